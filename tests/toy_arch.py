"""A toy architecture made only of things defined in this file plus registered built-in parts,
registered from outside the package: a mixer whose state is the running sum of its inputs (fixed size
per request, no pages), a mixer that keeps one latent vector per token in the paged cache (one tensor per
token, no keys and values), a feed-forward that is one linear map and one that routes every token to one of
three experts, a rotary encoding with interleaved pairs
(not the fused kernel's form), a layer order that runs layer 0 twice and lets the last call read the
cache another call wrote. Used on the GPU (tests/test_parts_gpu.py) and, with the plain kernel twins,
on the CPU (tests/test_engine_cpu.py): through the step function with explicit cuts (`run_toy`) and through
`LLM.generate`, scheduler, decode graphs and steps run one ahead (`run_toy_engine`). The mixers use device
operations only (no value travels to the host inside `forward`), which is what lets a decode step that
contains them be captured as a graph."""
import tempfile

import torch

import helpers
import plain_qwen3 as P
from mini_engine_amd.cache.manager import CacheManager
from mini_engine_amd.config.model_config import register_config
from mini_engine_amd.engine.runner import ModelRunner
from mini_engine_amd.models.model import DecoderModel, WeightSource
from mini_engine_amd.parts import (PAGE, CacheNeed, FeedForward, LayerCall, Mixer, PageTensor, ParamSpec,
                                   PositionEncoding, StateNeed, make_part, register_part, registered)
from mini_engine_amd.parts.embedding import LMHead, TokenEmbedding
from mini_engine_amd.registry import build_model, register_architecture
from mini_engine_amd.weights.random_init import fill_random, write_random_model


PRIOR_COUNT = 2.0      # the running mean starts as if it had seen this many zero vectors


def half_to_one(shape, generator, device):
    """An init function of a part's own: uniform in [0.5, 1)."""
    return 0.5 + 0.5 * torch.rand(shape, generator=generator, dtype=torch.float32, device=device)


@register_part("mixer", "toy_running_mean")
class RunningMean(Mixer):
    """y_t = W . (gain * (x_0 + .. + x_t) / (t + 1 + PRIOR_COUNT)). State per request: [hidden + 1] = (sum of
    inputs, count); the count of a request that has seen nothing is PRIOR_COUNT, not zero (`StateNeed.initial`),
    and `gain` is drawn by a function of this file (`ParamSpec.init`)."""

    def __init__(self, hidden_size):
        super().__init__()
        self.hidden_size = hidden_size
        self.add_param("weight", ParamSpec((hidden_size, hidden_size), init="matrix", dtype="compute"))
        self.add_param("gain", ParamSpec((hidden_size,), init=half_to_one, dtype="float32"))

    def state_need(self):
        return StateNeed((self.hidden_size + 1,), "float32", initial=(0.0,) * self.hidden_size + (PRIOR_COUNT,))

    def forward(self, x, step, cache, state):
        T = x.shape[0]
        seq, cu, slots = step.seq_of_token.long(), step.cu_seqlens.long(), step.state_slots.long()
        xs = x.float()
        cs = xs.cumsum(0)
        first = cu[seq]                                   # a request's tokens are consecutive and in order
        within = cs - (cs[first] - xs[first])             # running sum over the request's tokens of this step
        held = state[slots]                               # [B, hidden + 1]
        sums = held[seq, :-1] + within
        counts = held[seq, -1] + (torch.arange(T, device=x.device) - first + 1).float()
        last = cu[1:] - 1
        state.index_copy_(0, slots, torch.cat([sums[last], counts[last, None]], 1))
        return (self.gain * sums / counts[:, None]).to(x.dtype) @ self.weight.T


@register_part("mixer", "toy_latent_mean")
class LatentMean(Mixer):
    """y_t = W_out . mean_{j <= t}(W_in x_j). The cache holds one float32 vector W_in x_j per token: a page
    is [page, latent], there are no heads, keys or values. Everything it reads comes through the block
    table, so it works for any cut of the tokens into steps."""

    def __init__(self, hidden_size, latent_size):
        super().__init__()
        self.latent_size = latent_size
        self.add_param("w_in", ParamSpec((latent_size, hidden_size), init="matrix", dtype="compute"))
        self.add_param("w_out", ParamSpec((hidden_size, latent_size), init="matrix", dtype="compute"))

    def cache_need(self):
        return CacheNeed((PageTensor("z", (PAGE, self.latent_size), "float32"),))

    def forward(self, x, step, cache, state):
        grp = step.groups[cache.group]
        store = cache.tensors["z"]                        # [pages + 1, page, latent]
        r, page = self.latent_size, cache.page_size
        store.view(-1, r).index_copy_(0, grp.slot_mapping.long(), (x @ self.w_in.T).float())
        table = grp.block_tables.long()                   # [B, MB], -1 where there is no page
        B, MB = table.shape
        held = store[table.clamp(min=0)].reshape(B, MB * page, r)[step.seq_of_token.long()]     # [T, MB * page, r]
        pos = step.positions.long()
        seen = torch.arange(MB * page, device=x.device)[None, :] <= pos[:, None]
        mean = torch.where(seen[..., None], held, torch.zeros((), device=x.device)).sum(1) / (pos + 1).float()[:, None]
        return mean.to(x.dtype) @ self.w_out.T


@register_part("feed_forward", "toy_linear")
class ToyLinear(FeedForward):
    def __init__(self, hidden_size):
        super().__init__()
        self.add_param("weight", ParamSpec((hidden_size, hidden_size), init="matrix", dtype="compute"))

    def forward(self, x):
        return x @ self.weight.T


@register_part("feed_forward", "toy_top1_experts")
class ToyExperts(FeedForward):
    """Every token goes to the expert with the largest router logit and is scaled by that expert's softmax
    weight: y = p_e . W_e x, e = argmax(R x). The router works in float32 whatever the compute dtype. Each
    token picks its expert's matrix on the device (no value travels to the host, so a decode step with this
    feed-forward can be captured as a graph)."""

    def __init__(self, hidden_size, num_experts, router_scale):
        super().__init__()
        self.num_experts, self.router_scale = num_experts, router_scale
        self.add_param("router", ParamSpec((num_experts, hidden_size), init="matrix", dtype="float32"))
        self.add_param("experts", ParamSpec((num_experts, hidden_size, hidden_size), init="matrix", dtype="compute"))

    def forward(self, x):
        logits = (x.float() @ self.router.T) * self.router_scale
        weight, chosen = torch.softmax(logits, -1).max(-1)
        y = torch.bmm(self.experts[chosen], x.unsqueeze(-1)).squeeze(-1)        # [T, n, k] x [T, k, 1]
        return (y.float() * weight[:, None]).to(x.dtype)


@register_part("position_encoding", "toy_interleaved_rotary")
class InterleavedRotary(PositionEncoding):
    """Rotates the pairs (x_2i, x_2i+1) instead of (x_i, x_i+D/2): not the fused kernel's form, so the
    attention mixer must go through `apply` and the stand-alone cache write."""

    def __init__(self, head_dim, theta):
        super().__init__()
        self.head_dim, self.theta = head_dim, theta

    def angles(self, positions):
        inv = self.theta ** (-torch.arange(0, self.head_dim, 2, dtype=torch.float32, device=positions.device) / self.head_dim)
        return positions.float()[:, None] * inv[None, :]

    def apply(self, q, k, positions):
        a = self.angles(positions)
        c, s = a.cos()[:, None, :], a.sin()[:, None, :]
        for x in (q, k):
            e, o = x[..., 0::2].float(), x[..., 1::2].float()
            ne, no = e * c - o * s, o * c + e * s
            x[..., 0::2] = ne.to(x.dtype)
            x[..., 1::2] = no.to(x.dtype)


ROUTER_SCALE = 400.0       # router logits of order 10: their softmax is far from uniform


@register_config("ToyForCausalLM")
class ToyConfig:
    def __init__(self, vocab_size, hidden_size, eps):
        self.vocab_size, self.hidden_size, self.eps = vocab_size, hidden_size, eps

    @classmethod
    def from_dict(cls, raw):
        return cls(raw["vocab_size"], raw["hidden_size"], raw["eps"])

    def to_dict(self):
        return {"architectures": ["ToyForCausalLM"], "vocab_size": self.vocab_size, "hidden_size": self.hidden_size,
                "eps": self.eps}


@register_architecture("ToyForCausalLM")
def build_toy(cfg):
    h = cfg.hidden_size
    def block(mixer, feed_forward=None):
        return make_part("block", "pre_norm", norm1=make_part("norm", "rms", size=h, eps=cfg.eps), mixer=mixer,
                         norm2=make_part("norm", "rms", size=h, eps=cfg.eps), feed_forward=feed_forward or ToyLinear(h))
    rot = InterleavedRotary(16, 1e4)
    att = dict(hidden_size=h, num_heads=2, num_kv_heads=1, head_dim=16, scale=0.25, position=rot)
    layers = [block(RunningMean(h)),
              block(make_part("mixer", "attention", qk_norm_eps=None, **att),
                    make_part("feed_forward", "toy_top1_experts", hidden_size=h, num_experts=3, router_scale=ROUTER_SCALE)),
              block(make_part("mixer", "attention", qk_norm_eps=1e-5, own_kv=False, **att)),   # queries only
              block(LatentMean(h, 12))]
    emb = TokenEmbedding(cfg.vocab_size, h)
    # layer 0 runs twice (state of its own each time); call 3 reads the cache that call 1 wrote
    order = [LayerCall(0), LayerCall(1), LayerCall(0), LayerCall(2, cache_of=1), LayerCall(3)]
    model = DecoderModel(cfg, emb, layers, order, make_part("norm", "rms", size=h, eps=cfg.eps),
                         LMHead(cfg.vocab_size, h, tied_to=emb), {})
    model.weight_sources = {name: [WeightSource("toy." + name)] for name, _, _, _ in model.named_specs()}
    return model


def _toy_plain(model, ids, margins=None):
    """Whole-sequence float64 evaluation of the toy model, written out directly. `margins` collects, for
    every routed token, (the gap between its two largest router logits, the expert it goes to)."""
    W = lambda t: t.double().cpu()
    def norm(p, x): return P.rms_norm(x, W(p.weight), p.eps)
    x = W(model.embedding.weight)[ids]
    res = torch.zeros_like(x)
    h = x
    T = len(ids)
    ang = torch.arange(T, dtype=torch.float64)[:, None] * (1e4 ** (-torch.arange(0, 16, 2, dtype=torch.float64) / 16))[None, :]
    def rot(t):          # interleaved pairs, as InterleavedRotary
        e, o = t[..., 0::2], t[..., 1::2]
        out = torch.empty_like(t)
        out[..., 0::2] = e * ang.cos()[:, None, :] - o * ang.sin()[:, None, :]
        out[..., 1::2] = o * ang.cos()[:, None, :] + e * ang.sin()[:, None, :]
        return out
    kept = {}
    for ci, call in enumerate(model.order):
        layer = model.layers[call.layer]
        res = res + h
        a = norm(layer.norm1, res)
        if isinstance(layer.mixer, RunningMean):
            count = torch.arange(1, T + 1, dtype=torch.float64) + PRIOR_COUNT
            a = (W(layer.mixer.gain) * a.cumsum(0) / count[:, None]) @ W(layer.mixer.weight).T
        elif isinstance(layer.mixer, LatentMean):
            z = a @ W(layer.mixer.w_in).T
            a = (z.cumsum(0) / torch.arange(1, T + 1, dtype=torch.float64)[:, None]) @ W(layer.mixer.w_out).T
        else:
            m = layer.mixer
            qkv = a @ W(m.qkv.weight).T
            q = qkv[:, :32].view(T, 2, 16)
            if m.own_kv:
                k, v = rot(qkv[:, 32:48].view(T, 1, 16)), qkv[:, 48:].view(T, 1, 16)
                kept[ci] = (k, v)
            else:
                q = P.rms_norm(q, W(m.q_norm_weight), m.qk_norm_eps)
                k, v = kept[call.cache_of]
            o = P.causal_attention(rot(q), k, v, 0.25)
            a = o.reshape(T, 32) @ W(m.o.weight).T
        res = res + a
        f = norm(layer.norm2, res)
        if isinstance(layer.feed_forward, ToyExperts):
            ff = layer.feed_forward
            logits = (f @ W(ff.router).T) * ff.router_scale
            top = logits.topk(2, -1).values
            p, e = torch.softmax(logits, -1).max(-1)
            if margins is not None:
                margins += zip((top[:, 0] - top[:, 1]).tolist(), e.tolist())
            h = torch.einsum("tk,tnk->tn", f, W(ff.experts)[e]) * p[:, None]      # one expert per token
        else:
            h = f @ W(layer.feed_forward.weight).T
    return norm(model.final_norm, res + h) @ W(model.embedding.weight).T




def run_toy(device, dtype, tol):
    assert "toy_running_mean" in registered("mixer") and "toy_linear" in registered("feed_forward")
    assert "toy_top1_experts" in registered("feed_forward")
    cfg = ToyConfig.from_dict({"vocab_size": 50, "hidden_size": 40, "eps": 1e-5})
    model = build_model(cfg)
    plan = model.cache_plan()
    assert "toy_interleaved_rotary" in registered("position_encoding")
    assert plan.state_needs[0] is not None and plan.state_needs[2] is not None and plan.state_needs[1] is None
    assert plan.call_group == [None, 0, None, 0, 1] and plan.call_writes == [False, True, False, False, True]
    assert plan.group_calls == [[1], [4]]                             # keys and values of call 1; latents of call 4
    fill_random(model, 4, device, dtype, 128)
    manager = CacheManager(8, 8, ModelRunner.windows_of(model), num_state_slots=3)
    runner = ModelRunner(model, manager, dtype, device, 128, poison_cache=True)
    assert runner.pool.states[0] is not runner.pool.states[2]      # each call of layer 0 has state of its own
    a, b = helpers.random_ids(30, 50, 54), helpers.random_ids(12, 50, 34)     # seeds with clear routing, see below
    d = helpers.Driver(runner, manager)
    d.step({"a": a[:11]}); d.step({"a": a[11:12], "b": b[:5]}); d.step({"b": b[5:6], "a": a[12:29]})
    d.step({"a": a[29:], "b": b[6:]}, end=["a"])
    c = helpers.random_ids(9, 50, 46)                                # takes over a's slot: must start from zero state
    d.step({"c": c}, end=["b", "c"])
    margins = []
    for ids, rid in ((a, "a"), (b, "b"), (c, "c")):
        ref = _toy_plain(model, ids, margins)
        assert helpers.rel_err(d.result(rid), ref) <= tol, rid
    # the comparison means something only if no token sits between two experts (bfloat16 rounding moves a
    # logit by a few tenths and would then decide) and the tokens do not all go one way
    assert len(margins) == 51 and min(g for g, _ in margins) > 5
    assert len({e for _, e in margins}) == 3


def _toy_greedy(model, prompt, n, checks=None):
    """n greedy tokens from the plain evaluation; `checks` collects (logits, chosen) of every token."""
    ids = list(prompt)
    for _ in range(n):
        z = _toy_plain(model, ids)[-1]
        ids.append(int(z.argmax()))
        if checks is not None:
            checks.append((z, ids[-1]))
    return ids[len(prompt):]


def run_toy_engine(device, dtype_name, capture):
    """The toy architecture from a written folder through `LLM.generate`: admission under a token budget,
    portions of prompts beside decoding requests, state slots and latent pages taken and given back as
    requests come and go, a pool so small that requests are evicted and fed again, decode steps through
    `DecodeGraphs` (captured on a GPU) and launched one ahead. Greedy tokens against the plain evaluation."""
    from mini_engine_amd import LLM, SamplingParams
    cfg = ToyConfig.from_dict({"vocab_size": 50, "hidden_size": 40, "eps": 1e-5})
    prompts = [helpers.random_ids(n, 50, 70 + n) for n in (30, 12, 9, 1, 21)]
    with tempfile.TemporaryDirectory() as folder:
        write_random_model(cfg, 4, folder, torch.float32)
        for pages, run_ahead in ((24, True), (9, True), (24, False)):
            llm = LLM(folder, dtype=dtype_name, device=device, kvcache_block_size=8, num_kvcache_blocks=pages, max_num_seqs=3,
                      max_num_batched_tokens=16, max_model_len=64, poison_cache=True, run_ahead=run_ahead)
            assert llm.manager.num_groups == 2 and llm.manager.num_state_slots == 3 and not llm.manager.prefix_caching
            outs = llm.generate(prompts, SamplingParams(temperature=0, max_tokens=10, ignore_eos=True), use_tqdm=False)
            graphs = llm.runner.graphs
            assert graphs.replays > 0, "no decode step went through the fixed-layout path"
            assert (llm.steps_run_ahead > 0) == run_ahead
            if capture:
                assert any(c.graph is not None for c in graphs.captured.values()), "no decode step was captured"
            if pages == 9:
                assert llm.scheduler.num_preemptions > 0, "the pool was large enough that nobody was evicted"
            llm.manager.check_invariants()
            assert all(llm.manager.num_free_pages(g) == pages for g in range(2)) and len(llm.manager.free_slots) == 3
            for p, o in zip(prompts, outs):
                ids = list(p)
                for tok in o["token_ids"]:
                    z = _toy_plain(llm.model, ids)[-1]
                    best = int(z.argmax())
                    # bfloat16 may pick another token only where the two logits lie within its rounding
                    close = dtype_name == "bfloat16" and float(z[best] - z[tok]) < 3e-2 * float(z.abs().max())
                    assert tok == best or close, f"{dtype_name}, {pages} pages: generated {tok}, plain gives {best}"
                    ids.append(tok)

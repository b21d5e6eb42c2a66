"""A toy architecture made only of things defined in this file plus registered built-in parts,
registered from outside the package: a mixer whose state is the running sum of its inputs (fixed size
per request, no pages), a feed-forward that is one linear map and one that routes every token to one of
three experts, a rotary encoding with interleaved pairs
(not the fused kernel's form), a layer order that runs layer 0 twice and lets the last call read the
cache another call wrote. Used on the GPU (tests/test_parts_gpu.py) and, with the plain kernel twins,
on the CPU (tests/test_engine_cpu.py)."""
import torch

import helpers
import plain_qwen3 as P
from mini_engine_amd.cache.manager import CacheManager
from mini_engine_amd.config.model_config import register_config
from mini_engine_amd.engine.runner import ModelRunner
from mini_engine_amd.models.model import DecoderModel, WeightSource
from mini_engine_amd.parts import (FeedForward, LayerCall, Mixer, ParamSpec, PositionEncoding, StateNeed, make_part,
                                   register_part, registered)
from mini_engine_amd.parts.embedding import LMHead, TokenEmbedding
from mini_engine_amd.registry import build_model, register_architecture
from mini_engine_amd.weights.random_init import fill_random


@register_part("mixer", "toy_running_mean")
class RunningMean(Mixer):
    """y_t = W . mean(x_0..x_t). State per request: [hidden + 1] = (sum of inputs, count)."""

    def __init__(self, hidden_size):
        super().__init__()
        self.hidden_size = hidden_size
        self.add_param("weight", ParamSpec((hidden_size, hidden_size), init="matrix", dtype="compute"))

    def state_need(self):
        return StateNeed((self.hidden_size + 1,), "float32")

    def forward(self, x, step, cache, state):
        out = torch.empty_like(x)
        o = 0
        slots = step.state_slots.tolist()
        for b, n in enumerate(step.q_lens):            # a request's tokens are consecutive and in order
            s = state[slots[b]]
            xs = x[o:o + n].float()
            sums = s[:-1] + xs.cumsum(0)
            counts = s[-1] + torch.arange(1, n + 1, device=x.device, dtype=torch.float32)
            out[o:o + n] = ((sums / counts[:, None]).to(x.dtype) @ self.weight.T)
            s[:-1] = sums[-1]; s[-1] = counts[-1]
            o += n
        return out


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
    weight: y = p_e . W_e x, e = argmax(R x). The router works in float32 whatever the compute dtype; the
    tokens are grouped by expert, so each expert sees its tokens as one matrix."""

    def __init__(self, hidden_size, num_experts, router_scale):
        super().__init__()
        self.num_experts, self.router_scale = num_experts, router_scale
        self.add_param("router", ParamSpec((num_experts, hidden_size), init="matrix", dtype="float32"))
        self.add_param("experts", ParamSpec((num_experts, hidden_size, hidden_size), init="matrix", dtype="compute"))

    def forward(self, x):
        logits = (x.float() @ self.router.T) * self.router_scale
        weight, chosen = torch.softmax(logits, -1).max(-1)
        out = torch.empty_like(x)
        for e in range(self.num_experts):
            rows = (chosen == e).nonzero().flatten()
            if rows.numel():
                y = (x[rows] @ self.experts[e].T).float() * weight[rows, None]
                out[rows] = y.to(x.dtype)
        return out


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
              block(make_part("mixer", "attention", qk_norm_eps=1e-5, own_kv=False, **att))]   # queries only
    emb = TokenEmbedding(cfg.vocab_size, h)
    # layer 0 runs twice (state of its own each time); the last call reads the cache that call 1 wrote
    order = [LayerCall(0), LayerCall(1), LayerCall(0), LayerCall(2, cache_of=1)]
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
            a = (a.cumsum(0) / torch.arange(1, T + 1, dtype=torch.float64)[:, None]) @ W(layer.mixer.weight).T
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
    assert plan.call_group == [None, 0, None, 0] and plan.call_writes == [False, True, False, False]
    assert plan.group_calls == [[1]]                                  # only call 1 owns pages
    fill_random(model, 4, device, dtype, 128)
    manager = CacheManager(8, 8, ModelRunner.windows_of(model), num_state_slots=3)
    runner = ModelRunner(model, manager, dtype, device, 128, poison_cache=True)
    assert runner.pool.states[0] is not runner.pool.states[2]      # each call of layer 0 has state of its own
    a, b = helpers.random_ids(30, 50, 50), helpers.random_ids(12, 50, 34)     # seeds with clear routing, see below
    d = helpers.Driver(runner, manager)
    d.step({"a": a[:11]}); d.step({"a": a[11:12], "b": b[:5]}); d.step({"b": b[5:6], "a": a[12:29]})
    d.step({"a": a[29:], "b": b[6:]}, end=["a"])
    c = helpers.random_ids(9, 50, 44)                                # takes over a's slot: must start from zero state
    d.step({"c": c}, end=["b", "c"])
    margins = []
    for ids, rid in ((a, "a"), (b, "b"), (c, "c")):
        ref = _toy_plain(model, ids, margins)
        assert helpers.rel_err(d.result(rid), ref) <= tol, rid
    # the comparison means something only if no token sits between two experts (bfloat16 rounding moves a
    # logit by a few tenths and would then decide) and the tokens do not all go one way
    assert len(margins) == 51 and min(g for g, _ in margins) > 5
    assert len({e for _, e in margins}) == 3

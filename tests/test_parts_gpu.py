"""Each part alone against its plain formula, and a toy mixer with state of its own, defined
here, registered, built and stepped without a change to the framework's files."""
import pytest
import torch

import helpers
import plain_qwen3 as P
from mini_engine_amd.cache.manager import CacheManager
from mini_engine_amd.config.model_config import register_config
from mini_engine_amd.engine.runner import ModelRunner, StepEntry
from mini_engine_amd.models.model import DecoderModel, WeightSource
from mini_engine_amd.parts import (FeedForward, LayerCall, Mixer, ParamSpec, StateNeed, make_part, register_part,
                                   registered)
from mini_engine_amd.parts.embedding import LMHead, TokenEmbedding
from mini_engine_amd.registry import build_model, register_architecture
from mini_engine_amd.weights.random_init import fill_random

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _bind(part, dtype):
    g = torch.Generator().manual_seed(0)
    for name, owner, local, spec in part.named_specs():
        t = torch.randn(spec.shape, generator=g) * (0.1 if spec.init == "matrix" else 0.05) + (1.0 if spec.init == "norm" else 0.0)
        owner.set_param(local, t.to(DEV).to(torch.float32 if spec.dtype == "float32" else dtype))
    for p in part.parts():
        p.finalize(torch.device(DEV), dtype, 256)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-6), (torch.bfloat16, 8e-3)])
def test_norm_part(dtype, tol):
    norm = make_part("norm", "rms", size=72, eps=3e-6); _bind(norm, dtype)
    x, r = torch.randn(9, 72, device=DEV).to(dtype), torch.randn(9, 72, device=DEV)
    y, res = norm.forward(x, r)
    yr, rr = P.add_rms_norm(x.double(), r.double(), norm.weight.double(), 3e-6)
    assert y.dtype == dtype and res.dtype == torch.float32
    assert float((y.double() - yr).abs().max() / yr.abs().max()) <= tol and torch.allclose(res.double(), rr, atol=1e-6)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-6), (torch.bfloat16, 1.5e-2)])
def test_feed_forward_part(dtype, tol):
    ff = make_part("feed_forward", "swiglu", hidden_size=80, intermediate_size=224); _bind(ff, dtype)
    x = torch.randn(11, 80, device=DEV).to(dtype)
    y = ff.forward(x)
    y = y.sum(0) if y.dim() == 3 else y
    w = ff.gate_up.weight.double()
    ref = P.silu_and_mul(x.double() @ w[:224].T, x.double() @ w[224:].T) @ ff.down.weight.double().T
    assert float((y.double() - ref).abs().max() / ref.abs().max()) <= tol


def test_rotary_part_matches_plain_tables_and_unfused_apply():
    rot = make_part("position_encoding", "rotary", head_dim=32, theta=1e6); _bind(rot, torch.float32)
    # angles are formed in float32 as the reference forms them (layers/rotary_embedding.py:13-18), so the
    # table equals the float32 evaluation of the formula closely, and the float64 one up to the rounding
    # of an angle of up to 255 rad (255 * 2^-24)
    cos32, sin32 = P.rope_tables(32, 256, 1e6, torch.float32)
    assert torch.allclose(rot.table[..., 0].cpu(), cos32[:, :16], atol=1e-6)
    assert torch.allclose(rot.table[..., 1].cpu(), sin32[:, :16], atol=1e-6)
    cos, sin = P.rope_tables(32, 256, 1e6)
    assert torch.allclose(rot.table[..., 0].double().cpu(), cos[:, :16], atol=3e-5)
    assert torch.allclose(rot.table[..., 1].double().cpu(), sin[:, :16], atol=3e-5)
    q, k = torch.randn(7, 3, 32, device=DEV), torch.randn(7, 1, 32, device=DEV)
    pos = torch.tensor([0, 5, 9, 100, 255, 1, 2], device=DEV, dtype=torch.int32)
    qr = P.apply_rope(q.double().cpu(), cos32.double(), sin32.double(), pos.long().cpu())   # float32 angles, as above
    rot.apply(q, k, pos)
    assert torch.allclose(q.double().cpu(), qr, atol=1e-5)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 2e-2)])
@pytest.mark.parametrize("window", [None, 10])
def test_attention_part_alone(dtype, tol, window):
    """The mixer by itself: a whole sequence in two portions against plain attention."""
    from mini_engine_amd.cache.pool import CachePool
    from mini_engine_amd.engine.context import GroupStep, StepContext
    h, Hq, Hkv, D, page, T = 72, 6, 3, 16, 8, 37
    rot = make_part("position_encoding", "rotary", head_dim=D, theta=1e4)
    att = make_part("mixer", "attention", hidden_size=h, num_heads=Hq, num_kv_heads=Hkv, head_dim=D, scale=D ** -0.5,
                    qk_norm_eps=1e-5, position=rot, window=window)
    _bind(att, dtype)
    x = torch.randn(T, h, device=DEV).to(dtype)
    k_cache = torch.full((6, Hkv, page, D), float("nan"), device=DEV, dtype=dtype)
    v_cache = torch.full((6, Hkv, D, page), float("nan"), device=DEV, dtype=dtype)
    from mini_engine_amd.parts import CacheView
    view = CacheView(0, k_cache, v_cache, page)
    table = [4, 1, 5, 0, 2]
    outs = []
    for a, b in ((0, 20), (20, T)):
        n = b - a
        i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
        ctx = StepContext(num_tokens=n, num_seqs=1, num_decodes=0, positions=i32(list(range(a, b))), seq_of_token=i32([0] * n),
                          context_lens=i32([b]), cu_seqlens=i32([0, n]), prefill_cu=i32([0, n]), max_decode_context=0,
                          groups=[GroupStep(i32([table]), i32([table[p // page] * page + p % page for p in range(a, b)]))])
        y = att.forward(x[a:b], ctx, view, None)
        outs.append(y.sum(0) if y.dim() == 3 else y)
    got = torch.cat(outs).double().cpu()
    xd = x.double().cpu()
    w = att.qkv.weight.double().cpu()
    q = P.rms_norm((xd @ w[:Hq * D].T).view(T, Hq, D), att.q_norm_weight.double().cpu(), 1e-5)
    k = P.rms_norm((xd @ w[Hq * D:(Hq + Hkv) * D].T).view(T, Hkv, D), att.k_norm_weight.double().cpu(), 1e-5)
    v = (xd @ w[(Hq + Hkv) * D:].T).view(T, Hkv, D)
    cos, sin = P.rope_tables(D, T, 1e4)
    o = P.causal_attention(P.apply_rope(q, cos, sin, torch.arange(T)), P.apply_rope(k, cos, sin, torch.arange(T)), v, D ** -0.5, window)
    ref = o.reshape(T, Hq * D) @ att.o.weight.double().cpu().T
    assert float((got - ref).abs().max() / ref.abs().max()) <= tol


# ----------------------------------------------------------------------------------------------
# A toy architecture made only of things defined in this file plus registered built-in parts:
# a mixer whose state is the running sum of its inputs (fixed size per request, no pages), a
# feed-forward that is one linear map, a layer order that runs layer 0 twice.

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
    def block(mixer):
        return make_part("block", "pre_norm", norm1=make_part("norm", "rms", size=h, eps=cfg.eps), mixer=mixer,
                         norm2=make_part("norm", "rms", size=h, eps=cfg.eps), feed_forward=ToyLinear(h))
    rot = make_part("position_encoding", "rotary", head_dim=16, theta=1e4)
    layers = [block(RunningMean(h)),
              block(make_part("mixer", "attention", hidden_size=h, num_heads=2, num_kv_heads=1, head_dim=16, scale=0.25,
                              qk_norm_eps=None, position=rot))]
    emb = TokenEmbedding(cfg.vocab_size, h)
    model = DecoderModel(cfg, emb, layers, [LayerCall(0), LayerCall(1), LayerCall(0)], make_part("norm", "rms", size=h, eps=cfg.eps),
                         LMHead(cfg.vocab_size, h, tied_to=emb), {})
    model.weight_sources = {name: [WeightSource("toy." + name)] for name, _, _, _ in model.named_specs()}
    return model


def _toy_plain(model, ids):
    """Whole-sequence float64 evaluation of the toy model, written out directly."""
    W = lambda t: t.double().cpu()
    def norm(p, x): return P.rms_norm(x, W(p.weight), p.eps)
    x = W(model.embedding.weight)[ids]
    res = torch.zeros_like(x)
    h = x
    T = len(ids)
    for call in model.order:
        layer = model.layers[call.layer]
        res = res + h
        a = norm(layer.norm1, res)
        if isinstance(layer.mixer, RunningMean):
            a = (a.cumsum(0) / torch.arange(1, T + 1, dtype=torch.float64)[:, None]) @ W(layer.mixer.weight).T
        else:
            m = layer.mixer
            qkv = a @ W(m.qkv.weight).T
            q, k, v = qkv[:, :32].view(T, 2, 16), qkv[:, 32:48].view(T, 1, 16), qkv[:, 48:].view(T, 1, 16)
            cos, sin = P.rope_tables(16, T, 1e4)
            o = P.causal_attention(P.apply_rope(q, cos, sin, torch.arange(T)), P.apply_rope(k, cos, sin, torch.arange(T)), v, 0.25)
            a = o.reshape(T, 32) @ W(m.o.weight).T
        res = res + a
        h = norm(layer.norm2, res) @ W(layer.feed_forward.weight).T
    return norm(model.final_norm, res + h) @ W(model.embedding.weight).T


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 3e-2)])
def test_toy_architecture_registers_builds_and_steps(dtype, tol):
    assert "toy_running_mean" in registered("mixer") and "toy_linear" in registered("feed_forward")
    cfg = ToyConfig.from_dict({"vocab_size": 50, "hidden_size": 40, "eps": 1e-5})
    model = build_model(cfg)
    plan = model.cache_plan()
    assert plan.state_needs[0] is not None and plan.state_needs[2] is not None and plan.state_needs[1] is None
    assert plan.call_group == [None, 0, None]
    fill_random(model, 4, DEV, dtype, 128)
    manager = CacheManager(8, 8, ModelRunner.windows_of(model), num_state_slots=3)
    runner = ModelRunner(model, manager, dtype, DEV, 128, poison_cache=True)
    assert runner.pool.states[0] is not runner.pool.states[2]      # each call of layer 0 has state of its own
    a, b = helpers.random_ids(30, 50, 1), helpers.random_ids(12, 50, 2)
    d = helpers.Driver(runner, manager)
    d.step({"a": a[:11]}); d.step({"a": a[11:12], "b": b[:5]}); d.step({"b": b[5:6], "a": a[12:29]})
    d.step({"a": a[29:], "b": b[6:]}, end=["a"])
    c = helpers.random_ids(9, 50, 3)                                 # takes over a's slot: must start from zero state
    d.step({"c": c}, end=["b", "c"])
    for ids, rid in ((a, "a"), (b, "b"), (c, "c")):
        ref = _toy_plain(model, ids)
        assert helpers.rel_err(d.result(rid), ref) <= tol, rid

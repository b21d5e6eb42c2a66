"""Each part alone against its plain formula, and a toy mixer with state of its own, defined
here, registered, built and stepped without a change to the framework's files."""
import pytest
import torch

import helpers
import plain_qwen3 as P
from mini_engine_amd.parts import make_part

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


@pytest.mark.parametrize("rows", [1, 2, 5])
def test_norm_handed_to_the_next_part_unrun(rows):
    """A part that `takes_pending_norm` gets the norm in front of it as a `PendingNorm`. Its first product runs
    the norm inside itself where there is a kernel for that (bfloat16, one or two rows), otherwise the norm runs
    in front of it: either way the part's output and the new residual are those of the plain formulas. A norm
    without `linear_behind` (a toy one, defined here) is simply run."""
    from mini_engine_amd.parts import PendingNorm
    from mini_engine_amd.parts.base import Norm
    dtype = torch.bfloat16
    norm = make_part("norm", "rms", size=80, eps=3e-6); _bind(norm, dtype)
    ff = make_part("feed_forward", "swiglu", hidden_size=80, intermediate_size=224); _bind(ff, dtype)
    assert ff.takes_pending_norm
    parts, r = torch.randn(3, rows, 80, device=DEV), torch.randn(rows, 80, device=DEV)
    xr, rr = P.add_rms_norm(parts.double().sum(0), r.double(), norm.weight.double(), 3e-6)
    w = ff.gate_up.weight.double()
    ref = P.silu_and_mul(xr @ w[:224].T, xr @ w[224:].T) @ ff.down.weight.double().T

    def check(pending):
        y = ff.forward(pending)
        y = y.sum(0) if y.dim() == 3 else y
        assert float((y.double() - ref).abs().max() / ref.abs().max()) <= 2e-2
        assert torch.allclose(pending.new_residual().double(), rr, atol=1e-5)

    pending = PendingNorm(norm, parts, r)
    check(pending)
    assert (pending._y is None) == (rows <= 2)             # one or two rows: the norm never ran on its own

    class PlainNorm(Norm):                                 # no partial sums, no fused form
        def forward(self, x, residual):
            return norm.forward(x, residual)

    check(PendingNorm(PlainNorm(), parts, r))
    late = PendingNorm(norm, parts, r)                     # asked for its value first: runs as a norm, once
    first = late.value()
    assert late.into_linear(ff.gate_up.weight) is None and late.value() is first


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
    view = CacheView(0, {"k": k_cache, "v": v_cache}, page)
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


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 3e-2)])
def test_toy_architecture_registers_builds_and_steps(dtype, tol):
    """A mixer with state of its own, another feed-forward, another position encoding and a new
    architecture, all defined in tests/toy_arch.py and registered from there: no framework file changes."""
    import toy_arch
    toy_arch.run_toy(DEV, dtype, tol)


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_toy_architecture_through_the_engine_and_captured_graphs(dtype_name):
    """The toy architecture (state of its own, a cache of one tensor per token) from a written folder through
    `LLM.generate`: its decode steps are captured as graphs and launched one ahead, with no framework file changed."""
    import toy_arch
    toy_arch.run_toy_engine(DEV, dtype_name, capture=True)

"""Each HIP kernel alone against its plain twin, at sizes other than the engine tests use.
Inputs are built so that faults show: NaN in every cache slot nobody owns, a far key made to
dominate among hundreds, window edges, page edges, sizes that are no power of two."""
import math

import pytest
import torch

import kernel_twins as twin
from mini_engine_amd.kernels import ops

pytestmark = pytest.mark.gpu
DEV = "cuda"


def hip():
    return ops.HipBackend()


def close(a, b, tol):
    a, b = a.double().cpu(), b.double().cpu()
    assert torch.isfinite(a).all()
    err = float((a - b).abs().max() / b.abs().max().clamp_min(1e-30))
    assert err <= tol, f"relative error {err:.3g} > {tol:g}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,width", [(7, 100), (300, 1024), (5, 3)])
def test_gather_rows(dtype, rows, width):
    src = torch.randn(rows, width, device=DEV).to(dtype)
    idx = torch.randint(0, rows, (41,), device=DEV, dtype=torch.int32)
    assert torch.equal(hip().gather_rows(src, idx), twin.gather_rows(src, idx))


def test_take_tokens():
    """Rows that name a row of the sampling call's output take its token; rows that name none (-1) keep theirs."""
    sampled = torch.randint(0, 1000, (37,), device=DEV, dtype=torch.int32)
    for rows in (1, 8, 300):
        tokens = torch.randint(1000, 2000, (rows,), device=DEV, dtype=torch.int32)
        take = torch.randint(-1, 37, (rows,), device=DEV, dtype=torch.int32)
        want = tokens.clone()
        twin.take_tokens(want, sampled, take)
        hip().take_tokens(tokens, sampled, take)
        assert torch.equal(tokens, want)
        assert torch.equal(tokens[take < 0], want[take < 0]) and (want[take >= 0] < 1000).all()


@pytest.mark.parametrize("T,n", [(1, 80), (13, 1000), (64, 4096), (3, 5120), (300, 1024), (257, 72), (1000, 1028),
                                 (300, 520), (257, 4104), (256, 5120), (260, 5128)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rms_norm(dtype, T, n):
    torch.manual_seed(T * n)
    x = (torch.randn(T, n, device=DEV) * 3).to(dtype)
    res = torch.randn(T, n, device=DEV)
    w = torch.rand(n, device=DEV) + 0.5
    tol = 1e-6 if dtype == torch.float32 else 4e-3
    y, r = hip().rms_norm(x, w, 1e-5, res, dtype)
    yt, rt = twin.rms_norm(x, w, 1e-5, res, dtype)
    close(y, yt, tol); close(r, rt, 1e-6)
    y, r = hip().rms_norm(x, w, 1e-5, None, dtype)            # start of the residual stream
    yt, rt = twin.rms_norm(x, w, 1e-5, None, dtype)
    close(y, yt, tol); assert torch.equal(r, x.float())
    y, r = hip().rms_norm(x, w, 1e-5, res, dtype, want_residual=False)
    assert r is None
    parts = torch.randn(3, T, n, device=DEV)                  # stacked float32 partial sums
    y, r = hip().rms_norm(parts, w, 1e-6, res, dtype)
    yt, rt = twin.rms_norm(parts, w, 1e-6, res, dtype)
    close(y, yt, tol); close(r, rt, 1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_silu_and_mul(dtype):
    gu = (torch.randn(37, 2 * 224, device=DEV) * 4).to(dtype)
    close(hip().silu_and_mul(gu), twin.silu_and_mul(gu), 1e-6 if dtype == torch.float32 else 4e-3)
    big = torch.tensor([[-100.0, 100.0, 0.0, 1.0, 2.0, 3.0]], device=DEV).to(dtype)   # no overflow at the ends
    assert torch.isfinite(hip().silu_and_mul(big)).all()


def _caches(pages, Hkv, page, D, dtype):
    k = torch.full((pages, Hkv, page, D), float("nan"), device=DEV, dtype=dtype)
    v = torch.full((pages, Hkv, D, page), float("nan"), device=DEV, dtype=dtype)
    return k, v


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("Hq,Hkv,D,page", [(4, 2, 16, 16), (6, 2, 32, 8), (5, 5, 48, 4), (16, 8, 128, 16), (2, 1, 256, 32)])
def test_qk_norm_rope_store(dtype, Hq, Hkv, D, page):
    torch.manual_seed(D)
    T, P = 29, 64
    qkv = torch.randn(T, (Hq + 2 * Hkv) * D, device=DEV).to(dtype)
    qw, kw = torch.rand(D, device=DEV) + 0.5, torch.rand(D, device=DEV) + 0.5
    ang = torch.outer(torch.arange(P, dtype=torch.float32), 1.0 / (1e4 ** (torch.arange(0, D, 2).float() / D)))
    table = torch.stack((ang.cos(), ang.sin()), -1).contiguous().to(DEV)
    pos = torch.randint(0, P, (T,), device=DEV, dtype=torch.int32)
    slots = torch.randperm(8 * page, device=DEV)[:T].to(torch.int32)
    slots[3] = -1                                              # a skipped token
    tol = 2e-6 if dtype == torch.float32 else 4e-3
    for use_norm, use_rope in ((True, True), (False, True), (True, False)):
        a, b = qkv.clone(), qkv.clone()
        ka, va = _caches(8, Hkv, page, D, dtype); kb, vb = _caches(8, Hkv, page, D, dtype)
        args = (qw if use_norm else None, kw if use_norm else None, 1e-5, table if use_rope else None, pos, slots)
        hip().qk_norm_rope_store(a, *args, ka, va, Hq, Hkv, D, page, True)
        twin.qk_norm_rope_store(b, *args, kb, vb, Hq, Hkv, D, page, True)
        close(a[:, :Hq * D], b[:, :Hq * D], tol)
        assert torch.equal(torch.isnan(ka), torch.isnan(kb)) and torch.equal(torch.isnan(va), torch.isnan(vb))
        close(torch.nan_to_num(ka), torch.nan_to_num(kb), tol)
        assert torch.equal(torch.nan_to_num(va), torch.nan_to_num(vb))          # values are copied bit-exactly
        assert torch.equal(a[:, Hq * D:], qkv[:, Hq * D:])                       # k, v rows themselves untouched
    # in-place form: q and k rewritten, nothing cached; and q-only rows
    a, b = qkv[:, :(Hq + Hkv) * D].clone(), qkv[:, :(Hq + Hkv) * D].clone()
    hip().qk_norm_rope_store(a, qw, kw, 1e-5, table, pos, None, None, None, Hq, Hkv, D, page, False)
    twin.qk_norm_rope_store(b, qw, kw, 1e-5, table, pos, None, None, None, Hq, Hkv, D, page, False)
    close(a, b, tol)
    a, b = qkv[:, :Hq * D].clone(), qkv[:, :Hq * D].clone()
    hip().qk_norm_rope_store(a, qw, qw, 1e-5, table, pos, None, None, None, Hq, 0, D, page, False)
    twin.qk_norm_rope_store(b, qw, qw, 1e-5, table, pos, None, None, None, Hq, 0, D, page, False)
    close(a, b, tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("Hq,Hkv,D,page", [(4, 2, 16, 16), (6, 2, 32, 8), (5, 5, 48, 8), (16, 8, 128, 16), (2, 1, 256, 32),
                                           (3, 3, 64, 24)])
def test_qk_norm_rope_store_many_tokens(dtype, Hq, Hkv, D, page):
    """The form for many tokens (8 per workgroup): prompts written to consecutive slots from page
    starts and from the middle of a page, a token count that is no multiple of 8, scattered slots,
    skipped tokens."""
    torch.manual_seed(D + page)
    T, P, pages = 203, 512, 40
    qkv = torch.randn(T, (Hq + 2 * Hkv) * D, device=DEV).to(dtype)
    qw, kw = torch.rand(D, device=DEV) + 0.5, torch.rand(D, device=DEV) + 0.5
    ang = torch.outer(torch.arange(P, dtype=torch.float32), 1.0 / (1e4 ** (torch.arange(0, D, 2).float() / D)))
    table = torch.stack((ang.cos(), ang.sin()), -1).contiguous().to(DEV)
    pos = torch.randint(0, P, (T,), device=DEV, dtype=torch.int32)
    slots = torch.empty(T, dtype=torch.int64)
    slots[:96] = torch.arange(96) + 5 * page                    # a prompt from a page start
    slots[96:150] = torch.arange(54) + 20 * page + 3            # a chunk that starts inside a page
    slots[150:] = (torch.randperm(8 * page)[:T - 150] + 30 * page)   # scattered
    slots[[7, 100, 160]] = -1
    slots = slots.to(torch.int32).to(DEV)
    tol = 2e-6 if dtype == torch.float32 else 4e-3
    a, b = qkv.clone(), qkv.clone()
    ka, va = _caches(pages, Hkv, page, D, dtype); kb, vb = _caches(pages, Hkv, page, D, dtype)
    hip().qk_norm_rope_store(a, qw, kw, 1e-5, table, pos, slots, ka, va, Hq, Hkv, D, page, True)
    twin.qk_norm_rope_store(b, qw, kw, 1e-5, table, pos, slots, kb, vb, Hq, Hkv, D, page, True)
    close(a[:, :Hq * D], b[:, :Hq * D], tol)
    assert torch.equal(torch.isnan(ka), torch.isnan(kb)) and torch.equal(torch.isnan(va), torch.isnan(vb))
    close(torch.nan_to_num(ka), torch.nan_to_num(kb), tol)
    assert torch.equal(torch.nan_to_num(va), torch.nan_to_num(vb))
    assert torch.equal(a[:, Hq * D:], qkv[:, Hq * D:])
    a, b = qkv[:, :(Hq + Hkv) * D].clone(), qkv[:, :(Hq + Hkv) * D].clone()
    hip().qk_norm_rope_store(a, None, None, 1e-5, table, pos, None, None, None, Hq, Hkv, D, page, False)
    twin.qk_norm_rope_store(b, None, None, 1e-5, table, pos, None, None, None, Hq, Hkv, D, page, False)
    close(a, b, tol)
    # a mixed step: 5 decode rows in front of two prompts that start at page starts, so that no group of 8 batch rows
    # is a group of 8 aligned slots, and the last aligned group ends with the last row
    slots = torch.cat((torch.tensor([9 * page + 3, 2 * page, 11 * page + 15, 3 * page + 8, 12 * page + 1]),
                       torch.arange(128) + 14 * page, torch.arange(64) + 32 * page)).to(torch.int32).to(DEV)
    T2 = slots.numel()
    a, b = qkv[:T2].clone(), qkv[:T2].clone()
    ka, va = _caches(pages, Hkv, page, D, dtype); kb, vb = _caches(pages, Hkv, page, D, dtype)
    hip().qk_norm_rope_store(a, qw, kw, 1e-5, table, pos[:T2], slots, ka, va, Hq, Hkv, D, page, True)
    twin.qk_norm_rope_store(b, qw, kw, 1e-5, table, pos[:T2], slots, kb, vb, Hq, Hkv, D, page, True)
    assert torch.equal(torch.isnan(va), torch.isnan(vb)) and torch.equal(torch.nan_to_num(va), torch.nan_to_num(vb))
    close(torch.nan_to_num(ka), torch.nan_to_num(kb), tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_store_kv_is_bit_exact_and_skips_negative_slots(dtype):
    T, Hkv, D, page = 50, 3, 40, 8
    packed = torch.randn(T, (2 + 2 * Hkv) * D, device=DEV).to(dtype)
    k = packed[:, 2 * D:(2 + Hkv) * D].view(T, Hkv, D)        # strided views of a packed row
    v = packed[:, (2 + Hkv) * D:].view(T, Hkv, D)
    slots = torch.randperm(9 * page, device=DEV)[:T].to(torch.int32)
    slots[[0, 17]] = -1
    ka, va = _caches(9, Hkv, page, D, dtype); kb, vb = _caches(9, Hkv, page, D, dtype)
    hip().store_kv(k, v, slots, ka, va, page)
    twin.store_kv(k, v, slots, kb, vb, page)
    for x, y in ((ka, kb), (va, vb)):
        assert torch.equal(torch.isnan(x), torch.isnan(y)) and torch.equal(torch.nan_to_num(x), torch.nan_to_num(y))
    assert int((~torch.isnan(ka)).sum()) == (T - 2) * Hkv * D


# ------------------------------------------------------------------------------- attention

def _attention_case(dtype, Hq, Hkv, D, page, seqs, window=None, seed=0, peak=None):
    """seqs: list of (context length after the step, new tokens). Builds a paged cache with
    shuffled pages and NaN everywhere else, runs kernel and twin."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    order = sorted(range(len(seqs)), key=lambda i: seqs[i][1] != 1)          # decodes first
    seqs = [seqs[i] for i in order]
    B = len(seqs)
    need = [-(-L // page) for L, _ in seqs]
    total_pages = sum(need) + 3
    perm = torch.randperm(total_pages, generator=g).tolist()
    k_cache, v_cache = _caches(total_pages, Hkv, page, D, dtype)
    MB = max(need)
    bt = torch.full((B, MB + 1), -1, dtype=torch.int32)
    q_rows, seq_of, positions, ctx, cu = [], [], [], [], [0]
    for b, (L, n) in enumerate(seqs):
        pages = [perm.pop() for _ in range(need[b])]
        bt[b, :need[b]] = torch.tensor(pages, dtype=torch.int32)
        K = torch.randn(L, Hkv, D, generator=g)
        V = torch.randn(L, Hkv, D, generator=g)
        Q = torch.randn(n, Hq, D, generator=g) * 2
        if peak is not None:                                     # one far key dominates the last query
            far = peak if peak < L else 0
            K[far] = Q[-1, ::Hq // Hkv][:Hkv] * 6
        lo = 0
        if window:                                               # pages wholly behind the window are not held
            lo = max(0, (L - n) - window + 1)
            for pi in range(lo // page):
                bt[b, pi] = -1
        for t in range(lo // page * page, L):
            pg, off = pages[t // page], t % page
            k_cache[pg, :, off, :] = K[t].to(dtype)
            v_cache[pg, :, :, off] = V[t].to(dtype)
        q_rows.append(Q.reshape(n, Hq * D))
        seq_of += [b] * n
        positions += list(range(L - n, L))
        ctx.append(L); cu.append(cu[-1] + n)
    Dn = sum(1 for _, n in seqs if n == 1)
    T = cu[-1]
    # q as a strided view of a wider row, as in the engine
    wide = torch.zeros(T, Hq * D + 2 * Hkv * D, device=DEV, dtype=dtype)
    wide[:, :Hq * D] = torch.cat(q_rows).to(DEV).to(dtype)
    q = wide[:, :Hq * D]
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
    args = (q, k_cache, v_cache, page, bt.to(DEV), i32(ctx), i32(seq_of), i32(positions),
            i32([c - cu[Dn] for c in cu[Dn:]]) if Dn < B else None, Dn,
            max([L for L, n in seqs if n == 1], default=0), D ** -0.5, window, Hq, Hkv, D)
    return args


@pytest.fixture(params=[0, 1], ids=["per_wave", "through_lds"])
def prefill_form(request, monkeypatch):
    """Both forms of the prefill kernel (the launcher would choose by the size of the launch)."""
    monkeypatch.setattr(ops, "PREFILL_THROUGH_LDS", request.param)
    return request.param


SHAPES = [(4, 2, 16, 16), (6, 2, 32, 8), (4, 1, 48, 16), (16, 8, 128, 16), (8, 8, 64, 32), (32, 1, 64, 16), (2, 2, 128, 64),
          (80, 1, 32, 16),      # more heads in a group than one round of a workgroup's columns
          (40, 8, 128, 16), (64, 8, 128, 16)]      # groups of 5 and of 8 at head size 128 (Qwen3-14B and 32B)


@pytest.mark.parametrize("Hq,Hkv,D,page", SHAPES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_prefill_ragged(prefill_form, dtype, Hq, Hkv, D, page):
    """Ragged prompts, chunks that attend to earlier chunks, lengths at tile and page edges."""
    seqs = [(5, 5), (33, 33), (64, 2), (65, 33), (129, 17), (page, page), (page + 1, 2), (200, 64), (31, 31)]
    args = _attention_case(dtype, Hq, Hkv, D, page, seqs, seed=D + page)
    close(hip().paged_attention(*args), twin.paged_attention(*args), 1e-5 if dtype == torch.float32 else 1.5e-2)


@pytest.mark.parametrize("Hq,Hkv,D,page", SHAPES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_decode_batches(dtype, Hq, Hkv, D, page):
    """Decode alone (small, long, mixed lengths: one partition and many) and beside prefill rows."""
    for seqs in ([(1, 1)], [(7, 1), (130, 1), (2, 1)], [(1500, 1)], [(700, 1), (33, 1), (900, 1), (128, 1), (129, 1)],
                 [(40, 1), (300, 1), (50, 50), (90, 7), (2, 2)]):
        args = _attention_case(dtype, Hq, Hkv, D, page, seqs, seed=len(seqs))
        close(hip().paged_attention(*args), twin.paged_attention(*args), 1e-5 if dtype == torch.float32 else 1.5e-2)


@pytest.mark.parametrize("Hq,Hkv,D,page", SHAPES + [(6, 3, 80, 8), (4, 4, 256, 16)])
@pytest.mark.parametrize("window", [None, 50])
def test_decode_step_in_one_launch(Hq, Hkv, D, page, window):
    """Norms, rotation, cache write and attention of a pure decode step as one kernel, against the twins of
    the separate kernels: outputs, what the pages hold afterwards (NaN wherever nothing was written), rows
    untouched. Contexts: the new token alone, at a page's first and last place, first and last of a 32-key
    block, in the last of many partitions; a padding row (context 0) writes nothing."""
    torch.manual_seed(D + page)
    P = 3200
    ang = torch.outer(torch.arange(P, dtype=torch.float32), 1.0 / (1e4 ** (torch.arange(0, D, 2).float() / D)))
    table = torch.stack((ang.cos(), ang.sin()), -1).contiguous().to(DEV)
    qw, kw = torch.rand(D, device=DEV) + 0.5, torch.rand(D, device=DEV) + 0.5
    for lens in ([1], [page, page + 1, 2 * page], [32, 33, 64, 65, 31], [1500, 7, 3000, 700], [130] * 9):
        args = _attention_case(torch.bfloat16, Hq, Hkv, D, page, [(L, 1) for L in lens], window=window, seed=len(lens))
        q, k_cache, v_cache, _, bt, ctx = args[:6]
        rows = q._base
        rows[:, Hq * D:] = torch.randn(len(lens), 2 * Hkv * D, device=DEV).to(torch.bfloat16)
        B = len(lens)
        # a padding row behind the others: context 0, a table without pages
        rows = torch.cat((rows, torch.randn(1, rows.shape[1], device=DEV).to(torch.bfloat16)))
        bt = torch.cat((bt, torch.full((1, bt.shape[1]), -1, dtype=torch.int32, device=DEV)))
        ctx = torch.cat((ctx, torch.zeros(1, dtype=torch.int32, device=DEV)))
        for b, L in enumerate(lens):                              # the new token's place holds nothing yet
            pg = int(bt[b, (L - 1) // page])
            k_cache[pg, :, (L - 1) % page, :] = float("nan")
            v_cache[pg, :, :, (L - 1) % page] = float("nan")
        for use_norm, use_rope in ((True, True), (False, True), (True, False)):
            ka, va, kb, vb = k_cache.clone(), v_cache.clone(), k_cache.clone(), v_cache.clone()
            before = rows.clone()
            common = (qw if use_norm else None, kw if use_norm else None, 1e-6, table if use_rope else None)
            tail = (page, bt, ctx, max(lens), D ** -0.5, window, Hq, Hkv, D)
            got = hip().decode_step_attention(rows, *common, ka, va, *tail)
            want = twin.decode_step_attention(rows, *common, kb, vb, *tail)
            assert torch.equal(rows, before)
            assert torch.equal(torch.isnan(ka), torch.isnan(kb)) and torch.equal(torch.isnan(va), torch.isnan(vb))
            close(torch.nan_to_num(ka), torch.nan_to_num(kb), 4e-3)
            assert torch.equal(torch.nan_to_num(va), torch.nan_to_num(vb))
            close(got[:B], want[:B], 1.5e-2)
            assert not got[B].isnan().any()
            # and the same bits as the two launches it stands for (the q and k it forms are rounded alike)
            k2, v2, r2 = k_cache.clone(), v_cache.clone(), rows[:B].clone()
            pos = (ctx[:B] - 1)
            slots = (bt[torch.arange(B, device=DEV), (pos // page).long()] * page + pos % page).to(torch.int32)
            hip().qk_norm_rope_store(r2, *common, pos.to(torch.int32), slots, k2, v2, Hq, Hkv, D, page, True)
            two = hip().paged_attention(r2[:, :Hq * D], k2, v2, page, bt[:B], ctx[:B], torch.arange(B, dtype=torch.int32, device=DEV),
                                        pos.to(torch.int32), None, B, max(lens), D ** -0.5, window, Hq, Hkv, D)
            close(got[:B], two, 4e-3)


@pytest.mark.parametrize("Hq,Hkv,D,page", [(16, 8, 128, 16), (6, 2, 32, 8), (64, 8, 128, 16)])
def test_attention_decode_equal_contexts_in_one_partition(Hq, Hkv, D, page):
    """Equally long contexts whose workgroups fill the compute units evenly (256 of them): one partition each, no
    reduce kernel."""
    n = -(-256 // Hkv)
    seqs = [(1500 + i % 20, 1) for i in range(n)]
    assert ops.decode_partitions(n, Hq, Hkv, 1519, True)[1] == 1 and ops.decode_partitions(n, Hq, Hkv, 1519, False)[1] > 1
    args = _attention_case(torch.bfloat16, Hq, Hkv, D, page, seqs, seed=3, peak=700)
    want = twin.paged_attention(*args)
    close(hip().paged_attention(*args, even_contexts=True), want, 1.5e-2)
    close(hip().paged_attention(*args, even_contexts=False), want, 1.5e-2)


@pytest.mark.parametrize("part", [128, 160, 192, 224, 256, 288, 352, 416, 544, 704, 1088, 1408])
@pytest.mark.parametrize("window", [None, 300])
def test_attention_decode_at_every_partition_size(monkeypatch, part, window):
    """The partition sizes that `decode_partitions` chooses among (multiples of 32 keys; with 129-256 keys a wave asks
    for the keys of its two blocks at once), forced one by one: contexts that end in a partition's first block, its
    last, or exactly at its edge, a short one among them, the one key that matters in the last partition's first
    block; at two shapes of heads."""
    lens = [3000, part * 3, part * 2 + 1, part + 33, 40]
    parts = -(-max(lens) // part)
    monkeypatch.setattr(ops, "decode_partitions", lambda *a, **k: (part, parts))
    peak = (3000 - 1) // part * part + 5
    args = _attention_case(torch.bfloat16, 16, 8, 128, 16, [(L, 1) for L in lens], window=window, seed=part, peak=peak if window is None else None)
    close(hip().paged_attention(*args), twin.paged_attention(*args), 1.5e-2)
    args = _attention_case(torch.bfloat16, 6, 2, 64, 8, [(L, 1) for L in lens], window=window, seed=part + 1)
    close(hip().paged_attention(*args), twin.paged_attention(*args), 1.5e-2)
    if part in (160, 192, 256, 544):            # other head sizes, with and without the keys of two blocks ahead
        for Hq, Hkv, D, page in ((4, 1, 48, 16), (4, 4, 256, 16), (10, 2, 80, 8), (2, 2, 16, 32)):
            args = _attention_case(torch.bfloat16, Hq, Hkv, D, page, [(L, 1) for L in lens[1:]], window=window, seed=part + D)
            close(hip().paged_attention(*args), twin.paged_attention(*args), 1.5e-2)


@pytest.mark.parametrize("window", [None, 100, 1000])
def test_attention_decode_contexts_of_very_different_lengths(window):
    """One batch with contexts from 1 to 3,000 keys: the partitions are those of the longest, so most
    sequences have partitions without keys (beyond their context, or wholly before their window), whose
    workgroups write nothing and which the reduce kernel must not read. The peak key sits in the first,
    a middle and the last partition of the long sequences."""
    torch.empty(1 << 24, device=DEV).fill_(float("nan"))      # what freed memory holds is not zero
    seqs = [(3000, 1), (40, 1), (1, 1), (700, 1), (2049, 1), (128, 1), (129, 1), (2999, 1)]
    for peak in (None, 0, 1500, 2998):
        if window is not None and peak is not None and peak < 2999 - window:
            continue                                           # a peak outside the window is seen by nobody
        args = _attention_case(torch.bfloat16, 16, 8, 128, 16, seqs, window=window, seed=7, peak=peak)
        close(hip().paged_attention(*args), twin.paged_attention(*args), 1.5e-2)
    many = [(100 + 37 * i % 1900, 1) for i in range(256)]     # 2,048 workgroups: one partition, no reduce
    args = _attention_case(torch.bfloat16, 16, 8, 128, 16, many, window=window, seed=8)
    close(hip().paged_attention(*args), twin.paged_attention(*args), 1.5e-2)
    # both orders of the grid (each request on one XCD, each request spread over all) give the same bits
    for seqs in ([(2070 + i % 3, 1) for i in range(16)], [(3000, 1), (40, 1), (700, 1)], many):
        args = _attention_case(torch.bfloat16, 16, 8, 128, 16, seqs, window=window, seed=9)
        assert torch.equal(hip().paged_attention(*args, even_contexts=True), hip().paged_attention(*args, even_contexts=False))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_far_key_stands_out(prefill_form, dtype):
    """One key among hundreds gets all the weight: a kernel that drops or misplaces a block,
    a partition or a page shows an O(1) error here that random scores would average away."""
    for peak in (0, 15, 16, 255, 256, 700, 1023):
        args = _attention_case(dtype, 4, 2, 64, 16, [(1024, 1), (1024, 40)], seed=peak, peak=peak)
        close(hip().paged_attention(*args), twin.paged_attention(*args), 1e-5 if dtype == torch.float32 else 1.5e-2)


@pytest.mark.parametrize("window", [None, 1000])
def test_attention_over_very_long_contexts(prefill_form, window):
    """One request of 70,000 keys decoding (61 partitions of 1,152 keys, the most the reduce kernel merges is 64)
    and a portion of 48 tokens behind 40,000 cached ones (cut into segments): the one key that matters lies far
    back, near the start of the context when all keys are visible, near the window's far edge otherwise."""
    for seqs, peak in (([(70000, 1)], 37 if window is None else 69100), ([(40048, 48)], 40000 - 900 if window else 11)):
        args = _attention_case(torch.bfloat16, 16, 8, 128, 16, seqs, window=window, seed=5, peak=peak)
        close(hip().paged_attention(*args), twin.paged_attention(*args), 1.5e-2)
    assert ops.decode_partitions(1, 16, 8, 70000)[1] == 61


@pytest.mark.parametrize("Hq,Hkv", [(40, 8), (64, 8)])
@pytest.mark.parametrize("window", [None, 100])
def test_attention_wide_groups_at_head_size_128(prefill_form, monkeypatch, Hq, Hkv, window):
    """Groups of 5 and 8 query heads at head size 128: a far key, a window's edge and long tiles cut into
    segments, decode and prompt rows in one step."""
    seqs = [(1024, 1), (150, 1), (700, 130), (1024, 40), (33, 33)]
    for peak, seg_keys in ((None, None), (0, None), (1023 if window is None else 950, None), (600 if window is None else 1000, 96)):
        monkeypatch.setattr(ops, "PREFILL_SEGMENT_KEYS", seg_keys)
        args = _attention_case(torch.bfloat16, Hq, Hkv, 128, 16, seqs, window=window, seed=Hq, peak=peak)
        close(hip().paged_attention(*args, max_prefill_context=1024), twin.paged_attention(*args), 1.5e-2)


@pytest.mark.parametrize("Hq,Hkv,D,page", [(4, 2, 16, 16), (6, 2, 32, 8), (16, 8, 128, 16), (40, 8, 128, 16)])
@pytest.mark.parametrize("window", [None, 50])
def test_decode_rows_through_the_prefill_kernel(prefill_form, Hq, Hkv, D, page, window):
    """Two implementations of decoding cross-checked: the same step with its single-token rows sent to the
    decode kernel, and with every row sent to the prefill kernel (`decode_as_prefill`), each against the
    plain twin (the reference's `unified` mode: layers/attention.py:66-68)."""
    for seqs in ([(7, 1), (130, 1), (2, 1), (1, 1)], [(700, 1), (33, 1), (900, 1), (128, 1), (129, 1)],
                 [(40, 1), (300, 1), (50, 50), (90, 7), (2, 2)]):
        args = _attention_case(torch.bfloat16, Hq, Hkv, D, page, seqs, window=window, seed=len(seqs) + D, peak=0)
        want = twin.paged_attention(*args)
        split = hip().paged_attention(*args)
        unified = hip().paged_attention(*args, decode_as_prefill=True)
        close(split, want, 1.5e-2)
        close(unified, want, 1.5e-2)
        close(unified, split, 2e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window", [1, 7, 16, 24, 100])
def test_attention_window_edges(prefill_form, dtype, window):
    """Keys just inside and just outside the window; pages behind it are not held (-1 in the
    table, NaN in memory)."""
    seqs = [(150, 1), (33, 1), (window, 1), (window + 1, 1), (150, 40), (70, 70), (window + 5, 3)]
    for peak in (None, 150 - window, 150 - window - 1):
        args = _attention_case(dtype, 6, 2, 32, 8, seqs, window=window, seed=window, peak=peak)
        close(hip().paged_attention(*args), twin.paged_attention(*args), 1e-5 if dtype == torch.float32 else 1.5e-2)


@pytest.mark.parametrize("seg_keys", [32, 96, 256])
@pytest.mark.parametrize("Hq,Hkv,D,page", [(4, 2, 64, 16), (16, 8, 128, 16), (6, 2, 32, 8), (3, 1, 48, 32)])
def test_attention_prefill_cut_into_segments(prefill_form, monkeypatch, seg_keys, Hq, Hkv, D, page):
    """Long tiles cut into key segments run by different workgroups and merged: every segment
    count from 1 up, a segment that holds none of a wave's keys, the peak in each segment, a
    window, and a context bound that is too small (the last segment then takes the rest)."""
    monkeypatch.setattr(ops, "PREFILL_SEGMENT_KEYS", seg_keys)
    seqs = [(700, 700), (40, 40), (513, 130), (300, 2), (1000, 64)]
    for peak, window, bound in ((None, None, 1000), (0, None, 1000), (450, None, 1000), (699, None, 1000),
                                (None, 200, 1000), (600, 200, 1000), (333, None, 300), (None, None, 0)):
        args = _attention_case(torch.bfloat16, Hq, Hkv, D, page, seqs, window=window, seed=seg_keys, peak=peak)
        close(hip().paged_attention(*args, max_prefill_context=bound), twin.paged_attention(*args), 1.5e-2)


@pytest.mark.parametrize("Hq,Hkv,page", [(16, 8, 16), (64, 8, 16), (2, 2, 64), (40, 8, 256), (80, 1, 32)])
def test_attention_prefill_lds_filled_by_the_loads_themselves(monkeypatch, Hq, Hkv, page):
    """Head size 128, pages of 16 keys or more: the loads write LDS directly, three buffers deep. Same
    products in the same order as the form that stages through registers, so the results are equal bit for bit;
    against the twin as everywhere. Contexts that end inside a block and inside a page (the cache holds NaN
    wherever no key was written), one block, fewer blocks than buffers, segments, a group of 80 heads (a token's
    columns take two rounds of the workgroup), and a launch large enough for three waves to a SIMD."""
    seqs = [(5, 5), (31, 31), (32, 32), (33, 33), (64, 2), (65, 33), (97, 96), (129, 17), (page + 1, 2), (700, 700), (1000, 64)]
    # (segment size, the key that stands out, window): windows whose lower edge lies inside a block, at a block's
    # start and at a page's start, with the pages behind them given back
    for seg_keys, peak, window in ((None, None, None), (96, 450, None), (256, 3, None), (None, None, 50), (96, 690, 200),
                                   (None, 940, 64), (256, None, 17)):
        monkeypatch.setattr(ops, "PREFILL_SEGMENT_KEYS", seg_keys)
        args = _attention_case(torch.bfloat16, Hq, Hkv, 128, page, seqs, window=window, seed=page + Hq, peak=peak)
        monkeypatch.setattr(ops, "PREFILL_THROUGH_LDS", 1)
        direct = hip().paged_attention(*args, max_prefill_context=1000)
        monkeypatch.setattr(ops, "PREFILL_THROUGH_LDS", 2)
        staged = hip().paged_attention(*args, max_prefill_context=1000)
        assert not torch.isnan(direct).any() and torch.equal(direct, staged)
        close(direct, twin.paged_attention(*args), 1.5e-2)
    if Hq == 64:      # the form with three waves to a SIMD, which the engine takes for launches larger than a test's
        monkeypatch.setattr(ops, "PREFILL_SEGMENT_KEYS", 0)
        monkeypatch.setattr(ops, "prefill_waves", lambda *a: 3)
        args = _attention_case(torch.bfloat16, Hq, Hkv, 128, page, [(2100, 2100)], seed=7, peak=1500)
        monkeypatch.setattr(ops, "PREFILL_THROUGH_LDS", 1)
        direct = hip().paged_attention(*args, max_prefill_context=2100)
        monkeypatch.setattr(ops, "PREFILL_THROUGH_LDS", 2)
        assert torch.equal(direct, hip().paged_attention(*args, max_prefill_context=2100))
        close(direct, twin.paged_attention(*args), 1.5e-2)


def test_attention_prefill_segments_chosen_automatically():
    """A short chunk at the end of a long context is cut by the engine's own rule."""
    seqs = [(2500, 33), (1100, 2)]
    assert ops.prefill_segments(2500, 0, 35, 4)[1] > 1 and ops.prefill_segments(900, 0, 900, 16) == (0, 1)
    for peak in (None, 3, 1200, 2467):
        args = _attention_case(torch.bfloat16, 4, 2, 64, 16, seqs, seed=5, peak=peak)
        close(hip().paged_attention(*args, max_prefill_context=2500), twin.paged_attention(*args), 1.5e-2)


def test_attention_generic_path_takes_odd_sizes():
    """Head size 24 and page 5 are outside the matrix-core kernel: the generic kernel takes them."""
    for dtype in (torch.float32, torch.bfloat16):
        args = _attention_case(dtype, 3, 1, 24, 5, [(40, 1), (23, 23), (9, 2)], seed=1)
        close(hip().paged_attention(*args), twin.paged_attention(*args), 1e-5 if dtype == torch.float32 else 1.5e-2)
    args = _attention_case(torch.bfloat16, 4, 2, 32, 24, [(100, 1), (50, 50), (30, 3)], seed=3)   # page 24: no power of two
    close(hip().paged_attention(*args), twin.paged_attention(*args), 1.5e-2)
    args = _attention_case(torch.bfloat16, 4, 2, 64, 16, [(300, 1), (70, 70)], seed=2)
    close(hip().paged_attention(*args, force_simple=True), twin.paged_attention(*args), 1.5e-2)
    close(hip().paged_attention(*args, force_simple=True), hip().paged_attention(*args), 1.5e-2)


def test_decode_partitions_rule():
    for S, Hq, Hkv, ctx in ((1, 16, 8, 2048), (8, 16, 8, 2048), (64, 16, 8, 2304), (1, 32, 8, 100), (3, 6, 2, 130000),
                            (256, 16, 8, 4096), (256, 16, 8, 4097), (128, 16, 8, 16384)):
        part, parts = ops.decode_partitions(S, Hq, Hkv, ctx)
        assert part % 32 == 0 and part >= 128 and part * parts >= ctx and part * (parts - 1) < ctx


# ------------------------------------------------------------------------------- products

@pytest.mark.parametrize("M,N,K", [(1, 100, 72), (5, 384, 80), (64, 1000, 224), (130, 96, 200), (300, 300, 31)])
def test_linear_float32_is_exact_product(M, N, K):
    x, w = torch.randn(M, K, device=DEV), torch.randn(N, K, device=DEV)
    close(hip().linear(x, w), x.double() @ w.double().t(), 2e-6)


@pytest.mark.parametrize("M", [1, 3, 8, 16, 17, 33, 64])
@pytest.mark.parametrize("N,K", [(384, 80), (1000, 224), (3072, 1024), (1024, 3072), (100, 2048)])
def test_linear_skinny_bf16(M, N, K):
    x = torch.randn(M, K, device=DEV).bfloat16()
    w = (torch.randn(N, K, device=DEV) * 0.05).bfloat16()
    ref = x.double() @ w.double().t()
    close(hip().linear(x, w), ref, 6e-3)                       # bf16 output rounding
    close(hip().linear(x, w, torch.float32), ref, 2e-5)        # float32 output: accumulation error only
    parts = hip().linear(x, w, None, allow_partials=True)      # may be split over K
    close(parts.sum(0) if parts.dim() == 3 else parts, ref, 6e-3 if parts.dim() == 2 else 2e-5)


@pytest.mark.parametrize("M", [1, 3, 8, 16])
@pytest.mark.parametrize("N,K", [(4100, 1024), (1024, 4096), (8200, 512), (2056, 2048)])
def test_linear_skinny_wide_loads(monkeypatch, M, N, K):
    """Weights of 4 M elements or more, up to 16 rows, K in whole steps of 128: a wave's load takes 256 contiguous bytes
    of each of four rows and the pieces reach their lanes through LDS. The same bits as the plain loads give, for one
    result, partial sums over slices of K and the gating epilogue; a last workgroup with fewer than 16 rows (or 8 gate
    features); rows of x and w that are longer than K."""
    assert ops.skinny_wide(N, K) and ops.skinny_takes(M, N, K)
    torch.manual_seed(M + N)
    x = torch.randn(M, K + 64, device=DEV).bfloat16()[:, :K]
    w = (torch.randn(N, K + 128, device=DEV) * 0.05).bfloat16()[:, :K]
    ref = x.double() @ w.double().t()
    def all_forms():
        parts = hip().linear(x, w, None, allow_partials=True)
        return (hip().linear(x, w), hip().linear(x, w, torch.float32), parts, hip().gated_linear(x, w))
    wide = all_forms()
    monkeypatch.setattr(ops, "SKINNY_WIDE_MIN_WEIGHT", 1 << 40)
    plain = all_forms()
    for a, b in zip(wide, plain):
        assert a.shape == b.shape and torch.equal(a, b)
    close(wide[0], ref, 6e-3)
    close(wide[1], ref, 2e-5)
    close(wide[2].sum(0) if wide[2].dim() == 3 else wide[2], ref, 6e-3 if wide[2].dim() == 2 else 2e-5)
    assert wide[2].dim() == (3 if ops.choose_ksplit(M, N, K) > 1 else 2)
    close(wide[3], twin.gated_linear(x, w, compute_dtype=torch.float64), 6e-3)


@pytest.mark.parametrize("M", [1, 2])
@pytest.mark.parametrize("N,K", [(4096, 1024), (6144, 1024), (384, 80), (1000, 224), (100, 2048), (1536, 4096)])
@pytest.mark.parametrize("S", [0, 1, 6])
def test_norm_inside_the_skinny_product(M, N, K, S):
    """RMSNorm (+ residual, + partial sums) and the product behind it as one kernel, against the twin with
    the kernel's rounding points and against the two kernels it stands for. S = 0: bfloat16 rows without a
    residual (a model's first layer); else float32 [S, M, K] with a residual."""
    torch.manual_seed(M * 31 + S)
    w = (torch.randn(N, K, device=DEV) * 0.05).bfloat16()
    gamma = torch.rand(K, device=DEV) + 0.5
    if S == 0:
        x, res = (torch.randn(M, K, device=DEV) * 3).bfloat16(), None
    else:
        x, res = torch.randn(S, M, K, device=DEV), torch.randn(M, K, device=DEV) * 2
        x[:, 0] *= 30                                     # rows of very different size: the scale is per row
    assert ops.norm_linear_fuses(x, w)
    assert not ops.norm_linear_fuses(x[..., :1, :].expand(*x.shape[:-2], 3, K).contiguous(), w)      # three rows: two launches
    y, r = hip().norm_linear(x, res, gamma, 1e-6, w)
    want_y, want_r = twin.norm_linear(x, res, gamma, 1e-6, w)
    assert torch.equal(r, want_r) if S <= 1 else True
    close(r, want_r, 1e-6)
    close(y, want_y, 6e-3)                                 # bf16 output rounding, as for the product alone
    normed, r2 = hip().rms_norm(x, gamma, 1e-6, res, torch.bfloat16)
    assert torch.equal(r, r2)                              # the residual is summed in the same order
    two = hip().linear(normed, w)
    rows = two.float().abs().amax(dim=1, keepdim=True).clamp_min(1e-30)
    assert float(((y.float() - two.float()).abs() / rows).max()) <= 1.5e-2      # row by row: bfloat16 rounding of the operand
    y32, _ = hip().norm_linear(x, res, gamma, 1e-6, w, out_dtype=torch.float32, want_residual=False)
    # float32 output, against the exact product of the operand that the kernel's own r rounds to (a last-bit
    # difference in r can round gamma * r to the other bfloat16): accumulation error only
    exact = twin.norm_linear(r, None, gamma, 1e-6, w, out_dtype=torch.float64, compute_dtype=torch.float64)[0]
    close(y32, exact, 2e-5)


@pytest.mark.parametrize("M", [1, 2, 5, 16])
@pytest.mark.parametrize("I,K", [(3072, 1024), (224, 80), (100, 72), (1536, 4096)])
def test_gating_in_the_gate_up_products_epilogue(M, I, K):
    """silu(gate) * up formed where the packed gate/up product merges its waves (8 gate and 8 up features to a
    workgroup), against the product in float64 and against the two kernels it stands for; and the same behind
    an RMSNorm inside the product, for the one or two rows that takes."""
    torch.manual_seed(M + I)
    w = (torch.randn(2 * I, K, device=DEV) * 0.05).bfloat16()
    x = torch.randn(M, K, device=DEV).bfloat16()
    assert ops.gated_linear_fuses(x, w)
    assert ops.gated_linear_fuses(torch.randn(17, K, device=DEV).bfloat16(), w) == (ops.mid_takes(33, 2 * I, K, False) == 1)
    got = hip().gated_linear(x, w)
    assert got.shape == (M, I)
    close(got, twin.gated_linear(x, w, compute_dtype=torch.float64), 6e-3)
    close(got, hip().silu_and_mul(hip().linear(x, w)), 1.5e-2)         # those round the product before the gating
    parts, res = torch.randn(3, M, K, device=DEV), torch.randn(M, K, device=DEV)
    assert ops.norm_linear_fuses(parts, w) == (M <= 2 and 2 * I * K <= ops.NORM_FUSE_MAX_WEIGHT)
    if ops.norm_linear_fuses(parts, w):
        gamma = torch.rand(K, device=DEV) + 0.5
        y, r = hip().norm_linear(parts, res, gamma, 1e-6, w, gated=True)
        assert y.shape == (M, I)
        want = twin.norm_linear(r, None, gamma, 1e-6, w, gated=True, out_dtype=torch.float64, compute_dtype=torch.float64)[0]
        close(y, want, 6e-3)


@pytest.mark.parametrize("M", [17, 32, 33, 65, 130, 256])
@pytest.mark.parametrize("I,K", [(3072, 1024), (100, 256), (36, 320), (1000, 2048)])
def test_gating_in_the_epilogue_for_a_few_hundred_rows(M, I, K):
    """The same for 33 to 256 rows over a small weight: the tiled kernel takes 32 gate features and their 32 up features
    to a workgroup; a last tile that is partly beyond I, and an I that is no multiple of 16."""
    torch.manual_seed(M + I)
    w = (torch.randn(2 * I, K, device=DEV) * 0.05).bfloat16()
    x = torch.randn(M, K, device=DEV).bfloat16()
    if M > 32 and ops.skinny_takes(M, 2 * I, K):       # 33-64 rows over the smaller weights: the skinny kernel has the product
        assert not ops.gated_linear_fuses(x, w)
        return
    assert ops.gated_linear_fuses(x, w) and ops.mid_takes(max(M, 33), 2 * I, K, False) == 1
    got = hip().gated_linear(x, w)
    assert got.shape == (M, I)
    close(got, twin.gated_linear(x, w, compute_dtype=torch.float64), 6e-3)
    close(got, hip().silu_and_mul(hip().linear(x, w)), 1.5e-2)         # those round the product before the gating
    # one gate feature far out, so that a gate paired with another feature's up value shows
    w2 = w.clone()
    w2[I // 2] *= 40
    close(hip().gated_linear(x, w2), twin.gated_linear(x, w2, compute_dtype=torch.float64), 6e-3)


@pytest.mark.parametrize("M", [1, 8, 16, 17, 40])
@pytest.mark.parametrize("N,I", [(1024, 3072), (80, 224), (72, 200)])
def test_silu_mul_linear(M, N, I):
    """Gating fused into the down product (few rows) and the two-kernel form give the twin's result."""
    gu = (torch.randn(M, 2 * I, device=DEV) * 2).bfloat16()
    w = (torch.randn(N, I, device=DEV) * 0.05).bfloat16()
    ref = twin.silu_and_mul(gu).double() @ w.double().t()        # the gated values rounded to bf16 once, as the kernel does
    got = hip().silu_mul_linear(gu, w, allow_partials=True)
    # float32 partial sums: what remains is that a gated value next to a rounding boundary may round to
    # the other bf16 neighbour than the twin's (expf against sigmoid): 2^-8 on a few percent of the terms
    close(got.sum(0) if got.dim() == 3 else got, ref, 6e-3 if got.dim() == 2 else 1e-3)
    close(hip().silu_mul_linear(gu, w), ref, 6e-3)


def test_linear_partials_are_used_where_tiles_are_few():
    x = torch.randn(8, 3072, device=DEV).bfloat16()
    w = torch.randn(1024, 3072, device=DEV).bfloat16()
    assert hip().linear(x, w, None, allow_partials=True).dim() == 3
    assert hip().linear(x, torch.randn(9000, 3072, device=DEV).bfloat16(), None, allow_partials=True).dim() == 2
    # 320 feature tiles over a long K: four splits, so that the compute units are evenly loaded; the ring
    # path with its fetches past the end (12.5 steps of 128 per split, K not a multiple of 128)
    for M, N, K in ((3, 5120, 6408), (16, 5104, 4096)):
        x = torch.randn(M, K, device=DEV).bfloat16()
        w = (torch.randn(N, K, device=DEV) * 0.05).bfloat16()
        parts = hip().linear(x, w, None, allow_partials=True)
        assert parts.shape == (4, M, N) and parts.dtype == torch.float32
        close(parts.sum(0), x.double() @ w.double().t(), 2e-5)


@pytest.mark.parametrize("M,N,K", [(24, 4096, 4096), (17, 4100, 4104), (20, 4000, 4224), (64, 1400, 12296), (32, 1368, 12288), (9, 1000, 16904)])
def test_linear_rows_kernel(monkeypatch, M, N, K):
    """17 to 64 rows over large weights (and fewer over a very long K), partial sums allowed: 64 features per
    workgroup, the tokens staged in LDS chunk by chunk; feature counts and K that are no multiples of 64, 128 or 512.
    (The tiled kernel's slices, which take some of these shapes first, are switched off here.)"""
    from mini_engine_amd.kernels import ops
    monkeypatch.setattr(ops, "USE_MID_PRODUCT", False)
    assert ops.rows_takes(M, N, K)
    x = torch.randn(M, K, device=DEV).bfloat16()
    w = (torch.randn(N, K, device=DEV) * 0.05).bfloat16()
    parts = hip().linear(x, w, None, allow_partials=True)
    assert parts.shape == (ops.rows_ksplit(K), M, N) and parts.dtype == torch.float32
    close(parts.sum(0), x.double() @ w.double().t(), 2e-5)
    xs = torch.randn(M, K + 8, device=DEV).bfloat16()[:, :K]   # a row stride that is not K
    close(hip().linear(xs, w, None, allow_partials=True).sum(0), xs.double() @ w.double().t(), 2e-5)


@pytest.mark.parametrize("M,N,K", [(24, 4096, 4096), (20, 4100, 4096), (32, 4160, 4096), (17, 5120, 8192)])
def test_linear_rows_kernel_wide_loads(monkeypatch, M, N, K):
    """The rows kernel with the weights read 256 contiguous bytes of four rows a load and passed through LDS (up to 32
    rows, two workgroups or more to a compute unit, K in whole chunks): the same bits as with the plain loads; a last
    workgroup whose waves have few rows or none; weight rows longer than K."""
    monkeypatch.setattr(ops, "USE_MID_PRODUCT", False)          # the tiled kernel's slices take some of these shapes first
    assert ops.rows_takes(M, N, K) and ops.rows_wide(M, N, ops.rows_ksplit(K)) == 1
    x = torch.randn(M, K, device=DEV).bfloat16()
    w = (torch.randn(N, K + 64, device=DEV) * 0.05).bfloat16()[:, :K]
    wide = hip().linear(x, w, None, allow_partials=True)
    monkeypatch.setattr(ops, "rows_wide", lambda *a: 0)
    plain = hip().linear(x, w, None, allow_partials=True)
    assert wide.shape == (ops.rows_ksplit(K), M, N) and torch.equal(wide, plain)
    close(wide.sum(0), x.double() @ w.double().t(), 2e-5)


@pytest.mark.parametrize("M,N,K", [(65, 4096, 1024), (256, 6144, 1024), (130, 1024, 2048), (200, 1024, 3072), (512, 1024, 2048),
                                   (100, 1000, 320), (40, 6144, 1024), (70, 68, 256), (77, 1028, 2112)])
def test_linear_a_few_hundred_rows_over_small_weights(M, N, K):
    """33-512 rows over weights of up to 8 M elements: the own kernel with tiles of 64 x 64 whose loads write LDS
    themselves; row and feature counts that are no multiples of 64 (the last tiles read the matrix's last row again
    and store nothing for it), K a multiple of 64 only, a row stride that is not K, bfloat16 and float32 results,
    and four slices of K as float32 partial sums where the features are few and the consumer adds them."""
    from mini_engine_amd.kernels import ops
    x = torch.randn(M, K, device=DEV).bfloat16()
    w = (torch.randn(N, K, device=DEV) * 0.05).bfloat16()
    ref = x.double() @ w.double().t()
    assert ops.mid_takes(M, N, K, False) == (1 if M <= 256 else 0) and not ops.skinny_takes(M, N, K)
    if M <= 256:
        close(hip().linear(x, w), ref, 6e-3)
        close(hip().linear(x, w, torch.float32), ref, 2e-5)
        xs = torch.randn(M, K + 8, device=DEV).bfloat16()[:, :K]
        close(hip().linear(xs, w), xs.double() @ w.double().t(), 6e-3)
    parts = hip().linear(x, w, None, allow_partials=True)
    if N <= 2048 and K >= 2048:
        slices = ops.mid_takes(M, N, K, True)
        assert slices in (2, 4, 8) and parts.shape == (slices, M, N) and parts.dtype == torch.float32
        close(parts.sum(0), ref, 2e-5)
    else:
        assert parts.dim() == 2
        close(parts, ref, 6e-3)


@pytest.mark.parametrize("M,N,K,route", [(48, 1024, 2048, "mid"), (64, 2048, 2048, "mid"), (64, 2560, 9728, "mid"), (40, 2560, 9728, "mid"),
                                         (64, 2048, 6144, "mid"), (128, 2560, 4096, "mid"), (64, 2560, 4096, "mid"), (128, 4096, 4096, "mid"),
                                         (24, 2560, 9728, "mid"), (17, 4096, 4096, "mid"), (200, 2560, 9728, "slices"), (64, 4096, 12288, "slices"),
                                         (64, 5120, 5120, "slices"), (32, 4096, 12288, "rows"), (32, 6144, 2560, "plain"), (64, 4096, 2048, "plain")])
def test_linear_routes_at_the_sizes_between_the_measured_ones(M, N, K, route):
    """Products of the 1.7B, 4B layer sizes at row counts where the rules were corrected: the route the rules name
    is the one that runs, and it gives the exact product."""
    x = torch.randn(M, K, device=DEV).bfloat16()
    w = (torch.randn(N, K, device=DEV) * 0.05).bfloat16()
    ref = x.double() @ w.double().t()
    parts = hip().linear(x, w, None, allow_partials=True)
    if route == "mid":
        assert ops.mid_takes(M, N, K, True) in (2, 4, 8) and parts.shape == (ops.mid_takes(M, N, K, True), M, N)
    elif route == "rows":
        assert ops.rows_takes(M, N, K) and parts.shape == (ops.rows_ksplit(K), M, N)
    elif route == "slices":
        assert parts.shape == (ops.library_splits(M, N, K), M, N) and parts.shape[0] > 1
    else:
        assert parts.dim() == 2 and not ops.skinny_takes(M, N, K) and ops.mid_takes(M, N, K, False) == 0
    if parts.dim() == 3:
        assert parts.dtype == torch.float32
        close(parts.sum(0), ref, 2e-5)
    else:
        close(parts, ref, 6e-3)
    close(hip().linear(x, w), ref, 6e-3)


@pytest.mark.parametrize("M,N,K", [(200, 384, 80), (2048, 1024, 1024), (65, 100, 200), (70, 96, 44)])
def test_linear_large_and_odd_bf16(M, N, K):
    """Above the skinny range the library product runs; K not a multiple of 8 takes the FMA kernel."""
    x = torch.randn(M, K, device=DEV).bfloat16()
    w = (torch.randn(N, K, device=DEV) * 0.05).bfloat16()
    ref = x.double() @ w.double().t()
    close(hip().linear(x, w), ref, 6e-3)
    close(hip().linear(x, w, torch.float32), ref, 2e-5)
    xs = torch.randn(M, K + 8, device=DEV).bfloat16()[:, :K]   # a row stride that is not K
    close(hip().linear(xs, w), xs.double() @ w.double().t(), 6e-3)


@pytest.mark.parametrize("M,N,K", [(200, 384, 80), (2048, 1024, 1024), (65, 100, 200), (4, 6000, 4096), (300, 1531, 1024), (1, 152000, 1024)])
def test_library_product_is_called_directly(M, N, K):
    """The library product goes through the core library's own call of hipBLASLt (the process's copy is
    found, so no step falls back to torch's route) and agrees with the exact product: bfloat16 and float32
    outputs, a row stride that is not K, a feature count that is no multiple of 8, graph capture."""
    from mini_engine_amd.kernels import ops
    x = torch.randn(M, K, device=DEV).bfloat16()
    w = (torch.randn(N, K, device=DEV) * 0.05).bfloat16()
    ref = x.double() @ w.double().t()
    close(ops.library_product(x, w, torch.bfloat16), ref, 6e-3)
    assert ops._library_direct is True and ops._library_workspace is not None
    close(ops.library_product(x, w, torch.float32), ref, 2e-5)
    xs = torch.randn(M, K + 8, device=DEV).bfloat16()[:, :K]
    close(ops.library_product(xs, w, torch.bfloat16), xs.double() @ w.double().t(), 6e-3)
    graph, side = torch.cuda.CUDAGraph(), torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            y = ops.library_product(x, w, torch.float32)
    for _ in range(3):                        # every replay, with eager work between them
        x.copy_(torch.randn(M, K, device=DEV))
        graph.replay()
        torch.cuda.synchronize()
        close(y, x.double() @ w.double().t(), 2e-5)
        close(ops.library_product(x, w, torch.float32), x.double() @ w.double().t(), 2e-5)


@pytest.mark.parametrize("M,N,K", [(33, 4096, 12288), (256, 4096, 4096), (200, 2560, 9728), (300, 4096, 12288), (700, 5120, 8192), (200, 1368, 12288 + 64)])
def test_linear_library_slices_of_k(M, N, K):
    """o and down at 33 to 1,024 rows over large weights (where the tiled kernel's slices are not ahead): the library
    runs slices of K as one strided batch and the consumer adds the float32 partial sums."""
    from mini_engine_amd.kernels import ops
    splits = ops.library_splits(M, N, K)
    assert ops.mid_takes(M, N, K, True) == 0
    assert splits == (8 if M <= 256 else 4 if M <= 512 else 2) and K % (8 * splits) == 0
    x = torch.randn(M, K, device=DEV).bfloat16()
    w = (torch.randn(N, K, device=DEV) * 0.05).bfloat16()
    parts = hip().linear(x, w, None, allow_partials=True)
    assert parts.shape == (splits, M, N) and parts.dtype == torch.float32
    close(parts.sum(0), x.double() @ w.double().t(), 2e-5)
    xs = torch.randn(M, K + 8, device=DEV).bfloat16()[:, :K]   # a row stride that is not K
    close(hip().linear(xs, w, None, allow_partials=True).sum(0), xs.double() @ w.double().t(), 2e-5)
    # the norm that follows takes them as they are
    res = torch.randn(M, N, device=DEV)
    nw = torch.rand(N, device=DEV) + 0.5
    y, new_res = hip().rms_norm(parts, nw, 1e-6, res, torch.bfloat16)
    want_y, want_res = twin.rms_norm(parts.sum(0), nw, 1e-6, res, torch.bfloat16)
    close(new_res, want_res, 1e-6)
    close(y, want_y, 6e-3)


# ------------------------------------------------------------------------------- sampling

def test_sample_greedy_and_noise():
    S, V = 9, 1531
    logits = torch.randn(S, V, device=DEV) * 3
    keys = torch.randint(-2 ** 31, 2 ** 31 - 1, (S, 2), device=DEV, dtype=torch.int32)
    zero = torch.zeros(S, device=DEV)
    assert hip().sample(logits, zero, keys).tolist() == logits.argmax(-1).tolist()
    tie = torch.zeros(2, 50, device=DEV); tie[:, [7, 30]] = 5.0
    assert hip().sample(tie, zero[:2], keys[:2]).tolist() == [7, 7]           # first of equal maxima
    temps = torch.tensor([0.0, 0.5, 1.0, 2.0, 0.8, 0.0, 1.5, 0.1, 1.0], device=DEV)
    got = hip().sample(logits, temps, keys)
    scores = twin.sample_scores(logits, temps, keys)
    picked = scores.gather(1, got.long()[:, None])[:, 0]
    assert torch.all(picked >= scores.max(-1).values - 1e-4)                  # the twin's argmax up to float noise
    assert hip().sample(logits, temps, keys).tolist() == got.tolist()         # same keys, same tokens
    other = hip().sample(logits, temps, keys.flip(1))
    assert other[temps > 0.4].tolist() != got[temps > 0.4].tolist()


def test_sample_frequencies_follow_softmax():
    """Over many keys the exponential race picks token i with probability softmax(z/T)_i."""
    V, n, T = 12, 20000, 0.7
    z = torch.randn(V, device=DEV)
    keys = torch.stack((torch.arange(n, device=DEV, dtype=torch.int32), torch.full((n,), 12345, device=DEV, dtype=torch.int32)), 1)
    got = hip().sample(z.expand(n, V).contiguous(), torch.full((n,), T, device=DEV), keys)
    freq = torch.bincount(got.long(), minlength=V).double().cpu() / n
    p = torch.softmax(z.double().cpu() / T, 0)
    chi2 = float((n * (freq - p) ** 2 / p).sum())
    assert chi2 < 40.0, f"chi-square {chi2:.1f} with 11 degrees of freedom"   # p < 1e-4 under the null


def test_kernels_allocate_nothing_beside_their_results(monkeypatch):
    """The kernels' own scratch memory (partial results of split decode attention, of prefill attention cut into
    segments, of the sampler's chunks) is kept between calls or lives in the library: once a shape has run, a call
    asks the allocator for its result and nothing else."""
    def allocations(fn):
        fn()                                                  # the first call of a shape may size the kept buffers
        torch.cuda.synchronize()
        before = torch.cuda.memory_stats()["allocation.all.allocated"]
        out = fn()
        torch.cuda.synchronize()
        return torch.cuda.memory_stats()["allocation.all.allocated"] - before, out

    logits = torch.randn(40, 20011, device=DEV)
    temps = torch.full((40,), 0.7, device=DEV)
    keys = torch.randint(-2 ** 31, 2 ** 31 - 1, (40, 2), device=DEV, dtype=torch.int32)
    n, tokens = allocations(lambda: hip().sample(logits, temps, keys))
    assert n == 1 and tokens.shape == (40,)
    big = torch.randn(1030, 300, device=DEV)                  # more rows than the library's array holds: the kept buffer
    no_noise, same_keys = torch.zeros(1030, device=DEV), keys[:1].expand(1030, 2).contiguous()
    n, tokens = allocations(lambda: hip().sample(big, no_noise, same_keys))
    assert n == 1 and tokens.tolist() == big.argmax(-1).tolist()
    # prefill attention cut into segments, decode attention in partitions, both in one step
    monkeypatch.setattr(ops, "PREFILL_SEGMENT_KEYS", 64)
    args = _attention_case(torch.bfloat16, 16, 8, 128, 16, [(700, 1), (300, 1), (400, 130), (90, 7)], seed=5)
    assert ops.decode_partitions(2, 16, 8, 700)[1] > 1 and ops.prefill_segments(400, 0, 137, 16)[1] > 1
    n, out = allocations(lambda: hip().paged_attention(*args))
    assert n == 1
    close(out, twin.paged_attention(*args), 1.5e-2)


def test_kernels_refuse_what_they_cannot_do():
    with pytest.raises(ops.KernelError, match="dtype"):
        hip().silu_and_mul(torch.zeros(2, 4, device=DEV, dtype=torch.float16))
    with pytest.raises(ops.KernelError):
        hip().linear(torch.zeros(2, 8, device=DEV), torch.zeros(4, 8, device=DEV).bfloat16())
    with pytest.raises(ops.KernelError, match="head_dim"):
        hip().qk_norm_rope_store(torch.zeros(1, 3 * 600, device=DEV), None, None, 0.0, None,
                                 torch.zeros(1, device=DEV, dtype=torch.int32), torch.zeros(1, device=DEV, dtype=torch.int32),
                                 torch.zeros(1, 1, 4, 600, device=DEV), torch.zeros(1, 1, 600, 4, device=DEV), 1, 1, 600, 4, True)

"""Plain torch twins of every kernel: same arguments and cache layout, straightforward math.

Two uses: (1) each HIP kernel is compared with its twin on the GPU; (2) installed as the
ops backend (`PlainBackend`) they let the engine's bookkeeping (step function, cache manager,
scheduler, replay) be exercised on a machine without a GPU. They are test code: the engine
itself has no implementation but the HIP kernels.

All arithmetic is float32 (or float64 where a test asks), whatever the storage dtype; results
are rounded once to the output dtype.
"""
from __future__ import annotations

import torch


def gather_rows(src, idx):
    return src[idx.long()].clone()


def take_tokens(tokens, sampled, take):
    chosen = take.long() >= 0
    tokens[chosen] = sampled[take.long()[chosen]].to(tokens.dtype)


def rms_norm(x, weight, eps, residual, out_dtype, want_residual=True):
    r = x.float().sum(0) if x.dim() == 3 else x.float()
    if residual is not None:
        r = r + residual
    y = weight * (r * torch.rsqrt(r.pow(2).mean(-1, keepdim=True) + eps))
    return y.to(out_dtype), (r if want_residual else None)


def silu_and_mul(gu):
    inter = gu.shape[1] // 2
    g, u = gu[:, :inter].float(), gu[:, inter:].float()
    return (g * torch.sigmoid(g) * u).to(gu.dtype)


def _norm_rope(x, w, eps, table, positions):
    """x: [T, H, D] float32."""
    if w is not None:
        x = w * (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps))
    if table is not None:
        cs = table[positions.long()]                        # [T, D/2, 2]
        c, s = cs[..., 0].unsqueeze(1), cs[..., 1].unsqueeze(1)
        half = x.shape[-1] // 2
        x1, x2 = x[..., :half], x[..., half:]
        x = torch.cat((x1 * c - x2 * s, x2 * c + x1 * s), dim=-1)
    return x


def write_pages(k, v, slots, k_cache, v_cache, page):
    """k, v: [T, Hkv, D] -> K [pages, Hkv, page, D], V [pages, Hkv, D, page]."""
    keep = slots >= 0
    s = slots[keep].long()
    pg, off = s // page, s % page
    k_cache[pg, :, off, :] = k[keep].to(k_cache.dtype)
    v_cache[pg, :, :, off] = v[keep].to(v_cache.dtype)


def qk_norm_rope_store(qkv, q_weight, k_weight, eps, table, positions, slots, k_cache, v_cache,
                       Hq, Hkv, D, page, store=True, position_bound=0):
    T = qkv.shape[0]
    if table is not None:
        # what the kernel's launcher refuses, and what it could not see: a position beyond the table
        assert position_bound <= table.shape[0], f"position bound {position_bound} beyond the table's {table.shape[0]} rows"
        assert T == 0 or int(positions[:T].max()) < table.shape[0], "a position beyond the rotation table"
    q = _norm_rope(qkv[:, :Hq * D].float().clone().view(T, Hq, D), q_weight, eps, table, positions)
    if Hkv:
        k = _norm_rope(qkv[:, Hq * D:(Hq + Hkv) * D].float().clone().view(T, Hkv, D), k_weight, eps, table, positions)
    qkv[:, :Hq * D] = q.reshape(T, Hq * D).to(qkv.dtype)
    if store:
        v = qkv[:, (Hq + Hkv) * D:].view(T, Hkv, D)
        write_pages(k.to(qkv.dtype), v, slots, k_cache, v_cache, page)
    elif Hkv:
        qkv[:, Hq * D:(Hq + Hkv) * D] = k.reshape(T, Hkv * D).to(qkv.dtype)


def store_kv(k, v, slots, k_cache, v_cache, page):
    write_pages(k, v, slots, k_cache, v_cache, page)


def paged_attention(q, k_cache, v_cache, page, block_tables, context_lens, seq_of_token, positions,
                    prefill_cu, num_decodes, max_decode_context, scale, window, Hq, Hkv, D,
                    force_simple=False, max_prefill_context=0, even_contexts=False, compute_dtype=torch.float32):
    """Token by token: gather the keys this token may see through its request's block table
    and nothing else (so unowned pages are never read), softmax, weighted sum."""
    T = q.shape[0]
    out = torch.empty((T, Hq * D), dtype=q.dtype, device=q.device)
    G = Hq // Hkv
    seqs, where, lens = seq_of_token[:T].tolist(), positions[:T].tolist(), context_lens.tolist()      # one trip to the host
    for t in range(T):
        b, pos = seqs[t], where[t]
        lo = max(0, pos - window + 1) if window else 0
        hi = min(pos + 1, lens[b])                         # a padding row (context 0) sees nothing
        if hi <= lo:
            out[t] = 0
            continue
        js = torch.arange(lo, hi, device=q.device)
        pages = block_tables[b, (js // page).long()].long()
        assert (pages >= 0).all(), "attention would read a page the request does not hold"
        offs = js % page
        k = k_cache[pages, :, offs, :].to(compute_dtype)             # [n, Hkv, D]
        v = v_cache[pages, :, :, offs].to(compute_dtype)             # [n, Hkv, D]
        qt = q[t].to(compute_dtype).view(Hkv, G, D)                  # query head h belongs to key head h // G
        s = torch.einsum("nkd,kgd->kgn", k, qt) * scale
        p = torch.softmax(s, dim=-1)
        out[t] = torch.einsum("kgn,nkd->kgd", p, v).reshape(Hq * D).to(q.dtype)
    return out


def decode_step_attention(qkv, q_weight, k_weight, eps, table, k_cache, v_cache, page, block_tables, context_lens,
                          max_context, scale, window, Hq, Hkv, D, even_contexts=False, compute_dtype=torch.float32):
    """The two twins above, one after the other, on a copy of the rows: row r is request r's new token at
    position context_lens[r] - 1, its slot is what the block table names for that position (a row with
    context 0 is padding: nothing is written for it and it sees nothing)."""
    B = qkv.shape[0]
    assert table is None or max_context <= table.shape[0], f"a context of {max_context} beyond the table's {table.shape[0]} rows"
    ctx = context_lens[:B].long()
    positions = (ctx - 1).clamp(min=0).to(torch.int32)
    pages = block_tables[torch.arange(B, device=qkv.device), (positions // page).long()].long()
    slots = torch.where((ctx > 0) & (pages >= 0), pages * page + positions.long() % page, torch.full_like(pages, -1)).to(torch.int32)
    rows = qkv.clone()
    qk_norm_rope_store(rows, q_weight, k_weight, eps, table, positions, slots, k_cache, v_cache, Hq, Hkv, D, page, store=True)
    seq = torch.arange(B, dtype=torch.int32, device=qkv.device)
    return paged_attention(rows[:, :Hq * D], k_cache, v_cache, page, block_tables, context_lens, seq, positions, None, B,
                           max_context, scale, window, Hq, Hkv, D, compute_dtype=compute_dtype)


def linear(x, w, out_dtype=None, allow_partials=False, out=None):
    y = (x.float() @ w.float().t()).to(out_dtype or x.dtype)
    if out is not None:
        out.copy_(y)
        return out
    return y


def _gate(y):
    """silu(first half of the columns) * second half, on unrounded sums."""
    inter = y.shape[1] // 2
    return y[:, :inter] * torch.sigmoid(y[:, :inter]) * y[:, inter:]


def gated_linear(x, w, compute_dtype=torch.float32):
    return _gate(x.to(compute_dtype) @ w.to(compute_dtype).t()).to(x.dtype)


def norm_linear(x, residual, norm_weight, eps, w, out_dtype=None, want_residual=True, gated=False, compute_dtype=torch.float32):
    """The fused kernel's rounding points: gamma * r to the weight's dtype, product, then 1 / rms(r)."""
    r = x.float().sum(0) if x.dim() == 3 else x.float()
    if residual is not None:
        r = r + residual
    inv = torch.rsqrt(r.to(compute_dtype).pow(2).mean(-1, keepdim=True) + eps)
    y = ((norm_weight * r).to(w.dtype).to(compute_dtype) @ w.to(compute_dtype).t()) * inv
    if gated:
        y = _gate(y)
    return y.to(out_dtype or w.dtype), (r if want_residual else None)


def silu_mul_linear(gu, w, allow_partials=False):
    return linear(silu_and_mul(gu), w)


def _fmix32(h):
    m = 0xFFFFFFFF
    h = h & m
    h ^= h >> 16
    h = (h * 0x85EBCA6B) & m
    h ^= h >> 13
    h = (h * 0xC2B2AE35) & m
    h ^= h >> 16
    return h


def row_key(seed, stream, index):
    """The two 32-bit words that key the noise of output number `index` of the request with noise stream
    `stream` under `seed`: three rounds of SplitMix64's output function (add the golden-ratio constant, two
    xor-shift-multiplies, a last xor-shift), each taking the next of (seed, stream, index) xored into the state;
    (low word, high word) of the result. Written with numpy's wrapping 64-bit integers."""
    import numpy as np
    u = np.uint64

    def mix(x):
        with np.errstate(over="ignore"):
            x = x + u(0x9E3779B97F4A7C15)
            x = (x ^ (x >> u(30))) * u(0xBF58476D1CE4E5B9)
            x = (x ^ (x >> u(27))) * u(0x94D049BB133111EB)
        return x ^ (x >> u(31))

    x = mix(u(seed % (1 << 64)))
    x = mix(x ^ u(stream % (1 << 64)))
    x = mix(x ^ u(index % (1 << 64)))
    return int(x & u(0xFFFFFFFF)), int(x >> u(32))


def exp_noise(keys, V, device):
    """E ~ Exp(1), [S, V], the kernel's hash: fmix32(fmix32(v ^ k0) + k1) -> 24 bits -> -log(u)."""
    k = keys.to(torch.int64) & 0xFFFFFFFF
    v = torch.arange(V, dtype=torch.int64, device=device)[None, :]
    r = _fmix32((_fmix32(v ^ k[:, 0:1]) + k[:, 1:2]) & 0xFFFFFFFF)
    u = ((r >> 8).to(torch.float32) + 0.5) * (1.0 / 16777216.0)
    return -torch.log(u)


def sample_scores(logits, temperatures, keys):
    """The quantity whose argmax the sampler returns, [S, V] float32."""
    t = temperatures[:, None]
    noisy = logits / torch.where(t > 0, t, torch.ones_like(t)) - torch.log(exp_noise(keys, logits.shape[1], logits.device))
    return torch.where(t > 0, noisy, logits)


def sample(logits, temperatures, keys):
    return sample_scores(logits, temperatures, keys).argmax(dim=-1).to(torch.int32)


class PlainBackend:
    name = "plain"
    gather_rows = staticmethod(gather_rows)
    take_tokens = staticmethod(take_tokens)
    rms_norm = staticmethod(rms_norm)
    silu_and_mul = staticmethod(silu_and_mul)
    qk_norm_rope_store = staticmethod(qk_norm_rope_store)
    store_kv = staticmethod(store_kv)
    paged_attention = staticmethod(paged_attention)
    decode_step_attention = staticmethod(decode_step_attention)
    linear = staticmethod(linear)
    silu_mul_linear = staticmethod(silu_mul_linear)
    norm_linear = staticmethod(norm_linear)
    gated_linear = staticmethod(gated_linear)
    sample = staticmethod(sample)

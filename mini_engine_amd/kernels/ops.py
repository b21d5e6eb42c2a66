"""The engine's operations: thin, checked calls into the HIP libraries.

Every function takes torch tensors on the GPU, checks on the host what the
kernel assumes about shapes, strides and dtypes, and launches on torch's current
stream. There is no other implementation behind these names: without a GPU or
without the built library a call raises. (Tests may install another backend with
`set_backend` to exercise the engine's bookkeeping on a machine without a GPU.)

Reference counterparts: layers/ops.py:23-57 (attention/cache bindings and the
v1/v2 decode dispatcher), and the eager torch ops named in each docstring.
"""
from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_float, c_int, c_int64, c_void_p

import torch

from . import build

ME_BF16, ME_F32 = 0, 1
_DT = {torch.bfloat16: ME_BF16, torch.float32: ME_F32}


class KernelError(RuntimeError):
    pass


def _code(dtype: torch.dtype) -> int:
    try:
        return _DT[dtype]
    except KeyError:
        raise KernelError(f"unsupported dtype {dtype}; the kernels take bfloat16 and float32") from None


# --------------------------------------------------------------------------- libraries

class _Lib:
    def __init__(self, path: str, protos: dict):
        self.path = path
        self.cdll = ctypes.CDLL(path)
        self.cdll.me_last_error.restype = c_char_p
        self.fns = {}
        for name, argtypes in protos.items():
            fn = getattr(self.cdll, name)
            fn.argtypes = argtypes
            fn.restype = c_int
            self.fns[name] = fn
        self.protos = protos

    def call(self, name: str, *args):
        if self.fns[name](*args) != 0:
            raise KernelError(f"{name}: {self.cdll.me_last_error().decode()}")


P, I, L, F = c_void_p, c_int, c_int64, c_float
_CORE_PROTOS = {
    "me_gather_rows": [P, P, P, L, L, L, P],
    "me_take_tokens": [P, P, P, I, I, P],
    "me_rms_norm": [P, I, I, L, P, P, P, P, I, L, I, F, P],
    "me_silu_and_mul": [P, P, I, L, I, P],
    "me_qk_norm_rope_store": [P, I, L, L, P, P, F, P, L, L, P, P, P, P, I, I, I, I, I, P],
    "me_store_kv": [P, P, I, L, L, L, P, P, P, I, I, I, P],
    "me_attn_simple": [P, L, P, L, I, P, P, P, I, P, P, P, L, I, I, I, I, F, I, P],
    "me_gemm_tiled": [P, L, P, L, P, L, I, I, I, I, I, P],
    "me_gemm_skinny_bf16": [P, L, P, L, P, L, I, P, I, I, I, I, I, I, I, P],
    "me_gemm_rows_bf16": [P, L, P, L, P, L, I, P, I, I, I, I, I, P],
    "me_gemm_skinny_norm_bf16": [P, I, I, P, P, P, F, P, L, P, L, I, I, I, I, I, P],
    "me_gemm_mid_bf16": [P, L, P, L, P, L, I, I, I, I, I, I, P],
    "me_gemm_library_bf16": [P, L, P, L, P, L, I, P, ctypes.c_size_t, I, I, I, I, P],
    "me_sample": [P, L, P, P, P, P, I, I, P],
    "me_sample_static": [P, L, P, P, P, I, I, P],
}
_ATTN_PROTOS = {
    "me_attn_prefill": [P, L, P, L, P, P, P, I, P, P, I, L, I, I, I, F, I, I, I, I, I, I, P, P, I, P],
    "me_attn_decode": [P, L, P, L, P, P, P, I, P, I, I, I, I, F, I, I, I, P, I, P],
    "me_attn_decode_fused": [P, L, P, L, P, P, F, P, I, P, P, P, I, P, I, I, I, I, I, F, I, I, I, P, I, P],
}

_core: _Lib | None = None
_attn: dict = {}


def _require_gpu() -> None:
    if not torch.cuda.is_available():
        raise KernelError("mini_engine_amd needs an AMD GPU (gfx950): torch.cuda.is_available() is False "
                          "and there is no CPU implementation")


def core() -> _Lib:
    global _core
    if _core is None:
        _require_gpu()
        _core = _Lib(build.core_library(), _CORE_PROTOS)
    return _core


def attn_lib(head_dim: int) -> _Lib:
    lib = _attn.get(head_dim)
    if lib is None:
        _require_gpu()
        lib = _Lib(build.attention_library(head_dim), _ATTN_PROTOS)
        lib.cdll.me_attn_head_dim.restype = c_int
        if lib.cdll.me_attn_head_dim() != head_dim:
            raise KernelError(f"{lib.path} was built for head size {lib.cdll.me_attn_head_dim()}, not {head_dim}")
        _attn[head_dim] = lib
    return lib


def loaded_libraries() -> list:
    return ([_core.path] if _core else []) + [l.path for l in _attn.values()]


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_device_index: int | None = None


def _stream() -> int:
    """The handle of torch's current stream (also inside a graph capture, which runs on a stream of its
    own). Asked for at every launch, so through the short way where torch offers it."""
    global _device_index
    if _raw_stream is None:
        return torch.cuda.current_stream().cuda_stream
    if _device_index is None:
        _device_index = torch.cuda.current_device()
    return _raw_stream(_device_index)


def _ptr(t: torch.Tensor | None) -> int | None:
    return None if t is None else t.data_ptr()


def _check(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelError(msg)


def _is_i32(t: torch.Tensor, n: int | None = None) -> bool:
    return t.dtype == torch.int32 and t.is_contiguous() and (n is None or t.numel() >= n)


# --------------------------------------------------------------------------- the HIP backend

LIBRARY_WORKSPACE_BYTES = 64 << 20
_library_workspace: torch.Tensor | None = None
_library_direct: bool | None = None      # None: not asked yet


def library_is_direct() -> bool:
    """Whether the core library found a hipBLASLt in the process that it can call itself. Without a GPU
    (the dispatch rules are also asked on their own) the answer is yes, as on every GPU box."""
    global _library_direct
    if _library_direct is None:
        if not torch.cuda.is_available():
            return True
        core().cdll.me_gemm_library_available.restype = c_int
        _library_direct = bool(core().cdll.me_gemm_library_available())
    return _library_direct


def library_product(x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype, splits: int = 1,
                    out: torch.Tensor | None = None) -> torch.Tensor:
    """x [M, K] . w[N, K]^T through hipBLASLt, bfloat16 operands, float32 accumulation (reference
    layers/linear.py:25-26: its F.linear is a library product too).

    Called through the core library, which keeps the descriptors and the chosen algorithm of every
    shape, so a call costs a few microseconds of host time; torch's own route to the same library
    kernel costs several times that for every call, which is what bounds steps that are not replayed
    from a graph. torch's route stays as the way out when the process holds no hipBLASLt that the core
    library can find, or when it offers nothing for a shape. The workspace is allocated once, outside
    any graph capture (the first product of a process is never a captured one: a step runs eagerly
    before it is captured).

    splits > 1: K is cut in that many equal slices, computed as one strided batch; the result is their
    float32 partial sums [splits, M, N] for a consumer that adds them, or None where only torch's
    route is open (the caller then takes its other path)."""
    global _library_workspace
    if library_is_direct() and _library_workspace is None and not torch.cuda.is_current_stream_capturing():
        _library_workspace = torch.empty(LIBRARY_WORKSPACE_BYTES, dtype=torch.uint8, device=x.device)
    if _library_direct and _library_workspace is not None:
        M, K = x.shape
        N = w.shape[0]
        y = out if out is not None else torch.empty((M, N) if splits == 1 else (splits, M, N), dtype=out_dtype, device=x.device)
        rc = core().fns["me_gemm_library_bf16"](x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0), y.data_ptr(), N,
                                               _code(out_dtype), _library_workspace.data_ptr(),
                                               LIBRARY_WORKSPACE_BYTES, M, N, K, splits, _stream())
        if rc == 0:
            return y
        if rc != -3:
            raise KernelError(f"me_gemm_library_bf16: {core().cdll.me_last_error().decode()}")
    if splits > 1:
        return None                 # partial sums over slices of K only through the direct call
    y = torch.mm(x, w.t(), out_dtype=torch.float32) if out_dtype == torch.float32 else torch.matmul(x, w.t())
    if out is not None:
        out.copy_(y)
        return out
    return y


class HipBackend:
    """Each method is one kernel (or one dispatch among kernels of the same meaning)."""

    name = "hip"

    # -- rows ----------------------------------------------------------------------------
    def gather_rows(self, src: torch.Tensor, idx: torch.Tensor) -> torch.Tensor:
        """out[r] = src[idx[r]] (embedding lookup: reference layers/embed_head.py:10-11;
        rows that want logits: layers/embed_head.py:20-22)."""
        _check(src.dim() == 2 and src.is_contiguous(), "gather_rows: source must be a contiguous matrix")
        _check(_is_i32(idx) and idx.dim() == 1, "gather_rows: indices must be int32 [n]")
        out = torch.empty((idx.numel(), src.shape[1]), dtype=src.dtype, device=src.device)
        core().call("me_gather_rows", src.data_ptr(), idx.data_ptr(), out.data_ptr(), idx.numel(),
                    src.shape[1] * src.element_size(), src.shape[0], _stream())
        return out

    def take_tokens(self, tokens: torch.Tensor, sampled: torch.Tensor, take: torch.Tensor) -> None:
        """tokens[r] = sampled[take[r]] where take[r] >= 0, in place (int32 [R], [S], [R]): the tokens of the last
        sampling call go into the rows of a step launched before they have reached the host."""
        R = tokens.numel()
        _check(_is_i32(tokens) and _is_i32(sampled) and _is_i32(take, R), "take_tokens: int32 tensors, one source row per token row")
        core().call("me_take_tokens", tokens.data_ptr(), sampled.data_ptr(), take.data_ptr(), R, sampled.numel(), _stream())

    # -- norm ----------------------------------------------------------------------------
    def rms_norm(self, x: torch.Tensor, weight: torch.Tensor, eps: float, residual: torch.Tensor | None,
                 out_dtype: torch.dtype, want_residual: bool = True):
        """y = w * r * rsqrt(mean(r^2) + eps), r = x (+ residual) in float32 (reference
        layers/layernorm.py:11-24). x: [T, n], or float32 partial sums [P, T, n] that are added
        first. Returns (y [T, n] in out_dtype, r [T, n] float32 or None)."""
        parts = 1
        if x.dim() == 3:
            parts = x.shape[0]
            _check(x.dtype == torch.float32, "rms_norm: stacked partial sums must be float32")
        _check(x.is_contiguous(), "rms_norm: x must be contiguous")
        T, n = x.shape[-2], x.shape[-1]
        _check(weight.dtype == torch.float32 and weight.shape == (n,) and weight.is_contiguous(),
               "rms_norm: weight must be float32 [n]")
        if residual is not None:
            _check(residual.dtype == torch.float32 and residual.shape == (T, n) and residual.is_contiguous(),
                   "rms_norm: residual must be contiguous float32 [T, n]")
        y = torch.empty((T, n), dtype=out_dtype, device=x.device)
        res_out = torch.empty((T, n), dtype=torch.float32, device=x.device) if want_residual else None
        core().call("me_rms_norm", x.data_ptr(), _code(x.dtype), parts, T * n, _ptr(residual), _ptr(res_out),
                    weight.data_ptr(), y.data_ptr(), _code(out_dtype), T, n, float(eps), _stream())
        return y, res_out

    # -- feed-forward activation ---------------------------------------------------------
    def silu_and_mul(self, gu: torch.Tensor) -> torch.Tensor:
        """silu(gu[:, :I]) * gu[:, I:] (reference layers/activation.py:5-7)."""
        _check(gu.dim() == 2 and gu.is_contiguous() and gu.shape[1] % 2 == 0, "silu_and_mul: [T, 2I] contiguous")
        inter = gu.shape[1] // 2
        out = torch.empty((gu.shape[0], inter), dtype=gu.dtype, device=gu.device)
        core().call("me_silu_and_mul", gu.data_ptr(), out.data_ptr(), _code(gu.dtype), gu.shape[0], inter, _stream())
        return out

    # -- q/k norm + rotary + cache write -------------------------------------------------
    def qk_norm_rope_store(self, qkv, q_weight, k_weight, eps, table, positions, slots, k_cache, v_cache,
                           Hq: int, Hkv: int, D: int, page: int, store: bool = True, position_bound: int = 0) -> None:
        """In place on packed rows: per-head RMSNorm of q and k (weights float32 [D] or None), then
        rotary by `table` [P, D/2, 2] float32 (or None), q written back. `position_bound`: every position
        of the step is below it (the longest context the step's layout allows; 0: not told); a bound beyond
        the table's rows is refused.

        store=True: rows are [T, (Hq+2Hkv)*D]; k and v are scattered to the pages at `slots`
        (slots < 0 skipped). store=False: rows are [T, (Hq+Hkv)*D] (Hkv may be 0); k is written
        back in place and nothing is cached. (reference models/qwen3.py:34-36,
        layers/rotary_embedding.py:20-25, csrc/kv_cache.cu:10-31.)"""
        T = qkv.shape[0]
        width = (Hq + (2 * Hkv if store else Hkv)) * D
        _check(qkv.dim() == 2 and qkv.stride(1) == 1 and qkv.shape[1] == width,
               f"qk_norm_rope_store: rows must be [T, {width}] with unit inner stride, got {tuple(qkv.shape)}")
        for w in (q_weight, k_weight):
            _check(w is None or (w.dtype == torch.float32 and w.shape == (D,) and w.is_contiguous()),
                   "qk_norm_rope_store: norm weights must be float32 [D]")
        _check((q_weight is None) == (k_weight is None), "qk_norm_rope_store: give both norm weights or neither")
        if table is not None:
            _check(table.dtype == torch.float32 and table.is_contiguous() and table.shape[1:] == (D // 2, 2),
                   "qk_norm_rope_store: rotary table must be float32 [P, D/2, 2]")
        _check(_is_i32(positions, T), "qk_norm_rope_store: positions must be int32 [T]")
        if store:
            _check(_is_i32(slots, T), "qk_norm_rope_store: slots must be int32 [T]")
            _check(k_cache.dtype == qkv.dtype and v_cache.dtype == qkv.dtype and k_cache.is_contiguous()
                   and v_cache.is_contiguous(), "qk_norm_rope_store: caches must be contiguous and of the rows' dtype")
            _check(k_cache.shape[1:] == (Hkv, page, D) and v_cache.shape[1:] == (Hkv, D, page),
                   "qk_norm_rope_store: caches must be K [pages, Hkv, page, D] and V [pages, Hkv, D, page]")
        core().call("me_qk_norm_rope_store", qkv.data_ptr(), _code(qkv.dtype), T, qkv.stride(0), _ptr(q_weight),
                    _ptr(k_weight), float(eps), _ptr(table), 0 if table is None else table.shape[0], int(position_bound),
                    positions.data_ptr(), _ptr(slots) if store else None, _ptr(k_cache) if store else None,
                    _ptr(v_cache) if store else None, Hq, Hkv, D, page, int(store), _stream())

    def store_kv(self, k, v, slots, k_cache, v_cache, page: int) -> None:
        """Scatter k, v [T, Hkv, D] (views with a token stride are fine) into the pages; slots < 0
        are skipped (reference csrc/kv_cache.cu:10-31; the copy is bit-exact)."""
        T, Hkv, D = k.shape
        _check(v.shape == k.shape and k.dtype == v.dtype == k_cache.dtype == v_cache.dtype, "store_kv: dtype/shape mismatch")
        for t in (k, v):
            _check(t.stride(2) == 1 and t.stride(1) == D, "store_kv: heads of a token must be one contiguous row")
        _check(k_cache.shape[1:] == (Hkv, page, D) and v_cache.shape[1:] == (Hkv, D, page) and k_cache.is_contiguous()
               and v_cache.is_contiguous(), "store_kv: caches must be K [pages, Hkv, page, D], V [pages, Hkv, D, page]")
        _check(_is_i32(slots, T), "store_kv: slots must be int32 [T]")
        core().call("me_store_kv", k.data_ptr(), v.data_ptr(), _code(k.dtype), T, k.stride(0), v.stride(0),
                    slots.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), Hkv, D, page, _stream())

    # -- attention -----------------------------------------------------------------------
    def paged_attention(self, q, k_cache, v_cache, page: int, block_tables, context_lens, seq_of_token,
                        positions, prefill_cu, num_decodes: int, max_decode_context: int, scale: float,
                        window: int | None, Hq: int, Hkv: int, D: int, force_simple: bool = False,
                        max_prefill_context: int = 0, even_contexts: bool = False, decode_as_prefill: bool = False):
        """Causal attention of this step's tokens over the paged keys of their requests.

        q: [T, Hq*D] (a strided view is fine). Rows are ordered decode requests first (one token
        each, `num_decodes` of them), then the others; `prefill_cu` int32 [B - num_decodes + 1]
        are prefix sums of the new-token counts of the others. `context_lens` int32 [B] counts keys
        after this step's write; `block_tables` int32 [B, MB]. `max_prefill_context`: the largest
        context among the others (a hint for cutting long key ranges; 0 = unknown). `even_contexts`: the
        decode requests' contexts are equally long (decode_contexts_even), which lets the decode kernel
        keep each request on one XCD. `decode_as_prefill` (or the module's DECODE_AS_PREFILL): the
        single-token rows go through the prefill kernel too, as prompts of one token: a second
        implementation of decoding to check the first against. Returns [T, Hq*D].
        (reference layers/attention.py:63-76: decode rows to the decode kernel, the rest to the
        prefill kernel, or all rows to the prefill kernel in its `unified` mode; csrc/paged_decode.cu,
        csrc/paged_prefill.cu.)"""
        T = q.shape[0]
        B = context_lens.numel()
        _check(q.dim() == 2 and q.shape[1] == Hq * D and q.stride(1) == 1, "attention: q must be [T, Hq*D], unit inner stride")
        _check(k_cache.shape[1:] == (Hkv, page, D) and v_cache.shape[1:] == (Hkv, D, page), "attention: cache layout mismatch")
        _check(k_cache.dtype == q.dtype and v_cache.dtype == q.dtype, "attention: cache dtype differs from q")
        _check(block_tables.dim() == 2 and block_tables.dtype == torch.int32 and block_tables.stride(1) == 1
               and block_tables.shape[0] >= B, "attention: block tables must be int32 [B, MB]")
        _check(_is_i32(context_lens) and _is_i32(seq_of_token, T) and _is_i32(positions, T), "attention: metadata must be int32")
        _check(0 <= num_decodes <= B and num_decodes <= T, "attention: bad decode count")
        out = torch.empty((T, Hq * D), dtype=q.dtype, device=q.device)
        win = int(window or 0)
        mfma = (q.dtype == torch.bfloat16 and D % 16 == 0 and 16 <= D <= 512 and page >= 8 and page & (page - 1) == 0
                and not force_simple)
        if not mfma:
            core().call("me_attn_simple", q.data_ptr(), q.stride(0), out.data_ptr(), out.stride(0), _code(q.dtype),
                        k_cache.data_ptr(), v_cache.data_ptr(), block_tables.data_ptr(), block_tables.stride(0),
                        seq_of_token.data_ptr(), positions.data_ptr(), context_lens.data_ptr(), T, Hq, Hkv, D, page,
                        float(scale), win, _stream())
            return out
        lib = attn_lib(D)
        es = q.element_size()
        if (decode_as_prefill or DECODE_AS_PREFILL) and num_decodes > 0:
            ones = torch.arange(num_decodes + 1, dtype=torch.int32, device=q.device)
            prefill_cu = ones if prefill_cu is None else torch.cat((ones[:-1], prefill_cu[:B - num_decodes + 1] + num_decodes))
            max_prefill_context = max(max_prefill_context, max_decode_context)
            num_decodes = 0
        if num_decodes > 0:
            part_size, num_parts = decode_partitions(num_decodes, Hq, Hkv, max_decode_context, even_contexts)
            scratch = _scratch(num_decodes * Hq * num_parts * (D + 2), q.device) if num_parts > 1 else None
            lib.call("me_attn_decode", q.data_ptr(), q.stride(0), out.data_ptr(), out.stride(0), k_cache.data_ptr(),
                     v_cache.data_ptr(), block_tables.data_ptr(), block_tables.stride(0), context_lens.data_ptr(),
                     num_decodes, Hq, Hkv, page, float(scale), win, part_size, num_parts, _ptr(scratch),
                     0 if even_contexts else 1, _stream())
        if T > num_decodes:
            _check(prefill_cu is not None and _is_i32(prefill_cu, B - num_decodes + 1), "attention: prefill_cu must be int32 [B-Dn+1]")
            Tp = T - num_decodes
            col_tiles = prefill_col_tiles(max_prefill_context, win, Tp, Hq, D)
            seg_keys, max_segs = prefill_segments(max_prefill_context, win, Tp, Hq, D, col_tiles)
            waves = prefill_waves(max_prefill_context, Tp, B - num_decodes, Hq, Hkv, col_tiles, max_segs)
            # the segments' partial results: in a buffer that is kept between steps (a step's decode rows have
            # finished with theirs before, on the same stream, but the two are kept apart all the same)
            pf = _scratch(Tp * Hq * max_segs * (D + 2), q.device, "prefill") if max_segs > 1 else None
            lib.call("me_attn_prefill", q.data_ptr() + num_decodes * q.stride(0) * es, q.stride(0),
                     out.data_ptr() + num_decodes * out.stride(0) * es, out.stride(0), k_cache.data_ptr(),
                     v_cache.data_ptr(), block_tables.data_ptr() + num_decodes * block_tables.stride(0) * 4,
                     block_tables.stride(0), context_lens.data_ptr() + num_decodes * 4, prefill_cu.data_ptr(),
                     B - num_decodes, Tp, Hq, Hkv, page, float(scale), win, col_tiles, PREFILL_THROUGH_LDS, waves, seg_keys, max_segs,
                     _ptr(pf), seq_of_token.data_ptr() + num_decodes * 4, num_decodes, _stream())
        return out

    def decode_step_attention(self, qkv, q_weight, k_weight, eps, table, k_cache, v_cache, page: int, block_tables,
                              context_lens, max_context: int, scale: float, window: int | None, Hq: int, Hkv: int,
                              D: int, even_contexts: bool = False):
        """A pure decode step's `qk_norm_rope_store` and `paged_attention` as one launch: rows [B, (Hq+2Hkv)*D]
        as the packed product left them (row r is request r's one new token, at position context_lens[r] - 1).
        The kernel norms and rotates q and the new key in float32, rounds them to bfloat16 as the separate
        kernel leaves them in the rows, writes the new key and value to the page the block table names for
        that position and attends over the pages. The rows stay as they were. Takes what `decode_step_fuses`
        admits. Returns [B, Hq*D]. (reference models/qwen3.py:34-38, layers/attention.py:63-70: the same
        four calls one after the other.)"""
        B = qkv.shape[0]
        _check(decode_step_fuses(qkv.dtype, D, page), "decode_step_attention: bfloat16 rows, head sizes in steps of 16 "
               "up to 512 and pages of a power of two from 8 on")
        _check(qkv.dim() == 2 and qkv.stride(1) == 1 and qkv.shape[1] == (Hq + 2 * Hkv) * D,
               f"decode_step_attention: rows must be [B, {(Hq + 2 * Hkv) * D}] with unit inner stride")
        for w in (q_weight, k_weight):
            _check(w is None or (w.dtype == torch.float32 and w.shape == (D,) and w.is_contiguous()),
                   "decode_step_attention: norm weights must be float32 [D]")
        _check((q_weight is None) == (k_weight is None), "decode_step_attention: give both norm weights or neither")
        if table is not None:
            _check(table.dtype == torch.float32 and table.is_contiguous() and table.shape[1:] == (D // 2, 2),
                   "decode_step_attention: rotary table must be float32 [P, D/2, 2]")
        _check(k_cache.shape[1:] == (Hkv, page, D) and v_cache.shape[1:] == (Hkv, D, page) and k_cache.is_contiguous()
               and v_cache.is_contiguous() and k_cache.dtype == qkv.dtype and v_cache.dtype == qkv.dtype,
               "decode_step_attention: caches must be K [pages, Hkv, page, D] and V [pages, Hkv, D, page] of the rows' dtype")
        _check(block_tables.dim() == 2 and block_tables.dtype == torch.int32 and block_tables.stride(1) == 1
               and block_tables.shape[0] >= B and _is_i32(context_lens) and context_lens.numel() >= B,
               "decode_step_attention: block tables int32 [B, MB], context lengths int32 [B]")
        _check(block_tables.shape[1] * page >= max_context, "decode_step_attention: block tables shorter than the longest context")
        out = torch.empty((B, Hq * D), dtype=qkv.dtype, device=qkv.device)
        part_size, num_parts = decode_partitions(B, Hq, Hkv, max_context, even_contexts)
        scratch = _scratch(B * Hq * num_parts * (D + 2), qkv.device) if num_parts > 1 else None
        attn_lib(D).call("me_attn_decode_fused", qkv.data_ptr(), qkv.stride(0), out.data_ptr(), out.stride(0),
                         _ptr(q_weight), _ptr(k_weight), float(eps), _ptr(table), 0 if table is None else table.shape[0],
                         k_cache.data_ptr(), v_cache.data_ptr(), block_tables.data_ptr(), block_tables.stride(0),
                         context_lens.data_ptr(), int(max_context), B, Hq, Hkv, page, float(scale), int(window or 0),
                         part_size, num_parts, _ptr(scratch), 0 if even_contexts else 1, _stream())
        return out

    # -- matrix products -----------------------------------------------------------------
    def linear(self, x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype | None = None,
               allow_partials: bool = False, out: torch.Tensor | None = None):
        """x [M, K] . w[N, K]^T (reference layers/linear.py:25-26: F.linear, no bias).

        float32: plain FMA kernel. bfloat16: the skinny MFMA kernel for up to 32 rows (64 for
        smaller weights or when K is split), the library product (hipBLASLt, library_product) above
        that, for the head over a large vocabulary and for large weights with several rows
        (library_streams_better), the FMA kernel for shapes the MFMA kernel refuses.
        With allow_partials the result may be float32 partial sums [S, M, N] over slices of K for a
        consumer that adds them: from the skinny kernel when the output features are few
        (choose_ksplit), from the rows kernel for 17-32 rows over large weights (rows_takes), from the tiled
        kernel for 33 to a few hundred rows over weights up to 27 M elements (mid_slices), from the
        library as a strided batch for 33-1,024 rows over larger weights (library_splits).
        `out` (not with allow_partials): a contiguous [M, N] tensor of the output dtype to write into."""
        _check(x.dim() == 2 and w.dim() == 2 and x.shape[1] == w.shape[1], f"linear: {tuple(x.shape)} x {tuple(w.shape)}^T")
        _check(x.dtype == w.dtype, f"linear: activation {x.dtype} and weight {w.dtype} differ")
        _check(x.stride(1) == 1 and w.stride(1) == 1, "linear: rows must be contiguous")
        M, K = x.shape
        N = w.shape[0]
        out_dtype = out_dtype or x.dtype
        if out is not None:
            _check(not allow_partials and out.shape == (M, N) and out.dtype == out_dtype and out.is_contiguous()
                   and out.device == x.device, "linear: `out` must be a contiguous [M, N] tensor of the output dtype")
        new = (lambda: out) if out is not None else (lambda: torch.empty((M, N), dtype=out_dtype, device=x.device))
        if x.dtype == torch.float32:
            _check(out_dtype == torch.float32, "linear: float32 inputs give float32 outputs")
            y = new()
            core().call("me_gemm_tiled", x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0), y.data_ptr(), N,
                        ME_F32, ME_F32, M, N, K, _stream())
            return y
        aligned = (K % 8 == 0 and x.stride(0) % 8 == 0 and w.stride(0) % 8 == 0
                   and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)
        if not aligned:
            y = new()
            core().call("me_gemm_tiled", x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0), y.data_ptr(), N,
                        ME_BF16, _code(out_dtype), M, N, K, _stream())
            return y
        mid_parts = mid_takes(M, N, K, True) if (allow_partials and out_dtype == x.dtype) else 0
        if mid_parts > 1:
            parts = torch.empty((mid_parts, M, N), dtype=torch.float32, device=x.device)
            core().call("me_gemm_mid_bf16", x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0), parts.data_ptr(), N,
                        ME_F32, mid_parts, M, N, K, 0, _stream())
            return parts
        splits = library_splits(M, N, K) if (allow_partials and out_dtype == x.dtype) else 1
        if splits > 1:
            parts = library_product(x, w, torch.float32, splits)
            if parts is not None:
                return parts
        if allow_partials and out_dtype == x.dtype and rows_takes(M, N, K):
            ksplit = rows_ksplit(K)
            parts = torch.empty((ksplit, M, N), dtype=torch.float32, device=x.device)
            core().call("me_gemm_rows_bf16", x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0), None, N,
                        ME_F32, parts.data_ptr(), ksplit, M, N, K, rows_wide(M, N, ksplit), _stream())
            return parts
        ksplit = choose_ksplit(M, N, K) if (allow_partials and M <= PARTIALS_MAX_M and out_dtype == x.dtype
                                            and (M <= SKINNY_MAX_M or N * K <= SKINNY_WIDE_MAX_WEIGHT)
                                            and not library_streams_better(M, N, K)) else 1
        if ksplit > 1:
            parts = torch.empty((ksplit, M, N), dtype=torch.float32, device=x.device)
            core().call("me_gemm_skinny_bf16", x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0), None, N,
                        ME_F32, parts.data_ptr(), ksplit, M, N, K, 0, 0, skinny_wide(N, K), _stream())
            return parts
        if skinny_takes(M, N, K):
            y = new()
            core().call("me_gemm_skinny_bf16", x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0), y.data_ptr(), N,
                        _code(out_dtype), None, 1, M, N, K, 0, 0, skinny_wide(N, K), _stream())
            return y
        if mid_takes(M, N, K, False) == 1:
            y = new()
            core().call("me_gemm_mid_bf16", x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0), y.data_ptr(), N,
                        _code(out_dtype), 1, M, N, K, 0, _stream())
            return y
        # many rows, or the head over a large vocabulary: the library product (float32 accumulation; the
        # float32 output form keeps the logits unrounded)
        return library_product(x, w, out_dtype, out=out)

    def gated_linear(self, x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
        """silu(x . w[:I]^T) * (x . w[I:]^T) for a packed gate/up weight w [2 I, K] (gate rows first), as one
        launch: the product's workgroups pair each gate feature with its up feature when they merge their waves,
        from the unrounded sums (the separate kernels round the product to bfloat16 first). For the row counts
        `gated_linear_fuses` admits. Returns [M, I]. (reference layers/linear.py:29-45, layers/activation.py:5-7.)"""
        _check(gated_linear_fuses(x, w), "gated_linear: bfloat16, few rows, see gated_linear_fuses")
        M, K = x.shape
        N = w.shape[0]
        y = torch.empty((M, N // 2), dtype=x.dtype, device=x.device)
        if M > GATED_EPILOGUE_MAX_M:        # a few hundred rows over a small weight: the gating in that kernel's epilogue
            core().call("me_gemm_mid_bf16", x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0), y.data_ptr(), N // 2,
                        ME_BF16, 1, M, N, K, 1, _stream())
            return y
        core().call("me_gemm_skinny_bf16", x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0), y.data_ptr(), N // 2,
                    ME_BF16, None, 1, M, N, K, 0, 1, skinny_wide(N, K), _stream())
        return y

    def norm_linear(self, x: torch.Tensor, residual: torch.Tensor | None, norm_weight: torch.Tensor, eps: float,
                    w: torch.Tensor, out_dtype: torch.dtype | None = None, want_residual: bool = True,
                    gated: bool = False):
        """`rms_norm` and `linear` behind it as one launch, for the few rows `norm_linear_fuses` admits:
        r = x (+ residual), x being rows [M, K] or float32 partial sums [S, M, K]; y = (norm_weight * r
        rounded to bfloat16) . w^T, scaled by 1 / rms(r) in float32 (the scale is one number per row, so
        it is applied to the finished sums; the separate kernels round norm_weight * r / rms(r) instead:
        the same relative rounding). `gated`: w is a packed gate/up weight and y is silu(gate) * up, [M, N/2],
        as in `gated_linear`. Returns (y [M, N], r float32 [M, K] or None).
        (reference layers/layernorm.py:11-24, layers/linear.py:25-26.)"""
        _check(norm_linear_fuses(x, w), "norm_linear: bfloat16 weights, few rows, see norm_linear_fuses")
        _check(not gated or w.shape[0] % 2 == 0, "norm_linear: a packed gate/up weight has an even number of rows")
        S = x.shape[0] if x.dim() == 3 else 1
        M, K = x.shape[-2], x.shape[-1]
        N = w.shape[0]
        _check(norm_weight.dtype == torch.float32 and norm_weight.shape == (K,) and norm_weight.is_contiguous(),
               "norm_linear: the norm's weight must be float32 [K]")
        if residual is not None:
            _check(residual.dtype == torch.float32 and residual.shape == (M, K) and residual.is_contiguous(),
                   "norm_linear: residual must be contiguous float32 [M, K]")
        out_dtype = out_dtype or w.dtype
        cols = N // 2 if gated else N
        y = torch.empty((M, cols), dtype=out_dtype, device=x.device)
        res_out = torch.empty((M, K), dtype=torch.float32, device=x.device) if want_residual else None
        core().call("me_gemm_skinny_norm_bf16", x.data_ptr(), _code(x.dtype), S, _ptr(residual), _ptr(res_out),
                    norm_weight.data_ptr(), float(eps), w.data_ptr(), w.stride(0), y.data_ptr(), cols, _code(out_dtype),
                    M, N, K, int(gated), _stream())
        return y, res_out

    def silu_mul_linear(self, gu: torch.Tensor, w: torch.Tensor, allow_partials: bool = False):
        """(silu(gu[:, :I]) * gu[:, I:]) . w[N, I]^T: the gating fused into the product for few
        rows and a moderate width (bfloat16, M <= 16, I <= 4096, where the product is a weight stream
        and the gating is free);
        otherwise the two kernels one after the other (reference models/qwen3.py:50-51)."""
        M, two_i = gu.shape
        inter = two_i // 2
        _check(w.shape[1] == inter and two_i == 2 * inter, f"silu_mul_linear: {tuple(gu.shape)} against {tuple(w.shape)}")
        fused = (gu.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and M <= GATED_MAX_M and inter % 8 == 0
                 and inter <= GATED_MAX_K and not library_streams_better(M, w.shape[0], inter)
                 and gu.is_contiguous() and w.stride(1) == 1 and w.stride(0) % 8 == 0
                 and gu.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)
        if not fused:
            return self.linear(self.silu_and_mul(gu), w, None, allow_partials)
        N = w.shape[0]
        ksplit = choose_ksplit(M, N, inter) if allow_partials else 1      # fused only for M <= GATED_MAX_M <= PARTIALS_MAX_M
        if ksplit > 1:
            parts = torch.empty((ksplit, M, N), dtype=torch.float32, device=gu.device)
            core().call("me_gemm_skinny_bf16", gu.data_ptr(), gu.stride(0), w.data_ptr(), w.stride(0), None, N,
                        ME_F32, parts.data_ptr(), ksplit, M, N, inter, 1, 0, 0, _stream())
            return parts
        y = torch.empty((M, N), dtype=gu.dtype, device=gu.device)
        core().call("me_gemm_skinny_bf16", gu.data_ptr(), gu.stride(0), w.data_ptr(), w.stride(0), y.data_ptr(), N,
                    ME_BF16, None, 1, M, N, inter, 1, 0, 0, _stream())
        return y

    # -- sampling ------------------------------------------------------------------------
    def sample(self, logits: torch.Tensor, temperatures: torch.Tensor, keys: torch.Tensor) -> torch.Tensor:
        """Token ids int32 [S] from float32 logits [S, V]: argmax where temperature is 0, else
        argmax(logits/T - log E) with E ~ Exp(1) a hash of (keys[s], vocabulary id)
        (reference layers/sampler.py:5-11)."""
        S, V = logits.shape
        _check(logits.dtype == torch.float32 and logits.stride(1) == 1, "sample: logits must be float32 rows")
        _check(temperatures.dtype == torch.float32 and temperatures.numel() == S and temperatures.is_contiguous(),
               "sample: temperatures must be float32 [S]")
        _check(keys.dtype == torch.int32 and keys.shape == (S, 2) and keys.is_contiguous(), "sample: keys must be int32 [S, 2]")
        out = torch.empty((S,), dtype=torch.int32, device=logits.device)
        if S <= SAMPLE_STATIC_MAX_ROWS:
            # the per-chunk partial results stay in a device array of the library: nothing is allocated for them.
            # (All calls on a GPU share that array; the engine samples on one stream, one call after the other.)
            core().call("me_sample_static", logits.data_ptr(), logits.stride(0), temperatures.data_ptr(), keys.data_ptr(),
                        out.data_ptr(), S, V, _stream())
            return out
        scratch = _scratch(2 * S * 32, logits.device, "sample")
        core().call("me_sample", logits.data_ptr(), logits.stride(0), temperatures.data_ptr(), keys.data_ptr(),
                    out.data_ptr(), scratch.data_ptr(), S, V, _stream())
        return out


# Dispatch rules. Every threshold below was measured on one MI355X at the layer sizes of Qwen3-0.6B, 8B and 32B;
# the tables behind each constant are kept in the repository's design notes, one line of reason here.
SKINNY_MAX_M = 32                          # rows up to which the skinny kernel beats the library product
SKINNY_WIDE_MAX_M = 64                     # ... for weights of up to SKINNY_WIDE_MAX_WEIGHT elements
SKINNY_WIDE_MAX_WEIGHT = 5 * 1024 * 1024
PARTIALS_MAX_M = 64                        # rows up to which a product split over K (float32 partial sums) pays
LIBRARY_MIN_N = 32768                      # outputs this wide (the head over the vocabulary) go to the library ...
WIDE_OUTPUT_SKINNY_ROWS = 12               # ... except up to this many rows, where the skinny kernel's wide loads win
LIBRARY_MIN_ROWS = 4                       # large weights go to the library from this many rows on ...
LIBRARY_MIN_ROWS_WIDE = 17                 # ... with the wide loads and K up to 4,096: never within their 16 rows
LIBRARY_MIN_ROWS_WIDE_LONG_K = 11          # ... over a longer K
LIBRARY_MIN_WEIGHT = 15 * 1024 * 1024
LIBRARY_MAX_K = 16384                      # the library's choice for a longer K is poor
ROWS_MIN_WEIGHT = 10 * 1024 * 1024
ROWS_FEW_FEATURES = 3072
PREFILL_SEGMENT_KEYS = None    # None: chosen by prefill_segments(); an int forces that many keys per segment (0: never cut)
# prefill attention, keys and values shared by a workgroup's waves through LDS: 0 never, 1 wherever it fits (written there
# by the loads themselves at head size 128 and pages of 16 keys or more), 2 as 1 but always staged through registers
PREFILL_THROUGH_LDS = 1
PREFILL_COL_TILES = 0     # 0: chosen by prefill_col_tiles(); 1 or 2 force the column tiles per wave
DECODE_AS_PREFILL = False      # True: single-token rows go through the prefill kernel (cross-check of the decode kernel)
USE_MID_PRODUCT = True          # False: products of 33-512 rows over small weights go to the library like the larger ones
MID_MAX_WEIGHT = 8 << 20
MID_SMALL_WEIGHT = 13 << 19     # 6.5 M elements: gate/up at the 0.6B sizes (6.3 M) keeps the own kernel and its gating epilogue
FUSE_GATE_INTO_GATE_UP = True  # False: silu(gate) * up is formed in front of the down product, not behind gate_up
GATED_EPILOGUE_MAX_M = 16
FUSE_NORM_INTO_LINEAR = True   # False: the norm kernel and the product behind it always run as two launches
NORM_FUSE_MAX_M = 2
NORM_FUSE_MAX_WEIGHT = 8 << 20
FUSE_DECODE_STEP = True        # False: pure decode steps run norm/rotation/cache write and attention as two launches
GATED_MAX_K = 4096             # the gating in front of the down product is formed in every workgroup: not over a longer K
GATED_MAX_M = 16
_COMPUTE_UNITS = 256
_DECODE_WORKGROUPS = 4096
_PREFILL_THREE_WAVES_WORKGROUPS = 2048
_DECODE_WHOLE_WORKGROUPS = 768
_DECODE_ONE_ROUND = 768           # workgroups of the decode kernel that run at once: three to a compute unit
_DECODE_WHOLE_MAX_KEYS = 4096
_DECODE_EVEN_WHOLE_WORKGROUPS = 192
_DECODE_EVEN_WHOLE_MAX_KEYS = 8192
_DECODE_MAX_PARTITION = 2048
SAMPLE_STATIC_MAX_ROWS = 1024     # ME_SAMPLE_STATIC_MAX_ROWS of csrc/sampling.h
_scratch_buf: dict = {}
_scratch_retired: list = []      # outgrown buffers stay alive: a captured graph may still write to them


def _scratch(num_floats: int, device, use: str = "decode") -> torch.Tensor:
    """Device memory for a kernel's partial results (4-byte words), kept between calls: one buffer per device
    and use, grown when a call needs more (by half as much again, so that a slowly growing need does not
    allocate at every step), never shrunk."""
    key = (device, use)
    buf = _scratch_buf.get(key)
    if buf is None or buf.numel() < num_floats:
        if buf is not None:
            _scratch_retired.append(buf)
        buf = torch.empty((max(num_floats + num_floats // 2, 1 << 20),), dtype=torch.float32, device=device)
        _scratch_buf[key] = buf
    return buf


def prefill_col_tiles(max_context: int, window: int, num_tokens: int, Hq: int, D: int = 128) -> int:
    """Column tiles (of 16 (token, head) pairs) per wave of the prefill kernel: 2 halves the reads of keys and
    values per product but needs twice the columns per workgroup, so it is for launches with many columns (32,768
    or more: 2,048 tokens of 16 heads), and for portions of 256 tokens or more of a prompt over 4,096 keys or
    more, where each tile walks a long range and `prefill_segments` cuts that range into enough workgroups.
    PREFILL_COL_TILES forces it."""
    if PREFILL_COL_TILES in (1, 2):
        return PREFILL_COL_TILES
    if D > 128:
        return 1
    cols = num_tokens * Hq
    span = min(max_context, window + 256) if window else max_context
    return 2 if cols >= 32768 or (cols >= 4096 and span >= 4096) else 1


def prefill_segments(max_context: int, window: int, num_tokens: int, Hq: int, D: int = 128, col_tiles: int | None = None) -> tuple:
    """(keys per segment, most segments per tile) for the prefill kernel; (0, 1): no cutting.

    A tile's key range grows with its position, and a step with few new tokens over a long context
    gives the kernel few workgroups, each walking the whole context. Cutting the ranges into
    segments of at least 512 keys (1,024 over ranges beyond 4,096), run by different workgroups and merged by a
    second kernel, evens the work out and fills the GPU: two segments for launches of 257 to 640 workgroups; three
    for 129 to 256 when the ranges start short (a prompt from its beginning: tiles of 64 to all keys,
    which thirds balance better than halves) and two when they are all long (a later portion of a
    prompt: twice the workgroups fill the slots evenly); as many as give 768 workgroups below that.
    A portion of a prompt that runs with two column tiles per wave before its launch has 32,768 columns
    (`prefill_col_tiles`) gets segments of 512 to 1,024 keys, as many as give about 512 workgroups.
    PREFILL_SEGMENT_KEYS forces a size."""
    span = min(max_context, window + 256) if window else max_context
    if PREFILL_SEGMENT_KEYS is not None:
        seg = PREFILL_SEGMENT_KEYS
        return (seg, -(-span // seg) + 1) if seg > 0 and span > seg else (0, 1)
    cols = num_tokens * Hq
    if col_tiles is None:
        col_tiles = prefill_col_tiles(max_context, window, num_tokens, Hq, D)
    most_by_memory = (1 << 28) // (cols * (D + 2) * 4) - 1      # the partial results are float32 [tokens, heads, segments + 1, D + 2]: under 256 MB
    if col_tiles == 2 and cols < 32768:
        tiles = -(-cols // 128)
        seg = min(1024, max(512, -(-(-(-span // -(-512 // tiles))) // 32) * 32))
        segs = min(-(-span // seg), most_by_memory)
        if segs <= 1:
            return 0, 1
        seg = -(-(-(-span // segs)) // 32) * 32
        return seg, -(-span // seg) + 1
    workgroups = max(1, cols // (128 if col_tiles == 2 else 64))
    if workgroups > 640:
        segs = 1
    elif workgroups > 256:
        segs = 2
    elif workgroups > 128:
        segs = 3 if 2 * (max_context - num_tokens) < span else 2
    else:
        segs = -(-768 // workgroups)
    segs = min(segs, span // (512 if span <= 4096 else 1024))      # segments of 512 keys or more, 1,024 over long ranges
    segs = min(segs, most_by_memory)
    if segs <= 1:
        return 0, 1
    seg = -(-(-(-span // segs)) // 32) * 32
    return seg, -(-span // seg) + 1


SKINNY_WIDE_MIN_WEIGHT = 1 << 22


def skinny_wide(N: int, K: int) -> int:
    """Whether the skinny product reads a weight [N, K] with its wide loads: a wave's load takes 256 contiguous bytes
    of each of four rows, marked as not to be kept by the caches, and the pieces reach their lanes through LDS. For
    weights of SKINNY_WIDE_MIN_WEIGHT elements or more (the kernel applies them to up to 16 rows and a K in whole
    steps of 128); small weights are over before the mark matters."""
    return 1 if N * K >= SKINNY_WIDE_MIN_WEIGHT else 0


def skinny_takes(M: int, N: int, K: int) -> bool:
    """Whether the skinny kernel (without a split over K) takes an aligned bfloat16 product."""
    rows_ok = M <= SKINNY_MAX_M or (M <= SKINNY_WIDE_MAX_M and N * K <= SKINNY_WIDE_MAX_WEIGHT)
    if N >= LIBRARY_MIN_N:
        rows_ok = M <= WIDE_OUTPUT_SKINNY_ROWS and K % 128 == 0 and skinny_wide(N, K) == 1
    return rows_ok and not library_streams_better(M, N, K)


LIBRARY_SPLIT_MIN_ROWS = 33
LIBRARY_SPLIT_MAX_ROWS = 1024
LIBRARY_SPLIT_MIN_WEIGHT = 10 << 20
LIBRARY_SPLIT_SURE_WEIGHT = 16 << 20


def library_splits(M: int, N: int, K: int) -> int:
    """In how many slices of K the library computes a product whose consumer adds float32 partial sums
    (1: not this way). o and down have few output features and a long K, so the library's plain call
    covers the output with too few tiles to fill the GPU (it has no split over K of its own for these
    shapes); as a strided batch over slices of K it runs the same large-tile kernels on 2-8 times the
    tiles. From 33 rows (below, the skinny and the rows kernel are as fast or faster) to 1,024 (above,
    the tiles suffice and the partial sums, S x M x N x 4 bytes written and read again, cost more than
    the split gains), for weights of 10 M elements or more."""
    if not (LIBRARY_SPLIT_MIN_ROWS <= M <= LIBRARY_SPLIT_MAX_ROWS) or N * K < LIBRARY_SPLIT_MIN_WEIGHT:
        return 1
    if N * K < LIBRARY_SPLIT_SURE_WEIGHT and K < 6144 and M < 128:
        return 1          # the smaller of these weights over a short K: the plain call is ahead below 128 rows
    if rows_has_few_features(M, N, K):
        return 1
    if not library_is_direct():
        return 1
    splits = 8 if M <= 256 else 4 if M <= 512 else 2
    while splits > 1 and (K % (8 * splits) or K // splits < 512):
        splits //= 2
    return splits


def rows_has_few_features(M: int, N: int, K: int) -> bool:
    """33 to 64 rows over a weight of up to ROWS_FEW_FEATURES output features and a K of 8,192 or more (down at the 4B
    sizes): the rows kernel's own split over K is ahead of the library's slices and of its plain call."""
    return 32 < M <= 64 and N <= ROWS_FEW_FEATURES and K >= 8192 and K % 8 == 0 and N * K >= ROWS_MIN_WEIGHT


def rows_takes(M: int, N: int, K: int) -> bool:
    """Whether a product whose consumer adds float32 partial sums goes to the rows kernel (64 features per
    workgroup, the tokens staged once per workgroup in LDS, K split over up to 8 workgroups): large
    weights with 17 to 64 rows, where the skinny kernel reads the tokens again for every 16 features and
    the library streams at 1.7-3.5 TB/s, and from 8 rows on over a K too long for the library that is no multiple
    of 128 (otherwise the skinny kernel's wide loads are ahead up to 16 rows); and 33 to 64 rows over a weight with
    few output features (up to ROWS_FEW_FEATURES) and a K of 8,192 or more, where the library's slices of K are poor."""
    if N * K < ROWS_MIN_WEIGHT or K < 4096 or K % 8 or M > 64:
        return False
    if rows_has_few_features(M, N, K):
        return True       # few output features over a long K: the library's slices have too few tiles here too
    if library_splits(M, N, K) > 1:
        return False
    if M > 16:
        return M <= 32 or K >= 12288
    return M >= 8 and K > LIBRARY_MAX_K and not (K % 128 == 0 and skinny_wide(N, K))


def rows_wide(M: int, N: int, ksplit: int) -> int:
    """Whether the rows kernel reads its weights with the wide loads of the skinny kernel (`skinny_wide`): up to 32
    rows and with two workgroups or more to a compute unit. The pass through LDS lengthens a wave's chain from load
    to product, which other workgroups on the compute unit must fill, and the wave tiles' 17 KB beside 48-64 KB of
    staged tokens leave room for one workgroup only."""
    return 1 if M <= 32 and -(-N // 64) * ksplit >= 2 * _COMPUTE_UNITS else 0


def rows_ksplit(K: int) -> int:
    """The most splits up to 8 that leave no split without one of the K/512 chunks."""
    chunks = -(-K // 512)
    for ks in range(min(8, chunks), 0, -1):
        if (ks - 1) * -(-chunks // ks) < chunks:
            return ks
    return 1


def library_streams_better(M: int, N: int, K: int) -> bool:
    """Whether a product of few rows goes to the library rather than the skinny kernel: every workgroup of the
    skinny kernel reads all of x, which at 8 to 16 rows is as much traffic as a large weight itself."""
    if N * K < LIBRARY_MIN_WEIGHT or K > LIBRARY_MAX_K:
        return False
    if K % 128 == 0 and M <= 16 and skinny_wide(N, K):
        return M >= (LIBRARY_MIN_ROWS_WIDE if K <= 4096 else LIBRARY_MIN_ROWS_WIDE_LONG_K)
    return M >= LIBRARY_MIN_ROWS


def choose_ksplit(M: int, N: int, K: int) -> int:
    """Workgroups over K for a skinny product whose consumer adds float32 partial sums (1: K is not split).

    A product's time goes with the rounds its workgroups make over the 256 compute units, each round as long as
    a workgroup's share of K: rounds(tiles x splits) / splits, plus a little for every further set of partial sums
    that the consumer reads. The split with the least of that is taken, each split keeping 512 of K or more (4
    steps of 128, one per wave); with 256 feature tiles or more only over a K of 4,096 or more, where an uneven
    count (320 tiles: one round and a quarter) costs a quarter of the stream, and only up to 32 rows (beyond, the
    library is level or ahead)."""
    tiles = -(-N // 16) * -(-M // 64)
    if tiles >= _COMPUTE_UNITS and (K < 4096 or M > SKINNY_MAX_M):
        return 1
    best, least = 1, None
    for splits in range(1, 9):
        if splits > 1 and K // splits < 512:
            break
        cost = -(-tiles * splits // _COMPUTE_UNITS) / splits + 0.02 * splits
        if least is None or cost < least - 1e-9:
            best, least = splits, cost
    return best


MID_SLICES_MAX_WEIGHT = 27 << 20


def mid_slices(M: int, N: int, K: int) -> int:
    """In how many slices of K (2, 4 or 8; 1: not so) the tiled kernel of csrc/gemm_mid.hip computes M rows against a
    weight [N, K] as float32 partial sums for a consumer that adds them: o and down of a layer at 33 to a few hundred
    rows. A tile of 64 x 64 is one workgroup, and a compute unit that draws its operands alone gets them slowly, so
    what counts is how many workgroups there are: as many slices as keep tiles x slices within 256 workgroups (two
    slices up to 320), each slice with 8 steps of 64 or more (4 where the workgroups are 128 at most). Where it is
    ahead of the skinny split, the rows kernel and the library's strided batch (us with the norm that adds the slices
    behind, this / those): weights up to 8 M elements with up to 2,048 features (1024 x 3072 at 64 rows in 8 slices
    8.3 / 9.4 in 4); up to 13 M and 2,560 features at up to 256 rows (2048 x 6144 at 64 rows 11.6 / 14.7, 2560 x 4096 at
    128 rows 13.7 / 20.9); up to 27 M and 4,096 features at up to 128 rows (2560 x 9728 at 64 rows 20.1 / 24.7, 4096 x
    4096 at 64 rows 13.4 / 17.2). Beyond (4096 x 12288, 5120 x 5120, 5120 x 17408, more rows) the library's larger tiles
    are level or ahead."""
    weight = N * K
    # from 17 rows over the larger weights (2048 x 6144 at 24 rows 10.2 / 12.0, 2560 x 4096 10.3 / 12.8, 2560 x 9728 17.6 /
    # 20.3 with the rows kernel); over the small ones the skinny kernel's split keeps 17-32 rows (1024 x 2048: 6.8 / 7.2)
    if (not USE_MID_PRODUCT or K % 64 or N % 4 or K < 2048 or M <= (32 if weight <= MID_MAX_WEIGHT else 16)
            or weight > MID_SLICES_MAX_WEIGHT):
        return 1
    if weight <= MID_MAX_WEIGHT:
        if N > 2048 or M > (512 if N <= 1024 else 256):
            return 1
        if M > 256:
            return 4
    elif weight <= 13 << 20:
        if N > 2560 or M > 256:
            return 1
    elif N > 4096 or M > 128:
        return 1
    tiles = -(-N // 64) * -(-M // 64)
    steps = K // 64
    for slices in (8, 4, 2):
        per = -(-steps // slices)                       # steps of a slice; the last may have fewer, none has none
        fills = tiles * slices <= 256 or (slices == 2 and tiles <= 160)
        if fills and (slices - 1) * per < steps and (per >= 8 or (per >= 4 and tiles * slices <= 128)):
            return slices
    return 1


def mid_takes(M: int, N: int, K: int, partials: bool) -> int:
    """Whether the product of M rows against a bfloat16 weight [N, K] goes to the own kernel for a few hundred rows
    (csrc/gemm_mid.hip), and in how many slices of K: 0 no, 1 one result, 2, 4 or 8 float32 partial sums over
    that many slices (only when the consumer adds them, `partials`: `mid_slices`). One result: its time is 7 us
    whatever the row count up to 256 (tiles of 64 x 64, one workgroup to a compute unit), where the library's grows
    with the rows; beyond 8 M weight elements and beyond these row counts the library's larger tiles win."""
    if not USE_MID_PRODUCT or K % 64 or N % 4 or K < 256 or M <= 16:
        return 0
    if partials:
        slices = mid_slices(M, N, K)
        if slices > 1:
            return slices
    if M <= 32:
        return 0
    if N * K > MID_MAX_WEIGHT:
        return 0
    if N * K > MID_SMALL_WEIGHT and M < 128:
        return 0          # the larger of the small weights with few rows: the library's tiles are ahead
    return 1 if M <= 256 else 0


def prefill_waves(max_context: int, num_tokens: int, num_seqs: int, Hq: int, Hkv: int, col_tiles: int, max_segs: int) -> int:
    """Waves per SIMD (2 or 3) of the prefill attention kernel whose loads write LDS themselves (head size 128).

    Three waves of 168 registers where two column tiles per wave are in use, the tiles are left whole, there are
    2,048 workgroups or more, and the prompts start at their beginning (the longest context at most twice the mean
    number of new tokens per sequence): tiles of all lengths are then under way at once and the third wave fills
    the others' waits. Portions over a long prefix, whose tiles are equally long and walk the same keys together,
    run better with two waves and 205 registers, and so do launches of few workgroups."""
    if col_tiles != 2 or max_segs != 1 or num_seqs < 1 or max_context <= 0:
        return 2
    group = max(1, Hq // max(1, Hkv))
    tok_tile = max(1, 128 // group)
    tiles = num_tokens // tok_tile + num_seqs
    if tiles * Hkv < _PREFILL_THREE_WAVES_WORKGROUPS or max_context * num_seqs > 2 * num_tokens:
        return 2
    return 3


_DECODE_PART_SIZES = tuple(range(128, 577, 32)) + tuple(range(640, 1409, 64))


def _decode_partition_cost(base: int, ctx: int, part: int) -> float:
    """What a launch of the split decode kernel costs with partitions of `part` keys, in units of one key's work on a
    compute unit: the keys of the busiest compute unit (its workgroups, each with about 64 keys' worth of work before
    and after its keys; a few workgroups beyond a multiple of the 256 units already make some unit that busy), 80 for
    every block that a wave takes after another (a trip to memory that nothing hides), and 300 for every round of
    workgroups beyond the 768 that run at once. Fitted to 86 launches timed over all sizes (1-32 requests of 300-66,000
    keys, 8 key heads with 2, 4 and 8 query heads each, 2 key heads of 64 channels): the size it puts first is 2 %
    behind the fastest on average (12 % at worst)."""
    parts = -(-ctx // part)
    workgroups = base * parts
    per_unit = workgroups / _COMPUTE_UNITS
    busiest = int(per_unit) + min(1.0, (per_unit - int(per_unit)) * 3) if per_unit > 1 else 1.0
    rounds = -(-workgroups // _DECODE_ONE_ROUND)
    return busiest * (part + 64) + 80 * -(-part // 128) + 300 * (rounds - 1)


def decode_partitions(num_seqs: int, Hq: int, Hkv: int, max_context: int, even: bool = False) -> tuple:
    """(keys per partition, number of partitions) for the split decode kernel.

    A workgroup's 4 waves take the 32-key blocks of its partition in turn, and three workgroups share a compute
    unit: 768 run at once. While there are fewer (sequence, kv head) pairs than compute units, the partition size is
    the one of 128, 160, ... 576, 640, ... 1,408 keys that `_decode_partition_cost` puts first (8 requests of 2,048
    keys: 8 partitions of 256; of 2,070 keys: 11 of 192, 704 workgroups at once, where 17 of 128 keys, 1,088
    workgroups in a round and a third, cost a fifth more; of 8,200 keys: 12 of 704), never more than 64 partitions to
    merge. Beyond that list, and from 256 pairs on: one round of workgroups while the pairs stay below 768, at least
    128 keys (one block per wave) and at most 512, and at most 2,048 keys as long as 64 partitions cover the
    context: a workgroup goes through its keys round by round, so in a batch with a few long contexts among short
    ones the long partitions are what is still running at the end.
    From 768 workgroups on (96 sequences x 8 kv heads) a context up to 2,048 keys (4,096 from 2,048 workgroups
    on) is one partition and needs no reduce kernel. `even` (the contexts are equally long,
    `decode_contexts_even`): from 192 workgroups on, a context up to 8,192 keys is one partition if the workgroups
    then fill the compute units evenly (a multiple of 256: 32 or 64 requests x 8 kv heads; 24 or 48 requests leave
    compute units idle or doubly loaded and run 12-14 % faster in partitions): every workgroup then has the same
    work, none waits for another's partial results and no reduce kernel follows; contexts of different lengths
    gain nothing from it and long ones among short ones lose.
    (The reference's rule: layers/ops.py:44-51, split when sequences x kv heads cannot fill the SMs, 256-key
    partitions.)"""
    col_tiles = (Hq // Hkv + 15) // 16
    base = max(1, num_seqs * Hkv * col_tiles)
    ctx = max(1, max_context)
    if base >= _DECODE_WHOLE_WORKGROUPS and ctx <= (_DECODE_WHOLE_MAX_KEYS if base >= 2048 else _DECODE_WHOLE_MAX_KEYS // 2):
        return -(-ctx // 128) * 128, 1
    if even and base >= _DECODE_EVEN_WHOLE_WORKGROUPS and base % _COMPUTE_UNITS == 0 and ctx <= _DECODE_EVEN_WHOLE_MAX_KEYS:
        return -(-ctx // 128) * 128, 1
    if base < _COMPUTE_UNITS:
        # fewer (request, head block) pairs than compute units: the size that a simple reckoning of the launch's time
        # puts first (sizes beyond the list only where 64 partitions of the largest do not cover the context)
        sizes = [p for p in _DECODE_PART_SIZES if -(-ctx // p) <= 64]
        if sizes:
            part = min(sizes, key=lambda p: (_decode_partition_cost(base, ctx, p), -p))
            return part, max(1, -(-ctx // part))
    if base <= _DECODE_ONE_ROUND:
        # one round of workgroups where the batch allows it
        per = -(-ctx // max(1, _DECODE_ONE_ROUND // base))
        part = min(512, max(128, -(-per // 64) * 64))
        part = max(part, -(-(-(-ctx // 64)) // 128) * 128)          # 64 partitions at most
        return part, max(1, -(-ctx // part))
    want = max(1, -(-_DECODE_WORKGROUPS // base), -(-ctx // _DECODE_MAX_PARTITION))
    want = min(64, want)
    part = max(128, -(-(-(-ctx // want)) // 128) * 128)
    parts = max(1, -(-ctx // part))
    return part, parts


def gated_linear_rows(rows: int, w: torch.Tensor) -> bool:
    """Whether `rows` rows against the packed gate/up weight w [2 I, K] are few enough, and w of a kind, for the
    gating to happen in the product's epilogue: a bfloat16 product that the unsplit skinny kernel takes, up to
    GATED_EPILOGUE_MAX_M rows, or one of 17-256 rows that the tiled kernel for small weights takes (`mid_takes`).
    In front of the down product the gating costs every one of that product's workgroups about 2 us; behind
    gate/up every gate is formed once."""
    if not FUSE_GATE_INTO_GATE_UP or w.dtype != torch.bfloat16 or w.dim() != 2:
        return False
    N, K = w.shape
    # over large weights the library takes the product from a row count on (library_streams_better), and the gating is
    # then a kernel of its own; without the skinny kernel's wide loads (K no multiple of 128) the skinny kernel with the
    # gating in its epilogue is still ahead of the two up to 8 rows over a K of 4,096
    takes = skinny_takes(rows, N, K) or (rows <= 8 and K <= 4096 and N < LIBRARY_MIN_N and rows <= SKINNY_MAX_M)
    aligned = N % 2 == 0 and K % 8 == 0 and w.stride(1) == 1 and w.stride(0) % 8 == 0 and w.data_ptr() % 16 == 0
    if rows > GATED_EPILOGUE_MAX_M:
        # the kernel for a few hundred rows over a small weight gates in its epilogue too, in place of a kernel of
        # its own behind it; and from 17 rows on, where the skinny kernel would have the product itself
        if not (aligned and N % 8 == 0):
            return False
        if rows <= 32:
            return mid_takes(33, N, K, False) == 1
        return not skinny_takes(rows, N, K) and mid_takes(rows, N, K, False) == 1
    return 1 <= rows and aligned and takes


def gated_linear_fuses(x: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether `gated_linear` takes rows x [M, K] and the packed gate/up weight w [2 I, K]."""
    return (x.dtype == torch.bfloat16 and x.dim() == 2 and w.dim() == 2 and x.shape[1] == w.shape[1] and x.stride(1) == 1
            and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0 and gated_linear_rows(x.shape[0], w))


def norm_linear_fuses(x: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether `norm_linear` takes rows x ([M, K], or float32 partial sums [S, M, K]) and weight w: a
    bfloat16 weight that the unsplit skinny kernel would take, one or two rows, a weight of at most
    NORM_FUSE_MAX_WEIGHT elements. Every workgroup forms the normed rows for itself, which costs each about
    2 us; the norm kernel costs 3 us in a chain of decode kernels, so it pays for one and two rows only."""
    if not FUSE_NORM_INTO_LINEAR or w.dtype != torch.bfloat16 or w.dim() != 2 or x.dim() not in (2, 3):
        return False
    S = x.shape[0] if x.dim() == 3 else 1
    M, K = x.shape[-2], x.shape[-1]
    N = w.shape[0]
    if x.dtype not in (torch.float32, torch.bfloat16) or (S > 1 and x.dtype != torch.float32) or S > 8:
        return False
    if not (1 <= M <= NORM_FUSE_MAX_M and K == w.shape[1] and K % 8 == 0 and x.is_contiguous() and w.stride(1) == 1
            and w.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0):
        return False
    if N * K > NORM_FUSE_MAX_WEIGHT or M * (K + 8) * 2 + 4416 > 64 * 1024:
        return False
    return skinny_takes(M, N, K)


def decode_step_fuses(dtype: torch.dtype, D: int, page: int) -> bool:
    """Whether `decode_step_attention` takes these rows: what the matrix-core attention kernels take."""
    return bool(FUSE_DECODE_STEP and dtype == torch.bfloat16 and D % 16 == 0 and 16 <= D <= 512 and page >= 8
                and page & (page - 1) == 0)


def decode_contexts_even(num_seqs: int, min_context: int, max_context: int) -> bool:
    """Whether the decode kernel may keep each request's work on one XCD (8 requests or more whose
    contexts differ by 5 % at most), or has to spread every request over the XCDs. With all of a request
    on one XCD, the XCD that draws the long contexts finishes last; with equal contexts the spread costs
    1-3 % for the block-table reads that a request's heads no longer share in one L2."""
    return num_seqs >= 8 and min_context > 0 and (max_context - min_context) * 20 <= max_context


# --------------------------------------------------------------------------- dispatch

_backend = None


def backend():
    global _backend
    if _backend is None:
        _require_gpu()
        _backend = HipBackend()
    return _backend


def set_backend(b) -> None:
    """Install another object with HipBackend's methods (tests only); None restores the default."""
    global _backend
    _backend = b


def gather_rows(*a, **k): return backend().gather_rows(*a, **k)
def take_tokens(*a, **k): return backend().take_tokens(*a, **k)
def rms_norm(*a, **k): return backend().rms_norm(*a, **k)
def silu_and_mul(*a, **k): return backend().silu_and_mul(*a, **k)
def qk_norm_rope_store(*a, **k): return backend().qk_norm_rope_store(*a, **k)
def store_kv(*a, **k): return backend().store_kv(*a, **k)
def paged_attention(*a, **k): return backend().paged_attention(*a, **k)
def decode_step_attention(*a, **k): return backend().decode_step_attention(*a, **k)
def linear(*a, **k): return backend().linear(*a, **k)
def silu_mul_linear(*a, **k): return backend().silu_mul_linear(*a, **k)
def norm_linear(*a, **k): return backend().norm_linear(*a, **k)
def gated_linear(*a, **k): return backend().gated_linear(*a, **k)
def sample(*a, **k): return backend().sample(*a, **k)

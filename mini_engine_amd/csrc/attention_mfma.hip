// Paged attention on the CDNA4 matrix cores (bfloat16 in, float32 accumulate), compiled once
// per head size with -DME_HEAD_DIM=<D> (a multiple of 16).
//
// What the reference has: csrc/paged_prefill.cu:177-247 (flash-style tiles over block-table
// K/V, causal cut, online softmax, P rounded to bf16 before P.V while the sum uses the
// unrounded values), csrc/paged_decode.cu:202-334 (one block per (sequence, kv head), split-K
// partitions and a reduce kernel merging (max, sum, unnormalised output)). Those are warp-32
// WMMA/shuffle designs fixed to D=128, page 16, group 2. This file is a different design:
//
//  * Everything is computed transposed, with v_mfma_f32_16x16x32_bf16:
//      S^T[key, col] = K[key, :] . Q[col, :]      (A = K rows, B = Q rows; both contiguous in d)
//      O^T[d, col]  += V^T[d, key] . P^T[key, col] (A = V^T rows, B = P^T)
//    A "column" is one (query token, query head) pair of one kv head. The accumulator layout of
//    S^T (lane = column + 16*g holds keys 4g..4g+3) becomes the B operand of the second product
//    without any data movement, by letting rows of the two S^T tiles stand for keys
//    8*(m/4)+(m%4) and 8*(m/4)+4+(m%4): lane group g then holds keys 8g..8g+7 of the 32-key block,
//    exactly the 8 consecutive k-slots it must supply.
//  * The cache keeps V transposed inside a page ([page][Hkv][D][page_size]) so the V^T operand
//    is one 16-byte load of 8 consecutive keys; K ([page][Hkv][page_size][D]) is one 16-byte
//    load of 8 consecutive channels. No LDS is used for operands.
//  * All softmax state (running max, sum, rescaling) is float32 and per column, i.e. per lane.
//
// Masked keys never contribute: scores are replaced (not multiplied), and V values of keys at
// or beyond the context length are zeroed before the product, so a cache full of NaN outside
// the owned range cannot leak.
#include "common.h"

#ifndef ME_HEAD_DIM
#error "compile with -DME_HEAD_DIM=<multiple of 16>"
#endif
static_assert(ME_HEAD_DIM % 16 == 0 && ME_HEAD_DIM >= 16 && ME_HEAD_DIM <= 512, "head size");

constexpr int HD = ME_HEAD_DIM;
constexpr int KS = (HD + 31) / 32;  // 32-channel steps of the score product
constexpr int DT = HD / 16;         // 16-channel tiles of the output
constexpr float NEG = -1e30f;       // "no key yet": finite, so that differences never give NaN

struct AttnArgs {
  const bf16_t* q;
  int64_t q_stride;  // elements between consecutive tokens; head h starts at h*HD
  bf16_t* out;
  int64_t out_stride;
  const bf16_t* k_cache;
  const bf16_t* v_cache;
  const int32_t* block_tables;  // [num_seqs, bt_stride] page ids of this group
  int bt_stride;
  const int32_t* context_lens;  // [num_seqs] keys visible after this step's write
  const int32_t* cu_seqlens;    // prefill: [num_seqs + 1] prefix sums of new tokens
  int num_seqs;
  int Hq, Hkv, G;
  int page, page_shift;         // page_shift >= 0 iff page is a power of two
  float scale;
  int window;                   // 0: all keys
  int tok_tile;                 // prefill: query tokens per workgroup
  int part_size;                // decode: keys per partition (multiple of 32)
  int num_parts;                // decode: partitions launched
  float* tmp_out;               // [num_seqs, Hq, num_parts, HD] unnormalised
  float* tmp_m;                 // [num_seqs, Hq, num_parts]
  float* tmp_l;
};

__device__ __forceinline__ bf16x8 zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = static_cast<bf16_t>(0.f);
  return z;
}
__device__ __forceinline__ bf16x8 ld8(const bf16_t* p) { return *reinterpret_cast<const bf16x8*>(p); }

__device__ __forceinline__ int page_index(int tok, int page, int shift) {
  return shift >= 0 ? (tok >> shift) : (tok / page);
}

// One 32-key block [t0, t0+32) against this wave's 16 columns.
//   n = lane & 15 (column for B operands / row for A operands), g = lane >> 4.
//   col_hi: last key position this lane's column may see (-1: column unused);
//   col_lo: first key position it may see. lo_min: smallest col_lo of the whole call site, a
//   bound below which pages may already have been given back (never loaded).
__device__ __forceinline__ void attend32(const AttnArgs& a, const int32_t* __restrict__ bt, int kvh,
                                         int t0, int L, int lo_min, const bf16x8 (&qb)[KS],
                                         int col_lo, int col_hi, float& m, float& l,
                                         f32x4 (&acc)[DT], int n, int g) {
  // ---- scores: two 16-key tiles, rows permuted as described above
  const int kgrp = t0 + 8 * (n >> 2);
  bool kgrp_ok = kgrp < L && kgrp + 7 >= lo_min;
  int kpi = 0, kpage = 0;
  if (kgrp_ok) {
    kpi = page_index(kgrp, a.page, a.page_shift);
    kpage = bt[kpi];
    kgrp_ok = kpage >= 0;  // a page that is not held is never dereferenced
  }
  const int koff = kgrp - kpi * a.page + (n & 3);
  f32x4 st[2];
#pragma unroll
  for (int tt = 0; tt < 2; ++tt) {
    const int tok = kgrp + (n & 3) + 4 * tt;
    const bool ok = kgrp_ok && tok < L;
    const bf16_t* kp = a.k_cache + (((int64_t)kpage * a.Hkv + kvh) * a.page + koff + 4 * tt) * HD + 8 * g;
    f32x4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const bf16x8 ka = (ok && (32 * ks + 8 * g) < HD) ? ld8(kp + 32 * ks) : zero8();
      s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka, qb[ks], s, 0, 0, 0);
    }
    st[tt] = s;
  }

  // ---- V^T operands (issued before the softmax arithmetic so the loads overlap it)
  const int vgrp = t0 + 8 * g;
  bool vgrp_ok = vgrp < L && vgrp + 7 >= lo_min;
  int vpi = 0, vpage = 0;
  if (vgrp_ok) {
    vpi = page_index(vgrp, a.page, a.page_shift);
    vpage = bt[vpi];
    vgrp_ok = vpage >= 0;
  }
  const bf16_t* vp = a.v_cache + (((int64_t)vpage * a.Hkv + kvh) * HD + n) * a.page + (vgrp - vpi * a.page);
  bf16x8 va[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) va[dt] = vgrp_ok ? ld8(vp + (int64_t)dt * 16 * a.page) : zero8();
  if (vgrp_ok && vgrp + 8 > L) {  // tail: keys at or past L hold foreign or unwritten data
    const int nv = L - vgrp;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int i = 0; i < 8; ++i)
        if (i >= nv) va[dt][i] = static_cast<bf16_t>(0.f);
  }

  // ---- mask, running max, probabilities (this lane: keys t0+8g+0..7 of column n)
  float s[8];
  bool keep[8];
  float bm = NEG;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int j = t0 + 8 * g + i;
    keep[i] = j <= col_hi && j >= col_lo;
    s[i] = keep[i] ? st[i >> 2][i & 3] * a.scale : NEG;
    bm = fmaxf(bm, s[i]);
  }
  bm = fmaxf(bm, __shfl_xor(bm, 16, ME_WAVE));
  bm = fmaxf(bm, __shfl_xor(bm, 32, ME_WAVE));
  const float m_new = fmaxf(m, bm);
  const float alpha = __expf(m - m_new);
  float psum = 0.f;
  bf16x8 pb;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const float p = keep[i] ? __expf(s[i] - m_new) : 0.f;
    psum += p;
    pb[i] = static_cast<bf16_t>(p);
  }
  l = l * alpha + psum;  // this lane's share of the column's sum; the 4 shares are added at the end
  m = m_new;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) {
    f32x4 o = acc[dt];
    o[0] *= alpha; o[1] *= alpha; o[2] *= alpha; o[3] *= alpha;
    acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va[dt], pb, o, 0, 0, 0);
  }
}

__device__ __forceinline__ void load_q(const bf16_t* qrow, bool valid, int g, bf16x8 (&qb)[KS]) {
#pragma unroll
  for (int ks = 0; ks < KS; ++ks)
    qb[ks] = (valid && (32 * ks + 8 * g) < HD) ? ld8(qrow + 32 * ks + 8 * g) : zero8();
}

__device__ __forceinline__ float column_sum(float l) {
  l += __shfl_xor(l, 16, ME_WAVE);
  l += __shfl_xor(l, 32, ME_WAVE);
  return l;
}

// =====================================================================================
// Prefill / chunk kernel: each wave owns 16 columns of a (tok_tile tokens x G heads) tile of
// one sequence and one kv head, and walks the keys [lo, hi) its columns may see.
// Grid: (floor(T / tok_tile) + num_seqs, Hkv). The first tile of sequence b is
// floor(cu[b] / tok_tile) + b, an upper bound of the tiles before it; surplus tiles exit.
// =====================================================================================
__global__ void __launch_bounds__(256) attn_prefill_kernel(AttnArgs a) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n = lane & 15, g = lane >> 4;
  const int kvh = blockIdx.y;
  const int x = blockIdx.x;
  // largest b with first_tile(b) <= x
  int lo_b = 0, hi_b = a.num_seqs - 1;
  while (lo_b < hi_b) {
    const int mid = (lo_b + hi_b + 1) >> 1;
    if (a.cu_seqlens[mid] / a.tok_tile + mid <= x) lo_b = mid; else hi_b = mid - 1;
  }
  const int b = lo_b;
  const int q0 = a.cu_seqlens[b], q_len = a.cu_seqlens[b + 1] - q0;
  const int local = x - (q0 / a.tok_tile + b);
  const int tok0 = local * a.tok_tile;
  if (tok0 >= q_len) return;
  const int L = a.context_lens[b];
  const int start = L - q_len;  // position of the sequence's first new token
  const int32_t* bt = a.block_tables + (int64_t)b * a.bt_stride;
  const int tile_tokens = min(a.tok_tile, q_len - tok0);
  const int ncols = tile_tokens * a.G;
  const int tile_lo = a.window > 0 ? max(0, start + tok0 - a.window + 1) : 0;

  for (int ct = wave; ct * 16 < ncols; ct += 4) {
    const int c = ct * 16 + n;
    const bool valid = c < ncols;
    const int tl = valid ? c / a.G : 0;
    const int hh = c - tl * a.G;
    const int64_t t = q0 + tok0 + tl;
    const int head = kvh * a.G + hh;
    const int pos = start + tok0 + tl;
    const int col_hi = valid ? pos : -1;
    const int col_lo = a.window > 0 ? max(0, pos - a.window + 1) : 0;
    bf16x8 qb[KS];
    load_q(a.q + t * a.q_stride + (int64_t)head * HD, valid, g, qb);
    // keys this wave needs: from the window start of its first column to its last column's position
    const int c_first = ct * 16, c_last = min(ncols, ct * 16 + 16) - 1;
    const int pos_first = start + tok0 + c_first / a.G, pos_last = start + tok0 + c_last / a.G;
    const int w_lo = a.window > 0 ? max(0, pos_first - a.window + 1) : 0;
    float m = NEG, l = 0.f;
    f32x4 acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) acc[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int t0 = w_lo & ~31; t0 <= pos_last; t0 += 32)
      attend32(a, bt, kvh, t0, L, tile_lo, qb, col_lo, col_hi, m, l, acc, n, g);
    l = column_sum(l);
    if (valid) {
      const float inv = l > 0.f ? 1.f / l : 0.f;
      bf16_t* o = a.out + t * a.out_stride + (int64_t)head * HD + 4 * g;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        bf16x4 r;
#pragma unroll
        for (int i = 0; i < 4; ++i) r[i] = static_cast<bf16_t>(acc[dt][i] * inv);
        *reinterpret_cast<bf16x4*>(o + 16 * dt) = r;
      }
    }
  }
}

// =====================================================================================
// Decode kernel: one query token per sequence. Grid (num_seqs, Hkv * col_tiles, num_parts);
// the 4 waves of a workgroup take the 32-key blocks of the partition in turn and are merged
// through LDS. With one partition the result is written directly; otherwise the partition's
// (max, sum, unnormalised output) go to scratch for the reduce kernel.
// =====================================================================================
__global__ void __launch_bounds__(256) attn_decode_kernel(AttnArgs a) {
  extern __shared__ float lds[];  // [4 waves][16 cols][HD + 2]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n = lane & 15, g = lane >> 4;
  const int b = blockIdx.x;
  const int col_tiles = (a.G + 15) / 16;
  const int kvh = blockIdx.y / col_tiles, ctile = blockIdx.y - kvh * col_tiles;
  const int part = blockIdx.z;
  const int L = a.context_lens[b];
  const int pos = L - 1;
  const int lo = a.window > 0 ? max(0, pos - a.window + 1) : 0;
  const int32_t* bt = a.block_tables + (int64_t)b * a.bt_stride;
  const int hh = ctile * 16 + n;
  const bool valid = hh < a.G;
  const int head = kvh * a.G + (valid ? hh : 0);
  const int64_t t = b;  // decode rows come first in the batch: token index == sequence index

  bf16x8 qb[KS];
  load_q(a.q + t * a.q_stride + (int64_t)head * HD, valid, g, qb);
  float m = NEG, l = 0.f;
  f32x4 acc[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) acc[dt] = f32x4{0.f, 0.f, 0.f, 0.f};

  const int p_lo = max(part * a.part_size, lo & ~31);
  const int p_hi = min((part + 1) * a.part_size, L);
  for (int t0 = p_lo + 32 * wave; t0 < p_hi; t0 += 128)
    attend32(a, bt, kvh, t0, L, lo, qb, lo, valid ? pos : -1, m, l, acc, n, g);
  l = column_sum(l);

  // ---- merge the 4 waves
  const int stride = HD + 2;
  float* mine = lds + ((wave * 16 + n) * stride);
  if (g == 0) { mine[HD] = m; mine[HD + 1] = l; }
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int i = 0; i < 4; ++i) mine[16 * dt + 4 * g + i] = acc[dt][i];
  __syncthreads();
  // thread -> (column, channel) pairs
  const int ncols = min(16, a.G - ctile * 16);
  for (int e = threadIdx.x; e < ncols * HD; e += 256) {
    const int c = e / HD, d = e - c * HD;
    float M = NEG;
#pragma unroll
    for (int w = 0; w < 4; ++w) M = fmaxf(M, lds[(w * 16 + c) * stride + HD]);
    float o = 0.f, ls = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float f = __expf(lds[(w * 16 + c) * stride + HD] - M);
      o += f * lds[(w * 16 + c) * stride + d];
      ls += f * lds[(w * 16 + c) * stride + HD + 1];
    }
    const int hq = kvh * a.G + ctile * 16 + c;
    if (a.num_parts == 1) {
      a.out[t * a.out_stride + (int64_t)hq * HD + d] = static_cast<bf16_t>(ls > 0.f ? o / ls : 0.f);
    } else {
      const int64_t row = ((int64_t)b * a.Hq + hq) * a.num_parts + part;
      a.tmp_out[row * HD + d] = o;
      if (d == 0) { a.tmp_m[row] = M; a.tmp_l[row] = ls; }
    }
  }
}

// Reduce over partitions: out = sum_p e^{m_p - M} o_p / sum_p e^{m_p - M} l_p. Grid (num_seqs, Hq).
__global__ void attn_reduce_kernel(AttnArgs a) {
  const int b = blockIdx.x, hq = blockIdx.y;
  const int64_t row0 = ((int64_t)b * a.Hq + hq) * a.num_parts;
  float M = NEG;
  for (int p = 0; p < a.num_parts; ++p) M = fmaxf(M, a.tmp_m[row0 + p]);
  float ls = 0.f;
  for (int p = 0; p < a.num_parts; ++p) ls += __expf(a.tmp_m[row0 + p] - M) * a.tmp_l[row0 + p];
  const float inv = ls > 0.f ? 1.f / ls : 0.f;
  for (int d = threadIdx.x; d < HD; d += blockDim.x) {
    float o = 0.f;
    for (int p = 0; p < a.num_parts; ++p) o += __expf(a.tmp_m[row0 + p] - M) * a.tmp_out[(row0 + p) * HD + d];
    a.out[(int64_t)b * a.out_stride + (int64_t)hq * HD + d] = static_cast<bf16_t>(o * inv);
  }
}

// =====================================================================================
// Host side
// =====================================================================================
#include "errors.inc"

extern "C" int me_attn_head_dim() { return HD; }

static int fill_common(AttnArgs& a, const void* q, int64_t q_stride, void* out, int64_t out_stride,
                       const void* k_cache, const void* v_cache, const int32_t* block_tables, int bt_stride,
                       const int32_t* context_lens, int num_seqs, int Hq, int Hkv, int page, float scale,
                       int window) {
  ME_CHECK(Hq >= 1 && Hkv >= 1 && Hq % Hkv == 0, "attention: %d query heads are not a multiple of %d key heads", Hq, Hkv);
  ME_CHECK(page >= 8 && page % 8 == 0, "attention (bf16 MFMA path): page size %d must be a multiple of 8", page);
  ME_CHECK(q_stride % 8 == 0 && out_stride % 4 == 0, "attention: token strides must keep 16-byte alignment");
  ME_CHECK((reinterpret_cast<uintptr_t>(q) % 16 == 0) && (reinterpret_cast<uintptr_t>(out) % 8 == 0) &&
               (reinterpret_cast<uintptr_t>(k_cache) % 16 == 0) && (reinterpret_cast<uintptr_t>(v_cache) % 16 == 0),
           "attention: q, out and cache pointers must be 16-byte aligned");
  ME_CHECK(window >= 0 && bt_stride >= 1, "attention: bad window or block-table stride");
  a.q = (const bf16_t*)q; a.q_stride = q_stride; a.out = (bf16_t*)out; a.out_stride = out_stride;
  a.k_cache = (const bf16_t*)k_cache; a.v_cache = (const bf16_t*)v_cache;
  a.block_tables = block_tables; a.bt_stride = bt_stride; a.context_lens = context_lens;
  a.cu_seqlens = nullptr; a.num_seqs = num_seqs; a.Hq = Hq; a.Hkv = Hkv; a.G = Hq / Hkv;
  a.page = page; a.page_shift = -1;
  for (int s = 0; s < 31; ++s) if ((1 << s) == page) a.page_shift = s;
  a.scale = scale; a.window = window; a.tok_tile = 1; a.part_size = 0; a.num_parts = 1;
  a.tmp_out = a.tmp_m = a.tmp_l = nullptr;
  return 0;
}

// q/out point at the first prefill token; cu_seqlens are relative to it; block_tables and
// context_lens at the first prefill sequence.
extern "C" int me_attn_prefill(const void* q, int64_t q_stride, void* out, int64_t out_stride,
                               const void* k_cache, const void* v_cache, const int32_t* block_tables,
                               int bt_stride, const int32_t* context_lens, const int32_t* cu_seqlens,
                               int num_seqs, int64_t num_tokens, int Hq, int Hkv, int page, float scale,
                               int window, hipStream_t stream) {
  if (num_seqs == 0 || num_tokens == 0) return 0;
  AttnArgs a;
  if (fill_common(a, q, q_stride, out, out_stride, k_cache, v_cache, block_tables, bt_stride, context_lens,
                  num_seqs, Hq, Hkv, page, scale, window)) return -1;
  a.cu_seqlens = cu_seqlens;
  a.tok_tile = a.G >= 64 ? 1 : 64 / a.G;
  const int64_t tiles = num_tokens / a.tok_tile + num_seqs;
  ME_CHECK(tiles < (1ll << 31), "attention: too many tiles");
  attn_prefill_kernel<<<dim3((unsigned)tiles, Hkv), dim3(256), 0, stream>>>(a);
  ME_LAUNCH_CHECK();
  return 0;
}

// Bytes of scratch the decode path needs for (num_seqs, Hq, num_parts): out, m, l.
extern "C" int64_t me_attn_decode_scratch_floats(int num_seqs, int Hq, int num_parts) {
  return (int64_t)num_seqs * Hq * num_parts * (HD + 2);
}

extern "C" int me_attn_decode(const void* q, int64_t q_stride, void* out, int64_t out_stride,
                              const void* k_cache, const void* v_cache, const int32_t* block_tables,
                              int bt_stride, const int32_t* context_lens, int num_seqs, int Hq, int Hkv,
                              int page, float scale, int window, int part_size, int num_parts,
                              float* scratch, hipStream_t stream) {
  if (num_seqs == 0) return 0;
  AttnArgs a;
  if (fill_common(a, q, q_stride, out, out_stride, k_cache, v_cache, block_tables, bt_stride, context_lens,
                  num_seqs, Hq, Hkv, page, scale, window)) return -1;
  ME_CHECK(num_parts >= 1 && num_parts <= 65535, "attention: %d partitions outside 1..65535", num_parts);
  ME_CHECK(num_parts == 1 || (part_size >= 32 && part_size % 32 == 0),
           "attention: partition size %d must be a multiple of 32", part_size);
  ME_CHECK(num_parts == 1 || scratch != nullptr, "attention: split decode needs scratch");
  a.part_size = num_parts == 1 ? (1 << 30) : part_size;
  a.num_parts = num_parts;
  if (num_parts > 1) {
    const int64_t rows = (int64_t)num_seqs * Hq * num_parts;
    a.tmp_out = scratch; a.tmp_m = scratch + rows * HD; a.tmp_l = a.tmp_m + rows;
  }
  const int col_tiles = (a.G + 15) / 16;
  ME_CHECK((int64_t)Hkv * col_tiles <= 65535, "attention: too many heads for one launch");
  const size_t lds = (size_t)4 * 16 * (HD + 2) * sizeof(float);
  static bool attr_set = false;
  if (lds > 64 * 1024 && !attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)attn_decode_kernel,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    ME_CHECK(e == hipSuccess, "attention: cannot get %zu bytes of LDS: %s", lds, hipGetErrorString(e));
    attr_set = true;
  }
  attn_decode_kernel<<<dim3(num_seqs, Hkv * col_tiles, num_parts), dim3(256), lds, stream>>>(a);
  ME_LAUNCH_CHECK();
  if (num_parts > 1) {
    attn_reduce_kernel<<<dim3(num_seqs, Hq), dim3(HD >= 128 ? 128 : 64), 0, stream>>>(a);
    ME_LAUNCH_CHECK();
  }
  return 0;
}

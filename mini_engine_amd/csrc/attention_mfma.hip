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
#include <cstdlib>

#ifndef ME_HEAD_DIM
#error "compile with -DME_HEAD_DIM=<multiple of 16>"
#endif
static_assert(ME_HEAD_DIM % 16 == 0 && ME_HEAD_DIM >= 16 && ME_HEAD_DIM <= 512, "head size");

constexpr int HD = ME_HEAD_DIM;
constexpr int KS = (HD + 31) / 32;  // 32-channel steps of the score product
constexpr int DT = HD / 16;         // 16-channel tiles of the output
constexpr float NEG = -1e30f;       // "no key yet": finite, so that differences never give NaN
// log2 units by which the max must rise before the accumulators are rescaled (0: follow the max exactly). With a
// step of 8 the reference point of the exponentials lags the running max by up to 8, so probabilities reach 2^8
// instead of 1 (harmless: the sums are float32, bfloat16's precision is relative, and sums and outputs share the
// reference point), and after the first blocks of a tile hardly any block rescales: a prompt of 2,048 tokens at
// 16x128 heads 58.3 -> 50.6 us, of 8,192 tokens 466 -> 378 us, of 32,768 tokens 5.39 -> 5.24 ms.
constexpr float RESCALE_STEP = 8.f;

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
  int page, page_shift;         // page = 1 << page_shift
  float scale;
  int window;                   // 0: all keys
  int tok_tile;                 // prefill: query tokens per workgroup
  int part_size;                // decode: keys per partition (multiple of 32)
  int num_parts;                // decode: partitions launched
  int spread_heads;             // decode: grid (heads, sequences, partitions) instead of (sequences, heads, partitions)
  float* tmp_out;               // [num_seqs, Hq, num_parts, HD] unnormalised
  float* tmp_m;                 // [num_seqs, Hq, num_parts]
  float* tmp_l;
  // prefill: a tile whose keys span more than seg_keys is cut into segments handled by different
  // workgroups (grid z); their partial results go to pf_scratch and are merged by a second kernel
  int seg_keys;                 // 0: no cutting; else a multiple of 32
  int max_segs;
  float* pf_scratch;            // [tokens, Hq, max_segs, HD + 2]: unnormalised output, max (log2 domain), sum
  const int32_t* seq_of_token;  // prefill: [tokens] index of the token's sequence among the prefill sequences + seq_base
  int seq_base;
  // decode with the step's prologue inside (attn_decode_kernel<true>): q and the new token's key and value are
  // taken as the packed projection left them; the kernel norms and rotates q and the key itself, attends to the
  // new key and value from LDS, and writes them to their place in the pages
  const bf16_t* raw_k;          // token 0's first key head in the packed row (token stride q_stride)
  const bf16_t* raw_v;
  const float* q_w;             // per-head RMSNorm weights [HD], or both nullptr: no norm
  const float* k_w;
  float eps;
  const float* rope;            // [positions, HD/2, 2] (cos, sin), or nullptr: no rotation
  bf16_t* k_cache_w;
  bf16_t* v_cache_w;
};

// Key range of the tile that holds new token `tl` (index within its sequence's new tokens) and the
// number of segments it is cut into; shared by the prefill kernel and the merge kernel.
struct TileRange {
  int tok0, tile_tokens, tile_lo, tile_base, pos_last, nseg;
};
__device__ __forceinline__ TileRange tile_range(const AttnArgs& a, int tok0, int q_len, int L) {
  TileRange r;
  const int start = L - q_len;
  r.tok0 = tok0;
  r.tile_tokens = min(a.tok_tile, q_len - tok0);
  r.tile_lo = a.window > 0 ? max(0, start + tok0 - a.window + 1) : 0;
  r.tile_base = r.tile_lo & ~31;
  r.pos_last = start + tok0 + r.tile_tokens - 1;
  // never more than the scratch has room for: the last segment then runs to the tile's end
  r.nseg = a.seg_keys > 0 ? min((r.pos_last + 1 - r.tile_base + a.seg_keys - 1) / a.seg_keys, a.max_segs) : 1;
  return r;
}

__device__ __forceinline__ bf16x8 zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = static_cast<bf16_t>(0.f);
  return z;
}
__device__ __forceinline__ bf16x8 ld8(const bf16_t* p) { return *reinterpret_cast<const bf16x8*>(p); }
// The same for data that is read once (a decode step's keys and values): marked as not to be kept by the caches,
// which this GPU's memory system answers with a higher rate (a plain read of 4 GB: 5.2-6.4 TB/s, marked 5.7-7.3).
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
template <bool STREAM>
__device__ __forceinline__ bf16x8 ld8s(const bf16_t* p) {
  if constexpr (STREAM) {
    const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
    return __builtin_bit_cast(bf16x8, v);
  } else {
    return ld8(p);
  }
}

// Max / sum over the four lanes n, n+16, n+32, n+48 that share a column, left in all four.
// v_permlane16_swap exchanges the odd 16-lane rows of its first operand with the even rows of
// its second, v_permlane32_swap the upper half of the first with the lower half of the second;
// with both operands equal, the two results hold the two partners of every lane.
__device__ __forceinline__ float max_over_groups(float v) {
  unsigned u = __float_as_uint(v);
  auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  v = fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
  u = __float_as_uint(v);
  auto r2 = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return fmaxf(__uint_as_float(r2[0]), __uint_as_float(r2[1]));
}
__device__ __forceinline__ float sum_over_groups(float v) {
  unsigned u = __float_as_uint(v);
  auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  v = __uint_as_float(r[0]) + __uint_as_float(r[1]);
  u = __float_as_uint(v);
  auto r2 = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __uint_as_float(r2[0]) + __uint_as_float(r2[1]);
}


// -------------------------------------------------------------------------------------
// A 32-key block [t0, t0+32) of one kv head, as the operands of the two products.
//   n = lane & 15 (row of an A operand), g = lane >> 4 (its 8-wide k-slot group).
// Loads are unconditional: a lane whose keys are not to be read (at or past the context
// length L, in a page behind a window that was given back, or in a table entry that holds no
// page) reads from page 0 instead, which is always mapped, and its values are replaced by
// zeros when they are used. So no load hides behind a branch and all of a block's loads are
// in flight together; callers fetch the next block while they compute on the current one.
// lo_min: a bound below which pages may already have been given back (never loaded).
// -------------------------------------------------------------------------------------
struct KVBlock {   // the keys of a block: fetched one block ahead of their use
  bf16x8 k[2][KS];
  bool kok[2];
  // where the block's values are (looked up with the keys' pages, fetched when the block is used:
  // they are needed only after the scores and the softmax, which cover their latency)
  int vpage, voff;
  int vkeys;  // how many of this lane's 8 keys of the V operand may be used (0: none)
};
struct VBlock {
  bf16x8 v[DT];
  uint32_t vmask[4];  // per 32-bit pair of this lane's 8 keys: which halves lie before L in a held page
};

// Page ids of a block, looked up one block before its keys and values are fetched, so that the
// table read and the reads it addresses are not one chain of two latencies.
struct BlockPages {
  int kpage, koff, vpage, voff;  // kpage/vpage: table entries as loaded, not yet looked at
  bool kgrp_ok, vgrp_ok;
};

// Only issues the two table reads; nothing here depends on what they return, so no wait is
// placed behind them (a wait would also stall on every key/value load issued before).
__device__ __forceinline__ void lookup_pages(const AttnArgs& a, const int32_t* __restrict__ bt, int t0, int L,
                                             int lo_min, int n, int g, BlockPages& pg) {
  const int kgrp = t0 + 8 * (n >> 2);
  pg.kgrp_ok = kgrp < L && kgrp + 7 >= lo_min;
  const int kpi = pg.kgrp_ok ? (kgrp >> a.page_shift) : 0;
  pg.kpage = bt[kpi];
  pg.koff = pg.kgrp_ok ? kgrp - kpi * a.page + (n & 3) : (n & 3);
  const int vgrp = t0 + 8 * g;
  pg.vgrp_ok = vgrp < L && vgrp + 7 >= lo_min;
  const int vpi = pg.vgrp_ok ? (vgrp >> a.page_shift) : 0;
  pg.vpage = bt[vpi];
  pg.voff = pg.vgrp_ok ? vgrp - vpi * a.page : 0;
}

template <bool STREAM = false>
__device__ __forceinline__ void load_kv(const AttnArgs& a, const BlockPages& pg, int kvh, int t0, int L, int n,
                                        int g, KVBlock& blk) {
  // a table entry that holds no page (-1) is treated like a key past the context: page 0, zeros
  const bool kgrp_ok = pg.kgrp_ok && pg.kpage >= 0;
  const int kpage = kgrp_ok ? pg.kpage : 0;
  const int koff = kgrp_ok ? pg.koff : (n & 3);
  // K rows: tile tt holds keys t0 + 8*(n/4) + 4*tt + (n%4)
  const int kgrp = t0 + 8 * (n >> 2);
#pragma unroll
  for (int tt = 0; tt < 2; ++tt) {
    blk.kok[tt] = kgrp_ok && (kgrp + (n & 3) + 4 * tt) < L;
    const bf16_t* kp = a.k_cache + (((int64_t)kpage * a.Hkv + kvh) * a.page + koff + 4 * tt) * HD;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d0 = 32 * ks + 8 * g;
      blk.k[tt][ks] = ld8s<STREAM>(kp + ((HD % 32 == 0 || d0 < HD) ? d0 : 0));
    }
  }
  const bool vgrp_ok = pg.vgrp_ok && pg.vpage >= 0;
  blk.vpage = vgrp_ok ? pg.vpage : 0;
  blk.voff = vgrp_ok ? pg.voff : 0;
  blk.vkeys = vgrp_ok ? L - (t0 + 8 * g) : 0;
}

// Makes the block's value-page fields exist in registers of their own from here on. They are
// selects on the table entry that lookup_pages fetched; left alone, the compiler forms them where
// they are used (when the values are fetched, late in a loop iteration), keeps the raw entry alive
// until then, and must copy the next lookup's result into its register at the end of the
// iteration, which waits for every load in flight.
__device__ __forceinline__ void settle_value_page(KVBlock& blk) {
  asm volatile("" : "+v"(blk.vpage), "+v"(blk.voff), "+v"(blk.vkeys));
}

// V^T rows: channel 16*dt + n, keys t0 + 8g .. t0 + 8g + 7
template <bool STREAM = false>
__device__ __forceinline__ void load_v(const AttnArgs& a, const KVBlock& blk, int kvh, int t0, int L, int n, int g,
                                       VBlock& vb) {
  const bf16_t* vp = a.v_cache + (((int64_t)blk.vpage * a.Hkv + kvh) * HD + n) * a.page + blk.voff;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) vb.v[dt] = ld8s<STREAM>(vp + (int64_t)dt * 16 * a.page);
  // keys at or past L hold foreign or unwritten data (possibly NaN): their bits are cleared
  const int nv = blk.vkeys;
#pragma unroll
  for (int j = 0; j < 4; ++j)
    vb.vmask[j] = (2 * j < nv ? 0x0000ffffu : 0u) | (2 * j + 1 < nv ? 0xffff0000u : 0u);
}

template <bool STREAM = false>
__device__ __forceinline__ void load_block(const AttnArgs& a, const int32_t* __restrict__ bt, int kvh, int t0,
                                           int L, int lo_min, int n, int g, KVBlock& blk) {
  BlockPages pg;
  lookup_pages(a, bt, t0, L, lo_min, n, g, pg);
  load_kv<STREAM>(a, pg, kvh, t0, L, n, g, blk);
}

// Scores of the block against one 16-column tile, online-softmax update, and P.V.
//   col_lo..col_hi: key positions this lane's column may see (col_hi = -1: column unused).
//   The running max m is kept in the log2 domain: m = max(score) * c, c = scale * log2(e), so a
//   probability is exp2(score * c - m): one fused multiply-add and one v_exp per score.
//   FULL: every key of the block is visible to every column of the wave and lies before L in a
//   held page, so nothing is masked or zeroed. Otherwise scores outside [col_lo, col_hi] are
//   replaced, K rows and V keys that must not be read are zeroed.
//   The accumulators are rescaled only when some column's max has risen (a wave-wide test).
template <bool FULL>
__device__ __forceinline__ void attend_block(const AttnArgs& a, const KVBlock& blk, const VBlock& vblk, int t0,
                                             const bf16x8 (&qb)[KS], int col_lo, int col_hi, float& m, float& l,
                                             f32x4 (&acc)[DT], int g) {
  const bf16x8 z = zero8();
  const float c = a.scale * 1.4426950408889634f;
  f32x4 st[2];
#pragma unroll
  for (int tt = 0; tt < 2; ++tt) {
    f32x4 sacc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const bool dok = HD % 32 == 0 || (32 * ks + 8 * g) < HD;
      const bf16x8 ka = ((FULL || blk.kok[tt]) && dok) ? blk.k[tt][ks] : z;
      sacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka, qb[ks], sacc, 0, 0, 0);
    }
    st[tt] = sacc;
  }
  // this lane: keys t0+8g+0..7 of its column
  float sv[8];
  float bm = NEG;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    sv[i] = st[i >> 2][i & 3];
    if (!FULL) {
      const int j = t0 + 8 * g + i;
      sv[i] = (j <= col_hi && j >= col_lo) ? sv[i] : NEG;
    }
    bm = fmaxf(bm, sv[i]);
  }
  bm = max_over_groups(bm);
  // The reference point m of the exponentials follows the running max lazily: it moves only when
  // the max has risen by more than RESCALE_STEP (in log2 units), so probabilities may reach
  // 2^RESCALE_STEP instead of 1 (harmless in float32 sums and in bfloat16, whose precision is
  // relative) and the accumulators are rescaled rarely. Sums and outputs share the same m, so the
  // result is the same softmax.
  const float m_blk = bm > 0.5f * NEG ? bm * c : NEG;
  const bool rose = m_blk > m + RESCALE_STEP;
  if (__any(rose)) {
    const float m_new = rose ? m_blk : m;
    const float alpha = __builtin_amdgcn_exp2f(m - m_new);
    l *= alpha;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      acc[dt][0] *= alpha; acc[dt][1] *= alpha; acc[dt][2] *= alpha; acc[dt][3] *= alpha;
    }
    m = m_new;
  }
  float psum = 0.f;
  bf16x8 pb;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    float p = __builtin_amdgcn_exp2f(fmaf(sv[i], c, -m));
    if (!FULL) p = sv[i] > 0.5f * NEG ? p : 0.f;
    psum += p;
    pb[i] = static_cast<bf16_t>(p);
  }
  l += psum;  // this lane's share of the column's sum; the 4 shares are added at the end
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) {
    bf16x8 va = vblk.v[dt];
    if (!FULL) {
      typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
      u32x4 vb = __builtin_bit_cast(u32x4, va);
      vb[0] &= vblk.vmask[0]; vb[1] &= vblk.vmask[1]; vb[2] &= vblk.vmask[2]; vb[3] &= vblk.vmask[3];
      va = __builtin_bit_cast(bf16x8, vb);
    }
    acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va, pb, acc[dt], 0, 0, 0);
  }
}

// The three phases of attend_block as separate steps, for a kernel that interleaves them with
// its fetches. hide_keys / hide_values zero, in place, what a block that is not FULL must not use.
__device__ __forceinline__ void hide_keys(KVBlock& blk) {
  const bf16x8 z = zero8();
#pragma unroll
  for (int tt = 0; tt < 2; ++tt)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) blk.k[tt][ks] = blk.kok[tt] ? blk.k[tt][ks] : z;
}
__device__ __forceinline__ void hide_values(VBlock& vb) {
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) {
    u32x4 w = __builtin_bit_cast(u32x4, vb.v[dt]);
    w[0] &= vb.vmask[0]; w[1] &= vb.vmask[1]; w[2] &= vb.vmask[2]; w[3] &= vb.vmask[3];
    vb.v[dt] = __builtin_bit_cast(bf16x8, w);
  }
}
__device__ __forceinline__ void block_scores(const KVBlock& blk, const bf16x8 (&qb)[KS], int g, f32x4 (&st)[2]) {
  const bf16x8 z = zero8();
#pragma unroll
  for (int tt = 0; tt < 2; ++tt) {
    f32x4 sacc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const bool dok = HD % 32 == 0 || (32 * ks + 8 * g) < HD;
      sacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(dok ? blk.k[tt][ks] : z, qb[ks], sacc, 0, 0, 0);
    }
    st[tt] = sacc;
  }
}
// Online-softmax update of one 16-column tile from its block scores (as in attend_block):
// rescales l and acc when some column's max has risen and returns the probabilities as the
// operand of the value product.
template <bool FULL>
__device__ __forceinline__ void block_softmax(const AttnArgs& a, const f32x4 (&st)[2], int t0, int col_lo,
                                              int col_hi, float& m, float& l, f32x4 (&acc)[DT], int g, bf16x8& pb) {
  const float c = a.scale * 1.4426950408889634f;
  float sv[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) sv[i] = st[i >> 2][i & 3];
  if (!FULL) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int j = t0 + 8 * g + i;
      sv[i] = (j <= col_hi && j >= col_lo) ? sv[i] : NEG;
    }
  }
  // The reference point m of a column is shared by its four lanes and moves only when some score of the block
  // lies more than RESCALE_STEP above it. Every lane tests its own 8 scores; only when one of the wave finds such
  // a score is the column's maximum formed across the lanes (the common block needs no exchange between lanes).
  float bm = NEG;
#pragma unroll
  for (int i = 0; i < 8; ++i) bm = fmaxf(bm, sv[i]);
  if (__any(bm > 0.5f * NEG && bm * c > m + RESCALE_STEP)) {
    bm = max_over_groups(bm);
    const float m_blk = bm > 0.5f * NEG ? bm * c : NEG;
    // A branch of the lanes, not of the wave: the lanes that stay out keep their values, so the accumulators are
    // scaled in the registers they are in (written as a choice per wave, the rescaled values get registers of their
    // own and every accumulator is copied in every block that does not rescale).
    if (m_blk > m + RESCALE_STEP) {
      const float alpha = __builtin_amdgcn_exp2f(m - m_blk);
      l *= alpha;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        acc[dt][0] *= alpha; acc[dt][1] *= alpha; acc[dt][2] *= alpha; acc[dt][3] *= alpha;
      }
      m = m_blk;
    }
  }
  float psum = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    // a masked score is NEG: while the column has seen no key m is NEG too, and exp2(NEG * c - NEG)
    // is not 0, hence the select
    float p = __builtin_amdgcn_exp2f(fmaf(sv[i], c, -m));
    if (!FULL) p = sv[i] > 0.5f * NEG ? p : 0.f;
    psum += p;
    pb[i] = static_cast<bf16_t>(p);
  }
  l += psum;
}

__device__ __forceinline__ void load_q(const bf16_t* qrow, bool valid, int g, bf16x8 (&qb)[KS]) {
  const bf16x8 z = zero8();
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    const int d0 = 32 * ks + 8 * g;
    const bool dok = HD % 32 == 0 || d0 < HD;
    const bf16x8 v = ld8(qrow + (dok ? d0 : 0));
    qb[ks] = (valid && dok) ? v : z;
  }
}

__device__ __forceinline__ float column_sum(float l) { return sum_over_groups(l); }

// =====================================================================================
// Prefill / chunk kernel: each wave owns CT tiles of 16 columns of a (tok_tile tokens x G heads)
// tile of one sequence and one kv head, and walks the keys [lo, hi) its columns may see, the next
// block being fetched while the current one is used. Every K/V register serves CT products.
// Grid: (floor(T / tok_tile) + num_seqs) * Hkv. The first tile of sequence b is
// floor(cu[b] / tok_tile) + b, an upper bound of the tiles before it; surplus tiles exit.
// =====================================================================================
// Two waves per SIMD, not more: a third (the narrow form would fit) only adds to the keys and values
// in flight, which then push each other out of the L1 (256 tokens over 8,192 keys: 126 against 88 us).
template <int CT>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) attn_prefill_kernel(AttnArgs a) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n = lane & 15, g = lane >> 4;
  // Workgroups go to the 8 XCDs in turn, each with an L2 of its own: consecutive ids take the kv
  // heads in turn, so that an XCD sees few heads (one, with 8 heads) and their keys stay in its
  // L2. Tiles are taken from the last, which has the longest key range, to the first.
  const int kvh = blockIdx.x % a.Hkv;
  const int x = gridDim.x / a.Hkv - 1 - blockIdx.x / a.Hkv;
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
  const TileRange tr = tile_range(a, tok0, q_len, L);
  const int tile_tokens = tr.tile_tokens;
  const int ncols = tile_tokens * a.G;
  const int tile_lo = tr.tile_lo;
  const int seg = blockIdx.z;
  if (seg >= tr.nseg) return;
  const int seg_lo = a.seg_keys > 0 ? tr.tile_base + seg * a.seg_keys : 0;          // keys [seg_lo, seg_hi)
  const int seg_hi = (a.seg_keys > 0 && seg + 1 < tr.nseg) ? seg_lo + a.seg_keys : (1 << 30);

  for (int c0 = wave * 16 * CT; c0 < ncols; c0 += 4 * 16 * CT) {
    bf16x8 qb[CT][KS];
    int col_lo[CT], col_hi[CT];
    int64_t tq[CT];
    int head[CT];
    bool valid[CT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
      const int c = c0 + 16 * ct + n;
      valid[ct] = c < ncols;
      const int tl = valid[ct] ? c / a.G : 0;
      const int hh = valid[ct] ? c - tl * a.G : 0;
      tq[ct] = q0 + tok0 + tl;
      head[ct] = kvh * a.G + hh;
      const int pos = start + tok0 + tl;
      col_hi[ct] = valid[ct] ? pos : -1;
      col_lo[ct] = a.window > 0 ? max(0, pos - a.window + 1) : 0;
      load_q(a.q + tq[ct] * a.q_stride + (int64_t)head[ct] * HD, valid[ct], g, qb[ct]);
    }
    // keys this wave needs: from the window start of its first column to its last column's position
    const int c_last = min(ncols, c0 + 16 * CT) - 1;
    const int pos_first = start + tok0 + c0 / a.G, pos_last = start + tok0 + c_last / a.G;
    const int w_lo = a.window > 0 ? max(0, pos_first - a.window + 1) : 0;
    float m[CT], l[CT];
    f32x4 acc[CT][DT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
      m[ct] = NEG; l[ct] = 0.f;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) acc[ct][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    // a block all of whose keys every column of this wave sees (below the first column's position,
    // above the last column's window start) needs no masks
    const int full_hi = pos_first - 31;                                   // t0 <= full_hi: all 32 keys visible
    const int full_lo = a.window > 0 ? max(0, pos_last - a.window + 1) : 0;  // t0 >= full_lo: none behind a window
    // One set of key registers and one of value registers, refilled as soon as the products that
    // read them are issued: the next keys arrive behind the softmax and the value product, the next
    // values behind the score product and the softmax. Page ids are looked up a block earlier
    // still. The fetches are unconditional, also past the last block (they then read page 0 and are
    // not used): a fetch behind a branch would make the waits of both paths merge into waits on the
    // newest loads. With single sets two waves fit on a SIMD. (Two sets per wave, the next block
    // fetched whole while this one is used, need more than 256 registers, leave one wave per
    // SIMD, and measured slower at every size: 2,048 tokens 93 against 78 us, 8,192 tokens 689
    // against 668 us.)
    int t0 = max(w_lo & ~31, seg_lo);
    const int last = min(pos_last, seg_hi - 1);      // last key of this wave inside the segment
    if (t0 <= last) {
      KVBlock K;
      VBlock V;
      BlockPages pn;
      // issued in the order of the loop (keys, page ids, values): the waits inside the loop are
      // placed for the worse of the two ways into it, and a different order here would make every
      // iteration wait as if the page ids had been fetched last
      load_block(a, bt, kvh, t0, L, tile_lo, n, g, K);
      settle_value_page(K);
      lookup_pages(a, bt, t0 + 32, L, tile_lo, n, g, pn);
      load_v(a, K, kvh, t0, L, n, g, V);
      // The scores of a block are issued at the end of the iteration before, behind the value
      // products of the block before: the matrix cores then work on both while the vector ALU
      // does the loop's bookkeeping and the first softmax, instead of each waiting for the other.
      bool full = t0 <= full_hi && t0 >= full_lo;
      if (!full) hide_keys(K);
      f32x4 st[CT][2];
#pragma unroll
      for (int ct = 0; ct < CT; ++ct) block_scores(K, qb[ct], g, st[ct]);
      while (true) {
        // here: st = scores of block t0, V = its values (in flight), K free for the next keys
        load_kv(a, pn, kvh, t0 + 32, L, n, g, K);
        settle_value_page(K);
        lookup_pages(a, bt, t0 + 64, L, tile_lo, n, g, pn);
        bf16x8 pb[CT];
        if (full) {
#pragma unroll
          for (int ct = 0; ct < CT; ++ct)
            block_softmax<true>(a, st[ct], t0, col_lo[ct], col_hi[ct], m[ct], l[ct], acc[ct], g, pb[ct]);
        } else {
#pragma unroll
          for (int ct = 0; ct < CT; ++ct)
            block_softmax<false>(a, st[ct], t0, col_lo[ct], col_hi[ct], m[ct], l[ct], acc[ct], g, pb[ct]);
          hide_values(V);
        }
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
#pragma unroll
          for (int dt = 0; dt < DT; ++dt)
            acc[ct][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(V.v[dt], pb[ct], acc[ct][dt], 0, 0, 0);
        load_v(a, K, kvh, t0 + 32, L, n, g, V);
        t0 += 32;
        if (t0 > last) break;
        full = t0 <= full_hi && t0 >= full_lo;
        if (!full) hide_keys(K);
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) block_scores(K, qb[ct], g, st[ct]);
      }
    }
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
      const float ls = column_sum(l[ct]);
      if (valid[ct] && tr.nseg > 1) {      // a segment's share: unnormalised, for the merge kernel
        float* p = a.pf_scratch + (((int64_t)tq[ct] * a.Hq + head[ct]) * a.max_segs + seg) * (HD + 2);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
          *reinterpret_cast<f32x4*>(p + 16 * dt + 4 * g) = acc[ct][dt];
        if (g == 0) { p[HD] = m[ct]; p[HD + 1] = ls; }
      } else if (valid[ct]) {
        const float inv = ls > 0.f ? 1.f / ls : 0.f;
        bf16_t* o = a.out + tq[ct] * a.out_stride + (int64_t)head[ct] * HD + 4 * g;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          bf16x4 r;
#pragma unroll
          for (int i = 0; i < 4; ++i) r[i] = static_cast<bf16_t>(acc[ct][dt][i] * inv);
          *reinterpret_cast<bf16x4*>(o + 16 * dt) = r;
        }
      }
    }
  }
}

// =====================================================================================
// Prefill / chunk kernel, keys and values shared through LDS (head sizes up to 128).
// The four waves of a workgroup need the same 32-key blocks. Fetched by each wave for itself
// they make four times the L2 traffic that the tile needs (the 32 KB L1 cannot hold what four
// waves have in flight), and that traffic, not arithmetic, is what bounds the kernel above. Here
// the 256 threads fetch a block once, each its 16-byte pieces, one block ahead into registers,
// and put it into LDS, from which every wave reads its matrix operands:
//   keys    [32 rows][HD + 8]: row tt*16 + n holds key 8*(n>>2) + 4*tt + (n&3) of the block, the
//           order in which the lanes of an A operand want them (see the top of the file); with
//           the 16 bytes of padding the 16 lanes of a read hit different banks;
//   values  [HD rows][32 + 8]: channel-major as in the cache.
// What must not be used (keys at or past the context, in pages that are not held) is zeroed when
// it is put into LDS. All waves walk the tile's whole key range in step, one barrier per block
// (two LDS buffers); a block outside a wave's own range is masked like any other.
// Same grid and tile geometry as attn_prefill_kernel.
// =====================================================================================
#define PF_KROW (2 * HD + 16)            // bytes per key row in LDS
#define PF_VROW 80                        // bytes per value row in LDS
#define PF_BUF (32 * PF_KROW + HD * PF_VROW)
#define PF_PIECES ((4 * HD + 255) / 256)  // 16-byte pieces of a block's keys (and of its values) per thread

struct StagedBlock {
  bf16x8 k[PF_PIECES], v[PF_PIECES];
  bool kok[PF_PIECES];
  int vkeys[PF_PIECES];
};
struct StagedPages {   // table entries as loaded, for the block after the staged one
  int k[PF_PIECES], v[PF_PIECES];
};

// INSIDE: every key of the block lies before the context length and no page of the sequence has
// been given back (no window), so nothing has to be tested, clamped or zeroed.
template <bool INSIDE>
__device__ __forceinline__ void pf_lookup(const AttnArgs& a, const int32_t* __restrict__ bt, int t0, int L,
                                          int lo_min, int tid, StagedPages& pg) {
#pragma unroll
  for (int j = 0; j < PF_PIECES; ++j) {
    const int p = tid + 256 * j;
    const bool in = p < 4 * HD;
    const int key = t0 + p / (HD / 8);                 // a key row
    const bool kok = in && (INSIDE || (key < L && key >= (lo_min & ~7)));
    pg.k[j] = bt[kok ? key >> a.page_shift : 0];
    const int key0 = t0 + 8 * (p & 3);                 // a group of 8 keys of one channel
    const bool vok = in && (INSIDE || (key0 < L && key0 + 7 >= lo_min));
    pg.v[j] = bt[vok ? key0 >> a.page_shift : 0];
  }
}

template <bool INSIDE>
__device__ __forceinline__ void pf_fetch(const AttnArgs& a, const StagedPages& pg, int kvh, int t0, int L,
                                         int lo_min, int tid, StagedBlock& st) {
  const int64_t page_stride = (int64_t)a.Hkv * a.page * HD;      // elements per page, keys and values alike
#pragma unroll
  for (int j = 0; j < PF_PIECES; ++j) {
    const int p = tid + 256 * j;
    const bool in = p < 4 * HD;
    const int row = p / (HD / 8), ch = p - row * (HD / 8);
    const int key = t0 + row;
    const bool kok = in && (INSIDE || (key < L && key >= (lo_min & ~7) && pg.k[j] >= 0));
    st.kok[j] = kok;
    const bf16_t* kp = a.k_cache + (int64_t)(kok ? pg.k[j] : 0) * page_stride +
                       ((kvh * a.page + (kok ? key & (a.page - 1) : 0)) * HD + 8 * ch);
    st.k[j] = ld8(kp);
    const int d = in ? p >> 2 : 0, key0 = t0 + 8 * (p & 3);
    const bool vok = in && (INSIDE || (key0 < L && key0 + 7 >= lo_min && pg.v[j] >= 0));
    st.vkeys[j] = INSIDE ? 8 : (vok ? L - key0 : 0);
    const bf16_t* vp = a.v_cache + (int64_t)(vok ? pg.v[j] : 0) * page_stride +
                       ((kvh * HD + d) * a.page + (vok ? key0 & (a.page - 1) : 0));
    st.v[j] = ld8(vp);
  }
}

template <bool INSIDE>
__device__ __forceinline__ void pf_commit(const StagedBlock& st, int tid, unsigned char* buf) {
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  const bf16x8 z = zero8();
#pragma unroll
  for (int j = 0; j < PF_PIECES; ++j) {
    const int p = tid + 256 * j;
    if (p < 4 * HD) {
      const int row = p / (HD / 8), ch = p - row * (HD / 8);
      const int lrow = ((row >> 2) & 1) * 16 + ((row & 3) | ((row >> 3) << 2));
      *reinterpret_cast<bf16x8*>(buf + lrow * PF_KROW + 16 * ch) = (INSIDE || st.kok[j]) ? st.k[j] : z;
      u32x4 w = __builtin_bit_cast(u32x4, st.v[j]);
      if (!INSIDE) {
        const int nv = st.vkeys[j];
#pragma unroll
        for (int i = 0; i < 4; ++i) w[i] &= (2 * i < nv ? 0x0000ffffu : 0u) | (2 * i + 1 < nv ? 0xffff0000u : 0u);
      }
      *reinterpret_cast<u32x4*>(buf + 32 * PF_KROW + (p >> 2) * PF_VROW + 16 * (p & 3)) = w;
    }
  }
}

// Blocks start at multiples of 32 keys, so most of a thread's address arithmetic is the same for every
// block: which table entry beyond the block's first its pieces use (pages below 32 keys), and where in
// a page they lie. For blocks that lie wholly inside the context (pf_lookup<true>, pf_fetch<true> in
// meaning) only the block's own part is added: its first table entry, its offset in a page of 32 keys
// or more, the page's base.
struct StagedInvariants {
  int kidx[PF_PIECES], vidx[PF_PIECES];   // table entries beyond (t0 >> page_shift)
  int koff[PF_PIECES], voff[PF_PIECES];   // element offsets inside a page, without the block's own part
};
__device__ __forceinline__ void pf_invariants(const AttnArgs& a, int kvh, int tid, StagedInvariants& iv) {
  const bool small = a.page < 32;
#pragma unroll
  for (int j = 0; j < PF_PIECES; ++j) {
    const int p = tid + 256 * j;
    const bool in = p < 4 * HD;
    const int row = p / (HD / 8), ch = p - row * (HD / 8);
    const int krow = small ? (row & (a.page - 1)) : row;
    iv.kidx[j] = (in && small) ? row >> a.page_shift : 0;
    iv.koff[j] = in ? (kvh * a.page + krow) * HD + 8 * ch : 0;
    const int d = in ? p >> 2 : 0, k8 = 8 * (p & 3);
    iv.vidx[j] = (in && small) ? k8 >> a.page_shift : 0;
    iv.voff[j] = in ? (kvh * HD + d) * a.page + (small ? (k8 & (a.page - 1)) : k8) : 0;
  }
}
__device__ __forceinline__ void pf_lookup_inside(const AttnArgs& a, const int32_t* __restrict__ bt, int t0,
                                                 const StagedInvariants& iv, StagedPages& pg) {
  const int32_t* first = bt + (t0 >> a.page_shift);
#pragma unroll
  for (int j = 0; j < PF_PIECES; ++j) {
    pg.k[j] = first[iv.kidx[j]];
    pg.v[j] = first[iv.vidx[j]];
  }
}
__device__ __forceinline__ void pf_fetch_inside(const AttnArgs& a, const StagedPages& pg, int t0,
                                                const StagedInvariants& iv, StagedBlock& st) {
  const int64_t page_stride = (int64_t)a.Hkv * a.page * HD;
  const int in_page = a.page >= 32 ? (t0 & (a.page - 1)) : 0;      // the same for every thread
  const bf16_t* kbase = a.k_cache + in_page * HD;
  const bf16_t* vbase = a.v_cache + in_page;
#pragma unroll
  for (int j = 0; j < PF_PIECES; ++j) {
    st.kok[j] = true;
    st.vkeys[j] = 8;
    st.k[j] = ld8(kbase + ((int64_t)pg.k[j] * page_stride + iv.koff[j]));
    st.v[j] = ld8(vbase + ((int64_t)pg.v[j] * page_stride + iv.voff[j]));
  }
}

// the LDS writes of this wave done, every wave at the same point, nothing moved across by the compiler
__device__ __forceinline__ void pf_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

template <int CT>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) attn_prefill_shared_kernel(AttnArgs a) {
  extern __shared__ __align__(16) unsigned char pf_lds[];   // [2][PF_BUF]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n = lane & 15, g = lane >> 4;
  const int kvh = blockIdx.x % a.Hkv;
  const int x = gridDim.x / a.Hkv - 1 - blockIdx.x / a.Hkv;
  int lo_b = 0, hi_b = a.num_seqs - 1;
  while (lo_b < hi_b) {
    const int mid = (lo_b + hi_b + 1) >> 1;
    if (a.cu_seqlens[mid] / a.tok_tile + mid <= x) lo_b = mid; else hi_b = mid - 1;
  }
  const int b = lo_b;
  const int q0 = a.cu_seqlens[b], q_len = a.cu_seqlens[b + 1] - q0;
  const int tok0 = (x - (q0 / a.tok_tile + b)) * a.tok_tile;
  if (tok0 >= q_len) return;
  const int L = a.context_lens[b];
  const int start = L - q_len;
  const int32_t* bt = a.block_tables + (int64_t)b * a.bt_stride;
  const TileRange tr = tile_range(a, tok0, q_len, L);
  const int ncols = tr.tile_tokens * a.G;
  const int tile_lo = tr.tile_lo;
  const int seg = blockIdx.z;
  if (seg >= tr.nseg) return;
  const int seg_lo = a.seg_keys > 0 ? tr.tile_base + seg * a.seg_keys : tr.tile_base;
  const int seg_hi = (a.seg_keys > 0 && seg + 1 < tr.nseg) ? seg_lo + a.seg_keys : (1 << 30);
  const int last = min(tr.pos_last, seg_hi - 1);   // the same key range for every wave of the workgroup
  const float c = a.scale * 1.4426950408889634f;
  (void)c;
  StagedInvariants inv;
  pf_invariants(a, kvh, tid, inv);

  // every wave runs every round (a wave without columns in a round masks everything and writes nothing)
  for (int c_base = 0; c_base < ncols; c_base += 4 * 16 * CT) {
    const bool active = c_base + wave * 16 * CT < ncols;
    const int c0 = active ? c_base + wave * 16 * CT : 0;
    bf16x8 qb[CT][KS];
    int col_lo[CT], col_hi[CT];
    int64_t tq[CT];
    int head[CT];
    bool valid[CT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
      const int cc = c0 + 16 * ct + n;
      valid[ct] = active && cc < ncols;
      const int tl = valid[ct] ? cc / a.G : 0;
      const int hh = valid[ct] ? cc - tl * a.G : 0;
      tq[ct] = q0 + tok0 + tl;
      head[ct] = kvh * a.G + hh;
      const int pos = start + tok0 + tl;
      col_hi[ct] = valid[ct] ? pos : -1;
      col_lo[ct] = a.window > 0 ? max(0, pos - a.window + 1) : 0;
      load_q(a.q + tq[ct] * a.q_stride + (int64_t)head[ct] * HD, valid[ct], g, qb[ct]);
    }
    const int c_last = min(ncols, c0 + 16 * CT) - 1;
    const int pos_first = start + tok0 + c0 / a.G, pos_last = start + tok0 + c_last / a.G;
    const int full_hi = active ? pos_first - 31 : -(1 << 30);
    const int full_lo = a.window > 0 ? max(0, pos_last - a.window + 1) : 0;
    float m[CT], l[CT];
    f32x4 acc[CT][DT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
      m[ct] = NEG; l[ct] = 0.f;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) acc[ct][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

    int t0 = seg_lo;
    StagedBlock stg;
    StagedPages pg;
    pf_barrier();                                    // the round before has finished with both buffers
    pf_lookup<false>(a, bt, t0, L, tile_lo, tid, pg);
    pf_fetch<false>(a, pg, kvh, t0, L, tile_lo, tid, stg);
    pf_lookup<false>(a, bt, t0 + 32, L, tile_lo, tid, pg);
    pf_commit<false>(stg, tid, pf_lds);
    int cur = 0;
    while (true) {
      pf_barrier();                                  // block t0 is in buffer cur
      // the next block, into registers; the page ids of the one after it
      const bool inside1 = a.window == 0 && t0 + 64 <= L, inside2 = a.window == 0 && t0 + 96 <= L;
      if (inside1) pf_fetch_inside(a, pg, t0 + 32, inv, stg);
      else pf_fetch<false>(a, pg, kvh, t0 + 32, L, tile_lo, tid, stg);
      if (inside2) pf_lookup_inside(a, bt, t0 + 64, inv, pg);
      else pf_lookup<false>(a, bt, t0 + 64, L, tile_lo, tid, pg);
      const unsigned char* kb = pf_lds + cur * PF_BUF;
      const unsigned char* vb = kb + 32 * PF_KROW;
      const bool full = t0 <= full_hi && t0 >= full_lo;
      f32x4 st[CT][2];
      const bf16x8 z = zero8();
#pragma unroll
      for (int tt = 0; tt < 2; ++tt) {
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) st[ct][tt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const bool dok = HD % 32 == 0 || (32 * ks + 8 * g) < HD;
          bf16x8 ka = *reinterpret_cast<const bf16x8*>(kb + (tt * 16 + n) * PF_KROW + (dok ? 64 * ks + 16 * g : 0));
          ka = dok ? ka : z;
#pragma unroll
          for (int ct = 0; ct < CT; ++ct)
            st[ct][tt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka, qb[ct][ks], st[ct][tt], 0, 0, 0);
        }
      }
      bf16x8 pb[CT];
      if (full) {
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
          block_softmax<true>(a, st[ct], t0, col_lo[ct], col_hi[ct], m[ct], l[ct], acc[ct], g, pb[ct]);
      } else {
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
          block_softmax<false>(a, st[ct], t0, col_lo[ct], col_hi[ct], m[ct], l[ct], acc[ct], g, pb[ct]);
      }
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        const bf16x8 va = *reinterpret_cast<const bf16x8*>(vb + (16 * dt + n) * PF_VROW + 16 * g);
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
          acc[ct][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va, pb[ct], acc[ct][dt], 0, 0, 0);
      }
      if (inside1) pf_commit<true>(stg, tid, pf_lds + (cur ^ 1) * PF_BUF);
      else pf_commit<false>(stg, tid, pf_lds + (cur ^ 1) * PF_BUF);
      cur ^= 1;
      t0 += 32;
      if (t0 > last) break;
    }

#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
      const float ls = column_sum(l[ct]);
      if (valid[ct] && tr.nseg > 1) {
        float* p = a.pf_scratch + (((int64_t)tq[ct] * a.Hq + head[ct]) * a.max_segs + seg) * (HD + 2);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
          *reinterpret_cast<f32x4*>(p + 16 * dt + 4 * g) = acc[ct][dt];
        if (g == 0) { p[HD] = m[ct]; p[HD + 1] = ls; }
      } else if (valid[ct]) {
        const float inv = ls > 0.f ? 1.f / ls : 0.f;
        bf16_t* o = a.out + tq[ct] * a.out_stride + (int64_t)head[ct] * HD + 4 * g;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          bf16x4 r;
#pragma unroll
          for (int i = 0; i < 4; ++i) r[i] = static_cast<bf16_t>(acc[ct][dt][i] * inv);
          *reinterpret_cast<bf16x4*>(o + 16 * dt) = r;
        }
      }
    }
  }
}

#if ME_HEAD_DIM == 128
// =====================================================================================
// Prefill / chunk kernel, keys and values brought into LDS by the memory system itself
// (global_load_lds_dwordx4: every lane names 16 bytes of memory, and the 64 pieces of a wave's
// instruction land in 1 KB of consecutive LDS), head size 128, pages of 16 keys or more.
// Against the form above this takes the staged block out of the registers and the LDS writes out of
// the instruction stream, and lets a block be asked for NB - 1 blocks before its use instead of one:
// in the form above an iteration cannot be shorter than the latency of its loads, which at two
// workgroups per compute unit is what bounds it (1.8 us a block measured, where its matrix and vector
// instructions account for 0.6).
//   keys    8 instructions of 4 key rows (4 x 256 B); instruction i = 4 tt + (n >> 2) holds the rows
//           tt * 16 + n of the operand order (see the top of the file), i.e. the 4 consecutive keys
//           8 (i & 3) + 4 (i >> 2) + 0..3 of the block, and starts at i * (1 KB + 64 B); inside a row
//           the 16-byte piece c lies at position c ^ (row & 3). A read of 16 rows n at one piece then
//           touches 16 different bank groups (the padding separates the instructions, the exchange
//           the rows inside one), and the exchange leaves 4 ks + (g ^ (n & 3)): the pieces of the
//           four ks steps stay 64 bytes apart.
//   values  [2 halves of 16 keys][128 channels][32 B]: an instruction is 32 channel rows of one half,
//           so with pages of 16 keys it reads one page; piece (g & 1) of a row lies at (g & 1) ^ (channel >> 3 & 1).
// A block that reaches beyond the context (the last one of a sequence), or back into pages behind a window that
// may have been given back (the first one of a tile, with pages of 16 keys), is loaded into registers, zeroed where
// it must not be used, and written to the same places.
// =====================================================================================
#define DMA_KINST 1088
#define DMA_KBYTES (8 * DMA_KINST)
#define DMA_VHALF 4096
#define DMA_BUF (DMA_KBYTES + 2 * DMA_VHALF)
#define DMA_NB 3                       // buffers: three workgroups of a compute unit hold 3 x 3 x 16.5 KB of its 160 KB

// 64 x 16 bytes from gbase + voff (bytes, per lane) to LDS at lds_addr + 16 * lane. The write to m0 needs one wait
// state before an instruction that reads it for an LDS address.
// gbase and lds_addr are the same in every lane; the first lane's values are taken so that they lie in scalar
// registers whatever the compiler has concluded about them.
__device__ __forceinline__ void dma16(const bf16_t* gbase, uint32_t voff, uint32_t lds_addr) {
  const uint64_t g = reinterpret_cast<uint64_t>(gbase);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(g >> 32)), lo = __builtin_amdgcn_readfirstlane((uint32_t)g);
  const uint64_t base = (uint64_t)hi << 32 | lo;      // (the builtin returns int: widened as it is, a low half with its top bit set would fill the high half)
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(__builtin_amdgcn_readfirstlane(lds_addr)), "v"(voff), "s"(base) : "memory");
}
template <int N>
__device__ __forceinline__ void dma_wait() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }

// Keeps the reads of a whole operand array where they are written: without it the compiler moves every read
// down to the product that uses it and waits for each in turn.
template <int N>
__device__ __forceinline__ void pin_operands(bf16x8 (&x)[N]) {
#pragma unroll
  for (int i = 0; i < N; ++i) asm volatile("" : "+v"(x[i]));
}
template <int N, int M>
__device__ __forceinline__ void pin_operands(bf16x8 (&x)[N][M]) {
#pragma unroll
  for (int i = 0; i < N; ++i)
#pragma unroll
    for (int j = 0; j < M; ++j) asm volatile("" : "+v"(x[i][j]));
}

// Reads of 16 bytes at addr + 512 i that the compiler does not know to be reads: it neither moves them to their
// use nor waits for them, so lds_reads_done() has to stand between them and the first use of what they return.
// Until then the values must stay in the registers they were read into (a copy or a spill made by the compiler in
// between would move what the registers held before): only for a kernel with registers to spare, which the form
// with two waves per SIMD is (205 of 256; its test compares it bit for bit with the form that reads as usual).
template <int I>
__device__ __forceinline__ void lds_read16_ahead(uint32_t addr, bf16x8 (&x)[DT]) {
  if constexpr (I < DT) {
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(x[I]) : "v"(addr), "n"(512 * I));
    lds_read16_ahead<I + 1>(addr, x);
  }
}
__device__ __forceinline__ void lds_reads_done(bf16x8 (&x)[DT]) {
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  pin_operands(x);
}

// A wave in its softmax goes first when the SIMD chooses whose instruction to issue: its vector instructions are
// what the next products wait for, while a wave that is issuing products needs a slot only every 16 cycles
// (with two waves per SIMD: 2,048 tokens over 8,192 keys 151 -> 142 us, 512 over 8,192 55.0 -> 53.7 us, a prompt of
// 2,048 tokens 45.7 -> 44.1 us; with three it changes nothing).
__device__ __forceinline__ void softmax_priority(bool on) {
  if (on) __builtin_amdgcn_s_setprio(1); else __builtin_amdgcn_s_setprio(0);
}

struct DmaPages { int k, v; };   // the page of this wave's two key instructions and of its two value instructions

template <int CT, int W, bool WINDOW>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(W, W))) attn_prefill_dma_kernel(AttnArgs a) {
  extern __shared__ __align__(16) unsigned char pf_lds[];   // [NB][DMA_BUF]
  constexpr int NB = DMA_NB, PD = NB - 1;                   // PD: blocks asked for ahead of the one in use
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 15, g = lane >> 4;
  const int kvh = blockIdx.x % a.Hkv;
  const int x = gridDim.x / a.Hkv - 1 - blockIdx.x / a.Hkv;
  int lo_b = 0, hi_b = a.num_seqs - 1;
  while (lo_b < hi_b) {
    const int mid = (lo_b + hi_b + 1) >> 1;
    if (a.cu_seqlens[mid] / a.tok_tile + mid <= x) lo_b = mid; else hi_b = mid - 1;
  }
  const int b = lo_b;
  const int q0 = a.cu_seqlens[b], q_len = a.cu_seqlens[b + 1] - q0;
  const int tok0 = (x - (q0 / a.tok_tile + b)) * a.tok_tile;
  if (tok0 >= q_len) return;
  const int L = a.context_lens[b];
  const int start = L - q_len;
  // The table is read through the constant address space: entries are the same for every lane, and only from
  // there does the compiler fetch them with scalar loads, which count apart from the loads into LDS (a vector
  // load would be waited for together with every block on its way).
  typedef const __attribute__((address_space(4))) int32_t* table_ptr;
  const table_ptr bt = (table_ptr)(uintptr_t)(a.block_tables + (int64_t)b * a.bt_stride);
  const TileRange tr = tile_range(a, tok0, q_len, L);
  const int ncols = tr.tile_tokens * a.G;
  const int seg = blockIdx.z;
  if (seg >= tr.nseg) return;
  const int seg_lo = a.seg_keys > 0 ? tr.tile_base + seg * a.seg_keys : tr.tile_base;
  const int seg_hi = (a.seg_keys > 0 && seg + 1 < tr.nseg) ? seg_lo + a.seg_keys : (1 << 30);
  const int last = min(tr.pos_last, seg_hi - 1);   // the same key range for every wave of the workgroup
  const int nblk = (last - seg_lo) / 32 + 1;
  // With a window, pages wholly behind it may have been given back: from the page that holds the tile's first
  // visible key on, every page is held (pages are 16 keys or more, so this is a multiple of 16).
  // (Without a window all of this is known when the kernel is compiled: the tests below cost the common case 2-7 %.)
  const int first_held = WINDOW ? (tr.tile_lo >> a.page_shift) << a.page_shift : 0;
  auto held = [&](int key) { return !WINDOW || key >= first_held; };

  const uint32_t lds0 = (uint32_t)(uintptr_t)pf_lds;
  // what a lane names in memory, relative to its instruction's first byte, and where it reads its operands
  const uint32_t voff_k = (lane >> 4) * 256 + (((lane & 15) ^ (lane >> 4)) * 16);
  const uint32_t voff_v = ((lane >> 1) * a.page + (((lane & 1) ^ ((lane >> 4) & 1)) * 8)) * 2;
  const uint32_t rd_k = (n >> 2) * DMA_KINST + (n & 3) * 256 + ((g ^ (n & 3)) * 16);
  const uint32_t rd_v = DMA_KBYTES + (g >> 1) * DMA_VHALF + n * 32 + (((g & 1) ^ (n >> 3)) * 16);
  const int kg0 = 8 * ((2 * wave) & 3) + 4 * (wave >> 1);   // first key of this wave's first key instruction; the second: + 8
  const int vh = wave >> 1, vrow0 = 64 * (wave & 1);        // this wave's value instructions: half vh, channel rows vrow0 + 32 j
  const uint32_t page_elems = (uint32_t)(a.Hkv * a.page * HD);                 // elements of a page, keys and values alike
  const bf16_t* k_head = a.k_cache + (int64_t)kvh * a.page * HD;
  const bf16_t* v_head = a.v_cache + ((int64_t)kvh * HD + vrow0) * a.page;

  // table entries of the block at t0, asked for one block before they are used
  auto lookup = [&](int t0) -> DmaPages {
    DmaPages pg;
    pg.k = (t0 + kg0 < L && held(t0 + kg0)) ? bt[(t0 + kg0) >> a.page_shift] : 0;
    pg.v = (t0 + 16 * vh < L && held(t0 + 16 * vh)) ? bt[(t0 + 16 * vh) >> a.page_shift] : 0;
    return pg;
  };
  auto stage = [&](int t0, const DmaPages& pg, int bi) {
    const uint32_t buf = bi * DMA_BUF;
    const int krow = (t0 + kg0 < L && held(t0 + kg0)) ? ((t0 + kg0) & (a.page - 1)) : 0;
    const int vkey = (t0 + 16 * vh < L && held(t0 + 16 * vh)) ? ((t0 + 16 * vh) & (a.page - 1)) : 0;
    const bf16_t* gk = k_head + (uint64_t)(uint32_t)pg.k * page_elems + krow * HD;
    const bf16_t* gv = v_head + (uint64_t)(uint32_t)pg.v * page_elems + vkey;
    if (t0 + 32 <= L && held(t0)) {
#pragma unroll
      for (int j = 0; j < 2; ++j) dma16(gk + 8 * j * HD, voff_k, lds0 + buf + (2 * wave + j) * DMA_KINST);
#pragma unroll
      for (int j = 0; j < 2; ++j)
        dma16(gv + (int64_t)32 * j * a.page, voff_v, lds0 + buf + DMA_KBYTES + vh * DMA_VHALF + (vrow0 / 32 + j) * 1024);
    } else {
      typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
      const bf16x8 z = zero8();
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int key = t0 + kg0 + 8 * j + (lane >> 4);
        // rows of a page that is held may be read beyond the context; without a page, page 0 is read
        const bool mapped = t0 + kg0 + 8 * j < L && held(t0 + kg0);
        const bf16_t* src = mapped ? gk + 8 * j * HD : k_head;
        const bf16x8 kk = ld8(reinterpret_cast<const bf16_t*>(reinterpret_cast<const unsigned char*>(src) + voff_k));
        *reinterpret_cast<bf16x8*>(pf_lds + buf + (2 * wave + j) * DMA_KINST + 16 * lane) = (key < L && held(key)) ? kk : z;
      }
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int key0 = t0 + 16 * vh + 8 * ((lane & 1) ^ ((lane >> 4) & 1));
        const int nv = held(key0) ? L - key0 : 0;    // (a piece of 8 keys lies wholly before or behind first_held)
        const bf16x8 vv = ld8(reinterpret_cast<const bf16_t*>(reinterpret_cast<const unsigned char*>(gv + (int64_t)32 * j * a.page) + voff_v));
        u32x4 w = __builtin_bit_cast(u32x4, vv);
#pragma unroll
        for (int i = 0; i < 4; ++i) w[i] &= (2 * i < nv ? 0x0000ffffu : 0u) | (2 * i + 1 < nv ? 0xffff0000u : 0u);
        *reinterpret_cast<u32x4*>(pf_lds + buf + DMA_KBYTES + vh * DMA_VHALF + (vrow0 / 32 + j) * 1024 + 16 * lane) = w;
      }
    }
  };

  // every wave runs every round (a wave without columns in a round masks everything and writes nothing)
  for (int c_base = 0; c_base < ncols; c_base += 4 * 16 * CT) {
    const bool active = c_base + wave * 16 * CT < ncols;
    const int c0 = active ? c_base + wave * 16 * CT : 0;
    bf16x8 qb[CT][KS];
    int col_lo[CT], col_hi[CT];
    int64_t tq[CT];
    int head[CT];
    bool valid[CT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
      const int cc = c0 + 16 * ct + n;
      valid[ct] = active && cc < ncols;
      const int tl = valid[ct] ? cc / a.G : 0;
      const int hh = valid[ct] ? cc - tl * a.G : 0;
      tq[ct] = q0 + tok0 + tl;
      head[ct] = kvh * a.G + hh;
      const int pos = start + tok0 + tl;
      col_hi[ct] = valid[ct] ? pos : -1;
      col_lo[ct] = WINDOW ? max(0, pos - a.window + 1) : 0;
      load_q(a.q + tq[ct] * a.q_stride + (int64_t)head[ct] * HD, valid[ct], g, qb[ct]);
    }
    const int c_last = min(ncols, c0 + 16 * CT) - 1;
    const int pos_first = start + tok0 + c0 / a.G, pos_last = start + tok0 + c_last / a.G;
    const int full_hi = active ? pos_first - 31 : -(1 << 30);
    const int full_lo = WINDOW ? max(0, pos_last - a.window + 1) : 0;
    float m[CT], l[CT];
    f32x4 acc[CT][DT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
      m[ct] = NEG; l[ct] = 0.f;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) acc[ct][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

    pf_barrier();                                    // the round before has finished with every buffer
    DmaPages pg = lookup(seg_lo);
#pragma unroll
    for (int k = 0; k < PD; ++k) {
      if (k < nblk) {
        const DmaPages now = pg;
        pg = lookup(seg_lo + 32 * (k + 1));
        stage(seg_lo + 32 * k, now, k);
      }
    }
    int cur = 0;
    // One block: the wait for it, the request for the block PD further on, scores, softmax, values. FULL: every key
    // of the block is visible to every column of this wave. Blocks are walked in ascending order, so a wave's FULL
    // blocks come first and form a loop of their own (with both forms of the softmax in one loop body the compiler
    // copies all accumulators in every iteration); every wave passes the same barriers in either loop.
    auto block_step = [&](auto full_tag, int k) {
      constexpr bool FULL = decltype(full_tag)::value;
      const int t0 = seg_lo + 32 * k;
      // block k has landed: at most the PD - 1 blocks asked for after it are still on their way
      if (k + PD <= nblk) dma_wait<4 * (PD - 1)>(); else dma_wait<0>();
      pf_barrier();                                  // ... for every wave, and buffer cur - 1 is free
      if (k + PD < nblk) {
        const DmaPages now = pg;
        pg = lookup(t0 + 32 * (PD + 1));
        stage(t0 + 32 * PD, now, cur == 0 ? NB - 1 : cur - 1);
      }
      const unsigned char* kb = pf_lds + cur * DMA_BUF + rd_k;
      f32x4 st[CT][2];
      bf16x8 pb[CT];
      if constexpr (W == 2) {
        // With 256 registers to a wave all of a block's key operands are asked for before the first score product,
        // and its value operands before the softmax, which takes longer than they do: one LDS latency for each,
        // not one for every pair of reads.
        bf16x8 ka[2][KS];
#pragma unroll
        for (int tt = 0; tt < 2; ++tt)
#pragma unroll
          for (int ks = 0; ks < KS; ++ks)
            ka[tt][ks] = *reinterpret_cast<const bf16x8*>(kb + tt * 4 * DMA_KINST + 64 * ks);
        pin_operands(ka);
#pragma unroll
        for (int tt = 0; tt < 2; ++tt) {
#pragma unroll
          for (int ct = 0; ct < CT; ++ct) st[ct][tt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int ks = 0; ks < KS; ++ks)
#pragma unroll
            for (int ct = 0; ct < CT; ++ct)
              st[ct][tt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka[tt][ks], qb[ct][ks], st[ct][tt], 0, 0, 0);
        }
        bf16x8 va[DT];
        lds_read16_ahead<0>(lds0 + cur * DMA_BUF + rd_v, va);
        softmax_priority(true);
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
          block_softmax<FULL>(a, st[ct], t0, col_lo[ct], col_hi[ct], m[ct], l[ct], acc[ct], g, pb[ct]);
        softmax_priority(false);
        lds_reads_done(va);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int ct = 0; ct < CT; ++ct)
            acc[ct][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va[dt], pb[ct], acc[ct][dt], 0, 0, 0);
      } else {
        // With 168 registers the operands are read where they are used, and the third wave fills the waits.
#pragma unroll
        for (int tt = 0; tt < 2; ++tt) {
#pragma unroll
          for (int ct = 0; ct < CT; ++ct) st[ct][tt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) {
            const bf16x8 ka = *reinterpret_cast<const bf16x8*>(kb + tt * 4 * DMA_KINST + 64 * ks);
#pragma unroll
            for (int ct = 0; ct < CT; ++ct)
              st[ct][tt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka, qb[ct][ks], st[ct][tt], 0, 0, 0);
          }
        }
        softmax_priority(true);
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
          block_softmax<FULL>(a, st[ct], t0, col_lo[ct], col_hi[ct], m[ct], l[ct], acc[ct], g, pb[ct]);
        softmax_priority(false);
        const unsigned char* vb = pf_lds + cur * DMA_BUF + rd_v;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          const bf16x8 va = *reinterpret_cast<const bf16x8*>(vb + 512 * dt);
#pragma unroll
          for (int ct = 0; ct < CT; ++ct)
            acc[ct][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va, pb[ct], acc[ct][dt], 0, 0, 0);
        }
      }
      cur = cur == NB - 1 ? 0 : cur + 1;
    };
    // blocks [first_full, end_full) lie wholly inside every column's range of this wave: behind the window's lower
    // edge (if there is a window) and before the diagonal
    const int end_full = full_hi >= seg_lo ? min(nblk, (full_hi - seg_lo) / 32 + 1) : 0;
    int k = 0;
    if constexpr (WINDOW) {
      const int first_full = full_lo > seg_lo ? min(end_full, (full_lo - seg_lo + 31) / 32) : 0;
      for (; k < first_full; ++k) block_step(std::false_type{}, k);
    }
    for (; k < end_full; ++k) block_step(std::true_type{}, k);
    for (; k < nblk; ++k) block_step(std::false_type{}, k);

#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
      const float ls = column_sum(l[ct]);
      if (valid[ct] && tr.nseg > 1) {
        float* p = a.pf_scratch + (((int64_t)tq[ct] * a.Hq + head[ct]) * a.max_segs + seg) * (HD + 2);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
          *reinterpret_cast<f32x4*>(p + 16 * dt + 4 * g) = acc[ct][dt];
        if (g == 0) { p[HD] = m[ct]; p[HD + 1] = ls; }
      } else if (valid[ct]) {
        const float inv = ls > 0.f ? 1.f / ls : 0.f;
        bf16_t* o = a.out + tq[ct] * a.out_stride + (int64_t)head[ct] * HD + 4 * g;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          bf16x4 r;
#pragma unroll
          for (int i = 0; i < 4; ++i) r[i] = static_cast<bf16_t>(acc[ct][dt][i] * inv);
          *reinterpret_cast<bf16x4*>(o + 16 * dt) = r;
        }
      }
    }
  }
}
#endif  // ME_HEAD_DIM == 128

// Merge of the segments of cut tiles: out = sum_s 2^(m_s - M) o_s / sum_s 2^(m_s - M) l_s.
// Sixteen lanes per (token, head), each with HD/16 consecutive values; 16 rows to a workgroup. Rows of
// tiles that were not cut already hold their result and return.
#define MERGE_EPL (HD / 16)
__global__ void __launch_bounds__(256) attn_prefill_merge_kernel(AttnArgs a, int64_t rows) {
  const int64_t row = (int64_t)blockIdx.x * 16 + (threadIdx.x >> 4);
  if (row >= rows) return;
  const int part = threadIdx.x & 15;
  const int64_t t = row / a.Hq;
  const int hq = (int)(row - t * a.Hq);
  const int b = a.seq_of_token[t] - a.seq_base;
  const int q0 = a.cu_seqlens[b], q_len = a.cu_seqlens[b + 1] - q0;
  const int tok0 = ((int)(t - q0) / a.tok_tile) * a.tok_tile;
  const TileRange tr = tile_range(a, tok0, q_len, a.context_lens[b]);
  if (tr.nseg <= 1) return;
  const float* p = a.pf_scratch + row * a.max_segs * (HD + 2);
  float M = NEG;
  for (int s = 0; s < tr.nseg; ++s) M = fmaxf(M, p[s * (HD + 2) + HD]);
  float ls = 0.f;
  float o[MERGE_EPL];
#pragma unroll
  for (int i = 0; i < MERGE_EPL; ++i) o[i] = 0.f;
  for (int s = 0; s < tr.nseg; ++s) {
    const float* ps = p + s * (HD + 2);
    const float w = exp2f(ps[HD] - M);
    ls += w * ps[HD + 1];
    float v[MERGE_EPL];
    if (MERGE_EPL % 2 == 0) {        // rows of HD + 2 floats keep 8-byte alignment only
#pragma unroll
      for (int i = 0; i < MERGE_EPL; i += 2) {
        const float2 u = *reinterpret_cast<const float2*>(ps + part * MERGE_EPL + i);
        v[i] = u.x; v[i + 1] = u.y;
      }
    } else {
#pragma unroll
      for (int i = 0; i < MERGE_EPL; ++i) v[i] = ps[part * MERGE_EPL + i];
    }
#pragma unroll
    for (int i = 0; i < MERGE_EPL; ++i) o[i] += w * v[i];
  }
  const float inv = ls > 0.f ? 1.f / ls : 0.f;
  bf16_t* dst = a.out + t * a.out_stride + (int64_t)hq * HD + part * MERGE_EPL;
#pragma unroll
  for (int i = 0; i < MERGE_EPL; ++i) dst[i] = static_cast<bf16_t>(o[i] * inv);
}

// =====================================================================================
// Decode kernel: one query token per sequence, one workgroup per (sequence, kv head, partition).
// Neighbours in dispatch order go to different XCDs, so the grid's x decides which XCD does what.
// spread_heads: grid (Hkv * col_tiles, num_seqs, num_parts): the kv heads of a sequence go round the
// XCDs and every XCD gets its share of every sequence, however different their lengths are. Otherwise
// grid (num_seqs, Hkv * col_tiles, num_parts): all work of a sequence lands on one XCD, whose L2 then
// holds the block-table entries that its heads share; 1-3 % faster when the contexts are equally long,
// and far slower when they are not (64 contexts of 100-2,048 keys: 58.6 us against 48.5 us spread; one
// context of 32 k keys among 255 short ones: 434 us against 138 us). The caller says which it is.
// The 4 waves of a workgroup take the 32-key blocks of the partition in turn and are merged
// through LDS. With one partition the result is written directly; otherwise the partition's
// (max, sum, unnormalised output) go to scratch for the reduce kernel.
// The number of partitions is that of the longest context in the batch. A sequence's partitions
// beyond its own context (or wholly before its window) have no keys: their workgroups leave at once
// and write nothing, and the reduce kernel reads only the range decode_part_range gives. The last
// partitions are dispatched first (grid z counts down): only long sequences have them, so in a batch
// of contexts of very different lengths the longest sequences start first instead of last.
// =====================================================================================
__device__ __forceinline__ void decode_part_range(const AttnArgs& a, int L, int& first, int& end) {
  const int lo = a.window > 0 ? max(0, L - a.window) : 0;
  first = min((lo & ~31) / a.part_size, a.num_parts - 1);
  end = max(first + 1, min(a.num_parts, (L + a.part_size - 1) / a.part_size));
}

// PROLOGUE: what precedes attention in a decode step happens here too (reference models/qwen3.py:34-36 the
// per-head norms, layers/rotary_embedding.py:20-25 the rotation, csrc/kv_cache.cu:10-31 the cache write). The
// new token sits at position L - 1. Every workgroup norms and rotates its own query heads (a wave per head, a
// lane per rotation pair) into LDS, rounded to bfloat16 as the stand-alone kernel leaves them in the row. The
// workgroups whose partition holds position L - 1 do the same for the new key and copy the new value: they
// attend to both from LDS, in place of what the page holds there, and the first column tile's workgroup writes
// them into the page. No workgroup reads what another one writes.
#ifndef ME_DECODE_STREAMS
#define ME_DECODE_STREAMS 1
#endif
constexpr bool DECODE_STREAMS = ME_DECODE_STREAMS != 0;
// AHEAD (for partitions of at most 256 keys, i.e. one or two blocks to a wave): the keys of a wave's two blocks are
// both asked for before the first is worked on, so the second block's keys do not wait for the first block's work.
// (The values of both ahead as well need 197 registers, which leaves two workgroups to a compute unit instead of
// three.)
template <bool PROLOGUE, bool AHEAD = false>
__global__ void __launch_bounds__(256, 3) attn_decode_kernel(AttnArgs a) {
  extern __shared__ float lds[];  // [4 waves][cols][HD + 2]; PROLOGUE: then bfloat16 [cols + 2][HD]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n = lane & 15, g = lane >> 4;
  const int b = a.spread_heads ? blockIdx.y : blockIdx.x;
  const int head_block = a.spread_heads ? blockIdx.x : blockIdx.y;
  const int col_tiles = (a.G + 15) / 16;
  const int kvh = head_block / col_tiles, ctile = head_block - kvh * col_tiles;
  const int part = a.num_parts - 1 - blockIdx.z;
  const int L = a.context_lens[b];
  if (a.num_parts > 1) {
    int first, end;
    decode_part_range(a, L, first, end);
    if (part < first || part >= end) return;
  }
  const int pos = L - 1;
  const int lo = a.window > 0 ? max(0, pos - a.window + 1) : 0;
  const int32_t* bt = a.block_tables + (int64_t)b * a.bt_stride;
  const int ncols = min(16, a.G - ctile * 16);
  const bool valid = n < ncols;
  const int head = kvh * a.G + ctile * 16 + (valid ? n : 0);
  const int64_t t = b;  // decode rows come first in the batch: token index == sequence index

  const int p_lo = max(part * a.part_size, lo & ~31);
  const int p_hi = min((part + 1) * a.part_size, L);
  float m = NEG, l = 0.f;
  f32x4 acc[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) acc[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int cmax = a.G < 16 ? a.G : 16;
  bf16_t* q_s = reinterpret_cast<bf16_t*>(lds + 4 * cmax * (HD + 2));   // [cols][HD]
  bf16_t* k_s = q_s + cmax * HD;                                        // [HD] the new key
  bf16_t* v_s = k_s + HD;                                               // [HD] the new value
  const bool holds_new = PROLOGUE && pos >= p_lo && pos < p_hi;
  constexpr int HALF = HD / 2, PPL = (HALF + 63) / 64;   // rotation pairs of a head, pairs per lane
  struct RawHead { float x1[PPL], x2[PPL], w1[PPL], w2[PPL], cs[PPL], sn[PPL]; };
  const int nheads = PROLOGUE ? ncols + (holds_new ? 1 : 0) : 0;
  const int pi = pos >> a.page_shift;
  const int new_page = holds_new ? bt[pi] : -1;
  const int new_off = pos - (pi << a.page_shift);
  // a head's values, norm weights and angles as they lie in memory: only asked for here
  auto fetch_head = [&](int h, RawHead& r) {
    const bool is_q = h < ncols;
    const bf16_t* src = is_q ? a.q + t * a.q_stride + (int64_t)(kvh * a.G + ctile * 16 + h) * HD
                             : a.raw_k + t * a.q_stride + (int64_t)kvh * HD;
    const float* w = is_q ? a.q_w : a.k_w;
#pragma unroll
    for (int i = 0; i < PPL; ++i) {
      const int j = lane + 64 * i;
      const int js = j < HALF ? j : 0;
      r.x1[i] = static_cast<float>(src[js]);
      r.x2[i] = static_cast<float>(src[HALF + js]);
      r.w1[i] = w ? w[js] : 1.f;
      r.w2[i] = w ? w[HALF + js] : 1.f;
      // a padding row has no token (L = 0): it reads the angles of position 0 and nothing comes of them
      const float2 c = a.rope ? *reinterpret_cast<const float2*>(a.rope + ((int64_t)(pos > 0 ? pos : 0) * HALF + js) * 2) : make_float2(1.f, 0.f);
      r.cs[i] = c.x; r.sn[i] = c.y;
    }
  };
  // norm, rotation, rounding; into LDS, and the key into its page as well
  auto finish_head = [&](int h, const RawHead& r) {
    const bool is_q = h < ncols;
    const bool writes = !is_q && ctile == 0 && new_page >= 0;
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < PPL; ++i)
      if (lane + 64 * i < HALF) ss += r.x1[i] * r.x1[i] + r.x2[i] * r.x2[i];
    float inv = 1.f;
    if (a.q_w) inv = rsqrtf(wave_sum(ss) / (float)HD + a.eps);
    bf16_t* dst = is_q ? q_s + h * HD : k_s;
    bf16_t* page_row = a.k_cache_w + (((int64_t)(writes ? new_page : 0) * a.Hkv + kvh) * a.page + new_off) * HD;
#pragma unroll
    for (int i = 0; i < PPL; ++i) {
      const int j = lane + 64 * i;
      float o1 = r.x1[i] * inv, o2 = r.x2[i] * inv;
      o1 *= r.w1[i]; o2 *= r.w2[i];
      const bf16_t r1 = static_cast<bf16_t>(o1 * r.cs[i] - o2 * r.sn[i]);
      const bf16_t r2 = static_cast<bf16_t>(o2 * r.cs[i] + o1 * r.sn[i]);
      if (j < HALF) {
        dst[j] = r1; dst[HALF + j] = r2;
        if (writes) { page_row[j] = r1; page_row[HALF + j] = r2; }
      }
    }
  };
  // One block buffer only: the registers saved let several workgroups share a compute unit,
  // and it is their interleaving that hides the load latency here (partitions are short).
  int t0 = p_lo + 32 * wave;
  const bool has_keys = t0 < p_hi;
  const bool has_second = AHEAD && t0 + 128 < p_hi;
  KVBlock A, A2;
  // the first block of keys (AHEAD: and the second; both table reads go out before the keys they address)
  auto first_keys = [&]() {
    if constexpr (AHEAD) {
      BlockPages pg, pg2;
      lookup_pages(a, bt, t0, L, lo, n, g, pg);
      if (has_second) lookup_pages(a, bt, t0 + 128, L, lo, n, g, pg2);
      load_kv<DECODE_STREAMS>(a, pg, kvh, t0, L, n, g, A);
      if (has_second) load_kv<DECODE_STREAMS>(a, pg2, kvh, t0 + 128, L, n, g, A2);
    } else {
      load_block<DECODE_STREAMS>(a, bt, kvh, t0, L, lo, n, g, A);
    }
  };
  if (PROLOGUE) {
    // the wave's first head is asked for before the first block of keys, and worked on while those are on
    // their way; the heads after it (more than three query heads to a key head) one by one
    RawHead first;
    if (wave < nheads) fetch_head(wave, first);
    bf16_t new_v = static_cast<bf16_t>(0.f);
    const int vd = threadIdx.x < HD ? threadIdx.x : 0;
    if (holds_new) new_v = a.raw_v[t * a.q_stride + (int64_t)kvh * HD + vd];
    if (has_keys) first_keys();
    if (wave < nheads) finish_head(wave, first);
    for (int h = wave + 4; h < nheads; h += 4) {
      RawHead r;
      fetch_head(h, r);
      finish_head(h, r);
    }
    if (holds_new) {
      const bool writes = ctile == 0 && new_page >= 0;
      bf16_t* page_col = a.v_cache_w + (((int64_t)(writes ? new_page : 0) * a.Hkv + kvh) * HD) * a.page + new_off;
      for (int d = threadIdx.x; d < HD; d += 256) {
        const bf16_t v = d == vd ? new_v : a.raw_v[t * a.q_stride + (int64_t)kvh * HD + d];
        v_s[d] = v;
        if (writes) page_col[(int64_t)d * a.page] = v;
      }
    }
    __syncthreads();
  } else if (has_keys) {
    first_keys();
  }
  if (has_keys) {
    bf16x8 qb[KS];
    if (PROLOGUE) load_q(q_s + (valid ? n : 0) * HD, valid, g, qb);
    else load_q(a.q + t * a.q_stride + (int64_t)head * HD, valid, g, qb);
    const int col_hi = valid ? pos : -1;
    // one block: what the new token brings comes from LDS, then scores, softmax and the weighted sum
    auto work_on = [&](KVBlock& A, VBlock& vb, int t0) {
      if (holds_new && pos >= t0 && pos < t0 + 32) {
        // the block with the new token: its key row and its value column come from LDS
        const int rel = pos - t0;
#pragma unroll
        for (int tt = 0; tt < 2; ++tt)
          if (8 * (n >> 2) + 4 * tt + (n & 3) == rel) {
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
              const int d0 = 32 * ks + 8 * g;
              A.k[tt][ks] = ld8(k_s + ((HD % 32 == 0 || d0 < HD) ? d0 : 0));
            }
            A.kok[tt] = true;
          }
        if ((rel >> 3) == g) {
          const int at = rel & 7;
#pragma unroll
          for (int dt = 0; dt < DT; ++dt) {
            const bf16_t nv = v_s[16 * dt + n];
#pragma unroll
            for (int e = 0; e < 8; ++e) vb.v[dt][e] = e == at ? nv : vb.v[dt][e];
          }
        }
      }
      if (t0 + 32 <= L && t0 >= lo) attend_block<true>(a, A, vb, t0, qb, lo, col_hi, m, l, acc, g);
      else attend_block<false>(a, A, vb, t0, qb, lo, col_hi, m, l, acc, g);
    };
    if constexpr (AHEAD) {
      VBlock vb;
      load_v<DECODE_STREAMS>(a, A, kvh, t0, L, n, g, vb);
      work_on(A, vb, t0);
      if (has_second) {
        load_v<DECODE_STREAMS>(a, A2, kvh, t0 + 128, L, n, g, vb);
        work_on(A2, vb, t0 + 128);
      }
      t0 += 256;
    }
    while (t0 < p_hi) {           // AHEAD: only partitions of more than 256 keys get here
      if (AHEAD) load_block<DECODE_STREAMS>(a, bt, kvh, t0, L, lo, n, g, A);
      VBlock vb;
      load_v<DECODE_STREAMS>(a, A, kvh, t0, L, n, g, vb);
      work_on(A, vb, t0);
      t0 += 128;
      if (!AHEAD && t0 < p_hi) load_block<DECODE_STREAMS>(a, bt, kvh, t0, L, lo, n, g, A);
    }
  }
  l = column_sum(l);

  // ---- merge the 4 waves: only the columns in use pass through LDS
  const int stride = HD + 2;
  if (valid) {
    float* mine = lds + ((wave * ncols + n) * stride);
    if (g == 0) { mine[HD] = m; mine[HD + 1] = l; }
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int i = 0; i < 4; ++i) mine[16 * dt + 4 * g + i] = acc[dt][i];
  }
  __syncthreads();
  for (int e = threadIdx.x; e < ncols * HD; e += 256) {
    const int c = e / HD, d = e - c * HD;
    float M = NEG;
#pragma unroll
    for (int w = 0; w < 4; ++w) M = fmaxf(M, lds[(w * ncols + c) * stride + HD]);
    float o = 0.f, ls = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float f = exp2f(lds[(w * ncols + c) * stride + HD] - M);
      o += f * lds[(w * ncols + c) * stride + d];
      ls += f * lds[(w * ncols + c) * stride + HD + 1];
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

// Reduce over partitions: out = sum_p e^{m_p - M} o_p / sum_p e^{m_p - M} l_p. Grid (num_seqs, Hq);
// the weights of the partitions are formed once, in LDS, then every thread sums its channel.
#define RED_MAX_PARTS 64
__global__ void __launch_bounds__(128) attn_reduce_kernel(AttnArgs a) {
  __shared__ float wgt[RED_MAX_PARTS];
  __shared__ float inv_s;
  const int b = blockIdx.x, hq = blockIdx.y;
  int part0, part_end;
  decode_part_range(a, a.context_lens[b], part0, part_end);
  const int64_t row0 = ((int64_t)b * a.Hq + hq) * a.num_parts + part0;
  const int P = part_end - part0;
  // the first 16 partitions' values of this thread's channel are asked for before the weights are
  // formed: they do not depend on them, and the two rounds of loads then overlap
  const int d0 = threadIdx.x;
  float first[16];
#pragma unroll
  for (int p = 0; p < 16; ++p)
    first[p] = a.tmp_out[(row0 + (p < P ? p : 0)) * HD + (d0 < HD ? d0 : 0)];
  if (threadIdx.x < 64) {
    const int p = threadIdx.x;
    const float mp = p < P ? a.tmp_m[row0 + p] : NEG;
    const float lp = p < P ? a.tmp_l[row0 + p] : 0.f;
    const float M = wave_max(mp);
    const float f = p < P ? exp2f(mp - M) : 0.f;
    const float ls = wave_sum(f * lp);
    wgt[p] = f;
    if (p == 0) inv_s = ls > 0.f ? 1.f / ls : 0.f;
  }
  __syncthreads();
  const float inv = inv_s;
  for (int d = d0; d < HD; d += blockDim.x) {
    float o = 0.f;
    int p0 = 0;
    if (d == d0) {                      // weights beyond P are zero
#pragma unroll
      for (int p = 0; p < 16; ++p) o += wgt[p] * first[p];
      p0 = 16;
    }
#pragma unroll 8
    for (int p = p0; p < P; ++p) o += wgt[p] * a.tmp_out[(row0 + p) * HD + d];
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
  ME_CHECK(page >= 8 && (page & (page - 1)) == 0, "attention (bf16 MFMA path): page size %d must be a power of two, 8 or more", page);
  ME_CHECK(q_stride % 8 == 0 && out_stride % 4 == 0, "attention: token strides must keep 16-byte alignment");
  ME_CHECK((reinterpret_cast<uintptr_t>(q) % 16 == 0) && (reinterpret_cast<uintptr_t>(out) % 8 == 0) &&
               (reinterpret_cast<uintptr_t>(k_cache) % 16 == 0) && (reinterpret_cast<uintptr_t>(v_cache) % 16 == 0),
           "attention: q, out and cache pointers must be 16-byte aligned");
  ME_CHECK(window >= 0 && bt_stride >= 1, "attention: bad window or block-table stride");
  ME_CHECK(scale > 0.f, "attention: the score scale must be positive");
  a.q = (const bf16_t*)q; a.q_stride = q_stride; a.out = (bf16_t*)out; a.out_stride = out_stride;
  a.k_cache = (const bf16_t*)k_cache; a.v_cache = (const bf16_t*)v_cache;
  a.block_tables = block_tables; a.bt_stride = bt_stride; a.context_lens = context_lens;
  a.cu_seqlens = nullptr; a.num_seqs = num_seqs; a.Hq = Hq; a.Hkv = Hkv; a.G = Hq / Hkv;
  a.page = page; a.page_shift = 0;
  while ((1 << a.page_shift) < page) ++a.page_shift;
  a.scale = scale; a.window = window; a.tok_tile = 1; a.part_size = 0; a.num_parts = 1; a.spread_heads = 1;
  a.tmp_out = a.tmp_m = a.tmp_l = nullptr;
  a.seg_keys = 0; a.max_segs = 1; a.pf_scratch = nullptr; a.seq_of_token = nullptr; a.seq_base = 0;
  a.raw_k = a.raw_v = nullptr; a.q_w = a.k_w = nullptr; a.eps = 0.f; a.rope = nullptr;
  a.k_cache_w = a.v_cache_w = nullptr;
  return 0;
}

// q/out point at the first prefill token; cu_seqlens are relative to it; block_tables and
// context_lens at the first prefill sequence.
extern "C" int me_attn_prefill(const void* q, int64_t q_stride, void* out, int64_t out_stride,
                               const void* k_cache, const void* v_cache, const int32_t* block_tables,
                               int bt_stride, const int32_t* context_lens, const int32_t* cu_seqlens,
                               int num_seqs, int64_t num_tokens, int Hq, int Hkv, int page, float scale,
                               int window, int col_tiles_per_wave, int shared, int waves, int seg_keys, int max_segs, float* pf_scratch,
                               const int32_t* seq_of_token, int seq_base, hipStream_t stream) {
  if (num_seqs == 0 || num_tokens == 0) return 0;
  AttnArgs a;
  if (fill_common(a, q, q_stride, out, out_stride, k_cache, v_cache, block_tables, bt_stride, context_lens,
                  num_seqs, Hq, Hkv, page, scale, window)) return -1;
  a.cu_seqlens = cu_seqlens;
  // column tiles per wave: 2 when the step has enough tokens to fill the GPU with the larger tiles
  const int ct = (col_tiles_per_wave == 1 || col_tiles_per_wave == 2) ? col_tiles_per_wave
                 : ((num_tokens * Hq >= 32768 && HD <= 128) ? 2 : 1);
  const int cols = 64 * ct;
  a.tok_tile = a.G >= cols ? 1 : cols / a.G;
  const int64_t tiles = num_tokens / a.tok_tile + num_seqs;
  ME_CHECK(tiles * Hkv < (1ll << 31), "attention: too many tiles");
  if (seg_keys > 0 && max_segs > 1) {
    ME_CHECK(seg_keys % 32 == 0 && max_segs <= 65535, "attention: bad segment size %d or count %d", seg_keys, max_segs);
    ME_CHECK(pf_scratch && seq_of_token, "attention: cutting tiles into segments needs scratch and seq_of_token");
    a.seg_keys = seg_keys; a.max_segs = max_segs; a.pf_scratch = pf_scratch;
    a.seq_of_token = seq_of_token; a.seq_base = seq_base;
  }
  const dim3 grid((unsigned)(tiles * Hkv), 1, a.max_segs);
  // Keys and values through LDS where the two buffers fit (head sizes up to 128); the caller cuts
  // long key ranges so that there are workgroups enough for that form to pay (with one workgroup
  // per CU its waves have no others to fill their waits at the barriers).
  // shared: 0 never, otherwise wherever it fits.
  const bool through_lds = 2 * PF_BUF <= 65536 && shared != 0;
#if ME_HEAD_DIM == 128
  // shared: 1 the memory system fills LDS where the kernel for that applies, 2 always through registers.
  // waves: 3 asks for three waves to a SIMD (168 registers each) instead of two, with two column tiles; the
  // caller knows the launches for which that pays.
  if (through_lds && shared == 1 && page >= 16 && (int64_t)Hkv * page * HD < (1ll << 31)) {
    const bool three = ct == 2 && waves == 3;
#define DMA_LAUNCH(CTV, WV)                                                                                    \
  do {                                                                                                         \
    if (window > 0) attn_prefill_dma_kernel<CTV, WV, true><<<grid, dim3(256), DMA_NB * DMA_BUF, stream>>>(a);  \
    else attn_prefill_dma_kernel<CTV, WV, false><<<grid, dim3(256), DMA_NB * DMA_BUF, stream>>>(a);            \
  } while (0)
    if (three) DMA_LAUNCH(2, 3); else if (ct == 2) DMA_LAUNCH(2, 2); else DMA_LAUNCH(1, 2);
#undef DMA_LAUNCH
  } else
#endif
  if (through_lds) {
    if (ct == 2) attn_prefill_shared_kernel<2><<<grid, dim3(256), 2 * PF_BUF, stream>>>(a);
    else attn_prefill_shared_kernel<1><<<grid, dim3(256), 2 * PF_BUF, stream>>>(a);
  } else {
    if (ct == 2) attn_prefill_kernel<2><<<grid, dim3(256), 0, stream>>>(a);
    else attn_prefill_kernel<1><<<grid, dim3(256), 0, stream>>>(a);
  }
  ME_LAUNCH_CHECK();
  if (a.max_segs > 1) {
    const int64_t rows = num_tokens * Hq;
    attn_prefill_merge_kernel<<<dim3((unsigned)((rows + 15) / 16)), dim3(256), 0, stream>>>(a, rows);
    ME_LAUNCH_CHECK();
  }
  return 0;
}

// Scratch of the split decode path: num_seqs * Hq * num_parts * (HD + 2) floats (out, m, l per partition).
static int launch_decode(AttnArgs& a, int num_seqs, int part_size, int num_parts, float* scratch, int spread_heads,
                         bool prologue, hipStream_t stream) {
  ME_CHECK(num_parts >= 1 && num_parts <= RED_MAX_PARTS, "attention: %d partitions outside 1..%d", num_parts, RED_MAX_PARTS);
  ME_CHECK(num_parts == 1 || (part_size >= 32 && part_size % 32 == 0),
           "attention: partition size %d must be a multiple of 32", part_size);
  ME_CHECK(num_parts == 1 || scratch != nullptr, "attention: split decode needs scratch");
  a.part_size = num_parts == 1 ? (1 << 30) : part_size;
  a.num_parts = num_parts;
  a.spread_heads = spread_heads ? 1 : 0;
  if (num_parts > 1) {
    const int64_t rows = (int64_t)num_seqs * a.Hq * num_parts;
    a.tmp_out = scratch; a.tmp_m = scratch + rows * HD; a.tmp_l = a.tmp_m + rows;
  }
  const int col_tiles = (a.G + 15) / 16;
  ME_CHECK((int64_t)a.Hkv * col_tiles <= 65535 && num_seqs <= 65535,
           "attention: %d sequences or %d head blocks exceed one launch", num_seqs, a.Hkv * col_tiles);
  const int cmax = a.G < 16 ? a.G : 16;
  const size_t lds = (size_t)4 * cmax * (HD + 2) * sizeof(float) + (prologue ? (size_t)(cmax + 2) * HD * sizeof(bf16_t) : 0);
  static size_t lds_allowed[2] = {64 * 1024, 64 * 1024};
  if (lds > lds_allowed[prologue]) {
    for (const void* kernel : {prologue ? (const void*)attn_decode_kernel<true, false> : (const void*)attn_decode_kernel<false, false>,
                               prologue ? (const void*)attn_decode_kernel<true, true> : (const void*)attn_decode_kernel<false, true>}) {
      hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      ME_CHECK(e == hipSuccess, "attention: cannot get %zu bytes of LDS: %s", lds, hipGetErrorString(e));
    }
    lds_allowed[prologue] = lds;
  }
  const dim3 grid = a.spread_heads ? dim3(a.Hkv * col_tiles, num_seqs, num_parts) : dim3(num_seqs, a.Hkv * col_tiles, num_parts);
  // partitions of 129-256 keys: a wave has up to two blocks and asks for the keys of both at once
  // (ME_DECODE_KEYS_AHEAD=0 in the environment leaves that form out, for timing one against the other)
  static const bool ahead_allowed = []() { const char* v = getenv("ME_DECODE_KEYS_AHEAD"); return v == nullptr || v[0] != '0'; }();
  const bool ahead = ahead_allowed && num_parts > 1 && part_size > 128 && part_size <= 256;
  if (prologue && ahead) attn_decode_kernel<true, true><<<grid, dim3(256), lds, stream>>>(a);
  else if (prologue) attn_decode_kernel<true, false><<<grid, dim3(256), lds, stream>>>(a);
  else if (ahead) attn_decode_kernel<false, true><<<grid, dim3(256), lds, stream>>>(a);
  else attn_decode_kernel<false, false><<<grid, dim3(256), lds, stream>>>(a);
  ME_LAUNCH_CHECK();
  if (num_parts > 1) {
    attn_reduce_kernel<<<dim3(num_seqs, a.Hq), dim3(128), 0, stream>>>(a);
    ME_LAUNCH_CHECK();
  }
  return 0;
}

extern "C" int me_attn_decode(const void* q, int64_t q_stride, void* out, int64_t out_stride,
                              const void* k_cache, const void* v_cache, const int32_t* block_tables,
                              int bt_stride, const int32_t* context_lens, int num_seqs, int Hq, int Hkv,
                              int page, float scale, int window, int part_size, int num_parts,
                              float* scratch, int spread_heads, hipStream_t stream) {
  if (num_seqs == 0) return 0;
  AttnArgs a;
  if (fill_common(a, q, q_stride, out, out_stride, k_cache, v_cache, block_tables, bt_stride, context_lens,
                  num_seqs, Hq, Hkv, page, scale, window)) return -1;
  return launch_decode(a, num_seqs, part_size, num_parts, scratch, spread_heads, false, stream);
}

// A whole decode step's attention from the packed projection rows [num_seqs, (Hq + 2 Hkv) * HD] (row r belongs
// to sequence r, its token stands at position context_lens[r] - 1): per-head norms of q and k (q_w, k_w
// float32 [HD], or both null), rotation by `rope` [rope_rows, HD/2, 2] (or null), the new key and value into
// their page (the one the block table names for that position), attention over the pages. The rows are left as
// they were. max_context: no context_lens entry is larger (checked against rope_rows here, since the kernel
// reads the table at context_lens[r] - 1).
extern "C" int me_attn_decode_fused(const void* qkv, int64_t row_stride, void* out, int64_t out_stride,
                                    const float* q_w, const float* k_w, float eps, const float* rope, int rope_rows,
                                    void* k_cache, void* v_cache, const int32_t* block_tables, int bt_stride,
                                    const int32_t* context_lens, int max_context, int num_seqs, int Hq, int Hkv,
                                    int page, float scale, int window, int part_size, int num_parts,
                                    float* scratch, int spread_heads, hipStream_t stream) {
  if (num_seqs == 0) return 0;
  AttnArgs a;
  if (fill_common(a, qkv, row_stride, out, out_stride, k_cache, v_cache, block_tables, bt_stride, context_lens,
                  num_seqs, Hq, Hkv, page, scale, window)) return -1;
  ME_CHECK((q_w == nullptr) == (k_w == nullptr), "attention: give both norm weights or neither");
  ME_CHECK(rope == nullptr || (max_context >= 0 && max_context <= rope_rows),
           "attention: a context of %d tokens is beyond the rotation table's %d positions", max_context, rope_rows);
  ME_CHECK(rope == nullptr || reinterpret_cast<uintptr_t>(rope) % 8 == 0, "attention: the rotation table must be 8-byte aligned");
  ME_CHECK(row_stride >= (int64_t)(Hq + 2 * Hkv) * HD, "attention: packed rows must hold q, k and v");
  a.raw_k = (const bf16_t*)qkv + (int64_t)Hq * HD;
  a.raw_v = a.raw_k + (int64_t)Hkv * HD;
  a.q_w = q_w; a.k_w = k_w; a.eps = eps; a.rope = rope;
  a.k_cache_w = (bf16_t*)k_cache; a.v_cache_w = (bf16_t*)v_cache;
  return launch_decode(a, num_seqs, part_size, num_parts, scratch, spread_heads, true, stream);
}

// Per-head RMSNorm of q and k, rotary position encoding, and the scatter of k and v
// into the paged cache, in one pass over the packed qkv rows.
//
// The reference does this with four eager steps and one kernel: q_norm/k_norm
// (models/qwen3.py:34-35), rotary (layers/rotary_embedding.py:20-25: out = x*cos +
// rotate_half(x)*sin, pairs (i, i + D/2)), and csrc/kv_cache.cu:10-31 (row copy into
// slot_mapping[t], negative slots skipped). Here the norm, the rotation angles' cos/sin
// and the products are all float32 and each value is rounded once.
//
// Cache layout (chosen for the MFMA attention kernels, not the reference's):
//   K: [num_pages, Hkv, page, D]      keys of a page and head are contiguous rows
//   V: [num_pages, Hkv, D, page]      transposed inside a page: for one channel the
//                                     page's tokens are contiguous (the P.V operand)
#include "common.h"

#define ME_MAX_PAIRS 4  // pairs per lane: head_dim <= 2 * 64 * ME_MAX_PAIRS

// A value head of token t into its transposed page.
// Tokens are taken 8 at a time (by the workgroup of the group's first token): when their slots
// are 8 consecutive places of one page, a channel's 8 values are one 16-byte store; a lane
// reads them with 8 loads that are each contiguous across the lanes.
template <typename T>
__device__ void store_value_head(const T* row, int64_t row_stride, int64_t t, int64_t num_tokens,
                                 const int32_t* slots, T* v_cache, int Hkv, int kvh, int D, int page, int lane) {
  if (t & 7) return;
  const int cnt = (int)min((int64_t)8, num_tokens - t);
  const int s0 = slots[t];
  bool run = cnt == 8 && s0 >= 0 && (s0 & 7) == 0 && page % 8 == 0;
  if (run) {
#pragma unroll
    for (int i = 1; i < 8; ++i) run = run && slots[t + i] == s0 + i;
  }
  if (run) {
    const int64_t pg = s0 / page, off = s0 - pg * page;
    T* dst = v_cache + ((pg * Hkv + kvh) * (int64_t)D) * page + off;
    for (int d = lane; d < D; d += 64) {
      alignas(16) T vals[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) vals[i] = row[i * row_stride + d];
      *reinterpret_cast<uint4*>(dst + (int64_t)d * page) = *reinterpret_cast<const uint4*>(vals);
      if (sizeof(T) == 4) *reinterpret_cast<uint4*>(dst + (int64_t)d * page + 4) = *reinterpret_cast<const uint4*>(vals + 4);
    }
    return;
  }
  for (int i = 0; i < cnt; ++i) {
    const int slot = slots[t + i];
    if (slot < 0) continue;
    const int64_t pg = slot / page, off = slot - pg * page;
    T* dst = v_cache + ((pg * Hkv + kvh) * (int64_t)D) * page + off;
    for (int d = lane; d < D; d += 64) dst[(int64_t)d * page] = row[i * row_stride + d];
  }
}

template <typename T>
__global__ void __launch_bounds__(256)
qk_norm_rope_store_kernel(T* __restrict__ qkv, int64_t row_stride, const float* __restrict__ q_w,
                          const float* __restrict__ k_w, float eps,
                          const float* __restrict__ table,  // [P, D/2, 2] cos,sin or null
                          const int32_t* __restrict__ positions, const int32_t* __restrict__ slots,
                          T* __restrict__ k_cache, T* __restrict__ v_cache, int Hq, int Hkv, int D,
                          int page, int store, int64_t num_tokens) {
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x & 63;
  const int head = blockIdx.y * 4 + (threadIdx.x >> 6);
  // store: rows hold q, k and v heads; k and v go to the pages. Otherwise rows hold q and Hkv
  // (possibly 0) k heads, all rewritten in place, and v is not touched.
  const int total_heads = Hq + (store ? 2 * Hkv : Hkv);
  if (head >= total_heads) return;
  T* row = qkv + t * row_stride + (int64_t)head * D;
  const int half = D >> 1;

  if (head >= Hq + Hkv) {  // a value head: copy into the transposed page
    store_value_head<T>(row, row_stride, t, num_tokens, slots, v_cache, Hkv, head - Hq - Hkv, D, page, lane);
    return;
  }

  const bool is_q = head < Hq;
  const float* w = is_q ? q_w : k_w;
  float x1[ME_MAX_PAIRS], x2[ME_MAX_PAIRS];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < ME_MAX_PAIRS; ++j) {
    const int p = lane + 64 * j;
    x1[j] = x2[j] = 0.f;
    if (p < half) {
      x1[j] = to_f32<T>(row[p]);
      x2[j] = to_f32<T>(row[p + half]);
      ss += x1[j] * x1[j] + x2[j] * x2[j];
    }
  }
  float inv = 1.f;
  if (w) {
    ss = wave_sum(ss);
    inv = rsqrtf(ss / (float)D + eps);
  }
  const int pos = positions[t];
  T* dst = row;
  if (!is_q && store) {
    const int slot = slots[t];
    if (slot < 0) return;
    const int kvh = head - Hq;
    const int64_t pg = slot / page, off = slot - pg * page;
    dst = k_cache + ((pg * Hkv + kvh) * (int64_t)page + off) * D;
  }
#pragma unroll
  for (int j = 0; j < ME_MAX_PAIRS; ++j) {
    const int p = lane + 64 * j;
    if (p < half) {
      float a = x1[j] * inv, b = x2[j] * inv;
      if (w) {
        a *= w[p];
        b *= w[p + half];
      }
      float o1 = a, o2 = b;
      if (table) {
        const float c = table[((int64_t)pos * half + p) * 2];
        const float s = table[((int64_t)pos * half + p) * 2 + 1];
        o1 = a * c - b * s;
        o2 = b * c + a * s;
      }
      dst[p] = from_f32<T>(o1);
      dst[p + half] = from_f32<T>(o2);
    }
  }
}

// ------------------------------------------------------------------ vectorised q/k form
// The same arithmetic with 4 pairs per lane: LPH = D/8 lanes share a head (a power of two), a wave
// takes 64/LPH heads, a lane reads x[4l..4l+3] and x[D/2+4l..], their 4 (cos, sin) and writes both
// quadruples back. blockIdx.y < qk_blocks: q and k heads; the rest: value heads (one per wave).
template <typename T> struct Quad;
template <> struct Quad<float> {
  static __device__ __forceinline__ void load(const float* p, float (&v)[4]) {
    const float4 t = *reinterpret_cast<const float4*>(p); v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
  }
  static __device__ __forceinline__ void store(float* p, const float (&v)[4]) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  }
};
template <> struct Quad<bf16_t> {
  static __device__ __forceinline__ void load(const bf16_t* p, float (&v)[4]) {
    const bf16x4 t = *reinterpret_cast<const bf16x4*>(p);
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = static_cast<float>(t[i]);
  }
  static __device__ __forceinline__ void store(bf16_t* p, const float (&v)[4]) {
    bf16x4 t;
#pragma unroll
    for (int i = 0; i < 4; ++i) t[i] = static_cast<bf16_t>(v[i]);
    *reinterpret_cast<bf16x4*>(p) = t;
  }
};

template <typename T, int LPH>
__global__ void __launch_bounds__(256)
qk_norm_rope_store_vec_kernel(T* __restrict__ qkv, int64_t row_stride, const float* __restrict__ q_w,
                              const float* __restrict__ k_w, float eps, const float* __restrict__ table,
                              const int32_t* __restrict__ positions, const int32_t* __restrict__ slots,
                              T* __restrict__ k_cache, T* __restrict__ v_cache, int Hq, int Hkv, int D, int page,
                              int store, int64_t num_tokens, int qk_blocks) {
  constexpr int HPW = 64 / LPH;
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int half = D >> 1;
  if ((int)blockIdx.y >= qk_blocks) {
    const int kvh = ((int)blockIdx.y - qk_blocks) * 4 + wave;
    if (kvh < Hkv) store_value_head<T>(qkv + t * row_stride + (int64_t)(Hq + Hkv + kvh) * D, row_stride, t, num_tokens,
                                       slots, v_cache, Hkv, kvh, D, page, lane);
    return;
  }
  const int head = (blockIdx.y * 4 + wave) * HPW + lane / LPH;
  const int l = lane % LPH;
  const bool active = head < Hq + Hkv;
  const bool is_q = head < Hq;
  T* row = qkv + t * row_stride + (int64_t)(active ? head : 0) * D;
  // Everything this thread reads is asked for at once: the position and the slot first (the table's
  // address hangs on the position), then the row and the norm's weight; the step is a chain of memory
  // latencies, and each load that waits for arithmetic it does not need adds one.
  const int pos = table ? positions[t] : 0;
  const int slot = store ? slots[t] : 0;
  const float* w = is_q ? q_w : k_w;
  float x1[4], x2[4];
  Quad<T>::load(row + 4 * l, x1);
  Quad<T>::load(row + half + 4 * l, x2);
  float w1[4] = {1.f, 1.f, 1.f, 1.f}, w2[4] = {1.f, 1.f, 1.f, 1.f};
  if (w) {
    Quad<float>::load(w + 4 * l, w1);
    Quad<float>::load(w + half + 4 * l, w2);
  }
  float c0[4] = {1.f, 0.f, 1.f, 0.f}, c1[4] = {1.f, 0.f, 1.f, 0.f};
  if (table) {
    const float* cs = table + ((int64_t)pos * half + 4 * l) * 2;   // (cos, sin) of 4 pairs: 8 floats
    Quad<float>::load(cs, c0);
    Quad<float>::load(cs + 4, c1);
  }
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) ss += x1[i] * x1[i] + x2[i] * x2[i];
  float inv = 1.f;
  if (w) {
#pragma unroll
    for (int off = LPH / 2; off > 0; off >>= 1) ss += __shfl_xor(ss, off, ME_WAVE);
    inv = rsqrtf(ss / (float)D + eps);
  }
  float o1[4], o2[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) { o1[i] = x1[i] * inv; o2[i] = x2[i] * inv; }
  if (w) {
#pragma unroll
    for (int i = 0; i < 4; ++i) { o1[i] *= w1[i]; o2[i] *= w2[i]; }
  }
  if (table) {
    const float c[4] = {c0[0], c0[2], c1[0], c1[2]}, sn[4] = {c0[1], c0[3], c1[1], c1[3]};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float a = o1[i], b = o2[i];
      o1[i] = a * c[i] - b * sn[i];
      o2[i] = b * c[i] + a * sn[i];
    }
  }
  if (!active) return;
  T* dst = row;
  if (!is_q && store) {
    if (slot < 0) return;
    const int64_t pg = slot / page, off = slot - pg * page;
    dst = k_cache + ((pg * Hkv + (head - Hq)) * (int64_t)page + off) * D;
  }
  Quad<T>::store(dst + 4 * l, o1);
  Quad<T>::store(dst + half + 4 * l, o2);
}

// ------------------------------------------------------------------ many tokens: 8 tokens per workgroup
// The same arithmetic for steps with many tokens (prefill). Grid (groups of 8 consecutive tokens,
// q/k workgroups + one value workgroup). q and k heads: LPH = D/16 lanes share a head, a lane reads 8 values of each
// half (16 bytes), their 8 (cos, sin), and writes both back. Value heads: a thread takes 8 channels
// of a head, reads them for 8 tokens, transposes the 8x8 block in registers and writes one
// 16-byte piece per channel into the transposed page (for 8 tokens whose slots are consecutive places of
// one page, starting at a multiple of 8, wherever in the batch their rows begin; otherwise value by value).
typedef bf16_t bf16x8r __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4r __attribute__((ext_vector_type(4)));

template <int LPH>
__global__ void __launch_bounds__(256)
qk_norm_rope_store_tile_kernel(bf16_t* __restrict__ qkv, int64_t row_stride, const float* __restrict__ q_w,
                               const float* __restrict__ k_w, float eps, const float* __restrict__ table,
                               const int32_t* __restrict__ positions, const int32_t* __restrict__ slots,
                               bf16_t* __restrict__ k_cache, bf16_t* __restrict__ v_cache, int Hq, int Hkv, int D,
                               int page, int store, int64_t num_tokens, int qk_groups) {
  const int64_t t0 = (int64_t)blockIdx.x * 8;
  const int cnt = (int)min((int64_t)8, num_tokens - t0);
  const int half = D >> 1;
  const int heads = Hq + Hkv;
  const int l = threadIdx.x % LPH;
  // ---- q and k heads: workgroups y < qk_groups, one (token, head) per LPH lanes
  if ((int)blockIdx.y < qk_groups) {
    const int item = blockIdx.y * (256 / LPH) + threadIdx.x / LPH;
    if (item >= cnt * heads) return;
    const int ti = item / heads, head = item - ti * heads;
    const int64_t t = t0 + ti;
    const bool is_q = head < Hq;
    bf16_t* row = qkv + t * row_stride + (int64_t)head * D;
    const bf16x8r a = *reinterpret_cast<const bf16x8r*>(row + 8 * l);
    const bf16x8r b = *reinterpret_cast<const bf16x8r*>(row + half + 8 * l);
    float x1[8], x2[8];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      x1[i] = static_cast<float>(a[i]); x2[i] = static_cast<float>(b[i]);
      ss += x1[i] * x1[i] + x2[i] * x2[i];
    }
    const float* w = is_q ? q_w : k_w;
    float inv = 1.f;
    if (w) {
#pragma unroll
      for (int off = LPH / 2; off > 0; off >>= 1) ss += __shfl_xor(ss, off, ME_WAVE);
      inv = rsqrtf(ss / (float)D + eps);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) { x1[i] *= inv; x2[i] *= inv; }
    if (w) {
      const float4 wa = *reinterpret_cast<const float4*>(w + 8 * l), wb = *reinterpret_cast<const float4*>(w + 8 * l + 4);
      const float4 wc = *reinterpret_cast<const float4*>(w + half + 8 * l), wd = *reinterpret_cast<const float4*>(w + half + 8 * l + 4);
      const float w1[8] = {wa.x, wa.y, wa.z, wa.w, wb.x, wb.y, wb.z, wb.w}, w2[8] = {wc.x, wc.y, wc.z, wc.w, wd.x, wd.y, wd.z, wd.w};
#pragma unroll
      for (int i = 0; i < 8; ++i) { x1[i] *= w1[i]; x2[i] *= w2[i]; }
    }
    if (table) {
      const float4* cs = reinterpret_cast<const float4*>(table + ((int64_t)positions[t] * half + 8 * l) * 2);
#pragma unroll
      for (int i = 0; i < 4; ++i) {   // a float4 holds (cos, sin) of two pairs
        const float4 c = cs[i];
        const float a0 = x1[2 * i], b0 = x2[2 * i], a1 = x1[2 * i + 1], b1 = x2[2 * i + 1];
        x1[2 * i] = a0 * c.x - b0 * c.y; x2[2 * i] = b0 * c.x + a0 * c.y;
        x1[2 * i + 1] = a1 * c.z - b1 * c.w; x2[2 * i + 1] = b1 * c.z + a1 * c.w;
      }
    }
    bf16_t* dst = row;
    if (!is_q && store) {
      const int slot = slots[t];
      if (slot < 0) return;
      const int64_t pg = slot / page, off = slot - pg * page;
      dst = k_cache + ((pg * Hkv + (head - Hq)) * (int64_t)page + off) * D;
    }
    bf16x8r o1, o2;
#pragma unroll
    for (int i = 0; i < 8; ++i) { o1[i] = static_cast<bf16_t>(x1[i]); o2[i] = static_cast<bf16_t>(x2[i]); }
    *reinterpret_cast<bf16x8r*>(dst + 8 * l) = o1;
    *reinterpret_cast<bf16x8r*>(dst + half + 8 * l) = o2;
    return;
  }
  // ---- value heads: the last workgroup of the 8 tokens
  // The values go into the transposed page [channel][place]. Eight tokens whose slots are the eight places of an
  // aligned group (consecutive, the first a multiple of 8) are written as one 16-byte piece per channel. Which rows
  // of the batch form such a group has nothing to do with where the workgroups' rows begin (decode rows stand in
  // front of the prompts' rows, a prompt is cut where the token budget ends), so the groups are found from the
  // slots: a row begins a group if its slot is a multiple of 8 or does not follow the slot of the row before it; the
  // group is that row and the rows behind it whose slots follow on, up to the end of the aligned eight. Every row
  // lies in exactly one group, and a group is written by the workgroup that holds its first row (which reads up to
  // seven rows of the workgroup behind it). Whole groups take the 16-byte way, the others value by value.
  const int dvecs = D >> 3;
  for (int i = 0; i < cnt; ++i) {
    const int64_t t = t0 + i;
    const int s0 = slots[t];
    if (s0 < 0) continue;
    const int lead = s0 & 7;
    if (lead != 0 && t > 0 && slots[t - 1] == s0 - 1) continue;       // belongs to the group of a row before it
    int n = 1;
    while (n < 8 - lead && t + n < num_tokens && slots[t + n] == s0 + n) ++n;
    const int64_t pg = s0 / page, off = s0 - pg * page;               // page % 8 == 0: a group lies within one page
    for (int unit = threadIdx.x; unit < Hkv * dvecs; unit += 256) {
      const int kvh = unit / dvecs, dv = unit - kvh * dvecs;
      const bf16_t* src = qkv + t * row_stride + (int64_t)(heads + kvh) * D + 8 * dv;
      bf16_t* dst = v_cache + ((pg * Hkv + kvh) * (int64_t)D + 8 * dv) * page + off;
      if (n == 8) {
        u32x4r tok[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) tok[j] = *reinterpret_cast<const u32x4r*>(src + j * row_stride);
#pragma unroll
        for (int d = 0; d < 8; ++d) {   // channel d of the 8 tokens: word d/2 of each token, low or high half
          u32x4r o;
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const uint32_t lo = tok[2 * j][d >> 1], hi = tok[2 * j + 1][d >> 1];
            o[j] = (d & 1) ? ((lo >> 16) | (hi & 0xffff0000u)) : ((lo & 0xffffu) | (hi << 16));
          }
          *reinterpret_cast<u32x4r*>(dst + (int64_t)d * page) = o;
        }
      } else {
        for (int j = 0; j < n; ++j) {
          const bf16x8r v = *reinterpret_cast<const bf16x8r*>(src + j * row_stride);
#pragma unroll
          for (int d = 0; d < 8; ++d) dst[(int64_t)d * page + j] = v[d];
        }
      }
    }
  }
}

extern "C" int me_qk_norm_rope_store(void* qkv, int dtype, int64_t num_tokens, int64_t row_stride,
                                     const float* q_w, const float* k_w, float eps,
                                     const float* table, int64_t table_positions, int64_t position_bound,
                                     const int32_t* positions, const int32_t* slots, void* k_cache,
                                     void* v_cache, int Hq, int Hkv, int D, int page, int store,
                                     hipStream_t stream) {
  if (num_tokens == 0) return 0;
  ME_CHECK(D >= 2 && D % 2 == 0 && D <= 2 * 64 * ME_MAX_PAIRS,
           "qk_norm_rope_store: head_dim %d must be even and <= %d", D, 2 * 64 * ME_MAX_PAIRS);
  ME_CHECK(Hq >= 1 && Hkv >= 0 && page >= 1, "qk_norm_rope_store: bad head counts or page size");
  ME_CHECK(!store || (Hkv >= 1 && k_cache && v_cache), "qk_norm_rope_store: storing needs kv heads and caches");
  ME_CHECK(row_stride >= (int64_t)(Hq + (store ? 2 * Hkv : Hkv)) * D, "qk_norm_rope_store: row stride too small");
  ME_CHECK(!table || table_positions > 0, "qk_norm_rope_store: empty rotary table");
  // position_bound: every position of the step is below it (what the host knows of the step; 0: not told)
  ME_CHECK(!table || position_bound <= table_positions,
           "qk_norm_rope_store: positions up to %lld are beyond the rotation table's %lld", (long long)position_bound - 1,
           (long long)table_positions);
  const int heads = Hq + (store ? 2 * Hkv : Hkv);
  ME_CHECK(dtype == ME_BF16 || dtype == ME_F32, "qk_norm_rope_store: bad dtype code %d", dtype);
  // vectorised form: D/8 lanes per head must be a power of two, rows and caches 16-byte aligned
  const int lph = D / 8;
  const int esz = dtype == ME_BF16 ? 2 : 4;
  const bool vec = D % 8 == 0 && lph >= 1 && lph <= 32 && (lph & (lph - 1)) == 0 && (row_stride * esz) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(qkv) % 16 == 0 && reinterpret_cast<uintptr_t>(k_cache) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(q_w) % 16 == 0 && reinterpret_cast<uintptr_t>(k_w) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(table) % 16 == 0;
  // many tokens of bfloat16: 8 tokens per workgroup group. From 128 tokens on: below that the steps are
  // decode steps, whose slots are scattered, and the form above is faster for those (64 tokens: 6.4 against 7.6 us).
  const int lph16 = D / 16;
  const bool tile = vec && dtype == ME_BF16 && num_tokens >= 128 && D % 16 == 0 && lph16 >= 1 && lph16 <= 64 &&
                    (lph16 & (lph16 - 1)) == 0 && (!store || (page % 8 == 0 && reinterpret_cast<uintptr_t>(v_cache) % 16 == 0));
  if (tile) {
    const int per_group = 256 / lph16;
    const int qk_groups = (8 * (Hq + Hkv) + per_group - 1) / per_group;
    dim3 grid((unsigned)((num_tokens + 7) / 8), qk_groups + (store ? 1 : 0)), block(256);
#define LAUNCH_TILE(L)                                                                                     \
  qk_norm_rope_store_tile_kernel<L><<<grid, block, 0, stream>>>((bf16_t*)qkv, row_stride, q_w, k_w, eps, table, \
                                                                positions, slots, (bf16_t*)k_cache,       \
                                                                (bf16_t*)v_cache, Hq, Hkv, D, page, store, num_tokens, qk_groups)
    switch (lph16) {
      case 1: LAUNCH_TILE(1); break; case 2: LAUNCH_TILE(2); break; case 4: LAUNCH_TILE(4); break;
      case 8: LAUNCH_TILE(8); break; case 16: LAUNCH_TILE(16); break; case 32: LAUNCH_TILE(32); break;
      default: LAUNCH_TILE(64); break;
    }
#undef LAUNCH_TILE
    ME_LAUNCH_CHECK();
    return 0;
  }
  if (vec) {
    const int hpw = 64 / lph;
    const int qk_blocks = (Hq + Hkv + 4 * hpw - 1) / (4 * hpw);
    const int v_blocks = store ? (Hkv + 3) / 4 : 0;
    dim3 grid(num_tokens, qk_blocks + v_blocks), block(256);
#define LAUNCH(TT, L)                                                                                       \
  qk_norm_rope_store_vec_kernel<TT, L><<<grid, block, 0, stream>>>((TT*)qkv, row_stride, q_w, k_w, eps, table, \
                                                                   positions, slots, (TT*)k_cache, (TT*)v_cache, \
                                                                   Hq, Hkv, D, page, store, num_tokens, qk_blocks)
#define PICK(TT)                                                                                            \
  do {                                                                                                      \
    if (lph == 1) LAUNCH(TT, 1); else if (lph == 2) LAUNCH(TT, 2); else if (lph == 4) LAUNCH(TT, 4);        \
    else if (lph == 8) LAUNCH(TT, 8); else if (lph == 16) LAUNCH(TT, 16); else LAUNCH(TT, 32);              \
  } while (0)
    if (dtype == ME_BF16) PICK(bf16_t); else PICK(float);
#undef PICK
#undef LAUNCH
    ME_LAUNCH_CHECK();
    return 0;
  }
  dim3 grid(num_tokens, (heads + 3) / 4), block(256);
  if (dtype == ME_BF16)
    qk_norm_rope_store_kernel<bf16_t><<<grid, block, 0, stream>>>(
        (bf16_t*)qkv, row_stride, q_w, k_w, eps, table, positions, slots, (bf16_t*)k_cache,
        (bf16_t*)v_cache, Hq, Hkv, D, page, store, num_tokens);
  else
    qk_norm_rope_store_kernel<float><<<grid, block, 0, stream>>>(
        (float*)qkv, row_stride, q_w, k_w, eps, table, positions, slots, (float*)k_cache,
        (float*)v_cache, Hq, Hkv, D, page, store, num_tokens);
  ME_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------------ stand-alone cache write
// k, v: [T, Hkv, D] with a token stride (views of a packed row are fine); bit-exact copies.
template <typename T>
__global__ void store_kv_kernel(const T* __restrict__ k, const T* __restrict__ v, int64_t k_stride,
                                int64_t v_stride, const int32_t* __restrict__ slots,
                                T* __restrict__ k_cache, T* __restrict__ v_cache, int Hkv, int D, int page) {
  const int64_t t = blockIdx.x;
  const int slot = slots[t];
  if (slot < 0) return;
  const int64_t pg = slot / page, off = slot - pg * page;
  const int n = Hkv * D;
  for (int e = threadIdx.x; e < n; e += blockDim.x) {
    const int h = e / D, d = e - h * D;
    k_cache[((pg * Hkv + h) * (int64_t)page + off) * D + d] = k[t * k_stride + e];
    v_cache[((pg * Hkv + h) * (int64_t)D + d) * page + off] = v[t * v_stride + e];
  }
}

extern "C" int me_store_kv(const void* k, const void* v, int dtype, int64_t num_tokens, int64_t k_stride,
                           int64_t v_stride, const int32_t* slots, void* k_cache, void* v_cache, int Hkv,
                           int D, int page, hipStream_t stream) {
  if (num_tokens == 0) return 0;
  ME_CHECK(Hkv >= 1 && D >= 1 && page >= 1, "store_kv: bad sizes");
  ME_CHECK(k_stride >= (int64_t)Hkv * D && v_stride >= (int64_t)Hkv * D, "store_kv: token stride too small");
  dim3 grid(num_tokens), block(256);
  if (dtype == ME_BF16)
    store_kv_kernel<bf16_t><<<grid, block, 0, stream>>>((const bf16_t*)k, (const bf16_t*)v, k_stride, v_stride,
                                                        slots, (bf16_t*)k_cache, (bf16_t*)v_cache, Hkv, D, page);
  else if (dtype == ME_F32)
    store_kv_kernel<float><<<grid, block, 0, stream>>>((const float*)k, (const float*)v, k_stride, v_stride,
                                                       slots, (float*)k_cache, (float*)v_cache, Hkv, D, page);
  else
    ME_CHECK(false, "store_kv: bad dtype code %d", dtype);
  ME_LAUNCH_CHECK();
  return 0;
}

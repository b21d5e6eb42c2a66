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

template <typename T>
__global__ void __launch_bounds__(256)
qk_norm_rope_store_kernel(T* __restrict__ qkv, int64_t row_stride, const float* __restrict__ q_w,
                          const float* __restrict__ k_w, float eps,
                          const float* __restrict__ table,  // [P, D/2, 2] cos,sin or null
                          const int32_t* __restrict__ positions, const int32_t* __restrict__ slots,
                          T* __restrict__ k_cache, T* __restrict__ v_cache, int Hq, int Hkv, int D,
                          int page, int store) {
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
    const int kvh = head - Hq - Hkv;
    const int slot = slots[t];
    if (slot < 0) return;
    const int64_t pg = slot / page, off = slot - pg * page;
    T* dst = v_cache + ((pg * Hkv + kvh) * (int64_t)D) * page + off;
    for (int d = lane; d < D; d += 64) dst[(int64_t)d * page] = row[d];
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

extern "C" int me_qk_norm_rope_store(void* qkv, int dtype, int64_t num_tokens, int64_t row_stride,
                                     const float* q_w, const float* k_w, float eps,
                                     const float* table, int64_t table_positions,
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
  const int heads = Hq + (store ? 2 * Hkv : Hkv);
  dim3 grid(num_tokens, (heads + 3) / 4), block(256);
  if (dtype == ME_BF16)
    qk_norm_rope_store_kernel<bf16_t><<<grid, block, 0, stream>>>(
        (bf16_t*)qkv, row_stride, q_w, k_w, eps, table, positions, slots, (bf16_t*)k_cache,
        (bf16_t*)v_cache, Hq, Hkv, D, page, store);
  else if (dtype == ME_F32)
    qk_norm_rope_store_kernel<float><<<grid, block, 0, stream>>>(
        (float*)qkv, row_stride, q_w, k_w, eps, table, positions, slots, (float*)k_cache,
        (float*)v_cache, Hq, Hkv, D, page, store);
  else
    ME_CHECK(false, "qk_norm_rope_store: bad dtype code %d", dtype);
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

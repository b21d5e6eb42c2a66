// Paged causal attention, the exact and slow form: one workgroup per (query token, head),
// scalar float32 arithmetic throughout. It is the float32 path of the engine and takes any
// head size, page size and head grouping.
//
// Formulas as in the reference's pure-torch paged path (layers/attention.py:21-40): key j of
// the request is kept iff j <= position of the query (and j < context length); scores are
// scale * q.k; softmax over kept keys; output = sum p_j v_j. A window w additionally keeps
// only j > position - w (not in the reference).
//
// Keys are processed in chunks whose boundaries are multiples of the chunk size counted from
// position 0 of the request, so the order of every sum for a given token is the same however
// the request was cut into steps or batched.
#include "common.h"

#define AS_THREADS 256

template <typename T>
__global__ void __launch_bounds__(AS_THREADS)
attn_simple_kernel(const T* __restrict__ q, int64_t q_stride, T* __restrict__ out, int64_t out_stride,
                   const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                   const int32_t* __restrict__ block_tables, int bt_stride,
                   const int32_t* __restrict__ seq_of_token, const int32_t* __restrict__ positions,
                   const int32_t* __restrict__ context_lens, int Hq, int Hkv, int D, int page, float scale,
                   int window) {
  extern __shared__ float lds[];
  float* qs = lds;                 // D
  float* sc = lds + D;             // AS_THREADS scores / probabilities
  __shared__ float red[16];

  const int64_t t = blockIdx.x;
  const int h = blockIdx.y;
  const int kvh = h / (Hq / Hkv);
  const int b = seq_of_token[t];
  const int pos = positions[t];
  const int32_t* bt = block_tables + (int64_t)b * bt_stride;
  const int tid = threadIdx.x;

  for (int d = tid; d < D; d += AS_THREADS) qs[d] = to_f32<T>(q[t * q_stride + (int64_t)h * D + d]);
  __syncthreads();

  // keys [lo, hi): up to the query's own position, never past the request's context (a padding
  // row has context 0 and sees nothing)
  const int hi = min(pos + 1, context_lens[b]);
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  float m = -INFINITY, l = 0.f;
  // thread d < D owns output channel d (two channels per thread when D > AS_THREADS)
  float acc0 = 0.f, acc1 = 0.f;

  for (int c0 = (lo / AS_THREADS) * AS_THREADS; c0 < hi; c0 += AS_THREADS) {
    const int j = c0 + tid;
    float s = -INFINITY;
    bool keep = j >= lo && j < hi;
    if (keep) {
      const int64_t pg = bt[j / page];
      keep = pg >= 0;                        // a page that is not held is never dereferenced
      if (keep) {
        const int off = j % page;
        const T* kr = k_cache + ((pg * Hkv + kvh) * (int64_t)page + off) * D;
        float dot = 0.f;
        for (int d = 0; d < D; ++d) dot += qs[d] * to_f32<T>(kr[d]);
        s = dot * scale;
      }
    }
    // chunk max
    float cm = wave_max(s);
    __syncthreads();
    if ((tid & 63) == 0) red[tid >> 6] = cm;
    __syncthreads();
    cm = red[0];
    for (int w = 1; w < AS_THREADS / 64; ++w) cm = fmaxf(cm, red[w]);
    const float m_new = fmaxf(m, cm);
    const float p = (keep && m_new > -INFINITY) ? expf(s - m_new) : 0.f;
    sc[tid] = p;
    float ps = wave_sum(p);
    __syncthreads();
    if ((tid & 63) == 0) red[8 + (tid >> 6)] = ps;
    __syncthreads();
    ps = 0.f;
    for (int w = 0; w < AS_THREADS / 64; ++w) ps += red[8 + w];
    const float alpha = (m == -INFINITY) ? 0.f : expf(m - m_new);   // m finite implies m_new finite
    l = l * alpha + ps;
    m = m_new;
    acc0 *= alpha;
    acc1 *= alpha;
    const int jb = max(c0, lo), je = min(c0 + AS_THREADS, hi);
    for (int dd = 0; dd < 2; ++dd) {
      const int d = tid + dd * AS_THREADS;
      if (d < D) {
        float a = 0.f;
        for (int jj = jb; jj < je; ++jj) {
          const int64_t pg = bt[jj / page];
          if (pg < 0) continue;                // its probability is 0
          const int off = jj % page;
          a += sc[jj - c0] * to_f32<T>(v_cache[((pg * Hkv + kvh) * (int64_t)D + d) * page + off]);
        }
        if (dd == 0) acc0 += a; else acc1 += a;
      }
    }
    __syncthreads();
  }
  const float inv = l > 0.f ? 1.f / l : 0.f;
  if (tid < D) out[t * out_stride + (int64_t)h * D + tid] = from_f32<T>(acc0 * inv);
  if (tid + AS_THREADS < D) out[t * out_stride + (int64_t)h * D + tid + AS_THREADS] = from_f32<T>(acc1 * inv);
}

extern "C" int me_attn_simple(const void* q, int64_t q_stride, void* out, int64_t out_stride, int dtype,
                              const void* k_cache, const void* v_cache, const int32_t* block_tables,
                              int bt_stride, const int32_t* seq_of_token, const int32_t* positions,
                              const int32_t* context_lens, int64_t num_tokens, int Hq, int Hkv, int D, int page, float scale, int window,
                              hipStream_t stream) {
  if (num_tokens == 0) return 0;
  ME_CHECK(Hq >= 1 && Hkv >= 1 && Hq % Hkv == 0, "attention: %d query heads are not a multiple of %d key heads", Hq, Hkv);
  ME_CHECK(D >= 1 && D <= 2 * AS_THREADS, "attention (float32 path): head_dim %d outside 1..%d", D, 2 * AS_THREADS);
  ME_CHECK(page >= 1 && window >= 0, "attention: bad page size or window");
  dim3 grid(num_tokens, Hq), block(AS_THREADS);
  size_t lds = (size_t)(D + AS_THREADS) * sizeof(float);
  if (dtype == ME_F32)
    attn_simple_kernel<float><<<grid, block, lds, stream>>>(
        (const float*)q, q_stride, (float*)out, out_stride, (const float*)k_cache, (const float*)v_cache,
        block_tables, bt_stride, seq_of_token, positions, context_lens, Hq, Hkv, D, page, scale, window);
  else if (dtype == ME_BF16)
    attn_simple_kernel<bf16_t><<<grid, block, lds, stream>>>(
        (const bf16_t*)q, q_stride, (bf16_t*)out, out_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache,
        block_tables, bt_stride, seq_of_token, positions, context_lens, Hq, Hkv, D, page, scale, window);
  else
    ME_CHECK(false, "attention: bad dtype code %d", dtype);
  ME_LAUNCH_CHECK();
  return 0;
}

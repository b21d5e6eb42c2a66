// Token choice from float32 logits: argmax at temperature 0, otherwise the exponential race of
// the reference's sampler (layers/sampler.py:5-11: argmax(softmax(z/T) / E), E ~ Exp(1)), which
// equals argmax(z/T - log E) and needs no softmax. One pass over the row, one workgroup per row.
//
// The noise is a function of (row key, vocabulary id) only, so a request's tokens do not depend
// on which other requests share the step (the reference draws from the global generator for the
// whole [S, V] matrix).
#include "common.h"

__device__ __forceinline__ uint32_t fmix32(uint32_t h) {
  h ^= h >> 16; h *= 0x85EBCA6Bu; h ^= h >> 13; h *= 0xC2B2AE35u; h ^= h >> 16;
  return h;
}

// E ~ Exp(1) for (key0, key1, v): u uniform in (0, 1) from 24 hashed bits, E = -log(u).
__device__ __forceinline__ float exp_noise(uint32_t key0, uint32_t key1, uint32_t v) {
  const uint32_t r = fmix32(fmix32(v ^ key0) + key1);
  const float u = ((float)(r >> 8) + 0.5f) * (1.0f / 16777216.0f);
  return -logf(u);
}

__global__ void __launch_bounds__(1024)
sample_kernel(const float* __restrict__ logits, int64_t ld, const float* __restrict__ temperatures,
              const uint32_t* __restrict__ keys, int32_t* __restrict__ out, int V) {
  __shared__ float bv[16];
  __shared__ int bi[16];
  const int row = blockIdx.x;
  const float* z = logits + (int64_t)row * ld;
  const float T = temperatures[row];
  const uint32_t k0 = keys[2 * row], k1 = keys[2 * row + 1];
  float best = -INFINITY;
  int best_i = 0x7fffffff;
  for (int v = threadIdx.x; v < V; v += blockDim.x) {
    float s = z[v];
    if (T > 0.f) s = s / T - logf(exp_noise(k0, k1, (uint32_t)v));
    if (s > best || (s == best && v < best_i)) { best = s; best_i = v; }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float ov = __shfl_xor(best, off, ME_WAVE);
    const int oi = __shfl_xor(best_i, off, ME_WAVE);
    if (ov > best || (ov == best && oi < best_i)) { best = ov; best_i = oi; }
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = (blockDim.x + 63) >> 6;
  if (lane == 0) { bv[wave] = best; bi[wave] = best_i; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < nwaves; ++w)
      if (bv[w] > best || (bv[w] == best && bi[w] < best_i)) { best = bv[w]; best_i = bi[w]; }
    out[row] = best_i == 0x7fffffff ? 0 : best_i;
  }
}

// keys: [S, 2] uint32 per row; temperatures: [S] float32 (0 = greedy); out: [S] int32.
extern "C" int me_sample(const float* logits, int64_t ld, const float* temperatures, const uint32_t* keys,
                         int32_t* out, int S, int V, hipStream_t stream) {
  if (S == 0) return 0;
  ME_CHECK(V >= 1 && ld >= V, "sample: bad vocabulary size or row stride");
  const int threads = V >= 4096 ? 1024 : (V >= 512 ? 256 : 64);
  sample_kernel<<<dim3(S), dim3(threads), 0, stream>>>(logits, ld, temperatures, keys, out, V);
  ME_LAUNCH_CHECK();
  return 0;
}

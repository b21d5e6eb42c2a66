// Token choice from float32 logits: argmax at temperature 0, otherwise the exponential race of
// the reference's sampler (layers/sampler.py:5-11: argmax(softmax(z/T) / E), E ~ Exp(1)), which
// equals argmax(z/T - log E) and needs no softmax. One pass over the row, one workgroup per row.
//
// The noise is a function of (row key, vocabulary id) only, so a request's tokens do not depend
// on which other requests share the step (the reference draws from the global generator for the
// whole [S, V] matrix).
#include "common.h"
#include "sampling.h"
#include <mutex>

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

// Stage 1: grid (chunks, rows). Each workgroup scans its share of the vocabulary and leaves its
// best (score, index). Stage 2: one wave per row takes the best of the chunks. Ties go to the
// lowest index at every stage, so the result does not depend on the number of chunks.
__device__ __forceinline__ bool better(float v, int i, float bv, int bi) { return v > bv || (v == bv && i < bi); }

__global__ void __launch_bounds__(256)
sample_scan_kernel(const float* __restrict__ logits, int64_t ld, const float* __restrict__ temperatures,
                   const uint32_t* __restrict__ keys, float* __restrict__ part_v, int32_t* __restrict__ part_i,
                   int V, int chunk) {
  __shared__ float bv[4];
  __shared__ int bi[4];
  const int row = blockIdx.y, c = blockIdx.x;
  const float* z = logits + (int64_t)row * ld;
  const float T = temperatures[row];
  const uint32_t k0 = keys[2 * row], k1 = keys[2 * row + 1];
  float best = -INFINITY;
  int best_i = 0x7fffffff;
  const int end = min(V, (c + 1) * chunk);
  for (int v = c * chunk + threadIdx.x; v < end; v += 256) {
    float s = z[v];
    if (T > 0.f) s = s / T - logf(exp_noise(k0, k1, (uint32_t)v));
    if (better(s, v, best, best_i)) { best = s; best_i = v; }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float ov = __shfl_xor(best, off, ME_WAVE);
    const int oi = __shfl_xor(best_i, off, ME_WAVE);
    if (better(ov, oi, best, best_i)) { best = ov; best_i = oi; }
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) { bv[wave] = best; bi[wave] = best_i; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 4; ++w)
      if (better(bv[w], bi[w], best, best_i)) { best = bv[w]; best_i = bi[w]; }
    part_v[(int64_t)row * gridDim.x + c] = best;
    part_i[(int64_t)row * gridDim.x + c] = best_i;
  }
}

__global__ void __launch_bounds__(64)
sample_merge_kernel(const float* __restrict__ part_v, const int32_t* __restrict__ part_i, int32_t* __restrict__ out,
                    int chunks) {
  const int row = blockIdx.x;
  float best = -INFINITY;
  int best_i = 0x7fffffff;
  for (int c = threadIdx.x; c < chunks; c += 64) {
    const float v = part_v[(int64_t)row * chunks + c];
    const int i = part_i[(int64_t)row * chunks + c];
    if (better(v, i, best, best_i)) { best = v; best_i = i; }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float ov = __shfl_xor(best, off, ME_WAVE);
    const int oi = __shfl_xor(best_i, off, ME_WAVE);
    if (better(ov, oi, best, best_i)) { best = ov; best_i = oi; }
  }
  if (threadIdx.x == 0) out[row] = best_i == 0x7fffffff ? 0 : best_i;
}

// Workgroups that share a row's vocabulary; the scratch holds (value, index) per row and chunk.
static int sample_chunks(int V) { return V >= 16384 ? 32 : (V >= 2048 ? 4 : 1); }

static int launch_sample(const float* logits, int64_t ld, const float* temperatures, const uint32_t* keys,
                         int32_t* out, void* scratch, int S, int V, hipStream_t stream) {
  ME_CHECK(V >= 1 && ld >= V, "sample: bad vocabulary size or row stride");
  ME_CHECK(S <= 65535, "sample: too many rows (%d)", S);
  const int chunks = sample_chunks(V);
  const int chunk = (V + chunks - 1) / chunks;
  float* pv = (float*)scratch;
  int32_t* pi = (int32_t*)scratch + (int64_t)S * chunks;
  sample_scan_kernel<<<dim3(chunks, S), dim3(256), 0, stream>>>(logits, ld, temperatures, keys, pv, pi, V, chunk);
  ME_LAUNCH_CHECK();
  sample_merge_kernel<<<dim3(S), dim3(64), 0, stream>>>(pv, pi, out, chunks);
  ME_LAUNCH_CHECK();
  return 0;
}

extern "C" int me_sample(const float* logits, int64_t ld, const float* temperatures, const uint32_t* keys,
                         int32_t* out, void* scratch, int S, int V, hipStream_t stream) {
  if (S == 0) return 0;
  ME_CHECK(scratch != nullptr, "sample: no scratch memory given");
  return launch_sample(logits, ld, temperatures, keys, out, scratch, S, V, stream);
}

// ---- the form that allocates nothing: its partial results live in this array.
// In host code the array's name is only a stand-in; the address that kernels and copies may use is
// asked for once per device (each GPU holds its own copy at its own address) and kept here.
static __device__ __align__(256) uint32_t g_sample_scratch[2 * ME_SAMPLE_STATIC_MAX_ROWS * 32];

#define ME_MAX_DEVICES 64
static void* g_sample_scratch_ptr[ME_MAX_DEVICES];      // per device; nullptr: not asked yet
static std::mutex g_sample_scratch_guard;

static int sample_scratch_of_current_device(void** ptr) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  ME_CHECK(e == hipSuccess, "sample_static: hipGetDevice: %s", hipGetErrorString(e));
  ME_CHECK(dev >= 0 && dev < ME_MAX_DEVICES, "sample_static: device %d beyond the %d this library keeps scratch for",
           dev, ME_MAX_DEVICES);
  std::lock_guard<std::mutex> hold(g_sample_scratch_guard);
  if (g_sample_scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(g_sample_scratch));
    ME_CHECK(e == hipSuccess && p != nullptr, "sample_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
    g_sample_scratch_ptr[dev] = p;
  }
  *ptr = g_sample_scratch_ptr[dev];
  return 0;
}

extern "C" int me_sample_static(const float* logits, int64_t ld, const float* temperatures, const uint32_t* keys,
                                int32_t* out, int S, int V, hipStream_t stream) {
  if (S == 0) return 0;
  ME_CHECK(S > 0 && S <= ME_SAMPLE_STATIC_MAX_ROWS,
           "sample_static: %d rows, the built-in scratch holds %d at most (use me_sample with a workspace)",
           S, ME_SAMPLE_STATIC_MAX_ROWS);
  void* scratch = nullptr;
  if (int rc = sample_scratch_of_current_device(&scratch)) return rc;
  return launch_sample(logits, ld, temperatures, keys, out, scratch, S, V, stream);
}

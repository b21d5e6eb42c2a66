// Shared device helpers for the gfx950 (CDNA4, wave64) kernels of mini_engine_amd.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdint>
#include <cstdio>
#include <cstring>

#define ME_WAVE 64

typedef __bf16 bf16_t;
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// Dtype codes shared with the Python binding.
enum { ME_BF16 = 0, ME_F32 = 1 };

// ---- error reporting: launchers return 0 or a negative code and leave a message here.
extern "C" const char* me_last_error();
void me_set_error(const char* fmt, ...);

#define ME_CHECK(cond, ...)              \
  do {                                   \
    if (!(cond)) {                       \
      me_set_error(__VA_ARGS__);         \
      return -1;                         \
    }                                    \
  } while (0)

#define ME_LAUNCH_CHECK()                                         \
  do {                                                            \
    hipError_t e_ = hipGetLastError();                            \
    if (e_ != hipSuccess) {                                       \
      me_set_error("kernel launch failed: %s", hipGetErrorString(e_)); \
      return -2;                                                  \
    }                                                             \
  } while (0)

template <typename T> __device__ __forceinline__ float to_f32(T v);
template <> __device__ __forceinline__ float to_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ float to_f32<bf16_t>(bf16_t v) { return static_cast<float>(v); }

template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float v) { return static_cast<bf16_t>(v); }

// Sum / max over the 64 lanes of a wave; every lane gets the result.
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, ME_WAVE);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, ME_WAVE));
  return v;
}

// Sum over a workgroup of up to 1024 threads; `scratch` holds >= 16 floats of LDS.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = (blockDim.x + 63) >> 6;
  v = wave_sum(v);
  __syncthreads();  // scratch may still be read from an earlier call
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < nwaves; ++w) total += scratch[w];
  return total;
}

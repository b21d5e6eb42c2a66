// Row gathers (embedding, logits rows), RMSNorm fused with the residual sum, SiLU-gating.
//
// What the reference does with eager torch ops: layers/embed_head.py:10-11 (gather),
// layers/layernorm.py:11-24 (RMSNorm, residual add), layers/activation.py:5-7 (SiLU*up).
// Here each is one kernel; the residual stream is kept in float32 and the sum, the
// mean of squares and the scaling are computed in float32.
#include "common.h"
#include "errors.inc"   // the core library's error channel lives in this file


// ------------------------------------------------------------------ gather rows
// out[r, :] = src[idx[r], :], rows of `row_bytes` bytes. One workgroup per row.
template <typename V>
__global__ void gather_rows_kernel(const V* __restrict__ src, const int32_t* __restrict__ idx,
                                   V* __restrict__ out, int64_t row_vecs, int64_t num_src_rows) {
  const int64_t r = blockIdx.x;
  int64_t s = idx[r];
  if (s < 0 || s >= num_src_rows) s = 0;  // the binding checks ids on the host; never read outside
  const V* a = src + s * row_vecs;
  V* b = out + r * row_vecs;
  for (int64_t i = threadIdx.x; i < row_vecs; i += blockDim.x) b[i] = a[i];
}

extern "C" int me_gather_rows(const void* src, const int32_t* idx, void* out, int64_t num_rows,
                              int64_t row_bytes, int64_t num_src_rows, hipStream_t stream) {
  if (num_rows == 0) return 0;
  ME_CHECK(row_bytes > 0 && num_src_rows > 0, "gather_rows: empty source");
  const bool a16 = row_bytes % 16 == 0 && (reinterpret_cast<uintptr_t>(src) % 16 == 0) &&
                   (reinterpret_cast<uintptr_t>(out) % 16 == 0);
  if (a16) {
    int64_t n = row_bytes / 16;
    int threads = n >= 256 ? 256 : (n > 64 ? 128 : 64);
    gather_rows_kernel<uint4><<<dim3(num_rows), dim3(threads), 0, stream>>>(
        (const uint4*)src, idx, (uint4*)out, n, num_src_rows);
  } else if (row_bytes % 2 == 0) {
    int64_t n = row_bytes / 2;
    gather_rows_kernel<uint16_t><<<dim3(num_rows), dim3(256), 0, stream>>>(
        (const uint16_t*)src, idx, (uint16_t*)out, n, num_src_rows);
  } else {
    gather_rows_kernel<uint8_t><<<dim3(num_rows), dim3(256), 0, stream>>>(
        (const uint8_t*)src, idx, (uint8_t*)out, row_bytes, num_src_rows);
  }
  ME_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------------ tokens handed over on the device
// tokens[r] = sampled[take[r]] for the rows whose take[r] >= 0; the other rows keep what they hold. A decode step
// that is launched before the step in flight has delivered its tokens takes them so from the sampling kernel's
// output (the reference fetches every token to the host first: engine/llm_engine.py:43-52).
__global__ void take_tokens_kernel(int32_t* __restrict__ tokens, const int32_t* __restrict__ sampled,
                                   const int32_t* __restrict__ take, int rows, int num_sampled) {
  const int r = blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= rows) return;
  const int t = take[r];
  if (t >= 0 && t < num_sampled) tokens[r] = sampled[t];
}

extern "C" int me_take_tokens(int32_t* tokens, const int32_t* sampled, const int32_t* take, int rows, int num_sampled,
                              hipStream_t stream) {
  if (rows <= 0) return 0;
  ME_CHECK(tokens && sampled && take && num_sampled > 0, "take_tokens: missing operand");
  take_tokens_kernel<<<dim3((rows + 255) / 256), dim3(256), 0, stream>>>(tokens, sampled, take, rows, num_sampled);
  ME_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------------ RMSNorm (+ residual)
// r = x (+ res_in)           summed in float32, kept in float32 as the new residual
// y = w * r * rsqrt(mean(r^2) + eps)
// x may be `num_partials` stacked float32 partial sums [P, T, n] (a split-K product whose
// partial results are added here, in a fixed order) or one tensor of the compute dtype.
// One workgroup per row; a thread owns groups of 4 consecutive elements, and all the loads of a
// group (every partial, the residual) are issued before any is used.
#define RN_MAX_PARTIALS 8

template <typename TX> struct Vec4;
template <> struct Vec4<float> {
  static __device__ __forceinline__ void load(const float* p, float (&v)[4]) {
    const float4 t = *reinterpret_cast<const float4*>(p);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
  }
  static __device__ __forceinline__ void store(float* p, const float (&v)[4]) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  }
};
template <> struct Vec4<bf16_t> {
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

// VEC: n % 4 == 0 and all pointers 16-byte aligned (rows then stay aligned); else scalar.
template <typename TX, typename TY, bool VEC>
__global__ void rms_norm_kernel(const TX* __restrict__ x, int num_partials, int64_t partial_stride,
                                const float* __restrict__ res_in, float* __restrict__ res_out,
                                const float* __restrict__ w, TY* __restrict__ y, int n, float eps) {
  __shared__ float scratch[16];
  extern __shared__ float row[];  // n floats: the summed row, so that it is read from memory once
  const int64_t t = blockIdx.x;
  const TX* xr = x + t * n;
  float ss = 0.f;
  if (VEC && n <= (int)blockDim.x * 4) {
    // every thread has at most one group of 4: it stays in registers, and the norm's weight is asked
    // for together with the row, so that nothing is fetched behind the workgroup's sum
    const int i = threadIdx.x * 4;
    const bool on = i < n;
    float part[RN_MAX_PARTIALS][4], r[4] = {0.f, 0.f, 0.f, 0.f}, wv[4] = {0.f, 0.f, 0.f, 0.f}, v[4] = {0.f, 0.f, 0.f, 0.f};
    if (on) {
#pragma unroll
      for (int p = 0; p < RN_MAX_PARTIALS; ++p)
        if (p < num_partials) Vec4<TX>::load(xr + p * partial_stride + i, part[p]);
      if (res_in) Vec4<float>::load(res_in + t * n + i, r);
      Vec4<float>::load(w + i, wv);
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = part[0][e];
#pragma unroll
      for (int p = 1; p < RN_MAX_PARTIALS; ++p)
        if (p < num_partials) {
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] += part[p][e];
        }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        v[e] += r[e];
        ss += v[e] * v[e];
      }
      if (res_out) Vec4<float>::store(res_out + t * n + i, v);
    }
    const float inv1 = rsqrtf(block_sum(ss, scratch) / (float)n + eps);
    if (on) {
      float o[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = wv[e] * (v[e] * inv1);
      Vec4<TY>::store(y + t * n + i, o);
    }
    return;
  }
  if (VEC) {
    for (int i = threadIdx.x * 4; i < n; i += blockDim.x * 4) {
      float part[RN_MAX_PARTIALS][4];
#pragma unroll
      for (int p = 0; p < RN_MAX_PARTIALS; ++p)
        if (p < num_partials) Vec4<TX>::load(xr + p * partial_stride + i, part[p]);
      float r[4] = {0.f, 0.f, 0.f, 0.f};
      if (res_in) Vec4<float>::load(res_in + t * n + i, r);
      float v[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = part[0][e];
#pragma unroll
      for (int p = 1; p < RN_MAX_PARTIALS; ++p)
        if (p < num_partials) {
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] += part[p][e];
        }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        v[e] += r[e];
        ss += v[e] * v[e];
        row[i + e] = v[e];
      }
      if (res_out) Vec4<float>::store(res_out + t * n + i, v);
    }
  } else {
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
      float v = to_f32<TX>(xr[i]);
      for (int p = 1; p < num_partials; ++p) v += to_f32<TX>(xr[p * partial_stride + i]);
      if (res_in) v += res_in[t * n + i];
      if (res_out) res_out[t * n + i] = v;
      row[i] = v;
      ss += v * v;
    }
  }
  const float total = block_sum(ss, scratch);
  const float inv = rsqrtf(total / (float)n + eps);
  if (VEC) {
    for (int i = threadIdx.x * 4; i < n; i += blockDim.x * 4) {
      float wv[4], o[4];
      Vec4<float>::load(w + i, wv);
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = wv[e] * (row[i + e] * inv);
      Vec4<TY>::store(y + t * n + i, o);
    }
  } else {
    for (int i = threadIdx.x; i < n; i += blockDim.x) y[t * n + i] = from_f32<TY>(w[i] * (row[i] * inv));
  }
}

// Many rows (prefill): one wave per row, the row held in registers, no LDS and no workgroup
// barrier; 4 rows per workgroup. A lane takes 8 consecutive values at a time (16 bytes of bfloat16,
// two 16-byte pieces of float32). Every load of the row is issued before the first value is used:
// a piece beyond the row's end is read from its start instead and not used.
#define RW_MAX_OCTS 10  // n <= 64 * 8 * RW_MAX_OCTS = 5120
template <typename T> struct Oct;
template <> struct Oct<float> {
  static __device__ __forceinline__ void load(const float* p, float (&v)[8]) {
    const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
  }
  static __device__ __forceinline__ void store(float* p, const float (&v)[8]) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
    *reinterpret_cast<float4*>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
  }
};
template <> struct Oct<bf16_t> {
  typedef bf16_t bf16x8v __attribute__((ext_vector_type(8)));
  static __device__ __forceinline__ void load(const bf16_t* p, float (&v)[8]) {
    const bf16x8v t = *reinterpret_cast<const bf16x8v*>(p);
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = static_cast<float>(t[i]);
  }
  static __device__ __forceinline__ void store(bf16_t* p, const float (&v)[8]) {
    bf16x8v t;
#pragma unroll
    for (int i = 0; i < 8; ++i) t[i] = static_cast<bf16_t>(v[i]);
    *reinterpret_cast<bf16x8v*>(p) = t;
  }
};

template <typename TX, typename TY, int OCTS>
__global__ void __launch_bounds__(256)
rms_norm_rows_kernel(const TX* __restrict__ x, const float* __restrict__ res_in, float* __restrict__ res_out,
                     const float* __restrict__ w, TY* __restrict__ y, int64_t num_rows, int n, float eps) {
  const int lane = threadIdx.x & 63;
  const int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= num_rows) return;
  float v[OCTS][8], r[OCTS][8];
#pragma unroll
  for (int q = 0; q < OCTS; ++q) {
    const int i = (q * 64 + lane) * 8;
    const int is = i < n ? i : 0;
    Oct<TX>::load(x + t * n + is, v[q]);
    if (res_in) Oct<float>::load(res_in + t * n + is, r[q]);
  }
  float ss = 0.f;
#pragma unroll
  for (int q = 0; q < OCTS; ++q) {
    const bool in = (q * 64 + lane) * 8 < n;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      if (res_in) v[q][e] += r[q][e];
      ss += in ? v[q][e] * v[q][e] : 0.f;
    }
    if (res_out && in) Oct<float>::store(res_out + t * n + (q * 64 + lane) * 8, v[q]);
  }
  const float inv = rsqrtf(wave_sum(ss) / (float)n + eps);
#pragma unroll
  for (int q = 0; q < OCTS; ++q) {
    const int i = (q * 64 + lane) * 8;
    if (i < n) {
      float wv[8], o[8];
      Oct<float>::load(w + i, wv);
#pragma unroll
      for (int e = 0; e < 8; ++e) o[e] = wv[e] * (v[q][e] * inv);
      Oct<TY>::store(y + t * n + i, o);
    }
  }
}

extern "C" int me_rms_norm(const void* x, int x_dtype, int num_partials, int64_t partial_stride,
                           const float* res_in, float* res_out, const float* w, void* y, int y_dtype,
                           int64_t num_rows, int n, float eps, hipStream_t stream) {
  if (num_rows == 0) return 0;
  ME_CHECK(n > 0 && n <= 36864, "rms_norm: width %d outside 1..36864", n);
  ME_CHECK(num_partials >= 1 && num_partials <= RN_MAX_PARTIALS, "rms_norm: %d partial sums outside 1..%d",
           num_partials, RN_MAX_PARTIALS);
  ME_CHECK(num_partials == 1 || x_dtype == ME_F32, "rms_norm: partial sums must be float32");
  auto al = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  const bool vec = n % 4 == 0 && al(x) && al(res_in) && al(res_out) && al(w) && al(y) &&
                   (num_partials == 1 || partial_stride % 4 == 0);
  if (vec && num_partials == 1 && num_rows >= 256 && n % 8 == 0 && n <= 64 * 8 * RW_MAX_OCTS) {
    dim3 grid((num_rows + 3) / 4), block(256);
    const int octs = (n + 511) / 512;
#define LAUNCH_ROWS(TX, TY, O) \
  rms_norm_rows_kernel<TX, TY, O><<<grid, block, 0, stream>>>((const TX*)x, res_in, res_out, w, (TY*)y, num_rows, n, eps)
#define PICK_ROWS(TX, TY)                                                                                   \
  do {                                                                                                      \
    if (octs <= 2) LAUNCH_ROWS(TX, TY, 2); else if (octs <= 4) LAUNCH_ROWS(TX, TY, 4);                      \
    else if (octs <= 8) LAUNCH_ROWS(TX, TY, 8); else LAUNCH_ROWS(TX, TY, RW_MAX_OCTS);                     \
  } while (0)
    if (x_dtype == ME_BF16 && y_dtype == ME_BF16) PICK_ROWS(bf16_t, bf16_t);
    else if (x_dtype == ME_F32 && y_dtype == ME_BF16) PICK_ROWS(float, bf16_t);
    else if (x_dtype == ME_F32 && y_dtype == ME_F32) PICK_ROWS(float, float);
    else if (x_dtype == ME_BF16 && y_dtype == ME_F32) PICK_ROWS(bf16_t, float);
    else ME_CHECK(false, "rms_norm: bad dtype codes %d %d", x_dtype, y_dtype);
#undef PICK_ROWS
#undef LAUNCH_ROWS
    ME_LAUNCH_CHECK();
    return 0;
  }
  int threads = vec ? (n / 4 >= 1024 ? 1024 : ((n / 4 + 63) / 64) * 64) : (n >= 512 ? 256 : (n >= 128 ? 128 : 64));
  if (threads < 64) threads = 64;
  size_t lds = (size_t)n * sizeof(float);
  dim3 grid(num_rows), block(threads);
#define LAUNCH(TX, TY)                                                                                    \
  do {                                                                                                    \
    if (vec)                                                                                              \
      rms_norm_kernel<TX, TY, true><<<grid, block, lds, stream>>>((const TX*)x, num_partials, partial_stride, \
                                                                  res_in, res_out, w, (TY*)y, n, eps);   \
    else                                                                                                  \
      rms_norm_kernel<TX, TY, false><<<grid, block, lds, stream>>>((const TX*)x, num_partials,            \
                                                                   partial_stride, res_in, res_out, w,   \
                                                                   (TY*)y, n, eps);                      \
  } while (0)
  if (x_dtype == ME_BF16 && y_dtype == ME_BF16) LAUNCH(bf16_t, bf16_t);
  else if (x_dtype == ME_F32 && y_dtype == ME_BF16) LAUNCH(float, bf16_t);
  else if (x_dtype == ME_F32 && y_dtype == ME_F32) LAUNCH(float, float);
  else if (x_dtype == ME_BF16 && y_dtype == ME_F32) LAUNCH(bf16_t, float);
  else ME_CHECK(false, "rms_norm: bad dtype codes %d %d", x_dtype, y_dtype);
#undef LAUNCH
  ME_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------------ SiLU(gate) * up
// gu: [T, 2I] with gate = first I columns (reference layers/activation.py:6); out: [T, I].
// VEC: a thread takes 16 bytes of gate and of up at a time (I a multiple of the vector length).
template <typename T, bool VEC>
__global__ void silu_and_mul_kernel(const T* __restrict__ gu, T* __restrict__ out, int64_t rows, int inter) {
  constexpr int W = VEC ? 16 / sizeof(T) : 1;
  const int per_row = inter / W;
  const int64_t total = rows * (int64_t)per_row;
  for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < total;
       e += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = e / per_row;
    const int i = (int)(e - t * per_row) * W;
    alignas(16) T g[W], u[W], o[W];
    if (VEC) {
      *reinterpret_cast<uint4*>(g) = *reinterpret_cast<const uint4*>(gu + t * 2 * inter + i);
      *reinterpret_cast<uint4*>(u) = *reinterpret_cast<const uint4*>(gu + t * 2 * inter + inter + i);
    } else {
      g[0] = gu[t * 2 * inter + i];
      u[0] = gu[t * 2 * inter + inter + i];
    }
#pragma unroll
    for (int j = 0; j < W; ++j) {
      const float gf = to_f32<T>(g[j]);
      o[j] = from_f32<T>(gf / (1.f + expf(-gf)) * to_f32<T>(u[j]));
    }
    if (VEC) *reinterpret_cast<uint4*>(out + t * inter + i) = *reinterpret_cast<const uint4*>(o);
    else out[t * inter + i] = o[0];
  }
}

extern "C" int me_silu_and_mul(const void* gu, void* out, int dtype, int64_t rows, int inter,
                               hipStream_t stream) {
  if (rows == 0) return 0;
  ME_CHECK(inter > 0, "silu_and_mul: intermediate size must be positive");
  ME_CHECK(dtype == ME_BF16 || dtype == ME_F32, "silu_and_mul: bad dtype code %d", dtype);
  const int w = dtype == ME_BF16 ? 8 : 4;
  const bool vec = inter % w == 0 && reinterpret_cast<uintptr_t>(gu) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0;
  const int64_t total = rows * (int64_t)(vec ? inter / w : inter);
  int64_t blocks = (total + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  dim3 grid(blocks), block(256);
  if (dtype == ME_BF16) {
    if (vec) silu_and_mul_kernel<bf16_t, true><<<grid, block, 0, stream>>>((const bf16_t*)gu, (bf16_t*)out, rows, inter);
    else silu_and_mul_kernel<bf16_t, false><<<grid, block, 0, stream>>>((const bf16_t*)gu, (bf16_t*)out, rows, inter);
  } else {
    if (vec) silu_and_mul_kernel<float, true><<<grid, block, 0, stream>>>((const float*)gu, (float*)out, rows, inter);
    else silu_and_mul_kernel<float, false><<<grid, block, 0, stream>>>((const float*)gu, (float*)out, rows, inter);
  }
  ME_LAUNCH_CHECK();
  return 0;
}

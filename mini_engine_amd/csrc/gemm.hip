// Matrix products y[M, N] = x[M, K] . w[N, K]^T (weights stored [out, in] as in the checkpoint;
// the reference calls F.linear for all of them: layers/linear.py:26,45, models/qwen3.py:21,47,
// layers/embed_head.py:23).
//
//  * me_gemm_tiled: any shape, float32 or bfloat16 inputs, float32 accumulation with plain FMAs
//    (no matrix-core, no reduced precision). Each output element is one thread's sequential sum
//    over K, so a row's result does not depend on the other rows of the batch. This is the
//    float32 path and the fallback for bf16 shapes the MFMA kernel refuses.
//  * me_gemm_skinny_bf16: the decode product, up to 64 rows (the caller decides from which row
//    count the library is faster). Pure weight streaming: each workgroup owns 16 output features, its 4 waves split
//    K, a wave reads 256 contiguous bytes of each of its 16 weight rows per step (each load takes 64
//    contiguous bytes per row; over large weights 256 contiguous bytes of each of four rows, see the wide loads
//    below), the fetches run one step ahead of the products, products on
//    v_mfma_f32_16x16x32_bf16 with the tokens as the 16-wide B operand, waves merged through
//    LDS. Optional split of K over workgroups writes float32 partial sums [S, M, N] that the
//    consumer (the fused residual + RMSNorm kernel) adds in a fixed order.
#include "common.h"


// ------------------------------------------------------------------ tiled FMA product
#define GT_TILE 64
#define GT_BK 16

template <typename TI, typename TO>
__global__ void __launch_bounds__(256)
gemm_tiled_kernel(const TI* __restrict__ x, int64_t ldx, const TI* __restrict__ w, int64_t ldw,
                  TO* __restrict__ y, int64_t ldy, int M, int N, int K) {
  __shared__ float xs[GT_BK][GT_TILE + 1];
  __shared__ float ws[GT_BK][GT_TILE + 1];
  const int tid = threadIdx.x;
  const int m0 = blockIdx.y * GT_TILE, n0 = blockIdx.x * GT_TILE;
  const int tm = (tid / 16) * 4, tn = (tid % 16) * 4;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += GT_BK) {
    // 64 rows x 16 k = 1024 elements per operand, 4 per thread; consecutive threads read along k
    for (int e = tid; e < GT_TILE * GT_BK; e += 256) {
      const int r = e / GT_BK, kk = e % GT_BK;
      const int k = k0 + kk;
      xs[kk][r] = (m0 + r < M && k < K) ? to_f32<TI>(x[(int64_t)(m0 + r) * ldx + k]) : 0.f;
      ws[kk][r] = (n0 + r < N && k < K) ? to_f32<TI>(w[(int64_t)(n0 + r) * ldw + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < GT_BK; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) { a[i] = xs[kk][tm + i]; b[i] = ws[kk][tn + i]; }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int m = m0 + tm + i, n = n0 + tn + j;
      if (m < M && n < N) y[(int64_t)m * ldy + n] = from_f32<TO>(acc[i][j]);
    }
}

extern "C" int me_gemm_tiled(const void* x, int64_t ldx, const void* w, int64_t ldw, void* y, int64_t ldy,
                             int in_dtype, int out_dtype, int M, int N, int K, hipStream_t stream) {
  if (M == 0 || N == 0) return 0;
  ME_CHECK(K >= 1 && ldx >= K && ldw >= K && ldy >= N, "gemm: bad leading dimensions");
  dim3 grid((N + GT_TILE - 1) / GT_TILE, (M + GT_TILE - 1) / GT_TILE), block(256);
  ME_CHECK(grid.y <= 65535, "gemm: too many rows (%d) for one launch", M);
#define LAUNCH(TI, TO) \
  gemm_tiled_kernel<TI, TO><<<grid, block, 0, stream>>>((const TI*)x, ldx, (const TI*)w, ldw, (TO*)y, ldy, M, N, K)
  if (in_dtype == ME_F32 && out_dtype == ME_F32) LAUNCH(float, float);
  else if (in_dtype == ME_BF16 && out_dtype == ME_BF16) LAUNCH(bf16_t, bf16_t);
  else if (in_dtype == ME_BF16 && out_dtype == ME_F32) LAUNCH(bf16_t, float);
  else ME_CHECK(false, "gemm: unsupported dtype pair %d -> %d", in_dtype, out_dtype);
#undef LAUNCH
  ME_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------------ skinny bf16 product on MFMA
__device__ __forceinline__ bf16x8 gz8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = static_cast<bf16_t>(0.f);
  return z;
}

// MT: 16-token tiles per workgroup. Grid (ceil(N/16), ceil(M/(16*MT)), ksplit).
// k-slot mapping of MFMA j (0..3) inside a 128-wide macro step s: lane group g supplies
// k = 128 s + 32 j + 8 g + 0..7 for both operands, so the four lanes of a row read 64 contiguous
// bytes with every load.
// GATED: x is [M, 2K] and the B operand is silu(x[:, k]) * x[:, K + k], formed in float32 and
// rounded once to bfloat16 (the SiLU-gating of the feed-forward fused into its down product).
__device__ __forceinline__ bf16x8 silu_mul8(const bf16x8 g, const bf16x8 u) {
  bf16x8 r;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const float gf = static_cast<float>(g[i]), uf = static_cast<float>(u[i]);
    // the hardware's exp2 and reciprocal (about 1 ulp each, far below the bfloat16 rounding that follows):
    // every workgroup gates its tokens for itself, and the exact forms cost it about 2 us
    r[i] = static_cast<bf16_t>(gf * __frcp_rn(1.f + __expf(-gf)) * uf);
  }
  return r;
}

// ---- wide loads of a weight that a launch reads once (skinny and rows kernels, large weights)
// A load of a wave in the plain pattern takes 64 bytes of each of sixteen rows, so that a row's 128-byte line is
// asked for by two loads; marked as not to be kept by the caches, the second asks the memory again, and the mark,
// which this GPU's memory answers with a higher rate, gains nothing. In the wide pattern load j of lane (piece r, g)
// takes piece r (16 bytes) of the step's 256 bytes from row 4 j + g of the wave's sixteen: whole lines, marked.
// The pieces then pass through a tile of the wave's own in LDS, 16 rows 272 bytes apart (so that the 16 rows a read
// takes at once are spread over all banks, and every address is a lane's base plus a constant), to the lanes that
// the matrix instruction wants them in: lane (row r, g) gets the pieces 4 j + g of row r. A wave's LDS operations
// run in the order they are issued, so what its lanes write, its lanes read behind it without a barrier.
#define WIDE_TILE_BYTES (16 * 272)
__device__ __forceinline__ bf16x8 wide_load(const bf16_t* w, uint32_t byte_offset) {
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  return __builtin_bit_cast(bf16x8, __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(
                                        reinterpret_cast<const unsigned char*>(w) + byte_offset)));
}
__device__ __forceinline__ void wide_to_lanes(unsigned char* tile, int r, int g, const bf16x8 (&loaded)[4], bf16x8 (&a)[4]) {
#pragma unroll
  for (int j = 0; j < 4; ++j) *reinterpret_cast<bf16x8*>(tile + (g * 272 + r * 16) + j * (4 * 272)) = loaded[j];
  asm volatile("" ::: "memory");
#pragma unroll
  for (int j = 0; j < 4; ++j) a[j] = *reinterpret_cast<const bf16x8*>(tile + (r * 272 + g * 16) + j * 64);
  asm volatile("" ::: "memory");
}

// One macro step's operands. Loads are unconditional (a row or a k beyond the matrix is read from
// row 0 / k 0 instead and zeroed afterwards), so they all go out together and the next step's
// loads are in flight while this step's products run.
// Keeps the loads issued so far where they are. A value that is loaded in one loop iteration and
// first used in the next reaches its use through a phi, and the compiler rewrites "phi of loads"
// into "load of a phi of addresses": the load then sits in front of its use and nothing is in
// flight ahead. Something that may write memory between the load and the end of its block forbids
// that rewrite; an empty statement that claims to do so costs no instruction and no wait.
__device__ __forceinline__ void pin_loads() { asm volatile("" ::: "memory"); }

// Operand sets in the ring: fetches run SKINNY_DEPTH - 1 steps ahead. One step ahead and 86 registers
// (5 waves per SIMD) streams faster than two or four steps ahead with fewer waves: measured on
// 34-524 MB weights, 3.8-5.1 TB/s against 3.2-4.6 and 2.6-4.2.
#define SKINNY_DEPTH 2

template <int MT, bool GATED>
struct SkinnyOperands {
  bf16x8 a[4];
  bf16x8 b[MT][4];
  bf16x8 u[GATED ? MT : 1][4];
};

// EXACT_K: K is a multiple of 128, so no k-slot of any step lies beyond K and nothing is zeroed.
// Rows beyond N or M are read from row 0 and not zeroed either: an output element depends on its
// own weight row and token row only, and the elements of such rows are never written.
// ACT (one tile of tokens, K not split): w is a packed gate/up weight [N = 2 I, K], gate rows first (reference
// layers/linear.py:29-45), and y is silu(gate) * up, [M, I] (layers/activation.py:5-7): a workgroup takes 8 gate
// features and the 8 up features that go with them as the 16 rows of its matrix operand and pairs them when it
// merges its waves, so every gate is formed once, from the unrounded sums.
// WIDE (one tile of tokens, EXACT_K, not GATED; for large weights): the weights come by the wide loads above (a
// kernel that only reads a 201-524 MB weight: 5.3-6.1 TB/s in the plain pattern, 5.9-6.9 so).
template <int MT, typename TO, bool GATED, bool EXACT_K, bool ACT = false, bool WIDE = false>
__global__ void __launch_bounds__(256, WIDE ? 5 : 1)
gemm_skinny_kernel(const bf16_t* __restrict__ x, int64_t ldx, const bf16_t* __restrict__ w, int64_t ldw,
                   TO* __restrict__ y, int64_t ldy, float* __restrict__ partials, int M, int N, int K,
                   int steps_per_split) {
  static_assert(!WIDE || (MT == 1 && !GATED && EXACT_K), "the wide loads are built for one tile of tokens and whole steps");
  __shared__ float red[4][MT][256];
  __shared__ __align__(16) unsigned char wtile[WIDE ? 4 : 1][WIDE ? WIDE_TILE_BYTES : 16];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * (ACT ? 8 : 16), m0 = blockIdx.y * 16 * MT;
  const int split = blockIdx.z;
  const int s_begin = split * steps_per_split;
  const int total_steps = (K + 127) / 128;
  const int s_end = min(total_steps, s_begin + steps_per_split);

  const int half = N >> 1;                 // ACT: gate features 0..half-1, their up features behind them
  int feature;
  if (ACT) feature = n0 + (r & 7) < half ? (r < 8 ? n0 + r : half + n0 + r - 8) : 0;
  else feature = n0 + r < N ? n0 + r : 0;
  const bf16_t* wrow = w + (int64_t)feature * ldw;
  // WIDE: load j of lane (piece r, g) takes piece r of the step from row 4 j + g of the workgroup's sixteen, as a
  // byte offset from w (the launcher admits weights under 2 GB) formed where it is used: four row addresses kept
  // would not fit the registers of five waves to a SIMD
  const uint32_t ldw_bytes = (uint32_t)ldw * 2u;
  auto wide_offset = [&](int j, int s) -> uint32_t {
    const int rr = 4 * j + g;
    int f;
    if (ACT) f = j < 2 ? min(n0 + rr, half - 1) : half + min(n0 + rr - 8, half - 1);
    else f = min(n0 + rr, N - 1);
    return (uint32_t)f * ldw_bytes + 16u * (uint32_t)r + 256u * (uint32_t)s;
  };
  const bf16_t* xrow[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = m0 + 16 * mt + r;
    xrow[mt] = x + (int64_t)(m < M ? m : 0) * ldx;
  }
  f32x4 acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
  const bf16x8 z = gz8();

  // A fetch for a step beyond the wave's last (live == false) reads the first 16 bytes of w and x in
  // every lane: one cache line for the whole wave instead of sixteen rows, and still no branch.
  auto fetch = [&](int s, bool live, SkinnyOperands<MT, GATED>& op) {
    const int kb = 128 * s + 8 * g;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int k = kb + 32 * j;
      const int ks = (EXACT_K || k < K) ? k : 0;
      if (WIDE) {
        op.a[j] = wide_load(w, live ? wide_offset(j, s) : 0u);
      } else {
        op.a[j] = *reinterpret_cast<const bf16x8*>(live ? wrow + ks : w);
      }
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        op.b[mt][j] = *reinterpret_cast<const bf16x8*>(live ? xrow[mt] + ks : x);
        if (GATED) op.u[mt][j] = *reinterpret_cast<const bf16x8*>(live ? xrow[mt] + K + ks : x);
      }
    }
  };
  auto product = [&](int s, const SkinnyOperands<MT, GATED>& op) {
    const int kb = 128 * s + 8 * g;
    bf16x8 wide_a[4];
    if (WIDE) wide_to_lanes(wtile[wave], r, g, op.a, wide_a);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const bool kok = EXACT_K || kb + 32 * j < K;
      const bf16x8 a = WIDE ? wide_a[j] : (kok ? op.a[j] : z);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        bf16x8 b = op.b[mt][j];
        if (GATED) b = silu_mul8(b, op.u[mt][j]);
        acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[mt], 0, 0, 0);
      }
    }
  };

  // This wave's macro steps are s_begin + wave, + 4, ... Up to two steps: both fetched at once.
  // More: a ring of SKINNY_DEPTH operand sets keeps the fetches of the next SKINNY_DEPTH - 1 steps
  // in flight while a step's products run; a fetch past the wave's last step reads one line (no
  // fetch sits behind a branch) and its products are skipped.
  int s = s_begin + wave;
  if (s < s_end) {
    const int last = s + ((s_end - 1 - s) >> 2 << 2);   // this wave's last step
    if (last <= s + 4) {
      SkinnyOperands<MT, GATED> first, second;
      fetch(s, true, first);
      if (last > s) fetch(last, true, second);
      pin_loads();
      product(s, first);
      if (last > s) product(last, second);
    } else {
      SkinnyOperands<MT, GATED> ring[SKINNY_DEPTH];
#pragma unroll
      for (int d = 0; d < SKINNY_DEPTH - 1; ++d) fetch(s + 4 * d, s + 4 * d <= last, ring[d]);
      pin_loads();
      while (s <= last) {
#pragma unroll
        for (int u = 0; u < SKINNY_DEPTH; ++u) {
          const int ahead = s + 4 * (SKINNY_DEPTH - 1);
          fetch(ahead, ahead <= last, ring[(u + SKINNY_DEPTH - 1) % SKINNY_DEPTH]);
          pin_loads();
          if (s <= last) product(s, ring[u]);
          s += 4;
        }
      }
    }
  }
  // accumulator: lane (token r, g) holds features n0 + 4g + i
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int i = 0; i < 4; ++i) red[wave][mt][r * 16 + 4 * g + i] = acc[mt][i];
  __syncthreads();
  if (ACT) {
    const int idx = threadIdx.x, m = idx >> 3, f = idx & 7;
    if (idx < 128 && m0 + m < M && n0 + f < half) {
      const int ig = m * 16 + f, iu = ig + 8;
      const float gate = red[0][0][ig] + red[1][0][ig] + red[2][0][ig] + red[3][0][ig];
      const float up = red[0][0][iu] + red[1][0][iu] + red[2][0][iu] + red[3][0][iu];
      y[(int64_t)(m0 + m) * ldy + n0 + f] = from_f32<TO>(gate / (1.f + expf(-gate)) * up);
    }
    return;
  }
  for (int e = threadIdx.x; e < MT * 256; e += 256) {
    const int mt = e >> 8, idx = e & 255;
    const int m = m0 + 16 * mt + (idx >> 4), n = n0 + (idx & 15);
    if (m < M && n < N) {
      const float v = red[0][mt][idx] + red[1][mt][idx] + red[2][mt][idx] + red[3][mt][idx];
      if (partials) partials[((int64_t)split * M + m) * N + n] = v;
      else y[(int64_t)m * ldy + n] = from_f32<TO>(v);
    }
  }
}

// ------------------------------------------------------------------ the same product for 17 to 64 tokens
// With that many tokens the skinny kernel's token fetches (all tokens again in every workgroup of 16
// features) outweigh its weight fetches several times. Here a workgroup owns 64 features, one tile of
// 16 per wave, and every wave walks the whole k-range of the split; the tokens of 512 k at a time are
// staged once per workgroup in LDS and serve all four waves, so they cost a quarter as much. Weights go
// from memory straight into the matrix operand registers, one step ahead, as in the skinny kernel.
// LDS layout: row m holds the chunk's 64 granules of 16 bytes; granule q lies at q ^ (m & 15) within
// its group of 16, which spreads the 16 rows a wave reads at once over all banks without padding.
#define ROWS_CHUNK 512                      // k per staged chunk: 4 steps of 128
#define ROWS_GRANULES (ROWS_CHUNK / 8)

// EXACT_K: K is a multiple of the chunk, so neither a step nor a staged granule lies beyond K.
// WIDE (EXACT_K only): the weights come by the wide loads, as in the skinny kernel.
template <int MT, typename TO, bool EXACT_K, bool WIDE = false>
__global__ void __launch_bounds__(256)
gemm_rows_kernel(const bf16_t* __restrict__ x, int64_t ldx, const bf16_t* __restrict__ w, int64_t ldw,
                 TO* __restrict__ y, int64_t ldy, float* __restrict__ partials, int M, int N, int K,
                 int chunks_per_split) {
  static_assert(!WIDE || EXACT_K, "the wide loads are built for whole steps");
  extern __shared__ __align__(16) unsigned char rows_lds[];
  __shared__ __align__(16) unsigned char wtile[WIDE ? 4 : 1][WIDE ? WIDE_TILE_BYTES : 16];
  bf16_t* xs = reinterpret_cast<bf16_t*>(rows_lds);     // [16 * MT][ROWS_CHUNK]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * 64 + wave * 16;
  const int split = blockIdx.z;
  const int total_chunks = (K + ROWS_CHUNK - 1) / ROWS_CHUNK;
  const int c_begin = split * chunks_per_split;
  const int c_end = min(total_chunks, c_begin + chunks_per_split);
  const bf16_t* wrow = w + (int64_t)(n0 + r < N ? n0 + r : 0) * ldw;
  const bf16x8 z = gz8();
  const int rows = min(M, 16 * MT);

  const uint32_t ldw_bytes = (uint32_t)ldw * 2u;        // WIDE: byte offsets from w (the launcher admits weights under 2 GB)
  auto fetch = [&](int s, bool live, bf16x8 (&a)[4]) {
    const int kb = 128 * s + 8 * g;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (WIDE) {
        a[j] = wide_load(w, live ? (uint32_t)min(n0 + 4 * j + g, N - 1) * ldw_bytes + 16u * (uint32_t)r + 256u * (uint32_t)s : 0u);
      } else {
        const int k = kb + 32 * j;
        a[j] = *reinterpret_cast<const bf16x8*>(live && (EXACT_K || k < K) ? wrow + k : w);
      }
    }
  };
  f32x4 acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int s_last = min((K + 127) / 128, 4 * c_end) - 1;       // the split's last step
  bf16x8 ring[2][4];
  fetch(4 * c_begin, true, ring[0]);
  pin_loads();

  for (int c = c_begin; c < c_end; ++c) {
    // the tokens of this chunk into LDS: 8 granules of a thread go out together
    const int total = rows * ROWS_GRANULES;
    for (int e0 = threadIdx.x; e0 < total; e0 += 256 * 8) {
      bf16x8 v[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int e = e0 + 256 * i < total ? e0 + 256 * i : e0;   // beyond the end: the first again, no branch
        const int m = e / ROWS_GRANULES, q = e % ROWS_GRANULES;
        const int k = ROWS_CHUNK * c + 8 * q;
        v[i] = *reinterpret_cast<const bf16x8*>(x + (int64_t)m * ldx + ((EXACT_K || k < K) ? k : 0));
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int e = e0 + 256 * i;
        if (e < total) {
          const int m = e / ROWS_GRANULES, q = e % ROWS_GRANULES;
          bf16x8 t = v[i];
          if (!EXACT_K && ROWS_CHUNK * c + 8 * q >= K) t = z;
          *reinterpret_cast<bf16x8*>(xs + m * ROWS_CHUNK + 8 * ((q & ~15) | ((q ^ m) & 15))) = t;
        }
      }
    }
    __syncthreads();
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int s = 4 * c + u;
      fetch(s + 1, s + 1 <= s_last, ring[(u + 1) & 1]);
      pin_loads();
      if (s <= s_last) {
        bf16x8 wide_a[4];
        if (WIDE) wide_to_lanes(wtile[wave], r, g, ring[u & 1], wide_a);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const bool kok = EXACT_K || 128 * s + 32 * j + 8 * g < K;
          const bf16x8 a = WIDE ? wide_a[j] : (kok ? ring[u & 1][j] : z);
          const int q = 16 * u + 4 * j + g;           // granule of k = 128 s + 32 j + 8 g inside the chunk
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) {
            const int m = 16 * mt + r < rows ? 16 * mt + r : 0;
            const bf16x8 b = *reinterpret_cast<const bf16x8*>(xs + m * ROWS_CHUNK + 8 * ((q & ~15) | ((q ^ m) & 15)));
            acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[mt], 0, 0, 0);
          }
        }
      }
    }
    __syncthreads();      // the next chunk overwrites what the slowest wave may still read
  }
  // accumulator: lane (token r, g) holds features n0 + 4g + i
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = 16 * mt + r, n = n0 + 4 * g;
    if (m < M) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (n + i < N) {
          if (partials) partials[((int64_t)split * M + m) * N + n + i] = acc[mt][i];
          else y[(int64_t)m * ldy + n + i] = from_f32<TO>(acc[mt][i]);
        }
    }
  }
}

// wide: the caller asks for the wide loads; they apply to a K in whole chunks and a weight under 2 GB.
extern "C" int me_gemm_rows_bf16(const void* x, int64_t ldx, const void* w, int64_t ldw, void* y, int64_t ldy,
                                 int out_dtype, float* partials, int ksplit, int M, int N, int K, int wide,
                                 hipStream_t stream) {
  if (M == 0 || N == 0) return 0;
  ME_CHECK(M <= 64, "rows gemm: at most 64 rows (%d)", M);
  ME_CHECK(K >= 8 && K % 8 == 0 && ldx % 8 == 0 && ldw % 8 == 0,
           "rows gemm: K=%d and the row strides must be multiples of 8", K);
  ME_CHECK((reinterpret_cast<uintptr_t>(x) % 16 == 0) && (reinterpret_cast<uintptr_t>(w) % 16 == 0),
           "rows gemm: operands must be 16-byte aligned");
  ME_CHECK(ksplit >= 1 && (ksplit == 1) == (partials == nullptr), "rows gemm: partials iff ksplit > 1");
  const int total_chunks = (K + ROWS_CHUNK - 1) / ROWS_CHUNK;
  const int chunks_per_split = (total_chunks + ksplit - 1) / ksplit;
  ME_CHECK((int64_t)(ksplit - 1) * chunks_per_split < total_chunks, "rows gemm: ksplit %d leaves a split without work", ksplit);
  const int mt = (M + 15) / 16;
  const size_t lds = (size_t)16 * mt * ROWS_CHUNK * sizeof(bf16_t);
  dim3 grid((N + 63) / 64, 1, ksplit), block(256);
  const bool exact = K % ROWS_CHUNK == 0;   // whole chunks: the staging reads no k beyond K either
#define LAUNCH1(MTV, TO, E)                                                                                     \
  gemm_rows_kernel<MTV, TO, E><<<grid, block, lds, stream>>>((const bf16_t*)x, ldx, (const bf16_t*)w, ldw, (TO*)y, \
                                                             ldy, partials, M, N, K, chunks_per_split)
#define LAUNCH_WIDE(MTV, TO)                                                                                          \
  gemm_rows_kernel<MTV, TO, true, true><<<grid, block, lds, stream>>>((const bf16_t*)x, ldx, (const bf16_t*)w, ldw,   \
                                                                      (TO*)y, ldy, partials, M, N, K, chunks_per_split)
  const bool wide_ok = wide && exact && (int64_t)(N - 1) * ldw + K <= (int64_t)0x3fffffff;
#define LAUNCH2(MTV, TO)                                                                                       \
  do {                                                                                                         \
    if (wide_ok) LAUNCH_WIDE(MTV, TO); else if (exact) LAUNCH1(MTV, TO, true); else LAUNCH1(MTV, TO, false);   \
  } while (0)
#define LAUNCH(TO)                                                                             \
  do {                                                                                         \
    if (mt == 1) LAUNCH2(1, TO); else if (mt == 2) LAUNCH2(2, TO); else if (mt == 3) LAUNCH2(3, TO); \
    else LAUNCH2(4, TO);                                                                       \
  } while (0)
  if (out_dtype == ME_F32 || partials) LAUNCH(float);
  else if (out_dtype == ME_BF16) LAUNCH(bf16_t);
  else ME_CHECK(false, "rows gemm: bad output dtype code %d", out_dtype);
#undef LAUNCH
#undef LAUNCH2
#undef LAUNCH_WIDE
#undef LAUNCH1
  ME_LAUNCH_CHECK();
  return 0;
}

// y: bf16 or float32 [M, N]; or, when ksplit > 1, `partials` float32 [ksplit, M, N] (y unused).
// gated: x is [M, 2K] and silu(x[:, :K]) * x[:, K:] is what is multiplied. act: w is a packed gate/up weight and y
// is silu(gate) * up, [M, N / 2] (at most 16 rows, K not split, not together with gated).
extern "C" int me_gemm_skinny_bf16(const void* x, int64_t ldx, const void* w, int64_t ldw, void* y,
                                   int64_t ldy, int out_dtype, float* partials, int ksplit, int M, int N,
                                   int K, int gated, int act, int wide, hipStream_t stream) {
  if (M == 0 || N == 0) return 0;
  // wide: the caller asks for the wide loads (large weights); they apply to one tile of tokens, K in whole steps of
  // 128, an ungated input and a weight under 2 GB, and are left out otherwise
  const bool wide_ok = wide && M <= 16 && !gated && K % 128 == 0 && (int64_t)(N - 1) * ldw + K <= (int64_t)0x3fffffff;
  if (act) {
    ME_CHECK(!gated && ksplit == 1 && partials == nullptr && M <= 16 && N % 2 == 0,
             "skinny gemm: the gating epilogue takes at most 16 rows, an unsplit K and an even number of weight rows");
    ME_CHECK(K >= 8 && K % 8 == 0 && ldx % 8 == 0 && ldw % 8 == 0 && ldy >= N / 2,
             "skinny gemm: K=%d and the row strides must be multiples of 8", K);
    ME_CHECK((reinterpret_cast<uintptr_t>(x) % 16 == 0) && (reinterpret_cast<uintptr_t>(w) % 16 == 0),
             "skinny gemm: operands must be 16-byte aligned");
    const int steps = (K + 127) / 128;
    dim3 grid((N / 2 + 7) / 8, 1, 1), block(256);
#define LAUNCH_ACT(TO, E)                                                                                    \
  gemm_skinny_kernel<1, TO, false, E, true><<<grid, block, 0, stream>>>((const bf16_t*)x, ldx, (const bf16_t*)w, ldw, \
                                                                        (TO*)y, ldy, nullptr, M, N, K, steps)
    if (out_dtype == ME_BF16 && wide_ok) {
      gemm_skinny_kernel<1, bf16_t, false, true, true, true><<<grid, block, 0, stream>>>(
          (const bf16_t*)x, ldx, (const bf16_t*)w, ldw, (bf16_t*)y, ldy, nullptr, M, N, K, steps);
    } else if (out_dtype == ME_BF16) { if (K % 128 == 0) LAUNCH_ACT(bf16_t, true); else LAUNCH_ACT(bf16_t, false); }
    else if (out_dtype == ME_F32) { if (K % 128 == 0) LAUNCH_ACT(float, true); else LAUNCH_ACT(float, false); }
    else ME_CHECK(false, "skinny gemm: bad output dtype code %d", out_dtype);
#undef LAUNCH_ACT
    ME_LAUNCH_CHECK();
    return 0;
  }
  ME_CHECK(K >= 8 && K % 8 == 0 && ldx % 8 == 0 && ldw % 8 == 0,
           "skinny gemm: K=%d and the row strides must be multiples of 8", K);
  ME_CHECK((reinterpret_cast<uintptr_t>(x) % 16 == 0) && (reinterpret_cast<uintptr_t>(w) % 16 == 0),
           "skinny gemm: operands must be 16-byte aligned");
  ME_CHECK(ksplit >= 1 && (ksplit == 1) == (partials == nullptr), "skinny gemm: partials iff ksplit > 1");
  const int total_steps = (K + 127) / 128;
  ME_CHECK(ksplit <= total_steps, "skinny gemm: ksplit %d exceeds the %d K-steps of 128", ksplit, total_steps);
  const int steps_per_split = (total_steps + ksplit - 1) / ksplit;
  const int mt = M > 32 ? 4 : (M > 16 ? 2 : 1);
  dim3 grid((N + 15) / 16, (M + 16 * mt - 1) / (16 * mt), ksplit), block(256);
  ME_CHECK(grid.y <= 65535, "skinny gemm: too many rows (%d)", M);
  ME_CHECK(!gated || ldx >= 2 * (int64_t)K, "skinny gemm: gated input rows must hold 2K values");
  const bool exact = K % 128 == 0;
#define LAUNCH1(MTV, TO, G, E)                                                                               \
  gemm_skinny_kernel<MTV, TO, G, E><<<grid, block, 0, stream>>>((const bf16_t*)x, ldx, (const bf16_t*)w, ldw, \
                                                                (TO*)y, ldy, partials, M, N, K, steps_per_split)
#define LAUNCH(MTV, TO)                                                                                      \
  do {                                                                                                       \
    if (exact) LAUNCH1(MTV, TO, false, true); else LAUNCH1(MTV, TO, false, false);                           \
  } while (0)
#define LAUNCH_GATED(TO)                                                                                     \
  do {                                                                                                       \
    if (exact) LAUNCH1(1, TO, true, true); else LAUNCH1(1, TO, true, false);                                 \
  } while (0)
  ME_CHECK(!gated || mt == 1, "skinny gemm: the gated form takes at most 16 rows (%d)", M);
  if (wide_ok && (out_dtype == ME_F32 || out_dtype == ME_BF16 || partials)) {
    if (out_dtype == ME_F32 || partials)
      gemm_skinny_kernel<1, float, false, true, false, true><<<grid, block, 0, stream>>>(
          (const bf16_t*)x, ldx, (const bf16_t*)w, ldw, (float*)y, ldy, partials, M, N, K, steps_per_split);
    else
      gemm_skinny_kernel<1, bf16_t, false, true, false, true><<<grid, block, 0, stream>>>(
          (const bf16_t*)x, ldx, (const bf16_t*)w, ldw, (bf16_t*)y, ldy, partials, M, N, K, steps_per_split);
  } else if (out_dtype == ME_F32 || partials) {
    if (gated) LAUNCH_GATED(float); else if (mt == 4) LAUNCH(4, float); else if (mt == 2) LAUNCH(2, float); else LAUNCH(1, float);
  } else if (out_dtype == ME_BF16) {
    if (gated) LAUNCH_GATED(bf16_t); else if (mt == 4) LAUNCH(4, bf16_t); else if (mt == 2) LAUNCH(2, bf16_t); else LAUNCH(1, bf16_t);
  } else {
    ME_CHECK(false, "skinny gemm: bad output dtype code %d", out_dtype);
  }
#undef LAUNCH_GATED
#undef LAUNCH
#undef LAUNCH1
  ME_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------------ the skinny product behind an RMSNorm
// y = (gamma * r / rms(r)) . w^T with r = the sum of the partial sums (+ the residual): what the norm kernel and
// the skinny product do one after the other (reference layers/layernorm.py:11-24, then layers/linear.py:25-26),
// as one launch, for a handful of rows. 1 / rms(r) is one number per row, so it is applied to the finished sums
// in float32; the product itself runs on gamma * r rounded to bfloat16. Every workgroup forms that operand for
// itself in LDS while its first weights are on their way (all M rows: M x K x (S + 1) floats out of L2) and adds
// up r^2; the first workgroup also writes r, the new residual. K is not split. For one or two rows over a small
// weight this saves about a microsecond of the six that the two launches take (1024 -> 4096: 5.4 against 6.4 us);
// from three rows on, and over weights whose stream the prologue delays (4096 -> 24576: 44.8 against 41.4 us), the
// two launches are faster, so the launcher takes at most NORM_MAX_ROWS rows.
#define NORM_MAX_PARTIALS 8
#define NORM_MAX_ROWS 2

template <typename TX> struct Quad4;
template <> struct Quad4<float> {
  static __device__ __forceinline__ void load(const float* p, float (&v)[4]) {
    const float4 t = *reinterpret_cast<const float4*>(p); v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
  }
};
template <> struct Quad4<bf16_t> {
  static __device__ __forceinline__ void load(const bf16_t* p, float (&v)[4]) {
    const bf16x4 t = *reinterpret_cast<const bf16x4*>(p);
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = static_cast<float>(t[i]);
  }
};

template <typename TX, typename TO, bool EXACT_K, bool ACT>
__global__ void __launch_bounds__(256)
gemm_skinny_norm_kernel(const TX* __restrict__ xp, int S, int64_t part_stride, const float* __restrict__ res_in,
                        float* __restrict__ res_out, const float* __restrict__ gamma, float eps,
                        const bf16_t* __restrict__ w, int64_t ldw, TO* __restrict__ y, int64_t ldy, int M, int N,
                        int K) {
  extern __shared__ __align__(16) unsigned char norm_lds[];
  const int ldx = K + 8;                                   // a row shifts by 16 bytes against the one before
  bf16_t* xs = reinterpret_cast<bf16_t*>(norm_lds);        // [M][ldx] gamma * r
  float* red = reinterpret_cast<float*>(norm_lds + (((size_t)M * ldx * sizeof(bf16_t) + 15) & ~(size_t)15));   // [4][256]
  float* ssw = red + 4 * 256;                              // [4 waves][16 rows] sums of r^2
  float* inv = ssw + 64;                                   // [16] 1 / rms
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * (ACT ? 8 : 16);
  const int total_steps = (K + 127) / 128;
  const int half = N >> 1;                                 // ACT: as in gemm_skinny_kernel
  int feature;
  if (ACT) feature = n0 + (r & 7) < half ? (r < 8 ? n0 + r : half + n0 + r - 8) : 0;
  else feature = n0 + r < N ? n0 + r : 0;
  const bf16_t* wrow = w + (int64_t)feature * ldw;
  const bf16x8 z = gz8();

  auto fetch = [&](int s, bool live, bf16x8 (&a)[4]) {
    const int kb = 128 * s + 8 * g;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int k = kb + 32 * j;
      a[j] = *reinterpret_cast<const bf16x8*>(live && (EXACT_K || k < K) ? wrow + k : w);
    }
  };
  bf16x8 ring[2][4];
  int s = wave;
  fetch(s, s < total_steps, ring[0]);
  pin_loads();

  // ---- the rows: r = partial sums + residual, r^2 added up, gamma * r into LDS
  constexpr int RA = NORM_MAX_ROWS;                        // rows whose loads go out together
  const int quads = K >> 2;
  for (int m0 = 0; m0 < M; m0 += RA) {
    float ssr[RA];
#pragma unroll
    for (int a = 0; a < RA; ++a) ssr[a] = 0.f;
    for (int q = threadIdx.x; q < quads; q += 256) {
      float part[RA][NORM_MAX_PARTIALS][4], res[RA][4], gq[4];
      Quad4<float>::load(gamma + 4 * q, gq);
#pragma unroll
      for (int a = 0; a < RA; ++a) {
        const int m = m0 + a < M ? m0 + a : m0;
#pragma unroll
        for (int p = 0; p < NORM_MAX_PARTIALS; ++p)
          if (p < S) Quad4<TX>::load(xp + p * part_stride + (int64_t)m * K + 4 * q, part[a][p]);
        if (res_in) Quad4<float>::load(res_in + (int64_t)m * K + 4 * q, res[a]);
      }
#pragma unroll
      for (int a = 0; a < RA; ++a) {
        const int m = m0 + a;
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = part[a][0][e];
#pragma unroll
        for (int p = 1; p < NORM_MAX_PARTIALS; ++p)
          if (p < S) {
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] += part[a][p][e];
          }
        if (res_in) {
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] += res[a][e];
        }
        if (m < M) {
          bf16x4 o;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            ssr[a] += v[e] * v[e];
            o[e] = static_cast<bf16_t>(gq[e] * v[e]);
          }
          *reinterpret_cast<bf16x4*>(xs + m * ldx + 4 * q) = o;
          if (blockIdx.x == 0 && res_out)
            *reinterpret_cast<float4*>(res_out + (int64_t)m * K + 4 * q) = make_float4(v[0], v[1], v[2], v[3]);
        }
      }
    }
#pragma unroll
    for (int a = 0; a < RA; ++a) {
      const float total = wave_sum(ssr[a]);
      if (lane == 0 && m0 + a < M) ssw[wave * 16 + m0 + a] = total;
    }
  }
  __syncthreads();
  if (threadIdx.x < M) {
    const int m = threadIdx.x;
    inv[m] = rsqrtf((ssw[m] + ssw[16 + m] + ssw[32 + m] + ssw[48 + m]) / (float)K + eps);
  }

  // ---- the product: weights from memory one step ahead, the rows from LDS
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  const bf16_t* xrow = xs + (r < M ? r : 0) * ldx;
  auto product = [&](int step, const bf16x8 (&a)[4]) {
    const int kb = 128 * step + 8 * g;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int k = kb + 32 * j;
      const bool kok = EXACT_K || k < K;
      const bf16x8 b = *reinterpret_cast<const bf16x8*>(xrow + (kok ? k : 0));
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kok ? a[j] : z, b, acc, 0, 0, 0);
    }
  };
  while (s < total_steps) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      fetch(s + 4, s + 4 < total_steps, ring[u ^ 1]);
      pin_loads();
      if (s < total_steps) product(s, ring[u]);
      s += 4;
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) red[wave * 256 + r * 16 + 4 * g + i] = acc[i];
  __syncthreads();
  const int idx = threadIdx.x;
  if (ACT) {
    const int m = idx >> 3, f = idx & 7;
    if (idx < 128 && m < M && n0 + f < half) {
      const int ig = m * 16 + f, iu = ig + 8;
      const float gate = (red[ig] + red[256 + ig] + red[512 + ig] + red[768 + ig]) * inv[m];
      const float up = (red[iu] + red[256 + iu] + red[512 + iu] + red[768 + iu]) * inv[m];
      y[(int64_t)m * ldy + n0 + f] = from_f32<TO>(gate / (1.f + expf(-gate)) * up);
    }
  } else {
    const int m = idx >> 4, n = n0 + (idx & 15);
    if (m < M && n < N) {
      const float v = red[idx] + red[256 + idx] + red[512 + idx] + red[768 + idx];
      y[(int64_t)m * ldy + n] = from_f32<TO>(v * inv[m]);
    }
  }
}

// xp: bfloat16 or float32 [S, M, K] (S = 1: the rows themselves), contiguous; res_in float32 [M, K] or null;
// res_out float32 [M, K] or null; gamma float32 [K]. y bfloat16 or float32 with row stride ldy: [M, N], or with
// act (w a packed gate/up weight, as in me_gemm_skinny_bf16) silu(gate) * up, [M, N / 2].
extern "C" int me_gemm_skinny_norm_bf16(const void* xp, int x_dtype, int S, const float* res_in, float* res_out,
                                        const float* gamma, float eps, const void* w, int64_t ldw, void* y,
                                        int64_t ldy, int out_dtype, int M, int N, int K, int act,
                                        hipStream_t stream) {
  if (M == 0 || N == 0) return 0;
  ME_CHECK(M <= NORM_MAX_ROWS, "norm + skinny gemm: at most %d rows (%d)", NORM_MAX_ROWS, M);
  ME_CHECK(S >= 1 && S <= NORM_MAX_PARTIALS, "norm + skinny gemm: %d partial sums outside 1..%d", S, NORM_MAX_PARTIALS);
  ME_CHECK(K >= 8 && K % 8 == 0 && ldw % 8 == 0, "norm + skinny gemm: K=%d and the weight's row stride must be multiples of 8", K);
  ME_CHECK(x_dtype == ME_F32 || (x_dtype == ME_BF16 && S == 1), "norm + skinny gemm: partial sums must be float32");
  for (const void* p : {xp, (const void*)res_in, (const void*)res_out, (const void*)gamma, w})
    ME_CHECK(reinterpret_cast<uintptr_t>(p) % 16 == 0, "norm + skinny gemm: operands must be 16-byte aligned");
  ME_CHECK(!act || N % 2 == 0, "norm + skinny gemm: a packed gate/up weight has an even number of rows (%d)", N);
  ME_CHECK(xp && gamma && w && y && ldy >= (act ? N / 2 : N), "norm + skinny gemm: null operand or short output rows");
  const size_t lds = ((size_t)M * (K + 8) * sizeof(bf16_t) + 15) / 16 * 16 + (4 * 256 + 64 + 16) * sizeof(float);
  ME_CHECK(lds <= 64 * 1024, "norm + skinny gemm: %d rows of %d do not fit the workgroup's LDS", M, K);
  dim3 grid(act ? (N / 2 + 7) / 8 : (N + 15) / 16), block(256);
  const bool exact = K % 128 == 0;
  const int64_t part_stride = (int64_t)M * K;
#define LAUNCH1(TX, TO, E, A)                                                                                \
  gemm_skinny_norm_kernel<TX, TO, E, A><<<grid, block, lds, stream>>>((const TX*)xp, S, part_stride, res_in, \
      res_out, gamma, eps, (const bf16_t*)w, ldw, (TO*)y, ldy, M, N, K)
#define LAUNCH2(TX, TO, E) do { if (act) LAUNCH1(TX, TO, E, true); else LAUNCH1(TX, TO, E, false); } while (0)
#define LAUNCH3(TX, TO) do { if (exact) LAUNCH2(TX, TO, true); else LAUNCH2(TX, TO, false); } while (0)
  if (x_dtype == ME_F32 && out_dtype == ME_BF16) LAUNCH3(float, bf16_t);
  else if (x_dtype == ME_BF16 && out_dtype == ME_BF16) LAUNCH3(bf16_t, bf16_t);
  else if (x_dtype == ME_F32 && out_dtype == ME_F32) LAUNCH3(float, float);
  else if (x_dtype == ME_BF16 && out_dtype == ME_F32) LAUNCH3(bf16_t, float);
  else ME_CHECK(false, "norm + skinny gemm: bad dtype codes %d -> %d", x_dtype, out_dtype);
#undef LAUNCH3
#undef LAUNCH2
#undef LAUNCH1
  ME_LAUNCH_CHECK();
  return 0;
}

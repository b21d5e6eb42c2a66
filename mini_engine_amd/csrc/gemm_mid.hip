// y[M, N] = x[M, K] . w[N, K]^T for 65 to a few hundred rows over weights of a few million elements: the decode
// products of large batches at small model widths (reference layers/linear.py:26,45: F.linear). These products
// are 1-3 GFLOP over a few megabytes; what they cost is the way from the first load to the last store.
//
// A workgroup owns a tile of 64 tokens x 64 features; its 4 waves are 2 x 2 sub-tiles of 32 x 32. K is walked
// 64 at a time. The loads write LDS themselves (global_load_lds_dwordx4: every lane names 16 bytes of memory,
// the 64 pieces of a wave's instruction land in 1 KB of consecutive LDS), three stages deep, so no operand
// passes through registers on its way in and an iteration does not wait for its own loads. A stage holds the
// tile's 64 token rows and 64 weight rows, 128 bytes each; the 16-byte piece c of row R lies at position
// c ^ (R >> 1 & 7), so that the 16 lanes of an operand read (rows R..R+15, one piece each) touch 16 different
// bank groups. Products on v_mfma_f32_16x16x32_bf16 with the weight rows as the A operand and the token rows
// as B: a lane then holds 4 consecutive features of one token. K may be split over workgroups (grid z): float32
// partial sums [S, M, N] for a consumer that adds them. Workgroups that share weight rows run on the same XCD.
// An iteration is a chain of wait, barrier, LDS reads and 8 products (about 500 cycles for 128 cycles of matrix
// work), so the kernel takes 7 us whatever the row count up to 256 and loses to the library's larger tiles
// beyond; the caller (ops.mid_takes) knows where it is ahead. Where K is a multiple of 128 an iteration walks 128 of
// K instead (BK = 128: rows of 256 bytes, 16 pieces, piece c of row R at position c ^ (R & 15); 96 KB of LDS for
// the three stages): half as many iterations, each with 16 products behind the same wait and barrier.
#include "common.h"

#define MID_TM 64
#define MID_TN 64
#define MID_NB 3                                      // stages in LDS (48 or 96 KB): two asked for ahead of the one in use

// gbase and lds_addr are the same in every lane; the first lane's values are taken so that they lie in scalar
// registers whatever the compiler has concluded about them. The write to m0 needs one wait state before an
// instruction that reads it for an LDS address.
__device__ __forceinline__ void mid_dma16(const bf16_t* gbase, uint32_t voff, uint32_t lds_addr) {
  const uint64_t g = reinterpret_cast<uint64_t>(gbase);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(g >> 32)), lo = __builtin_amdgcn_readfirstlane((uint32_t)g);
  const uint64_t base = (uint64_t)hi << 32 | lo;
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(__builtin_amdgcn_readfirstlane(lds_addr)), "v"(voff), "s"(base) : "memory");
}
template <int N>
__device__ __forceinline__ void mid_wait() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }
__device__ __forceinline__ void mid_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// ACT: w is a packed gate/up weight [2 I, K] (gate rows first, N = 2 I); the tile's 64 weight rows are 32 gate rows and
// the 32 up rows that go with them, a wave's two feature tiles are 16 gate features and their up features, and what
// is written is silu(gate) * up [M, I], formed from the unrounded sums (reference layers/activation.py:5-7).
template <typename TO, bool PARTIAL, bool ACT, int MID_BK>
__global__ void __launch_bounds__(256)
gemm_mid_kernel(const bf16_t* __restrict__ x, int64_t ldx, const bf16_t* __restrict__ w, int64_t ldw,
                TO* __restrict__ y, int64_t ldy, int M, int N, int K, int steps_per_split, int m_tiles, int n_tiles) {
  extern __shared__ __align__(16) unsigned char mid_lds[];   // [MID_NB][MID_STAGE]
  static_assert(MID_BK == 64 || MID_BK == 128, "a row of a stage is 128 or 256 bytes");
  constexpr int ROW = 2 * MID_BK;                                    // bytes of a row in LDS
  constexpr int MID_STAGE = (MID_TM + MID_TN) * ROW;                // bytes
  constexpr int ROWS_PER_DMA = 1024 / ROW;                           // rows that one instruction of a wave brings
  constexpr int MID_DMA_PER_WAVE = (MID_TM + MID_TN) / ROWS_PER_DMA / 4;
  constexpr int PIECES = ROW / 16;                                   // 16-byte pieces of a row
  constexpr int PD = MID_NB - 1;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 15, g = lane >> 4;
  // consecutive workgroup ids go to different XCDs: the low 3 bits pick the feature tile's XCD, and the token
  // tiles of one feature tile follow each other on it
  const int id = blockIdx.x;
  const int rest = id >> 3;
  const int mt = rest % m_tiles;
  const int nt = (rest / m_tiles) * 8 + (id & 7);
  if (nt >= n_tiles) return;
  const int I = N / 2;                              // ACT only
  const int m0 = mt * MID_TM, n0 = nt * (ACT ? MID_TN / 2 : MID_TN);
  const int steps = K / MID_BK;
  const int s_lo = blockIdx.z * steps_per_split;
  const int s_hi = min(steps, s_lo + steps_per_split);
  const int nsteps = s_hi - s_lo;

  // what a lane names in memory for each of its wave's instructions of a stage: 8 rows of 128 bytes; rows beyond
  // the matrix are read from its last row and never stored
  uint32_t voff[MID_DMA_PER_WAVE];
  bool is_x[MID_DMA_PER_WAVE];
#pragma unroll
  for (int q = 0; q < MID_DMA_PER_WAVE; ++q) {
    const int inst = wave + 4 * q;                 // 0 .. (TM + TN) / rows per instruction - 1; token rows first
    const int R = ROWS_PER_DMA * inst + lane / PIECES;
    const int c = (lane % PIECES) ^ (MID_BK == 64 ? (R >> 1) & 7 : R & 15);
    is_x[q] = inst < MID_TM / ROWS_PER_DMA;
    const int wr = R - MID_TM;                      // weight row of the tile
    const int64_t row = is_x[q] ? min(m0 + R, M - 1)
                        : ACT ? (wr < 32 ? min(n0 + wr, I - 1) : I + min(n0 + wr - 32, I - 1))
                              : min(n0 + wr, N - 1);
    voff[q] = (uint32_t)(row * (is_x[q] ? ldx : ldw) * 2 + 16 * c);
  }
  const uint32_t lds0 = (uint32_t)(uintptr_t)mid_lds;
  auto stage = [&](int s, int bi) {
#pragma unroll
    for (int q = 0; q < MID_DMA_PER_WAVE; ++q) {
      const int inst = wave + 4 * q;
      mid_dma16((is_x[q] ? x : w) + (int64_t)s * MID_BK, voff[q], lds0 + bi * MID_STAGE + inst * 1024);
    }
  };
  // where this lane reads its operands: token rows of the wave's half, weight rows of its half
  const int wm = wave >> 1, wn = wave & 1;
  const int swz = MID_BK == 64 ? (n >> 1) & 7 : n;
  constexpr int KS = MID_BK / 32;                  // matrix instructions' steps of 32 along K in a stage
  uint32_t rd_b[KS], rd_a[KS];
#pragma unroll
  for (int s = 0; s < KS; ++s) {
    rd_b[s] = (wm * 32 + n) * ROW + (((4 * s + g) ^ swz) * 16);
    rd_a[s] = (MID_TM + wn * (ACT ? 16 : 32) + n) * ROW + (((4 * s + g) ^ swz) * 16);
  }
  f32x4 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

#pragma unroll
  for (int k = 0; k < PD; ++k)
    if (k < nsteps) stage(s_lo + k, k);
  int cur = 0;
  for (int k = 0; k < nsteps; ++k) {
    // stage k has landed: at most the PD - 1 stages asked for after it are still on their way
    if (k + PD <= nsteps) mid_wait<MID_DMA_PER_WAVE * (PD - 1)>(); else mid_wait<0>();
    mid_barrier();                                 // ... for every wave, and the buffer of stage k - 1 is free
    if (k + PD < nsteps) stage(s_lo + k + PD, cur == 0 ? MID_NB - 1 : cur - 1);
    const unsigned char* buf = mid_lds + cur * MID_STAGE;
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      bf16x8 a[2], b[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) a[i] = *reinterpret_cast<const bf16x8*>(buf + rd_a[s] + (ACT ? 32 : 16) * ROW * i);
#pragma unroll
      for (int j = 0; j < 2; ++j) b[j] = *reinterpret_cast<const bf16x8*>(buf + rd_b[s] + 16 * ROW * j);
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
    }
    cur = cur == MID_NB - 1 ? 0 : cur + 1;
  }
  // lane (n, g) of tile (i, j): features n0 + 32 wn + 16 i + 4 g .. + 3 of token m0 + 32 wm + 16 j + n
  // (ACT: tile 0 holds the gates and tile 1 the up values of features n0 + 16 wn + 4 g .. + 3)
  TO* out = PARTIAL ? y + (int64_t)blockIdx.z * M * ldy : y;
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int t = m0 + wm * 32 + 16 * j + n;
    if constexpr (ACT) {
      const int f = n0 + wn * 16 + 4 * g;
      if (t < M && f < I) {
        typedef TO out4 __attribute__((ext_vector_type(4)));
        out4 r;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float gate = acc[0][j][e];
          r[e] = from_f32<TO>(gate / (1.f + __expf(-gate)) * acc[1][j][e]);
        }
        *reinterpret_cast<out4*>(out + (int64_t)t * ldy + f) = r;
      }
    } else {
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int f = n0 + wn * 32 + 16 * i + 4 * g;
        if (t < M && f < N) {
          if constexpr (PARTIAL) {
            *reinterpret_cast<f32x4*>(out + (int64_t)t * ldy + f) = acc[i][j];
          } else {
            typedef TO out4 __attribute__((ext_vector_type(4)));
            out4 r;
#pragma unroll
            for (int e = 0; e < 4; ++e) r[e] = from_f32<TO>(acc[i][j][e]);
            *reinterpret_cast<out4*>(out + (int64_t)t * ldy + f) = r;
          }
        }
      }
    }
  }
}

// y: [M, N] of out_dtype (ksplit 1), or float32 partial sums [ksplit, M, N] with ldy = N; act: w is a packed
// gate/up weight [N = 2 I, K] and y is silu(gate) * up [M, I] (bfloat16, ksplit 1).
extern "C" int me_gemm_mid_bf16(const void* x, int64_t ldx, const void* w, int64_t ldw, void* y, int64_t ldy,
                                int out_dtype, int ksplit, int M, int N, int K, int act, hipStream_t stream) {
  if (M == 0 || N == 0) return 0;
  ME_CHECK(K >= 64 && K % 64 == 0, "mid gemm: K=%d must be a multiple of 64", K);
  ME_CHECK(N % 4 == 0 && ldy % 4 == 0 && ldx % 8 == 0 && ldw % 8 == 0, "mid gemm: N=%d and the row strides must keep 16-byte pieces whole", N);
  ME_CHECK((reinterpret_cast<uintptr_t>(x) % 16 == 0) && (reinterpret_cast<uintptr_t>(w) % 16 == 0) &&
               (reinterpret_cast<uintptr_t>(y) % 16 == 0), "mid gemm: operands must be 16-byte aligned");
  ME_CHECK((int64_t)M * ldx * 2 < (1ll << 32) && (int64_t)N * ldw * 2 < (1ll << 32), "mid gemm: an operand beyond 4 GB");
  ME_CHECK(ksplit >= 1 && ksplit <= K / 64, "mid gemm: %d slices of %d steps", ksplit, K / 64);
  ME_CHECK(ksplit == 1 || out_dtype == ME_F32, "mid gemm: partial sums are float32");
  // steps of 128 where K is in whole steps of 128 and every slice still gets one; else steps of 64
  bool wide_steps = K % 128 == 0 && (int64_t)(ksplit - 1) * ((K / 128 + ksplit - 1) / ksplit) < K / 128;
  const int bk = wide_steps ? 128 : 64;
  const int steps = K / bk;
  const int steps_per_split = (steps + ksplit - 1) / ksplit;
  ME_CHECK((int64_t)(ksplit - 1) * steps_per_split < steps, "mid gemm: ksplit %d leaves a slice without work", ksplit);
  ME_CHECK(!act || (ksplit == 1 && out_dtype == ME_BF16 && N % 8 == 0), "mid gemm: the gating wants one bfloat16 result and I a multiple of 4");
  const int m_tiles = (M + MID_TM - 1) / MID_TM, n_tiles = act ? (N / 2 + MID_TN / 2 - 1) / (MID_TN / 2) : (N + MID_TN - 1) / MID_TN;
  const int64_t ids = (int64_t)((n_tiles + 7) / 8) * 8 * m_tiles;
  ME_CHECK(ids < (1ll << 31), "mid gemm: too many tiles");
  const dim3 grid((unsigned)ids, 1, ksplit), block(256);
  const size_t lds = (size_t)MID_NB * (MID_TM + MID_TN) * 2 * bk;
#define MID_LAUNCH1(TO, P, A, BK)                                                                                        \
  gemm_mid_kernel<TO, P, A, BK><<<grid, block, lds, stream>>>((const bf16_t*)x, ldx, (const bf16_t*)w, ldw, (TO*)y, ldy, \
                                                             M, N, K, steps_per_split, m_tiles, n_tiles)
#define MID_LAUNCH(TO, P, A)                                                                                       \
  do {                                                                                                             \
    if (wide_steps) {                                                                                              \
      static bool allowed = false;                   /* 96 KB of LDS: more than a kernel may have unasked */       \
      if (!allowed) {                                                                                              \
        hipError_t e = hipFuncSetAttribute((const void*)gemm_mid_kernel<TO, P, A, 128>,                            \
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);                  \
        ME_CHECK(e == hipSuccess, "mid gemm: cannot get %zu bytes of LDS: %s", lds, hipGetErrorString(e));         \
        allowed = true;                                                                                            \
      }                                                                                                            \
      MID_LAUNCH1(TO, P, A, 128);                                                                                  \
    } else {                                                                                                       \
      MID_LAUNCH1(TO, P, A, 64);                                                                                   \
    }                                                                                                              \
  } while (0)
  if (act) MID_LAUNCH(bf16_t, false, true);
  else if (ksplit > 1) MID_LAUNCH(float, true, false);
  else if (out_dtype == ME_F32) MID_LAUNCH(float, false, false);
  else MID_LAUNCH(bf16_t, false, false);
#undef MID_LAUNCH
#undef MID_LAUNCH1
  ME_LAUNCH_CHECK();
  return 0;
}

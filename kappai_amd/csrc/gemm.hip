// Matrix products  C[M,N] = A[M,K] * W[N,K]^T (+ bias[N])  for every projection and the
// output head.  W is a weight matrix [out, in] with `in` contiguous, as stored in the
// checkpoint (kappai: y[n] = sum_k W[n,k] x[k], src/backend/cpu/scalar/quants.c:1398-1414).
//
//   gemm_f32         true 32-bit on the vector ALUs: every product and sum is an fp32 FMA in
//                    the order k = 0..K-1, so a row's result does not depend on M.
//   gemm_bf16_block256  large products (K a multiple of 128 per K range): bf16 inputs, fp32
//                    accumulation on the matrix cores (v_mfma_f32_32x32x16_bf16), 256x256 or
//                    128x128 blocks, tiles of 64 of K loaded straight into LDS.
//   gemm_bf16_tile   any K that is a multiple of 8: 256x128 or 128x128 blocks staged through
//                    registers into LDS.
//   gemm_bf16_skinny M <= 64 (decode): every block streams 16 or 32 rows of W once, its 4 to 16
//                    waves split K and meet in LDS (v_mfma_f32_16x16x32_bf16).
//   gemm_bf16_shared_rows  17 <= M <= 64 and a W with many rows: as above, but two waves that
//                    stream different rows of W share the rows of A through LDS.
//   gemm_bf16_rows32 25 <= M <= 128: the same idea with 32 x 32 tiles (v_mfma_f32_32x32x16_bf16),
//                    W from its fragment-order copy.
//   gemm_bf16_any    K or a row stride that is no multiple of 8: a plain kernel, so that no
//                    width is refused.
#include "common.h"
#include "gemm_rules.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;

// ---------------------------------------------------------------------------------------
// true fp32
// ---------------------------------------------------------------------------------------
#define F32_BM 64
#define F32_BN 64
#define F32_BK 16
#define F32_SUM_TILES 8

__global__ __launch_bounds__(256) void gemm_f32_kernel(const float* __restrict__ A,
                                                       const float* __restrict__ W,
                                                       const float* __restrict__ bias,
                                                       float* __restrict__ C, int M, int N, int K,
                                                       int lda, int ldc) {
  __shared__ float As[F32_BK][F32_BM + 4];
  __shared__ float Ws[F32_BK][F32_BN + 4];
  const int tid = threadIdx.x;
  const int tx = tid % 16, ty = tid / 16;
  const int m0 = blockIdx.y * F32_BM, n0 = blockIdx.x * F32_BN;
  // Sums in two levels: `acc` runs over F32_SUM_TILES tiles of K (128 values), then goes into
  // `tot`.  A single running sum over K = 8192 loses about sqrt(K) roundings; this way it is
  // sqrt(128) + sqrt(K / 128), a quarter of that, for one more addition per 128 products.
  float acc[4][4], tot[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = tot[i][j] = 0.f;

  int tiles_in_acc = 0;
  for (int k0 = 0; k0 < K; k0 += F32_BK) {
    if (tiles_in_acc == F32_SUM_TILES) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          tot[i][j] += acc[i][j];
          acc[i][j] = 0.f;
        }
      tiles_in_acc = 0;
    }
    ++tiles_in_acc;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int idx = tid + e * 256;         // 0..1023
      const int r = idx / F32_BK, kk = idx % F32_BK;
      const int gm = m0 + r, gn = n0 + r, gk = k0 + kk;
      As[kk][r] = (gm < M && gk < K) ? A[(size_t)gm * lda + gk] : 0.f;
      Ws[kk][r] = (gn < N && gk < K) ? W[(size_t)gn * K + gk] : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < F32_BK; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = Ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int gm = m0 + ty * 4 + i;
    if (gm >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int gn = n0 + tx * 4 + j;
      if (gn < N) C[(size_t)gm * ldc + gn] = (tot[i][j] + acc[i][j]) + (bias ? bias[gn] : 0.f);
    }
  }
}

extern "C" int kappai_gemm_f32(const float* A, const float* W, const float* bias, float* C, int M,
                               int N, int K, int lda, int ldc, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  dim3 grid((N + F32_BN - 1) / F32_BN, (M + F32_BM - 1) / F32_BM);
  hipLaunchKernelGGL(gemm_f32_kernel, grid, dim3(256), 0, stream, A, W, bias, C, M, N, K, lda,
                     ldc);
  KAPPAI_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------------
// bf16 on the matrix cores
// ---------------------------------------------------------------------------------------
__device__ __forceinline__ u32x4_t load16(const bf16_t* p) {
  return *reinterpret_cast<const u32x4_t*>(p);
}
__device__ __forceinline__ bf16x8_t as_bf16x8(u32x4_t v) {
  return __builtin_bit_cast(bf16x8_t, v);
}
__device__ __forceinline__ void store_out(float* p, float v) { *p = v; }
__device__ __forceinline__ void store_out(bf16_t* p, float v) { *p = f32_to_bf16(v); }

// silu(g) = g / (1 + e^-g) for the epilogues that store bfloat16: the hardware's 2^x and reciprocal
// (each good to about an ulp of float, far below a bfloat16's rounding) instead of expf and a
// division, which were 9 of the 132 us of gate/up at 2048 rows.  e^-g overflows to infinity for
// g < -88: the reciprocal is then 0 and the result -0, as it should be.
__device__ __forceinline__ float silu_f(float g) {
  return g * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * g));
}

// Block = WAVES_M x WAVES_N waves, each owning (WM*32) x (WN*32) of the result as WM*WN
// accumulator tiles of 32x32: per 16 of K a wave reads WM+WN fragments from LDS for WM*WN
// matrix instructions, so large wave tiles keep LDS traffic below what the matrix cores
// consume.  Tiles of A (BM x BK) and W (BN x BK) go global -> registers -> LDS,
// double-buffered: the loads of tile k+1 are in flight while tile k is multiplied, one
// barrier a tile.
// Blocks are renumbered so that the blocks that run on one XCD (every eighth) work on
// neighbouring tiles and share their L2.
//
// EPI 1 (SwiGLU): W holds gate and up rows interleaved in groups of 16 (16 gate rows, the 16 up
// rows of the same columns, ...); the kernel writes silu(gate) * up, N/2 columns wide
// (kappai: src/backend/cpu/quants.h:369-371, src/recipe/builders.c:344-370).
// Block number -> (row tile, column tile).  Consecutive block numbers go to the 8 XCDs in
// turn, each with an L2 of its own.  An XCD is given a band of column tiles (an eighth of W, so
// that W is fetched from memory once) and walks it in groups of up to 8 x 8 tiles, row tiles
// fastest: the blocks that run on it at one time then share both their rows of A and their
// rows of W in its L2.
__device__ __forceinline__ int2 xcd_tile(int b, int tiles_m, int tiles_n) {
  constexpr int XCDS = 8, GROUP = 8;
  if (tiles_n % XCDS != 0) return make_int2(b / tiles_n, b % tiles_n);
  const int band = tiles_n / XCDS;             // column tiles of one XCD
  const int xcd = b % XCDS;
  int j = b / XCDS;                            // position in the XCD's own order
  const int per_group = GROUP * band;
  const int groups = (tiles_m + GROUP - 1) / GROUP;
  const int g = min(j / per_group, groups - 1);
  j -= g * per_group;
  const int gm = min(GROUP, tiles_m - g * GROUP);
  return make_int2(g * GROUP + j % gm, xcd * band + j / gm);
}

template <typename TO, int EPI, int WAVES_M, int WAVES_N, int WM, int WN, int BK, int NBUF,
          int OCC>
__global__ __launch_bounds__(WAVES_M * WAVES_N * WAVE)
    __attribute__((amdgpu_waves_per_eu(OCC, OCC))) void gemm_bf16_tile_kernel(
        const bf16_t* __restrict__ A, const bf16_t* __restrict__ W,
        const float* __restrict__ bias, TO* __restrict__ C, int M, int N, int K, int lda, int ldc,
        int tiles_n, int w_frag) {
  constexpr int BM = WAVES_M * WM * 32, BN = WAVES_N * WN * 32;
  constexpr int LDS_STRIDE = BK + 8;   // in bf16: rows stay 16-byte aligned, banks are spread
  constexpr int THREADS = WAVES_M * WAVES_N * WAVE;
  constexpr int CPR = BK / 8;                              // 16-byte chunks a row
  constexpr int A_CHUNKS = BM * CPR / THREADS;             // chunks a thread stages
  constexpr int W_CHUNKS = BN * CPR / THREADS;
  extern __shared__ __attribute__((aligned(16))) bf16_t lds[];
  // LDS: the A tiles of the NBUF buffers, then their W tiles
  constexpr int A_TILE = BM * LDS_STRIDE, W_TILE = BN * LDS_STRIDE;
  const int tid = threadIdx.x;
  const int lane = tid % WAVE, wave = tid / WAVE;
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  // block -> tile, XCD-aware
  const int2 tile = xcd_tile(blockIdx.x, gridDim.x / tiles_n, tiles_n);
  const int m0 = tile.x * BM, n0 = tile.y * BN;
  // gridDim.y > 1 splits K over blocks: block y writes its partial sums to C + y * M * ldc
  const int kblk = ((K + BK * (int)gridDim.y - 1) / (BK * (int)gridDim.y)) * BK;
  const int kbeg = blockIdx.y * kblk, kend = min(K, kbeg + kblk);
  C += (size_t)blockIdx.y * M * ldc;

  f32x16_t acc[WM][WN];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  // Staging: a thread copies 16-byte chunks; consecutive lanes take consecutive chunks of a
  // row, so that a row's bytes are asked for by neighbouring lanes and coalesce.
  const u32x4_t zero = {0u, 0u, 0u, 0u};
  u32x4_t ra[A_CHUNKS], rw[W_CHUNKS];
  auto chunk_row = [&](int idx) { return idx / CPR; };
  auto chunk_col = [&](int idx) { return (idx % CPR) * 8; };
  auto fetch = [&](int k0) {
#pragma unroll
    for (int c = 0; c < A_CHUNKS; ++c) {
      const int idx = tid + c * THREADS;
      const int r = chunk_row(idx), gk = k0 + chunk_col(idx);
      ra[c] = (m0 + r < M && gk < kend) ? load16(A + (size_t)(m0 + r) * lda + gk) : zero;
    }
#pragma unroll
    for (int c = 0; c < W_CHUNKS; ++c) {
      const int idx = tid + c * THREADS;
      const int r = chunk_row(idx), gk = k0 + chunk_col(idx);
      // (w_frag: W in fragment order, see gemm_bf16_skinny_kernel: the chunk of row n0 + r at gk)
      const size_t wr = (size_t)(n0 + r);
      const bf16_t* wp = w_frag ? W + (wr / 16) * 16 * K + (size_t)(gk / 32) * 512 +
                                      (((gk % 32) / 8) * 16 + wr % 16) * 8
                                : W + wr * K + gk;
      rw[c] = (n0 + r < N && gk < kend) ? load16(wp) : zero;
    }
  };
  auto stage = [&](int buf) {
#pragma unroll
    for (int c = 0; c < A_CHUNKS; ++c) {
      const int idx = tid + c * THREADS;
      *reinterpret_cast<u32x4_t*>(lds + buf * A_TILE + chunk_row(idx) * LDS_STRIDE +
                                  chunk_col(idx)) = ra[c];
    }
#pragma unroll
    for (int c = 0; c < W_CHUNKS; ++c) {
      const int idx = tid + c * THREADS;
      *reinterpret_cast<u32x4_t*>(lds + NBUF * A_TILE + buf * W_TILE +
                                  chunk_row(idx) * LDS_STRIDE + chunk_col(idx)) = rw[c];
    }
  };
  // While tile k is multiplied out of LDS, the loads of tile k+1 are in flight into registers;
  // after the products they are written to LDS: into the other buffer (NBUF 2, one barrier a
  // tile) or, after a barrier, into the same one (NBUF 1: half the LDS, so that two blocks fit
  // a CU even with long tiles, whose products give the loads more time to arrive).
  fetch(kbeg);
  stage(0);
  __syncthreads();
  int buf = 0;
  for (int k0 = kbeg; k0 < kend; k0 += BK) {
    const bool more = k0 + BK < kend;
    if (more) fetch(k0 + BK);
    const bf16_t* as =
        lds + buf * A_TILE + (wm * WM * 32 + lane % 32) * LDS_STRIDE + (lane / 32) * 8;
    const bf16_t* ws = lds + NBUF * A_TILE + buf * W_TILE +
                       (wn * WN * 32 + lane % 32) * LDS_STRIDE + (lane / 32) * 8;
    bf16x8_t a[2][WM], w[2][WN];
    auto frags = [&](int fb, int ks) {
#pragma unroll
      for (int i = 0; i < WM; ++i)
        a[fb][i] = as_bf16x8(*reinterpret_cast<const u32x4_t*>(as + i * 32 * LDS_STRIDE + ks));
#pragma unroll
      for (int j = 0; j < WN; ++j)
        w[fb][j] = as_bf16x8(*reinterpret_cast<const u32x4_t*>(ws + j * 32 * LDS_STRIDE + ks));
    };
    frags(0, 0);
#pragma unroll
    for (int s2 = 0; s2 < BK / 16; ++s2) {
      if (s2 + 1 < BK / 16) frags((s2 + 1) & 1, (s2 + 1) * 16);
#pragma unroll
      for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int j = 0; j < WN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[s2 & 1][i], w[s2 & 1][j],
                                                              acc[i][j], 0, 0, 0);
    }
    if (NBUF == 1) {
      __syncthreads();
      if (more) stage(0);
    } else {
      if (more) stage(buf ^ 1);
      buf ^= 1;
    }
    __syncthreads();
  }
  // D[m][n] of a 32x32 tile: lane holds column lane%32, rows 8*(v/4) + 4*(lane/32) + v%4
  if (EPI == 1) {
    // a 32-column tile is 16 gate columns and their 16 up columns: lane c < 16 holds gate,
    // lane c + 16 the matching up
#pragma unroll
    for (int i = 0; i < WM; ++i)
#pragma unroll
      for (int j = 0; j < WN; ++j) {
        const int c = lane % 32;
        const int gcol = n0 + (wn * WN + j) * 32;        // first interleaved column of the tile
        const int on = gcol / 2 + c;                     // output column for c < 16
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const float other = __shfl_xor(acc[i][j][v], 16, WAVE);
          const int gm = m0 + (wm * WM + i) * 32 + 8 * (v / 4) + 4 * (lane / 32) + v % 4;
          if (c < 16 && gm < M && gcol + c < N)
            store_out(C + (size_t)gm * ldc + on, silu_f(acc[i][j][v]) * other);
        }
      }
    return;
  }
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j) {
      const int gn = n0 + (wn * WN + j) * 32 + lane % 32;
      if (gn >= N) continue;
      const float bv = (bias && blockIdx.y == 0) ? bias[gn] : 0.f;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int gm = m0 + (wm * WM + i) * 32 + 8 * (v / 4) + 4 * (lane / 32) + v % 4;
        if (gm < M) store_out(C + (size_t)gm * ldc + gn, acc[i][j][v] + bv);
      }
    }
}

template <typename TO, int EPI, int WAVES_M, int WAVES_N, int WM, int WN, int BK, int NBUF,
          int OCC>
static void launch_tile_cfg(const bf16_t* A, const bf16_t* W, const float* bias, TO* C, int M,
                            int n_rows_w, int K, int lda, int ldc, int ksplit,
                            hipStream_t stream, int w_frag = 0) {
  constexpr int BM = WAVES_M * WM * 32, BN = WAVES_N * WN * 32;
  constexpr size_t lds_bytes = (size_t)NBUF * (BM + BN) * (BK + 8) * sizeof(bf16_t);
  auto kern = gemm_bf16_tile_kernel<TO, EPI, WAVES_M, WAVES_N, WM, WN, BK, NBUF, OCC>;
  static bool attr_set = false;       // more than 64 KB of LDS has to be asked for once
  if (!attr_set) {
    (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)lds_bytes);
    attr_set = true;
  }
  const int tn = (n_rows_w + BN - 1) / BN, tm = (M + BM - 1) / BM;
  hipLaunchKernelGGL(kern, dim3(tm * tn, ksplit), dim3(WAVES_M * WAVES_N * WAVE), lds_bytes,
                     stream, A, W, bias, C, M, n_rows_w, K, lda, ldc, tn, w_frag);
}

// ---------------------------------------------------------------------------------------
// 256 x 256 blocks for large products (prefill)
// ---------------------------------------------------------------------------------------
// Four waves, one on each SIMD, each owning 128 x 128 of the result as 4 x 4 accumulator tiles
// (256 accumulator registers): per 16 of K a wave reads 8 fragments from LDS for 16 matrix
// instructions.  Tiles of 64 of K (128-byte rows, whole cache lines) go from global memory
// straight into LDS (global_load_lds), two buffers; the 16-byte chunks of a row are permuted
// by (chunk ^ (row / 2) % 8) on the way in, so that the 16 lanes of a fragment read (16 rows,
// one chunk each) fall on 16 different 16-byte bank groups without padding.  The order of LDS reads, loads and matrix instructions is written out slot by slot
// and fenced, one wave has to hide every latency by itself: while the products of one 16 of K
// run, the fragments of the next are read; the loads of tile k+2 are issued as soon as the
// barrier of tile k has shown that everybody is done with its buffer.
//
// The matrix instruction takes the W fragment as its first operand: a lane then holds one row
// of C and 4 consecutive columns per register group, which the epilogue packs, transposes
// through LDS and stores as whole 16-byte chunks of rows (the SwiGLU pairs gate and up in one
// lane: registers v and v + 8).
//
// Host side guarantees: K / gridDim.y is a multiple of 128, rows of W a multiple of 8 (32 with
// SwiGLU), C and its row stride 16-byte aligned, M * lda and N * K below 2^31 elements.
#define KAPPAI_GPTR(p) ((const __attribute__((address_space(1))) void*)(p))
#define KAPPAI_LPTR(p) ((__attribute__((address_space(3))) void*)(p))
#define SCHED_FENCE() __builtin_amdgcn_sched_barrier(0)

template <int N> struct IntC { static constexpr int value = N; };

template <typename TO, int EPI, int WT, bool DEEP = false, int WN_ = 0>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4 / WT, 4 / WT)))
void gemm_bf16_block256_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ W,
                               const float* __restrict__ bias, TO* __restrict__ C, int M, int N,
                               int K, int lda, int ldc, int tiles_n, int w_frag) {
  // WTM x WTN accumulator tiles of 32 x 32 a wave (WTN = WT unless WN_ is given): 4 x 4 ->
  // 256 x 256 blocks, 2 x 2 -> 128 x 128, 4 x 3 -> 256 rows x 192 columns (for a product whose
  // 256 x 256 blocks would leave a quarter of the chip without one)
  constexpr int WTM = WT, WTN = WN_ ? WN_ : WT;
  static_assert(!DEEP || (WTM == 2 && WTN == 2), "four LDS buffers: the 128 x 128 form only");
  static_assert(WTN <= WTM && 2 * WTN >= WTM, "the load slots are laid out for the rows' side");
  constexpr int BM = WTM * 64, BN = WTN * 64, BK = 64;
  constexpr int WROWS_M = WTM * 32, WROWS_N = WTN * 32;        // rows, columns of a wave's tile
  constexpr int NPROD = WTM * WTN, NREAD = WTM + WTN;          // per 16 of K
  // load instructions a wave and tile: the waves that bring A issue NLOAD, those that bring W
  // the first NLOAD_W of the same slots
  constexpr int NLOAD = 4 * WTM, NLOAD_W = 4 * WTN, HALF = NLOAD / 2;
  constexpr int A_TILE = BM * BK, BUF = (BM + BN) * BK;        // in bf16
  extern __shared__ __attribute__((aligned(1024))) bf16_t lds[];
  const int tid = threadIdx.x, lane = tid % WAVE;
  const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
  const int wm = wave / 2, wn = wave % 2;
  const int2 tile = xcd_tile(blockIdx.x, gridDim.x / tiles_n, tiles_n);
  const int m0 = tile.x * BM, n0 = tile.y * BN;
  const int kblk = K / (int)gridDim.y;
  const int nk = kblk / BK;
  C += (size_t)blockIdx.y * M * ldc;

  f32x16_t acc[WTM][WTN];
#pragma unroll
  for (int i = 0; i < WTM; ++i)
#pragma unroll
    for (int j = 0; j < WTN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  // One load instruction = 8 rows x 128 bytes: lane -> (row lane/8, LDS chunk lane%8), which
  // receives the row's chunk (lane%8) ^ ((row/2)%8).  Waves 0, 1 bring the A tile, waves 2, 3 the W
  // tile, NLOAD instructions each; rows past the end of the matrix repeat its last row (their
  // products are never stored).
  //
  // w_frag: W lies in fragment order ([rows / 16][K / 32] pieces of 16 rows x 32 of K, 1 KB each,
  // the lane's 16 bytes at lane = (k % 32) / 8 * 16 + row % 16; see gemm_bf16_skinny_kernel).  A
  // load instruction of the W waves then brings one piece, instruction i the piece (16 rows
  // number i / 2 of the wave's rows, 32 of K number i % 2 of the tile), which lands in LDS as it
  // lies in memory: a fragment read (16 lanes = 16 rows of one group of 8 of K = 256 contiguous
  // bytes) is free of bank conflicts without a permutation.
  const bool brings_a = wave < 2;
  const bool frag_w = !brings_a && w_frag;
  const char* gk = reinterpret_cast<const char*>(brings_a ? A : W) +
                   (size_t)blockIdx.y * kblk * (frag_w ? 16 : 1) * sizeof(bf16_t);
  const int ld = brings_a ? lda : K;
  const int last_row = (brings_a ? M : N) - 1;
  const int row0 = brings_a ? m0 + wave * WROWS_M : n0 + (wave - 2) * WROWS_N;
  const int lds_row0 = brings_a ? wave * WROWS_M : BM + (wave - 2) * WROWS_N;   // in the buffer
  const int my_loads = brings_a ? NLOAD : NLOAD_W;
  const int lrow = lane / 8;
  uint32_t roff[NLOAD];
#pragma unroll
  for (int i = 0; i < NLOAD; ++i) {
    const int lchunk = (lane % 8) ^ (((i * 8 + lrow) >> 1) & 7);
    roff[i] = (uint32_t)(min(row0 + i * 8 + lrow, last_row) * ld + lchunk * 8) *
              (uint32_t)sizeof(bf16_t);
    if (frag_w)
      roff[i] = (uint32_t)(min(row0 / 16 + i / 2, last_row / 16) * 16 * K + (i % 2) * 512 +
                           lane * 8) * (uint32_t)sizeof(bf16_t);
  }
  // bytes from one tile of 64 of K to the next: a row's 128 bytes, or two pieces
  const uint32_t kstep = frag_w ? 2048u : (uint32_t)(BK * sizeof(bf16_t));
  // the address of a load is a wave-uniform 64-bit base (the tile's first column) plus the
  // lane's 32-bit row offset; pinning the base into scalar registers keeps the compiler from
  // folding the two into sixteen 64-bit per-lane pointers
  auto tile_base = [&](int kt) {
    const uint64_t p = reinterpret_cast<uint64_t>(gk) + (uint64_t)kt * kstep;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)p);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(p >> 32));
    return reinterpret_cast<const char*>(((uint64_t)hi << 32) | lo);
  };
  auto load_one = [&](int buf, const char* base, int i) {
    if (NLOAD_W < NLOAD && i >= my_loads) return;       // (uniform over the wave)
    __builtin_amdgcn_global_load_lds(KAPPAI_GPTR(base + roff[i]),
                                     KAPPAI_LPTR(lds + buf * BUF + (lds_row0 + i * 8) * BK), 16,
                                     0, 0);
  };
  // fragments of the 16 of K number s: chunks 2s and 2s+1; lane -> (row lane%32, chunk 2s+lane/32)
  const int r_in = lane % 32, hh = lane / 32;
  int aoff[4], woff[4];
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    aoff[s] = (wm * WROWS_M + r_in) * BK + (((s * 2 + hh) ^ ((r_in >> 1) & 7)) * 8);
    woff[s] = A_TILE + (wn * WROWS_N + r_in) * BK + (((s * 2 + hh) ^ ((r_in >> 1) & 7)) * 8);
    if (w_frag)     // piece (r_in / 16, s / 2) of the wave's rows, group (s % 2) * 2 + hh of its K
      woff[s] = A_TILE + wn * WROWS_N * BK + ((r_in / 16) * 2 + s / 2) * 512 +
                (((s % 2) * 2 + hh) * 16 + r_in % 16) * 8;
  }
  bf16x8_t fa[2][WTM], fw[2][WTN];
  // in the order the products ask for them: w0 a0, the other w, the other a
  auto read_one = [&](int fb, int buf, int s, int idx) {
    const bool is_w = idx == 0 || (idx >= 2 && idx <= WTN);
    const int n = idx <= 1 ? 0 : idx <= WTN ? idx - 1 : idx - WTN;
    if (is_w)
      fw[fb][n] = as_bf16x8(
          *reinterpret_cast<const u32x4_t*>(lds + buf * BUF + woff[s] + n * 32 * BK));
    else
      fa[fb][n] = as_bf16x8(
          *reinterpret_cast<const u32x4_t*>(lds + buf * BUF + aoff[s] + n * 32 * BK));
  };
  auto product = [&](int fb, int t) {
    const int i = t / WTN, j = t % WTN;
    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fw[fb][j], fa[fb][i], acc[i][j], 0, 0, 0);
  };
  // One tile of K out of buffer U.  next: there is a tile kt+1 (its second half is loaded
  // here, its first fragments are read at the end); next2: there is a tile kt+2 (its first
  // half is loaded into this tile's buffer once the barrier has passed).  Both are uniform.
  auto tile_step = [&](auto u_c, int kt, bool next, bool next2) {
    constexpr int U = decltype(u_c)::value;
    const char* base1 = tile_base(kt + 1);
    const char* base2 = tile_base(kt + 2);
#pragma unroll
    for (int s = 0; s < 3; ++s) {
#pragma unroll
      for (int t = 0; t < NPROD; ++t) {
        if (t < NREAD) read_one((s + 1) & 1, U, s + 1, t);
        if (s == 0 && t >= NPROD - HALF && next) load_one(U ^ 1, base1, HALF + t - (NPROD - HALF));
        product(s & 1, t);
        SCHED_FENCE();
      }
    }
    // the last 16 of K: a few products first, so that the matrix cores have work while the
    // wave waits at the barrier
    constexpr int PRE = WTM == 4 ? 4 : 1;
    constexpr int REST = NPROD - PRE;
    constexpr int SPREAD = REST < 8 ? REST : 8;         // slots that also read and load
    constexpr int READS_PER = (NREAD + SPREAD - 1) / SPREAD;
    constexpr int LOADS_PER = (HALF + SPREAD - 1) / SPREAD;
#pragma unroll
    for (int t = 0; t < PRE; ++t) {
      product(1, t);
      SCHED_FENCE();
    }
    if (next) {
      __builtin_amdgcn_s_waitcnt(0x0F70);       // vmcnt(0): tile kt+1 has landed
      __builtin_amdgcn_s_barrier();
    }
    SCHED_FENCE();
#pragma unroll
    for (int t = PRE; t < NPROD; ++t) {
      const int k = t - PRE;
#pragma unroll
      for (int q = 0; q < READS_PER; ++q)
        if (k * READS_PER + q < NREAD && next) read_one(0, U ^ 1, 0, k * READS_PER + q);
#pragma unroll
      for (int q = 0; q < LOADS_PER; ++q)
        if (k * LOADS_PER + q < HALF && next2) load_one(U, base2, k * LOADS_PER + q);
      product(1, t);
      SCHED_FENCE();
    }
  };

  if constexpr (DEEP) {
    // Four LDS buffers, the block alone on its CU (128 KB): a 128 x 128 block's products of one
    // tile take about 0.2 us, far less than a tile's way from memory, so with two buffers a
    // block that has no neighbour on its CU waits for every tile (0.62 us each).  Here the loads
    // of tile kt+3 are issued while tile kt is multiplied: three tiles are under way.
    // Buffer of tile kt: kt % 4.  After the barrier of step kt-1 nobody reads tile kt-1's
    // buffer any more, which is where tile kt+3 goes.
    auto load_deep = [&](int kt, const char* base, int i) {
      __builtin_amdgcn_global_load_lds(
          KAPPAI_GPTR(base + roff[i]),
          KAPPAI_LPTR(lds + (kt & 3) * BUF + (lds_row0 + i * 8) * BK), 16, 0, 0);
    };
    auto read_deep = [&](int fb, const bf16_t* buf, int s, int idx) {
      const bool is_w = idx == 0 || (idx >= 2 && idx <= WTN);
      const int n = idx <= 1 ? 0 : idx <= WTN ? idx - 1 : idx - WTN;
      if (is_w)
        fw[fb][n] = as_bf16x8(*reinterpret_cast<const u32x4_t*>(buf + woff[s] + n * 32 * BK));
      else
        fa[fb][n] = as_bf16x8(*reinterpret_cast<const u32x4_t*>(buf + aoff[s] + n * 32 * BK));
    };
    const int pre = min(nk, 3);
    for (int p = 0; p < pre; ++p) {
      const char* base = tile_base(p);
#pragma unroll
      for (int i = 0; i < NLOAD; ++i) load_deep(p, base, i);
    }
    // tile 0 has landed when only the loads of the tiles after it are outstanding
    if (pre == 3)
      __builtin_amdgcn_s_waitcnt(0x4F70);         // vmcnt(16)
    else if (pre == 2)
      __builtin_amdgcn_s_waitcnt(0x0F78);         // vmcnt(8)
    else
      __builtin_amdgcn_s_waitcnt(0x0F70);         // vmcnt(0)
    __builtin_amdgcn_s_barrier();
    SCHED_FENCE();
#pragma unroll
    for (int t = 0; t < NREAD; ++t) read_deep(0, lds, 0, t);
    static_assert(NLOAD == 2 * NPROD, "one load a slot over the first two 16s of K");
    for (int kt = 0; kt < nk; ++kt) {
      const bf16_t* cur = lds + (kt & 3) * BUF;
      const bf16_t* nxt = lds + ((kt + 1) & 3) * BUF;
      const bool has1 = kt + 1 < nk, has2 = kt + 2 < nk, has3 = kt + 3 < nk;
      const char* base3 = tile_base(kt + 3);
#pragma unroll
      for (int s = 0; s < 3; ++s) {
#pragma unroll
        for (int t = 0; t < NPROD; ++t) {
          if (t < NREAD) read_deep((s + 1) & 1, cur, s + 1, t);
          if (s < 2 && has3) load_deep(kt + 3, base3, s * NPROD + t);
          product(s & 1, t);
          SCHED_FENCE();
        }
      }
      product(1, 0);
      SCHED_FENCE();
      if (has1) {
        // tile kt+1 has landed when only the loads of tiles kt+2 and kt+3 are outstanding
        if (has3)
          __builtin_amdgcn_s_waitcnt(0x4F70);     // vmcnt(16)
        else if (has2)
          __builtin_amdgcn_s_waitcnt(0x0F78);     // vmcnt(8)
        else
          __builtin_amdgcn_s_waitcnt(0x0F70);     // vmcnt(0)
        __builtin_amdgcn_s_barrier();
      }
      SCHED_FENCE();
#pragma unroll
      for (int t = 1; t < NPROD; ++t) {
        if (has1) {
          if (t == 1) {
            read_deep(0, nxt, 0, 0);
            read_deep(0, nxt, 0, 1);
          } else if (t == 2) {
            read_deep(0, nxt, 0, 2);
            read_deep(0, nxt, 0, 3);
          }
        }
        product(1, t);
        SCHED_FENCE();
      }
    }
  } else {
#pragma unroll
  for (int i = 0; i < NLOAD; ++i) load_one(0, tile_base(0), i);
#pragma unroll
  for (int i = 0; i < HALF; ++i) load_one(1, tile_base(1), i);
  __builtin_amdgcn_s_waitcnt(0x0F70 | HALF);    // vmcnt(HALF): tile 0 has landed
  __builtin_amdgcn_s_barrier();
  SCHED_FENCE();
#pragma unroll
  for (int t = 0; t < NREAD; ++t) read_one(0, 0, 0, t);

  // nk is even: the loop body is straight-line code for the accumulators (a conditional
  // second tile would merge two versions of all 256 of them)
  for (int kt = 0; kt < nk; kt += 2) {
    const bool more = kt + 2 < nk;
    tile_step(IntC<0>{}, kt, true, more);
    tile_step(IntC<1>{}, kt + 1, more, more);
  }
  }

  // Epilogue: a wave turns 32 rows of its tile at a time through its own piece of LDS.
  // acc[i][j][4g + e] is C[row (wm*WT+i)*32 + lane%32][column (wn*WT+j)*32 + 8g + 4*(lane/32) + e].
  __syncthreads();                               // everybody is done with the last tile
  constexpr int OUT_COLS = EPI == 1 ? WROWS_N / 2 : WROWS_N;   // columns a wave writes
  constexpr int ROW_BYTES = OUT_COLS * (int)sizeof(TO) + 16;
  char* mine = reinterpret_cast<char*>(lds) + wave * 32 * ROW_BYTES;
  const int out_n = EPI == 1 ? N / 2 : N;
  const int col0 = EPI == 1 ? (n0 + wn * WROWS_N) / 2 : n0 + wn * WROWS_N;
#pragma unroll
  for (int i = 0; i < WTM; ++i) {
    char* wrow = mine + r_in * ROW_BYTES;
#pragma unroll
    for (int j = 0; j < WTN; ++j) {
#pragma unroll
      for (int g = 0; g < (EPI == 1 ? 2 : 4); ++g) {
        float v4[4];
        int c;                                   // first of the 4 columns, within the wave's
        if (EPI == 1) {
          c = j * 16 + 8 * g + 4 * hh;
#pragma unroll
          for (int e = 0; e < 4; ++e) v4[e] = silu_f(acc[i][j][4 * g + e]) * acc[i][j][4 * g + 8 + e];
        } else {
          c = j * 32 + 8 * g + 4 * hh;
#pragma unroll
          for (int e = 0; e < 4; ++e) v4[e] = acc[i][j][4 * g + e];
          if (bias && blockIdx.y == 0) {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (col0 + c + e < out_n) v4[e] += bias[col0 + c + e];
          }
        }
        if (sizeof(TO) == 2) {
          uint2 pk;
          pk.x = pack_bf16x2(v4[0], v4[1]);
          pk.y = pack_bf16x2(v4[2], v4[3]);
          *reinterpret_cast<uint2*>(wrow + c * 2) = pk;
        } else {
          *reinterpret_cast<float4*>(wrow + c * 4) = make_float4(v4[0], v4[1], v4[2], v4[3]);
        }
      }
    }
    // rows back out, 16 bytes a lane
    constexpr int CHUNKS = OUT_COLS * (int)sizeof(TO) / 16;   // per row
    constexpr int ROWS_PER = WAVE / CHUNKS;                   // (lanes left over sit out)
    constexpr int PER = 16 / (int)sizeof(TO);                 // columns a chunk
    constexpr bool EVEN = WAVE % CHUNKS == 0 && 32 % ROWS_PER == 0;
#pragma unroll
    for (int it = 0; it < (32 + ROWS_PER - 1) / ROWS_PER; ++it) {
      const int rr = it * ROWS_PER + lane / CHUNKS, ch = lane % CHUNKS;
      if (!EVEN && (lane >= ROWS_PER * CHUNKS || rr >= 32)) continue;
      const u32x4_t v = *reinterpret_cast<const u32x4_t*>(mine + rr * ROW_BYTES + ch * 16);
      const int gm = m0 + (wm * WTM + i) * 32 + rr, gn = col0 + ch * PER;
      if (gm < M && gn < out_n) *reinterpret_cast<u32x4_t*>(C + (size_t)gm * ldc + gn) = v;
    }
  }
}

template <typename TO, int EPI>
static bool block256_fits(const bf16_t* A, const bf16_t* W, TO* C, int M, int n_rows_w, int K,
                          int lda, int ldc, int ksplit) {
  const long long limit = 1ll << 31;
  return K % (128 * ksplit) == 0 && n_rows_w % (EPI == 1 ? 32 : 8) == 0 &&
         ((uintptr_t)C % 16) == 0 && ((size_t)ldc * sizeof(TO)) % 16 == 0 &&
         (long long)M * lda < limit && (long long)n_rows_w * K < limit;
}

template <typename TO, int EPI, int WT, bool DEEP = false, int WN_ = 0>
static void launch_block256(const bf16_t* A, const bf16_t* W, const float* bias, TO* C, int M,
                            int n_rows_w, int K, int lda, int ldc, int ksplit,
                            hipStream_t stream, int w_frag = 0) {
  constexpr int B = WT * 64, BN = (WN_ ? WN_ : WT) * 64;       // block: B rows x BN columns
  constexpr size_t lds_bytes = (DEEP ? 4 : 2) * (B + BN) * 64 * sizeof(bf16_t);
  auto kern = gemm_bf16_block256_kernel<TO, EPI, WT, DEEP, WN_>;
  static bool attr_set = false;
  if (!attr_set) {
    (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)lds_bytes);
    attr_set = true;
  }
  const int tn = (n_rows_w + BN - 1) / BN, tm = (M + B - 1) / B;
  hipLaunchKernelGGL(kern, dim3(tm * tn, ksplit), dim3(256), lds_bytes, stream, A, W, bias, C, M,
                     n_rows_w, K, lda, ldc, tn, w_frag);
}

// The 256 x 256 form (one block a CU, 40-55 us per round of up to 256 blocks at K = 2048) against
// the 128 x 128 form (two blocks a CU): from 140 blocks on when one round does it, and with more
// rounds when the last one is not mostly idle (idle CU-rounds under 30 % of the blocks); from a
// sweep of the layer shapes at 1024 to 8192 rows.
static bool use_256_form(long blocks256) {
  if (blocks256 <= 256) return blocks256 >= 140;
  const long rem = blocks256 % 256;
  return rem == 0 || (256 - rem) * 10 < 3 * blocks256;
}

// shape: 0 = chosen by size, 1 = 128x128 blocks of two waves, 2 = 256x128 blocks (tiles of 32
// of K, two LDS buffers), 3 = 256x128 blocks (tiles of 64 of K, one LDS buffer), 4 = 256x256
// blocks of the same kernel (tiles of 64 of K), 5 = the 256x256 kernel with one wave a SIMD, 6 = its
// 128x128 form (when the sizes fit them, else 3), 8 = the 128x128 form with four LDS buffers, one
// block a CU, 9 = the one-wave-a-SIMD kernel with blocks of 256 rows x 192 columns
template <typename TO, int EPI>
static void launch_tile(const bf16_t* A, const bf16_t* W, const float* bias, TO* C, int M,
                        int n_rows_w, int K, int lda, int ldc, int ksplit, int shape,
                        hipStream_t stream, const bf16_t* Wf = nullptr) {
  const bool fits = EPI != 2 && block256_fits<TO, EPI>(A, W, C, M, n_rows_w, K, lda, ldc, ksplit);
  if (shape == 0) {
    const int big = ((M + 255) / 256) * ((n_rows_w + 127) / 128) * ksplit;
    const int blocks256 = ((M + 255) / 256) * ((n_rows_w + 255) / 256) * ksplit;
    // the one-wave-a-SIMD kernel when its 256 x 256 blocks fill most of the chip, its
    // 128 x 128 form (two blocks a CU) below that
    // 128 x 128 blocks that would each have a CU to themselves anyway, and a long K: the form
    // with four LDS buffers (0.46 against 0.62-0.87 us per 64 of K; its start costs 2 us more)
    const long blocks128 = (long)((M + 127) / 128) * ((n_rows_w + 127) / 128) * ksplit;
    const bool deep = blocks128 <= 256 && K / ksplit >= 2048;
    // (up to 128 rows a block of 256 rows would be half empty)
    shape = !fits ? (big >= 128 ? 3 : 1) : (M > 128 && use_256_form(blocks256)) ? 5 : deep ? 8 : 6;
    if (shape == 5 && EPI == 0) {
      // blocks of 256 rows x 192 columns when they fill their rounds and come to fewer rounds'
      // worth of work than 256 x 256 (in_proj of 2048 rows: 192 blocks of 256 x 256 leave 64 CUs
      // idle, 256 blocks of 256 x 192 none: 49 against 55 us).  Only against the 256 x 256 form:
      // where the 128 x 128 form was chosen (rows or columns that fill their last tiles badly, K
      // split into ranges) the 192 form was measured slower (2063 x 2048 x 7168: 88 against 74 us).
      const long blocks192 = (long)((M + 255) / 256) * ((n_rows_w + 191) / 192) * ksplit;
      const long r256 = (blocks256 + 255) / 256, r192 = (blocks192 + 255) / 256;
      if (use_256_form(blocks192) && r192 * (192 + 16) < r256 * (256 + 16)) shape = 9;
    }
  }
  if ((shape == 5 || shape == 6 || shape == 8 || shape == 9) && !fits) shape = 3;
  if (shape == 9 && EPI != 0) shape = 5;
  // Wf: W in fragment order (W may then be null).  The one-wave-a-SIMD kernel reads it as fast as
  // rows or a little faster (gate/up of 2048 rows 119.5 against 122-124 us in turns on one box, the
  // other products equal: a tile's loads are pieces of 1 KB), the older tile kernel a little
  // slower (47 against 43 us), so that one takes the rows when there are any.
  const bool block_form = shape == 5 || shape == 6 || shape == 8 || shape == 9;
  const int w_frag = Wf != nullptr && (W == nullptr || block_form);
  if (w_frag) W = Wf;
  switch (shape) {
    case 5:
      if constexpr (EPI != 2)
        launch_block256<TO, EPI, 4>(A, W, bias, C, M, n_rows_w, K, lda, ldc, ksplit, stream, w_frag);
      break;
    case 6:
      if constexpr (EPI != 2)
        launch_block256<TO, EPI, 2>(A, W, bias, C, M, n_rows_w, K, lda, ldc, ksplit, stream, w_frag);
      break;
    case 8:
      if constexpr (EPI != 2)
        launch_block256<TO, EPI, 2, true>(A, W, bias, C, M, n_rows_w, K, lda, ldc, ksplit, stream, w_frag);
      break;
    case 9:
      if constexpr (EPI == 0)
        launch_block256<TO, EPI, 4, false, 3>(A, W, bias, C, M, n_rows_w, K, lda, ldc, ksplit,
                                              stream, w_frag);
      break;
    case 1:
      launch_tile_cfg<TO, EPI, 1, 2, 4, 2, 32, 2, 2>(A, W, bias, C, M, n_rows_w, K, lda, ldc, ksplit,
                                                  stream, w_frag);
      break;
    case 2:
      launch_tile_cfg<TO, EPI, 2, 2, 4, 2, 32, 2, 2>(A, W, bias, C, M, n_rows_w, K, lda, ldc, ksplit,
                                                  stream, w_frag);
      break;
    case 3:
      launch_tile_cfg<TO, EPI, 2, 2, 4, 2, 64, 1, 2>(A, W, bias, C, M, n_rows_w, K, lda, ldc, ksplit,
                                                  stream, w_frag);
      break;
    default:
      launch_tile_cfg<TO, EPI, 2, 2, 4, 4, 64, 2, 1>(A, W, bias, C, M, n_rows_w, K, lda, ldc, ksplit,
                                                  stream, w_frag);
      break;
  }
}

// M <= 16*MT (decode).  Bound by reading W once: a block owns 16 columns of the result and
// streams their 16 rows of W; its NW waves split K into contiguous ranges and meet in LDS.
// Every wave issues SK_UNROLL independent 16-byte loads of W per lane before it consumes
// them, so that enough bytes are in flight to keep HBM busy.  A fragment: lane holds row
// lane%16, k-group lane/16; W fragment: lane holds column lane%16, k-group lane/16; result:
// lane holds column lane%16, rows 4*(lane/16) + v.
#define SK_UNROLL 8

// EPI 1 (SwiGLU, see the tile kernel): a block owns 16 output columns = 16 gate rows and
// their 16 up rows of the interleaved W; N is the number of output columns.
// gridDim.y > 1 splits K over blocks as well: block (x, y) writes its partial sums to
// C + y * M * ldc (float), which the consumer adds up in a fixed order.
// EPI 2 (gated short convolution, one decoded row a request; kappai:
// src/backend/cpu/common.c:2393-2431): W is the conv layer's in_proj [3N, K]; a block owns 16
// channels and streams their B, C and x rows (N rows apart), then bx = B*x meets the request's
// state, the taps give s, the kernel writes C*s and shifts the state.
struct ConvStep {
  const float* taps;       // [N, L]
  const float* conv_bias;  // [N] or null
  float* state;            // [slots, N, L-1]
  const int* seg_pos0;     // [M]: position of the row (0: no history)
  const int* seg_slot;     // [M]
  int L;
};

// Two ways of saving the RMSNorm kernel between two products of a decode step (one row tile,
// at most 16 rows).  RMSNorm(x) W^T = (x * w) W^T / rms(x) row by row (kappai:
// src/backend/cpu/scalar/quants.c:1507-1512 for the norm), so the product can run on x * w and
// be scaled afterwards:
//   ResidOut (a product whose result is added to the residual stream, plain epilogue, float, K
//     not split over blocks): resid[m][n] += sum (+ bias) in place, in float; and when `rows` is
//     set the block also writes what the next product reads, rows[m][n] = bf16(resid[m][n] *
//     norm_w[n]) (row order, or the fragment order of add_rmsnorm when rows_frag), and
//     ss[blockIdx.x][m] = the sum of resid[m][n]^2 over its 8 columns (gemm_bf16_into_resid);
//   RowScale (the product that follows): its rows are such x * w, and every result is
//     multiplied by 1 / sqrt(sum_p ss[p][m] / K + eps) before bias and epilogue.
struct RowScale {
  const float* ss;   // [n_parts][16] (a row's value at [p][m]), or null: rows are used as they are
  int n_parts;
  float eps;
};
struct ResidOut {
  float* resid;          // [M, ldr], or null: the result goes to C
  int ldr;
  const float* norm_w;   // [N]; null: no rows for a next product
  bf16_t* rows;          // [M, N] or 16 rows in fragment order
  int rows_frag;
  float* ss;             // [gridDim.x][16]: a part holds one value a row, rows beyond M unwritten
};

template <typename TO, int MT, int NW, int EPI, int NT>
__global__ __launch_bounds__((NW < 16 ? NW + 1 : NW) * WAVE) void gemm_bf16_skinny_kernel(
    const bf16_t* __restrict__ A, const bf16_t* __restrict__ W, const float* __restrict__ bias,
    TO* __restrict__ C, int M, int N, int K, int lda, int ldc, ConvStep cs, RowScale rsc,
    int w_frag, int a_frag, int c_frag) {
  static_assert(NT == 1 || EPI == 0, "several column tiles a wave: plain products only");
  // c_frag (one row tile, the SwiGLU and conv epilogues): the result is written as 16 rows in
  // fragment order, which is how the product that follows likes to read it (see a_frag)
  auto out_at = [&](int gm, int gn_) {
    return c_frag ? ((size_t)(gn_ / 8) * 16 + gm) * 8 + gn_ % 8 : (size_t)gm * ldc + gn_;
  };
  // row groups of W a block streams: gate/up, the three conv gates, or NT column tiles
  constexpr int NG = EPI == 1 ? 2 : (EPI == 2 ? 3 : (EPI == 3 ? 2 : NT));
  __shared__ float red[NW][NG * MT][WAVE][4];
  const int tid = threadIdx.x;
  const int lane = tid % WAVE, wave = tid / WAVE;
  const int n0 = blockIdx.x * (EPI == 3 ? 8 : 16 * NT);
  const int col = lane % 16, kg = (lane / 16) * 8;
  // EPI 3: columns 0-7 and 8-15 are the same 8 channels (of two different gates)
  const int gn = n0 + (EPI == 3 ? col % 8 : col);
  const u32x4_t zero = {0u, 0u, 0u, 0u};
  f32x4_t acc[NG * MT];
#pragma unroll
  for (int t = 0; t < NG * MT; ++t) acc[t] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
  // plain: row gn (and 16 further for the next column tile).  SwiGLU: gate row 32*block + col, up
  // row 16 further.  Conv: rows gn, N + gn, 2N + gn.
  // EPI 3 (the conv step with 8 channels a block, twice as many blocks for narrow models): row
  // group 0 is the B gate's rows in columns 0-7 and the C gate's in columns 8-15, row group 1 the
  // x gate's rows in columns 0-7 (columns 8-15 stay zero).
  const size_t wr0 = EPI == 1 ? (size_t)blockIdx.x * 32 + col
                              : (EPI == 3 && col >= 8 ? (size_t)N + gn : (size_t)gn);
  const size_t group_rows = EPI == 2 ? (size_t)N : (EPI == 3 ? 2 * (size_t)N : 16);
  // W as it is stored ([rows, K]), or its copy in fragment order (w_frag): [rows / 16][K / 32]
  // pieces of 1 KB, each what one load instruction of a wave wants, lane by lane (lane =
  // (k % 32) / 8 * 16 + row % 16, 8 values a lane).  A wave's loads then touch every cache line
  // once instead of twice, and neighbouring lines: the products with 1-16 rows are bound by the
  // number of lines asked for as much as by bytes (gate/up at 8 rows: 14.7 against 18.2 us).
  // One step of 32 along K is 32 elements here and 512 there.
  const size_t wr1 = gn < N ? wr0 : 0;
  const int kmul = w_frag ? 16 : 1;
  const bf16_t* wrow = w_frag ? W + (wr1 / 16) * 16 * K + ((size_t)(kg / 8) * 16 + wr1 % 16) * 8
                              : W + wr1 * K + kg;
  auto group_ok = [&](int r) { return EPI == 3 ? (r == 0 || col < 8) : true; };
  const bf16_t* arow[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int gm = t * 16 + col;
    // a_frag (at most 16 rows): the rows lie in fragment order too, [K / 32][(k % 32) / 8][16 rows]
    // [8 values] (add_rmsnorm writes them so): a load then takes whole lines of neighbouring rows
    arow[t] = a_frag ? A + ((size_t)(kg / 8) * 16 + (gm < M ? gm : 0)) * 8
                     : A + (size_t)(gm < M ? gm : 0) * lda + kg;
  }
  __shared__ float row_ss[16];
  if (wave == NW) {
    // The block's extra wave (launched only with a RowScale) adds up the rows' sums of squares
    // while the others stream W: a lane takes parts lane, lane + 64, ... of all rows at once (a
    // part is 16 floats, one a row), four parts' loads in flight, then the lanes are summed.
    float q[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) q[i] = 0.f;
    for (int p0 = 0; p0 < rsc.n_parts; p0 += 4 * WAVE) {
      float4 v[4][4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int p = p0 + u * WAVE + lane;
        const float4* src = reinterpret_cast<const float4*>(rsc.ss + (size_t)p * 16);
#pragma unroll
        for (int j = 0; j < 4; ++j)
          v[u][j] = (p < rsc.n_parts && 4 * j < M) ? src[j] : make_float4(0.f, 0.f, 0.f, 0.f);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          q[4 * j] += v[u][j].x; q[4 * j + 1] += v[u][j].y;
          q[4 * j + 2] += v[u][j].z; q[4 * j + 3] += v[u][j].w;
        }
    }
    // (all 16 without a branch between them, so that the sixteen chains of exchanges overlap)
#pragma unroll
    for (int i = 0; i < 16; ++i) q[i] = wave_sum(q[i]);
    if (lane < 16) {
      float t = q[0];
#pragma unroll
      for (int i = 1; i < 16; ++i) t = lane == i ? q[i] : t;
      row_ss[lane] = t;
    }
  }
  // The conv step's epilogue (EPI 2, 3) needs the rows' state, the channel's taps and the biases:
  // asked for now by the lanes that will use them (two round trips, the slot first), so that they
  // have arrived when the stream of W has gone through.  Up to CONV_PRE taps are held this way;
  // a longer filter reads the rest when it gets there.
  constexpr int CONV_PRE = 4;
  float st_pre[4][CONV_PRE], tap_pre[CONV_PRE + 1], conv_bias_pre = 0.f;
  float gate_bias_pre[3] = {0.f, 0.f, 0.f};
  bool fresh_pre[4] = {true, true, true, true};
  float* st_ptr[4] = {nullptr, nullptr, nullptr, nullptr};
  if ((EPI == 2 || EPI == 3) && wave < MT && gn < N && (EPI != 3 || col < 8)) {
    const int H = cs.L - 1;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int gm = wave * 16 + 4 * (lane / 16) + v;
      if (gm < M) {
        fresh_pre[v] = cs.seg_pos0[gm] == 0;
        st_ptr[v] = cs.state + ((size_t)cs.seg_slot[gm] * N + gn) * H;
      }
    }
#pragma unroll
    for (int v = 0; v < 4; ++v)
#pragma unroll
      for (int k = 0; k < CONV_PRE; ++k)
        st_pre[v][k] = (st_ptr[v] != nullptr && !fresh_pre[v] && k < H) ? st_ptr[v][k] : 0.f;
#pragma unroll
    for (int k = 0; k <= CONV_PRE; ++k) tap_pre[k] = k <= H ? cs.taps[(size_t)gn * cs.L + k] : 0.f;
    if (cs.conv_bias) conv_bias_pre = cs.conv_bias[gn];
    if (bias) {
      gate_bias_pre[0] = bias[gn];
      gate_bias_pre[1] = bias[N + gn];
      gate_bias_pre[2] = bias[2 * N + gn];
    }
  }
  const int kblk = ((K + 32 * (int)gridDim.y - 1) / (32 * (int)gridDim.y)) * 32;   // K a block
  const int kb0 = blockIdx.y * kblk, kb1 = min(K, kb0 + kblk);
  const int kper = ((kb1 - kb0 + 32 * NW - 1) / (32 * NW)) * 32;
  const int k0 = kb0 + wave * kper;
  const int k1 = min(kb1, k0 + kper);
  C += (size_t)blockIdx.y * M * ldc;
  // loads in flight a lane: U * (NG + MT)
  constexpr int U = (NG + MT) <= 3 ? SK_UNROLL : ((NG + MT) <= 6 ? 4 : 2);
  auto products = [&](const u32x4_t (&wv)[U][NG], const u32x4_t (&av)[U][MT]) {
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int r = 0; r < NG; ++r)
#pragma unroll
        for (int t = 0; t < MT; ++t)
          acc[r * MT + t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
              as_bf16x8(av[u][t]), as_bf16x8(wv[u][r]), acc[r * MT + t], 0, 0, 0);
  };
  {
    for (int k = k0; k < k1; k += 32 * U) {
      // the loads of W and of A alternate, in the order of K
      u32x4_t wv[U][NG], av[U][MT];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int gk = k + 32 * u;
        const bool kin = gk + kg < k1;
#pragma unroll
        for (int r = 0; r < NG; ++r)
          wv[u][r] = (kin && gn + (EPI == 0 ? r * 16 : 0) < N && group_ok(r))
                         ? load16(wrow + r * group_rows * K + (size_t)gk * kmul)
                         : zero;
#pragma unroll
        for (int t = 0; t < MT; ++t)
          av[u][t] = (kin && t * 16 + col < M) ? load16(arow[t] + (size_t)gk * (a_frag ? 16 : 1)) : zero;
      }
      products(wv, av);
    }
  }
  if (wave < NW) {
#pragma unroll
    for (int t = 0; t < NG * MT; ++t)
#pragma unroll
      for (int v = 0; v < 4; ++v) red[wave][t][lane][v] = acc[t][v];
  }
  __syncthreads();
  if (wave >= NW) return;
  auto scale_of = [&](int gm) {
    return rsc.ss != nullptr ? 1.0f / sqrtf(row_ss[gm] / (float)K + rsc.eps) : 1.0f;
  };
  // the first MT waves each sum one row tile over the NW partial results, in a fixed order
  if (EPI == 0 && NT > 1) {
    // waves take the NT * MT tiles in turn
    for (int tile = wave; tile < NT * MT; tile += NW) {
      const int r = tile / MT, t = tile % MT;
      const int gnr = gn + r * 16;
      if (gnr >= N) continue;
      const float bv = (bias && blockIdx.y == 0) ? bias[gnr] : 0.f;
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int gm = t * 16 + 4 * (lane / 16) + v;
        if (gm >= M) continue;
        float sum = red[0][tile][lane][v];
#pragma unroll
        for (int w = 1; w < NW; ++w) sum += red[w][tile][lane][v];
        store_out(C + (size_t)gm * ldc + gnr, sum * scale_of(gm) + bv);
      }
    }
  } else if (wave < MT && gn < N && (EPI != 3 || col < 8)) {
    const int t = wave;
    const float bv = (bias && blockIdx.y == 0) ? bias[gn] : 0.f;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int gm = t * 16 + 4 * (lane / 16) + v;
      if (gm < M) {
        const float rs = scale_of(gm);
        float sum = red[0][t][lane][v];
#pragma unroll
        for (int w = 1; w < NW; ++w) sum += red[w][t][lane][v];
        sum *= rs;
        if (EPI == 1) {
          float up = red[0][MT + t][lane][v];
#pragma unroll
          for (int w = 1; w < NW; ++w) up += red[w][MT + t][lane][v];
          store_out(C + out_at(gm, gn), silu_f(sum) * (up * rs));
        } else if (EPI == 2 || EPI == 3) {
          // where the other two gates of this channel lie: EPI 2 in row groups 1 and 2 of this
          // lane, EPI 3 the C gate 8 columns further in group 0 and the x gate in group 1
          const int cg_t = EPI == 2 ? MT + t : t, cg_lane = EPI == 2 ? lane : lane + 8;
          const int xg_t = EPI == 2 ? 2 * MT + t : MT + t;
          float cg = red[0][cg_t][cg_lane][v], xg = red[0][xg_t][lane][v];
#pragma unroll
          for (int w = 1; w < NW; ++w) {
            cg += red[w][cg_t][cg_lane][v];
            xg += red[w][xg_t][lane][v];
          }
          cg *= rs;
          xg *= rs;
          const float bg = sum + gate_bias_pre[0];
          cg += gate_bias_pre[1];
          xg += gate_bias_pre[2];
          // the three gates are rounded as the unfused path stores them
          const float bx = to_f32(f32_to_bf16(bg)) * to_f32(f32_to_bf16(xg));
          const int H = cs.L - 1;
          const bool fresh = fresh_pre[v];
          float* st = st_ptr[v];
          const float* wc = cs.taps + (size_t)gn * cs.L;
          float s = conv_bias_pre;
          if (H <= CONV_PRE) {
            // everything is in registers already
            float prev = st_pre[v][0];
#pragma unroll
            for (int k = 0; k < CONV_PRE; ++k) {
              if (k < H) {
                s += tap_pre[k] * prev;
                const float next = (k + 1 < H) ? st_pre[v][k + 1 < CONV_PRE ? k + 1 : 0] : bx;
                st[k] = next;
                prev = next;
              }
            }
            float last = tap_pre[0];
#pragma unroll
            for (int k = 1; k <= CONV_PRE; ++k) last = k == H ? tap_pre[k] : last;
            s += last * bx;
          } else {
            float prev = fresh ? 0.f : st[0];
            for (int k = 0; k < H; ++k) {
              s += wc[k] * prev;
              const float next = (k + 1 < H) ? (fresh ? 0.f : st[k + 1]) : bx;
              st[k] = next;
              prev = next;
            }
            s += wc[H] * bx;
          }
          store_out(C + out_at(gm, gn), to_f32(f32_to_bf16(cg)) * s);
        } else {
          store_out(C + (size_t)gm * ldc + gn, sum + bv);
        }
      }
    }
  }
}

// A product whose result joins the residual stream (ResidOut; at most 16 rows, K in one piece).
// Such products have few columns (the model's width), so a block owns 8 of them, and the two
// halves of the matrix tile's 16 columns take the two halves of K: column j < 8 is row n0 + j of
// W over K's first half, column j + 8 the same row over the second half.  The rows of A of the
// two halves meet the one fragment of W in two matrix instructions, whose valid halves are added
// at the end.  Twice as many blocks stream W as with 16 columns a block, and K needs no split
// over blocks, so the residual sum can be made here, in a fixed order.
template <int NW>
__global__ __launch_bounds__(NW * WAVE) void gemm_bf16_into_resid_kernel(
    const bf16_t* __restrict__ A, const bf16_t* __restrict__ W, const float* __restrict__ bias,
    int M, int N, int K, int lda, ResidOut ro, int w_frag, int a_frag) {
  __shared__ float red[NW][2][WAVE][4];
  const int tid = threadIdx.x;
  const int lane = tid % WAVE, wave = tid / WAVE;
  const int col = lane % 16, kg = (lane / 16) * 8;
  const int half = col / 8;
  const int gn = blockIdx.x * 8 + col % 8;               // the lane's row of W
  const int khalf = ((K / 2 + 31) / 32) * 32;            // the second half starts here
  const u32x4_t zero = {0u, 0u, 0u, 0u};
  // what the epilogue needs, asked for before the stream of W
  float resid_in[4] = {0.f, 0.f, 0.f, 0.f};
  float norm_w_in = 0.f;
  if (wave == 0 && half == 0 && gn < N) {
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int gm = 4 * (lane / 16) + v;
      if (gm < M) resid_in[v] = ro.resid[(size_t)gm * ro.ldr + gn];
    }
    if (ro.rows != nullptr) norm_w_in = ro.norm_w[gn];
  }
  const size_t wr = gn < N ? gn : 0;
  const int kmul = w_frag ? 16 : 1;                      // see the kernel above for the two orders
  const bf16_t* wrow = (w_frag ? W + (wr / 16) * 16 * K + ((size_t)(kg / 8) * 16 + wr % 16) * 8
                               : W + wr * K + kg) + (size_t)half * khalf * kmul;
  const int am = col < M ? col : 0;                      // the lane's row of A
  const int amul = a_frag ? 16 : 1;
  const bf16_t* arow = a_frag ? A + ((size_t)(kg / 8) * 16 + am) * 8 : A + (size_t)am * lda + kg;
  const int kper = ((khalf + 32 * NW - 1) / (32 * NW)) * 32;
  const int k0 = wave * kper, k1 = min(khalf, k0 + kper);
  f32x4_t acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
  constexpr int U = SK_UNROLL;
  for (int k = k0; k < k1; k += 32 * U) {
    u32x4_t wv[U], a0[U], a1[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int gk = k + 32 * u;
      const bool in0 = gk + kg < k1 && gk + kg < K;       // within the wave's range of a half
      const bool in1 = in0 && khalf + gk + kg < K;        // and, for the second half, within K
      wv[u] = ((half ? in1 : in0) && gn < N) ? load16(wrow + (size_t)gk * kmul) : zero;
      a0[u] = (in0 && col < M) ? load16(arow + (size_t)gk * amul) : zero;
      a1[u] = (in1 && col < M) ? load16(arow + (size_t)(khalf + gk) * amul) : zero;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      acc0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(a0[u]), as_bf16x8(wv[u]), acc0, 0, 0, 0);
      acc1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(a1[u]), as_bf16x8(wv[u]), acc1, 0, 0, 0);
    }
  }
#pragma unroll
  for (int v = 0; v < 4; ++v) {
    red[wave][0][lane][v] = acc0[v];
    red[wave][1][lane][v] = acc1[v];
  }
  __syncthreads();
  if (wave != 0) return;
  // columns 0-7: the first half's sums of this lane and the second half's of the lane 8 further
  const bool mine = half == 0 && gn < N;
  const float bv = (bias && mine) ? bias[gn] : 0.f;
#pragma unroll
  for (int v = 0; v < 4; ++v) {
    const int gm = 4 * (lane / 16) + v;
    float q = 0.f;
    if (mine && gm < M) {
      float lo = red[0][0][lane][v], hi = red[0][1][lane + 8][v];
#pragma unroll
      for (int w = 1; w < NW; ++w) {
        lo += red[w][0][lane][v];
        hi += red[w][1][lane + 8][v];
      }
      const float x = resid_in[v] + ((lo + hi) + bv);
      ro.resid[(size_t)gm * ro.ldr + gn] = x;
      if (ro.rows != nullptr) {
        const size_t at = ro.rows_frag ? ((size_t)(gn / 8) * 16 + gm) * 8 + gn % 8
                                       : (size_t)gm * N + gn;
        ro.rows[at] = f32_to_bf16(x * norm_w_in);
      }
      q = x * x;
    }
    if (ro.rows != nullptr) {
      // the sum of squares over the block's 8 columns, row by row
      q += __shfl_xor(q, 1, WAVE);
      q += __shfl_xor(q, 2, WAVE);
      q += __shfl_xor(q, 4, WAVE);
      if (col == 0 && gm < M) ro.ss[(size_t)blockIdx.x * 16 + gm] = q;
    }
  }
}

static void launch_into_resid(const bf16_t* A, const bf16_t* W, const float* bias, int M, int N,
                              int K, int lda, const ResidOut& ro, hipStream_t stream,
                              const bf16_t* Wf, int a_frag) {
  const int w_frag = Wf != nullptr;
  if (Wf) W = Wf;
  const dim3 grid((N + 7) / 8);
  // K a wave: 128 or more where K allows it
  if (K >= 4096)
    hipLaunchKernelGGL((gemm_bf16_into_resid_kernel<16>), grid, dim3(16 * WAVE), 0, stream, A, W,
                       bias, M, N, K, lda, ro, w_frag, a_frag);
  else if (K >= 1024)
    hipLaunchKernelGGL((gemm_bf16_into_resid_kernel<8>), grid, dim3(8 * WAVE), 0, stream, A, W,
                       bias, M, N, K, lda, ro, w_frag, a_frag);
  else
    hipLaunchKernelGGL((gemm_bf16_into_resid_kernel<4>), grid, dim3(4 * WAVE), 0, stream, A, W,
                       bias, M, N, K, lda, ro, w_frag, a_frag);
}

struct Fuse {
  RowScale rsc;
  ResidOut ro;
  int c_frag = 0;
};

template <typename TO, int MT, int NW, int EPI, int NT = 1>
static void launch_skinny(const bf16_t* A, const bf16_t* W, const float* bias, TO* C, int M, int N,
                          int K, int lda, int ldc, int ksplit, ConvStep cs, hipStream_t stream,
                          const Fuse& fuse = Fuse{}, const bf16_t* Wf = nullptr, int a_frag = 0) {
  // Wf: the copy of W in fragment order (see the kernel), or null
  const int w_frag = Wf != nullptr;
  if (Wf) W = Wf;
  const dim3 grid(EPI == 3 ? (N + 7) / 8 : (N + 16 * NT - 1) / (16 * NT), ksplit);
  // one wave more when there are row scales to make (launch_skinny_mt keeps NW below 16 then)
  const int waves = fuse.rsc.ss != nullptr ? NW + 1 : NW;
  if (waves * WAVE > 1024) return;
  hipLaunchKernelGGL((gemm_bf16_skinny_kernel<TO, MT, NW, EPI, NT>), grid, dim3(waves * WAVE), 0,
                     stream, A, W, bias, C, M, N, K, lda, ldc, cs, fuse.rsc, w_frag, a_frag,
                     (MT == 1 && EPI != 0) ? fuse.c_frag : 0);
}

// more waves a block when there are few blocks, so that about 2048 waves or more stream W
template <typename TO, int MT, int EPI>
static void launch_skinny_mt(const bf16_t* A, const bf16_t* W, const float* bias, TO* C, int M,
                             int N, int K, int lda, int ldc, int ksplit, ConvStep cs,
                             hipStream_t stream, const Fuse& fuse = Fuse{},
                             const bf16_t* Wf = nullptr, int a_frag = 0) {
  // several row tiles and a plain product: a wave takes two column tiles for every fragment
  // of A it loads, which halves the reads of A (every block reads all of it)
  if constexpr (EPI == 0 && MT >= 2) {
    if (N >= 64) {
      launch_skinny<TO, MT, 4, EPI, 2>(A, W, bias, C, M, N, K, lda, ldc, ksplit, cs, stream,
                                       Fuse{}, Wf, a_frag);
      return;
    }
  }
  // 8 to 16 rows and columns enough (the output head): four column tiles for every fragment of
  // A (58 against 62 us for 65,536 columns at 8 rows, 62 against 74 at 16; slower below 8 rows).
  // With W in fragment order one tile a wave is the faster up to 11 rows (50 against 56 us at 8
  // rows, 56 either way at 12, 62 against 56 at 16).
  if constexpr (EPI == 0 && MT == 1) {
    if (M >= (Wf ? 12 : 8) && (long)(N / 64) * ksplit >= 512) {
      launch_skinny<TO, MT, 4, EPI, 4>(A, W, bias, C, M, N, K, lda, ldc, ksplit, cs, stream,
                                       fuse, Wf, a_frag);
      return;
    }
  }
  const int blocks = (EPI == 3 ? (N + 7) / 8 : (N + 15) / 16) * ksplit;
  const int kb = K / ksplit;                              // K a block
  constexpr int NG = EPI == 1 ? 2 : (EPI == 2 ? 3 : (EPI == 3 ? 2 : 1));
  constexpr int MAXW = 48 / (MT * NG);                    // 1 KB of LDS a wave, group and row tile
  if (blocks * 4 >= 2048 || kb <= 512 || MAXW < 8)
    launch_skinny<TO, MT, 4, EPI>(A, W, bias, C, M, N, K, lda, ldc, ksplit, cs, stream, fuse, Wf, a_frag);
  else if (blocks * 8 >= 2048 || kb <= 1024 || MAXW < 16)
    launch_skinny<TO, MT, (MAXW >= 8 ? 8 : 4), EPI>(A, W, bias, C, M, N, K, lda, ldc, ksplit, cs,
                                                    stream, fuse, Wf, a_frag);
  else if (fuse.rsc.ss != nullptr)      // (the block needs room for the wave that makes the scales)
    launch_skinny<TO, MT, (MAXW >= 8 ? 8 : 4), EPI>(A, W, bias, C, M, N, K, lda, ldc, ksplit, cs,
                                                    stream, fuse, Wf, a_frag);
  else
    launch_skinny<TO, MT, (MAXW >= 16 ? 16 : 4), EPI>(A, W, bias, C, M, N, K, lda, ldc, ksplit, cs,
                                                      stream, fuse, Wf, a_frag);
}

// ---------------------------------------------------------------------------------------
// 17 to 64 rows (decode at larger batches): the activations go through LDS
// ---------------------------------------------------------------------------------------
// With several row tiles every wave of the kernel above reads all rows of A for its K range
// from L2 again, which at 64 rows is twice the bytes of W it streams.  Here a block is
// NWN x NWK waves: wave (wn, wk) owns 32 rows of W (two column tiles, or the gate and up rows
// of 16 SwiGLU columns) and the wk-th part of the block's K range, and the NWN waves with the
// same wk share the rows of A: chunk by chunk of KC of K they are loaded once, straight into
// LDS (global_load_lds, two buffers, 16-byte chunks permuted so that a fragment read is free of
// bank conflicts), while W goes from global memory into registers, one chunk ahead.  The waves
// meet in LDS at the end to add their K parts in a fixed order.
//
// Host side guarantees: K / gridDim.y is a multiple of NWK * KC, M * lda < 2^31.  Rows of A
// past M and rows of W past the end repeat the last row (their products are not stored).
template <int MT, int NWN, int NWK, int KC>
struct SharedRows {
  static constexpr int NW = NWN * NWK, ROWS = 16 * MT, CH = KC / 8, UK = KC / 32;
  static constexpr int RPI = 64 / CH;                        // rows a load instruction brings
  static constexpr int INSTR = NWK * ROWS / RPI;             // load instructions a chunk
  static constexpr int PER_WAVE = (INSTR + NW - 1) / NW;
  static constexpr int BUF = NWK * ROWS * KC;                // bf16 elements a buffer
  static constexpr size_t stage_bytes = 2 * (size_t)BUF * sizeof(bf16_t);
  static constexpr size_t red_bytes = (size_t)NW * 2 * MT * WAVE * sizeof(f32x4_t);
  static constexpr size_t lds_bytes = stage_bytes > red_bytes ? stage_bytes : red_bytes;
  __device__ static int swz(int row) { return CH == 16 ? (row & 15) : ((row >> 1) & 7); }
};

template <typename TO, int MT, int EPI, int NWN, int NWK, int KC, int NSETS>
__global__ __launch_bounds__(NWN * NWK * WAVE) void gemm_bf16_shared_rows_kernel(
    const bf16_t* __restrict__ A, const bf16_t* __restrict__ W, const float* __restrict__ bias,
    TO* __restrict__ C, int M, int n_rows_w, int K, int lda, int ldc, int w_frag) {
  static_assert(NSETS % 2 == 0 && 2 * (KC / 32) * (NSETS - 1) < 64, "register sets");
  using S = SharedRows<MT, NWN, NWK, KC>;
  constexpr int NW = S::NW, UK = S::UK, CH = S::CH;
  extern __shared__ __attribute__((aligned(1024))) bf16_t lds[];
  const int tid = threadIdx.x, lane = tid % WAVE;
  const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
  const int wn = wave / NWK, wk = wave % NWK;
  const int col = lane % 16, kgi = lane / 16;
  const int kblk = K / (int)gridDim.y;               // K of the block
  const int kper = kblk / NWK;                       // K of a wave
  const int nchunks = kper / KC;
  const int kb0 = blockIdx.y * kblk;
  C += (size_t)blockIdx.y * M * ldc;

  // rows of W of this wave: group r = rows wrow0 + 16 r + (0..15)
  const int wrow0 = (blockIdx.x * NWN + wn) * 32;
  const bf16_t* wptr[2];
#pragma unroll
  for (int r = 0; r < 2; ++r) {
    // W as stored, or its copy in fragment order (see gemm_bf16_skinny_kernel): a step of 32
    // along K is 32 elements here and 512 there
    const size_t row = (size_t)min(wrow0 + 16 * r + col, n_rows_w - 1);
    const size_t kbase = (size_t)kb0 + (size_t)wk * kper;
    wptr[r] = w_frag ? W + (row / 16) * 16 * K + kbase * 16 + ((size_t)kgi * 16 + row % 16) * 8
                     : W + row * K + kbase + kgi * 8;
  }
  const int kmul = w_frag ? 16 : 1;

  // the block's load instructions for a chunk of A, dealt round the waves: instruction j
  // brings rows (j % (ROWS / RPI)) * RPI + lane / CH of K part j / (ROWS / RPI)
  uint32_t aoff[S::PER_WAVE];
#pragma unroll
  for (int i = 0; i < S::PER_WAVE; ++i) {
    const int j = i * NW + wave;
    const int part = j / (S::ROWS / S::RPI), row = (j % (S::ROWS / S::RPI)) * S::RPI + lane / CH;
    const int chunk = (lane % CH) ^ S::swz(row);
    aoff[i] = (uint32_t)(min(row, M - 1) * lda + kb0 + part * kper + chunk * 8) *
              (uint32_t)sizeof(bf16_t);
  }
  auto stage = [&](int buf, int c) {
    const uint64_t p = reinterpret_cast<uint64_t>(A) + (uint64_t)c * (KC * sizeof(bf16_t));
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)p);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(p >> 32));
    const char* base = reinterpret_cast<const char*>(((uint64_t)hi << 32) | lo);
#pragma unroll
    for (int i = 0; i < S::PER_WAVE; ++i) {
      const int j = i * NW + wave;
      if (S::INSTR % NW == 0 || j < S::INSTR)
        __builtin_amdgcn_global_load_lds(KAPPAI_GPTR(base + aoff[i]),
                                         KAPPAI_LPTR(lds + buf * S::BUF + j * 512), 16, 0, 0);
    }
  };
  auto load_w = [&](u32x4_t (&wv)[UK][2], int c) {
#pragma unroll
    for (int u = 0; u < UK; ++u)
#pragma unroll
      for (int r = 0; r < 2; ++r) wv[u][r] = load16(wptr[r] + (size_t)(c * KC + 32 * u) * kmul);
  };
  f32x4_t acc[2 * MT];
#pragma unroll
  for (int t = 0; t < 2 * MT; ++t) acc[t] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
  // fragment of A: lane holds row 16 t + col, the 8 of K number 4 u + kgi of the chunk
  int roff[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) roff[t] = (wk * S::ROWS + 16 * t + col) * KC;
  auto products = [&](const u32x4_t (&wv)[UK][2], int buf) {
#pragma unroll
    for (int u = 0; u < UK; ++u) {
      u32x4_t av[MT];
#pragma unroll
      for (int t = 0; t < MT; ++t)
        av[t] = *reinterpret_cast<const u32x4_t*>(
            lds + buf * S::BUF + roff[t] + (((4 * u + kgi) ^ S::swz(16 * t + col)) * 8));
#pragma unroll
      for (int r = 0; r < 2; ++r)
#pragma unroll
        for (int t = 0; t < MT; ++t)
          acc[r * MT + t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
              as_bf16x8(av[t]), as_bf16x8(wv[u][r]), acc[r * MT + t], 0, 0, 0);
    }
  };

  // W is loaded NSETS - 1 chunks ahead into register sets used in turn; A one chunk ahead.  In
  // every pass of the loop the loads of A are issued before those of W, and loads come back in
  // the order they were issued: waiting until only the latest pass's loads of W are out means that
  // the chunk of A issued before them has landed.  NSETS is even, so that the LDS buffer of a pass
  // is known at compile time (else the compiler waits for every load before it reads LDS).
  u32x4_t wv[NSETS][UK][2];
  stage(0, 0);
#pragma unroll
  for (int s = 0; s < NSETS - 1; ++s)
    if (s < nchunks) load_w(wv[s], s);
  constexpr int VM_ROUND = 0x0F70 | ((2 * UK) & 15) | (((2 * UK) >> 4) << 14);
  constexpr int VM_FIRST = 0x0F70 | ((2 * UK * (NSETS - 1)) & 15) | (((2 * UK * (NSETS - 1)) >> 4) << 14);
  for (int c = 0; c < nchunks; c += NSETS) {
#pragma unroll
    for (int s = 0; s < NSETS; ++s) {
      const int cc = c + s;
      if (cc >= nchunks) break;
      // chunk cc of A was issued in round cc - 1 and after it that round's chunk of W, if there
      // was one left to load (before the loop: chunk 0 of A, then NSETS - 1 chunks of W)
      if (cc == 0 && nchunks >= NSETS - 1)
        __builtin_amdgcn_s_waitcnt(VM_FIRST);
      else if (cc > 0 && cc + NSETS - 2 < nchunks)
        __builtin_amdgcn_s_waitcnt(VM_ROUND);
      else
        __builtin_amdgcn_s_waitcnt(0x0F70);
      // everybody's part of chunk cc is there and nobody reads the other buffer any more (a
      // bare barrier: a fence would wait for the loads of W that are meant to stay in flight)
      __builtin_amdgcn_s_barrier();
      SCHED_FENCE();
      if (cc + 1 < nchunks) stage((s + 1) & 1, cc + 1);
      if (cc + NSETS - 1 < nchunks) load_w(wv[(s + NSETS - 1) % NSETS], cc + NSETS - 1);
      products(wv[s], s & 1);
    }
  }
  __syncthreads();
  // the K parts meet: wave (wn, wk) adds up and stores row tiles wk, wk + NWK, ...
  f32x4_t* red = reinterpret_cast<f32x4_t*>(lds);
#pragma unroll
  for (int t = 0; t < 2 * MT; ++t) red[(wave * 2 * MT + t) * WAVE + lane] = acc[t];
  __syncthreads();
  for (int t = wk; t < MT; t += NWK) {
    f32x4_t sum[2];
#pragma unroll
    for (int r = 0; r < 2; ++r) {
      sum[r] = red[((wn * NWK) * 2 * MT + r * MT + t) * WAVE + lane];
#pragma unroll
      for (int w = 1; w < NWK; ++w) sum[r] += red[((wn * NWK + w) * 2 * MT + r * MT + t) * WAVE + lane];
    }
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int gm = 16 * t + 4 * kgi + v;
      if (gm >= M) continue;
      if (EPI == 1) {
        const int on = wrow0 / 2 + col;                 // 16 output columns a wave
        if (wrow0 + 16 + col < n_rows_w)
          store_out(C + (size_t)gm * ldc + on, silu_f(sum[0][v]) * sum[1][v]);
      } else {
#pragma unroll
        for (int r = 0; r < 2; ++r) {
          const int gn = wrow0 + 16 * r + col;
          if (gn < n_rows_w)
            store_out(C + (size_t)gm * ldc + gn,
                      sum[r][v] + ((bias && blockIdx.y == 0) ? bias[gn] : 0.f));
        }
      }
    }
  }
}

template <int NWK, int KC>
static bool shared_rows_fits(int M, int K, int lda, int ksplit) {
  return M > 16 && M <= 64 && ksplit >= 1 && K % (ksplit * NWK * KC) == 0 &&
         (long)M * lda < (1L << 31) - 8 * (long)KC;
}

template <typename TO, int MT, int EPI, int NWN, int NWK, int KC, int NSETS>
static void launch_shared_rows_cfg(const bf16_t* A, const bf16_t* W, const float* bias, TO* C,
                                   int M, int n_rows_w, int K, int lda, int ldc, int ksplit,
                                   hipStream_t stream, const bf16_t* Wf) {
  using S = SharedRows<MT, NWN, NWK, KC>;
  auto kern = gemm_bf16_shared_rows_kernel<TO, MT, EPI, NWN, NWK, KC, NSETS>;
  static bool attr_set = false;       // more than 64 KB of LDS has to be asked for once
  if (!attr_set) {
    (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)S::lds_bytes);
    attr_set = true;
  }
  hipLaunchKernelGGL(kern, dim3((n_rows_w + 32 * NWN - 1) / (32 * NWN), ksplit),
                     dim3(S::NW * WAVE), S::lds_bytes, stream, A, Wf ? Wf : W, bias, C, M, n_rows_w, K,
                     lda, ldc, Wf ? 1 : 0);
}

// 2 x 4 waves, chunks of 128 of K, two register sets of W.  (4 x 4 waves leave half the CUs
// without a block on the layer shapes; more register sets or 16 waves with chunks of 64 gain
// nothing.)  Returns false when the shape does not fit.
#define SR_NWN 2
#define SR_NWK 4
#define SR_KC 128
template <typename TO, int EPI>
static bool launch_shared_rows(const bf16_t* A, const bf16_t* W, const float* bias, TO* C, int M,
                               int n_rows_w, int K, int lda, int ldc, int ksplit,
                               hipStream_t stream, const bf16_t* Wf) {
  if (!shared_rows_fits<SR_NWK, SR_KC>(M, K, lda, ksplit)) return false;
  if (M <= 32)
    launch_shared_rows_cfg<TO, 2, EPI, SR_NWN, SR_NWK, SR_KC, 2>(A, W, bias, C, M, n_rows_w, K, lda,
                                                                 ldc, ksplit, stream, Wf);
  else if (M <= 48)
    launch_shared_rows_cfg<TO, 3, EPI, SR_NWN, SR_NWK, SR_KC, 2>(A, W, bias, C, M, n_rows_w, K, lda,
                                                                 ldc, ksplit, stream, Wf);
  else
    launch_shared_rows_cfg<TO, 4, EPI, SR_NWN, SR_NWK, SR_KC, 2>(A, W, bias, C, M, n_rows_w, K, lda,
                                                                 ldc, ksplit, stream, Wf);
  return true;
}

// ---------------------------------------------------------------------------------------
// 25 to 128 rows (decode at batches of that size, short prompt portions): 32 x 32 tiles, rows
// via LDS
// ---------------------------------------------------------------------------------------
// The block kernels above need hundreds of rows to fill their tiles, and the kernel for 17 to 64
// rows reads every fragment of A once per 16 x 16 tile (it still runs where this one does not
// fit: a matrix kept as rows, a K range that is no multiple of 256).  Here a block is 2 x 4 waves: wave
// (wn, wk) owns 32 rows of W (one 32 x 32 tile of the result for each 32 rows of A,
// v_mfma_f32_32x32x16_bf16: half the LDS reads per product of the 16 x 16 form) and, of every
// run of 256 of the block's K range, the 64 number wk.  The block's rows of A go through LDS run
// by run (global_load_lds, two buffers of rows x 256, rows of 128 bytes per 64 of K permuted as
// in the block kernel: a fragment read is free of bank conflicts), W comes from its
// fragment-order copy straight into registers, one run ahead: a load instruction takes the two
// pieces of the wave's 32 rows, 256 bytes of each of two groups of 8 of K.  The waves meet in LDS
// at the end to add their K parts in a fixed order.  K can be cut over blocks as well (float
// partial sums), which is what fills the chip for the products with few rows of W.
// Measured at the LFM2-1.2B shapes, W cold, 128 rows: gate/up 23.2 against 26.7 us (the 128 x 128
// block form), in_proj 13.0 against 14.1, qkv 9.1 against 12.4, out_proj 7.4 against 8.0, down
// 15.5 against 20.6; 64 rows against the kernel for 17 to 64 rows: gate/up 18.4 against 20.5, qkv
// 7.0 against 10.7, in_proj 10.0 against 11.0.  A wave that owns 64 rows of W (half the reads of A
// from L2 and LDS) was slower (29 us for gate/up at 128 rows), and so were 4 x 2 waves.
//
// Host side guarantees: W in fragment order, K / gridDim.y a multiple of 256, lda a multiple of
// 8, M * lda < 2^31.  Rows of A past M repeat the last row, pieces of W past the end the last
// piece (their products are not stored).
#define R32_NWN 2
#define R32_NWK 4
static_assert(R32_NWK * 64 == KAPPAI_ROWS32_RUN, "the rule for K ranges counts in runs");
template <typename TO, int MT, int EPI>
__global__ __launch_bounds__(R32_NWN * R32_NWK * WAVE) void gemm_bf16_rows32_kernel(
    const bf16_t* __restrict__ A, const bf16_t* __restrict__ Wf, const float* __restrict__ bias,
    TO* __restrict__ C, int M, int n_rows_w, int K, int lda, int ldc) {
  constexpr int NWN = R32_NWN, NWK = R32_NWK, NW = NWN * NWK, ROWS = 32 * MT, RUN = NWK * 64;
  constexpr int BUF = ROWS * RUN;                       // bf16 elements a buffer
  constexpr int INSTR = ROWS * NWK / 8;                 // load instructions a run (8 rows x 128 B)
  constexpr int PER_WAVE = INSTR / NW;
  static_assert(INSTR % NW == 0, "the loads of a run are dealt round the waves evenly");
  extern __shared__ __attribute__((aligned(1024))) bf16_t lds[];
  const int tid = threadIdx.x, lane = tid % WAVE;
  const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
  const int wn = wave / NWK, wk = wave % NWK;
  const int r_in = lane % 32, hh = lane / 32;
  const int kblk = K / (int)gridDim.y;
  const int nruns = kblk / RUN;
  const int kb0 = blockIdx.y * kblk;
  C += (size_t)blockIdx.y * M * ldc;

  // W: lane -> row wrow0 + r_in, the 8 of K number hh (+ 2 for the second 16) of a piece of 16
  // rows x 32 of K; step s of a run (16 of K) lies in piece s / 2, half s % 2
  const int wrow0 = (blockIdx.x * NWN + wn) * 32;
  const int piece_row = min((wrow0 + r_in) / 16, n_rows_w / 16 - 1);
  const bf16_t* wbase = Wf + ((size_t)piece_row * (K / 32) + (kb0 + wk * 64) / 32) * 512 +
                        (hh * 16 + r_in % 16) * 8;
  auto load_w = [&](u32x4_t (&wv)[4], int run) {
    const bf16_t* p = wbase + (size_t)run * (RUN / 32) * 512;
#pragma unroll
    for (int s = 0; s < 4; ++s) wv[s] = load16(p + (s / 2) * 512 + (s % 2) * 256);
  };

  // A: instruction j of a run brings rows (j % (ROWS / 8)) * 8 + lane / 8 of the 64 number
  // j / (ROWS / 8) of the run; in LDS: the four 64s one after the other, rows of 128 bytes
  uint32_t aoff[PER_WAVE];
#pragma unroll
  for (int i = 0; i < PER_WAVE; ++i) {
    const int j = i * NW + wave;
    const int slice = j / (ROWS / 8), row = (j % (ROWS / 8)) * 8 + lane / 8;
    const int chunk = (lane % 8) ^ ((row >> 1) & 7);
    aoff[i] = (uint32_t)(min(row, M - 1) * lda + kb0 + slice * 64 + chunk * 8) *
              (uint32_t)sizeof(bf16_t);
  }
  auto stage = [&](int buf, int run) {
    const uint64_t p = reinterpret_cast<uint64_t>(A) + (uint64_t)run * (RUN * sizeof(bf16_t));
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)p);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(p >> 32));
    const char* base = reinterpret_cast<const char*>(((uint64_t)hi << 32) | lo);
#pragma unroll
    for (int i = 0; i < PER_WAVE; ++i) {
      const int j = i * NW + wave;
      const int slice = j / (ROWS / 8), rowblk = j % (ROWS / 8);
      __builtin_amdgcn_global_load_lds(
          KAPPAI_GPTR(base + aoff[i]),
          KAPPAI_LPTR(lds + buf * BUF + (slice * ROWS + rowblk * 8) * 64), 16, 0, 0);
    }
  };

  f32x16_t acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[t][v] = 0.f;
  // fragment of A: lane -> row 32 t + r_in, chunk 2 s + hh of the wave's 64
  int roff[4];
#pragma unroll
  for (int s = 0; s < 4; ++s)
    roff[s] = (wk * ROWS + r_in) * 64 + (((2 * s + hh) ^ ((r_in >> 1) & 7)) * 8);
  auto products = [&](const u32x4_t (&wv)[4], int buf) {
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      u32x4_t av[MT];
#pragma unroll
      for (int t = 0; t < MT; ++t)
        av[t] = *reinterpret_cast<const u32x4_t*>(lds + buf * BUF + roff[s] + t * 32 * 64);
#pragma unroll
      for (int t = 0; t < MT; ++t)
        acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(wv[s]), as_bf16x8(av[t]), acc[t],
                                                         0, 0, 0);
    }
  };

  // W one run ahead in two register sets used in turn, A one run ahead in the other LDS buffer.
  // In every pass of the loop the loads of A are issued before those of W, and loads come back in
  // the order they were issued: waiting until only the latest pass's four loads of W are out means
  // that the run of A issued before them has landed (and the run of W before that).
  u32x4_t wv[2][4];
  stage(0, 0);
  load_w(wv[0], 0);
  for (int c = 0; c < nruns; c += 2) {
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const int cc = c + s;
      if (cc >= nruns) break;
      // run cc of A was issued before the four loads of run cc of W, which may stay out
      __builtin_amdgcn_s_waitcnt(0x0F70 | 4);       // vmcnt(4)
      // everybody's part of run cc is there and nobody reads the other buffer any more (a bare
      // barrier: a fence would wait for the loads of W that are meant to stay in flight)
      __builtin_amdgcn_s_barrier();
      SCHED_FENCE();
      if (cc + 1 < nruns) {
        stage((s + 1) & 1, cc + 1);
        load_w(wv[(s + 1) & 1], cc + 1);
      }
      products(wv[s], s & 1);
    }
  }
  // the K parts meet: wave (wn, wk) adds up and stores row tiles wk, wk + 4, ...
  // acc[t][v] is C[row 32 t + r_in][column wrow0 + 8 (v / 4) + 4 hh + v % 4]
  __syncthreads();
  float* red = reinterpret_cast<float*>(lds);
  constexpr int RSTRIDE = MT * 16 * WAVE;               // floats a wave
#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int v = 0; v < 16; ++v) red[wave * RSTRIDE + (t * 16 + v) * WAVE + lane] = acc[t][v];
  __syncthreads();
  for (int t = wk; t < MT; t += NWK) {
    float sum[16];
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      sum[v] = red[(wn * NWK) * RSTRIDE + (t * 16 + v) * WAVE + lane];
#pragma unroll
      for (int w = 1; w < NWK; ++w)
        sum[v] += red[(wn * NWK + w) * RSTRIDE + (t * 16 + v) * WAVE + lane];
    }
    const int gm = 32 * t + r_in;
    if (gm >= M) continue;
    if (EPI == 1) {
      // rows 0..15 of the wave's W are gate rows, 16..31 the up rows of the same 16 columns:
      // registers v and v + 8 of a lane
      if (wrow0 + 16 < n_rows_w) {
#pragma unroll
        for (int g = 0; g < 2; ++g) {
          uint2 pk;
          pk.x = pack_bf16x2(silu_f(sum[4 * g]) * sum[4 * g + 8],
                             silu_f(sum[4 * g + 1]) * sum[4 * g + 9]);
          pk.y = pack_bf16x2(silu_f(sum[4 * g + 2]) * sum[4 * g + 10],
                             silu_f(sum[4 * g + 3]) * sum[4 * g + 11]);
          if constexpr (sizeof(TO) == 2)
            *reinterpret_cast<uint2*>(C + (size_t)gm * ldc + wrow0 / 2 + 8 * g + 4 * hh) = pk;
        }
      }
    } else {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int gn = wrow0 + 8 * g + 4 * hh;
        if (gn >= n_rows_w) continue;
        float o[4];
#pragma unroll
        for (int e = 0; e < 4; ++e)
          o[e] = sum[4 * g + e] + ((bias && blockIdx.y == 0) ? bias[gn + e] : 0.f);
        TO* dst = C + (size_t)gm * ldc + gn;
        if constexpr (sizeof(TO) == 2) {
          uint2 pk;
          pk.x = pack_bf16x2(o[0], o[1]);
          pk.y = pack_bf16x2(o[2], o[3]);
          *reinterpret_cast<uint2*>(dst) = pk;
        } else {
          *reinterpret_cast<float4*>(dst) = make_float4(o[0], o[1], o[2], o[3]);
        }
      }
    }
  }
}

template <typename TO, int MT, int EPI>
static void launch_rows32_cfg(const bf16_t* A, const bf16_t* Wf, const float* bias, TO* C, int M,
                              int n_rows_w, int K, int lda, int ldc, int ksplit,
                              hipStream_t stream) {
  constexpr int NW = R32_NWN * R32_NWK, ROWS = 32 * MT, RUN = R32_NWK * 64;
  constexpr size_t stage_bytes = 2 * (size_t)ROWS * RUN * sizeof(bf16_t);
  constexpr size_t red_bytes = (size_t)NW * MT * 16 * WAVE * sizeof(float);
  constexpr size_t lds_bytes = stage_bytes > red_bytes ? stage_bytes : red_bytes;
  static_assert(lds_bytes <= 160 * 1024, "a block's LDS");
  auto kern = gemm_bf16_rows32_kernel<TO, MT, EPI>;
  static bool attr_set = false;       // more than 64 KB of LDS has to be asked for once
  if (!attr_set) {
    (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)lds_bytes);
    attr_set = true;
  }
  hipLaunchKernelGGL(kern, dim3((n_rows_w + 32 * R32_NWN - 1) / (32 * R32_NWN), ksplit),
                     dim3(NW * WAVE), lds_bytes, stream, A, Wf, bias, C, M, n_rows_w, K, lda, ldc);
}

// Returns false when the shape does not fit (the caller then takes a block kernel).  The output
// must allow the kernel's stores of four values (8 or 16 bytes).
template <typename TO, int EPI>
static bool launch_rows32(const bf16_t* A, const bf16_t* Wf, const float* bias, TO* C, int M,
                          int n_rows_w, int K, int lda, int ldc, int ksplit, hipStream_t stream) {
  const int out_cols = EPI == 1 ? n_rows_w / 2 : n_rows_w;
  if (Wf == nullptr || M < 1 || M > KAPPAI_ROWS32_MAX_ROWS || ksplit < 1 || K % (ksplit * R32_NWK * 64) ||
      n_rows_w % (EPI == 1 ? 32 : 16) || (lda % 8) || (long)M * lda >= (1L << 31) - 2048 ||
      (out_cols % 4) || (ldc % 4) || ((uintptr_t)C % 16) || (EPI == 1 && sizeof(TO) != 2))
    return false;
  switch ((M + 31) / 32) {
    case 1: launch_rows32_cfg<TO, 1, EPI>(A, Wf, bias, C, M, n_rows_w, K, lda, ldc, ksplit, stream); break;
    case 2: launch_rows32_cfg<TO, 2, EPI>(A, Wf, bias, C, M, n_rows_w, K, lda, ldc, ksplit, stream); break;
    case 3: launch_rows32_cfg<TO, 3, EPI>(A, Wf, bias, C, M, n_rows_w, K, lda, ldc, ksplit, stream); break;
    default: launch_rows32_cfg<TO, 4, EPI>(A, Wf, bias, C, M, n_rows_w, K, lda, ldc, ksplit, stream); break;
  }
  return true;
}

template <typename TO, int EPI>
static int launch_bf16(const bf16_t* A, const bf16_t* W, const float* bias, TO* C, int M, int N,
                       int K, int lda, int ldc, int force_kernel, int ksplit, hipStream_t stream,
                       ConvStep cs = ConvStep{}, const bf16_t* Wf = nullptr, int a_frag = 0,
                       const Fuse& fuse = Fuse{}) {
  // a_frag: the rows of A lie in fragment order, which only the kernel for 1 to 16 rows reads
  if (a_frag && (M > 16 || force_kernel == 1 || force_kernel >= 3)) return (int)hipErrorInvalidValue;
  // so are the row scale and the residual epilogue (and the latter only with K in one piece)
  const bool fused = fuse.rsc.ss != nullptr || fuse.ro.resid != nullptr || fuse.c_frag;
  if (fuse.c_frag && (EPI == 0 || (N % 32))) return (int)hipErrorInvalidValue;
  if (fused && (M > 16 || force_kernel == 1 || force_kernel >= 3)) return (int)hipErrorInvalidValue;
  if (fuse.ro.resid != nullptr) {
    if (EPI != 0 || ksplit != 1 || fuse.rsc.ss != nullptr) return (int)hipErrorInvalidValue;
    launch_into_resid(A, W, bias, M, N, K, lda, fuse.ro, stream, Wf, a_frag);
    KAPPAI_RETURN_LAUNCH_STATUS();
  }
  if (fuse.rsc.ss != nullptr && ksplit != 1) return (int)hipErrorInvalidValue;
  // Wf: W in fragment order (see the kernel for 1 to 16 rows); W may be null when Wf is there
  // N counts output columns; with the SwiGLU epilogue W has 2N rows
  // a very wide plain product (the output head) with more than 32 rows streams faster through
  // the 128 x 128 blocks than through the decode kernel, which reads the rows once per 32 columns
  const bool wide_head = EPI == 0 && M > 32 && N >= 16384 && force_kernel == 0 && ksplit == 1 &&
                         block256_fits<TO, EPI>(A, W, C, M, N, K, lda, ldc, ksplit);
  // 25 to 128 rows: 32 x 32 tiles with the rows through LDS, when W is there in fragment order
  // and the shape fits (else the kernels below)
  if constexpr (EPI != 2) {
    if (force_kernel == 12 || (force_kernel == 0 && M > KAPPAI_ROWS32_MIN_ROWS &&
                               M <= KAPPAI_ROWS32_MAX_ROWS &&
                               Wf != nullptr && !wide_head)) {
      if (launch_rows32<TO, EPI>(A, Wf, bias, C, M, EPI == 1 ? 2 * N : N, K, lda, ldc, ksplit,
                                 stream))
        KAPPAI_RETURN_LAUNCH_STATUS();
      if (force_kernel == 12) return (int)hipErrorInvalidValue;
    }
  } else if (force_kernel == 12) {
    return (int)hipErrorInvalidValue;
  }
  // 17 to 64 rows and blocks enough to fill half the chip: the rows go through LDS
  if constexpr (EPI != 2) {
    const int n_rows_w = EPI == 1 ? 2 * N : N;
    const long sr_blocks = (long)((n_rows_w + 32 * SR_NWN - 1) / (32 * SR_NWN)) * ksplit;
    // (with W in fragment order the kernel for few rows keeps up to 24 rows: gate/up 16.6
    // against 17.5 us at 24 rows, 15.7 against 17.6 at 17)
    if (force_kernel == 9 ||
        (force_kernel == 0 && M > (Wf ? 24 : 16) && M <= 64 && sr_blocks >= 128 && !wide_head)) {
      if (launch_shared_rows<TO, EPI>(A, W, bias, C, M, n_rows_w, K, lda, ldc, ksplit, stream, Wf))
        KAPPAI_RETURN_LAUNCH_STATUS();
      if (force_kernel == 9) return (int)hipErrorInvalidValue;
    }
  } else if (force_kernel == 9) {
    return (int)hipErrorInvalidValue;
  }
  if (M <= 64 && force_kernel != 1 && force_kernel < 3 && !wide_head) {
    const int mt = (M + 15) / 16;
    switch (mt) {
      case 1:
        launch_skinny_mt<TO, 1, EPI>(A, W, bias, C, M, N, K, lda, ldc, ksplit, cs, stream, fuse,
                                     Wf, a_frag);
        break;
      case 2:
        launch_skinny_mt<TO, 2, EPI>(A, W, bias, C, M, N, K, lda, ldc, ksplit, cs, stream, Fuse{},
                                     Wf);
        break;
      case 3:
        launch_skinny_mt<TO, 3, EPI>(A, W, bias, C, M, N, K, lda, ldc, ksplit, cs, stream, Fuse{},
                                     Wf);
        break;
      default:
        launch_skinny_mt<TO, 4, EPI>(A, W, bias, C, M, N, K, lda, ldc, ksplit, cs, stream, Fuse{},
                                     Wf);
        break;
    }
  } else {
    // rows of W = columns the tiles run over
    launch_tile<TO, EPI>(A, W, bias, C, M, EPI == 1 ? 2 * N : N, K, lda, ldc, ksplit,
                         force_kernel >= 3 ? force_kernel - 2 : (wide_head && M <= 64 ? 6 : 0),
                         stream, Wf);
  }
  KAPPAI_RETURN_LAUNCH_STATUS();
}

// K, lda must be multiples of 8 and A, W 16-byte aligned (checked by the caller).
// force_kernel: 0 = by M, 1 = tile kernel, 2 = skinny kernel (M <= 64 only), 3..8 = tile kernel
// with block shape 1..6 (see launch_tile), 9 = shared-rows kernel (17 to 64 rows, K / ksplit a
// multiple of 512), 10 = block shape 8, 11 = block shape 9, 12 = the kernel for 25 to 128 rows
// (1 to 128 rows, W in fragment order, K / ksplit a multiple of 256); for tests and tuning.
// ksplit > 1 (float output only): C is [ksplit][M][ldc] partial sums over K ranges.
// W_frag: null, or W in fragment order (K a multiple of 32, rows a multiple of 16); W may then
// be null: every kernel reads the fragment order (only kappai_gemm_bf16_any needs rows).
static bool frag_ok(const void* W_frag, int rows, int K) {
  return W_frag == nullptr || (K % 32 == 0 && rows % 16 == 0 && ((uintptr_t)W_frag % 16) == 0);
}

// The fused forms (at most 16 rows, see RowScale and ResidOut in the kernel for 1 to 16 rows):
// scale_ss [scale_parts][16] (or null) scales every result row by 1 / sqrt(sum of its parts / K +
// scale_eps); resid [M, ldr] (or null; float output, ksplit 1) receives the result added in place
// instead of C, and with norm_w also rows_out (bf16(resid * norm_w), [M, N] or fragment order)
// and ss_out [(N + 7) / 8][16].
static bool fuse_ok(const Fuse& f, int M, int N, int K, int out_is_f32, int ksplit) {
  if (f.rsc.ss != nullptr && (M > 16 || f.rsc.n_parts < 1 || ksplit != 1)) return false;
  if (f.c_frag && M > 16) return false;
  if (f.ro.resid != nullptr) {
    if (M > 16 || !out_is_f32 || ksplit != 1 || f.ro.ldr < N) return false;
    if (f.ro.norm_w != nullptr && (f.ro.rows == nullptr || f.ro.ss == nullptr)) return false;
    if (f.ro.rows_frag && (N % 32)) return false;
  } else if (f.ro.norm_w != nullptr || f.ro.rows != nullptr) {
    return false;
  }
  return true;
}

extern "C" int kappai_gemm_bf16(const void* A, const void* W, const void* W_frag, const float* bias,
                                void* C, int M, int N, int K, int lda, int ldc, int out_is_f32,
                                int force_kernel, int ksplit, int a_frag, const float* scale_ss,
                                int scale_parts, float scale_eps, float* resid, int ldr,
                                const float* norm_w, void* rows_out, int rows_frag, float* ss_out,
                                hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if ((K % 8) || (lda % 8) || ksplit < 1 || ksplit > 64) return (int)hipErrorInvalidValue;
  if (!frag_ok(W_frag, N, K) || (a_frag && (K % 32))) return (int)hipErrorInvalidValue;
  if (force_kernel == 2 && M > 64) return (int)hipErrorInvalidValue;
  if (ksplit > 1 && !out_is_f32) return (int)hipErrorInvalidValue;
  Fuse fuse{RowScale{scale_ss, scale_parts, scale_eps},
            ResidOut{resid, ldr, resid && rows_out ? norm_w : nullptr,
                     resid ? (bf16_t*)rows_out : nullptr, rows_frag, ss_out}};
  if (!fuse_ok(fuse, M, N, K, out_is_f32, ksplit)) return (int)hipErrorInvalidValue;
  if (out_is_f32)
    return launch_bf16<float, 0>((const bf16_t*)A, (const bf16_t*)W, bias, (float*)C, M, N, K, lda,
                                 ldc, force_kernel, ksplit, stream, ConvStep{},
                                 (const bf16_t*)W_frag, a_frag, fuse);
  return launch_bf16<bf16_t, 0>((const bf16_t*)A, (const bf16_t*)W, bias, (bf16_t*)C, M, N, K, lda,
                                ldc, force_kernel, 1, stream, ConvStep{}, (const bf16_t*)W_frag,
                                a_frag, fuse);
}

// C[M, F] = silu(A Wg^T) * (A Wu^T) with W = gate and up rows interleaved in groups of 16,
// [2F, K]; F must be a multiple of 16.
extern "C" int kappai_gemm_bf16_swiglu(const void* A, const void* W, const void* W_frag, void* C,
                                       int M, int F, int K, int lda, int ldc, int force_kernel,
                                       int a_frag, const float* scale_ss, int scale_parts,
                                       float scale_eps, int c_frag, hipStream_t stream) {
  if (M <= 0 || F <= 0) return 0;
  if ((K % 8) || (lda % 8) || (F % 16)) return (int)hipErrorInvalidValue;
  if (force_kernel == 2 && M > 64) return (int)hipErrorInvalidValue;
  if (!frag_ok(W_frag, 2 * F, K) || (a_frag && (K % 32))) return (int)hipErrorInvalidValue;
  Fuse fuse{RowScale{scale_ss, scale_parts, scale_eps}, ResidOut{}, c_frag};
  if (!fuse_ok(fuse, M, F, K, 0, 1)) return (int)hipErrorInvalidValue;
  return launch_bf16<bf16_t, 1>((const bf16_t*)A, (const bf16_t*)W, nullptr, (bf16_t*)C, M, F, K,
                                lda, ldc, force_kernel, 1, stream, ConvStep{},
                                (const bf16_t*)W_frag, a_frag, fuse);
}

// Conv layer decode step in one kernel: C[M, D] = Cgate * conv(Bgate * x | state) from A [M, K]
// and the in_proj matrix W [3D, K]; M <= 64, one row a request; D a multiple of 16.
extern "C" int kappai_gemm_bf16_shortconv_step(const void* A, const void* W, const void* W_frag,
                                               const float* bias,
                                               void* C, int M, int D, int K, int lda,
                                               const float* taps, const float* conv_bias,
                                               float* state, const int* seg_pos0,
                                               const int* seg_slot, int L, int a_frag,
                                               const float* scale_ss, int scale_parts,
                                               float scale_eps, int c_frag, hipStream_t stream) {
  if (M <= 0 || D <= 0) return 0;
  if ((K % 8) || (lda % 8) || (D % 16) || M > 64 || L < 2) return (int)hipErrorInvalidValue;
  if (!frag_ok(W_frag, 3 * D, K) || (a_frag && ((K % 32) || M > 16)))
    return (int)hipErrorInvalidValue;
  Fuse fuse{RowScale{scale_ss, scale_parts, scale_eps}, ResidOut{}, c_frag};
  if (!fuse_ok(fuse, M, D, K, 0, 1) || (c_frag && (D % 32))) return (int)hipErrorInvalidValue;
  const bf16_t* wf = (const bf16_t*)W_frag;
  ConvStep cs{taps, conv_bias, state, seg_pos0, seg_slot, L};
  if (D / 16 < 256) {
    // too few blocks of 16 channels for the chip: 8 channels a block
    const bf16_t* a = (const bf16_t*)A;
    const bf16_t* w = (const bf16_t*)W;
    bf16_t* c = (bf16_t*)C;
    switch ((M + 15) / 16) {
      case 1:
        launch_skinny_mt<bf16_t, 1, 3>(a, w, bias, c, M, D, K, lda, D, 1, cs, stream, fuse, wf,
                                       a_frag);
        break;
      case 2:
        launch_skinny_mt<bf16_t, 2, 3>(a, w, bias, c, M, D, K, lda, D, 1, cs, stream, Fuse{}, wf);
        break;
      case 3:
        launch_skinny_mt<bf16_t, 3, 3>(a, w, bias, c, M, D, K, lda, D, 1, cs, stream, Fuse{}, wf);
        break;
      default:
        launch_skinny_mt<bf16_t, 4, 3>(a, w, bias, c, M, D, K, lda, D, 1, cs, stream, Fuse{}, wf);
        break;
    }
    KAPPAI_RETURN_LAUNCH_STATUS();
  }
  return launch_bf16<bf16_t, 2>((const bf16_t*)A, (const bf16_t*)W, bias, (bf16_t*)C, M, D, K, lda,
                                D, 2, 1, stream, cs, wf, a_frag, fuse);
}

// ---------------------------------------------------------------------------------------
// bf16 at any size and alignment (K or a row stride that is no multiple of 8): one wave per
// row and four output columns, lanes stride over K with 2-byte loads, float sums added up
// across the wave.  Slow, and only there so that no width is refused.
// ---------------------------------------------------------------------------------------
template <typename TO>
__global__ __launch_bounds__(WAVE) void gemm_bf16_any_kernel(
    const bf16_t* __restrict__ A, const bf16_t* __restrict__ W, const float* __restrict__ bias,
    TO* __restrict__ C, int M, int N, int K, int lda, int ldc) {
  const int m = blockIdx.y, n0 = blockIdx.x * 4, lane = threadIdx.x;
  const bf16_t* a = A + (size_t)m * lda;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  for (int k = lane; k < K; k += WAVE) {
    const float x = bf16_to_f32(a[k]);
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (n0 + j < N) acc[j] = fmaf(x, bf16_to_f32(W[(size_t)(n0 + j) * K + k]), acc[j]);
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const float sum = wave_sum(acc[j]);
    if (lane == 0 && n0 + j < N)
      store_out(C + (size_t)m * ldc + n0 + j, sum + (bias ? bias[n0 + j] : 0.f));
  }
}

extern "C" int kappai_gemm_bf16_any(const void* A, const void* W, const float* bias, void* C,
                                    int M, int N, int K, int lda, int ldc, int out_is_f32,
                                    hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K < 1 || M > 65535) return (int)hipErrorInvalidValue;
  const dim3 grid((N + 3) / 4, M);
  if (out_is_f32)
    hipLaunchKernelGGL(gemm_bf16_any_kernel<float>, grid, dim3(WAVE), 0, stream, (const bf16_t*)A,
                       (const bf16_t*)W, bias, (float*)C, M, N, K, lda, ldc);
  else
    hipLaunchKernelGGL(gemm_bf16_any_kernel<bf16_t>, grid, dim3(WAVE), 0, stream,
                       (const bf16_t*)A, (const bf16_t*)W, bias, (bf16_t*)C, M, N, K, lda, ldc);
  KAPPAI_RETURN_LAUNCH_STATUS();
}

// Matrix products  C[M,N] = A[M,K] * W[N,K]^T (+ bias[N])  for every projection and the
// output head.  W is a weight matrix [out, in] with `in` contiguous, as stored in the
// checkpoint (kappai: y[n] = sum_k W[n,k] x[k], src/backend/cpu/scalar/quants.c:1398-1414).
//
//   gemm_f32         true 32-bit on the vector ALUs: every product and sum is an fp32 FMA in
//                    the order k = 0..K-1, so a row's result does not depend on M.
//   gemm_bf16_tile   bf16 inputs, fp32 accumulation on the matrix cores
//                    (v_mfma_f32_32x32x16_bf16), 128x128x32 block tiles staged through LDS.
//   gemm_bf16_skinny M <= 64 (decode): every block streams 16 rows of W once, its four
//                    waves split K and meet in LDS (v_mfma_f32_16x16x32_bf16).
#include "common.h"

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
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += F32_BK) {
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
      if (gn < N) C[(size_t)gm * ldc + gn] = acc[i][j] + (bias ? bias[gn] : 0.f);
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

#define T_BM 128
#define T_BN 128
#define T_BK 32
#define T_LDS (T_BK + 8)  // row stride in bf16: 80 bytes keeps 16-byte alignment, spreads banks

template <typename TO>
__global__ __launch_bounds__(256) void gemm_bf16_tile_kernel(const bf16_t* __restrict__ A,
                                                             const bf16_t* __restrict__ W,
                                                             const float* __restrict__ bias,
                                                             TO* __restrict__ C, int M, int N,
                                                             int K, int lda, int ldc) {
  __shared__ __attribute__((aligned(16))) bf16_t As[T_BM * T_LDS];
  __shared__ __attribute__((aligned(16))) bf16_t Ws[T_BN * T_LDS];
  const int tid = threadIdx.x;
  const int lane = tid % WAVE, wave = tid / WAVE;
  const int wm = wave / 2, wn = wave % 2;
  const int m0 = blockIdx.y * T_BM, n0 = blockIdx.x * T_BN;

  // global -> register staging: thread loads 16 bytes of rows lr and lr+64 of each tile
  const int lr = tid / 4, lc = (tid % 4) * 8;
  f32x16_t acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  const u32x4_t zero = {0u, 0u, 0u, 0u};
  u32x4_t ra[2], rw[2];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int r = lr + h * 64;
      const int gk = k0 + lc;
      const int gm = m0 + r, gn = n0 + r;
      ra[h] = (gm < M && gk < K) ? load16(A + (size_t)gm * lda + gk) : zero;
      rw[h] = (gn < N && gk < K) ? load16(W + (size_t)gn * K + gk) : zero;
    }
  };
  fetch(0);
  for (int k0 = 0; k0 < K; k0 += T_BK) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int r = lr + h * 64;
      *reinterpret_cast<u32x4_t*>(&As[r * T_LDS + lc]) = ra[h];
      *reinterpret_cast<u32x4_t*>(&Ws[r * T_LDS + lc]) = rw[h];
    }
    __syncthreads();
    if (k0 + T_BK < K) fetch(k0 + T_BK);
#pragma unroll
    for (int ks = 0; ks < T_BK; ks += 16) {
      bf16x8_t a[2], b[2];
      const int kc = ks + (lane / 32) * 8;
#pragma unroll
      for (int i = 0; i < 2; ++i)
        a[i] = as_bf16x8(*reinterpret_cast<const u32x4_t*>(
            &As[(wm * 64 + i * 32 + lane % 32) * T_LDS + kc]));
#pragma unroll
      for (int j = 0; j < 2; ++j)
        b[j] = as_bf16x8(*reinterpret_cast<const u32x4_t*>(
            &Ws[(wn * 64 + j * 32 + lane % 32) * T_LDS + kc]));
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
    }
    __syncthreads();
  }
  // D[m][n] of a 32x32 tile: lane holds column lane%32, rows 8*(v/4) + 4*(lane/32) + v%4
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int gn = n0 + wn * 64 + j * 32 + lane % 32;
      if (gn >= N) continue;
      const float bv = bias ? bias[gn] : 0.f;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int gm = m0 + wm * 64 + i * 32 + 8 * (v / 4) + 4 * (lane / 32) + v % 4;
        if (gm < M) store_out(C + (size_t)gm * ldc + gn, acc[i][j][v] + bv);
      }
    }
}

// M <= 16*MT.  Block = 4 waves = 16 columns of the result; wave w takes the k-chunks
// c = w, w+4, ... of 32 elements.  A fragment: lane holds row lane%16, k-group lane/16;
// W fragment: lane holds column lane%16, k-group lane/16; result: lane holds column
// lane%16, rows 4*(lane/16) + v.
template <typename TO, int MT>
__global__ __launch_bounds__(256) void gemm_bf16_skinny_kernel(const bf16_t* __restrict__ A,
                                                               const bf16_t* __restrict__ W,
                                                               const float* __restrict__ bias,
                                                               TO* __restrict__ C, int M, int N,
                                                               int K, int lda, int ldc) {
  __shared__ float red[4][MT][WAVE][4];
  const int tid = threadIdx.x;
  const int lane = tid % WAVE, wave = tid / WAVE;
  const int n0 = blockIdx.x * 16;
  const int col = lane % 16, kg = (lane / 16) * 8;
  const int gn = n0 + col;
  const u32x4_t zero = {0u, 0u, 0u, 0u};
  f32x4_t acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
  const bf16_t* wrow = W + (size_t)(gn < N ? gn : 0) * K;
  for (int k0 = wave * 32; k0 < K; k0 += 128) {
    const int gk = k0 + kg;
    const bool kin = gk < K;
    const u32x4_t wv = (kin && gn < N) ? load16(wrow + gk) : zero;
    u32x4_t av[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      const int gm = t * 16 + col;
      av[t] = (kin && gm < M) ? load16(A + (size_t)gm * lda + gk) : zero;
    }
#pragma unroll
    for (int t = 0; t < MT; ++t)
      acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(av[t]), as_bf16x8(wv), acc[t], 0,
                                                       0, 0);
  }
#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int v = 0; v < 4; ++v) red[wave][t][lane][v] = acc[t][v];
  __syncthreads();
  if (wave == 0 && gn < N) {
    const float bv = bias ? bias[gn] : 0.f;
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int gm = t * 16 + 4 * (lane / 16) + v;
        if (gm < M) {
          const float s = ((red[0][t][lane][v] + red[1][t][lane][v]) + red[2][t][lane][v]) +
                          red[3][t][lane][v];
          store_out(C + (size_t)gm * ldc + gn, s + bv);
        }
      }
  }
}

template <typename TO>
static int launch_bf16(const bf16_t* A, const bf16_t* W, const float* bias, TO* C, int M, int N,
                       int K, int lda, int ldc, hipStream_t stream) {
  if (M <= 64) {
    dim3 grid((N + 15) / 16), block(256);
    const int mt = (M + 15) / 16;
    switch (mt) {
      case 1:
        hipLaunchKernelGGL((gemm_bf16_skinny_kernel<TO, 1>), grid, block, 0, stream, A, W, bias, C,
                           M, N, K, lda, ldc);
        break;
      case 2:
        hipLaunchKernelGGL((gemm_bf16_skinny_kernel<TO, 2>), grid, block, 0, stream, A, W, bias, C,
                           M, N, K, lda, ldc);
        break;
      case 3:
        hipLaunchKernelGGL((gemm_bf16_skinny_kernel<TO, 3>), grid, block, 0, stream, A, W, bias, C,
                           M, N, K, lda, ldc);
        break;
      default:
        hipLaunchKernelGGL((gemm_bf16_skinny_kernel<TO, 4>), grid, block, 0, stream, A, W, bias, C,
                           M, N, K, lda, ldc);
        break;
    }
  } else {
    dim3 grid((N + T_BN - 1) / T_BN, (M + T_BM - 1) / T_BM);
    hipLaunchKernelGGL(gemm_bf16_tile_kernel<TO>, grid, dim3(256), 0, stream, A, W, bias, C, M, N,
                       K, lda, ldc);
  }
  KAPPAI_RETURN_LAUNCH_STATUS();
}

// K, lda must be multiples of 8 and A, W 16-byte aligned (checked by the caller).
// force_kernel: 0 = by M, 1 = tile kernel, 2 = skinny kernel (M <= 64 only); for tests.
extern "C" int kappai_gemm_bf16(const void* A, const void* W, const float* bias, void* C, int M,
                                int N, int K, int lda, int ldc, int out_is_f32, int force_kernel,
                                hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if ((K % 8) || (lda % 8)) return (int)hipErrorInvalidValue;
  if (force_kernel == 2 && M > 64) return (int)hipErrorInvalidValue;
  if (force_kernel == 1) {
    dim3 grid((N + T_BN - 1) / T_BN, (M + T_BM - 1) / T_BM);
    if (out_is_f32)
      hipLaunchKernelGGL(gemm_bf16_tile_kernel<float>, grid, dim3(256), 0, stream,
                         (const bf16_t*)A, (const bf16_t*)W, bias, (float*)C, M, N, K, lda, ldc);
    else
      hipLaunchKernelGGL(gemm_bf16_tile_kernel<bf16_t>, grid, dim3(256), 0, stream,
                         (const bf16_t*)A, (const bf16_t*)W, bias, (bf16_t*)C, M, N, K, lda, ldc);
    KAPPAI_RETURN_LAUNCH_STATUS();
  }
  if (out_is_f32)
    return launch_bf16<float>((const bf16_t*)A, (const bf16_t*)W, bias, (float*)C, M, N, K, lda,
                              ldc, stream);
  return launch_bf16<bf16_t>((const bf16_t*)A, (const bf16_t*)W, bias, (bf16_t*)C, M, N, K, lda,
                             ldc, stream);
}

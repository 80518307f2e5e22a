// Shared device helpers for the gfx950 kernels: raw bfloat16 storage, wave (64 lanes)
// and block reductions, and the error convention of the host launchers.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef uint16_t bf16_t;  // storage of a bfloat16; arithmetic is always done in float

#define WAVE 64

// every launcher returns 0 or the hipError_t of its launch
#define KAPPAI_RETURN_LAUNCH_STATUS() return (int)hipGetLastError()

__device__ __forceinline__ float bf16_to_f32(bf16_t v) {
  return __uint_as_float(((uint32_t)v) << 16);
}

// round to nearest, ties to even; NaN stays NaN (gfx950 converts in hardware: v_cvt_pk_bf16_f32)
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
  return __builtin_bit_cast(bf16_t, (__bf16)f);
}

// two floats to two bfloat16 in one 32-bit word, `lo` in the low half
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
  const bf16x2_t v = {(__bf16)lo, (__bf16)hi};
  return __builtin_bit_cast(uint32_t, v);
}

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16_t v) { return bf16_to_f32(v); }
__device__ __forceinline__ void from_f32(float* p, float v) { *p = v; }
__device__ __forceinline__ void from_f32(bf16_t* p, float v) { *p = f32_to_bf16(v); }

// eight consecutive values as floats (16- or 32-byte loads and stores)
__device__ __forceinline__ void load8(const float* p, float* v) {
  const float4 a = *reinterpret_cast<const float4*>(p);
  const float4 b = *reinterpret_cast<const float4*>(p + 4);
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
__device__ __forceinline__ void load8(const bf16_t* p, float* v) {
  const uint4 a = *reinterpret_cast<const uint4*>(p);
  const uint32_t w[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    v[2 * i] = __uint_as_float(w[i] << 16);
    v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
  }
}
__device__ __forceinline__ void store8(float* p, const float* v) {
  *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  *reinterpret_cast<float4*>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
}
__device__ __forceinline__ void store8(bf16_t* p, const float* v) {
  uint4 o;
  o.x = (uint32_t)f32_to_bf16(v[0]) | ((uint32_t)f32_to_bf16(v[1]) << 16);
  o.y = (uint32_t)f32_to_bf16(v[2]) | ((uint32_t)f32_to_bf16(v[3]) << 16);
  o.z = (uint32_t)f32_to_bf16(v[4]) | ((uint32_t)f32_to_bf16(v[5]) << 16);
  o.w = (uint32_t)f32_to_bf16(v[6]) | ((uint32_t)f32_to_bf16(v[7]) << 16);
  *reinterpret_cast<uint4*>(p) = o;
}

// Exchanges inside a wave without a trip through LDS: the partner lane ^ 1 or ^ 2 (inside a quad)
// and the lanes 4 and 8 further in a row of 16 come by data-parallel moves, the partners lane ^ 16
// and lane ^ 32 by the row and half swaps of gfx950.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  return __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(v), CTRL, 0xf, 0xf, false));
}
__device__ __forceinline__ float lane_xor16(float x) {
  const uint32_t u = __float_as_uint(x);
  const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  // r[0] = the even rows' values in both rows of a pair, r[1] = the odd rows'
  return __uint_as_float((threadIdx.x & 16) ? r[0] : r[1]);
}
__device__ __forceinline__ float lane_xor32(float x) {
  const uint32_t u = __float_as_uint(x);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __uint_as_float((threadIdx.x & 32) ? r[0] : r[1]);
}

// Sum and maximum over the 64 lanes, the same value in every lane, in a fixed order: quads, the
// row of 16 (two rotations), the pair of rows, the two halves.
__device__ __forceinline__ float wave_sum(float v) {
  v += dpp_move<0xB1>(v);     // quad_perm [1, 0, 3, 2]
  v += dpp_move<0x4E>(v);     // quad_perm [2, 3, 0, 1]
  v += dpp_move<0x124>(v);    // row_ror 4
  v += dpp_move<0x128>(v);    // row_ror 8
  v += lane_xor16(v);
  v += lane_xor32(v);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, dpp_move<0xB1>(v));
  v = fmaxf(v, dpp_move<0x4E>(v));
  v = fmaxf(v, dpp_move<0x124>(v));
  v = fmaxf(v, dpp_move<0x128>(v));
  v = fmaxf(v, lane_xor16(v));
  v = fmaxf(v, lane_xor32(v));
  return v;
}

// The same for integers (the moves carry bits, whatever they mean).
__device__ __forceinline__ int wave_sum(int v) {
  const auto mv = [](auto f, int x) { return __float_as_int(f(__int_as_float(x))); };
  v += mv(dpp_move<0xB1>, v);
  v += mv(dpp_move<0x4E>, v);
  v += mv(dpp_move<0x124>, v);
  v += mv(dpp_move<0x128>, v);
  v += mv(lane_xor16, v);
  v += mv(lane_xor32, v);
  return v;
}

__device__ __forceinline__ int wave_max(int v) {
  const auto mv = [](auto f, int x) { return __float_as_int(f(__int_as_float(x))); };
  v = max(v, mv(dpp_move<0xB1>, v));
  v = max(v, mv(dpp_move<0x4E>, v));
  v = max(v, mv(dpp_move<0x124>, v));
  v = max(v, mv(dpp_move<0x128>, v));
  v = max(v, mv(lane_xor16, v));
  v = max(v, mv(lane_xor32, v));
  return v;
}

// Sum over a block of up to 1024 threads; `red` is LDS for 16 floats.  All threads get
// the result.  Ends with a barrier so that `red` may be used again at once.
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int nw = (blockDim.x + WAVE - 1) / WAVE;
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float t = 0.f;
  for (int i = 0; i < nw; ++i) t += red[i];
  __syncthreads();
  return t;
}

__device__ __forceinline__ float block_max(float v, float* red) {
  v = wave_max(v);
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int nw = (blockDim.x + WAVE - 1) / WAVE;
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float t = red[0];
  for (int i = 1; i < nw; ++i) t = fmaxf(t, red[i]);
  __syncthreads();
  return t;
}

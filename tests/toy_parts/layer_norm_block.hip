// A toy norm and a toy arrangement of parts, for the tests: LayerNorm (mean taken off, weight and
// bias) and a block whose mixer and feed-forward both read the same normalised rows,
//   h = norm(x);  x += mixer(h);  x += feed_forward(h).
// This file holds what they bring along to run their steps from C: two kernels, the launchers
// that the host's parts call too, and runners for the walk of csrc/engine.hip (a norm's and a
// block's), which the host registers under names.  Nothing in the framework's own files knows of
// them.
#include "common.h"
#include "engine.h"

struct toy_layer_norm {           // what the norm's runner reads (mirrored by the test's ctypes)
  const float* w;                 // [width]
  const float* b;                 // [width]
  float eps;
};

struct toy_parallel_block {       // what the block's runner reads
  kappai_norm_part norm;
  kappai_part mixer;
  kappai_part feed_forward;
};

__device__ __forceinline__ float toy_wave_sum(float v) {
  for (int o = WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
  return v;
}

// One wave per output row i (row r = rows ? rows[i] : i of the stream): x = resid[r] + delta[r],
// written back unless `rows` is given; out[i] = (x - mean) / sqrt(var + eps) * w + b.
template <typename TD, typename TO>
__global__ __launch_bounds__(WAVE) void toy_layer_norm_kernel(
    float* __restrict__ resid, const TD* __restrict__ delta, const float* __restrict__ w,
    const float* __restrict__ b, TO* __restrict__ out, const int* __restrict__ rows, int D,
    float eps) {
  const int i = blockIdx.x, lane = threadIdx.x;
  const int r = rows ? rows[i] : i;
  float* x = resid + (size_t)r * D;
  float sum = 0.f;
  for (int c = lane; c < D; c += WAVE) {
    float v = x[c];
    if (delta != nullptr) {
      if constexpr (sizeof(TD) == 2) v += bf16_to_f32(delta[(size_t)r * D + c]);
      else v += delta[(size_t)r * D + c];
      if (rows == nullptr) x[c] = v;
    }
    sum += v;
  }
  const float mean = toy_wave_sum(sum) / (float)D;
  auto value = [&](int c) {
    float v = x[c];
    if (delta != nullptr && rows != nullptr) {       // (the stream was left alone)
      if constexpr (sizeof(TD) == 2) v += bf16_to_f32(delta[(size_t)r * D + c]);
      else v += delta[(size_t)r * D + c];
    }
    return v;
  };
  float sq = 0.f;
  for (int c = lane; c < D; c += WAVE) {
    const float d = value(c) - mean;
    sq += d * d;
  }
  const float inv = 1.0f / sqrtf(toy_wave_sum(sq) / (float)D + eps);
  for (int c = lane; c < D; c += WAVE) {
    const float y = (value(c) - mean) * inv * w[c] + b[c];
    if constexpr (sizeof(TO) == 2) out[(size_t)i * D + c] = f32_to_bf16(y);
    else out[(size_t)i * D + c] = y;
  }
}

// delta: null, bfloat16 (delta_kind 1) or float32 (delta_kind 2) rows [M, D]
extern "C" int toy_layer_norm_launch(float* resid, const void* delta, int delta_kind,
                                     const float* w, const float* b, void* out, int out_bf16,
                                     const int* rows, int n, int D, float eps,
                                     hipStream_t stream) {
  if (n < 1 || D < 1 || (delta != nullptr && delta_kind != 1 && delta_kind != 2))
    return (int)hipErrorInvalidValue;
  const dim3 grid(n), block(WAVE);
#define TOY_LN(TD, TO)                                                                          \
  hipLaunchKernelGGL((toy_layer_norm_kernel<TD, TO>), grid, block, 0, stream, resid,            \
                     (const TD*)delta, w, b, (TO*)out, rows, D, eps)
  if (delta != nullptr && delta_kind == 1) {
    if (out_bf16) TOY_LN(bf16_t, bf16_t); else TOY_LN(bf16_t, float);
  } else {
    if (out_bf16) TOY_LN(float, bf16_t); else TOY_LN(float, float);
  }
#undef TOY_LN
  return (int)hipGetLastError();
}

template <typename TD>
__global__ void toy_add_kernel(float* __restrict__ resid, const TD* __restrict__ delta, long n) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  if constexpr (sizeof(TD) == 2) resid[i] += bf16_to_f32(delta[i]);
  else resid[i] += delta[i];
}

extern "C" int toy_add_launch(float* resid, const void* delta, int delta_is_f32, long n,
                              hipStream_t stream) {
  if (n < 1) return (int)hipErrorInvalidValue;
  const dim3 grid((unsigned)((n + 255) / 256)), block(256);
  if (delta_is_f32)
    hipLaunchKernelGGL(toy_add_kernel<float>, grid, block, 0, stream, resid, (const float*)delta, n);
  else
    hipLaunchKernelGGL(toy_add_kernel<bf16_t>, grid, block, 0, stream, resid,
                       (const bf16_t*)delta, n);
  return (int)hipGetLastError();
}

// The norm as the C walk runs it.  It knows nothing of the framework's shortcuts: what arrives
// (the embedding still to be looked up, partial sums, scaled rows) is brought to a plain update
// first, and its rows go out plain whoever takes them.
extern "C" kappai_rows toy_layer_norm_run(kappai_step* s, const void* desc, float* resid,
                                          kappai_carry carry, int M, const int* rows, int n_rows,
                                          const kappai_part* consumer) {
  (void)consumer;
  const kappai_step_api& api = *s->api;
  const toy_layer_norm& d = *static_cast<const toy_layer_norm*>(desc);
  const int bf16 = api.model(s)->compute_bf16, D = api.model(s)->width;
  carry = api.plain_carry(s, carry, resid, M);
  const int n = rows ? n_rows : M;
  kappai_rows out = {};
  out.is_bf16 = bf16;
  out.M = n;
  out.D = D;
  out.ld = D;
  out.data = api.take(s, KAPPAI_REGION_BLOCK, (size_t)n * D * (bf16 ? 2 : 4));
  const void* delta = carry.kind == KAPPAI_CARRY_DELTA ? carry.data : nullptr;
  if (!api.dry(s) && api.ok(s))
    api.launched(s, toy_layer_norm_launch(resid, delta, carry.is_f32 ? 2 : 1, d.w, d.b, out.data,
                                          bf16, rows, n, D, d.eps, api.stream(s)));
  return out;
}

// The block as the C walk runs it: the host's forward() in C.
extern "C" kappai_carry toy_parallel_block_run(kappai_step* s, const void* desc, float* resid,
                                               kappai_carry carry,
                                               const kappai_norm_part* after_norm,
                                               const kappai_part* after_consumer) {
  (void)after_norm;
  (void)after_consumer;                 // (it folds nothing into what comes after it)
  const kappai_step_api& api = *s->api;
  const toy_parallel_block& d = *static_cast<const toy_parallel_block*>(desc);
  const int M = api.batch(s)->n_rows, D = api.model(s)->width;
  kappai_rows h = d.norm.run(s, d.norm.desc, resid, carry, M, nullptr, 0, &d.mixer);
  h = api.plain_rows(s, h, resid);      // (a norm of the framework's may have deferred them)
  kappai_carry mixed = d.mixer.run(s, d.mixer.desc, h, resid, nullptr);
  mixed = api.plain_carry(s, mixed, resid, M);
  if (mixed.kind == KAPPAI_CARRY_DELTA && !api.dry(s) && api.ok(s))
    api.launched(s, toy_add_launch(resid, mixed.data, mixed.is_f32, (long)M * D, api.stream(s)));
  return d.feed_forward.run(s, d.feed_forward.desc, h, resid, nullptr);
}

extern "C" int toy_layer_norm_desc_bytes(void) { return (int)sizeof(toy_layer_norm); }
extern "C" int toy_parallel_block_desc_bytes(void) { return (int)sizeof(toy_parallel_block); }

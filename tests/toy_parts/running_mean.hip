// A toy token mixer with a state of its own, for the tests: out_t = mean(x_0 .. x_t) per channel,
// then a projection.  Its state is the running sum [width] of a request (the count is the
// position).  This file holds what a part from outside the framework brings along to run its
// steps from C: a kernel, the launcher that the host's part calls too, and a runner for the walk
// of csrc/engine.hip, which the host registers under a name.  Nothing in the framework's own
// files knows of it.
#include "common.h"
#include "engine.h"

struct toy_running_mean {         // what the runner reads (mirrored by the test's ctypes struct)
  kappai_linear proj;
  float* state;                   // [slots, width]
};

template <typename T>
__global__ void running_mean_kernel(const T* __restrict__ x, int ld, T* __restrict__ out,
                                    float* __restrict__ state, const int* __restrict__ seg_start,
                                    const int* __restrict__ seg_pos0,
                                    const int* __restrict__ seg_slot, int D) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  const int s = blockIdx.y;
  if (c >= D) return;
  float* st = state + (size_t)seg_slot[s] * D;
  const int pos0 = seg_pos0[s];
  float sum = pos0 == 0 ? 0.f : st[c];          // a fresh request has no history
  float count = (float)pos0;
  for (int t = seg_start[s]; t < seg_start[s + 1]; ++t) {
    float v;
    if constexpr (sizeof(T) == 2) v = bf16_to_f32(x[(size_t)t * ld + c]);
    else v = x[(size_t)t * ld + c];
    sum += v;
    count += 1.f;
    const float mean = sum / count;
    if constexpr (sizeof(T) == 2) out[(size_t)t * D + c] = f32_to_bf16(mean);
    else out[(size_t)t * D + c] = mean;
  }
  st[c] = sum;
}

extern "C" int toy_running_mean_launch(const void* x, int ld, void* out, float* state,
                                       const int* seg_start, const int* seg_pos0,
                                       const int* seg_slot, int n_segments, int D, int is_bf16,
                                       hipStream_t stream) {
  if (n_segments < 1 || D < 1 || n_segments > 65535) return (int)hipErrorInvalidValue;
  const dim3 grid((D + 127) / 128, n_segments), block(128);
  if (is_bf16)
    hipLaunchKernelGGL(running_mean_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)x, ld,
                       (bf16_t*)out, state, seg_start, seg_pos0, seg_slot, D);
  else
    hipLaunchKernelGGL(running_mean_kernel<float>, grid, block, 0, stream, (const float*)x, ld,
                       (float*)out, state, seg_start, seg_pos0, seg_slot, D);
  return (int)hipGetLastError();
}

// The mixer as the C walk runs it: the host's forward() in C.
extern "C" kappai_carry toy_running_mean_run(kappai_step* s, const void* desc, kappai_rows x,
                                             float* resid, const kappai_into* into) {
  const kappai_step_api& api = *s->api;
  const toy_running_mean& d = *static_cast<const toy_running_mean*>(desc);
  const kappai_batch& b = *api.batch(s);
  const int bf16 = api.model(s)->compute_bf16;
  const int region = api.carry_region(s);
  x = api.plain_rows(s, x, resid);              // (it announced no flags: rows come plain anyway)
  void* mean = api.take(s, KAPPAI_REGION_BLOCK, (size_t)x.M * x.D * (bf16 ? 2 : 4));
  if (!api.dry(s) && api.ok(s))
    api.launched(s, toy_running_mean_launch(x.data, x.ld, mean, d.state, b.seg_start, b.seg_pos0,
                                            b.seg_slot, b.n_segments, x.D, bf16, api.stream(s)));
  kappai_rows m = {};
  m.data = mean;
  m.is_bf16 = bf16;
  m.M = x.M;
  m.D = x.D;
  m.ld = x.D;
  return api.linear(s, m, &d.proj, bf16, 0, into, region);
}

extern "C" int toy_running_mean_desc_bytes(void) { return (int)sizeof(toy_running_mean); }

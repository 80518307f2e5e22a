// Gated short convolution over a batch of segments (kappai: src/backend/cpu/common.c:2393-2431,
// second statement in src/backend/vulkan/shaders/shortconv.comp:29-52).
//
// proj[t] = (B | C | x), each D wide.  bx = B*x;  s_t[c] = bias[c] + sum_k w[c,k] bx_{t-(L-1)+k}[c];
// out = C * s.  Values before a segment's first row come from the request's state
// state[slot][c][0..L-2] (oldest first), or are zero when the segment starts at position 0
// (src/recipe/ops_hybrid.c:353-354).  A second kernel then moves the last L-1 values of bx
// into the state; segments shorter than L-1 shift the old state through.
#include "common.h"

template <typename T>
__global__ void shortconv_out_kernel(const T* __restrict__ proj, const float* __restrict__ w,
                                     const float* __restrict__ bias,
                                     const float* __restrict__ state, T* __restrict__ out,
                                     const int* __restrict__ row_seg,
                                     const int* __restrict__ seg_start,
                                     const int* __restrict__ seg_pos0,
                                     const int* __restrict__ seg_slot, int D, int L) {
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  const int t = blockIdx.x;
  if (c >= D) return;
  const int seg = row_seg[t];
  const int r = t - seg_start[seg];          // row index inside the segment
  const bool fresh = seg_pos0[seg] == 0;
  const int H = L - 1;
  const float* st = state + ((size_t)seg_slot[seg] * D + c) * H;
  const float* wc = w + (size_t)c * L;
  float sum = bias ? bias[c] : 0.f;
  for (int k = 0; k < L; ++k) {
    const int src = r - H + k;               // segment-relative row of the tap's input
    float bx;
    if (src >= 0) {
      const T* p = proj + (size_t)(t - r + src) * 3 * D;
      bx = to_f32(p[c]) * to_f32(p[2 * D + c]);
    } else {
      bx = fresh ? 0.f : st[H + src];
    }
    sum += wc[k] * bx;
  }
  const float cg = to_f32(proj[(size_t)t * 3 * D + D + c]);
  from_f32(out + (size_t)t * D + c, cg * sum);
}

template <typename T>
__global__ void shortconv_state_kernel(const T* __restrict__ proj, float* __restrict__ state,
                                       const int* __restrict__ seg_start,
                                       const int* __restrict__ seg_pos0,
                                       const int* __restrict__ seg_slot, int D, int L) {
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  const int seg = blockIdx.x;
  if (c >= D) return;
  const int t0 = seg_start[seg];
  const int n = seg_start[seg + 1] - t0;
  const bool fresh = seg_pos0[seg] == 0;
  const int H = L - 1;
  float* st = state + ((size_t)seg_slot[seg] * D + c) * H;
  // new[j] = bx at segment row n-H+j, or old[n+j] when that row lies before the segment.
  // n >= 1, so old[n+j] is read before any new[j'] with j' >= n+j is written.
  for (int j = 0; j < H; ++j) {
    const int src = n - H + j;
    float v;
    if (src >= 0) {
      const T* p = proj + (size_t)(t0 + src) * 3 * D;
      v = to_f32(p[c]) * to_f32(p[2 * D + c]);
    } else {
      v = fresh ? 0.f : st[n + j];
    }
    st[j] = v;
  }
}

// Every segment is a single row (decode): one thread per (segment, channel) computes the output
// and shifts the state, which nobody else reads.
template <typename T>
__global__ void shortconv_step_kernel(const T* __restrict__ proj, const float* __restrict__ w,
                                      const float* __restrict__ bias, float* __restrict__ state,
                                      T* __restrict__ out, const int* __restrict__ seg_pos0,
                                      const int* __restrict__ seg_slot, int D, int L) {
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  const int t = blockIdx.x;
  if (c >= D) return;
  const bool fresh = seg_pos0[t] == 0;
  const int H = L - 1;
  float* st = state + ((size_t)seg_slot[t] * D + c) * H;
  const float* wc = w + (size_t)c * L;
  const T* p = proj + (size_t)t * 3 * D;
  const float bx = to_f32(p[c]) * to_f32(p[2 * D + c]);
  float sum = (bias ? bias[c] : 0.f);
  float prev = fresh ? 0.f : st[0];
  for (int k = 0; k < H; ++k) {
    sum += wc[k] * prev;                       // tap k meets history entry k
    const float next = (k + 1 < H) ? (fresh ? 0.f : st[k + 1]) : bx;
    st[k] = next;                              // shift: entry k becomes entry k+1, the last bx
    prev = next;
  }
  sum += wc[H] * bx;
  from_f32(out + (size_t)t * D + c, to_f32(p[D + c]) * sum);
}

extern "C" int kappai_shortconv(const void* proj, const float* w, const float* bias, float* state,
                                void* out, const int* row_seg, const int* seg_start,
                                const int* seg_pos0, const int* seg_slot, int T, int S, int D,
                                int L, int is_bf16, hipStream_t stream) {
  if (T <= 0 || S <= 0) return 0;
  if (L < 2) return (int)hipErrorInvalidValue;
  const int threads = D >= 256 ? 256 : 64;
  dim3 g1(T, (D + threads - 1) / threads), g2(S, (D + threads - 1) / threads);
  if (T == S) {   // one row a segment: row t is segment t
    if (is_bf16)
      hipLaunchKernelGGL(shortconv_step_kernel<bf16_t>, g1, dim3(threads), 0, stream,
                         (const bf16_t*)proj, w, bias, state, (bf16_t*)out, seg_pos0, seg_slot, D,
                         L);
    else
      hipLaunchKernelGGL(shortconv_step_kernel<float>, g1, dim3(threads), 0, stream,
                         (const float*)proj, w, bias, state, (float*)out, seg_pos0, seg_slot, D, L);
    KAPPAI_RETURN_LAUNCH_STATUS();
  }
  if (is_bf16) {
    hipLaunchKernelGGL(shortconv_out_kernel<bf16_t>, g1, dim3(threads), 0, stream,
                       (const bf16_t*)proj, w, bias, (const float*)state, (bf16_t*)out, row_seg,
                       seg_start, seg_pos0, seg_slot, D, L);
    hipLaunchKernelGGL(shortconv_state_kernel<bf16_t>, g2, dim3(threads), 0, stream,
                       (const bf16_t*)proj, state, seg_start, seg_pos0, seg_slot, D, L);
  } else {
    hipLaunchKernelGGL(shortconv_out_kernel<float>, g1, dim3(threads), 0, stream,
                       (const float*)proj, w, bias, (const float*)state, (float*)out, row_seg,
                       seg_start, seg_pos0, seg_slot, D, L);
    hipLaunchKernelGGL(shortconv_state_kernel<float>, g2, dim3(threads), 0, stream,
                       (const float*)proj, state, seg_start, seg_pos0, seg_slot, D, L);
  }
  KAPPAI_RETURN_LAUNCH_STATUS();
}

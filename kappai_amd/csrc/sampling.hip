// Token choice on the device (kappai: src/sampler.c).
//   temperature <= 0 : argmax, ties to the lowest id (src/sampler.c:125-136)
//   else             : softmax(logit / T) over the whole vocabulary and an inverse-CDF draw with
//                      the row's uniform u in [0,1) (src/sampler.c:234-258); sums in double.
// One block per row.  Also the repeat penalty of src/sampler.c:205-216 as a scatter.
#include "common.h"

#define SAMPLE_THREADS 1024

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_rows_kernel(
    const float* __restrict__ logits, const float* __restrict__ temperature,
    const float* __restrict__ uniform, int* __restrict__ out, int V) {
  __shared__ float redf[SAMPLE_THREADS / WAVE];
  __shared__ int redi[SAMPLE_THREADS / WAVE];
  __shared__ double part[SAMPLE_THREADS];
  __shared__ int found;
  const int r = blockIdx.x, tid = threadIdx.x;
  const int lane = tid % WAVE, wave = tid / WAVE, nw = SAMPLE_THREADS / WAVE;
  const float* lg = logits + (size_t)r * V;
  const float temp = temperature[r];

  // ---- max and its lowest index -------------------------------------------------------
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  for (int i = tid; i < V; i += SAMPLE_THREADS) {
    const float v = lg[i];
    if (v > bv || (v == bv && i < bi)) { bv = v; bi = i; }
  }
#pragma unroll
  for (int m = WAVE / 2; m > 0; m >>= 1) {
    const float ov = __shfl_xor(bv, m, WAVE);
    const int oi = __shfl_xor(bi, m, WAVE);
    if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
  }
  if (lane == 0) { redf[wave] = bv; redi[wave] = bi; }
  __syncthreads();
  bv = redf[0];
  bi = redi[0];
  for (int w = 1; w < nw; ++w)
    if (redf[w] > bv || (redf[w] == bv && redi[w] < bi)) { bv = redf[w]; bi = redi[w]; }
  if (!(temp > 0.f)) {
    if (tid == 0) out[r] = bi == 0x7fffffff ? 0 : bi;
    return;
  }

  // ---- e_i = exp(l_i/T - max/T); every thread owns one contiguous range ------------------
  const float inv_t = 1.0f / temp;
  const float mx = bv * inv_t;
  const int chunk = (V + SAMPLE_THREADS - 1) / SAMPLE_THREADS;
  const int i0 = min(tid * chunk, V), i1 = min(i0 + chunk, V);
  double s = 0.0;
  for (int i = i0; i < i1; ++i) s += (double)expf(lg[i] * inv_t - mx);
  part[tid] = s;
  if (tid == 0) found = V - 1;
  __syncthreads();
  // inclusive scan over the threads' sums (Hillis-Steele)
  for (int off = 1; off < SAMPLE_THREADS; off <<= 1) {
    const double add = tid >= off ? part[tid - off] : 0.0;
    __syncthreads();
    part[tid] += add;
    __syncthreads();
  }
  const double total = part[SAMPLE_THREADS - 1];
  const double target = (double)uniform[r] * total;
  const double before = tid ? part[tid - 1] : 0.0;
  if (before <= target && target < part[tid]) {   // exactly one thread unless target >= total
    double acc = before;
    int pick = i1 - 1;
    for (int i = i0; i < i1; ++i) {
      acc += (double)expf(lg[i] * inv_t - mx);
      if (target < acc) { pick = i; break; }
    }
    found = pick;
  }
  __syncthreads();
  if (tid == 0) out[r] = found;
}

extern "C" int kappai_sample_rows(const float* logits, const float* temperature,
                                  const float* uniform, int* out, int n_rows, int V,
                                  hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (V < 1) return (int)hipErrorInvalidValue;
  hipLaunchKernelGGL(sample_rows_kernel, dim3(n_rows), dim3(SAMPLE_THREADS), 0, stream, logits,
                     temperature, uniform, out, V);
  KAPPAI_RETURN_LAUNCH_STATUS();
}

// logits[row[i], tok[i]] is divided by penalty[i] when positive, multiplied otherwise.  The
// caller lists every token of a row's window once per occurrence, as the reference applies
// the penalty once per occurrence; entries of one (row, token) must therefore be serialised:
// one thread walks the whole list of a row.
__global__ void repeat_penalty_kernel(float* __restrict__ logits, const int* __restrict__ row_start,
                                      const int* __restrict__ toks,
                                      const float* __restrict__ penalty, int V) {
  const int r = blockIdx.x;
  if (threadIdx.x != 0) return;
  const float pen = penalty[r];
  if (pen == 1.0f) return;
  float* lg = logits + (size_t)r * V;
  for (int i = row_start[r]; i < row_start[r + 1]; ++i) {
    const int tok = toks[i];
    if (tok < 0 || tok >= V) continue;
    lg[tok] = lg[tok] > 0.f ? lg[tok] / pen : lg[tok] * pen;
  }
}

extern "C" int kappai_repeat_penalty(float* logits, const int* row_start, const int* toks,
                                     const float* penalty, int n_rows, int V,
                                     hipStream_t stream) {
  if (n_rows <= 0) return 0;
  hipLaunchKernelGGL(repeat_penalty_kernel, dim3(n_rows), dim3(WAVE), 0, stream, logits, row_start,
                     toks, penalty, V);
  KAPPAI_RETURN_LAUNCH_STATUS();
}

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
  if (V % 4 == 0) {   // rows are 16-byte aligned: four values a load, all loads independent
    const float4* lg4 = reinterpret_cast<const float4*>(lg);
    for (int i = tid; i < V / 4; i += SAMPLE_THREADS) {
      const float4 q = lg4[i];
      const float vs[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (vs[e] > bv) { bv = vs[e]; bi = 4 * i + e; }   // indices only grow within a thread
    }
  } else {
    for (int i = tid; i < V; i += SAMPLE_THREADS) {
      const float v = lg[i];
      if (v > bv) { bv = v; bi = i; }
    }
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

// ---------------------------------------------------------------------------------------
// Draw with narrowed candidates (kappai: src/sampler.c:218-332): the `keep` largest logits
// (top-k, or the best 1024 when only top-p / min-p narrow), sorted by descending logit;
// softmax of logit/T in float; top-p keeps the token that crosses the mass; min-p is relative
// to the best; inverse-CDF draw at the row's uniform over what is left.  One block per row:
// radix select of the keep-th largest value, gather, bitonic sort in LDS, then one thread walks
// the (at most 1024) candidates in the reference's order of operations.
// ---------------------------------------------------------------------------------------
#define FILT_THREADS 1024
#define FILT_MAX_KEEP 1024

__device__ __forceinline__ uint32_t order_key(float f) {   // larger float -> larger key
  const uint32_t u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__global__ __launch_bounds__(FILT_THREADS) void sample_filtered_kernel(
    const float* __restrict__ logits, const int* __restrict__ rows, const int* __restrict__ keep_n,
    const float* __restrict__ temperature, const float* __restrict__ top_p,
    const float* __restrict__ min_p, const float* __restrict__ uniform, int* __restrict__ out,
    int V) {
  __shared__ uint32_t hist[256];
  __shared__ uint32_t sh_prefix, sh_remaining, sh_count;
  __shared__ uint32_t scan[FILT_THREADS];
  __shared__ float cval[FILT_MAX_KEEP];
  __shared__ int cidx[FILT_MAX_KEEP];
  const int i = blockIdx.x, tid = threadIdx.x;
  const float* lg = logits + (size_t)rows[i] * V;
  const int keep = min(min(keep_n[i], V), FILT_MAX_KEEP);

  // ---- the keep-th largest key, byte by byte from the top --------------------------------
  if (tid == 0) { sh_prefix = 0; sh_remaining = keep; }
  __syncthreads();
  for (int shift = 24; shift >= 0; shift -= 8) {
    if (tid < 256) hist[tid] = 0;
    __syncthreads();
    const uint32_t prefix = sh_prefix;
    const uint32_t mask = shift == 24 ? 0u : (0xffffffffu << (shift + 8));
    for (int e = tid; e < V; e += FILT_THREADS) {
      const uint32_t k = order_key(lg[e]);
      if ((k & mask) == prefix) atomicAdd(&hist[(k >> shift) & 0xff], 1u);
    }
    __syncthreads();
    if (tid == 0) {
      uint32_t rem = sh_remaining, above = 0;
      int b = 255;
      for (; b > 0; --b) {
        if (above + hist[b] >= rem) break;
        above += hist[b];
      }
      sh_prefix = prefix | ((uint32_t)b << shift);
      sh_remaining = rem - above;
    }
    __syncthreads();
  }
  const uint32_t thr = sh_prefix;            // key of the keep-th largest
  const uint32_t n_ties = sh_remaining;      // how many elements with exactly this key are kept
  // ---- gather: everything above the threshold, then the first ties in index order ---------
  if (tid == 0) sh_count = 0;
  __syncthreads();
  const int chunk = (V + FILT_THREADS - 1) / FILT_THREADS;
  const int e0 = min(tid * chunk, V), e1 = min(e0 + chunk, V);
  uint32_t my_ties = 0;
  for (int e = e0; e < e1; ++e) {
    const float v = lg[e];
    const uint32_t k = order_key(v);
    if (k > thr) {
      const uint32_t slot = atomicAdd(&sh_count, 1u);
      cval[slot] = v;
      cidx[slot] = e;
    } else if (k == thr) {
      ++my_ties;
    }
  }
  scan[tid] = my_ties;
  __syncthreads();
  for (int off = 1; off < FILT_THREADS; off <<= 1) {
    const uint32_t add = tid >= off ? scan[tid - off] : 0u;
    __syncthreads();
    scan[tid] += add;
    __syncthreads();
  }
  {
    const uint32_t n_above = sh_count;
    uint32_t rank = scan[tid] - my_ties;      // ties before this thread's range
    for (int e = e0; e < e1 && rank < n_ties; ++e) {
      const float v = lg[e];
      if (order_key(v) == thr) {
        cval[n_above + rank] = v;
        cidx[n_above + rank] = e;
        ++rank;
      }
    }
  }
  __syncthreads();
  // pad to a power of two for the sort
  int n2 = 1;
  while (n2 < keep) n2 <<= 1;
  for (int e = keep + tid; e < n2; e += FILT_THREADS) { cval[e] = -INFINITY; cidx[e] = 0x7fffffff; }
  __syncthreads();
  // ---- bitonic sort: descending value, ascending index on ties ----------------------------
  for (int k = 2; k <= n2; k <<= 1)
    for (int j = k >> 1; j > 0; j >>= 1) {
      const int a = tid, b = tid ^ j;
      if (a < n2 && b > a) {
        const bool desc = (a & k) == 0;
        const float va = cval[a], vb = cval[b];
        const int ia = cidx[a], ib = cidx[b];
        const bool a_first = va > vb || (va == vb && ia < ib);   // a belongs before b
        if (a_first != desc) { cval[a] = vb; cval[b] = va; cidx[a] = ib; cidx[b] = ia; }
      }
      __syncthreads();
    }
  // ---- one thread: temperature, top-p, min-p, draw (float, in the reference's order) -------
  if (tid == 0) {
    const float inv_t = 1.0f / temperature[i];
    const float mx = cval[0] * inv_t;
    float sum = 0.f;
    for (int e = 0; e < keep; ++e) {
      const float p = expf(cval[e] * inv_t - mx);
      cval[e] = p;
      sum += p;
    }
    int kept = keep;
    const float tp = top_p[i];
    if (tp < 1.0f) {
      float cum = 0.f;
      for (int e = 0; e < keep; ++e) {
        cum += cval[e] / sum;
        if (cum > tp) { kept = e + 1; break; }
      }
    }
    const float mp = min_p[i];
    if (mp > 0.f) {
      const float floor_p = mp * (cval[0] / sum);
      int n = 0;
      while (n < kept && (cval[n] / sum) >= floor_p) ++n;
      kept = n > 0 ? n : 1;
    }
    float psum = 0.f;
    for (int e = 0; e < kept; ++e) psum += cval[e];
    const float target = uniform[i] * psum;
    float acc = 0.f;
    int pick = kept - 1;
    for (int e = 0; e < kept; ++e) {
      acc += cval[e];
      if (target < acc) { pick = e; break; }
    }
    out[rows[i]] = cidx[pick];
  }
}

// rows[i] names the row of `logits` (and of `out`) that entry i samples for; keep_n[i] <= 1024.
extern "C" int kappai_sample_filtered(const float* logits, const int* rows, const int* keep_n,
                                      const float* temperature, const float* top_p,
                                      const float* min_p, const float* uniform, int* out,
                                      int n_entries, int V, hipStream_t stream) {
  if (n_entries <= 0) return 0;
  if (V < 1) return (int)hipErrorInvalidValue;
  hipLaunchKernelGGL(sample_filtered_kernel, dim3(n_entries), dim3(FILT_THREADS), 0, stream,
                     logits, rows, keep_n, temperature, top_p, min_p, uniform, out, V);
  KAPPAI_RETURN_LAUNCH_STATUS();
}

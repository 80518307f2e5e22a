// Token choice on the device (kappai: src/sampler.c).
//   temperature <= 0 : argmax, ties to the lowest id (src/sampler.c:125-136)
//   else             : softmax(logit / T) over the whole vocabulary and an inverse-CDF draw with
//                      the row's uniform u in [0,1) (src/sampler.c:234-258); sums in double.
// One block per row.  Also the repeat penalty of src/sampler.c:205-216 as a scatter.
#include "common.h"

#define SAMPLE_THREADS 1024

// The chosen token goes to `out` and, when given, to `out2` as well (the token table of the
// step that comes next, so that no copy runs between two decode steps queued back to back).
__device__ __forceinline__ void put(int* __restrict__ out, int* __restrict__ out2, int at, int token) {
  out[at] = token;
  if (out2 != nullptr) out2[at] = token;
}

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_rows_kernel(
    const float* __restrict__ logits, const float* __restrict__ temperature,
    const float* __restrict__ uniform, int* __restrict__ out, int* __restrict__ out2, int V) {
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
    if (tid == 0) put(out, out2, r, bi == 0x7fffffff ? 0 : bi);
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
  if (tid == 0) put(out, out2, r, found);
}

// The same for rows of at most SAMPLE_THREADS * 4 * SR_STEPS values, which a block keeps in
// registers: every wave owns a contiguous part of the row and reads it 256 values a step (16
// bytes a lane), so that the order of the values is (wave, step, lane, place in the lane).  The
// exponentials are summed in double per (wave, step), one wave finds the part that holds the
// drawn point of the distribution, and its owner finds the lane and the value.
#define SR_STEPS 16
#define SR_WAVES (SAMPLE_THREADS / WAVE)

__device__ __forceinline__ double wave_sum_f64(double v) {
#pragma unroll
  for (int m = WAVE / 2; m > 0; m >>= 1) v += __shfl_xor(v, m, WAVE);
  return v;
}

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_rows_held_kernel(
    const float* __restrict__ logits, const float* __restrict__ temperature,
    const float* __restrict__ uniform, int* __restrict__ out, int* __restrict__ out2, int V) {
  __shared__ float redf[SR_WAVES];
  __shared__ int redi[SR_WAVES];
  __shared__ double part[SR_WAVES * SR_STEPS];
  __shared__ double sh_before, sh_target;
  __shared__ int sh_part, found;
  const int r = blockIdx.x, tid = threadIdx.x;
  const int lane = tid % WAVE, wave = tid / WAVE;
  const float* lg = logits + (size_t)r * V;
  const float temp = temperature[r];
  const int region = (((V + SR_WAVES - 1) / SR_WAVES) + 255) / 256 * 256;
  const int w0 = min(wave * region, V), w1 = min(w0 + region, V);
  const bool vec = V % 4 == 0 && (reinterpret_cast<uintptr_t>(lg) % 16) == 0;
  float x[SR_STEPS][4];
#pragma unroll
  for (int st = 0; st < SR_STEPS; ++st) {
    const int idx = w0 + 256 * st + 4 * lane;
    if (vec) {
      float4 q = {-INFINITY, -INFINITY, -INFINITY, -INFINITY};
      if (idx < w1) q = *reinterpret_cast<const float4*>(lg + idx);
      x[st][0] = q.x; x[st][1] = q.y; x[st][2] = q.z; x[st][3] = q.w;
    } else {
#pragma unroll
      for (int c = 0; c < 4; ++c) x[st][c] = idx + c < w1 ? lg[idx + c] : -INFINITY;
    }
  }
  // ---- max and its lowest index (a lane's indices grow with step and place) ---------------
  float bv = -INFINITY;
  int bi = 0x7fffffff;
#pragma unroll
  for (int st = 0; st < SR_STEPS; ++st)
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int idx = w0 + 256 * st + 4 * lane + c;
      if (idx < w1 && x[st][c] > bv) { bv = x[st][c]; bi = idx; }
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
  for (int w = 1; w < SR_WAVES; ++w)
    if (redf[w] > bv || (redf[w] == bv && redi[w] < bi)) { bv = redf[w]; bi = redi[w]; }
  if (!(temp > 0.f)) {
    if (tid == 0) put(out, out2, r, bi == 0x7fffffff ? 0 : bi);
    return;
  }
  // ---- e = exp(l/T - max/T); sums per (wave, step) in double ---------------------------------
  const float inv_t = 1.0f / temp;
  const float mx = bv * inv_t;
  double lane_sum[SR_STEPS];
#pragma unroll
  for (int st = 0; st < SR_STEPS; ++st) {
    double sum = 0.0;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int idx = w0 + 256 * st + 4 * lane + c;
      x[st][c] = idx < w1 ? expf(x[st][c] * inv_t - mx) : 0.f;
      sum += (double)x[st][c];
    }
    lane_sum[st] = sum;
    const double all = wave_sum_f64(sum);
    if (lane == 0) part[wave * SR_STEPS + st] = all;
  }
  if (tid == 0) { found = V - 1; sh_part = -1; }
  __syncthreads();
  // ---- the part that holds the drawn point: one wave scans the 256 sums in order -----------
  if (wave == 0) {
    constexpr int PER = SR_WAVES * SR_STEPS / WAVE;       // 4 parts a lane
    double mine[PER], incl = 0.0;
#pragma unroll
    for (int j = 0; j < PER; ++j) { mine[j] = part[PER * lane + j]; incl += mine[j]; }
    // inclusive sums over the lanes
#pragma unroll
    for (int off = 1; off < WAVE; off <<= 1) {
      const double o = __shfl_up(incl, off, WAVE);
      if (lane >= off) incl += o;
    }
    const double total = __shfl(incl, WAVE - 1, WAVE);
    const double target = (double)uniform[r] * total;
    // sum of the parts before this lane's: the lane below's inclusive sum itself, so that the
    // intervals of neighbouring lanes meet exactly (0 for the first)
    double before = __shfl_up(incl, 1, WAVE);
    if (lane == 0) before = 0.0;
    // the lane's last part ends where the next lane begins (the last lane's at the total), so
    // that the parts cover [0, total) without a gap whatever the rounding of the sums
    double next = __shfl_down(before, 1, WAVE);
    if (lane == WAVE - 1) next = total;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const double end = j + 1 < PER ? before + mine[j] : next;
      if (before <= target && target < end) {               // one part, unless target >= total
        sh_part = PER * lane + j;
        sh_before = before;
        sh_target = target;
      }
      before = end;
    }
  }
  __syncthreads();
  const int p = sh_part;
  if (p < 0 || wave != p / SR_STEPS) {
    if (p < 0 && tid == 0) put(out, out2, r, found);                // the draw fell on the very end
    return;
  }
  // ---- the wave that owns the part finds the lane, the lane its value --------------------------
  const int st_p = p % SR_STEPS;
  double mine = 0.0;
  float e[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int st = 0; st < SR_STEPS; ++st)
    if (st == st_p) {
      mine = lane_sum[st];
#pragma unroll
      for (int c = 0; c < 4; ++c) e[c] = x[st][c];
    }
  double incl = mine;
#pragma unroll
  for (int off = 1; off < WAVE; off <<= 1) {
    const double o = __shfl_up(incl, off, WAVE);
    if (lane >= off) incl += o;
  }
  double below = __shfl_up(incl, 1, WAVE);
  if (lane == 0) below = 0.0;
  const double before = sh_before + below, target = sh_target;
  const bool here = before <= target && target < sh_before + incl;   // ends where the next begins
  // rounding may leave the point just past the last lane's sum: the last lane with values takes it
  const unsigned long long any = __ballot(here);
  if (any == 0ull) {
    if (lane == 0) put(out, out2, r, min(w0 + 256 * st_p + 255, w1 - 1));
    return;
  }
  if (here) {
    // the lane's sum was made in this order, so the last step reaches it exactly; values past
    // the end of the row are zero and cannot be the one at which the sum passes the point
    double acc = before;
    int pick = 3;
    for (int c = 0; c < 4; ++c) {
      acc += (double)e[c];
      if (target < acc) { pick = c; break; }
    }
    put(out, out2, r, min(w0 + 256 * st_p + 4 * lane + pick, w1 - 1));
  }
}

extern "C" int kappai_sample_rows(const float* logits, const float* temperature,
                                  const float* uniform, int* out, int* out2, int n_rows, int V,
                                  hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (V < 1) return (int)hipErrorInvalidValue;
  if (V <= SAMPLE_THREADS * 4 * SR_STEPS)
    hipLaunchKernelGGL(sample_rows_held_kernel, dim3(n_rows), dim3(SAMPLE_THREADS), 0, stream,
                       logits, temperature, uniform, out, out2, V);
  else
    hipLaunchKernelGGL(sample_rows_kernel, dim3(n_rows), dim3(SAMPLE_THREADS), 0, stream, logits,
                       temperature, uniform, out, out2, V);
  KAPPAI_RETURN_LAUNCH_STATUS();
}

// logits[row[i], tok[i]] is divided by penalty[i] when positive, multiplied otherwise.  The
// caller lists every token of a row's window once per occurrence, as the reference applies
// the penalty once per occurrence (src/sampler.c:205-216).  One wave per row: a lane takes the
// entries lane, lane + 64, ...; the lane that holds a token's first entry counts the token's
// entries and applies the penalty to that one logit as many times, one after the other in a
// register, which gives the bits of the reference's walk over the list (entries of different
// tokens do not touch each other, and a logit keeps its sign under the penalty, so the order
// among them does not matter).
__global__ __launch_bounds__(WAVE) void repeat_penalty_kernel(
    float* __restrict__ logits, const int* __restrict__ row_start, const int* __restrict__ toks,
    const float* __restrict__ penalty, int V) {
  const int r = blockIdx.x, lane = threadIdx.x;
  const float pen = penalty[r];
  if (pen == 1.0f) return;
  float* lg = logits + (size_t)r * V;
  const int lo = row_start[r], hi = row_start[r + 1];
  for (int i = lo + lane; i < hi; i += WAVE) {
    const int tok = toks[i];
    if (tok < 0 || tok >= V) continue;
    bool first = true;
    for (int j = lo; j < i && first; ++j) first = toks[j] != tok;
    if (!first) continue;
    int times = 1;
    for (int j = i + 1; j < hi; ++j) times += toks[j] == tok ? 1 : 0;
    float v = lg[tok];
    for (int t = 0; t < times; ++t) v = v > 0.f ? v / pen : v * pen;
    lg[tok] = v;
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
// The tokens a request has seen, kept on the GPU: history[slot] is a ring of `cap` token ids and
// seen[slot] counts what went into it.  With it the repeat penalty needs nothing from the host
// at the time of a step, so a step can be queued before the tokens of the one before it have
// been read.  (kappai keeps the same ring on the host: src/sampler.c recent / recent_head.)
// ---------------------------------------------------------------------------------------
// history[slots[i]] := toks[starts[i] .. starts[i + 1]) (at most cap tokens, the oldest first)
__global__ __launch_bounds__(WAVE) void history_set_kernel(
    int* __restrict__ history, int* __restrict__ seen, const int* __restrict__ slots,
    const int* __restrict__ starts, const int* __restrict__ toks, int cap) {
  const int i = blockIdx.x, lane = threadIdx.x;
  const int slot = slots[i], lo = starts[i], n = min(starts[i + 1] - lo, cap);
  for (int j = lane; j < n; j += WAVE) history[(size_t)slot * cap + j] = toks[lo + j];
  if (lane == 0) seen[slot] = n;
}

// entry i: the penalty of row rows[i] over the last last_n[i] tokens of history[slots[i]], as
// repeat_penalty_kernel applies it to a list
__global__ __launch_bounds__(WAVE) void repeat_penalty_history_kernel(
    float* __restrict__ logits, const int* __restrict__ rows, const int* __restrict__ slots,
    const float* __restrict__ penalty, const int* __restrict__ last_n,
    const int* __restrict__ history, const int* __restrict__ seen, int V, int cap) {
  const int i = blockIdx.x, lane = threadIdx.x;
  const float pen = penalty[i];
  if (pen == 1.0f) return;
  float* lg = logits + (size_t)rows[i] * V;
  const int slot = slots[i];
  const int* ring = history + (size_t)slot * cap;
  const int total = seen[slot];
  const int n = min(min(last_n[i], total), cap);
  const int first = total - n;                          // the window: tokens first .. total - 1
  auto at = [&](int j) { return ring[(first + j) % cap]; };
  for (int j = lane; j < n; j += WAVE) {
    const int tok = at(j);
    if (tok < 0 || tok >= V) continue;
    bool is_first = true;
    for (int e = 0; e < j && is_first; ++e) is_first = at(e) != tok;
    if (!is_first) continue;
    int times = 1;
    for (int e = j + 1; e < n; ++e) times += at(e) == tok ? 1 : 0;
    float v = lg[tok];
    for (int t = 0; t < times; ++t) v = v > 0.f ? v / pen : v * pen;
    lg[tok] = v;
  }
}

// entry i: the token chosen for row rows[i] joins history[slots[i]]
__global__ void history_append_kernel(const int* __restrict__ chosen, const int* __restrict__ rows,
                                      const int* __restrict__ slots, int* __restrict__ history,
                                      int* __restrict__ seen, int n, int cap) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int slot = slots[i];
  const int total = seen[slot];
  history[(size_t)slot * cap + total % cap] = chosen[rows[i]];
  seen[slot] = total + 1;         // (a request's tokens are far fewer than an int counts)
}

extern "C" int kappai_history_set(int* history, int* seen, const int* slots, const int* starts,
                                  const int* toks, int n, int cap, hipStream_t stream) {
  if (n <= 0) return 0;
  if (cap < 1) return (int)hipErrorInvalidValue;
  hipLaunchKernelGGL(history_set_kernel, dim3(n), dim3(WAVE), 0, stream, history, seen, slots,
                     starts, toks, cap);
  KAPPAI_RETURN_LAUNCH_STATUS();
}

extern "C" int kappai_repeat_penalty_history(float* logits, const int* rows, const int* slots,
                                             const float* penalty, const int* last_n,
                                             const int* history, const int* seen, int n, int V,
                                             int cap, hipStream_t stream) {
  if (n <= 0) return 0;
  if (cap < 1 || V < 1) return (int)hipErrorInvalidValue;
  hipLaunchKernelGGL(repeat_penalty_history_kernel, dim3(n), dim3(WAVE), 0, stream, logits, rows,
                     slots, penalty, last_n, history, seen, V, cap);
  KAPPAI_RETURN_LAUNCH_STATUS();
}

extern "C" int kappai_history_append(const int* chosen, const int* rows, const int* slots,
                                     int* history, int* seen, int n, int cap,
                                     hipStream_t stream) {
  if (n <= 0) return 0;
  if (cap < 1) return (int)hipErrorInvalidValue;
  hipLaunchKernelGGL(history_append_kernel, dim3((n + 63) / 64), dim3(64), 0, stream, chosen, rows,
                     slots, history, seen, n, cap);
  KAPPAI_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------------
// Draw with narrowed candidates (kappai: src/sampler.c:218-332): the `keep` largest logits
// (top-k, or the best 1024 when only top-p / min-p narrow), sorted by descending logit;
// softmax of logit/T in float; top-p keeps the token that crosses the mass; min-p is relative
// to the best; inverse-CDF draw at the row's uniform over what is left.  One block per row:
// radix select of the keep-th largest value, gather, bitonic sort in LDS, then the (at most
// 1024) candidates in the reference's order of operations: the exponentials and quotients are
// computed by all threads, the running sums by one.
//
// Every wave owns a contiguous part of the row and reads it 256 values a step (16 bytes a
// lane).  Logits share their high bits, so in the first radix pass all lanes add to a handful
// of counters: the digits are 11 bits wide (sign, exponent and two bits of the mantissa in the
// first) and every counter exists 4 times (lane % 4, in different LDS banks).
// ---------------------------------------------------------------------------------------
#define FILT_THREADS 1024
#define FILT_WAVES (FILT_THREADS / WAVE)
#define FILT_MAX_KEEP 1024
#define FILT_BINS 2048
#define FILT_SUBS 4

__device__ __forceinline__ uint32_t order_key(float f) {   // larger float -> larger key
  const uint32_t u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float key_value(uint32_t k) {   // the float a key came from
  return __uint_as_float((k & 0x80000000u) ? (k ^ 0x80000000u) : ~k);
}

// p(e) = exp(l_e/T - max/T) and q(e) = p(e) / sum of the candidates in descending order: top-p
// keeps the token that crosses the mass, min-p is relative to the best, then the inverse-CDF
// draw at u over what is left (src/sampler.c:271-332).  Returns the place of the chosen one.
template <typename P, typename Q>
__device__ __forceinline__ int narrow_and_draw(P&& p, Q&& q, int keep, float tp, float mp,
                                               float u) {
  int kept = keep;
  if (tp < 1.0f) {
    float cum = 0.f;
    for (int e = 0; e < keep; ++e) {
      cum += q(e);
      if (cum > tp) { kept = e + 1; break; }
    }
  }
  if (mp > 0.f) {
    const float floor_p = mp * q(0);
    int n = 0;
    while (n < kept && q(n) >= floor_p) ++n;
    kept = n > 0 ? n : 1;
  }
  float psum = 0.f;
  for (int e = 0; e < kept; ++e) psum += p(e);
  const float target = u * psum;
  float acc = 0.f;
  for (int e = 0; e < kept; ++e) {
    acc += p(e);
    if (target < acc) return e;
  }
  return kept - 1;
}

// CACHED: the row has at most FILT_THREADS * 4 * FILT_STEPS values, and every lane keeps its
// share of the row (4 values of each of the wave's steps) in registers from the first read on.
#define FILT_STEPS 16
template <bool CACHED>
__global__ __launch_bounds__(FILT_THREADS) void sample_filtered_kernel(
    const float* __restrict__ logits, const int* __restrict__ rows, const int* __restrict__ keep_n,
    const float* __restrict__ temperature, const float* __restrict__ top_p,
    const float* __restrict__ min_p, const float* __restrict__ uniform, int* __restrict__ out,
    int* __restrict__ out2, int V) {
  __shared__ uint32_t hist_p[FILT_BINS][FILT_SUBS];
  __shared__ uint32_t hist[FILT_BINS];
  __shared__ uint32_t sh_prefix, sh_remaining, sh_count;
  __shared__ uint32_t wave_ties[FILT_WAVES];
  __shared__ float cval[FILT_MAX_KEEP];
  __shared__ float cq[FILT_MAX_KEEP];
  __shared__ int cidx[FILT_MAX_KEEP];
  __shared__ float sh_sum;
  const int i = blockIdx.x, tid = threadIdx.x;
  const int lane = tid % WAVE, wave = tid / WAVE;
  const float* lg = logits + (size_t)rows[i] * V;
  const int keep = min(min(keep_n[i], V), FILT_MAX_KEEP);

  // the wave's part of the row, a whole number of 256-value steps
  const int region = (((V + FILT_WAVES - 1) / FILT_WAVES) + 255) / 256 * 256;
  const int w0 = min(wave * region, V), w1 = min(w0 + region, V);
  const bool vec = V % 4 == 0 && (reinterpret_cast<uintptr_t>(lg) % 16) == 0;
  // keys of the values base + 4 lane + (0..3) of a step; 0 (below every number's key) past the
  // end of the part
  auto load4 = [&](int base, uint32_t (&k)[4]) {
    const int idx = base + 4 * lane;
    if (vec) {
      const bool in = idx < w1;          // V and the parts are multiples of 4
      float4 q = {0.f, 0.f, 0.f, 0.f};
      if (in) q = *reinterpret_cast<const float4*>(lg + idx);
      k[0] = in ? order_key(q.x) : 0u;
      k[1] = in ? order_key(q.y) : 0u;
      k[2] = in ? order_key(q.z) : 0u;
      k[3] = in ? order_key(q.w) : 0u;
    } else {
#pragma unroll
      for (int c = 0; c < 4; ++c) k[c] = idx + c < w1 ? order_key(lg[idx + c]) : 0u;
    }
  };
  // every step of the wave's part in turn: f(first index of the step, this lane's four keys)
  uint32_t held[CACHED ? FILT_STEPS : 1][4];
  if (CACHED) {
#pragma unroll
    for (int st = 0; st < FILT_STEPS; ++st) load4(w0 + 256 * st, held[st]);
  }
  auto each_step = [&](auto&& f) {
    if (CACHED) {
#pragma unroll
      for (int st = 0; st < FILT_STEPS; ++st) f(w0 + 256 * st, held[st]);
    } else {
      for (int base = w0; base < w1; base += 256) {
        uint32_t k[4];
        load4(base, k);
        f(base, k);
      }
    }
  };

  // ---- the keep-th largest key, 11, 11 and 10 bits at a time from the top ------------------
  if (tid == 0) { sh_prefix = 0; sh_remaining = keep; }
#pragma unroll 1
  for (int pass = 0; pass < 3; ++pass) {
    const int shift = pass == 0 ? 21 : (pass == 1 ? 10 : 0);
    const uint32_t digit = pass == 2 ? 0x3ffu : 0x7ffu;
    for (int e = tid; e < FILT_BINS * FILT_SUBS; e += FILT_THREADS) (&hist_p[0][0])[e] = 0;
    __syncthreads();
    const uint32_t prefix = sh_prefix;
    const uint32_t mask = pass == 0 ? 0u : (0xffffffffu << (pass == 1 ? 21 : 10));
    uint32_t* mine = &hist_p[0][lane % FILT_SUBS];
    each_step([&](int base, const uint32_t (&k)[4]) {
      // after the first pass few values still match the prefix: one test for the lane's four
      bool hit[4];
#pragma unroll
      for (int c = 0; c < 4; ++c) hit[c] = k[c] != 0u && (k[c] & mask) == prefix;
      if (!(hit[0] || hit[1] || hit[2] || hit[3])) return;
#pragma unroll
      for (int c = 0; c < 4; ++c)
        if (hit[c]) atomicAdd(mine + ((k[c] >> shift) & digit) * FILT_SUBS, 1u);
    });
    __syncthreads();
    for (int bin = tid; bin < FILT_BINS; bin += FILT_THREADS) {
      uint32_t sum = 0;
#pragma unroll
      for (int sub = 0; sub < FILT_SUBS; ++sub) sum += hist_p[bin][sub];
      hist[bin] = sum;
    }
    __syncthreads();
    if (wave == 0) {
      // the largest bin b whose count together with all bins above it reaches what is still
      // wanted: lane holds bins PER lane .. PER lane + PER - 1; sums from the top by a suffix
      // scan over the lanes
      constexpr int PER = FILT_BINS / WAVE;
      uint32_t mine_sum = 0;
      for (int j = 0; j < PER; ++j) mine_sum += hist[PER * lane + j];
      uint32_t suf = mine_sum;
#pragma unroll
      for (int off = 1; off < WAVE; off <<= 1) {
        const uint32_t o = __shfl_down(suf, off, WAVE);
        if (lane + off < WAVE) suf += o;
      }
      const uint32_t rem = sh_remaining;
      // count of the bins >= b falls with b: the bins that reach `rem` are 0..cnt-1
      int cnt = 0;
      uint32_t from = suf;                 // count of bins >= PER lane + j
      for (int j = 0; j < PER; ++j) {
        cnt += from >= rem ? 1 : 0;
        from -= hist[PER * lane + j];
      }
#pragma unroll
      for (int m = WAVE / 2; m > 0; m >>= 1) cnt += __shfl_xor(cnt, m, WAVE);
      const int b = max(cnt - 1, 0);
      if (lane == b / PER) {
        uint32_t above = suf;              // count of bins > b
        for (int j = 0; j <= b % PER; ++j) above -= hist[PER * lane + j];
        sh_prefix = prefix | ((uint32_t)b << shift);
        sh_remaining = rem - above;
      }
    }
    __syncthreads();
  }
  const uint32_t thr = sh_prefix;            // key of the keep-th largest
  const uint32_t n_ties = sh_remaining;      // how many elements with exactly this key are kept
  // ---- gather: everything above the threshold, then the first ties in index order ---------
  if (tid == 0) sh_count = 0;
  __syncthreads();
  uint32_t my_ties = 0;
  each_step([&](int base, const uint32_t (&k)[4]) {
    if (max(max(k[0], k[1]), max(k[2], k[3])) < thr) return;      // the usual case
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      if (k[c] > thr) {                     // thr is a number's key: above the 0 of the padding
        const uint32_t slot = atomicAdd(&sh_count, 1u);
        cval[slot] = key_value(k[c]);
        cidx[slot] = base + 4 * lane + c;
      } else if (k[c] == thr) {
        ++my_ties;
      }
    }
  });
#pragma unroll
  for (int m = WAVE / 2; m > 0; m >>= 1) my_ties += __shfl_xor(my_ties, m, WAVE);
  if (lane == 0) wave_ties[wave] = my_ties;
  __syncthreads();
  {
    const uint32_t n_above = sh_count;      // = keep - n_ties
    uint32_t running = 0;                   // ties in the parts before this wave's
    for (int w = 0; w < wave; ++w) running += wave_ties[w];
    if (my_ties > 0 && running < n_ties) {
      // index order inside a step: lane, then the lane's four values
      const uint64_t below = lane == 0 ? 0ull : (~0ull >> (WAVE - lane));
      each_step([&](int base, const uint32_t (&k)[4]) {
        if (running >= n_ties) return;
        uint32_t before = 0, in_step = 0;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          const uint64_t m = __ballot(k[c] == thr);
          before += (uint32_t)__popcll(m & below);
          in_step += (uint32_t)__popcll(m);
        }
        uint32_t r = running + before;
#pragma unroll
        for (int c = 0; c < 4; ++c)
          if (k[c] == thr) {
            if (r < n_ties) {
              cval[n_above + r] = key_value(thr);
              cidx[n_above + r] = base + 4 * lane + c;
            }
            ++r;
          }
        running += in_step;
      });
    }
  }
  __syncthreads();
  // pad to a power of two for the sort
  int n2 = 1;
  while (n2 < keep) n2 <<= 1;
  if (n2 <= WAVE) {
    // few candidates (the usual top-k): the first wave sorts them in registers, one a lane, and
    // finishes alone, without block barriers
    if (wave != 0) return;
    float v = lane < keep ? cval[lane] : -INFINITY;
    int id = lane < keep ? cidx[lane] : 0x7fffffff;
    for (int k = 2; k <= n2; k <<= 1)
      for (int j = k >> 1; j > 0; j >>= 1) {
        const float ov = __shfl_xor(v, j, WAVE);
        const int oi = __shfl_xor(id, j, WAVE);
        const bool lower = (lane & j) == 0, desc = (lane & k) == 0;
        const bool mine_first = v > ov || (v == ov && id < oi);
        const bool keep_mine = lower ? (mine_first == desc) : (mine_first != desc);
        if (!keep_mine) { v = ov; id = oi; }
      }
    // lane e holds candidate e; the running sums go through the lanes in order, every lane
    // computing the same
    const float inv_t = 1.0f / temperature[i];
    const float mx = __shfl(v, 0, WAVE) * inv_t;
    const float p = expf(v * inv_t - mx);
    auto p_of = [&](int e) { return __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(p), e)); };
    float sum = 0.f;
    for (int e = 0; e < keep; ++e) sum += p_of(e);
    const float q = p / sum;
    auto q_of = [&](int e) { return __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(q), e)); };
    const int pick = narrow_and_draw(p_of, q_of, keep, top_p[i], min_p[i], uniform[i]);
    if (lane == 0) put(out, out2, rows[i], __builtin_amdgcn_readlane(id, pick));
    return;
  }
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
  // ---- temperature, top-p, min-p, draw (float, in the reference's order) -------------------
  const float inv_t = 1.0f / temperature[i];
  const float mx = cval[0] * inv_t;
  __syncthreads();
  if (tid < keep) cval[tid] = expf(cval[tid] * inv_t - mx);
  __syncthreads();
  if (tid == 0) {
    float sum = 0.f;
    for (int e = 0; e < keep; ++e) sum += cval[e];
    sh_sum = sum;
  }
  __syncthreads();
  if (tid < keep) cq[tid] = cval[tid] / sh_sum;
  __syncthreads();
  if (tid == 0)
    put(out, out2, rows[i],
        cidx[narrow_and_draw([&](int e) { return cval[e]; }, [&](int e) { return cq[e]; }, keep,
                             top_p[i], min_p[i], uniform[i])]);
}

// ---------------------------------------------------------------------------------------
// The same draw for a top-k above 1024 (kappai keeps any top-k below the vocabulary,
// src/sampler.c:218-223): the candidates no longer fit LDS.  One block per entry sorts the
// whole row with its indices in a workspace in global memory (bitonic, descending value,
// ascending index on ties: the passes that stay inside 4096 neighbours run in LDS, the others
// in place), takes the first `keep`, and walks them in the reference's order of operations:
// exponentials by all threads, every running sum by one thread, chunk by chunk through LDS.
// A setting for experiments, not for serving: 2 to 3 ms for a vocabulary of 65,536.
// ---------------------------------------------------------------------------------------
#define WIDE_CHUNK 4096
__global__ __launch_bounds__(FILT_THREADS) void sample_filtered_wide_kernel(
    const float* __restrict__ logits, const int* __restrict__ rows, const int* __restrict__ keep_n,
    const float* __restrict__ temperature, const float* __restrict__ top_p,
    const float* __restrict__ min_p, const float* __restrict__ uniform, int* __restrict__ out,
    int* __restrict__ out2, int V, int n2, float* __restrict__ ws_val, int* __restrict__ ws_idx) {
  __shared__ float s_val[WIDE_CHUNK];
  __shared__ int s_idx[WIDE_CHUNK];
  __shared__ int sh_stop, sh_int;
  const int i = blockIdx.x, tid = threadIdx.x;
  const float* lg = logits + (size_t)rows[i] * V;
  float* val = ws_val + (size_t)i * n2;
  int* idx = ws_idx + (size_t)i * n2;
  const int keep = max(1, min(keep_n[i], V));
  for (int e = tid; e < n2; e += FILT_THREADS) {
    val[e] = e < V ? lg[e] : -INFINITY;
    idx[e] = e < V ? e : 0x7fffffff;
  }
  __syncthreads();
  // ---- the sort ---------------------------------------------------------------------------
  const int len = min(WIDE_CHUNK, n2);           // both powers of two
  // stages k_from..k_to, of each the passes with j < len, chunk by chunk in LDS
  auto local_passes = [&](int k_from, int k_to) {
    for (int c0 = 0; c0 < n2; c0 += len) {
      for (int e = tid; e < len; e += FILT_THREADS) {
        s_val[e] = val[c0 + e];
        s_idx[e] = idx[c0 + e];
      }
      __syncthreads();
      for (int k = k_from; k <= k_to; k <<= 1)
        for (int j = min(k >> 1, len >> 1); j > 0; j >>= 1) {
          for (int a = tid; a < len; a += FILT_THREADS) {
            const int b = a ^ j;
            if (b > a) {
              const bool desc = ((c0 + a) & k) == 0;
              const float va = s_val[a], vb = s_val[b];
              const int ia = s_idx[a], ib = s_idx[b];
              const bool a_first = va > vb || (va == vb && ia < ib);
              if (a_first != desc) { s_val[a] = vb; s_val[b] = va; s_idx[a] = ib; s_idx[b] = ia; }
            }
          }
          __syncthreads();
        }
      for (int e = tid; e < len; e += FILT_THREADS) {
        val[c0 + e] = s_val[e];
        idx[c0 + e] = s_idx[e];
      }
      __syncthreads();
    }
  };
  local_passes(2, len);
  for (int k = 2 * len; k <= n2; k <<= 1) {
    for (int j = k >> 1; j >= len; j >>= 1) {
      for (int a = tid; a < n2; a += FILT_THREADS) {
        const int b = a ^ j;
        if (b > a) {
          const bool desc = (a & k) == 0;
          const float va = val[a], vb = val[b];
          const int ia = idx[a], ib = idx[b];
          const bool a_first = va > vb || (va == vb && ia < ib);
          if (a_first != desc) { val[a] = vb; val[b] = va; idx[a] = ib; idx[b] = ia; }
        }
      }
      __syncthreads();
    }
    local_passes(k, k);
  }
  // ---- temperature: val[e] becomes p(e) -----------------------------------------------------
  const float inv_t = 1.0f / temperature[i];
  const float mx = val[0] * inv_t;
  __syncthreads();
  for (int e = tid; e < keep; e += FILT_THREADS) val[e] = expf(val[e] * inv_t - mx);
  __syncthreads();
  // thread 0 walks p(0..n) in order, a chunk at a time out of LDS; body(e, p) returns true to stop
  auto walk = [&](int n, auto&& body) {
    for (int c0 = 0; c0 < n; c0 += WIDE_CHUNK) {
      const int m = min(WIDE_CHUNK, n - c0);
      for (int e = tid; e < m; e += FILT_THREADS) s_val[e] = val[c0 + e];
      if (tid == 0) sh_stop = 0;
      __syncthreads();
      if (tid == 0)
        for (int e = 0; e < m; ++e)
          if (body(c0 + e, s_val[e])) { sh_stop = 1; break; }
      __syncthreads();
      if (sh_stop) break;
    }
  };
  auto share = [&](int v) {                      // thread 0's value, for everybody
    __syncthreads();
    if (tid == 0) sh_int = v;
    __syncthreads();
    return sh_int;
  };
  // (src/sampler.c:271-332, as narrow_and_draw above; only thread 0's numbers mean anything)
  float sum = 0.f;
  walk(keep, [&](int, float p) { sum += p; return false; });
  const float tp = top_p[i], mp = min_p[i];
  int kept = keep;
  if (tp < 1.0f) {
    float cum = 0.f;
    int k1 = keep;
    walk(keep, [&](int e, float p) {
      cum += p / sum;
      if (cum > tp) { k1 = e + 1; return true; }
      return false;
    });
    kept = share(k1);
  }
  if (mp > 0.f) {
    float floor_p = 0.f;
    int n = 0;
    walk(kept, [&](int e, float p) {
      const float q = p / sum;
      if (e == 0) floor_p = mp * q;
      if (q >= floor_p) { n = e + 1; return false; }
      return true;
    });
    kept = share(n > 0 ? n : 1);
  }
  float psum = 0.f;
  walk(kept, [&](int, float p) { psum += p; return false; });
  const float target = uniform[i] * psum;
  float acc = 0.f;
  int pick = kept - 1;
  walk(kept, [&](int e, float p) {
    acc += p;
    if (target < acc) { pick = e; return true; }
    return false;
  });
  if (tid == 0) put(out, out2, rows[i], idx[pick]);
}

// The workspace of the kernel above: floats and ints for `n_entries` rows of `n2` values each,
// n2 the power of two that holds the vocabulary.
extern "C" int kappai_sample_filtered_wide_n2(int V) {
  int n2 = 1;
  while (n2 < V) n2 <<= 1;
  return n2;
}

// As kappai_sample_filtered, for any keep_n[i] up to the vocabulary; ws_val and ws_idx hold
// n_entries * kappai_sample_filtered_wide_n2(V) values each.
extern "C" int kappai_sample_filtered_wide(const float* logits, const int* rows, const int* keep_n,
                                           const float* temperature, const float* top_p,
                                           const float* min_p, const float* uniform, int* out,
                                           int* out2, int n_entries, int V, float* ws_val,
                                           int* ws_idx, hipStream_t stream) {
  if (n_entries <= 0) return 0;
  if (V < 1 || V > (1 << 30) || ws_val == nullptr || ws_idx == nullptr)
    return (int)hipErrorInvalidValue;
  hipLaunchKernelGGL(sample_filtered_wide_kernel, dim3(n_entries), dim3(FILT_THREADS), 0, stream,
                     logits, rows, keep_n, temperature, top_p, min_p, uniform, out, out2, V,
                     kappai_sample_filtered_wide_n2(V), ws_val, ws_idx);
  KAPPAI_RETURN_LAUNCH_STATUS();
}

// rows[i] names the row of `logits` (and of `out`) that entry i samples for; keep_n[i] <= 1024.
extern "C" int kappai_sample_filtered(const float* logits, const int* rows, const int* keep_n,
                                      const float* temperature, const float* top_p,
                                      const float* min_p, const float* uniform, int* out,
                                      int* out2, int n_entries, int V, hipStream_t stream) {
  if (n_entries <= 0) return 0;
  if (V < 1) return (int)hipErrorInvalidValue;
  if (V <= FILT_THREADS * 4 * FILT_STEPS)
    hipLaunchKernelGGL(sample_filtered_kernel<true>, dim3(n_entries), dim3(FILT_THREADS), 0, stream,
                       logits, rows, keep_n, temperature, top_p, min_p, uniform, out, out2, V);
  else
    hipLaunchKernelGGL(sample_filtered_kernel<false>, dim3(n_entries), dim3(FILT_THREADS), 0,
                       stream, logits, rows, keep_n, temperature, top_p, min_p, uniform, out, out2, V);
  KAPPAI_RETURN_LAUNCH_STATUS();
}

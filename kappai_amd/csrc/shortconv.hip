// Gated short convolution over a batch of segments (kappai: src/backend/cpu/common.c:2393-2431,
// second statement in src/backend/vulkan/shaders/shortconv.comp:29-52).
//
// proj[t] = (B | C | x), each D wide.  bx = B*x;  s_t[c] = bias[c] + sum_k w[c,k] bx_{t-(L-1)+k}[c];
// out = C * s.  Values before a segment's first row come from the request's state
// state[slot][c][0..L-2] (oldest first), or are zero when the segment starts at position 0
// (src/recipe/ops_hybrid.c:353-354).  A second kernel then moves the last L-1 values of bx
// into the state; segments shorter than L-1 shift the old state through.
#include "common.h"

// The projection as the kernels below read it: a tensor [T, 3D], or (PartsIn) the float sums
// over n_parts ranges of its input dimension, [n_parts][T][3D] (a product split over K): they are
// added in order and rounded to bfloat16, which is what the unsplit product would have stored.
template <typename T>
struct RowsIn {
  const T* proj;
  __device__ float at(size_t i) const { return to_f32(proj[i]); }
};
struct PartsIn {
  const float* parts;
  int n_parts;
  size_t plane;      // T * 3D
  __device__ float at(size_t i) const {
    float sum = parts[i];
    for (int s = 1; s < n_parts; ++s) sum += parts[s * plane + i];
    return to_f32(f32_to_bf16(sum));
  }
};

template <typename T, typename IN>
__global__ void shortconv_out_kernel(IN in, const float* __restrict__ w,
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
      const size_t p = (size_t)(t - r + src) * 3 * D;
      bx = in.at(p + c) * in.at(p + 2 * D + c);
    } else {
      bx = fresh ? 0.f : st[H + src];
    }
    sum += wc[k] * bx;
  }
  const float cg = in.at((size_t)t * 3 * D + D + c);
  from_f32(out + (size_t)t * D + c, cg * sum);
}

// bfloat16, D a multiple of 8, L <= 4: a thread takes 8 channels and a run of SC_RUN rows, 16
// bytes a load, every load of the run in flight at once.  It carries the last L-1 values of bx
// from row to row; at the run's first row (and where a new segment begins inside the run) they
// come from the rows before, or from the state when those lie before the segment.
#define SC_RUN 4
#define SC_HMAX 3
typedef __attribute__((ext_vector_type(4))) uint32_t sc_u32x4_t;

__device__ __forceinline__ void sc_unpack8(sc_u32x4_t v, float* f) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f[2 * i] = __uint_as_float(v[i] << 16);
    f[2 * i + 1] = __uint_as_float(v[i] & 0xffff0000u);
  }
}

// PARTS: the projection comes as float sums over n_parts ranges of its input dimension (see
// PartsIn); 8 channels of a gate are then two loads of 16 bytes a range, and a thread takes one
// row only (RUN 1): the steps that come this way have few rows, and the sums are the work.
template <int L, bool PARTS, int RUN>
__global__ __launch_bounds__(256) void shortconv_out_vec_kernel(
    const bf16_t* __restrict__ proj, const float* __restrict__ parts, int n_parts,
    const float* __restrict__ w, const float* __restrict__ bias,
    const float* __restrict__ state, bf16_t* __restrict__ out, const int* __restrict__ row_seg,
    const int* __restrict__ seg_start, const int* __restrict__ seg_pos0,
    const int* __restrict__ seg_slot, int T, int D) {
  constexpr int H = L - 1;
  const int c0 = (blockIdx.y * blockDim.x + threadIdx.x) * 8;
  const int t0 = blockIdx.x * RUN;
  if (c0 >= D) return;
  const size_t ld = (size_t)3 * D;
  // 8 channels of a gate of one row (at: the row's offset plus the gate's), as bfloat16
  auto gate8 = [&](size_t at) -> sc_u32x4_t {
    if (!PARTS) return *reinterpret_cast<const sc_u32x4_t*>(proj + at);
    const size_t plane = (size_t)T * ld;
    float4 lo = *reinterpret_cast<const float4*>(parts + at);
    float4 hi = *reinterpret_cast<const float4*>(parts + at + 4);
    for (int s = 1; s < n_parts; ++s) {
      const float4 a = *reinterpret_cast<const float4*>(parts + s * plane + at);
      const float4 b = *reinterpret_cast<const float4*>(parts + s * plane + at + 4);
      lo.x += a.x; lo.y += a.y; lo.z += a.z; lo.w += a.w;
      hi.x += b.x; hi.y += b.y; hi.z += b.z; hi.w += b.w;
    }
    sc_u32x4_t r;
    r[0] = pack_bf16x2(lo.x, lo.y);
    r[1] = pack_bf16x2(lo.z, lo.w);
    r[2] = pack_bf16x2(hi.x, hi.y);
    r[3] = pack_bf16x2(hi.z, hi.w);
    return r;
  };
  // rows t0-H .. t0+RUN-1: the gates of the run and of the rows just before it
  sc_u32x4_t vb[RUN + H], vx[RUN + H], vc[RUN];
  const sc_u32x4_t zero = {0u, 0u, 0u, 0u};
#pragma unroll
  for (int i = 0; i < RUN + H; ++i) {
    const int t = t0 - H + i;
    const bool in = t >= 0 && t < T;
    const size_t p = (size_t)(in ? t : 0) * ld + c0;
    vb[i] = in ? gate8(p) : zero;
    vx[i] = in ? gate8(p + 2 * D) : zero;
    if (i >= H) vc[i - H] = in ? gate8(p + D) : zero;
  }
  // the 8 channels' taps lie together: 8 L floats from a 16-byte aligned address
  float wt[8 * L], bs[8];
  {
    const float4* wp = reinterpret_cast<const float4*>(w + (size_t)c0 * L);
#pragma unroll
    for (int i = 0; i < 2 * L; ++i) {
      const float4 v = wp[i];
      wt[4 * i] = v.x, wt[4 * i + 1] = v.y, wt[4 * i + 2] = v.z, wt[4 * i + 3] = v.w;
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) bs[j] = 0.f;
    if (bias) {
      const float4 b0 = *reinterpret_cast<const float4*>(bias + c0);
      const float4 b1 = *reinterpret_cast<const float4*>(bias + c0 + 4);
      bs[0] = b0.x, bs[1] = b0.y, bs[2] = b0.z, bs[3] = b0.w;
      bs[4] = b1.x, bs[5] = b1.y, bs[6] = b1.z, bs[7] = b1.w;
    }
  }
  float bx[RUN + H][8];
#pragma unroll
  for (int i = 0; i < RUN + H; ++i) {
    float b[8], x[8];
    sc_unpack8(vb[i], b);
    sc_unpack8(vx[i], x);
#pragma unroll
    for (int j = 0; j < 8; ++j) bx[i][j] = b[j] * x[j];
  }
#pragma unroll
  for (int r = 0; r < RUN; ++r) {
    const int t = t0 + r;
    if (t >= T) break;
    const int seg = row_seg[t];
    const int first = seg_start[seg];
    const bool fresh = seg_pos0[seg] == 0;
    const float* st = state + ((size_t)seg_slot[seg] * D + c0) * H;
    float cg[8], res[8];
    sc_unpack8(vc[r], cg);
#pragma unroll
    for (int j = 0; j < 8; ++j) res[j] = bs[j];
    // tap k meets the row t - H + k, which is loaded row r + k
#pragma unroll
    for (int k = 0; k < L; ++k) {
      const int src = t - H + k;
      if (src >= first) {
#pragma unroll
        for (int j = 0; j < 8; ++j) res[j] = fmaf(wt[j * L + k], bx[r + k][j], res[j]);
      } else if (!fresh) {
        const int e = H + (src - first);            // entry of the state: H-1 is the newest
#pragma unroll
        for (int j = 0; j < 8; ++j) res[j] = fmaf(wt[j * L + k], st[(size_t)j * H + e], res[j]);
      }
    }
    sc_u32x4_t o;
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = pack_bf16x2(cg[2 * i] * res[2 * i], cg[2 * i + 1] * res[2 * i + 1]);
    *reinterpret_cast<sc_u32x4_t*>(out + (size_t)t * D + c0) = o;
  }
}

template <typename IN>
__global__ void shortconv_state_kernel(IN in, float* __restrict__ state,
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
      const size_t p = (size_t)(t0 + src) * 3 * D;
      v = in.at(p + c) * in.at(p + 2 * D + c);
    } else {
      v = fresh ? 0.f : st[n + j];
    }
    st[j] = v;
  }
}

// Every segment is a single row (decode): one thread per (segment, channel) computes the output
// and shifts the state, which nobody else reads.
__device__ __forceinline__ float shortconv_step_one(float bg, float cg, float xg,
                                                    const float* __restrict__ wc, float cbias,
                                                    float* __restrict__ st, bool fresh, int L) {
  const int H = L - 1;
  const float bx = bg * xg;
  float sum = cbias;
  float prev = fresh ? 0.f : st[0];
  for (int k = 0; k < H; ++k) {
    sum += wc[k] * prev;                       // tap k meets history entry k
    const float next = (k + 1 < H) ? (fresh ? 0.f : st[k + 1]) : bx;
    st[k] = next;                              // shift: entry k becomes entry k+1, the last bx
    prev = next;
  }
  sum += wc[H] * bx;
  return cg * sum;
}

template <typename T>
__global__ void shortconv_step_kernel(const T* __restrict__ proj, const float* __restrict__ w,
                                      const float* __restrict__ bias, float* __restrict__ state,
                                      T* __restrict__ out, const int* __restrict__ seg_pos0,
                                      const int* __restrict__ seg_slot, int D, int L) {
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  const int t = blockIdx.x;
  if (c >= D) return;
  const T* p = proj + (size_t)t * 3 * D;
  float* st = state + ((size_t)seg_slot[t] * D + c) * (L - 1);
  from_f32(out + (size_t)t * D + c,
           shortconv_step_one(to_f32(p[c]), to_f32(p[D + c]), to_f32(p[2 * D + c]),
                              w + (size_t)c * L, bias ? bias[c] : 0.f, st, seg_pos0[t] == 0, L));
}

// The same step when the projection arrives as float sums over n_parts ranges of its input
// dimension, [n_parts][T][3D] (a product split over K): they are added in order and rounded to
// bfloat16, which is what the unsplit product would have stored.
__global__ void shortconv_step_parts_kernel(const float* __restrict__ parts, int n_parts,
                                            const float* __restrict__ w,
                                            const float* __restrict__ bias,
                                            float* __restrict__ state, bf16_t* __restrict__ out,
                                            const int* __restrict__ seg_pos0,
                                            const int* __restrict__ seg_slot, int T, int D, int L) {
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  const int t = blockIdx.x;
  if (c >= D) return;
  const size_t plane = (size_t)T * 3 * D;
  const float* p = parts + (size_t)t * 3 * D + c;
  float g[3];
#pragma unroll
  for (int i = 0; i < 3; ++i) {
    float sum = p[(size_t)i * D];
    for (int s = 1; s < n_parts; ++s) sum += p[s * plane + (size_t)i * D];
    g[i] = to_f32(f32_to_bf16(sum));
  }
  float* st = state + ((size_t)seg_slot[t] * D + c) * (L - 1);
  from_f32(out + (size_t)t * D + c,
           shortconv_step_one(g[0], g[1], g[2], w + (size_t)c * L, bias ? bias[c] : 0.f, st,
                              seg_pos0[t] == 0, L));
}

// proj [T, 3D] (float32 or bfloat16), or null with `parts` [n_parts][T][3D]: float sums over
// ranges of the projection's input dimension (the result is then bfloat16).
static int shortconv_launch(const void* proj, const float* parts, int n_parts, const float* w,
                            const float* bias, float* state, void* out, const int* row_seg,
                            const int* seg_start, const int* seg_pos0, const int* seg_slot, int T,
                            int S, int D, int L, int is_bf16, hipStream_t stream) {
  if (T <= 0 || S <= 0) return 0;
  if (L < 2) return (int)hipErrorInvalidValue;
  const int threads = D >= 256 ? 256 : 64;
  dim3 g1(T, (D + threads - 1) / threads), g2(S, (D + threads - 1) / threads);
  const PartsIn pin{parts, n_parts, (size_t)T * 3 * D};
  if (T == S) {   // one row a segment: row t is segment t
    if (parts)
      hipLaunchKernelGGL(shortconv_step_parts_kernel, g1, dim3(threads), 0, stream, parts, n_parts,
                         w, bias, state, (bf16_t*)out, seg_pos0, seg_slot, T, D, L);
    else if (is_bf16)
      hipLaunchKernelGGL(shortconv_step_kernel<bf16_t>, g1, dim3(threads), 0, stream,
                         (const bf16_t*)proj, w, bias, state, (bf16_t*)out, seg_pos0, seg_slot, D,
                         L);
    else
      hipLaunchKernelGGL(shortconv_step_kernel<float>, g1, dim3(threads), 0, stream,
                         (const float*)proj, w, bias, state, (float*)out, seg_pos0, seg_slot, D, L);
    KAPPAI_RETURN_LAUNCH_STATUS();
  }
  const void* in_ptr = parts ? (const void*)parts : proj;
  if (is_bf16 && D % 8 == 0 && L <= SC_HMAX + 1 && ((uintptr_t)in_ptr % 16) == 0 &&
      ((uintptr_t)out % 16) == 0 && ((uintptr_t)w % 16) == 0 && (!bias || ((uintptr_t)bias % 16) == 0)) {
    const int groups = D / 8;
    const int th = groups >= 256 ? 256 : 64;
    const int run = parts ? 1 : SC_RUN;
    const dim3 gv((T + run - 1) / run, (groups + th - 1) / th);
#define SC_LAUNCH_AS(LL, PP)                                                                     \
  hipLaunchKernelGGL((shortconv_out_vec_kernel<LL, PP, (PP ? 1 : SC_RUN)>), gv, dim3(th), 0, stream, \
                     (const bf16_t*)proj, parts, n_parts, w, bias, (const float*)state,          \
                     (bf16_t*)out, row_seg, seg_start, seg_pos0, seg_slot, T, D)
#define SC_LAUNCH(LL)                                                                            \
  if (parts) SC_LAUNCH_AS(LL, true);                                                             \
  else SC_LAUNCH_AS(LL, false)
    if (L == 2) { SC_LAUNCH(2); }
    else if (L == 3) { SC_LAUNCH(3); }
    else { SC_LAUNCH(4); }
#undef SC_LAUNCH
#undef SC_LAUNCH_AS
  } else if (parts) {
    hipLaunchKernelGGL((shortconv_out_kernel<bf16_t, PartsIn>), g1, dim3(threads), 0, stream, pin, w,
                       bias, (const float*)state, (bf16_t*)out, row_seg, seg_start, seg_pos0,
                       seg_slot, D, L);
  } else if (is_bf16) {
    hipLaunchKernelGGL((shortconv_out_kernel<bf16_t, RowsIn<bf16_t>>), g1, dim3(threads), 0, stream,
                       RowsIn<bf16_t>{(const bf16_t*)proj}, w, bias, (const float*)state,
                       (bf16_t*)out, row_seg, seg_start, seg_pos0, seg_slot, D, L);
  } else {
    hipLaunchKernelGGL((shortconv_out_kernel<float, RowsIn<float>>), g1, dim3(threads), 0, stream,
                       RowsIn<float>{(const float*)proj}, w, bias, (const float*)state, (float*)out,
                       row_seg, seg_start, seg_pos0, seg_slot, D, L);
  }
  // then the state: the last L - 1 values of B * x of every segment
  if (parts)
    hipLaunchKernelGGL(shortconv_state_kernel<PartsIn>, g2, dim3(threads), 0, stream, pin, state,
                       seg_start, seg_pos0, seg_slot, D, L);
  else if (is_bf16)
    hipLaunchKernelGGL(shortconv_state_kernel<RowsIn<bf16_t>>, g2, dim3(threads), 0, stream,
                       RowsIn<bf16_t>{(const bf16_t*)proj}, state, seg_start, seg_pos0, seg_slot, D,
                       L);
  else
    hipLaunchKernelGGL(shortconv_state_kernel<RowsIn<float>>, g2, dim3(threads), 0, stream,
                       RowsIn<float>{(const float*)proj}, state, seg_start, seg_pos0, seg_slot, D, L);
  KAPPAI_RETURN_LAUNCH_STATUS();
}

extern "C" int kappai_shortconv(const void* proj, const float* w, const float* bias, float* state,
                                void* out, const int* row_seg, const int* seg_start,
                                const int* seg_pos0, const int* seg_slot, int T, int S, int D,
                                int L, int is_bf16, hipStream_t stream) {
  return shortconv_launch(proj, nullptr, 0, w, bias, state, out, row_seg, seg_start, seg_pos0,
                          seg_slot, T, S, D, L, is_bf16, stream);
}

// The same from the float partial sums of the projection, [n_parts][T][3D], for segments of any
// length; the result is bfloat16.
extern "C" int kappai_shortconv_parts(const float* parts, int n_parts, const float* w,
                                      const float* bias, float* state, void* out,
                                      const int* row_seg, const int* seg_start,
                                      const int* seg_pos0, const int* seg_slot, int T, int S, int D,
                                      int L, hipStream_t stream) {
  if (parts == nullptr || n_parts < 1 || D < 1) return (int)hipErrorInvalidValue;
  return shortconv_launch(nullptr, parts, n_parts, w, bias, state, out, row_seg, seg_start,
                          seg_pos0, seg_slot, T, S, D, L, 1, stream);
}

// Attention over the paged cache.
//
//   qk_norm_rope_store  per-head RMSNorm of q and k (src/backend/cpu/scalar/quants.c:1521-1531),
//                       rotation at the row's absolute position
//                       (src/backend/cpu/quants.h:395-438: rotate-half or interleaved pairs),
//                       q rewritten in place, k and v stored into their pages
//                       (src/backend/cpu/common.c:1603-1622).  The projection may also arrive
//                       as float partial sums of a product split over its input dimension.
//   paged_attention_rows  one wave per (row, head): causal softmax(q.k/sqrt(d)) v over the keys
//                       lo..pos of the row's request, read through its block table
//                       (src/backend/cpu/scalar/core.c:383-433, 623-666), online softmax in float.
//
// The key pool is [page][kv_head][page_size][head_dim]; the value pool is stored transposed,
// [page][kv_head][head_dim][page_size], which is what the matrix-core kernels want.  Token p of
// a request lives in page block_table[p / page_size] at offset p % page_size.
#include "common.h"

#define MAX_HEAD_DIM 512

// rot_mode: 0 none, 1 rotate-half pairs (j, j+rot/2), 2 interleaved pairs (2j, 2j+1)
// A block of QKS_WAVES waves takes QKS_SLOTS heads (q, k or v) of one row, a wave a head at a
// time, each wave with its own piece of LDS.
#define QKS_WAVES 4
#define QKS_SLOTS 16
template <typename T>
__global__ __launch_bounds__(QKS_WAVES * WAVE) void qk_norm_rope_store_kernel(
    T* __restrict__ qkv, int row_stride, const float* __restrict__ q_norm_w,
    const float* __restrict__ k_norm_w, float eps, const float* __restrict__ cos_tab,
    const float* __restrict__ sin_tab, int rot_dim, int rot_mode, T* __restrict__ k_pool,
    T* __restrict__ v_pool, const int* __restrict__ row_pos, const int* __restrict__ row_seg,
    const int* __restrict__ block_tables, int max_blocks, int H, int G, int d, int ps,
    int n_slots, const float* __restrict__ parts, int n_parts, T* __restrict__ q_out,
    int q_stride) {
  __shared__ float bufs[QKS_WAVES][MAX_HEAD_DIM];
  const int t = blockIdx.x, lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
  float* buf = bufs[wave];
  const int pos = row_pos[t];
  if (rot_mode == 0) rot_dim = 0;
  const int half = rot_dim / 2;
  const float* ct = cos_tab + (size_t)pos * half;
  const float* st = sin_tab + (size_t)pos * half;
  const int* bt = block_tables + (size_t)row_seg[t] * max_blocks;
  const int slot_end = min(n_slots, (int)(blockIdx.y + 1) * QKS_SLOTS);
  for (int slot = blockIdx.y * QKS_SLOTS + wave; slot < slot_end; slot += QKS_WAVES) {
    const size_t at = (size_t)t * row_stride + (size_t)slot * d;
    // with `parts` the row arrives as float sums over n_parts ranges of the projection's input
    // dimension, [n_parts][rows][row_stride]; added in order and rounded to T they are what the
    // unsplit projection would have stored, and q goes to a buffer of its own
    const size_t plane = (size_t)gridDim.x * row_stride;
    auto value = [&](int e) -> float {
      if (!parts) return to_f32(qkv[at + e]);
      float sum = parts[at + e];
      for (int k = 1; k < n_parts; ++k) sum += parts[k * plane + at + e];
      T rounded;
      from_f32(&rounded, sum);
      return to_f32(rounded);
    };
    T* dst = parts ? q_out + (size_t)t * q_stride + (size_t)slot * d : qkv + at;
    if (slot >= H) {
      const int g = (slot - H) % G;
      const size_t pg = (size_t)bt[pos / ps] * G + g;
      if (slot >= H + G) {  // v: copied into its page, transposed
        T* vdst = v_pool + pg * d * ps + pos % ps;
        for (int e = lane; e < d; e += WAVE) from_f32(vdst + (size_t)e * ps, value(e));
        continue;
      }
      dst = k_pool + (pg * ps + pos % ps) * d;
    }
    const float* nw = slot < H ? q_norm_w : k_norm_w;
    float ss = 0.f;
    for (int e = lane; e < d; e += WAVE) {
      const float v = value(e);
      buf[e] = v;
      ss += v * v;
    }
    if (nw) {
      ss = wave_sum(ss);
      const float sc = 1.0f / sqrtf(ss / (float)d + eps);
      for (int e = lane; e < d; e += WAVE) buf[e] = buf[e] * sc * nw[e];
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    for (int j = lane; j < half; j += WAVE) {
      const int i0 = rot_mode == 1 ? j : 2 * j;
      const int i1 = rot_mode == 1 ? j + half : 2 * j + 1;
      const float c = ct[j], s = st[j];
      const float v0 = buf[i0], v1 = buf[i1];
      from_f32(dst + i0, v0 * c - v1 * s);
      from_f32(dst + i1, v0 * s + v1 * c);
    }
    for (int e = rot_dim + lane; e < d; e += WAVE) from_f32(dst + e, buf[e]);
    // the next head overwrites the wave's piece of LDS
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
  }
}

// bfloat16, the whole head rotated in halves (or not at all), d / 8 a power of two up to 64:
// a lane takes 8 consecutive elements of a head, so that a wave works on 512 / d heads at once
// without LDS; the sum of squares and the rotation's partner (the lane d / 16 away) come by
// shuffles.
typedef __attribute__((ext_vector_type(4))) uint32_t qks_u32x4_t;
template <int LPH, bool PARTS>
__global__ __launch_bounds__(256) void qk_norm_rope_store_vec_kernel(
    bf16_t* __restrict__ qkv, int row_stride, const float* __restrict__ q_norm_w,
    const float* __restrict__ k_norm_w, float eps, const float* __restrict__ cos_tab,
    const float* __restrict__ sin_tab, int rotate, bf16_t* __restrict__ k_pool,
    bf16_t* __restrict__ v_pool, const int* __restrict__ row_pos,
    const int* __restrict__ row_seg, const int* __restrict__ block_tables, int max_blocks, int T,
    int H, int G, int ps, int n_slots, const float* __restrict__ parts, int n_parts,
    bf16_t* __restrict__ q_out, int q_stride) {
  constexpr int d = LPH * 8, half = d / 2;
  const long long total = (long long)T * n_slots * LPH;
  const long long gid = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const bool active = gid < total;
  const long long idx = active ? gid : total - 1;
  const int part = (int)(idx % LPH);
  const long long head = idx / LPH;
  const int t = (int)(head / n_slots), slot = (int)(head % n_slots);
  const int pos = row_pos[t];
  const int e0 = 8 * part;
  const size_t at = (size_t)t * row_stride + (size_t)slot * d + e0;
  qks_u32x4_t raw;
  if (PARTS) {
    // float sums over n_parts ranges of the projection's input dimension, added in order and
    // rounded to bfloat16: what the unsplit projection would have stored
    const size_t plane = (size_t)T * row_stride;
    float4 lo = *reinterpret_cast<const float4*>(parts + at);
    float4 hi = *reinterpret_cast<const float4*>(parts + at + 4);
    for (int k = 1; k < n_parts; ++k) {
      const float4 a = *reinterpret_cast<const float4*>(parts + k * plane + at);
      const float4 b = *reinterpret_cast<const float4*>(parts + k * plane + at + 4);
      lo.x += a.x; lo.y += a.y; lo.z += a.z; lo.w += a.w;
      hi.x += b.x; hi.y += b.y; hi.z += b.z; hi.w += b.w;
    }
    raw[0] = pack_bf16x2(lo.x, lo.y);
    raw[1] = pack_bf16x2(lo.z, lo.w);
    raw[2] = pack_bf16x2(hi.x, hi.y);
    raw[3] = pack_bf16x2(hi.z, hi.w);
  } else {
    raw = *reinterpret_cast<const qks_u32x4_t*>(qkv + at);
  }
  float v[8];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    v[2 * i] = __uint_as_float(raw[i] << 16);
    v[2 * i + 1] = __uint_as_float(raw[i] & 0xffff0000u);
  }
  const bool is_v = slot >= H + G;
  const float* nw = slot < H ? q_norm_w : k_norm_w;
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) ss = fmaf(v[i], v[i], ss);
#pragma unroll
  for (int m = LPH / 2; m >= 1; m /= 2) ss += __shfl_xor(ss, m, WAVE);
  if (nw && !is_v) {
    const float sc = 1.0f / sqrtf(ss / (float)d + eps);
    const float4 w0 = *reinterpret_cast<const float4*>(nw + e0);
    const float4 w1 = *reinterpret_cast<const float4*>(nw + e0 + 4);
    const float wv[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = v[i] * sc * wv[i];
  }
  float r[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) r[i] = v[i];
  if (LPH >= 2) {
    // partner element e +- d/2 lives in the lane LPH/2 away, same place
    float other[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) other[i] = __shfl_xor(v[i], LPH / 2 > 0 ? LPH / 2 : 1, WAVE);
    if (rotate && !is_v) {
      const bool low = e0 < half;
      const int j0 = low ? e0 : e0 - half;
      const float* ct = cos_tab + (size_t)pos * half + j0;
      const float* st = sin_tab + (size_t)pos * half + j0;
      const float4 c0 = *reinterpret_cast<const float4*>(ct), c1 = *reinterpret_cast<const float4*>(ct + 4);
      const float4 s0 = *reinterpret_cast<const float4*>(st), s1 = *reinterpret_cast<const float4*>(st + 4);
      const float cv[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
      const float sv[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
#pragma unroll
      for (int i = 0; i < 8; ++i)
        r[i] = low ? v[i] * cv[i] - other[i] * sv[i] : other[i] * sv[i] + v[i] * cv[i];
    }
  }
  if (!active) return;
  if (slot < H) {
    qks_u32x4_t o;
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = pack_bf16x2(r[2 * i], r[2 * i + 1]);
    bf16_t* qdst = PARTS ? q_out + (size_t)t * q_stride + (size_t)slot * d + e0 : qkv + at;
    *reinterpret_cast<qks_u32x4_t*>(qdst) = o;
    return;
  }
  const int g = (slot - H) % G;
  const int* bt = block_tables + (size_t)row_seg[t] * max_blocks;
  const size_t pg = (size_t)bt[pos / ps] * G + g;
  if (is_v) {
    bf16_t* vdst = v_pool + (pg * d + e0) * ps + pos % ps;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      vdst[(size_t)(2 * i) * ps] = (bf16_t)(raw[i] & 0xffffu);
      vdst[(size_t)(2 * i + 1) * ps] = (bf16_t)(raw[i] >> 16);
    }
    return;
  }
  qks_u32x4_t o;
#pragma unroll
  for (int i = 0; i < 4; ++i) o[i] = pack_bf16x2(r[2 * i], r[2 * i + 1]);
  *reinterpret_cast<qks_u32x4_t*>(k_pool + (pg * ps + pos % ps) * d + e0) = o;
}

extern "C" int kappai_qk_norm_rope_store(void* qkv, int row_stride, const float* q_norm_w,
                                         const float* k_norm_w, float eps, const float* cos_tab,
                                         const float* sin_tab, int rot_dim, int rot_mode,
                                         void* k_pool, void* v_pool, const int* row_pos,
                                         const int* row_seg, const int* block_tables,
                                         int max_blocks, int T, int H, int G, int d, int ps,
                                         int store_kv, int is_bf16, const float* parts,
                                         int n_parts, void* q_out, int q_stride,
                                         hipStream_t stream) {
  // parts != null: the projection as [n_parts][T][row_stride] float partial sums instead of
  // qkv; q is then written to q_out [T][q_stride] (bfloat16 only)
  if (T <= 0) return 0;
  if (d > MAX_HEAD_DIM || d < 1 || rot_dim > d || (rot_dim & 1)) return (int)hipErrorInvalidValue;
  if (parts && (!is_bf16 || n_parts < 1 || !q_out)) return (int)hipErrorInvalidValue;
  const int n_slots = store_kv ? H + 2 * G : H;
  const bool whole_rot = rot_mode == 0 || rot_dim == 0 || (rot_mode == 1 && rot_dim == d);
  const int lph = d / 8;
  if (is_bf16 && whole_rot && d % 8 == 0 && lph >= 2 && lph <= 64 && (lph & (lph - 1)) == 0 &&
      row_stride % 8 == 0 && ((uintptr_t)qkv % 16) == 0 && ((uintptr_t)k_pool % 16) == 0 &&
      ((uintptr_t)parts % 16) == 0 && ((uintptr_t)q_out % 16) == 0 && q_stride % 8 == 0 &&
      ((uintptr_t)cos_tab % 16) == 0 && ((uintptr_t)sin_tab % 16) == 0 &&
      (!q_norm_w || ((uintptr_t)q_norm_w % 16) == 0) &&
      (!k_norm_w || ((uintptr_t)k_norm_w % 16) == 0)) {
    const int rotate = rot_mode == 1 && rot_dim == d;
    const long long total = (long long)T * n_slots * lph;
    const dim3 gv((unsigned)((total + 255) / 256));
#define QKS_LAUNCH_AS(N, P)                                                                      \
  hipLaunchKernelGGL((qk_norm_rope_store_vec_kernel<N, P>), gv, dim3(256), 0, stream,            \
                     (bf16_t*)qkv, row_stride, q_norm_w, k_norm_w, eps, cos_tab, sin_tab,        \
                     rotate, (bf16_t*)k_pool, (bf16_t*)v_pool, row_pos, row_seg, block_tables,   \
                     max_blocks, T, H, G, ps, n_slots, parts, n_parts, (bf16_t*)q_out, q_stride)
#define QKS_LAUNCH(N)                                                                            \
  if (parts) QKS_LAUNCH_AS(N, true);                                                             \
  else QKS_LAUNCH_AS(N, false)
    switch (lph) {
      case 2: QKS_LAUNCH(2); break;
      case 4: QKS_LAUNCH(4); break;
      case 8: QKS_LAUNCH(8); break;
      case 16: QKS_LAUNCH(16); break;
      case 32: QKS_LAUNCH(32); break;
      default: QKS_LAUNCH(64); break;
    }
#undef QKS_LAUNCH
#undef QKS_LAUNCH_AS
    KAPPAI_RETURN_LAUNCH_STATUS();
  }
  dim3 grid(T, (n_slots + QKS_SLOTS - 1) / QKS_SLOTS);
  if (is_bf16)
    hipLaunchKernelGGL(qk_norm_rope_store_kernel<bf16_t>, grid, dim3(QKS_WAVES * WAVE), 0, stream,
                       (bf16_t*)qkv, row_stride, q_norm_w, k_norm_w, eps, cos_tab, sin_tab,
                       rot_dim, rot_mode, (bf16_t*)k_pool, (bf16_t*)v_pool, row_pos, row_seg,
                       block_tables, max_blocks, H, G, d, ps, n_slots, parts, n_parts,
                       (bf16_t*)q_out, q_stride);
  else
    hipLaunchKernelGGL(qk_norm_rope_store_kernel<float>, grid, dim3(QKS_WAVES * WAVE), 0, stream, (float*)qkv,
                       row_stride, q_norm_w, k_norm_w, eps, cos_tab, sin_tab, rot_dim, rot_mode,
                       (float*)k_pool, (float*)v_pool, row_pos, row_seg, block_tables, max_blocks,
                       H, G, d, ps, n_slots, nullptr, 0, nullptr, 0);
  KAPPAI_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------------
__device__ __forceinline__ float dot_row(const float* __restrict__ qs, const float* __restrict__ k,
                                         int d) {
  float s = 0.f;
  for (int e = 0; e < d; e += 4) {
    const float4 kv = *reinterpret_cast<const float4*>(k + e);
    s = fmaf(qs[e], kv.x, s);
    s = fmaf(qs[e + 1], kv.y, s);
    s = fmaf(qs[e + 2], kv.z, s);
    s = fmaf(qs[e + 3], kv.w, s);
  }
  return s;
}

__device__ __forceinline__ float dot_row(const float* __restrict__ qs,
                                         const bf16_t* __restrict__ k, int d) {
  float s = 0.f;
  for (int e = 0; e < d; e += 8) {
    const uint4 kv = *reinterpret_cast<const uint4*>(k + e);
    const uint32_t w[4] = {kv.x, kv.y, kv.z, kv.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      s = fmaf(qs[e + 2 * i], __uint_as_float(w[i] << 16), s);
      s = fmaf(qs[e + 2 * i + 1], __uint_as_float(w[i] & 0xffff0000u), s);
    }
  }
  return s;
}

#define ATT_NPL (MAX_HEAD_DIM / WAVE)

template <typename T>
__global__ __launch_bounds__(64) void paged_attention_rows_kernel(
    const T* __restrict__ q, int q_stride, const T* __restrict__ k_pool,
    const T* __restrict__ v_pool, T* __restrict__ out, int out_stride,
    const int* __restrict__ row_pos, const int* __restrict__ row_seg,
    const int* __restrict__ block_tables, int max_blocks, int H, int G, int d, int ps, int window,
    float scale) {
  __shared__ float qs[MAX_HEAD_DIM];
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int g = h / (H / G);
  const int pos = row_pos[t];
  const int* bt = block_tables + (size_t)row_seg[t] * max_blocks;
  const int lo = (window > 0 && pos + 1 > window) ? pos + 1 - window : 0;
  const T* qr = q + (size_t)t * q_stride + (size_t)h * d;
  for (int e = lane; e < d; e += WAVE) qs[e] = to_f32(qr[e]);
  __syncthreads();

  float m = -INFINITY, l = 0.f;
  float acc[ATT_NPL];
#pragma unroll
  for (int i = 0; i < ATT_NPL; ++i) acc[i] = 0.f;

  for (int base = lo; base <= pos; base += WAVE) {
    const int tk = base + lane;
    const bool valid = tk <= pos;
    float s = -INFINITY;
    unsigned long long voff = 0;
    if (valid) {
      const size_t pg = (size_t)bt[tk / ps] * G + g;
      s = dot_row(qs, k_pool + (pg * ps + tk % ps) * d, d) * scale;
      voff = (unsigned long long)(pg * d * ps + tk % ps);
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float p = valid ? expf(s - m_new) : 0.f;
    const float corr = expf(m - m_new);
    l = l * corr + wave_sum(p);
#pragma unroll
    for (int i = 0; i < ATT_NPL; ++i) acc[i] *= corr;
    const int nk = min(WAVE, pos - base + 1);
    for (int kk = 0; kk < nk; ++kk) {
      const float pk = __shfl(p, kk, WAVE);
      const unsigned lo32 = __shfl((unsigned)(voff & 0xffffffffull), kk, WAVE);
      const unsigned hi32 = __shfl((unsigned)(voff >> 32), kk, WAVE);
      const T* vr = v_pool + (((unsigned long long)hi32 << 32) | lo32);
#pragma unroll
      for (int i = 0; i < ATT_NPL; ++i) {
        const int e = lane + i * WAVE;
        if (e < d) acc[i] = fmaf(pk, to_f32(vr[(size_t)e * ps]), acc[i]);
      }
    }
    m = m_new;
  }
  const float inv = 1.0f / l;
  T* o = out + (size_t)t * out_stride + (size_t)h * d;
#pragma unroll
  for (int i = 0; i < ATT_NPL; ++i) {
    const int e = lane + i * WAVE;
    if (e < d) from_f32(o + e, acc[i] * inv);
  }
}

extern "C" int kappai_paged_attention_rows(const void* q, int q_stride, const void* k_pool,
                                           const void* v_pool, void* out, int out_stride,
                                           const int* row_pos, const int* row_seg,
                                           const int* block_tables, int max_blocks, int T, int H,
                                           int G, int d, int ps, int window, float scale,
                                           int is_bf16, hipStream_t stream) {
  if (T <= 0) return 0;
  if (d > MAX_HEAD_DIM || d % 8 || G < 1 || H % G || H > 65535) return (int)hipErrorInvalidValue;
  dim3 grid(T, H);
  if (is_bf16)
    hipLaunchKernelGGL(paged_attention_rows_kernel<bf16_t>, grid, dim3(WAVE), 0, stream,
                       (const bf16_t*)q, q_stride, (const bf16_t*)k_pool, (const bf16_t*)v_pool,
                       (bf16_t*)out, out_stride, row_pos, row_seg, block_tables, max_blocks, H, G,
                       d, ps, window, scale);
  else
    hipLaunchKernelGGL(paged_attention_rows_kernel<float>, grid, dim3(WAVE), 0, stream,
                       (const float*)q, q_stride, (const float*)k_pool, (const float*)v_pool,
                       (float*)out, out_stride, row_pos, row_seg, block_tables, max_blocks, H, G, d,
                       ps, window, scale);
  KAPPAI_RETURN_LAUNCH_STATUS();
}

// bfloat16 attention over the paged cache on the matrix cores, for one head size
// (HEAD_DIM, a multiple of 16, set when the file is compiled).
//
// Both kernels keep "one query per lane column".  For a tile of keys they compute
//     S^T = K Q^T        A = K rows (a key per lane row, 8 consecutive d per lane)
//                        B = Q     (a query per lane column)
//     O^T += V^T P^T     A = V^T   (a d index per lane row, 8 key slots per lane)
//                        B = P^T   (the lane's own values of S^T, no data movement)
// so that a lane holds, for ITS query, scores of several keys and later outputs of several d
// indices: the running maximum, the running sum and the rescaling are per lane, in float.
// The value pool is stored transposed, [page][kv_head][head_dim][page_size], which makes the
// 8 key slots of the A operand two 8-byte loads.  page_size must be a multiple of 16.
//
//   attn_prefill   v_mfma_f32_32x32x16_bf16; one block per (tile of 32 rows of a segment, head),
//                  its waves sharing out the key tiles
//   attn_decode    v_mfma_f32_16x16x32_bf16; one wave per (row, kv head, split of the keys): the
//                  query heads that share the kv head are the columns; partial results are
//                  merged by attn_merge.
// Formulas: softmax(q.k/sqrt(d)) v over keys lo..pos (kappai: src/backend/cpu/scalar/core.c:383-433,
// 623-666), online softmax as in its flash form (:386-413).
#include "common.h"
#include "no_alloc.h"
#include <stdio.h>

#ifndef HEAD_DIM
#error "compile with -DHEAD_DIM=<multiple of 16>"
#endif
static_assert(HEAD_DIM % 16 == 0 && HEAD_DIM >= 16 && HEAD_DIM <= 256, "unsupported head size");

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2_t;

__device__ __forceinline__ bf16x8_t as_frag(u32x4_t v) { return __builtin_bit_cast(bf16x8_t, v); }
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) { return pack_bf16x2(lo, hi); }
// 2^x for x <= 0 straight from the hardware (v_exp_f32); results below the normal range flush
// to zero, which is what a softmax weight that small is worth
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
// keep the j-th of four bf16 values only if keep bit j is set
__device__ __forceinline__ u32x2_t mask4(u32x2_t v, int keep) {
  const uint32_t m0 = ((keep & 1) ? 0x0000ffffu : 0u) | ((keep & 2) ? 0xffff0000u : 0u);
  const uint32_t m1 = ((keep & 4) ? 0x0000ffffu : 0u) | ((keep & 8) ? 0xffff0000u : 0u);
  return (u32x2_t){v.x & m0, v.y & m1};
}

#define LOG2E 1.4426950408889634f

// the value that lane ^ 32 holds, by one swap of the wave's halves (no trip through LDS)
__device__ __forceinline__ float other_half(float x) {
  const uint32_t u = __float_as_uint(x);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  // r[0] = the lower half's values in both halves, r[1] = the upper half's
  return __uint_as_float((threadIdx.x & 32) ? r[0] : r[1]);
}

// four key slots of V^T for d index `dd`, keys key0..key0+3 (one 16-key group: one page);
// keys outside [lo, hi] read as zero
__device__ __forceinline__ u32x2_t load_vt4(const bf16_t* __restrict__ vt_pool,
                                            const int* __restrict__ bt, int G, int g, int ps,
                                            int dd, int key0, int lo, int hi) {
  u32x2_t z = {0u, 0u};
  if (dd >= HEAD_DIM || key0 > hi || key0 + 3 < lo) return z;
  const int page = bt[key0 / ps];
  if (page < 0) return z;
  const bf16_t* p = vt_pool + (((size_t)page * G + g) * HEAD_DIM + dd) * ps + key0 % ps;
  u32x2_t v = *reinterpret_cast<const u32x2_t*>(p);
  int keep = 0;
#pragma unroll
  for (int i = 0; i < 4; ++i)
    if (key0 + i >= lo && key0 + i <= hi) keep |= 1 << i;
  return keep == 15 ? v : mask4(v, keep);
}

// the same with the page already looked up.  The load itself is unconditional (from the pool's
// first page when the keys are not wanted) and its result is masked, so that the compiler
// keeps it in straight-line code and can leave it in flight across other work.
__device__ __forceinline__ u32x2_t load_vt4_pg(const bf16_t* __restrict__ vt_pool, int page, int G,
                                               int g, int ps, int dd, int key0, int lo, int hi) {
  const bool want = dd < HEAD_DIM && key0 <= hi && key0 + 3 >= lo && page >= 0;
  const size_t off =
      want ? (((size_t)page * G + g) * HEAD_DIM + dd) * ps + key0 % ps : (size_t)0;
  u32x2_t v = *reinterpret_cast<const u32x2_t*>(vt_pool + off);
  int keep = 0;
#pragma unroll
  for (int i = 0; i < 4; ++i)
    if (want && key0 + i >= lo && key0 + i <= hi) keep |= 1 << i;
  return mask4(v, keep);
}

// eight key slots of V^T for d index `dd`, keys key0..key0+7 (half a 16-key group: one page),
// the page already looked up; keys outside [lo, hi] read as zero
__device__ __forceinline__ u32x4_t load_vt8_pg(const bf16_t* __restrict__ vt_pool, int page, int G,
                                               int g, int ps, int dd, int key0, int lo, int hi) {
  const bool want = dd < HEAD_DIM && key0 <= hi && key0 + 7 >= lo && page >= 0;
  const size_t off =
      want ? (((size_t)page * G + g) * HEAD_DIM + dd) * ps + key0 % ps : (size_t)0;
  const u32x4_t v = *reinterpret_cast<const u32x4_t*>(vt_pool + off);
  uint32_t m[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const bool k0 = want && key0 + 2 * i >= lo && key0 + 2 * i <= hi;
    const bool k1 = want && key0 + 2 * i + 1 >= lo && key0 + 2 * i + 1 <= hi;
    m[i] = (k0 ? 0x0000ffffu : 0u) | (k1 ? 0xffff0000u : 0u);
  }
  return (u32x4_t){v.x & m[0], v.y & m[1], v.z & m[2], v.w & m[3]};
}

__device__ __forceinline__ u32x4_t load_k8_pg(const bf16_t* __restrict__ k_pool, int page, int G,
                                              int g, int ps, int key, int d0, int lo, int hi) {
  const bool want = d0 < HEAD_DIM && key >= lo && key <= hi && page >= 0;
  const size_t off = want ? (((size_t)page * G + g) * ps + key % ps) * HEAD_DIM + d0 : (size_t)0;
  u32x4_t v = *reinterpret_cast<const u32x4_t*>(k_pool + off);
  const uint32_t m = want ? 0xffffffffu : 0u;
  return (u32x4_t){v.x & m, v.y & m, v.z & m, v.w & m};
}

// eight consecutive d of key `key` starting at d0; zero outside [lo, hi] or beyond the head
__device__ __forceinline__ u32x4_t load_k8(const bf16_t* __restrict__ k_pool,
                                           const int* __restrict__ bt, int G, int g, int ps,
                                           int key, int d0, int lo, int hi) {
  u32x4_t z = {0u, 0u, 0u, 0u};
  if (d0 >= HEAD_DIM || key < lo || key > hi) return z;
  const int page = bt[key / ps];
  if (page < 0) return z;
  return *reinterpret_cast<const u32x4_t*>(
      k_pool + (((size_t)page * G + g) * ps + key % ps) * HEAD_DIM + d0);
}

// ---------------------------------------------------------------------------------------
// prefill: q_tiles[tile] = (segment, first row, rows <= 32, unused)
// ---------------------------------------------------------------------------------------
#define P_KS (HEAD_DIM / 16)            // k-steps of S^T over d
#define P_MT ((HEAD_DIM + 31) / 32)     // row tiles of O^T over d

// waves of a block: they share one q tile and take its key tiles in turn, which shortens the
// longest chain of dependent work fourfold; their partial results meet in LDS
#define P_NW (HEAD_DIM <= 128 ? 4 : 1)

__global__ __launch_bounds__(P_NW * WAVE) void attn_prefill_kernel(
    const bf16_t* __restrict__ q, int q_stride, const bf16_t* __restrict__ k_pool,
    const bf16_t* __restrict__ vt_pool, bf16_t* __restrict__ out, int out_stride,
    const int* __restrict__ q_tiles, const int* __restrict__ row_pos,
    const int* __restrict__ block_tables, int max_blocks, int H, int G, int ps, int window,
    float scale) {
  // later tiles of a segment have more keys: they are started first
  const int tile = gridDim.x - 1 - blockIdx.x, h = blockIdx.y;
  const int lane = threadIdx.x % WAVE;
  // the wave's number in scalar registers: everything that depends only on the key tile (its
  // pages, its base addresses, whether it is masked) is then scalar work
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
  const int seg = q_tiles[4 * tile], r0 = q_tiles[4 * tile + 1], nr = q_tiles[4 * tile + 2];
  const int g = h / (H / G);
  const int col = lane % 32, hh = lane / 32;
  const int* bt = block_tables + (size_t)seg * max_blocks;
  const int pos_first = row_pos[r0], pos_last = pos_first + nr - 1;
  const bool row_ok = col < nr;
  const int my_pos = row_ok ? pos_first + col : -1;
  const int my_lo = (window > 0 && my_pos + 1 > window) ? my_pos + 1 - window : 0;
  const int lo_tile = (window > 0 && pos_first + 1 > window) ? pos_first + 1 - window : 0;

  bf16x8_t qf[P_KS];
  {
    const bf16_t* qr = q + (size_t)(r0 + (row_ok ? col : 0)) * q_stride + (size_t)h * HEAD_DIM;
#pragma unroll
    for (int ks = 0; ks < P_KS; ++ks) {
      u32x4_t v = {0u, 0u, 0u, 0u};
      if (row_ok) v = *reinterpret_cast<const u32x4_t*>(qr + 16 * ks + 8 * hh);
      qf[ks] = as_frag(v);
    }
  }
  f32x16_t o[P_MT];
#pragma unroll
  for (int mt = 0; mt < P_MT; ++mt)
#pragma unroll
    for (int v = 0; v < 16; ++v) o[mt][v] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;
  const float sc = scale * LOG2E;

  // A tile of 32 keys is "whole" when every row of the q tile sees all of its keys: then nothing
  // is masked, and addresses are a base that is the same for all lanes of a 16-key group (its
  // page) plus an offset that a lane computes once.  The tiles at the window's lower edge and at
  // the diagonal take the general path.  Either way the loads of the next tile are issued
  // before the current one is worked on.
  const int lo_last = (window > 0 && pos_last + 1 > window) ? pos_last + 1 - window : 0;
  auto whole = [&](int kb) { return kb >= lo_last && kb + 31 <= pos_first; };
  const int k_lane = (col % 16) * HEAD_DIM + 8 * hh;       // + 16*ks
  const int v_lane = col * ps + 4 * hh;                    // + 32*mt*ps (+ 8)
  constexpr bool P_AHEAD = HEAD_DIM <= 128;      // beyond that the registers do not suffice
  constexpr int P_NB = P_AHEAD ? 2 : 1;
  u32x4_t kfr[P_NB][P_KS];
  u32x2_t vfa[P_NB][2][P_MT], vfb[P_NB][2][P_MT];
  auto fetch = [&](int buf, int kb) {
    const int g0 = min(kb / ps, max_blocks - 1), g1 = min((kb + 16) / ps, max_blocks - 1);
    const int pg0 = kb <= pos_last ? bt[g0] : -1;
    const int pg1 = kb + 16 <= pos_last ? bt[g1] : -1;
    if (whole(kb)) {
      const bf16_t* kb0p = k_pool + (((size_t)pg0 * G + g) * ps + kb % ps) * HEAD_DIM;
      const bf16_t* kb1p = k_pool + (((size_t)pg1 * G + g) * ps + (kb + 16) % ps) * HEAD_DIM;
      const bf16_t* kp = (col < 16 ? kb0p : kb1p) + k_lane;
#pragma unroll
      for (int ks = 0; ks < P_KS; ++ks)
        kfr[buf][ks] = *reinterpret_cast<const u32x4_t*>(kp + 16 * ks);
#pragma unroll
      for (int st = 0; st < 2; ++st) {
        const bf16_t* vp = vt_pool + ((size_t)(st == 0 ? pg0 : pg1) * G + g) * HEAD_DIM * ps +
                           (kb + 16 * st) % ps + v_lane;
#pragma unroll
        for (int mt = 0; mt < P_MT; ++mt) {
          const bool dok = HEAD_DIM % 32 == 0 || 32 * mt + col < HEAD_DIM;
          const bf16_t* vq = vp + (dok ? 32 * mt * ps : -v_lane);
          u32x2_t a = *reinterpret_cast<const u32x2_t*>(vq);
          u32x2_t b = *reinterpret_cast<const u32x2_t*>(vq + 8);
          if (!dok) a = b = (u32x2_t){0u, 0u};
          vfa[buf][st][mt] = a;
          vfb[buf][st][mt] = b;
        }
      }
      return;
    }
    const int my_key = kb + col;
    const int my_pg = col < 16 ? pg0 : pg1;
#pragma unroll
    for (int ks = 0; ks < P_KS; ++ks)
      kfr[buf][ks] =
          load_k8_pg(k_pool, my_pg, G, g, ps, my_key, 16 * ks + 8 * hh, lo_tile, pos_last);
#pragma unroll
    for (int st = 0; st < 2; ++st) {
      const int key0 = kb + 16 * st + 4 * hh;
      const int pg = st == 0 ? pg0 : pg1;
#pragma unroll
      for (int mt = 0; mt < P_MT; ++mt) {
        const int dd = 32 * mt + col;
        vfa[buf][st][mt] = load_vt4_pg(vt_pool, pg, G, g, ps, dd, key0, lo_tile, pos_last);
        vfb[buf][st][mt] = load_vt4_pg(vt_pool, pg, G, g, ps, dd, key0 + 8, lo_tile, pos_last);
      }
    }
  };
  auto work = [&](int buf, int kb) {
    // ---- S^T tile: 32 keys x 32 queries -------------------------------------------------
    f32x16_t s;
#pragma unroll
    for (int v = 0; v < 16; ++v) s[v] = 0.f;
#pragma unroll
    for (int ks = 0; ks < P_KS; ++ks)
      s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_frag(kfr[buf][ks]), qf[ks], s, 0, 0, 0);
    // lane holds, for query `col`, keys kb + 8*(v/4) + 4*hh + v%4
    float mloc = -INFINITY;
    if (whole(kb)) {
#pragma unroll
      for (int v = 0; v < 16; ++v) mloc = fmaxf(mloc, s[v]);
      mloc *= sc;           // sc > 0: scaling commutes with the maximum
    } else {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int key = kb + 8 * (v / 4) + 4 * hh + v % 4;
        const bool ok = key <= my_pos && key >= my_lo;
        s[v] = ok ? s[v] : -INFINITY;
        mloc = fmaxf(mloc, s[v] * sc);
      }
    }
    mloc = fmaxf(mloc, other_half(mloc));
    const float m_new = fmaxf(m_run, mloc);
    const float m_safe = m_new == -INFINITY ? 0.f : m_new;
    const float corr = fast_exp2(m_run - m_safe);
    float lsum = 0.f;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      s[v] = fast_exp2(fmaf(s[v], sc, -m_safe));
      lsum += s[v];
    }
    lsum += other_half(lsum);
    l_run = l_run * corr + lsum;
    m_run = m_new;
#pragma unroll
    for (int mt = 0; mt < P_MT; ++mt)
#pragma unroll
      for (int v = 0; v < 16; ++v) o[mt][v] *= corr;
    // ---- O^T += V^T P^T, two k-steps of 16 keys ---------------------------------------
#pragma unroll
    for (int st = 0; st < 2; ++st) {
      const u32x4_t pw = {pack_bf16(s[8 * st + 0], s[8 * st + 1]),
                          pack_bf16(s[8 * st + 2], s[8 * st + 3]),
                          pack_bf16(s[8 * st + 4], s[8 * st + 5]),
                          pack_bf16(s[8 * st + 6], s[8 * st + 7])};
      const bf16x8_t pf = as_frag(pw);
#pragma unroll
      for (int mt = 0; mt < P_MT; ++mt) {
        const u32x4_t vw = {vfa[buf][st][mt].x, vfa[buf][st][mt].y, vfb[buf][st][mt].x,
                            vfb[buf][st][mt].y};
        o[mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_frag(vw), pf, o[mt], 0, 0, 0);
      }
    }
  };
  // wave w takes the key tiles kb0 + 32 * (w + P_NW * i)
  const int kb0 = (lo_tile / 32) * 32 + 32 * wave;
  constexpr int KSTEP = 32 * P_NW;
  if (P_AHEAD) {
    if (kb0 <= pos_last) fetch(0, kb0);
    for (int kb = kb0; kb <= pos_last; kb += 2 * KSTEP) {
      if (kb + KSTEP <= pos_last) fetch(P_NB - 1, kb + KSTEP);
      work(0, kb);
      if (kb + KSTEP <= pos_last) {
        if (kb + 2 * KSTEP <= pos_last) fetch(0, kb + 2 * KSTEP);
        work(P_NB - 1, kb + KSTEP);
      }
    }
  } else {
    for (int kb = kb0; kb <= pos_last; kb += KSTEP) {
      fetch(0, kb);
      work(0, kb);
    }
  }
  if (P_NW > 1) {
    // merge: every wave rescales to the common maximum; waves 1.. hand their sums to wave 0
    __shared__ float sh_m[P_NW][32], sh_l[P_NW][32];
    __shared__ float sh_o[P_NW > 1 ? P_NW - 1 : 1][P_MT * 16][WAVE];
    if (hh == 0) sh_m[wave][col] = m_run;
    __syncthreads();
    float M = sh_m[0][col];
#pragma unroll
    for (int w = 1; w < P_NW; ++w) M = fmaxf(M, sh_m[w][col]);
    const float f = m_run == -INFINITY ? 0.f : fast_exp2(m_run - M);
    l_run *= f;
    if (hh == 0) sh_l[wave][col] = l_run;
    if (wave > 0) {
#pragma unroll
      for (int mt = 0; mt < P_MT; ++mt)
#pragma unroll
        for (int v = 0; v < 16; ++v) sh_o[wave - 1][mt * 16 + v][lane] = o[mt][v] * f;
    }
    __syncthreads();
    if (wave > 0) return;
    l_run = sh_l[0][col];
#pragma unroll
    for (int w = 1; w < P_NW; ++w) l_run += sh_l[w][col];
#pragma unroll
    for (int mt = 0; mt < P_MT; ++mt)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        float acc = o[mt][v] * f;
#pragma unroll
        for (int w = 1; w < P_NW; ++w) acc += sh_o[w - 1][mt * 16 + v][lane];
        o[mt][v] = acc;
      }
  }
  if (!row_ok) return;
  const float inv = l_run > 0.f ? 1.0f / l_run : 0.f;
  bf16_t* orow = out + (size_t)(r0 + col) * out_stride + (size_t)h * HEAD_DIM;
#pragma unroll
  for (int mt = 0; mt < P_MT; ++mt)
#pragma unroll
    for (int v4 = 0; v4 < 4; ++v4) {
      const int dd = 32 * mt + 8 * v4 + 4 * hh;     // four consecutive d: v = 4*v4 .. 4*v4+3
      if (dd < HEAD_DIM) {
        u32x2_t w = {pack_bf16(o[mt][4 * v4] * inv, o[mt][4 * v4 + 1] * inv),
                     pack_bf16(o[mt][4 * v4 + 2] * inv, o[mt][4 * v4 + 3] * inv)};
        *reinterpret_cast<u32x2_t*>(orow + dd) = w;
      }
    }
}

// ---------------------------------------------------------------------------------------
// prefill, key tiles shared by the query heads of a kv head
// ---------------------------------------------------------------------------------------
// One block = two q tiles (32 rows each) of one segment x four query heads of one kv head, a
// wave each.  The eight waves walk the same key tiles, so a tile of K (32 keys x d) and of V^T
// (d x 32 keys) is brought from global memory once, straight into LDS (global_load_lds, three
// buffers, two tiles ahead), and every wave reads its matrix operands from there.  Pairing an
// early q tile with a late one gives every block the same number of keys to walk.  K rows keep their 16-byte chunks permuted (chunk ^ f(key)) so that the
// 16 keys of a fragment read fall on different banks; V^T lies as [16-key group][d][16 keys],
// every other 8 rows with their two halves of 8 keys swapped, for the same reason.
// The running maximum is only moved when a tile's maximum exceeds it by more than 2^8: most
// tiles then leave the output accumulators alone (no rescaling), and the weights stay <= 256.
#if HEAD_DIM == 64 || HEAD_DIM == 128
#define PG_OK 1
#define PG_NBUF 3
#define PG_SUB 2
template <int N> struct PgBuf { static constexpr int value = N; };
#define PG_GPTR(p) ((const __attribute__((address_space(1))) void*)(p))
#define PG_LPTR(p) ((__attribute__((address_space(3))) void*)(p))

__global__ __launch_bounds__(8 * WAVE) void attn_prefill_shared_kernel(
    const bf16_t* __restrict__ q, int q_stride, const bf16_t* __restrict__ k_pool,
    const bf16_t* __restrict__ vt_pool, bf16_t* __restrict__ out, int out_stride,
    const int* __restrict__ q_tiles, const int* __restrict__ row_pos,
    const int* __restrict__ block_tables, int max_blocks, int H, int G, int ps, int window,
    float scale) {
  constexpr int ROWB = HEAD_DIM * 2;                // bytes of a key's row
  constexpr int KTILE = 32 * ROWB, VGROUP = HEAD_DIM * 32, BUF = KTILE + 2 * VGROUP;   // bytes
  constexpr int CPR = ROWB / 16;                    // 16-byte chunks a K row
  constexpr int K_ROWS_PER = 1024 / ROWB;           // K rows one load instruction brings
  constexpr int NL = 8 / K_ROWS_PER;                // loads a wave issues per tile: a K wave
                                                    // brings 8 keys, a V wave half a 16-key group
  static_assert(NL == (HEAD_DIM / 2) / 32, "K and V waves issue the same number of loads");
  // a buffer holds PG_SUB key tiles: one barrier for that many tiles
  __shared__ __attribute__((aligned(1024))) char lds[PG_NBUF * PG_SUB * BUF];
  const int t_a = gridDim.x - 1 - blockIdx.x;
  // The block's second q tile.  q_tiles[t][3] = (index of the tile within its segment) |
  // (tiles of the segment << 16), 0 if unknown.  Without a window tile j is paired with tile
  // n-1-j, so that every block walks about the same number of keys; with a window, with its
  // neighbour, whose keys are nearly the same.  The later tile of a pair has no block of its own.
  int t_b = -1;
  {
    const int info = q_tiles[4 * t_a + 3];
    const int j = info & 0xffff, n = info >> 16;
    if (n > 0) {
      if (window == 0) {
        if (2 * j > n - 1) return;
        if (2 * j < n - 1) t_b = t_a + (n - 1 - 2 * j);
      } else {
        if (j & 1) return;
        if (j + 1 < n) t_b = t_a + 1;
      }
    }
  }
  const int rep = H / G, quads = rep / 4;
  const int g = blockIdx.y / quads;
  const int lane = threadIdx.x % WAVE;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
  const int grp = wave / 4;                         // 0: tile a, 1: tile b
  const int h = g * rep + (blockIdx.y % quads) * 4 + wave % 4;
  const int tile = grp == 0 ? t_a : t_b;
  const bool has_tile = tile >= 0;
  const int seg = q_tiles[4 * t_a];                 // both tiles are of one segment
  const int r0 = has_tile ? q_tiles[4 * tile + 1] : 0, nr = has_tile ? q_tiles[4 * tile + 2] : 0;
  const int col = lane % 32, hh = lane / 32;
  const int* bt = block_tables + (size_t)seg * max_blocks;
  const int pos_first = row_pos[r0], pos_last = pos_first + nr - 1;
  const bool row_ok = col < nr;
  const int my_pos = row_ok ? pos_first + col : -1;
  const int my_lo = (window > 0 && my_pos + 1 > window) ? my_pos + 1 - window : 0;
  const int lo_tile = (window > 0 && pos_first + 1 > window) ? pos_first + 1 - window : 0;
  const int lo_last = (window > 0 && pos_last + 1 > window) ? pos_last + 1 - window : 0;
  // the keys the block walks: from the first key of either tile to the last key of either
  int blk_first, blk_last;
  {
    const int ra = q_tiles[4 * t_a + 1], pa0 = row_pos[ra], pa1 = pa0 + q_tiles[4 * t_a + 2] - 1;
    blk_first = (window > 0 && pa0 + 1 > window) ? pa0 + 1 - window : 0;
    blk_last = pa1;
    if (t_b >= 0) {
      const int rb = q_tiles[4 * t_b + 1], pb0 = row_pos[rb], pb1 = pb0 + q_tiles[4 * t_b + 2] - 1;
      blk_first = min(blk_first, (window > 0 && pb0 + 1 > window) ? pb0 + 1 - window : 0);
      blk_last = max(blk_last, pb1);
    }
  }

  bf16x8_t qf[P_KS];
  {
    const bf16_t* qr = q + (size_t)(r0 + (row_ok ? col : 0)) * q_stride + (size_t)h * HEAD_DIM;
#pragma unroll
    for (int ks = 0; ks < P_KS; ++ks) {
      u32x4_t v = {0u, 0u, 0u, 0u};
      if (row_ok) v = *reinterpret_cast<const u32x4_t*>(qr + 16 * ks + 8 * hh);
      qf[ks] = as_frag(v);
    }
  }
  f32x16_t o[P_MT];
#pragma unroll
  for (int mt = 0; mt < P_MT; ++mt)
#pragma unroll
    for (int v = 0; v < 16; ++v) o[mt][v] = 0.f;
  // The sums of the weights come from the matrix cores too: a V^T fragment of ones gives a
  // tile whose every row is the sum over the keys, of the same rounded weights the output is made
  // of.  (The kernel is bound by the issue of vector instructions: 16 additions and an exchange
  // between half waves less per tile.)  Only at head size 64: at 128 the 16 registers more spill.
  constexpr bool MFMA_SUM = HEAD_DIM == 64;
  float l_add = 0.f;
  f32x16_t o_sum;
#pragma unroll
  for (int v = 0; v < 16; ++v) o_sum[v] = 0.f;
  const bf16x8_t ones = as_frag((u32x4_t){0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u});
  float m_ref = -INFINITY;
  const float sc = scale * LOG2E;

  const int kbase = (blk_first / 32) * 32;
  const int n_tiles = (blk_last - kbase) / 32 + 1;
  auto swz = [](int key) { return HEAD_DIM == 64 ? (key >> 1) & 7 : key & 15; };
  // what this lane brings: waves 0-3 eight rows of K each, waves 4-7 half a 16-key group of V^T
  const int k_row_in = lane / CPR, k_slot = lane % CPR;
  const int vw = wave - 4, v_st = vw / 2, v_d0 = (vw % 2) * (HEAD_DIM / 2) + lane / 2;
  const int v_half = lane % 2;
  // The buffer of a tile is a compile-time constant (the tile loop is unrolled three times):
  // only then can the compiler tell that the loads it issues into one buffer do not touch
  // the buffer it reads from, and leave them in flight across the reads.
  // Tiles are issued in order, so the wave keeps the place of its next keys (block table
  // index, offset in the page) and looks the next page up one tile ahead; a group past the
  // last key (or given back by the window) is read from the pool's first page instead and
  // masked when it is used.  A wave's keys (8 of K, 16 of V^T) lie in one page.
  int nx_key = kbase + (wave < 4 ? 8 * wave : 16 * v_st);
  int nx_pidx = nx_key / ps, nx_off = nx_key % ps;
  auto lookup = [&]() {
    const int page = nx_key <= blk_last ? bt[min(nx_pidx, max_blocks - 1)] : 0;
    return max(page, 0);
  };
  int nx_page = lookup();
  auto issue_one = [&](char* buf) {
    if (wave < 4) {
      const bf16_t* base = k_pool + (((size_t)nx_page * G + g) * ps + nx_off) * HEAD_DIM;
#pragma unroll
      for (int i = 0; i < NL; ++i) {
        const int row = i * K_ROWS_PER + k_row_in;               // 0..7 within the wave's keys
        const int chunk = k_slot ^ swz(8 * wave + row);
        __builtin_amdgcn_global_load_lds(PG_GPTR(base + row * HEAD_DIM + chunk * 8),
                                         PG_LPTR(buf + (8 * wave + i * K_ROWS_PER) * ROWB), 16, 0,
                                         0);
      }
    } else {
      const bf16_t* base = vt_pool + ((size_t)nx_page * G + g) * HEAD_DIM * ps + nx_off;
#pragma unroll
      for (int i = 0; i < NL; ++i) {
        const int dd = v_d0 + 32 * i;
        // rows 8 apart would meet on the same banks: every other group of 8 rows keeps its two
        // 16-byte halves swapped
        __builtin_amdgcn_global_load_lds(
            PG_GPTR(base + (size_t)dd * ps + 8 * (v_half ^ ((dd >> 3) & 1))),
            PG_LPTR(buf + KTILE + v_st * VGROUP + ((vw % 2) * (HEAD_DIM / 2) + 32 * i) * 32), 16, 0,
            0);
      }
    }
    nx_key += 32;
    nx_off += 32;
    while (nx_off >= ps) {
      nx_off -= ps;
      ++nx_pidx;
    }
    nx_page = lookup();
  };
  auto issue = [&](auto buf_c) {
#pragma unroll
    for (int sub = 0; sub < PG_SUB; ++sub)
      issue_one(lds + (decltype(buf_c)::value * PG_SUB + sub) * BUF);
  };
  auto whole = [&](int kb) { return kb >= lo_last && kb + 31 <= pos_first; };
  auto work = [&](auto buf_c, auto sub_c, int it) {
    const int kb = kbase + 32 * it;
    const char* buf = lds + (decltype(buf_c)::value * PG_SUB + decltype(sub_c)::value) * BUF;
    const bool full = whole(kb);
    // ---- S^T tile: 32 keys x 32 queries -------------------------------------------------
    f32x16_t s;
#pragma unroll
    for (int v = 0; v < 16; ++v) s[v] = 0.f;
#pragma unroll
    for (int ks = 0; ks < P_KS; ++ks) {
      const u32x4_t kf = *reinterpret_cast<const u32x4_t*>(
          buf + col * ROWB + (((2 * ks + hh) ^ swz(col)) * 16));
      s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_frag(kf), qf[ks], s, 0, 0, 0);
    }
    // V^T operands: d index 32*mt + col, keys 16*st + 4*hh .. +3 and 8 more
    u32x2_t va[2][P_MT], vb[2][P_MT];
#pragma unroll
    for (int st = 0; st < 2; ++st)
#pragma unroll
      for (int mt = 0; mt < P_MT; ++mt) {
        const int sw = ((col >> 3) & 1) * 16;      // this row's halves are swapped
        const char* vp = buf + KTILE + st * VGROUP + (32 * mt + col) * 32 + 8 * hh;
        va[st][mt] = *reinterpret_cast<const u32x2_t*>(vp + sw);
        vb[st][mt] = *reinterpret_cast<const u32x2_t*>(vp + (16 - sw));
      }
    // lane holds, for query `col`, keys kb + 8*(v/4) + 4*hh + v%4
    float mloc = -INFINITY;
    if (full) {
#pragma unroll
      for (int v = 0; v < 16; ++v) mloc = fmaxf(mloc, s[v]);
      mloc *= sc;           // sc > 0: scaling commutes with the maximum
    } else {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int key = kb + 8 * (v / 4) + 4 * hh + v % 4;
        const bool ok = key <= my_pos && key >= my_lo;
        s[v] = ok ? s[v] : -INFINITY;
        mloc = fmaxf(mloc, s[v] * sc);
      }
      // what lies in LDS for keys outside the tile's range is not cache content: zero it
#pragma unroll
      for (int st = 0; st < 2; ++st) {
        int keep_a = 0, keep_b = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int ka = kb + 16 * st + 4 * hh + i, kbb = ka + 8;
          if (ka >= lo_tile && ka <= pos_last) keep_a |= 1 << i;
          if (kbb >= lo_tile && kbb <= pos_last) keep_b |= 1 << i;
        }
#pragma unroll
        for (int mt = 0; mt < P_MT; ++mt) {
          va[st][mt] = mask4(va[st][mt], keep_a);
          vb[st][mt] = mask4(vb[st][mt], keep_b);
        }
      }
    }
    mloc = fmaxf(mloc, other_half(mloc));
    // move the reference only when it is far off (or unset): uniform for the wave's branch
    const bool move = mloc > m_ref + 8.0f;
    if (__builtin_amdgcn_ballot_w64(move) != 0) {
      const float m_new = move ? mloc : m_ref;
      const float m_safe = m_new == -INFINITY ? 0.f : m_new;
      const float corr = move ? fast_exp2(m_ref - m_safe) : 1.0f;
      if (MFMA_SUM) {
#pragma unroll
        for (int v = 0; v < 16; ++v) o_sum[v] *= corr;
      } else {
        l_add *= corr;
      }
#pragma unroll
      for (int mt = 0; mt < P_MT; ++mt)
#pragma unroll
        for (int v = 0; v < 16; ++v) o[mt][v] *= corr;
      m_ref = m_new;
    }
    const float m_safe = m_ref == -INFINITY ? 0.f : m_ref;
    float lsum = 0.f;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      s[v] = fast_exp2(fmaf(s[v], sc, -m_safe));
      if (!MFMA_SUM) lsum += s[v];
    }
    if (!MFMA_SUM) {
      lsum += other_half(lsum);
      l_add += lsum;
    }
    // ---- O^T += V^T P^T, two k-steps of 16 keys ---------------------------------------
#pragma unroll
    for (int st = 0; st < 2; ++st) {
      const u32x4_t pw = {pack_bf16(s[8 * st + 0], s[8 * st + 1]),
                          pack_bf16(s[8 * st + 2], s[8 * st + 3]),
                          pack_bf16(s[8 * st + 4], s[8 * st + 5]),
                          pack_bf16(s[8 * st + 6], s[8 * st + 7])};
      const bf16x8_t pf = as_frag(pw);
      if (MFMA_SUM) o_sum = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ones, pf, o_sum, 0, 0, 0);
#pragma unroll
      for (int mt = 0; mt < P_MT; ++mt) {
        const u32x4_t vw4 = {va[st][mt].x, va[st][mt].y, vb[st][mt].x, vb[st][mt].y};
        o[mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_frag(vw4), pf, o[mt], 0, 0, 0);
      }
    }
  };

  // Both tiles of a buffer when neither needs a mask (most steps of a long history): the
  // products of the second tile's scores are issued before the first tile's exponentials, so
  // that the matrix cores work while the vector unit does the softmax of the tile before.
  auto work2 = [&](auto buf_c) {
    const char* buf0 = lds + (decltype(buf_c)::value * PG_SUB) * BUF;
    const char* buf1 = buf0 + BUF;
    auto scores = [&](const char* buf) {
      f32x16_t s;
#pragma unroll
      for (int v = 0; v < 16; ++v) s[v] = 0.f;
#pragma unroll
      for (int ks = 0; ks < P_KS; ++ks) {
        const u32x4_t kf = *reinterpret_cast<const u32x4_t*>(
            buf + col * ROWB + (((2 * ks + hh) ^ swz(col)) * 16));
        s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_frag(kf), qf[ks], s, 0, 0, 0);
      }
      return s;
    };
    // the running reference moves only when a tile's maximum is far above it (rare: a branch)
    auto update_reference = [&](const f32x16_t& s) {
      float mloc = -INFINITY;
#pragma unroll
      for (int v = 0; v < 16; ++v) mloc = fmaxf(mloc, s[v]);
      mloc *= sc;
      mloc = fmaxf(mloc, other_half(mloc));
      const bool move = mloc > m_ref + 8.0f;
      if (__builtin_amdgcn_ballot_w64(move) != 0) {
        const float m_new = move ? mloc : m_ref;
        const float m_safe = m_new == -INFINITY ? 0.f : m_new;
        const float corr = move ? fast_exp2(m_ref - m_safe) : 1.0f;
        if (MFMA_SUM) {
#pragma unroll
          for (int v = 0; v < 16; ++v) o_sum[v] *= corr;
        } else {
          l_add *= corr;
        }
#pragma unroll
        for (int mt = 0; mt < P_MT; ++mt)
#pragma unroll
          for (int v = 0; v < 16; ++v) o[mt][v] *= corr;
        m_ref = m_new;
      }
    };
    auto weights_and_output = [&](const char* buf, f32x16_t s) {
      u32x2_t va[2][P_MT], vb[2][P_MT];
#pragma unroll
      for (int st = 0; st < 2; ++st)
#pragma unroll
        for (int mt = 0; mt < P_MT; ++mt) {
          const int sw = ((col >> 3) & 1) * 16;
          const char* vp = buf + KTILE + st * VGROUP + (32 * mt + col) * 32 + 8 * hh;
          va[st][mt] = *reinterpret_cast<const u32x2_t*>(vp + sw);
          vb[st][mt] = *reinterpret_cast<const u32x2_t*>(vp + (16 - sw));
        }
      const float m_safe = m_ref == -INFINITY ? 0.f : m_ref;
      float lsum = 0.f;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        s[v] = fast_exp2(fmaf(s[v], sc, -m_safe));
        if (!MFMA_SUM) lsum += s[v];
      }
      if (!MFMA_SUM) {
        lsum += other_half(lsum);
        l_add += lsum;
      }
#pragma unroll
      for (int st = 0; st < 2; ++st) {
        const u32x4_t pw = {pack_bf16(s[8 * st + 0], s[8 * st + 1]),
                            pack_bf16(s[8 * st + 2], s[8 * st + 3]),
                            pack_bf16(s[8 * st + 4], s[8 * st + 5]),
                            pack_bf16(s[8 * st + 6], s[8 * st + 7])};
        const bf16x8_t pf = as_frag(pw);
        if (MFMA_SUM) o_sum = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ones, pf, o_sum, 0, 0, 0);
#pragma unroll
        for (int mt = 0; mt < P_MT; ++mt) {
          const u32x4_t vw4 = {va[st][mt].x, va[st][mt].y, vb[st][mt].x, vb[st][mt].y};
          o[mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_frag(vw4), pf, o[mt], 0, 0, 0);
        }
      }
    };
    // the second tile's score products stand between the first tile's maximum and its
    // exponentials: nothing in them depends on the other
    const f32x16_t s0 = scores(buf0);
    update_reference(s0);
    const f32x16_t s1 = scores(buf1);
    weights_and_output(buf0, s0);
    update_reference(s1);
    weights_and_output(buf1, s1);
  };

  // `it` counts buffers' worth of tiles (PG_SUB each)
  const int n_steps = (n_tiles + PG_SUB - 1) / PG_SUB;
  auto step = [&](auto buf_c, int it) {
    constexpr int B = decltype(buf_c)::value;
    // the tiles of this step have landed (this wave's part; the barrier makes it everybody's),
    // those of the next step may still be on their way
    if (it + 1 < n_steps) __builtin_amdgcn_s_waitcnt(0x0F70 | (PG_SUB * NL));
    else __builtin_amdgcn_s_waitcnt(0x0F70);
    __builtin_amdgcn_s_barrier();     // no fence: a fence would wait for the loads in flight
    // step it+2 goes into the buffer of step it-1: everybody is done with it
    if (it + 2 < n_steps) issue(PgBuf<(B + 2) % PG_NBUF>{});
    const int kb = kbase + 32 * PG_SUB * it;
    if (HEAD_DIM == 64 && has_tile && whole(kb) && whole(kb + 32)) {   // (128: registers spill)
      work2(buf_c);
      return;
    }
    if (has_tile && kb + 31 >= lo_tile && kb <= pos_last) work(buf_c, PgBuf<0>{}, PG_SUB * it);
    if (has_tile && kb + 63 >= lo_tile && kb + 32 <= pos_last)
      work(buf_c, PgBuf<1>{}, PG_SUB * it + 1);
  };
  static_assert(PG_SUB == 2, "the step works on two tiles");
  issue(PgBuf<0>{});
  if (n_steps > 1) issue(PgBuf<1>{});
  for (int it = 0; it < n_steps; it += PG_NBUF) {
    step(PgBuf<0>{}, it);
    if (it + 1 < n_steps) step(PgBuf<1>{}, it + 1);
    if (it + 2 < n_steps) step(PgBuf<2>{}, it + 2);
  }
  if (!row_ok) return;
  const float l_run = MFMA_SUM ? o_sum[0] : l_add;
  const float inv = l_run > 0.f ? 1.0f / l_run : 0.f;
  bf16_t* orow = out + (size_t)(r0 + col) * out_stride + (size_t)h * HEAD_DIM;
#pragma unroll
  for (int mt = 0; mt < P_MT; ++mt)
#pragma unroll
    for (int v4 = 0; v4 < 4; ++v4) {
      const int dd = 32 * mt + 8 * v4 + 4 * hh;     // four consecutive d: v = 4*v4 .. 4*v4+3
      u32x2_t w = {pack_bf16(o[mt][4 * v4] * inv, o[mt][4 * v4 + 1] * inv),
                   pack_bf16(o[mt][4 * v4 + 2] * inv, o[mt][4 * v4 + 3] * inv)};
      *reinterpret_cast<u32x2_t*>(orow + dd) = w;
    }
}
#else
#define PG_OK 0
#endif

// ---------------------------------------------------------------------------------------
// decode: one row a request; columns are the query heads of one kv head (at most 16)
// ---------------------------------------------------------------------------------------
#define D_KS ((HEAD_DIM + 31) / 32)     // k-steps of S^T over d (32 each)
#define D_MT (HEAD_DIM / 16)            // row tiles of O^T over d
// keys whose loads a wave has in flight at once (their registers: keys * HEAD_DIM / 64)
#define D_KPW (HEAD_DIM <= 64 ? 128 : (HEAD_DIM <= 128 ? 64 : 32))

// head sizes whose decode kernel can take the prologue below: the rotation's partner d / 2 further
// must lie in the same lane, and the registers must hold it beside a chunk of keys
#define D_QK_FUSABLE (HEAD_DIM % 64 == 0 && HEAD_DIM <= 128)

// The per-head RMSNorm, the rotation and the storing of a decoded row's own key and value, done in
// the attention kernel's prologue instead of a kernel of their own (kappai: QK-norm, then RoPE,
// then the cache write, src/models/lfm.c:36-44).  For head sizes of 64 and 128; rotate-half over
// the whole head.
struct QkFuse {
  int on;                   // 0: q is ready and the row's key and value are in the pools
  int kv;                   // the row's own key and value come from the projection beside q (k of
                            // kv head g at column (H + g) d, v at (H + G + g) d) and go to the pools
  const float* q_norm_w;    // [d] or null
  const float* k_norm_w;
  float eps;
  const float* cos_tab;     // [positions][d / 2], or null: no rotation
  const float* sin_tab;
  bf16_t* k_pool_w;         // the pools once more, to be written
  bf16_t* vt_pool_w;
};

// What the prologue reads beside the projection, asked for before the first keys so that it has
// arrived when they have: the lane's norm weights at d = 32 ks + 8 kg and, for the first half of
// the head, the cosines and sines of its position.
struct QkTables {
  float wq[(HEAD_DIM + 31) / 32][8], wk[(HEAD_DIM + 31) / 32][8];
  float cs[(HEAD_DIM + 63) / 64][8], sn[(HEAD_DIM + 63) / 64][8];
};

__device__ __forceinline__ void load8f(const float* __restrict__ p, float (&v)[8]) {
  const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}

__device__ __forceinline__ void qk_load_tables(const QkFuse& qk, int pos, int kg, QkTables& tb) {
  constexpr int KS = (HEAD_DIM + 31) / 32, HALF = HEAD_DIM / 2;
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    if (qk.q_norm_w != nullptr) load8f(qk.q_norm_w + 32 * ks + 8 * kg, tb.wq[ks]);
    if (qk.k_norm_w != nullptr && qk.kv) load8f(qk.k_norm_w + 32 * ks + 8 * kg, tb.wk[ks]);
  }
  if (qk.cos_tab != nullptr) {
#pragma unroll
    for (int ks = 0; ks < KS / 2; ++ks) {
      load8f(qk.cos_tab + (size_t)pos * HALF + 32 * ks + 8 * kg, tb.cs[ks]);
      load8f(qk.sin_tab + (size_t)pos * HALF + 32 * ks + 8 * kg, tb.sn[ks]);
    }
  }
}

// raw[ks] = the lane's eight values at d = 32 ks + 8 kg of one head; returns them normalised over
// the head (the four lanes kg = 0..3 with the same lane % 16 hold a head together), weighted
// (w: the lane's weights, when has_w) and rotated (cs, sn, when rotate), rounded to bfloat16
__device__ __forceinline__ void qk_norm_rotate(u32x4_t (&raw)[(HEAD_DIM + 31) / 32], bool has_w,
                                               const float (&w)[(HEAD_DIM + 31) / 32][8], float eps,
                                               bool rotate,
                                               const float (&cs)[(HEAD_DIM + 63) / 64][8],
                                               const float (&sn)[(HEAD_DIM + 63) / 64][8]) {
  constexpr int KS = (HEAD_DIM + 31) / 32;
  float x[KS][8];
  float ss = 0.f;
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    const uint32_t r[4] = {raw[ks].x, raw[ks].y, raw[ks].z, raw[ks].w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      x[ks][2 * i] = __uint_as_float(r[i] << 16);
      x[ks][2 * i + 1] = __uint_as_float(r[i] & 0xffff0000u);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) ss = fmaf(x[ks][i], x[ks][i], ss);
  }
  ss += __shfl_xor(ss, 16, WAVE);
  ss += other_half(ss);
  if (has_w) {
    const float sc = 1.0f / sqrtf(ss / (float)HEAD_DIM + eps);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int i = 0; i < 8; ++i) x[ks][i] = x[ks][i] * sc * w[ks][i];
  }
  if (rotate) {
#pragma unroll
    for (int ks = 0; ks < KS / 2; ++ks)
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float lo = x[ks][i], hi = x[ks + KS / 2][i];
        x[ks][i] = lo * cs[ks][i] - hi * sn[ks][i];
        x[ks + KS / 2][i] = lo * sn[ks][i] + hi * cs[ks][i];
      }
  }
#pragma unroll
  for (int ks = 0; ks < KS; ++ks)
    raw[ks] = (u32x4_t){pack_bf16(x[ks][0], x[ks][1]), pack_bf16(x[ks][2], x[ks][3]),
                        pack_bf16(x[ks][4], x[ks][5]), pack_bf16(x[ks][6], x[ks][7])};
}

// One wave's share of a row's attention: the query heads of kv head g (columns) against the keys
// of the chunks c0 = first, first + stride, ... below k_end (D_KPW keys each), with a running
// maximum and sum per column.  Leaves the unnormalised output in o (lane: column lane % 16, d
// rows 16 mt + 4 (lane / 16) + v), the maximum (in units of log 2) in m_run, the sum in l_run.
template <bool FUSABLE>
__device__ __forceinline__ void attn_decode_wave(
    const bf16_t* __restrict__ q, int q_stride, const bf16_t* __restrict__ k_pool,
    const bf16_t* __restrict__ vt_pool, const int* __restrict__ bt, int max_blocks, int t, int g,
    int H, int G, int ps, float scale, int lo, int hi, int first, int stride, int k_end,
    f32x4_t (&o)[D_MT], float& m_run, float& l_run, const QkFuse& qk, int pos) {
  const int lane = threadIdx.x % WAVE;
  const int rep = H / G;
  const int col = lane % 16, kg = lane / 16;
  const bool head_ok = col < rep;
  const int h = g * rep + (head_ok ? col : 0);
  // the page ids of the first chunk of keys: asked for before anything else, so that the keys
  // can be asked for as soon as they are there, whatever else is still on its way
  auto ask_pages = [&](int c0) {
    const int first_page = c0 / ps;
    int my_page = -1;
    if (first_page + lane < max_blocks && (first_page + lane) * ps <= hi)
      my_page = bt[first_page + lane];
    return my_page;
  };
  int pages_first = first < k_end ? ask_pages(first) : -1;
  bf16x8_t qf[D_KS];
  u32x4_t qraw[D_KS];
  u32x4_t k_new[D_KS];                 // the row's own key, in the K fragment's order of d
  uint32_t v_new[D_MT];                // its value at d = 16 mt + col
  QkTables tb;
  const bool fused = FUSABLE && D_QK_FUSABLE && qk.on;
  const bool own_kv = fused && qk.kv;
  {
    const bf16_t* row = q + (size_t)t * q_stride;
    const bf16_t* qr = row + (size_t)h * HEAD_DIM;
#pragma unroll
    for (int ks = 0; ks < D_KS; ++ks) {
      u32x4_t v = {0u, 0u, 0u, 0u};
      const int d0 = 32 * ks + 8 * kg;
      if (head_ok && d0 < HEAD_DIM) v = *reinterpret_cast<const u32x4_t*>(qr + d0);
      qraw[ks] = v;
    }
    if constexpr (FUSABLE && D_QK_FUSABLE) {
      if (fused) {
        // everything the prologue needs is asked for here; it is worked on when the first keys
        // have been asked for as well
        if (own_kv) {
          const bf16_t* kr = row + (size_t)(H + g) * HEAD_DIM;
          const bf16_t* vr = row + (size_t)(H + G + g) * HEAD_DIM;
#pragma unroll
          for (int ks = 0; ks < D_KS; ++ks)
            k_new[ks] = *reinterpret_cast<const u32x4_t*>(kr + 32 * ks + 8 * kg);
#pragma unroll
          for (int mt = 0; mt < D_MT; ++mt) v_new[mt] = vr[16 * mt + col];
        }
        qk_load_tables(qk, pos, kg, tb);
      }
    }
    if (!fused) {
#pragma unroll
      for (int ks = 0; ks < D_KS; ++ks) qf[ks] = as_frag(qraw[ks]);
    }
  }
  bool prologue_due = fused;
  // the wave whose chunks hold the row's own position puts its key and value into the pools
  const bool owner = own_kv && pos >= first && pos < k_end &&
                     ((pos - first) / D_KPW) % (stride / D_KPW) == 0;
#pragma unroll
  for (int mt = 0; mt < D_MT; ++mt) o[mt] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
  m_run = -INFINITY;
  l_run = 0.f;
  const float sc = scale * LOG2E;

  // A wave takes its keys in chunks of D_KPW: first the chunk's page ids (one load, handed
  // round by shuffles), then every key and value load of the chunk at once (16 bytes a lane
  // each), then the matrix products and the softmax: two memory round trips a chunk, whatever
  // its length.  (Two chunks' loads in flight at once were measured: the registers they take
  // halve the waves a SIMD holds, and 64 requests at 4096 keys took 140 us instead of 100.)
  constexpr int NCH = D_KPW / 32;
  struct Chunk {
    u32x4_t kf[NCH][2][D_KS];
    u32x4_t vv[NCH][D_MT];
  };
  auto ask = [&](int c0, int my_page, Chunk& ch) {
    const int first_page = c0 / ps;
    // Row r of the key tile tt (of the 32 keys from kb) is key kb + 8 (r / 4) + 4 tt + r % 4:
    // the lane that holds rows 4 kg .. 4 kg + 3 of both tiles' scores then holds the keys
    // kb + 8 kg .. + 7 in order, and their values are ONE 16-byte piece of a V^T row.
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
      const int kb = c0 + 32 * c;
#pragma unroll
      for (int tt = 0; tt < 2; ++tt) {
        const int key = kb + 8 * (col / 4) + 4 * tt + col % 4;
        const int page = __shfl(my_page, min(key / ps - first_page, WAVE - 1), WAVE);
#pragma unroll
        for (int ks = 0; ks < D_KS; ++ks)
          ch.kf[c][tt][ks] = load_k8_pg(k_pool, page, G, g, ps, key, 32 * ks + 8 * kg, lo, hi);
      }
      const int pv = __shfl(my_page, min((kb + 8 * kg) / ps - first_page, WAVE - 1), WAVE);
#pragma unroll
      for (int mt = 0; mt < D_MT; ++mt)
        ch.vv[c][mt] = load_vt8_pg(vt_pool, pv, G, g, ps, 16 * mt + col, kb + 8 * kg, lo, hi);
    }
  };
  // the pools do not hold the row's own key and value yet (or only just): the chunk that holds
  // the row's position takes them from the registers
  auto own = [&](int c0, Chunk& ch) {
    if (!(own_kv && pos >= c0 && pos < c0 + D_KPW)) return;
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
      const int kb = c0 + 32 * c;
#pragma unroll
      for (int tt = 0; tt < 2; ++tt) {
        if (kb + 8 * (col / 4) + 4 * tt + col % 4 == pos) {
#pragma unroll
          for (int ks = 0; ks < D_KS; ++ks) ch.kf[c][tt][ks] = k_new[ks];
        }
      }
      const int e = pos - (kb + 8 * kg);
      if (e >= 0 && e < 8) {
        const uint32_t keep = (e & 1) ? 0x0000ffffu : 0xffff0000u;
#pragma unroll
        for (int mt = 0; mt < D_MT; ++mt) {
          const uint32_t put = (v_new[mt] & 0xffffu) << ((e & 1) * 16);
          uint32_t w[4] = {ch.vv[c][mt].x, ch.vv[c][mt].y, ch.vv[c][mt].z, ch.vv[c][mt].w};
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (i == e / 2) w[i] = (w[i] & keep) | put;
          ch.vv[c][mt] = (u32x4_t){w[0], w[1], w[2], w[3]};
        }
      }
    }
  };
  auto work = [&](int c0, const Chunk& ch) {
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
      const int kb = c0 + 32 * c;
      if (kb >= k_end) break;
      f32x4_t s[2];
#pragma unroll
      for (int tt = 0; tt < 2; ++tt) {
        s[tt] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < D_KS; ++ks)
          s[tt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_frag(ch.kf[c][tt][ks]), qf[ks], s[tt],
                                                          0, 0, 0);
      }
      // lane holds, for head `col`, keys kb + 8*kg + 4*tt + v
      float mloc = -INFINITY;
#pragma unroll
      for (int tt = 0; tt < 2; ++tt)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const int key = kb + 8 * kg + 4 * tt + v;
          const bool ok = key >= lo && key <= hi;
          s[tt][v] = ok ? s[tt][v] * sc : -INFINITY;
          mloc = fmaxf(mloc, s[tt][v]);
        }
      mloc = fmaxf(mloc, __shfl_xor(mloc, 16, WAVE));
      mloc = fmaxf(mloc, other_half(mloc));
      const float m_new = fmaxf(m_run, mloc);
      const float m_safe = m_new == -INFINITY ? 0.f : m_new;
      const float corr = fast_exp2(m_run - m_safe);
      float lsum = 0.f;
#pragma unroll
      for (int tt = 0; tt < 2; ++tt)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          s[tt][v] = fast_exp2(s[tt][v] - m_safe);
          lsum += s[tt][v];
        }
      lsum += __shfl_xor(lsum, 16, WAVE);
      lsum += other_half(lsum);
      l_run = l_run * corr + lsum;
      m_run = m_new;
      const u32x4_t pw = {pack_bf16(s[0][0], s[0][1]), pack_bf16(s[0][2], s[0][3]),
                          pack_bf16(s[1][0], s[1][1]), pack_bf16(s[1][2], s[1][3])};
      const bf16x8_t pf = as_frag(pw);
#pragma unroll
      for (int mt = 0; mt < D_MT; ++mt) {
        o[mt] = o[mt] * corr;
        o[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_frag(ch.vv[c][mt]), pf, o[mt], 0, 0, 0);
      }
    }
  };
  for (int c0 = first; c0 < k_end; c0 += stride) {
    Chunk ca;
    ask(c0, c0 == first ? pages_first : ask_pages(c0), ca);
    if constexpr (FUSABLE && D_QK_FUSABLE) {
      if (prologue_due) {
        prologue_due = false;
        if (own_kv) qk_norm_rotate(k_new, qk.k_norm_w != nullptr, tb.wk, qk.eps,
                                   qk.cos_tab != nullptr, tb.cs, tb.sn);
        qk_norm_rotate(qraw, qk.q_norm_w != nullptr, tb.wq, qk.eps, qk.cos_tab != nullptr, tb.cs,
                       tb.sn);
#pragma unroll
        for (int ks = 0; ks < D_KS; ++ks)
          qf[ks] = as_frag(head_ok ? qraw[ks] : (u32x4_t){0u, 0u, 0u, 0u});
        if (owner) {
          const size_t pg = (size_t)bt[pos / ps] * G + g;
          if (col == 0) {
#pragma unroll
            for (int ks = 0; ks < D_KS; ++ks)
              *reinterpret_cast<u32x4_t*>(qk.k_pool_w + (pg * ps + pos % ps) * HEAD_DIM + 32 * ks +
                                          8 * kg) = k_new[ks];
          }
          if (kg == 0) {
#pragma unroll
            for (int mt = 0; mt < D_MT; ++mt)
              qk.vt_pool_w[(pg * HEAD_DIM + 16 * mt + col) * ps + pos % ps] = (bf16_t)v_new[mt];
          }
        }
      }
    }
    own(c0, ca);
    work(c0, ca);
  }
}

// How many keys a split takes in this step.  The host sizes the grid for up to n_splits splits of
// at least kps_min keys from the step's longest context; what the rows really hold decides here:
// as many keys a split that the rows' keys together give D_TARGET_WAVES waves work (requests of
// mixed lengths then get shorter splits than their longest context alone would give them, and
// no wave walks a long row's keys by itself while the rest of the chip has nothing to do), and
// no fewer than the longest row needs to fit into n_splits.  Every wave of the step computes the
// same number from the same table; splits past a row's keys do nothing and are not merged.
#define D_TARGET_WAVES 2048
__device__ __forceinline__ int keys_of_row(int pos, int window) {
  const int lo = (window > 0 && pos + 1 > window) ? pos + 1 - window : 0;
  return pos + 1 - (lo / 32) * 32;
}
__device__ __forceinline__ int step_keys_per_split(const int* __restrict__ row_pos,
                                                   const int* __restrict__ row_ids, int n_rows,
                                                   int window, int G, int kps_min, int n_splits) {
  const int lane = threadIdx.x % WAVE;
  int total32 = 0, longest = 0;                  // the sum in units of 32 keys, rounded up by row
  for (int i = lane; i < n_rows; i += WAVE) {
    const int n = keys_of_row(row_pos[row_ids ? row_ids[i] : i], window);
    total32 += (n + 31) / 32;
    longest = max(longest, n);
  }
  total32 = wave_sum(total32);
  longest = wave_max(longest);
  const long long want = ((long long)total32 * G * 32 + D_TARGET_WAVES - 1) / D_TARGET_WAVES;
  int kps = want > (1 << 30) ? (1 << 30) : (int)want;
  kps = max(kps, (longest + n_splits - 1) / n_splits);
  kps = max(kps, kps_min);
  return (kps + D_KPW - 1) / D_KPW * D_KPW;
}

// The keys of a row split over blocks: block (t, g, split) is one wave that takes the keys
// k_begin + split * kps .. (kps: step_keys_per_split, at least the caller's keys_per_split) and
// writes its partial result; attn_merge adds up those of the splits that had keys.
// (FUSED: with the prologue of QkFuse; a kernel of its own, because the prologue's registers would
// halve the waves a SIMD holds for the steps that do not use it)
// (PLAN: the keys per split come from step_keys_per_split, else they are the caller's: a kernel of
// its own, because the rule's code costs half a microsecond even where it is skipped)
template <bool FUSED, bool PLAN>
__global__ __launch_bounds__(64) void attn_decode_kernel(
    const bf16_t* __restrict__ q, int q_stride, const bf16_t* __restrict__ k_pool,
    const bf16_t* __restrict__ vt_pool, float* __restrict__ part_o, float* __restrict__ part_ml,
    const int* __restrict__ row_pos, const int* __restrict__ row_seg,
    const int* __restrict__ block_tables, int max_blocks, int H, int G, int ps, int window,
    float scale, int keys_per_split, int n_splits, QkFuse qk, const int* __restrict__ row_ids) {
  // (row_ids: the kernel's rows are these rows of the step, partial results are kept by their
  // place in the list)
  // Blocks go to the CUs in the order of their numbers, the row's number fastest: with a number
  // of rows that divides the number of CUs, a CU would get the same row in every (kv head,
  // split), and rows of different lengths would load the CUs unevenly.  Hence the rows are
  // taken in an order that turns with the kv head and the split.
  const int g = blockIdx.y, split = blockIdx.z, lane = threadIdx.x;
  const int ti = (int)((blockIdx.x + 7u * (blockIdx.y + gridDim.y * blockIdx.z)) % gridDim.x);
  const int t = row_ids ? row_ids[ti] : ti;
  const int rep = H / G;
  const int col = lane % 16, kg = lane / 16;
  const int pos = row_pos[t];
  const int seg = row_seg[t];
  const int kps = PLAN ? step_keys_per_split(row_pos, row_ids, (int)gridDim.x, window, G,
                                             keys_per_split, n_splits)
                       : keys_per_split;
  const int* bt = block_tables + (size_t)seg * max_blocks;
  const int lo = (window > 0 && pos + 1 > window) ? pos + 1 - window : 0;
  const int k_begin = (lo / 32) * 32 + split * kps;
  if (k_begin > pos) return;                                   // a split past the row's keys
  const int k_end = min(k_begin + kps, pos + 1);                // exclusive
  const bool head_ok = col < rep;
  const int h = g * rep + (head_ok ? col : 0);
  const size_t pbase = ((size_t)ti * H + h) * n_splits + split;
  f32x4_t o[D_MT];
  float m_run, l_run;
  attn_decode_wave<FUSED>(q, q_stride, k_pool, vt_pool, bt, max_blocks, t, g, H, G, ps, scale, lo,
                          k_end - 1, k_begin, D_KPW, k_end, o, m_run, l_run, qk, pos);
  if (!head_ok) return;
  if (kg == 0) {
    part_ml[2 * pbase] = m_run;
    part_ml[2 * pbase + 1] = l_run;
  }
  float* po = part_o + pbase * HEAD_DIM;
#pragma unroll
  for (int mt = 0; mt < D_MT; ++mt)
    *reinterpret_cast<f32x4_t*>(po + 16 * mt + 4 * kg) = o[mt];
}

// (eight waves at most: a wave keeps a whole chunk's loads in registers, which 16 waves a block
// would not leave room for)
#define D_BLOCK_MAX_WAVES 8
// The keys of a row split over the waves of one block (t, g): wave w takes the chunks w, w + NW,
// ... of D_KPW keys, the waves' results meet in LDS and are added up there in the order of the
// waves, so that nothing goes through memory and no second kernel is needed.  The split of a row's
// keys depends on the row's own position and on the number of waves only.  For batches with
// (rows x kv heads) enough to fill the chip, or contexts short enough for one block.
// LDS: sh_o [NW][rep][HEAD_DIM], then sh_m [NW][16], sh_l [NW][16] (floats).
__global__ __launch_bounds__(D_BLOCK_MAX_WAVES * WAVE) void attn_decode_block_kernel(
    const bf16_t* __restrict__ q, int q_stride, const bf16_t* __restrict__ k_pool,
    const bf16_t* __restrict__ vt_pool, bf16_t* __restrict__ out, int out_stride,
    const int* __restrict__ row_pos, const int* __restrict__ row_seg,
    const int* __restrict__ block_tables, int max_blocks, int H, int G, int ps, int window,
    float scale) {
  extern __shared__ float sh_dec[];
  const int t = blockIdx.x, g = blockIdx.y;
  const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE, NW = blockDim.x / WAVE;
  const int rep = H / G;
  const int col = lane % 16, kg = lane / 16;
  const int pos = row_pos[t];
  const int* bt = block_tables + (size_t)row_seg[t] * max_blocks;
  const int lo = (window > 0 && pos + 1 > window) ? pos + 1 - window : 0;
  const int k_begin = (lo / 32) * 32;
  const int k_end = pos + 1;
  f32x4_t o[D_MT];
  float m_run, l_run;
  // (without the prologue: eight waves a block leave no registers for it, and every wave would
  // do it again)
  attn_decode_wave<false>(q, q_stride, k_pool, vt_pool, bt, max_blocks, t, g, H, G, ps, scale, lo,
                          pos, k_begin + wave * D_KPW, NW * D_KPW, k_end, o, m_run, l_run,
                          QkFuse{}, pos);
  float* sh_o = sh_dec;
  float* sh_m = sh_dec + (size_t)NW * rep * HEAD_DIM;
  float* sh_l = sh_m + NW * 16;
  if (col < rep) {
    float* po = sh_o + ((size_t)wave * rep + col) * HEAD_DIM;
#pragma unroll
    for (int mt = 0; mt < D_MT; ++mt)
      *reinterpret_cast<f32x4_t*>(po + 16 * mt + 4 * kg) = o[mt];
    if (kg == 0) {
      sh_m[wave * 16 + col] = m_run;
      sh_l[wave * 16 + col] = l_run;
    }
  }
  __syncthreads();
  // out[t, g rep + c, e] for (c, e) in turn over the block's threads
  for (int i = threadIdx.x; i < rep * HEAD_DIM; i += blockDim.x) {
    const int c = i / HEAD_DIM, e = i % HEAD_DIM;
    float M = -INFINITY;
    for (int w = 0; w < NW; ++w) M = fmaxf(M, sh_m[w * 16 + c]);
    float L = 0.f, acc = 0.f;
    for (int w = 0; w < NW; ++w) {
      const float m = sh_m[w * 16 + c];
      const float wgt = m == -INFINITY ? 0.f : fast_exp2(m - M);
      L += sh_l[w * 16 + c] * wgt;
      acc = fmaf(sh_o[((size_t)w * rep + c) * HEAD_DIM + e], wgt, acc);
    }
    const float inv = L > 0.f ? 1.0f / L : 0.f;
    out[(size_t)t * out_stride + (size_t)(g * rep + c) * HEAD_DIM + e] = f32_to_bf16(acc * inv);
  }
}

// out[t, h, :] = sum_s o_s 2^(m_s - M) / sum_s l_s 2^(m_s - M).  Four waves share the splits
// (wave w takes s = w, w+4, ...); each computes its splits' weights one per lane.  The partial
// outputs of MERGE_AHEAD splits are asked for before the maxima, so that with up to 32 splits
// the kernel waits for memory once.
#define MERGE_WAVES 4
#define MERGE_AHEAD 8
__global__ __launch_bounds__(MERGE_WAVES * WAVE) void attn_merge_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_ml,
    bf16_t* __restrict__ out, int out_stride, int H, int splits_stride,
    const int* __restrict__ row_ids, const int* __restrict__ row_pos, int window, int G,
    int kps_min, int planned) {
  constexpr int NPL = (HEAD_DIM + WAVE - 1) / WAVE;
  __shared__ float sh_acc[MERGE_WAVES][NPL * WAVE];
  __shared__ float sh_l[MERGE_WAVES];
  const int t = row_ids ? row_ids[blockIdx.x] : blockIdx.x, h = blockIdx.y;
  const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
  const size_t base = ((size_t)blockIdx.x * H + h) * splits_stride;
  // the partial outputs of this wave's splits number j .. j + MERGE_AHEAD - 1, of the first
  // `bound` splits
  float o[MERGE_AHEAD][NPL];
  auto ask = [&](int j, int bound) {
#pragma unroll
    for (int k = 0; k < MERGE_AHEAD; ++k) {
      const int sk = wave + MERGE_WAVES * (j + k);
#pragma unroll
      for (int i = 0; i < NPL; ++i) {
        const int e = lane + i * WAVE;
        o[k][i] = (sk < bound && e < HEAD_DIM) ? part_o[(base + sk) * HEAD_DIM + e] : 0.f;
      }
    }
  };
  // The first partial outputs and maxima are asked for before the number of splits that had keys
  // is known (it takes the row's position): whatever the grid has room for is loaded, and what
  // lies past the row's splits (never written, or by an earlier step) is dropped afterwards.
  ask(0, splits_stride);
  const float m_first = lane < splits_stride ? part_ml[2 * (base + lane)] : -INFINITY;
  float2 ml_first = make_float2(-INFINITY, 0.f);        // of the split wave + MERGE_WAVES * lane
  if (wave + MERGE_WAVES * lane < splits_stride)
    ml_first = *reinterpret_cast<const float2*>(part_ml + 2 * (base + wave + MERGE_WAVES * lane));
  // the splits of this row that had keys (the decode kernel's own rule)
  const int kps = planned ? step_keys_per_split(row_pos, row_ids, (int)gridDim.x, window, G,
                                                kps_min, splits_stride)
                          : kps_min;
  const int n_splits = (keys_of_row(row_pos[t], window) + kps - 1) / kps;
#pragma unroll
  for (int k = 0; k < MERGE_AHEAD; ++k)
#pragma unroll
    for (int i = 0; i < NPL; ++i)
      if (wave + MERGE_WAVES * k >= n_splits) o[k][i] = 0.f;
  float M = lane < n_splits ? m_first : -INFINITY;
  for (int s = lane + WAVE; s < n_splits; s += WAVE) M = fmaxf(M, part_ml[2 * (base + s)]);
  M = wave_max(M);
  float L = 0.f;
  float acc[NPL];
#pragma unroll
  for (int i = 0; i < NPL; ++i) acc[i] = 0.f;
  // this wave's splits, 64 at a time: split index s = wave + MERGE_WAVES * j
  for (int j0 = 0; wave + MERGE_WAVES * j0 < n_splits; j0 += WAVE) {
    const int s = wave + MERGE_WAVES * (j0 + lane);
    float wgt = 0.f, l = 0.f;
    if (s < n_splits) {
      const float2 ml = j0 == 0 ? ml_first
                                : *reinterpret_cast<const float2*>(part_ml + 2 * (base + s));
      wgt = ml.x == -INFINITY ? 0.f : fast_exp2(ml.x - M);
      l = ml.y * wgt;
    }
    L += wave_sum(l);
    for (int k0 = 0; k0 < WAVE; k0 += MERGE_AHEAD) {
      if (wave + MERGE_WAVES * (j0 + k0) >= n_splits) break;
      if (j0 + k0 > 0) ask(j0 + k0, n_splits);
#pragma unroll
      for (int k = 0; k < MERGE_AHEAD; ++k) {
        // a split past the end has the weight 0 and the partial output 0
        const float wk = __shfl(wgt, k0 + k, WAVE);
#pragma unroll
        for (int i = 0; i < NPL; ++i) acc[i] = fmaf(o[k][i], wk, acc[i]);
      }
    }
  }
#pragma unroll
  for (int i = 0; i < NPL; ++i) sh_acc[wave][i * WAVE + lane] = acc[i];
  if (lane == 0) sh_l[wave] = L;
  __syncthreads();
  if (wave != 0) return;
  L = (sh_l[0] + sh_l[1]) + (sh_l[2] + sh_l[3]);
  const float inv = L > 0.f ? 1.0f / L : 0.f;
  bf16_t* dst = out + (size_t)t * out_stride + (size_t)h * HEAD_DIM;
#pragma unroll
  for (int i = 0; i < NPL; ++i) {
    const int e = lane + i * WAVE;
    const float v = (sh_acc[0][i * WAVE + lane] + sh_acc[1][i * WAVE + lane]) +
                    (sh_acc[2][i * WAVE + lane] + sh_acc[3][i * WAVE + lane]);
    if (e < HEAD_DIM) dst[e] = f32_to_bf16(v * inv);
  }
}

extern "C" int kappai_attn_keys_per_wave(void) { return D_KPW; }

// Waves of a block of the decode kernel that merges in LDS, for `rep` query heads a kv head:
// as many as 64 KB of LDS hold partial results for (D_BLOCK_MAX_WAVES at most), 0 if not even two.
extern "C" int kappai_attn_decode_block_waves(int rep) {
  if (rep < 1 || rep > 16) return 0;
  const int per_wave = (rep * HEAD_DIM + 32) * (int)sizeof(float);
  int nw = (64 * 1024) / per_wave;
  nw = nw > D_BLOCK_MAX_WAVES ? D_BLOCK_MAX_WAVES : nw;
  return nw >= 2 ? nw : 0;
}

// Decode attention with the keys of a row split over the `n_waves` waves of one block per (row, kv
// head); no workspace, no second kernel.
extern "C" int kappai_attn_decode_block(const void* q, int q_stride, const void* k_pool,
                                        const void* vt_pool, void* out, int out_stride,
                                        const int* row_pos, const int* row_seg,
                                        const int* block_tables, int max_blocks, int T, int H,
                                        int G, int ps, int window, float scale, int n_waves,
                                        hipStream_t stream) {
  if (T <= 0) return 0;
  if (ps % 16 || G < 1 || H % G || H / G > 16 || G > 65535 || (q_stride % 8) || n_waves < 1 ||
      n_waves > kappai_attn_decode_block_waves(H / G))
    return (int)hipErrorInvalidValue;
  const int rep = H / G;
  const size_t lds = (size_t)n_waves * (rep * HEAD_DIM + 32) * sizeof(float);
  hipLaunchKernelGGL(attn_decode_block_kernel, dim3(T, G), dim3(n_waves * WAVE), lds, stream,
                     (const bf16_t*)q, q_stride, (const bf16_t*)k_pool, (const bf16_t*)vt_pool,
                     (bf16_t*)out, out_stride, row_pos, row_seg, block_tables, max_blocks, H, G, ps,
                     window, scale);
  KAPPAI_RETURN_LAUNCH_STATUS();
}

// 1 when the decode kernel of this head size that splits the keys over blocks can do the per-head
// norm, the rotation and the storing of the rows' own keys and values itself
// (kappai_attn_decode_qk)
extern "C" int kappai_attn_decode_takes_qk(void) { return D_QK_FUSABLE ? 1 : 0; }

// The arguments that kappai_attn_decode_qk adds: qkv [T, row_stride] is the projection as it
// comes out of its product (q heads, then with store_kv the k heads and the v heads); q_norm_w /
// k_norm_w [d] float or null; cos_tab / sin_tab [positions, d / 2] float (rotate-half over the
// whole head) or both null; the pools are written at each row's own position when store_kv.
static bool qk_args_ok(const void* qkv, int row_stride, const float* q_norm_w,
                       const float* k_norm_w, const float* cos_tab, const float* sin_tab,
                       const void* k_pool, const void* vt_pool) {
  return D_QK_FUSABLE && row_stride % 8 == 0 && ((uintptr_t)qkv % 16) == 0 &&
         ((uintptr_t)q_norm_w % 16) == 0 && ((uintptr_t)k_norm_w % 16) == 0 &&
         ((uintptr_t)cos_tab % 16) == 0 && ((uintptr_t)sin_tab % 16) == 0 &&
         (cos_tab == nullptr) == (sin_tab == nullptr) && ((uintptr_t)k_pool % 16) == 0 &&
         vt_pool != nullptr;
}

extern "C" int kappai_attn_head_dim(void) { return HEAD_DIM; }

// variant: 0 = chosen by shape, 1 = one block per (tile, head), 2 = key tiles shared by four
// query heads of a kv head (head sizes 64 and 128, a multiple of four heads per kv head).
extern "C" int kappai_attn_prefill(const void* q, int q_stride, const void* k_pool,
                                   const void* vt_pool, void* out, int out_stride,
                                   const int* q_tiles, int n_tiles, const int* row_pos,
                                   const int* block_tables, int max_blocks, int H, int G, int ps,
                                   int window, float scale, int variant, hipStream_t stream) {
  if (n_tiles <= 0) return 0;
  if (ps % 16 || G < 1 || H % G || H > 65535 || (q_stride % 8) || (out_stride % 4))
    return (int)hipErrorInvalidValue;
  const int rep = H / G;
  const bool shared_ok = PG_OK && rep % 4 == 0;
  if (variant == 2 && !shared_ok) return (int)hipErrorInvalidValue;
  // sharing pays when there are blocks enough to fill the chip without splitting the keys of
  // a q tile over waves
  const bool shared = variant == 2 || (variant == 0 && shared_ok && n_tiles * (H / 4) >= 256);
#if PG_OK
  if (shared) {
    hipLaunchKernelGGL(attn_prefill_shared_kernel, dim3(n_tiles, H / 4), dim3(8 * WAVE), 0, stream,
                       (const bf16_t*)q, q_stride, (const bf16_t*)k_pool, (const bf16_t*)vt_pool,
                       (bf16_t*)out, out_stride, q_tiles, row_pos, block_tables, max_blocks, H, G,
                       ps, window, scale);
    KAPPAI_RETURN_LAUNCH_STATUS();
  }
#endif
  hipLaunchKernelGGL(attn_prefill_kernel, dim3(n_tiles, H), dim3(P_NW * WAVE), 0, stream,
                     (const bf16_t*)q, q_stride, (const bf16_t*)k_pool, (const bf16_t*)vt_pool,
                     (bf16_t*)out, out_stride, q_tiles, row_pos, block_tables, max_blocks, H, G,
                     ps, window, scale);
  KAPPAI_RETURN_LAUNCH_STATUS();
}

static int launch_decode(const void* q, int q_stride, const void* k_pool, const void* vt_pool,
                         void* out, int out_stride, float* part_o, float* part_ml,
                         const int* row_pos, const int* row_seg, const int* block_tables,
                         int max_blocks, int T, int H, int G, int ps, int window, float scale,
                         int keys_per_split, int n_splits, const QkFuse& qk, const int* row_ids,
                         hipStream_t stream) {
  if (T <= 0) return 0;
  if (ps % 16 || G < 1 || H % G || H / G > 16 || G > 65535 || n_splits < 1 || n_splits > 65535 ||
      keys_per_split < D_KPW || keys_per_split % D_KPW || (q_stride % 8))
    return (int)hipErrorInvalidValue;
  // The rows' own lengths decide the keys per split when the grid has more blocks than the waves
  // aimed at (else they could not ask for longer splits than the grid's own), and not in the form
  // with the prologue, which runs for a few rows and has no registers to spare.
  const bool plan = !qk.on && (long long)T * G * n_splits > D_TARGET_WAVES;
#define KAPPAI_DECODE(FUSED, PLAN)                                                               \
  hipLaunchKernelGGL((attn_decode_kernel<FUSED, PLAN>), dim3(T, G, n_splits), dim3(WAVE), 0,     \
                     stream, (const bf16_t*)q, q_stride, (const bf16_t*)k_pool,                  \
                     (const bf16_t*)vt_pool, part_o, part_ml, row_pos, row_seg, block_tables,    \
                     max_blocks, H, G, ps, window, scale, keys_per_split, n_splits, qk, row_ids)
  if (qk.on) KAPPAI_DECODE(true, false);
  else if (plan) KAPPAI_DECODE(false, true);
  else KAPPAI_DECODE(false, false);
#undef KAPPAI_DECODE
  hipLaunchKernelGGL(attn_merge_kernel, dim3(T, H), dim3(MERGE_WAVES * WAVE), 0, stream,
                     (const float*)part_o, (const float*)part_ml, (bf16_t*)out, out_stride, H,
                     n_splits, row_ids, row_pos, window, G, keys_per_split, plan ? 1 : 0);
  KAPPAI_RETURN_LAUNCH_STATUS();
}

extern "C" int kappai_attn_decode(const void* q, int q_stride, const void* k_pool,
                                  const void* vt_pool, void* out, int out_stride, float* part_o,
                                  float* part_ml, const int* row_pos, const int* row_seg,
                                  const int* block_tables, int max_blocks, int T, int H, int G,
                                  int ps, int window, float scale, int keys_per_split,
                                  int n_splits, hipStream_t stream) {
  return launch_decode(q, q_stride, k_pool, vt_pool, out, out_stride, part_o, part_ml, row_pos,
                       row_seg, block_tables, max_blocks, T, H, G, ps, window, scale,
                       keys_per_split, n_splits, QkFuse{}, nullptr, stream);
}

// kappai_attn_decode for some rows of a step: row_ids [T] names them (rows of q, row_pos, row_seg
// and out), part_o / part_ml hold T rows.  For the single decoded tokens of a step that also
// holds prompt portions: a row that stands alone over a long context is one tile for the tiled
// kernel, whose block then walks all its keys by itself.
extern "C" int kappai_attn_decode_rows(const void* q, int q_stride, const void* k_pool,
                                       const void* vt_pool, void* out, int out_stride,
                                       float* part_o, float* part_ml, const int* row_ids,
                                       const int* row_pos, const int* row_seg,
                                       const int* block_tables, int max_blocks, int T, int H,
                                       int G, int ps, int window, float scale, int keys_per_split,
                                       int n_splits, hipStream_t stream) {
  if (row_ids == nullptr) return (int)hipErrorInvalidValue;
  return launch_decode(q, q_stride, k_pool, vt_pool, out, out_stride, part_o, part_ml, row_pos,
                       row_seg, block_tables, max_blocks, T, H, G, ps, window, scale,
                       keys_per_split, n_splits, QkFuse{}, row_ids, stream);
}

// kappai_attn_decode with the norm, the rotation and the store of the rows' own keys and values in
// the kernel's prologue (see qk_args_ok for the added arguments).  Every split of
// a row must find the row's position inside the keys the splits cover: the caller's n_splits *
// keys_per_split reach beyond the longest context, as for kappai_attn_decode.
extern "C" int kappai_attn_decode_qk(const void* qkv, int row_stride, void* k_pool, void* vt_pool,
                                     void* out, int out_stride, float* part_o, float* part_ml,
                                     const int* row_pos, const int* row_seg,
                                     const int* block_tables, int max_blocks, int T, int H, int G,
                                     int ps, int window, float scale, int keys_per_split,
                                     int n_splits, const float* q_norm_w, const float* k_norm_w,
                                     float eps, const float* cos_tab, const float* sin_tab,
                                     int store_kv, hipStream_t stream) {
  if (!qk_args_ok(qkv, row_stride, q_norm_w, k_norm_w, cos_tab, sin_tab, k_pool, vt_pool))
    return (int)hipErrorInvalidValue;
  const QkFuse qk{1, store_kv ? 1 : 0, q_norm_w, k_norm_w, eps, cos_tab, sin_tab, (bf16_t*)k_pool,
                  (bf16_t*)vt_pool};
  return launch_decode(qkv, row_stride, k_pool, vt_pool, out, out_stride, part_o, part_ml, row_pos,
                       row_seg, block_tables, max_blocks, T, H, G, ps, window, scale,
                       keys_per_split, n_splits, qk, nullptr, stream);
}

// ---------------------------------------------------------------------------------------
// the decode attention for callers that cannot allocate: partial results in a device array
// of the library's own
// ---------------------------------------------------------------------------------------
static __device__ __align__(256) float scratch[KAPPAI_ATTN_STATIC_SCRATCH_FLOATS];

#define KAPPAI_MAX_DEVICES 64
// the address of each device's copy of `scratch`; in host code the array's name is only a
// stand-in for the symbol, never an address that a kernel could use
static float* g_scratch_ptr[KAPPAI_MAX_DEVICES];
static thread_local char g_static_error[256];

extern "C" int kappai_attn_decode_static_capacity(void) { return KAPPAI_ATTN_STATIC_SCRATCH_FLOATS; }

extern "C" const char* kappai_attn_decode_static_error(void) { return g_static_error; }

static int static_scratch_of_current_device(float** ptr) {
  int dev = -1;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return (int)err;
  if (dev < 0 || dev >= KAPPAI_MAX_DEVICES) {
    snprintf(g_static_error, sizeof g_static_error,
             "kappai_attn_decode_static: device %d is beyond the %d this library keeps track of",
             dev, KAPPAI_MAX_DEVICES);
    return (int)hipErrorInvalidDevice;
  }
  float* p = __atomic_load_n(&g_scratch_ptr[dev], __ATOMIC_ACQUIRE);
  if (p == nullptr) {
    void* sym = nullptr;
    err = hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch));
    if (err != hipSuccess || sym == nullptr) {
      snprintf(g_static_error, sizeof g_static_error,
               "kappai_attn_decode_static: hipGetSymbolAddress failed on device %d: %s", dev,
               hipGetErrorString(err));
      return (int)(err != hipSuccess ? err : hipErrorInvalidSymbol);
    }
    p = static_cast<float*>(sym);
    __atomic_store_n(&g_scratch_ptr[dev], p, __ATOMIC_RELEASE);   // the same value from any thread
  }
  *ptr = p;
  return 0;
}

extern "C" int kappai_attn_decode_static_init(void) {
  float* p = nullptr;
  return static_scratch_of_current_device(&p);
}

extern "C" int kappai_attn_decode_static(const void* q, int q_stride, const void* k_pool,
                                         const void* vt_pool, void* out, int out_stride,
                                         const int* row_pos, const int* row_seg,
                                         const int* block_tables, int max_blocks, int T, int H,
                                         int G, int ps, int window, float scale,
                                         int keys_per_split, int n_splits, hipStream_t stream) {
  g_static_error[0] = 0;
  if (T <= 0) return 0;
  if (H < 1 || n_splits < 1) {
    snprintf(g_static_error, sizeof g_static_error,
             "kappai_attn_decode_static: H = %d heads and n_splits = %d must be positive", H,
             n_splits);
    return (int)hipErrorInvalidValue;
  }
  const long long entries = (long long)T * H * n_splits;
  const long long need = entries * (HEAD_DIM + 2);
  if (need > KAPPAI_ATTN_STATIC_SCRATCH_FLOATS) {
    snprintf(g_static_error, sizeof g_static_error,
             "kappai_attn_decode_static: %d rows x %d heads x %d splits need %lld floats of partial "
             "results (head size %d); the library's array holds %d: use fewer splits or rows, or "
             "kappai_attn_decode with a workspace of the caller's",
             T, H, n_splits, need, HEAD_DIM, KAPPAI_ATTN_STATIC_SCRATCH_FLOATS);
    return (int)hipErrorInvalidValue;
  }
  float* base = nullptr;
  const int rc = static_scratch_of_current_device(&base);
  if (rc != 0) return rc;
  // part_o first (a multiple of 16 floats, so part_ml stays 16-byte aligned as well)
  float* part_o = base;
  float* part_ml = base + entries * HEAD_DIM;
  const int status = kappai_attn_decode(q, q_stride, k_pool, vt_pool, out, out_stride, part_o,
                                        part_ml, row_pos, row_seg, block_tables, max_blocks, T, H,
                                        G, ps, window, scale, keys_per_split, n_splits, stream);
  if (status == (int)hipErrorInvalidValue)
    snprintf(g_static_error, sizeof g_static_error,
             "kappai_attn_decode_static: an argument that kappai_attn_decode refuses (page size "
             "%d, %d heads over %d kv heads, %d keys a split, q stride %d)",
             ps, H, G, keys_per_split, q_stride);
  return status;
}

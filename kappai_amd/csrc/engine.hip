// kappai_forward: a whole step launched from C (see engine.h).
//
// This file holds no kernel.  It is the host side of the framework's own parts, written once more
// in C: the order of kernels of a pre-norm block, the choices that depend on the number of rows
// (which product kernel, partial sums over K, rows in fragment order, the residual sum and the
// norm folded into products), and a workspace that the activations of a step are cut from.  The
// same step run from the host's parts, kernel by kernel, gives bit for bit the same logits; the
// host keeps that path for models with parts this file does not know and for timing by stage.
//
// Order of a block as kappai's (src/models/lfm.c:7-62, src/recipe/builders.c:378-388):
// x += mixer(norm(x)); x += ffn(norm(x)).
#include "engine.h"

#include <stdio.h>
#include <string.h>

namespace {

thread_local char g_error[320];

// ---------------------------------------------------------------------------------------------
// workspace: four regions, each a stack that a dry run measures first
// ---------------------------------------------------------------------------------------------
enum Region { R_STEP = 0, R_CARRY_A = 1, R_CARRY_B = 2, R_BLOCK = 3, N_REGIONS = 4 };

struct Arena {
  char* base = nullptr;              // null: dry run, only the sizes are followed
  size_t offset[N_REGIONS] = {0, 0, 0, 0};
  size_t used[N_REGIONS] = {0, 0, 0, 0};
  size_t peak[N_REGIONS] = {0, 0, 0, 0};
  size_t limit[N_REGIONS] = {0, 0, 0, 0};
  bool overflow = false;

  void* take(Region r, size_t bytes) {
    bytes = (bytes + 255) / 256 * 256;
    const size_t at = used[r];
    used[r] += bytes;
    if (used[r] > peak[r]) peak[r] = used[r];
    if (base == nullptr) return reinterpret_cast<void*>((uintptr_t)256);   // never dereferenced
    if (used[r] > limit[r]) {
      overflow = true;
      return nullptr;
    }
    return base + offset[r] + at;
  }
  void reset(Region r) { used[r] = 0; }
};

// ---------------------------------------------------------------------------------------------
// what travels between kernels
// ---------------------------------------------------------------------------------------------
// Rows on their way into a product: plain [M, D] with a row stride, 16 row slots in fragment
// order, or either of the two still to be divided by the rows' root mean square (scaled).
struct Rows {
  void* data = nullptr;
  int is_bf16 = 0;
  int M = 0, D = 0, ld = 0;
  int frag = 0;
  const float* ss = nullptr;       // scaled rows: [ss_parts][16]
  int ss_parts = 0;
  float eps = 0.f;
  const kappai_norm* norm = nullptr;   // the norm the scaled rows were made for
};

// What a part hands to the norm after it.
enum CarryKind { C_NOTHING = 0, C_DELTA = 1, C_PARTS = 2, C_SCALED = 3 };
struct Carry {
  CarryKind kind = C_NOTHING;      // nothing: the sum is in the residual stream already
  void* data = nullptr;            // delta [M, D] / partial sums [parts][M][D] float
  int is_f32 = 0;
  int parts = 1;
  Rows scaled;                     // C_SCALED
};

struct Into {                      // ops.AddInto
  float* resid = nullptr;
  const kappai_norm* norm = nullptr;
};

struct Ctx {
  const kappai_model* m;
  const kappai_batch* b;
  Arena* a;
  hipStream_t stream;
  bool dry;
  int status = 0;
  int carry_turn = 0;

  // The region for what a part hands to the norm after it.  What the region held is two parts
  // old by now and has been consumed (the part's own input lies in the other region).
  Region next_carry_region() {
    const Region r = (carry_turn++ & 1) ? R_CARRY_B : R_CARRY_A;
    a->reset(r);
    return r;
  }
  bool ok() const { return status == 0 && !a->overflow; }
};

#define LAUNCH(ctx, call)                         \
  do {                                            \
    if (!(ctx).dry && (ctx).ok()) {               \
      const int rc_ = (call);                     \
      if (rc_ != 0) (ctx).status = rc_;           \
    }                                             \
  } while (0)

inline size_t elem(int is_bf16) { return is_bf16 ? 2 : 4; }

// ---------------------------------------------------------------------------------------------
// how many K ranges (the rule the host's parts use as well)
// ---------------------------------------------------------------------------------------------
// K ranges for a product with more than 64 rows whose consumer adds partial sums: the number
// that a model of the block kernel's time likes best.  A 128 x 128 block that has a CU to itself
// takes about 0.62 us per 64 of K, so a product with few blocks gains from being cut until the
// chip is full (with 140 blocks of 256 x 256 or more the kernel takes its 256 x 256 form, about
// 1 us per 64 of K) or the float partial sums cost more than the cut saves.
int split_k_large(int M, int N, int K) {
  int best = 1;
  double best_t = -1.0;
  for (int split = 1; split < 9; ++split) {
    if (K % (128 * split) || (split > 1 && K / split < 256)) continue;
    const double steps = (double)K / split / 64.0;
    const long blocks256 = (long)((M + 255) / 256) * ((N + 255) / 256) * split;
    const long rem = blocks256 % 256;
    double t;
    if ((140 <= blocks256 && blocks256 <= 256) ||
        (blocks256 > 256 && (rem == 0 || (256 - rem) * 10 < 3 * blocks256))) {
      t = (double)((blocks256 + 255) / 256) * (steps * 1.0 + 4.5);
    } else {
      const long blocks = (long)((M + 127) / 128) * ((N + 127) / 128) * split;
      t = (double)((blocks + 511) / 512) * (steps * 0.62 * (blocks > 256 ? 1.25 : 1.0) + 2.5);
    }
    t += (split > 1 ? (double)split * M * N * 8 : (double)M * N * 4) / 5e6;
    if (best_t < 0 || t < best_t - 1e-9) {
      best = split;
      best_t = t;
    }
  }
  return best;
}

int split_k_for(int M, int N, int K) {
  if (M > 64) return split_k_large(M, N, K);
  if (M > 16) {
    // the kernel that shares the rows through LDS: blocks of 64 columns, K ranges that are
    // multiples of 512 and at least 1024 long, 128 blocks or more
    int split = K / 1024 < 8 ? K / 1024 : 8;
    while (split > 1 && K % (512 * split)) --split;
    if (split >= 1 && K % (512 * split) == 0 && (long)((N + 63) / 64) * split >= 128) return split;
  }
  const int col_groups = (N + 15) / 16;
  int s = 8;
  if (512 / col_groups < s) s = 512 / col_groups;
  if (K / 512 < s) s = K / 512;
  return s < 1 ? 1 : s;
}

// ---------------------------------------------------------------------------------------------
// the products
// ---------------------------------------------------------------------------------------------
bool aligned16(const void* p) { return ((uintptr_t)p % 16) == 0; }

// Can the kernel for 1 to 16 rows of this matrix read rows in fragment order / scale its results?
bool takes_kernel_order(const kappai_linear& lin, int D) {
  return !lin.w_is_f32 && lin.k == D && aligned16(lin.w) && lin.k % 8 == 0;
}

bool fragment_fits(const Ctx& c, int M, int D) {         // ops.FragmentRows.fits for bfloat16
  return c.m->compute_bf16 && M >= 1 && M <= 16 && D % 32 == 0 && D <= 8192;
}

// RMSNorm by its own kernel.  rows: only these (the residual is then left alone).
Rows norm_kernel(Ctx& c, const kappai_norm& norm, float* resid, const Carry& carry, int M,
                 const int* rows, int n_rows, bool fragment) {
  const int D = c.m->width;
  const int n = rows ? n_rows : M;
  Rows out;
  out.is_bf16 = c.m->compute_bf16;
  out.M = n;
  out.D = D;
  out.ld = D;
  out.frag = fragment ? 1 : 0;
  out.norm = &norm;
  out.data = c.a->take(R_BLOCK, (size_t)(fragment ? 16 : n) * D * elem(out.is_bf16));
  const void* delta = nullptr;
  int delta_f32 = 0, n_part = 1;
  long pstride = 0;
  if (carry.kind == C_DELTA) {
    delta = carry.data;
    delta_f32 = carry.is_f32;
  } else if (carry.kind == C_PARTS) {
    delta = carry.data;
    delta_f32 = 1;
    n_part = carry.parts;
    pstride = (long)M * D;
  }
  LAUNCH(c, c.m->kernels->add_rmsnorm(resid, delta, delta_f32, n_part, pstride, norm.w, out.data,
                                      rows, n, D, norm.eps, rows ? 0 : 1, out.is_bf16,
                                      fragment ? 1 : 0, c.stream));
  return out;
}

// The rows that the product `consumer` reads after `norm` (RMSNorm.add_norm with defer): scaled
// rows made for this norm go through as they are, else the norm's kernel runs, writing fragment
// order when that suits the number of rows and the consumer.
Rows normed(Ctx& c, const kappai_norm& norm, float* resid, const Carry& carry, int M,
            const kappai_linear& consumer) {
  const int D = c.m->width;
  if (carry.kind == C_SCALED) {
    if (carry.scaled.norm == &norm && takes_kernel_order(consumer, D)) return carry.scaled;
    Carry none;                                  // the sum is in the residual already
    return norm_kernel(c, norm, resid, none, M, nullptr, 0, false);
  }
  const bool fragment = M >= c.m->fragment_rows_min && fragment_fits(c, M, D) &&
                        (carry.kind != C_PARTS || carry.parts <= 8) &&
                        takes_kernel_order(consumer, D);
  return norm_kernel(c, norm, resid, carry, M, nullptr, 0, fragment);
}

// The first norm of a step together with the embedding that fills the residual stream.
Rows embedded_and_normed(Ctx& c, const kappai_norm& norm, float* resid, int M,
                         const kappai_linear& consumer) {
  const int D = c.m->width;
  const bool fragment = M >= c.m->fragment_rows_min && fragment_fits(c, M, D) &&
                        takes_kernel_order(consumer, D);
  Rows out;
  out.is_bf16 = c.m->compute_bf16;
  out.M = M;
  out.D = D;
  out.ld = D;
  out.frag = fragment ? 1 : 0;
  out.norm = &norm;
  out.data = c.a->take(R_BLOCK, (size_t)(fragment ? 16 : M) * D * elem(out.is_bf16));
  LAUNCH(c, c.m->kernels->embed_rmsnorm(c.b->tokens, c.m->embed_table, c.m->embed_is_bf16, resid,
                                        norm.w, out.data, M, D, norm.eps, out.is_bf16,
                                        fragment ? 1 : 0, c.stream));
  return out;
}

void* cast_to(Ctx& c, const void* x, size_t n, int from_bf16, int to_bf16) {
  void* out = c.a->take(R_BLOCK, n * elem(to_bf16));
  LAUNCH(c, c.m->kernels->cast(x, out, (long)n, from_bf16, to_bf16, c.stream));
  return out;
}

// ops.linear.  out_bf16: the dtype of a plain result.  partial_sums: the result may come as float
// planes over K ranges.  into: the product may add its result into the residual stream.
// region: where a result that outlives the block goes (the carry to the next norm).
Carry linear(Ctx& c, Rows x, const kappai_linear& lin, int out_bf16, bool partial_sums,
             const Into* into, Region region) {
  const kappai_kernels& k = *c.m->kernels;
  Carry out;
  const int M = x.M, K = x.D, N = lin.n;
  if (lin.k != K) {
    snprintf(g_error, sizeof g_error, "kappai_forward: rows of width %d meet a matrix [%d, %d]", K,
             lin.n, lin.k);
    c.status = (int)hipErrorInvalidValue;
    return out;
  }
  if (lin.w_is_f32) {
    // a matrix stored in 32 bits: true 32-bit arithmetic whatever the activations are
    const float* xf = x.is_bf16 ? (const float*)cast_to(c, x.data, (size_t)M * K, 1, 0)
                                : (const float*)x.data;
    const int lda = x.is_bf16 ? K : x.ld;
    float* o = (float*)c.a->take(out_bf16 ? R_BLOCK : region, (size_t)M * N * 4);
    LAUNCH(c, k.gemm_f32(xf, (const float*)lin.w, lin.bias, o, M, N, K, M > 1 ? lda : K, N,
                         c.stream));
    out.kind = C_DELTA;
    if (out_bf16) {
      out.data = c.a->take(region, (size_t)M * N * 2);
      LAUNCH(c, k.cast(o, out.data, (long)M * N, 0, 1, c.stream));
      out.is_f32 = 0;
    } else {
      out.data = o;
      out.is_f32 = 1;
    }
    return out;
  }
  const void* xb = x.data;
  int lda = x.ld;
  if (!x.is_bf16) {
    xb = cast_to(c, x.data, (size_t)M * K, 0, 1);
    lda = K;
  }
  if (M <= 1) lda = K;
  const bool scaled = x.ss != nullptr;
  if (!(K % 8 == 0 && lda % 8 == 0 && aligned16(xb) && aligned16(lin.w))) {
    // the matrix-core kernels read 16 bytes at a time; anything else goes the plain way
    if (lin.w == nullptr) {
      snprintf(g_error, sizeof g_error, "kappai_forward: a matrix kept in fragment order met "
                                        "rows that are not 16-byte aligned (K = %d, row stride %d)",
               K, lda);
      c.status = (int)hipErrorInvalidValue;
      return out;
    }
    if (scaled || x.frag) {
      snprintf(g_error, sizeof g_error, "kappai_forward: rows in kernel order reached the plain "
                                        "product kernel (K = %d)", K);
      c.status = (int)hipErrorInvalidValue;
      return out;
    }
    out.kind = C_DELTA;
    out.is_f32 = out_bf16 ? 0 : 1;
    out.data = c.a->take(region, (size_t)M * N * elem(out_bf16));
    LAUNCH(c, k.gemm_bf16_any(xb, lin.w, lin.bias, out.data, M, N, K, lda, N, out_bf16 ? 0 : 1,
                              c.stream));
    return out;
  }
  if (into != nullptr && M <= c.m->fused_max_rows) {
    // the result joins the residual stream inside the kernel
    const kappai_norm* norm = into->norm;
    void* rows = nullptr;
    float* ss = nullptr;
    int fragment = 0;
    if (norm != nullptr) {
      fragment = (M >= c.m->fragment_rows_from && fragment_fits(c, M, N)) ? 1 : 0;
      rows = c.a->take(region, (size_t)(fragment ? 16 : M) * N * 2);
      ss = (float*)c.a->take(region, (size_t)((N + 7) / 8) * 16 * 4);
    }
    LAUNCH(c, k.gemm_bf16(xb, lin.w, lin.w_frag, lin.bias, nullptr, M, N, K, lda, N, 1, 0, 1,
                          x.frag, scaled ? x.ss : nullptr, scaled ? x.ss_parts : 0,
                          scaled ? x.eps : 0.f, into->resid, N, norm ? norm->w : nullptr, rows,
                          fragment, ss, c.stream));
    if (norm == nullptr) return out;             // C_NOTHING
    out.kind = C_SCALED;
    out.scaled.data = rows;
    out.scaled.is_bf16 = 1;
    out.scaled.M = M;
    out.scaled.D = N;
    out.scaled.ld = N;
    out.scaled.frag = fragment;
    out.scaled.ss = ss;
    out.scaled.ss_parts = (N + 7) / 8;
    out.scaled.eps = norm->eps;
    out.scaled.norm = norm;
    return out;
  }
  const int ksplit = (partial_sums && !scaled) ? split_k_for(M, N, K) : 1;
  if (ksplit > 1) {
    out.kind = C_PARTS;
    out.is_f32 = 1;
    out.parts = ksplit;
    out.data = c.a->take(region, (size_t)ksplit * M * N * 4);
  } else {
    out.kind = C_DELTA;
    out.is_f32 = out_bf16 ? 0 : 1;
    out.data = c.a->take(region, (size_t)M * N * elem(out_bf16));
  }
  LAUNCH(c, k.gemm_bf16(xb, lin.w, lin.w_frag, lin.bias, out.data, M, N, K, lda, N,
                        (ksplit > 1 || !out_bf16) ? 1 : 0, 0, ksplit, x.frag,
                        scaled ? x.ss : nullptr, scaled ? x.ss_parts : 0, scaled ? x.eps : 0.f,
                        nullptr, 0, nullptr, nullptr, 0, nullptr, c.stream));
  return out;
}

// Scaled rows or rows in fragment order that a kernel cannot take are made by the norm's own
// kernel from the residual stream instead (ops.ScaledRows.materialize).
Rows plain_rows(Ctx& c, const Rows& x, float* resid) {
  if (x.ss == nullptr && !x.frag) return x;
  Carry none;
  return norm_kernel(c, *x.norm, resid, none, x.M, nullptr, 0, false);
}

Rows as_rows(const Carry& y, int M, int D, int is_bf16) {
  Rows r;
  r.data = y.data;
  r.is_bf16 = is_bf16;
  r.M = M;
  r.D = D;
  r.ld = D;
  return r;
}

// ---------------------------------------------------------------------------------------------
// the parts
// ---------------------------------------------------------------------------------------------
// When in_proj and qkv hand their consumer partial sums over K ranges (tuning.takes_partial_sums)
bool takes_partial_sums(const Ctx& c, int M) {
  return M > c.m->partial_sums_min_rows &&
         (M <= c.m->partial_sums_max_rows || c.b->max_segment_rows == 1);
}

// parts/shortconv.py
Carry conv_mixer(Ctx& c, const kappai_layer_call& L, Rows x, float* resid, const Into& into) {
  const kappai_kernels& k = *c.m->kernels;
  const kappai_batch& b = *c.b;
  const int M = x.M, D = c.m->width, taps = L.taps_per_channel;
  const Region region = c.next_carry_region();
  const bool wide_enough = D >= c.m->fused_step_min_width ||
                           (D >= c.m->fused_step_narrow_width && M <= c.m->fused_step_narrow_rows);
  Carry none;
  if (b.max_segment_rows == 1 && M <= 64 && x.is_bf16 && !L.in_proj.w_is_f32 && D % 16 == 0 &&
      wide_enough) {
    // decode: projection, convolution and state shift in one kernel
    if (!(takes_kernel_order(L.in_proj, D))) x = plain_rows(c, x, resid);
    const int c_frag = (M >= c.m->fragment_rows_from && M <= c.m->fused_max_rows && D % 32 == 0 &&
                        takes_kernel_order(L.out_proj, D));
    void* y = c.a->take(R_BLOCK, (size_t)(c_frag ? 16 : M) * D * 2);
    LAUNCH(c, k.gemm_bf16_shortconv_step(x.data, L.in_proj.w, L.in_proj.w_frag, L.in_proj.bias, y,
                                         M, D, D, M > 1 ? x.ld : D, L.taps, L.conv_bias, L.state,
                                         b.seg_pos0, b.seg_slot, taps, x.frag, x.ss, x.ss_parts,
                                         x.eps, c_frag, c.stream));
    Rows yr = as_rows(Carry{C_DELTA, y}, M, D, 1);
    yr.frag = c_frag;
    return linear(c, yr, L.out_proj, c.m->compute_bf16, true, &into, region);
  }
  // more than 16 rows (decode at any batch size, short prompt portions): the projection may come
  // as sums over ranges of its input dimension, which the conv kernel adds up
  const bool parts = takes_partial_sums(c, M);
  Carry proj = linear(c, x, L.in_proj, c.m->compute_bf16, parts, nullptr, R_BLOCK);
  if (!c.ok() && !c.dry) return none;
  void* y;
  int y_bf16;
  if (proj.kind == C_PARTS) {
    y_bf16 = 1;
    y = c.a->take(R_BLOCK, (size_t)M * D * 2);
    LAUNCH(c, k.shortconv_parts((const float*)proj.data, proj.parts, L.taps, L.conv_bias, L.state,
                                y, b.row_seg, b.seg_start, b.seg_pos0, b.seg_slot, M, b.n_segments,
                                D, taps, c.stream));
  } else {
    y_bf16 = proj.is_f32 ? 0 : 1;
    y = c.a->take(R_BLOCK, (size_t)M * D * elem(y_bf16));
    LAUNCH(c, k.shortconv(proj.data, L.taps, L.conv_bias, L.state, y, b.row_seg, b.seg_start,
                          b.seg_pos0, b.seg_slot, M, b.n_segments, D, taps, y_bf16, c.stream));
  }
  return linear(c, as_rows(Carry{C_DELTA, y}, M, D, y_bf16), L.out_proj, c.m->compute_bf16, true,
                &into, region);
}

// ops.decode_form: few keys go to the kernel that splits them over the waves of a block
int decode_keys(const Ctx& c, const kappai_layer_call& L) {
  int n_keys = c.b->max_position + 1;
  if (L.window) n_keys = (n_keys < L.window ? n_keys : L.window) + 32;
  return n_keys;
}
bool decode_block_form(const Ctx& c, const kappai_layer_call& L, int rep) {
  return L.mfma->decode_block_waves(rep) > 0 && decode_keys(c, L) <= c.m->decode_block_max_keys;
}

// how the split decode kernel cuts n_keys keys of `rows` rows (ops._decode_split)
void decode_splits(const Ctx& c, const kappai_layer_call& L, int rows, int G, int n_keys,
                   int* keys_per_split, int* n_splits) {
  const int kpw = L.mfma->keys_per_wave();
  int s = c.m->decode_max_splits;
  if ((n_keys + kpw - 1) / kpw < s) s = (n_keys + kpw - 1) / kpw;
  int by_waves = c.m->decode_waves / (rows * G);
  if (by_waves < 1) by_waves = 1;
  if (by_waves < s) s = by_waves;
  if (s < 1) s = 1;
  *keys_per_split = ((n_keys + s - 1) / s + kpw - 1) / kpw * kpw;
  *n_splits = (n_keys + *keys_per_split - 1) / *keys_per_split;
}

// parts/attention.py with ops.qk_norm_rope_store and ops.paged_attention
Carry attention_mixer(Ctx& c, const kappai_layer_call& L, Rows x, float* resid, const Into& into) {
  const kappai_kernels& k = *c.m->kernels;
  const kappai_batch& b = *c.b;
  const int M = x.M, H = L.heads, G = L.kv_heads, d = L.head_dim, ps = c.m->page_size;
  const Region region = c.next_carry_region();
  Carry none;
  kappai_linear qkv = L.qkv;
  if (L.shared_cache) {          // the q rows of the stacked matrix, whole pieces of 16 rows
    qkv.n = H * d;
    if (qkv.w_frag != nullptr && (H * d) % 16) qkv.w_frag = nullptr;
  }
  if (!takes_kernel_order(qkv, x.D)) x = plain_rows(c, x, resid);
  const bool parts = takes_partial_sums(c, M);
  Carry proj = linear(c, x, qkv, c.m->compute_bf16, parts, nullptr, R_BLOCK);
  if (!c.ok() && !c.dry) return none;
  if (L.rot_mode != 0 && b.max_position >= L.rot_positions) {
    snprintf(g_error, sizeof g_error, "kappai_forward: position %d is beyond the rotation table of "
                                      "%d positions", b.max_position, L.rot_positions);
    c.status = (int)hipErrorInvalidValue;
    return none;
  }
  if (L.group < 0 || L.group >= b.n_groups) {
    c.status = (int)hipErrorInvalidValue;
    snprintf(g_error, sizeof g_error, "kappai_forward: the batch has no block tables of group %d",
             L.group);
    return none;
  }
  const int* tables = b.block_tables[L.group];
  const int max_blocks = b.max_blocks[L.group];
  const int store = L.shared_cache ? 0 : 1;
  const bool single = b.max_segment_rows == 1;
  // decode: the attention kernels take the projection as it is and do norm, rotation and store
  // themselves (parts/attention.py: _prologue_in_kernel)
  const bool qk_in_kernel =
      M <= c.m->fused_qk && single && proj.kind == C_DELTA && !proj.is_f32 && L.mfma != nullptr &&
      H / G <= 16 && qkv.n % 8 == 0 && aligned16(proj.data) && ps % 16 == 0 && d % 16 == 0 &&
      d <= 256 && (L.rot_mode == 0 || (L.rot_mode == 1 && L.rot_dim == d)) &&
      L.mfma->decode_takes_qk != nullptr && L.mfma->decode_takes_qk() &&
      !decode_block_form(c, L, H / G);
  // q in place in the projection, or (from partial sums) a new bfloat16 [M, H d]
  void* q;
  int q_stride, q_bf16;
  if (qk_in_kernel) {
    q_bf16 = 1;
    q_stride = qkv.n;
    q = proj.data;
  } else if (proj.kind == C_PARTS) {
    q_bf16 = 1;
    q_stride = H * d;
    q = c.a->take(R_BLOCK, (size_t)M * H * d * 2);
    LAUNCH(c, k.qk_norm_rope_store(nullptr, qkv.n, L.q_norm_w, L.k_norm_w, L.qk_eps, L.cos_table,
                                   L.sin_table, L.rot_mode ? L.rot_dim : 0, L.rot_mode, L.k_pool,
                                   L.v_pool, b.row_pos, b.row_seg, store ? tables : nullptr,
                                   store ? max_blocks : 0, M, H, G, d, ps, store, 1,
                                   (const float*)proj.data, proj.parts, q, H * d, c.stream));
  } else {
    q_bf16 = proj.is_f32 ? 0 : 1;
    q_stride = qkv.n;
    q = proj.data;
    LAUNCH(c, k.qk_norm_rope_store(q, q_stride, L.q_norm_w, L.k_norm_w, L.qk_eps, L.cos_table,
                                   L.sin_table, L.rot_mode ? L.rot_dim : 0, L.rot_mode, L.k_pool,
                                   L.v_pool, b.row_pos, b.row_seg, store ? tables : nullptr,
                                   store ? max_blocks : 0, M, H, G, d, ps, store, q_bf16, nullptr,
                                   0, nullptr, H * d, c.stream));
  }
  void* ctx = c.a->take(R_BLOCK, (size_t)M * H * d * elem(q_bf16));
  const float* cos_t = L.rot_mode ? L.cos_table : nullptr;
  const float* sin_t = L.rot_mode ? L.sin_table : nullptr;
  const bool mfma_ok = q_bf16 && L.mfma != nullptr && ps % 16 == 0 && d % 16 == 0 && d <= 256 &&
                       q_stride % 8 == 0 && aligned16(q);
  if (mfma_ok && single && H / G <= 16) {
    const int n_keys = decode_keys(c, L);
    const int block_waves = L.mfma->decode_block_waves(H / G);
    if (decode_block_form(c, L, H / G)) {
      LAUNCH(c, L.mfma->attn_decode_block(q, q_stride, L.k_pool, L.v_pool, ctx, H * d, b.row_pos,
                                          b.row_seg, tables, max_blocks, M, H, G, ps, L.window,
                                          L.scale, block_waves, c.stream));
    } else {
      int keys_per_split, n_splits;
      decode_splits(c, L, M, G, n_keys, &keys_per_split, &n_splits);
      float* part_o = (float*)c.a->take(R_BLOCK, (size_t)M * H * n_splits * d * 4);
      float* part_ml = (float*)c.a->take(R_BLOCK, (size_t)M * H * n_splits * 2 * 4);
      if (qk_in_kernel)
        LAUNCH(c, L.mfma->attn_decode_qk(q, q_stride, L.k_pool, L.v_pool, ctx, H * d, part_o,
                                         part_ml, b.row_pos, b.row_seg, tables, max_blocks, M, H,
                                         G, ps, L.window, L.scale, keys_per_split, n_splits,
                                         L.q_norm_w, L.k_norm_w, L.qk_eps, cos_t, sin_t, store,
                                         c.stream));
      else
        LAUNCH(c, L.mfma->attn_decode(q, q_stride, L.k_pool, L.v_pool, ctx, H * d, part_o, part_ml,
                                      b.row_pos, b.row_seg, tables, max_blocks, M, H, G, ps,
                                      L.window, L.scale, keys_per_split, n_splits, c.stream));
    }
  } else if (mfma_ok && b.q_tiles != nullptr) {
    LAUNCH(c, L.mfma->attn_prefill(q, q_stride, L.k_pool, L.v_pool, ctx, H * d, b.q_tiles,
                                   b.n_tiles, b.row_pos, tables, max_blocks, H, G, ps, L.window,
                                   L.scale, 0, c.stream));
    if (b.lone_rows != nullptr && b.n_lone_rows > 0) {
      // the single decoded tokens beside the portions: keys split over blocks (ops._decode_split)
      if (H / G > 16 || b.max_lone_position < 0) {
        snprintf(g_error, sizeof g_error, "kappai_forward: rows left out of the tiles need the "
                                          "decode kernel and their largest position");
        c.status = (int)hipErrorInvalidValue;
        return none;
      }
      const int R = b.n_lone_rows;
      int n_keys = b.max_lone_position + 1;
      if (L.window) n_keys = (n_keys < L.window ? n_keys : L.window) + 32;
      int keys_per_split, n_splits;
      decode_splits(c, L, R, G, n_keys, &keys_per_split, &n_splits);
      float* part_o = (float*)c.a->take(R_BLOCK, (size_t)R * H * n_splits * d * 4);
      float* part_ml = (float*)c.a->take(R_BLOCK, (size_t)R * H * n_splits * 2 * 4);
      LAUNCH(c, L.mfma->attn_decode_rows(q, q_stride, L.k_pool, L.v_pool, ctx, H * d, part_o,
                                         part_ml, b.lone_rows, b.row_pos, b.row_seg, tables,
                                         max_blocks, R, H, G, ps, L.window, L.scale,
                                         keys_per_split, n_splits, c.stream));
    }
  } else {
    LAUNCH(c, k.paged_attention_rows(q, q_stride, L.k_pool, L.v_pool, ctx, H * d, b.row_pos,
                                     b.row_seg, tables, max_blocks, M, H, G, d, ps, L.window,
                                     L.scale, q_bf16, c.stream));
  }
  return linear(c, as_rows(Carry{C_DELTA, ctx}, M, H * d, q_bf16), L.attn_out, c.m->compute_bf16,
                true, &into, region);
}

// parts/feed_forward.py
Carry swiglu_ffn(Ctx& c, const kappai_layer_call& L, Rows x, float* resid, const Into& into) {
  const kappai_kernels& k = *c.m->kernels;
  const int M = x.M, D = c.m->width, F = L.hidden;
  const Region region = c.next_carry_region();
  Carry none;
  if (L.ffn_fused && x.is_bf16) {
    if (!takes_kernel_order(L.gate_up, D)) x = plain_rows(c, x, resid);
    const int c_frag = (M >= c.m->fragment_rows_from && M <= c.m->fused_max_rows && F % 32 == 0 &&
                        takes_kernel_order(L.down, F));
    void* act = c.a->take(R_BLOCK, (size_t)(c_frag ? 16 : M) * F * 2);
    LAUNCH(c, k.gemm_bf16_swiglu(x.data, L.gate_up.w, L.gate_up.w_frag, act, M, F, D,
                                 M > 1 ? x.ld : D, F, 0, x.frag, x.ss, x.ss_parts, x.eps, c_frag,
                                 c.stream));
    Rows ar = as_rows(Carry{C_DELTA, act}, M, F, 1);
    ar.frag = c_frag;
    return linear(c, ar, L.down, c.m->compute_bf16, true, &into, region);
  }
  Carry gu = linear(c, x, L.gate_up, c.m->compute_bf16, false, nullptr, R_BLOCK);
  if (!c.ok() && !c.dry) return none;
  const int act_bf16 = gu.is_f32 ? 0 : 1;
  void* act = c.a->take(R_BLOCK, (size_t)M * F * elem(act_bf16));
  LAUNCH(c, k.swiglu(gu.data, act, M, F, act_bf16, c.stream));
  return linear(c, as_rows(Carry{C_DELTA, act}, M, F, act_bf16), L.down, c.m->compute_bf16, true,
                &into, region);
}

bool model_ok(const kappai_model* m) {
  if (m == nullptr || m->abi != KAPPAI_ENGINE_ABI || m->kernels == nullptr || m->n_calls < 0 ||
      m->width < 1 || m->vocab < 1 || (m->n_calls > 0 && m->calls == nullptr)) {
    snprintf(g_error, sizeof g_error, "kappai_forward: the model description is incomplete or was "
                                      "filled in for another version of this library");
    return false;
  }
  return true;
}

int run(const kappai_model* m, const kappai_batch* b, Arena& arena, float* logits,
        hipStream_t stream, bool dry) {
  Ctx c{m, b, &arena, stream, dry};
  const kappai_kernels& k = *m->kernels;
  const int T = b->n_rows, D = m->width;
  float* resid = (float*)arena.take(R_STEP, (size_t)T * D * 4);
  // the embedding and the first call's norm are one kernel where the norm's row kernel takes
  // the width (the same arithmetic as the two kernels, bit for bit)
  const bool embed_with_norm = m->n_calls > 0 && D % 8 == 0 && D <= 8192 &&
                               (m->embed_is_bf16 != 2 || D % 32 == 0) &&
                               aligned16(m->embed_table) && aligned16(m->calls[0].mixer_norm.w);
  if (!embed_with_norm)
    LAUNCH(c, k.embed_rows(b->tokens, m->embed_table, m->embed_is_bf16, resid, T, D, stream));
  Carry carry;
  for (int ci = 0; ci < m->n_calls && c.ok(); ++ci) {
    const kappai_layer_call& L = m->calls[ci];
    const kappai_layer_call* next = ci + 1 < m->n_calls ? &m->calls[ci + 1] : nullptr;
    arena.reset(R_BLOCK);
    const bool conv = L.mixer == KAPPAI_MIXER_CONV;
    const kappai_linear& first = conv ? L.in_proj : L.qkv;
    Rows x = (ci == 0 && embed_with_norm) ? embedded_and_normed(c, L.mixer_norm, resid, T, first)
                                          : normed(c, L.mixer_norm, resid, carry, T, first);
    const Into into_ffn{resid, &L.ffn_norm};
    const Carry mixed = conv ? conv_mixer(c, L, x, resid, into_ffn)
                             : attention_mixer(c, L, x, resid, into_ffn);
    if (!c.ok()) break;
    Rows x2 = normed(c, L.ffn_norm, resid, mixed, T, L.gate_up);
    // the norm after the last call is the final one; the head can take rows made for it when
    // every row of the step wants its logits, in the rows' order
    const kappai_norm* after = next ? &next->mixer_norm
                               : (b->logits_of_every_row && b->n_logit_rows == T &&
                                  takes_kernel_order(m->head, D)) ? &m->final_norm : nullptr;
    const Into into_next{resid, after};
    carry = swiglu_ffn(c, L, x2, resid, into_next);
  }
  if (c.ok() && b->n_logit_rows > 0) {
    arena.reset(R_BLOCK);
    const int n = b->n_logit_rows;
    Rows xb;
    if (carry.kind == C_SCALED && carry.scaled.norm == &m->final_norm) {
      xb = carry.scaled;               // the last product made the rows, the head divides by rms
    } else {
      Carry for_norm = carry;
      if (carry.kind == C_SCALED) for_norm = Carry();      // made for no norm that runs here
      const bool fragment = n >= m->fragment_rows_min && fragment_fits(c, n, D) &&
                            (for_norm.kind != C_PARTS || for_norm.parts <= 8) &&
                            takes_kernel_order(m->head, D);
      xb = norm_kernel(c, m->final_norm, resid, for_norm, T, b->logit_rows, n, fragment);
    }
    // the head: a plain product with float results, straight into the caller's tensor
    const kappai_linear& head = m->head;
    if (head.w_is_f32) {
      const float* xf = xb.is_bf16 ? (const float*)cast_to(c, xb.data, (size_t)n * D, 1, 0)
                                   : (const float*)xb.data;
      LAUNCH(c, k.gemm_f32(xf, (const float*)head.w, head.bias, logits, n, head.n, D, D, head.n,
                           stream));
    } else {
      const void* xh = xb.data;
      if (!xb.is_bf16) xh = cast_to(c, xb.data, (size_t)n * D, 0, 1);
      if (D % 8 == 0 && aligned16(xh) && aligned16(head.w))
        LAUNCH(c, k.gemm_bf16(xh, head.w, head.w_frag, head.bias, logits, n, head.n, D, D, head.n,
                              1, 0, 1, xb.frag, xb.ss, xb.ss ? xb.ss_parts : 0,
                              xb.ss ? xb.eps : 0.f, nullptr, 0, nullptr, nullptr, 0, nullptr,
                              stream));
      else if (head.w != nullptr)
        LAUNCH(c, k.gemm_bf16_any(xh, head.w, head.bias, logits, n, head.n, D, D, head.n, 1,
                                  stream));
      else
        c.status = (int)hipErrorInvalidValue;    // (a matrix in fragment order has D % 32 == 0)
    }
  }
  if (arena.overflow) {
    snprintf(g_error, sizeof g_error, "kappai_forward: the workspace is smaller than "
                                      "kappai_forward_workspace_bytes says this batch needs");
    return (int)hipErrorInvalidValue;
  }
  return c.status;
}

bool batch_ok(const kappai_model* m, const kappai_batch* b) {
  if (b == nullptr || b->n_rows < 1 || b->n_segments < 1 || b->n_logit_rows < 0 ||
      b->n_groups < 0 || b->n_groups > KAPPAI_MAX_GROUPS) {
    snprintf(g_error, sizeof g_error, "kappai_forward: a step needs rows and segments");
    return false;
  }
  (void)m;
  return true;
}

}  // namespace

extern "C" int kappai_engine_layout(int* sizes, int n) {
  const int mine[8] = {KAPPAI_ENGINE_ABI,
                       (int)sizeof(kappai_kernels),
                       (int)sizeof(kappai_attention_kernels),
                       (int)sizeof(kappai_linear),
                       (int)sizeof(kappai_norm),
                       (int)sizeof(kappai_layer_call),
                       (int)sizeof(kappai_model),
                       (int)sizeof(kappai_batch)};
  for (int i = 0; i < n && i < 8; ++i) sizes[i] = mine[i];
  return 8;
}

extern "C" const char* kappai_forward_error(void) { return g_error; }

extern "C" int kappai_split_k_for(int M, int N, int K) { return split_k_for(M, N, K); }

extern "C" size_t kappai_forward_workspace_bytes(const kappai_model* model,
                                                 const kappai_batch* batch) {
  g_error[0] = 0;
  if (!model_ok(model) || !batch_ok(model, batch)) return 0;
  Arena arena;
  if (run(model, batch, arena, nullptr, nullptr, true) != 0) return 0;
  size_t total = 0;
  for (int r = 0; r < N_REGIONS; ++r) total += arena.peak[r];
  return total + 256;
}

extern "C" int kappai_forward(const kappai_model* model, const kappai_batch* batch,
                              void* workspace, size_t workspace_bytes, float* logits,
                              hipStream_t stream) {
  g_error[0] = 0;
  if (!model_ok(model) || !batch_ok(model, batch)) return (int)hipErrorInvalidValue;
  if (workspace == nullptr || (batch->n_logit_rows > 0 && logits == nullptr)) {
    snprintf(g_error, sizeof g_error, "kappai_forward: no workspace or no place for the logits");
    return (int)hipErrorInvalidValue;
  }
  // first the sizes of the four regions (the same walk without launches), then the step
  Arena dry;
  const int rc = run(model, batch, dry, nullptr, nullptr, true);
  if (rc != 0) return rc;
  Arena arena;
  char* base = reinterpret_cast<char*>(((uintptr_t)workspace + 255) / 256 * 256);
  size_t at = 0;
  for (int r = 0; r < N_REGIONS; ++r) {
    arena.offset[r] = at;
    arena.limit[r] = dry.peak[r];
    at += dry.peak[r];
  }
  if ((size_t)(base - (char*)workspace) + at > workspace_bytes) {
    snprintf(g_error, sizeof g_error, "kappai_forward: this batch needs %zu bytes of workspace, "
                                      "%zu were given", at + 256, workspace_bytes);
    return (int)hipErrorInvalidValue;
  }
  arena.base = base;
  return run(model, batch, arena, logits, stream, false);
}

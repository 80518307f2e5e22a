// kappai_forward: a whole step launched from C (see engine.h).
//
// This file holds no kernel and knows no part by name.  It owns what every part needs: the
// workspace that the activations of a step are cut from, the products with their choices by
// number of rows (which kernel, partial sums over K, rows in fragment order, the residual sum and
// a norm folded in), the registry of runners, and the walk itself: embedding, every call of the
// schedule through the function its description names, final norm and head.  The framework's own
// parts are registered from engine_parts.hip like anybody else's.
//
// kappai: an operation list run through a table of handlers that each operation registered
// (src/recipe.h:577-580, src/recipe/exec.c:467-517); order of a step src/recipe/exec.c:704-758.
#include "engine.h"
#include "gemm_rules.h"

#include <stdio.h>
#include <string.h>

#include <mutex>
#include <string>
#include <vector>

namespace {

thread_local char g_error[320];

// ---------------------------------------------------------------------------------------------
// workspace: four regions, each a stack that a dry run measures first
// ---------------------------------------------------------------------------------------------
enum Region { R_STEP = KAPPAI_REGION_STEP, R_CARRY_A = 1, R_CARRY_B = 2,
              R_BLOCK = KAPPAI_REGION_BLOCK, N_REGIONS = 4 };

struct Arena {
  char* base = nullptr;              // null: dry run, only the sizes are followed
  size_t offset[N_REGIONS] = {0, 0, 0, 0};
  size_t used[N_REGIONS] = {0, 0, 0, 0};
  size_t peak[N_REGIONS] = {0, 0, 0, 0};
  size_t limit[N_REGIONS] = {0, 0, 0, 0};
  bool overflow = false;

  void* take(int r, size_t bytes) {
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
  void reset(int r) { used[r] = 0; }
};

// The step as the walk sees it; runners see its first member only.
struct Step : kappai_step {
  const kappai_model* m;
  const kappai_batch* b;
  Arena* a;
  hipStream_t stream;
  bool dry;
  int status = 0;
  int carry_turn = 0;
  bool ok() const { return status == 0 && !a->overflow; }
};

Step& of(kappai_step* s) { return *static_cast<Step*>(s); }

#define LAUNCH(ctx, call)                         \
  do {                                            \
    if (!(ctx).dry && (ctx).ok()) {               \
      const int rc_ = (call);                     \
      if (rc_ != 0) (ctx).status = rc_;           \
    }                                             \
  } while (0)

inline size_t elem(int is_bf16) { return is_bf16 ? 2 : 4; }

void refuse(Step& c, const char* message) {
  snprintf(g_error, sizeof g_error, "kappai_forward: %s", message);
  c.status = (int)hipErrorInvalidValue;
}

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

// 25 to 128 rows: the kernel with 32 x 32 tiles gives a block 64 columns and takes K ranges that
// are multiples of 256; as many equal ranges (at most 8: the norm's row kernel adds up to eight
// planes, more take its slower form, 13 against 5 us) that up to 256 blocks stream the matrix
// (from sweeps at the 1.2B and 350M shapes: in_proj two and four, qkv four, out_proj eight and
// four, down eight and six; twice as many blocks were 5 to 40 % slower)
int split_k_rows32(int N, int K) {
  const long col_blocks = (N + 63) / 64;
  const int runs = K / KAPPAI_ROWS32_RUN;
  int split = 1;
  for (int d = 2; d <= 8 && d <= runs; ++d)
    if (runs % d == 0 && col_blocks * d <= 256) split = d;
  return split;
}

int split_k_for(int M, int N, int K) {
  if (M > KAPPAI_ROWS32_MIN_ROWS && M <= KAPPAI_ROWS32_MAX_ROWS && K % KAPPAI_ROWS32_RUN == 0 &&
      N % 16 == 0)
    return split_k_rows32(N, K);
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

// how the split decode kernel cuts n_keys keys of `rows` rows
void decode_splits(int kpw, int max_splits, int waves, int rows, int G, int n_keys,
                   int* keys_per_split, int* n_splits) {
  int s = max_splits;
  if ((n_keys + kpw - 1) / kpw < s) s = (n_keys + kpw - 1) / kpw;
  int by_waves = waves / (rows * G);
  if (by_waves < 1) by_waves = 1;
  if (by_waves < s) s = by_waves;
  if (s < 1) s = 1;
  *keys_per_split = ((n_keys + s - 1) / s + kpw - 1) / kpw * kpw;
  *n_splits = (n_keys + *keys_per_split - 1) / *keys_per_split;
}

// ---------------------------------------------------------------------------------------------
// what every part may ask of the step
// ---------------------------------------------------------------------------------------------
bool aligned16(const void* p) { return ((uintptr_t)p % 16) == 0; }

// Can the kernel for 1 to 16 rows of this matrix read rows in fragment order / scale its results?
int takes_kernel_order(const kappai_linear* lin, int D) {
  return lin != nullptr && !lin->w_is_f32 && lin->k == D && aligned16(lin->w) && lin->k % 8 == 0;
}

void* cast_to(Step& c, const void* x, size_t n, int from_bf16, int to_bf16) {
  void* out = c.a->take(R_BLOCK, n * elem(to_bf16));
  LAUNCH(c, c.m->kernels->cast(x, out, (long)n, from_bf16, to_bf16, c.stream));
  return out;
}

// RMSNorm by its own kernel.  rows: only these (the residual is then left alone).
kappai_rows rms_norm(Step& c, const kappai_fold* norm, float* resid, const kappai_carry& carry,
                     int M, const int* rows, int n_rows, int fragment) {
  const int D = c.m->width;
  const int n = rows ? n_rows : M;
  kappai_rows out = {};
  out.is_bf16 = c.m->compute_bf16;
  out.M = n;
  out.D = D;
  out.ld = D;
  out.frag = fragment ? 1 : 0;
  out.norm = norm;
  out.data = c.a->take(R_BLOCK, (size_t)(fragment ? 16 : n) * D * elem(out.is_bf16));
  const void* delta = nullptr;
  int delta_f32 = 0, n_part = 1;
  long pstride = 0;
  if (carry.kind == KAPPAI_CARRY_DELTA) {
    delta = carry.data;
    delta_f32 = carry.is_f32;
  } else if (carry.kind == KAPPAI_CARRY_PARTS) {
    delta = carry.data;
    delta_f32 = 1;
    n_part = carry.parts;
    pstride = (long)M * D;
  } else if (carry.kind == KAPPAI_CARRY_EMBEDDING) {
    refuse(c, "a norm kernel was asked for rows of a residual stream that is not filled yet");
    return out;
  }
  LAUNCH(c, c.m->kernels->add_rmsnorm(resid, delta, delta_f32, n_part, pstride, norm->w, out.data,
                                      rows, n, D, norm->eps, rows ? 0 : 1, out.is_bf16,
                                      fragment ? 1 : 0, c.stream));
  return out;
}

// Scaled rows or rows in fragment order that a kernel cannot take are made by the norm's own
// kernel from the residual stream instead.
kappai_rows plain_rows(Step& c, const kappai_rows& x, float* resid) {
  if (x.ss == nullptr && !x.frag) return x;
  if (x.norm == nullptr) {
    refuse(c, "rows in kernel order that name no norm cannot be made anew");
    return x;
  }
  kappai_carry none = {};
  return rms_norm(c, x.norm, resid, none, x.M, nullptr, 0, 0);
}

kappai_carry plain_carry(Step& c, kappai_carry carry, float* resid, int M) {
  const int D = c.m->width;
  kappai_carry out = {};
  switch (carry.kind) {
    case KAPPAI_CARRY_EMBEDDING:
      LAUNCH(c, c.m->kernels->embed_rows(c.b->tokens, c.m->embed_table, c.m->embed_is_bf16, resid,
                                         M, D, c.stream));
      return out;
    case KAPPAI_CARRY_SCALED:
      return out;                          // the sum is in the stream already
    case KAPPAI_CARRY_PARTS:
      out.kind = KAPPAI_CARRY_DELTA;
      out.is_f32 = 1;
      out.parts = 1;
      out.data = c.a->take(R_BLOCK, (size_t)M * D * 4);
      LAUNCH(c, c.m->kernels->sum_partials((const float*)carry.data, carry.parts, (long)M * D,
                                           (float*)out.data, c.stream));
      return out;
    default:
      return carry;
  }
}

bool fragment_fits(const Step& c, int M, int D) {         // 8 to 16 bfloat16 rows of whole pieces
  return c.m->compute_bf16 && M >= 1 && M <= 16 && D % 32 == 0 && D <= 8192;
}

// The products.  out_bf16: the dtype of a plain result.  partial_sums: the result may come as
// float planes over K ranges.  into: the product may add its result into the residual stream.
// region: where a result that outlives the block goes (the carry to the next norm).
kappai_carry linear(Step& c, kappai_rows x, const kappai_linear& lin, int out_bf16,
                    bool partial_sums, const kappai_into* into, int region) {
  const kappai_kernels& k = *c.m->kernels;
  const kappai_tuning& tune = c.m->tuning;
  kappai_carry out = {};
  out.parts = 1;
  const int M = x.M, K = x.D, N = lin.n;
  if (region < 0 || region >= N_REGIONS) {
    refuse(c, "a product was given a region of the workspace that does not exist");
    return out;
  }
  if (lin.k != K) {
    snprintf(g_error, sizeof g_error, "kappai_forward: rows of width %d meet a matrix [%d, %d]", K,
             lin.n, lin.k);
    c.status = (int)hipErrorInvalidValue;
    return out;
  }
  if (lin.w_is_f32) {
    // a matrix stored in 32 bits: true 32-bit arithmetic whatever the activations are
    if (x.ss != nullptr || x.frag) {
      refuse(c, "rows in kernel order reached a matrix stored in 32 bits");
      return out;
    }
    const float* xf = x.is_bf16 ? (const float*)cast_to(c, x.data, (size_t)M * K, 1, 0)
                                : (const float*)x.data;
    const int lda = x.is_bf16 ? K : x.ld;
    float* o = (float*)c.a->take(out_bf16 ? R_BLOCK : region, (size_t)M * N * 4);
    LAUNCH(c, k.gemm_f32(xf, (const float*)lin.w, lin.bias, o, M, N, K, M > 1 ? lda : K, N,
                         c.stream));
    out.kind = KAPPAI_CARRY_DELTA;
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
    out.kind = KAPPAI_CARRY_DELTA;
    out.is_f32 = out_bf16 ? 0 : 1;
    out.data = c.a->take(region, (size_t)M * N * elem(out_bf16));
    LAUNCH(c, k.gemm_bf16_any(xb, lin.w, lin.bias, out.data, M, N, K, lda, N, out_bf16 ? 0 : 1,
                              c.stream));
    return out;
  }
  if (into != nullptr && M <= tune.fused_max_rows) {
    // the result joins the residual stream inside the kernel
    const kappai_fold* norm = into->norm;
    void* rows = nullptr;
    float* ss = nullptr;
    int fragment = 0;
    if (norm != nullptr) {
      fragment = (M >= tune.fragment_rows_from && fragment_fits(c, M, N)) ? 1 : 0;
      rows = c.a->take(region, (size_t)(fragment ? 16 : M) * N * 2);
      ss = (float*)c.a->take(region, (size_t)((N + 7) / 8) * 16 * 4);
    }
    LAUNCH(c, k.gemm_bf16(xb, lin.w, lin.w_frag, lin.bias, nullptr, M, N, K, lda, N, 1, 0, 1,
                          x.frag, scaled ? x.ss : nullptr, scaled ? x.ss_parts : 0,
                          scaled ? x.eps : 0.f, into->resid, N, norm ? norm->w : nullptr, rows,
                          fragment, ss, c.stream));
    if (norm == nullptr) return out;             // nothing left to add
    out.kind = KAPPAI_CARRY_SCALED;
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
    out.kind = KAPPAI_CARRY_PARTS;
    out.is_f32 = 1;
    out.parts = ksplit;
    out.data = c.a->take(region, (size_t)ksplit * M * N * 4);
  } else {
    out.kind = KAPPAI_CARRY_DELTA;
    out.is_f32 = out_bf16 ? 0 : 1;
    out.data = c.a->take(region, (size_t)M * N * elem(out_bf16));
  }
  LAUNCH(c, k.gemm_bf16(xb, lin.w, lin.w_frag, lin.bias, out.data, M, N, K, lda, N,
                        (ksplit > 1 || !out_bf16) ? 1 : 0, 0, ksplit, x.frag,
                        scaled ? x.ss : nullptr, scaled ? x.ss_parts : 0, scaled ? x.eps : 0.f,
                        nullptr, 0, nullptr, nullptr, 0, nullptr, c.stream));
  return out;
}

// ---- the same, as runners call it -------------------------------------------------------------
const kappai_model* api_model(kappai_step* s) { return of(s).m; }
const kappai_batch* api_batch(kappai_step* s) { return of(s).b; }
hipStream_t api_stream(kappai_step* s) { return of(s).stream; }
int api_dry(kappai_step* s) { return of(s).dry ? 1 : 0; }
int api_ok(kappai_step* s) { return of(s).ok() ? 1 : 0; }
void* api_take(kappai_step* s, int region, size_t bytes) {
  if (region < 0 || region >= N_REGIONS) {
    refuse(of(s), "a part asked for memory from a region of the workspace that does not exist");
    return nullptr;
  }
  return of(s).a->take(region, bytes);
}
// The region for what a part hands to the norm after it.  What the region held is two parts old
// by now and has been consumed (the part's own input lies in the other region).
int api_carry_region(kappai_step* s) {
  Step& c = of(s);
  const int r = (c.carry_turn++ & 1) ? R_CARRY_B : R_CARRY_A;
  c.a->reset(r);
  return r;
}
void api_launched(kappai_step* s, int status) {
  if (status != 0 && of(s).status == 0) of(s).status = status;
}
void api_fail(kappai_step* s, const char* message) { refuse(of(s), message); }
kappai_carry api_linear(kappai_step* s, kappai_rows x, const kappai_linear* lin, int out_bf16,
                        int partial_sums, const kappai_into* into, int region) {
  return linear(of(s), x, *lin, out_bf16, partial_sums != 0, into, region);
}
kappai_rows api_plain_rows(kappai_step* s, kappai_rows x, float* resid) {
  return plain_rows(of(s), x, resid);
}
kappai_carry api_plain_carry(kappai_step* s, kappai_carry carry, float* resid, int M) {
  return plain_carry(of(s), carry, resid, M);
}
void* api_cast(kappai_step* s, const void* x, size_t n, int from_bf16, int to_bf16) {
  return cast_to(of(s), x, n, from_bf16, to_bf16);
}
kappai_rows api_rms_norm(kappai_step* s, const kappai_fold* norm, float* resid, kappai_carry carry,
                         int M, const int* rows, int n_rows, int fragment) {
  return rms_norm(of(s), norm, resid, carry, M, rows, n_rows, fragment);
}

const kappai_step_api g_api = {api_model,      api_batch,       api_stream,    api_dry,
                               api_ok,         api_take,        api_carry_region, api_launched,
                               api_fail,       api_linear,      api_plain_rows, api_plain_carry,
                               api_cast,       takes_kernel_order, api_rms_norm};

// ---------------------------------------------------------------------------------------------
// the registry of runners
// ---------------------------------------------------------------------------------------------
struct Runner {
  std::string name;
  int kind;
  void* fn;
  int desc_bytes;
};
std::mutex& registry_lock() {
  static std::mutex m;
  return m;
}
std::vector<Runner>& registry() {
  static std::vector<Runner> r;
  return r;
}

// ---------------------------------------------------------------------------------------------
// the walk
// ---------------------------------------------------------------------------------------------
bool model_ok(const kappai_model* m) {
  if (m == nullptr || m->abi != KAPPAI_ENGINE_ABI || m->kernels == nullptr || m->n_calls < 0 ||
      m->width < 1 || m->vocab < 1 || (m->n_calls > 0 && m->calls == nullptr) ||
      m->final_norm.run == nullptr) {
    snprintf(g_error, sizeof g_error, "kappai_forward: the model description is incomplete or was "
                                      "filled in for another version of this library");
    return false;
  }
  for (int ci = 0; ci < m->n_calls; ++ci)
    if (m->calls[ci].run == nullptr) {
      snprintf(g_error, sizeof g_error, "kappai_forward: call %d of the schedule names no runner",
               ci);
      return false;
    }
  return true;
}

int run(const kappai_model* m, const kappai_batch* b, Arena& arena, float* logits,
        hipStream_t stream, bool dry) {
  Step c;
  c.api = &g_api;
  c.m = m;
  c.b = b;
  c.a = &arena;
  c.stream = stream;
  c.dry = dry;
  const kappai_kernels& k = *m->kernels;
  const int T = b->n_rows, D = m->width;
  float* resid = (float*)arena.take(R_STEP, (size_t)T * D * 4);
  // The head as the part that takes the final norm's rows.
  kappai_part head_part = {};
  head_part.flags = KAPPAI_TAKES_DEFERRED_ROWS;
  head_part.first = &m->head;
  // After the last call comes the final norm, whose rows the head takes; a block can make them
  // only when every row wants its logits, in the rows' order, and the head reads such rows.
  const bool every_row = b->logits_of_every_row && b->n_logit_rows == T &&
                         takes_kernel_order(&m->head, D);
  // the embedding is looked up by the first norm that runs (which may do both in one kernel)
  kappai_carry carry = {};
  carry.kind = KAPPAI_CARRY_EMBEDDING;
  if (m->on_embedding.run != nullptr) {
    // something changes the embedded rows: they are looked up now
    carry = plain_carry(c, carry, resid, T);
    m->on_embedding.run(&c, m->on_embedding.desc, resid, T);
  }
  for (int ci = 0; ci < m->n_calls && c.ok(); ++ci) {
    const kappai_call& call = m->calls[ci];
    const kappai_call* next = ci + 1 < m->n_calls ? &m->calls[ci + 1] : nullptr;
    arena.reset(R_BLOCK);
    const kappai_norm_part* after_norm = next ? next->first_norm
                                              : (every_row ? &m->final_norm : nullptr);
    const kappai_part* after_consumer = next ? next->first_consumer
                                             : (every_row ? &head_part : nullptr);
    carry = call.run(&c, call.desc, resid, carry, after_norm, after_consumer);
  }
  if (c.ok() && b->n_logit_rows > 0) {
    arena.reset(R_BLOCK);
    const int n = b->n_logit_rows;
    // rows made for the final norm by the last product stand for all rows in order
    const bool made = carry.kind == KAPPAI_CARRY_SCALED && every_row;
    kappai_rows xb = m->final_norm.run(&c, m->final_norm.desc, resid, carry, T,
                                       made ? nullptr : b->logit_rows, made ? 0 : n, &head_part);
    if (c.ok() && (xb.M != n || xb.D != D)) refuse(c, "the final norm returned rows of another shape");
    // the head: a plain product with float results, straight into the caller's tensor
    const kappai_linear& head = m->head;
    if (!c.ok()) {
    } else if (head.w_is_f32) {
      xb = plain_rows(c, xb, resid);
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
      else if (head.w != nullptr && !xb.frag && xb.ss == nullptr)
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

bool batch_ok(const kappai_batch* b) {
  if (b == nullptr || b->n_rows < 1 || b->n_segments < 1 || b->n_logit_rows < 0 ||
      b->n_groups < 0 || b->n_groups > KAPPAI_MAX_GROUPS) {
    snprintf(g_error, sizeof g_error, "kappai_forward: a step needs rows and segments");
    return false;
  }
  return true;
}

}  // namespace

extern "C" int kappai_register_runner(const char* name, int kind, void* fn, int desc_bytes) {
  if (name == nullptr || fn == nullptr || kind < KAPPAI_RUNNER_PART || kind > KAPPAI_RUNNER_EMBEDDED ||
      desc_bytes < 0) {
    snprintf(g_error, sizeof g_error, "kappai_register_runner: a runner needs a name, a kind and "
                                      "a function");
    return (int)hipErrorInvalidValue;
  }
  std::lock_guard<std::mutex> hold(registry_lock());
  for (const Runner& r : registry())
    if (r.name == name && r.kind == kind) {
      if (r.fn == fn && r.desc_bytes == desc_bytes) return 0;
      snprintf(g_error, sizeof g_error, "kappai_register_runner: '%s' is registered already, with "
                                        "another function or description", name);
      return (int)hipErrorInvalidValue;
    }
  registry().push_back(Runner{name, kind, fn, desc_bytes});
  return 0;
}

extern "C" void* kappai_runner(const char* name, int kind, int* desc_bytes) {
  if (name == nullptr) return nullptr;
  std::lock_guard<std::mutex> hold(registry_lock());
  for (const Runner& r : registry())
    if (r.name == name && r.kind == kind) {
      if (desc_bytes != nullptr) *desc_bytes = r.desc_bytes;
      return r.fn;
    }
  return nullptr;
}

extern "C" int kappai_engine_layout(int* sizes, int n) {
  const int mine[] = {KAPPAI_ENGINE_ABI,
                      (int)sizeof(kappai_kernels),
                      (int)sizeof(kappai_attention_kernels),
                      (int)sizeof(kappai_linear),
                      (int)sizeof(kappai_fold),
                      (int)sizeof(kappai_rows),
                      (int)sizeof(kappai_carry),
                      (int)sizeof(kappai_part),
                      (int)sizeof(kappai_norm_part),
                      (int)sizeof(kappai_call),
                      (int)sizeof(kappai_tuning),
                      (int)sizeof(kappai_model),
                      (int)sizeof(kappai_batch)};
  const int count = (int)(sizeof mine / sizeof mine[0]);
  for (int i = 0; i < n && i < count; ++i) sizes[i] = mine[i];
  return count;
}

extern "C" const char* kappai_forward_error(void) { return g_error; }

extern "C" int kappai_split_k_for(int M, int N, int K) { return split_k_for(M, N, K); }

extern "C" void kappai_decode_splits(int keys_per_wave, int max_splits, int waves, int rows, int G,
                                     int n_keys, int* keys_per_split, int* n_splits) {
  decode_splits(keys_per_wave, max_splits, waves, rows, G, n_keys, keys_per_split, n_splits);
}

extern "C" size_t kappai_forward_workspace_bytes(const kappai_model* model,
                                                 const kappai_batch* batch) {
  g_error[0] = 0;
  if (!model_ok(model) || !batch_ok(batch)) return 0;
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
  if (!model_ok(model) || !batch_ok(batch)) return (int)hipErrorInvalidValue;
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

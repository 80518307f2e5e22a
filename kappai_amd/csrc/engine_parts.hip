// The runners of the framework's own parts: RMSNorm, the gated short convolution, grouped-query
// attention over the paged cache, the SwiGLU feed-forward and the pre-norm block.
//
// Each is the host side of the part of the same name (parts/*.py) written once more in C: the
// order of its kernels and the choices that depend on the number of rows.  The same step run from
// the host's parts, kernel by kernel, gives bit for bit the same logits.  They reach the step
// through kappai_step_api only and register themselves under a name when the library is loaded,
// as a part from anywhere else would (kappai: RECIPE_REGISTER, src/recipe.h:577-580).
//
// Order of a block as kappai's (src/models/lfm.c:7-62, src/recipe/builders.c:378-388):
// x += mixer(norm(x)); x += ffn(norm(x)).
#include "engine_parts.h"

#include <stdio.h>

namespace {

#define LAUNCH(s, call)                                         \
  do {                                                          \
    if (!(s)->api->dry(s) && (s)->api->ok(s)) (s)->api->launched((s), (call)); \
  } while (0)

inline size_t elem(int is_bf16) { return is_bf16 ? 2 : 4; }
bool aligned16(const void* p) { return ((uintptr_t)p % 16) == 0; }

bool fragment_fits(const kappai_model& m, int M, int D) {   // 8 to 16 bfloat16 rows, whole pieces
  return m.compute_bf16 && M >= 1 && M <= 16 && D % 32 == 0 && D <= 8192;
}

kappai_rows rows_of(void* data, int M, int D, int is_bf16) {
  kappai_rows r = {};
  r.data = data;
  r.is_bf16 = is_bf16;
  r.M = M;
  r.D = D;
  r.ld = D;
  return r;
}

// ---------------------------------------------------------------------------------------------
// "norm.rms" (parts/norm.py)
// ---------------------------------------------------------------------------------------------
// The rows that `consumer` reads after the norm: scaled rows made for this norm go through as
// they are, else the norm's kernel runs, writing fragment order when that suits the number of
// rows and the consumer.  The first norm of a step looks the embedding up in the same kernel.
kappai_rows rms_norm(kappai_step* s, const void* desc, float* resid, kappai_carry carry, int M,
                     const int* rows, int n_rows, const kappai_part* consumer) {
  const kappai_step_api& api = *s->api;
  const kappai_fold* norm = static_cast<const kappai_fold*>(desc);
  const kappai_model& m = *api.model(s);
  const int D = m.width;
  const bool kernel_order = consumer != nullptr && (consumer->flags & KAPPAI_TAKES_DEFERRED_ROWS) &&
                            api.takes_kernel_order(consumer->first, D);
  const int n = rows ? n_rows : M;
  if (carry.kind == KAPPAI_CARRY_EMBEDDING) {
    // the embedding and this norm are one kernel where the norm's row kernel takes the width
    // (the same arithmetic as the two kernels, bit for bit)
    const bool both = rows == nullptr && D % 8 == 0 && D <= 8192 &&
                      (m.embed_is_bf16 != 2 || D % 32 == 0) && aligned16(m.embed_table) &&
                      aligned16(norm->w);
    if (both) {
      const bool fragment = kernel_order && M >= m.tuning.fragment_rows_min &&
                            fragment_fits(m, M, D);
      kappai_rows out = rows_of(nullptr, M, D, m.compute_bf16);
      out.frag = fragment ? 1 : 0;
      out.norm = norm;
      out.data = api.take(s, KAPPAI_REGION_BLOCK, (size_t)(fragment ? 16 : M) * D * elem(out.is_bf16));
      LAUNCH(s, m.kernels->embed_rmsnorm(api.batch(s)->tokens, m.embed_table, m.embed_is_bf16,
                                         resid, norm->w, out.data, M, D, norm->eps, out.is_bf16,
                                         fragment ? 1 : 0, api.stream(s)));
      return out;
    }
    carry = api.plain_carry(s, carry, resid, M);
  }
  if (carry.kind == KAPPAI_CARRY_SCALED) {
    if (rows == nullptr && carry.scaled.norm == norm && kernel_order) return carry.scaled;
    carry = kappai_carry{};                      // the sum is in the residual already
    return api.rms_norm(s, norm, resid, carry, M, rows, n_rows, 0);
  }
  const bool fragment = kernel_order && n >= m.tuning.fragment_rows_min && fragment_fits(m, n, D) &&
                        (carry.kind != KAPPAI_CARRY_PARTS || carry.parts <= 8);
  return api.rms_norm(s, norm, resid, carry, M, rows, n_rows, fragment ? 1 : 0);
}

// ---------------------------------------------------------------------------------------------
// "mixer.conv" (parts/shortconv.py)
// ---------------------------------------------------------------------------------------------
// When in_proj and qkv hand their consumer partial sums over K ranges
bool takes_partial_sums(const kappai_model& m, const kappai_batch& b, int M) {
  return M > m.tuning.partial_sums_min_rows &&
         (M <= m.tuning.partial_sums_max_rows || b.max_segment_rows == 1);
}

kappai_carry conv_mixer(kappai_step* s, const void* desc, kappai_rows x, float* resid,
                        const kappai_into* into) {
  const kappai_step_api& api = *s->api;
  const kappai_conv_mixer& L = *static_cast<const kappai_conv_mixer*>(desc);
  const kappai_model& m = *api.model(s);
  const kappai_kernels& k = *m.kernels;
  const kappai_batch& b = *api.batch(s);
  const kappai_tuning& tune = m.tuning;
  const int M = x.M, D = m.width, taps = L.taps_per_channel;
  const int region = api.carry_region(s);
  const bool wide_enough = D >= tune.fused_step_min_width ||
                           (D >= tune.fused_step_narrow_width && M <= tune.fused_step_narrow_rows);
  kappai_carry none = {};
  if (b.max_segment_rows == 1 && M <= 64 && x.is_bf16 && !L.in_proj.w_is_f32 && D % 16 == 0 &&
      wide_enough) {
    // decode: projection, convolution and state shift in one kernel
    if (!api.takes_kernel_order(&L.in_proj, D)) x = api.plain_rows(s, x, resid);
    const int c_frag = (M >= tune.fragment_rows_from && M <= tune.fused_max_rows && D % 32 == 0 &&
                        api.takes_kernel_order(&L.out_proj, D));
    void* y = api.take(s, KAPPAI_REGION_BLOCK, (size_t)(c_frag ? 16 : M) * D * 2);
    LAUNCH(s, k.gemm_bf16_shortconv_step(x.data, L.in_proj.w, L.in_proj.w_frag, L.in_proj.bias, y,
                                         M, D, D, M > 1 ? x.ld : D, L.taps, L.conv_bias, L.state,
                                         b.seg_pos0, b.seg_slot, taps, x.frag, x.ss, x.ss_parts,
                                         x.eps, c_frag, api.stream(s)));
    kappai_rows yr = rows_of(y, M, D, 1);
    yr.frag = c_frag;
    return api.linear(s, yr, &L.out_proj, m.compute_bf16, 1, into, region);
  }
  // more than 16 rows (decode at any batch size, short prompt portions): the projection may come
  // as sums over ranges of its input dimension, which the conv kernel adds up
  const bool parts = takes_partial_sums(m, b, M);
  kappai_carry proj = api.linear(s, x, &L.in_proj, m.compute_bf16, parts, nullptr,
                                 KAPPAI_REGION_BLOCK);
  if (!api.ok(s)) return none;
  void* y;
  int y_bf16;
  if (proj.kind == KAPPAI_CARRY_PARTS) {
    y_bf16 = 1;
    y = api.take(s, KAPPAI_REGION_BLOCK, (size_t)M * D * 2);
    LAUNCH(s, k.shortconv_parts((const float*)proj.data, proj.parts, L.taps, L.conv_bias, L.state,
                                y, b.row_seg, b.seg_start, b.seg_pos0, b.seg_slot, M, b.n_segments,
                                D, taps, api.stream(s)));
  } else {
    y_bf16 = proj.is_f32 ? 0 : 1;
    y = api.take(s, KAPPAI_REGION_BLOCK, (size_t)M * D * elem(y_bf16));
    LAUNCH(s, k.shortconv(proj.data, L.taps, L.conv_bias, L.state, y, b.row_seg, b.seg_start,
                          b.seg_pos0, b.seg_slot, M, b.n_segments, D, taps, y_bf16,
                          api.stream(s)));
  }
  return api.linear(s, rows_of(y, M, D, y_bf16), &L.out_proj, m.compute_bf16, 1, into, region);
}

// ---------------------------------------------------------------------------------------------
// "mixer.attention" (parts/attention.py with ops.qk_norm_rope_store and ops.paged_attention)
// ---------------------------------------------------------------------------------------------
// few keys go to the kernel that splits them over the waves of a block (ops.decode_form)
int decode_keys(const kappai_batch& b, const kappai_attention_mixer& L) {
  int n_keys = b.max_position + 1;
  if (L.window) n_keys = (n_keys < L.window ? n_keys : L.window) + 32;
  return n_keys;
}
bool decode_block_form(const kappai_model& m, const kappai_batch& b,
                       const kappai_attention_mixer& L, int rep) {
  return L.mfma->decode_block_waves(rep) > 0 &&
         decode_keys(b, L) <= m.tuning.decode_block_max_keys;
}

kappai_carry attention_mixer(kappai_step* s, const void* desc, kappai_rows x, float* resid,
                             const kappai_into* into) {
  const kappai_step_api& api = *s->api;
  const kappai_attention_mixer& L = *static_cast<const kappai_attention_mixer*>(desc);
  const kappai_model& m = *api.model(s);
  const kappai_kernels& k = *m.kernels;
  const kappai_batch& b = *api.batch(s);
  const kappai_tuning& tune = m.tuning;
  hipStream_t stream = api.stream(s);
  const int M = x.M, H = L.heads, G = L.kv_heads, d = L.head_dim, ps = m.page_size;
  const int region = api.carry_region(s);
  kappai_carry none = {};
  kappai_linear qkv = L.qkv;
  if (L.shared_cache) {          // the q rows of the stacked matrix, whole pieces of 16 rows
    qkv.n = H * d;
    if (qkv.w_frag != nullptr && (H * d) % 16) qkv.w_frag = nullptr;
  }
  if (!api.takes_kernel_order(&qkv, x.D)) x = api.plain_rows(s, x, resid);
  const bool parts = takes_partial_sums(m, b, M);
  kappai_carry proj = api.linear(s, x, &qkv, m.compute_bf16, parts, nullptr, KAPPAI_REGION_BLOCK);
  if (!api.ok(s)) return none;
  char msg[200];
  if (L.rot_mode != 0 && b.max_position >= L.rot_positions) {
    snprintf(msg, sizeof msg, "position %d is beyond the rotation table of %d positions",
             b.max_position, L.rot_positions);
    api.fail(s, msg);
    return none;
  }
  if (L.group < 0 || L.group >= b.n_groups) {
    snprintf(msg, sizeof msg, "the batch has no block tables of group %d", L.group);
    api.fail(s, msg);
    return none;
  }
  const int* tables = b.block_tables[L.group];
  const int max_blocks = b.max_blocks[L.group];
  const int store = L.shared_cache ? 0 : 1;
  const bool single = b.max_segment_rows == 1;
  // decode: the attention kernels take the projection as it is and do norm, rotation and store
  // themselves (parts/attention.py: _prologue_in_kernel)
  const bool qk_in_kernel =
      M <= tune.fused_qk && single && proj.kind == KAPPAI_CARRY_DELTA && !proj.is_f32 &&
      L.mfma != nullptr && H / G <= 16 && qkv.n % 8 == 0 && aligned16(proj.data) && ps % 16 == 0 &&
      d % 16 == 0 && d <= 256 && (L.rot_mode == 0 || (L.rot_mode == 1 && L.rot_dim == d)) &&
      L.mfma->decode_takes_qk != nullptr && L.mfma->decode_takes_qk() &&
      !decode_block_form(m, b, L, H / G);
  // q in place in the projection, or (from partial sums) a new bfloat16 [M, H d]
  void* q;
  int q_stride, q_bf16;
  if (qk_in_kernel) {
    q_bf16 = 1;
    q_stride = qkv.n;
    q = proj.data;
  } else if (proj.kind == KAPPAI_CARRY_PARTS) {
    q_bf16 = 1;
    q_stride = H * d;
    q = api.take(s, KAPPAI_REGION_BLOCK, (size_t)M * H * d * 2);
    LAUNCH(s, k.qk_norm_rope_store(nullptr, qkv.n, L.q_norm_w, L.k_norm_w, L.qk_eps, L.cos_table,
                                   L.sin_table, L.rot_mode ? L.rot_dim : 0, L.rot_mode, L.k_pool,
                                   L.v_pool, b.row_pos, b.row_seg, store ? tables : nullptr,
                                   store ? max_blocks : 0, M, H, G, d, ps, store, 1,
                                   (const float*)proj.data, proj.parts, q, H * d, stream));
  } else {
    q_bf16 = proj.is_f32 ? 0 : 1;
    q_stride = qkv.n;
    q = proj.data;
    LAUNCH(s, k.qk_norm_rope_store(q, q_stride, L.q_norm_w, L.k_norm_w, L.qk_eps, L.cos_table,
                                   L.sin_table, L.rot_mode ? L.rot_dim : 0, L.rot_mode, L.k_pool,
                                   L.v_pool, b.row_pos, b.row_seg, store ? tables : nullptr,
                                   store ? max_blocks : 0, M, H, G, d, ps, store, q_bf16, nullptr,
                                   0, nullptr, H * d, stream));
  }
  void* ctx = api.take(s, KAPPAI_REGION_BLOCK, (size_t)M * H * d * elem(q_bf16));
  const float* cos_t = L.rot_mode ? L.cos_table : nullptr;
  const float* sin_t = L.rot_mode ? L.sin_table : nullptr;
  const bool mfma_ok = q_bf16 && L.mfma != nullptr && ps % 16 == 0 && d % 16 == 0 && d <= 256 &&
                       q_stride % 8 == 0 && aligned16(q);
  // the tables that the host's part asked the step for (AttentionTiles): the segments' tiles, the
  // single rows left out of them and the largest of their positions
  auto table_ok = [](int at) { return at >= 0 && at < KAPPAI_MAX_TABLES; };
  const int* q_tiles = table_ok(L.tiles_table) ? b.tables[L.tiles_table] : nullptr;
  const int n_tiles = table_ok(L.tiles_table) ? b.table_rows[L.tiles_table] : 0;
  const int* lone_rows = table_ok(L.lone_table) ? b.tables[L.lone_table] : nullptr;
  const int n_lone_rows = table_ok(L.lone_table) ? b.table_rows[L.lone_table] : 0;
  const int max_lone_position = table_ok(L.lone_number) ? b.numbers[L.lone_number] : -1;
  if (mfma_ok && single && H / G <= 16) {
    const int n_keys = decode_keys(b, L);
    const int block_waves = L.mfma->decode_block_waves(H / G);
    if (decode_block_form(m, b, L, H / G)) {
      LAUNCH(s, L.mfma->attn_decode_block(q, q_stride, L.k_pool, L.v_pool, ctx, H * d, b.row_pos,
                                          b.row_seg, tables, max_blocks, M, H, G, ps, L.window,
                                          L.scale, block_waves, stream));
    } else {
      int keys_per_split, n_splits;
      kappai_decode_splits(L.mfma->keys_per_wave(), tune.decode_max_splits, tune.decode_waves, M,
                           G, n_keys, &keys_per_split, &n_splits);
      float* part_o = (float*)api.take(s, KAPPAI_REGION_BLOCK, (size_t)M * H * n_splits * d * 4);
      float* part_ml = (float*)api.take(s, KAPPAI_REGION_BLOCK, (size_t)M * H * n_splits * 2 * 4);
      if (qk_in_kernel)
        LAUNCH(s, L.mfma->attn_decode_qk(q, q_stride, L.k_pool, L.v_pool, ctx, H * d, part_o,
                                         part_ml, b.row_pos, b.row_seg, tables, max_blocks, M, H,
                                         G, ps, L.window, L.scale, keys_per_split, n_splits,
                                         L.q_norm_w, L.k_norm_w, L.qk_eps, cos_t, sin_t, store,
                                         stream));
      else
        LAUNCH(s, L.mfma->attn_decode(q, q_stride, L.k_pool, L.v_pool, ctx, H * d, part_o, part_ml,
                                      b.row_pos, b.row_seg, tables, max_blocks, M, H, G, ps,
                                      L.window, L.scale, keys_per_split, n_splits, stream));
    }
  } else if (mfma_ok && q_tiles != nullptr) {
    LAUNCH(s, L.mfma->attn_prefill(q, q_stride, L.k_pool, L.v_pool, ctx, H * d, q_tiles,
                                   n_tiles, b.row_pos, tables, max_blocks, H, G, ps, L.window,
                                   L.scale, 0, stream));
    if (lone_rows != nullptr && n_lone_rows > 0) {
      // the single decoded tokens beside the portions: keys split over blocks
      if (H / G > 16 || max_lone_position < 0) {
        api.fail(s, "rows left out of the tiles need the decode kernel and their largest position");
        return none;
      }
      const int R = n_lone_rows;
      int n_keys = max_lone_position + 1;
      if (L.window) n_keys = (n_keys < L.window ? n_keys : L.window) + 32;
      int keys_per_split, n_splits;
      kappai_decode_splits(L.mfma->keys_per_wave(), tune.decode_max_splits, tune.decode_waves, R,
                           G, n_keys, &keys_per_split, &n_splits);
      float* part_o = (float*)api.take(s, KAPPAI_REGION_BLOCK, (size_t)R * H * n_splits * d * 4);
      float* part_ml = (float*)api.take(s, KAPPAI_REGION_BLOCK, (size_t)R * H * n_splits * 2 * 4);
      LAUNCH(s, L.mfma->attn_decode_rows(q, q_stride, L.k_pool, L.v_pool, ctx, H * d, part_o,
                                         part_ml, lone_rows, b.row_pos, b.row_seg, tables,
                                         max_blocks, R, H, G, ps, L.window, L.scale,
                                         keys_per_split, n_splits, stream));
    }
  } else {
    LAUNCH(s, k.paged_attention_rows(q, q_stride, L.k_pool, L.v_pool, ctx, H * d, b.row_pos,
                                     b.row_seg, tables, max_blocks, M, H, G, d, ps, L.window,
                                     L.scale, q_bf16, stream));
  }
  return api.linear(s, rows_of(ctx, M, H * d, q_bf16), &L.out, m.compute_bf16, 1, into, region);
}

// ---------------------------------------------------------------------------------------------
// "feed_forward.swiglu" (parts/feed_forward.py)
// ---------------------------------------------------------------------------------------------
kappai_carry swiglu_ffn(kappai_step* s, const void* desc, kappai_rows x, float* resid,
                        const kappai_into* into) {
  const kappai_step_api& api = *s->api;
  const kappai_swiglu& L = *static_cast<const kappai_swiglu*>(desc);
  const kappai_model& m = *api.model(s);
  const kappai_kernels& k = *m.kernels;
  const kappai_tuning& tune = m.tuning;
  const int M = x.M, D = m.width, F = L.hidden;
  const int region = api.carry_region(s);
  kappai_carry none = {};
  if (L.fused && x.is_bf16) {
    if (!api.takes_kernel_order(&L.gate_up, D)) x = api.plain_rows(s, x, resid);
    const int c_frag = (M >= tune.fragment_rows_from && M <= tune.fused_max_rows && F % 32 == 0 &&
                        api.takes_kernel_order(&L.down, F));
    void* act = api.take(s, KAPPAI_REGION_BLOCK, (size_t)(c_frag ? 16 : M) * F * 2);
    LAUNCH(s, k.gemm_bf16_swiglu(x.data, L.gate_up.w, L.gate_up.w_frag, act, M, F, D,
                                 M > 1 ? x.ld : D, F, 0, x.frag, x.ss, x.ss_parts, x.eps, c_frag,
                                 api.stream(s)));
    kappai_rows ar = rows_of(act, M, F, 1);
    ar.frag = c_frag;
    return api.linear(s, ar, &L.down, m.compute_bf16, 1, into, region);
  }
  kappai_carry gu = api.linear(s, x, &L.gate_up, m.compute_bf16, 0, nullptr, KAPPAI_REGION_BLOCK);
  if (!api.ok(s)) return none;
  const int act_bf16 = gu.is_f32 ? 0 : 1;
  void* act = api.take(s, KAPPAI_REGION_BLOCK, (size_t)M * F * elem(act_bf16));
  LAUNCH(s, k.swiglu(gu.data, act, M, F, act_bf16, api.stream(s)));
  return api.linear(s, rows_of(act, M, F, act_bf16), &L.down, m.compute_bf16, 1, into, region);
}

// ---------------------------------------------------------------------------------------------
// "block.pre_norm" (parts/block.py)
// ---------------------------------------------------------------------------------------------
// The norm that `producer`'s last product may fold in: one that can be folded, before a part that
// takes rows still to be divided by their root mean square.
const kappai_fold* fold_for(const kappai_norm_part* norm, const kappai_part* consumer) {
  if (norm == nullptr || consumer == nullptr || norm->fold == nullptr) return nullptr;
  return (consumer->flags & KAPPAI_TAKES_DEFERRED_ROWS) ? norm->fold : nullptr;
}

kappai_carry pre_norm_block(kappai_step* s, const void* desc, float* resid, kappai_carry carry,
                            const kappai_norm_part* after_norm, const kappai_part* after_consumer) {
  const kappai_step_api& api = *s->api;
  const kappai_pre_norm_block& B = *static_cast<const kappai_pre_norm_block*>(desc);
  const int T = api.batch(s)->n_rows;
  kappai_carry none = {};
  kappai_rows x = B.mixer_norm.run(s, B.mixer_norm.desc, resid, carry, T, nullptr, 0, &B.mixer);
  if (!api.ok(s)) return none;
  const kappai_into into_ffn = {resid, fold_for(&B.ffn_norm, &B.feed_forward)};
  const kappai_carry mixed = B.mixer.run(
      s, B.mixer.desc, x, resid, (B.mixer.flags & KAPPAI_ADDS_RESIDUAL) ? &into_ffn : nullptr);
  if (!api.ok(s)) return none;
  kappai_rows x2 = B.ffn_norm.run(s, B.ffn_norm.desc, resid, mixed, T, nullptr, 0, &B.feed_forward);
  if (!api.ok(s)) return none;
  const kappai_into into_next = {resid, fold_for(after_norm, after_consumer)};
  return B.feed_forward.run(s, B.feed_forward.desc, x2, resid,
                            (B.feed_forward.flags & KAPPAI_ADDS_RESIDUAL) ? &into_next : nullptr);
}

// registered when the library is loaded
struct Registration {
  Registration() {
    kappai_register_runner("norm.rms", KAPPAI_RUNNER_NORM, (void*)rms_norm, sizeof(kappai_fold));
    kappai_register_runner("mixer.conv", KAPPAI_RUNNER_PART, (void*)conv_mixer,
                           sizeof(kappai_conv_mixer));
    kappai_register_runner("mixer.attention", KAPPAI_RUNNER_PART, (void*)attention_mixer,
                           sizeof(kappai_attention_mixer));
    kappai_register_runner("feed_forward.swiglu", KAPPAI_RUNNER_PART, (void*)swiglu_ffn,
                           sizeof(kappai_swiglu));
    kappai_register_runner("block.pre_norm", KAPPAI_RUNNER_BLOCK, (void*)pre_norm_block,
                           sizeof(kappai_pre_norm_block));
  }
} g_registration;

}  // namespace

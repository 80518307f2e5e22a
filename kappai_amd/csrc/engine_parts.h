// The descriptions of the framework's own parts, as their runners in engine_parts.hip read them
// and as the host's part classes fill them in (parts/*.py).  Nothing outside these two places
// reads them: to the walk in engine.hip they are bytes behind a pointer.
#pragma once
#include "engine.h"

#ifdef __cplusplus
extern "C" {
#endif

// "norm.rms" reads a kappai_fold.

// "mixer.conv": gated short convolution (parts/shortconv.py)
typedef struct kappai_conv_mixer {
  kappai_linear in_proj, out_proj;
  const float* taps;                // [width, taps_per_channel]
  const float* conv_bias;           // [width] or null
  int taps_per_channel;
  float* state;                     // [slots, width, taps_per_channel - 1]
} kappai_conv_mixer;

// "mixer.attention": grouped-query attention over the paged cache (parts/attention.py)
typedef struct kappai_attention_mixer {
  kappai_linear qkv;                // q, k, v rows stacked (q first)
  kappai_linear out;
  const float* q_norm_w;            // [head_dim] or null
  const float* k_norm_w;
  float qk_eps;
  int heads, kv_heads, head_dim, window;
  float scale;
  const float* cos_table;           // [positions, rot_dim / 2] or null
  const float* sin_table;
  int rot_dim, rot_mode, rot_positions;
  void* k_pool;                     // [pages, kv_heads, page, head_dim]
  void* v_pool;                     // [pages, kv_heads, head_dim, page]
  int group;                        // which block tables of the batch
  int shared_cache;                 // reads the keys another call stored: q only, nothing stored
  const kappai_attention_kernels* mfma;
  // places in kappai_batch::tables / numbers: the tiles of the step's segments ([tiles, 4]), the
  // single rows left out of them, and the largest position among those (see AttentionTiles in
  // parts/attention.py)
  int tiles_table, lone_table, lone_number;
} kappai_attention_mixer;

// "feed_forward.swiglu" (parts/feed_forward.py)
typedef struct kappai_swiglu {
  kappai_linear gate_up;            // gate and up rows (interleaved in 16s when fused)
  kappai_linear down;
  int hidden;
  int fused;
} kappai_swiglu;

// "block.pre_norm": x += mixer(norm(x)); x += feed_forward(norm(x)) (parts/block.py)
typedef struct kappai_pre_norm_block {
  kappai_norm_part mixer_norm;
  kappai_part mixer;
  kappai_norm_part ffn_norm;
  kappai_part feed_forward;
} kappai_pre_norm_block;

#ifdef __cplusplus
}
#endif

// The C side of a step: one call that launches every kernel of a forward pass.
//
// kappai's entry points are C (engine_init / engine_run / engine_shutdown, src/engine.h:12-17;
// one forward call compute_forward_rows over a row description, src/compute.h:120-149,
// src/recipe/exec.c:704-758).  Here the host that owns requests, cache bookkeeping and scheduling
// is Python; what it hands down for a step is what this header describes: the model as a flat list
// of layer calls with the addresses of their tensors (kappai_model), the rows of the step with
// their tables (kappai_batch), a workspace, and the place for the logits.  kappai_forward then
// runs the whole step on the given stream without returning to the host in between.
//
// The description covers what the framework's own parts are: pre-norm blocks (RMSNorm) around a
// gated short convolution or a grouped-query attention over the paged cache, and a SwiGLU
// feed-forward.  A model with parts of another kind runs its steps from the host, part by part.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define KAPPAI_ENGINE_ABI 8          // bumped with every change of the structs below
#define KAPPAI_MAX_GROUPS 8          // paged groups a batch can carry block tables for

// ---- the kernels' launchers, by address (they live in libraries of their own) ---------------
typedef struct kappai_kernels {
  int (*embed_rows)(const int*, const void*, int, float*, int, int, hipStream_t);
  int (*embed_rmsnorm)(const int*, const void*, int, float*, const float*, void*, int, int, float,
                       int, int, hipStream_t);
  int (*add_rmsnorm)(float*, const void*, int, int, long, const float*, void*, const int*, int, int,
                     float, int, int, int, hipStream_t);
  int (*swiglu)(const void*, void*, int, int, int, hipStream_t);
  int (*cast)(const void*, void*, long, int, int, hipStream_t);
  int (*gemm_f32)(const float*, const float*, const float*, float*, int, int, int, int, int,
                  hipStream_t);
  int (*gemm_bf16)(const void*, const void*, const void*, const float*, void*, int, int, int, int,
                   int, int, int, int, int, const float*, int, float, float*, int, const float*,
                   void*, int, float*, hipStream_t);
  int (*gemm_bf16_any)(const void*, const void*, const float*, void*, int, int, int, int, int, int,
                       hipStream_t);
  int (*gemm_bf16_swiglu)(const void*, const void*, const void*, void*, int, int, int, int, int,
                          int, int, const float*, int, float, int, hipStream_t);
  int (*gemm_bf16_shortconv_step)(const void*, const void*, const void*, const float*, void*, int,
                                  int, int, int, const float*, const float*, float*, const int*,
                                  const int*, int, int, const float*, int, float, int, hipStream_t);
  int (*shortconv)(const void*, const float*, const float*, float*, void*, const int*, const int*,
                   const int*, const int*, int, int, int, int, int, hipStream_t);
  int (*shortconv_parts)(const float*, int, const float*, const float*, float*, void*, const int*,
                         const int*, const int*, const int*, int, int, int, int, hipStream_t);
  int (*qk_norm_rope_store)(void*, int, const float*, const float*, float, const float*,
                            const float*, int, int, void*, void*, const int*, const int*,
                            const int*, int, int, int, int, int, int, int, int, const float*, int,
                            void*, int, hipStream_t);
  int (*paged_attention_rows)(const void*, int, const void*, const void*, void*, int, const int*,
                              const int*, const int*, int, int, int, int, int, int, int, float, int,
                              hipStream_t);
} kappai_kernels;

// the matrix-core attention kernels of one head size (null where no such library fits)
typedef struct kappai_attention_kernels {
  int (*keys_per_wave)(void);
  int (*decode_block_waves)(int);
  int (*attn_prefill)(const void*, int, const void*, const void*, void*, int, const int*, int,
                      const int*, const int*, int, int, int, int, int, float, int, hipStream_t);
  int (*attn_decode)(const void*, int, const void*, const void*, void*, int, float*, float*,
                     const int*, const int*, const int*, int, int, int, int, int, int, float, int,
                     int, hipStream_t);
  int (*attn_decode_block)(const void*, int, const void*, const void*, void*, int, const int*,
                           const int*, const int*, int, int, int, int, int, int, float, int,
                           hipStream_t);
  // the decode kernel that splits the keys over blocks, with the per-head norm, the rotation and
  // the store of the rows' own keys and values in its prologue (decode_takes_qk() says whether
  // this head size has it)
  // kappai_attn_decode for the rows that a list names
  int (*attn_decode_rows)(const void*, int, const void*, const void*, void*, int, float*, float*,
                          const int*, const int*, const int*, const int*, int, int, int, int, int,
                          int, float, int, int, hipStream_t);
  int (*decode_takes_qk)(void);
  int (*attn_decode_qk)(const void*, int, void*, void*, void*, int, float*, float*, const int*,
                        const int*, const int*, int, int, int, int, int, int, float, int, int,
                        const float*, const float*, float, const float*, const float*, int,
                        hipStream_t);
} kappai_attention_kernels;

// ---- the model --------------------------------------------------------------------------------
typedef struct kappai_linear {
  const void* w;        // [n, k], bfloat16 or float32; null when the matrix is kept in w_frag only
  const void* w_frag;   // the bfloat16 matrix in fragment order, or null
  const float* bias;    // [n] or null
  int n, k;
  int w_is_f32;
} kappai_linear;

typedef struct kappai_norm {
  const float* w;       // [width]
  float eps;
} kappai_norm;

enum { KAPPAI_MIXER_CONV = 0, KAPPAI_MIXER_ATTENTION = 1 };

// One call of the schedule: a pre-norm block and the cache it uses.
typedef struct kappai_layer_call {
  int mixer;                        // KAPPAI_MIXER_*
  kappai_norm mixer_norm, ffn_norm;
  // gated short convolution
  kappai_linear in_proj, out_proj;
  const float* taps;                // [width, taps_per_channel]
  const float* conv_bias;           // [width] or null
  int taps_per_channel;
  float* state;                     // [slots, width, taps_per_channel - 1]
  // grouped-query attention
  kappai_linear qkv;                // q, k, v rows stacked (q first)
  kappai_linear attn_out;
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
  // SwiGLU feed-forward
  kappai_linear gate_up;            // gate and up rows (interleaved in 16s when ffn_fused)
  kappai_linear down;
  int hidden;
  int ffn_fused;
} kappai_layer_call;

typedef struct kappai_model {
  int abi;                          // KAPPAI_ENGINE_ABI of the side that filled this in
  int compute_bf16;                 // activations and cache in bfloat16 (else float32)
  int width, vocab, page_size;
  const void* embed_table;          // [vocab, width]
  int embed_is_bf16;                // 0: float32 rows, 1: bfloat16 rows, 2: bfloat16 in fragment order
  int n_calls;
  const kappai_layer_call* calls;
  kappai_norm final_norm;
  kappai_linear head;
  const kappai_kernels* kernels;
  // the choices that the parts make by size (the same numbers the host's parts use)
  int fused_step_min_width, fused_step_narrow_width, fused_step_narrow_rows;
  int partial_sums_min_rows;        // projections hand on partial sums above this many rows
  int partial_sums_max_rows;        // and up to this many (more, when every segment is one row)
  int fragment_rows_min;            // the norm writes fragment order from this many rows on
  int fragment_rows_from;           // products write fragment order from this many rows on
  int fused_max_rows;               // rows up to which products fold residual sum and norm in
  int decode_waves, decode_max_splits, decode_block_max_keys;
  int attention_tile_rows;
  int fused_qk;                     // rows up to which decode attention does norm, rotation and
                                    // store itself (0: never)
} kappai_model;

// ---- the rows of a step -------------------------------------------------------------------------
typedef struct kappai_batch {
  int n_rows, n_segments, n_logit_rows, max_position, max_segment_rows;
  int logits_of_every_row;          // logit_rows is 0, 1, ..., n_rows - 1
  const int* tokens;                // [n_rows]
  const int* row_pos;               // [n_rows]
  const int* row_seg;               // [n_rows]
  const int* seg_start;             // [n_segments + 1]
  const int* seg_pos0;              // [n_segments]
  const int* seg_slot;              // [n_segments]
  const int* logit_rows;            // [n_logit_rows]
  const int* q_tiles;               // [n_tiles, 4] or null
  int n_tiles;
  const int* lone_rows;             // [n_lone_rows] or null: single decoded tokens beside prompt
  int n_lone_rows;                  // portions that q_tiles leaves out
  int max_lone_position;
  int n_groups;
  const int* block_tables[KAPPAI_MAX_GROUPS];   // [n_segments, max_blocks[g]]
  int max_blocks[KAPPAI_MAX_GROUPS];
} kappai_batch;

// The sizes of the structs above as this library sees them (abi, kernels, attention kernels,
// linear, norm, layer call, model, batch), for the host to check its own layout against.
int kappai_engine_layout(int* sizes, int n);

// Bytes of workspace that kappai_forward needs for this batch (it depends on the batch's sizes
// only, not on its tables), or 0 when the model or the batch is one it refuses.
size_t kappai_forward_workspace_bytes(const kappai_model* model, const kappai_batch* batch);

// Runs the step: embedding, every layer call, final norm and head for the rows that want logits.
// `logits` receives float [n_logit_rows, vocab].  Every kernel goes to `stream`; nothing waits.
// Returns 0, a hipError_t of a launch, or hipErrorInvalidValue with a message that
// kappai_forward_error() returns.
int kappai_forward(const kappai_model* model, const kappai_batch* batch, void* workspace,
                   size_t workspace_bytes, float* logits, hipStream_t stream);

const char* kappai_forward_error(void);

// How many K ranges a product of these sizes is cut into when its consumer adds partial sums (the
// host's parts ask the same function).
int kappai_split_k_for(int M, int N, int K);

#ifdef __cplusplus
}
#endif

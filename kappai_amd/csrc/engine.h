// The C side of a step: one call that launches every kernel of a forward pass.
//
// kappai's entry points are C (engine_init / engine_run / engine_shutdown, src/engine.h:12-17;
// one forward call compute_forward_rows over a row description, src/compute.h:120-149,
// src/recipe/exec.c:704-758), and its executor runs a list of operations through a table of
// handlers that each operation registered itself in (RECIPE_REGISTER, src/recipe.h:577-580;
// src/recipe/exec.c:467-517).  Here the host that owns requests, cache bookkeeping and scheduling
// is Python; what it hands down for a step is what this header describes: the model as a flat list
// of calls (kappai_model), the rows of the step with their tables (kappai_batch), a workspace, and
// the place for the logits.  kappai_forward then runs the whole step on the given stream without
// returning to the host in between.
//
// The walk knows no part by name.  A call of the schedule is a block: a function and a
// description that only that function reads.  A block is put together from norms, a mixer and a
// feed-forward, each again a function and its description.  The functions ("runners") are
// registered under names (kappai_register_runner); the host asks for them by name when it
// builds the model's description, so a part that the framework has never heard of runs from C
// once its library has registered a runner for it and its host class hands out a description.
// A runner sees the step only through kappai_step_api: memory from the step's workspace, the
// batch's tables, the stream, the products (kappai_step_api::linear) and what travels between
// parts (kappai_rows, kappai_carry).
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define KAPPAI_ENGINE_ABI 11         // bumped with every change of the structs below
#define KAPPAI_MAX_GROUPS 8          // paged groups a batch can carry block tables for
#define KAPPAI_MAX_TABLES 8         // tables and numbers of the parts' own in a step

// ---- the kernels' launchers, by address (they live in libraries of their own) ---------------
typedef struct kappai_kernels {
  int (*embed_rows)(const int*, const void*, int, float*, int, int, hipStream_t);
  int (*embed_rmsnorm)(const int*, const void*, int, float*, const float*, void*, int, int, float,
                       int, int, hipStream_t);
  int (*add_rmsnorm)(float*, const void*, int, int, long, const float*, void*, const int*, int, int,
                     float, int, int, int, hipStream_t);
  int (*swiglu)(const void*, void*, int, int, int, hipStream_t);
  int (*cast)(const void*, void*, long, int, int, hipStream_t);
  int (*sum_partials)(const float*, int, long, float*, hipStream_t);
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
  // kappai_attn_decode for the rows that a list names
  int (*attn_decode_rows)(const void*, int, const void*, const void*, void*, int, float*, float*,
                          const int*, const int*, const int*, const int*, int, int, int, int, int,
                          int, float, int, int, hipStream_t);
  // the decode kernel that splits the keys over blocks, with the per-head norm, the rotation and
  // the store of the rows' own keys and values in its prologue (decode_takes_qk() says whether
  // this head size has it)
  int (*decode_takes_qk)(void);
  int (*attn_decode_qk)(const void*, int, void*, void*, void*, int, float*, float*, const int*,
                        const int*, const int*, int, int, int, int, int, int, float, int, int,
                        const float*, const float*, float, const float*, const float*, int,
                        hipStream_t);
} kappai_attention_kernels;

// ---- what parts are made of and what travels between them -------------------------------------
typedef struct kappai_linear {
  const void* w;        // [n, k], bfloat16 or float32; null when the matrix is kept in w_frag only
  const void* w_frag;   // the bfloat16 matrix in fragment order, or null
  const float* bias;    // [n] or null
  int n, k;
  int w_is_f32;
} kappai_linear;

// y = x * w / sqrt(mean(x^2) + eps): what a product needs to know of a norm to fold it in (it
// hands on x * w and the sums of squares, and the product after the norm divides)
typedef struct kappai_fold {
  const float* w;       // [width]
  float eps;
} kappai_fold;

// Rows on their way into a product: plain [M, D] with a row stride, 16 row slots in fragment
// order, or either of the two still to be divided by the rows' root mean square (ss != null).
typedef struct kappai_rows {
  void* data;
  int is_bf16;
  int M, D, ld;
  int frag;
  const float* ss;                 // scaled rows: [ss_parts][16] sums of squares
  int ss_parts;
  float eps;
  const kappai_fold* norm;         // the norm the scaled rows were made for
} kappai_rows;

// What a part hands to the norm after it.
enum {
  KAPPAI_CARRY_NOTHING = 0,        // the sum is in the residual stream already
  KAPPAI_CARRY_DELTA = 1,          // data [M, D] in the compute dtype or float32
  KAPPAI_CARRY_PARTS = 2,          // data [parts][M][D] float: sums over ranges of K
  KAPPAI_CARRY_SCALED = 3,         // the sum is in the stream, and `scaled` holds the next rows
  KAPPAI_CARRY_EMBEDDING = 4       // the residual stream is not filled yet: the embedding's rows
};                                 // are still to be looked up (the first norm may do both)
typedef struct kappai_carry {
  int kind;
  void* data;
  int is_f32;
  int parts;
  kappai_rows scaled;
} kappai_carry;

// Where a part's last product may add its result, and the norm it may fold in (or null).
typedef struct kappai_into {
  float* resid;
  const kappai_fold* norm;
} kappai_into;

// The regions of the step's workspace: what lives for the whole step, what a part hands to the
// next norm (kappai_step_api::carry_region names the one to use), and what a block needs only
// while it runs (given back when the next call of the schedule starts).
enum { KAPPAI_REGION_STEP = 0, KAPPAI_REGION_BLOCK = 3 };

struct kappai_model;
struct kappai_batch;
struct kappai_part;
typedef struct kappai_step kappai_step;

// What a runner may ask of the step.  Every function takes the step it was given.
typedef struct kappai_step_api {
  const struct kappai_model* (*model)(kappai_step*);
  const struct kappai_batch* (*batch)(kappai_step*);
  hipStream_t (*stream)(kappai_step*);
  // 1 while the walk only measures the workspace: take() as usual, launch nothing
  int (*dry)(kappai_step*);
  // 0 once a launch has failed or the workspace has run out: a runner may return early
  int (*ok)(kappai_step*);
  // bytes from a region of the workspace (256-byte aligned; never null while ok())
  void* (*take)(kappai_step*, int region, size_t bytes);
  // the region for what this part hands on to the next norm; to be asked once per part run
  int (*carry_region)(kappai_step*);
  // the status a kernel's launcher returned (0 or a hipError_t)
  void (*launched)(kappai_step*, int status);
  // refuses the step with a message that kappai_forward_error() returns
  void (*fail)(kappai_step*, const char* message);
  // y = x W^T (+ bias).  out_bf16: the dtype of a plain result.  partial_sums: the result may come
  // as float planes over ranges of K (the caller hands it to a norm or a kernel that adds them).
  // into: the product may add its result into the residual stream (up to 16 bfloat16 rows), and
  // fold into->norm in; null: never.  region: where a result that outlives the block goes.
  kappai_carry (*linear)(kappai_step*, kappai_rows x, const kappai_linear* lin, int out_bf16,
                         int partial_sums, const kappai_into* into, int region);
  // rows any kernel can read: scaled rows or rows in fragment order are made anew by the norm
  // they were made for, from the residual stream
  kappai_rows (*plain_rows)(kappai_step*, kappai_rows x, float* resid);
  // a carry as a norm takes it that knows nothing of the framework's shortcuts: the embedding
  // looked up, partial sums added up (KAPPAI_CARRY_DELTA, float), scaled rows dropped (NOTHING)
  kappai_carry (*plain_carry)(kappai_step*, kappai_carry carry, float* resid, int M);
  // n elements to the other of the two dtypes, in the block's region
  void* (*cast)(kappai_step*, const void* x, size_t n, int from_bf16, int to_bf16);
  // whether the products for 1 to 16 rows read this matrix from rows of width D in kernel
  // order (fragment order, scaled rows)
  int (*takes_kernel_order)(const kappai_linear* lin, int D);
  // the RMSNorm kernel: adds `carry` (nothing, a delta or partial sums) into the residual stream
  // and writes the normalised rows, in fragment order if asked (up to 16 bfloat16 rows);
  // rows != null: only these n_rows rows, and the stream is left alone
  kappai_rows (*rms_norm)(kappai_step*, const kappai_fold* norm, float* resid, kappai_carry carry,
                          int M, const int* rows, int n_rows, int fragment);
} kappai_step_api;

struct kappai_step {
  const kappai_step_api* api;      // the rest of the step is the walk's own
};

// ---- parts, norms, blocks: a function and the description it reads ----------------------------
enum { KAPPAI_TAKES_DEFERRED_ROWS = 1,   // x may arrive scaled or in fragment order
       KAPPAI_ADDS_RESIDUAL = 2 };       // the part takes `into` for its last product

// A mixer or a feed-forward: the normalised rows in, what it hands to the next norm out.
typedef kappai_carry (*kappai_part_fn)(kappai_step*, const void* desc, kappai_rows x, float* resid,
                                       const kappai_into* into);
typedef struct kappai_part {
  kappai_part_fn run;
  const void* desc;
  int flags;
  const kappai_linear* first;      // the product that takes the part's input rows, if it is a
} kappai_part;                     // product that takes them (else null)

// A norm: adds what the part before it handed on into the residual stream and returns the
// normalised rows for `consumer`.  rows != null: only these n_rows rows, the stream is left alone.
typedef kappai_rows (*kappai_norm_fn)(kappai_step*, const void* desc, float* resid,
                                      kappai_carry carry, int M, const int* rows, int n_rows,
                                      const kappai_part* consumer);
typedef struct kappai_norm_part {
  kappai_norm_fn run;
  const void* desc;
  const kappai_fold* fold;         // set when a product can fold this norm in, else null
} kappai_norm_part;

// A call of the schedule: an arrangement of parts around the residual stream.  `carry`: what the
// call before handed on.  after_norm / after_consumer: the first norm of what runs next and the
// part that takes its rows (the final norm and the head after the last call when every row wants
// its logits; null when nothing can be folded).  Returns what it hands on.
typedef kappai_carry (*kappai_block_fn)(kappai_step*, const void* desc, float* resid,
                                        kappai_carry carry, const kappai_norm_part* after_norm,
                                        const kappai_part* after_consumer);
typedef struct kappai_call {
  kappai_block_fn run;
  const void* desc;
  const kappai_norm_part* first_norm;     // what a block before this one may fold in (or null)
  const kappai_part* first_consumer;
} kappai_call;

// The numbers by which parts choose between forms of a kernel (the host's parts use the same).
typedef struct kappai_tuning {
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
} kappai_tuning;

// What may change the embedded rows before the first call of the schedule (an encoding of
// positions that is added to them): resid holds the step's M rows, looked up already.
typedef void (*kappai_embedded_fn)(kappai_step*, const void* desc, float* resid, int M);
typedef struct kappai_embedded_part {
  kappai_embedded_fn run;          // null: nothing does
  const void* desc;
} kappai_embedded_part;

typedef struct kappai_model {
  int abi;                          // KAPPAI_ENGINE_ABI of the side that filled this in
  int compute_bf16;                 // activations and cache in bfloat16 (else float32)
  int width, vocab, page_size;
  const void* embed_table;          // [vocab, width]
  int embed_is_bf16;                // 0: float32 rows, 1: bfloat16 rows, 2: bfloat16 in fragment order
  int n_calls;
  const kappai_call* calls;
  kappai_norm_part final_norm;
  kappai_linear head;
  const kappai_kernels* kernels;
  kappai_tuning tuning;
  kappai_embedded_part on_embedding;
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
  // What the parts' own layouts made for this step (parts.base.StepTables): tables on the GPU
  // and numbers, by the places the plan gave their names (CPlan.table / CPlan.number).  A table
  // that was not laid out in this step is null with 0 rows, such a number is -1.
  const int* tables[KAPPAI_MAX_TABLES];
  int table_rows[KAPPAI_MAX_TABLES];        // the table's first dimension
  int numbers[KAPPAI_MAX_TABLES];
  int n_groups;
  const int* block_tables[KAPPAI_MAX_GROUPS];   // [n_segments, max_blocks[g]]
  int max_blocks[KAPPAI_MAX_GROUPS];
} kappai_batch;

// ---- the registry of runners ----------------------------------------------------------------
enum { KAPPAI_RUNNER_PART = 0, KAPPAI_RUNNER_NORM = 1, KAPPAI_RUNNER_BLOCK = 2,
       KAPPAI_RUNNER_EMBEDDED = 3 };

// Registers `fn` (a kappai_part_fn, kappai_norm_fn, kappai_block_fn or kappai_embedded_fn, as
// `kind` says) under
// `name`; desc_bytes is the size of the description it reads, which the host checks its own
// layout against.  A name can be registered again with the same function only.  Returns 0, or
// hipErrorInvalidValue (the message through kappai_forward_error).
int kappai_register_runner(const char* name, int kind, void* fn, int desc_bytes);
// The function registered under `name` with this kind, or null; desc_bytes receives the size.
void* kappai_runner(const char* name, int kind, int* desc_bytes);

// ---- entry points -------------------------------------------------------------------------------
// The sizes of the structs above as this library sees them, for the host to check its own layout
// against (the order is that of kappai_engine_layout's definition).
int kappai_engine_layout(int* sizes, int n);

// Bytes of workspace that kappai_forward needs for this batch (it depends on the batch's sizes
// only, not on its tables), or 0 when the model or the batch is one it refuses.
size_t kappai_forward_workspace_bytes(const kappai_model* model, const kappai_batch* batch);

// Runs the step: embedding, every call of the schedule, final norm and head for the rows that
// want logits.  `logits` receives float [n_logit_rows, vocab].  Every kernel goes to `stream`;
// nothing waits.  Returns 0, a hipError_t of a launch, or hipErrorInvalidValue with a message that
// kappai_forward_error() returns.
int kappai_forward(const kappai_model* model, const kappai_batch* batch, void* workspace,
                   size_t workspace_bytes, float* logits, hipStream_t stream);

const char* kappai_forward_error(void);

// How many K ranges a product of these sizes is cut into when its consumer adds partial sums (the
// host's parts ask the same function).
int kappai_split_k_for(int M, int N, int K);

// How the decode attention that splits a row's keys over blocks cuts n_keys keys of `rows` rows
// over G kv heads: the fewest keys a split and the most splits a row (the host asks the same
// function).  keys_per_wave: what a wave of the kernel keeps in flight.
void kappai_decode_splits(int keys_per_wave, int max_splits, int waves, int rows, int G,
                          int n_keys, int* keys_per_split, int* n_splits);

#ifdef __cplusplus
}
#endif

// The engine behind a C API.
//
// kappai's own entry points are C: engine_init / engine_init_config / engine_run /
// engine_shutdown (src/engine.h:12-17) over a session that prefills and decodes
// (src/context.h:100-137), and one forward call over a row description (src/compute.h:120-149).
// Here requests, scheduling and cache bookkeeping are Python (kappai_amd.engine.Engine); this
// library is a shell over them for callers written in C: it holds an interpreter (its own when
// the process has none, else the process's), and every function below is one call into the
// engine.  Token ids in, token ids out; nothing here tokenizes text.
//
// All functions are safe to call from any thread, one at a time per engine.  A function that
// fails returns a negative number (or null) and kappai_engine_error() says why.
#pragma once
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct kappai_engine kappai_engine;

// Options with kappai's meanings where it has them (src/config.c:48-61, 84-154): 0 or null
// leaves an option at the engine's default.
typedef struct kappai_engine_config {
  const char* model;        // -m: folder with config.json and model.safetensors (required)
  const char* dtype;        // "bfloat16" (default) or "float32"
  int device;               // index of the GPU
  int ctx_size;             // -c: longest sequence; 0: the model's
  int page_size;            // tokens a cache page
  int num_pages;            // cache pages; 0: from free memory
  int max_batch;            // requests live at a time
  int token_budget;         // most tokens a step
  int chunk;                // longest prompt portion
  int decode_graphs;        // 0: default (on), 1: on, -1: off
} kappai_engine_config;

// Generation options with kappai's names, meanings and defaults (src/config.c:156-172).
typedef struct kappai_sampling {
  float temperature;        // -t: <= 0 is greedy
  int top_k;                // -k: 0 disabled, 1 greedy
  float top_p;              // -P: 1 disabled
  float min_p;              // -M: 0 disabled
  float repeat_penalty;     // 1 disabled
  int repeat_last_n;
  uint64_t seed;            // -s: 0 = from the operating system
  int n_predict;            // -n: most tokens to generate; -1: until the context ends
} kappai_sampling;

// What a step reports for a request: the token it got (-1: none), whether it ended, and why
// (0 not ended, 1 end-of-sequence token, 2 n_predict reached, 3 context full, 4 failed,
// 5 aborted, 6 shutdown).
typedef struct kappai_step_output {
  int request_id;
  int token;
  int finished;
  int reason;
} kappai_step_output;

// One request's part of a raw step: its next tokens and the places among them whose logits are
// wanted.  A request id that the engine has not seen opens a request of the raw step function
// (these ids are apart from those that kappai_engine_add_request returns).
typedef struct kappai_forward_entry {
  int request_id;
  const int* tokens;
  int n_tokens;
  const int* want;
  int n_want;
} kappai_forward_entry;

typedef struct kappai_engine_stats {
  double steps, prompt_tokens, prompt_seconds, decoded_tokens, decode_seconds, first_token_ms,
         graph_replays, preemptions, free_pages, vocab_size, ctx_size;
} kappai_engine_stats;

void kappai_engine_config_default(kappai_engine_config* config);
void kappai_sampling_default(kappai_sampling* sampling);      // kappai's defaults
void kappai_sampling_greedy(kappai_sampling* sampling, int n_predict);

// kappai: engine_init_config.  Loads the model, sizes the cache, warms the kernels.
kappai_engine* kappai_engine_create(const kappai_engine_config* config);
// kappai: engine_shutdown.
void kappai_engine_destroy(kappai_engine* engine);

// Queues a prompt; returns its request id (>= 0).
int kappai_engine_add_request(kappai_engine* engine, const int* token_ids, int n_tokens,
                              const kappai_sampling* sampling);
int kappai_engine_abort(kappai_engine* engine, int request_id);       // 1: stopped, 0: had ended
int kappai_engine_has_work(kappai_engine* engine);                    // 1 while requests are live
// One step of the engine (schedule, run the model, sample): up to `capacity` outputs are written,
// the rest is kept for the next call.  Returns how many were written.
int kappai_engine_step(kappai_engine* engine, kappai_step_output* outputs, int capacity);
// The tokens a request has generated so far: up to `capacity` are written, the total is returned.
int kappai_engine_output(kappai_engine* engine, int request_id, int* tokens, int capacity);
int kappai_engine_release(kappai_engine* engine, int request_id);     // forget an ended request

// kappai: engine_run.  One prompt to its end (blocking); returns the number of tokens generated,
// of which up to `capacity` are written.
int kappai_engine_generate(kappai_engine* engine, const int* token_ids, int n_tokens,
                           const kappai_sampling* sampling, int* tokens, int capacity);

// The raw step function (kappai: compute_forward_rows): runs the entries' tokens as one batch
// from the cache that earlier calls left and writes float32 logits [wanted, vocab] in the order
// of the entries and of their `want`.  Returns the number of wanted rows.
int kappai_engine_forward(kappai_engine* engine, const kappai_forward_entry* entries,
                          int n_entries, float* logits, size_t capacity_floats);
int kappai_engine_end(kappai_engine* engine, int request_id);         // a raw request is finished

int kappai_engine_get_stats(kappai_engine* engine, kappai_engine_stats* stats);

// The message of this thread's last failed call ("" if none).
const char* kappai_engine_error(void);

#ifdef __cplusplus
}
#endif

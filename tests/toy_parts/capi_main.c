/* A caller of the engine's C API that is no Python program: it loads the library, creates an
 * engine for a model folder, runs two prompts side by side step by step, one more through the
 * blocking call, one raw step, and prints what it got as lines of numbers for the test to compare
 * with the Python engine.
 *
 *   capi_main <engine_api.so> <model folder> <dtype> <n_predict>
 */
#include <dlfcn.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "engine_api.h"

#define LOAD(name)                                             \
  __typeof__(&name) p_##name = (__typeof__(&name))dlsym(lib, #name); \
  if (p_##name == NULL) {                                      \
    fprintf(stderr, "no symbol %s\n", #name);                  \
    return 2;                                                  \
  }

int main(int argc, char** argv) {
  if (argc < 5) {
    fprintf(stderr, "usage: capi_main <engine_api.so> <model> <dtype> <n_predict>\n");
    return 2;
  }
  void* lib = dlopen(argv[1], RTLD_NOW | RTLD_GLOBAL);
  if (lib == NULL) {
    fprintf(stderr, "dlopen: %s\n", dlerror());
    return 2;
  }
  LOAD(kappai_engine_config_default)
  LOAD(kappai_sampling_greedy)
  LOAD(kappai_engine_create)
  LOAD(kappai_engine_destroy)
  LOAD(kappai_engine_add_request)
  LOAD(kappai_engine_has_work)
  LOAD(kappai_engine_step)
  LOAD(kappai_engine_output)
  LOAD(kappai_engine_generate)
  LOAD(kappai_engine_forward)
  LOAD(kappai_engine_end)
  LOAD(kappai_engine_get_stats)
  LOAD(kappai_engine_error)
  const int n_predict = atoi(argv[4]);

  /* before any engine exists (and before this process has an interpreter) a call is refused */
  if (p_kappai_engine_has_work(NULL) != -1 || strstr(p_kappai_engine_error(), "no engine") == NULL) {
    fprintf(stderr, "a call without an engine was not refused\n");
    return 1;
  }

  kappai_engine_config config;
  p_kappai_engine_config_default(&config);
  config.model = argv[2];
  config.dtype = argv[3];
  config.num_pages = 64;
  config.max_batch = 4;
  kappai_engine* engine = p_kappai_engine_create(&config);
  if (engine == NULL) {
    fprintf(stderr, "create: %s\n", p_kappai_engine_error());
    return 1;
  }
  kappai_sampling greedy;
  p_kappai_sampling_greedy(&greedy, n_predict);

  /* two prompts side by side, step by step */
  const int a[] = {3, 200, 17, 17, 0, 255, 9};
  const int b[] = {41, 41, 100, 7, 8, 9, 250, 1, 2, 3, 4, 5};
  const int ra = p_kappai_engine_add_request(engine, a, 7, &greedy);
  const int rb = p_kappai_engine_add_request(engine, b, 12, &greedy);
  if (ra < 0 || rb < 0) {
    fprintf(stderr, "add_request: %s\n", p_kappai_engine_error());
    return 1;
  }
  int ended = 0, reported = 0;
  while (p_kappai_engine_has_work(engine) == 1) {
    kappai_step_output out[8];
    const int n = p_kappai_engine_step(engine, out, 8);
    if (n < 0) {
      fprintf(stderr, "step: %s\n", p_kappai_engine_error());
      return 1;
    }
    for (int i = 0; i < n; ++i) {
      reported += out[i].token >= 0;
      ended += out[i].finished;
    }
  }
  int tokens[64];
  const int ids[2] = {ra, rb};
  for (int r = 0; r < 2; ++r) {
    const int n = p_kappai_engine_output(engine, ids[r], tokens, 64);
    printf("request %d:", r);
    for (int i = 0; i < n && i < 64; ++i) printf(" %d", tokens[i]);
    printf("\n");
  }
  printf("reported %d ended %d\n", reported, ended);

  /* the blocking call */
  const int n = p_kappai_engine_generate(engine, a, 7, &greedy, tokens, 64);
  if (n < 0) {
    fprintf(stderr, "generate: %s\n", p_kappai_engine_error());
    return 1;
  }
  printf("generate:");
  for (int i = 0; i < n && i < 64; ++i) printf(" %d", tokens[i]);
  printf("\n");

  /* the raw step function: the first five tokens of b, then two more beside a new request */
  kappai_engine_stats stats;
  if (p_kappai_engine_get_stats(engine, &stats) != 0) return 1;
  const int vocab = (int)stats.vocab_size;
  float* logits = (float*)malloc(sizeof(float) * 3 * vocab);
  const int want_last[] = {4};
  kappai_forward_entry first = {7, b, 5, want_last, 1};
  int rows = p_kappai_engine_forward(engine, &first, 1, logits, (size_t)3 * vocab);
  if (rows != 1) {
    fprintf(stderr, "forward: %s\n", p_kappai_engine_error());
    return 1;
  }
  int best = 0;
  for (int v = 1; v < vocab; ++v)
    if (logits[v] > logits[best]) best = v;
  printf("forward argmax %d\n", best);
  const int want_both[] = {0, 1}, want_one[] = {2};
  kappai_forward_entry second[2] = {{7, b + 5, 2, want_both, 2}, {8, a, 3, want_one, 1}};
  rows = p_kappai_engine_forward(engine, second, 2, logits, (size_t)3 * vocab);
  if (rows != 3) {
    fprintf(stderr, "forward (2): %s\n", p_kappai_engine_error());
    return 1;
  }
  for (int r = 0; r < 3; ++r) {
    best = 0;
    for (int v = 1; v < vocab; ++v)
      if (logits[r * vocab + v] > logits[r * vocab + best]) best = v;
    printf("forward row %d argmax %d\n", r, best);
  }
  /* a refused call says why */
  rows = p_kappai_engine_forward(engine, second, 2, logits, 10);
  printf("refused %d: %s\n", rows, p_kappai_engine_error());
  p_kappai_engine_end(engine, 7);
  p_kappai_engine_end(engine, 8);
  p_kappai_engine_get_stats(engine, &stats);
  printf("stats steps %.0f decoded %.0f vocab %.0f\n", stats.steps, stats.decoded_tokens,
         stats.vocab_size);
  free(logits);
  p_kappai_engine_destroy(engine);
  return 0;
}

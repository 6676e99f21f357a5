/* A host program in C against the engine's C interface (csrc/engine_api/ninfer_c_api.h), as a
   program written for the reference's C API would use it: load, a session, prefill, then
   greedy decoding through ninfer_sample; a second session decoded beside the first through
   ninfer_decode_batch. Prints the generated ids, one line per request.
   usage: c_api_host MODEL_DIR N_NEW TOKEN [TOKEN ...] */
#include <stdio.h>
#include <stdlib.h>

#include "ninfer_c_api.h"

static void die(const char* what) {
  fprintf(stderr, "%s: %s\n", what, ninfer_last_error());
  exit(1);
}

int main(int argc, char** argv) {
  if (argc < 4) return 2;
  const int n_new = atoi(argv[2]), n_prompt = argc - 3;
  long long* prompt = malloc(sizeof(long long) * n_prompt);
  for (int i = 0; i < n_prompt; ++i) prompt[i] = atoll(argv[3 + i]);

  ninfer_options_t opt = {128, 8, 2, 0, NULL, "f32", NULL};
  ninfer_engine_t* eng = NULL;
  if (ninfer_load(argv[1], &opt, &eng) != 0) die("ninfer_load");
  const int vocab = ninfer_vocab_size(eng);
  if (vocab <= 0 || ninfer_max_context(eng) != 128 || ninfer_num_sequences(eng) != 2 ||
      ninfer_device_count(eng) != 1)
    die("engine figures");
  float* logits = malloc(sizeof(float) * 2 * vocab);

  /* request a alone: prefill, then token by token */
  ninfer_session_t* a = ninfer_session_create(eng);
  if (!a) die("ninfer_session_create");
  if (ninfer_prefill(a, prompt, n_prompt, logits, vocab) != 0) die("ninfer_prefill");
  printf("a:");
  long long tok_a[64];
  for (int i = 0; i < n_new; ++i) {
    tok_a[i] = ninfer_sample(eng, logits, 0.f, 0, 1.f, 1.f, 0);
    if (tok_a[i] < 0) die("ninfer_sample");
    printf(" %lld", tok_a[i]);
    if (ninfer_decode(a, tok_a[i], logits, vocab) != 0) die("ninfer_decode");
  }
  printf("\n");
  if (ninfer_session_length(a) != n_prompt + n_new) die("session length");

  /* the same request again in a new session beside a second one, decoded as a batch: the
     same tokens must come out for it */
  ninfer_session_reset(a);
  ninfer_session_t* b = ninfer_session_create(eng);
  if (!b) die("second session");
  if (ninfer_session_create(eng) != NULL) die("a third session where two are allowed");
  if (ninfer_prefill(b, prompt + 1, n_prompt - 1, logits + vocab, vocab) != 0) die("prefill b");
  if (ninfer_prefill(a, prompt, n_prompt, logits, vocab) != 0) die("prefill a");
  ninfer_session_t* both[2] = {a, b};
  printf("batch:");
  for (int i = 0; i < n_new; ++i) {
    long long t[2];
    t[0] = ninfer_sample(eng, logits, 0.f, 0, 1.f, 1.f, 0);
    t[1] = ninfer_sample(eng, logits + vocab, 0.f, 0, 1.f, 1.f, 0);
    printf(" %lld", t[0]);
    if (ninfer_decode_batch(eng, both, t, 2, logits, 2 * vocab) != 0) die("ninfer_decode_batch");
  }
  printf("\n");
  if (ninfer_decode_batch(eng, both, tok_a, 2, logits, vocab) != -3) die("a short buffer must give -3");

  const long long total = ninfer_kv_pages_total(eng);
  if (total <= 0 || ninfer_kv_pages_free(eng) >= total) die("pages in use");
  ninfer_session_free(a);
  ninfer_session_free(b);
  if (ninfer_kv_pages_free(eng) != total) die("pages given back");
  printf("pages: %lld\n", total);

  /* the engine's own scheduler: the same request and a second one, step by step */
  const long long ra = ninfer_request_add(eng, prompt, n_prompt, n_new, 0.f, 0, 1.f, 1.f, 0, NULL, 0);
  const long long rb = ninfer_request_add(eng, prompt + 2, n_prompt - 2, n_new, 0.f, 0, 1.f, 1.f, 0, NULL, 0);
  if (ra < 0 || rb < 0 || ra == rb) die("ninfer_request_add");
  long long out[64];
  if (ninfer_request_take(eng, ra, out, 64) != -4) die("a request that has not run yet is not finished");
  int left, steps = 0;
  while ((left = ninfer_run_step(eng)) > 0) ++steps;
  if (left < 0) die("ninfer_run_step");
  const int got = ninfer_request_take(eng, ra, out, 64);
  if (got != n_new) die("ninfer_request_take");
  printf("scheduled:");
  for (int i = 0; i < got; ++i) printf(" %lld", out[i]);
  printf("\n");
  if (ninfer_request_take(eng, ra, out, 64) != -1) die("a request is taken once");
  if (ninfer_request_take(eng, rb, out, 64) != n_new) die("the second request");
  if (ninfer_kv_pages_free(eng) != total || steps < n_new) die("after the scheduler");
  ninfer_engine_free(eng);
  return 0;
}

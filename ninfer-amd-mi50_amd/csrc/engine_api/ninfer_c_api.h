// The engine's C interface (extern "C"): loading, sessions, prefill / decode / batched
// decode, cache figures and sampling, with the names, argument lists and return codes of the
// reference's C API (src/api/ninfer_c_api.h:17-82), so that a host program written against
// that header links against this library instead.
//
// The engine itself is the Python package beside this folder; this library starts a Python
// interpreter inside the calling process at the first ninfer_load (or joins the one that is
// already running, when the caller is itself a Python process that loaded it through ctypes)
// and hands every call to ninfer_amd.api.c_bridge. Calls may come from any thread; they take
// the interpreter's lock and run one at a time.
//
// What differs from the reference, by what this engine is:
//   * one GPU: gpu_count must be 0 or 1, parallel null or "pp";
//   * quant: null, "fp16" or "bf16" all mean the engine's bfloat16 (there is no fp16 path),
//     "f32" the true 32-bit path; "q4" is refused;
//   * no tokenizer: ninfer_tokenize / ninfer_detokenize return -1;
//   * the cache is paged: ninfer_kv_seq_stride_elems returns 0 (there is no per-sequence
//     slab), and ninfer_kv_pages_total / _free / _reused report the pages instead;
//   * ninfer_last_error gives the text of the last failure of the calling thread's calls (the
//     reference logs it to stderr).
// Beyond the reference, for what it leaves to an outside scheduler: ninfer_step (one mixed
// batch: portions of prompts beside decoded tokens), the engine's own scheduler
// (ninfer_request_add, ninfer_run_step, ninfer_request_take) and ninfer_tensor_read (what the
// engine holds under a checkpoint name, for models whose weights were generated on the device).
#ifndef NINFER_AMD_C_API_H_
#define NINFER_AMD_C_API_H_

#ifdef __cplusplus
extern "C" {
#endif

typedef struct ninfer_engine ninfer_engine_t;
typedef struct ninfer_session ninfer_session_t;

typedef struct ninfer_options {
  int max_context;      // most tokens a request may hold (0: 32768)
  int prefill_chunk;    // rows of one prefill step (0: 512)
  int num_sequences;    // requests that may be live at a time (0: 1)
  int gpu_count;        // 0 or 1
  const int* gpus;      // ignored beyond the check of gpu_count
  const char* quant;    // see above
  const char* parallel; // see above
} ninfer_options_t;

// ---- engine ---------------------------------------------------------------------------
// 0 on success, negative on error (ninfer_last_error says what).
int ninfer_load(const char* model_dir, const ninfer_options_t* options, ninfer_engine_t** out_engine);
void ninfer_engine_free(ninfer_engine_t* engine);

int ninfer_vocab_size(ninfer_engine_t* engine);
int ninfer_max_context(ninfer_engine_t* engine);
int ninfer_num_sequences(ninfer_engine_t* engine);
int ninfer_device_count(ninfer_engine_t* engine);

long long ninfer_kv_bytes_per_token(ninfer_engine_t* engine);
long long ninfer_kv_total_bytes(ninfer_engine_t* engine);
long long ninfer_kv_seq_stride_elems(ninfer_engine_t* engine);
// Pages of all cache groups together; `reused`: pages handed out again after they came back.
long long ninfer_kv_pages_total(ninfer_engine_t* engine);
long long ninfer_kv_pages_free(ninfer_engine_t* engine);
long long ninfer_kv_pages_reused(ninfer_engine_t* engine);
// `count` numbers from flat index `offset` of the checkpoint tensor `name`, as the engine holds
// it now, as 32-bit floats. 0, or -1.
int ninfer_tensor_read(ninfer_engine_t* engine, const char* name, long long offset, long long count,
                       float* out);

int ninfer_tokenize(ninfer_engine_t* engine, const char* text, long long* out_ids, int capacity);
int ninfer_detokenize(ninfer_engine_t* engine, const long long* ids, int count, char* out_text,
                      int capacity);

// ---- sessions (one per live request) ------------------------------------------------------
ninfer_session_t* ninfer_session_create(ninfer_engine_t* engine);   // null when no slot is free
void ninfer_session_free(ninfer_session_t* session);                // gives the pages back
void ninfer_session_reset(ninfer_session_t* session);
int ninfer_session_slot(ninfer_session_t* session);
int ninfer_session_length(ninfer_session_t* session);

// Feeds `count` tokens in portions of prefill_chunk; the logits of the last one go to
// out_logits (capacity >= vocab_size floats). 0, or -1 (error), -3 (capacity too small).
int ninfer_prefill(ninfer_session_t* session, const long long* tokens, int count, float* out_logits,
                   int capacity);
int ninfer_decode(ninfer_session_t* session, long long token, float* out_logits, int capacity);
// One token for each of n sessions in one step; row i of out_logits (n * vocab_size floats)
// belongs to sessions[i].
int ninfer_decode_batch(ninfer_engine_t* engine, ninfer_session_t** sessions, const long long* tokens,
                        int n, float* out_logits, int capacity);

// One step for several sessions at once, each bringing its next q_len[i] tokens (a portion of
// its prompt, or one decoded token): `tokens` holds them one session after the other, T =
// sum of q_len; logit_rows[R] names the rows (0 .. T - 1, ascending) whose logits are wanted,
// which go to out_logits [R, vocab_size] in that order (R may be 0). 0, -1 or -3.
int ninfer_step(ninfer_engine_t* engine, ninfer_session_t** sessions, const int* q_len, int n_sessions,
                const long long* tokens, const int* logit_rows, int n_rows, float* out_logits,
                int capacity);

// ---- the engine's scheduler -----------------------------------------------------------------
// A request for up to max_new_tokens tokens after `prompt`; generation also ends at any of
// stop_ids (which is not part of the output). Returns the request's id (>= 0), or -1.
long long ninfer_request_add(ninfer_engine_t* engine, const long long* prompt, int count, int max_new_tokens,
                             float temperature, int top_k, float top_p, float repetition_penalty,
                             unsigned long long seed, const long long* stop_ids, int n_stop);
// One step of the scheduler (admission, portions under the token budget, decoding, sampling,
// finishing). Returns how many requests are still waiting or running, or -1.
int ninfer_run_step(ninfer_engine_t* engine);
// The output of a finished request: its tokens go to out_tokens, their number is returned and
// the request is forgotten. -4: not finished yet; -3: capacity too small (nothing is forgotten);
// -1: unknown id, or the request failed (ninfer_last_error says why; it is forgotten).
int ninfer_request_take(ninfer_engine_t* engine, long long id, long long* out_tokens, int capacity);

// ---- sampling ---------------------------------------------------------------------------
// The sampled token id, or negative on error. seed 0: a fresh seed.
long long ninfer_sample(ninfer_engine_t* engine, const float* logits, float temperature, int top_k,
                        float top_p, float repetition_penalty, unsigned long long seed);

const char* ninfer_last_error(void);

#ifdef __cplusplus
}  // extern "C"
#endif

#endif  // NINFER_AMD_C_API_H_

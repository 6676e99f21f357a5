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
//     slab), and ninfer_kv_pages reports the pages instead;
//   * ninfer_last_error gives the text of the last failure on the calling thread's engine
//     calls (the reference logs it to stderr).
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
// Pages of all cache groups together: total and free (either pointer may be null).
int ninfer_kv_pages(ninfer_engine_t* engine, long long* total, long long* free_pages);

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

// ---- sampling ---------------------------------------------------------------------------
// The sampled token id, or negative on error. seed 0: a fresh seed.
long long ninfer_sample(ninfer_engine_t* engine, const float* logits, float temperature, int top_k,
                        float top_p, float repetition_penalty, unsigned long long seed);

const char* ninfer_last_error(void);

#ifdef __cplusplus
}  // extern "C"
#endif

#endif  // NINFER_AMD_C_API_H_

// Arguments of paged attention. One struct serves the plain kernel and the
// MFMA kernels; the entry point picks by dtype, head size and batch shape.
#pragma once
#include "common.h"

namespace ninfer {

struct AttnArgs {
  const void* q;            // [T, q_stride] rows; head h of row t at q + t*q_stride + h*D
  const void* kpool;        // [pages, Hkv, page_size, D]
  const void* vpool;
  void* out;                // [T, Hq*D]
  const int* block_table;   // [S, bt_stride] page of each logical page, -1 when given back
  const int* positions;     // [T] absolute position of each row
  const int* row_seq;       // [T] request (index in this step) of each row
  const int* seq_row_start; // [S + 1] first row of each request, then T
  const int* seq_qlen;      // [S]
  const int* seq_pos0;      // [S]
  float* workspace;         // split-KV partial results, or null
  int64_t workspace_floats;
  int q_stride;
  int bt_stride;
  int T;
  int S;
  int Hq;
  int Hkv;
  int D;
  int page_size;
  int window;               // 0: all keys
  float scale;
  int dtype;
  int max_qlen;             // host-side bounds used to size launches
  int max_kv_len;
  int single_rows;          // the first single_rows requests bring one row each: rows
                            // 0 .. single_rows - 1 (0 when the caller does not sort them)
  const float* slopes;      // [Hq] or null: head h's scores get slopes[h] * (key position - row's
                            // position) added before the softmax (a distance-based position bias)
};

int attention_check(const AttnArgs& a);
int attention_generic(const void* q, int q_stride, const void* kpool, const void* vpool,
                      const int* block_table, int bt_stride, const int* positions,
                      const int* row_seq, void* out, int T, int Hq, int Hkv, int D, int page_size,
                      int window, float scale, const float* slopes, int dtype, hipStream_t stream);

int64_t attention_decode_workspace_floats(int T, int Hq, int D, int max_kv_len);
bool attention_decode_takes(const AttnArgs& a);
int attention_decode(const AttnArgs& a, hipStream_t stream);
void attention_decode_plan(const AttnArgs& a, bool* heads, int* chunk, int* n_chunks);
bool attention_decode_heads_takes(const AttnArgs& a);
int attention_decode_heads(const AttnArgs& a, int chunk, int n_chunks, hipStream_t stream);
bool attention_prefill_takes(const AttnArgs& a);
int attention_prefill(const AttnArgs& a, hipStream_t stream);

}  // namespace ninfer

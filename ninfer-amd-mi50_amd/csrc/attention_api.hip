// Entry point of paged attention: checks the arguments and picks a kernel.
#include "attention.h"

using namespace ninfer;

namespace ninfer {
// What every kernel of the family assumes of the arguments.
int attention_check(const AttnArgs& args) {
  const AttnArgs* a = &args;
  NINFER_REQUIRE(a->T > 0 && a->S > 0, "paged_attention: T=%d S=%d must be positive", a->T, a->S);
  NINFER_REQUIRE(a->Hq > 0 && a->Hkv > 0 && a->Hq % a->Hkv == 0,
                 "paged_attention: %d query heads are not a multiple of %d kv heads", a->Hq,
                 a->Hkv);
  NINFER_REQUIRE(a->D > 0 && a->D % 2 == 0, "paged_attention: head size %d must be even", a->D);
  NINFER_REQUIRE(a->page_size > 0 && a->bt_stride > 0, "paged_attention: bad page size %d or "
                 "table width %d", a->page_size, a->bt_stride);
  NINFER_REQUIRE(a->scale > 0.f, "paged_attention: scale %g must be positive", (double)a->scale);
  NINFER_REQUIRE(a->window >= 0, "paged_attention: window %d must be >= 0", a->window);
  NINFER_REQUIRE(a->dtype == kF32 || a->dtype == kBF16, "paged_attention: unknown dtype %d",
                 a->dtype);
  NINFER_REQUIRE(a->q_stride >= a->Hq * a->D, "paged_attention: row stride %d < %d", a->q_stride,
                 a->Hq * a->D);
  NINFER_REQUIRE(a->max_qlen >= 1 && a->max_kv_len >= 1, "paged_attention: bad size hints");
  NINFER_REQUIRE(a->single_rows >= 0 && a->single_rows <= a->S && a->single_rows <= a->T,
                 "paged_attention: %d single rows of %d requests", a->single_rows, a->S);
  return 0;
}
}  // namespace ninfer

// force_generic != 0 runs the plain one-wave-per-(row, head) kernel whatever
// the shape (tests compare the fast kernels with it).
extern "C" int ninfer_paged_attention(const AttnArgs* a, int force_generic, hipStream_t stream) {
  if (int rc = attention_check(*a)) return rc;
  if (!force_generic && a->max_qlen == 1 && attention_decode_takes(*a))
    return attention_decode(*a, stream);
  if (!force_generic && a->single_rows > 0 && a->single_rows < a->S &&
      attention_decode_takes(*a) && attention_prefill_takes(*a)) {
    // A step that mixes decoded tokens with prompt portions: the single rows, which come
    // first, walk their contexts split over many blocks; in the prompt kernel each would be
    // one block that walks its whole context alone.
    const int n = a->single_rows;
    AttnArgs d = *a;
    d.T = n;
    d.S = n;
    d.max_qlen = 1;
    if (int rc = attention_decode(d, stream)) return rc;
    AttnArgs p = *a;   // rows and their positions stay where they are: only the requests move
    p.seq_row_start += n;
    p.seq_qlen += n;
    p.seq_pos0 += n;
    p.block_table += (int64_t)n * a->bt_stride;
    p.S = a->S - n;
    p.T = a->T - n;
    return attention_prefill(p, stream);
  }
  if (!force_generic && attention_prefill_takes(*a)) return attention_prefill(*a, stream);
  return attention_generic(a->q, a->q_stride, a->kpool, a->vpool, a->block_table, a->bt_stride,
                           a->positions, a->row_seq, a->out, a->T, a->Hq, a->Hkv, a->D,
                           a->page_size, a->window, a->scale, a->slopes, a->dtype, stream);
}

// 32-bit floats of workspace the split-KV decode kernel needs for this shape.
extern "C" long long ninfer_attention_workspace_floats(int T, int Hq, int D, int max_kv_len) {
  return attention_decode_workspace_floats(T, Hq, D, max_kv_len);
}

// How a step of single-token rows would run (nothing is launched): kernel 0 = the plain
// kernel, 1 = split contexts on scalar FMAs, 2 = split contexts on the matrix cores (grouped
// heads); the keys per chunk and the number of chunks the merge kernel adds up. Tests name
// the kernel variant they mean to reach with it.
extern "C" int ninfer_attention_decode_plan(const AttnArgs* a, int* kernel, int* chunk, int* n_chunks) {
  *kernel = 0;
  *chunk = *n_chunks = 0;
  if (int rc = attention_check(*a)) return rc;
  if (!attention_decode_takes(*a)) return 0;
  bool heads;
  attention_decode_plan(*a, &heads, chunk, n_chunks);
  *kernel = heads ? 2 : 1;
  return 0;
}

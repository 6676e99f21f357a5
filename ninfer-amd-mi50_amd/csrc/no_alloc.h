// An entry point that allocates nothing.
//
// It has no counterpart in the reference. It is for callers that cannot
// allocate device memory: code under HIP graph capture, tight serving loops,
// harnesses that forbid hipMalloc. The existing ninfer_paged_attention needs a
// workspace from its caller for decode steps (the partial results of the
// chunks a context is cut into); the entry point here runs the same kernels on
// the same arguments with that workspace in a fixed array of device memory
// inside the library.
//
// Limits and rules:
//  - single-token rows only (max_qlen == 1), bf16, the shapes the split-context
//    kernels take (head sizes 16, 32, 64, 128, 256, a page size that is a power
//    of two); anything else is refused with an error, never run another way;
//  - T * Hq * ceil(max_kv_len / 128) * (D + 2) floats must fit in
//    ninfer_decode_attention_static_max_floats() (4 Mi floats = 16 MiB, which
//    every GPU the library runs on holds until the process ends): 8 rows of 16
//    heads of 128 at 30,000 keys, or 64 rows at 3,900; beyond that the call is
//    refused;
//  - max_kv_len must exceed every position in `positions` (it sizes the launch and the
//    chunks a row's partial results are laid out in); a position at or beyond it is read
//    as max_kv_len - 1, so nothing is written or read outside the array, and the row's
//    result is then that of the shorter context;
//  - ninfer_decode_attention_static_init() is best called once per device at set-up and
//    outside any graph capture: the first lookup of the array's address on a device may
//    load the library's code object there;
//  - the workspace and workspace_floats fields of the arguments are ignored;
//  - nothing in the array has to start at zero: pass 1 writes every entry that
//    the merge reads, so the last call's contents do not matter;
//  - every call on a GPU shares that GPU's array: calls that overlap on one GPU
//    (two streams, two threads) race. Calls on one stream are ordered.
// Neither call allocates or frees device or pinned memory.
#pragma once
#include "attention.h"

extern "C" {
// Looks up the array's address on the current device (once per device). Optional: the
// entry point does it at its first call on a device. 0 on success.
int ninfer_decode_attention_static_init();
// Most floats of workspace a call may need.
long long ninfer_decode_attention_static_max_floats();
// Paged attention of single-token rows, as ninfer_paged_attention runs them, into a->out.
int ninfer_decode_attention_static(const ninfer::AttnArgs* a, hipStream_t stream);
}

// Arguments of the product family C = A W^T (+ bias | SwiGLU), dense or
// grouped by expert. One struct serves every kernel of the family; the entry
// point picks the kernel from the dtype and the shape.
#pragma once
#include "common.h"

namespace ninfer {

enum Epilogue : int { kEpilogueNone = 0, kEpilogueSwiGLU = 1 };

struct GemmArgs {
  const void* A;         // [rows, lda] activations
  const void* W;         // [groups, N (2N for SwiGLU), K] weights
  void* C;               // [rows, ldc]
  const float* bias;     // [N] or null
  const int* offsets;    // [groups + 1] sorted-row ranges per group, or null (dense)
  const int* a_index;    // sorted row -> a_index[r] / a_div is the row of A, or null
  const int* c_index;    // sorted row -> row of C, or null
  int64_t w_group_stride;  // elements between the weights of two groups
  int M;                 // rows (dense) or number of sorted rows (grouped)
  int N;                 // output features (per SwiGLU half)
  int K;
  int lda;
  int ldc;
  int groups;
  int a_div;
  int in_dtype;          // of A and W
  int out_dtype;         // of C
  int epilogue;
};

int gemm_check(const GemmArgs& a);
int gemm_generic(const GemmArgs& a, hipStream_t stream);

}  // namespace ninfer

// Arguments of the product family C = A W^T (+ bias | SwiGLU), dense or
// grouped by expert. One struct serves every kernel of the family; the entry
// point picks the kernel from the dtype and the shape.
#pragma once
#include "common.h"

namespace ninfer {

// A gated epilogue forms act(x Wg^T) * (x Wu^T) from the two halves of W's rows; the
// activation is SiLU (SwiGLU) or the tanh form of GELU (GeGLU).
enum Epilogue : int { kEpilogueNone = 0, kEpilogueSwiGLU = 1, kEpilogueGeGLU = 2 };
inline bool epilogue_gated(int e) { return e == kEpilogueSwiGLU || e == kEpilogueGeGLU; }

// Both activations are g * sigmoid(z): z = g for SiLU; for GELU's tanh form,
// 0.5 g (1 + tanh(c (g + 0.044715 g^3))) with c = sqrt(2 / pi), z = 2 c (g + 0.044715 g^3).
__device__ __forceinline__ float gate_logit(float g, bool gelu) {
  return gelu ? 1.5957691216057308f * (g + 0.044715f * g * g * g) : g;
}

struct GemmArgs {
  const void* A;         // [rows, lda] activations
  const void* W;         // [groups, N (2N with a gated epilogue), K] weights
  void* C;               // [rows, ldc]
  const float* bias;     // [N] ([2N] with a gated epilogue: the gate's, then the other half's) or null
  const int* offsets;    // [groups + 1] sorted-row ranges per group, or null (dense)
  const int* a_index;    // sorted row -> a_index[r] / a_div is the row of A, or null
  const int* c_index;    // sorted row -> row of C, or null
  const int* tiles16;    // grouped: {expert, first row, end row, 0} per 16-row tile, or null
  const int* tiles_big;  // the same for the tall tiles (256 rows: gemm_tile_direct's)
  const int* tile_counts;  // {number of 16-row tiles, number of big tiles}
  int64_t w_group_stride;  // elements between the weights of two groups
  int M;                 // rows (dense) or number of sorted rows (grouped)
  int N;                 // output features (per half of a gated product)
  int K;
  int lda;
  int ldc;
  int groups;
  int a_div;
  int in_dtype;          // of A and W
  int out_dtype;         // of C
  int epilogue;
  int k_parts;           // the K range is cut into this many parts, one per blockIdx.z, part z
                         // writing its sums to C + z * M * ldc (0 or 1: no cut); set by
                         // gemm_split, not by callers
  float* workspace;      // 32-bit scratch for a product cut along K, or null
  int64_t workspace_floats;
  // What tests and measurements ask of one call (all 0: the library chooses). Per call, not
  // state of the library: a caller that forgets to reset it changes nothing for the next.
  int64_t split_min_bytes;  // least bytes of weights for a cut along K (0: 48 MB)
  int force_kernel;      // many-row kernel: 1, 2, 3 = tiles of 64, 128, 256 rows (grouped
                         // products run 256-row tiles unless told otherwise here)
  int skinny_two;        // few-row grouped products with two feature sets per block: 1 = whenever
                         // the shape allows, -1 = never
};

// Which rows does tile `ti` of the grouped enumeration cover? Tiles of
// `tile_rows` sorted rows are counted expert by expert from the device-side
// offsets. Called by every thread of the block; the first wave scans 64 groups
// at a time. info (LDS, 3 ints) receives {first row, end row of the expert,
// expert}; returns false when the tile does not exist.
__device__ inline bool find_tile(const int* __restrict__ offsets, int groups, int tile_rows,
                                 int ti, int* info) {
  if (threadIdx.x < 64) {
    const int lane = threadIdx.x;
    int base = 0, found = 0;
    for (int g0 = 0; g0 < groups && !found; g0 += 64) {
      int g = g0 + lane, b = 0, e = 0;
      if (g < groups) {
        b = offsets[g];
        e = offsets[g + 1];
      }
      int nt = (e - b + tile_rows - 1) / tile_rows;
      int incl = nt;
#pragma unroll
      for (int off = 1; off < 64; off <<= 1) {
        int v = __shfl_up(incl, off, 64);
        if (lane >= off) incl += v;
      }
      int lo = base + incl - nt, hi = base + incl;
      bool mine = ti >= lo && ti < hi;
      if (__ballot(mine)) {
        found = 1;
        if (mine) {
          info[0] = b + (ti - lo) * tile_rows;
          info[1] = e;
          info[2] = g;
        }
      }
      base += __shfl(incl, 63, 64);
    }
    if (!found && lane == 0) info[2] = -1;
  }
  __syncthreads();
  return info[2] >= 0;
}

// The rows of tile `ti`: from the tile list routing wrote (one 16-byte load),
// or by scanning the offsets when there is no list. `info` is 3 ints of LDS.
__device__ inline bool grouped_tile(const GemmArgs& a, const int* __restrict__ tiles, int which,
                                    int tile_rows, int ti, int* info) {
  if (!tiles) return find_tile(a.offsets, a.groups, tile_rows, ti, info);
  int count = a.tile_counts[which];
  int4 t = ((const int4*)tiles)[ti];
  if (ti >= count) return false;
  info[0] = t.y;
  info[1] = t.z;
  info[2] = t.x;
  return true;
}

int gemm_check(const GemmArgs& a);
bool gemm_skinny_takes(const GemmArgs& a);
int gemm_skinny(const GemmArgs& a, hipStream_t stream);
bool gemm_skinny_rows_takes(const GemmArgs& a);
int gemm_skinny_rows(const GemmArgs& a, hipStream_t stream);
bool gemm_skinny_pair_takes(const GemmArgs& a, const GemmArgs& b);
int gemm_skinny_pair(const GemmArgs& a, const GemmArgs& b, hipStream_t stream);
struct RouteArgs;
bool gemm_skinny_route_takes(const GemmArgs& a, const RouteArgs& rt);
int gemm_skinny_route(const GemmArgs& a, const RouteArgs& rt, hipStream_t stream);
bool gemm_skinny_route_pair_takes(const GemmArgs& a, const GemmArgs& b, const RouteArgs& rt);
int gemm_skinny_route_pair(const GemmArgs& a, const GemmArgs& b, const RouteArgs& rt,
                           hipStream_t stream);
bool gemm_tile_takes(const GemmArgs& a);
int gemm_tile(const GemmArgs& a, hipStream_t stream);
int gemm_generic(const GemmArgs& a, hipStream_t stream);
// Dense products of 33 to 512 rows whose output tiles are too few to fill the GPU: cut
// along K over more blocks, partial sums in the workspace, then added up in a fixed order.
int gemm_split_parts(const GemmArgs& a);   // parts the product would be cut into (< 2: not cut)
int gemm_split(const GemmArgs& a, hipStream_t stream);

}  // namespace ninfer

// Routing on the device, as functions of a wave (softmax + top-k of a row) and of a
// block (rows grouped by expert): the routing kernels are made of them, and so is the
// block of the few-row product kernel that routes the rows whose logits it has just
// computed. The reference does both on the host with a stream sync per layer
// (src/ops/moe.hip:49-106).
#pragma once
#include "common.h"

namespace ninfer {

// Where routing writes (all on the device).
struct RouteArgs {
  int* ids;          // [T, k] chosen experts, best first
  float* wts;        // [T, k] their weights
  int* offsets;      // [E + 1] ranges of `order` per expert
  int* order;        // [T k] flat (row, choice) indices grouped by expert
  int* tiles16;      // tile lists (see align_block), or all three null
  int* tiles64;
  int* tile_counts;
  int E;
  int k;
  int renorm;
  int big_rows;      // rows of a tile in tiles64: 64, 128 or 256
};

constexpr int kMaxExpertsPerLane = 16;  // up to 1024 experts

// One wave per row. p = softmax(logits) over all E; the k largest p in
// descending order, ties to the lower expert index; weights p (renorm: p / sum
// of the chosen). Reference formulas: src/ops/moe.hip:65-82.
// Returns the expert that lane j < k chose as its j-th (the same value it writes to ids[j]).
// NPL: experts a lane looks after (64 NPL >= E).
template <int NPL>
__device__ __forceinline__ int route_row(const float* __restrict__ row, int E, int k, int renorm,
                                         int* __restrict__ ids, float* __restrict__ wts,
                                         int lane) {
  float p[NPL];
  float m = -INFINITY;
#pragma unroll
  for (int i = 0; i < NPL; ++i) {
    int e = lane + i * 64;
    p[i] = e < E ? row[e] : -INFINITY;
    m = fmaxf(m, p[i]);
  }
  m = wave_max(m);
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < NPL; ++i) {
    int e = lane + i * 64;
    p[i] = e < E ? expf(p[i] - m) : 0.f;
    sum += p[i];
  }
  sum = wave_sum(sum);
  // A row with a NaN or an infinite logit has no softmax. The choice stays total all the
  // same (every probability counts as 0, so the first k experts are taken: ids are always
  // valid indices) and the weights come out NaN, so the fault stays visible downstream.
  const bool bad = !(sum > 0.f && sum < INFINITY);
#pragma unroll
  for (int i = 0; i < NPL; ++i) {
    int e = lane + i * 64;
    p[i] = e < E ? (bad ? 0.f : p[i] / sum) : -1.f;  // -1 marks "not a candidate"
  }
  float chosen_sum = 0.f, my_w = 0.f;
  int my_id = 0;
  for (int j = 0; j < k; ++j) {
    float best = -1.f;
    int best_e = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < NPL; ++i) {
      int e = lane + i * 64;
      if (p[i] > best) {  // ascending e within a lane: the first maximum is the lowest index
        best = p[i];
        best_e = e;
      }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      float ob = __shfl_xor(best, off, 64);
      int oe = __shfl_xor(best_e, off, 64);
      if (ob > best || (ob == best && oe < best_e)) {
        best = ob;
        best_e = oe;
      }
    }
#pragma unroll
    for (int i = 0; i < NPL; ++i)
      if (lane + i * 64 == best_e) p[i] = -1.f;
    chosen_sum += best;
    if (lane == j) {  // lane j keeps choice j
      my_w = best;
      my_id = best_e;
    }
  }
  if (lane < k) {
    ids[lane] = my_id;
    wts[lane] = bad ? __builtin_nanf("") : (renorm ? my_w / chosen_sum : my_w);
  }
  return my_id;
}

// Rows grouped by expert, by one block: offsets[e] .. offsets[e+1] are the
// positions in `order` of the flat (row, choice) indices routed to expert e.
// The order inside an expert is not fixed (atomic cursors), which no result
// depends on: every routed row is computed on its own and written back by its
// index. Also writes the lists of 16-row and 64-row tiles the grouped products
// walk: {expert, first row, end row, 0} per tile, and their counts.
// `cnt` is E + 1 ints of LDS; ids may be in LDS or global memory.
__device__ inline void align_block(const int* ids, int n, int E, int* __restrict__ offsets,
                            int* __restrict__ order, int* __restrict__ tiles16,
                            int* __restrict__ tiles64, int* __restrict__ tile_counts, int big, int* cnt) {
  for (int e = threadIdx.x; e < E; e += blockDim.x) cnt[e] = 0;
  __syncthreads();
  // ids from outside this file are clamped into [0, E): never an index out of bounds
  for (int i = threadIdx.x; i < n; i += blockDim.x) atomicAdd(&cnt[min(max(ids[i], 0), E - 1)], 1);
  __syncthreads();
  if (threadIdx.x < 64) {
    // the first wave scans 64 experts at a time: rows, 16-row tiles, 64-row tiles
    const int lane = threadIdx.x;
    int run0 = 0, n16 = 0, n64 = 0;
    for (int e0 = 0; e0 < E; e0 += 64) {
      const int e = e0 + lane;
      const int c = e < E ? cnt[e] : 0;
      const int t16 = (c + 15) / 16, t64 = (c + big - 1) / big;
      int ic = c, i16 = t16, i64 = t64;
#pragma unroll
      for (int off = 1; off < 64; off <<= 1) {
        int a1 = __shfl_up(ic, off, 64), a2 = __shfl_up(i16, off, 64), a3 = __shfl_up(i64, off, 64);
        if (lane >= off) {
          ic += a1;
          i16 += a2;
          i64 += a3;
        }
      }
      const int run = run0 + ic - c;
      if (e < E) {
        offsets[e] = run;
        cnt[e] = run;
        if (tiles16) {
          int p16 = n16 + i16 - t16, p64 = n64 + i64 - t64;
          for (int r = run; r < run + c; r += 16) ((int4*)tiles16)[p16++] = make_int4(e, r, run + c, 0);
          for (int r = run; r < run + c; r += big) ((int4*)tiles64)[p64++] = make_int4(e, r, run + c, 0);
        }
      }
      run0 += __shfl(ic, 63, 64);
      n16 += __shfl(i16, 63, 64);
      n64 += __shfl(i64, 63, 64);
    }
    if (lane == 0) {
      offsets[E] = run0;
      if (tile_counts) {
        tile_counts[0] = n16;
        tile_counts[1] = n64;
      }
    }
  }
  __syncthreads();
  for (int i = threadIdx.x; i < n; i += blockDim.x)
    order[atomicAdd(&cnt[min(max(ids[i], 0), E - 1)], 1)] = i;
}

}  // namespace ninfer

extern "C" int ninfer_router_topk(const float* logits, int ld, int T, int E, int k, int renorm,
                                  int* ids, float* wts, hipStream_t stream);
extern "C" int ninfer_moe_align(const int* ids, int n, int E, int* offsets, int* order,
                                int* tiles16, int* tiles64, int* tile_counts, int big_rows,
                                hipStream_t stream);
extern "C" int ninfer_moe_route_small(const float* logits, int ld, int T, int E, int k,
                                      int renorm, int* ids, float* wts, int* offsets, int* order,
                                      int* tiles16, int* tiles64, int* tile_counts, int big_rows,
                                      hipStream_t stream);

// Routing on the device, as functions of a wave (softmax + top-k of a row) and of a
// block (rows grouped by expert): the routing kernels are made of them, and so is the
// block of the few-row product kernel that routes the rows whose logits it has just
// computed. The reference does both on the host with a stream sync per layer
// (src/ops/moe.hip:49-106).
#pragma once
#include "common.h"

namespace ninfer {

enum RouteScore : int { kScoreSoftmax = 0, kScoreSigmoid = 1 };

// What a router computes from its logits, and where routing writes (all on the device).
//   s_e = softmax(logits)_e, or sigmoid(logits_e)            (`score`)
//   candidates = all experts, or with `n_group` > 1 those of the `topk_group` groups (of E /
//            n_group neighbouring experts each) whose largest s_e + choice_bias_e is largest,
//            ties to the lower group
//   chosen = the k candidates with the largest s_e + choice_bias_e, ties to the lower index
//   w_e    = s_e of the chosen (the bias decides the choice only), divided by their sum when
//            `renorm`, times `scale`
// Softmax without bias, scale 1: the reference's router (src/ops/moe.hip:65-82), which
// always renormalises.
struct RouteArgs {
  int* ids;          // [T, k] chosen experts, best first
  float* wts;        // [T, k] their weights
  int* offsets;      // [E + 1] ranges of `order` per expert
  int* order;        // [T k] flat (row, choice) indices grouped by expert
  int* tiles16;      // tile lists (see align_block), or all three null
  int* tiles_big;
  int* tile_counts;
  const float* choice_bias;  // [E] added to the scores for the choice only, or null
  int* parts;        // [ceil(T / kAlignRowsPerBlock), E] scratch for the routing of many rows
                     // (counts of the chosen experts per block of rows), or null
  int E;
  int k;
  int renorm;
  int score;         // RouteScore
  float scale;       // factor on every weight
  int n_group;       // groups of experts for a group-limited choice (0 or 1: none; at most 64)
  int topk_group;    // groups whose experts are candidates
};

// A group-limited choice asks: groups of equal size, at most 64 of them, and enough candidates
// left for k choices.
inline bool route_groups_ok(const RouteArgs& rt) {
  if (rt.n_group <= 1) return rt.n_group >= 0;
  return rt.n_group <= 64 && rt.E % rt.n_group == 0 && rt.topk_group >= 1 &&
         rt.topk_group <= rt.n_group && (long)rt.topk_group * (rt.E / rt.n_group) >= rt.k;
}

constexpr int kMaxExpertsPerLane = 16;  // up to 1024 experts
// Many rows: the grouping runs as blocks of this many rows side by side (a launch that counts
// what each block's rows chose, then one that places them).
constexpr int kAlignRowsPerBlock = 1024;

// One wave per row: scores, choice and weights as RouteArgs says; writes ids[0..k) and
// wts[0..k). Returns the expert that lane j < k chose as its j-th (the value it writes to
// ids[j]). NPL: experts a lane looks after (64 NPL >= E).
template <int NPL>
__device__ __forceinline__ int route_row(const float* __restrict__ row, const RouteArgs& rt,
                                         int* __restrict__ ids, float* __restrict__ wts,
                                         int lane) {
  const int E = rt.E, k = rt.k;
  float p[NPL];     // scores
  float sel[NPL];   // what the choice compares: score (+ bias); -inf: not a candidate
  bool bad = false;
  if (rt.score == kScoreSigmoid) {
#pragma unroll
    for (int i = 0; i < NPL; ++i) {
      const int e = lane + i * 64;
      p[i] = e < E ? 1.f / (1.f + expf(-row[e])) : 0.f;
      bad |= p[i] != p[i];
    }
  } else {
    float m = -INFINITY;
#pragma unroll
    for (int i = 0; i < NPL; ++i) {
      const int e = lane + i * 64;
      p[i] = e < E ? row[e] : -INFINITY;
      m = fmaxf(m, p[i]);
    }
    m = wave_max(m);
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < NPL; ++i) {
      const int e = lane + i * 64;
      p[i] = e < E ? expf(p[i] - m) : 0.f;
      sum += p[i];
    }
    sum = wave_sum(sum);
    bad = !(sum > 0.f && sum < INFINITY);
#pragma unroll
    for (int i = 0; i < NPL; ++i) p[i] = p[i] / sum;
  }
#pragma unroll
  for (int i = 0; i < NPL; ++i) {
    const int e = lane + i * 64;
    const float b = rt.choice_bias && e < E ? rt.choice_bias[e] : 0.f;
    sel[i] = p[i] + b;
    bad |= !(fabsf(b) < INFINITY);
  }
  // A row with a NaN or an infinite logit (or a bias that is not finite) has no scores. The choice stays
  // total all the same (every candidate counts as 0, so the first k experts are taken: ids
  // are always valid indices) and the weights come out NaN, so the fault stays visible
  // downstream.
  bad = __any(bad);
#pragma unroll
  for (int i = 0; i < NPL; ++i) sel[i] = lane + i * 64 < E ? (bad ? 0.f : sel[i]) : -INFINITY;
  if (rt.n_group > 1 && rt.topk_group < rt.n_group) {
    // the groups that may be chosen from: topk_group times the group of the best remaining score
    const int per_group = E / rt.n_group;
    unsigned long long open_groups = 0;
    for (int j = 0; j < rt.topk_group; ++j) {
      float best = -INFINITY;
      int best_g = 0x7fffffff;
#pragma unroll
      for (int i = 0; i < NPL; ++i) {
        const int e = lane + i * 64;
        if (e >= E) continue;
        const int g = e / per_group;
        if ((open_groups >> g) & 1ull) continue;
        if (sel[i] > best || (sel[i] == best && g < best_g)) {
          best = sel[i];
          best_g = g;
        }
      }
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) {
        const float ob = __shfl_xor(best, off, 64);
        const int og = __shfl_xor(best_g, off, 64);
        if (ob > best || (ob == best && og < best_g)) {
          best = ob;
          best_g = og;
        }
      }
      open_groups |= 1ull << best_g;
    }
#pragma unroll
    for (int i = 0; i < NPL; ++i) {
      const int e = lane + i * 64;
      if (e < E && !((open_groups >> (e / per_group)) & 1ull)) sel[i] = -INFINITY;
    }
  }
  float chosen_sum = 0.f, my_w = 0.f;
  int my_id = 0;
  for (int j = 0; j < k; ++j) {
    float best = -INFINITY, best_p = 0.f;
    int best_e = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < NPL; ++i) {
      const int e = lane + i * 64;
      if (sel[i] > best) {  // ascending e within a lane: the first maximum is the lowest index
        best = sel[i];
        best_p = p[i];
        best_e = e;
      }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const float ob = __shfl_xor(best, off, 64), op = __shfl_xor(best_p, off, 64);
      const int oe = __shfl_xor(best_e, off, 64);
      if (ob > best || (ob == best && oe < best_e)) {
        best = ob;
        best_p = op;
        best_e = oe;
      }
    }
#pragma unroll
    for (int i = 0; i < NPL; ++i)
      if (lane + i * 64 == best_e) sel[i] = -INFINITY;
    chosen_sum += best_p;
    if (lane == j) {  // lane j keeps choice j
      my_w = best_p;
      my_id = best_e;
    }
  }
  if (lane < k) {
    ids[lane] = my_id;
    wts[lane] = bad ? __builtin_nanf("") : (rt.renorm ? my_w / chosen_sum : my_w) * rt.scale;
  }
  return my_id;
}

// Rows grouped by expert, by one block: offsets[e] .. offsets[e+1] are the
// positions in `order` of the flat (row, choice) indices routed to expert e.
// The order inside an expert is not fixed (atomic cursors), which no result
// depends on: every routed row is computed on its own and written back by its
// index. Also writes the lists of 16-row and of kGroupedTileRows-row tiles the grouped
// products walk: {expert, first row, end row, 0} per tile, and their counts.
// `cnt` is E + 1 ints of LDS; ids may be in LDS or global memory.
__device__ inline void align_block(const int* ids, int n, int E, int* __restrict__ offsets,
                            int* __restrict__ order, int* __restrict__ tiles16,
                            int* __restrict__ tiles_big, int* __restrict__ tile_counts, int* cnt) {
  constexpr int big = kGroupedTileRows;
  for (int e = threadIdx.x; e < E; e += blockDim.x) cnt[e] = 0;
  __syncthreads();
  // ids from outside this file are clamped into [0, E): never an index out of bounds
  for (int i = threadIdx.x; i < n; i += blockDim.x) atomicAdd(&cnt[min(max(ids[i], 0), E - 1)], 1);
  __syncthreads();
  if (threadIdx.x < 64) {
    // the first wave scans 64 experts at a time: rows, 16-row tiles, tall tiles
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
          for (int r = run; r < run + c; r += big) ((int4*)tiles_big)[p64++] = make_int4(e, r, run + c, 0);
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

// Entry points (all only enqueue work). `rt` carries the router's parameters and outputs;
// router_topk reads E, k, renorm, score, scale, choice_bias, ids, wts of it.
extern "C" int ninfer_router_topk(const float* logits, int ld, int T, const ninfer::RouteArgs* rt,
                                  hipStream_t stream);
extern "C" int ninfer_moe_align(const int* ids, int n, int E, int* offsets, int* order,
                                int* tiles16, int* tiles_big, int* tile_counts,
                                hipStream_t stream);
// Scores + top-k and the grouping of many rows (T > 16) in three launches whose blocks work
// side by side; needs rt->parts. Without it (or for few rows) callers run ninfer_router_topk
// and ninfer_moe_align, whose grouping is one block.
extern "C" int ninfer_moe_route_many(const float* logits, int ld, int T,
                                     const ninfer::RouteArgs* rt, hipStream_t stream);
extern "C" int ninfer_moe_route_small(const float* logits, int ld, int T,
                                      const ninfer::RouteArgs* rt, hipStream_t stream);

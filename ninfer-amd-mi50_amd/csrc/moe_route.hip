// Routing on the device: scores + top-k per row, then rows grouped by expert.
// The reference does both on the host with a stream sync per layer
// (src/ops/moe.hip:49-106).
#include "moe_route.h"

namespace ninfer {

template <int NPL>
__global__ __launch_bounds__(64) void router_topk_kernel(const float* __restrict__ logits, int ld,
                                                         RouteArgs rt) {
  const int t = blockIdx.x;
  route_row<NPL>(logits + (int64_t)t * ld, rt, rt.ids + (int64_t)t * rt.k,
                 rt.wts + (int64_t)t * rt.k, threadIdx.x);
}

__global__ void moe_align_kernel(const int* __restrict__ ids, int n, int E,
                                 int* __restrict__ offsets, int* __restrict__ order,
                                 int* __restrict__ tiles16, int* __restrict__ tiles_big,
                                 int* __restrict__ tile_counts) {
  extern __shared__ int cnt[];
  align_block(ids, n, E, offsets, order, tiles16, tiles_big, tile_counts, cnt);
}

// Many rows, after the top-k kernel: block b counts the experts that rows
// [b, b + 1) x kAlignRowsPerBlock chose; the counts go to parts[b][E].
__global__ __launch_bounds__(1024) void moe_count_kernel(int T, RouteArgs rt) {
  extern __shared__ int cnt[];   // E
  const int E = rt.E;
  for (int e = threadIdx.x; e < E; e += blockDim.x) cnt[e] = 0;
  __syncthreads();
  const int i0 = blockIdx.x * kAlignRowsPerBlock * rt.k, i1 = min(T * rt.k, i0 + kAlignRowsPerBlock * rt.k);
  for (int i = i0 + threadIdx.x; i < i1; i += blockDim.x) atomicAdd(&cnt[min(max(rt.ids[i], 0), E - 1)], 1);
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += blockDim.x) rt.parts[(int64_t)blockIdx.x * E + e] = cnt[e];
}

// Many rows, last launch: block b groups rows [b, b + 1) x kAlignRowsPerBlock. Every block
// adds up the counts of all blocks (an expert's total, and what lies before its own rows), scans the totals into the experts' ranges, and places its rows with cursors of its
// own in LDS; block 0 also writes the ranges and the tile lists. The order inside an expert
// is rows of earlier blocks first; within a block it is not fixed (no result depends on it).
__global__ __launch_bounds__(1024) void moe_align_parts_kernel(int T, RouteArgs rt, int n_parts) {
  extern __shared__ int lds[];   // total[E], cursor[E], one more
  int* total = lds;
  int* cursor = lds + rt.E;
  const int E = rt.E, k = rt.k;
  const int first_part = blockIdx.x;
  for (int e = threadIdx.x; e < E; e += blockDim.x) total[e] = cursor[e] = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < n_parts * E; i += blockDim.x) {   // (sums of ints: any order)
    const int c = rt.parts[i];
    if (c) {
      atomicAdd(&total[i % E], c);
      if (i / E < first_part) atomicAdd(&cursor[i % E], c);
    }
  }
  __syncthreads();
  if (threadIdx.x < 64) {
    // the first wave scans 64 experts at a time: rows, 16-row tiles, tall tiles
    constexpr int big = kGroupedTileRows;
    const int lane = threadIdx.x;
    const bool writes = blockIdx.x == 0;
    int run0 = 0, n16 = 0, nbig = 0;
    for (int e0 = 0; e0 < E; e0 += 64) {
      const int e = e0 + lane;
      const int c = e < E ? total[e] : 0;
      const int t16 = (c + 15) / 16, tb = (c + big - 1) / big;
      int ic = c, i16 = t16, ib = tb;
#pragma unroll
      for (int off = 1; off < 64; off <<= 1) {
        int a1 = __shfl_up(ic, off, 64), a2 = __shfl_up(i16, off, 64), a3 = __shfl_up(ib, off, 64);
        if (lane >= off) {
          ic += a1;
          i16 += a2;
          ib += a3;
        }
      }
      const int run = run0 + ic - c;
      if (e < E) {
        cursor[e] += run;
        if (writes) {
          rt.offsets[e] = run;
          if (rt.tiles16) {
            int p16 = n16 + i16 - t16, pb = nbig + ib - tb;
            for (int r = run; r < run + c; r += 16) ((int4*)rt.tiles16)[p16++] = make_int4(e, r, run + c, 0);
            for (int r = run; r < run + c; r += big) ((int4*)rt.tiles_big)[pb++] = make_int4(e, r, run + c, 0);
          }
        }
      }
      run0 += __shfl(ic, 63, 64);
      n16 += __shfl(i16, 63, 64);
      nbig += __shfl(ib, 63, 64);
    }
    if (writes && lane == 0) {
      rt.offsets[E] = run0;
      if (rt.tile_counts) {
        rt.tile_counts[0] = n16;
        rt.tile_counts[1] = nbig;
      }
    }
  }
  __syncthreads();
  const int i0 = blockIdx.x * kAlignRowsPerBlock * k, i1 = min(T * k, i0 + kAlignRowsPerBlock * k);
  for (int i = i0 + threadIdx.x; i < i1; i += blockDim.x)
    rt.order[atomicAdd(&cursor[min(max(rt.ids[i], 0), E - 1)], 1)] = i;
}

// Few rows (decode): scores + top-k of every row and the grouping by expert
// in one launch of one block.
template <int NPL>
__global__ __launch_bounds__(1024) void moe_route_small_kernel(
    const float* __restrict__ logits, int ld, int T, RouteArgs rt, int ids_in_lds) {
  extern __shared__ int cnt[];   // E + 1 counters, then (if they fit) a copy of the chosen ids
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
  const int E = rt.E, k = rt.k;
  int* ids_s = ids_in_lds ? cnt + E + 1 : nullptr;
  for (int t = wave; t < T; t += waves) {
    const int mine = route_row<NPL>(logits + (int64_t)t * ld, rt, rt.ids + (int64_t)t * k,
                                    rt.wts + (int64_t)t * k, lane);
    // the grouping below reads the ids from LDS: no trip through global memory in between
    if (ids_s && lane < k) ids_s[t * k + lane] = mine;
  }
  __syncthreads();  // what this block wrote above is read below by other threads of this block
  align_block(ids_s ? ids_s : rt.ids, T * k, E, rt.offsets, rt.order, rt.tiles16, rt.tiles_big,
              rt.tile_counts, cnt);
}

}  // namespace ninfer

using namespace ninfer;

// What every routing entry point asks of the router's parameters.
static int route_args_check(const char* who, const RouteArgs& rt, int ld) {
  NINFER_REQUIRE(rt.E > 0 && rt.E <= 64 * kMaxExpertsPerLane, "%s: %d experts not in [1, %d]", who,
                 rt.E, 64 * kMaxExpertsPerLane);
  NINFER_REQUIRE(rt.k >= 1 && rt.k <= rt.E && rt.k <= 64, "%s: k=%d not in [1, min(%d, 64)]", who,
                 rt.k, rt.E);
  NINFER_REQUIRE(ld >= rt.E, "%s: row stride %d < %d experts", who, ld, rt.E);
  NINFER_REQUIRE(rt.score == kScoreSoftmax || rt.score == kScoreSigmoid,
                 "%s: score function %d is neither softmax (0) nor sigmoid (1)", who, rt.score);
  NINFER_REQUIRE(rt.scale == rt.scale && fabsf(rt.scale) < INFINITY, "%s: the scale is not finite",
                 who);
  NINFER_REQUIRE(rt.ids && rt.wts, "%s: no place for the chosen experts and weights", who);
  NINFER_REQUIRE(route_groups_ok(rt), "%s: %d groups of which %d are open do not fit %d experts and "
                 "k=%d (equal groups, at most 64, enough candidates)", who, rt.n_group, rt.topk_group,
                 rt.E, rt.k);
  return 0;
}

extern "C" int ninfer_router_topk(const float* logits, int ld, int T, const RouteArgs* rt,
                                  hipStream_t stream) {
  NINFER_REQUIRE(T > 0, "router_topk: T=%d must be positive", T);
  int rc = route_args_check("router_topk", *rt, ld);
  if (rc) return rc;
  // a lane looks after 1, 4 or 16 experts: the loops of the common sizes stay short
  if (rt->E <= 64)
    router_topk_kernel<1><<<T, 64, 0, stream>>>(logits, ld, *rt);
  else if (rt->E <= 256)
    router_topk_kernel<4><<<T, 64, 0, stream>>>(logits, ld, *rt);
  else
    router_topk_kernel<kMaxExpertsPerLane><<<T, 64, 0, stream>>>(logits, ld, *rt);
  NINFER_LAUNCH_CHECK();
  return 0;
}

// tiles16 / tiles_big / tile_counts may be null (no tile lists). tiles16 holds
// 4 ints for each of up to min(n, n / 16 + E) tiles of 16 rows, tiles_big for up
// to n / kGroupedTileRows + E tall tiles.
extern "C" int ninfer_moe_align(const int* ids, int n, int E, int* offsets, int* order,
                                int* tiles16, int* tiles_big, int* tile_counts,
                                hipStream_t stream) {
  NINFER_REQUIRE(n > 0 && E > 0, "moe_align: n=%d E=%d must be positive", n, E);
  NINFER_REQUIRE(E <= 8192, "moe_align: %d experts exceed 8192", E);
  NINFER_REQUIRE((!tiles16) == (!tiles_big) && (!tiles16) == (!tile_counts),
                 "moe_align: tile lists come together or not at all");
  moe_align_kernel<<<1, 1024, (E + 1) * sizeof(int), stream>>>(ids, n, E, offsets, order, tiles16,
                                                               tiles_big, tile_counts);
  NINFER_LAUNCH_CHECK();
  return 0;
}

extern "C" int ninfer_moe_route_many(const float* logits, int ld, int T, const RouteArgs* rt,
                                     hipStream_t stream) {
  NINFER_REQUIRE(T > 0, "moe_route_many: T=%d must be positive", T);
  int rc = route_args_check("moe_route_many", *rt, ld);
  if (rc) return rc;
  NINFER_REQUIRE(rt->offsets && rt->order && rt->parts, "moe_route_many: no place for the grouping "
                 "or its counts");
  NINFER_REQUIRE((!rt->tiles16) == (!rt->tiles_big) && (!rt->tiles16) == (!rt->tile_counts),
                 "moe_route_many: tile lists come together or not at all");
  NINFER_REQUIRE((int64_t)T * rt->k < (1LL << 31), "moe_route_many: %d rows of %d choices are too many", T,
                 rt->k);
  const int E = rt->E;
  rc = ninfer_router_topk(logits, ld, T, rt, stream);
  if (rc) return rc;
  const int blocks = (T + kAlignRowsPerBlock - 1) / kAlignRowsPerBlock;
  moe_count_kernel<<<blocks, 1024, E * sizeof(int), stream>>>(T, *rt);
  NINFER_LAUNCH_CHECK();
  moe_align_parts_kernel<<<blocks, 1024, (2 * E + 1) * sizeof(int), stream>>>(T, *rt, blocks);
  NINFER_LAUNCH_CHECK();
  return 0;
}

// Routing of few rows in one launch: top-k and grouping (T <= 256).
extern "C" int ninfer_moe_route_small(const float* logits, int ld, int T, const RouteArgs* rt,
                                      hipStream_t stream) {
  NINFER_REQUIRE(T > 0 && T <= 256, "moe_route_small: T=%d not in [1, 256]", T);
  int rc = route_args_check("moe_route_small", *rt, ld);
  if (rc) return rc;
  NINFER_REQUIRE(rt->offsets && rt->order, "moe_route_small: no place for the grouping");
  NINFER_REQUIRE((!rt->tiles16) == (!rt->tiles_big) && (!rt->tiles16) == (!rt->tile_counts),
                 "moe_route_small: tile lists come together or not at all");
  const int E = rt->E, k = rt->k;
  int threads = T >= 16 ? 1024 : 64 * T;
  const int ids_in_lds = T * k <= 4096;
  const size_t lds = (E + 1 + (ids_in_lds ? T * k : 0)) * sizeof(int);
#define NINFER_ROUTE_SMALL(NPL) \
  moe_route_small_kernel<NPL><<<1, threads, lds, stream>>>(logits, ld, T, *rt, ids_in_lds)
  if (E <= 64)
    NINFER_ROUTE_SMALL(1);
  else if (E <= 256)
    NINFER_ROUTE_SMALL(4);
  else
    NINFER_ROUTE_SMALL(kMaxExpertsPerLane);
#undef NINFER_ROUTE_SMALL
  NINFER_LAUNCH_CHECK();
  return 0;
}

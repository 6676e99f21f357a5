// Routing on the device: softmax + top-k per row, then rows grouped by expert.
// The reference does both on the host with a stream sync per layer
// (src/ops/moe.hip:49-106).
#include "moe_route.h"

namespace ninfer {

template <int NPL>
__global__ __launch_bounds__(64) void router_topk_kernel(const float* __restrict__ logits, int ld,
                                                         int E, int k, int renorm,
                                                         int* __restrict__ ids,
                                                         float* __restrict__ wts) {
  const int t = blockIdx.x;
  route_row<NPL>(logits + (int64_t)t * ld, E, k, renorm, ids + (int64_t)t * k, wts + (int64_t)t * k,
                 threadIdx.x);
}

__global__ void moe_align_kernel(const int* __restrict__ ids, int n, int E,
                                 int* __restrict__ offsets, int* __restrict__ order,
                                 int* __restrict__ tiles16, int* __restrict__ tiles64,
                                 int* __restrict__ tile_counts, int big) {
  extern __shared__ int cnt[];
  align_block(ids, n, E, offsets, order, tiles16, tiles64, tile_counts, big, cnt);
}

// Few rows (decode): softmax + top-k of every row and the grouping by expert
// in one launch of one block.
template <int NPL>
__global__ __launch_bounds__(1024) void moe_route_small_kernel(
    const float* __restrict__ logits, int ld, int T, int E, int k, int renorm,
    int* __restrict__ ids, float* __restrict__ wts, int* __restrict__ offsets,
    int* __restrict__ order, int* __restrict__ tiles16, int* __restrict__ tiles64,
    int* __restrict__ tile_counts, int big, int ids_in_lds) {
  extern __shared__ int cnt[];   // E + 1 counters, then (if they fit) a copy of the chosen ids
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
  int* ids_s = ids_in_lds ? cnt + E + 1 : nullptr;
  for (int t = wave; t < T; t += waves) {
    const int mine = route_row<NPL>(logits + (int64_t)t * ld, E, k, renorm, ids + (int64_t)t * k,
                                    wts + (int64_t)t * k, lane);
    // the grouping below reads the ids from LDS: no trip through global memory in between
    if (ids_s && lane < k) ids_s[t * k + lane] = mine;
  }
  __syncthreads();  // what this block wrote above is read below by other threads of this block
  align_block(ids_s ? ids_s : ids, T * k, E, offsets, order, tiles16, tiles64, tile_counts, big, cnt);
}

}  // namespace ninfer

using namespace ninfer;

extern "C" int ninfer_router_topk(const float* logits, int ld, int T, int E, int k, int renorm,
                                  int* ids, float* wts, hipStream_t stream) {
  NINFER_REQUIRE(T > 0 && E > 0, "router_topk: T=%d E=%d must be positive", T, E);
  NINFER_REQUIRE(E <= 64 * kMaxExpertsPerLane, "router_topk: %d experts exceed %d", E,
                 64 * kMaxExpertsPerLane);
  NINFER_REQUIRE(k >= 1 && k <= E && k <= 64, "router_topk: k=%d not in [1, min(%d, 64)]", k, E);
  NINFER_REQUIRE(ld >= E, "router_topk: row stride %d < %d experts", ld, E);
  // a lane looks after 1, 4 or 16 experts: the loops of the common sizes stay short
  if (E <= 64)
    router_topk_kernel<1><<<T, 64, 0, stream>>>(logits, ld, E, k, renorm, ids, wts);
  else if (E <= 256)
    router_topk_kernel<4><<<T, 64, 0, stream>>>(logits, ld, E, k, renorm, ids, wts);
  else
    router_topk_kernel<kMaxExpertsPerLane><<<T, 64, 0, stream>>>(logits, ld, E, k, renorm, ids, wts);
  NINFER_LAUNCH_CHECK();
  return 0;
}

// tiles16 / tiles64 / tile_counts may be null (no tile lists). tiles16 holds
// 4 ints for each of up to min(n, n / 16 + E) tiles of 16 rows, tiles64 for up
// to n / 64 + E tiles of big_rows (64, 128 or 256) rows.
extern "C" int ninfer_moe_align(const int* ids, int n, int E, int* offsets, int* order,
                                int* tiles16, int* tiles64, int* tile_counts, int big_rows,
                                hipStream_t stream) {
  NINFER_REQUIRE(big_rows == 64 || big_rows == 128 || big_rows == 256, "moe_align: big tiles of %d rows", big_rows);
  NINFER_REQUIRE(n > 0 && E > 0, "moe_align: n=%d E=%d must be positive", n, E);
  NINFER_REQUIRE(E <= 8192, "moe_align: %d experts exceed 8192", E);
  NINFER_REQUIRE((!tiles16) == (!tiles64) && (!tiles16) == (!tile_counts),
                 "moe_align: tile lists come together or not at all");
  moe_align_kernel<<<1, 1024, (E + 1) * sizeof(int), stream>>>(ids, n, E, offsets, order, tiles16,
                                                             tiles64, tile_counts, big_rows);
  NINFER_LAUNCH_CHECK();
  return 0;
}

// Routing of few rows in one launch: top-k and grouping (T <= 256).
extern "C" int ninfer_moe_route_small(const float* logits, int ld, int T, int E, int k,
                                      int renorm, int* ids, float* wts, int* offsets, int* order,
                                      int* tiles16, int* tiles64, int* tile_counts, int big_rows,
                                      hipStream_t stream) {
  NINFER_REQUIRE(big_rows == 64 || big_rows == 128 || big_rows == 256, "moe_route_small: big tiles of %d rows",
                 big_rows);
  NINFER_REQUIRE(T > 0 && T <= 256, "moe_route_small: T=%d not in [1, 256]", T);
  NINFER_REQUIRE(E > 0 && E <= 64 * kMaxExpertsPerLane, "moe_route_small: %d experts exceed %d", E,
                 64 * kMaxExpertsPerLane);
  NINFER_REQUIRE(k >= 1 && k <= E && k <= 64, "moe_route_small: k=%d not in [1, min(%d, 64)]", k, E);
  NINFER_REQUIRE(ld >= E, "moe_route_small: row stride %d < %d experts", ld, E);
  NINFER_REQUIRE((!tiles16) == (!tiles64) && (!tiles16) == (!tile_counts),
                 "moe_route_small: tile lists come together or not at all");
  int threads = T >= 16 ? 1024 : 64 * T;
  const int ids_in_lds = T * k <= 4096;
  const size_t lds = (E + 1 + (ids_in_lds ? T * k : 0)) * sizeof(int);
#define NINFER_ROUTE_SMALL(NPL)                                                                \
  moe_route_small_kernel<NPL><<<1, threads, lds, stream>>>(logits, ld, T, E, k, renorm, ids, wts, \
                                                           offsets, order, tiles16, tiles64,  \
                                                           tile_counts, big_rows, ids_in_lds)
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

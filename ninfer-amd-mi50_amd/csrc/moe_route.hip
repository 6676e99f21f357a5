// Routing on the device: softmax + top-k per row, then rows grouped by expert.
// The reference does both on the host with a stream sync per layer
// (src/ops/moe.hip:49-106).
#include "common.h"

namespace ninfer {

constexpr int kMaxExpertsPerLane = 16;  // up to 1024 experts

// One wave per row. p = softmax(logits) over all E; the k largest p in
// descending order, ties to the lower expert index; weights p (renorm: p / sum
// of the chosen). Reference formulas: src/ops/moe.hip:65-82.
__global__ __launch_bounds__(64) void router_topk_kernel(const float* __restrict__ logits, int ld,
                                                         int E, int k, int renorm,
                                                         int* __restrict__ ids,
                                                         float* __restrict__ wts) {
  const int t = blockIdx.x, lane = threadIdx.x;
  const float* row = logits + (int64_t)t * ld;
  float p[kMaxExpertsPerLane];
  float m = -INFINITY;
#pragma unroll
  for (int i = 0; i < kMaxExpertsPerLane; ++i) {
    int e = lane + i * 64;
    p[i] = e < E ? row[e] : -INFINITY;
    m = fmaxf(m, p[i]);
  }
  m = wave_max(m);
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < kMaxExpertsPerLane; ++i) {
    int e = lane + i * 64;
    p[i] = e < E ? expf(p[i] - m) : 0.f;
    sum += p[i];
  }
  sum = wave_sum(sum);
#pragma unroll
  for (int i = 0; i < kMaxExpertsPerLane; ++i) {
    int e = lane + i * 64;
    p[i] = e < E ? p[i] / sum : -1.f;  // -1 marks "not a candidate"
  }
  float chosen_sum = 0.f;
  float my_w = 0.f;
  int my_id = 0;
  for (int j = 0; j < k; ++j) {
    float best = -1.f;
    int best_e = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < kMaxExpertsPerLane; ++i) {
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
    for (int i = 0; i < kMaxExpertsPerLane; ++i)
      if (lane + i * 64 == best_e) p[i] = -1.f;
    chosen_sum += best;
    if (lane == j) {  // lane j keeps choice j
      my_w = best;
      my_id = best_e;
    }
  }
  if (lane < k) {
    ids[(int64_t)t * k + lane] = my_id;
    wts[(int64_t)t * k + lane] = renorm ? my_w / chosen_sum : my_w;
  }
}

// Rows grouped by expert: offsets[e] .. offsets[e+1] are the positions in
// `order` of the flat (row, choice) indices routed to expert e. One block; the
// order inside an expert is not fixed (atomic cursors), which no result depends
// on: every routed row is computed on its own and written back by its index.
__global__ void moe_align_kernel(const int* __restrict__ ids, int n, int E,
                                 int* __restrict__ offsets, int* __restrict__ order) {
  extern __shared__ int cnt[];  // [E] counts, then cursors
  for (int e = threadIdx.x; e < E; e += blockDim.x) cnt[e] = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < n; i += blockDim.x) atomicAdd(&cnt[ids[i]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int run = 0;
    for (int e = 0; e < E; ++e) {
      int c = cnt[e];
      offsets[e] = run;
      cnt[e] = run;
      run += c;
    }
    offsets[E] = run;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < n; i += blockDim.x) order[atomicAdd(&cnt[ids[i]], 1)] = i;
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
  router_topk_kernel<<<T, 64, 0, stream>>>(logits, ld, E, k, renorm, ids, wts);
  NINFER_LAUNCH_CHECK();
  return 0;
}

extern "C" int ninfer_moe_align(const int* ids, int n, int E, int* offsets, int* order,
                                hipStream_t stream) {
  NINFER_REQUIRE(n > 0 && E > 0, "moe_align: n=%d E=%d must be positive", n, E);
  NINFER_REQUIRE(E <= 8192, "moe_align: %d experts exceed 8192", E);
  moe_align_kernel<<<1, 1024, E * sizeof(int), stream>>>(ids, n, E, offsets, order);
  NINFER_LAUNCH_CHECK();
  return 0;
}

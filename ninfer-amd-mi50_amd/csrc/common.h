// Shared device helpers for the gfx950 kernels: element types, 64-lane wave
// reductions, and the error convention of the C entry points.
//
// Every entry point returns 0 on success and a negative code on a refused
// call (bad size, bad dtype); the message is kept per thread and read with
// ninfer_last_error(). Entry points only enqueue work on the given stream.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <stdint.h>

namespace ninfer {

enum DType : int { kF32 = 0, kBF16 = 1 };

typedef __hip_bfloat16 bf16;

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16 v) { return __bfloat162float(v); }
template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16 from_f32<bf16>(float v) { return __float2bfloat16(v); }

constexpr int kWave = 64;
// gfx950 (the one target) has 8 XCDs, each with an L2 of its own; the hardware deals
// workgroups to them in turn (block id mod 8). Kernels that share operands through L2 map
// block ids to work with this number.
constexpr int kXcds = 8;
// Rows of a tall tile of the grouped products (the height of gemm_tile_direct's tiles):
// what routing's list of tall tiles is made for.
constexpr int kGroupedTileRows = 256;

// Butterfly reductions over the 64 lanes of a wave: offsets 32 -> 1.
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
  return v;
}

// Sum over a block of up to 1024 threads; `red` holds 16 floats of LDS.
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  int nw = (blockDim.x + 63) >> 6;
  __syncthreads();
  if (lane == 0) red[w] = v;
  __syncthreads();
  float t = 0.f;
  for (int i = 0; i < nw; ++i) t += red[i];  // same order in every thread
  return t;
}

// A workgroup barrier that waits for this wave's LDS traffic only. The plain
// __syncthreads() also drains every global load in flight, which undoes
// software prefetching: loads issued for a later tile would be waited for at
// the next barrier. Use where the barrier only orders LDS reads and writes.
__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// A load of data that this kernel reads once and no other block reads soon (the cache of a
// decode step): marked non-temporal, so that it does not push out of the caches what is read
// again. Measured on decode attention over 8 x 8,192 keys, where a wave's load covers whole
// 128-byte lines: the cache streams at 5.6 instead of 5.0 TB/s. Not for the weights of the
// few-row products: their lanes take a line in pieces over several loads, and those kernels
// lost 5 to 12% with it.
template <typename V> __device__ __forceinline__ V stream_load(const V* p) {
  return __builtin_nontemporal_load(p);
}

int set_error(int code, const char* fmt, ...);

// Compute units of the current device (asked once per device; 256 if the runtime cannot
// say). Launch heuristics count blocks against it.
int device_cu_count();

#define NINFER_REQUIRE(cond, ...)                         \
  do {                                                    \
    if (!(cond)) return ::ninfer::set_error(-1, __VA_ARGS__); \
  } while (0)

#define NINFER_LAUNCH_CHECK()                                               \
  do {                                                                      \
    hipError_t e_ = hipGetLastError();                                      \
    if (e_ != hipSuccess)                                                   \
      return ::ninfer::set_error(-2, "kernel launch failed: %s", hipGetErrorString(e_)); \
  } while (0)

}  // namespace ninfer

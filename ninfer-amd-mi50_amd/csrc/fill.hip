// Fills: seeded random weights, and NaN into cache pages that were given back.
// The reference has neither (it loads checkpoints only and gives no page back).
//
// Random numbers are a pure function of a 64-bit key (from the seed and the
// tensor's name, made on the host) and the element's flat index, so a tensor's
// values do not depend on how it is cut over blocks, on the device, or on
// whether the host or the GPU computes them: the host mirror
// (weights/counter_random.py) gives the same bits. Element i hashes the three
// counters 3i, 3i + 1, 3i + 2 (splitmix64's finalizer over key + counter *
// golden ratio); the twelve 16-bit fields of the three hashes are added up (an
// integer between 0 and 12 * 65535, mean 6 * 65535, standard deviation 65536 up
// to 1e-10: the sum of twelve uniform numbers, the classic approximation of a
// normal one, cut at +-6 sigma) and z = (sum - mean) / 65536 exactly in 32-bit.
// The value is mean + std * z with one rounding for the product and one for
// the sum, then one to the storage type.
#include "common.h"

namespace ninfer {

__device__ __forceinline__ uint64_t mix64(uint64_t z) {
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

__device__ __forceinline__ float counter_normal(uint64_t key, uint64_t i) {
  int sum = 0;
#pragma unroll
  for (int j = 0; j < 3; ++j) {
    const uint64_t h = mix64(key + (3 * i + j) * 0x9E3779B97F4A7C15ull);
    sum += (int)(h & 0xffff) + (int)((h >> 16) & 0xffff) + (int)((h >> 32) & 0xffff) + (int)(h >> 48);
  }
  return (float)(sum - 6 * 65535) * (1.f / 65536.f);   // exact: |sum - mean| < 2^19
}

// mean + std * z with the product rounded before the sum, as the host computes it: the
// compiler must not contract the two into one fused multiply-add (which rounds once).
__device__ __forceinline__ float scale_shift(float z, float std, float mean) {
#pragma clang fp contract(off)
  const float prod = std * z;
  return mean + prod;
}

template <typename T>
__global__ void fill_random_kernel(T* __restrict__ out, int64_t n, uint64_t key, float std, float mean) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x)
    out[i] = from_f32<T>(scale_shift(counter_normal(key, (uint64_t)i), std, mean));
}

// NaN into pages[0 .. n) of a pool whose pages hold per_page numbers each.
template <typename T>
__global__ void fill_nan_pages_kernel(T* __restrict__ pool, const int* __restrict__ pages,
                                      int num_pages, int64_t per_page) {
  const int page = pages[blockIdx.y];
  if (page < 0 || page >= num_pages) return;   // never outside the pool, whatever the list holds
  T* dst = pool + (int64_t)page * per_page;
  const T nan = from_f32<T>(__builtin_nanf(""));
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < per_page;
       i += (int64_t)gridDim.x * blockDim.x)
    dst[i] = nan;
}

// A kernel that only reads: every wave walks a contiguous part of the buffer from one end to
// the other (whole 1 KB pieces per instruction, 16-byte non-temporal loads, eight on their
// way per lane: the pattern that streams fastest on this part) and writes nothing unless the
// words add up to a value they never add up to (which keeps the loads). What it reaches is
// the rate at which memory that is read once streams: the measure a decode step's weights
// and cache are held against.
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void read_probe_kernel(const u32x4* __restrict__ p, int64_t n_vec,
                                                         unsigned* __restrict__ sink) {
  const int64_t waves = (int64_t)gridDim.x * (blockDim.x >> 6);
  const int64_t wave = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  const int64_t per = (n_vec / 64 + waves - 1) / waves * 64;   // vectors of a wave's part
  const int64_t end = min(n_vec, (wave + 1) * per);
  int64_t i = wave * per + lane;
  unsigned acc = 0;
  for (; i + 7 * 64 < end; i += 8 * 64) {
    u32x4 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = __builtin_nontemporal_load(p + i + 64 * u);
#pragma unroll
    for (int u = 0; u < 8; ++u) acc += v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  }
  for (; i < end; i += 64) {
    const u32x4 a = __builtin_nontemporal_load(p + i);
    acc += a.x ^ a.y ^ a.z ^ a.w;
  }
  if (acc == 0x9e3779b9u && sink) *sink = acc;
}

}  // namespace ninfer

using namespace ninfer;

// Reads `bytes` bytes from `p` (16-byte aligned; a tail of fewer than 16 bytes is not read)
// and writes nothing: for measuring the rate of a plain read.
extern "C" int ninfer_read_probe(const void* p, long long bytes, hipStream_t stream) {
  NINFER_REQUIRE(p && bytes >= 16 && ((uintptr_t)p & 15) == 0, "read_probe: %lld bytes at %p", bytes, p);
  const int blocks = 16 * device_cu_count();
  read_probe_kernel<<<blocks, 256, 0, stream>>>((const u32x4*)p, bytes / 16, nullptr);
  NINFER_LAUNCH_CHECK();
  return 0;
}

extern "C" int ninfer_fill_random(void* out, long long n, unsigned long long key, float std,
                                  float mean, int dtype, hipStream_t stream) {
  NINFER_REQUIRE(n > 0, "fill_random: %lld elements", n);
  NINFER_REQUIRE(dtype == kF32 || dtype == kBF16, "fill_random: unknown dtype %d", dtype);
  const long long want = (n + 255) / 256;
  const unsigned blocks = (unsigned)(want < 65536 ? want : 65536);
  if (dtype == kF32)
    fill_random_kernel<float><<<blocks, 256, 0, stream>>>((float*)out, n, key, std, mean);
  else
    fill_random_kernel<bf16><<<blocks, 256, 0, stream>>>((bf16*)out, n, key, std, mean);
  NINFER_LAUNCH_CHECK();
  return 0;
}

extern "C" int ninfer_fill_nan_pages(void* pool, const int* pages, int n, int num_pages,
                                     long long per_page, int dtype, hipStream_t stream) {
  NINFER_REQUIRE(n > 0 && num_pages > 0 && per_page > 0, "fill_nan_pages: n=%d pages=%d per_page=%lld",
                 n, num_pages, per_page);
  NINFER_REQUIRE(n <= 65535, "fill_nan_pages: %d pages at once exceed 65535", n);
  NINFER_REQUIRE(dtype == kF32 || dtype == kBF16, "fill_nan_pages: unknown dtype %d", dtype);
  const long long want = (per_page + 255) / 256;
  dim3 grid((unsigned)(want < 64 ? want : 64), n);
  if (dtype == kF32)
    fill_nan_pages_kernel<float><<<grid, 256, 0, stream>>>((float*)pool, pages, num_pages, per_page);
  else
    fill_nan_pages_kernel<bf16><<<grid, 256, 0, stream>>>((bf16*)pool, pages, num_pages, per_page);
  NINFER_LAUNCH_CHECK();
  return 0;
}

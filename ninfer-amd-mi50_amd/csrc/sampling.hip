// Sampling on the device, one block per row of logits.
//
// Order of operations as in the reference's CPU sampler
// (src/runtime/engine.cpp:18-82): repetition penalty -> greedy if
// temperature <= 0 -> / temperature -> top-k -> softmax -> top-p -> draw.
// Differences, all deliberate: the penalty arrives as (token, count) pairs
// (a token seen c times is penalised c times, as the reference's loop over
// the history does); top-k and top-p are found by radix selection on the
// ordered bit pattern of the scaled logits instead of a sort, and of the tokens
// tied at the threshold the first ones in index order are kept, so the kept set
// is the prefix a stable sort by descending logit would give (top_k = 1 is the
// greedy choice, ties included); probabilities are held as 32.32 fixed-point
// integers so every sum is exact and the draw does not depend on the order of
// additions; the draw walks the kept tokens in index order with a uniform
// number `u` in [0,1) that the caller derives from (seed, request, draw
// index), so it does not depend on what else is in the batch. top_k <= 0
// keeps all tokens (the reference clamps to >= 1).
#include "common.h"

namespace ninfer {

constexpr int kSampleThreads = 1024;

__device__ __forceinline__ uint32_t ordered_key(float v) {
  uint32_t b = __float_as_uint(v);
  if (b == 0x80000000u) b = 0;   // -0 and +0 are one value, as in a comparison of floats
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);  // ascending with the float order
}

// Largest key t such that the sum of weight(i) over kept i with key(i) >= t
// reaches `target`. 4 passes of an 8-bit histogram. `hist` is 256 uint64 in LDS.
template <typename KeyFn, typename WeightFn>
__device__ uint32_t radix_select(int V, unsigned long long target, unsigned long long* hist,
                                 uint32_t* shared_out, KeyFn key, WeightFn weight) {
  uint32_t prefix = 0, mask = 0;
  for (int shift = 24; shift >= 0; shift -= 8) {
    for (int b = threadIdx.x; b < 256; b += blockDim.x) hist[b] = 0;
    __syncthreads();
    for (int i = threadIdx.x; i < V; i += blockDim.x) {
      uint32_t k = key(i);
      if ((k & mask) == prefix) {
        unsigned long long w = weight(i, k);
        if (w) atomicAdd(&hist[(k >> shift) & 255], w);
      }
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      unsigned long long run = 0;
      int b = 255;
      for (; b > 0; --b) {
        if (run + hist[b] >= target) break;
        run += hist[b];
      }
      shared_out[0] = (uint32_t)b;
      // mass above the chosen bin no longer counts towards the target
      ((unsigned long long*)(shared_out + 2))[0] = run;
    }
    __syncthreads();
    uint32_t b = shared_out[0];
    target -= ((unsigned long long*)(shared_out + 2))[0];
    prefix |= b << shift;
    mask |= 255u << shift;
    __syncthreads();
  }
  return prefix;
}

__global__ __launch_bounds__(kSampleThreads) void sample_kernel(
    const float* __restrict__ logits, int ld, int V, float* __restrict__ work,
    const float* __restrict__ temperature, const int* __restrict__ top_k,
    const float* __restrict__ top_p, const float* __restrict__ rep_penalty,
    const int* __restrict__ pen_tokens, const int* __restrict__ pen_counts,
    const int* __restrict__ pen_offsets, const float* __restrict__ uniform,
    const int* __restrict__ index_map, int* __restrict__ out) {
  __shared__ unsigned long long hist[256];
  __shared__ unsigned long long sums[kSampleThreads];
  __shared__ float fred[kSampleThreads / 64];
  __shared__ int ired[kSampleThreads / 64];
  __shared__ __align__(8) uint32_t sel[4];

  const int r = blockIdx.x, tid = threadIdx.x;
  const float* row = logits + (int64_t)r * ld;
  float* w = work + (int64_t)r * V;
  const float temp = temperature[r];

  // repetition penalty on a copy of the row (greedy rows without a penalty read the row itself)
  float rp = rep_penalty ? rep_penalty[r] : 1.f;
  const bool penalised = rp != 1.f && pen_offsets && pen_offsets[r + 1] > pen_offsets[r];
  if (!(temp > 0.f) && !penalised) {
    w = const_cast<float*>(row);
  } else {
    for (int i = tid; i < V; i += blockDim.x) w[i] = row[i];
  }
  __syncthreads();
  if (penalised) {
    for (int e = pen_offsets[r] + tid; e < pen_offsets[r + 1]; e += blockDim.x) {
      int tok = pen_tokens[e];
      if (tok < 0 || tok >= V) continue;
      float v = w[tok];
      for (int c = 0; c < pen_counts[e]; ++c) v = v > 0.f ? v / rp : v * rp;
      w[tok] = v;
    }
  }
  __syncthreads();

  // max and argmax (ties: lowest index); four loads in flight per thread
  float best = -INFINITY;
  int best_i = 0x7fffffff;
  for (int i0 = tid; i0 < V; i0 += 4 * blockDim.x) {
    float v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      int i = i0 + u * blockDim.x;
      v[u] = i < V ? w[i] : -INFINITY;
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (v[u] > best) {
        best = v[u];
        best_i = i0 + u * blockDim.x;
      }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    float ob = __shfl_xor(best, off, 64);
    int oi = __shfl_xor(best_i, off, 64);
    if (ob > best || (ob == best && oi < best_i)) {
      best = ob;
      best_i = oi;
    }
  }
  if ((tid & 63) == 0) {
    fred[tid >> 6] = best;
    ired[tid >> 6] = best_i;
  }
  __syncthreads();
  best = fred[0];
  best_i = ired[0];
  for (int i = 1; i < (int)(blockDim.x >> 6); ++i) {
    if (fred[i] > best || (fred[i] == best && ired[i] < best_i)) {
      best = fred[i];
      best_i = ired[i];
    }
  }
  // (the row may be a list of candidates: index_map gives the token behind each place)
  const int* map = index_map ? index_map + (int64_t)r * V : nullptr;
  if (!(temp > 0.f)) {
    if (tid == 0) out[r] = map ? map[best_i] : best_i;
    return;
  }
  __syncthreads();

  const float inv_t = 1.f / temp;
  const float m = best * inv_t;  // max of the scaled logits (temp > 0)
  typedef unsigned long long u64;
  auto key = [&](int i) { return ordered_key(w[i] * inv_t); };
  // probability of a token as 32.32 fixed point; tokens of equal key have equal mass
  auto mass_of = [&](int i) -> u64 { return (u64)(expf(w[i] * inv_t - m) * 4294967296.f); };
  auto mass_at = [&](uint32_t kk) -> u64 {
    const uint32_t bits = (kk & 0x80000000u) ? (kk & 0x7fffffffu) : ~kk;   // ordered_key's inverse
    return (u64)(expf(__uint_as_float(bits) - m) * 4294967296.f);
  };
  auto block_sum = [&](u64 v) -> u64 {
    sums[tid] = v;
    __syncthreads();
    for (int off = kSampleThreads / 2; off > 0; off >>= 1) {
      if (tid < off) sums[tid] += sums[tid + off];
      __syncthreads();
    }
    const u64 t = sums[0];
    __syncthreads();
    return t;
  };
  // tokens with a key above t (their count and mass) and with key t (their count)
  auto stats = [&](uint32_t t, u64& cnt_gt, u64& mass_gt, u64& cnt_eq) {
    u64 c = 0, ms = 0, e = 0;
    for (int i = tid; i < V; i += blockDim.x) {
      const uint32_t kk = key(i);
      if (kk > t) {
        ++c;
        ms += mass_of(i);
      } else if (kk == t) {
        ++e;
      }
    }
    cnt_gt = block_sum(c);
    mass_gt = block_sum(ms);
    cnt_eq = block_sum(e);
  };

  // The kept set is a prefix of the tokens ordered by (logit descending, index ascending),
  // as a sort would give it: every token with a key above `thr`, and of the tokens with key
  // `thr` the first `quota` in index order. Keeping all is thr = 0 with no token at it.
  uint32_t thr = 0;
  u64 cnt_gt, mass_gt, cnt_eq;
  const int k = top_k ? top_k[r] : 0;
  if (k > 0 && k < V)   // top-k: the k-th largest key
    thr = radix_select(V, (u64)k, hist, sel, key, [](int, uint32_t) { return 1ull; });
  stats(thr, cnt_gt, mass_gt, cnt_eq);
  u64 quota = (k > 0 && k < V) ? (u64)k - cnt_gt : cnt_eq;   // 1 .. cnt_eq with top-k
  u64 mass_thr = mass_at(thr);
  u64 total = mass_gt + quota * mass_thr;

  // top-p: the shortest prefix of that order whose mass reaches top_p of the total
  const float pp = top_p ? top_p[r] : 1.f;
  if (pp < 1.f) {
    u64 target = (u64)((double)pp * (double)total);
    if (target < 1) target = 1;
    if (target <= mass_gt) {   // it ends among the keys above thr
      const uint32_t floor_key = thr;
      thr = radix_select(V, target, hist, sel, key, [&](int i, uint32_t kk) -> u64 {
        return kk > floor_key ? mass_of(i) : 0ull;
      });
      stats(thr, cnt_gt, mass_gt, cnt_eq);
      mass_thr = mass_at(thr);
      quota = cnt_eq;
    }
    // mass_gt < target <= mass_gt + quota * mass_thr
    if (mass_thr > 0) {
      const u64 need = (target - mass_gt + mass_thr - 1) / mass_thr;
      if (need < quota) quota = need;
    }
    total = mass_gt + quota * mass_thr;
  }

  // inverse CDF over the kept tokens in index order; a thread owns a run of indices
  u64 goal = (u64)((double)uniform[r] * (double)total);
  if (goal >= total) goal = total - 1;
  const int chunk = (V + blockDim.x - 1) / blockDim.x;
  const int c0 = min(V, tid * chunk), c1 = min(V, c0 + chunk);
  auto shfl_up64 = [](u64 v, int d) -> u64 {
    const uint32_t lo = __shfl_up((uint32_t)v, d, 64), hi = __shfl_up((uint32_t)(v >> 32), d, 64);
    return ((u64)hi << 32) | lo;
  };
  auto scan = [&](u64 mine) -> u64 {   // sum over the threads before this one
    const int lane = tid & 63, wv = tid >> 6;
    u64 incl = mine;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const u64 o = shfl_up64(incl, d);
      if (lane >= d) incl += o;
    }
    if (lane == 63) sums[wv] = incl;
    __syncthreads();
    u64 base = 0;
    for (int i = 0; i < wv; ++i) base += sums[i];   // at most 15 wave totals
    __syncthreads();
    return base + incl - mine;
  };
  // ranks among the tokens tied at the threshold are needed only when not all of them are kept
  u64 eq_before = 0;
  if (quota < cnt_eq) {
    u64 eq_mine = 0;
    for (int i = c0; i < c1; ++i) eq_mine += key(i) == thr;
    eq_before = scan(eq_mine);
  }
  auto walk = [&](u64 start, bool pick_it) -> u64 {   // mass of the run; or the token at `goal`
    u64 run = start, rank = eq_before;
    for (int i = c0; i < c1; ++i) {
      const uint32_t kk = key(i);
      u64 ms = 0;
      if (kk > thr) ms = mass_of(i);
      else if (kk == thr && rank++ < quota) ms = mass_thr;
      if (pick_it && ms && goal < run + ms) return (u64)i;
      run += ms;
    }
    return pick_it ? (u64)(c1 - 1) : run - start;
  };
  const u64 mine = walk(0, false);
  const u64 before = scan(mine);
  if (mine > 0 && goal >= before && goal < before + mine) {
    const int pick = (int)walk(before, true);
    out[r] = map ? map[pick] : pick;
  }
}

// Candidates for rows that keep few tokens (greedy, or top-k up to kCandPerSlice): the row is
// cut into slices of kSlice tokens, one block each, so that the whole GPU reads the logits
// instead of one CU. A block holds its slice in LDS, applies the repetition penalty to it, and
// writes out, in index order, its own k best tokens under the order (scaled logit descending,
// index ascending). Every token of the row's k best is among its slice's k best, so the
// sampling kernel run on the candidates (sample_kernel with an index map) keeps the same set,
// sums the same masses and draws the same token as on the whole row.
constexpr int kSlice = 4096;
constexpr int kCandPerSlice = 64;
constexpr int kCandThreads = 256;

__global__ __launch_bounds__(kCandThreads) void sample_candidates_kernel(
    const float* __restrict__ logits, int ld, int V, const float* __restrict__ temperature,
    const int* __restrict__ top_k, const float* __restrict__ rep_penalty,
    const int* __restrict__ pen_tokens, const int* __restrict__ pen_counts,
    const int* __restrict__ pen_offsets, float* __restrict__ cand_val, int* __restrict__ cand_idx) {
  __shared__ float vals[kSlice];
  __shared__ unsigned long long hist[256];
  __shared__ __align__(8) uint32_t sel[4];
  __shared__ int wave_tot[kCandThreads / 64];
  const int r = blockIdx.y, b = blockIdx.x, tid = threadIdx.x;
  const int s0 = b * kSlice, n = min(kSlice, V - s0);
  const int C = gridDim.x * kCandPerSlice;
  const float* row = logits + (int64_t)r * ld;
  for (int i = tid; i < kSlice; i += kCandThreads) vals[i] = i < n ? row[s0 + i] : -INFINITY;
  __syncthreads();
  const float rp = rep_penalty ? rep_penalty[r] : 1.f;
  if (rp != 1.f && pen_offsets) {
    for (int e = pen_offsets[r] + tid; e < pen_offsets[r + 1]; e += kCandThreads) {
      const int tok = pen_tokens[e] - s0;
      if (tok < 0 || tok >= n) continue;
      float v = vals[tok];
      for (int c = 0; c < pen_counts[e]; ++c) v = v > 0.f ? v / rp : v * rp;
      vals[tok] = v;
    }
    __syncthreads();
  }
  const float temp = temperature[r];
  const float inv_t = temp > 0.f ? 1.f / temp : 1.f;
  int k = temp > 0.f ? top_k[r] : 1;            // greedy is the best one
  if (k < 1 || k > kCandPerSlice) k = kCandPerSlice;   // (not this entry's rows: kept in bounds)
  auto key = [&](int i) { return ordered_key(vals[i] * inv_t); };
  // the slice's k-th largest key, and how many of the tokens tied at it are kept
  uint32_t thr = 0;
  int quota = kSlice;
  if (k < n) {
    thr = radix_select(n, (unsigned long long)k, hist, sel, key, [](int, uint32_t) { return 1ull; });
    int above = 0;
    for (int i = tid; i < n; i += kCandThreads) above += key(i) > thr;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) above += __shfl_xor(above, off, 64);
    if ((tid & 63) == 0) wave_tot[tid >> 6] = above;
    __syncthreads();
    above = 0;
    for (int i = 0; i < kCandThreads / 64; ++i) above += wave_tot[i];
    __syncthreads();
    quota = k - above;
  }
  // in index order: a thread owns a run of consecutive tokens
  constexpr int RUN = kSlice / kCandThreads;
  auto scan = [&](int mine) -> int {   // sum over the threads before this one
    const int lane = tid & 63, wv = tid >> 6;
    int incl = mine;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int o = __shfl_up(incl, d, 64);
      if (lane >= d) incl += o;
    }
    if (lane == 63) wave_tot[wv] = incl;
    __syncthreads();
    int base = 0;
    for (int i = 0; i < wv; ++i) base += wave_tot[i];
    __syncthreads();
    return base + incl - mine;
  };
  const int i0 = tid * RUN, i1 = min(n, i0 + RUN);
  int eq = 0;
  for (int i = i0; i < i1; ++i) eq += key(i) == thr;
  int rank = scan(eq);
  int kept = 0;
  bool keep[RUN];
#pragma unroll
  for (int u = 0; u < RUN; ++u) {
    const int i = i0 + u;
    keep[u] = false;
    if (i < i1) {
      const uint32_t kk = key(i);
      keep[u] = kk > thr || (kk == thr && rank++ < quota);
    }
    kept += keep[u];
  }
  int pos = scan(kept);
  float* cv = cand_val + (int64_t)r * C + b * kCandPerSlice;
  int* ci = cand_idx + (int64_t)r * C + b * kCandPerSlice;
#pragma unroll
  for (int u = 0; u < RUN; ++u)
    if (keep[u]) {   // at most min(k, n) <= kCandPerSlice places
      cv[pos] = vals[i0 + u];
      ci[pos] = s0 + i0 + u;
      ++pos;
    }
  // the places left over hold nothing: never the largest, no mass
  const int total = min(k, n);
  for (int i = total + tid; i < kCandPerSlice; i += kCandThreads) {
    cv[i] = -INFINITY;
    ci[i] = 0;
  }
}

}  // namespace ninfer

using namespace ninfer;

// logits [R, ld] (V used); work [R, V] scratch; per-row temperature, top_k,
// top_p, rep_penalty, uniform; penalties as (token, count) pairs in
// pen_tokens/pen_counts[pen_offsets[r] .. pen_offsets[r+1]) (null: none);
// out [R] token ids.
extern "C" int ninfer_sample(const float* logits, int ld, int V, int R, float* work,
                             const float* temperature, const int* top_k, const float* top_p,
                             const float* rep_penalty, const int* pen_tokens,
                             const int* pen_counts, const int* pen_offsets, const float* uniform,
                             int* out, hipStream_t stream) {
  NINFER_REQUIRE(R > 0 && V > 0, "sample: R=%d V=%d must be positive", R, V);
  NINFER_REQUIRE(ld >= V, "sample: row stride %d < vocabulary %d", ld, V);
  NINFER_REQUIRE(temperature && uniform && work && out, "sample: a required array is null");
  sample_kernel<<<R, kSampleThreads, 0, stream>>>(logits, ld, V, work, temperature, top_k, top_p,
                                                  rep_penalty, pen_tokens, pen_counts, pen_offsets,
                                                  uniform, nullptr, out);
  NINFER_LAUNCH_CHECK();
  return 0;
}

// Places per row that ninfer_sample_few needs in each of cand_val, cand_idx and work.
extern "C" long long ninfer_sample_few_places(int V) {
  return (long long)((V + kSlice - 1) / kSlice) * kCandPerSlice;
}

// The same for rows that all keep few tokens: every row greedy (temperature <= 0) or with
// 1 <= top_k <= 64, which the caller asserts (a row with another top_k would be cut to its 64
// best per slice). Same result as ninfer_sample, from two launches that use the whole GPU.
// cand_val, cand_idx, work: [R, ninfer_sample_few_places(V)].
extern "C" int ninfer_sample_few(const float* logits, int ld, int V, int R, float* cand_val,
                                 int* cand_idx, float* work, const float* temperature,
                                 const int* top_k, const float* top_p, const float* rep_penalty,
                                 const int* pen_tokens, const int* pen_counts,
                                 const int* pen_offsets, const float* uniform, int* out,
                                 hipStream_t stream) {
  NINFER_REQUIRE(R > 0 && V > 0, "sample: R=%d V=%d must be positive", R, V);
  NINFER_REQUIRE(ld >= V, "sample: row stride %d < vocabulary %d", ld, V);
  NINFER_REQUIRE(temperature && top_k && uniform && cand_val && cand_idx && work && out,
                 "sample: a required array is null");
  const int slices = (V + kSlice - 1) / kSlice, C = slices * kCandPerSlice;
  NINFER_REQUIRE(R <= 65535, "sample: %d rows are too many", R);
  sample_candidates_kernel<<<dim3(slices, R), kCandThreads, 0, stream>>>(
      logits, ld, V, temperature, top_k, rep_penalty, pen_tokens, pen_counts, pen_offsets, cand_val,
      cand_idx);
  NINFER_LAUNCH_CHECK();
  sample_kernel<<<R, kSampleThreads, 0, stream>>>(cand_val, C, C, work, temperature, top_k, top_p,
                                                  nullptr, nullptr, nullptr, nullptr, uniform,
                                                  cand_idx, out);
  NINFER_LAUNCH_CHECK();
  return 0;
}

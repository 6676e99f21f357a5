// Paged attention, plain form: one wave per (row, query head).
//
// A row at position p of its request sees the keys of that request at
// positions lo..p, lo = max(0, p - window + 1) (window 0: all). Keys are
// walked in tiles of 64 aligned to absolute positions, with an online softmax
// (running max m, running sum l, rescale by exp(m_old - m_new): reference
// src/ops/attention.hip:62-75, :228-241; normalised at the end :92, :265), so
// the order of every sum depends only on the row's own position, never on how
// the request was cut into steps or what else is in the batch. Query head h
// reads kv head h / (Hq / Hkv) (reference src/ops/attention.hip:27-28).
// Scores, softmax and the value sum are 32-bit. This is the kernel of the true
// 32-bit path and of head sizes the MFMA kernels refuse.
#include "common.h"

namespace ninfer {

constexpr int kMaxDPerLane = 8;  // head sizes up to 512

template <typename T>
__global__ __launch_bounds__(64) void paged_attention_generic_kernel(
    const T* __restrict__ q, int q_stride, const T* __restrict__ kpool,
    const T* __restrict__ vpool, const int* __restrict__ block_table, int bt_stride,
    const int* __restrict__ positions, const int* __restrict__ row_seq, T* __restrict__ out,
    int Hq, int Hkv, int D, int page_size, int window, float scale,
    const float* __restrict__ slopes) {
  extern __shared__ float smem[];
  float* q_s = smem;                 // [D]
  float* p_s = smem + D;             // [64]
  int64_t* off_s = (int64_t*)(p_s + 64);  // [64] element offset of each key's row

  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int g = h / (Hq / Hkv);
  const int pos = positions[t];
  const int* bt = block_table + (int64_t)row_seq[t] * bt_stride;
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  const float slope = slopes ? slopes[h] : 0.f;

  const T* qr = q + (int64_t)t * q_stride + h * D;
  for (int d = lane; d < D; d += 64) q_s[d] = to_f32(qr[d]);
  __syncthreads();

  float m = -INFINITY, l = 0.f;
  float acc[kMaxDPerLane];
#pragma unroll
  for (int i = 0; i < kMaxDPerLane; ++i) acc[i] = 0.f;

  for (int tile = (lo / 64) * 64; tile <= pos; tile += 64) {
    int j = tile + lane;
    bool valid = j >= lo && j <= pos;
    float s = -INFINITY;
    int64_t off = 0;
    if (valid) {
      int page = bt[j / page_size];
      off = (((int64_t)page * Hkv + g) * page_size + (j % page_size)) * D;
      const T* kr = kpool + off;
      float dot = 0.f;
      for (int d = 0; d < D; ++d) dot = fmaf(q_s[d], to_f32(kr[d]), dot);
      s = fmaf(slope, (float)(j - pos), dot * scale);
    }
    float m_new = fmaxf(m, wave_max(s));
    float p = valid ? expf(s - m_new) : 0.f;
    float alpha = expf(m - m_new);  // 0 on the first tile (m = -inf)
    l = l * alpha + wave_sum(p);
    m = m_new;
    p_s[lane] = p;
    off_s[lane] = off;
    __syncthreads();
    int n_keys = min(64, pos - tile + 1);
    int first = max(0, lo - tile);
#pragma unroll
    for (int i = 0; i < kMaxDPerLane; ++i) {
      int d = lane + i * 64;
      if (d < D) {
        float a = acc[i] * alpha;
        for (int jj = first; jj < n_keys; ++jj) a = fmaf(p_s[jj], to_f32(vpool[off_s[jj] + d]), a);
        acc[i] = a;
      }
    }
    __syncthreads();
  }
  T* orow = out + ((int64_t)t * Hq + h) * D;
  float inv = 1.f / l;
#pragma unroll
  for (int i = 0; i < kMaxDPerLane; ++i) {
    int d = lane + i * 64;
    if (d < D) orow[d] = from_f32<T>(acc[i] * inv);
  }
}

int attention_generic(const void* q, int q_stride, const void* kpool, const void* vpool,
                      const int* block_table, int bt_stride, const int* positions,
                      const int* row_seq, void* out, int T, int Hq, int Hkv, int D, int page_size,
                      int window, float scale, const float* slopes, int dtype, hipStream_t stream) {
  NINFER_REQUIRE(D <= 64 * kMaxDPerLane, "paged_attention: head size %d exceeds %d", D,
                 64 * kMaxDPerLane);
  dim3 grid(T, Hq);
  size_t lds = (D + 64) * sizeof(float) + 64 * sizeof(int64_t);
  if (dtype == kF32)
    paged_attention_generic_kernel<float><<<grid, 64, lds, stream>>>(
        (const float*)q, q_stride, (const float*)kpool, (const float*)vpool, block_table, bt_stride,
        positions, row_seq, (float*)out, Hq, Hkv, D, page_size, window, scale, slopes);
  else
    paged_attention_generic_kernel<bf16><<<grid, 64, lds, stream>>>(
        (const bf16*)q, q_stride, (const bf16*)kpool, (const bf16*)vpool, block_table, bt_stride,
        positions, row_seq, (bf16*)out, Hq, Hkv, D, page_size, window, scale, slopes);
  NINFER_LAUNCH_CHECK();
  return 0;
}

}  // namespace ninfer

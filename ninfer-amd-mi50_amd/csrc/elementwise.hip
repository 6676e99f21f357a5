// Row-wise kernels: embedding gather, RMSNorm with the residual sum fused in,
// bias + rotary + paged cache write, and the expert combine.
//
// The residual stream is 32-bit in both precisions; activations are `T`
// (float or bf16). Sums of squares, rsqrt, rotation angles and weighted sums
// are 32-bit.
#include "common.h"

namespace ninfer {

// x[t,:] = table[token[t],:]   (reference src/ops/kernels.hip:150-159)
// [+ pos_table[position[t],:], learned absolute positions: a second gather, summed in 32-bit;
// a position beyond the table reads its last row, which the host refuses beforehand]
template <typename T>
__global__ void embed_kernel(const int* __restrict__ tokens, const T* __restrict__ table,
                             float* __restrict__ out, int H, const int* __restrict__ positions,
                             const T* __restrict__ pos_table, int pos_rows) {
  int64_t t = blockIdx.x;
  const T* src = table + (int64_t)tokens[t] * H;
  float* dst = out + t * H;
  if (pos_table) {
    const T* psrc = pos_table + (int64_t)min(max(positions[t], 0), pos_rows - 1) * H;
    for (int i = threadIdx.x; i < H; i += blockDim.x) dst[i] = to_f32(src[i]) + to_f32(psrc[i]);
  } else {
    for (int i = threadIdx.x; i < H; i += blockDim.x) dst[i] = to_f32(src[i]);
  }
}

// A weighted sum of rows that a sparse feed-forward leaves to be added to the
// residual: sum_j w[t,j] * y[t*k + j,:] + sigmoid(gate[t * gate_stride]) * shared[t,:]
// (gate null: factor 1; shared null: no such term; y null: nothing).
struct MoeSum {
  const void* y;
  const float* w;
  const void* shared;
  const float* gate;
  int gate_stride;
  int k;
};

constexpr int kNormPerThread = 8;

// VEC consecutive elements as floats (VEC = 4: one 16-byte or 8-byte load).
template <int VEC>
__device__ __forceinline__ void load_vec(const float* p, float* f) {
  if constexpr (VEC == 4) {
    float4 v = *(const float4*)p;
    f[0] = v.x; f[1] = v.y; f[2] = v.z; f[3] = v.w;
  } else {
    f[0] = p[0];
  }
}
template <int VEC>
__device__ __forceinline__ void load_vec(const bf16* p, float* f) {
  if constexpr (VEC == 4) {
    uint2 v = *(const uint2*)p;   // four bf16: the upper halves of four floats
    f[0] = __uint_as_float(v.x << 16); f[1] = __uint_as_float(v.x & 0xffff0000u);
    f[2] = __uint_as_float(v.y << 16); f[3] = __uint_as_float(v.y & 0xffff0000u);
  } else {
    f[0] = to_f32(p[0]);
  }
}
template <int VEC>
__device__ __forceinline__ void store_vec(float* p, const float* f) {
  if constexpr (VEC == 4) *(float4*)p = make_float4(f[0], f[1], f[2], f[3]);
  else p[0] = f[0];
}
template <int VEC>
__device__ __forceinline__ void store_vec(bf16* p, const float* f) {
#pragma unroll
  for (int e = 0; e < VEC; ++e) p[e] = __float2bfloat16(f[e]);
}

// y = (x [+ delta] [+ moe sum]) * rsqrt(mean(.^2) + eps) * gain  (reference
// src/ops/kernels.hip:17-41 and :100-129). With rows == nullptr the sum is
// written back to x; with rows the kernel reads row rows[i] and leaves x alone.
// Every thread keeps its (at most 8) elements in registers between the two
// passes, in groups of VEC consecutive elements; all loads of a thread are
// independent of each other, so they are in flight together. The reduction
// order depends only on H, VEC and the block size, never on the number of rows.
template <typename T, int VEC>
__global__ void rmsnorm_kernel(float* __restrict__ x, const T* __restrict__ delta, MoeSum ms,
                               const float* __restrict__ gain, T* __restrict__ out,
                               const int* __restrict__ rows, int H, float eps) {
  constexpr int G = kNormPerThread / VEC;   // groups per thread
  __shared__ float red[16];
  int64_t r_out = blockIdx.x;
  int64_t r_in = rows ? rows[r_out] : r_out;
  float* xr = x + r_in * H;
  const T* dr = delta ? delta + r_in * H : nullptr;
  T* orow = out + r_out * H;
  float vals[G][VEC];
#pragma unroll
  for (int c = 0; c < G; ++c) {
    int i = VEC * (threadIdx.x + c * blockDim.x);
#pragma unroll
    for (int e = 0; e < VEC; ++e) vals[c][e] = 0.f;
    if (i < H) {
      load_vec<VEC>(xr + i, vals[c]);
      if (dr) {
        float d[VEC];
        load_vec<VEC>(dr + i, d);
#pragma unroll
        for (int e = 0; e < VEC; ++e) vals[c][e] += d[e];
      }
    }
  }
  if (ms.y) {
    const T* y = (const T*)ms.y + r_in * ms.k * H;
    const float* w = ms.w + r_in * ms.k;
    for (int j0 = 0; j0 < ms.k; j0 += 4) {   // four routed rows at a time, loads independent
      float wj[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) wj[j] = j0 + j < ms.k ? w[j0 + j] : 0.f;
#pragma unroll
      for (int c = 0; c < G; ++c) {
        int i = VEC * (threadIdx.x + c * blockDim.x);
        if (i < H) {
          float yv[4][VEC];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            if (j0 + j < ms.k) {
              load_vec<VEC>(y + (int64_t)(j0 + j) * H + i, yv[j]);
            } else {
#pragma unroll
              for (int e = 0; e < VEC; ++e) yv[j][e] = 0.f;
            }
          }
#pragma unroll
          for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int e = 0; e < VEC; ++e) vals[c][e] += wj[j] * yv[j][e];
        }
      }
    }
    if (ms.shared) {
      float g = ms.gate ? 1.f / (1.f + expf(-ms.gate[r_in * ms.gate_stride])) : 1.f;
      const T* sh = (const T*)ms.shared + r_in * H;
#pragma unroll
      for (int c = 0; c < G; ++c) {
        int i = VEC * (threadIdx.x + c * blockDim.x);
        if (i < H) {
          float sv[VEC];
          load_vec<VEC>(sh + i, sv);
#pragma unroll
          for (int e = 0; e < VEC; ++e) vals[c][e] += g * sv[e];
        }
      }
    }
  }
  float acc = 0.f;
#pragma unroll
  for (int c = 0; c < G; ++c)
#pragma unroll
    for (int e = 0; e < VEC; ++e) acc += vals[c][e] * vals[c][e];
  float total = block_sum(acc, red);
  float inv = rsqrtf(total / (float)H + eps);
  const bool write_back = !rows && (dr || ms.y);
#pragma unroll
  for (int c = 0; c < G; ++c) {
    int i = VEC * (threadIdx.x + c * blockDim.x);
    if (i < H) {
      if (write_back) store_vec<VEC>(xr + i, vals[c]);
      float gv[VEC], o[VEC];
      load_vec<VEC>(gain + i, gv);
#pragma unroll
      for (int e = 0; e < VEC; ++e) o[e] = vals[c][e] * inv * gv[e];
      store_vec<VEC>(orow + i, o);
    }
  }
}

// One block per row of the fused q|k|v activations. Adds the bias, rotates q
// heads in place and k heads on their way into the page; v heads are copied.
// Pairs are (i, i + rot/2) within the first `rot` dims of a head (reference
// src/ops/kernels.hip:86-91, full rotation there), or neighbours (2i, 2i + 1)
// when `interleaved`; pair i turns by pos * inv_freq[i]; dims >= rot pass through.
// A work item is one rotating pair or one pass-through element, read and
// written by one thread, so q can be rewritten in place without a barrier.
// Page lookup: logical page pos / page_size of the row's request.
template <typename T>
__global__ void rope_kv_write_kernel(T* __restrict__ qkv, const float* __restrict__ bias,
                                     const int* __restrict__ positions,
                                     const int* __restrict__ row_seq,
                                     const float* __restrict__ inv_freq, int rot, int Hq, int Hkv,
                                     int D, T* __restrict__ kpool, T* __restrict__ vpool,
                                     const int* __restrict__ block_table, int bt_stride,
                                     int page_size, int write_kv, int interleaved) {
  const int t = blockIdx.x;
  const int half = rot >> 1;
  const int per_head = half + (D - rot);          // items of a rotated head
  const int n_heads = write_kv ? Hq + 2 * Hkv : Hq;
  const int W = (Hq + 2 * Hkv) * D;
  T* row = qkv + (int64_t)t * W;
  const int pos = positions[t];
  const int page = write_kv ? block_table[(int64_t)row_seq[t] * bt_stride + pos / page_size] : 0;
  const int slot = pos % page_size;
  for (int it = blockIdx.y * blockDim.x + threadIdx.x; it < n_heads * per_head;
       it += gridDim.y * blockDim.x) {
    const int head = it / per_head, i = it % per_head;
    const bool is_q = head < Hq, is_k = !is_q && head < Hq + Hkv;
    const int base = head * D;
    int d0, d1 = -1;                               // element(s) of this item
    float v0, v1 = 0.f;
    if (i < half) {
      d0 = interleaved ? 2 * i : i;
      d1 = interleaved ? 2 * i + 1 : i + half;
      v0 = to_f32(row[base + d0]) + (bias ? bias[base + d0] : 0.f);
      v1 = to_f32(row[base + d1]) + (bias ? bias[base + d1] : 0.f);
      if (is_q || is_k) {
        float phi = (float)pos * inv_freq[i];
        float c, s;
        sincosf(phi, &s, &c);   // one range reduction for both
        float r0 = v0 * c - v1 * s, r1 = v0 * s + v1 * c;
        v0 = r0;
        v1 = r1;
      }
    } else {
      d0 = rot + (i - half);
      v0 = to_f32(row[base + d0]) + (bias ? bias[base + d0] : 0.f);
    }
    if (is_q) {
      row[base + d0] = from_f32<T>(v0);
      if (d1 >= 0) row[base + d1] = from_f32<T>(v1);
    } else {
      const int kvh = is_k ? head - Hq : head - Hq - Hkv;
      T* dst = (is_k ? kpool : vpool) + (((int64_t)page * Hkv + kvh) * page_size + slot) * D;
      dst[d0] = from_f32<T>(v0);
      if (d1 >= 0) dst[d1] = from_f32<T>(v1);
    }
  }
}

// The same for query and key heads that are normed before they turn: head vector
// v = x + bias, v * rsqrt(mean(v^2) + eps) * gain[d] (one gain vector for the query heads, one
// for the key heads; value heads pass as they are), then the rotation. One wave per (row,
// head): the head lies in LDS in 32-bit between the norm and the rotation.
template <typename T>
__global__ __launch_bounds__(256) void rope_kv_write_normed_kernel(
    T* __restrict__ qkv, const float* __restrict__ bias, const int* __restrict__ positions,
    const int* __restrict__ row_seq, const float* __restrict__ inv_freq, int rot, int Hq, int Hkv,
    int D, T* __restrict__ kpool, T* __restrict__ vpool, const int* __restrict__ block_table,
    int bt_stride, int page_size, int write_kv, int interleaved, const float* __restrict__ q_gain,
    const float* __restrict__ k_gain, float eps) {
  extern __shared__ float heads_s[];   // [waves][D]
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n_heads = write_kv ? Hq + 2 * Hkv : Hq;
  const int head = blockIdx.y * (blockDim.x >> 6) + wave;
  if (head >= n_heads) return;   // (no block-wide barrier below: a wave works alone)
  float* v = heads_s + wave * D;
  const int half = rot >> 1;
  const int W = (Hq + 2 * Hkv) * D;
  T* row = qkv + (int64_t)t * W;
  const int pos = positions[t];
  const bool is_q = head < Hq, is_k = !is_q && head < Hq + Hkv;
  const int base = head * D;
  float sq = 0.f;
  for (int d = lane; d < D; d += 64) {
    const float x = to_f32(row[base + d]) + (bias ? bias[base + d] : 0.f);
    v[d] = x;
    sq += x * x;
  }
  const float* gain = is_q ? q_gain : (is_k ? k_gain : nullptr);
  if (gain) {
    const float inv = rsqrtf(wave_sum(sq) / (float)D + eps);
    for (int d = lane; d < D; d += 64) v[d] = v[d] * inv * gain[d];   // each lane its own elements
  }
  __builtin_amdgcn_wave_barrier();
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the wave's LDS writes are done before its reads
  T* dst = row + base;
  if (!is_q) {
    const int page = block_table[(int64_t)row_seq[t] * bt_stride + pos / page_size];
    const int kvh = is_k ? head - Hq : head - Hq - Hkv;
    dst = (is_k ? kpool : vpool) + (((int64_t)page * Hkv + kvh) * page_size + pos % page_size) * D;
  }
  const int per_head = half + (D - rot);
  for (int i = lane; i < per_head; i += 64) {
    if (i < half && (is_q || is_k)) {
      const int d0 = interleaved ? 2 * i : i, d1 = interleaved ? 2 * i + 1 : i + half;
      float c, s;
      sincosf((float)pos * inv_freq[i], &s, &c);
      dst[d0] = from_f32<T>(v[d0] * c - v[d1] * s);
      dst[d1] = from_f32<T>(v[d0] * s + v[d1] * c);
    } else if (i < half) {   // a value head: both elements of the pair pass
      const int d0 = interleaved ? 2 * i : i, d1 = interleaved ? 2 * i + 1 : i + half;
      dst[d0] = from_f32<T>(v[d0]);
      dst[d1] = from_f32<T>(v[d1]);
    } else {
      const int d0 = rot + (i - half);
      dst[d0] = from_f32<T>(v[d0]);
    }
  }
}

// Eight consecutive elements at once (16 or 32 bytes).
__device__ __forceinline__ void load8(const float* p, float* f) {
  const float4 a = *(const float4*)p, b = *(const float4*)(p + 4);
  f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w; f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
}
__device__ __forceinline__ void load8(const bf16* p, float* f) {
  typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
  const bf16x8 v = *(const bf16x8*)p;
#pragma unroll
  for (int e = 0; e < 8; ++e) f[e] = (float)v[e];
}
__device__ __forceinline__ void store8(float* p, const float* f) {
  *(float4*)p = make_float4(f[0], f[1], f[2], f[3]);
  *(float4*)(p + 4) = make_float4(f[4], f[5], f[6], f[7]);
}
__device__ __forceinline__ void store8(bf16* p, const float* f) {
  typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
  bf16x8 v;
#pragma unroll
  for (int e = 0; e < 8; ++e) v[e] = (__bf16)f[e];
  *(bf16x8*)p = v;
}

// The same as rope_kv_write_kernel for many rows, eight elements per access:
// a work item is eight rotating pairs (dims i .. i + 7 and their partners at
// + rot / 2) or eight pass-through elements. One block per row; the row's
// cosines and sines are computed once, into LDS, for all its heads. Needs
// rot / 2, D - rot and D to be multiples of 8 and 16-byte aligned rows.
template <typename T>
__global__ __launch_bounds__(256) void rope_kv_write_rows_kernel(
    T* __restrict__ qkv, const float* __restrict__ bias, const int* __restrict__ positions,
    const int* __restrict__ row_seq, const float* __restrict__ inv_freq, int rot, int Hq, int Hkv,
    int D, T* __restrict__ kpool, T* __restrict__ vpool, const int* __restrict__ block_table,
    int bt_stride, int page_size, int write_kv) {
  extern __shared__ float trig[];   // [rot / 2] cosines, [rot / 2] sines
  const int t = blockIdx.x;
  const int half = rot >> 1;
  const int W = (Hq + 2 * Hkv) * D;
  T* row = qkv + (int64_t)t * W;
  const int pos = positions[t];
  const int page = write_kv ? block_table[(int64_t)row_seq[t] * bt_stride + pos / page_size] : 0;
  const int slot = pos % page_size;
  for (int i = threadIdx.x; i < half; i += blockDim.x) {
    const float phi = (float)pos * inv_freq[i];
    sincosf(phi, &trig[half + i], &trig[i]);   // one range reduction for both
  }
  __syncthreads();
  const int rot_items = half / 8, pass_items = (D - rot) / 8;   // of a rotated head
  const int per_qk = rot_items + pass_items, per_v = D / 8;
  const int n_qk = (write_kv ? Hq + Hkv : Hq) * per_qk;
  const int n_items = n_qk + (write_kv ? Hkv * per_v : 0);
  for (int it = threadIdx.x; it < n_items; it += blockDim.x) {
    int head, d0;
    bool rotate = false;
    if (it < n_qk) {
      head = it / per_qk;
      const int i = it % per_qk;
      rotate = i < rot_items;
      d0 = rotate ? 8 * i : rot + 8 * (i - rot_items);
    } else {
      head = Hq + Hkv + (it - n_qk) / per_v;
      d0 = 8 * ((it - n_qk) % per_v);
    }
    const int base = head * D;
    T* dst = row + base;      // q: in place
    if (head >= Hq) {
      const bool is_k = head < Hq + Hkv;
      const int kvh = is_k ? head - Hq : head - Hq - Hkv;
      dst = (is_k ? kpool : vpool) + (((int64_t)page * Hkv + kvh) * page_size + slot) * D;
    }
    float v0[8], v1[8];
    load8(row + base + d0, v0);
    if (bias) {
#pragma unroll
      for (int e = 0; e < 8; ++e) v0[e] += bias[base + d0 + e];
    }
    if (rotate) {
      load8(row + base + d0 + half, v1);
      if (bias) {
#pragma unroll
        for (int e = 0; e < 8; ++e) v1[e] += bias[base + d0 + half + e];
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float c = trig[d0 + e], s = trig[half + d0 + e];
        const float r0 = v0[e] * c - v1[e] * s, r1 = v0[e] * s + v1[e] * c;
        v0[e] = r0;
        v1[e] = r1;
      }
      store8(dst + d0 + half, v1);
    }
    store8(dst + d0, v0);
  }
}

// residual[t,:] += sum_j w[t,j] * y[t*k + j,:] + sigmoid(gate[t]) * shared[t,:]
// in that order, in 32-bit (the reference scales and scatter-adds rounded
// rows: src/ops/kernels.hip:216-223, src/ops/moe.hip:22-31).
template <typename T>
__global__ void moe_combine_kernel(float* __restrict__ residual, const T* __restrict__ y,
                                   const float* __restrict__ w, const T* __restrict__ shared,
                                   const float* __restrict__ gate, int gate_stride, int H, int k) {
  const int64_t t = blockIdx.x;
  const int i = blockIdx.y * blockDim.x + threadIdx.x;
  if (i >= H) return;
  float acc = 0.f;
  for (int j = 0; j < k; ++j) acc += w[t * k + j] * to_f32(y[(t * k + j) * H + i]);
  if (shared) {
    float g = gate ? 1.f / (1.f + expf(-gate[t * gate_stride])) : 1.f;
    acc += g * to_f32(shared[t * H + i]);
  }
  residual[t * H + i] += acc;
}

}  // namespace ninfer

using namespace ninfer;

// positions / pos_table / pos_rows: learned absolute positions [pos_rows, H] of the table's
// dtype, gathered by positions [T] and added; all null / 0: none.
extern "C" int ninfer_embed(const int* tokens, const void* table, float* out, int T, int H,
                            int dtype, const int* positions, const void* pos_table, int pos_rows,
                            hipStream_t stream) {
  NINFER_REQUIRE(T > 0 && H > 0, "embed: T=%d H=%d must be positive", T, H);
  NINFER_REQUIRE(dtype == kF32 || dtype == kBF16, "embed: unknown dtype %d", dtype);
  NINFER_REQUIRE(!pos_table || (positions && pos_rows > 0),
                 "embed: a table of positions needs the rows' positions and its row count (%d)", pos_rows);
  if (dtype == kF32)
    embed_kernel<float><<<T, 256, 0, stream>>>(tokens, (const float*)table, out, H, positions,
                                               (const float*)pos_table, pos_rows);
  else
    embed_kernel<bf16><<<T, 256, 0, stream>>>(tokens, (const bf16*)table, out, H, positions,
                                              (const bf16*)pos_table, pos_rows);
  NINFER_LAUNCH_CHECK();
  return 0;
}

// moe_* describe an optional weighted sum of rows added before the norm (all
// null / 0: none): y [rows * k, H], w [rows, k], shared [rows, H], gate logits
// with stride gate_stride.
extern "C" int ninfer_rmsnorm(float* x, const void* delta, const float* gain, void* out,
                              const int* rows, int n_rows, int H, float eps, int dtype,
                              const void* moe_y, const float* moe_w, const void* moe_shared,
                              const float* moe_gate, int moe_gate_stride, int moe_k,
                              hipStream_t stream) {
  NINFER_REQUIRE(n_rows > 0 && H > 0, "rmsnorm: rows=%d H=%d must be positive", n_rows, H);
  NINFER_REQUIRE(dtype == kF32 || dtype == kBF16, "rmsnorm: unknown dtype %d", dtype);
  NINFER_REQUIRE(H <= 1024 * kNormPerThread, "rmsnorm: width %d exceeds %d", H,
                 1024 * kNormPerThread);
  NINFER_REQUIRE(!moe_y || (moe_w && moe_k > 0), "rmsnorm: a row sum needs weights and k");
  MoeSum ms{moe_y, moe_w, moe_shared, moe_gate, moe_gate_stride, moe_k};
  // groups of 4 consecutive elements when every row pointer stays 16-byte aligned
  auto aligned = [](const void* p) { return ((uintptr_t)p & 15) == 0; };
  const bool vec = H % 4 == 0 && aligned(x) && aligned(delta) && aligned(out) && aligned(gain) &&
                   aligned(moe_y) && aligned(moe_shared);
  // few elements per thread (short chains of loads), at most 1024 threads
  int per_thread = vec ? 4 : 2;
  int block = ((H + per_thread - 1) / per_thread + 63) / 64 * 64;
  if (block < 64) block = 64;
  if (block > 1024) block = 1024;
  if (dtype == kF32) {
    if (vec)
      rmsnorm_kernel<float, 4><<<n_rows, block, 0, stream>>>(x, (const float*)delta, ms, gain,
                                                            (float*)out, rows, H, eps);
    else
      rmsnorm_kernel<float, 1><<<n_rows, block, 0, stream>>>(x, (const float*)delta, ms, gain,
                                                            (float*)out, rows, H, eps);
  } else {
    if (vec)
      rmsnorm_kernel<bf16, 4><<<n_rows, block, 0, stream>>>(x, (const bf16*)delta, ms, gain,
                                                           (bf16*)out, rows, H, eps);
    else
      rmsnorm_kernel<bf16, 1><<<n_rows, block, 0, stream>>>(x, (const bf16*)delta, ms, gain,
                                                           (bf16*)out, rows, H, eps);
  }
  NINFER_LAUNCH_CHECK();
  return 0;
}

extern "C" int ninfer_rope_kv_write(void* qkv, const float* bias, const int* positions,
                                    const int* row_seq, const float* inv_freq, int rot_dim, int Hq,
                                    int Hkv, int D, void* kpool, void* vpool,
                                    const int* block_table, int bt_stride, int page_size,
                                    int write_kv, int interleaved, int T, int dtype,
                                    const float* q_gain, const float* k_gain, float norm_eps,
                                    hipStream_t stream) {
  NINFER_REQUIRE(T > 0, "rope_kv_write: T=%d must be positive", T);
  NINFER_REQUIRE((!q_gain) == (!k_gain), "rope_kv_write: the gains of the query heads' and of the key "
                 "heads' norm come together or not at all");
  NINFER_REQUIRE(D > 0 && D <= 1024, "rope_kv_write: head size %d not in [1,1024]", D);
  NINFER_REQUIRE(rot_dim >= 0 && rot_dim <= D && rot_dim % 2 == 0,
                 "rope_kv_write: rotary size %d must be even and <= head size %d", rot_dim, D);
  NINFER_REQUIRE(rot_dim == 0 || inv_freq, "rope_kv_write: rotary size %d without a table", rot_dim);
  NINFER_REQUIRE(dtype == kF32 || dtype == kBF16, "rope_kv_write: unknown dtype %d", dtype);
  NINFER_REQUIRE(page_size > 0 && bt_stride > 0, "rope_kv_write: bad page size or table width");
  if (q_gain) {
    // query and key heads normed before they turn: one wave per (row, head)
    NINFER_REQUIRE(norm_eps >= 0.f && norm_eps == norm_eps, "rope_kv_write: the norm's eps is not a number >= 0");
    const int heads = write_kv ? Hq + 2 * Hkv : Hq;
    const dim3 grid(T, (heads + 3) / 4);
    const size_t lds = 4 * (size_t)D * sizeof(float);
    if (dtype == kF32)
      rope_kv_write_normed_kernel<float><<<grid, 256, lds, stream>>>(
          (float*)qkv, bias, positions, row_seq, inv_freq, rot_dim, Hq, Hkv, D, (float*)kpool,
          (float*)vpool, block_table, bt_stride, page_size, write_kv, interleaved, q_gain, k_gain,
          norm_eps);
    else
      rope_kv_write_normed_kernel<bf16><<<grid, 256, lds, stream>>>(
          (bf16*)qkv, bias, positions, row_seq, inv_freq, rot_dim, Hq, Hkv, D, (bf16*)kpool,
          (bf16*)vpool, block_table, bt_stride, page_size, write_kv, interleaved, q_gain, k_gain,
          norm_eps);
    NINFER_LAUNCH_CHECK();
    return 0;
  }
  // many rows of a shape that takes 8-element accesses: one block per row, vectorised
  // (half-split pairs only: neighbouring pairs stay on the kernel of single items)
  const bool vec_ok = !interleaved && (rot_dim / 2) % 8 == 0 && (D - rot_dim) % 8 == 0 && D % 8 == 0 &&
                      ((uintptr_t)qkv % 32 == 0) && ((uintptr_t)kpool % 32 == 0) &&
                      ((uintptr_t)vpool % 32 == 0);
  if (T >= 256 && vec_ok) {
    const size_t lds = rot_dim * sizeof(float);
    if (dtype == kF32)
      rope_kv_write_rows_kernel<float><<<T, 256, lds, stream>>>(
          (float*)qkv, bias, positions, row_seq, inv_freq, rot_dim, Hq, Hkv, D, (float*)kpool,
          (float*)vpool, block_table, bt_stride, page_size, write_kv);
    else
      rope_kv_write_rows_kernel<bf16><<<T, 256, lds, stream>>>(
          (bf16*)qkv, bias, positions, row_seq, inv_freq, rot_dim, Hq, Hkv, D, (bf16*)kpool,
          (bf16*)vpool, block_table, bt_stride, page_size, write_kv);
    NINFER_LAUNCH_CHECK();
    return 0;
  }
  // few rows: spread a row's items over several blocks; many rows: one block per row
  int items = (Hq + 2 * Hkv) * (rot_dim / 2 + D - rot_dim);
  int per_row = T >= 256 ? 1 : (items + 255) / 256;
  dim3 grid(T, per_row);
  int block = 256;
  if (dtype == kF32)
    rope_kv_write_kernel<float><<<grid, block, 0, stream>>>(
        (float*)qkv, bias, positions, row_seq, inv_freq, rot_dim, Hq, Hkv, D, (float*)kpool,
        (float*)vpool, block_table, bt_stride, page_size, write_kv, interleaved);
  else
    rope_kv_write_kernel<bf16><<<grid, block, 0, stream>>>(
        (bf16*)qkv, bias, positions, row_seq, inv_freq, rot_dim, Hq, Hkv, D, (bf16*)kpool,
        (bf16*)vpool, block_table, bt_stride, page_size, write_kv, interleaved);
  NINFER_LAUNCH_CHECK();
  return 0;
}

extern "C" int ninfer_moe_combine(float* residual, const void* y, const float* w,
                                  const void* shared, const float* gate, int gate_stride, int T,
                                  int H, int k, int dtype, hipStream_t stream) {
  NINFER_REQUIRE(T > 0 && H > 0 && k > 0, "moe_combine: T=%d H=%d k=%d must be positive", T, H, k);
  NINFER_REQUIRE(dtype == kF32 || dtype == kBF16, "moe_combine: unknown dtype %d", dtype);
  if (dtype == kF32)
    moe_combine_kernel<float><<<dim3(T, (H + 255) / 256), 256, 0, stream>>>(residual, (const float*)y, w,
                                                    (const float*)shared, gate, gate_stride, H, k);
  else
    moe_combine_kernel<bf16><<<dim3(T, (H + 255) / 256), 256, 0, stream>>>(residual, (const bf16*)y, w,
                                                   (const bf16*)shared, gate, gate_stride, H, k);
  NINFER_LAUNCH_CHECK();
  return 0;
}

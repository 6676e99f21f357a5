// q, k, v = x Wqkv^T + b for few rows (decode), rotated and written where they
// belong, in one kernel: q (rotated) into the row's qkv buffer, k (rotated) and v
// into the pages of the row's request. Few-row steps otherwise pay a launch for
// the product and one for the rotation, each a chain of dependent loads.
//
// The product runs as in the few-row kernel (gemm_skinny.hip): weight rows are
// the A operand of v_mfma_f32_16x16x32_bf16, the K range is split over the
// waves of the block, partial tiles meet in LDS. What differs is which 16
// weight rows a block owns: up to 8 dims d0 .. d0 + P - 1 of one head and their
// rotation partners at + D / 2 (half-split pairs, reference
// src/ops/kernels.hip:86-91), so that the block's epilogue holds both elements
// of every pair it rotates. Angles, cosines and sines are 32-bit
// (pos * inv_freq[i], sincosf), as in the rotation kernel of elementwise.hip.
// The reference fuses rotation and cache write into its one-row GEMV the same
// way (src/ops/gemv.hip:271-324).
#include "gemm.h"

namespace ninfer {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

struct QkvRopeArgs {
  const void* x;          // [T, lda] normed rows (bf16)
  const void* w;          // [(Hq + 2 Hkv) D, K] (bf16)
  const float* bias;      // [(Hq + 2 Hkv) D] or null
  void* qkv;              // [T, (Hq + 2 Hkv) D]: only the q part is written
  const int* positions;   // [T]
  const int* row_seq;     // [T]
  const float* inv_freq;  // [D / 2]
  void* kpool;            // [pages, Hkv, page_size, D]
  void* vpool;
  const int* block_table; // [S, bt_stride]
  int T;
  int K;
  int lda;
  int Hq;
  int Hkv;
  int D;
  int bt_stride;
  int page_size;
  int write_kv;           // 0: a layer that reads another layer's cache writes q only
};

template <int WAVES>
__global__ __launch_bounds__(WAVES * 64) void qkv_rope_kernel(QkvRopeArgs a, int pairs) {
  __shared__ float red[WAVES][256];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, j = lane >> 4;
  const int D = a.D, half = D >> 1, K = a.K;
  const int per_head = half / pairs;               // blocks of a head
  const int head = blockIdx.x / per_head;
  const int d0 = (blockIdx.x % per_head) * pairs;
  const int row0 = blockIdx.y * 16;

  // weight row of lane r: pair r % 8 (if the block has that many), its low or high element
  const int pr = r & 7;
  const bool w_valid = pr < pairs;
  const int n = head * D + d0 + min(pr, pairs - 1) + (r >> 3) * half;
  const bf16* wrow = (const bf16*)a.w + (int64_t)n * K + 8 * j;
  const int mrow = row0 + r;
  const bool m_valid = mrow < a.T;
  const bf16* xrow = (const bf16*)a.x + (int64_t)(m_valid ? mrow : 0) * a.lda + 8 * j;

  // The same weight rows as the loads see them: whole 128-byte lines, lane l at row
  // 8 q + l / 8 (of the block's 16), byte 16 (l % 8) of a 128-byte piece; they reach the
  // operand's layout through 2 KB of LDS per wave (as in the few-row product kernel).
  const bf16* wline[2];
  bool line_valid[2];
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    const int R = 8 * q + (lane >> 3), p8 = R & 7;
    line_valid[q] = p8 < pairs;
    const int nn = head * D + d0 + min(p8, pairs - 1) + (R >> 3) * half;
    wline[q] = (const bf16*)a.w + (int64_t)nn * K + 8 * (lane & 7);
  }
  __shared__ __attribute__((aligned(16))) unsigned char stage[WAVES * 2048];
  unsigned char* my_stage = stage + wave * 2048;
  const int st_write = ((lane >> 3) * 128) + 16 * ((lane & 7) ^ ((lane >> 3) & 7));   // + 1024 q
  const int st_read = r * 128;   // + 16 * ((4 i + j) ^ (r % 8))

  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  // a wave's chunks of four steps lie side by side: it walks its part of every row in order
  const int steps = K / 32;
  const int chunks = (steps + 3) / 4, per_wave = (chunks + WAVES - 1) / WAVES;
  for (int c = wave * per_wave; c < min((wave + 1) * per_wave, chunks); ++c) {
    const int s0 = c * 4;
    if (s0 + 4 <= steps) {
      bf16x8 wl[2][2], x[4];   // [piece][q]
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int q = 0; q < 2; ++q)
          wl[h][q] = line_valid[q] ? stream_load((const bf16x8*)(wline[q] + s0 * 32 + h * 64)) : zero;
#pragma unroll
      for (int i = 0; i < 4; ++i) x[i] = m_valid ? *(const bf16x8*)(xrow + (s0 + i) * 32) : zero;
#pragma unroll
      for (int h = 0; h < 2; ++h) {
#pragma unroll
        for (int q = 0; q < 2; ++q) *(bf16x8*)(my_stage + st_write + 1024 * q) = wl[h][q];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          const bf16x8 wf = *(const bf16x8*)(my_stage + st_read + 16 * ((4 * i + j) ^ (r & 7)));
          acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf, x[2 * h + i], acc, 0, 0, 0);
        }
      }
    } else {
      for (int s = s0; s < steps; ++s) {
        bf16x8 w = w_valid ? *(const bf16x8*)(wrow + s * 32) : zero;
        bf16x8 x = m_valid ? *(const bf16x8*)(xrow + s * 32) : zero;
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w, x, acc, 0, 0, 0);
      }
    }
  }
  // partial tiles -> LDS, element (weight row f, token m) at [m * 16 + f]
#pragma unroll
  for (int v = 0; v < 4; ++v) red[wave][r * 16 + 4 * j + v] = acc[v];
  __syncthreads();

  // thread (m, p): pair p of row m
  if (threadIdx.x < 128) {
    const int m = threadIdx.x >> 3, p = threadIdx.x & 7;
    const int row = row0 + m;
    if (row < a.T && p < pairs) {
      float lo = 0.f, hi = 0.f;
#pragma unroll
      for (int w = 0; w < WAVES; ++w) {
        lo += red[w][m * 16 + p];
        hi += red[w][m * 16 + 8 + p];
      }
      const int d = d0 + p;
      if (a.bias) {
        lo += a.bias[head * D + d];
        hi += a.bias[head * D + d + half];
      }
      const int pos = a.positions[row];
      const bool is_q = head < a.Hq, is_k = !is_q && head < a.Hq + a.Hkv;
      if (is_q || is_k) {
        const float phi = (float)pos * a.inv_freq[d];
        float c, s;
        sincosf(phi, &s, &c);
        const float r0 = lo * c - hi * s, r1 = lo * s + hi * c;
        lo = r0;
        hi = r1;
      }
      bf16* dst;
      if (is_q) {
        dst = (bf16*)a.qkv + (int64_t)row * (a.Hq + 2 * a.Hkv) * D + head * D;
      } else {
        const int page = a.block_table[(int64_t)a.row_seq[row] * a.bt_stride + pos / a.page_size];
        const int kvh = is_k ? head - a.Hq : head - a.Hq - a.Hkv;
        dst = (bf16*)(is_k ? a.kpool : a.vpool) +
              (((int64_t)page * a.Hkv + kvh) * a.page_size + pos % a.page_size) * D;
      }
      dst[d] = from_f32<bf16>(lo);
      dst[d + half] = from_f32<bf16>(hi);
    }
  }
}

}  // namespace ninfer

using namespace ninfer;

// Shapes the fused kernel takes (bf16 only; the caller keeps other cases on the two
// separate kernels): full rotation of heads whose size is a multiple of 16, K a multiple
// of 32, 16-byte aligned rows.
extern "C" int ninfer_qkv_rope_takes(int T, int K, int lda, int D, int rot_dim) {
  return T >= 1 && T <= 32 && rot_dim == D && D % 16 == 0 && K % 32 == 0 && lda % 8 == 0;
}

extern "C" int ninfer_qkv_rope(const QkvRopeArgs* args, hipStream_t stream) {
  const QkvRopeArgs& a = *args;
  NINFER_REQUIRE(ninfer_qkv_rope_takes(a.T, a.K, a.lda, a.D, a.D),
                 "qkv_rope: %d rows of width %d (row stride %d), heads of %d are not taken", a.T,
                 a.K, a.lda, a.D);
  NINFER_REQUIRE(a.Hq > 0 && a.Hkv > 0 && a.page_size > 0 && a.bt_stride > 0,
                 "qkv_rope: bad head counts, page size or table width");
  NINFER_REQUIRE(((uintptr_t)a.x % 16 == 0) && ((uintptr_t)a.w % 16 == 0),
                 "qkv_rope: operands must be 16-byte aligned");
  const int heads = a.write_kv ? a.Hq + 2 * a.Hkv : a.Hq;
  const int m_tiles = (a.T + 15) / 16;
  const long total_pairs = (long)heads * (a.D / 2);
  // eight pairs per block, whole tiles of the matrix instruction: blocks of fewer pairs would
  // spread more evenly over the CUs but measured slower (each re-reads the rows of x)
  const int pairs = 8;
  const long blocks = total_pairs / pairs;
  NINFER_REQUIRE(blocks < (1L << 31), "qkv_rope: %ld blocks are too many", blocks);
  dim3 grid((unsigned)blocks, m_tiles);
  const int chunks = a.K / 128;
  const int cus = device_cu_count();
  if (blocks * m_tiles < 2 * cus && chunks >= 16)
    qkv_rope_kernel<16><<<grid, 16 * 64, 0, stream>>>(a, pairs);
  else if (blocks * m_tiles < 8 * cus && chunks >= 8)
    qkv_rope_kernel<8><<<grid, 8 * 64, 0, stream>>>(a, pairs);
  else
    qkv_rope_kernel<4><<<grid, 4 * 64, 0, stream>>>(a, pairs);
  NINFER_LAUNCH_CHECK();
  return 0;
}

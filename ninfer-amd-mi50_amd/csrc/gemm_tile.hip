// C = A W^T for many rows (prompt portions) on the matrix cores: dense, or
// grouped by expert with one launch for all experts, with a bias or a SwiGLU
// epilogue. bf16 inputs, 32-bit accumulation, bf16 or 32-bit output.
//
// A block of 4 waves owns 64 rows of A (sorted rows of one expert in the
// grouped form) and 256 rows of W: each wave 64 x 64 as 2 x 2 tiles of
// v_mfma_f32_32x32x16_bf16. W rows are the A operand (lane l: row l % 32,
// k = 8 (l / 32) .. +7), activation rows the B operand, so a lane's accumulator
// holds, for token l % 32, four consecutive output features per register
// quad: C^T[feature 8 (v / 4) + 4 (l / 32) + v % 4][token l % 32]. With the
// SwiGLU epilogue a wave's 64 W rows are 32 gate rows and their 32 up rows, so
// silu(g) * u is formed in registers and the block writes 128 output features.
// Tiles go global -> registers -> LDS with the next tile's loads in flight
// during the products (two LDS buffers, one barrier per 32-wide k step).
// The reference sends these products to rocBLAS, one call per expert
// (src/models/model.hip:406-425, src/ops/linear.hip:21-35).
#include "gemm.h"

namespace ninfer {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int TM = 64;         // rows of A per block
constexpr int TN = 256;        // rows of W per block
constexpr int TK = 32;
constexpr int TPAD = TK + 8;   // bf16 per LDS row

template <bool SWIGLU, typename TC>
__global__ __launch_bounds__(256) void gemm_tile_kernel(GemmArgs a) {
  __shared__ __attribute__((aligned(16))) bf16 xs[2][TM * TPAD];
  __shared__ __attribute__((aligned(16))) bf16 ws[2][TN * TPAD];
  __shared__ int tile_info[3];

  int row0, row_end, group = 0;
  if (a.offsets) {
    if (!grouped_tile(a, a.tiles64, 1, TM, blockIdx.x, tile_info)) return;
    __syncthreads();
    group = tile_info[2];
    row0 = tile_info[0];
    row_end = tile_info[1];
  } else {
    row0 = blockIdx.x * TM;
    row_end = a.M;
    if (row0 >= row_end) return;
  }
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int K = a.K, N = a.N;
  const bf16* W = (const bf16*)a.W + (int64_t)group * a.w_group_stride;
  const int out0 = blockIdx.y * (SWIGLU ? TN / 2 : TN);   // first output feature of the block

  // which W row does LDS row r (0..255) hold?
  auto w_row_of = [&](int r) -> int {
    if (SWIGLU) {
      int w = r >> 6, i = r & 63;                 // wave, row within the wave's 64
      int f = min(out0 + 32 * w + (i & 31), N - 1);
      return i < 32 ? f : f + N;
    }
    return min(out0 + r, N - 1);
  };

  // global -> register staging: 1 vector of A, 4 of W per thread and k tile
  const int xr = tid >> 2, kv = tid & 3;
  const bf16* xsrc = nullptr;
  if (row0 + xr < row_end) {
    int64_t ar = a.a_index ? a.a_index[row0 + xr] / a.a_div : row0 + xr;
    xsrc = (const bf16*)a.A + ar * a.lda + 8 * kv;
  }
  const bf16* wsrc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) wsrc[i] = W + (int64_t)w_row_of(xr + 64 * i) * K + 8 * kv;

  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  bf16x8 xreg, wreg[4];
  auto load_tile = [&](int k0) {
    xreg = xsrc ? *(const bf16x8*)(xsrc + k0) : zero;
#pragma unroll
    for (int i = 0; i < 4; ++i) wreg[i] = *(const bf16x8*)(wsrc[i] + k0);
  };
  auto store_tile = [&](int buf) {
    *(bf16x8*)(xs[buf] + xr * TPAD + 8 * kv) = xreg;
#pragma unroll
    for (int i = 0; i < 4; ++i) *(bf16x8*)(ws[buf] + (xr + 64 * i) * TPAD + 8 * kv) = wreg[i];
  };

  f32x16 acc[2][2];   // [W 32-row block][token 32-row block]
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int jj = 0; jj < 2; ++jj)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][jj][v] = 0.f;

  const int lr = lane & 31, lk = lane >> 5;
  const int nk = K / TK;
  load_tile(0);
  store_tile(0);
  __syncthreads();
  for (int kt = 0; kt < nk; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < nk) load_tile((kt + 1) * TK);
#pragma unroll
    for (int kk = 0; kk < TK / 16; ++kk) {
      bf16x8 wf[2], xf[2];
#pragma unroll
      for (int i = 0; i < 2; ++i)
        wf[i] = *(const bf16x8*)(ws[buf] + (wave * 64 + 32 * i + lr) * TPAD + 16 * kk + 8 * lk);
#pragma unroll
      for (int jj = 0; jj < 2; ++jj)
        xf[jj] = *(const bf16x8*)(xs[buf] + (32 * jj + lr) * TPAD + 16 * kk + 8 * lk);
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int jj = 0; jj < 2; ++jj)
          acc[i][jj] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[i], xf[jj], acc[i][jj], 0, 0, 0);
    }
    if (kt + 1 < nk) store_tile(buf ^ 1);
    __syncthreads();
  }

  // epilogue: lane holds token 32 jj + lr; features 32 i + 8 q + 4 lk + r (q = v / 4, r = v % 4)
  TC* C = (TC*)a.C;
#pragma unroll
  for (int jj = 0; jj < 2; ++jj) {
    const int row = row0 + 32 * jj + lr;
    if (row >= row_end) continue;
    const int64_t c_row = a.c_index ? a.c_index[row] : row;
    TC* crow = C + c_row * a.ldc;
    if (SWIGLU) {
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          int f = out0 + 32 * wave + 8 * q + 4 * lk + r;
          if (f < N) {
            float g = acc[0][jj][4 * q + r], u = acc[1][jj][4 * q + r];
            crow[f] = from_f32<TC>(g / (1.f + __expf(-g)) * u);
          }
        }
    } else {
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            int f = out0 + 64 * wave + 32 * i + 8 * q + 4 * lk + r;
            if (f < N) {
              float v = acc[i][jj][4 * q + r];
              if (a.bias) v += a.bias[f];
              crow[f] = from_f32<TC>(v);
            }
          }
    }
  }
}

bool gemm_tile_takes(const GemmArgs& a) {
  return a.in_dtype == kBF16 && a.K % TK == 0 && a.lda % 8 == 0 && ((uintptr_t)a.A % 16 == 0) &&
         ((uintptr_t)a.W % 16 == 0) && a.w_group_stride % 8 == 0;
}

int gemm_tile(const GemmArgs& a, hipStream_t stream) {
  bool swiglu = a.epilogue == kEpilogueSwiGLU;
  int m_tiles = (a.M + TM - 1) / TM + (a.offsets ? a.groups : 0);
  int per_block = swiglu ? TN / 2 : TN;
  dim3 grid(m_tiles, (a.N + per_block - 1) / per_block);
  if (a.out_dtype == kF32) {
    if (swiglu)
      gemm_tile_kernel<true, float><<<grid, 256, 0, stream>>>(a);
    else
      gemm_tile_kernel<false, float><<<grid, 256, 0, stream>>>(a);
  } else {
    if (swiglu)
      gemm_tile_kernel<true, bf16><<<grid, 256, 0, stream>>>(a);
    else
      gemm_tile_kernel<false, bf16><<<grid, 256, 0, stream>>>(a);
  }
  NINFER_LAUNCH_CHECK();
  return 0;
}

}  // namespace ninfer

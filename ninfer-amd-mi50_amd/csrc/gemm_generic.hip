// C = A W^T (+ bias), optionally grouped by expert and with a SwiGLU epilogue:
// the plain tiled kernel of the product family. 32-bit accumulation by FMA in
// a fixed order (k ascending) for every output element, whatever M is and
// wherever the row sits in its tile, so a row's result does not depend on the
// batch it came in. This is the kernel of the true 32-bit path and the
// fallback of the bf16 path for shapes its MFMA kernels refuse.
//
// Linear weights are [out, in] row-major, y = x W^T, as in the reference
// (src/ops/ops.h:16-18). Grouped form: sorted row r belongs to the expert g
// with offsets[g] <= r < offsets[g+1]; it reads row a_index[r] / a_div of A
// and writes row c_index[r] of C (identity when the index is null). The
// reference loops experts on the host with one library call each
// (src/models/model.hip:355-427).
#include "gemm.h"

namespace ninfer {

constexpr int BM = 64, BN = 64, BK = 16;

template <typename T, typename TC, bool SWIGLU>
__global__ __launch_bounds__(256) void gemm_generic_kernel(GemmArgs a) {
  __shared__ float As[BK][BM + 4];
  __shared__ float Ws[BK][BN + 4];
  __shared__ float Us[SWIGLU ? BK : 1][BN + 4];
  __shared__ int tile_info[3];

  // which rows: dense, or the tile `blockIdx.y` of the grouped enumeration
  int row0, row_end, group = 0;
  if (a.offsets) {
    if (!find_tile(a.offsets, a.groups, BM, blockIdx.y, tile_info)) return;
    group = tile_info[2];
    row0 = tile_info[0];
    row_end = tile_info[1];
  } else {
    row0 = blockIdx.y * BM;
    row_end = a.M;
    if (row0 >= row_end) return;
  }
  const int n0 = blockIdx.x * BN;
  const T* A = (const T*)a.A;
  const T* W = (const T*)a.W + (int64_t)group * a.w_group_stride;
  const int tid = threadIdx.x;
  const int tx = tid & 15, ty = tid >> 4;

  // each thread loads 4 elements of the A tile and 4 of the W tile per k-step
  const int lrow = tid >> 2;        // 0..63
  const int lk = (tid & 3) * 4;     // 0,4,8,12
  int64_t a_row = -1;
  {
    int r = row0 + lrow;
    if (r < row_end) a_row = a.a_index ? a.a_index[r] / a.a_div : r;
  }
  const int w_row = n0 + lrow;

  float acc[4][4] = {};
  float accu[SWIGLU ? 4 : 1][4] = {};

  for (int k0 = 0; k0 < a.K; k0 += BK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      int k = k0 + lk + i;
      float av = 0.f, wv = 0.f, uv = 0.f;
      if (k < a.K) {
        if (a_row >= 0) av = to_f32(A[a_row * a.lda + k]);
        if (w_row < a.N) {
          wv = to_f32(W[(int64_t)w_row * a.K + k]);
          if (SWIGLU) uv = to_f32(W[(int64_t)(w_row + a.N) * a.K + k]);
        }
      }
      As[lk + i][lrow] = av;
      Ws[lk + i][lrow] = wv;
      if (SWIGLU) Us[lk + i][lrow] = uv;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < BK; ++k) {
      float av[4], wv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = As[k][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) wv[j] = Ws[k][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
      if (SWIGLU) {
        float uv[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) uv[j] = Us[k][tx * 4 + j];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j) accu[i][j] = fmaf(av[i], uv[j], accu[i][j]);
      }
    }
    __syncthreads();
  }

  TC* C = (TC*)a.C;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    int r = row0 + ty * 4 + i;
    if (r >= row_end) continue;
    int64_t c_row = a.c_index ? a.c_index[r] : r;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      int n = n0 + tx * 4 + j;
      if (n >= a.N) continue;
      float v = acc[i][j];
      if (SWIGLU) {
        float g = v + (a.bias ? a.bias[n] : 0.f);
        const float u = accu[i][j] + (a.bias ? a.bias[a.N + n] : 0.f);
        v = g / (1.f + expf(-gate_logit(g, a.epilogue == kEpilogueGeGLU))) * u;
      } else if (a.bias) {
        v += a.bias[n];
      }
      C[c_row * a.ldc + n] = from_f32<TC>(v);
    }
  }
}

template <typename T, typename TC>
static void launch(const GemmArgs& a, hipStream_t stream) {
  int m_tiles = (a.M + BM - 1) / BM + (a.offsets ? a.groups : 0);
  dim3 grid((a.N + BN - 1) / BN, m_tiles);
  if (epilogue_gated(a.epilogue))
    gemm_generic_kernel<T, TC, true><<<grid, 256, 0, stream>>>(a);
  else
    gemm_generic_kernel<T, TC, false><<<grid, 256, 0, stream>>>(a);
}

int gemm_check(const GemmArgs& a) {
  NINFER_REQUIRE(a.M > 0 && a.N > 0 && a.K > 0, "gemm: M=%d N=%d K=%d must be positive", a.M, a.N,
                 a.K);
  NINFER_REQUIRE(a.in_dtype == kF32 || a.in_dtype == kBF16, "gemm: unknown input dtype %d",
                 a.in_dtype);
  NINFER_REQUIRE(a.out_dtype == kF32 || a.out_dtype == kBF16, "gemm: unknown output dtype %d",
                 a.out_dtype);
  NINFER_REQUIRE(!(a.in_dtype == kF32 && a.out_dtype == kBF16),
                 "gemm: 32-bit inputs with a bfloat16 output are not supported");
  NINFER_REQUIRE(a.lda >= a.K && a.ldc >= a.N, "gemm: lda=%d < K=%d or ldc=%d < N=%d", a.lda, a.K,
                 a.ldc, a.N);
  NINFER_REQUIRE(a.groups >= 1, "gemm: groups=%d must be >= 1", a.groups);
  NINFER_REQUIRE(a.offsets || a.groups == 1, "gemm: %d groups without offsets", a.groups);
  NINFER_REQUIRE(!a.a_index || a.a_div >= 1, "gemm: a_div=%d must be >= 1", a.a_div);
  NINFER_REQUIRE(a.epilogue == kEpilogueNone || epilogue_gated(a.epilogue),
                 "gemm: unknown epilogue %d", a.epilogue);
  NINFER_REQUIRE(!(epilogue_gated(a.epilogue) && a.bias && a.offsets),
                 "gemm: a grouped product with a gated epilogue takes no bias");
  NINFER_REQUIRE(a.k_parts <= 1, "gemm: k_parts is set by the library, not by callers");
  NINFER_REQUIRE(!a.workspace || a.workspace_floats > 0, "gemm: a workspace of %ld floats",
                 (long)a.workspace_floats);
  return 0;
}

int gemm_generic(const GemmArgs& a, hipStream_t stream) {
  if (a.in_dtype == kF32) {
    launch<float, float>(a, stream);
  } else if (a.out_dtype == kF32) {
    launch<bf16, float>(a, stream);
  } else {
    launch<bf16, bf16>(a, stream);
  }
  NINFER_LAUNCH_CHECK();
  return 0;
}

}  // namespace ninfer

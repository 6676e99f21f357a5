// C = A W^T for many rows (prompt portions) on the matrix cores: dense, or
// grouped by expert with one launch for all experts, with a bias or a SwiGLU
// epilogue. bf16 inputs, 32-bit accumulation, bf16 or 32-bit output.
//
// A block of 4 waves owns TM rows of A (sorted rows of one expert in the
// grouped form) and TN rows of W; the waves form a WGM x WGN grid, each with
// FI x FJ tiles of v_mfma_f32_32x32x16_bf16. W rows are the A operand (lane l:
// row l % 32, k = 8 (l / 32) .. +7), activation rows the B operand, so a lane's
// accumulator holds, for token l % 32, four consecutive output features per
// register quad: C^T[feature 8 (v / 4) + 4 (l / 32) + v % 4][token l % 32].
// With the SwiGLU epilogue the first half of a wave's W rows are gate rows and
// the second half their up rows, so silu(g) * u is formed in registers and the
// block writes TN / 2 output features. Tiles go global -> registers -> LDS with
// the next tile's loads in flight during the products (two LDS buffers, one
// barrier per k step of TK). 32-row blocks of tokens beyond the tile's last row
// are skipped. The reference sends these products to rocBLAS, one call per
// expert (src/models/model.hip:406-425, src/ops/linear.hip:21-35).
#include "gemm.h"
#include <type_traits>

namespace ninfer {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

template <int TM, int TN, int TK, int WGM, int P, bool SWIGLU, typename TC>
__global__ __launch_bounds__(256) void gemm_tile_kernel(GemmArgs a) {
  constexpr int WGN = 4 / WGM;
  constexpr int FI = TN / WGM / 32;      // 32-row blocks of W per wave
  constexpr int FJ = TM / WGN / 32;      // 32-row blocks of tokens per wave
  constexpr int TPAD = TK + 8;           // bf16 per LDS row
  constexpr int VPR = TK / 8;            // 16-byte vectors per row and k tile
  constexpr int XV = TM * VPR / 256;     // vectors of A per thread and k tile
  constexpr int WV = TN * VPR / 256;     // vectors of W per thread and k tile
  static_assert(FI >= 1 && FJ >= 1 && XV >= 1 && WV >= 1, "tile too small for the block");
  static_assert(!SWIGLU || FI % 2 == 0, "SwiGLU needs gate and up rows in every wave");
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  bf16* xs = (bf16*)smem;                       // [2][TM * TPAD]
  bf16* ws = xs + 2 * TM * TPAD;                // [2][TN * TPAD]
  __shared__ int tile_info[3];

  // Which tile? Blocks go to the 8 XCDs in turn (block id mod 8), and each XCD
  // has its own L2: block ids that are congruent mod 8 get neighbouring work,
  // and work is ordered so that neighbours share their W tile (the row tiles of
  // one expert, four at a time) and then their rows of A.
  int bx, by;
  {
    const int total = gridDim.x * gridDim.y;
    const int id = blockIdx.x + gridDim.x * blockIdx.y;
    // ids congruent to x mod 8 number total / 8 (one more for x < total % 8): a bijection
    const int x = id % 8, q = total / 8, rem8 = total % 8;
    const int w = x * q + min(x, rem8) + id / 8;
    const int nt = gridDim.y, mt = gridDim.x;
    const int chunk = w / (4 * nt), rem = w % (4 * nt);
    const int full = mt / 4;   // chunks of four row tiles; the rest is walked one by one
    if (chunk < full) {
      by = rem / 4;
      bx = chunk * 4 + rem % 4;
    } else {
      const int w2 = w - full * 4 * nt, left = mt - full * 4;
      by = w2 / left;
      bx = full * 4 + w2 % left;
    }
  }
  int row0, row_end, group = 0;
  if (a.offsets) {
    if (!grouped_tile(a, a.tiles64, 1, TM, bx, tile_info)) return;
    __syncthreads();
    group = tile_info[2];
    row0 = tile_info[0];
    row_end = tile_info[1];
  } else {
    row0 = bx * TM;
    row_end = a.M;
    if (row0 >= row_end) return;
  }
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave % WGM, wn = wave / WGM;
  const int K = a.K, N = a.N;
  const bf16* W = (const bf16*)a.W + (int64_t)group * a.w_group_stride;
  constexpr int OUT_PER_BLOCK = SWIGLU ? TN / 2 : TN;
  constexpr int OUT_PER_WAVE = OUT_PER_BLOCK / WGM;
  const int out0 = by * OUT_PER_BLOCK;

  // which W row does LDS row r (0 .. TN-1) hold? LDS rows are grouped by wave.
  auto w_row_of = [&](int r) -> int {
    int w = r / (TN / WGM), i = r % (TN / WGM);
    if (SWIGLU) {
      int f = min(out0 + OUT_PER_WAVE * w + i % OUT_PER_WAVE, N - 1);
      return i < OUT_PER_WAVE ? f : f + N;
    }
    return min(out0 + OUT_PER_WAVE * w + i, N - 1);
  };

  const bf16* xsrc[XV];
  const bf16* wsrc[WV];
#pragma unroll
  for (int i = 0; i < XV; ++i) {
    int v = tid + i * 256, r = v / VPR, kv = v % VPR;
    // rows beyond the tile's last read its first row: their results are never stored
    int rr = row0 + r < row_end ? row0 + r : row0;
    int64_t ar = a.a_index ? a.a_index[rr] / a.a_div : rr;
    xsrc[i] = (const bf16*)a.A + ar * a.lda + 8 * kv;
  }
#pragma unroll
  for (int i = 0; i < WV; ++i) {
    int v = tid + i * 256, r = v / VPR, kv = v % VPR;
    wsrc[i] = W + (int64_t)w_row_of(r) * K + 8 * kv;
  }
  // P register stages: the loads of k tile t + P are issued while tile t is multiplied
  bf16x8 xreg[P][XV], wreg[P][WV];
  auto load_tile = [&](int st, int k0) {
#pragma unroll
    for (int i = 0; i < XV; ++i) xreg[st][i] = *(const bf16x8*)(xsrc[i] + k0);
#pragma unroll
    for (int i = 0; i < WV; ++i) wreg[st][i] = *(const bf16x8*)(wsrc[i] + k0);
  };
  auto store_tile = [&](int st, int buf) {
#pragma unroll
    for (int i = 0; i < XV; ++i) {
      int v = tid + i * 256;
      *(bf16x8*)(xs + buf * TM * TPAD + (v / VPR) * TPAD + 8 * (v % VPR)) = xreg[st][i];
    }
#pragma unroll
    for (int i = 0; i < WV; ++i) {
      int v = tid + i * 256;
      *(bf16x8*)(ws + buf * TN * TPAD + (v / VPR) * TPAD + 8 * (v % VPR)) = wreg[st][i];
    }
  };

  f32x16 acc[FI][FJ];
#pragma unroll
  for (int i = 0; i < FI; ++i)
#pragma unroll
    for (int jj = 0; jj < FJ; ++jj)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][jj][v] = 0.f;

  // token blocks of this wave that hold at least one row
  const int rows_here = min(TM, row_end - row0);
  const int tok0 = wn * (TM / WGN);
  int n_jj = 0;
#pragma unroll
  for (int jj = 0; jj < FJ; ++jj)
    if (tok0 + 32 * jj < rows_here) n_jj = jj + 1;

  const int lr = lane & 31, lk = lane >> 5;
  const int nk = K / TK;
  // products of one k tile from LDS buffer `buf`; NJ token blocks are live (a
  // compile-time count, so the loop body is straight-line code)
  auto multiply = [&](int buf, auto nj_tag) {
    constexpr int NJ = decltype(nj_tag)::value;
    if constexpr (NJ == 0) return;   // a wave without rows still loads, stores and meets barriers
    const bf16* xb = xs + buf * TM * TPAD;
    const bf16* wb = ws + buf * TN * TPAD;
#pragma unroll
    for (int kk = 0; kk < TK / 16; ++kk) {
      bf16x8 wf[FI], xf[NJ > 0 ? NJ : 1];
#pragma unroll
      for (int i = 0; i < FI; ++i)
        wf[i] = *(const bf16x8*)(wb + (wm * (TN / WGM) + 32 * i + lr) * TPAD + 16 * kk + 8 * lk);
#pragma unroll
      for (int jj = 0; jj < NJ; ++jj)
        xf[jj] = *(const bf16x8*)(xb + (tok0 + 32 * jj + lr) * TPAD + 16 * kk + 8 * lk);
#pragma unroll
      for (int jj = 0; jj < NJ; ++jj)
#pragma unroll
        for (int i = 0; i < FI; ++i)
          acc[i][jj] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[i], xf[jj], acc[i][jj], 0, 0, 0);
    }
  };
  // The k loop, unrolled by the P register stages so that every stage index is
  // a constant and no load sits under a condition: the compiler can then wait
  // for exactly the loads a store needs. Tile t is in LDS buffer t & 1 and was
  // loaded into stage t % P; while tile t is multiplied, tile t + P is loaded
  // into that stage and tile t + 1 moves from its stage to the other buffer.
  auto run = [&](auto nj_tag) {
#pragma unroll
    for (int st = 0; st < P; ++st) load_tile(st, st * TK);
    store_tile(0, 0);
    lds_barrier();
    int kt0 = 0;
    for (; kt0 + 2 * P <= nk; kt0 += P) {
#pragma unroll
      for (int st = 0; st < P; ++st) {
        const int kt = kt0 + st;
        load_tile(st, (kt + P) * TK);
        __builtin_amdgcn_sched_barrier(0);   // keep these loads ahead of the products
        multiply(kt & 1, nj_tag);
        __builtin_amdgcn_sched_barrier(0);
        store_tile((st + 1) % P, (kt & 1) ^ 1);
        lds_barrier();
      }
    }
#pragma unroll
    for (int st = 0; st < P; ++st) {   // the last P tiles: nothing left to load
      const int kt = kt0 + st;
      multiply(kt & 1, nj_tag);
      if (st + 1 < P) store_tile(st + 1, (kt & 1) ^ 1);
      lds_barrier();
    }
  };
  if (n_jj == FJ) {
    run(std::integral_constant<int, FJ>{});
  } else if (n_jj == 0) {
    run(std::integral_constant<int, 0>{});
  } else if (FJ > 1 && n_jj == 1) {
    run(std::integral_constant<int, 1>{});
  } else {
    run(std::integral_constant<int, FJ>{});
  }

  // epilogue: lane holds token tok0 + 32 jj + lr; features 8 q + 4 lk + r of each 32-row block
  TC* C = (TC*)a.C;
#pragma unroll
  for (int jj = 0; jj < FJ; ++jj) {
    const int row = row0 + tok0 + 32 * jj + lr;
    if (row >= row_end || tok0 + 32 * jj + lr >= TM) continue;
    const int64_t c_row = a.c_index ? a.c_index[row] : row;
    TC* crow = C + c_row * a.ldc;
    if (SWIGLU) {
#pragma unroll
      for (int i = 0; i < FI / 2; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            int f = out0 + OUT_PER_WAVE * wm + 32 * i + 8 * q + 4 * lk + r;
            if (f < N) {
              float g = acc[i][jj][4 * q + r], u = acc[i + (SWIGLU ? FI / 2 : 0)][jj][4 * q + r];
              crow[f] = from_f32<TC>(g / (1.f + __expf(-g)) * u);
            }
          }
    } else {
#pragma unroll
      for (int i = 0; i < FI; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            int f = out0 + OUT_PER_WAVE * wm + 32 * i + 8 * q + 4 * lk + r;
            if (f < N) {
              float v = acc[i][jj][4 * q + r];
              if (a.bias) v += a.bias[f];
              crow[f] = from_f32<TC>(v);
            }
          }
    }
  }
}

// K must be a whole number of pipeline rounds (2 k tiles of 64) and at least two.
bool gemm_tile_takes(const GemmArgs& a) {
  return a.in_dtype == kBF16 && a.K % 128 == 0 && a.K >= 256 && a.lda % 8 == 0 && ((uintptr_t)a.A % 16 == 0) &&
         ((uintptr_t)a.W % 16 == 0) && a.w_group_stride % 8 == 0;
}

static int g_tile_variant = 0;   // tests: 0 = choose by shape

template <int TM, int TN, int TK, int WGM, int P>
static int launch_tile(const GemmArgs& a, hipStream_t stream) {
  if (a.offsets && a.tiles64 && TM != (a.big_rows ? a.big_rows : 64))
    return set_error(-1, "gemm: the grouped tile lists are made for %d rows, not %d", a.big_rows, TM);
  const bool swiglu = a.epilogue == kEpilogueSwiGLU;
  const int m_tiles = (a.M + TM - 1) / TM + (a.offsets ? a.groups : 0);
  const int per_block = swiglu ? TN / 2 : TN;
  const dim3 grid(m_tiles, (a.N + per_block - 1) / per_block);
  const size_t lds = 2 * (TM + TN) * (TK + 8) * sizeof(bf16);
#define NINFER_TILE_LAUNCH(SW, TYPE)                                                        \
  do {                                                                                      \
    auto kern = gemm_tile_kernel<TM, TN, TK, WGM, P, SW, TYPE>;                               \
    if (lds > 48 * 1024) {                                                                  \
      hipError_t e = hipFuncSetAttribute((const void*)kern,                                 \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, lds);  \
      if (e != hipSuccess) return set_error(-2, "gemm: cannot get %zu bytes of LDS", lds);  \
    }                                                                                       \
    kern<<<grid, 256, lds, stream>>>(a);                                                    \
  } while (0)
  if (a.out_dtype == kF32) {
    if (swiglu) NINFER_TILE_LAUNCH(true, float); else NINFER_TILE_LAUNCH(false, float);
  } else {
    if (swiglu) NINFER_TILE_LAUNCH(true, bf16); else NINFER_TILE_LAUNCH(false, bf16);
  }
#undef NINFER_TILE_LAUNCH
  NINFER_LAUNCH_CHECK();
  return 0;
}

int gemm_tile(const GemmArgs& a, hipStream_t stream) {
  // 128-row tiles when there are rows to fill them: twice the work per weight read.
  // g_tile_variant (tests): 1 forces 64-row tiles, 2 forces 128-row tiles on dense products.
  bool big = a.offsets ? a.big_rows == 128 : a.M >= 256;
  if (!a.offsets && g_tile_variant == 1) big = false;
  if (!a.offsets && g_tile_variant == 2) big = true;
  if (big) return launch_tile<128, 128, 64, 2, 2>(a, stream);
  return launch_tile<64, 128, 64, 2, 2>(a, stream);
}

}  // namespace ninfer

extern "C" void ninfer_set_tile_variant(int v) { ninfer::g_tile_variant = v; }

// What the many-row product kernels share: the map from block ids to tiles,
// the W rows a block stages, and the epilogue that writes a wave's accumulators.
#pragma once
#include "gemm.h"
#include <type_traits>

namespace ninfer {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

// Which tile does this block work on? bx: row tile (0 .. gridDim.x - 1), by: tile
// of output features.
// Dense: blocks go to the 8 XCDs in turn (block id mod 8), and each XCD has its
// own L2: block ids that are congruent mod 8 get neighbouring work, and work is
// ordered so that neighbours share their W tile (four row tiles at a time) and
// then their rows of A.
// Grouped: the blocks that an XCD runs at the same time are the feature tiles of
// few experts (row tile x + 8 i for XCD x, its feature tiles side by side), so
// that an expert's rows of A are fetched into that L2 once and found there by
// the other feature tiles; every (expert, feature tile) panel of W is read by
// one block and streams from HBM whatever the order. The launcher rounds the
// row tiles up to a multiple of 8, which makes this a bijection.
__device__ inline void block_to_tile(bool grouped, int& bx, int& by) {
  if (grouped) {
    const int id = blockIdx.x + gridDim.x * blockIdx.y;
    const int x = id % kXcds, slot = id / kXcds;
    bx = x + kXcds * (slot / (int)gridDim.y);
    by = slot % (int)gridDim.y;
    return;
  }
  const int total = gridDim.x * gridDim.y;
  const int id = blockIdx.x + gridDim.x * blockIdx.y;
  // ids congruent to x mod 8 number total / 8 (one more for x < total % 8): a bijection
  const int x = id % kXcds, q = total / kXcds, rem8 = total % kXcds;
  const int w = x * q + min(x, rem8) + id / kXcds;
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

// The rows of A of tile bx: {first row, end of the rows it may take}, and the
// group whose weights it meets. False when the tile does not exist. `info` is
// 3 ints of LDS.
template <int TM>
__device__ inline bool tile_rows(const GemmArgs& a, int bx, int* info, int& row0, int& row_end,
                                 int& group) {
  group = 0;
  if (a.offsets) {
    // the tile list is made for the tall tiles; other heights count their tiles from the offsets
    if (!grouped_tile(a, TM == kGroupedTileRows ? a.tiles_big : nullptr, 1, TM, bx, info))
      return false;
    __syncthreads();
    group = info[2];
    row0 = info[0];
    row_end = info[1];
    return true;
  }
  row0 = bx * TM;
  row_end = a.M;
  return row0 < row_end;
}

// Which W row does staged row r (0 .. TN-1) of a block hold? Staged rows are
// grouped by wave row (WGM of them, TN / WGM each); with the SwiGLU epilogue
// the first half of a wave's rows are gate rows and the second half their up
// rows. Rows beyond N repeat row N - 1 and are never stored.
template <int TN, int WGM, bool SWIGLU>
__device__ inline int staged_w_row(int r, int out0, int N) {
  constexpr int PER_WAVE = TN / WGM;
  constexpr int OUT_PER_WAVE = SWIGLU ? PER_WAVE / 2 : PER_WAVE;
  const int w = r / PER_WAVE, i = r % PER_WAVE;
  if (SWIGLU) {
    const int f = min(out0 + OUT_PER_WAVE * w + i % OUT_PER_WAVE, N - 1);
    return i < OUT_PER_WAVE ? f : f + N;
  }
  return min(out0 + OUT_PER_WAVE * w + i, N - 1);
}

// act(g) * u with the hardware's reciprocal (1 ulp) in place of an IEEE division: a tile's
// epilogue forms 128 of them per lane, and the division is ten instructions each.
__device__ __forceinline__ float gated_times(float g, float u, bool gelu) {
  return g * __builtin_amdgcn_rcpf(1.f + __expf(-gate_logit(g, gelu))) * u;
}

__device__ inline void store_quad(float* p, const float (&v)[4]) {
  *(float4*)p = make_float4(v[0], v[1], v[2], v[3]);
}
__device__ inline void store_quad(bf16* p, const float (&v)[4]) {
  typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
  *(bf16x4*)p = (bf16x4){(__bf16)v[0], (__bf16)v[1], (__bf16)v[2], (__bf16)v[3]};
}

// A wave's accumulators to C. The lane holds staged token row tok0 + 32 jj +
// lane % 32, which is row row_of(..) of the tile, and of every 32-row block of
// W rows the features 8 q + 4 (lane / 32) + r in register 4 q + r.
// feat0: first output feature of the wave.
template <int FI, int FJ, bool SWIGLU, typename TC, typename RowOf>
__device__ inline void write_accumulators(const GemmArgs& a, const f32x16 (&acc)[FI][FJ], int tok0,
                                          int row0, int rows_here, int feat0, RowOf row_of) {
  const int lane = threadIdx.x & 63, lr = lane & 31, lk = lane >> 5;
  const int N = a.N;
  TC* C = (TC*)a.C;
  // four features side by side go out in one store when every such group is whole and aligned
  const bool whole_quads = N % 4 == 0 && a.ldc % 4 == 0 && ((uintptr_t)a.C & 15) == 0;
  const bool gelu = a.epilogue == kEpilogueGeGLU;
#pragma unroll
  for (int jj = 0; jj < FJ; ++jj) {
    const int r_tile = row_of(tok0 + 32 * jj + lr);
    if (r_tile >= rows_here) continue;
    const int row = row0 + r_tile;
    const int64_t c_row = a.c_index ? a.c_index[row] : row;
    TC* crow = C + c_row * a.ldc;
    if (SWIGLU) {
#pragma unroll
      for (int i = 0; i < FI / 2; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int f0 = feat0 + 32 * i + 8 * q + 4 * lk;
          float v[4];
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            float g = acc[i][jj][4 * q + r], u = acc[i + (SWIGLU ? FI / 2 : 0)][jj][4 * q + r];
            if (a.bias && f0 + r < N) {
              g += a.bias[f0 + r];
              u += a.bias[N + f0 + r];
            }
            v[r] = gated_times(g, u, gelu);
          }
          if (whole_quads) {
            if (f0 < N) store_quad(crow + f0, v);
          } else {
#pragma unroll
            for (int r = 0; r < 4; ++r)
              if (f0 + r < N) crow[f0 + r] = from_f32<TC>(v[r]);
          }
        }
    } else {
#pragma unroll
      for (int i = 0; i < FI; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int f0 = feat0 + 32 * i + 8 * q + 4 * lk;
          float v[4];
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            v[r] = acc[i][jj][4 * q + r];
            if (a.bias && f0 + r < N) v[r] += a.bias[f0 + r];
          }
          if (whole_quads) {   // N % 4 == 0: the four features are in or out together
            if (f0 < N) store_quad(crow + f0, v);
          } else {
#pragma unroll
            for (int r = 0; r < 4; ++r)
              if (f0 + r < N) crow[f0 + r] = from_f32<TC>(v[r]);
          }
        }
    }
  }
}

// The same for bf16 output, through LDS, so that rows of C are written in whole
// 16-byte pieces side by side (the accumulator layout gives a lane 4 features
// of 32 different rows). `stage` is LDS of the wave's own, FJ * 32 rows of
// FEAT * 2 bytes; the 16-byte pieces of a row are stored in the order
// v ^ (row % pieces), which spreads the lanes of a write over the banks.
// Needs N % 8 == 0, ldc % 8 == 0 and C aligned to 16 bytes.
template <int FI, int FJ, bool SWIGLU, typename RowOf>
__device__ inline void write_accumulators_staged(const GemmArgs& a, const f32x16 (&acc)[FI][FJ],
                                                 unsigned char* stage, int tok0, int row0,
                                                 int rows_here, int feat0, RowOf row_of) {
  typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
  constexpr int FB = SWIGLU ? FI / 2 : FI;     // 32-feature blocks the wave writes
  constexpr int RB = FB * 64;                  // bytes of a staged row
  constexpr int U = RB / 16;                   // 16-byte pieces of a row
  constexpr int ROWS = FJ * 32;
  constexpr int RPI = 64 / U;                  // rows one store instruction covers
  static_assert(U >= 2 && U <= 64 && (U & (U - 1)) == 0, "row pieces");
  const int lane = threadIdx.x & 63, lr = lane & 31, lk = lane >> 5;
  const int N = a.N;
  const bool gelu = a.epilogue == kEpilogueGeGLU;
#pragma unroll
  for (int jj = 0; jj < FJ; ++jj) {
    const int tok = 32 * jj + lr;
#pragma unroll
    for (int i = 0; i < FB; ++i)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        bf16x4 val;
        if (SWIGLU) {
          float bg[4] = {0.f, 0.f, 0.f, 0.f}, bu[4] = {0.f, 0.f, 0.f, 0.f};
          const int f = feat0 + 32 * i + 8 * q + 4 * lk;
          if (a.bias && f < N) {   // N % 4 == 0: four features are in or out together
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              bg[r] = a.bias[f + r];
              bu[r] = a.bias[N + f + r];
            }
          }
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const float g = acc[i][jj][4 * q + r] + bg[r];
            const float u = acc[i + (SWIGLU ? FI / 2 : 0)][jj][4 * q + r] + bu[r];
            val[r] = (__bf16)gated_times(g, u, gelu);
          }
        } else {
          float b[4] = {0.f, 0.f, 0.f, 0.f};
          const int f = feat0 + 32 * i + 8 * q + 4 * lk;
          if (a.bias && f < N) {   // N % 4 == 0: four features are in or out together
#pragma unroll
            for (int r = 0; r < 4; ++r) b[r] = a.bias[f + r];
          }
#pragma unroll
          for (int r = 0; r < 4; ++r) val[r] = (__bf16)(acc[i][jj][4 * q + r] + b[r]);
        }
        const int v = 4 * i + q;
        *(bf16x4*)(stage + tok * RB + ((v ^ (tok & (U - 1))) << 4) + 8 * lk) = val;
      }
  }
  // row of C for staged rows lane and lane + 64 (-1: not a row of the tile)
  int c_row[(ROWS + 63) / 64];
#pragma unroll
  for (int h = 0; h < (ROWS + 63) / 64; ++h) {
    const int tok = 64 * h + lane;
    const int r_tile = tok < ROWS ? row_of(tok0 + tok) : rows_here;
    c_row[h] = -1;
    if (r_tile < rows_here) c_row[h] = a.c_index ? a.c_index[row0 + r_tile] : row0 + r_tile;
  }
  // LDS serves the accesses of one wave in order: its reads below see its writes above
  bf16* C = (bf16*)a.C;
  const int c = lane % U;
#pragma unroll
  for (int it = 0; it < ROWS / RPI; ++it) {
    const int tok = it * RPI + lane / U;
    const int dst = __shfl(c_row[(it * RPI) / 64], tok & 63, 64);
    const bf16x8 val = *(const bf16x8*)(stage + tok * RB + ((c ^ (tok & (U - 1))) << 4));
    const int f = feat0 + 8 * c;
    if (dst >= 0 && f < N) *(bf16x8*)(C + (int64_t)dst * a.ldc + f) = val;
  }
}

// Can C be written in whole 16-byte pieces?
__device__ inline bool c_takes_vectors(const GemmArgs& a) {
  return a.N % 8 == 0 && a.ldc % 8 == 0 && ((uintptr_t)a.C & 15) == 0;
}

// The epilogue of a wave: through LDS when C is bf16 and takes 16-byte pieces,
// element by element otherwise. The caller has made sure (a barrier) that no
// wave still reads the LDS that `stage` reuses; a wave needs FJ * 32 rows of
// 64 bytes per 32 features it writes.
template <int FI, int FJ, bool SWIGLU, typename TC, typename RowOf>
__device__ inline void write_tile(const GemmArgs& a, const f32x16 (&acc)[FI][FJ], unsigned char* stage,
                                  int tok0, int row0, int rows_here, int feat0, RowOf row_of) {
  if constexpr (std::is_same<TC, bf16>::value) {
    if (c_takes_vectors(a)) {
      write_accumulators_staged<FI, FJ, SWIGLU>(a, acc, stage, tok0, row0, rows_here, feat0, row_of);
      return;
    }
  }
  write_accumulators<FI, FJ, SWIGLU, TC>(a, acc, tok0, row0, rows_here, feat0, row_of);
}

bool gemm_tile_direct_takes(const GemmArgs& a);
int gemm_tile_direct(const GemmArgs& a, hipStream_t stream);

}  // namespace ninfer

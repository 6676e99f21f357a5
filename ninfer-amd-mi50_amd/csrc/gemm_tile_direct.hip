// C = A W^T for very many rows per weight matrix (bf16): 256 x 256 tiles, loaded
// from global memory straight into LDS (global_load_lds_dwordx4), so that no
// registers stage the tiles, in k tiles of 64 (whole 128-byte lines of every
// row): two buffers for the rows of A, which neighbours share through L2, and
// three for the rows of W, which come from HBM and are the bytes that have to
// be on their way (all 160 KB of a CU's LDS). Dense or grouped by expert, bias or SwiGLU epilogue, as
// the staged kernel beside it; the reference sends these products to rocBLAS
// (src/ops/linear.hip:21-35, src/models/model.hip:406-425).
//
// A block has 8 waves, two per SIMD, as a 4 x 2 grid; each wave owns 64 W rows
// x 128 tokens = 2 x 4 tiles of v_mfma_f32_32x32x16_bf16 (128 accumulator
// registers). Four waves of 128 x 128 read a third less from LDS per product,
// but on this part a CU's loads into LDS and its matrix instructions do not
// overlap (a block's time is their sum, whatever the order of issue), and what
// is left to hide is the rest: with two waves per SIMD the epilogue and the
// waits at the barrier of one run beside the products of the other (3 to 15%
// on the experts' products of 1,024 to 8,192 tokens).
// A wave column multiplies only its 32-row blocks that hold rows (the tile's rows
// fill the columns' blocks one after the other, the first column's first), and
// after the first two k tiles a wave loads only the pieces of A that hold rows,
// so a tile with few rows costs little more than its share: one tile height
// serves every count of rows per expert.
//
// LDS rows are 128 bytes (64 bf16) and unpadded, because a wave's load writes
// 1 KB contiguously (lane l at 16 l); the eight 16-byte chunks of row r are
// stored in the order c ^ ((r / 2) % 8), chosen on the global side, so that the
// 16 rows which one pass of a fragment read touches fall into 16 different
// 16-byte columns of the banks.
//
// One barrier per k tile, before its last quarter: when a wave passes the
// barrier of tile t, tile t + 1 has landed for every wave and every wave holds
// the last fragments of tile t in registers, so the loads of A's tile t + 2 and
// of W's tile t + 3 may overwrite tile t. The fragments of every quarter are read while the products
// of the quarter before run, across the barrier too.
#include "gemm_tile.h"
#include <type_traits>

namespace ninfer {

namespace direct {
constexpr int TM = 256, TN = 256;
constexpr int WGM = 4, WGN = 2;
constexpr int WAVES = WGM * WGN;
constexpr int COL = TM / WGN;             // staged token rows per wave column
constexpr int FI = TN / WGM / 32, FJ = TM / WGN / 32;
}  // namespace direct

// Wait until at most N of this wave's loads are under way (and, with LDS, until its LDS
// reads have returned).
template <int N> __device__ __forceinline__ void wait_loads() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
template <int N> __device__ __forceinline__ void wait_loads_and_lds() {
  asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(N) : "memory");
}

template <int TK, bool SWIGLU, typename TC>
__global__ __launch_bounds__(direct::WAVES * 64, 1) void gemm_tile_direct_kernel(GemmArgs a) {
  using namespace direct;
  constexpr int KK = TK / 16;                // parts of a k tile: one MFMA depth each
  constexpr int ROW_BYTES = TK * 2;
  constexpr int CPR = ROW_BYTES / 16;        // 16-byte chunks of a staged row
  constexpr int RPP = 64 / CPR;              // rows of a 1 KB piece
  constexpr int X_BYTES = TM * ROW_BYTES, W_BYTES = TN * ROW_BYTES;
  constexpr int NBX = 2, NBW = 3;            // buffers of A rows, of W rows
  constexpr int W_BASE = NBX * X_BYTES;
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];

  int bx, by;
  block_to_tile(a.offsets != nullptr, bx, by);
  int row0, row_end, group;
  // the search's three ints lie in the buffers: no load may land before every wave has them
  if (!tile_rows<TM>(a, bx, (int*)smem, row0, row_end, group)) return;
  __syncthreads();

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // the same in every lane: a scalar
  const int wm = wave % WGM, wn = wave / WGM;
  const int K = a.K, N = a.N;
  const bf16* W = (const bf16*)a.W + (int64_t)group * a.w_group_stride;
  constexpr int OUT_PER_BLOCK = SWIGLU ? TN / 2 : TN;
  constexpr int OUT_PER_WAVE = OUT_PER_BLOCK / WGM;
  const int out0 = by * OUT_PER_BLOCK;
  const int rows_here = min(TM, row_end - row0);
  // The tile's rows go to the two wave columns in whole blocks of 32, the first column
  // taking the odd one: a SIMD holds a wave of each column, so its matrix instructions are
  // those of both, and 137 rows cost it five blocks (3 + 2) where rows dealt in turn would
  // cost six (69 + 68 rows). Staged row l of column l / COL holds the tile's row
  // (l / COL) * rows0 + l % COL, or none (TM: beyond every tile's rows).
  static_assert(WGN == 2, "the rows are dealt to two wave columns");
  const int n_blocks = (rows_here + 31) / 32;
  const int rows0 = min(rows_here, 32 * ((n_blocks + 1) / 2));   // rows of the first column
  auto row_of = [&](int l) -> int {
    const int i = l % COL;
    if (l < COL) return i < rows0 ? i : TM;
    return rows0 + i < rows_here ? rows0 + i : TM;
  };

  // Loads: instruction i of wave w fills the 1 KB piece i * 4 + w of the X (and
  // of the W) part of a buffer: RPP rows, lane l at row l / CPR, stored chunk
  // l % CPR, which holds the row's chunk (l % CPR) ^ swizzle(row), where
  // swizzle(row) = (row / (16 / CPR)) % CPR.
  constexpr int NL = TM * ROW_BYTES / 1024 / WAVES;   // load instructions per wave, k tile and operand
  constexpr int NLT = 2 * NL;                     // loads per wave and k tile
  // the row's part of the swizzle that the piece's number leaves: pieces i * 4 + w differ
  // in multiples of 4 RPP rows between the loads of a wave, which the swizzle does not see
  const int chunk = (lane % CPR) ^ (((wave * RPP + lane / CPR) / (16 / CPR)) % CPR);
  static_assert((WAVES * RPP / (16 / CPR)) % CPR == 0, "the loads of a wave must share their swizzle");
  const bf16* xsrc[NL];
  const bf16* wsrc[NL];
  int x_row[NL];
  unsigned x_live = 0;   // bit i: piece i of this wave's loads of A holds rows of the tile
#pragma unroll
  for (int i = 0; i < NL; ++i) {
    const int l = (i * WAVES + wave) * RPP + lane / CPR;
    const int r = row_of(l);
    // rows beyond the tile's last read its first row (one line, from L1): their results are
    // never stored
    x_row[i] = r < rows_here ? row0 + r : row0;
    // a piece none of whose rows the tile has is loaded with the first tiles only (what the
    // fragments read there afterwards goes into sums that are never stored); staged rows
    // of a piece are neighbours in one column, so its first row decides
    if (row_of((i * WAVES + wave) * RPP) < rows_here) x_live |= 1u << i;
    wsrc[i] = W + (int64_t)staged_w_row<TN, WGM, SWIGLU>(l, out0, N) * K + 8 * chunk;
  }
  if (a.a_index) {   // the index loads in flight together
    int idx[NL];
#pragma unroll
    for (int i = 0; i < NL; ++i) idx[i] = a.a_index[x_row[i]];
#pragma unroll
    for (int i = 0; i < NL; ++i) x_row[i] = idx[i] / a.a_div;
  }
#pragma unroll
  for (int i = 0; i < NL; ++i) xsrc[i] = (const bf16*)a.A + (int64_t)x_row[i] * a.lda + 8 * chunk;
  typedef const __attribute__((address_space(1))) void* gptr;
  typedef __attribute__((address_space(3))) void* lptr;
  // Every lane of every load takes part: with some lanes switched off, a load into LDS did
  // not leave the other lanes' bytes where this layout expects them (products came out wrong).
  // Every block walks the k tiles in a circle from a start of its own: blocks that start
  // together would otherwise read the same columns of rows that lie a power of two apart at
  // the same time, which fall on few memory channels.
  const int nk_all = K / TK;
  // (Grouped: the start depends on the expert, not on the row tile, so that a row's sum has the
  // same order whichever tile of its expert the grouping put it in.)
  const int phase = (int)(((a.offsets ? group : bx) * 5u + by * 3u) % (unsigned)nk_all);
  // the t-th k tile of this block's walk: A rows into their buffer t % NBX, W rows into
  // theirs at byte w_off (the caller's count of t % NBW)
  auto issue_x = [&](int t) {
    unsigned char* buf = smem + (t % NBX) * X_BYTES + wave * 1024;
    int kt = t + phase;
    kt = kt >= nk_all ? kt - nk_all : kt;
#pragma unroll
    for (int i = 0; i < NL; ++i)
      if (t < NBX || (x_live & (1u << i)))
        __builtin_amdgcn_global_load_lds((gptr)(xsrc[i] + kt * TK), (lptr)(buf + i * (WAVES * 1024)), 16, 0, 0);
  };
  // An expert whose rows fit one tile (or a dense product of one row tile) has its W panel read
  // by this block alone: those loads
  // are marked non-temporal (the last argument: 2), so that they do not push the rows of A,
  // which the expert's other feature tiles read again, out of L2 (6 to 9% at 137 rows per
  // expert; with two tiles per expert the second finds the panel in L2 and the mark costs 4%).
  const bool w_once = a.offsets != nullptr ? row_end - a.offsets[group] <= TM : a.M <= TM;
  auto issue_w = [&](int t, int w_off) {
    unsigned char* buf = smem + W_BASE + w_off + wave * 1024;
    int kt = t + phase;
    kt = kt >= nk_all ? kt - nk_all : kt;
    if (w_once) {
#pragma unroll
      for (int i = 0; i < NL; ++i)
        __builtin_amdgcn_global_load_lds((gptr)(wsrc[i] + kt * TK), (lptr)(buf + i * (WAVES * 1024)), 16, 0, 2);
    } else {
#pragma unroll
      for (int i = 0; i < NL; ++i)
        __builtin_amdgcn_global_load_lds((gptr)(wsrc[i] + kt * TK), (lptr)(buf + i * (WAVES * 1024)), 16, 0, 0);
    }
  };
  auto next_w = [](int w_off) { return w_off == (NBW - 1) * W_BYTES ? 0 : w_off + W_BYTES; };

  f32x16 acc[FI][FJ];
#pragma unroll
  for (int i = 0; i < FI; ++i)
#pragma unroll
    for (int jj = 0; jj < FJ; ++jj)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][jj][v] = 0.f;

  // rows dealt to this wave's column, and its 32-row blocks that hold any
  const int col_rows = wn == 0 ? rows0 : rows_here - rows0;
  const int n_jj = (col_rows + 31) / 32;
  const int tok0 = wn * COL;

  // fragment addresses: lane reads row lr of a 32-row block, k chunk 2 kk + lk, stored at
  // chunk (2 kk + lk) ^ swizzle(lr) (the block's first row is a multiple of 16)
  const int lr = lane & 31, lk = lane >> 5;
  const int sw = (lr / (16 / CPR)) % CPR;
  const int x_lane = (tok0 + lr) * ROW_BYTES;
  const int w_lane = W_BASE + (wm * (TN / WGM) + lr) * ROW_BYTES;
  int c_part[KK];
#pragma unroll
  for (int kk = 0; kk < KK; ++kk) c_part[kk] = 16 * ((2 * kk + lk) ^ sw);
  const int nk = K / TK;

  auto run = [&](auto nj_tag) {
    constexpr int NJ = decltype(nj_tag)::value;
    constexpr int NX = NJ > 0 ? NJ : 1;
    bf16x8 wf[2][FI], xf[2][NX];
    // fragments of k part kk of the tile in A's buffer t % NBX and W's buffer at w_off
    auto read_part = [&](int set, int t, int w_off, int kk) {
      if constexpr (NJ == 0) return;
      const unsigned char* xb = smem + (t % NBX) * X_BYTES + c_part[kk];
      const unsigned char* wb = smem + w_off + c_part[kk];
#pragma unroll
      for (int i = 0; i < FI; ++i) wf[set][i] = *(const bf16x8*)(wb + w_lane + i * 32 * ROW_BYTES);
#pragma unroll
      for (int jj = 0; jj < NJ; ++jj) xf[set][jj] = *(const bf16x8*)(xb + x_lane + jj * 32 * ROW_BYTES);
    };
    auto multiply = [&](int set) {
#pragma unroll
      for (int jj = 0; jj < NJ; ++jj)
#pragma unroll
        for (int i = 0; i < FI; ++i)
          acc[i][jj] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[set][i], xf[set][jj], acc[i][jj], 0, 0, 0);
    };
    // The order of a quarter: every fragment read of the next quarter goes between two
    // products of this one, so that it has returned when its products begin.
    auto interleave = [&]() {
#pragma unroll
      for (int i = 0; i < FI + NJ; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // one MFMA
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // one LDS read
      }
      __builtin_amdgcn_sched_group_barrier(0x008, FI * NJ > FI + NJ ? FI * NJ - FI - NJ : 0, 0);
    };
    // A wave's loads return in the order of their issue: A 0, W 0, A 1, W 1, W 2, then per
    // tile t A t + 2, W t + 3. When tile t + 1 is needed, the only younger loads are W's
    // tile t + 2 (NL loads), which stay on their way.
    issue_x(0);
    issue_w(0, 0);
    if (nk > 1) {
      issue_x(1);
      issue_w(1, W_BYTES);
    }
    if (nk > 2) issue_w(2, 2 * W_BYTES);
    if (nk > 2) wait_loads<3 * NL>();
    else if (nk > 1) wait_loads<2 * NL>();
    else wait_loads<0>();
    __builtin_amdgcn_s_barrier();
    read_part(0, 0, 0, 0);
    int t = 0, w_cur = 0;   // w_cur: where W's tile t lies
    // steady state, free of conditions: W's tile t + 3 exists
    for (; t + NBW < nk; ++t) {
#pragma unroll
      for (int kk = 0; kk + 1 < KK; ++kk) {
        read_part((kk + 1) & 1, t, w_cur, kk + 1);
        multiply(kk & 1);
        interleave();
      }
      // this wave's loads of tile t + 1 have landed and its last fragments of tile t are in
      // registers; after the barrier that holds for every wave, and tile t's buffers are free
      wait_loads_and_lds<NL>();
      __builtin_amdgcn_s_barrier();
      issue_x(t + NBX);
      issue_w(t + NBW, w_cur);
      w_cur = next_w(w_cur);
      read_part(KK & 1, t + 1, w_cur, 0);
      multiply((KK - 1) & 1);
      interleave();
    }
    // the last NBW tiles: A's tile t + 2 still to issue while it exists
    for (; t < nk; ++t) {
#pragma unroll
      for (int kk = 0; kk + 1 < KK; ++kk) {
        read_part((kk + 1) & 1, t, w_cur, kk + 1);
        multiply(kk & 1);
      }
      if (t + NBW == nk) wait_loads_and_lds<NL>();   // W's last tile may stay on its way
      else wait_loads_and_lds<0>();
      __builtin_amdgcn_s_barrier();
      if (t + NBX < nk) issue_x(t + NBX);
      w_cur = next_w(w_cur);
      if (t + 1 < nk) read_part(KK & 1, t + 1, w_cur, 0);
      multiply((KK - 1) & 1);
    }
  };
  // one straight-line instance per count of live token blocks
  switch (n_jj) {
    case 0: run(std::integral_constant<int, 0>{}); break;
    case 1: run(std::integral_constant<int, 1>{}); break;
    case 2: run(std::integral_constant<int, 2>{}); break;
    case 3: run(std::integral_constant<int, 3>{}); break;
    default: run(std::integral_constant<int, 4>{}); break;
  }
  static_assert(WAVES * FJ * 32 * FI * 64 <= NBX * X_BYTES + NBW * W_BYTES, "the epilogue's stage exceeds the buffers");
  __syncthreads();   // every wave has read its last fragments: the buffers become the epilogue's stage
  write_tile<FI, FJ, SWIGLU, TC>(a, acc, smem + wave * (FJ * 32 * FI * 64), tok0, row0, rows_here,
                                 out0 + OUT_PER_WAVE * wm, row_of);
}

bool gemm_tile_direct_takes(const GemmArgs& a) {
  return a.in_dtype == kBF16 && a.K % 64 == 0 && a.lda % 8 == 0 &&
         ((uintptr_t)a.A % 16 == 0) && ((uintptr_t)a.W % 16 == 0) && a.w_group_stride % 8 == 0;
}

template <int TK>
static int launch_direct(const GemmArgs& a, hipStream_t stream) {
  using namespace direct;
  constexpr int LDS_BYTES = (2 * TM + 3 * TN) * TK * 2;
  const bool swiglu = epilogue_gated(a.epilogue);
  int m_tiles = (a.M + TM - 1) / TM + (a.offsets ? a.groups : 0);
  if (a.offsets) m_tiles = (m_tiles + kXcds - 1) / kXcds * kXcds;   // block_to_tile's bijection
  const int per_block = swiglu ? TN / 2 : TN;
  const dim3 grid(m_tiles, (a.N + per_block - 1) / per_block);
#define NINFER_DIRECT_LAUNCH(SW, TYPE)                                                          \
  do {                                                                                          \
    auto kern = gemm_tile_direct_kernel<TK, SW, TYPE>;                                    \
    hipError_t e = hipFuncSetAttribute((const void*)kern,                                       \
                                       hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);  \
    if (e != hipSuccess) return set_error(-2, "gemm: cannot get %d bytes of LDS", LDS_BYTES);   \
    kern<<<grid, direct::WAVES * 64, LDS_BYTES, stream>>>(a);                                                  \
  } while (0)
  if (a.out_dtype == kF32) {
    if (swiglu) NINFER_DIRECT_LAUNCH(true, float); else NINFER_DIRECT_LAUNCH(false, float);
  } else {
    if (swiglu) NINFER_DIRECT_LAUNCH(true, bf16); else NINFER_DIRECT_LAUNCH(false, bf16);
  }
#undef NINFER_DIRECT_LAUNCH
  NINFER_LAUNCH_CHECK();
  return 0;
}

int gemm_tile_direct(const GemmArgs& a, hipStream_t stream) {
  static_assert(direct::TM == kGroupedTileRows, "the grouped tile lists are made for this height");
  // k tiles of 64: measured faster than tiles of 32 in twice the buffers (whole 128-byte
  // lines per row beat the deeper queue of loads)
  return launch_direct<64>(a, stream);
}

}  // namespace ninfer

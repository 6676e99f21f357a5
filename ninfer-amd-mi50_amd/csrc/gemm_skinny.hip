// C = A W^T for few rows (decode): every weight is read once from HBM and
// multiplied on the matrix cores.
//
// One block owns 16 output features (16 rows of W; with the SwiGLU epilogue
// the 16 gate rows and their 16 up rows) and up to 16 rows of A. The weight
// rows are the A operand of v_mfma_f32_16x16x32_bf16 (lane l supplies row
// l % 16, k = 8 (l / 16) .. +7, i.e. 16 contiguous bytes), the activations are
// the B operand (lane l supplies token l % 16, same k), so the accumulator
// holds a 16 x 16 tile out[feature 4 (l / 16) + v][token l % 16]. The K range is
// split over the waves of the block, each wave a contiguous part that it walks
// in chunks of 128; partial tiles meet in LDS and are summed in wave order, so
// the result does not depend on timing. Activations are read straight from
// global memory (they stay in cache: few rows). Weights are loaded as whole
// 128-byte lines (8 rows per instruction, four instructions in flight per
// chunk), non-temporal, and reach the operand's layout through 2 KB of LDS per
// wave: read that way they stream at 6.4 TB/s, against 5.5 when every lane
// loads the 16 bytes of its operand itself.
//
// A dense product whose 16-feature tiles would be few is cut into tiles of
// fewer features (some of each matrix instruction's rows stay empty, which
// costs nothing where the weights' way into the CUs is the bound), so that the
// blocks are a whole multiple of the CUs and all CUs pull equally.
//
// Grouped form as in the plain kernel: tiles of 16 sorted rows per expert are
// enumerated from the device-side offsets; a block whose tile does not exist
// exits. The reference runs these products as one GEMV per row (decode,
// src/ops/gemv.hip:52-93) or one library call per expert
// (src/models/model.hip:355-427).
#include "gemm.h"
#include "moe_route.h"

namespace ninfer {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int SM = 16;  // rows of A per tile

// What a wave multiplies: SETS sets of 16 weight rows against up to 16 rows of A.
template <int SETS>
struct SkinnyOperands {
  const bf16* wrow[SETS];       // lane (r, j): weight row r of the set at k = 8 j (the operand's view)
  const bf16* wline[SETS][2];   // lane l: row 8 q + l / 8 at byte 16 (l % 8) (whole lines)
  bool line_valid[2];
  bool w_valid;                 // lanes of rows the tile does not have load nothing
  const bf16* xrow;             // lane (r, j): row r of A at k = 8 j
  bool m_valid;
  bool w_again;                 // another block beside this one reads the same weights (a dense
                                // product of several row tiles): they are to stay in L2
};

// One wave's part of the K range: `waves` waves split K in chunks of four steps (256 bytes
// of a row); a wave's chunks lie side by side, so that it walks its part of every row from
// one end to the other (measured with loads alone: 5.9 TB/s, against 5.6 with the waves'
// chunks interleaved). `my_stage`: this wave's 2 KB of LDS, 16 rows of 128 bytes, the
// 16-byte units of row R stored in the order u ^ (R % 8), so that the writes (a row per 8
// lanes) and the fragment reads (lane (r, j): row r, unit 4 i + j) both spread evenly over
// the banks.
template <int SETS, bool AGAIN = false>
__device__ __forceinline__ void skinny_walk(const SkinnyOperands<SETS>& o, int K, int wave,
                                            int waves, unsigned char* my_stage, int lane,
                                            f32x4 (&acc)[SETS]) {
  const int r = lane & 15, j = lane >> 4;
  const int st_write = ((lane >> 3) * 128) + 16 * ((lane & 7) ^ ((lane >> 3) & 7));   // + 1024 q
  const int st_read = r * 128;   // + 16 * ((4 i + j) ^ (r % 8))
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  const int steps = K / 32;
  const int chunks = (steps + 3) / 4, per_wave = (chunks + waves - 1) / waves;
  for (int c = wave * per_wave; c < min((wave + 1) * per_wave, chunks); ++c) {
    const int s0 = c * 4;
    if (s0 + 4 <= steps) {
      // A chunk is two pieces of 128 bytes per row. Weights are read once and by this wave
      // alone: whole lines, 8 rows per instruction, marked non-temporal (measured with loads
      // alone, with each wave walking its part of the rows in order: 6.6 TB/s, against 5.9
      // when every lane loads its own 16 bytes of the matrix instruction's operand, 64 bytes
      // of a row per instruction). They reach the operand's layout through LDS.
      bf16x8 wl[SETS][2][2], x[4];   // [set][piece][q]
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int s = 0; s < SETS; ++s)
#pragma unroll
          for (int q = 0; q < 2; ++q)
            wl[s][h][q] = !o.line_valid[q] ? zero
                          : AGAIN ? *(const bf16x8*)(o.wline[s][q] + s0 * 32 + h * 64)
                                  : stream_load((const bf16x8*)(o.wline[s][q] + s0 * 32 + h * 64));
#pragma unroll
      for (int i = 0; i < 4; ++i) x[i] = o.m_valid ? *(const bf16x8*)(o.xrow + (s0 + i) * 32) : zero;
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int s = 0; s < SETS; ++s) {
#pragma unroll
          for (int q = 0; q < 2; ++q) *(bf16x8*)(my_stage + st_write + 1024 * q) = wl[s][h][q];
#pragma unroll
          for (int i = 0; i < 2; ++i) {
            const bf16x8 wf = *(const bf16x8*)(my_stage + st_read + 16 * ((4 * i + j) ^ (r & 7)));
            acc[s] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf, x[2 * h + i], acc[s], 0, 0, 0);
          }
        }
    } else {
      for (int st = s0; st < steps; ++st) {
        bf16x8 x = o.m_valid ? *(const bf16x8*)(o.xrow + st * 32) : zero;
#pragma unroll
        for (int s = 0; s < SETS; ++s) {
          bf16x8 w = o.w_valid ? *(const bf16x8*)(o.wrow[s] + st * 32) : zero;
          acc[s] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w, x, acc[s], 0, 0, 0);
        }
      }
    }
  }
}

// A dense product of several row tiles is launched as one line of blocks in which the row
// tiles of a feature tile lie side by side on one XCD (blocks go to the XCDs in turn): the
// weights then come from HBM once and from that XCD's L2 for the other row tiles (with plain
// loads: SkinnyOperands::w_again). line_ids: the blocks of such a line; line_tile: the tile of
// block `id`, false for the ids that pad the line.
__host__ __device__ inline int line_ids(int grid_x, int grid_y) {
  return (grid_x + kXcds - 1) / kXcds * kXcds * grid_y;
}
__device__ __forceinline__ bool line_tile(int id, int grid_x, int grid_y, int& bx, int& by) {
  const int x = id % kXcds, slot = id / kXcds;
  by = slot % grid_y;
  bx = (slot / grid_y) * kXcds + x;
  return bx < grid_x;
}

// The work of one block: tile (bx, by) of the product `a`. WAVES > 0 fixes the waves that
// share the K range at compile time; WAVES == 0 takes them from `waves_arg` (waves of the
// block beyond that number must not call). `red` holds waves x (2 with SwiGLU, else 1) x 256
// floats.
// TWO: the block owns 32 output features, as two groups of 16 that meet the same activations
// (for products with many small tiles: half the blocks, each activation row read once for
// twice the weights). Not with SwiGLU, whose blocks have two sets of W rows already (gate
// and up): four sets were measured 7% slower at 2048 x 1408, 3% faster at 3584 x 2560.
template <int WAVES, bool FULL, bool SWIGLU, typename TC, bool TWO = false>
__device__ __forceinline__ void skinny_block(const GemmArgs& a, int rows_arg, int waves_arg,
                                             int bx, int by, float* red, unsigned char* stage,
                                             int* tile_info) {
  static_assert(!(TWO && SWIGLU) && (!TWO || FULL), "two feature groups: whole tiles, no SwiGLU");
  constexpr int HALVES = SWIGLU ? 2 : 1;     // sets per feature group
  constexpr int FG = TWO ? 2 : 1;            // feature groups
  constexpr int SETS = HALVES * FG;
  const int waves = WAVES > 0 ? WAVES : waves_arg;
  int row0, row_end, group = 0;
  if (a.offsets && a.tiles16) {
    // every thread reads the tile's entry itself: no barrier before the first loads
    int count = a.tile_counts[0];
    int4 t = ((const int4*)a.tiles16)[by];
    if (by >= count) return;
    group = t.x;
    row0 = t.y;
    row_end = t.z;
  } else if (a.offsets) {
    if (!find_tile(a.offsets, a.groups, SM, by, tile_info)) return;
    group = tile_info[2];
    row0 = tile_info[0];
    row_end = tile_info[1];
  } else {
    row0 = by * SM;
    row_end = a.M;
    if (row0 >= row_end) return;
  }

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, j = lane >> 4;
  const int rows = FULL ? 16 : rows_arg;   // features per group, at most 16
  const int n0 = bx * (TWO ? 32 : rows);
  const bool w_valid = FULL || r < rows;   // lanes of the empty rows load nothing
  const int K = a.K;

  const bf16* W = (const bf16*)a.W + (int64_t)group * a.w_group_stride;
  SkinnyOperands<SETS> o;
  o.w_valid = w_valid;
  o.w_again = !a.offsets && a.M > SM;
  // set s: feature group s / HALVES; with SwiGLU the odd sets are the up rows, N rows further
#pragma unroll
  for (int s = 0; s < SETS; ++s)
    o.wrow[s] = W + ((int64_t)min(n0 + 16 * (s / HALVES) + r, a.N - 1) + (s % HALVES ? a.N : 0)) * K +
                8 * j;
  // The same rows as the loads see them: whole 128-byte lines. Lane l reads 16 bytes at row
  // 8 q + l / 8, byte 16 (l % 8) of a 128-byte piece (q = 0, 1).
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    const int R = 8 * q + (lane >> 3);
    o.line_valid[q] = FULL || R < rows;
#pragma unroll
    for (int s = 0; s < SETS; ++s)
      o.wline[s][q] = W + ((int64_t)min(n0 + 16 * (s / HALVES) + R, a.N - 1) + (s % HALVES ? a.N : 0)) * K +
                      8 * (lane & 7);
  }
  const int mrow = row0 + r;
  o.m_valid = mrow < row_end;
  int64_t a_row = 0;
  if (o.m_valid) a_row = a.a_index ? a.a_index[mrow] / a.a_div : mrow;
  o.xrow = (const bf16*)a.A + a_row * a.lda + 8 * j;

  f32x4 acc[SETS];
#pragma unroll
  for (int s = 0; s < SETS; ++s) acc[s] = f32x4{0.f, 0.f, 0.f, 0.f};
  if (o.w_again)
    skinny_walk<SETS, true>(o, K, wave, waves, stage + wave * 2048, lane, acc);
  else
    skinny_walk<SETS>(o, K, wave, waves, stage + wave * 2048, lane, acc);

  // partial tiles -> LDS, element (feature f, token m) of set s at [m * 16 + f]
#pragma unroll
  for (int v = 0; v < 4; ++v) {
    int f = 4 * j + v;
#pragma unroll
    for (int s = 0; s < SETS; ++s) red[(wave * SETS + s) * 256 + r * 16 + f] = acc[s][v];
  }
  __syncthreads();
  if (threadIdx.x < 256) {
    const int m = threadIdx.x >> 4, f = threadIdx.x & 15;
    const int row = row0 + m;
    if (row < row_end && n0 + f < a.N && f < rows) {
      float sum[SETS];
#pragma unroll
      for (int s = 0; s < SETS; ++s) sum[s] = 0.f;
#pragma unroll
      for (int w = 0; w < (WAVES > 0 ? WAVES : 16); ++w) {
        if (WAVES == 0 && w >= waves) break;
#pragma unroll
        for (int s = 0; s < SETS; ++s) sum[s] += red[(w * SETS + s) * 256 + threadIdx.x];
      }
      const int64_t c_row = a.c_index ? a.c_index[row] : row;
#pragma unroll
      for (int fg = 0; fg < FG; ++fg) {
        const int col = n0 + 16 * fg + f;
        if (col >= a.N) break;
        float v = sum[fg * HALVES];
        if (SWIGLU) {
          float u = sum[fg * HALVES + (SWIGLU ? 1 : 0)];
          if (a.bias) {
            v += a.bias[col];
            u += a.bias[a.N + col];
          }
          v = v / (1.f + __expf(-gate_logit(v, a.epilogue == kEpilogueGeGLU))) * u;
        } else if (a.bias) {
          v += a.bias[col];
        }
        ((TC*)a.C)[c_row * a.ldc + col] = from_f32<TC>(v);
      }
    }
  }
}

template <int WAVES, bool FULL, bool SWIGLU, typename TC, bool TWO = false>
__global__ __launch_bounds__(WAVES * 64) void gemm_skinny_kernel(GemmArgs a, int rows_arg) {
  __shared__ float red[WAVES * (SWIGLU ? 2 : 1) * (TWO ? 2 : 1) * 256];
  __shared__ __attribute__((aligned(16))) unsigned char stage[WAVES * 2048];
  __shared__ int tile_info[3];
  int bx = blockIdx.x, by = blockIdx.y;
  if (!a.offsets && a.M > SM) {   // launched as one line of blocks (line_tile)
    if (!line_tile(blockIdx.x, (a.N + rows_arg - 1) / rows_arg, (a.M + SM - 1) / SM, bx, by)) return;
  }
  skinny_block<WAVES, FULL, SWIGLU, TC, TWO>(a, rows_arg, WAVES, bx, by, red, stage, tile_info);
}

// Two products that do not depend on each other in one launch: the first blocks are the
// tiles of `b` (the dense product, whose blocks run longest), the rest the tiles of `a`.
// With few rows every launch costs a fixed
// time next to which the products themselves are short; together they pay it once and
// their loads overlap. The block has the waves of the larger need; waves a problem
// does not use leave at once.
struct SkinnyPlan {
  int waves;    // waves that share the K range
  int rows;     // features per block (32 with `two`)
  int grid_x;
  int grid_y;
  bool two;     // two sets of 16 features per block
};

template <bool FULL_A, bool SW_A, typename TC_A, bool FULL_B, bool SW_B, typename TC_B,
          bool TWO_A = false>
__global__ __launch_bounds__(1024) void gemm_skinny_pair_kernel(GemmArgs a, SkinnyPlan pa,
                                                               GemmArgs b, SkinnyPlan pb) {
  // LDS by the block's waves (the launch passes blockDim.x / 64 * 4 KB): 2 KB of partial sums
  // (two sets of 256) and 2 KB of weight lines per wave; a fixed array for 16 waves would
  // hold blocks of 4 waves down to two per CU
  extern __shared__ __attribute__((aligned(16))) unsigned char pair_lds[];
  __shared__ int tile_info[3];
  float* red = (float*)pair_lds;
  unsigned char* stage = pair_lds + (blockDim.x >> 6) * 2048;
  const int wave = threadIdx.x >> 6;
  int id = blockIdx.x;
  // (the dense product's blocks come first, so that its line starts at an XCD's turn)
  const int blocks_b = pb.grid_y > 1 ? line_ids(pb.grid_x, pb.grid_y) : pb.grid_x;
  if (id < blocks_b) {
    if (wave >= pb.waves) return;
    int bx = id, by = 0;
    if (pb.grid_y > 1 && !line_tile(id, pb.grid_x, pb.grid_y, bx, by)) return;
    skinny_block<0, FULL_B, SW_B, TC_B>(b, pb.rows, pb.waves, bx, by, red, stage, tile_info);
  } else {
    id -= blocks_b;
    if (wave >= pa.waves) return;
    skinny_block<0, FULL_A, SW_A, TC_A, TWO_A>(a, pa.rows, pa.waves, id % pa.grid_x,
                                               id / pa.grid_x, red, stage, tile_info);
  }
}

// A router's logits and the routing they decide, by one block: the product `a` (dense, at
// most 16 rows, at most kRouteMaxFeatures features, 32-bit out) is small enough for one
// block, whose 16 waves share it as feature groups of 16 x parts of the K range; the block
// then holds every logit of every row and routes the rows itself (softmax, top-k, grouping
// by expert) out of LDS. As a kernel of its own the routing is a launch and a chain of
// dependent loads between the router's product and the experts' first one.
// `red`: 32 x 256 floats; `stage`: 32 KB (the waves' weight lines, then logits, counters
// and chosen experts). Every thread of the block must call.
constexpr int kRouteMaxFeatures = 80;

template <int NPL>
__device__ __forceinline__ void skinny_route_block(const GemmArgs& a, const RouteArgs& rt,
                                                   float* red, unsigned char* stage) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
  const int r = lane & 15, j = lane >> 4;
  const int N = a.N, K = a.K, T = a.M;
  const int groups = (N + 15) / 16;
  // A wave multiplies GS feature groups of 16 over its part of K; the waves are shared out as
  // sets of GS groups x parts of K. Rows beyond N repeat row N - 1: they are computed and
  // never used. The fewer parts of K per wave, the shorter the chain of dependent loads that
  // this block, the launch's longest, consists of.
  constexpr int GS = 2;
  const int sets = (groups + GS - 1) / GS, parts = waves / sets;
  const int g = wave / parts, part = wave % parts;   // waves beyond sets x parts have no share
  if (g < sets) {
    const bf16* W = (const bf16*)a.W;
    SkinnyOperands<GS> o;
    o.w_valid = true;
    o.w_again = false;
#pragma unroll
    for (int s = 0; s < GS; ++s) o.wrow[s] = W + (int64_t)min(16 * (GS * g + s) + r, N - 1) * K + 8 * j;
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      const int R = 8 * q + (lane >> 3);
      o.line_valid[q] = true;
#pragma unroll
      for (int s = 0; s < GS; ++s)
        o.wline[s][q] = W + (int64_t)min(16 * (GS * g + s) + R, N - 1) * K + 8 * (lane & 7);
    }
    o.m_valid = r < T;
    o.xrow = (const bf16*)a.A + (int64_t)(o.m_valid ? r : 0) * a.lda + 8 * j;
    f32x4 acc[GS];
#pragma unroll
    for (int s = 0; s < GS; ++s) acc[s] = f32x4{0.f, 0.f, 0.f, 0.f};
    skinny_walk<GS>(o, K, part, parts, stage + wave * 2048, lane, acc);
    // partial tile of group GS g + s from K part `part`: at ((GS g + s) * parts + part) * 256
#pragma unroll
    for (int s = 0; s < GS; ++s)
#pragma unroll
      for (int v = 0; v < 4; ++v)
        red[((GS * g + s) * parts + part) * 256 + r * 16 + 4 * j + v] = acc[s][v];
  }
  __syncthreads();   // the partial tiles are complete, and the weight lines' LDS is free
  // logit (row m, feature n): the parts of its group summed in their order; kept in LDS and
  // written out (the caller may read further columns than the experts', as a gate's logit)
  const int ldl = 16 * groups;
  float* logits_s = (float*)stage;
  for (int i = threadIdx.x; i < T * ldl; i += blockDim.x) {
    const int m = i / ldl, n = i % ldl;
    float sum = 0.f;
    for (int p = 0; p < parts; ++p) sum += red[((n >> 4) * parts + p) * 256 + m * 16 + (n & 15)];
    logits_s[i] = sum;
    if (n < N) ((float*)a.C)[(int64_t)m * a.ldc + n] = sum;
  }
  __syncthreads();
  int* cnt = (int*)(logits_s + 16 * ldl);   // E + 1 counters, then the chosen experts
  int* ids_s = cnt + rt.E + 1;
  for (int t = wave; t < T; t += waves) {
    const int mine = route_row<NPL>(logits_s + t * ldl, rt, rt.ids + (int64_t)t * rt.k,
                                    rt.wts + (int64_t)t * rt.k, lane);
    if (lane < rt.k) ids_s[t * rt.k + lane] = mine;
  }
  __syncthreads();
  align_block(ids_s, T * rt.k, rt.E, rt.offsets, rt.order, rt.tiles16, rt.tiles_big,
              rt.tile_counts, cnt);
}

// The first block is the router's (product `a` and routing `rt`), the others are the tiles of
// the dense product `b`, which does not depend on it (a shared expert's gate and up).
template <bool FULL_B, bool SW_B, typename TC_B>
__global__ __launch_bounds__(1024) void gemm_skinny_route_pair_kernel(GemmArgs a, RouteArgs rt,
                                                                     GemmArgs b, SkinnyPlan pb) {
  extern __shared__ __attribute__((aligned(16))) unsigned char pair_lds[];   // 16 waves x 4 KB
  __shared__ int tile_info[3];
  float* red = (float*)pair_lds;
  unsigned char* stage = pair_lds + (blockDim.x >> 6) * 2048;
  if (blockIdx.x == 0) {
    if (rt.E <= 64) skinny_route_block<1>(a, rt, red, stage);
    else skinny_route_block<4>(a, rt, red, stage);
    return;
  }
  const int id = blockIdx.x - 1;
  if ((int)(threadIdx.x >> 6) >= pb.waves) return;
  skinny_block<0, FULL_B, SW_B, TC_B>(b, pb.rows, pb.waves, id % pb.grid_x, id / pb.grid_x, red,
                                      stage, tile_info);
}

// The router's block alone (a router with nothing to launch beside it).
__global__ __launch_bounds__(1024) void gemm_skinny_route_kernel(GemmArgs a, RouteArgs rt) {
  extern __shared__ __attribute__((aligned(16))) unsigned char pair_lds[];   // 16 waves x 4 KB
  float* red = (float*)pair_lds;
  unsigned char* stage = pair_lds + (blockDim.x >> 6) * 2048;
  if (rt.E <= 64) skinny_route_block<1>(a, rt, red, stage);
  else skinny_route_block<4>(a, rt, red, stage);
}

template <int WAVES>
static void launch_skinny(const GemmArgs& a, int rows, bool two, hipStream_t stream) {
  int m_tiles = a.offsets ? min((a.M + SM - 1) / SM + a.groups, a.M) : (a.M + SM - 1) / SM;
  dim3 grid((a.N + rows - 1) / rows, m_tiles);   // as plan_skinny counts them
  if (!a.offsets && m_tiles > 1)   // one line of blocks, the row tiles of a feature tile side by side
    grid = dim3(line_ids(grid.x, m_tiles), 1);
  dim3 block(WAVES * 64);
  bool swiglu = epilogue_gated(a.epilogue);
  if (two) {   // whole tiles, no SwiGLU (plan_skinny)
    if (a.out_dtype == kF32)
      gemm_skinny_kernel<WAVES, true, false, float, true><<<grid, block, 0, stream>>>(a, 16);
    else
      gemm_skinny_kernel<WAVES, true, false, bf16, true><<<grid, block, 0, stream>>>(a, 16);
    return;
  }
#define NINFER_SKINNY(FULL)                                                                   \
  do {                                                                                        \
    if (a.out_dtype == kF32) {                                                                \
      if (swiglu)                                                                             \
        gemm_skinny_kernel<WAVES, FULL, true, float><<<grid, block, 0, stream>>>(a, rows);    \
      else                                                                                    \
        gemm_skinny_kernel<WAVES, FULL, false, float><<<grid, block, 0, stream>>>(a, rows);   \
    } else {                                                                                  \
      if (swiglu)                                                                             \
        gemm_skinny_kernel<WAVES, FULL, true, bf16><<<grid, block, 0, stream>>>(a, rows);     \
      else                                                                                    \
        gemm_skinny_kernel<WAVES, FULL, false, bf16><<<grid, block, 0, stream>>>(a, rows);    \
    }                                                                                         \
  } while (0)
  if (rows == 16) NINFER_SKINNY(true); else NINFER_SKINNY(false);
#undef NINFER_SKINNY
}

// Shapes the kernel takes: bf16 inputs, K a multiple of 32, rows 16-byte aligned.
bool gemm_skinny_takes(const GemmArgs& a) {
  return a.in_dtype == kBF16 && a.K % 32 == 0 && a.lda % 8 == 0 &&
         ((uintptr_t)a.A % 16 == 0) && ((uintptr_t)a.W % 16 == 0) && a.w_group_stride % 8 == 0;
}

constexpr long kSkinnyTwoMinBlocks = 4096;   // GemmArgs::skinny_two overrides the choice for tests

static SkinnyPlan plan_skinny(const GemmArgs& a) {
  SkinnyPlan p;
  // more waves per block when the grid alone would leave CUs idle (grouped: at most one tile
  // per sorted row, and one partial tile per group)
  p.grid_y = a.offsets ? min((a.M + SM - 1) / SM + a.groups, a.M) : (a.M + SM - 1) / SM;
  int m_tiles = p.grid_y;
  long blocks = (long)((a.N + 15) / 16) * m_tiles;
  int chunks = a.K / 128;
  // features per block: 16, or for a dense product with few tiles the count that makes the
  // blocks a whole multiple of the CUs
  p.rows = 16;
  const int cus = device_cu_count();
  if (!a.offsets && m_tiles == 1 && blocks < 8 * cus) {
    const int per_cu = (a.N + 16 * cus - 1) / (16 * cus);          // blocks each CU gets
    p.rows = (a.N + per_cu * cus - 1) / (per_cu * cus);
  } else if (a.offsets && a.M <= 8 && blocks < 8 * cus) {
    // a single token's choices: one tile per sorted row (its experts differ), counted alike
    const long per_cu = ((long)a.N * m_tiles + 16 * cus - 1) / (16 * cus);
    p.rows = (int)(((long)a.N * m_tiles + per_cu * cus - 1) / (per_cu * cus));
  }
  // (16 waves only while the blocks are fewer than the CUs: a block of 16 waves is alone on its
  // CU, and with more blocks than CUs they follow each other there with nothing overlapping
  // their starts and ends; two blocks of 8 waves side by side: a batch-1 step 1.5 to 2% faster)
  p.waves = (blocks < cus && chunks >= 16) ? 16 : (blocks < 8 * cus && chunks >= 8) ? 8 : 4;
  // a grouped product without SwiGLU whose tiles are many and short (K small): two feature
  // sets per block, so that blocks are half as many and each does twice the work
  p.two = a.skinny_two >= 0 && a.offsets && a.epilogue == kEpilogueNone && p.rows == 16 &&
          p.waves == 4 && blocks >= (a.skinny_two > 0 ? 1 : kSkinnyTwoMinBlocks) && a.N % 32 == 0;
  if (p.two) p.rows = 32;
  p.grid_x = (a.N + p.rows - 1) / p.rows;
  return p;
}

int gemm_skinny(const GemmArgs& a, hipStream_t stream) {
  const SkinnyPlan p = plan_skinny(a);
  if (p.waves == 16)
    launch_skinny<16>(a, p.rows, false, stream);
  else if (p.waves == 8)
    launch_skinny<8>(a, p.rows, false, stream);
  else
    launch_skinny<4>(a, p.rows, p.two, stream);
  NINFER_LAUNCH_CHECK();
  return 0;
}

// The pairs that have a kernel: (dense, 32-bit out) beside (dense SwiGLU), as a router's
// logits beside a shared expert's gate and up; (grouped) beside (dense), as the experts'
// down products beside the shared expert's. Both bf16 in, the second bf16 out.
bool gemm_skinny_pair_takes(const GemmArgs& a, const GemmArgs& b) {
  if (!gemm_skinny_takes(a) || !gemm_skinny_takes(b) || a.bias || b.bias) return false;
  const bool dense_b = !b.offsets && b.out_dtype == kBF16;
  const bool first = !a.offsets && a.out_dtype == kF32 && a.epilogue == kEpilogueNone &&
                     dense_b && epilogue_gated(b.epilogue);
  const bool second = a.offsets && a.out_dtype == kBF16 && a.epilogue == kEpilogueNone &&
                      dense_b && b.epilogue == kEpilogueNone;
  return first || second;
}

int gemm_skinny_pair(const GemmArgs& a, const GemmArgs& b, hipStream_t stream) {
  SkinnyPlan pa = plan_skinny(a), pb = plan_skinny(b);
  // beside a grouped product with many blocks, which are small, the dense one takes the same
  // few waves: blocks as wide as the larger need would hold up the small blocks' places
  if (a.offsets && !pa.two) {   // the pair's grouped kernel has whole tiles of 16 features
    pa.rows = 16;
    pa.grid_x = (a.N + 15) / 16;
  }
  if (a.offsets && (long)pa.grid_x * pa.grid_y >= 2048) pb.waves = pa.waves;
  // ... and 8 waves at most where the launch has more blocks than there are CUs (a block has
  // the places of the larger need, and blocks of 16 waves follow each other on a CU with
  // nothing overlapping their starts and ends): batch 1 and 2 steps 1.5 to 2% faster
  if (pb.waves == 16 && pa.waves <= 8 &&
      (long)pa.grid_x * pa.grid_y + (long)pb.grid_x * pb.grid_y >= device_cu_count())
    pb.waves = 8;
  const int threads = 64 * max(pa.waves, pb.waves);
  const size_t lds = (size_t)(threads / 64) * 4096;   // partial sums and weight lines, per wave
  const long blocks = (long)pa.grid_x * pa.grid_y +
                      (pb.grid_y > 1 ? (long)line_ids(pb.grid_x, pb.grid_y) : (long)pb.grid_x);
  NINFER_REQUIRE(blocks < (1L << 31), "gemm pair: %ld blocks are too many", blocks);
  if (!a.offsets)
    gemm_skinny_pair_kernel<false, false, float, false, true, bf16>
        <<<(unsigned)blocks, threads, lds, stream>>>(a, pa, b, pb);
  else if (pa.two)
    gemm_skinny_pair_kernel<true, false, bf16, false, false, bf16, true>
        <<<(unsigned)blocks, threads, lds, stream>>>(a, pa, b, pb);
  else
    gemm_skinny_pair_kernel<true, false, bf16, false, false, bf16>
        <<<(unsigned)blocks, threads, lds, stream>>>(a, pa, b, pb);
  NINFER_LAUNCH_CHECK();
  return 0;
}

// The pair (router's logits, a dense SwiGLU) with the routing of the logits in the same
// launch: few rows (one tile of 16), few router features (one block streams their weights in
// the time the other product's blocks take anyway).
// A router's product of few rows and few features, and the routing by it, in one block.
bool gemm_skinny_route_takes(const GemmArgs& a, const RouteArgs& rt) {
  // the routing block reads A by row and writes C by row: no row indices, one group
  if (!gemm_skinny_takes(a) || a.offsets || a.a_index || a.c_index || a.groups > 1 || a.bias ||
      a.out_dtype != kF32 || a.epilogue != kEpilogueNone)
    return false;
  return a.M <= SM && a.N <= kRouteMaxFeatures && a.N >= rt.E && (int64_t)a.N * a.K <= (1 << 19) &&
         rt.E >= 1 && rt.k >= 1 && rt.k <= rt.E && rt.k <= 64;
}

int gemm_skinny_route(const GemmArgs& a, const RouteArgs& rt, hipStream_t stream) {
  gemm_skinny_route_kernel<<<1, 1024, 16 * 4096, stream>>>(a, rt);
  NINFER_LAUNCH_CHECK();
  return 0;
}

bool gemm_skinny_route_pair_takes(const GemmArgs& a, const GemmArgs& b, const RouteArgs& rt) {
  return gemm_skinny_pair_takes(a, b) && gemm_skinny_route_takes(a, rt);
}

int gemm_skinny_route_pair(const GemmArgs& a, const GemmArgs& b, const RouteArgs& rt,
                           hipStream_t stream) {
  const SkinnyPlan pb = plan_skinny(b);
  // The router's block has work for 16 waves and is the launch's longest beside a short
  // dense product. But a block of 16 waves is alone on its CU, and the dense product's blocks
  // then follow each other with nothing overlapping their starts and ends (they stream at 5.5
  // TB/s instead of 6.8): beside a long dense product (100 MB of weights and more) every block
  // has the dense product's waves, and the router's block makes do with them.
  const bool long_b = (int64_t)b.N * b.K * (epilogue_gated(b.epilogue) ? 4 : 2) >= (100LL << 20);
  const int threads = long_b ? 64 * max(pb.waves, 8) : 1024;
  const size_t lds = (size_t)(threads / 64) * 4096;
  // the router's block: 5 KB of logits, E + 1 counters and 16 k chosen experts in its 32 KB
  static_assert(16 * kRouteMaxFeatures * 4 + (kRouteMaxFeatures + 1) * 4 + 16 * 64 * 4 <= 8 * 2048,
                "the routing block's LDS (8 waves' stage at least)");
  static_assert((kRouteMaxFeatures + 15) / 16 <= 8, "a wave's two feature groups x 8 waves hold them");
  const long blocks = 1 + (long)pb.grid_x * pb.grid_y;
  NINFER_REQUIRE(blocks < (1L << 31), "gemm pair: %ld blocks are too many", blocks);
  gemm_skinny_route_pair_kernel<false, true, bf16>
      <<<(unsigned)blocks, threads, lds, stream>>>(a, rt, b, pb);
  NINFER_LAUNCH_CHECK();
  return 0;
}

}  // namespace ninfer



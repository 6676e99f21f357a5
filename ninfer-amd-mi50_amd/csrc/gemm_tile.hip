// C = A W^T for many rows (prompt portions) on the matrix cores: dense, or
// grouped by expert with one launch for all experts, with a bias or a SwiGLU
// epilogue. bf16 inputs, 32-bit accumulation, bf16 or 32-bit output.
//
// A block of NW waves owns TM rows of A (sorted rows of one expert in the
// grouped form) and TN rows of W; the waves form a WGM x WGN grid, each with
// FI x FJ tiles of v_mfma_f32_32x32x16_bf16. W rows are the A operand (lane l:
// row l % 32, k = 8 (l / 32) .. +7), activation rows the B operand, so a lane's
// accumulator holds, for token l % 32, four consecutive output features per
// register quad: C^T[feature 8 (v / 4) + 4 (l / 32) + v % 4][token l % 32].
// With the SwiGLU epilogue the first half of a wave's W rows are gate rows and
// the second half their up rows, so silu(g) * u is formed in registers and the
// block writes TN / 2 output features.
//
// What bounds this kernel is the traffic from L2 into LDS (every block reads
// its W panel and its A panel over the whole K), so tiles are as large as the
// rows allow: 256 x 256 with 8 waves when an expert has many rows. The rows of
// a tile are dealt to the WGN wave columns in turn (row r to column r % WGN),
// so a partly filled tile keeps all columns equally busy, and 32-row blocks
// without rows are skipped. Tiles go global -> registers -> LDS with the loads
// of later tiles in flight during the products (P register stages, two LDS
// buffers, one LDS-only barrier per k step). Block ids are mapped to tiles so
// that the blocks of one XCD (its own L2) work on neighbouring tiles. The
// reference sends these products to rocBLAS, one call per expert
// (src/models/model.hip:406-425, src/ops/linear.hip:21-35).
#include "gemm_tile.h"
#include <type_traits>

namespace ninfer {

template <int TM, int TN, int TK, int NW, int WGM, int P, int OCC, bool SWIGLU, typename TC>
__global__ __launch_bounds__(NW * 64, OCC) void gemm_tile_kernel(GemmArgs a) {
  constexpr int NT = NW * 64;            // threads
  constexpr int WGN = NW / WGM;
  constexpr int COL = TM / WGN;          // tile rows of one wave column
  constexpr int FI = TN / WGM / 32;      // 32-row blocks of W per wave
  constexpr int FJ = COL / 32;           // 32-row blocks of tokens per wave
  constexpr int TPAD = TK + 8;           // bf16 per LDS row
  constexpr int VPR = TK / 8;            // 16-byte vectors per row and k tile
  constexpr int XV = TM * VPR / NT;     // vectors of A per thread and k tile
  constexpr int WV = TN * VPR / NT;     // vectors of W per thread and k tile
  static_assert(FI >= 1 && FJ >= 1 && XV >= 1 && WV >= 1, "tile too small for the block");
  static_assert(!SWIGLU || FI % 2 == 0, "SwiGLU needs gate and up rows in every wave");
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  bf16* xs = (bf16*)smem;                       // [2][TM * TPAD]
  bf16* ws = xs + 2 * TM * TPAD;                // [2][TN * TPAD]
  __shared__ int tile_info[3];

  int bx, by;
  block_to_tile(a.offsets != nullptr, bx, by);
  int row0, row_end, group;
  if (!tile_rows<TM>(a, bx, tile_info, row0, row_end, group)) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave % WGM, wn = wave / WGM;
  const int K = a.K, N = a.N;
  const bf16* W = (const bf16*)a.W + (int64_t)group * a.w_group_stride;
  // a product cut along K: this block's k tiles are kt_first .. kt_first + nk - 1, and its
  // sums go to part blockIdx.z of C
  int nk = K / TK, kt_first = 0;
  if (a.k_parts > 1) {
    const int per = (nk + a.k_parts - 1) / a.k_parts;
    kt_first = blockIdx.z * per;
    nk = min(per, nk - kt_first);
    a.C = (TC*)a.C + (int64_t)blockIdx.z * a.M * a.ldc;
  }
  constexpr int OUT_PER_BLOCK = SWIGLU ? TN / 2 : TN;
  constexpr int OUT_PER_WAVE = OUT_PER_BLOCK / WGM;
  const int out0 = by * OUT_PER_BLOCK;
  const int rows_here = min(TM, row_end - row0);

  // LDS row l holds the tile's row (l % COL) * WGN + l / COL: column l / COL gets every WGN-th row
  auto row_of = [&](int l) -> int { return (l % COL) * WGN + l / COL; };
  const bf16* xsrc[XV];
  const bf16* wsrc[WV];
#pragma unroll
  for (int i = 0; i < XV; ++i) {
    int v = tid + i * NT, r = row_of(v / VPR), kv = v % VPR;
    // rows beyond the tile's last read its first row: their results are never stored
    int rr = r < rows_here ? row0 + r : row0;
    int64_t ar = a.a_index ? a.a_index[rr] / a.a_div : rr;
    xsrc[i] = (const bf16*)a.A + ar * a.lda + 8 * kv + kt_first * TK;
  }
#pragma unroll
  for (int i = 0; i < WV; ++i) {
    int v = tid + i * NT, r = v / VPR, kv = v % VPR;
    wsrc[i] = W + (int64_t)staged_w_row<TN, WGM, SWIGLU>(r, out0, N) * K + 8 * kv + kt_first * TK;
  }
  // Every block walks its k tiles in a circle from a start of its own: blocks that start
  // together would otherwise read the same columns of rows that lie a power of two apart at
  // the same time, which fall on few memory channels.
  // (Grouped: the start depends on the expert, not on the row tile, so that a row's sum has the
  // same order whichever tile of its expert the grouping put it in.)
  const int phase = (int)(((a.offsets ? group : bx) * 5u + by * 3u) % (unsigned)nk);
  // An expert whose rows fit one tile (or a dense product of one row tile) has its W panel
  // read by this block alone: non-temporal loads, so that they do not push out of L2 the rows
  // of A that the other feature tiles read again.
  const bool w_once = a.offsets != nullptr ? row_end - a.offsets[group] <= TM : a.M <= TM;
  // P register stages: the loads of k tile t + P are issued while tile t is multiplied
  bf16x8 xreg[P][XV], wreg[P][WV];
  auto load_tile = [&](int st, int k_lin) {   // k_lin: the tile's place in this block's walk, times TK
    int kt = k_lin / TK + phase;
    kt = kt >= nk ? kt - nk : kt;
    const int k0 = kt * TK;
#pragma unroll
    for (int i = 0; i < XV; ++i) xreg[st][i] = *(const bf16x8*)(xsrc[i] + k0);
    if (w_once) {
#pragma unroll
      for (int i = 0; i < WV; ++i) wreg[st][i] = stream_load((const bf16x8*)(wsrc[i] + k0));
    } else {
#pragma unroll
      for (int i = 0; i < WV; ++i) wreg[st][i] = *(const bf16x8*)(wsrc[i] + k0);
    }
  };
  auto store_tile = [&](int st, int buf) {
#pragma unroll
    for (int i = 0; i < XV; ++i) {
      int v = tid + i * NT;
      *(bf16x8*)(xs + buf * TM * TPAD + (v / VPR) * TPAD + 8 * (v % VPR)) = xreg[st][i];
    }
#pragma unroll
    for (int i = 0; i < WV; ++i) {
      int v = tid + i * NT;
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

  // rows dealt to this wave's column, and its 32-row blocks that hold any
  const int col_rows = rows_here > wn ? (rows_here - wn + WGN - 1) / WGN : 0;
  const int n_jj = (col_rows + 31) / 32;
  const int tok0 = wn * COL;

  const int lr = lane & 31, lk = lane >> 5;
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
    for (int st = 0; st < P; ++st)
      if (st < nk) load_tile(st, st * TK);
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
    // the last tiles (fewer than 2 P): loads only while tiles remain
    for (; kt0 < nk; kt0 += P) {
#pragma unroll
      for (int st = 0; st < P; ++st) {
        const int kt = kt0 + st;
        if (kt < nk) {
          if (kt + P < nk) load_tile(st, (kt + P) * TK);
          multiply(kt & 1, nj_tag);
          if (kt + 1 < nk) store_tile((st + 1) % P, (kt & 1) ^ 1);
          lds_barrier();
        }
      }
    }
  };
  // one straight-line instance per count of live token blocks
  if (n_jj == 0) {
    run(std::integral_constant<int, 0>{});
  } else if (FJ > 1 && n_jj == 1) {
    run(std::integral_constant<int, 1>{});
  } else if (FJ > 2 && n_jj == 2) {
    run(std::integral_constant<int, (FJ > 2 ? 2 : FJ)>{});
  } else if (FJ > 3 && n_jj == 3) {
    run(std::integral_constant<int, (FJ > 3 ? 3 : FJ)>{});
  } else {
    run(std::integral_constant<int, FJ>{});
  }

  static_assert(NW * FJ * 32 * FI * 64 <= 2 * (TM + TN) * TPAD * 2, "the epilogue's stage exceeds the tiles' LDS");
  __syncthreads();   // every wave has read its last fragments: the buffers become the epilogue's stage
  write_tile<FI, FJ, SWIGLU, TC>(a, acc, smem + wave * (FJ * 32 * FI * 64), tok0, row0, rows_here,
                                 out0 + OUT_PER_WAVE * wm, row_of);
}

// K must be a whole number of k tiles of 64.
bool gemm_tile_takes(const GemmArgs& a) {
  return a.in_dtype == kBF16 && a.K % 64 == 0 && a.lda % 8 == 0 && ((uintptr_t)a.A % 16 == 0) &&
         ((uintptr_t)a.W % 16 == 0) && a.w_group_stride % 8 == 0;
}

constexpr int64_t kSplitMinBytes = 48 << 20;   // GemmArgs::split_min_bytes lowers it for tests

template <int TM, int TN, int TK, int NW, int WGM, int P, int OCC = 2>
static int launch_tile(const GemmArgs& a, hipStream_t stream) {
  const bool swiglu = epilogue_gated(a.epilogue);
  int m_tiles = (a.M + TM - 1) / TM + (a.offsets ? a.groups : 0);
  if (a.offsets) m_tiles = (m_tiles + kXcds - 1) / kXcds * kXcds;   // block_to_tile's bijection
  const int per_block = swiglu ? TN / 2 : TN;
  const dim3 grid(m_tiles, (a.N + per_block - 1) / per_block, a.k_parts > 1 ? a.k_parts : 1);
  const size_t lds = 2 * (TM + TN) * (TK + 8) * sizeof(bf16);
#define NINFER_TILE_LAUNCH(SW, TYPE)                                                        \
  do {                                                                                      \
    auto kern = gemm_tile_kernel<TM, TN, TK, NW, WGM, P, OCC, SW, TYPE>;                             \
    if (lds > 48 * 1024) {                                                                  \
      hipError_t e = hipFuncSetAttribute((const void*)kern,                                 \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, lds);  \
      if (e != hipSuccess) return set_error(-2, "gemm: cannot get %zu bytes of LDS", lds);  \
    }                                                                                       \
    kern<<<grid, NW * 64, lds, stream>>>(a);                                               \
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
  // Tile height. Grouped: the tall tile (it loads and multiplies only the 32-row blocks that
  // hold rows, so it beats the lower ones from 17 rows per expert on, the fewest that come
  // here). Dense: the tallest tile that still gives every CU a block (taller tiles read less
  // per product, but fewer of them fill the chip). force_kernel (tests) forces 64, 128 or
  // 256 rows.
  int rows;
  if (a.force_kernel >= 1 && a.force_kernel <= 3) {
    rows = 32 << a.force_kernel;
  } else if (a.offsets) {
    rows = kGroupedTileRows;
  } else {
    const int n_units = epilogue_gated(a.epilogue) ? 2 * a.N : a.N;   // W rows
    auto blocks = [&](int tm, int tn) { return ((a.M + tm - 1) / tm) * ((n_units + tn - 1) / tn); };
    const int cus = device_cu_count();
    rows = blocks(256, 256) >= cus ? 256 : blocks(128, 128) >= cus ? 128 : 64;
    if (a.M <= 64) rows = 64;           // and no taller than the rows there are
    else if (a.M <= 128 && rows > 128) rows = 128;
  }
  if (rows == 256) return gemm_tile_direct(a, stream);
  if (rows == 128) return launch_tile<128, 128, 64, 4, 2, 2>(a, stream);
  return launch_tile<64, 128, 64, 4, 2, 2>(a, stream);
}

// out[m][n] = sum over the parts, in their order, of ws[z][m][n] (+ bias[n]); four features a thread.
template <typename TC>
__global__ void sum_parts_kernel(const float* __restrict__ ws, int parts, int M, int N,
                                 const float* __restrict__ bias, TC* __restrict__ out, int ldc) {
  const int64_t q = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;   // quad of features
  const int quads = N / 4;
  if (q >= (int64_t)M * quads) return;
  const int m = q / quads, n = 4 * (q % quads);
  float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int z = 0; z < parts; ++z) {
    const float4 v = *(const float4*)(ws + ((int64_t)z * M + m) * N + n);
    s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
  }
  if (bias) {
    s.x += bias[n]; s.y += bias[n + 1]; s.z += bias[n + 2]; s.w += bias[n + 3];
  }
  const float v[4] = {s.x, s.y, s.z, s.w};
  store_quad(out + (int64_t)m * ldc + n, v);
}

// The cut along K pays where the tiles of the output (64 x 128, or 128 x 128 beyond 128 rows)
// are fewer than the CUs, K is long, and the weights are many enough (48 MB and more) that
// their stream outweighs the second launch that adds the parts up (measured against the
// library's product at 3584 x 20480: 41 against 99 us at 64 rows, 111 against 226 at 512;
// no gain at 25 MB; at 8192 x 8192 and 384 rows the library is faster, hence K >= 2 N beyond
// 128 rows). Parts so that about two blocks per CU exist, each with at least four k tiles,
// and no part is empty.
int gemm_split_parts(const GemmArgs& a) {
  if (a.offsets || a.epilogue != kEpilogueNone || !a.workspace || !gemm_tile_takes(a)) return 1;
  if (a.M <= 32 || a.M > 512 || a.N % 4 || a.ldc % 4 || ((uintptr_t)a.C & 15)) return 1;
  if ((int64_t)a.N * a.K * 2 < (a.split_min_bytes > 0 ? a.split_min_bytes : kSplitMinBytes)) return 1;
  if (a.M > 128 && a.K < 2 * a.N) return 1;   // beyond 128 rows only where K is long against N
  const int cus = device_cu_count(), tk = 64;
  const int tm = a.M > 128 ? 128 : 64;
  const int tiles = ((a.M + tm - 1) / tm) * ((a.N + 127) / 128), nk = a.K / tk;
  if (tiles >= cus) return 1;
  const int64_t fit = a.workspace_floats / ((int64_t)a.M * a.N);
  int parts = (int)min((int64_t)min(min(16, 2 * cus / tiles), nk / 4), fit);
  if (parts < 2) return 1;
  const int per = (nk + parts - 1) / parts;
  return (nk + per - 1) / per;
}

int gemm_split(const GemmArgs& a, hipStream_t stream) {
  const int parts = gemm_split_parts(a);
  NINFER_REQUIRE(parts >= 2, "gemm: this product is not cut along K");
  GemmArgs b = a;
  b.C = a.workspace;
  b.ldc = a.N;
  b.out_dtype = kF32;
  b.bias = nullptr;
  b.k_parts = parts;
  int rc = a.M > 128 ? launch_tile<128, 128, 64, 4, 2, 2>(b, stream)
                     : launch_tile<64, 128, 64, 4, 2, 2>(b, stream);
  if (rc) return rc;
  const int64_t quads = (int64_t)a.M * (a.N / 4);
  const unsigned blocks = (unsigned)((quads + 255) / 256);
  if (a.out_dtype == kF32)
    sum_parts_kernel<float><<<blocks, 256, 0, stream>>>(a.workspace, parts, a.M, a.N, a.bias,
                                                        (float*)a.C, a.ldc);
  else
    sum_parts_kernel<bf16><<<blocks, 256, 0, stream>>>(a.workspace, parts, a.M, a.N, a.bias,
                                                       (bf16*)a.C, a.ldc);
  NINFER_LAUNCH_CHECK();
  return 0;
}

}  // namespace ninfer


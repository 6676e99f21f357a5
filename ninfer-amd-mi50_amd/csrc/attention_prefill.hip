// Paged attention for prompt portions (bf16) on the matrix cores.
//
// One block owns NQ * 32 consecutive rows of one request and one query head
// (128 or 64 rows: every key and value it loads serves that many). It has
// 2 NQ waves: rows are dealt to NQ groups of 32, and two waves share a group,
// one for the first and one for the second 32 keys of every tile, each with a
// running max, sum and output of its own that are merged at the end. So every
// SIMD holds two waves, and the softmax arithmetic of one overlaps the matrix
// products of the other. Keys and values are walked in tiles of
// 64 aligned to absolute positions, through LDS, both as stored ([key][d]); they
// are loaded from the cache's pages straight into LDS (global_load_lds_dwordx4: no
// staging registers, no LDS stores), two or three tiles deep. With
// v_mfma_f32_32x32x16_bf16 the wave computes
//   S^T[key][q] = K Q^T      (A = K rows from LDS, B = Q held in registers)
// whose accumulator layout gives lane l the scores of query l % 32 for keys
// 8 (v / 4) + 4 (l / 32) + v % 4 of every 32-key block: the softmax of a query
// runs in the two lanes that share l % 32 (one cross-lane step), and the
// probabilities, packed to bf16 in place, are already the B operand of
//   O^T[d][q] += V^T P^T     (A = V^T rows: ds_read_b64_tr_b16 hands a lane four keys of one
//                             dim out of the [key][d] tile, no transposing store needed)
// if the contraction index is numbered the way the lanes hold it; so
// probabilities never leave registers, and the running max and sum of a query
// live in the lanes that hold its output column. Online softmax as in the
// reference's prefill kernel (src/ops/attention.hip:228-241, normalised at the
// end :265), which runs 16 queries x 32 keys per step in scalar FMAs.
// Scores, max, sum and the output accumulator are 32-bit.
//
// A row at position p sees keys lo..p, lo = max(0, p - window + 1). Pages that
// a window has passed may be gone (block-table entry -1): their keys are never
// visible, and the last key's row is loaded in their place.
//
// The same kernel serves decoding for models whose kv heads are shared by three
// or more query heads (HEADS): the 32 "rows" of a block are then the query
// heads of one kv head for one decoded token, all at one position, and the block
// walks one chunk of CHUNK keys and writes its running max, sum and output to the
// workspace, which the decode path's merge kernel adds up. Each key and value is
// then read once for all heads of its group, and the products run on the matrix
// cores instead of one scalar FMA per head, key and dim.
#include "attention.h"
#include "gemm.h"

namespace ninfer {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) short4v lds_short4;

constexpr int PK = 64;   // keys per tile

// Two transposing LDS reads (ds_read_b64_tr_b16) at byte offsets OFF0 and OFF1 from `addr`,
// issued and not waited for: `wait_values` must come before the results are used. They are
// written in assembly because the compiler makes the intrinsic wait for every load into LDS
// that is under way (it cannot tell that those fill other stages); what it does not see it
// does not wait for. LDS operations return in order and only add to the counter the
// compiler's own waits count against, so those stay sufficient.
template <int OFF0, int OFF1>
__device__ __forceinline__ void tr_read2(unsigned addr, short4v& r0, short4v& r1) {
  asm volatile("ds_read_b64_tr_b16 %0, %2 offset:%3\n\tds_read_b64_tr_b16 %1, %2 offset:%4"
               : "=&v"(r0), "=&v"(r1)
               : "v"(addr), "n"(OFF0), "n"(OFF1));
}

template <int D, int NQ, bool HEADS>   // HEADS: rows are the query heads of one token (decode)
__global__ __launch_bounds__(NQ * 128, 2) void attn_prefill_kernel(AttnArgs a, int CHUNK,
                                                                   int paired) {
  constexpr int KH = 2;             // waves per group of 32 rows: each meets one half of a tile's keys
  constexpr int NW = NQ * KH;       // waves
  constexpr int NT = NW * 64;
  constexpr int NKB = 2 / KH;       // 32-key blocks of a tile that one wave meets
  constexpr int PQ = NQ * 32;       // query rows per block
  constexpr int KS = D / 16;        // k-steps of Q K^T
  constexpr int DB = D / 32;        // 32-row blocks of O^T
  // Keys and values lie in LDS as they lie in the cache, [key][d], rows of 2 D bytes without
  // padding: they are loaded from global memory straight into LDS (global_load_lds_dwordx4:
  // no staging registers, no LDS stores), and such a load fills 1 KB of LDS contiguously,
  // lane l at byte 16 l. Bank conflicts of the reads are avoided by a swizzle made on the
  // global side instead: position p of a row's 16-byte chunks holds the row's chunk
  // p ^ swizzle(row), one swizzle for the keys' row-wise reads, another for the values'
  // transposing reads.
  constexpr int ROW_BYTES = 2 * D;
  constexpr int CPR = ROW_BYTES / 16;        // 16-byte chunks of a row
  constexpr int RPP = 64 / CPR;              // rows that one load of a wave fills (1 KB)
  constexpr int TILE_BYTES = PK * ROW_BYTES; // of the keys, and of the values, of a tile
  constexpr int KPT = PK / RPP / NW;         // loads per wave for a tile's keys (as many for its values)
  static_assert(PK % (RPP * NW) == 0, "tile does not divide over the block's waves");
  // Tiles in LDS: the one being multiplied and NST - 1 on their way. Three where one block
  // fills a CU anyway; two for the blocks of four waves, so that two of them fit a CU.
  constexpr int NST = NQ == 4 ? 3 : 2;
  // All LDS reads of a phase are issued before the matrix instructions that need them.
  constexpr bool EARLY = true;
  // All stages lie in one array of dynamic LDS, a tile's keys, then its values, stage after
  // stage; tile_info's three ints and the merge's (max, sum) pairs behind them.
  constexpr int STAGE_BYTES = 2 * TILE_BYTES;
  extern __shared__ __attribute__((aligned(1024))) unsigned char stages[];   // NST x STAGE_BYTES + kPrefillExtra
  // At the end the stages merge the two key halves: the output registers of a group of 32
  // rows' second wave, 16 DB floats per lane stored [register][lane], two groups to a stage.
  static_assert(2 * 16 * DB * 64 * 4 <= STAGE_BYTES && NQ <= 4, "two groups' outputs fit a stage");
  float (*const merge_ml)[64][2] = (float (*)[64][2])(stages + NST * STAGE_BYTES + 16);   // [NQ][64][2]
  int* const tile_info = (int*)(stages + NST * STAGE_BYTES);

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int c = lane & 31, j = lane >> 5;
  // this lane's part in a transposing read of V (see read_values): group lane / 16 holds dims
  // 16 (group % 2) .. + 15 and keys 4 (group / 2) .. + 3
  const int tr_key = 4 * (lane >> 5) + ((lane & 15) >> 2), tr_dim = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
  const int group = a.Hq / a.Hkv;
  int row0, n_rows, seq, g, h, pos_first, pos_last, lo_first, chunk_id = 0;
  if constexpr (HEADS) {
    // grid (kv heads, chunks, rows): heads fastest, so that blocks in flight share pages
    row0 = blockIdx.z;
    g = blockIdx.x;
    chunk_id = blockIdx.y;
    const int pos = min(a.positions[row0], a.max_kv_len - 1);   // as the merge kernel reads it
    const int lo = a.window > 0 ? max(0, pos - a.window + 1) : 0;
    const int c0 = chunk_id * CHUNK;
    if (c0 > pos || c0 + CHUNK <= lo) return;   // chunk outside the row's keys
    n_rows = group;
    seq = a.row_seq[row0];
    h = g * group;                               // the lane's head is h + c
    pos_first = pos;
    pos_last = min(pos, c0 + CHUNK - 1);         // last key this block meets
    lo_first = max(lo, c0);
  } else {
    // Blocks go to the 8 XCDs in turn (block id mod 8) and each XCD has its own L2: ids
    // that are congruent mod 8 get neighbouring work, heads outermost, so that an XCD
    // meets the keys and values of few heads; within a head the later row tiles, which
    // see the most keys, come first.
    const int total = gridDim.x * gridDim.y;
    const int id = blockIdx.x + gridDim.x * blockIdx.y;
    int tile;
    if (paired > 0) {
      // Two blocks fit a CU and all blocks are resident at once: nothing is dealt out later,
      // so what a CU gets at the start decides when it ends. The device deals block ids to
      // the CUs in turn, the first `paired` ids one to each, the rest as their second: id k
      // of the first gets the k-th longest piece of work (later row tiles see more keys),
      // id paired + k the k-th shortest, so that every CU holds about the same.
      const int rank = id < paired ? id : total - 1 - (id - paired);   // 0: the longest
      tile = gridDim.x - 1 - rank / (int)gridDim.y;
      h = rank % (int)gridDim.y;
    } else {
      const int x = id % kXcds, q = total / kXcds, rem8 = total % kXcds;
      const int w = x * q + min(x, rem8) + id / kXcds;   // a bijection: x < rem8 own one id more
      h = w / gridDim.x;
      tile = gridDim.x - 1 - w % gridDim.x;
    }
    if (!find_tile(a.seq_row_start, a.S, PQ, tile, tile_info)) return;
    row0 = tile_info[0];
    seq = tile_info[2];
    g = h / group;
    pos_first = a.positions[row0];               // rows of a request are consecutive
    n_rows = min(PQ, tile_info[1] - row0);
    pos_last = pos_first + n_rows - 1;
    lo_first = a.window > 0 ? max(0, pos_first - a.window + 1) : 0;
  }
  const int* bt = a.block_table + (int64_t)seq * a.bt_stride;
  const bf16* kpool = (const bf16*)a.kpool;
  const bf16* vpool = (const bf16*)a.vpool;
  // the page size divides the tile of 64 keys: a power of two
  const int ps_shift = __builtin_ctz(a.page_size), ps_mask = a.page_size - 1, Hkv = a.Hkv;

  // this lane's query (B operand): row q = qg * 32 + c, dims 16 ks + 8 j .. +7; the wave
  // meets the 32 NKB keys from 32 NKB kh of every tile
  const int qg = wave % NQ, kh = wave / NQ;
  const int q_local = qg * 32 + c;
  const bool q_valid = q_local < n_rows;
  const bool wave_live = qg * 32 < n_rows;    // a wave without rows only helps to load
  const int q_pos = HEADS ? pos_first : pos_first + q_local;
  const int q_lo = HEADS ? lo_first : (a.window > 0 ? max(0, q_pos - a.window + 1) : 0);
  // keys this wave's rows can see: tiles outside are loaded for the others but not multiplied
  const int wave_pos_last = HEADS ? pos_last : pos_first + min(qg * 32 + 31, n_rows - 1);
  const int wave_lo = HEADS ? lo_first
                            : (a.window > 0 ? max(0, pos_first + qg * 32 - a.window + 1) : 0);
  // keys that every row of the wave sees, rows without a query included: a block of keys
  // inside needs no mask
  const int all_see_last = HEADS ? pos_first : pos_first + qg * 32;
  const int all_see_first =
      HEADS ? lo_first : (a.window > 0 ? max(0, pos_first + qg * 32 + 31 - a.window + 1) : 0);
  bf16x8 qf[KS];
  {
    const int ql = q_valid ? q_local : 0;
    const bf16* qr = (const bf16*)a.q + (int64_t)(row0 + (HEADS ? 0 : ql)) * a.q_stride +
                     (h + (HEADS ? ql : 0)) * D + 8 * j;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = *(const bf16x8*)(qr + 16 * ks);
  }

  f32x16 o[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int v = 0; v < 16; ++v) o[db][v] = 0.f;
  // scores are kept in units of log 2, so that a probability is one v_exp_f32
  const float scale2 = a.scale * 1.44269504088896f;
  // a distance-based bias: slope of this lane's head, in units of the unscaled scores (the
  // scale is applied to score + bias together)
  const bool biased = a.slopes != nullptr;
  const float slope_raw = biased ? a.slopes[h + (HEADS ? (q_valid ? q_local : 0) : 0)] / a.scale : 0.f;
  float m = -1e30f, l = 0.f;

  // Loads. Load i of wave w fills piece i NW + w of a tile's keys (and the same piece of its
  // values): RPP rows, lane l at row l / CPR, position l % CPR, which takes the row's chunk
  // (l % CPR) ^ swizzle(row). A key and its value lie at the same place of their pools.
  // Every load is unconditional: for a key that is not there (beyond the last key, or on a
  // page that a window has passed and given back) the row of the last key is loaded in its
  // place. Such a key lies in a block that is masked, and the mask replaces its scores whatever
  // they are; its value must be finite, since its probability is 0 and 0 x NaN is not
  // (pages that were given back may hold anything): the last key's value is.
  typedef const __attribute__((address_space(1))) void* gptr;
  typedef __attribute__((address_space(3))) void* lptr;
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const int l_row = lane / CPR, l_pos = lane % CPR;
  auto k_swizzle = [](int row) { return (row / (16 / CPR)) % CPR; };
  auto v_swizzle = [](int row) { return 4 * ((row / (16 / CPR)) % (CPR / 4)); };
  // A tile starts at a multiple of the page size, so the place of a lane's row inside its
  // page is the same in every tile: address = pool + page * page_stride + in_page + chunk.
  const int64_t page_stride = ((int64_t)Hkv << ps_shift) * D;
  int in_page[KPT], k_chunk[KPT], v_chunk[KPT];   // in elements
#pragma unroll
  for (int i = 0; i < KPT; ++i) {
    const int row = (i * NW + wave_u) * RPP + l_row;
    in_page[i] = (((int64_t)g << ps_shift) + (row & ps_mask)) * D;
    k_chunk[i] = 8 * (l_pos ^ k_swizzle(row));
    v_chunk[i] = 8 * (l_pos ^ v_swizzle(row));
  }
  const int pos_last_u = __builtin_amdgcn_readfirstlane(pos_last);
  const int64_t last_at =
      (int64_t)bt[pos_last >> ps_shift] * page_stride + (((int64_t)g << ps_shift) + (pos_last & ps_mask)) * D;
  // Page numbers, fetched NST tiles ahead of the keys with scalar loads: the rows of one load
  // lie in one page (a page holds at least RPP rows: see attention_prefill_takes), so its
  // number is the same in every lane, and scalar loads do not count among the vector loads
  // that the waits below count. (The table is read through the constant address space, which
  // is what makes the compiler use scalar loads; nothing writes it while the kernel runs.)
  typedef const __attribute__((address_space(4))) int* table_ptr;
  // (the same in every lane, and said so: an address the compiler took for a lane's own
  // would become a vector load, which the waits below would have to count)
  // (the halves go through unsigned: the intrinsic returns an int, and a low half with its top
  // bit set would otherwise widen with ones all over the high half)
  const uintptr_t bt_bits = (uintptr_t)bt;
  const unsigned bt_hi = (unsigned)__builtin_amdgcn_readfirstlane((int)(bt_bits >> 32));
  const unsigned bt_lo = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)bt_bits);
  const table_ptr bt_c = (table_ptr)(((uintptr_t)bt_hi << 32) | (uintptr_t)bt_lo);
  int kpage[NST][KPT];
  auto load_pages = [&](int slot, int t0) {
#pragma unroll
    for (int i = 0; i < KPT; ++i) {
      const int kp = t0 + (i * NW + wave_u) * RPP;   // the load's first row
      kpage[slot][i] = bt_c[__builtin_amdgcn_readfirstlane(min(kp, pos_last_u) >> ps_shift)];   // always a table entry of the request
    }
  };
  // the tile at keys t0.. into stage `buf`, with the page numbers of slot `slot`
  auto issue_tile = [&](int buf, int slot, int t0) {
    unsigned char* kb = stages + buf * STAGE_BYTES + wave_u * 1024;
    unsigned char* vb = kb + TILE_BYTES;
#pragma unroll
    for (int i = 0; i < KPT; ++i) {
      const int page = kpage[slot][i];
      const int kp = t0 + (i * NW + wave_u) * RPP + l_row;
      const int64_t at = (page >= 0 && kp <= pos_last) ? page * page_stride + in_page[i] : last_at;
      // decoding reads every key once a step (marked non-temporal: the last argument); a
      // prompt's keys serve many blocks of rows from L2
      __builtin_amdgcn_global_load_lds((gptr)(kpool + at + k_chunk[i]), (lptr)(kb + i * (NW * 1024)), 16, 0,
                                       HEADS ? 2 : 0);
      __builtin_amdgcn_global_load_lds((gptr)(vpool + at + v_chunk[i]), (lptr)(vb + i * (NW * 1024)), 16, 0,
                                       HEADS ? 2 : 0);
    }
  };

  // This lane's part in the transposing reads of V (see the output products below): its key
  // row tr_key of the wave's 32 keys, dims 32 db + tr_dim .. + 3, as a byte offset into a
  // stage. Rows + 8, + 16 and + 24 have the row's swizzle: constant offsets reach them.
  unsigned v_at[DB];
  {
    const int row = 32 * NKB * kh + tr_key;
#pragma unroll
    for (int db = 0; db < DB; ++db)
      v_at[db] = TILE_BYTES + row * ROW_BYTES + 16 * ((4 * db + tr_dim / 8) ^ v_swizzle(row)) + 2 * (tr_dim % 8);
  }
  // the products of this wave's part of the tile at keys t0.. in LDS buffer buf
  auto multiply = [&](int buf, int t0) {
    const int k0 = t0 + 32 * NKB * kh;
    // not for tiles beyond the last key, or out of sight of every row of the wave
    if (!wave_live || k0 > wave_pos_last || k0 + 32 * NKB <= wave_lo) return;
    const unsigned char* k_s = stages + buf * STAGE_BYTES;
    // Left alone, the compiler reads each fragment from LDS just before the matrix instruction
    // that needs it (it keeps registers few), and that instruction then waits a whole LDS
    // latency: 24 such waits in a row per tile. Where registers allow (EARLY), all reads of a
    // phase are issued first; nothing moves across the asm statement that follows them.
    // S^T = K Q^T : NKB key blocks of 32 x 32 queries
    f32x16 s[NKB];
    bf16x8 kf[NKB][KS];
    auto read_keys = [&](int kb, int ks) {
      const int row = (NKB * kh + kb) * 32 + c;
      kf[kb][ks] = *(const bf16x8*)(k_s + row * ROW_BYTES + 16 * ((2 * ks + j) ^ k_swizzle(row)));
    };
    if constexpr (EARLY) {
#pragma unroll
      for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) read_keys(kb, ks);
      // the first fragment passes through the statement, so the chain begins after it
      asm volatile("" : "+v"(kf[0][0]) : : "memory");
    }
#pragma unroll
    for (int kb = 0; kb < NKB; ++kb) {
#pragma unroll
      for (int v = 0; v < 16; ++v) s[kb][v] = 0.f;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        if constexpr (!EARLY) read_keys(kb, ks);
        s[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[kb][ks], qf[ks], s[kb], 0, 0, 0);
      }
    }
    // The values are read here, while the vector units form the probabilities.
    // The transposing read works in groups of 16 lanes: lane s of a group fetches 8 bytes from
    // an address of its own, and lane i receives element i % 4 of what lanes i / 4 + 4 v
    // fetched, v = 0 .. 3. With lane s at key v = s / 4, dims 4 (s % 4) .. + 3 of the group's
    // 16 dims, lane i gets four consecutive keys of dim i: half of the operand's 8 keys.
    static_assert(NKB == 1, "one block of 32 keys per wave and tile");
    short4v vlo[DB][2], vhi[DB][2];
    {
      const unsigned base = (unsigned)(uintptr_t)(lds_short4*)k_s;
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        tr_read2<0, 8 * ROW_BYTES>(base + v_at[db], vlo[db][0], vhi[db][0]);
        tr_read2<16 * ROW_BYTES, 24 * ROW_BYTES>(base + v_at[db], vlo[db][1], vhi[db][1]);
      }
    }
    // lane holds, for query c, keys k0 + 32 kb + 8 (v / 4) + 4 j + v % 4
    if (biased) {
#pragma unroll
      for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int kp = k0 + 32 * kb + 8 * (v >> 2) + 4 * j + (v & 3);
          s[kb][v] = fmaf(slope_raw, (float)(kp - q_pos), s[kb][v]);
        }
    }
    float mx = -1e30f;
    if (k0 + 32 * NKB - 1 > all_see_last || k0 < all_see_first) {
#pragma unroll
      for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          int kp = k0 + 32 * kb + 8 * (v >> 2) + 4 * j + (v & 3);
          // minus infinity, so that the probability is exactly 0 whatever the row's maximum
          // (the maximum itself starts at -1e30 and stays finite)
          float val = (kp <= q_pos && kp >= q_lo) ? s[kb][v] : -__builtin_inff();
          s[kb][v] = val;
          mx = fmaxf(mx, val);
        }
    } else {
#pragma unroll
      for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
        for (int v = 0; v < 16; ++v) mx = fmaxf(mx, s[kb][v]);
    }
    mx *= scale2;   // the scale is positive: the largest score stays the largest
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    // The reference point m of a row's exponents follows its maximum only in jumps: while the
    // maximum stays within 2^8 of it, probabilities are formed against the old m (they may
    // exceed 1, by up to 2^8: nothing for 32-bit sums or for bf16, which rounds relative to
    // size) and neither the sum nor the 64 output registers are rescaled. The result is the
    // same quotient; at the end the two halves and the chunks are merged by their own m.
    const bool moved = __any(mx > m + 8.f);
    float psum = 0.f;
    if (moved) {
      asm volatile("" ::: "memory");   // a real branch: as selects the products would always run
      const float m_new = fmaxf(m, mx);
      const float alpha = __builtin_amdgcn_exp2f(m - m_new);
      l *= alpha;
#pragma unroll
      for (int db = 0; db < DB; ++db) o[db] *= alpha;
      m = m_new;
    }
    // pf[kb][h]: the 16-key step h of key block kb; slot i of lane j is key 16 h + 8 (i / 4) + 4 j + i % 4
    bf16x8 pf[NKB][2];
#pragma unroll
    for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        float p = __builtin_amdgcn_exp2f(fmaf(s[kb][v], scale2, -m));
        psum += p;
        pf[kb][v >> 3][v & 7] = (__bf16)p;
      }
    l += psum;
    // the values have arrived (every register the reads fill passes through this statement)
    if constexpr (DB == 4)
      asm volatile("s_waitcnt lgkmcnt(0)"
                   : "+v"(vlo[0][0]), "+v"(vhi[0][0]), "+v"(vlo[0][1]), "+v"(vhi[0][1]), "+v"(vlo[1][0]),
                     "+v"(vhi[1][0]), "+v"(vlo[1][1]), "+v"(vhi[1][1]), "+v"(vlo[2][0]), "+v"(vhi[2][0]),
                     "+v"(vlo[2][1]), "+v"(vhi[2][1]), "+v"(vlo[3][0]), "+v"(vhi[3][0]), "+v"(vlo[3][1]),
                     "+v"(vhi[3][1]));
    else
      asm volatile("s_waitcnt lgkmcnt(0)"
                   : "+v"(vlo[0][0]), "+v"(vhi[0][0]), "+v"(vlo[0][1]), "+v"(vhi[0][1]), "+v"(vlo[1][0]),
                     "+v"(vhi[1][0]), "+v"(vlo[1][1]), "+v"(vhi[1][1]));
    static_assert(DB == 4 || DB == 2, "head sizes 128 and 64");
#pragma unroll
    for (int db = 0; db < DB; ++db) {
#pragma unroll
      for (int hs = 0; hs < 2; ++hs) {
        typedef short short8v __attribute__((ext_vector_type(8)));
        const short4v lo4 = vlo[db][hs], hi4 = vhi[db][hs];
        const short8v both = {lo4[0], lo4[1], lo4[2], lo4[3], hi4[0], hi4[1], hi4[2], hi4[3]};
        o[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, both), pf[0][hs], o[db], 0, 0, 0);
      }
    }
  };

  // A wave's loads return in the order of their issue. Per tile it issues 2 KPT loads into
  // LDS (and nothing else that the vector memory counter counts); when tile i is needed, the
  // loads issued after its own are those of the NST - 2 tiles after it.
  constexpr int YOUNGER = (NST - 2) * 2 * KPT;
  const int t_first = (lo_first / PK) * PK;
#pragma unroll
  for (int st = 0; st < NST; ++st) load_pages(st, t_first + st * PK);
#pragma unroll
  for (int st = 0; st + 1 < NST; ++st) {
    issue_tile(st, st, t_first + st * PK);
    load_pages(st, t_first + (NST + st) * PK);
  }
  // NST tiles per turn, so that the stage and the page slot of each are constants. Nothing
  // in the loop stands under a condition: tiles beyond the last key are loaded (the last
  // key's row, over and over) and skipped by the products, so the wait counts exactly the
  // loads issued after the ones it needs.
  for (int t0 = t_first; t0 <= pos_last; t0 += NST * PK) {
#pragma unroll
    for (int u = 0; u < NST; ++u) {
      // this wave's part of tile u has landed; after the barrier everybody's has, and the
      // tile before has been read by every wave (one statement: nothing moves across it)
      asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(YOUNGER) : "memory");
      constexpr int FREE = (NST - 1);   // (u + NST - 1) % NST: the stage of the tile before
      issue_tile((u + FREE) % NST, (u + FREE) % NST, t0 + (u + NST - 1) * PK);
      load_pages((u + FREE) % NST, t0 + (u + 2 * NST - 1) * PK);
      multiply(u, t0 + u * PK);
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // nothing may land in LDS after this
  __syncthreads();

  // Merge the two key halves of every row group: the waves of the second half hand their
  // max, sum and output over through LDS (the last barrier of the loop has freed it).
  float* mine = (float*)(stages + (qg >> 1) * STAGE_BYTES) + (qg & 1) * (16 * DB * 64) + lane;
  if (kh == 1) {
    merge_ml[qg][lane][0] = m;
    merge_ml[qg][lane][1] = l;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int v = 0; v < 16; ++v) mine[(16 * db + v) * 64] = o[db][v];
  }
  __syncthreads();
  if (kh == 1) return;
  float m_all;
  {
    const float m1 = merge_ml[qg][lane][0], l1 = merge_ml[qg][lane][1];
    m_all = fmaxf(m, m1);
    const float a0 = __builtin_amdgcn_exp2f(m - m_all), a1 = __builtin_amdgcn_exp2f(m1 - m_all);
    l = l * a0 + l1 * a1;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int v = 0; v < 16; ++v) o[db][v] = o[db][v] * a0 + mine[(16 * db + v) * 64] * a1;
  }
  // the two lanes of a query hold partial sums of l
  l += __shfl_xor(l, 32, 64);
  if constexpr (HEADS) {
    // the chunk's max (in natural-log units, as the merge kernel takes it), sum and
    // unnormalised output of head h + c
    if (q_valid) {
      float* ws = a.workspace + (((int64_t)row0 * a.Hq + h + c) * gridDim.y + chunk_id) * (D + 2);
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int qd = 0; qd < 4; ++qd) {
          float* dst = ws + db * 32 + 8 * qd + 4 * j;   // D + 2 is even: 8-byte aligned
          *(float2*)dst = make_float2(o[db][4 * qd], o[db][4 * qd + 1]);
          *(float2*)(dst + 2) = make_float2(o[db][4 * qd + 2], o[db][4 * qd + 3]);
        }
      if (j == 0) {
        ws[D] = m_all * 0.693147180559945f;
        ws[D + 1] = l;
      }
    }
    return;
  }
  if (q_valid) {
    // lane holds, of its query's output, dims 32 db + 8 (v / 4) + 4 j + v % 4
    const float inv = 1.f / l;
    bf16* orow = (bf16*)a.out + ((int64_t)(row0 + q_local) * a.Hq + h) * D;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int qd = 0; qd < 4; ++qd) {
        bf16x4 val = {(__bf16)(o[db][4 * qd] * inv), (__bf16)(o[db][4 * qd + 1] * inv),
                      (__bf16)(o[db][4 * qd + 2] * inv), (__bf16)(o[db][4 * qd + 3] * inv)};
        *(bf16x4*)(orow + db * 32 + 8 * qd + 4 * j) = val;
      }
  }
}

// LDS of a block beside its stages: tile_info, then the merge's (max, sum) pairs.
constexpr int kPrefillExtra = 16 + 4 * 64 * 2 * 4;

// Bytes of dynamic LDS of attn_prefill_kernel<D, NQ, .> (as the kernel lays them out).
static size_t prefill_lds(int D, int nq) {
  const int stages = nq == 4 ? 3 : 2;
  return (size_t)stages * 2 * PK * 2 * D + kPrefillExtra;
}

// Pages the matrix-core kernels take: a power of two that divides the tile of 64 keys and
// holds the rows that one load into LDS fills (1 KB: 4 rows of heads of 128, 8 of 64), so
// that a load's rows share their page.
static bool prefill_page_ok(const AttnArgs& a) {
  return PK % a.page_size == 0 && a.page_size * 2 * a.D >= 1024;
}

template <int D, int NQ, bool HEADS>
static int launch_attn(const AttnArgs& a, dim3 grid, int chunk, int paired, hipStream_t stream) {
  auto kern = attn_prefill_kernel<D, NQ, HEADS>;
  const size_t lds = prefill_lds(D, NQ);
  if (lds > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return set_error(-2, "paged_attention: cannot get %zu bytes of LDS", lds);
  }
  kern<<<grid, NQ * 128, lds, stream>>>(a, chunk, paired);
  NINFER_LAUNCH_CHECK();
  return 0;
}

// Decoding with grouped heads: bf16, head size 64 or 128, 3 to 32 query heads per kv head.
bool attention_decode_heads_takes(const AttnArgs& a) {
  const int group = a.Hq / a.Hkv;
  return a.dtype == kBF16 && (a.D == 64 || a.D == 128) && a.q_stride % 8 == 0 &&
         prefill_page_ok(a) && group >= 3 && group <= 32 && a.workspace != nullptr &&
         a.row_seq != nullptr;
}

// Pass 1 of split-context decoding for grouped heads; the caller merges the chunks.
// Blocks of four waves: two multiply (the key halves of the one group of 32 rows), the
// other two only help to load, which keeps each wave's staging registers few.
int attention_decode_heads(const AttnArgs& a, int chunk, int n_chunks, hipStream_t stream) {
  NINFER_REQUIRE(chunk > 0 && chunk % PK == 0, "paged_attention: chunks of %d keys are no "
                 "multiple of %d", chunk, PK);
  dim3 grid(a.Hkv, n_chunks, a.T);
  if (a.D == 128) return launch_attn<128, 2, true>(a, grid, chunk, 0, stream);
  return launch_attn<64, 2, true>(a, grid, chunk, 0, stream);
}

bool attention_prefill_takes(const AttnArgs& a) {
  return a.dtype == kBF16 && (a.D == 64 || a.D == 128) && a.q_stride % 8 == 0 &&
         prefill_page_ok(a) && a.seq_row_start != nullptr;
}

// Row tiles of PQ rows that the launch enumerates (one more per request than whole tiles:
// a request's last tile may be partial; tiles that do not exist exit at once).
static int prefill_tiles(const AttnArgs& a, int pq) { return (a.T + pq - 1) / pq + a.S; }

template <int NQ>
static int launch_prefill(const AttnArgs& a, int paired, hipStream_t stream) {
  constexpr int PQ = NQ * 32;
  dim3 grid(prefill_tiles(a, PQ), a.Hq);
  if (a.D == 128) return launch_attn<128, NQ, false>(a, grid, 0, paired, stream);
  return launch_attn<64, NQ, false>(a, grid, 0, paired, stream);
}

int attention_prefill(const AttnArgs& a, hipStream_t stream) {
  // 128 rows per block when requests bring that many: every key loaded serves more rows.
  // But a causal prompt's row tiles differ in length by their number, and while the 128-row
  // blocks are no more than the CUs, each CU gets at most one and the longest decides (2,048
  // rows of 16 heads: 256 blocks, the last of 16 times the first's length). Blocks of 64 rows
  // fit two to a CU: twice as many, all resident at once, and when they are more than the
  // CUs they are handed out so that every CU holds a long and a short one (measured at 16
  // heads of 128: 40 against 44 us at 2,048 rows, 21.5 against 26 at 1,024, 15 against 18 at
  // 512; from 3,072 rows on the 128-row blocks win, 62 against 70 us).
  const int cus = device_cu_count();
  if (a.max_qlen > 64) {
    // (tiles that hold rows; the launch enumerates a few more, which exit at once)
    const long big = (long)((a.T + 127) / 128) * a.Hq, small = (long)((a.T + 63) / 64) * a.Hq;
    if (big > cus) return launch_prefill<4>(a, 0, stream);
    return launch_prefill<2>(a, small > cus ? cus : 0, stream);
  }
  return launch_prefill<2>(a, 0, stream);
}

}  // namespace ninfer

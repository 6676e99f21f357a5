// Paged attention for prompt portions (bf16) on the matrix cores.
//
// One block owns NQ * 32 consecutive rows of one request and one query head
// (128 or 64 rows: every key and value it loads serves that many). It has
// 2 NQ waves: rows are dealt to NQ groups of 32, and two waves share a group,
// one for the first and one for the second 32 keys of every tile, each with a
// running max, sum and output of its own that are merged at the end. So every
// SIMD holds two waves, and the softmax arithmetic of one overlaps the matrix
// products of the other. Keys and values are walked in tiles of
// 64 aligned to absolute positions, through LDS, both as stored ([key][d]). With
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
// visible and are loaded as zeros.
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

template <int D, int NQ, bool HEADS>   // HEADS: rows are the query heads of one token (decode)
__global__ __launch_bounds__(NQ * 128, 2) void attn_prefill_kernel(AttnArgs a, int CHUNK) {
  constexpr int KH = 2;             // waves per group of 32 rows: each meets one half of a tile's keys
  constexpr int NT = NQ * KH * 64;
  constexpr int NS = 2;              // tiles on their way in registers
  constexpr int NKB = 2 / KH;       // 32-key blocks of a tile that one wave meets
  constexpr int PQ = NQ * 32;       // query rows per block
  constexpr int KS = D / 16;        // k-steps of Q K^T
  constexpr int DB = D / 32;        // 32-row blocks of O^T
  constexpr int KPAD = D + 8;       // bf16 per K row in LDS
  constexpr int VROW = D + 16;      // bf16 per V row in LDS: 32 bytes more than a row, so that the 4 keys x
                                    // 4 dim quads that 16 lanes of a transposing read touch fall on 32 banks
  constexpr int K_TILE = PK * KPAD, V_TILE = PK * VROW;   // bf16 of a tile in LDS
  constexpr bool EARLY = NQ == 4;   // 512 threads stage half as much each: registers to spare
  constexpr int MERGE = 2 + DB * 16 + 1;                   // floats a lane hands over at the end (odd stride)
  constexpr int TILES_BYTES = 2 * (K_TILE + V_TILE) * 2, MERGE_BYTES = NQ * 64 * MERGE * 4;
  // two tiles of each (one read, one written); at the end the same memory merges the two key halves
  __shared__ __attribute__((aligned(16))) unsigned char lds_raw[TILES_BYTES > MERGE_BYTES ? TILES_BYTES : MERGE_BYTES];
  bf16* const k_lds = (bf16*)lds_raw;                  // [2][K_TILE]
  bf16* const vt_lds = k_lds + 2 * K_TILE;             // [2][V_TILE]
  __shared__ int tile_info[3];

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
    const int x = id % kXcds, q = total / kXcds, rem8 = total % kXcds;
    const int w = x * q + min(x, rem8) + id / kXcds;   // a bijection: x < rem8 own one id more
    h = w / gridDim.x;
    const int tile = gridDim.x - 1 - w % gridDim.x;
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
  float m = -1e30f, l = 0.f;

  // global -> LDS mapping, the same for K and V: thread loads 16 bytes (8 dims) of a key's row.
  // Both lie in LDS as they lie in the cache ([key][d]); the output products read V through the
  // transposing LDS read (ds_read_b64_tr_b16), which hands a lane four keys of one dim.
  constexpr int K_VECS = PK * D / 8;                  // 16-byte vectors in a K tile
  constexpr int K_PER_THREAD = (K_VECS + NT - 1) / NT;
  static_assert(K_VECS % NT == 0, "tile does not divide over the block");

  // A tile's keys and values travel global -> registers (stage i % NS) -> LDS. Tile i is
  // multiplied from LDS buffer i % 2 while tile i + 1 moves from its registers to
  // the other buffer, the loads of tile i + 1 + NS are issued into those registers,
  // and the page numbers of tile i + 1 + 2 NS are fetched: no load waits for another
  // inside the loop.
  bf16x8 kreg[NS][K_PER_THREAD], vreg[NS][K_PER_THREAD];
  int kpage[NS][K_PER_THREAD];   // K and V of a key lie at the same place of their pools
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  // Every load below is unconditional (a select replaces what is not there by zeros): a
  // load under a condition would have to be waited for where the condition ends.
  auto load_pages = [&](int st, int t0) {
#pragma unroll
    for (int i = 0; i < K_PER_THREAD; ++i) {
      int kp = t0 + (tid + i * NT) / (D / 8);
      kpage[st][i] = bt[min(kp, pos_last) >> ps_shift];   // always a table entry of the request
    }
  };
  // A tile starts at a multiple of the page size, so the place of a thread's piece inside
  // its page is the same in every tile: address = pool + page * page_stride + in_page.
  const int64_t page_stride = ((int64_t)Hkv << ps_shift) * D;
  int64_t k_in_page[K_PER_THREAD];
#pragma unroll
  for (int i = 0; i < K_PER_THREAD; ++i) {
    const int vec = tid + i * NT;
    k_in_page[i] = (((int64_t)g << ps_shift) + ((vec / (D / 8)) & ps_mask)) * D + 8 * (vec % (D / 8));
  }
  auto load_regs = [&](int st, int t0) {
#pragma unroll
    for (int i = 0; i < K_PER_THREAD; ++i) {
      // For a key that is not there, a row of the last key's page (beyond it) or of the
      // pool's first page (a page given back) is read in its place. Such a key lies in a
      // block that is masked, and the mask replaces its scores whatever they are; its value
      // must be zero: its probability is, but 0 x anything is not.
      const int page = kpage[st][i];
      const int64_t at = max(page, 0) * page_stride + k_in_page[i];
      const int kp = t0 + (tid + i * NT) / (D / 8);
      // decoding reads every key once a step; a prompt's keys serve many blocks of rows from L2
      kreg[st][i] = HEADS ? stream_load((const bf16x8*)(kpool + at)) : *(const bf16x8*)(kpool + at);
      const bf16x8 got = HEADS ? stream_load((const bf16x8*)(vpool + at)) : *(const bf16x8*)(vpool + at);
      vreg[st][i] = (page >= 0 && kp <= pos_last) ? got : zero8;
    }
  };
  auto store_regs = [&](int st, int buf) {
    bf16* k_s = k_lds + buf * K_TILE;
    bf16* v_s = vt_lds + buf * V_TILE;
#pragma unroll
    for (int i = 0; i < K_PER_THREAD; ++i) {
      int vec = tid + i * NT;
      *(bf16x8*)(k_s + (vec / (D / 8)) * KPAD + 8 * (vec % (D / 8))) = kreg[st][i];
      *(bf16x8*)(v_s + (vec / (D / 8)) * VROW + 8 * (vec % (D / 8))) = vreg[st][i];
    }
  };

  // the products of this wave's part of the tile at keys t0.. in LDS buffer buf
  auto multiply = [&](int buf, int t0) {
    const int k0 = t0 + 32 * NKB * kh;
    // not for tiles beyond the last key, or out of sight of every row of the wave
    if (!wave_live || k0 > wave_pos_last || k0 + 32 * NKB <= wave_lo) return;
    const bf16* k_s = k_lds + buf * K_TILE;
    const bf16* vt_s = vt_lds + buf * V_TILE;
    // Left alone, the compiler reads each fragment from LDS just before the matrix instruction
    // that needs it (it keeps registers few), and that instruction then waits a whole LDS
    // latency: 24 such waits in a row per tile. Where registers allow (EARLY), all reads of a
    // phase are issued first; nothing moves across the asm statement that follows them.
    // S^T = K Q^T : NKB key blocks of 32 x 32 queries
    f32x16 s[NKB];
    bf16x8 kf[NKB][KS];
    auto read_keys = [&](int kb, int ks) {
      kf[kb][ks] = *(const bf16x8*)(k_s + ((NKB * kh + kb) * 32 + c) * KPAD + 16 * ks + 8 * j);
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
    // the values: with EARLY read here, while the vector units form the probabilities
    bf16x8 vf[DB][NKB][2];
    // The transposing read works in groups of 16 lanes: lane s of a group fetches 8 bytes from
    // an address of its own, and lane i receives element i % 4 of what lanes i / 4 + 4 v
    // fetched, v = 0 .. 3. With lane s at key v = s / 4, dims 4 (s % 4) .. + 3 of the group's
    // 16 dims, lane i gets four consecutive keys of dim i: half of the operand's 8 keys.
    auto read_values = [&](int db, int kb, int hs) {
      const bf16* vr = vt_s + (32 * (NKB * kh + kb) + 16 * hs + tr_key) * VROW + db * 32 + tr_dim;
      const short4v lo4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4*)vr);
      const short4v hi4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4*)(vr + 8 * VROW));
      typedef short short8v __attribute__((ext_vector_type(8)));
      const short8v both = {lo4[0], lo4[1], lo4[2], lo4[3], hi4[0], hi4[1], hi4[2], hi4[3]};
      vf[db][kb][hs] = __builtin_bit_cast(bf16x8, both);
    };
    if constexpr (EARLY) {
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
          for (int hs = 0; hs < 2; ++hs) read_values(db, kb, hs);
      asm volatile("" ::: "memory");
    }
    // lane holds, for query c, keys k0 + 32 kb + 8 (v / 4) + 4 j + v % 4
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
#pragma unroll
    for (int db = 0; db < DB; ++db) {
#pragma unroll
      for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
        for (int hs = 0; hs < 2; ++hs) {
          if constexpr (!EARLY) read_values(db, kb, hs);
          o[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[db][kb][hs], pf[kb][hs], o[db], 0, 0, 0);
        }
    }
  };

  const int t_first = (lo_first / PK) * PK;
#pragma unroll
  for (int st = 0; st < NS; ++st) load_pages(st, t_first + st * PK);
#pragma unroll
  for (int st = 0; st < NS; ++st) {
    load_regs(st, t_first + st * PK);
    load_pages(st, t_first + (NS + st) * PK);
  }
  store_regs(0, 0);
  load_regs(0, t_first + NS * PK);
  load_pages(0, t_first + 2 * NS * PK);
  lds_barrier();
  // NS tiles per turn, so that the register stage and the buffer of each are constants.
  // Nothing in the loop stands under a condition: tiles beyond the last key are loaded as
  // zeros and skipped by the products, so the wait before a store counts exactly the loads
  // issued after the ones it needs.
  for (int t0 = t_first; t0 <= pos_last; t0 += NS * PK) {
#pragma unroll
    for (int u = 0; u < NS; ++u) {
      const int st = (u + 1) % NS;
      store_regs(st, (u + 1) % 2);
      load_regs(st, t0 + (u + 1 + NS) * PK);
      load_pages(st, t0 + (u + 1 + 2 * NS) * PK);
      multiply(u % 2, t0 + u * PK);
      lds_barrier();   // the next tile is whole, this one has been read by every wave
    }
  }

  // Merge the two key halves of every row group: the waves of the second half hand their
  // max, sum and output over through LDS (the last barrier of the loop has freed it).
  float* mine = (float*)lds_raw + (qg * 64 + lane) * MERGE;
  if (kh == 1) {
    mine[0] = m;
    mine[1] = l;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int v = 0; v < 16; ++v) mine[2 + 16 * db + v] = o[db][v];
  }
  __syncthreads();
  if (kh == 1) return;
  float m_all;
  {
    const float m1 = mine[0], l1 = mine[1];
    m_all = fmaxf(m, m1);
    const float a0 = __builtin_amdgcn_exp2f(m - m_all), a1 = __builtin_amdgcn_exp2f(m1 - m_all);
    l = l * a0 + l1 * a1;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int v = 0; v < 16; ++v) o[db][v] = o[db][v] * a0 + mine[2 + 16 * db + v] * a1;
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

// Decoding with grouped heads: bf16, head size 64 or 128, 3 to 32 query heads per kv head.
bool attention_decode_heads_takes(const AttnArgs& a) {
  const int group = a.Hq / a.Hkv;
  return a.dtype == kBF16 && (a.D == 64 || a.D == 128) && a.q_stride % 8 == 0 &&
         PK % a.page_size == 0 && group >= 3 && group <= 32 && a.workspace != nullptr &&
         a.row_seq != nullptr;
}

// Pass 1 of split-context decoding for grouped heads; the caller merges the chunks.
// Blocks of four waves: two multiply (the key halves of the one group of 32 rows), the
// other two only help to load, which keeps each wave's staging registers few.
int attention_decode_heads(const AttnArgs& a, int chunk, int n_chunks, hipStream_t stream) {
  NINFER_REQUIRE(chunk > 0 && chunk % PK == 0, "paged_attention: chunks of %d keys are no "
                 "multiple of %d", chunk, PK);
  dim3 grid(a.Hkv, n_chunks, a.T);
  if (a.D == 128)
    attn_prefill_kernel<128, 2, true><<<grid, 256, 0, stream>>>(a, chunk);
  else
    attn_prefill_kernel<64, 2, true><<<grid, 256, 0, stream>>>(a, chunk);
  NINFER_LAUNCH_CHECK();
  return 0;
}

bool attention_prefill_takes(const AttnArgs& a) {
  return a.dtype == kBF16 && (a.D == 64 || a.D == 128) && a.q_stride % 8 == 0 &&
         PK % a.page_size == 0 && a.seq_row_start != nullptr;
}

template <int NQ>
static int launch_prefill(const AttnArgs& a, hipStream_t stream) {
  constexpr int PQ = NQ * 32;
  dim3 grid((a.T + PQ - 1) / PQ + a.S, a.Hq);
  if (a.D == 128)
    attn_prefill_kernel<128, NQ, false><<<grid, NQ * 128, 0, stream>>>(a, 0);
  else
    attn_prefill_kernel<64, NQ, false><<<grid, NQ * 128, 0, stream>>>(a, 0);
  NINFER_LAUNCH_CHECK();
  return 0;
}

int attention_prefill(const AttnArgs& a, hipStream_t stream) {
  // 128 rows per block when requests bring that many: every key loaded serves more rows
  if (a.max_qlen > 64) return launch_prefill<4>(a, stream);
  return launch_prefill<2>(a, stream);
}

}  // namespace ninfer

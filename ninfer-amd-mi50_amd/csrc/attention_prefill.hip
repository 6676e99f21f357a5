// Paged attention for prompt portions (bf16) on the matrix cores.
//
// One block of 4 waves owns 64 consecutive rows of one request and one query
// head; each wave owns 16 of the rows. Keys and values are walked in tiles of
// 64 aligned to absolute positions, through LDS: K as stored ([key][d]), V
// transposed ([d][key]) so that both products read their contraction index
// contiguously. With v_mfma_f32_16x16x32_bf16 the wave computes
//   S^T[key][q] = K Q^T      (A = K rows from LDS, B = Q held in registers)
// whose accumulator layout gives lane l the scores of query l % 16 for keys
// 4 (l / 16) + v of every 16-key block: the softmax of a query runs in the four
// lanes that share l % 16 (two cross-lane steps), and the probabilities, packed
// to bf16 in place, are already the B operand of
//   O^T[d][q] += V^T P^T     (A = V^T rows from LDS)
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
#include "attention.h"
#include "gemm.h"

namespace ninfer {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int PQ = 64;   // query rows per block
constexpr int PK = 64;   // keys per tile

template <int D>
__global__ __launch_bounds__(256) void attn_prefill_kernel(AttnArgs a) {
  constexpr int KS = D / 32;        // k-steps of Q K^T
  constexpr int DB = D / 16;        // 16-row blocks of O^T
  constexpr int KPAD = D + 8;       // bf16 per K row in LDS
  constexpr int VPAD = PK + 8;      // bf16 per V^T row in LDS
  __shared__ __attribute__((aligned(16))) bf16 k_s[PK * KPAD];
  __shared__ __attribute__((aligned(16))) bf16 vt_s[D * VPAD];
  __shared__ int tile_info[3];

  if (!find_tile(a.seq_row_start, a.S, PQ, blockIdx.x, tile_info)) return;
  const int row0 = tile_info[0], row_end = tile_info[1], seq = tile_info[2];
  const int h = blockIdx.y;
  const int g = h / (a.Hq / a.Hkv);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int c = lane & 15, j = lane >> 4;

  const int pos_first = a.positions[row0];               // rows of a request are consecutive
  const int n_rows = min(PQ, row_end - row0);
  const int pos_last = pos_first + n_rows - 1;
  const int lo_first = a.window > 0 ? max(0, pos_first - a.window + 1) : 0;
  const int* bt = a.block_table + (int64_t)seq * a.bt_stride;
  const bf16* kpool = (const bf16*)a.kpool;
  const bf16* vpool = (const bf16*)a.vpool;
  const int ps = a.page_size, Hkv = a.Hkv;

  // this lane's query (B operand): row q = wave * 16 + c, dims 32 ks + 8 j .. +7
  const int q_local = wave * 16 + c;
  const bool q_valid = q_local < n_rows;
  const int q_pos = pos_first + q_local;
  const int q_lo = a.window > 0 ? max(0, q_pos - a.window + 1) : 0;
  bf16x8 qf[KS];
  {
    const bf16* qr = (const bf16*)a.q + (int64_t)(row0 + (q_valid ? q_local : 0)) * a.q_stride +
                     h * D + 8 * j;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = *(const bf16x8*)(qr + 32 * ks);
  }

  f32x4 o[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db) o[db] = (f32x4){0.f, 0.f, 0.f, 0.f};
  float m = -1e30f, l = 0.f;

  // global -> LDS mapping. K: thread loads 16 bytes (8 dims) of a key row.
  // V: thread loads a 4-key x 8-dim block and stores it transposed.
  constexpr int K_VECS = PK * D / 8;                  // 16-byte vectors in a K tile
  constexpr int K_PER_THREAD = K_VECS / 256;
  constexpr int V_BLOCKS = (PK / 4) * (D / 8);        // 4 x 8 blocks in a V tile
  static_assert(K_VECS % 256 == 0, "tile does not divide over the block");

  // A tile's keys and values travel global -> registers -> LDS; the next
  // tile's loads are issued before the products of the current one.
  constexpr int V_PER_THREAD = (V_BLOCKS + 255) / 256;
  bf16x8 kreg[2][K_PER_THREAD], vreg[2][V_PER_THREAD][4];
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  auto load_regs = [&](int st, int t0) {
#pragma unroll
    for (int i = 0; i < K_PER_THREAD; ++i) {
      int vec = tid + i * 256;
      int key = vec / (D / 8), dv = vec % (D / 8);
      int kp = t0 + key;
      kreg[st][i] = zero8;
      if (kp <= pos_last) {
        int page = bt[kp / ps];
        if (page >= 0)
          kreg[st][i] = *(const bf16x8*)(kpool + (((int64_t)page * Hkv + g) * ps + kp % ps) * D + 8 * dv);
      }
    }
#pragma unroll
    for (int i = 0; i < V_PER_THREAD; ++i) {
      int blk = tid + i * 256;
      int kg = blk % (PK / 4), dv = blk / (PK / 4);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        int kp = t0 + 4 * kg + r;
        vreg[st][i][r] = zero8;
        if (blk < V_BLOCKS && kp <= pos_last) {
          int page = bt[kp / ps];
          if (page >= 0)
            vreg[st][i][r] = *(const bf16x8*)(vpool + (((int64_t)page * Hkv + g) * ps + kp % ps) * D + 8 * dv);
        }
      }
    }
  };
  auto store_regs = [&](int st) {
#pragma unroll
    for (int i = 0; i < K_PER_THREAD; ++i) {
      int vec = tid + i * 256;
      *(bf16x8*)(k_s + (vec / (D / 8)) * KPAD + 8 * (vec % (D / 8))) = kreg[st][i];
    }
#pragma unroll
    for (int i = 0; i < V_PER_THREAD; ++i) {
      int blk = tid + i * 256;
      if (blk < V_BLOCKS) {
        int kg = blk % (PK / 4), dv = blk / (PK / 4);
#pragma unroll
        for (int d = 0; d < 8; ++d) {
          bf16x4 col = {vreg[st][i][0][d], vreg[st][i][1][d], vreg[st][i][2][d], vreg[st][i][3][d]};
          *(bf16x4*)(vt_s + (8 * dv + d) * VPAD + 4 * kg) = col;
        }
      }
    }
  };

  // Tiles alternate between two register stages: the loads of tile t + 2 are
  // issued as soon as tile t has moved to LDS, and are consumed two tiles later.
  auto tile = [&](int st, int t0) {
    lds_barrier();   // the previous tile has been consumed
    store_regs(st);
    lds_barrier();
    if (t0 + 2 * PK <= pos_last) load_regs(st, t0 + 2 * PK);

    // S^T = K Q^T : 4 key blocks of 16
    f32x4 s[4];
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
      s[kb] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        bf16x8 kf = *(const bf16x8*)(k_s + (kb * 16 + c) * KPAD + 32 * ks + 8 * j);
        s[kb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[ks], s[kb], 0, 0, 0);
      }
    }
    // lane holds, for query c, keys t0 + 16 kb + 4 j + v
    float mx = -1e30f;
#pragma unroll
    for (int kb = 0; kb < 4; ++kb)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        int kp = t0 + 16 * kb + 4 * j + v;
        float val = (kp <= q_pos && kp >= q_lo) ? s[kb][v] * a.scale : -1e30f;
        s[kb][v] = val;
        mx = fmaxf(mx, val);
      }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m, mx);
    const float alpha = __expf(m - m_new);
    float psum = 0.f;
    bf16x8 pf[2];
#pragma unroll
    for (int kb = 0; kb < 4; ++kb)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        float p = __expf(s[kb][v] - m_new);
        psum += p;
        pf[kb >> 1][(kb & 1) * 4 + v] = (__bf16)p;
      }
    l = l * alpha + psum;
    m = m_new;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      o[db] *= alpha;
      // contraction slot (j, i): key 32 ks + 4 j + i for i < 4, 32 ks + 16 + 4 j + i - 4 else
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        const bf16* vr = vt_s + (db * 16 + c) * VPAD + 32 * ks + 4 * j;
        bf16x4 lo4 = *(const bf16x4*)vr;
        bf16x4 hi4 = *(const bf16x4*)(vr + 16);
        bf16x8 vf = {lo4[0], lo4[1], lo4[2], lo4[3], hi4[0], hi4[1], hi4[2], hi4[3]};
        o[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf[ks], o[db], 0, 0, 0);
      }
    }
  };
  const int t_first = (lo_first / PK) * PK;
  load_regs(0, t_first);
  if (t_first + PK <= pos_last) load_regs(1, t_first + PK);
  for (int t0 = t_first; t0 <= pos_last; t0 += 2 * PK) {
    tile(0, t0);
    if (t0 + PK <= pos_last) tile(1, t0 + PK);
  }

  // the four lanes of a query hold partial sums of l
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);
  if (q_valid) {
    const float inv = 1.f / l;
    bf16* orow = (bf16*)a.out + ((int64_t)(row0 + q_local) * a.Hq + h) * D;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      bf16x4 val = {(__bf16)(o[db][0] * inv), (__bf16)(o[db][1] * inv), (__bf16)(o[db][2] * inv),
                    (__bf16)(o[db][3] * inv)};
      *(bf16x4*)(orow + db * 16 + 4 * j) = val;
    }
  }
}

bool attention_prefill_takes(const AttnArgs& a) {
  return a.dtype == kBF16 && (a.D == 64 || a.D == 128) && a.q_stride % 8 == 0 &&
         PK % a.page_size == 0 && a.seq_row_start != nullptr;
}

int attention_prefill(const AttnArgs& a, hipStream_t stream) {
  dim3 grid((a.T + PQ - 1) / PQ + a.S, a.Hq);
  if (a.D == 128)
    attn_prefill_kernel<128><<<grid, 256, 0, stream>>>(a);
  else
    attn_prefill_kernel<64><<<grid, 256, 0, stream>>>(a);
  NINFER_LAUNCH_CHECK();
  return 0;
}

}  // namespace ninfer

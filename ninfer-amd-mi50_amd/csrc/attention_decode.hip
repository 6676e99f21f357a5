// Paged attention for decode rows (bf16): the context of every row is split
// into chunks of keys that different blocks walk at the same time
// (flash-decoding), then a second kernel merges the chunks. The reference
// walks the whole context in one block per head with a serial softmax tail
// (src/ops/attention.hip:14-94); at long context and small batch that leaves
// most of the GPU idle.
//
// Pass 1, grid (kv heads x head groups, chunks, rows), 4 waves per block: blocks that start
// together read the heads of the same pages, which lie side by side in the pool. A
// key row of D = 8 LPK elements is read by LPK adjacent lanes, 16 bytes each,
// so one wave instruction fetches 64 / LPK whole keys, contiguous in the page.
// The dot product is reduced over those LPK lanes; each lane group keeps its
// own online softmax (m, l, acc) over the keys it sees, for up to GQ query
// heads that share the kv head, so keys and values are read once for all of
// them. Lane groups, then waves, are merged by the usual log-sum-exp rule and
// the chunk's (m, l, acc) goes to the workspace.
// Pass 2, grid (rows, query heads): merges the chunks of a row in a fixed order.
// With three or more query heads per kv head (and heads of 64 or 128), pass 1 is the
// matrix-core kernel of attention_prefill.hip with the heads of a kv head as its rows;
// it writes the same (m, l, acc) per chunk, and pass 2 is the same.
//
// Scores, softmax and sums are 32-bit. A row sees keys lo..pos with
// lo = max(0, pos - window + 1); chunks are aligned to absolute positions.
#include "attention.h"

namespace ninfer {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr int kDecWaves = 4;

// Keys per block: 128, or 256 above 24 blocks a CU. Blocks live long (all of a CU's share
// the CU's part of the memory system), so with few rounds of them the last ones to finish
// leave the device half empty for a while, and shorter blocks end more evenly: 8 rows x 8,192
// keys take 82 us with 128 keys a block against 85 to 87 with 256, and the step 1.5% less
// (4,991 to 5,025 against 5,064 to 5,104 us in one process). From 16 rows on the larger
// blocks win the step (7,964 to 7,975 against 8,003 to 8,098 us; 64 rows: 633 against 651 us
// a layer: half the partial results to write and merge). At 24 blocks a CU: 8 rows x 12,288
// keys 6,005 to 6,011 us a step against 6,058, 12 rows x 8,192 the same; at 32 (8 x 16,384)
// the larger blocks by 1%.
static int decode_chunk(int T, int Hkv, int max_kv_len) {
  long blocks = (long)T * Hkv * ((max_kv_len + 255) / 256);
  return blocks <= 24L * device_cu_count() ? 128 : 256;
}

__device__ __forceinline__ void cvt8(const bf16x8& v, float* f) {
#pragma unroll
  for (int i = 0; i < 8; ++i) f[i] = (float)v[i];
}

template <int LPK, int GQ, int kChunk>
__global__ __launch_bounds__(kDecWaves * 64) void attn_decode_kernel(AttnArgs a, int head_groups) {
  constexpr int D = 8 * LPK;
  constexpr int KPI = 64 / LPK;             // keys per wave instruction
  constexpr int KEYS_PER_WAVE = kChunk / kDecWaves;
  constexpr int ITERS = KEYS_PER_WAVE / KPI;
  constexpr int UNROLL = ITERS >= 4 ? 4 : ITERS;
  __shared__ float merge[kDecWaves][GQ][D + 2];

  const int t = blockIdx.z;
  const int g = blockIdx.x / head_groups;            // kv head
  const int hg = blockIdx.x % head_groups;           // which GQ-group of its query heads
  const int group = a.Hq / a.Hkv;
  const int h0 = g * group + hg * GQ;                // first query head of this block
  const int n_heads = min(GQ, group - hg * GQ);
  // (a position beyond the host's bound max_kv_len would index past the chunks the launch
  // and the workspace were sized for: it is read as the last position inside the bound)
  const int pos = min(a.positions[t], a.max_kv_len - 1);
  const int lo = a.window > 0 ? max(0, pos - a.window + 1) : 0;
  const int chunk_id = blockIdx.y;
  const int c0 = chunk_id * kChunk;
  if (c0 > pos || c0 + kChunk <= lo) return;          // chunk outside the row's keys
  const int n_chunks = gridDim.y;

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int sub = lane % LPK, kslot = lane / LPK;
  const int* bt = a.block_table + (int64_t)a.row_seq[t] * a.bt_stride;
  const bf16* kpool = (const bf16*)a.kpool;
  const bf16* vpool = (const bf16*)a.vpool;
  // the page size is a power of two (attention_decode_takes)
  const int ps_shift = __builtin_ctz(a.page_size), ps_mask = a.page_size - 1, Hkv = a.Hkv;

  float q[GQ][8];
#pragma unroll
  for (int i = 0; i < GQ; ++i) {
    if (i < n_heads) {
      bf16x8 v = *(const bf16x8*)((const bf16*)a.q + (int64_t)t * a.q_stride + (h0 + i) * D + 8 * sub);
      cvt8(v, q[i]);
#pragma unroll
      for (int d = 0; d < 8; ++d) q[i][d] *= a.scale;
    } else {
#pragma unroll
      for (int d = 0; d < 8; ++d) q[i][d] = 0.f;
    }
  }
  // a distance-based bias on the scores: slope of each of the block's heads (0: none)
  float slope[GQ];
#pragma unroll
  for (int i = 0; i < GQ; ++i) slope[i] = a.slopes && i < n_heads ? a.slopes[h0 + i] : 0.f;
  float m[GQ], l[GQ], acc[GQ][8];
#pragma unroll
  for (int i = 0; i < GQ; ++i) {
    m[i] = -1e30f;
    l[i] = 0.f;
#pragma unroll
    for (int d = 0; d < 8; ++d) acc[i][d] = 0.f;
  }

  // Every load is unconditional: a key outside lo..pos is read at the nearest key inside
  // (a page the request holds) and its values are not used. First the page numbers of all
  // the wave's keys, then keys and values, none waiting for another.
  const int wbase = c0 + wave * KEYS_PER_WAVE;
  int64_t koff[ITERS];
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int j = min(max(wbase + it * KPI + kslot, lo), pos);
    const int page = bt[j >> ps_shift];
    koff[it] = ((((int64_t)page * Hkv + g) << ps_shift) + (j & ps_mask)) * D + 8 * sub;
  }
#pragma unroll
  for (int it0 = 0; it0 < ITERS; it0 += UNROLL) {
    bf16x8 kf[UNROLL], vf[UNROLL];
    bool ok[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int j = wbase + (it0 + u) * KPI + kslot;
      ok[u] = j >= lo && j <= pos;
      kf[u] = stream_load((const bf16x8*)(kpool + koff[it0 + u]));
      vf[u] = stream_load((const bf16x8*)(vpool + koff[it0 + u]));
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const float dist = (float)(wbase + (it0 + u) * KPI + kslot - pos);   // key's position - row's
      float kk[8], vv[8];
      if (ok[u]) {
        cvt8(kf[u], kk);
        cvt8(vf[u], vv);
      } else {
#pragma unroll
        for (int d = 0; d < 8; ++d) kk[d] = vv[d] = 0.f;
      }
#pragma unroll
      for (int i = 0; i < GQ; ++i) {
        float s = 0.f;
#pragma unroll
        for (int d = 0; d < 8; ++d) s = fmaf(q[i][d], kk[d], s);
#pragma unroll
        for (int off = LPK / 2; off > 0; off >>= 1) s += __shfl_xor(s, off, 64);
        s = fmaf(slope[i], dist, s);
        if (ok[u]) {
          float m_new = fmaxf(m[i], s);
          float alpha = __expf(m[i] - m_new);
          float p = __expf(s - m_new);
          l[i] = l[i] * alpha + p;
#pragma unroll
          for (int d = 0; d < 8; ++d) acc[i][d] = fmaf(p, vv[d], acc[i][d] * alpha);
          m[i] = m_new;
        }
      }
    }
  }

  // merge the KPI lane groups of the wave
#pragma unroll
  for (int i = 0; i < GQ; ++i) {
#pragma unroll
    for (int off = LPK; off < 64; off <<= 1) {
      float om = __shfl_xor(m[i], off, 64);
      float ol = __shfl_xor(l[i], off, 64);
      float m_new = fmaxf(m[i], om);
      float sa = __expf(m[i] - m_new), sb = __expf(om - m_new);
      l[i] = l[i] * sa + ol * sb;
#pragma unroll
      for (int d = 0; d < 8; ++d) {
        float oa = __shfl_xor(acc[i][d], off, 64);
        acc[i][d] = acc[i][d] * sa + oa * sb;
      }
      m[i] = m_new;
    }
    if (kslot == 0) {
#pragma unroll
      for (int d = 0; d < 8; ++d) merge[wave][i][8 * sub + d] = acc[i][d];
      if (sub == 0) {
        merge[wave][i][D] = m[i];
        merge[wave][i][D + 1] = l[i];
      }
    }
  }
  __syncthreads();
  // merge the waves; one thread per (head, dim)
  for (int e = threadIdx.x; e < n_heads * D; e += blockDim.x) {
    int i = e / D, d = e % D;
    float mm = merge[0][i][D];
#pragma unroll
    for (int w = 1; w < kDecWaves; ++w) mm = fmaxf(mm, merge[w][i][D]);
    float ll = 0.f, aa = 0.f;
#pragma unroll
    for (int w = 0; w < kDecWaves; ++w) {
      float sc = __expf(merge[w][i][D] - mm);
      ll += merge[w][i][D + 1] * sc;
      aa += merge[w][i][d] * sc;
    }
    float* ws = a.workspace + (((int64_t)t * a.Hq + h0 + i) * n_chunks + chunk_id) * (D + 2);
    ws[d] = aa;
    if (d == 0) {
      ws[D] = mm;
      ws[D + 1] = ll;
    }
  }
}

// out[t, h, :] = sum_c acc_c exp(m_c - M) / sum_c l_c exp(m_c - M).
// Block of 512 threads: the chunks' m and l come in with one round of loads and stay in
// LDS; then thread (d, part) sums the chunks c = part mod parts of dim d, all loads in
// flight at once, and the parts are added in part order (fixed, so the result does not
// depend on timing).
constexpr int kMergeThreads = 512;

__global__ __launch_bounds__(kMergeThreads) void attn_decode_merge_kernel(AttnArgs a, int n_chunks,
                                                                         int kChunk) {
  extern __shared__ float merge_s[];   // [n_chunks] scale, [n_chunks] l, [kMergeThreads] partial sums
  float* scale_s = merge_s;
  float* l_s = merge_s + n_chunks;
  float* part_s = merge_s + 2 * n_chunks;
  __shared__ float red[2 * kMergeThreads / 64];
  const int t = blockIdx.x, h = blockIdx.y, D = a.D, tid = threadIdx.x;
  const int pos = min(a.positions[t], a.max_kv_len - 1);   // as in pass 1: never past n_chunks
  const int lo = a.window > 0 ? max(0, pos - a.window + 1) : 0;
  const int c_lo = lo / kChunk, c_hi = min(pos / kChunk, n_chunks - 1);
  const float* ws = a.workspace + ((int64_t)t * a.Hq + h) * n_chunks * (D + 2);
  float mx = -1e30f;
  for (int c = c_lo + tid; c <= c_hi; c += kMergeThreads) {
    const float m = ws[c * (D + 2) + D], l = ws[c * (D + 2) + D + 1];
    scale_s[c] = m;
    l_s[c] = l;
    mx = fmaxf(mx, m);
  }
  mx = wave_max(mx);
  if ((tid & 63) == 0) red[tid >> 6] = mx;
  __syncthreads();
  float M = red[0];
#pragma unroll
  for (int w = 1; w < kMergeThreads / 64; ++w) M = fmaxf(M, red[w]);
  float lsum = 0.f;
  for (int c = c_lo + tid; c <= c_hi; c += kMergeThreads) {
    const float sc = __expf(scale_s[c] - M);
    scale_s[c] = sc;
    lsum += l_s[c] * sc;
  }
  lsum = wave_sum(lsum);
  if ((tid & 63) == 0) red[kMergeThreads / 64 + (tid >> 6)] = lsum;
  __syncthreads();
  float total = 0.f;
#pragma unroll
  for (int w = 0; w < kMergeThreads / 64; ++w) total += red[kMergeThreads / 64 + w];
  const int parts = kMergeThreads / D;          // D <= 256: at least 2
  const int d = tid % D, part = tid / D;
  float acc = 0.f;
  if (part < parts) {
#pragma unroll 8
    for (int c = c_lo + part; c <= c_hi; c += parts) acc = fmaf(ws[c * (D + 2) + d], scale_s[c], acc);
  }
  part_s[tid] = acc;
  __syncthreads();
  if (tid < D) {
    float sum = 0.f;
    for (int p = 0; p < parts; ++p) sum += part_s[p * D + tid];
    ((bf16*)a.out)[((int64_t)t * a.Hq + h) * D + tid] = __float2bfloat16(sum / total);
  }
}

int64_t attention_decode_workspace_floats(int T, int Hq, int D, int max_kv_len) {
  int n_chunks = (max_kv_len + 127) / 128;   // the smaller chunk size bounds the need
  return (int64_t)T * Hq * n_chunks * (D + 2);
}

bool attention_decode_takes(const AttnArgs& a) {
  int d = a.D;
  bool d_ok = d == 16 || d == 32 || d == 64 || d == 128 || d == 256;
  bool ps_ok = (a.page_size & (a.page_size - 1)) == 0;
  return a.dtype == kBF16 && d_ok && ps_ok && a.q_stride % 8 == 0 && a.workspace != nullptr;
}

template <int LPK, int CHUNK>
static void launch_decode(const AttnArgs& a, int n_chunks, hipStream_t stream) {
  int group = a.Hq / a.Hkv;
  dim3 block(kDecWaves * 64);
  if (group == 1) {
    attn_decode_kernel<LPK, 1, CHUNK><<<dim3(a.Hkv, n_chunks, a.T), block, 0, stream>>>(a, 1);
  } else if (group == 2) {
    attn_decode_kernel<LPK, 2, CHUNK><<<dim3(a.Hkv, n_chunks, a.T), block, 0, stream>>>(a, 1);
  } else {
    int hg = (group + 3) / 4;
    attn_decode_kernel<LPK, 4, CHUNK><<<dim3(a.Hkv * hg, n_chunks, a.T), block, 0, stream>>>(a, hg);
  }
}

template <int LPK>
static void launch_decode_chunk(const AttnArgs& a, int chunk, int n_chunks, hipStream_t stream) {
  if (chunk == 128)
    launch_decode<LPK, 128>(a, n_chunks, stream);
  else
    launch_decode<LPK, 256>(a, n_chunks, stream);
}

// Which pass-1 kernel a decode step runs and how it cuts the contexts: the matrix-core
// kernel for grouped heads (`heads`) or the scalar one, chunks of `chunk` keys.
void attention_decode_plan(const AttnArgs& a, bool* heads, int* chunk, int* n_chunks) {
  *heads = attention_decode_heads_takes(a);
  *chunk = decode_chunk(a.T, a.Hkv, a.max_kv_len);
  if (*heads) {
    // the matrix-core kernel has a start-up of several tiles: the largest chunk that still
    // gives every CU two blocks
    *chunk = 128;
    for (int c = 1024; c > 128; c /= 2)
      if ((long)a.T * a.Hkv * ((a.max_kv_len + c - 1) / c) >= 2L * device_cu_count()) {
        *chunk = c;
        break;
      }
  }
  *n_chunks = (a.max_kv_len + *chunk - 1) / *chunk;
}

int attention_decode(const AttnArgs& a, hipStream_t stream) {
  bool heads;
  int chunk, n_chunks;
  attention_decode_plan(a, &heads, &chunk, &n_chunks);
  NINFER_REQUIRE(a.workspace_floats >= attention_decode_workspace_floats(a.T, a.Hq, a.D, a.max_kv_len),
                 "paged_attention: workspace of %lld floats is too small", (long long)a.workspace_floats);
  const size_t merge_lds = (2 * (size_t)n_chunks + kMergeThreads) * sizeof(float);
  NINFER_REQUIRE(merge_lds <= 48 * 1024, "paged_attention: a context of %d keys has too many chunks to merge",
                 a.max_kv_len);
  if (heads) {
    // three or more query heads per kv head: their products go to the matrix cores
    if (int rc = attention_decode_heads(a, chunk, n_chunks, stream)) return rc;
  } else {
    switch (a.D) {
      case 16: launch_decode_chunk<2>(a, chunk, n_chunks, stream); break;
      case 32: launch_decode_chunk<4>(a, chunk, n_chunks, stream); break;
      case 64: launch_decode_chunk<8>(a, chunk, n_chunks, stream); break;
      case 128: launch_decode_chunk<16>(a, chunk, n_chunks, stream); break;
      case 256: launch_decode_chunk<32>(a, chunk, n_chunks, stream); break;
      default: return set_error(-1, "paged_attention: decode kernel does not take head size %d", a.D);
    }
  }
  NINFER_LAUNCH_CHECK();
  attn_decode_merge_kernel<<<dim3(a.T, a.Hq), kMergeThreads, merge_lds, stream>>>(a, n_chunks, chunk);
  NINFER_LAUNCH_CHECK();
  return 0;
}

}  // namespace ninfer

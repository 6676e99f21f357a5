// C = A W^T (+ bias) for a dense product of 33 to 64 rows: every weight is read once from
// HBM, as in the few-row kernel (gemm_skinny.hip), and meets all the rows in the block that
// read it.
//
// The few-row kernel gives every 16 rows of A a block of their own, which reads the weights
// again (from L2, but with all of a block's fixed work); the tile kernels want many rows per
// weight to pay for their tiles. Between them a block here owns 32 output features (FG = 2
// groups of 16) and all the rows: RT row tiles of 16, each with an accumulator of its own,
// multiplied by the same weight fragment. The K range is split over the block's 8 waves, each a contiguous
// part walked in chunks of 128; weights are loaded as whole 128-byte lines, non-temporal,
// and reach the matrix instruction's layout through 2 KB of LDS per wave; activations come
// straight from global memory (64 rows stay in cache). Partial tiles meet in LDS and are
// summed in wave order, so a row's result depends neither on timing nor on the other rows.
//
// Every block reads all of A (from L2): twice the bytes of its weights at 64 rows. Measured
// against the library's kernels in a replayed decode step of 64 rows: 6144 features of K =
// 2048 15.2 against 13.2 us; 2048 features (16 features a block, 128 blocks) 18.7 against
// 12.0 (K = 2048) and 18.5 (K = 5632); 151,936 features 244 us (the activations' 1.2 GB from
// L2 bound it). On the device the library's kernels are the faster ones, then; but a launch
// here costs the host 3 us and the library's call 18, and the steps that bring 33 to 64
// rows eagerly (short prompt portions, portions beside decoded tokens) are bound by the
// host: 4.9 against 5.3 ms with the qkv product here, replayed decode steps of 40 to 64 rows
// the same within 0.3%. So the kernel takes products of 4,096 to 32,768 features, where its
// blocks fill the device and the activations' traffic stays small; the others stay with the
// library. The reference sends all products of this size to the library
// (src/ops/linear.hip:21-35).
#include "gemm.h"

namespace ninfer {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kRowsWaves = 8;
constexpr int kRowsMinFeatures = 4096, kRowsMaxFeatures = 32768;

template <int RT, int FG, typename TC>
__global__ __launch_bounds__(kRowsWaves * 64) void gemm_skinny_rows_kernel(GemmArgs a) {
  // partial tiles: [wave][feature group][row tile][token 16][feature 16]; the first bytes
  // are the waves' 2 KB each of weight lines while the K range is walked
  __shared__ __attribute__((aligned(16))) float red[kRowsWaves * FG * RT * 256];
  unsigned char* stage = (unsigned char*)red;
  static_assert(FG * RT * 1024 >= 2048, "the weight lines fit in the partial tiles' memory");
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, j = lane >> 4;
  const int n0 = blockIdx.x * 16 * FG, K = a.K;
  const bf16* W = (const bf16*)a.W;
  // weights as the loads see them: lane l reads 16 bytes of row 8 q + l / 8 at byte
  // 16 (l % 8) of a 128-byte piece
  const bf16* wline[FG][2];
#pragma unroll
  for (int s = 0; s < FG; ++s)
#pragma unroll
    for (int q = 0; q < 2; ++q)
      wline[s][q] = W + (int64_t)(n0 + 16 * s + 8 * q + (lane >> 3)) * K + 8 * (lane & 7);
  // activations as the matrix instruction wants them: lane (r, j) has row r of a row tile at
  // k = 8 j
  const bf16* xrow[RT];
  bool m_valid[RT];
#pragma unroll
  for (int t = 0; t < RT; ++t) {
    const int row = 16 * t + r;
    m_valid[t] = row < a.M;
    xrow[t] = (const bf16*)a.A + (int64_t)(m_valid[t] ? row : 0) * a.lda + 8 * j;
  }
  f32x4 acc[FG][RT];
#pragma unroll
  for (int s = 0; s < FG; ++s)
#pragma unroll
    for (int t = 0; t < RT; ++t) acc[s][t] = f32x4{0.f, 0.f, 0.f, 0.f};

  // this wave's 2 KB of LDS: 16 rows of 128 bytes, the 16-byte units of row R in the order
  // u ^ (R % 8), so that the writes (a row per 8 lanes) and the fragment reads (lane (r, j):
  // row r, unit 4 i + j) both spread evenly over the banks
  unsigned char* my_stage = stage + wave * 2048;
  const int st_write = ((lane >> 3) * 128) + 16 * ((lane & 7) ^ ((lane >> 3) & 7));   // + 1024 q
  const int st_read = r * 128;
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  const int chunks = K / 128, per_wave = (chunks + kRowsWaves - 1) / kRowsWaves;
  const int c_end = min((wave + 1) * per_wave, chunks);
  // the weights of a chunk are asked for a chunk ahead of its products (with K = 2048 a wave
  // has two chunks: all its weights are under way before the first product); the activations,
  // which come from L2, with the chunk itself (both a chunk ahead: the registers spill)
  bf16x8 wl[2][FG][2][2], x[RT][4];   // [buffer][feature group][half of the chunk][q]
  auto load_w = [&](int c, int b) {
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int s = 0; s < FG; ++s)
#pragma unroll
        for (int q = 0; q < 2; ++q)
          wl[b][s][h][q] = stream_load((const bf16x8*)(wline[s][q] + c * 128 + h * 64));
  };
  auto multiply = [&](int c, int b) {
#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        x[t][i] = m_valid[t] ? *(const bf16x8*)(xrow[t] + c * 128 + i * 32) : zero;
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int s = 0; s < FG; ++s) {
#pragma unroll
        for (int q = 0; q < 2; ++q) *(bf16x8*)(my_stage + st_write + 1024 * q) = wl[b][s][h][q];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          const bf16x8 wf = *(const bf16x8*)(my_stage + st_read + 16 * ((4 * i + j) ^ (r & 7)));
#pragma unroll
          for (int t = 0; t < RT; ++t)
            acc[s][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf, x[t][2 * h + i], acc[s][t], 0, 0, 0);
        }
      }
  };
  int c = wave * per_wave;
  if (c < c_end) load_w(c, 0);
  for (; c + 1 < c_end; c += 2) {
    load_w(c + 1, 1);
    multiply(c, 0);
    if (c + 2 < c_end) load_w(c + 2, 0);
    multiply(c + 1, 1);
  }
  if (c < c_end) multiply(c, 0);

  __syncthreads();   // every wave is done with its weight lines
  // the accumulator holds out[feature 4 j + v][token r]; stored as [token][feature]
#pragma unroll
  for (int s = 0; s < FG; ++s)
#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
      for (int v = 0; v < 4; ++v)
        red[((wave * FG + s) * RT + t) * 256 + r * 16 + 4 * j + v] = acc[s][t][v];
  __syncthreads();
  for (int idx = threadIdx.x; idx < FG * RT * 256; idx += kRowsWaves * 64) {
    const int st = idx >> 8, s = st / RT, t = st % RT, m = (idx >> 4) & 15, f = idx & 15;
    const int row = 16 * t + m, col = n0 + 16 * s + f;
    if (row >= a.M) continue;
    float sum = 0.f;
#pragma unroll
    for (int w = 0; w < kRowsWaves; ++w) sum += red[((w * FG + s) * RT + t) * 256 + (idx & 255)];
    if (a.bias) sum += a.bias[col];
    ((TC*)a.C)[(int64_t)row * a.ldc + col] = from_f32<TC>(sum);
  }
}

bool gemm_skinny_rows_takes(const GemmArgs& a) {
  return !a.offsets && !a.a_index && !a.c_index && a.groups <= 1 && a.epilogue == kEpilogueNone &&
         a.in_dtype == kBF16 && a.M > 32 && a.M <= 64 && a.N % 32 == 0 && a.N >= kRowsMinFeatures &&
         a.N <= kRowsMaxFeatures && a.K % 128 == 0 &&
         a.lda % 8 == 0 && ((uintptr_t)a.A % 16 == 0) && ((uintptr_t)a.W % 16 == 0);
}

template <int RT>
static void launch_rows(const GemmArgs& a, hipStream_t stream) {
  const unsigned blocks = (unsigned)(a.N / 32);
  if (a.out_dtype == kF32)
    gemm_skinny_rows_kernel<RT, 2, float><<<blocks, kRowsWaves * 64, 0, stream>>>(a);
  else
    gemm_skinny_rows_kernel<RT, 2, bf16><<<blocks, kRowsWaves * 64, 0, stream>>>(a);
}

int gemm_skinny_rows(const GemmArgs& a, hipStream_t stream) {
  NINFER_REQUIRE(gemm_skinny_rows_takes(a), "gemm: not a dense product of 33 to 64 rows");
  if (a.M <= 48)
    launch_rows<3>(a, stream);
  else
    launch_rows<4>(a, stream);
  NINFER_LAUNCH_CHECK();
  return 0;
}

}  // namespace ninfer

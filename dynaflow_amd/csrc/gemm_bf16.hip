// bf16 GEMM for gfx950:  C[M,N] = A[M,K] * W[N,K]^T, fp32 accumulate, bf16 out.
//
// Both operands are K-contiguous, which is the layout the 32x32x16 bf16 MFMA
// wants: every lane feeds 8 consecutive k of one row.  A workgroup owns a
// BM x BN tile of C and walks K in slabs of 64.  Each slab of A and W is
// fetched with 16-byte global loads into registers while the previous slab is
// being multiplied, then parked in LDS (two buffers, one barrier per slab).
// LDS rows are padded from 128 to 144 bytes so that the 16-byte fragment reads
// of 16 consecutive rows fall into 16 different 16-byte bank groups.
//
// The MFMA is issued with W as its first operand and A as its second, i.e. it
// produces the transposed 32x32 block.  In the accumulator layout of
// v_mfma_f32_32x32x16 a lane then holds ONE row m of C and runs of 4
// consecutive columns n, which lets the epilogue store 8 bytes per lane
// instead of 2.
#include "dfhip_common.h"

namespace {

constexpr int BK = 64;              // k extent of one slab
constexpr int LDS_ROW = BK + 8;     // padded row, in bf16 elements (144 bytes)
constexpr int CHUNKS = BK / 8;      // 16-byte chunks per slab row

template <int BM, int BN, int WAVES_M, int WAVES_N>
struct Shape {
  static constexpr int THREADS = WAVES_M * WAVES_N * 64;
  static constexpr int WTM = BM / WAVES_M;   // wave tile
  static constexpr int WTN = BN / WAVES_N;
  static constexpr int TM = WTM / 32;        // 32x32 MFMA blocks per wave
  static constexpr int TN = WTN / 32;
  static constexpr int A_LOADS = BM * CHUNKS / THREADS;  // 16-byte loads per thread per slab
  static constexpr int W_LOADS = BN * CHUNKS / THREADS;
  static constexpr int ROWS_PER_PASS = THREADS / CHUNKS;
  static constexpr int LDS_BYTES = 2 * (BM + BN) * LDS_ROW * 2;
  static_assert(BM % (WAVES_M * 32) == 0 && BN % (WAVES_N * 32) == 0, "wave tile must be MFMA blocks");
  static_assert((BM * CHUNKS) % THREADS == 0 && (BN * CHUNKS) % THREADS == 0, "loads must divide evenly");
};

template <int BM, int BN, int WAVES_M, int WAVES_N>
__global__ void __launch_bounds__(WAVES_M * WAVES_N * 64)
gemm_bf16_nt_kernel(const uint16_t* __restrict__ A, const uint16_t* __restrict__ W,
                    uint16_t* __restrict__ C, int M, int N, int K, int64_t lda, int64_t ldw,
                    int64_t ldc, int tiles_m, int tiles_n) {
  using S = Shape<BM, BN, WAVES_M, WAVES_N>;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  uint16_t* lds = reinterpret_cast<uint16_t*>(smem);
  // buffer b: A slab at b*(BM+BN)*LDS_ROW, W slab right after it
  constexpr int BUF_ELEMS = (BM + BN) * LDS_ROW;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wave_m = wave % WAVES_M;
  const int wave_n = wave / WAVES_M;

  // M-fastest tile order inside each XCD's contiguous range: the workgroups
  // that run together share one column block of W and all of A.
  const int tile = remap_xcd(blockIdx.x, tiles_m * tiles_n);
  const int tile_m = tile % tiles_m;
  const int tile_n = tile / tiles_m;
  const int m0 = tile_m * BM;
  const int n0 = tile_n * BN;

  // ---- global -> register staging: thread owns chunk `ld_chunk` of rows ld_row + p*ROWS_PER_PASS
  const int ld_row = tid / CHUNKS;
  const int ld_chunk = tid % CHUNKS;
  const uint16_t* a_src[S::A_LOADS];
  const uint16_t* w_src[S::W_LOADS];
#pragma unroll
  for (int p = 0; p < S::A_LOADS; ++p) {
    int row = m0 + ld_row + p * S::ROWS_PER_PASS;
    row = row < M ? row : M - 1;  // rows past the edge re-read the last row; never stored
    a_src[p] = A + (int64_t)row * lda + ld_chunk * 8;
  }
#pragma unroll
  for (int p = 0; p < S::W_LOADS; ++p) {
    int row = n0 + ld_row + p * S::ROWS_PER_PASS;
    row = row < N ? row : N - 1;
    w_src[p] = W + (int64_t)row * ldw + ld_chunk * 8;
  }
  u32x4 a_reg[S::A_LOADS];
  u32x4 w_reg[S::W_LOADS];

  auto fetch = [&](int kt) {
    const int koff = kt * BK;
#pragma unroll
    for (int p = 0; p < S::A_LOADS; ++p) a_reg[p] = *reinterpret_cast<const u32x4*>(a_src[p] + koff);
#pragma unroll
    for (int p = 0; p < S::W_LOADS; ++p) w_reg[p] = *reinterpret_cast<const u32x4*>(w_src[p] + koff);
  };
  auto park = [&](int buf) {
    uint16_t* a_dst = lds + buf * BUF_ELEMS + ld_row * LDS_ROW + ld_chunk * 8;
    uint16_t* w_dst = a_dst + BM * LDS_ROW;
#pragma unroll
    for (int p = 0; p < S::A_LOADS; ++p)
      *reinterpret_cast<u32x4*>(a_dst + p * S::ROWS_PER_PASS * LDS_ROW) = a_reg[p];
#pragma unroll
    for (int p = 0; p < S::W_LOADS; ++p)
      *reinterpret_cast<u32x4*>(w_dst + p * S::ROWS_PER_PASS * LDS_ROW) = w_reg[p];
  };

  // ---- fragment addressing: lane reads row (lane % 32), k chunk (lane / 32) of each k16 step
  const int frag_row = lane & 31;
  const int frag_half = lane >> 5;
  const int a_frag_off = (wave_m * S::WTM + frag_row) * LDS_ROW + frag_half * 8;
  const int w_frag_off = BM * LDS_ROW + (wave_n * S::WTN + frag_row) * LDS_ROW + frag_half * 8;

  f32x16 acc[S::TM][S::TN];
#pragma unroll
  for (int i = 0; i < S::TM; ++i)
#pragma unroll
    for (int j = 0; j < S::TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  const int KT = K / BK;
  fetch(0);
  park(0);
  __syncthreads();

  for (int kt = 0; kt < KT; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < KT) fetch(kt + 1);

    const uint16_t* base = lds + buf * BUF_ELEMS;
    bf16x8 fa[2][S::TM];
    bf16x8 fw[2][S::TN];
    auto load_frags = [&](int ks, int slot) {
#pragma unroll
      for (int i = 0; i < S::TM; ++i)
        fa[slot][i] = *reinterpret_cast<const bf16x8*>(base + a_frag_off + i * 32 * LDS_ROW + ks * 16);
#pragma unroll
      for (int j = 0; j < S::TN; ++j)
        fw[slot][j] = *reinterpret_cast<const bf16x8*>(base + w_frag_off + j * 32 * LDS_ROW + ks * 16);
    };
    load_frags(0, 0);
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      const int slot = ks & 1;
      if (ks + 1 < BK / 16) load_frags(ks + 1, slot ^ 1);
#pragma unroll
      for (int i = 0; i < S::TM; ++i)
#pragma unroll
        for (int j = 0; j < S::TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fw[slot][j], fa[slot][i], acc[i][j], 0, 0, 0);
    }

    if (kt + 1 < KT) park(buf ^ 1);
    __syncthreads();
  }

  // ---- epilogue: lane holds row m = lane%32 of each block, columns 8*g + 4*(lane/32) + 0..3
  const int m_lane = m0 + wave_m * S::WTM + frag_row;
  const int n_lane = n0 + wave_n * S::WTN + frag_half * 4;
#pragma unroll
  for (int i = 0; i < S::TM; ++i) {
    const int m = m_lane + i * 32;
    if (m >= M) continue;
    uint16_t* c_row = C + (int64_t)m * ldc;
#pragma unroll
    for (int j = 0; j < S::TN; ++j) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int n = n_lane + j * 32 + g * 8;
        if (n < N) {  // N % 8 == 0 and n % 4 == 0: the 4-wide run is entirely inside or outside
          u32x2 v;
          v[0] = pack2_bf16(acc[i][j][4 * g + 0], acc[i][j][4 * g + 1]);
          v[1] = pack2_bf16(acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]);
          *reinterpret_cast<u32x2*>(c_row + n) = v;
        }
      }
    }
  }
}

template <int BM, int BN, int WAVES_M, int WAVES_N>
int launch(const void* A, int64_t lda, const void* W, int64_t ldw, void* C, int64_t ldc, int M, int N,
           int K, hipStream_t stream) {
  using S = Shape<BM, BN, WAVES_M, WAVES_N>;
  auto kernel = gemm_bf16_nt_kernel<BM, BN, WAVES_M, WAVES_N>;
  static bool lds_opted_in = false;  // attribute is per function, set once per process
  if (!lds_opted_in) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            S::LDS_BYTES) != hipSuccess)
      return DFHIP_ERR_LAUNCH;
    lds_opted_in = true;
  }
  const int tiles_m = (M + BM - 1) / BM;
  const int tiles_n = (N + BN - 1) / BN;
  hipLaunchKernelGGL(kernel, dim3(tiles_m * tiles_n), dim3(S::THREADS), S::LDS_BYTES, stream,
                     static_cast<const uint16_t*>(A), static_cast<const uint16_t*>(W),
                     static_cast<uint16_t*>(C), M, N, K, lda, ldw, ldc, tiles_m, tiles_n);
  return dfhip_check_launch();
}

int check_args(const void* A, int64_t lda, const void* W, int64_t ldw, void* C, int64_t ldc, int M, int N,
               int K) {
  if (!A || !W || !C) return DFHIP_ERR_NULL_POINTER;
  if (M < 1 || N < 1 || K < 1 || K % BK != 0 || N % 8 != 0) return DFHIP_ERR_BAD_SHAPE;
  if (lda < K || ldw < K || ldc < N) return DFHIP_ERR_BAD_STRIDE;
  if (lda % 8 || ldw % 8 || ldc % 8 || !dfhip_aligned16(A) || !dfhip_aligned16(W) || !dfhip_aligned16(C))
    return DFHIP_ERR_BAD_ALIGNMENT;
  return DFHIP_OK;
}

}  // namespace

extern "C" int dfhip_gemm_bf16_nt_variant(const void* A, int64_t lda, const void* W, int64_t ldw, void* C,
                                          int64_t ldc, int M, int N, int K, int variant,
                                          dfhip_stream_t stream) {
  if (int rc = check_args(A, lda, W, ldw, C, ldc, M, N, K)) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (variant) {
    case 0: return launch<256, 256, 2, 2>(A, lda, W, ldw, C, ldc, M, N, K, s);
    case 1: return launch<256, 256, 2, 4>(A, lda, W, ldw, C, ldc, M, N, K, s);
    case 2: return launch<128, 128, 2, 2>(A, lda, W, ldw, C, ldc, M, N, K, s);
    case 3: return launch<256, 128, 2, 2>(A, lda, W, ldw, C, ldc, M, N, K, s);
    default: return DFHIP_ERR_BAD_ARGUMENT;
  }
}

extern "C" int dfhip_gemm_bf16_nt(const void* A, int64_t lda, const void* W, int64_t ldw, void* C,
                                  int64_t ldc, int M, int N, int K, dfhip_stream_t stream) {
  // Big tiles when they still give the 256 CUs at least one tile each.
  const int64_t big_tiles = (int64_t)((M + 255) / 256) * ((N + 255) / 256);
  int variant = 2;
  if (M > 128 && big_tiles >= 256) variant = 0;
  else if (M > 128 && (int64_t)((M + 255) / 256) * ((N + 127) / 128) >= 192) variant = 3;
  return dfhip_gemm_bf16_nt_variant(A, lda, W, ldw, C, ldc, M, N, K, variant, stream);
}

// fp32 GEMM for gfx950:  C[M,N] = A[M,K] * W[N,K]^T with v_mfma_f32_32x32x2_f32.
//
// Serves the small fp32 configuration, where agreement with an fp32 host
// result to 1e-5 matters and speed does not: a 128x128 tile per workgroup,
// K walked in slabs of 16 through one LDS buffer.  LDS rows hold 16 floats
// padded to 17 so that the 32 lanes of a fragment read (one float each, rows
// 17 words apart) hit 32 different banks.
#include "dfhip_common.h"

namespace {

constexpr int FBM = 128, FBN = 128, FBK = 16, FROW = FBK + 1, FTHREADS = 256;

__global__ void __launch_bounds__(FTHREADS)
gemm_f32_nt_kernel(const float* __restrict__ A, const float* __restrict__ W, float* __restrict__ C, int M,
                   int N, int K, int64_t lda, int64_t ldw, int64_t ldc) {
  __shared__ float a_lds[FBM * FROW];
  __shared__ float w_lds[FBN * FROW];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wave_m = wave & 1, wave_n = wave >> 1;  // 2 x 2 waves, 64 x 64 each
  const int m0 = blockIdx.y * FBM, n0 = blockIdx.x * FBN;

  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  const int frag_row = lane & 31, frag_k = lane >> 5;
  for (int k0 = 0; k0 < K; k0 += FBK) {
    // 128 rows x 4 float4 chunks per operand = 512 chunks, 2 per thread
#pragma unroll
    for (int p = 0; p < 2; ++p) {
      const int idx = tid + p * FTHREADS;
      const int r = idx >> 2, c = (idx & 3) * 4;
      int ar = m0 + r; ar = ar < M ? ar : M - 1;
      int wr = n0 + r; wr = wr < N ? wr : N - 1;
      f32x4 av = {0.f, 0.f, 0.f, 0.f}, wv = {0.f, 0.f, 0.f, 0.f};
      if (k0 + c < K) {  // K % 4 == 0: a chunk is entirely inside or outside
        av = *reinterpret_cast<const f32x4*>(A + (int64_t)ar * lda + k0 + c);
        wv = *reinterpret_cast<const f32x4*>(W + (int64_t)wr * ldw + k0 + c);
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        a_lds[r * FROW + c + e] = av[e];
        w_lds[r * FROW + c + e] = wv[e];
      }
    }
    __syncthreads();
#pragma unroll
    for (int ks = 0; ks < FBK / 2; ++ks) {
      float fa[2], fw[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) fa[i] = a_lds[(wave_m * 64 + i * 32 + frag_row) * FROW + ks * 2 + frag_k];
#pragma unroll
      for (int j = 0; j < 2; ++j) fw[j] = w_lds[(wave_n * 64 + j * 32 + frag_row) * FROW + ks * 2 + frag_k];
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fw[j], fa[i], acc[i][j], 0, 0, 0);
    }
    __syncthreads();
  }

  // W was the first MFMA operand: a lane holds row m = lane%32 and 4-wide runs of n
  const int m_lane = m0 + wave_m * 64 + frag_row;
  const int n_lane = n0 + wave_n * 64 + frag_k * 4;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int m = m_lane + i * 32;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int g = 0; g < 4; ++g)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int n = n_lane + j * 32 + g * 8 + e;
          if (n < N) C[(int64_t)m * ldc + n] = acc[i][j][4 * g + e];
        }
  }
}

}  // namespace

extern "C" int dfhip_gemm_f32_nt(const void* A, int64_t lda, const void* W, int64_t ldw, void* C, int64_t ldc,
                                 int M, int N, int K, dfhip_stream_t stream) {
  if (!A || !W || !C) return DFHIP_ERR_NULL_POINTER;
  if (M < 1 || N < 1 || K < 1 || K % 4 != 0) return DFHIP_ERR_BAD_SHAPE;
  if (lda < K || ldw < K || ldc < N) return DFHIP_ERR_BAD_STRIDE;
  if (lda % 4 || ldw % 4 || !dfhip_aligned16(A) || !dfhip_aligned16(W) ||
      (reinterpret_cast<uintptr_t>(C) & 3u))
    return DFHIP_ERR_BAD_ALIGNMENT;
  dim3 grid((N + FBN - 1) / FBN, (M + FBM - 1) / FBM);
  hipLaunchKernelGGL(gemm_f32_nt_kernel, grid, dim3(FTHREADS), 0, static_cast<hipStream_t>(stream),
                     static_cast<const float*>(A), static_cast<const float*>(W), static_cast<float*>(C), M, N,
                     K, lda, ldw, ldc);
  return dfhip_check_launch();
}

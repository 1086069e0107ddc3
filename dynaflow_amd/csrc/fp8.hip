// fp8 (OCP e4m3fn) path: per-tensor dynamic quantisation, SiLU*mul with amax,
// and the fp8 GEMM  C = bf16(a_scale * w_scale[n] * A[M,K] * W[N,K]^T).
//
// The GEMMs have the byte geometry of the bf16 ones (a K slab row is 128 bytes, here
// 128 fp8 values) and multiply with the scaled fp8 MFMAs (scale exponents fixed at 2^0):
// v_mfma_scale_f32_16x16x128_f8f6f4 in the ring kernels, ..._32x32x64_... in the
// register-staged one - twice the bf16 rate.  A lane feeds 32 consecutive bytes of one
// row; both operands use the same lane->k mapping, so the contraction is exact whatever
// order the hardware walks those bytes in.
//
// gemm_fp8_ring_kernel  256x256 tile, the LDS-DMA ring / pinned-schedule design of the
//                       bf16 ring kernel: five 32 KiB LDS units, 1.5 slabs in flight,
//                       XOR-swizzled 128-byte rows, one LDS read or DMA issue behind every
//                       MFMA, barrier between the two column halves of a slab, staged epilogue.
// gemm_fp8_nt_kernel    register-staged double buffer for small shapes.
#include "dfhip_common.h"

namespace {

typedef int i32x8 __attribute__((ext_vector_type(8)));

constexpr float FP8_MAX = 448.0f;
constexpr int QT = 256;      // threads of the elementwise fp8 kernels
constexpr int QUNROLL = 4;

DFHIP_DEVICE float silu_f32(float g) { return silu_fast(g); }   // one formula for every bf16 path

DFHIP_DEVICE void atomic_max_nonneg(float* cell, float v) {
  // non-negative floats order like their bit patterns
  atomicMax(reinterpret_cast<unsigned int*>(cell), __float_as_uint(v));
}

DFHIP_DEVICE void block_max_to(float* cell, float v) {
  __shared__ float partial[QT / 64];
  v = wave_max(v);
  if ((threadIdx.x & 63) == 0) partial[threadIdx.x >> 6] = v;
  __syncthreads();
  if (threadIdx.x == 0) {
    float m = partial[0];
#pragma unroll
    for (int w = 1; w < QT / 64; ++w) m = fmaxf(m, partial[w]);
    atomic_max_nonneg(cell, m);
  }
}

// amax[0] = max(amax[0], max |x|) over a row-strided bf16 matrix; group = 8 values
__global__ void __launch_bounds__(QT)
absmax_bf16_kernel(const uint16_t* __restrict__ x, int64_t ld, uint32_t groups, uint32_t per_row,
                   float* __restrict__ amax) {
  float m = 0.0f;
  for (uint32_t gi = blockIdx.x * QT + threadIdx.x; gi < groups; gi += gridDim.x * QT) {
    const uint32_t row = gi / per_row, col = (gi - row * per_row) * 8;
    const u32x4 v = *reinterpret_cast<const u32x4*>(x + (int64_t)row * ld + col);
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      m = fmaxf(m, fabsf(bf16_bits_to_f32(v[w] & 0xffffu)));
      m = fmaxf(m, fabsf(__uint_as_float(v[w] & 0xffff0000u)));
    }
  }
  block_max_to(amax, m);
}

DFHIP_DEVICE uint32_t quant4(float a, float b, float c, float d, float scale) {
  a = fminf(fmaxf(a / scale, -FP8_MAX), FP8_MAX);
  b = fminf(fmaxf(b / scale, -FP8_MAX), FP8_MAX);
  c = fminf(fmaxf(c / scale, -FP8_MAX), FP8_MAX);
  d = fminf(fmaxf(d / scale, -FP8_MAX), FP8_MAX);
  uint32_t r = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);  // bytes 0,1
  r = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, r, true);            // bytes 2,3
  return r;
}

// q = e4m3fn(x / scale), scale = max(amax, 1e-12) / 448; group = 8 values -> 8 bytes
__global__ void __launch_bounds__(QT)
quant_fp8_bf16_kernel(const uint16_t* __restrict__ x, int64_t ld, uint8_t* __restrict__ q, int64_t ld_q,
                      uint32_t groups, uint32_t per_row, const float* __restrict__ amax,
                      float* __restrict__ scale_out) {
  const float scale = fmaxf(amax[0], 1e-12f) / FP8_MAX;
  if (blockIdx.x == 0 && threadIdx.x == 0 && scale_out != nullptr) scale_out[0] = scale;
  for (uint32_t gi = blockIdx.x * QT + threadIdx.x; gi < groups; gi += gridDim.x * QT) {
    const uint32_t row = gi / per_row, col = (gi - row * per_row) * 8;
    const u32x4 v = *reinterpret_cast<const u32x4*>(x + (int64_t)row * ld + col);
    u32x2 o;
    o[0] = quant4(bf16_bits_to_f32(v[0] & 0xffffu), __uint_as_float(v[0] & 0xffff0000u),
                  bf16_bits_to_f32(v[1] & 0xffffu), __uint_as_float(v[1] & 0xffff0000u), scale);
    o[1] = quant4(bf16_bits_to_f32(v[2] & 0xffffu), __uint_as_float(v[2] & 0xffff0000u),
                  bf16_bits_to_f32(v[3] & 0xffffu), __uint_as_float(v[3] & 0xffff0000u), scale);
    *reinterpret_cast<u32x2*>(q + (int64_t)row * ld_q + col) = o;
  }
}

// out = bf16(silu(g) * u) (optional store) and amax over the rounded values
__global__ void __launch_bounds__(QT)
silu_mul_absmax_kernel(const uint16_t* __restrict__ gate, int64_t ld_gate, const uint16_t* __restrict__ up,
                       int64_t ld_up, uint16_t* __restrict__ out, int64_t ld_out, uint32_t groups,
                       uint32_t per_row, float* __restrict__ amax) {
  float m = 0.0f;
  for (uint32_t gi = blockIdx.x * QT + threadIdx.x; gi < groups; gi += gridDim.x * QT) {
    const uint32_t row = gi / per_row, col = (gi - row * per_row) * 8;
    const u32x4 g = *reinterpret_cast<const u32x4*>(gate + (int64_t)row * ld_gate + col);
    const u32x4 u = *reinterpret_cast<const u32x4*>(up + (int64_t)row * ld_up + col);
    u32x4 o;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float lo = silu_f32(bf16_bits_to_f32(g[w] & 0xffffu)) * bf16_bits_to_f32(u[w] & 0xffffu);
      const float hi = silu_f32(__uint_as_float(g[w] & 0xffff0000u)) * __uint_as_float(u[w] & 0xffff0000u);
      o[w] = pack2_bf16(lo, hi);
      m = fmaxf(m, fabsf(bf16_bits_to_f32(o[w] & 0xffffu)));
      m = fmaxf(m, fabsf(__uint_as_float(o[w] & 0xffff0000u)));
    }
    if (out != nullptr) *reinterpret_cast<u32x4*>(out + (int64_t)row * ld_out + col) = o;
  }
  block_max_to(amax, m);
}

// ------------------------------------------------------------------ fp8 GEMM
constexpr int FBK = 128;            // fp8 values (= bytes) per slab row
constexpr int FROW = FBK + 16;      // padded LDS row in bytes
constexpr int FCHUNKS = FBK / 16;   // 16-byte chunks per slab row

template <int BM, int BN>
__global__ void __launch_bounds__(256)
gemm_fp8_nt_kernel(const uint8_t* __restrict__ A, const uint8_t* __restrict__ W, uint16_t* __restrict__ C,
                   const float* __restrict__ a_scale, const float* __restrict__ w_scale, int M, int N, int K,
                   int64_t lda, int64_t ldw, int64_t ldc, int tiles_m, int tiles_n) {
  constexpr int THREADS = 256;
  constexpr int WTM = BM / 2, WTN = BN / 2, TM = WTM / 32, TN = WTN / 32;
  constexpr int A_LOADS = BM * FCHUNKS / THREADS, W_LOADS = BN * FCHUNKS / THREADS;
  constexpr int ROWS_PER_PASS = THREADS / FCHUNKS;
  constexpr int BUF_BYTES = (BM + BN) * FROW;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wave_m = wave & 1, wave_n = wave >> 1;
  const int tile = remap_xcd(blockIdx.x, tiles_m * tiles_n);
  const int m0 = (tile % tiles_m) * BM, n0 = (tile / tiles_m) * BN;

  const int ld_row = tid / FCHUNKS, ld_chunk = tid % FCHUNKS;
  const uint8_t* a_src[A_LOADS];
  const uint8_t* w_src[W_LOADS];
#pragma unroll
  for (int p = 0; p < A_LOADS; ++p) {
    int row = m0 + ld_row + p * ROWS_PER_PASS;
    row = row < M ? row : M - 1;
    a_src[p] = A + (int64_t)row * lda + ld_chunk * 16;
  }
#pragma unroll
  for (int p = 0; p < W_LOADS; ++p) {
    int row = n0 + ld_row + p * ROWS_PER_PASS;
    row = row < N ? row : N - 1;
    w_src[p] = W + (int64_t)row * ldw + ld_chunk * 16;
  }
  u32x4 a_reg[A_LOADS], w_reg[W_LOADS];
  auto fetch = [&](int kt) {
#pragma unroll
    for (int p = 0; p < A_LOADS; ++p) a_reg[p] = *reinterpret_cast<const u32x4*>(a_src[p] + kt * FBK);
#pragma unroll
    for (int p = 0; p < W_LOADS; ++p) w_reg[p] = *reinterpret_cast<const u32x4*>(w_src[p] + kt * FBK);
  };
  auto park = [&](int buf) {
    uint8_t* a_dst = smem + buf * BUF_BYTES + ld_row * FROW + ld_chunk * 16;
    uint8_t* w_dst = a_dst + BM * FROW;
#pragma unroll
    for (int p = 0; p < A_LOADS; ++p) *reinterpret_cast<u32x4*>(a_dst + p * ROWS_PER_PASS * FROW) = a_reg[p];
#pragma unroll
    for (int p = 0; p < W_LOADS; ++p) *reinterpret_cast<u32x4*>(w_dst + p * ROWS_PER_PASS * FROW) = w_reg[p];
  };

  // lane reads 32 consecutive bytes: row lane%32, byte offset 64*ks + 32*(lane/32)
  const int frag_row = lane & 31, frag_half = lane >> 5;
  const int a_frag_off = (wave_m * WTM + frag_row) * FROW + frag_half * 32;
  const int w_frag_off = BM * FROW + (wave_n * WTN + frag_row) * FROW + frag_half * 32;

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  const int KT = K / FBK;
  fetch(0);
  park(0);
  __syncthreads();
  for (int kt = 0; kt < KT; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < KT) fetch(kt + 1);
    const uint8_t* base = smem + buf * BUF_BYTES;
#pragma unroll
    for (int ks = 0; ks < FBK / 64; ++ks) {
      i32x8 fa[TM], fw[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const u32x4 lo = *reinterpret_cast<const u32x4*>(base + a_frag_off + i * 32 * FROW + ks * 64);
        const u32x4 hi = *reinterpret_cast<const u32x4*>(base + a_frag_off + i * 32 * FROW + ks * 64 + 16);
        fa[i] = i32x8{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
      }
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const u32x4 lo = *reinterpret_cast<const u32x4*>(base + w_frag_off + j * 32 * FROW + ks * 64);
        const u32x4 hi = *reinterpret_cast<const u32x4*>(base + w_frag_off + j * 32 * FROW + ks * 64 + 16);
        fw[j] = i32x8{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
      }
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fw[j], fa[i], acc[i][j], 0, 0, 0, 0x7f7f7f7f,
                                                                     0, 0x7f7f7f7f);
    }
    if (kt + 1 < KT) park(buf ^ 1);
    __syncthreads();
  }

  // W was the first operand: lane holds row m = lane%32, columns 8g + 4*(lane/32) + 0..3
  const float sa = a_scale[0];
  const int m_lane = m0 + wave_m * WTM + frag_row;
  const int n_lane = n0 + wave_n * WTN + frag_half * 4;
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int m = m_lane + i * 32;
    if (m >= M) continue;
    uint16_t* c_row = C + (int64_t)m * ldc;
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int n = n_lane + j * 32 + g * 8;
        if (n < N) {
          const f32x4 ws = *reinterpret_cast<const f32x4*>(w_scale + n);
          u32x2 v;
          v[0] = pack2_bf16(acc[i][j][4 * g + 0] * (sa * ws[0]), acc[i][j][4 * g + 1] * (sa * ws[1]));
          v[1] = pack2_bf16(acc[i][j][4 * g + 2] * (sa * ws[2]), acc[i][j][4 * g + 3] * (sa * ws[3]));
          *reinterpret_cast<u32x2*>(c_row + n) = v;
        }
      }
  }
}


// ------------------------------------------------------------------ fp8 ring kernel
constexpr int F8_UNIT = 32768, F8_NUNITS = 5, F8_RING_LDS = F8_UNIT * F8_NUNITS;
constexpr int F8_GROUP_M = 4, F8_EROW = 272;

// FUSED: the W half of a slab holds 128 rows of W (gate) and the matching 128 rows of W2 (up); the tile
// then is 256 x 128 outputs, N counts those, and the epilogue writes act = bf16(silu(bf16 g) * bf16 u) -
// the roundings of the separate GEMMs and of silu_mul_absmax_kernel, so the same bits - and folds
// max |act| into amax[0].
template <bool FUSED>
__global__ void __launch_bounds__(256)
gemm_fp8_ring_kernel(const uint8_t* __restrict__ A, const uint8_t* __restrict__ W, const uint8_t* __restrict__ W2,
                     uint16_t* __restrict__ C, const float* __restrict__ a_scale, const float* __restrict__ w_scale,
                     const float* __restrict__ w2_scale, float* __restrict__ amax, int M, int N, int K, int64_t lda,
                     int64_t ldw, int64_t ldc, int tiles_m, int tiles_n) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wave_m = wave & 1, wave_n = wave >> 1;
  constexpr int TILE_N = FUSED ? 128 : 256;    // output columns of a tile

  const int tile = remap_xcd(blockIdx.x, tiles_m * tiles_n);
  const int per_panel = F8_GROUP_M * tiles_n;
  const int first_m = (tile / per_panel) * F8_GROUP_M;
  const int rows_in_panel = (tiles_m - first_m) < F8_GROUP_M ? (tiles_m - first_m) : F8_GROUP_M;
  const int in_panel = tile % per_panel;
  const int m0 = (first_m + in_panel % rows_in_panel) * 256;
  const int n0 = (in_panel / rows_in_panel) * TILE_N;
  const int KT = K / FBK;

  // DMA addresses: a wave-uniform tile base (scalar registers, advanced per slab) plus a 32-bit byte
  // offset per lane.  FUSED: rows 0..127 of the W half come from W (waves 0, 1), rows 128..255 from W2.
  uint32_t a_off[8], w_off[8];
#pragma unroll
  for (int t = 0; t < 8; ++t) {
    const int row = (wave * 8 + t) * 8 + (lane >> 3);
    const int chunk = (lane & 7) ^ ((row >> 1) & 7);
    int ar = m0 + row; ar = ar < M ? ar : M - 1;
    a_off[t] = (uint32_t)((int64_t)(ar - m0) * lda + chunk * 16);
    int wr = n0 + (FUSED ? (row & 127) : row); wr = wr < N ? wr : N - 1;
    w_off[t] = (uint32_t)((int64_t)(wr - n0) * ldw + chunk * 16);
  }
  const uint8_t* const a_tile = A + (int64_t)m0 * lda;
  const uint8_t* const w_tile = ((FUSED && wave >= 2) ? W2 : W) + (int64_t)n0 * ldw;
  const uint32_t wave_lds = wave * 8 * 1024;
  auto dma_a = [&](int t, int slab, int unit) {
    const int s = slab < KT ? slab : KT - 1;
    dma16_base(unit * F8_UNIT + wave_lds + t * 1024, a_tile + (int64_t)s * FBK, a_off[t]);
  };
  auto dma_w = [&](int t, int slab, int unit) {
    const int s = slab < KT ? slab : KT - 1;
    dma16_base(unit * F8_UNIT + wave_lds + t * 1024, w_tile + (int64_t)s * FBK, w_off[t]);
  };

  // v_mfma_scale_f32_16x16x128_f8f6f4: one instruction covers the 128 bytes of k of a slab.  A fragment of a
  // 16-row block is 32 bytes per lane = chunks 2*(lane/16) and 2*(lane/16) + 1 of row lane%16, swizzled by
  // (row/2)%8.  acc[i][j] (W block j first operand, A block i second): lane holds
  // C[16 i + lane%16][16 j + 4 (lane/16) + r], r = 0..3.
  const int frow = lane & 15, fquad = lane >> 4, fswz = (frow >> 1) & 7;
  int koff[2];
#pragma unroll
  for (int part = 0; part < 2; ++part) koff[part] = ((2 * fquad + part) ^ fswz) * 16;
  const int a_lane = (wave_m * 128 + frow) * 128, w_lane = (wave_n * 128 + frow) * 128;

  f32x4 acc[8][8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[i][j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

#pragma unroll
  for (int t = 0; t < 8; ++t) dma_a(t, 0, 0);
#pragma unroll
  for (int t = 0; t < 8; ++t) dma_w(t, 0, 1);
#pragma unroll
  for (int t = 0; t < 8; ++t) dma_a(t, 1, 2);
#pragma unroll
  for (int t = 0; t < 8; ++t) dma_w(t, 1, 3);
  wait_vmcnt<16>();
  workgroup_barrier();

  // A whole slab of fragments is 128 registers per operand; both operands double-buffered would not fit.
  // The slab is multiplied in two column halves instead: W blocks 0..3 (fwa), then W blocks 4..7 (fwb), both
  // against all eight A blocks.  The A blocks are double-buffered across slabs, each W half is read while the
  // other one is in use.
  u32x4 fa[2][8][2], fwa[4][2], fwb[4][2];   // [..][block][low / high 16 bytes]
  auto read_a = [&](int half_idx, int slot, int unit_a) {   // half_idx 0..15: block half_idx/2, low / high half
    const int blk = half_idx >> 1, part = half_idx & 1;
    fa[slot][blk][part] = *reinterpret_cast<const u32x4*>(smem + unit_a * F8_UNIT + a_lane + koff[part] + blk * 2048);
  };
  auto read_w = [&](int half_idx, bool second, int unit_w) {   // half_idx 0..7 within the column half
    const int blk = half_idx >> 1, part = half_idx & 1;
    const u32x4 v = *reinterpret_cast<const u32x4*>(smem + unit_w * F8_UNIT + w_lane + koff[part] + ((second ? 4 : 0) + blk) * 2048);
    if (second) fwb[blk][part] = v; else fwa[blk][part] = v;
  };
  const int unit_scale = 0x7f7f7f7f;   // e8m0 scales 2^0
  auto mfma = [&](int q, int slot, bool second) {   // snake over 8 A blocks x 4 W blocks
    const int i = q >> 2, jj = (i & 1) ? 3 - (q & 3) : (q & 3);
    const u32x4 (&w)[2] = second ? fwb[jj] : fwa[jj];
    const i32x8 av = {(int)fa[slot][i][0][0], (int)fa[slot][i][0][1], (int)fa[slot][i][0][2], (int)fa[slot][i][0][3],
                      (int)fa[slot][i][1][0], (int)fa[slot][i][1][1], (int)fa[slot][i][1][2], (int)fa[slot][i][1][3]};
    const i32x8 wv = {(int)w[0][0], (int)w[0][1], (int)w[0][2], (int)w[0][3], (int)w[1][0], (int)w[1][1], (int)w[1][2], (int)w[1][3]};
    // written out so that the accumulator keeps its registers
    asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %3 op_sel_hi:[0,0,0]"
                 : "+a"(acc[i][second ? 4 + jj : jj]) : "v"(wv), "v"(av), "v"(unit_scale));
  };
  // reads of the next slab in the order its first MFMAs need them: W block 0, A block 0, W blocks 1..3, A 1..7
  auto read_next = [&](int pos, int slot, int unit_a, int unit_w) {   // pos 0..23 (fragment halves)
    if (pos < 2) read_w(pos, false, unit_w);
    else if (pos < 4) read_a(pos - 2, slot, unit_a);
    else if (pos < 10) read_w(pos - 2, false, unit_w);
    else read_a(pos - 8, slot, unit_a);
  };

  int ua = 0, uw = 1, ia = 4, iw = 0;
#pragma unroll
  for (int pos = 0; pos < 24; ++pos) read_next(pos, 0, ua, uw);
  // one slab; `sl` (0 / 1, a constant at each call) is the A fragment buffer this slab multiplies from
  auto slab = [&](int kt, int sl) {
    // first column half: the fragments of W blocks 4..7 behind MFMAs 0..7, the DMA of A(kt+2) behind every
    // other MFMA after that
#pragma unroll
    for (int q = 0; q < 32; ++q) {
      mfma(q, sl, false);
      if (q < 8) read_w(q, true, uw);
      else if (q % 2 == 0 && q < 24) dma_a((q - 8) / 2, kt + 2, ia);
      DFHIP_PIN;
    }
    // every LDS read of slab kt has been issued; slab kt+1 must have landed, only A(kt+2) may be in flight
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    wait_vmcnt<8>();
    workgroup_barrier();
    int na = ua + 2; if (na >= F8_NUNITS) na -= F8_NUNITS;
    int nw = uw + 2; if (nw >= F8_NUNITS) nw -= F8_NUNITS;
    // second column half: the DMA of W(kt+2) behind every other MFMA, the 24 fragment halves of slab kt+1
    // (all of A, W blocks 0..3) behind the others
#pragma unroll
    for (int q = 0; q < 32; ++q) {
      mfma(q, sl, true);
      if (q < 16) { if (q % 2 == 0) dma_w(q / 2, kt + 2, iw); else read_next(q / 2, sl ^ 1, na, nw); }
      else read_next(8 + (q - 16), sl ^ 1, na, nw);
      DFHIP_PIN;
    }
    ua = na; uw = nw;
    ia += 2; if (ia >= F8_NUNITS) ia -= F8_NUNITS;
    iw += 2; if (iw >= F8_NUNITS) iw -= F8_NUNITS;
  };
  int kt = 0;
  for (; kt + 1 < KT; kt += 2) {
    slab(kt, 0);
    slab(kt + 1, 1);
  }
  if (kt < KT) slab(kt, 0);
  wait_vmcnt<0>();
  workgroup_barrier();
  asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");   // the last MFMAs have written their accumulators
  // (the compiler does not know that the statements above write the accumulators late: every later use
  // of an accumulator is tied behind the wait states)
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) asm volatile("" : "+a"(acc[i][j]));

  // scale, round to bf16, park the wave's 128x128 block in LDS, store whole 256-byte row pieces
  const float sa = a_scale[0];
  uint8_t* park = smem + wave * (128 * F8_EROW);
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    int n = n0 + (FUSED ? 0 : wave_n * 128) + j * 16 + fquad * 4;
    n = n < N ? n : N - 4;   // columns past the edge are never stored; keep the scale load in bounds
    const f32x4 ws = *reinterpret_cast<const f32x4*>((FUSED && wave_n ? w2_scale : w_scale) + n);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      u32x2 v;
      v[0] = pack2_bf16(acc[i][j][0] * (sa * ws[0]), acc[i][j][1] * (sa * ws[1]));
      v[1] = pack2_bf16(acc[i][j][2] * (sa * ws[2]), acc[i][j][3] * (sa * ws[3]));
      *reinterpret_cast<u32x2*>(park + (i * 16 + frow) * F8_EROW + (j * 16 + fquad * 4) * 2) = v;
    }
  }
  DFHIP_PIN;
  if (FUSED) {
    // gate blocks sit in the parks of waves 0, 1 (rows 0..127, 128..255), up blocks in those of waves 2, 3;
    // wave w combines rows (w & 1) * 128 + (w >> 1) * 64 .. + 64 of the tile
    __syncthreads();
    const uint8_t* gpark = smem + (wave & 1) * (128 * F8_EROW);
    const uint8_t* upark = smem + ((wave & 1) + 2) * (128 * F8_EROW);
    const int row0 = (wave >> 1) * 64;
    float vmax = 0.0f;
#pragma unroll 4
    for (int p = 0; p < 16; ++p) {
      const int id = p * 64 + lane;
      const int row = row0 + (id >> 4), c = id & 15;
      const u32x4 gv = *reinterpret_cast<const u32x4*>(gpark + row * F8_EROW + c * 16);
      const u32x4 uv = *reinterpret_cast<const u32x4*>(upark + row * F8_EROW + c * 16);
      u32x4 o;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const float lo = silu_f32(bf16_bits_to_f32(gv[w] & 0xffffu)) * bf16_bits_to_f32(uv[w] & 0xffffu);
        const float hi = silu_f32(__uint_as_float(gv[w] & 0xffff0000u)) * __uint_as_float(uv[w] & 0xffff0000u);
        o[w] = pack2_bf16(lo, hi);
      }
      const int m = m0 + (wave & 1) * 128 + row, n = n0 + c * 8;
      if (m < M && n < N) {
        *reinterpret_cast<u32x4*>(C + (int64_t)m * ldc + n) = o;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          vmax = fmaxf(vmax, fabsf(bf16_bits_to_f32(o[w] & 0xffffu)));
          vmax = fmaxf(vmax, fabsf(__uint_as_float(o[w] & 0xffff0000u)));
        }
      }
    }
    vmax = wave_max(vmax);
    if (lane == 0) atomic_max_nonneg(amax, vmax);
    return;
  }
  const int m_base = m0 + wave_m * 128, n_base = n0 + wave_n * 128;
#pragma unroll 4
  for (int p = 0; p < 32; ++p) {
    const int id = p * 64 + lane;
    const int row = id >> 4, c = id & 15;
    const u32x4 v = *reinterpret_cast<const u32x4*>(park + row * F8_EROW + c * 16);
    const int m = m_base + row, n = n_base + c * 8;
    if (m < M && n < N) *reinterpret_cast<u32x4*>(C + (int64_t)m * ldc + n) = v;
  }
}

int launch_fp8_ring(const void* A, int64_t lda, const void* W, int64_t ldw, void* C, int64_t ldc,
                    const float* a_scale, const float* w_scale, int M, int N, int K, hipStream_t stream) {
  static std::atomic<uint64_t> lds_opted_in{0};   // per instantiation, one bit per device
  if (int rc = dfhip_opt_in_lds(reinterpret_cast<const void*>(gemm_fp8_ring_kernel<false>), F8_RING_LDS, lds_opted_in)) return rc;
  const int tiles_m = (M + 255) / 256, tiles_n = (N + 255) / 256;
  hipLaunchKernelGGL(gemm_fp8_ring_kernel<false>, dim3(tiles_m * tiles_n), dim3(256), F8_RING_LDS, stream,
                     static_cast<const uint8_t*>(A), static_cast<const uint8_t*>(W), nullptr,
                     static_cast<uint16_t*>(C), a_scale, w_scale, nullptr, nullptr, M, N, K, lda, ldw, ldc, tiles_m,
                     tiles_n);
  return dfhip_check_launch();
}

int launch_fp8_ring_fused(const void* A, int64_t lda, const void* Wg, const void* Wu, int64_t ldw, void* act,
                          int64_t ld_act, const float* a_scale, const float* wg_scale, const float* wu_scale,
                          float* amax, int M, int I, int K, hipStream_t stream) {
  static std::atomic<uint64_t> lds_opted_in{0};   // per instantiation, one bit per device
  if (int rc = dfhip_opt_in_lds(reinterpret_cast<const void*>(gemm_fp8_ring_kernel<true>), F8_RING_LDS, lds_opted_in)) return rc;
  const int tiles_m = (M + 255) / 256, tiles_n = (I + 127) / 128;
  hipLaunchKernelGGL(gemm_fp8_ring_kernel<true>, dim3(tiles_m * tiles_n), dim3(256), F8_RING_LDS, stream,
                     static_cast<const uint8_t*>(A), static_cast<const uint8_t*>(Wg), static_cast<const uint8_t*>(Wu),
                     static_cast<uint16_t*>(act), a_scale, wg_scale, wu_scale, amax, M, I, K, lda, ldw, ld_act,
                     tiles_m, tiles_n);
  return dfhip_check_launch();
}


// ------------------------------------------------------------------ fp8 ring kernel, 256 x 224 tile
// The same ring with 4 waves stacked along M, each 64 x 224 = 4 x 14 MFMA blocks: column counts of
// the form 7 * 2^k (28672 = 128 * 224) then fill the rounds of 256 workgroups exactly.
constexpr int F8_TBN = 224, F8_TROW = F8_TBN * 2 + 16;

__global__ void __launch_bounds__(256)
gemm_fp8_ring224_kernel(const uint8_t* __restrict__ A, const uint8_t* __restrict__ W, uint16_t* __restrict__ C,
                        const float* __restrict__ a_scale, const float* __restrict__ w_scale, int M, int N, int K,
                        int64_t lda, int64_t ldw, int64_t ldc, int tiles_m, int tiles_n) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  const int tile = remap_xcd(blockIdx.x, tiles_m * tiles_n);
  const int per_panel = F8_GROUP_M * tiles_n;
  const int first_m = (tile / per_panel) * F8_GROUP_M;
  const int rows_in_panel = (tiles_m - first_m) < F8_GROUP_M ? (tiles_m - first_m) : F8_GROUP_M;
  const int in_panel = tile % per_panel;
  const int m0 = (first_m + in_panel % rows_in_panel) * 256;
  const int n0 = (in_panel / rows_in_panel) * F8_TBN;
  const int KT = K / FBK;

  uint32_t a_off[8], w_off[7];   // byte offsets from the tile's first row; the tile base sits in scalar registers
#pragma unroll
  for (int t = 0; t < 8; ++t) {
    const int row = (wave * 8 + t) * 8 + (lane >> 3);
    const int chunk = (lane & 7) ^ ((row >> 1) & 7);
    int ar = m0 + row; ar = ar < M ? ar : M - 1;
    a_off[t] = (uint32_t)((int64_t)(ar - m0) * lda + chunk * 16);
  }
#pragma unroll
  for (int t = 0; t < 7; ++t) {
    const int row = (wave * 7 + t) * 8 + (lane >> 3);
    const int chunk = (lane & 7) ^ ((row >> 1) & 7);
    int wr = n0 + row; wr = wr < N ? wr : N - 1;
    w_off[t] = (uint32_t)((int64_t)(wr - n0) * ldw + chunk * 16);
  }
  const uint8_t* const a_tile = A + (int64_t)m0 * lda;
  const uint8_t* const w_tile = W + (int64_t)n0 * ldw;
  auto dma_a = [&](int t, int slab, int unit) {
    const int s = slab < KT ? slab : KT - 1;
    dma16_base(unit * F8_UNIT + (wave * 8 + t) * 1024, a_tile + (int64_t)s * FBK, a_off[t]);
  };
  auto dma_w = [&](int t, int slab, int unit) {
    const int s = slab < KT ? slab : KT - 1;
    dma16_base(unit * F8_UNIT + (wave * 7 + t) * 1024, w_tile + (int64_t)s * FBK, w_off[t]);
  };

  // fragments and accumulators as in gemm_fp8_ring_kernel (16x16x128 instruction); the slab is multiplied in
  // two column halves of 7 W blocks against the wave's 4 A blocks
  const int frow = lane & 15, fquad = lane >> 4, fswz = (frow >> 1) & 7;
  int koff[2];
#pragma unroll
  for (int part = 0; part < 2; ++part) koff[part] = ((2 * fquad + part) ^ fswz) * 16;
  const int a_lane = (wave * 64 + frow) * 128, w_lane = frow * 128;

  f32x4 acc[4][14];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 14; ++j) acc[i][j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

#pragma unroll
  for (int t = 0; t < 8; ++t) dma_a(t, 0, 0);
#pragma unroll
  for (int t = 0; t < 7; ++t) dma_w(t, 0, 1);
#pragma unroll
  for (int t = 0; t < 8; ++t) dma_a(t, 1, 2);
#pragma unroll
  for (int t = 0; t < 7; ++t) dma_w(t, 1, 3);
  wait_vmcnt<15>();
  workgroup_barrier();

  u32x4 fa[2][4][2], fwa[7][2], fwb[7][2];   // [..][block][low / high 16 bytes]
  auto read_a = [&](int half_idx, int slot, int unit_a) {
    const int blk = half_idx >> 1, part = half_idx & 1;
    fa[slot][blk][part] = *reinterpret_cast<const u32x4*>(smem + unit_a * F8_UNIT + a_lane + koff[part] + blk * 2048);
  };
  auto read_w = [&](int half_idx, bool second, int unit_w) {   // half_idx 0..13 within the column half
    const int blk = half_idx >> 1, part = half_idx & 1;
    const u32x4 v = *reinterpret_cast<const u32x4*>(smem + unit_w * F8_UNIT + w_lane + koff[part] + ((second ? 7 : 0) + blk) * 2048);
    if (second) fwb[blk][part] = v; else fwa[blk][part] = v;
  };
  const int unit_scale = 0x7f7f7f7f;   // e8m0 scales 2^0
  auto mfma = [&](int q, int slot, bool second) {   // snake over 4 A blocks x 7 W blocks
    const int i = q / 7, jj = (i & 1) ? 6 - q % 7 : q % 7;
    const u32x4 (&w)[2] = second ? fwb[jj] : fwa[jj];
    const i32x8 av = {(int)fa[slot][i][0][0], (int)fa[slot][i][0][1], (int)fa[slot][i][0][2], (int)fa[slot][i][0][3],
                      (int)fa[slot][i][1][0], (int)fa[slot][i][1][1], (int)fa[slot][i][1][2], (int)fa[slot][i][1][3]};
    const i32x8 wv = {(int)w[0][0], (int)w[0][1], (int)w[0][2], (int)w[0][3], (int)w[1][0], (int)w[1][1], (int)w[1][2], (int)w[1][3]};
    asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %3 op_sel_hi:[0,0,0]"
                 : "+a"(acc[i][second ? 7 + jj : jj]) : "v"(wv), "v"(av), "v"(unit_scale));
  };
  // reads of the next slab in the order its first MFMAs need them: W block 0, A block 0, W blocks 1..6, A 1..3
  auto read_next = [&](int pos, int slot, int unit_a, int unit_w) {   // pos 0..21 (fragment halves)
    if (pos < 2) read_w(pos, false, unit_w);
    else if (pos < 4) read_a(pos - 2, slot, unit_a);
    else if (pos < 16) read_w(pos - 2, false, unit_w);
    else read_a(pos - 14, slot, unit_a);
  };

  int ua = 0, uw = 1, ia = 4, iw = 0;
#pragma unroll
  for (int pos = 0; pos < 22; ++pos) read_next(pos, 0, ua, uw);
  auto slab = [&](int kt, int sl) {
    // first column half: the 14 fragment halves of W blocks 7..13 and the 8 DMA instructions of A(kt+2)
#pragma unroll
    for (int q = 0; q < 28; ++q) {
      mfma(q, sl, false);
      if (q < 14) read_w(q, true, uw);
      if (q % 2 == 1 && q < 16) dma_a(q / 2, kt + 2, ia);
      DFHIP_PIN;
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    wait_vmcnt<8>();
    workgroup_barrier();
    int na = ua + 2; if (na >= F8_NUNITS) na -= F8_NUNITS;
    int nw = uw + 2; if (nw >= F8_NUNITS) nw -= F8_NUNITS;
    // second column half: the 7 DMA instructions of W(kt+2), then the 22 fragment halves of slab kt+1
#pragma unroll
    for (int q = 0; q < 28; ++q) {
      mfma(q, sl, true);
      if (q % 2 == 0 && q < 14) dma_w(q / 2, kt + 2, iw);
      if (q >= 6) read_next(q - 6, sl ^ 1, na, nw);
      DFHIP_PIN;
    }
    ua = na; uw = nw;
    ia += 2; if (ia >= F8_NUNITS) ia -= F8_NUNITS;
    iw += 2; if (iw >= F8_NUNITS) iw -= F8_NUNITS;
  };
  int kt = 0;
  for (; kt + 1 < KT; kt += 2) {
    slab(kt, 0);
    slab(kt + 1, 1);
  }
  if (kt < KT) slab(kt, 0);
  wait_vmcnt<0>();
  workgroup_barrier();
  asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");   // the last MFMAs have written their accumulators
  // (the compiler does not know that the statements above write the accumulators late: every later use
  // of an accumulator is tied behind the wait states)
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 14; ++j) asm volatile("" : "+a"(acc[i][j]));

  const float sa = a_scale[0];
  uint8_t* park = smem + wave * (64 * F8_TROW);
#pragma unroll
  for (int j = 0; j < 14; ++j) {
    int n = n0 + j * 16 + fquad * 4;
    n = n < N ? n : N - 4;
    const f32x4 ws = *reinterpret_cast<const f32x4*>(w_scale + n);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      u32x2 v;
      v[0] = pack2_bf16(acc[i][j][0] * (sa * ws[0]), acc[i][j][1] * (sa * ws[1]));
      v[1] = pack2_bf16(acc[i][j][2] * (sa * ws[2]), acc[i][j][3] * (sa * ws[3]));
      *reinterpret_cast<u32x2*>(park + (i * 16 + frow) * F8_TROW + (j * 16 + fquad * 4) * 2) = v;
    }
  }
  DFHIP_PIN;
  const int m_base = m0 + wave * 64;
#pragma unroll 4
  for (int p = 0; p < 28; ++p) {
    const int id = p * 64 + lane;
    const int row = id / 28, c = id - row * 28;
    const u32x4 v = *reinterpret_cast<const u32x4*>(park + row * F8_TROW + c * 16);
    const int m = m_base + row, n = n0 + c * 8;
    if (m < M && n < N) *reinterpret_cast<u32x4*>(C + (int64_t)m * ldc + n) = v;
  }
}

int launch_fp8_ring224(const void* A, int64_t lda, const void* W, int64_t ldw, void* C, int64_t ldc,
                       const float* a_scale, const float* w_scale, int M, int N, int K, hipStream_t stream) {
  static std::atomic<uint64_t> lds_opted_in{0};   // per instantiation, one bit per device
  if (int rc = dfhip_opt_in_lds(reinterpret_cast<const void*>(gemm_fp8_ring224_kernel), F8_RING_LDS, lds_opted_in)) return rc;
  const int tiles_m = (M + 255) / 256, tiles_n = (N + F8_TBN - 1) / F8_TBN;
  hipLaunchKernelGGL(gemm_fp8_ring224_kernel, dim3(tiles_m * tiles_n), dim3(256), F8_RING_LDS, stream,
                     static_cast<const uint8_t*>(A), static_cast<const uint8_t*>(W), static_cast<uint16_t*>(C),
                     a_scale, w_scale, M, N, K, lda, ldw, ldc, tiles_m, tiles_n);
  return dfhip_check_launch();
}

// Fraction of the CU-rounds that do work when [M, N] is cut into 256 x tile_n tiles dealt to 256 CUs in rounds.
double fp8_round_fill(int M, int N, int tile_n) {
  const int64_t tiles = (int64_t)((M + 255) / 256) * ((N + tile_n - 1) / tile_n);
  const int64_t rounds = (tiles + 255) / 256;
  return (double)M * N / ((double)rounds * 256 * 256 * tile_n);
}

template <int BM, int BN>
int launch_fp8(const void* A, int64_t lda, const void* W, int64_t ldw, void* C, int64_t ldc, const float* a_scale,
               const float* w_scale, int M, int N, int K, hipStream_t stream) {
  constexpr int LDS_BYTES = 2 * (BM + BN) * FROW;
  auto kernel = gemm_fp8_nt_kernel<BM, BN>;
  static std::atomic<uint64_t> lds_opted_in{0};   // per instantiation, one bit per device
  if (int rc = dfhip_opt_in_lds(reinterpret_cast<const void*>(kernel), LDS_BYTES, lds_opted_in)) return rc;
  const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
  hipLaunchKernelGGL(kernel, dim3(tiles_m * tiles_n), dim3(256), LDS_BYTES, stream, static_cast<const uint8_t*>(A),
                     static_cast<const uint8_t*>(W), static_cast<uint16_t*>(C), a_scale, w_scale, M, N, K, lda, ldw,
                     ldc, tiles_m, tiles_n);
  return dfhip_check_launch();
}

int check_q(const void* x, int64_t ld, int M, int D) {
  if (!x) return DFHIP_ERR_NULL_POINTER;
  if (M < 1 || D < 8 || D % 8 != 0 || (int64_t)M * (D / 8) >= (int64_t)1 << 31) return DFHIP_ERR_BAD_SHAPE;
  if (ld < D) return DFHIP_ERR_BAD_STRIDE;
  if (ld % 8 || !dfhip_aligned16(x)) return DFHIP_ERR_BAD_ALIGNMENT;
  return DFHIP_OK;
}

unsigned grid_for(uint32_t groups) {
  uint32_t blocks = (groups + QT * QUNROLL - 1) / (QT * QUNROLL);
  return blocks < 1 ? 1 : (blocks > 4096 ? 4096 : blocks);
}

}  // namespace

extern "C" int dfhip_absmax_bf16(const void* x, int64_t ld, int M, int D, float* amax, dfhip_stream_t stream) {
  if (int rc = check_q(x, ld, M, D)) return rc;
  if (!amax) return DFHIP_ERR_NULL_POINTER;
  const uint32_t per_row = D / 8, groups = (uint32_t)M * per_row;
  hipLaunchKernelGGL(absmax_bf16_kernel, dim3(grid_for(groups)), dim3(QT), 0, static_cast<hipStream_t>(stream),
                     static_cast<const uint16_t*>(x), ld, groups, per_row, amax);
  return dfhip_check_launch();
}

extern "C" int dfhip_quant_fp8_bf16(const void* x, int64_t ld, void* q, int64_t ld_q, int M, int D,
                                    const float* amax, float* scale_out, dfhip_stream_t stream) {
  if (int rc = check_q(x, ld, M, D)) return rc;
  if (!q || !amax) return DFHIP_ERR_NULL_POINTER;
  if (ld_q < D) return DFHIP_ERR_BAD_STRIDE;
  if (ld_q % 8 || (reinterpret_cast<uintptr_t>(q) & 7u)) return DFHIP_ERR_BAD_ALIGNMENT;
  const uint32_t per_row = D / 8, groups = (uint32_t)M * per_row;
  hipLaunchKernelGGL(quant_fp8_bf16_kernel, dim3(grid_for(groups)), dim3(QT), 0, static_cast<hipStream_t>(stream),
                     static_cast<const uint16_t*>(x), ld, static_cast<uint8_t*>(q), ld_q, groups, per_row, amax,
                     scale_out);
  return dfhip_check_launch();
}

extern "C" int dfhip_silu_mul_absmax_bf16(const void* gate, int64_t ld_gate, const void* up, int64_t ld_up,
                                          void* out, int64_t ld_out, int M, int D, float* amax,
                                          dfhip_stream_t stream) {
  if (int rc = check_q(gate, ld_gate, M, D)) return rc;
  if (int rc = check_q(up, ld_up, M, D)) return rc;
  if (!amax) return DFHIP_ERR_NULL_POINTER;
  if (out) {
    if (ld_out < D) return DFHIP_ERR_BAD_STRIDE;
    if (ld_out % 8 || !dfhip_aligned16(out)) return DFHIP_ERR_BAD_ALIGNMENT;
  }
  const uint32_t per_row = D / 8, groups = (uint32_t)M * per_row;
  hipLaunchKernelGGL(silu_mul_absmax_kernel, dim3(grid_for(groups)), dim3(QT), 0, static_cast<hipStream_t>(stream),
                     static_cast<const uint16_t*>(gate), ld_gate, static_cast<const uint16_t*>(up), ld_up,
                     static_cast<uint16_t*>(out), ld_out, groups, per_row, amax);
  return dfhip_check_launch();
}

extern "C" int dfhip_gemm_fp8_nt_variant(const void* A, int64_t lda, const void* W, int64_t ldw, void* C,
                                         int64_t ldc, const float* a_scale, const float* w_scale, int M, int N,
                                         int K, int variant, dfhip_stream_t stream) {
  if (!A || !W || !C || !a_scale || !w_scale) return DFHIP_ERR_NULL_POINTER;
  if (M < 1 || N < 1 || K < 1 || K % FBK != 0 || N % 8 != 0) return DFHIP_ERR_BAD_SHAPE;
  if (lda < K || ldw < K || ldc < N) return DFHIP_ERR_BAD_STRIDE;
  if (lda >= (1 << 23) || ldw >= (1 << 23)) return DFHIP_ERR_BAD_STRIDE;   // 256 rows of a tile within 32-bit byte offsets
  if (lda % 16 || ldw % 16 || ldc % 8 || !dfhip_aligned16(A) || !dfhip_aligned16(W) || !dfhip_aligned16(C) ||
      !dfhip_aligned16(w_scale))
    return DFHIP_ERR_BAD_ALIGNMENT;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (variant < 0) {   // the planned kernel
    const int64_t big_tiles = (int64_t)((M + 255) / 256) * ((N + 255) / 256);
    variant = 1;
    if (M > 128 && N > 128 && big_tiles >= 32)
      variant = fp8_round_fill(M, N, F8_TBN) > fp8_round_fill(M, N, 256) + 0.05 ? 2 : 0;
  }
  switch (variant) {
    case 0: return launch_fp8_ring(A, lda, W, ldw, C, ldc, a_scale, w_scale, M, N, K, s);
    case 1: return launch_fp8<128, 128>(A, lda, W, ldw, C, ldc, a_scale, w_scale, M, N, K, s);
    case 2: return launch_fp8_ring224(A, lda, W, ldw, C, ldc, a_scale, w_scale, M, N, K, s);
    default: return DFHIP_ERR_BAD_ARGUMENT;
  }
}

extern "C" int dfhip_gemm_fp8_gate_up_silu_absmax(const void* A, int64_t lda, const void* W_gate, const void* W_up,
                                                  int64_t ldw, void* act, int64_t ld_act, const float* a_scale,
                                                  const float* w_gate_scale, const float* w_up_scale, float* amax,
                                                  int M, int I, int K, dfhip_stream_t stream) {
  if (!A || !W_gate || !W_up || !act || !a_scale || !w_gate_scale || !w_up_scale || !amax)
    return DFHIP_ERR_NULL_POINTER;
  if (M < 1 || I < 8 || K < 1 || K % FBK != 0 || I % 8 != 0) return DFHIP_ERR_BAD_SHAPE;
  if (lda < K || ldw < K || ld_act < I) return DFHIP_ERR_BAD_STRIDE;
  if (lda >= (1 << 23) || ldw >= (1 << 23)) return DFHIP_ERR_BAD_STRIDE;
  if (lda % 16 || ldw % 16 || ld_act % 8 || !dfhip_aligned16(A) || !dfhip_aligned16(W_gate) ||
      !dfhip_aligned16(W_up) || !dfhip_aligned16(act) || !dfhip_aligned16(w_gate_scale) ||
      !dfhip_aligned16(w_up_scale))
    return DFHIP_ERR_BAD_ALIGNMENT;
  return launch_fp8_ring_fused(A, lda, W_gate, W_up, ldw, act, ld_act, a_scale, w_gate_scale, w_up_scale, amax, M, I,
                               K, static_cast<hipStream_t>(stream));
}

extern "C" int dfhip_gemm_fp8_nt(const void* A, int64_t lda, const void* W, int64_t ldw, void* C, int64_t ldc,
                                 const float* a_scale, const float* w_scale, int M, int N, int K,
                                 dfhip_stream_t stream) {
  return dfhip_gemm_fp8_nt_variant(A, lda, W, ldw, C, ldc, a_scale, w_scale, M, N, K, -1, stream);
}

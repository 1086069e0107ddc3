// bf16 GEMM for gfx950:  C[M,N] = A[M,K] * W[N,K]^T, fp32 accumulate, bf16 out.
//
// Both operands are K-contiguous, the layout the bf16 MFMAs want: every lane feeds
// 8 consecutive k of one row.  The MFMA is issued with W as its first operand and A
// as its second, i.e. it produces the transposed block; in the accumulator layout a
// lane then holds ONE row m of C and runs of 4 consecutive columns n.  The ring
// kernels multiply with v_mfma_f32_16x16x32_bf16, the weight-streaming and the
// register-staged kernels with v_mfma_f32_32x32x16_bf16.
//
// Two kernels:
//
// gemm_bf16_ring_kernel (the fast path, 256x256 tile, 4 waves of 128x128)
//   * K is walked in slabs of 64.  A slab of A (256 rows x 128 bytes) and a slab of
//     W are "halves" of 32 KiB each; halves are copied global->LDS by the DMA path
//     (global_load_lds_dwordx4, no registers involved) into a ring of five 32 KiB
//     units (160 KiB, the whole LDS), so that one and a half slabs are in flight
//     while one slab is being multiplied.
//   * LDS rows are 128 bytes with the 16-byte chunk index XOR-ed by (row/2)%8; the
//     DMA writes 1 KiB (8 rows) per instruction contiguously, the swizzle is applied
//     on the global side by choosing which chunk each lane fetches.  Fragment reads
//     (ds_read_b128, row = lane%32, chunk = 2*ks + lane/32) are then conflict free.
//   * one wave per SIMD means nothing hides a stall, so the loop body is pinned
//     instruction by instruction: the two k-steps of a slab go into one accumulator
//     block as a pair of MFMAs (the second adds to what the first has just written),
//     behind a pair comes at most one LDS read or one DMA issue, fragments are read
//     into registers that the walk over the 8 x 8 blocks has just freed, and the
//     workgroup barrier that hands LDS units back sits in the middle of a slab.
//   * the loop is branch free: halves past the end of K re-read the last slab into
//     units nobody reads, so the count of outstanding DMA instructions is the same in
//     every iteration (s_waitcnt vmcnt(8) before the barrier).
//   * epilogue: each wave parks its 128x128 block in LDS and stores whole 256-byte
//     row pieces (16 bytes per lane).
//   * tiles are numbered so that the ~32 workgroups resident on one XCD form a
//     4 (M) x 8 (N) block of tiles and share operand slabs in that XCD's L2.
//
// gemm_bf16_nt_kernel (generic, register staged, any tile shape of the template)
//   16-byte global loads into registers while the previous slab multiplies, parked
//   in two padded LDS buffers, one barrier per slab.  Used for small shapes.
#include <mutex>
#include <type_traits>

#include "dfhip_common.h"

// Split-K scratch of dfhip_gemm_bf16_nt_splitk_static: arrival counters followed by fp32 partial blocks,
// laid out like a caller's workspace.  One copy per GPU, held until the process ends.  In host code this
// name is only a handle for hipGetSymbolAddress; the device address it yields is what launches receive.
static __device__ __align__(256) unsigned char scratch[DFHIP_SPLITK_STATIC_BYTES];

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

// bf16(x + r) on packed pairs: the product is rounded to bf16 first (x is such a rounded value), the
// sum is rounded again - the roundings of a GEMM followed by a separate bf16 addition.
DFHIP_DEVICE uint32_t add2_bf16(uint32_t x, uint32_t r) {
  return pack2_bf16(bf16_bits_to_f32(x & 0xffffu) + bf16_bits_to_f32(r & 0xffffu),
                    __uint_as_float(x & 0xffff0000u) + __uint_as_float(r & 0xffff0000u));
}

// R (may be null): residual [M, N] with the leading dimension of C, added in the epilogue.
template <int BM, int BN, int WAVES_M, int WAVES_N>
__global__ void __launch_bounds__(WAVES_M * WAVES_N * 64)
gemm_bf16_nt_kernel(const uint16_t* __restrict__ A, const uint16_t* __restrict__ W,
                    const uint16_t* __restrict__ R, uint16_t* __restrict__ C, int M, int N, int K, int64_t lda,
                    int64_t ldw, int64_t ldc, int tiles_m, int tiles_n) {
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
          if (R) {
            const u32x2 r = *reinterpret_cast<const u32x2*>(R + (int64_t)m * ldc + n);
            v[0] = add2_bf16(v[0], r[0]);
            v[1] = add2_bf16(v[1], r[1]);
          }
          *reinterpret_cast<u32x2*>(c_row + n) = v;
        }
      }
    }
  }
}


// ------------------------------------------------------------------ ring kernel
// Results leave the ring kernels through non-temporal stores (`nt`): an output row is written once and read by
// a later kernel, never by this one, so it should not displace the operand slabs that the workgroups of an
// XCD share through its L2, nor sit there dirty until the end of the launch (measured on the 8B shapes:
// gate/up/SiLU launch 3 % faster together with the stores spread over the next tile, down projection 2 %).
constexpr int RBM = 256, RBN = 256, RTHREADS = 256;
constexpr int UNIT = 32768, NUNITS = 5, RING_LDS = UNIT * NUNITS;
constexpr int GROUP_M = 4;   // tiles of one XCD are walked in panels of GROUP_M tile rows
constexpr int EROW = 272;    // padded row of the epilogue staging area (bytes)
// Split-K: the bound of the last part's wait for the others (sleeps of about a microsecond: a second).
constexpr int SPLITK_SPIN_LIMIT = 1 << 20;

// 16-byte store / load that is coherent across the XCDs (sc1: written through to, and read
// from, the memory side instead of the XCD-private L2).  Used for split-K partial blocks so
// that no L2-wide write-back or invalidate is needed to hand them from one XCD to another.
// A store of more than 8 bytes reads its data registers for a few cycles after issue and the compiler
// cannot see that this statement is one: the wait states keep the next write to those registers away.
DFHIP_DEVICE void store_f32x4_device_coherent(f32x4* p, f32x4 v) {
  asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" ::"v"(p), "v"(v) : "memory");
}
DFHIP_DEVICE f32x4 load_f32x4_device_coherent(const f32x4* p) {
  f32x4 v;
  asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=v"(v) : "v"(p) : "memory");
  return v;
}
// The loads above are invisible to the compiler's own wait-count bookkeeping: a value may only
// be used after this, which ties the wait to the register so that the use cannot move above it.
DFHIP_DEVICE void wait_loaded(f32x4& v) { asm volatile("s_waitcnt vmcnt(0)" : "+v"(v)::"memory"); }

// Split-K workspaces start with the arrival counters.  Both split-K kernels use the same size of
// counter area for a workspace (at least 4 KiB), so that the fp32 blocks one of them leaves behind
// never lie where the other expects counters that are zero.
size_t counter_area(size_t tiles) {
  const size_t need = ((tiles * sizeof(int)) + 255) & ~(size_t)255;
  return need > 4096 ? need : 4096;
}

// Which output the W row at position `pos` of a run of paired MFMA blocks belongs to.  MFMA block j = pos / 16
// hands lane quad q = (pos % 16) / 4 the four outputs r = pos % 4; blocks are paired (0,1), (2,3), ... over 32
// outputs each, and quad q owns outputs 8q .. 8q+3 of a pair through the even block and 8q+4 .. 8q+7 through the
// odd one: eight consecutive outputs per lane and pair, one 16-byte store, four lanes a 64-byte run.
DFHIP_DEVICE int fused_pair_output_of(int pos) {
  const int j = pos >> 4, n = pos & 15;
  return 32 * (j >> 1) + 8 * (n >> 2) + 4 * (j & 1) + (n & 3);
}

template <int I, int N, class F>
DFHIP_DEVICE void static_for(F& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for<I + 1, N>(f);
  }
}

// FUSED = false: C[M,N] = A W^T.
// FUSED = true : C[M,N] = silu(A W^T) * (A W2^T) with W = gate weight, W2 = up weight, N = the
//   intermediate size.  A tile is 256 rows x 128 columns; its "W half" holds 128 gate rows and 128 up
//   rows arranged so that every wave owns gate AND up accumulators of the same 128x64 block: the
//   SiLU*mul happens in registers with the roundings of the two-kernel path (bf16 projections, bf16
//   silu, bf16 product) so that the result has the same bits, and only the product is written.
// The products are v_mfma_f32_16x16x32_bf16: a wave's 128 x 128 block is 8 x 8 blocks of 16 x 16, a slab
// of 64 is two k-steps of 32.  Per flop the instruction reads half as many accumulator registers as the
// 32x32x16 one; a loop of nothing but this instruction sustains about 15 % more at the package power
// limit, and this kernel ran 9-10 % faster than its 32x32x16 predecessor with the same ring.  The two
// k-steps of a slab go into a block as one pair of instructions: the second takes the accumulator straight
// from the first (a loop of nothing but such pairs sustains another 6 % at the power limit; this kernel gained
// 1.3 % over walking all 64 blocks per k-step, after paying 1.8 % more cycles for the order of its reads).
//   fragment of a 16-row block for k-step ks: lane -> row lane%16, 16-byte chunk 4*ks + lane/16
//   acc[i][j] (W block j first operand, A block i second): lane holds
//     C[16 i + lane%16][16 j + 4 (lane/16) + r], r = 0..3
// FUSED: blocks j = 0..3 are the gate, j = 4..7 the up projection of the same 64 outputs.
template <bool FUSED>
__global__ void __launch_bounds__(RTHREADS)
gemm_bf16_ring_kernel(const uint16_t* __restrict__ A, const uint16_t* __restrict__ W,
                      const uint16_t* __restrict__ W2, uint16_t* __restrict__ C,
                      int M, int N, int K, int64_t lda, int64_t ldw, int64_t ldc, int tiles_m, int tiles_n,
                      int split_k, int lead_slabs, float* __restrict__ partials, int* __restrict__ arrivals) {
  constexpr int TILE_N = FUSED ? 128 : RBN;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wave_m = wave & 1, wave_n = wave >> 1;

  int tile, part;
  splitk_work_of(blockIdx.x, tiles_m * tiles_n, tile, part);
  const int per_panel = GROUP_M * tiles_n;
  const int first_m = (tile / per_panel) * GROUP_M;
  const int rows_in_panel = (tiles_m - first_m) < GROUP_M ? (tiles_m - first_m) : GROUP_M;
  const int in_panel = tile % per_panel;
  const int m0 = (first_m + in_panel % rows_in_panel) * RBM;
  const int n0 = (in_panel / rows_in_panel) * TILE_N;
  // K split: parts 0 .. split_k-2 take lead_slabs slabs each, the last part takes the rest
  const int slabs_total = K / BK;
  const int slab0 = part * lead_slabs;
  const int KT = part == split_k - 1 ? slabs_total - slab0 : lead_slabs;

  uint32_t a_off[8], w_off[8];
#pragma unroll
  for (int t = 0; t < 8; ++t) {
    const int row = (wave * 8 + t) * 8 + (lane >> 3);
    const int chunk = (lane & 7) ^ ((row >> 1) & 7);
    int ar = m0 + row; ar = ar < M ? ar : M - 1;
    a_off[t] = (uint32_t)((int64_t)(ar - m0) * lda * 2 + chunk * 16);
    // FUSED: the 64 outputs of a wave column are dealt to its four gate (and four up) MFMA blocks in pairs, so that
    // a lane ends with 8 consecutive outputs per pair (fused_pair_output_of)
    int wr = FUSED ? n0 + (row >> 7) * 64 + fused_pair_output_of(row & 63) : n0 + row;
    wr = wr < N ? wr : N - 1;
    w_off[t] = (uint32_t)((int64_t)(wr - n0) * ldw * 2 + chunk * 16);
  }
  const uint8_t* const a_tile = reinterpret_cast<const uint8_t*>(A + (int64_t)m0 * lda);
  const uint8_t* const w_tile = reinterpret_cast<const uint8_t*>(((FUSED && (wave & 1)) ? W2 : W) + (int64_t)n0 * ldw);
  const uint32_t wave_lds = wave * 8 * 1024;
  auto dma_a = [&](int t, int slab, int unit) {
    const int s = slab0 + (slab < KT ? slab : KT - 1);
    dma16_base(unit * UNIT + wave_lds + t * 1024, a_tile + (int64_t)s * (BK * 2), a_off[t]);
  };
  auto dma_w = [&](int t, int slab, int unit) {
    const int s = slab0 + (slab < KT ? slab : KT - 1);
    dma16_base(unit * UNIT + wave_lds + t * 1024, w_tile + (int64_t)s * (BK * 2), w_off[t]);
  };

  const int frow = lane & 15, fquad = lane >> 4, fswz = (frow >> 1) & 7;
  int koff[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) koff[ks] = ((4 * ks + fquad) ^ fswz) * 16;
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
  wait_vmcnt<16>();   // slab 0 has landed; slab 1 may still be in flight
  workgroup_barrier();

  // K loop.  The two k-steps of a slab go into one 16 x 16 block back to back: the second product adds to the
  // accumulator that the first one has just written, which the matrix pipe hands over without the round trip
  // through the register file - less energy per product, and energy is what bounds this kernel.  For that, the W
  // fragments of a slab (both k-steps, 16 fragments) are in registers before its first product, and the 8 x 8
  // blocks are walked so that registers free up on the way:
  //   top half    rows 0 .. 3, row by row; behind the pairs of row i, the A fragments of row i + 1 and of row
  //               4 + i (and, in row 0, the W fragments of column 7, whose registers the last slab used to its end);
  //   bottom half rows 4 .. 7, column by column; behind column j its W fragments are dead and the registers
  //               take those of the next slab, which row 0 needs first.
  // A pair is one statement (nothing between its two instructions); behind a pair comes at most one LDS read
  // or one DMA issue.
  bf16x8 fa_top[2][2], fa_bot[4][2], fw[2][8];   // [row parity][k-step], [row - 4][k-step], [k-step][block]
  auto a_frag = [&](int row, int ks, int unit) {
    return *reinterpret_cast<const bf16x8*>(smem + unit * UNIT + a_lane + koff[ks] + row * 2048);
  };
  auto read_w = [&](int blk, int ks, int unit) {
    fw[ks][blk] = *reinterpret_cast<const bf16x8*>(smem + unit * UNIT + w_lane + koff[ks] + blk * 2048);
  };
  // written out so that the accumulator stays in its own registers (the compiler otherwise gives result and
  // addend different registers and moves 64 accumulators around in every iteration)
  auto mfma_pair = [&](int i, int j) {
    if (i < 4)
      asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0\n\tv_mfma_f32_16x16x32_bf16 %0, %3, %4, %0"
                   : "+a"(acc[i][j])
                   : "v"(fw[0][j]), "v"(fa_top[i & 1][0]), "v"(fw[1][j]), "v"(fa_top[i & 1][1]));
    else
      asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0\n\tv_mfma_f32_16x16x32_bf16 %0, %3, %4, %0"
                   : "+a"(acc[i][j])
                   : "v"(fw[0][j]), "v"(fa_bot[i - 4][0]), "v"(fw[1][j]), "v"(fa_bot[i - 4][1]));
  };
  // a pair with one DMA instruction behind it, as one statement: m0 is set ahead of the pair (which also is the
  // wait state that the DMA instruction needs after the move), so that only the DMA instruction itself stands
  // between this pair and the next
  auto mfma_pair_dma = [&](int i, int j, uint32_t lds_addr, const void* base, uint32_t offset) {
    if (i < 4)
      asm volatile("s_mov_b32 m0, %5\n\tv_mfma_f32_16x16x32_bf16 %0, %1, %2, %0\n\tv_mfma_f32_16x16x32_bf16 %0, %3, %4, %0"
                   "\n\tglobal_load_lds_dwordx4 %6, %7"
                   : "+a"(acc[i][j])
                   : "v"(fw[0][j]), "v"(fa_top[i & 1][0]), "v"(fw[1][j]), "v"(fa_top[i & 1][1]), "s"(lds_addr),
                     "v"(offset), "s"(base)
                   : "memory", "m0");
    else
      asm volatile("s_mov_b32 m0, %5\n\tv_mfma_f32_16x16x32_bf16 %0, %1, %2, %0\n\tv_mfma_f32_16x16x32_bf16 %0, %3, %4, %0"
                   "\n\tglobal_load_lds_dwordx4 %6, %7"
                   : "+a"(acc[i][j])
                   : "v"(fw[0][j]), "v"(fa_bot[i - 4][0]), "v"(fw[1][j]), "v"(fa_bot[i - 4][1]), "s"(lds_addr),
                     "v"(offset), "s"(base)
                   : "memory", "m0");
  };
  auto slab_of = [&](int slab) { return slab0 + (slab < KT ? slab : KT - 1); };
  // the zeros are in the accumulators before the first product reads them (the compiler would otherwise move
  // them in right in front of it, and does not know the wait states that a product needs after such a move)
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) asm volatile("" : "+a"(acc[i][j]));
  asm volatile("s_nop 7" ::: "memory");

  int ua = 0, uw = 1;   // units of the slab being multiplied
  int ia = 4, iw = 0;   // units that A(kt+2) and W(kt+2) go to
#pragma unroll
  for (int j = 0; j < 8; ++j) { read_w(j, 0, uw); read_w(j, 1, uw); }
  fa_top[0][0] = a_frag(0, 0, ua);
  fa_top[0][1] = a_frag(0, 1, ua);
  // all of them have landed before the loop: the loop's first wait then has to cover what an iteration leaves
  // in flight (the refills of the last columns), not the order of the reads above
#pragma unroll
  for (int j = 0; j < 8; ++j) asm volatile("" ::"v"(fw[0][j]), "v"(fw[1][j]));
  asm volatile("" ::"v"(fa_top[0][0]), "v"(fa_top[0][1]));
  for (int kt = 0; kt < KT; ++kt) {
    // top half.  Behind pair j of row i: row 0 starts with the two W fragments of column 7 (from this slab's unit:
    // at kt = 0 that reads again what is there); then the two A fragments of row i + 1, the two of row 4 + i; in
    // rows 1 .. 3 the DMA of A(kt+2) behind the last three pairs
#pragma unroll
    for (int p = 0; p < 32; ++p) {
      const int i = p >> 3, j = p & 7;
      const int first = i == 0 ? 2 : 0;
      const int t = (i - 1) * 3 + j - 5;               // DMA instruction of A(kt+2) behind this pair, if any
      if (i >= 1 && j >= 5 && t < 8) {
        mfma_pair_dma(i, j, ia * UNIT + wave_lds + t * 1024, a_tile + (int64_t)slab_of(kt + 2) * (BK * 2), a_off[t]);
      } else {
        mfma_pair(i, j);
        if (i == 0 && j < 2) read_w(7, j, uw);
        else if (j - first < 2) { if (i < 3) fa_top[(i + 1) & 1][j - first] = a_frag(i + 1, j - first, ua); }
        else if (j - first < 4) fa_bot[i][j - first - 2] = a_frag(4 + i, j - first - 2, ua);
      }
      DFHIP_PIN;
    }
    // every LDS read of slab kt has been issued; once they have landed its two units are free.
    // Slab kt+1 must have landed too; only the 8 instructions of A(kt+2) may still be in flight.
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    wait_vmcnt<8>();
    workgroup_barrier();
    int na = ua + 2; if (na >= NUNITS) na -= NUNITS;
    int nw = uw + 2; if (nw >= NUNITS) nw -= NUNITS;
    // bottom half.  Column j is four pairs: behind the second and third, the W fragments of slab kt+1 for column
    // j - 1 (column 0: its A fragments of row 0); behind the first and last of columns 0 .. 3, the DMA of
    // W(kt+2) into the unit A(kt) just left
#pragma unroll
    for (int p = 0; p < 32; ++p) {
      const int j = p >> 2, r = p & 3, i = 4 + r;
      if (r == 1 || r == 2) {
        mfma_pair(i, j);
        if (j == 0) fa_top[0][r - 1] = a_frag(0, r - 1, na);
        else read_w(j - 1, r - 1, nw);
      } else if (j < 4) {
        const int t = j * 2 + (r == 3);
        mfma_pair_dma(i, j, iw * UNIT + wave_lds + t * 1024, w_tile + (int64_t)slab_of(kt + 2) * (BK * 2), w_off[t]);
      } else {
        mfma_pair(i, j);
      }
      DFHIP_PIN;
    }
    ua = na; uw = nw;
    ia += 2; if (ia >= NUNITS) ia -= NUNITS;
    iw += 2; if (iw >= NUNITS) iw -= NUNITS;
  }
  wait_vmcnt<0>();      // the padding halves issued by the last iterations
  workgroup_barrier();  // other waves may still be reading fragments where this wave parks its block
  asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");   // the last MFMAs have written their accumulators
  // (the compiler does not know that the statements above write the accumulators late: every later use
  // of an accumulator is tied behind the wait states)
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) asm volatile("" : "+a"(acc[i][j]));

  uint32_t* const poison_cell = reinterpret_cast<uint32_t*>(smem + RING_LDS - 16);   // behind the parked blocks
  if (!FUSED && split_k > 1) {
    // Parts 0 .. split_k-2 of a tile leave their fp32 block in `partials`, count themselves in and are
    // done; the last part waits for that count, adds the blocks to its own accumulators in part order (so the
    // sum has one order) and writes the tile.  The launch is part-major (splitk_work_of), so the last part has
    // the highest launch index of its tile, and workgroups are dispatched in launch order: whoever it waits for
    // is already running or finished - and those never wait for anybody.  The wait is bounded; a tile whose
    // parts never arrived is filled with NaN.
    int* const counter = arrivals + tile;
    if (part != split_k - 1) {
      f32x4* mine = reinterpret_cast<f32x4*>(partials) + ((int64_t)tile * split_k + part) * (64 * RTHREADS) + tid;
#pragma unroll
      for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) store_f32x4_device_coherent(mine + (i * 8 + j) * RTHREADS, acc[i][j]);
      wait_vmcnt<0>();
      __syncthreads();
      if (tid == 0) __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      return;
    }
    if (tid == 0) {
      int spins = 0;
      while (__hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < split_k - 1 &&
             spins < SPLITK_SPIN_LIMIT) {
        __builtin_amdgcn_s_sleep(16);
        ++spins;
      }
      // OR-ed into every stored pair of bf16 values: all exponent bits and a mantissa bit, i.e. NaN
      *poison_cell = spins < SPLITK_SPIN_LIMIT ? 0u : 0x7fc07fc0u;
      __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // counters are left at zero
    }
    __syncthreads();
    const f32x4* all = reinterpret_cast<const f32x4*>(partials) + (int64_t)tile * split_k * (64 * RTHREADS) + tid;
    for (int p = 0; p < split_k - 1; ++p) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        f32x4 v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = load_f32x4_device_coherent(all + ((int64_t)p * 64 + i * 8 + j) * RTHREADS);
#pragma unroll
        for (int j = 0; j < 8; ++j) wait_loaded(v[j]);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          acc[i][j] += v[j];
          asm volatile("" : "+a"(acc[i][j]));   // back to its accumulation registers: no copies pile up
        }
      }
    }
  }

  if (FUSED) {
    // silu(gate) * up in registers (blocks j and j + 4 hold the two projections of the same outputs) and stores
    // straight from them: 8 consecutive outputs of one row per lane and pair of blocks
    auto product = [&](int i, int j) {
      u32x2 packed;
#pragma unroll
      for (int h = 0; h < 2; ++h) {   // two outputs at a time: every rounding is one packed conversion
        const uint32_t g2 = pack2_bf16(acc[i][j][2 * h], acc[i][j][2 * h + 1]);
        const uint32_t u2 = pack2_bf16(acc[i][j + 4][2 * h], acc[i][j + 4][2 * h + 1]);
        const uint32_t s2 = pack2_bf16(silu_fast(bf16_lo_to_f32(g2)), silu_fast(bf16_hi_to_f32(g2)));
        packed[h] = pack2_bf16(bf16_lo_to_f32(s2) * bf16_lo_to_f32(u2), bf16_hi_to_f32(s2) * bf16_hi_to_f32(u2));
      }
      return packed;
    };
    const int m_first = m0 + wave_m * 128 + frow, n_first = n0 + wave_n * 64 + fquad * 8;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int m = m_first + i * 16;
#pragma unroll
      for (int pr = 0; pr < 2; ++pr) {
        const u32x2 even = product(i, 2 * pr), odd = product(i, 2 * pr + 1);
        const u32x4 v = {even[0], even[1], odd[0], odd[1]};
        const int n = n_first + pr * 32;   // N % 8 == 0: a run is entirely inside or outside
        if (m < M && n < N) __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(C + (int64_t)m * ldc + n));
      }
    }
    return;
  }

  uint8_t* park = smem + wave * (128 * EROW);
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      u32x2 v;
      v[0] = pack2_bf16(acc[i][j][0], acc[i][j][1]);
      v[1] = pack2_bf16(acc[i][j][2], acc[i][j][3]);
      *reinterpret_cast<u32x2*>(park + (i * 16 + frow) * EROW + (j * 16 + fquad * 4) * 2) = v;
    }
  DFHIP_PIN;
  const uint32_t poison = split_k > 1 ? *poison_cell : 0u;   // NaN pattern if the other parts of the tile never came
  const int m_base = m0 + wave_m * 128, n_base = n0 + wave_n * 128;
#pragma unroll 4
  for (int p = 0; p < 32; ++p) {
    const int id = p * 64 + lane;
    const int row = id >> 4, c = id & 15;
    u32x4 v = *reinterpret_cast<const u32x4*>(park + row * EROW + c * 16);
    const int m = m_base + row, n = n_base + c * 8;
    if (m < M && n < N) {
      if (W2) {            // not FUSED: W2 is the optional residual [M, N] (leading dimension ldc)
        const u32x4 r = *reinterpret_cast<const u32x4*>(W2 + (int64_t)m * ldc + n);
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = add2_bf16(v[e], r[e]);
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] |= poison;
      __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(C + (int64_t)m * ldc + n));
    }
  }
}

template <bool FUSED>
int launch_ring(const void* A, int64_t lda, const void* W, const void* W2, int64_t ldw, void* C, int64_t ldc, int M,
                int N, int K, int split_k, void* workspace, hipStream_t stream) {
  auto kernel = gemm_bf16_ring_kernel<FUSED>;
  static std::atomic<uint64_t> lds_opted_in{0};   // per instantiation, one bit per device
  if (int rc = dfhip_opt_in_lds(reinterpret_cast<const void*>(kernel), RING_LDS, lds_opted_in)) return rc;
  const int tiles_m = (M + RBM - 1) / RBM;
  const int tiles_n = FUSED ? (N + 127) / 128 : (N + RBN - 1) / RBN;
  int* arrivals = static_cast<int*>(workspace);
  float* partials = nullptr;
  int lead_slabs = K / BK;
  if (split_k > 1) {
    partials = reinterpret_cast<float*>(static_cast<uint8_t*>(workspace) + counter_area((size_t)tiles_m * tiles_n));
    lead_slabs = (K / BK) / split_k;   // an even split measured best (a smaller share for the parts that only leave a block did not pay)
  }
  hipLaunchKernelGGL(kernel, dim3(tiles_m * tiles_n * split_k), dim3(RTHREADS), RING_LDS, stream,
                     static_cast<const uint16_t*>(A), static_cast<const uint16_t*>(W),
                     static_cast<const uint16_t*>(W2), static_cast<uint16_t*>(C), M, N, K, lda, ldw, ldc, tiles_m,
                     tiles_n, split_k, lead_slabs, partials, arrivals);
  return dfhip_check_launch();
}


// ------------------------------------------------------------------ ring kernel, 256 x 224 tile
// Same LDS-DMA ring as above with a tile of 256 rows x 224 columns: 4 waves stacked along M, each
// 64 x 224 = 4 x 14 MFMA blocks of 16 x 16 (224 accumulator registers).  Column counts that are multiples of
// 7 * 2^k (Llama's 14336 = 64 * 224) then give a tile count that divides evenly over the 256 CUs
// (512 tiles instead of 448 of 256 x 256: 2 full rounds instead of 1.75 rounded up to 2).
// FUSED: the W half holds 112 gate rows then 112 up rows, so a lane's accumulators of blocks j and
// j + 7 are the two projections of the same outputs: bf16(bf16(silu(g)) * u) - the roundings of the
// two-kernel path - is computed in registers and stored from there, 8 bytes per lane.
constexpr int TBN = 224;
// The column count is a template parameter: 224 as described, and 128 (4 x 8 blocks per wave, not FUSED) for
// shapes whose 256 x 256 tiling has at most half as many tiles as the GPU has CUs - 256 x 128 tiles then fill
// a round without a split along K and its fp32 partial blocks.

// Fused 224-wide tile: which of the tile's 112 outputs the W row at position `pos` (0..111 within the gate or
// the up part of the W half) belongs to.  MFMA block j = pos / 16 hands lane quad q = (pos % 16) / 4 the four
// outputs r = pos % 4.  Blocks are paired: (0,1), (2,3), (4,5) cover 32 outputs each, and quad q owns outputs
// 8q .. 8q+3 of a pair through the even block and 8q+4 .. 8q+7 through the odd one - eight consecutive
// outputs, one 16-byte store, four lanes a 64-byte run (the size of a write request; with four outputs per lane
// a tile went out as twice as many 32-byte requests).  The seventh block keeps the plain order.
DFHIP_DEVICE int fused224_output_of(int pos) { return pos < 96 ? fused_pair_output_of(pos) : pos; }

template <bool FUSED, int TN>
__global__ void __launch_bounds__(RTHREADS)
gemm_bf16_ring224_kernel(const uint16_t* __restrict__ A, const uint16_t* __restrict__ W,
                         const uint16_t* __restrict__ W2, uint16_t* __restrict__ C,
                         int M, int N, int K, int64_t lda, int64_t ldw, int64_t ldc, int tiles_m, int tiles_n) {
  constexpr int OUT_N = FUSED ? TN / 2 : TN;
  constexpr int JB = TN / 16;          // 16-column MFMA blocks of a wave: 14 or 8
  constexpr int WP = TN / 32;          // DMA instructions of a W half per wave: 7 or 4
  constexpr int NR = 4 + JB;           // fragment reads per k-step
  constexpr int MQ = 4 * JB;           // MFMAs per k-step
  constexpr int TROW = TN * 2 + 16;    // padded row of the staging area (bytes)
  static_assert(!FUSED || TN == TBN, "the fused form exists for the 224-wide tile only");
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  const int tile = remap_xcd(blockIdx.x, tiles_m * tiles_n);
  const int per_panel = GROUP_M * tiles_n;
  const int first_m = (tile / per_panel) * GROUP_M;
  const int rows_in_panel = (tiles_m - first_m) < GROUP_M ? (tiles_m - first_m) : GROUP_M;
  const int in_panel = tile % per_panel;
  const int m0 = (first_m + in_panel % rows_in_panel) * RBM;
  const int n0 = (in_panel / rows_in_panel) * OUT_N;
  const int KT = K / BK;

  // DMA sources.  A half: 32 instructions of 8 rows, 8 per wave.  W half: 28 instructions, 7 per wave
  // (FUSED: 14 of gate rows, then 14 of up rows: waves 0, 1 read W, waves 2, 3 read W2).  The address is a
  // wave-uniform tile base (scalar registers, advanced per slab) plus a 32-bit byte offset per lane.
  uint32_t a_off[8], w_off[WP];
#pragma unroll
  for (int t = 0; t < 8; ++t) {
    const int row = (wave * 8 + t) * 8 + (lane >> 3);
    const int chunk = (lane & 7) ^ ((row >> 1) & 7);
    int ar = m0 + row; ar = ar < M ? ar : M - 1;
    a_off[t] = (uint32_t)((int64_t)(ar - m0) * lda * 2 + chunk * 16);
  }
#pragma unroll
  for (int t = 0; t < WP; ++t) {
    const int row = (wave * WP + t) * 8 + (lane >> 3);
    const int chunk = (lane & 7) ^ ((row >> 1) & 7);
    int wr = n0 + (FUSED ? fused224_output_of(row >= OUT_N ? row - OUT_N : row) : row);
    wr = wr < N ? wr : N - 1;
    w_off[t] = (uint32_t)((int64_t)(wr - n0) * ldw * 2 + chunk * 16);
  }
  const uint8_t* const a_tile = reinterpret_cast<const uint8_t*>(A + (int64_t)m0 * lda);
  const uint8_t* const w_tile = reinterpret_cast<const uint8_t*>(((FUSED && wave >= 2) ? W2 : W) + (int64_t)n0 * ldw);
  auto dma_a = [&](int t, int slab, int unit) {
    const int s = slab < KT ? slab : KT - 1;
    dma16_base(unit * UNIT + (wave * 8 + t) * 1024, a_tile + (int64_t)s * (BK * 2), a_off[t]);
  };
  auto dma_w = [&](int t, int slab, int unit) {
    const int s = slab < KT ? slab : KT - 1;
    dma16_base(unit * UNIT + (wave * WP + t) * 1024, w_tile + (int64_t)s * (BK * 2), w_off[t]);
  };

  const int frow = lane & 15, fquad = lane >> 4, fswz = (frow >> 1) & 7;
  int koff[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) koff[ks] = ((4 * ks + fquad) ^ fswz) * 16;
  const int a_lane = (wave * 64 + frow) * 128, w_lane = frow * 128;

  f32x4 acc[4][JB];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < JB; ++j) acc[i][j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

#pragma unroll
  for (int t = 0; t < 8; ++t) dma_a(t, 0, 0);
#pragma unroll
  for (int t = 0; t < WP; ++t) dma_w(t, 0, 1);
#pragma unroll
  for (int t = 0; t < 8; ++t) dma_a(t, 1, 2);
#pragma unroll
  for (int t = 0; t < WP; ++t) dma_w(t, 1, 3);
  wait_vmcnt<8 + WP>();   // slab 0 has landed; slab 1 may still be in flight
  workgroup_barrier();

  bf16x8 fa[2][4], fw[2][JB];
  // fragments in the order the MFMAs need them: W block 0, A block 0, W blocks 1.., A blocks 1..3
  auto read_frag = [&](int pos, int ks, int slot, int unit_a, int unit_w) {
    const bool is_a = pos == 1 || pos > JB;
    const int blk = pos <= 1 ? 0 : pos <= JB ? pos - 1 : pos - JB;
    if (is_a)
      fa[slot][blk] = *reinterpret_cast<const bf16x8*>(smem + unit_a * UNIT + a_lane + koff[ks] + blk * 2048);
    else
      fw[slot][blk] = *reinterpret_cast<const bf16x8*>(smem + unit_w * UNIT + w_lane + koff[ks] + blk * 2048);
  };
  auto mfma = [&](int q, int slot) {   // snake order: odd rows walk the W blocks backwards
    const int i = q / JB, j = (i & 1) ? JB - 1 - q % JB : q % JB;
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc[i][j]) : "v"(fw[slot][j]), "v"(fa[slot][i]));
  };

  int ua = 0, uw = 1;   // units of the slab being multiplied
  int ia = 4, iw = 0;   // units that A(kt+2) and W(kt+2) go to
#pragma unroll
  for (int pos = 0; pos < NR; ++pos) read_frag(pos, 0, 0, ua, uw);
  for (int kt = 0; kt < KT; ++kt) {
    // k-step 0: the fragments of k-step 1 behind the first MFMAs, the 8 pieces of A(kt+2) spread over the rest
    constexpr int A0 = TN == TBN ? NR + 2 : NR, AS = (MQ - A0) / 8;
#pragma unroll
    for (int q = 0; q < MQ; ++q) {
      mfma(q, 0);
      if (q < NR) read_frag(q, 1, 1, ua, uw);
      else if (q >= A0 && (q - A0) % AS == 0 && (q - A0) / AS < 8) dma_a((q - A0) / AS, kt + 2, ia);
      DFHIP_PIN;
    }
    // all LDS reads of slab kt issued; slab kt+1 must have landed, only A(kt+2) may be in flight
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    wait_vmcnt<8>();
    workgroup_barrier();
    int na = ua + 2; if (na >= NUNITS) na -= NUNITS;
    int nw = uw + 2; if (nw >= NUNITS) nw -= NUNITS;
    // k-step 1: the pieces of W(kt+2) behind every fourth MFMA, then the fragments of slab kt+1, k-step 0
#pragma unroll
    for (int q = 0; q < MQ; ++q) {
      mfma(q, 1);
      if (q < 4 * WP) { if (q % 4 == 0) dma_w(q / 4, kt + 2, iw); }
      else if (q < 4 * WP + NR) read_frag(q - 4 * WP, 0, 0, na, nw);
      DFHIP_PIN;
    }
    ua = na; uw = nw;
    ia += 2; if (ia >= NUNITS) ia -= NUNITS;
    iw += 2; if (iw >= NUNITS) iw -= NUNITS;
  }
  wait_vmcnt<0>();
  workgroup_barrier();
  asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");   // the last MFMAs have written their accumulators
  // (the compiler does not know that the statements above write the accumulators late: every later use
  // of an accumulator is tied behind the wait states)
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < JB; ++j) asm volatile("" : "+a"(acc[i][j]));

  if (FUSED) {
    // silu(gate) * up in registers (blocks j and j + 7 hold the two projections of the same outputs) and
    // stores straight from the registers: a lane owns 8 consecutive outputs of one row per pair of blocks
    // (see fused224_output_of) and 4 of the seventh block
    const int m_first = m0 + wave * 64 + frow;
    auto product = [&](int i, int j) {
      u32x2 packed;
#pragma unroll
      for (int h = 0; h < 2; ++h) {   // two outputs at a time: every rounding is one packed conversion
        const uint32_t g2 = pack2_bf16(acc[i][j][2 * h], acc[i][j][2 * h + 1]);
        const uint32_t u2 = pack2_bf16(acc[i][j + JB / 2][2 * h], acc[i][j + JB / 2][2 * h + 1]);
        const uint32_t s2 = pack2_bf16(silu_fast(bf16_lo_to_f32(g2)), silu_fast(bf16_hi_to_f32(g2)));
        packed[h] = pack2_bf16(bf16_lo_to_f32(s2) * bf16_lo_to_f32(u2), bf16_hi_to_f32(s2) * bf16_hi_to_f32(u2));
      }
      return packed;
    };
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = m_first + i * 16;
#pragma unroll
      for (int pr = 0; pr < 3; ++pr) {
        const u32x2 even = product(i, 2 * pr), odd = product(i, 2 * pr + 1);
        const u32x4 v = {even[0], even[1], odd[0], odd[1]};
        const int n = n0 + pr * 32 + fquad * 8;   // N % 8 == 0: the run is entirely inside or outside
        if (m < M && n < N) __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(C + (int64_t)m * ldc + n));
      }
      const u32x2 v = product(i, 6);
      const int n = n0 + 96 + fquad * 4;
      if (m < M && n < N) __builtin_nontemporal_store(v, reinterpret_cast<u32x2*>(C + (int64_t)m * ldc + n));
    }
    return;
  }
  // park 64 rows x 224 columns per wave as bf16, then store whole row pieces
  uint8_t* park = smem + wave * (64 * TROW);
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < JB; ++j) {
      u32x2 v;
      v[0] = pack2_bf16(acc[i][j][0], acc[i][j][1]);
      v[1] = pack2_bf16(acc[i][j][2], acc[i][j][3]);
      *reinterpret_cast<u32x2*>(park + (i * 16 + frow) * TROW + (j * 16 + fquad * 4) * 2) = v;
    }
  DFHIP_PIN;
  const int m_base = m0 + wave * 64;
  constexpr int CPR = TN / 8;   // 16-byte pieces of a row
#pragma unroll 4
  for (int p = 0; p < CPR; ++p) {
    const int id = p * 64 + lane;
    const int row = id / CPR, c = id - row * CPR;
    u32x4 v = *reinterpret_cast<const u32x4*>(park + row * TROW + c * 16);
    const int m = m_base + row, n = n0 + c * 8;
    if (m < M && n < N) {
      if (W2) {            // not FUSED: W2 is the optional residual [M, N] (leading dimension ldc)
        const u32x4 r = *reinterpret_cast<const u32x4*>(W2 + (int64_t)m * ldc + n);
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = add2_bf16(v[e], r[e]);
      }
      __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(C + (int64_t)m * ldc + n));
    }
  }
}

template <bool FUSED, int TN = TBN>
int launch_ring224(const void* A, int64_t lda, const void* W, const void* W2, int64_t ldw, void* C, int64_t ldc,
                   int M, int N, int K, hipStream_t stream) {
  auto kernel = gemm_bf16_ring224_kernel<FUSED, TN>;
  static std::atomic<uint64_t> lds_opted_in{0};   // per instantiation, one bit per device
  if (int rc = dfhip_opt_in_lds(reinterpret_cast<const void*>(kernel), RING_LDS, lds_opted_in)) return rc;
  constexpr int OUT_N = FUSED ? TN / 2 : TN;
  const int tiles_m = (M + RBM - 1) / RBM;
  const int tiles_n = (N + OUT_N - 1) / OUT_N;
  hipLaunchKernelGGL(kernel, dim3(tiles_m * tiles_n), dim3(RTHREADS), RING_LDS, stream,
                     static_cast<const uint16_t*>(A), static_cast<const uint16_t*>(W),
                     static_cast<const uint16_t*>(W2), static_cast<uint16_t*>(C), M, N, K, lda, ldw, ldc, tiles_m,
                     tiles_n);
  return dfhip_check_launch();
}


// ------------------------------------------------------------------ fused 256 x 224 kernel that walks its tiles
// gate/up projection with the SiLU*mul epilogue, as gemm_bf16_ring224_kernel<true>, with one workgroup per
// compute unit that walks several tiles (the tiles the same unit would get round by round) and never lets
// the ring run dry:
//   * the DMA of a tile's last two iterations fetches the first slabs of the NEXT tile, so a tile starts with
//     its operands in LDS;
//   * a tile's results (56 registers of packed bf16 per lane) are stored during the first iterations of the
//     next tile's K loop, a few store instructions per slab, instead of all at once at the end of a round.
// The first MFMAs of a tile take a zero addend instead of the accumulator, so nothing is cleared in between.
// Full tiles only: M % 256 == 0, N % 112 == 0, K / 64 >= WALK_MIN_SLABS.
#ifndef WALK_STORES_PER_SLAB
#define WALK_STORES_PER_SLAB 4
#endif
constexpr int WALK_STORES = WALK_STORES_PER_SLAB;    // stores behind one slab of the next tile
constexpr int WALK_PEEL = 16 / WALK_STORES;          // iterations of the next tile that carry stores
constexpr int WALK_MIN_SLABS = WALK_PEEL + 3;

__global__ void __launch_bounds__(RTHREADS)
gemm_bf16_gate_up_silu_walk_kernel(const uint16_t* __restrict__ A, const uint16_t* __restrict__ W,
                                   const uint16_t* __restrict__ W2, uint16_t* __restrict__ C,
                                   int M, int N, int K, int64_t lda, int64_t ldw, int64_t ldc, int tiles_m,
                                   int tiles_n) {
  constexpr int TN = TBN, OUT_N = TN / 2, JB = TN / 16, WP = TN / 32, NR = 4 + JB, MQ = 4 * JB;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int KT = K / BK;

  // Tiles of this workgroup: workgroup b runs on XCD b % 8 and is slot b / 8 there; an XCD owns a contiguous
  // range of tiles (as remap_xcd deals them) and slot s takes tiles s, s + slots, s + 2 slots, ... of it.
  const int total = tiles_m * tiles_n;
  const int slots = gridDim.x / 8;
  const int xcd = blockIdx.x % 8, slot = blockIdx.x / 8;
  const int share = total / 8, rest = total % 8;
  const int first_tile = xcd * share + (xcd < rest ? xcd : rest);
  const int count = share + (xcd < rest ? 1 : 0);
  const int n_tiles = slot < count ? (count - slot + slots - 1) / slots : 0;
  if (n_tiles == 0) return;

  const uint8_t* const w_base = reinterpret_cast<const uint8_t*>(wave >= 2 ? W2 : W);
  const int per_panel = GROUP_M * tiles_n;
  auto origin = [&](int walk, int& m0, int& n0) {
    const int tile = first_tile + slot + walk * slots;
    const int first_m = (tile / per_panel) * GROUP_M;
    const int rows_in_panel = (tiles_m - first_m) < GROUP_M ? (tiles_m - first_m) : GROUP_M;
    const int in_panel = tile % per_panel;
    m0 = (first_m + in_panel % rows_in_panel) * RBM;
    n0 = (in_panel / rows_in_panel) * OUT_N;
  };

  // DMA sources: instruction t of a wave fetches rows 8 t .. 8 t + 7 of the wave's share of a half.  The
  // swizzled chunk a lane fetches depends on t only through its parity, so two per-lane byte offsets per
  // operand do; the 16 rows between instructions t and t + 2 go into the wave-uniform base.
  uint32_t a_off[2], w_off[4];
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    const int row = (wave * 8 + t) * 8 + (lane >> 3);
    const int chunk = (lane & 7) ^ ((row >> 1) & 7);
    a_off[t] = (uint32_t)((int64_t)row * lda * 2 + chunk * 16);
  }
  // W: the rows of a half are dealt to the MFMA blocks by fused224_output_of.  Instructions 0 .. 4 of a wave lie
  // in paired blocks, where the rows of instruction t are those of instruction t & 1 shifted by a wave-uniform
  // number of rows; instructions 5 and 6 (the seventh block, for the odd waves) have offsets of their own.
  auto w_pos = [&](int t) { return ((wave & 1) * WP + t) * 8; };   // first position of instruction t in its part
  auto w_lane_off = [&](int t) {
    const int row = (wave * WP + t) * 8 + (lane >> 3);              // row of the W half in LDS
    const int chunk = (lane & 7) ^ ((row >> 1) & 7);
    return (uint32_t)((int64_t)fused224_output_of(w_pos(t) + (lane >> 3)) * ldw * 2 + chunk * 16);
  };
  w_off[0] = w_lane_off(0);
  w_off[1] = w_lane_off(1);
  w_off[2] = w_lane_off(5);
  w_off[3] = w_lane_off(6);
  const int64_t a_rows16 = 16 * lda * 2;
  auto dma_a = [&](int t, const uint8_t* slab, int unit) {
    dma16_base(unit * UNIT + (wave * 8 + t) * 1024, slab + (t >> 1) * a_rows16, a_off[t & 1]);
  };
  auto dma_w = [&](int t, const uint8_t* slab, int unit) {
    if (t < 5) {
      const int shift = fused224_output_of(w_pos(t)) - fused224_output_of(w_pos(t & 1));
      dma16_base(unit * UNIT + (wave * WP + t) * 1024, slab + shift * (ldw * 2), w_off[t & 1]);
    } else {
      dma16_base(unit * UNIT + (wave * WP + t) * 1024, slab, w_off[t - 3]);
    }
  };

  const int frow = lane & 15, fquad = lane >> 4, fswz = (frow >> 1) & 7;
  int koff[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) koff[ks] = ((4 * ks + fquad) ^ fswz) * 16;
  const int a_lane = (wave * 64 + frow) * 128, w_lane = frow * 128;

  f32x4 acc[4][JB];       // defined by the first MFMAs of every tile (zero addend)
  // the finished tile, waiting to be stored: per 16 rows three runs of 8 outputs and one of 4 (fused224_output_of)
  u32x4 out16[4][3];
  u32x2 out8[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
#pragma unroll
    for (int j = 0; j < 3; ++j) out16[i][j] = u32x4{0u, 0u, 0u, 0u};
    out8[i] = u32x2{0u, 0u};
  }

  int m0, n0;
  origin(0, m0, n0);
  const uint8_t* a_cur = reinterpret_cast<const uint8_t*>(A + (int64_t)m0 * lda);
  const uint8_t* w_cur = w_base + (int64_t)n0 * ldw * 2;
  // where the slabs behind the end of the current tile come from: the next tile, or (last tile) its own last two
  const uint8_t* a_nxt = a_cur + (int64_t)(KT - 2) * (BK * 2);
  const uint8_t* w_nxt = w_cur + (int64_t)(KT - 2) * (BK * 2);
  if (n_tiles > 1) {
    int m1, n1;
    origin(1, m1, n1);
    a_nxt = reinterpret_cast<const uint8_t*>(A + (int64_t)m1 * lda);
    w_nxt = w_base + (int64_t)n1 * ldw * 2;
  }
  // results: wave-uniform address of the wave's 64 rows of the tile + a 32-bit byte offset per lane
  uint8_t* c_cur = reinterpret_cast<uint8_t*>(C + ((int64_t)(m0 + wave * 64)) * ldc + n0);
  uint8_t* c_pend = c_cur;
  const int64_t c_rows16 = 16 * ldc * 2;
  const uint32_t c_lane16 = (uint32_t)((frow * ldc + fquad * 8) * 2), c_lane8 = (uint32_t)((frow * ldc + fquad * 4) * 2);

#pragma unroll
  for (int t = 0; t < 8; ++t) dma_a(t, a_cur, 0);
#pragma unroll
  for (int t = 0; t < WP; ++t) dma_w(t, w_cur, 1);
#pragma unroll
  for (int t = 0; t < 8; ++t) dma_a(t, a_cur + BK * 2, 2);
#pragma unroll
  for (int t = 0; t < WP; ++t) dma_w(t, w_cur + BK * 2, 3);
  wait_vmcnt<8 + WP>();   // slab 0 has landed; slab 1 may still be in flight
  workgroup_barrier();

  bf16x8 fa[2][4], fw[2][JB];
  auto read_frag = [&](int pos, int ks, int slot_, int unit_a, int unit_w) {
    const bool is_a = pos == 1 || pos > JB;
    const int blk = pos <= 1 ? 0 : pos <= JB ? pos - 1 : pos - JB;
    if (is_a)
      fa[slot_][blk] = *reinterpret_cast<const bf16x8*>(smem + unit_a * UNIT + a_lane + koff[ks] + blk * 2048);
    else
      fw[slot_][blk] = *reinterpret_cast<const bf16x8*>(smem + unit_w * UNIT + w_lane + koff[ks] + blk * 2048);
  };
  auto mfma = [&](int q, int slot_) {   // snake order: odd rows walk the W blocks backwards
    const int i = q / JB, j = (i & 1) ? JB - 1 - q % JB : q % JB;
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc[i][j]) : "v"(fw[slot_][j]), "v"(fa[slot_][i]));
  };
  auto mfma_first = [&](int q) {        // first k-step of a tile: zero addend, the old accumulator is dead
    const int i = q / JB, j = (i & 1) ? JB - 1 - q % JB : q % JB;
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, 0" : "=a"(acc[i][j]) : "v"(fw[0][j]), "v"(fa[0][i]));
  };
  auto store_out = [&](int idx) {   // store idx of the 16 of a tile
    const int i = idx / 4, run = idx % 4;
    // written out for the addressing mode: uniform base in scalar registers + the lane's 32-bit offset (the
    // wait states: the base may have come out of a vector register just before, which a memory instruction
    // may only read five cycles later, and the compiler does not look into this statement)
    if (run < 3)
      asm volatile("s_nop 4\n\tglobal_store_dwordx4 %0, %1, %2 nt" ::"v"(c_lane16), "v"(out16[i][run]),
                   "s"(c_pend + i * c_rows16 + run * 64)
                   : "memory");
    else
      asm volatile("s_nop 4\n\tglobal_store_dwordx2 %0, %1, %2 nt" ::"v"(c_lane8), "v"(out8[i]),
                   "s"(c_pend + i * c_rows16 + 192)
                   : "memory");
  };

  int ua = 0, uw = 1;   // units of the slab being multiplied
  int ia = 4, iw = 0;   // units that the A and W halves two slabs ahead go to
  // One iteration = one slab.  FIRST: first slab of a tile (zero addend).  The iteration issues stores
  // [STORE0, STORE0 + STORES) of the previous tile (if there is one) ahead of the DMA instructions of its second
  // k-step: memory instructions complete in order, so by the wait of the next iteration - which needs those
  // DMA pieces anyway - the stores are no younger than what is waited for, and the count of 8 stays exact.
  bool pending = false;
  auto iteration = [&](int kt, auto first_c, auto store0_c, auto stores_c) {
    constexpr bool FIRST = decltype(first_c)::value;
    constexpr int STORE0 = decltype(store0_c)::value, STORES = decltype(stores_c)::value;
    constexpr int A0 = NR + 2, AS = (MQ - A0) / 8;
    const int s2 = kt + 2;
    const uint8_t* const pa = s2 < KT ? a_cur + (int64_t)s2 * (BK * 2) : a_nxt + (int64_t)(s2 - KT) * (BK * 2);
    const uint8_t* const pw = s2 < KT ? w_cur + (int64_t)s2 * (BK * 2) : w_nxt + (int64_t)(s2 - KT) * (BK * 2);
#pragma unroll
    for (int q = 0; q < MQ; ++q) {
      if (FIRST) mfma_first(q); else mfma(q, 0);
      if (q < NR) read_frag(q, 1, 1, ua, uw);
      else if (q >= A0 && (q - A0) % AS == 0 && (q - A0) / AS < 8) dma_a((q - A0) / AS, pa, ia);
      DFHIP_PIN;
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    wait_vmcnt<8>();
    workgroup_barrier();
    int na = ua + 2; if (na >= NUNITS) na -= NUNITS;
    int nw = uw + 2; if (nw >= NUNITS) nw -= NUNITS;
    if (STORES > 0 && pending) {
#pragma unroll
      for (int t = 0; t < STORES; ++t) store_out(STORE0 + t);
    }
    DFHIP_PIN;
#pragma unroll
    for (int q = 0; q < MQ; ++q) {
      mfma(q, 1);
      if (q < 4 * WP) { if (q % 4 == 0) dma_w(q / 4, pw, iw); }
      else if (q < 4 * WP + NR) read_frag(q - 4 * WP, 0, 0, na, nw);
      DFHIP_PIN;
    }
    ua = na; uw = nw;
    ia += 2; if (ia >= NUNITS) ia -= NUNITS;
    iw += 2; if (iw >= NUNITS) iw -= NUNITS;
  };
  using std::integral_constant;
  auto peeled = [&](auto p_c) {   // iteration p of a tile
    constexpr int P = decltype(p_c)::value;
    iteration(P, integral_constant<bool, P == 0>{}, integral_constant<int, P * WALK_STORES>{},
              integral_constant<int, WALK_STORES>{});
  };

#pragma unroll
  for (int pos = 0; pos < NR; ++pos) read_frag(pos, 0, 0, ua, uw);
  for (int walk = 0; walk < n_tiles; ++walk) {
    static_for<0, WALK_PEEL>(peeled);
    for (int kt = WALK_PEEL; kt < KT; ++kt)
      iteration(kt, integral_constant<bool, false>{}, integral_constant<int, 0>{}, integral_constant<int, 0>{});

    // the tile is complete once the last MFMAs have written their accumulators (the compiler does not know
    // that they write late: every later use of an accumulator is tied behind the wait states)
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
    // silu(gate) * up with the roundings of the separate kernels (blocks j and j + 7 hold the two projections).
    // The accumulators are read out here, group by group, by written-out moves: left to the compiler, all of
    // them were copied out ahead of the arithmetic and did not fit.
    auto product = [&](int i, int j) {
      float ga[4], ub[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(ga[e]) : "a"(acc[i][j][e]));
        asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(ub[e]) : "a"(acc[i][j + JB / 2][e]));
      }
      u32x2 packed;
#pragma unroll
      for (int h = 0; h < 2; ++h) {   // two outputs at a time: every rounding is one packed conversion
        const uint32_t g2 = pack2_bf16(ga[2 * h], ga[2 * h + 1]), u2 = pack2_bf16(ub[2 * h], ub[2 * h + 1]);
        const uint32_t s2 = pack2_bf16(silu_fast(bf16_lo_to_f32(g2)), silu_fast(bf16_hi_to_f32(g2)));
        packed[h] = pack2_bf16(bf16_lo_to_f32(s2) * bf16_lo_to_f32(u2), bf16_hi_to_f32(s2) * bf16_hi_to_f32(u2));
      }
      DFHIP_PIN;
      return packed;
    };
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
      for (int run = 0; run < 3; ++run) {
        const u32x2 even = product(i, 2 * run), odd = product(i, 2 * run + 1);
        out16[i][run] = u32x4{even[0], even[1], odd[0], odd[1]};
      }
      out8[i] = product(i, 6);
    }
    // the first fragments of the next tile (the last iteration read them too, into registers that the code
    // above was free to use: read again rather than kept alive through it)
#pragma unroll
    for (int pos = 0; pos < NR; ++pos) read_frag(pos, 0, 0, ua, uw);
    c_pend = c_cur;
    pending = true;
    // on to the next tile: its first slabs are in LDS or on their way
    a_cur = a_nxt;
    w_cur = w_nxt;
    if (walk + 1 < n_tiles) {
      origin(walk + 1, m0, n0);
      c_cur = reinterpret_cast<uint8_t*>(C + ((int64_t)(m0 + wave * 64)) * ldc + n0);
    }
    if (walk + 2 < n_tiles) {
      int m2, n2;
      origin(walk + 2, m2, n2);
      a_nxt = reinterpret_cast<const uint8_t*>(A + (int64_t)m2 * lda);
      w_nxt = w_base + (int64_t)n2 * ldw * 2;
    } else {
      a_nxt = a_cur + (int64_t)(KT - 2) * (BK * 2);
      w_nxt = w_cur + (int64_t)(KT - 2) * (BK * 2);
    }
  }
  // the last tile has no successor to hide behind
#pragma unroll
  for (int idx = 0; idx < 16; ++idx) store_out(idx);
  wait_vmcnt<0>();   // no DMA may be in flight when the workgroup gives its LDS back
}

int compute_units_of_current_device() {
  static std::atomic<int> cached[64];
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return 0;
  int n = cached[device].load(std::memory_order_relaxed);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess) return 0;
    cached[device].store(n, std::memory_order_relaxed);
  }
  return n;
}

bool walk_kernel_fits(int M, int N, int K) {
  return M % RBM == 0 && N % (TBN / 2) == 0 && K / BK >= WALK_MIN_SLABS;
}

int launch_walk(const void* A, int64_t lda, const void* W, const void* W2, int64_t ldw, void* C, int64_t ldc,
                int M, int N, int K, hipStream_t stream) {
  auto kernel = gemm_bf16_gate_up_silu_walk_kernel;
  static std::atomic<uint64_t> lds_opted_in{0};
  if (int rc = dfhip_opt_in_lds(reinterpret_cast<const void*>(kernel), RING_LDS, lds_opted_in)) return rc;
  const int tiles_m = M / RBM, tiles_n = N / (TBN / 2);
  int grid = compute_units_of_current_device() / 8 * 8;   // one workgroup per compute unit, a multiple of the XCDs
  if (grid < 8) return DFHIP_ERR_NO_DEVICE;
  const int rounds = (tiles_m * tiles_n + grid - 1) / grid;
  // no more workgroups than the longest walk needs: an XCD's tiles spread evenly over its slots
  const int per_xcd = (tiles_m * tiles_n + 7) / 8;
  const int slots = (per_xcd + rounds - 1) / rounds;
  if (slots * 8 < grid) grid = slots * 8;
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(RTHREADS), RING_LDS, stream, static_cast<const uint16_t*>(A),
                     static_cast<const uint16_t*>(W), static_cast<const uint16_t*>(W2), static_cast<uint16_t*>(C),
                     M, N, K, lda, ldw, ldc, tiles_m, tiles_n);
  return dfhip_check_launch();
}


// ------------------------------------------------------------------ weight-streaming kernel, M <= 1024
// Decode-sized activations (a nano-batch of single-token queries): the GEMM is bound by reading W
// once from HBM.  Tile 128 rows x 128 columns, 4 waves of 64 x 64, K in slabs of 64 through
// a ring of four 32 KiB units (A half + W half of a slab) filled by LDS-DMA, three slabs in flight per
// workgroup.  K is split over `split_k` workgroups per tile so that up to 256 workgroups (one round) stream
// different parts of W at the same time; the parts meet through the same ticket scheme as above.
// Workgroups of one K part are neighbours (they share the A columns of that part in one XCD's L2),
// and with more than 128 rows the row tiles of one column tile are direct neighbours: W leaves HBM
// once and the other row tiles find it in that XCD's L2.  Results leave through ordinary stores, not the
// non-temporal ones of the large-tile kernels: they are a few MB that the next kernel of the chain reads at once
// (decode step 16.85 -> 16.72 ms).
// (a ring of five units, one more slab in flight, measured no faster on any decode shape)
constexpr int SK_BM = 128, SK_BN = 128, SK_UNITS = 4, SK_UNIT = 32768, SK_LDS = SK_UNITS * SK_UNIT;
constexpr int SK_AHEAD = SK_UNITS - 1;          // slabs issued ahead of the one being multiplied
constexpr int SK_FLIGHT = (SK_AHEAD - 2) * 8;   // DMA instructions of a wave that may still be in flight at a barrier
constexpr int SK_MAX_M = 1024;

// FUSED: C[M, N] = silu(A W^T) * (A W2^T) (gate and up weights, N = the intermediate size, K not split):
// a tile is 128 rows x 64 columns, its W half holds, per wave column, 32 gate rows and the 32 matching up
// rows, so MFMA block j = 0 is the gate and j = 1 the up projection of the same outputs.
template <bool FUSED>
__global__ void __launch_bounds__(RTHREADS)
gemm_bf16_skinny_kernel(const uint16_t* __restrict__ A, const uint16_t* __restrict__ W,
                        const uint16_t* __restrict__ W2, uint16_t* __restrict__ C,
                        int M, int N, int K, int64_t lda, int64_t ldw, int64_t ldc, int tiles_m, int tiles_n,
                        int split_k, float* __restrict__ partials, int* __restrict__ arrivals) {
  constexpr int TILE_N = FUSED ? SK_BN / 2 : SK_BN;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wave_m = wave & 1, wave_n = wave >> 1;
  const int tiles = tiles_m * tiles_n;
  const int work = remap_xcd(blockIdx.x, tiles * split_k);
  const int part = work / tiles;
  const int tile = work - part * tiles;        // column tile major, row tile minor
  const int tile_n = tile / tiles_m;
  const int m0 = (tile - tile_n * tiles_m) * SK_BM;
  const int n0 = tile_n * TILE_N;
  const int slabs_total = K / BK;
  const int slab0 = (int)((int64_t)slabs_total * part / split_k);
  const int KT = (int)((int64_t)slabs_total * (part + 1) / split_k) - slab0;

  // DMA: a half is 128 rows x 128 bytes = 16 instructions of 8 rows, 4 per wave
  const uint8_t* a_src[4];
  const uint8_t* w_src[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const int row = (wave * 4 + t) * 8 + (lane >> 3);
    const int chunk = (lane & 7) ^ ((row >> 1) & 7);
    const int ar = m0 + row < M ? m0 + row : M - 1;
    a_src[t] = reinterpret_cast<const uint8_t*>(A + (int64_t)ar * lda + chunk * 8);
    if (FUSED) {
      const int block = row >> 5;                       // 32-row block: wave column block/2, (0: gate, 1: up)
      int wr = n0 + (block >> 1) * 32 + (row & 31); wr = wr < N ? wr : N - 1;
      w_src[t] = reinterpret_cast<const uint8_t*>(((block & 1) ? W2 : W) + (int64_t)wr * ldw + chunk * 8);
    } else {
      int wr = n0 + row; wr = wr < N ? wr : N - 1;
      w_src[t] = reinterpret_cast<const uint8_t*>(W + (int64_t)wr * ldw + chunk * 8);
    }
  }
  auto issue = [&](int slab, int unit) {
    const int64_t off = (int64_t)(slab0 + (slab < KT ? slab : KT - 1)) * (BK * 2);
#pragma unroll
    for (int t = 0; t < 4; ++t) dma16(unit * SK_UNIT + (wave * 4 + t) * 1024, a_src[t] + off);
#pragma unroll
    for (int t = 0; t < 4; ++t) dma16(unit * SK_UNIT + 16384 + (wave * 4 + t) * 1024, w_src[t] + off);
  };

  const int frow = lane & 31, fhalf = lane >> 5, fswz = (frow >> 1) & 7;
  int koff[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) koff[ks] = ((2 * ks + fhalf) ^ fswz) * 16;
  const int a_lane = (wave_m * 64 + frow) * 128, w_lane = 16384 + (wave_n * 64 + frow) * 128;

  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  // Fragments are double-buffered by hand: the reads of k-step s+1 (or of the next slab's first k-step)
  // are issued before the MFMAs of step s, so no LDS latency is exposed inside a slab or across slabs.
  bf16x8 fa[2][2], fw[2][2];
  auto read_frags = [&](int slab, int ks, int slot) {
    const uint8_t* u = smem + (slab % SK_UNITS) * SK_UNIT;
#pragma unroll
    for (int i = 0; i < 2; ++i) fa[slot][i] = *reinterpret_cast<const bf16x8*>(u + a_lane + i * 4096 + koff[ks]);
#pragma unroll
    for (int j = 0; j < 2; ++j) fw[slot][j] = *reinterpret_cast<const bf16x8*>(u + w_lane + j * 4096 + koff[ks]);
  };
#pragma unroll
  for (int u = 0; u < SK_AHEAD; ++u) issue(u, u);
  wait_vmcnt<SK_FLIGHT>();   // slabs 0 and 1 have landed
  workgroup_barrier();
  read_frags(0, 0, 0);
  for (int kt = 0; kt < KT; ++kt) {
    issue(kt + SK_AHEAD, (kt + SK_AHEAD) % SK_UNITS);   // into the unit of slab kt-1: everybody passed the barrier after it
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      const int slot = ks & 1;
      if (ks < 3) read_frags(kt, ks + 1, slot ^ 1); else read_frags(kt + 1, 0, slot ^ 1);   // slab kt+1 has landed
      DFHIP_PIN;
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fw[slot][j], fa[slot][i], acc[i][j], 0, 0, 0);
      DFHIP_PIN;
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // every read of slab kt (and the prefetch) has returned
    wait_vmcnt<SK_FLIGHT>();   // slab kt+2 has landed; only the slabs after it may be in flight
    workgroup_barrier();
  }
  wait_vmcnt<0>();
  workgroup_barrier();

  if (split_k > 1) {
    f32x4* mine = reinterpret_cast<f32x4*>(partials) + ((int64_t)tile * split_k + part) * (16 * RTHREADS) + tid;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          f32x4 v = {acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
          store_f32x4_device_coherent(mine + ((i * 2 + j) * 4 + g) * RTHREADS, v);
        }
    wait_vmcnt<0>();
    __syncthreads();
    int* ticket_cell = reinterpret_cast<int*>(smem);
    if (tid == 0) *ticket_cell = atomicAdd(arrivals + tile, 1);
    __syncthreads();
    const int ticket = *ticket_cell;
    __syncthreads();
    if (ticket != split_k - 1) return;
    if (tid == 0) atomicExch(arrivals + tile, 0);
    // the last arriver adds the parts in part order (its own is read back like the others)
    const f32x4* all = reinterpret_cast<const f32x4*>(partials) + (int64_t)tile * split_k * (16 * RTHREADS) + tid;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
    for (int p = 0; p < split_k; ++p) {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        f32x4 v[8];
#pragma unroll
        for (int c = 0; c < 8; ++c) v[c] = load_f32x4_device_coherent(all + ((int64_t)p * 16 + h * 8 + c) * RTHREADS);
#pragma unroll
        for (int c = 0; c < 8; ++c) wait_loaded(v[c]);
#pragma unroll
        for (int c = 0; c < 8; ++c) {
          const int i = h, j = c >> 2, g = c & 3;
          acc[i][j][4 * g] += v[c][0];
          acc[i][j][4 * g + 1] += v[c][1];
          acc[i][j][4 * g + 2] += v[c][2];
          acc[i][j][4 * g + 3] += v[c][3];
        }
      }
    }
  }

  if (FUSED) {
    // the roundings of the separate kernels: bf16 projections, bf16 silu, bf16 product
    constexpr int FROW = 80;
    uint8_t* fpark = smem + wave * (64 * FROW);
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        float p[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float gt = bf16_bits_to_f32(f32_to_bf16_bits(acc[i][0][4 * g + e]));
          const float ut = bf16_bits_to_f32(f32_to_bf16_bits(acc[i][1][4 * g + e]));
          p[e] = bf16_bits_to_f32(f32_to_bf16_bits(silu_fast(gt))) * ut;
        }
        u32x2 v;
        v[0] = pack2_bf16(p[0], p[1]);
        v[1] = pack2_bf16(p[2], p[3]);
        *reinterpret_cast<u32x2*>(fpark + (i * 32 + frow) * FROW + (g * 8 + fhalf * 4) * 2) = v;
      }
    DFHIP_PIN;
    const int fm_base = m0 + wave_m * 64, fn_base = n0 + wave_n * 32;
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      const int id = p * 64 + lane;
      const int row = id >> 2, c = id & 3;
      const u32x4 v = *reinterpret_cast<const u32x4*>(fpark + row * FROW + c * 16);
      const int m = fm_base + row, n = fn_base + c * 8;
      if (m < M && n < N) *reinterpret_cast<u32x4*>(C + (int64_t)m * ldc + n) = v;
    }
    return;
  }

  // park 64 rows x 64 columns per wave (144-byte rows), then whole 128-byte row pieces
  constexpr int PROW = 144;
  uint8_t* park = smem + wave * (64 * PROW);
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        u32x2 v;
        v[0] = pack2_bf16(acc[i][j][4 * g + 0], acc[i][j][4 * g + 1]);
        v[1] = pack2_bf16(acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]);
        *reinterpret_cast<u32x2*>(park + (i * 32 + frow) * PROW + (j * 32 + g * 8 + fhalf * 4) * 2) = v;
      }
  DFHIP_PIN;
  const int m_base = m0 + wave_m * 64, n_base = n0 + wave_n * 64;
#pragma unroll 4
  for (int p = 0; p < 8; ++p) {
    const int id = p * 64 + lane;
    const int row = id >> 3, c = id & 7;
    u32x4 v = *reinterpret_cast<const u32x4*>(park + row * PROW + c * 16);
    const int m = m_base + row, n = n_base + c * 8;
    if (m < M && n < N) {
      if (W2) {            // not FUSED: W2 is the optional residual [M, N] (leading dimension ldc)
        const u32x4 r = *reinterpret_cast<const u32x4*>(W2 + (int64_t)m * ldc + n);
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = add2_bf16(v[e], r[e]);
      }
      *reinterpret_cast<u32x4*>(C + (int64_t)m * ldc + n) = v;
    }
  }
}

// The fused launch with twice the columns per workgroup: 128 rows x 128 outputs (128 gate rows and 128 up rows of
// W per slab), 4 waves of 64 rows x 64 outputs (two gate and two up blocks of 32 rows each).  Half as many
// workgroups move half as many activation bytes through LDS per weight byte and meet at half as many barriers;
// a unit of the ring is A 16 KiB | W 32 KiB and three of them fit, so a slab's first fragments are read after the
// barrier that follows its landing (no read ahead across slabs) and two slabs are in flight meanwhile.  For two
// launches that share the GPU (2 x 112 workgroups at 14336 outputs: one round together) and for 129 .. 256 rows.
// Same instruction and same order of K as gemm_bf16_skinny_kernel<true>: the same bits.
constexpr int SKW_BN = 128, SKW_UNIT = 49152, SKW_UNITS = 3, SKW_LDS = SKW_UNITS * SKW_UNIT;

__global__ void __launch_bounds__(RTHREADS)
gemm_bf16_skinny_wide_kernel(const uint16_t* __restrict__ A, const uint16_t* __restrict__ W,
                             const uint16_t* __restrict__ W2, uint16_t* __restrict__ C, int M, int N, int K,
                             int64_t lda, int64_t ldw, int64_t ldc, int tiles_m, int tiles_n) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wave_m = wave & 1, wave_n = wave >> 1;
  const int tile = remap_xcd(blockIdx.x, tiles_m * tiles_n);   // column tile major, row tile minor
  const int tile_n = tile / tiles_m;
  const int m0 = (tile - tile_n * tiles_m) * SK_BM;
  const int n0 = tile_n * SKW_BN;
  const int KT = K / BK;

  // DMA: the A part is 128 rows x 128 bytes = 16 instructions of 8 rows (4 per wave), the W part 256 rows = 32
  // instructions (8 per wave); W row r of the unit: wave column r / 128, (gate, up) = (r / 64) % 2, output r % 64
  const uint8_t* a_src[4];
  const uint8_t* w_src[8];
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const int row = (wave * 4 + t) * 8 + (lane >> 3);
    const int chunk = (lane & 7) ^ ((row >> 1) & 7);
    const int ar = m0 + row < M ? m0 + row : M - 1;
    a_src[t] = reinterpret_cast<const uint8_t*>(A + (int64_t)ar * lda + chunk * 8);
  }
#pragma unroll
  for (int t = 0; t < 8; ++t) {
    const int row = (wave * 8 + t) * 8 + (lane >> 3);
    const int chunk = (lane & 7) ^ ((row >> 1) & 7);
    int wr = n0 + (row >> 7) * 64 + (row & 63);
    wr = wr < N ? wr : N - 1;
    w_src[t] = reinterpret_cast<const uint8_t*>((((row >> 6) & 1) ? W2 : W) + (int64_t)wr * ldw + chunk * 8);
  }
  auto issue = [&](int slab, int unit) {
    const int64_t off = (int64_t)(slab < KT ? slab : KT - 1) * (BK * 2);
#pragma unroll
    for (int t = 0; t < 4; ++t) dma16(unit * SKW_UNIT + (wave * 4 + t) * 1024, a_src[t] + off);
#pragma unroll
    for (int t = 0; t < 8; ++t) dma16(unit * SKW_UNIT + 16384 + (wave * 8 + t) * 1024, w_src[t] + off);
  };

  const int frow = lane & 31, fhalf = lane >> 5, fswz = (frow >> 1) & 7;
  int koff[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) koff[ks] = ((2 * ks + fhalf) ^ fswz) * 16;
  const int a_lane = (wave_m * 64 + frow) * 128, w_lane = 16384 + (wave_n * 128 + frow) * 128;

  f32x16 acc[2][4];   // [row block][gate 0, gate 1, up 0, up 1]
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  bf16x8 fa[2][2], fw[2][4];
  auto read_frags = [&](int unit, int ks, int slot) {
    const uint8_t* u = smem + unit * SKW_UNIT;
#pragma unroll
    for (int i = 0; i < 2; ++i) fa[slot][i] = *reinterpret_cast<const bf16x8*>(u + a_lane + i * 4096 + koff[ks]);
#pragma unroll
    for (int j = 0; j < 4; ++j) fw[slot][j] = *reinterpret_cast<const bf16x8*>(u + w_lane + j * 4096 + koff[ks]);
  };
  issue(0, 0);
  issue(1, 1);
  wait_vmcnt<12>();          // slab 0 has landed
  workgroup_barrier();
  int unit = 0;
  for (int kt = 0; kt < KT; ++kt) {
    read_frags(unit, 0, 0);
    const int free_unit = unit == 0 ? SKW_UNITS - 1 : unit - 1;   // slab kt-1: everybody passed the barrier after it
    issue(kt + 2, free_unit);
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      const int slot = ks & 1;
      if (ks < 3) read_frags(unit, ks + 1, slot ^ 1);
      DFHIP_PIN;
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fw[slot][j], fa[slot][i], acc[i][j], 0, 0, 0);
      DFHIP_PIN;
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // every read of slab kt has returned
    wait_vmcnt<12>();        // slab kt+1 has landed; only slab kt+2 may be in flight
    workgroup_barrier();
    unit = unit == SKW_UNITS - 1 ? 0 : unit + 1;
  }
  wait_vmcnt<0>();
  workgroup_barrier();

  // the roundings of the separate kernels (bf16 projections, bf16 silu, bf16 product); 64 rows x 64 outputs per
  // wave are parked in LDS (144-byte rows) and leave as whole 128-byte row pieces
  constexpr int PROW = 144;
  uint8_t* park = smem + wave * (64 * PROW);
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int jj = 0; jj < 2; ++jj)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        float p[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float gt = bf16_bits_to_f32(f32_to_bf16_bits(acc[i][jj][4 * g + e]));
          const float ut = bf16_bits_to_f32(f32_to_bf16_bits(acc[i][2 + jj][4 * g + e]));
          p[e] = bf16_bits_to_f32(f32_to_bf16_bits(silu_fast(gt))) * ut;
        }
        u32x2 v;
        v[0] = pack2_bf16(p[0], p[1]);
        v[1] = pack2_bf16(p[2], p[3]);
        *reinterpret_cast<u32x2*>(park + (i * 32 + frow) * PROW + (jj * 32 + g * 8 + fhalf * 4) * 2) = v;
      }
  DFHIP_PIN;
  const int m_base = m0 + wave_m * 64, n_base = n0 + wave_n * 64;
#pragma unroll 4
  for (int p = 0; p < 8; ++p) {
    const int id = p * 64 + lane;
    const int row = id >> 3, c = id & 7;
    const u32x4 v = *reinterpret_cast<const u32x4*>(park + row * PROW + c * 16);
    const int m = m_base + row, n = n_base + c * 8;
    if (m < M && n < N) *reinterpret_cast<u32x4*>(C + (int64_t)m * ldc + n) = v;
  }
}

size_t skinny_tiles(int M, int N) { return (size_t)((M + SK_BM - 1) / SK_BM) * ((N + SK_BN - 1) / SK_BN); }
size_t skinny_counter_bytes(int M, int N) { return counter_area(skinny_tiles(M, N)); }

template <bool FUSED>
int launch_skinny(const void* A, int64_t lda, const void* W, const void* W2, int64_t ldw, void* C, int64_t ldc, int M,
                  int N, int K, int split_k, void* workspace, hipStream_t stream) {
  if (M > SK_MAX_M || (FUSED && split_k != 1)) return DFHIP_ERR_BAD_SHAPE;
  auto kernel = gemm_bf16_skinny_kernel<FUSED>;
  static std::atomic<uint64_t> lds_opted_in{0};   // per instantiation, one bit per device
  if (int rc = dfhip_opt_in_lds(reinterpret_cast<const void*>(kernel), SK_LDS, lds_opted_in)) return rc;
  constexpr int TILE_N = FUSED ? SK_BN / 2 : SK_BN;
  const int tiles_m = (M + SK_BM - 1) / SK_BM;
  const int tiles_n = (N + TILE_N - 1) / TILE_N;
  int* arrivals = static_cast<int*>(workspace);
  float* partials = nullptr;
  if (split_k > 1) partials = reinterpret_cast<float*>(static_cast<uint8_t*>(workspace) + skinny_counter_bytes(M, N));
  hipLaunchKernelGGL(kernel, dim3(tiles_m * tiles_n * split_k), dim3(RTHREADS), SK_LDS, stream,
                     static_cast<const uint16_t*>(A), static_cast<const uint16_t*>(W),
                     static_cast<const uint16_t*>(W2), static_cast<uint16_t*>(C), M, N, K, lda, ldw, ldc, tiles_m,
                     tiles_n, split_k, partials, arrivals);
  return dfhip_check_launch();
}

int launch_skinny_wide(const void* A, int64_t lda, const void* W, const void* W2, int64_t ldw, void* C, int64_t ldc,
                       int M, int N, int K, hipStream_t stream) {
  if (M > SK_MAX_M || K / BK < 2) return DFHIP_ERR_BAD_SHAPE;
  auto kernel = gemm_bf16_skinny_wide_kernel;
  static std::atomic<uint64_t> lds_opted_in{0};
  if (int rc = dfhip_opt_in_lds(reinterpret_cast<const void*>(kernel), SKW_LDS, lds_opted_in)) return rc;
  const int tiles_m = (M + SK_BM - 1) / SK_BM;
  const int tiles_n = (N + SKW_BN - 1) / SKW_BN;
  hipLaunchKernelGGL(kernel, dim3(tiles_m * tiles_n), dim3(RTHREADS), SKW_LDS, stream,
                     static_cast<const uint16_t*>(A), static_cast<const uint16_t*>(W),
                     static_cast<const uint16_t*>(W2), static_cast<uint16_t*>(C), M, N, K, lda, ldw, ldc, tiles_m,
                     tiles_n);
  return dfhip_check_launch();
}

template <int BM, int BN, int WAVES_M, int WAVES_N>
int launch(const void* A, int64_t lda, const void* W, int64_t ldw, void* C, int64_t ldc, int M, int N,
           int K, hipStream_t stream, const void* R = nullptr) {
  using S = Shape<BM, BN, WAVES_M, WAVES_N>;
  auto kernel = gemm_bf16_nt_kernel<BM, BN, WAVES_M, WAVES_N>;
  static std::atomic<uint64_t> lds_opted_in{0};   // per instantiation, one bit per device
  if (int rc = dfhip_opt_in_lds(reinterpret_cast<const void*>(kernel), S::LDS_BYTES, lds_opted_in)) return rc;
  const int tiles_m = (M + BM - 1) / BM;
  const int tiles_n = (N + BN - 1) / BN;
  hipLaunchKernelGGL(kernel, dim3(tiles_m * tiles_n), dim3(S::THREADS), S::LDS_BYTES, stream,
                     static_cast<const uint16_t*>(A), static_cast<const uint16_t*>(W),
                     static_cast<const uint16_t*>(R), static_cast<uint16_t*>(C), M, N, K, lda, ldw, ldc, tiles_m,
                     tiles_n);
  return dfhip_check_launch();
}

// Fraction of the CU-rounds that do work when [M, N] is cut into 256 x tile_n tiles and the
// tiles are dealt to 256 CUs in rounds, weighted by the columns of a tile that exist.
// `share` launches of this shape run side by side and take their rounds together.
double round_fill(int M, int N, int tile_n, int share = 1) {
  const int64_t tiles = (int64_t)((M + RBM - 1) / RBM) * ((N + tile_n - 1) / tile_n) * share;
  const int64_t rounds = (tiles + 255) / 256;
  return (double)M * N * share / ((double)rounds * 256 * RBM * tile_n);
}

int check_args(const void* A, int64_t lda, const void* W, int64_t ldw, void* C, int64_t ldc, int M, int N,
               int K) {
  if (!A || !W || !C) return DFHIP_ERR_NULL_POINTER;
  if (M < 1 || N < 1 || K < 1 || K % BK != 0 || N % 8 != 0) return DFHIP_ERR_BAD_SHAPE;
  if (lda < K || ldw < K || ldc < N) return DFHIP_ERR_BAD_STRIDE;
  if (lda >= (1 << 22) || ldw >= (1 << 22)) return DFHIP_ERR_BAD_STRIDE;   // 256 rows of a tile within 32-bit byte offsets
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
    case 0: return launch_ring<false>(A, lda, W, nullptr, ldw, C, ldc, M, N, K, 1, nullptr, s);
    case 4: return launch<256, 256, 2, 2>(A, lda, W, ldw, C, ldc, M, N, K, s);
    case 1: return launch<256, 256, 2, 4>(A, lda, W, ldw, C, ldc, M, N, K, s);
    case 2: return launch<128, 128, 2, 2>(A, lda, W, ldw, C, ldc, M, N, K, s);
    case 3: return launch<256, 128, 2, 2>(A, lda, W, ldw, C, ldc, M, N, K, s);
    case 5: return launch_ring224<false>(A, lda, W, nullptr, ldw, C, ldc, M, N, K, s);
    case 7: return launch_ring224<false, 128>(A, lda, W, nullptr, ldw, C, ldc, M, N, K, s);
    case 6: return launch_skinny<false>(A, lda, W, nullptr, ldw, C, ldc, M, N, K, 1, nullptr, s);
    default: return DFHIP_ERR_BAD_ARGUMENT;
  }
}

extern "C" int dfhip_gemm_bf16_plan(int M, int N, int K, int* variant, int* split_k) {
  return dfhip_gemm_bf16_plan_shared(M, N, K, 1, variant, split_k);
}

extern "C" int dfhip_gemm_bf16_plan_shared(int M, int N, int K, int share, int* variant, int* split_k) {
  if (!variant || !split_k) return DFHIP_ERR_NULL_POINTER;
  if (M < 1 || N < 1 || K < 1) return DFHIP_ERR_BAD_SHAPE;
  if (share < 1 || share > 16) return DFHIP_ERR_BAD_ARGUMENT;
  // The 256x256 ring kernel whenever the problem has more than half a tile of rows and columns
  // and enough tiles to occupy a good part of the 256 CUs; the small register-staged tile
  // otherwise.  With at most half as many tiles as CUs, K is split so that every CU gets a part.
  const int64_t big_tiles = (int64_t)((M + 255) / 256) * ((N + 255) / 256);
  *variant = 2;
  *split_k = 1;
  // decode-sized activations: up to 128 rows always, up to 512 rows (1024 with K <= 8192: with a longer K the
  // 256 x 256 tiles with K split win) while the 128 x 128 tiles fit one round of 256 workgroups; beyond that
  // the 256 x 256 tiles below move fewer bytes through LDS per flop
  const int tiles = (int)skinny_tiles(M, N);
  const bool one_round = tiles <= 256 && (M <= 512 || (M <= SK_MAX_M && K <= 8192));
  if ((M <= SK_BM || one_round) && M >= 16 && N >= 1024 && K >= 1024) {
    // stream W with as many workgroups as fit ONE round of 256 (a second round costs more than it brings), but
    // at least 12 slabs per part: shorter loops fall below a workgroup's fixed costs and every further part is
    // another fp32 block written and read (measured over the 8B shapes at 128 and 256 rows, parts 2 .. 12)
    int s = 256 / (tiles * share);            // launches that run side by side take the round together
    if (s < 1) s = 1;
    if (s > 16) s = 16;
    while (s > 1 && K / BK < 12 * s) --s;
    *variant = 6;
    *split_k = s;
    return DFHIP_OK;
  }
  if (M > 128 && N > 128 && big_tiles >= 32) {
    *variant = 0;
    int s = (int)(256 / (big_tiles * share));   // launches that run side by side fill the compute units together
    if (s > 8) s = 8;
    while (s > 1 && K / BK < 16 * s) --s;   // keep at least 16 slabs per part
    if (s > 1) *split_k = s;
    // few tiles and a short K: 256 x 128 tiles fill the CUs without the fp32 partial blocks of a split
    // (with K = 14336 the split 256 x 256 tiles are as fast or faster)
    if (s > 1 && K <= 8192) {
      *variant = 7;
      *split_k = 1;
      return DFHIP_OK;
    }
    // 256 x 224 tiles when they fill the rounds of 256 workgroups clearly better (N = 7 * 2^k)
    if (s <= 1 && round_fill(M, N, TBN, share) > round_fill(M, N, RBN, share) + 0.05) *variant = 5;
  }
  return DFHIP_OK;
}

extern "C" int dfhip_gemm_bf16_nt(const void* A, int64_t lda, const void* W, int64_t ldw, void* C,
                                  int64_t ldc, int M, int N, int K, dfhip_stream_t stream) {
  int variant = 2, split_k = 1;
  if (int rc = dfhip_gemm_bf16_plan(M, N, K, &variant, &split_k)) return rc;
  return dfhip_gemm_bf16_nt_variant(A, lda, W, ldw, C, ldc, M, N, K, variant, stream);
}

extern "C" size_t dfhip_gemm_bf16_splitk_workspace_bytes(int M, int N, int split_k) {
  if (M < 1 || N < 1 || split_k < 2) return 0;
  const size_t tiles = (size_t)((M + RBM - 1) / RBM) * ((N + RBN - 1) / RBN);
  const size_t ring = counter_area(tiles) + tiles * split_k * (size_t)RBM * RBN * sizeof(float);
  if (M > SK_MAX_M) return ring;
  // the weight-streaming kernel (M <= 1024) has its own layout; a caller sizes for whichever is used
  const size_t skinny = skinny_counter_bytes(M, N) + skinny_tiles(M, N) * split_k * (size_t)SK_BM * SK_BN * sizeof(float);
  return ring > skinny ? ring : skinny;
}

extern "C" int dfhip_gemm_bf16_nt_splitk(const void* A, int64_t lda, const void* W, int64_t ldw, void* C,
                                         int64_t ldc, int M, int N, int K, int split_k, void* workspace,
                                         size_t workspace_bytes, dfhip_stream_t stream) {
  if (int rc = check_args(A, lda, W, ldw, C, ldc, M, N, K)) return rc;
  if (split_k < 1 || split_k > 16 || K / BK < split_k) return DFHIP_ERR_BAD_ARGUMENT;
  if (split_k > 1) {
    if (!workspace) return DFHIP_ERR_NULL_POINTER;
    if (!dfhip_aligned16(workspace)) return DFHIP_ERR_BAD_ALIGNMENT;
    if (workspace_bytes < dfhip_gemm_bf16_splitk_workspace_bytes(M, N, split_k)) return DFHIP_ERR_BAD_ARGUMENT;
  }
  int variant = 0, planned = 1;
  dfhip_gemm_bf16_plan(M, N, K, &variant, &planned);
  if (variant == 6)
    return launch_skinny<false>(A, lda, W, nullptr, ldw, C, ldc, M, N, K, split_k, workspace,
                                static_cast<hipStream_t>(stream));
  if (split_k > 8) return DFHIP_ERR_BAD_ARGUMENT;
  return launch_ring<false>(A, lda, W, nullptr, ldw, C, ldc, M, N, K, split_k, workspace,
                            static_cast<hipStream_t>(stream));
}

extern "C" int dfhip_gemm_bf16_splitk_work(int launch_index, int tiles, int split_k, int* tile, int* part) {
  if (!tile || !part) return DFHIP_ERR_NULL_POINTER;
  if (tiles < 1 || split_k < 1 || launch_index < 0 || (int64_t)launch_index >= (int64_t)tiles * split_k)
    return DFHIP_ERR_BAD_ARGUMENT;
  splitk_work_of(launch_index, tiles, *tile, *part);
  return DFHIP_OK;
}

extern "C" int dfhip_gemm_bf16_gate_up_silu(const void* A, int64_t lda, const void* W_gate, const void* W_up,
                                            int64_t ldw, void* Out, int64_t ldo, int M, int I, int K,
                                            dfhip_stream_t stream) {
  return dfhip_gemm_bf16_gate_up_silu_shared(A, lda, W_gate, W_up, ldw, Out, ldo, M, I, K, 1, stream);
}

extern "C" int dfhip_gemm_bf16_gate_up_silu_shared(const void* A, int64_t lda, const void* W_gate, const void* W_up,
                                                   int64_t ldw, void* Out, int64_t ldo, int M, int I, int K,
                                                   int share, dfhip_stream_t stream) {
  if (!W_up) return DFHIP_ERR_NULL_POINTER;
  if (share < 1 || share > 16) return DFHIP_ERR_BAD_ARGUMENT;
  if (int rc = check_args(A, lda, W_gate, ldw, Out, ldo, M, I, K)) return rc;
  if (!dfhip_aligned16(W_up)) return DFHIP_ERR_BAD_ALIGNMENT;
  if (M <= 2 * SK_BM && I >= 1024 && K >= 1024) {   // decode-sized activations: stream both weights once
    // 128 outputs per workgroup when the launches that run side by side, or the two row tiles of 129 .. 256
    // rows, then still give every compute unit a workgroup's worth of the round; 64 outputs otherwise
    // (8B shape, us: a pair of 128-row launches on two streams 99.5 -> 88, one 256-row launch 88.6 -> 75.9, but a
    // lone 128-row launch 55 -> 71 with its 112 workgroups)
    const int64_t wide = (int64_t)((M + SK_BM - 1) / SK_BM) * ((I + SKW_BN - 1) / SKW_BN) * share;
    if (wide >= 192)
      return launch_skinny_wide(A, lda, W_gate, W_up, ldw, Out, ldo, M, I, K, static_cast<hipStream_t>(stream));
    return launch_skinny<true>(A, lda, W_gate, W_up, ldw, Out, ldo, M, I, K, 1, nullptr,
                               static_cast<hipStream_t>(stream));
  }
  // the 256 x (112 + 112) tile when it fills the rounds of 256 workgroups clearly better than the 256 x (128 + 128)
  // one, which moves fewer bytes through LDS per flop; launches that run side by side take their rounds together
  // (two launches of the 8B shape at 2048 rows: 2 x 896 square tiles are exactly 7 rounds)
  if (round_fill(M, I, TBN / 2, share) > round_fill(M, I, 128, share) + 0.05) {
    // a launch that has the GPU to itself and more than one round of tiles: workgroups that walk their tiles hide
    // a tile's stores behind the next one (they hold their compute units to the end, so nothing runs beside them)
    if (share == 1 && walk_kernel_fits(M, I, K) && ldo < (1 << 22) && (int64_t)(M / RBM) * (I / (TBN / 2)) > 256)
      return launch_walk(A, lda, W_gate, W_up, ldw, Out, ldo, M, I, K, static_cast<hipStream_t>(stream));
    return launch_ring224<true>(A, lda, W_gate, W_up, ldw, Out, ldo, M, I, K, static_cast<hipStream_t>(stream));
  }
  // (a walking form of this tile - each launch of a pair on half the compute units, seven tiles per workgroup -
  // was measured on the 8B shape and is 1 % slower than one tile per workgroup: under the package power limit a
  // hidden epilogue buys nothing, and a launch that walks cannot give its idle units to the other one)
  return launch_ring<true>(A, lda, W_gate, W_up, ldw, Out, ldo, M, I, K, 1, nullptr,
                           static_cast<hipStream_t>(stream));
}

extern "C" int dfhip_gemm_bf16_nt_add(const void* A, int64_t lda, const void* W, int64_t ldw, const void* R, void* C,
                                      int64_t ldc, int M, int N, int K, int split_k, void* workspace,
                                      size_t workspace_bytes, dfhip_stream_t stream) {
  if (!R) return DFHIP_ERR_NULL_POINTER;
  if (int rc = check_args(A, lda, W, ldw, C, ldc, M, N, K)) return rc;
  if (!dfhip_aligned16(R)) return DFHIP_ERR_BAD_ALIGNMENT;
  int variant = 2, planned = 1;
  if (int rc = dfhip_gemm_bf16_plan(M, N, K, &variant, &planned)) return rc;
  if (split_k < 1 || split_k > 16 || K / BK < split_k) return DFHIP_ERR_BAD_ARGUMENT;
  if (split_k > 1) {
    if (variant != 0 && variant != 6) return DFHIP_ERR_BAD_ARGUMENT;   // the planned kernel does not split K
    if (variant == 0 && split_k > 8) return DFHIP_ERR_BAD_ARGUMENT;
    if (!workspace) return DFHIP_ERR_NULL_POINTER;
    if (!dfhip_aligned16(workspace)) return DFHIP_ERR_BAD_ALIGNMENT;
    if (workspace_bytes < dfhip_gemm_bf16_splitk_workspace_bytes(M, N, split_k)) return DFHIP_ERR_BAD_ARGUMENT;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (variant) {
    case 0: return launch_ring<false>(A, lda, W, R, ldw, C, ldc, M, N, K, split_k, workspace, s);
    case 5: return launch_ring224<false>(A, lda, W, R, ldw, C, ldc, M, N, K, s);
    case 7: return launch_ring224<false, 128>(A, lda, W, R, ldw, C, ldc, M, N, K, s);
    case 6: return launch_skinny<false>(A, lda, W, R, ldw, C, ldc, M, N, K, split_k, workspace, s);
    default: return launch<128, 128, 2, 2>(A, lda, W, ldw, C, ldc, M, N, K, s, R);
  }
}

namespace {
constexpr int MAX_DEVICES = 64;
std::mutex scratch_mutex;
void* scratch_ptr[MAX_DEVICES];   // device address of `scratch` on each GPU, looked up on first use

// The address of this GPU's copy of `scratch` (null: not known and not to be looked up now).  The lookup
// (hipGetSymbolAddress, once per device) may set up the code object's device variables, which is not a thing to
// do while a stream is capturing: with `may_look_up` false only an address found earlier is returned.  No
// allocation happens here.
void* scratch_on_current_device(bool may_look_up) {
  int device = -1;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= MAX_DEVICES) return nullptr;
  std::lock_guard<std::mutex> guard(scratch_mutex);
  if (!scratch_ptr[device] && may_look_up) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess) {
      (void)hipGetLastError();
      return nullptr;
    }
    scratch_ptr[device] = p;
  }
  return scratch_ptr[device];
}
}  // namespace

extern "C" int dfhip_gemm_bf16_nt_splitk_static(const void* A, int64_t lda, const void* W, int64_t ldw, void* C,
                                                int64_t ldc, int M, int N, int K, int split_k,
                                                dfhip_stream_t stream) {
  if (int rc = check_args(A, lda, W, ldw, C, ldc, M, N, K)) return rc;
  if (split_k < 1 || split_k > 16 || K / BK < split_k) return DFHIP_ERR_BAD_ARGUMENT;
  const size_t need = dfhip_gemm_bf16_splitk_workspace_bytes(M, N, split_k);
  if (need > (size_t)DFHIP_SPLITK_STATIC_BYTES) return DFHIP_ERR_TOO_LARGE;
  void* ws = nullptr;
  if (split_k > 1) {
    // the first call on a device finds the array's address and must not be part of a capture
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(static_cast<hipStream_t>(stream), &capturing) != hipSuccess) {
      (void)hipGetLastError();
      return DFHIP_ERR_LAUNCH;
    }
    ws = scratch_on_current_device(capturing == hipStreamCaptureStatusNone);
    if (!ws) return capturing == hipStreamCaptureStatusNone ? DFHIP_ERR_NO_DEVICE : DFHIP_ERR_BAD_ARGUMENT;
    // The array keeps what the last call left.  Completed launches leave the counters at zero; they are
    // cleared all the same (a fill kernel, not a memset node), so that a launch that never finished cannot
    // poison the next one.  The two split-K kernels size their counter areas differently; the larger one is
    // cleared (what lies behind the counters are partial blocks, written before they are read).
    const size_t tiles_ring = (size_t)((M + RBM - 1) / RBM) * ((N + RBN - 1) / RBN);
    size_t counters = counter_area(tiles_ring);
    if (M <= SK_MAX_M && skinny_counter_bytes(M, N) > counters) counters = skinny_counter_bytes(M, N);
    if (int rc = dfhip_fill_u32(ws, 0u, (int64_t)(counters / 4), stream)) return rc;
  }
  return dfhip_gemm_bf16_nt_splitk(A, lda, W, ldw, C, ldc, M, N, K, split_k, ws, need, stream);
}

// Causal grouped-query attention for prefill (bf16, head_dim 128), flash-attention style: scores and
// probabilities never leave the registers.
//
// One workgroup = 4 waves x 64 query rows that share one (sequence, kv head): the same 64 rows of 4 query heads
// of the group (HPW = 4: every wave has the same diagonal block, so no wave waits for another one's masked
// tiles, and no tile lies wholly above the diagonal), 128 rows of 2 heads, or 256 rows of one head, whichever
// the group size allows.  K and V are staged
// in LDS in blocks of 64 positions by LDS-DMA (3 stages in flight).  Both products are computed
// transposed so that no operand ever needs a transpose:
//   S^T[pos, qrow] = K Q^T   A = K rows from LDS, B = Q fragments held in registers for the whole kernel
//   O^T[dim, qrow] = V^T P^T A = V in the blocked layout (8 consecutive positions of one dim are 16
//                            contiguous bytes), B = P^T = the score accumulators themselves
// MFMA row m of a score tile is mapped to position pi(m) (the two middle groups of 4 rows of every 16
// are swapped) - K rows sit in LDS in that order - so that accumulator registers 0..7 of lane
// (qrow, half) are the probabilities of positions 8*half .. 8*half+7: exactly the lane's B fragment of
// the first 16-position k-step of P V; registers 8..15 are the second.  Every accumulator of a lane
// belongs to the lane's own query row, so the softmax statistics and the rescaling are lane-local.
//
// Two passes in one kernel.  The fast pass never rescales: every row keeps the maximum of its first tile
// as the reference of its exponentials (mathematically the reference is arbitrary).  That removes all
// arithmetic on the 128 output accumulators from the loop - they stay in the accumulation registers from
// first to last tile.  Exponentials and sums can only overflow if later scores exceed the row's first maximum
// by far; a workgroup in which a row's sum of exponentials ends beyond SAFE_SUM runs the safe pass behind the
// fast one (running maximum, rescaling whenever the maximum moves by more than 2^RESCALE_THRESHOLD) and
// stores its rows again.
#include <type_traits>

#include "dfhip_common.h"

namespace {

constexpr int AD = 128;          // head dim
constexpr int WAVE_ROWS = 64;    // query rows per wave
constexpr int KVB = 64;          // positions per staged block
constexpr int STAGES = 4;
constexpr int K_BYTES = KVB * AD * 2;            // 16 KiB
constexpr int STAGE_BYTES = 2 * K_BYTES;         // K block + V block
constexpr int ATT_LDS = STAGES * STAGE_BYTES;    // 128 KiB
constexpr float RESCALE_THRESHOLD = 8.0f;        // in units of log2: stale maxima up to 2^8 are tolerated
constexpr float SAFE_SUM = 0x1p64f;               // fast pass: a row sum beyond this (relative to the row's reference) is redone

// maximum of three without the quieting of signalling NaNs that fmaxf implies (one instruction)
DFHIP_DEVICE float max3(float a, float b, float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}

// The score products of the fast pass, written out with their register classes: the result tile in VECTOR
// registers, where the softmax reads it with ordinary instructions, and the Q fragment - which is only ever an MFMA
// operand - in ACCUMULATION registers.  Left to the compiler the score tiles sit in accumulation registers and
// every score costs a v_accvgpr_read_b32, which beside running MFMAs takes about three times as long as an
// ordinary vector instruction (take-it-out timing).  The compiler does not know that these are MFMAs, so it puts
// no wait states between one of them and a vector instruction that reads its result (an 8-pass MFMA needs 11).
// The invariant that stands in for them: a score tile is first read two or more MFMAs (64 cycles) after the last
// product into it.  It is kept in the source, not left to the scheduler - the statements are volatile (their order
// among themselves and against the other pinned statements is the written one), inside a step every MFMA and the
// softmax slices behind it sit between scheduling barriers, and where no MFMAs separate a tile's last product from
// its first reader (the prologue) scores_settled() spends the wait states and ties the tile behind them.  The
// accumulating form reads exactly the registers it writes, the one dependent sequence that the matrix pipe
// forwards by itself.
DFHIP_DEVICE f32x16 mfma_scores_first(bf16x8 k_rows, bf16x8 q_frag) {
  f32x16 d;
  asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(d) : "v"(k_rows), "a"(q_frag));
  return d;
}
DFHIP_DEVICE void mfma_scores_next(f32x16& d, bf16x8 k_rows, bf16x8 q_frag) {
  asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(d) : "v"(k_rows), "a"(q_frag));
}
// 12 wait states, and every later use of the two halves of a score tile tied behind them.
DFHIP_DEVICE void scores_settled(f32x16 (&s)[2]) {
  asm volatile("s_nop 7\n\ts_nop 3" : "+v"(s[0]), "+v"(s[1]));
  DFHIP_PIN;
}

DFHIP_DEVICE int pi(int m) {   // MFMA row -> position inside a 32-position tile
  const int g = (m >> 2) & 3;
  const int g2 = ((g & 1) << 1) | (g >> 1);      // 0,1,2,3 -> 0,2,1,3
  return (m & 16) | (g2 << 2) | (m & 3);
}

// workgroup -> (sequence, kv head, first query head, query block) for workgroups of HPW heads x QROWS rows.  All
// query heads of a (sequence, kv head) pair run on ONE XCD (its K and V stay in that XCD's L2); inside an XCD's
// range the heavy query blocks (late rows, many K/V blocks) come first.
template <int HPW>
DFHIP_DEVICE void map_workgroup(int B, int S, int q_heads, int kv_heads, int& b, int& kvh, int& hq, int& qb) {
  constexpr int QROWS = WAVE_ROWS * 4 / HPW;
  const int group = q_heads / kv_heads / HPW;    // workgroups per (sequence, kv head, query block)
  const int nqb = (S + QROWS - 1) / QROWS;
  const int sets = B * kv_heads;
  int hg;
  if (sets % 8 == 0) {
    const int total = sets * group * nqb;
    const int t = remap_xcd(blockIdx.x, total);
    const int range = total / 8, sets_x = sets / 8;
    const int local = t % range;
    const int per_level = sets_x * group;
    qb = nqb - 1 - local / per_level;
    const int within = local % per_level;
    const int set = (t / range) * sets_x + within / group;
    hg = within % group;
    b = set / kv_heads;
    kvh = set % kv_heads;
  } else {
    const int t = blockIdx.x;
    hg = t % group;
    const int set = (t / group) % sets;
    qb = nqb - 1 - t / (group * sets);
    b = set / kv_heads;
    kvh = set % kv_heads;
  }
  hq = (kvh * group + hg) * HPW;
}

// The fast pass is software-pipelined: with one wave per SIMD nothing else fills the matrix pipe while a
// wave does its softmax, so every step holds three independent pieces of work, interleaved by hand and
// pinned - the P V MFMAs of tile t, the score MFMAs of tile t+2, and the softmax (VALU) of tile t+1.  Score
// tiles and probability fragments alternate between two register sets (A: even tiles, B: odd tiles).  K/V
// blocks live in a ring of 4 stages: block j (V in use), j+1 (K in use), j+2 and j+3 landing.
template <int HPW>
__global__ void __launch_bounds__(256)
causal_attention_kernel(const uint16_t* __restrict__ q, int64_t ld_q, const uint16_t* __restrict__ k, int64_t ld_k,
                        const uint16_t* __restrict__ v_blk, uint16_t* __restrict__ out, int64_t ld_o, int B, int S,
                        int q_heads, int kv_heads, float scale_log2) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int col = lane & 31, half = lane >> 5;
  constexpr int WPH = 4 / HPW;                 // waves per head
  constexpr int QROWS = WAVE_ROWS * WPH;       // query rows per workgroup
  int b, kvh, hq, qb;
  map_workgroup<HPW>(B, S, q_heads, kv_heads, b, kvh, hq, qb);
  hq += wave / WPH;                            // this wave's query head ...
  const int wrow = wave % WPH;                 // ... and its 64 rows of the workgroup's query block
  const int q0 = qb * QROWS;
  const int last_block_wg = ((q0 + QROWS < S ? q0 + QROWS : S) + KVB - 1) / KVB - 1;
  int last_block_wave = q0 / KVB + wrow;                        // the wave's diagonal block
  if (last_block_wave > last_block_wg) last_block_wave = last_block_wg;   // a wave of rows past S (never stored)

  // ---- DMA sources: uniform bases that advance by one block, per-lane offsets fixed for the whole kernel
  // (per block: 4 K instructions + 4 V instructions per wave, 1 KiB each)
  const uint8_t* kseq = reinterpret_cast<const uint8_t*>(k + (int64_t)b * S * ld_k + (int64_t)kvh * AD);
  const uint8_t* vseq = reinterpret_cast<const uint8_t*>(v_blk) + ((int64_t)(b * kv_heads + kvh) * S) * (AD * 2) +
                        wave * 4096;
  const int64_t k_block_bytes = (int64_t)KVB * ld_k * 2;
  uint32_t k_off[4], v_off[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const int row = (wave * 4 + t) * 4 + (lane >> 4);          // LDS row 0..63 (MFMA row order)
    const int slot = lane & 15;
    const int pos = (row & 32) | pi(row & 31);                 // position inside the block
    const int chunk = (slot & 8) | ((slot & 7) ^ (row & 7));   // logical 16-byte chunk held by this slot
    k_off[t] = (uint32_t)(pos * ld_k * 2 + chunk * 16);
    v_off[t] = (uint32_t)(t * 1024 + lane * 16);
  }
  // piece t of block j: 4 K instructions (t = 0..3), then 4 V instructions; nothing past the last block
  auto issue_piece = [&](int j, int t) {
    if (j > last_block_wg) return;
    const int stage = j % STAGES;
    if (t < 4) dma16_base(stage * STAGE_BYTES + (wave * 4 + t) * 1024, kseq + j * k_block_bytes, k_off[t]);
    else dma16_base(stage * STAGE_BYTES + K_BYTES + (wave * 4 + t - 4) * 1024, vseq + (int64_t)j * (KVB * AD * 2),
                    v_off[t - 4]);
  };
  auto issue_block = [&](int j) {
#pragma unroll
    for (int t = 0; t < 8; ++t) issue_piece(j, t);
  };
  // The same for the steps of the main loop, without a branch: a piece past the last block re-reads the last
  // block into the stage that its own block would have taken, which nobody reads any more.  (A branch here cuts
  // the step into basic blocks, and the compiler then sinks the step's softmax across them to its first use in
  // the next step: 32 exponentials in one run with no MFMA over them.)
  auto issue_piece_or_dummy = [&](int j, int t) {
    const int src = j < last_block_wg ? j : last_block_wg;
    const int stage = j % STAGES;
    if (t < 4) dma16_base(stage * STAGE_BYTES + (wave * 4 + t) * 1024, kseq + src * k_block_bytes, k_off[t]);
    else dma16_base(stage * STAGE_BYTES + K_BYTES + (wave * 4 + t - 4) * 1024, vseq + (int64_t)src * (KVB * AD * 2),
                    v_off[t - 4]);
  };

  issue_block(0);
  issue_block(1);
  issue_block(2);
  // ---- Q fragments (behind the first K/V blocks, so that everything is in flight together): B operand of
  // S^T, lane supplies Q[qrow][16 ks + 8 half .. +8]
  bf16x8 qf[2][8];
#pragma unroll
  for (int nb = 0; nb < 2; ++nb) {
    int qrow = q0 + wrow * WAVE_ROWS + nb * 32 + col;
    qrow = qrow < S ? qrow : S - 1;
    const uint16_t* qp = q + ((int64_t)b * S + qrow) * ld_q + (int64_t)hq * AD + 8 * half;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) qf[nb][ks] = *reinterpret_cast<const bf16x8*>(qp + 16 * ks);
  }


  f32x16 o[4][2];
#pragma unroll
  for (int db = 0; db < 4; ++db)
#pragma unroll
    for (int nb = 0; nb < 2; ++nb)
#pragma unroll
      for (int r = 0; r < 16; ++r) o[db][nb][r] = 0.0f;
  const int k_read = col * 256;
  const int my_qrow0 = q0 + wrow * WAVE_ROWS + col;

  // LDS addresses of the A fragments: V pair p = (t, db) of tile [block, sb], K k-step ks of tile [block, sb]
  auto v_frag = [&](int block, int sb, int p) {
    const int t = p >> 2, db = p & 3;
    return *reinterpret_cast<const bf16x8*>(smem + (block % STAGES) * STAGE_BYTES + K_BYTES +
                                            ((sb * 4 + t * 2 + half) * AD + db * 32 + col) * 16);
  };
  auto k_frag = [&](int block, int sb, int ks) {
    const int chunk = 2 * ks + half;
    const int slot = (chunk & 8) | ((chunk & 7) ^ (col & 7));
    return *reinterpret_cast<const bf16x8*>(smem + (block % STAGES) * STAGE_BYTES + sb * 8192 + k_read + slot * 16);
  };

  // The reference of a row's exponentials (times scale_log2, negated): the maximum of its first tile.
  float neg_ref[2] = {0.0f, 0.0f};
  auto first_tile_reference = [&](bool diag, const f32x16 (&s)[2]) {
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) {
      const int qrow = my_qrow0 + 32 * nb;
      float tmax = -INFINITY;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const bool masked = diag && 8 * half + 16 * (r >> 3) + (r & 7) > qrow;   // tile 0 starts at position 0
        tmax = fmaxf(tmax, masked ? -INFINITY : s[nb][r]);
      }
      neg_ref[nb] = -fmaxf(tmax, __shfl_xor(tmax, 32, 64)) * scale_log2;
    }
  };
  // The softmax of one score tile in the fast pass is 32 slices (16 per half of the query rows), one behind
  // nearly every MFMA of a step: a slice turns one score into a probability (an even register's waits for its
  // odd neighbour to be packed with it).  No maximum is taken and no sum: the row sums come out of the matrix
  // pipe (an all-ones A operand against the probabilities), and whether a row's scores outgrew its reference
  // shows in that sum at the end.
  float held = 0.0f;                          // the probability of an even register until its odd neighbour follows
  auto softmax_slice = [&](auto diag, int i, int block, int sb, const f32x16 (&s)[2], bf16x8 (&pf)[2][2]) {
    const int nb = i >> 4, r = i & 15;
    float x = s[nb][r];
    if (decltype(diag)::value) {
      const int pos = block * KVB + sb * 32 + 8 * half + 16 * (r >> 3) + (r & 7);
      const int qrow = my_qrow0 + 32 * nb;
      if (pos > qrow) x = -INFINITY;
    }
    const float e = __builtin_amdgcn_exp2f(fmaf(x, scale_log2, neg_ref[nb]));
    if (r & 1) {
      pf[nb][r >> 3][(r & 7) - 1] = static_cast<bf16_t>(held);
      pf[nb][r >> 3][r & 7] = static_cast<bf16_t>(e);
    } else {
      held = e;
    }
  };

  // Hazard invariant of a step (see mfma_scores_first): s_out's last products are the step's last two MFMAs (nb = 0,
  // then nb = 1); the next step reads s_in[0] behind its second MFMA at the earliest and s_in[1] sixteen slices
  // later, i.e. two or more MFMAs after the last product into the registers it reads, and the scheduling barrier
  // behind every MFMA keeps it so.
  // One step: P V of tile [vb, vsb] (probabilities pf_in) with the two row-sum MFMAs of each k-step behind
  // it, then - DO_S - the scores of tile [kb, ksb] into s_out, with - DO_SM - the softmax of tile [mb, msb]
  // (scores s_in -> pf_out) sliced between the MFMAs.  A fragments are read AHEAD MFMA pairs ahead; the
  // first of a step are read by the step before (vpre), which is why the P V pairs come first: the V block of
  // the next step has always landed already.
  constexpr int AHEAD = 4;                     // fragment-consuming pairs between a fragment's read and its use
  bf16x8 vpre[AHEAD];
  bf16x8 ones;
#pragma unroll
  for (int e = 0; e < 8; ++e) ones[e] = static_cast<bf16_t>(1.0f);
  f32x16 l_acc[2];                             // every element: the row sum of the lane's query row
#pragma unroll
  for (int nb = 0; nb < 2; ++nb)
#pragma unroll
    for (int r = 0; r < 16; ++r) l_acc[nb][r] = 0.0f;
  auto step = [&](auto do_s, auto do_sm, auto diag, int vb, int vsb, const bf16x8 (&pf_in)[2][2], int kb, int ksb,
                  f32x16 (&s_out)[2], int mb, int msb, const f32x16 (&s_in)[2], bf16x8 (&pf_out)[2][2], int nvb,
                  int nvsb, int dma_block) {
    constexpr bool DO_S = decltype(do_s)::value, DO_SM = decltype(do_sm)::value;
    constexpr int FRAGS = DO_S ? 16 : 8;       // pairs that consume an A fragment: 8 of P V, 8 of the scores
    constexpr int PAIRS = FRAGS + 2;           // + the row sums of the two k-steps
    bf16x8 fr[FRAGS + AHEAD];
#pragma unroll
    for (int a = 0; a < AHEAD; ++a) fr[a] = vpre[a];
#pragma unroll
    for (int pq = 0; pq < PAIRS; ++pq) {
      // pair order: pv0..pv3, sum(t=0), pv4..pv7, sum(t=1), score k-steps 0..7
      const bool is_sum = pq == 4 || pq == 9;
      const int f = pq < 4 ? pq : pq < 9 ? pq - 1 : pq - 2;      // fragment index of a consuming pair
      // the 8 LDS-DMA instructions of the block that enters the ring in this iteration, spread over the step
      // (4 waves issuing them in one burst keep the address unit, and with it the waves, busy for ~500 cycles)
      if (dma_block >= 0) {
        if (DO_S ? (pq & 1) && pq < 16 : pq < 8) issue_piece_or_dummy(dma_block, DO_S ? pq >> 1 : pq);
      }
      if (!is_sum) {
        const int n = f + AHEAD;               // the fragment to fetch now
        if (n < 8) fr[n] = v_frag(vb, vsb, n);
        else if (n < FRAGS) fr[n] = k_frag(kb, ksb, n - 8);
        else fr[n] = v_frag(nvb, nvsb, n - FRAGS);
      }
#pragma unroll
      for (int nb = 0; nb < 2; ++nb) {
        if (is_sum) {
          l_acc[nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ones, pf_in[nb][pq == 4 ? 0 : 1], l_acc[nb], 0, 0, 0);
        } else if (f < 8) {
          const int t = f >> 2, db = f & 3;
          o[db][nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fr[f], pf_in[nb][t], o[db][nb], 0, 0, 0);
        } else if (f == 8) {
          s_out[nb] = mfma_scores_first(fr[f], qf[nb][0]);
        } else {
          mfma_scores_next(s_out[nb], fr[f], qf[nb][f - 8]);
        }
        if (DO_SM) {
          const int m = 2 * pq + nb;           // slices [32 m / (2 PAIRS), 32 (m+1) / (2 PAIRS))
#pragma unroll
          for (int i = 32 * m / (2 * PAIRS); i < 32 * (m + 1) / (2 * PAIRS); ++i)
            softmax_slice(diag, i, mb, msb, s_in, pf_out);
        }
        DFHIP_PIN;
      }
    }
#pragma unroll
    for (int a = 0; a < AHEAD; ++a) vpre[a] = fr[FRAGS + a];
  };
  constexpr int NO_DMA = -1;
  using yes = std::true_type;
  using no = std::false_type;

  f32x16 sA[2], sB[2];
  bf16x8 pfA[2][2], pfB[2][2];
  wait_vmcnt<0>();                           // Q and the first blocks have landed
  workgroup_barrier();
  // from here on the Q fragments live in accumulation registers (see mfma_scores_first)
#pragma unroll
  for (int nb = 0; nb < 2; ++nb)
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) asm volatile("" : "+a"(qf[nb][ks]));
  // prologue (not overlapped): scores of tiles 0 and 1, softmax of tile 0
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    f32x16 (&sd)[2] = t == 0 ? sA : sB;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      const bf16x8 kf = k_frag(0, t, ks);
#pragma unroll
      for (int nb = 0; nb < 2; ++nb) {
        if (ks == 0) sd[nb] = mfma_scores_first(kf, qf[nb][0]);
        else mfma_scores_next(sd[nb], kf, qf[nb][ks]);
      }
    }
  }
  // nothing but the products into sB separates sA's last product from its first reader, and the scheduler is
  // free to put those elsewhere: the wait states are spent here, for both tiles
  scores_settled(sA);
  scores_settled(sB);
  first_tile_reference(last_block_wave == 0, sA);
  if (last_block_wave == 0) {
#pragma unroll
    for (int i = 0; i < 32; ++i) softmax_slice(yes{}, i, 0, 0, sA, pfA);
  } else {
#pragma unroll
    for (int i = 0; i < 32; ++i) softmax_slice(no{}, i, 0, 0, sA, pfA);
  }
#pragma unroll
  for (int a = 0; a < AHEAD; ++a) vpre[a] = v_frag(0, 0, a);

  // Every wave passes last_block_wg + 1 barriers: full iterations up to its diagonal block, the drain of
  // the diagonal block, then the staging duty only.  The three phases follow each other (no branch
  // around code that touches the output accumulators, so they never leave the accumulation registers).
  // Before iteration j block j+1 must have landed; only block j+2 (when there is one) may be in flight.
  auto turn_ring = [&](int j) {
    if (j + 2 <= last_block_wg) wait_vmcnt<8>();
    else wait_vmcnt<0>();
    workgroup_barrier();                     // block j+1 is there for every wave; everybody is done with block j-1
  };                                         // ... so block j+3 may enter the ring (first step of the iteration)
  // While a wave runs steps, every iteration issues exactly 8 pieces (block j+3 or its stand-in), so "at most 8
  // in flight" always means that block j+1 has landed.
  auto turn_ring_in_steps = [&]() {
    wait_vmcnt<8>();
    workgroup_barrier();
  };
  int j = 0;
  for (; j + 1 < last_block_wave; ++j) {
    turn_ring_in_steps();
    step(yes{}, yes{}, no{}, j, 0, pfA, j + 1, 0, sA, j, 1, sB, pfB, j, 1, j + 3);
    step(yes{}, yes{}, no{}, j, 1, pfB, j + 1, 1, sB, j + 1, 0, sA, pfA, j + 1, 0, NO_DMA);
  }
  if (j < last_block_wave) {                 // the block before the diagonal one: its second softmax is masked
    turn_ring_in_steps();
    step(yes{}, yes{}, no{}, j, 0, pfA, j + 1, 0, sA, j, 1, sB, pfB, j, 1, j + 3);
    step(yes{}, yes{}, yes{}, j, 1, pfB, j + 1, 1, sB, j + 1, 0, sA, pfA, j + 1, 0, NO_DMA);
    ++j;
  }
  turn_ring_in_steps();
  step(no{}, yes{}, yes{}, j, 0, pfA, 0, 0, sA, j, 1, sB, pfB, j, 1, j + 3);
  step(no{}, no{}, no{}, j, 1, pfB, 0, 0, sA, 0, 0, sB, pfA, j, 1, NO_DMA);
  wait_vmcnt<0>();                           // the last pieces (stand-ins, possibly) are out of the way of what follows
  // The output goes from the registers straight to memory (a lane holds runs of 4 dims of its query rows), so
  // a wave that is done stores while the others still work; its remaining duty is the ring.
  auto store_rows = [&](const float (&row_sum)[2]) {
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) {
      const float inv = 1.0f / row_sum[nb];
      const int qrow = q0 + wrow * WAVE_ROWS + nb * 32 + col;
      uint16_t* orow = out + ((int64_t)b * S + qrow) * ld_o + (int64_t)hq * AD + 4 * half;
      if (qrow < S) {
#pragma unroll
        for (int db = 0; db < 4; ++db)
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            u32x2 w;
            w[0] = pack2_bf16(o[db][nb][4 * g + 0] * inv, o[db][nb][4 * g + 1] * inv);
            w[1] = pack2_bf16(o[db][nb][4 * g + 2] * inv, o[db][nb][4 * g + 3] * inv);
            *reinterpret_cast<u32x2*>(orow + db * 32 + 8 * g) = w;
          }
      }
    }
  };
  const float fast_sum[2] = {l_acc[0][0], l_acc[1][0]};
  store_rows(fast_sum);
  for (++j; j <= last_block_wg; ++j) {
    turn_ring(j);
    issue_block(j + 3);
  }

  // ---- Did the scores of any row of the workgroup outgrow the row's reference?  Then exponentials or sums
  // may have overflowed.  (The ring is idle: the last turns waited for everything in flight.)
  __syncthreads();
  const bool wave_risk = __any(fast_sum[0] > SAFE_SUM || fast_sum[1] > SAFE_SUM);
  if (lane == 0) reinterpret_cast<int*>(smem)[wave] = wave_risk;
  __syncthreads();
  const int4 risks = *reinterpret_cast<const int4*>(smem);
  if ((risks.x | risks.y | risks.z | risks.w) == 0) return;
  __syncthreads();                           // everybody has read the four words before the ring restarts

  // ---- The safe pass (rare): the whole workgroup again, tile by tile with a running maximum; the output
  // accumulators are rescaled whenever the maximum moves by more than 2^RESCALE_THRESHOLD.  Same lanes, same
  // addresses: the second store of a lane lands behind its first.
#pragma unroll
  for (int db = 0; db < 4; ++db)
#pragma unroll
    for (int nb = 0; nb < 2; ++nb)
#pragma unroll
      for (int r = 0; r < 16; ++r) o[db][nb][r] = 0.0f;
  float m_run[2] = {-INFINITY, -INFINITY};   // running (possibly stale) maximum of the raw scores
  float l_run[2] = {0.0f, 0.0f};             // this lane's share of the row sum
  issue_block(0);
  for (int jb = 0; jb <= last_block_wg; ++jb) {
    issue_block(jb + 1);                     // into a stage that neither block jb nor block jb-1 uses
    if (jb + 1 <= last_block_wg) wait_vmcnt<8>();
    else wait_vmcnt<0>();
    workgroup_barrier();                     // block jb is there for every wave; everybody is done with jb-1
    if (jb > last_block_wave) continue;
    const bool diagonal = jb == last_block_wave;
#pragma clang loop unroll(disable)
    for (int sb = 0; sb < 2; ++sb) {
      f32x16 s[2];
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) {
        const bf16x8 kf = k_frag(jb, sb, ks);
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) {
          const f32x16 zero = {};
          s[nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[nb][ks], ks == 0 ? zero : s[nb], 0, 0, 0);
        }
      }
      // register r of this lane: position p_base + 16*(r/8) + (r%8), query row my_qrow0 + 32 nb
      const int p_base = jb * KVB + sb * 32 + 8 * half;
      bf16x8 pf[2][2];
#pragma unroll
      for (int nb = 0; nb < 2; ++nb) {
        if (diagonal) {
          const int qrow = my_qrow0 + 32 * nb;
#pragma unroll
          for (int r = 0; r < 16; ++r)
            if (p_base + 16 * (r >> 3) + (r & 7) > qrow) s[nb][r] = -INFINITY;
        }
        float tmax = s[nb][0];
#pragma unroll
        for (int r = 1; r < 16; ++r) tmax = fmaxf(tmax, s[nb][r]);
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
        if (__any((tmax - m_run[nb]) * scale_log2 > RESCALE_THRESHOLD)) {
          const float m_new = fmaxf(m_run[nb], tmax);
          const float alpha = __builtin_amdgcn_exp2f((m_run[nb] - m_new) * scale_log2);   // 0 on the first block
          m_run[nb] = m_new;
          l_run[nb] *= alpha;
#pragma unroll
          for (int db = 0; db < 4; ++db)
#pragma unroll
            for (int r = 0; r < 16; ++r) o[db][nb][r] *= alpha;
        }
        const float mc = m_run[nb] * scale_log2;
        float lsum = 0.0f;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float p = __builtin_amdgcn_exp2f(fmaf(s[nb][r], scale_log2, -mc));
          lsum += p;
          pf[nb][r >> 3][r & 7] = static_cast<bf16_t>(p);
        }
        l_run[nb] += lsum;
      }
#pragma unroll
      for (int p = 0; p < 8; ++p) {
        const bf16x8 vf = v_frag(jb, sb, p);
        o[p & 3][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf[0][p >> 2], o[p & 3][0], 0, 0, 0);
        o[p & 3][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf[1][p >> 2], o[p & 3][1], 0, 0, 0);
      }
    }
  }
  const float safe_sum[2] = {l_run[0] + __shfl_xor(l_run[0], 32, 64), l_run[1] + __shfl_xor(l_run[1], 32, 64)};
  store_rows(safe_sum);
}

// v[T, ld_v] (head h at column h*128) -> v_blk[B][kv_heads][S/8][128][8]
__global__ void __launch_bounds__(128)
pack_v_kernel(const uint16_t* __restrict__ v, int64_t ld_v, uint16_t* __restrict__ v_blk, int S, int kv_heads) {
  const int pbs = S / 8;
  const int pb = blockIdx.x % pbs;
  const int h = (blockIdx.x / pbs) % kv_heads;
  const int b = blockIdx.x / (pbs * kv_heads);
  const int d = threadIdx.x;
  const uint16_t* src = v + ((int64_t)b * S + pb * 8) * ld_v + (int64_t)h * AD + d;
  uint32_t w[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) w[i] = (uint32_t)src[(2 * i) * ld_v] | ((uint32_t)src[(2 * i + 1) * ld_v] << 16);
  u32x4 o = {w[0], w[1], w[2], w[3]};
  *reinterpret_cast<u32x4*>(v_blk + ((((int64_t)b * kv_heads + h) * pbs + pb) * AD + d) * 8) = o;
}

}  // namespace

extern "C" int dfhip_pack_v_bf16(const void* v, int64_t ld_v, void* v_blk, int B, int S, int kv_heads, int head_dim,
                                 dfhip_stream_t stream) {
  if (!v || !v_blk) return DFHIP_ERR_NULL_POINTER;
  if (B < 1 || S < 8 || S % 8 != 0 || kv_heads < 1 || head_dim != AD ||
      (int64_t)B * kv_heads * (S / 8) >= (int64_t)1 << 31)
    return DFHIP_ERR_BAD_SHAPE;
  if (ld_v < (int64_t)kv_heads * AD) return DFHIP_ERR_BAD_STRIDE;
  if (!dfhip_aligned16(v_blk)) return DFHIP_ERR_BAD_ALIGNMENT;
  hipLaunchKernelGGL(pack_v_kernel, dim3(B * kv_heads * (S / 8)), dim3(128), 0, static_cast<hipStream_t>(stream),
                     static_cast<const uint16_t*>(v), ld_v, static_cast<uint16_t*>(v_blk), S, kv_heads);
  return dfhip_check_launch();
}

extern "C" int dfhip_causal_attention_bf16(const void* q, int64_t ld_q, const void* k, int64_t ld_k,
                                           const void* v_blk, void* out, int64_t ld_o, int B, int S, int q_heads,
                                           int kv_heads, int head_dim, float scale, dfhip_stream_t stream) {
  if (!q || !k || !v_blk || !out) return DFHIP_ERR_NULL_POINTER;
  if (B < 1 || S < KVB || S % KVB != 0 || q_heads < 1 || kv_heads < 1 || q_heads % kv_heads != 0 || head_dim != AD)
    return DFHIP_ERR_BAD_SHAPE;
  const int group = q_heads / kv_heads;
  const int hpw = group % 4 == 0 ? 4 : group % 2 == 0 ? 2 : 1;      // query heads per workgroup
  const int wg_rows = WAVE_ROWS * 4 / hpw;
  const int64_t groups = (int64_t)B * (q_heads / hpw) * ((S + wg_rows - 1) / wg_rows);
  if (groups >= (int64_t)1 << 31) return DFHIP_ERR_BAD_SHAPE;
  if (ld_q < (int64_t)q_heads * AD || ld_k < (int64_t)kv_heads * AD || ld_o < (int64_t)q_heads * AD ||
      ld_k >= (int64_t)1 << 24)   // a K block's byte offsets are kept in 32 bits
    return DFHIP_ERR_BAD_STRIDE;
  if (ld_q % 8 || ld_k % 8 || ld_o % 8 || !dfhip_aligned16(q) || !dfhip_aligned16(k) || !dfhip_aligned16(v_blk) ||
      !dfhip_aligned16(out))
    return DFHIP_ERR_BAD_ALIGNMENT;
  auto launch = [&](auto heads_per_workgroup) {
    constexpr int HPW = decltype(heads_per_workgroup)::value;
    static std::atomic<uint64_t> lds_opted_in{0};   // per instantiation, one bit per device
    if (int rc = dfhip_opt_in_lds(reinterpret_cast<const void*>(causal_attention_kernel<HPW>), ATT_LDS, lds_opted_in))
      return rc;
    hipLaunchKernelGGL(causal_attention_kernel<HPW>, dim3((unsigned)groups), dim3(256), ATT_LDS,
                       static_cast<hipStream_t>(stream), static_cast<const uint16_t*>(q), ld_q,
                       static_cast<const uint16_t*>(k), ld_k, static_cast<const uint16_t*>(v_blk),
                       static_cast<uint16_t*>(out), ld_o, B, S, q_heads, kv_heads, scale * 1.4426950408889634f);
    return dfhip_check_launch();
  };
  if (hpw == 4) return launch(std::integral_constant<int, 4>{});
  if (hpw == 2) return launch(std::integral_constant<int, 2>{});
  return launch(std::integral_constant<int, 1>{});
}

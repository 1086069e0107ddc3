// Decode step (one new token per sequence) against a static KV cache: RoPE + cache append, and
// grouped-query attention of the new token over the cached positions.  Both are HBM-bound: the
// attention kernel reads every cached K and V element of a sequence exactly once.
//
// Cache layout (bf16, head_dim 128, `capacity` positions per sequence slot, capacity % 32 == 0):
//   K cache [slots][kv_heads][capacity][128]        - a position's 128 dims are contiguous
//   V cache [slots][kv_heads][capacity/8][128][8]   - 8 consecutive positions of one dim are contiguous
// Both layouts are what the 16x16x32 MFMA operands want as 16-byte per-lane loads straight from
// global memory (no LDS staging, no transposes):
//   scores^T = K Q^T : A = K rows (lane: one position, 8 consecutive dims)
//   out      = P V   : B = V     (lane: one dim, 8 consecutive positions)
#include "dfhip_common.h"

namespace {

constexpr int HD = 128;           // head dim
constexpr int DEC_THREADS = 256;  // 4 waves
constexpr int CHUNK = 32;         // positions per softmax step of a wave
constexpr int MAX_GROUP = 16;     // query heads per kv head (rows of the MFMA tile)

DFHIP_DEVICE f32x4 mfma16(bf16x8 a, bf16x8 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

// The rotation of one pair (x[i], x[i + 64]) of a head by the angle of its position: the one formula of both kernels
// below, so that they round alike.
// (The fused multiply-adds are spelt out: left to the compiler the two kernels could contract the expressions
// differently.)
DFHIP_DEVICE void rotate_pair(float lo, float hi, float c, float s, bf16_t& out_lo, bf16_t& out_hi) {
  out_lo = static_cast<bf16_t>(__builtin_fmaf(lo, c, -(hi * s)));
  out_hi = static_cast<bf16_t>(__builtin_fmaf(hi, c, lo * s));
}
DFHIP_DEVICE uint16_t bits_of(bf16_t v) { return __builtin_bit_cast(uint16_t, v); }

struct KVFrags {
  bf16x8 k[2][4];   // [set][k-step]
  bf16x8 v[8];      // [dim block]
};

// One workgroup per (token, kv head).  Wave w takes the chunks w, w+4, ... of 32 positions.
// MFMA row i of a score tile is mapped to position 8*(i/4) + i%4 (+4 for the second tile of the
// chunk), so that after the two tiles lane (head = lane%16, g = lane/16) holds the scores of its
// head for positions 8g .. 8g+7 - which is exactly the A-operand fragment of P for the P V product.
//
// APPEND: the workgroup first does what rope_kv_append_kernel does for its share of the token - `q` is the
// token's row of the q / k / v product, the group's query heads are rotated in registers, the kv head's new key
// is rotated and, with the new value, written to the caches at position lengths[t] - 1 - and then attends.  The
// wave whose chunks include that position does the append and keeps the new key and value in LDS for its own
// fragments of that position, which it patches when it gets there (no read of what was just written and no
// barrier: the wave that wrote the LDS words is the one that reads them; the other three waves only rotate their
// copies of the query heads).
template <bool APPEND>
__global__ void __launch_bounds__(DEC_THREADS)
decode_attention_kernel(const uint16_t* __restrict__ q, int64_t ld_q, uint16_t* __restrict__ kc,
                        uint16_t* __restrict__ vc, const int32_t* __restrict__ slots,
                        const int32_t* __restrict__ lengths, uint16_t* __restrict__ out, int64_t ld_out,
                        int kv_heads, int group, int num_slots, int capacity, float scale_log2,
                        const float* __restrict__ cos_t, const float* __restrict__ sin_t, int table_rows) {
  // partial results of the four waves, sized by the launch for the real group (a workgroup that asks for
  // little LDS leaves room for a GEMM workgroup of the other nano-batch on the same CU)
  extern __shared__ __attribute__((aligned(16))) float combine_lds[];
  float* const o_lds = combine_lds;                       // [4][group][HD]
  float* const m_lds = combine_lds + 4 * group * HD;      // [4][group]
  float* const l_lds = m_lds + 4 * group;                 // [4][group]
  const int t = blockIdx.x / kv_heads, kvh = blockIdx.x - t * kv_heads;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int hq = lane & 15, g = lane >> 4;
  const int slot = slots[t];
  int len = lengths[t];
  uint16_t* out_row = out + (int64_t)t * ld_out + (int64_t)kvh * group * HD;
  if (slot < 0 || slot >= num_slots || len < 1) {   // nothing to attend to: defined output, no access
    for (int idx = tid; idx < group * HD; idx += DEC_THREADS) out_row[idx] = 0;
    return;
  }
  const int pos = len - 1;                     // APPEND: the new token's position (before the clamp below)
  const bool append = APPEND && pos < capacity;
  len = len < capacity ? len : capacity;
  const int64_t head_base = ((int64_t)slot * kv_heads + kvh) * capacity * HD;
  uint16_t* kbase = kc + head_base;
  uint16_t* vbase = vc + head_base;
  const int trow = pos < table_rows ? pos : table_rows - 1;
  const uint16_t* const token_row = q + (int64_t)t * ld_q;                  // APPEND: q | k | v of the token
  uint16_t* const new_k = reinterpret_cast<uint16_t*>(l_lds + 4 * group);   // [HD], APPEND only
  uint16_t* const new_v = new_k + HD;                                        // [HD]

  bf16x8 qf[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) {
    if (hq < group) {
      qf[ks] = *reinterpret_cast<const bf16x8*>(q + (int64_t)t * ld_q + (int64_t)(kvh * group + hq) * HD + 32 * ks + 8 * g);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) qf[ks][e] = static_cast<bf16_t>(0.0f);
    }
  }
  const int krow = 8 * (hq >> 2) + (hq & 3);
  const uint16_t* k_lane = kbase + (int64_t)krow * HD + 8 * g;
  const uint16_t* v_lane = vbase + ((int64_t)g * HD + hq) * 8;

  // every cached element is read once per step and by nobody else: non-temporal loads, which do not displace
  // what the caches hold for the kernels that run beside this one (128 sequences x 2048 positions: 187 -> 158 us)
  auto load = [&](KVFrags& f, int chunk) {
    const uint16_t* kp = k_lane + (int64_t)chunk * (CHUNK * HD);
    const uint16_t* vp = v_lane + (int64_t)chunk * (CHUNK * HD);
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int ks = 0; ks < 4; ++ks)
        f.k[s][ks] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(kp + s * 4 * HD + 32 * ks));
#pragma unroll
    for (int nb = 0; nb < 8; ++nb) f.v[nb] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(vp + nb * 16 * 8));
  };

  float m = -INFINITY, l = 0.0f;
  f32x4 o[8];
#pragma unroll
  for (int nb = 0; nb < 8; ++nb) o[nb] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

  auto step = [&](KVFrags& f, int c) {
    if (APPEND && append && c == pos / CHUNK) {
      // the chunk of the new token: its key row and value column come from LDS, whatever the loads returned
      const int krow_pos = c * CHUNK + 8 * (hq >> 2) + (hq & 3);
#pragma unroll
      for (int s = 0; s < 2; ++s)
        if (krow_pos + 4 * s == pos) {
#pragma unroll
          for (int ks = 0; ks < 4; ++ks) f.k[s][ks] = *reinterpret_cast<const bf16x8*>(new_k + 32 * ks + 8 * g);
        }
      if (pos / 8 == c * (CHUNK / 8) + g) {
#pragma unroll
        for (int nb = 0; nb < 8; ++nb) {
          const uint16_t v = new_v[nb * 16 + hq];
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (e == (pos & 7)) f.v[nb][e] = __builtin_bit_cast(bf16_t, v);
        }
      }
    }
    if ((c + 1) * CHUNK > len) {
      // the last chunk of the sequence: positions from len on may hold anything (a cache that was never
      // written there, NaN bit patterns included) and their probability 0 would not silence a NaN in the
      // product, so their V elements are zeroed.  Their K rows need nothing: their scores are replaced below.
#pragma unroll
      for (int nb = 0; nb < 8; ++nb)
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (c * CHUNK + 8 * g + e >= len) f.v[nb][e] = static_cast<bf16_t>(0.0f);
    }
    f32x4 s1 = {0.0f, 0.0f, 0.0f, 0.0f}, s2 = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      s1 = mfma16(f.k[0][ks], qf[ks], s1);
      s2 = mfma16(f.k[1][ks], qf[ks], s2);
    }
    // this lane: head hq, positions c*32 + 8g + 0..7
    const int p_first = c * CHUNK + 8 * g;
    float sc[8];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      sc[r] = (p_first + r < len) ? s1[r] * scale_log2 : -INFINITY;
      sc[4 + r] = (p_first + 4 + r < len) ? s2[r] * scale_log2 : -INFINITY;
    }
    float cmax = sc[0];
#pragma unroll
    for (int r = 1; r < 8; ++r) cmax = fmaxf(cmax, sc[r]);
    cmax = fmaxf(cmax, __shfl_xor(cmax, 16, 64));
    cmax = fmaxf(cmax, __shfl_xor(cmax, 32, 64));
    const float m_new = fmaxf(m, cmax);       // finite: every chunk has at least one valid position
    const float alpha = exp2f(m - m_new);
    float psum = 0.0f;
    bf16x8 pf;
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      const float p = exp2f(sc[r] - m_new);
      psum += p;
      pf[r] = static_cast<bf16_t>(p);
    }
    psum += __shfl_xor(psum, 16, 64);
    psum += __shfl_xor(psum, 32, 64);
    l = l * alpha + psum;
    m = m_new;
    // the accumulators of this lane belong to heads 4g + r: their factors live in lanes 4g + r
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float a = __shfl(alpha, 4 * g + r, 64);
#pragma unroll
      for (int nb = 0; nb < 8; ++nb) o[nb][r] *= a;
    }
#pragma unroll
    for (int nb = 0; nb < 8; ++nb) o[nb] = mfma16(pf, f.v[nb], o[nb]);
  };

  // two fragment sets in turn: the loads of the next chunk are in flight while one is multiplied
  const int chunks = (len + CHUNK - 1) / CHUNK;
  KVFrags fa, fb;
  if (wave < chunks) load(fa, wave);
  // (the first chunk's loads are on their way while the query heads are rotated)
  if (APPEND) {
    // the lane's fragments ks and ks + 2 hold the two halves of the pairs i = 32 ks + 8 g + e, ks = 0, 1
#pragma unroll
    for (int ks = 0; ks < 2; ++ks)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int i = 32 * ks + 8 * g + e;
        const float c = cos_t[trow * (HD / 2) + i], s = sin_t[trow * (HD / 2) + i];
        bf16_t lo, hi;
        rotate_pair(static_cast<float>(qf[ks][e]), static_cast<float>(qf[ks + 2][e]), c, s, lo, hi);
        qf[ks][e] = lo;
        qf[ks + 2][e] = hi;
      }
    // The wave whose chunks include the new position appends: lane i rotates the pair (i, i + 64) of the new key
    // and copies two elements of the new value - to the caches for the later steps, to LDS for this wave's own
    // fragments of that position (the same wave writes and reads them: no barrier).
    if (append && wave == (pos / CHUNK) % 4) {
      const int q_heads = kv_heads * group;
      const uint16_t* k_in = token_row + (int64_t)(q_heads + kvh) * HD;
      const uint16_t* v_in = token_row + (int64_t)(q_heads + kv_heads + kvh) * HD;
      bf16_t lo, hi;
      rotate_pair(bf16_bits_to_f32(k_in[lane]), bf16_bits_to_f32(k_in[lane + 64]), cos_t[trow * (HD / 2) + lane],
                  sin_t[trow * (HD / 2) + lane], lo, hi);
      new_k[lane] = bits_of(lo);
      new_k[lane + 64] = bits_of(hi);
      kbase[(int64_t)pos * HD + lane] = bits_of(lo);
      kbase[(int64_t)pos * HD + lane + 64] = bits_of(hi);
#pragma unroll
      for (int d = lane; d < HD; d += 64) {
        const uint16_t v = v_in[d];
        new_v[d] = v;
        vbase[((int64_t)(pos >> 3) * HD + d) * 8 + (pos & 7)] = v;
      }
    }
  }
  for (int c = wave; c < chunks; c += 8) {
    if (c + 4 < chunks) load(fb, c + 4);
    step(fa, c);
    if (c + 4 < chunks) {
      if (c + 8 < chunks) load(fa, c + 8);
      step(fb, c + 4);
    }
  }

  // combine the four waves
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int h = 4 * g + r;
    if (h < group) {
#pragma unroll
      for (int nb = 0; nb < 8; ++nb) o_lds[(wave * group + h) * HD + nb * 16 + hq] = o[nb][r];
    }
  }
  if (g == 0 && hq < group) {
    m_lds[wave * group + hq] = m;
    l_lds[wave * group + hq] = l;
  }
  __syncthreads();
  for (int idx = tid; idx < group * HD; idx += DEC_THREADS) {
    const int h = idx >> 7, dim = idx & (HD - 1);
    float mm = m_lds[h];
#pragma unroll
    for (int w = 1; w < 4; ++w) mm = fmaxf(mm, m_lds[w * group + h]);
    float num = 0.0f, den = 0.0f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float f = exp2f(m_lds[w * group + h] - mm);   // 0 for a wave that had no chunk (m = -inf)
      num += o_lds[(w * group + h) * HD + dim] * f;
      den += l_lds[w * group + h] * f;
    }
    out_row[idx] = static_cast<uint16_t>(f32_to_bf16_bits(num / den));
  }
}

// One workgroup per token: rotate q and k of the new token (position lengths[t] - 1), store q,
// append k and v to the caches of slot slots[t].
__global__ void __launch_bounds__(256)
rope_kv_append_kernel(const uint16_t* __restrict__ qkv, int64_t ld_qkv, uint16_t* __restrict__ q_out, int64_t ld_q,
                      uint16_t* __restrict__ kc, uint16_t* __restrict__ vc, const int32_t* __restrict__ slots,
                      const int32_t* __restrict__ lengths, const float* __restrict__ cos_t,
                      const float* __restrict__ sin_t, int q_heads, int kv_heads, int num_slots, int capacity,
                      int table_rows) {
  const int t = blockIdx.x, tid = threadIdx.x;
  const int slot = slots[t], pos = lengths[t] - 1;
  const bool cache_ok = slot >= 0 && slot < num_slots && pos >= 0 && pos < capacity;
  const int trow = pos < 0 ? 0 : (pos < table_rows ? pos : table_rows - 1);
  const uint16_t* row = qkv + (int64_t)t * ld_qkv;
  const int64_t slot_base = (int64_t)slot * kv_heads;
  for (int idx = tid; idx < (q_heads + kv_heads) * (HD / 2); idx += 256) {
    const int head = idx >> 6, i = idx & 63;
    const float lo = bf16_bits_to_f32(row[head * HD + i]), hi = bf16_bits_to_f32(row[head * HD + i + 64]);
    const float c = cos_t[trow * (HD / 2) + i], s = sin_t[trow * (HD / 2) + i];
    bf16_t olo, ohi;
    rotate_pair(lo, hi, c, s, olo, ohi);
    if (head < q_heads) {
      uint16_t* dst = q_out + (int64_t)t * ld_q + head * HD + i;
      dst[0] = bits_of(olo);
      dst[64] = bits_of(ohi);
    } else if (cache_ok) {
      uint16_t* dst = kc + ((slot_base + (head - q_heads)) * capacity + pos) * HD + i;
      dst[0] = bits_of(olo);
      dst[64] = bits_of(ohi);
    }
  }
  if (!cache_ok) return;
  const uint16_t* vrow = row + (q_heads + kv_heads) * HD;
  for (int idx = tid; idx < kv_heads * HD; idx += 256) {
    const int kh = idx >> 7, dim = idx & (HD - 1);
    vc[(((slot_base + kh) * (capacity / 8) + (pos >> 3)) * HD + dim) * 8 + (pos & 7)] = vrow[idx];
  }
}

}  // namespace

extern "C" int dfhip_rope_kv_append_bf16(const void* qkv, int64_t ld_qkv, void* q_out, int64_t ld_q, void* k_cache,
                                         void* v_cache, const int32_t* slots, const int32_t* lengths,
                                         const float* cos_table, const float* sin_table, int T, int q_heads,
                                         int kv_heads, int head_dim, int num_slots, int capacity, int table_rows,
                                         dfhip_stream_t stream) {
  if (!qkv || !q_out || !k_cache || !v_cache || !slots || !lengths || !cos_table || !sin_table)
    return DFHIP_ERR_NULL_POINTER;
  if (T < 1 || q_heads < 1 || kv_heads < 1 || head_dim != HD || num_slots < 1 || capacity < CHUNK ||
      capacity % CHUNK != 0 || table_rows < 1)
    return DFHIP_ERR_BAD_SHAPE;
  if (ld_qkv < (int64_t)(q_heads + 2 * kv_heads) * HD || ld_q < (int64_t)q_heads * HD) return DFHIP_ERR_BAD_STRIDE;
  hipLaunchKernelGGL(rope_kv_append_kernel, dim3(T), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const uint16_t*>(qkv), ld_qkv, static_cast<uint16_t*>(q_out), ld_q,
                     static_cast<uint16_t*>(k_cache), static_cast<uint16_t*>(v_cache), slots, lengths, cos_table,
                     sin_table, q_heads, kv_heads, num_slots, capacity, table_rows);
  return dfhip_check_launch();
}

extern "C" int dfhip_decode_attention_bf16(const void* q, int64_t ld_q, const void* k_cache, const void* v_cache,
                                           const int32_t* slots, const int32_t* lengths, void* out, int64_t ld_out,
                                           int T, int q_heads, int kv_heads, int head_dim, int num_slots,
                                           int capacity, float scale, dfhip_stream_t stream) {
  if (!q || !k_cache || !v_cache || !slots || !lengths || !out) return DFHIP_ERR_NULL_POINTER;
  if (T < 1 || q_heads < 1 || kv_heads < 1 || q_heads % kv_heads != 0 || q_heads / kv_heads > MAX_GROUP ||
      head_dim != HD || num_slots < 1 || capacity < CHUNK || capacity % CHUNK != 0 ||
      (int64_t)T * kv_heads >= (int64_t)1 << 31)
    return DFHIP_ERR_BAD_SHAPE;
  if (ld_q < (int64_t)q_heads * HD || ld_out < (int64_t)q_heads * HD) return DFHIP_ERR_BAD_STRIDE;
  if (ld_q % 8 || !dfhip_aligned16(q) || !dfhip_aligned16(k_cache) || !dfhip_aligned16(v_cache))
    return DFHIP_ERR_BAD_ALIGNMENT;
  const float scale_log2 = scale * 1.4426950408889634f;
  const int group = q_heads / kv_heads;
  const size_t combine_bytes = (size_t)4 * group * (HD + 2) * sizeof(float);
  hipLaunchKernelGGL(decode_attention_kernel<false>, dim3(T * kv_heads), dim3(DEC_THREADS), combine_bytes,
                     static_cast<hipStream_t>(stream), static_cast<const uint16_t*>(q), ld_q,
                     static_cast<uint16_t*>(const_cast<void*>(k_cache)), static_cast<uint16_t*>(const_cast<void*>(v_cache)),
                     slots, lengths, static_cast<uint16_t*>(out), ld_out, kv_heads, group, num_slots, capacity,
                     scale_log2, nullptr, nullptr, 1);
  return dfhip_check_launch();
}

extern "C" int dfhip_decode_attention_append_bf16(const void* qkv, int64_t ld_qkv, void* k_cache, void* v_cache,
                                                  const int32_t* slots, const int32_t* lengths,
                                                  const float* cos_table, const float* sin_table, void* out,
                                                  int64_t ld_out, int T, int q_heads, int kv_heads, int head_dim,
                                                  int num_slots, int capacity, int table_rows, float scale,
                                                  dfhip_stream_t stream) {
  if (!qkv || !k_cache || !v_cache || !slots || !lengths || !cos_table || !sin_table || !out)
    return DFHIP_ERR_NULL_POINTER;
  if (T < 1 || q_heads < 1 || kv_heads < 1 || q_heads % kv_heads != 0 || q_heads / kv_heads > MAX_GROUP ||
      head_dim != HD || num_slots < 1 || capacity < CHUNK || capacity % CHUNK != 0 || table_rows < 1 ||
      (int64_t)T * kv_heads >= (int64_t)1 << 31)
    return DFHIP_ERR_BAD_SHAPE;
  if (ld_qkv < (int64_t)(q_heads + 2 * kv_heads) * HD || ld_out < (int64_t)q_heads * HD) return DFHIP_ERR_BAD_STRIDE;
  if (ld_qkv % 8 || !dfhip_aligned16(qkv) || !dfhip_aligned16(k_cache) || !dfhip_aligned16(v_cache))
    return DFHIP_ERR_BAD_ALIGNMENT;
  const int group = q_heads / kv_heads;
  const size_t lds_bytes = (size_t)4 * group * (HD + 2) * sizeof(float) + 2 * HD * sizeof(uint16_t);
  hipLaunchKernelGGL(decode_attention_kernel<true>, dim3(T * kv_heads), dim3(DEC_THREADS), lds_bytes,
                     static_cast<hipStream_t>(stream), static_cast<const uint16_t*>(qkv), ld_qkv,
                     static_cast<uint16_t*>(k_cache), static_cast<uint16_t*>(v_cache), slots, lengths,
                     static_cast<uint16_t*>(out), ld_out, kv_heads, group, num_slots, capacity,
                     scale * 1.4426950408889634f, cos_table, sin_table, table_rows);
  return dfhip_check_launch();
}

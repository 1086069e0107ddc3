// HBM-bound kernels of the MLP path: SiLU*mul, RMSNorm, transpose, fill.
//
// All of them move 16 bytes per lane per access (global_load/store_dwordx4) from
// many small workgroups and do their arithmetic in fp32 with a single rounding at
// the store.
#include "dfhip_common.h"

namespace {

constexpr int EW_THREADS = 256;
constexpr int EW_UNROLL = 1;  // 16-byte groups per lane per array: one is fastest here (6.5 vs 5.4 TB/s with four):
                              // occupancy hides the latency better than a longer per-lane queue does

DFHIP_DEVICE float silu_f32(float g) { return g / (1.0f + expf(-g)); }

// out[t, j] = bf16(silu(gate[t, j]) * up[t, j]); a "group" is 8 consecutive j.
template <bool ROUND_SILU>
__global__ void __launch_bounds__(EW_THREADS)
silu_mul_bf16_kernel(const uint16_t* __restrict__ gate, int64_t ld_gate, const uint16_t* __restrict__ up,
                     int64_t ld_up, uint16_t* __restrict__ out, int64_t ld_out, uint32_t groups,
                     uint32_t groups_per_row) {
  const uint32_t first = blockIdx.x * (EW_THREADS * EW_UNROLL) + threadIdx.x;
  u32x4 g[EW_UNROLL], u[EW_UNROLL];
  uint32_t row[EW_UNROLL], col[EW_UNROLL];
#pragma unroll
  for (int p = 0; p < EW_UNROLL; ++p) {
    const uint32_t gi = first + p * EW_THREADS;
    row[p] = gi / groups_per_row;
    col[p] = (gi - row[p] * groups_per_row) * 8;
    if (gi < groups) {
      g[p] = *reinterpret_cast<const u32x4*>(gate + (int64_t)row[p] * ld_gate + col[p]);
      u[p] = *reinterpret_cast<const u32x4*>(up + (int64_t)row[p] * ld_up + col[p]);
    }
  }
#pragma unroll
  for (int p = 0; p < EW_UNROLL; ++p) {
    const uint32_t gi = first + p * EW_THREADS;
    if (gi >= groups) continue;
    u32x4 o;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      float g_lo = bf16_bits_to_f32(g[p][w] & 0xffffu), g_hi = __uint_as_float(g[p][w] & 0xffff0000u);
      float u_lo = bf16_bits_to_f32(u[p][w] & 0xffffu), u_hi = __uint_as_float(u[p][w] & 0xffff0000u);
      float s_lo = silu_fast(g_lo), s_hi = silu_fast(g_hi);   // same formula as the GEMM epilogues: same bits
      if (ROUND_SILU) {
        s_lo = bf16_bits_to_f32(f32_to_bf16_bits(s_lo));
        s_hi = bf16_bits_to_f32(f32_to_bf16_bits(s_hi));
      }
      o[w] = pack2_bf16(s_lo * u_lo, s_hi * u_hi);
    }
    *reinterpret_cast<u32x4*>(out + (int64_t)row[p] * ld_out + col[p]) = o;
  }
}

// fp32 flavour; a group is 4 consecutive j.
__global__ void __launch_bounds__(EW_THREADS)
silu_mul_f32_kernel(const float* __restrict__ gate, int64_t ld_gate, const float* __restrict__ up,
                    int64_t ld_up, float* __restrict__ out, int64_t ld_out, uint32_t groups,
                    uint32_t groups_per_row) {
  const uint32_t first = blockIdx.x * (EW_THREADS * EW_UNROLL) + threadIdx.x;
  f32x4 g[EW_UNROLL], u[EW_UNROLL];
  uint32_t row[EW_UNROLL], col[EW_UNROLL];
#pragma unroll
  for (int p = 0; p < EW_UNROLL; ++p) {
    const uint32_t gi = first + p * EW_THREADS;
    row[p] = gi / groups_per_row;
    col[p] = (gi - row[p] * groups_per_row) * 4;
    if (gi < groups) {
      g[p] = *reinterpret_cast<const f32x4*>(gate + (int64_t)row[p] * ld_gate + col[p]);
      u[p] = *reinterpret_cast<const f32x4*>(up + (int64_t)row[p] * ld_up + col[p]);
    }
  }
#pragma unroll
  for (int p = 0; p < EW_UNROLL; ++p) {
    const uint32_t gi = first + p * EW_THREADS;
    if (gi >= groups) continue;
    f32x4 o;
#pragma unroll
    for (int w = 0; w < 4; ++w) o[w] = silu_f32(g[p][w]) * u[p][w];
    *reinterpret_cast<f32x4*>(out + (int64_t)row[p] * ld_out + col[p]) = o;
  }
}

// One workgroup per row; the whole row lives in registers between the two passes.
constexpr int NORM_THREADS = 256;
constexpr int NORM_MAX_CHUNKS = 8;  // 8 chunks * 8 elements * 256 lanes = 16384 columns

__global__ void __launch_bounds__(NORM_THREADS)
rmsnorm_bf16_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ residual,
                    const uint16_t* __restrict__ weight, uint16_t* __restrict__ out,
                    uint16_t* __restrict__ residual_out, int H, float eps) {
  __shared__ float partial[NORM_THREADS / 64];
  const int64_t row_off = (int64_t)blockIdx.x * H;
  const int chunks = H / 8;
  u32x4 h[NORM_MAX_CHUNKS];
  float sumsq = 0.0f;
#pragma unroll
  for (int p = 0; p < NORM_MAX_CHUNKS; ++p) {
    const int c = threadIdx.x + p * NORM_THREADS;
    if (c < chunks) h[p] = *reinterpret_cast<const u32x4*>(x + row_off + c * 8);
  }
  if (residual != nullptr) {
#pragma unroll
    for (int p = 0; p < NORM_MAX_CHUNKS; ++p) {
      const int c = threadIdx.x + p * NORM_THREADS;
      if (c < chunks) {
        const u32x4 r = *reinterpret_cast<const u32x4*>(residual + row_off + c * 8);
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          // bf16 add: fp32 sum rounded back to bf16, like a bf16 tensor add
          const float lo = bf16_bits_to_f32(h[p][w] & 0xffffu) + bf16_bits_to_f32(r[w] & 0xffffu);
          const float hi = __uint_as_float(h[p][w] & 0xffff0000u) + __uint_as_float(r[w] & 0xffff0000u);
          h[p][w] = pack2_bf16(lo, hi);
        }
        if (residual_out != nullptr) *reinterpret_cast<u32x4*>(residual_out + row_off + c * 8) = h[p];
      }
    }
  }
#pragma unroll
  for (int p = 0; p < NORM_MAX_CHUNKS; ++p) {
    const int c = threadIdx.x + p * NORM_THREADS;
    if (c < chunks) {
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const float lo = bf16_bits_to_f32(h[p][w] & 0xffffu);
        const float hi = __uint_as_float(h[p][w] & 0xffff0000u);
        sumsq += lo * lo;
        sumsq += hi * hi;
      }
    }
  }
  sumsq = wave_sum(sumsq);
  if ((threadIdx.x & 63) == 0) partial[threadIdx.x >> 6] = sumsq;
  __syncthreads();
  float total = 0.0f;
#pragma unroll
  for (int w = 0; w < NORM_THREADS / 64; ++w) total += partial[w];
  const float inv = rsqrtf(total / (float)H + eps);
#pragma unroll
  for (int p = 0; p < NORM_MAX_CHUNKS; ++p) {
    const int c = threadIdx.x + p * NORM_THREADS;
    if (c < chunks) {
      const u32x4 wv = *reinterpret_cast<const u32x4*>(weight + c * 8);
      u32x4 o;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        // scale, round to bf16, then multiply by the weight and round again
        const float lo = bf16_bits_to_f32(f32_to_bf16_bits(bf16_bits_to_f32(h[p][w] & 0xffffu) * inv));
        const float hi = bf16_bits_to_f32(f32_to_bf16_bits(__uint_as_float(h[p][w] & 0xffff0000u) * inv));
        o[w] = pack2_bf16(lo * bf16_bits_to_f32(wv[w] & 0xffffu), hi * __uint_as_float(wv[w] & 0xffff0000u));
      }
      *reinterpret_cast<u32x4*>(out + row_off + c * 8) = o;
    }
  }
}

// out[n, k] = in[k, n]; 64x64 tiles through LDS (padded against bank conflicts).
constexpr int TR_TILE = 64;
__global__ void __launch_bounds__(256)
transpose_bf16_kernel(const uint16_t* __restrict__ in, int64_t ld_in, uint16_t* __restrict__ out,
                      int64_t ld_out, int K, int N) {
  __shared__ uint16_t tile[TR_TILE][TR_TILE + 2];
  const int k0 = blockIdx.y * TR_TILE;
  const int n0 = blockIdx.x * TR_TILE;
  for (int i = threadIdx.x; i < TR_TILE * TR_TILE; i += 256) {
    const int r = i / TR_TILE, c = i % TR_TILE;
    if (k0 + r < K && n0 + c < N) tile[r][c] = in[(int64_t)(k0 + r) * ld_in + n0 + c];
  }
  __syncthreads();
  for (int i = threadIdx.x; i < TR_TILE * TR_TILE; i += 256) {
    const int r = i / TR_TILE, c = i % TR_TILE;  // r indexes n, c indexes k
    if (n0 + r < N && k0 + c < K) out[(int64_t)(n0 + r) * ld_out + k0 + c] = tile[c][r];
  }
}

// Rotary embedding, half-split pairs (x[i], x[i + d/2]) of every head, position = row % seq_len:
//   out_lo = lo*cos - hi*sin,  out_hi = hi*cos + lo*sin   (fp32, one rounding)
// One lane rotates 8 pairs: 16 bytes of the low half and the matching 16 bytes of the high half.
__global__ void __launch_bounds__(EW_THREADS)
rope_bf16_kernel(const uint16_t* __restrict__ x, int64_t ld_x, uint16_t* __restrict__ out, int64_t ld_out,
                 const float* __restrict__ cos_t, const float* __restrict__ sin_t, uint32_t groups, int heads,
                 int half, int seq_len) {
  const uint32_t gi = blockIdx.x * EW_THREADS + threadIdx.x;
  if (gi >= groups) return;
  const uint32_t per_head = half / 8;                 // groups of 8 pairs per head
  const uint32_t per_row = per_head * heads;
  const uint32_t row = gi / per_row;
  const uint32_t in_row = gi - row * per_row;
  const uint32_t head = in_row / per_head;
  const uint32_t pair0 = (in_row - head * per_head) * 8;
  const uint32_t pos = row % (uint32_t)seq_len;
  const int64_t lo_off = (int64_t)head * (2 * half) + pair0;
  const u32x4 lo = *reinterpret_cast<const u32x4*>(x + (int64_t)row * ld_x + lo_off);
  const u32x4 hi = *reinterpret_cast<const u32x4*>(x + (int64_t)row * ld_x + lo_off + half);
  const f32x4 c0 = *reinterpret_cast<const f32x4*>(cos_t + (int64_t)pos * half + pair0);
  const f32x4 c1 = *reinterpret_cast<const f32x4*>(cos_t + (int64_t)pos * half + pair0 + 4);
  const f32x4 s0 = *reinterpret_cast<const f32x4*>(sin_t + (int64_t)pos * half + pair0);
  const f32x4 s1 = *reinterpret_cast<const f32x4*>(sin_t + (int64_t)pos * half + pair0 + 4);
  u32x4 olo, ohi;
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    const float c_a = w < 2 ? c0[2 * w] : c1[2 * w - 4], c_b = w < 2 ? c0[2 * w + 1] : c1[2 * w - 3];
    const float s_a = w < 2 ? s0[2 * w] : s1[2 * w - 4], s_b = w < 2 ? s0[2 * w + 1] : s1[2 * w - 3];
    const float lo_a = bf16_bits_to_f32(lo[w] & 0xffffu), lo_b = __uint_as_float(lo[w] & 0xffff0000u);
    const float hi_a = bf16_bits_to_f32(hi[w] & 0xffffu), hi_b = __uint_as_float(hi[w] & 0xffff0000u);
    olo[w] = pack2_bf16(lo_a * c_a - hi_a * s_a, lo_b * c_b - hi_b * s_b);
    ohi[w] = pack2_bf16(hi_a * c_a + lo_a * s_a, hi_b * c_b + lo_b * s_b);
  }
  *reinterpret_cast<u32x4*>(out + (int64_t)row * ld_out + lo_off) = olo;
  *reinterpret_cast<u32x4*>(out + (int64_t)row * ld_out + lo_off + half) = ohi;
}

__global__ void __launch_bounds__(256) fill_u32_kernel(uint32_t* dst, uint32_t value, int64_t count) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < count; i += (int64_t)gridDim.x * 256)
    dst[i] = value;
}

int check_rowwise(const void* gate, int64_t ld_gate, const void* up, int64_t ld_up, const void* out,
                  int64_t ld_out, int M, int D, int vec) {
  if (!gate || !up || !out) return DFHIP_ERR_NULL_POINTER;
  if (M < 1 || D < 1 || D % vec != 0) return DFHIP_ERR_BAD_SHAPE;
  if ((int64_t)M * (D / vec) >= (int64_t)1 << 31) return DFHIP_ERR_BAD_SHAPE;
  if (ld_gate < D || ld_up < D || ld_out < D) return DFHIP_ERR_BAD_STRIDE;
  if (ld_gate % vec || ld_up % vec || ld_out % vec || !dfhip_aligned16(gate) || !dfhip_aligned16(up) ||
      !dfhip_aligned16(out))
    return DFHIP_ERR_BAD_ALIGNMENT;
  return DFHIP_OK;
}

}  // namespace

extern "C" int dfhip_silu_mul_bf16(const void* gate, int64_t ld_gate, const void* up, int64_t ld_up, void* out,
                                   int64_t ld_out, int M, int D, int round_inputs_product,
                                   dfhip_stream_t stream) {
  if (int rc = check_rowwise(gate, ld_gate, up, ld_up, out, ld_out, M, D, 8)) return rc;
  const uint32_t per_row = D / 8;
  const uint32_t groups = (uint32_t)M * per_row;
  const uint32_t blocks = (groups + EW_THREADS * EW_UNROLL - 1) / (EW_THREADS * EW_UNROLL);
  auto g = static_cast<const uint16_t*>(gate);
  auto u = static_cast<const uint16_t*>(up);
  auto o = static_cast<uint16_t*>(out);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (round_inputs_product)
    hipLaunchKernelGGL(silu_mul_bf16_kernel<true>, dim3(blocks), dim3(EW_THREADS), 0, s, g, ld_gate, u, ld_up, o,
                       ld_out, groups, per_row);
  else
    hipLaunchKernelGGL(silu_mul_bf16_kernel<false>, dim3(blocks), dim3(EW_THREADS), 0, s, g, ld_gate, u, ld_up,
                       o, ld_out, groups, per_row);
  return dfhip_check_launch();
}

extern "C" int dfhip_silu_mul_f32(const void* gate, int64_t ld_gate, const void* up, int64_t ld_up, void* out,
                                  int64_t ld_out, int M, int D, dfhip_stream_t stream) {
  if (int rc = check_rowwise(gate, ld_gate, up, ld_up, out, ld_out, M, D, 4)) return rc;
  const uint32_t per_row = D / 4;
  const uint32_t groups = (uint32_t)M * per_row;
  const uint32_t blocks = (groups + EW_THREADS * EW_UNROLL - 1) / (EW_THREADS * EW_UNROLL);
  hipLaunchKernelGGL(silu_mul_f32_kernel, dim3(blocks), dim3(EW_THREADS), 0, static_cast<hipStream_t>(stream),
                     static_cast<const float*>(gate), ld_gate, static_cast<const float*>(up), ld_up,
                     static_cast<float*>(out), ld_out, groups, per_row);
  return dfhip_check_launch();
}

extern "C" int dfhip_rmsnorm_bf16(const void* x, const void* residual, const void* weight, void* out,
                                  void* residual_out, int M, int H, float eps, dfhip_stream_t stream) {
  if (!x || !weight || !out) return DFHIP_ERR_NULL_POINTER;
  if (M < 1 || H < 8 || H % 8 != 0 || H > NORM_MAX_CHUNKS * 8 * NORM_THREADS) return DFHIP_ERR_BAD_SHAPE;
  if (!dfhip_aligned16(x) || !dfhip_aligned16(weight) || !dfhip_aligned16(out) ||
      (residual && !dfhip_aligned16(residual)) || (residual_out && !dfhip_aligned16(residual_out)))
    return DFHIP_ERR_BAD_ALIGNMENT;
  hipLaunchKernelGGL(rmsnorm_bf16_kernel, dim3(M), dim3(NORM_THREADS), 0, static_cast<hipStream_t>(stream),
                     static_cast<const uint16_t*>(x), static_cast<const uint16_t*>(residual),
                     static_cast<const uint16_t*>(weight), static_cast<uint16_t*>(out),
                     static_cast<uint16_t*>(residual_out), H, eps);
  return dfhip_check_launch();
}

extern "C" int dfhip_transpose_bf16(const void* in, int64_t ld_in, void* out, int64_t ld_out, int K, int N,
                                    dfhip_stream_t stream) {
  if (!in || !out) return DFHIP_ERR_NULL_POINTER;
  if (K < 1 || N < 1) return DFHIP_ERR_BAD_SHAPE;
  if (ld_in < N || ld_out < K) return DFHIP_ERR_BAD_STRIDE;
  dim3 grid((N + TR_TILE - 1) / TR_TILE, (K + TR_TILE - 1) / TR_TILE);
  hipLaunchKernelGGL(transpose_bf16_kernel, grid, dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const uint16_t*>(in), ld_in, static_cast<uint16_t*>(out), ld_out, K, N);
  return dfhip_check_launch();
}

extern "C" int dfhip_fill_u32(void* dst, uint32_t value, int64_t count, dfhip_stream_t stream) {
  if (!dst) return DFHIP_ERR_NULL_POINTER;
  if (count < 1) return DFHIP_ERR_BAD_SHAPE;
  int64_t blocks = (count + 255) / 256;
  if (blocks > 1024) blocks = 1024;
  hipLaunchKernelGGL(fill_u32_kernel, dim3((unsigned)blocks), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<uint32_t*>(dst), value, count);
  return dfhip_check_launch();
}

extern "C" int dfhip_rope_bf16(const void* x, int64_t ld_x, void* out, int64_t ld_out, const float* cos_table,
                               const float* sin_table, int T, int heads, int head_dim, int seq_len,
                               dfhip_stream_t stream) {
  if (!x || !out || !cos_table || !sin_table) return DFHIP_ERR_NULL_POINTER;
  if (T < 1 || heads < 1 || head_dim < 16 || head_dim % 16 != 0 || seq_len < 1) return DFHIP_ERR_BAD_SHAPE;
  if ((int64_t)T * heads * (head_dim / 16) >= (int64_t)1 << 31) return DFHIP_ERR_BAD_SHAPE;
  if (ld_x < (int64_t)heads * head_dim || ld_out < (int64_t)heads * head_dim) return DFHIP_ERR_BAD_STRIDE;
  if (ld_x % 8 || ld_out % 8 || !dfhip_aligned16(x) || !dfhip_aligned16(out) || !dfhip_aligned16(cos_table) ||
      !dfhip_aligned16(sin_table))
    return DFHIP_ERR_BAD_ALIGNMENT;
  const int half = head_dim / 2;
  const uint32_t groups = (uint32_t)T * heads * (half / 8);
  hipLaunchKernelGGL(rope_bf16_kernel, dim3((groups + EW_THREADS - 1) / EW_THREADS), dim3(EW_THREADS), 0,
                     static_cast<hipStream_t>(stream), static_cast<const uint16_t*>(x), ld_x,
                     static_cast<uint16_t*>(out), ld_out, cos_table, sin_table, groups, heads, half, seq_len);
  return dfhip_check_launch();
}

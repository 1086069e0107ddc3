/*
 * Plain-C restatement of the arithmetic on the batch-split MLP path.
 * TEST INFRASTRUCTURE: built into oracle/libmlp_ref.so by oracle/Makefile and
 * loaded only by tests, smoke() and the cpu_baseline leg of bench.py.
 *
 *   ref_silu_mul_bf16   examples/ae/up-silu-overlap.cu:75-90 (silu_one / silu8):
 *                       o = bf16( (g / (1 + expf(-g))) * u ), fp32 inside
 *   ref_rmsnorm_bf16    examples/ae/scheduler/vllm/tokenweave-kernels/csrc/
 *                       tokenweave.cu:85-109: fp32 sum of squares,
 *                       rsqrtf(var / H + eps), scale, then * weight, each
 *                       rounded to bf16
 *   ref_gemm_nt_f32     C = A * W^T with a double accumulator (the `linear` node)
 *   ref_gemm_nt_bf16    same on bf16 storage, result rounded to bf16
 *
 * bf16 values are uint16_t holding the upper half of an IEEE fp32.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

static float bf16_to_f32(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

static uint16_t f32_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u); /* NaN stays NaN */
  u += 0x7fffu + ((u >> 16) & 1u); /* round to nearest even */
  return (uint16_t)(u >> 16);
}

void ref_silu_mul_bf16(const uint16_t* gate, long ld_gate, const uint16_t* up, long ld_up, uint16_t* out,
                       long ld_out, long M, long D, int round_silu) {
  for (long t = 0; t < M; ++t)
    for (long j = 0; j < D; ++j) {
      float g = bf16_to_f32(gate[t * ld_gate + j]);
      float u = bf16_to_f32(up[t * ld_up + j]);
      float s = g / (1.0f + expf(-g));
      if (round_silu) s = bf16_to_f32(f32_to_bf16(s));
      out[t * ld_out + j] = f32_to_bf16(s * u);
    }
}

void ref_silu_mul_f32(const float* gate, const float* up, float* out, long n) {
  for (long i = 0; i < n; ++i) out[i] = (gate[i] / (1.0f + expf(-gate[i]))) * up[i];
}

void ref_rmsnorm_bf16(const uint16_t* x, const uint16_t* weight, uint16_t* out, long M, long H, float eps) {
  for (long t = 0; t < M; ++t) {
    float var = 0.0f;
    for (long j = 0; j < H; ++j) {
      float v = bf16_to_f32(x[t * H + j]);
      var += v * v;
    }
    float inv = 1.0f / sqrtf(var / (float)H + eps);
    for (long j = 0; j < H; ++j) {
      float n = bf16_to_f32(f32_to_bf16(bf16_to_f32(x[t * H + j]) * inv));
      out[t * H + j] = f32_to_bf16(n * bf16_to_f32(weight[j]));
    }
  }
}

void ref_gemm_nt_f32(const float* A, const float* W, float* C, long M, long N, long K) {
  for (long m = 0; m < M; ++m)
    for (long n = 0; n < N; ++n) {
      double acc = 0.0;
      for (long k = 0; k < K; ++k) acc += (double)A[m * K + k] * (double)W[n * K + k];
      C[m * N + n] = (float)acc;
    }
}

void ref_gemm_nt_bf16(const uint16_t* A, const uint16_t* W, uint16_t* C, long M, long N, long K) {
  for (long m = 0; m < M; ++m)
    for (long n = 0; n < N; ++n) {
      double acc = 0.0;
      for (long k = 0; k < K; ++k) acc += (double)bf16_to_f32(A[m * K + k]) * (double)bf16_to_f32(W[n * K + k]);
      C[m * N + n] = f32_to_bf16((float)acc);
    }
}

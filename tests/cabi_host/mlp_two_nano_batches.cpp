// A host program with no Python and no PyTorch in it: the batch-split SwiGLU MLP through the C ABI of
// libdynaflow_hip.so, two nano-batches on two HIP streams (gate/up projection with the SiLU*mul epilogue, then
// the down projection), checked against the plain-C restatement of the arithmetic (oracle/libmlp_ref.so).
// TEST INFRASTRUCTURE: built by tests/cabi_host/Makefile, run by tests/test_gpu_cabi_from_c.py on a GPU.
//
// What a maintainer of the reference would write behind `ctx.execute(op, func)` of a scheduler
// (dynaflow/executor/engine.py:374-381 runs the sub-graph's callable on the current stream): the same calls,
// with the framework's tensors' pointers and the current stream's handle.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <vector>

#include "dynaflow_hip.h"

extern "C" {
void ref_silu_mul_bf16(const uint16_t* gate, long ld_gate, const uint16_t* up, long ld_up, uint16_t* out,
                       long ld_out, long M, long D, int round_silu);
void ref_gemm_nt_bf16(const uint16_t* A, const uint16_t* W, uint16_t* C, long M, long N, long K);
}

namespace {

uint16_t to_bf16(float f) {          // round to nearest even
  uint32_t u;
  std::memcpy(&u, &f, 4);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
float to_f32(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  std::memcpy(&f, &u, 4);
  return f;
}
std::vector<uint16_t> uniform_bf16(size_t n, float scale, uint32_t seed) {
  std::vector<uint16_t> v(n);
  uint32_t s = seed;
  for (size_t i = 0; i < n; ++i) {
    s = s * 1664525u + 1013904223u;
    v[i] = to_bf16(((float)(s >> 8) / 8388608.0f - 1.0f) * scale);
  }
  return v;
}

#define HIP_OK(call)                                                                          \
  do {                                                                                        \
    hipError_t e_ = (call);                                                                   \
    if (e_ != hipSuccess) {                                                                   \
      std::fprintf(stderr, "%s: %s\n", #call, hipGetErrorString(e_));                         \
      return 2;                                                                               \
    }                                                                                         \
  } while (0)
#define DF_OK(call)                                                                           \
  do {                                                                                        \
    int s_ = (call);                                                                          \
    if (s_ != DFHIP_OK) {                                                                     \
      std::fprintf(stderr, "%s: %s\n", #call, dfhip_status_string(s_));                       \
      return 3;                                                                               \
    }                                                                                         \
  } while (0)

}  // namespace

int main() {
  const int T = 256, H = 512, I = 1408, lanes = 2, rows = T / lanes;
  std::printf("library %d for %s\n", dfhip_version(), dfhip_arch());
  std::fflush(stdout);
  const std::vector<uint16_t> x = uniform_bf16((size_t)T * H, 1.0f, 1), wg = uniform_bf16((size_t)I * H, 0.05f, 2),
                              wu = uniform_bf16((size_t)I * H, 0.05f, 3), wd = uniform_bf16((size_t)H * I, 0.05f, 4);
  uint16_t *dx, *dwg, *dwu, *dwd, *dact, *dout;
  HIP_OK(hipMalloc(&dx, x.size() * 2));
  HIP_OK(hipMalloc(&dwg, wg.size() * 2));
  HIP_OK(hipMalloc(&dwu, wu.size() * 2));
  HIP_OK(hipMalloc(&dwd, wd.size() * 2));
  HIP_OK(hipMalloc(&dact, (size_t)T * I * 2));
  HIP_OK(hipMalloc(&dout, (size_t)T * H * 2));
  HIP_OK(hipMemcpy(dx, x.data(), x.size() * 2, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(dwg, wg.data(), wg.size() * 2, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(dwu, wu.data(), wu.size() * 2, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(dwd, wd.data(), wd.size() * 2, hipMemcpyHostToDevice));

  // the C ABI refuses what it cannot run, with a status instead of a fault
  if (dfhip_gemm_bf16_nt(dx, H, dwg, H, dact, I, 0, I, H, nullptr) != DFHIP_ERR_BAD_SHAPE ||
      dfhip_gemm_bf16_nt(nullptr, H, dwg, H, dact, I, rows, I, H, nullptr) != DFHIP_ERR_NULL_POINTER) {
    std::fprintf(stderr, "bad arguments were not refused\n");
    return 4;
  }

  hipStream_t stream[lanes];
  for (int b = 0; b < lanes; ++b) HIP_OK(hipStreamCreate(&stream[b]));   // default priority
  for (int b = 0; b < lanes; ++b) {
    const uint16_t* xb = dx + (size_t)b * rows * H;
    uint16_t* actb = dact + (size_t)b * rows * I;
    uint16_t* outb = dout + (size_t)b * rows * H;      // the nano-batches' outputs land in one buffer: no concatenation
    DF_OK(dfhip_gemm_bf16_gate_up_silu(xb, H, dwg, dwu, H, actb, I, rows, I, H, stream[b]));
    DF_OK(dfhip_gemm_bf16_nt(actb, I, dwd, I, outb, H, rows, H, I, stream[b]));
  }
  for (int b = 0; b < lanes; ++b) HIP_OK(hipStreamSynchronize(stream[b]));
  std::vector<uint16_t> got((size_t)T * H);
  HIP_OK(hipMemcpy(got.data(), dout, got.size() * 2, hipMemcpyDeviceToHost));

  // the unsplit layer on the host: cat_b MLP(x_b) == MLP(x) row by row
  std::vector<uint16_t> g((size_t)T * I), u((size_t)T * I), act((size_t)T * I), want((size_t)T * H);
  ref_gemm_nt_bf16(x.data(), wg.data(), g.data(), T, I, H);
  ref_gemm_nt_bf16(x.data(), wu.data(), u.data(), T, I, H);
  ref_silu_mul_bf16(g.data(), I, u.data(), I, act.data(), I, T, I, 1);
  ref_gemm_nt_bf16(act.data(), wd.data(), want.data(), T, H, I);
  double worst = 0.0, scale = 0.0;
  for (size_t i = 0; i < got.size(); ++i) {
    worst = std::fmax(worst, std::fabs((double)to_f32(got[i]) - (double)to_f32(want[i])));
    scale = std::fmax(scale, std::fabs((double)to_f32(want[i])));
  }
  const double rel = worst / scale;
  std::printf("max |got - want| / max |want| = %.3e (bf16 tolerance 2e-2)\n", rel);
  for (int b = 0; b < lanes; ++b) HIP_OK(hipStreamDestroy(stream[b]));
  for (void* p : {(void*)dx, (void*)dwg, (void*)dwu, (void*)dwd, (void*)dact, (void*)dout}) HIP_OK(hipFree(p));
  if (!(rel < 2e-2) || !(scale > 0.0)) {
    std::fprintf(stderr, "result differs from the host restatement\n");
    return 1;
  }
  std::printf("ok\n");
  return 0;
}

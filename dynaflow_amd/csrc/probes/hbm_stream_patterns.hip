// Calibration probe (not part of the library): the read-only streaming rate of a weight matrix against
// workgroup count and access pattern - what a weight-streaming (decode-sized) GEMM can reach at best.
// The matrix has 8 KiB rows (K = 4096 bf16); a workgroup of 4 waves reads blocks of 128 rows, 32 loads of
// 16 bytes a lane in flight per wave at most.  Three regions of 800 MiB rotate so that no cache keeps the data.
// Every address is computed from (row < 128, 16-byte column < 512) of a block inside the buffer.
// Build: make -C dynaflow_amd/csrc probes.  Run: probes/hbm_stream_patterns
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
#define CK(x) do{hipError_t e=(x); if(e!=hipSuccess){printf("HIP error %s at %d\n",hipGetErrorString(e),__LINE__); exit(1);} }while(0)
constexpr int ROWS = 28672, ROW16 = 512;           // uint4 per row
typedef unsigned int u4 __attribute__((ext_vector_type(4)));
// PAT 0: a workgroup streams 128 rows; one step = 128 bytes of each row (wave instruction: 8 rows x 128 B)
// PAT 1: the same bytes, a workgroup's rows as one contiguous 1 MiB piece (wave instruction: 1 KiB contiguous)
// PAT 2: like 0 but wave instruction = 32 rows x 32 B (MFMA operand layout)
template <int PAT>
__global__ void __launch_bounds__(256) stream_kernel(const u4* __restrict__ W, u4* __restrict__ out, int row_blocks) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  u4 acc = {0, 0, 0, 0};
  for (int rb = blockIdx.x; rb < row_blocks; rb += gridDim.x) {
    const u4* base = W + (size_t)rb * 128 * ROW16;
    auto addr = [&](int t, int j) -> const u4* {     // step t in 0..63, instruction j in 0..3
      if (PAT == 0) { const int row = wave * 32 + j * 8 + (lane >> 3), c = t * 8 + (lane & 7); return base + (size_t)row * ROW16 + c; }
      if (PAT == 2) { const int row = wave * 32 + (lane & 31), c = t * 8 + j * 2 + (lane >> 5); return base + (size_t)row * ROW16 + c; }
      return base + ((size_t)(t * 4 + j) * 4 + wave) * 64 + lane;    // 65536 uint4 = 64 steps x 4 x 4 waves x 64 lanes
    };
    u4 a[16], b[16];
#pragma unroll
    for (int q = 0; q < 16; ++q) a[q] = *addr(q >> 2, q & 3);
    for (int g = 0; g < 16; g += 2) {
#pragma unroll
      for (int q = 0; q < 16; ++q) b[q] = *addr((g + 1) * 4 + (q >> 2), q & 3);
#pragma unroll
      for (int q = 0; q < 16; ++q) acc ^= a[q];
      if (g + 2 < 16) {
#pragma unroll
        for (int q = 0; q < 16; ++q) a[q] = *addr((g + 2) * 4 + (q >> 2), q & 3);
      }
#pragma unroll
      for (int q = 0; q < 16; ++q) acc ^= b[q];
    }
  }
  if (acc[0] == 0x12345678u && acc[1] == 0x9abcdef0u) out[threadIdx.x] = acc;   // keeps the loads alive
}
int main() {
  const int COP = 12; const size_t per = (size_t)ROWS * ROW16;   // 12 x 224 = 2688 blocks of 1 MiB
  u4 *dW, *dO; CK(hipMalloc(&dW, per * 16 * COP)); CK(hipMalloc(&dO, 4096)); CK(hipMemset(dW, 0x3c, per * 16 * COP));
  hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
  for (int rep = 0; rep < 2; ++rep)
  for (int pat = 0; pat < 3; ++pat) for (int wgs : {128, 192, 224, 256, 512}) {
    const int blocks = 2 * wgs;                       // two 1 MiB row blocks per workgroup; 3 regions of 800 blocks rotate
    auto run = [&](int i) { const u4* W = dW + (size_t)(i % 3) * 800 * 128 * ROW16;
      if (pat == 0) hipLaunchKernelGGL(stream_kernel<0>, dim3(wgs), dim3(256), 0, 0, W, dO, blocks);
      else if (pat == 1) hipLaunchKernelGGL(stream_kernel<1>, dim3(wgs), dim3(256), 0, 0, W, dO, blocks);
      else hipLaunchKernelGGL(stream_kernel<2>, dim3(wgs), dim3(256), 0, 0, W, dO, blocks); };
    for (int i = 0; i < 6; ++i) run(i);
    CK(hipEventRecord(e0)); const int it = 48; for (int i = 0; i < it; ++i) run(i); CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
    float ms; CK(hipEventElapsedTime(&ms, e0, e1)); const double us = ms / it * 1e3;
    if (rep) printf("pattern %d workgroups %3d: %6.1f us -> %.2f TB/s\n", pat, wgs, us, blocks * 1048576.0 / us / 1e6); fflush(stdout);
  }
  CK(hipDeviceSynchronize());
  return 0;
}

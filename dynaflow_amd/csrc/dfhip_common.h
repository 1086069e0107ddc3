// Internal helpers shared by the kernel sources (not part of the C ABI).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "../../include/dynaflow_hip.h"

typedef __bf16 bf16_t;
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

#define DFHIP_DEVICE __device__ __forceinline__

static inline bool dfhip_aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Opt a kernel in to `bytes` of dynamic LDS.  The attribute belongs to the (function, device) pair, so `done`
// - one word per kernel instantiation - carries one bit per device; setting the attribute twice from two
// threads is harmless, reading a torn flag is not, hence the atomic.
static inline int dfhip_opt_in_lds(const void* kernel, int bytes, std::atomic<uint64_t>& done) {
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) return DFHIP_ERR_NO_DEVICE;
  const uint64_t bit = 1ull << (device & 63);
  if (done.load(std::memory_order_acquire) & bit) return DFHIP_OK;
  if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess)
    return DFHIP_ERR_LAUNCH;
  done.fetch_or(bit, std::memory_order_release);
  return DFHIP_OK;
}

static inline int dfhip_check_launch() {
  return hipGetLastError() == hipSuccess ? DFHIP_OK : DFHIP_ERR_LAUNCH;
}

// bf16 <-> fp32 on raw 16-bit storage
DFHIP_DEVICE float bf16_bits_to_f32(uint32_t bits16) { return __uint_as_float(bits16 << 16); }

// round-to-nearest-even fp32 -> bf16 (quiet NaN preserved)
DFHIP_DEVICE uint32_t f32_to_bf16_bits(float f) {
  bf16_t h = static_cast<bf16_t>(f);
  return static_cast<uint32_t>(__builtin_bit_cast(uint16_t, h));
}

// two values rounded and packed by one v_cvt_pk_bf16_f32 (same rounding as f32_to_bf16_bits, lo in bits 0..15)
DFHIP_DEVICE uint32_t pack2_bf16(float lo, float hi) {
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  const f32x2 v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}
// the two bf16 values of a packed pair, as fp32
DFHIP_DEVICE float bf16_lo_to_f32(uint32_t pair) { return __uint_as_float(pair << 16); }
DFHIP_DEVICE float bf16_hi_to_f32(uint32_t pair) { return __uint_as_float(pair & 0xffff0000u); }

// silu(g) = g / (1 + e^-g) on the hardware exponential and reciprocal (a few fp32 ulp; the bf16 paths
// round the result to 8 bits of mantissa right after).  -inf gives NaN like the exact quotient.
DFHIP_DEVICE float silu_fast(float g) {
  return g * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * g));
}

// 64-lane reductions through DPP-free shuffles (wave64)
DFHIP_DEVICE float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}
DFHIP_DEVICE float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

// The 8 XCDs of the chip take workgroups round-robin (workgroup i runs on XCD
// i % 8) and each XCD has a private L2.  remap_xcd turns the launch index into
// a tile index such that every XCD walks one contiguous range of tiles, so the
// tiles that are resident together on an XCD are neighbours and share operand
// rows/columns in that XCD's L2.  (Also compiled for the host: the mapping is
// replayed by CPU tests.)
__host__ __device__ __forceinline__ int remap_xcd(int pid, int total) {
  constexpr int XCDS = 8;
  const int xcd = pid % XCDS;
  const int local = pid / XCDS;
  const int base = total / XCDS;
  const int rem = total % XCDS;
  const int start = xcd * base + (xcd < rem ? xcd : rem);
  return start + local;
}

// Work item of a workgroup of the 256 x 256 split-K launch (`tiles` tiles, K of every tile cut into
// `split_k` parts): the launch is part-major - launch indices [p * tiles, (p + 1) * tiles) are part p of
// every tile, dealt to the XCDs like the tiles of an unsplit launch.  The last part of a tile, which waits
// for the others, therefore has the highest launch index of that tile for every tile count, and the parts
// it waits for were dispatched before it.
__host__ __device__ __forceinline__ void splitk_work_of(int pid, int tiles, int& tile, int& part) {
  part = pid / tiles;
  tile = remap_xcd(pid - part * tiles, tiles);
}

// ---- hand-ordered memory operations of the LDS-DMA GEMM kernels ------------------------------
// One LDS-DMA instruction: 64 lanes x 16 bytes from per-lane global addresses to
// LDS[lds_addr + 16*lane].  The compiler does not see the memory effect; ordering is kept by
// hand with wait_vmcnt / workgroup_barrier.
DFHIP_DEVICE void dma16(uint32_t lds_addr, const void* g) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_addr), "v"(g)
               : "memory", "m0");
}
// The same with a wave-uniform base (scalar registers) and a 32-bit per-lane byte offset.
DFHIP_DEVICE void dma16_base(uint32_t lds_addr, const void* base, uint32_t offset) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(offset), "s"(base)
               : "memory", "m0");
}
template <int N>
DFHIP_DEVICE void wait_vmcnt() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
DFHIP_DEVICE void workgroup_barrier() { asm volatile("s_barrier" ::: "memory"); }
#define DFHIP_PIN __builtin_amdgcn_sched_barrier(0)

// Calibration probe (not part of the library): the sustained MFMA throughput of this GPU with nothing
// but MFMA instructions on normally distributed operands, 256 workgroups x 4 waves, each wave on a
// 128 x 128 accumulator tile - the ceiling any GEMM kernel on the box works under once the package
// power limit sets the clock.  bf16 with both instruction shapes, and fp8 e4m3 (32x32x64, scales 2^0).  Build: make -C dynaflow_amd/csrc probes.  Run: probes/mfma_ceiling
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <math.h>
#include <vector>
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef int i32x8 __attribute__((ext_vector_type(8)));
#define CK(x) do{hipError_t e=(x); if(e!=hipSuccess){printf("HIP error %s line %d\n",hipGetErrorString(e),__LINE__); exit(1);} }while(0)
template<int KIND>
__global__ void __launch_bounds__(256) mfma_tile(const bf16x8* __restrict__ data, int iters, float* out){
  const int lane = threadIdx.x;
  if (KIND==0) {
    bf16x8 a[4], b[4];
    for (int i=0;i<4;++i){ a[i]=data[(i*256+lane)]; b[i]=data[((4+i)*256+lane)]; }
    f32x16 acc[4][4]; for(int i=0;i<4;++i) for(int j=0;j<4;++j) for(int r=0;r<16;++r) acc[i][j][r]=0.f;
    for(int it=0;it<iters;++it){
      #pragma unroll
      for(int i=0;i<4;++i)
      #pragma unroll
        for(int j=0;j<4;++j) acc[i][j]=__builtin_amdgcn_mfma_f32_32x32x16_bf16(b[j],a[i],acc[i][j],0,0,0);
    }
    float s=0; for(int i=0;i<4;++i) for(int j=0;j<4;++j) for(int r=0;r<16;++r) s+=acc[i][j][r];
    out[blockIdx.x*256+threadIdx.x]=s;
  } else if (KIND==2) {
    // fp8: a lane feeds 32 bytes per operand; the bf16 sample's bytes are re-read as e4m3 codes with the
    // exponent's top bit cleared (|value| < 2), which keeps every code finite
    i32x8 a[4], b[4];
    const int* words = reinterpret_cast<const int*>(data);
    for (int i=0;i<4;++i) for (int w=0;w<8;++w){ a[i][w]=words[(i*8+w)*256+lane] & 0xbfbfbfbf; b[i][w]=words[((4+i)*8+w)*256+lane] & 0xbfbfbfbf; }
    f32x16 acc[4][4]; for(int i=0;i<4;++i) for(int j=0;j<4;++j) for(int r=0;r<16;++r) acc[i][j][r]=0.f;
    for(int it=0;it<iters;++it){
      #pragma unroll
      for(int i=0;i<4;++i)
      #pragma unroll
        for(int j=0;j<4;++j) acc[i][j]=__builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(b[j],a[i],acc[i][j],0,0,0,0x7f7f7f7f,0,0x7f7f7f7f);
    }
    float s=0; for(int i=0;i<4;++i) for(int j=0;j<4;++j) for(int r=0;r<16;++r) s+=acc[i][j][r];
    out[blockIdx.x*256+threadIdx.x]=s;
  } else if (KIND==3) {
    // fp8 with the 16x16x128 shape: 8 x 8 blocks of 16 x 16, 32 bytes per lane and operand
    i32x8 a[8], b[8];
    const int* words = reinterpret_cast<const int*>(data);
    for (int i=0;i<8;++i) for (int w=0;w<8;++w){ a[i][w]=words[((i&3)*8+w)*256+lane] & 0xbfbfbfbf; b[i][w]=words[((4+(i&3))*8+w)*256+lane] & 0xbfbfbfbf; }
    f32x4 acc[8][8]; for(int i=0;i<8;++i) for(int j=0;j<8;++j) for(int r=0;r<4;++r) acc[i][j][r]=0.f;
    for(int it=0;it<iters;++it){
      #pragma unroll
      for(int i=0;i<8;++i)
      #pragma unroll
        for(int j=0;j<8;++j) acc[i][j]=__builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(b[j],a[i],acc[i][j],0,0,0,0x7f7f7f7f,0,0x7f7f7f7f);
    }
    float s=0; for(int i=0;i<8;++i) for(int j=0;j<8;++j) for(int r=0;r<4;++r) s+=acc[i][j][r];
    out[blockIdx.x*256+threadIdx.x]=s;
  } else {
    bf16x8 a[8], b[8];
    for (int i=0;i<8;++i){ a[i]=data[(i*256+lane)]; b[i]=data[((8+i)*256+lane)]; }
    f32x4 acc[8][8]; for(int i=0;i<8;++i) for(int j=0;j<8;++j) for(int r=0;r<4;++r) acc[i][j][r]=0.f;
    for(int it=0;it<iters;++it){
      #pragma unroll
      for(int i=0;i<8;++i)
      #pragma unroll
        for(int j=0;j<8;++j) acc[i][j]=__builtin_amdgcn_mfma_f32_16x16x32_bf16(b[j],a[i],acc[i][j],0,0,0);
    }
    float s=0; for(int i=0;i<8;++i) for(int j=0;j<8;++j) for(int r=0;r<4;++r) s+=acc[i][j][r];
    out[blockIdx.x*256+threadIdx.x]=s;
  }
}
static uint16_t f2bf(float f){ uint32_t u; memcpy(&u,&f,4); u += 0x7fff + ((u>>16)&1); return (uint16_t)(u>>16);}
int main(){
  std::vector<uint16_t> h(64*256*8); srand(1);
  for(auto& v:h){ float u1=(rand()+1.0f)/(RAND_MAX+2.0f), u2=(rand()+1.0f)/(RAND_MAX+2.0f); v=f2bf(sqrtf(-2*logf(u1))*cosf(6.2831853f*u2)*0.3f); }
  bf16x8* d; CK(hipMalloc(&d,h.size()*2)); CK(hipMemcpy(d,h.data(),h.size()*2,hipMemcpyHostToDevice));
  float* out; CK(hipMalloc(&out,256*256*4));
  hipEvent_t e0,e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
  // per iteration and wave, a 128 x 128 tile: 16 x 32768 flop (32x32x16) = 524288; 64 x 16384 (16x16x32) = 1048576;
  // 16 x 131072 (fp8 32x32x64) = 2097152
  for(int round=0; round<3; ++round) for(int kind=0; kind<4; ++kind){
    int iters = kind==0 ? 400000 : kind==3 ? 100000 : 200000;   // an fp8 instruction is 4x the flop of a bf16 one at twice the rate   // 256 WG x 4 waves x 4e5 x 524288 flop = 2.1e14 -> ~0.15 s at 1.4 PF; loop launches for ~3 s
    CK(hipEventRecord(e0));
    for(int rep=0; rep<20; ++rep){
      if(kind==0) hipLaunchKernelGGL((mfma_tile<0>),dim3(256),dim3(256),0,0,d,iters,out);
      else if(kind==1) hipLaunchKernelGGL((mfma_tile<1>),dim3(256),dim3(256),0,0,d,iters,out);
      else if(kind==2) hipLaunchKernelGGL((mfma_tile<2>),dim3(256),dim3(256),0,0,d,iters,out);
      else hipLaunchKernelGGL((mfma_tile<3>),dim3(256),dim3(256),0,0,d,iters,out);
    }
    CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1)); float ms; CK(hipEventElapsedTime(&ms,e0,e1));
    double flops=20.0*256*4*(double)iters*524288.0*(kind==3?8.0:kind==2?4.0:kind==1?2.0:1.0);
    printf("round %d %s: %.1f ms  %.1f TFLOP/s\n",round,kind==0?"bf16 32x32x16":kind==1?"bf16 16x16x32":kind==2?"fp8 32x32x64":"fp8 16x16x128",ms,flops/ms/1e9); fflush(stdout);
  }
  return 0;
}

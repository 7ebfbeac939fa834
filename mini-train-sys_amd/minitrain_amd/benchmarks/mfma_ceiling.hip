// What the matrix pipes of this GPU sustain with nothing else going on: a register-only loop of
// bf16 MFMAs (no LDS, no memory), one 256-thread block per SIMD pair, operands either constant
// or eight pseudo-random register sets rotated from instruction to instruction.  The chip is
// power-limited under MFMA load, and operands that toggle cost clock: this is the calibration
// the expert-GEMM figures are read against.
//
// build: hipcc -O3 --offload-arch=gfx950 -Xclang -target-feature -Xclang -packed-fp32-ops \
//              -Wno-unused-value -o mfma_ceiling.bin mfma_ceiling.hip
// run:   ./mfma_ceiling.bin
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdint.h>
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
__device__ __forceinline__ uint32_t rnd(uint32_t& s){ s = s*1664525u + 1013904223u; return s; }
// MODE 0: 32x32x16, MODE 1: 16x16x32.  TOGGLE: operands are NS different pseudo-random register sets, rotated every MFMA
template <int MODE, bool TOGGLE>
__global__ __launch_bounds__(256) void k(float* out, int iters){
  constexpr int NS = 8;
  bf16x8 a[NS], b[NS];
  uint32_t s = threadIdx.x*2654435761u + blockIdx.x*97u + 12345u;
  for (int n=0;n<NS;n++) for (int i=0;i<8;i++){
    float va = TOGGLE ? ((int)(rnd(s)>>8)%2001-1000)*0.001f : 0.5f;
    float vb = TOGGLE ? ((int)(rnd(s)>>8)%2001-1000)*0.00002f : 0.01f;
    a[n][i]=(__bf16)va; b[n][i]=(__bf16)vb; }
  float total = 0.f;
  if (MODE == 0) {
    f32x16 acc[8];
    for (int j=0;j<8;j++) for(int i=0;i<16;i++) acc[j][i]=0.f;
    for (int it=0; it<iters; it+=8){
#pragma unroll
      for (int r=0;r<8;r++)
#pragma unroll
      for (int j=0;j<8;j++) acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(j+3*r)&7],b[(j+r)&7],acc[j],0,0,0);
    }
    for (int j=0;j<8;j++) for(int i=0;i<16;i++) total+=acc[j][i];
  } else {
    f32x4 acc[16];
    for (int j=0;j<16;j++) for(int i=0;i<4;i++) acc[j][i]=0.f;
    for (int it=0; it<iters; it+=8){
#pragma unroll
      for (int r=0;r<8;r++)
#pragma unroll
      for (int j=0;j<16;j++) acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[(j+3*r)&7],b[(j+r)&7],acc[j],0,0,0);
    }
    for (int j=0;j<16;j++) for(int i=0;i<4;i++) total+=acc[j][i];
  }
  out[blockIdx.x*256+threadIdx.x]=total;
}
template <int MODE, bool TOGGLE> void run(const char* name, float* d){
  hipEvent_t e0,e1; hipEventCreate(&e0); hipEventCreate(&e1);
  int blocks = 512, iters = 20000;
  k<MODE,TOGGLE><<<blocks,256>>>(d, 2000); hipDeviceSynchronize();
  hipEventRecord(e0); k<MODE,TOGGLE><<<blocks,256>>>(d, iters); hipEventRecord(e1); hipEventSynchronize(e1);
  float ms; hipEventElapsedTime(&ms,e0,e1);
  double per_it = MODE == 0 ? 8*32768.0 : 16*16384.0;
  double flops = (double)blocks*4*iters*per_it;
  printf("%s: %.3f ms, %.1f TFLOP/s\n", name, ms, flops/ms/1e9); fflush(stdout);
}
int main(){
  float* d; hipMalloc(&d, 4096*256*4);
  for (int rep=0; rep<2; ++rep){
    run<0,false>("32x32x16 constant operands", d);
    run<0,true>("32x32x16 random operands  ", d);
    run<1,false>("16x16x32 constant operands", d);
    run<1,true>("16x16x32 random operands  ", d);
  }
  return 0;
}

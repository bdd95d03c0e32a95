// Diagnostic, not part of the library: sustained v_mfma_f32_32x32x16 rate on gfx950 with constant
// and with random N(0,1)-like operands, fp16 and bf16.  Random operands toggle more of the
// datapath, the package hits its power limit and the clock drops, so this is the MFMA ceiling a
// real workload can see.  Build: python -m flash_colreduce_amd.build --tools ; run: flash_colreduce_amd/mfma_rate
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
#include <vector>
#include <string.h>
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
#define CHECK(x) do{hipError_t e=(x); if(e!=hipSuccess){printf("err %s line %d\n",hipGetErrorString(e),__LINE__);exit(1);}}while(0)
template<int BF> __global__ __launch_bounds__(256) void k(const u32x4* in, float* out, int iters) {
  u32x4 a[8], b[8];
  for (int i=0;i<8;++i){ a[i]=in[(threadIdx.x*16+i)]; b[i]=in[(threadIdx.x*16+8+i)]; }
  f32x16 acc0={0}, acc1={0};
  for (int it=0; it<iters; ++it) {
#pragma unroll
    for (int i=0;i<8;++i) {
      if (BF) { acc0=__builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8,a[i]),__builtin_bit_cast(bf16x8,b[i]),acc0,0,0,0);
                acc1=__builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8,b[i]),__builtin_bit_cast(bf16x8,a[(i+1)&7]),acc1,0,0,0); }
      else { acc0=__builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8,a[i]),__builtin_bit_cast(f16x8,b[i]),acc0,0,0,0);
             acc1=__builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8,b[i]),__builtin_bit_cast(f16x8,a[(i+1)&7]),acc1,0,0,0); }
    }
    if ((it & 63) == 63) { for (int r=0;r<16;++r){acc0[r]*=1e-30f; acc1[r]*=1e-30f;} }
  }
  float s=0; for(int i=0;i<16;++i) s+=acc0[i]+acc1[i];
  if (s==12345.678f) out[threadIdx.x]=s;
}
static unsigned short f2h(float f){ _Float16 h=(_Float16)f; unsigned short u; memcpy(&u,&h,2); return u; }
static unsigned short f2bf(float f){ unsigned u; memcpy(&u,&f,4); return (unsigned short)((u+0x8000)>>16); }
int main(){
  int n=256*16*8; std::vector<unsigned short> h(n);
  u32x4* d; float* o; CHECK(hipMalloc(&d,n*2)); CHECK(hipMalloc(&o,4096));
  hipEvent_t e0,e1; CHECK(hipEventCreate(&e0)); CHECK(hipEventCreate(&e1));
  for (int mode=0; mode<4; ++mode) {
    bool bf = mode&1, rnd = mode&2;
    srand(1);
    for (int i=0;i<n;++i){ float v = rnd ? ( (rand()/(float)RAND_MAX + rand()/(float)RAND_MAX + rand()/(float)RAND_MAX -1.5f)*2.0f ) : 1.0f; h[i]= bf? f2bf(v): f2h(v); }
    CHECK(hipMemcpy(d,h.data(),n*2,hipMemcpyHostToDevice));
    for (int rep=0; rep<2; ++rep) {
      int iters = rep? 40000: 2000;
      CHECK(hipEventRecord(e0));
      if (bf) k<1><<<512,256>>>(d,o,iters); else k<0><<<512,256>>>(d,o,iters);
      CHECK(hipEventRecord(e1)); CHECK(hipEventSynchronize(e1));
      float ms; CHECK(hipEventElapsedTime(&ms,e0,e1));
      if (rep) printf("%s %s: %.2f ms  %.0f TFLOP/s\n", bf?"bf16":"f16 ", rnd?"random  ":"constant", ms, 512.0*4*iters*16*32768.0/(ms*1e-3)/1e12);
    }
  }
  return 0;
}

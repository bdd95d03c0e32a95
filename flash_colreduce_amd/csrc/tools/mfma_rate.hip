// Diagnostic, not part of the library: what MFMA rate gfx950 sustains under the package power limit.
//   1. back-to-back v_mfma_f32_32x32x16 and v_mfma_f32_16x16x32, fp16 and bf16, with constant and with
//      random N(0,1)-like operands (random operands toggle more of the datapath, the clock drops);
//   2. the column-reduction kernels' instruction mix without any memory traffic: per sub-step of 64
//      resident x 32 streamed rows at D = 128 the MFMAs of one sub-step next to one fma + exp2 + add per
//      score of the previous one, random operands, both MFMA shapes.
// Build: python -m flash_colreduce_amd.build --tools ; run: flash_colreduce_amd/mfma_rate
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
#include <vector>
#include <string.h>
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
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
template<int BF> __global__ __launch_bounds__(256) void k16(const u32x4* in, float* out, int iters) {
  u32x4 a[8], b[8];
  for (int i=0;i<8;++i){ a[i]=in[(threadIdx.x*16+i)]; b[i]=in[(threadIdx.x*16+8+i)]; }
  f32x4 acc0={0}, acc1={0}, acc2={0}, acc3={0};
  for (int it=0; it<iters; ++it) {
#pragma unroll
    for (int i=0;i<8;++i) {
      if (BF) {
        acc0=__builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8,a[i]),__builtin_bit_cast(bf16x8,b[i]),acc0,0,0,0);
        acc1=__builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8,b[i]),__builtin_bit_cast(bf16x8,a[(i+1)&7]),acc1,0,0,0);
        acc2=__builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8,a[i]),__builtin_bit_cast(bf16x8,a[(i+3)&7]),acc2,0,0,0);
        acc3=__builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8,b[i]),__builtin_bit_cast(bf16x8,b[(i+5)&7]),acc3,0,0,0);
      } else {
        acc0=__builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8,a[i]),__builtin_bit_cast(f16x8,b[i]),acc0,0,0,0);
        acc1=__builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8,b[i]),__builtin_bit_cast(f16x8,a[(i+1)&7]),acc1,0,0,0);
        acc2=__builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8,a[i]),__builtin_bit_cast(f16x8,a[(i+3)&7]),acc2,0,0,0);
        acc3=__builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8,b[i]),__builtin_bit_cast(f16x8,b[(i+5)&7]),acc3,0,0,0);
      }
    }
    if ((it & 63) == 63) { for (int r=0;r<4;++r){acc0[r]*=1e-30f; acc1[r]*=1e-30f; acc2[r]*=1e-30f; acc3[r]*=1e-30f;} }
  }
  float s=0; for(int i=0;i<4;++i) s+=acc0[i]+acc1[i]+acc2[i]+acc3[i];
  if (s==12345.678f) out[threadIdx.x]=s;
}
static unsigned short f2h(float f){ _Float16 h=(_Float16)f; unsigned short u; memcpy(&u,&h,2); return u; }
static unsigned short f2bf(float f){ unsigned u; memcpy(&u,&f,4); return (unsigned short)((u+0x8000)>>16); }
#define H8(x) __builtin_bit_cast(f16x8,(x))
// one "sub-step": 64 resident rows x 32 streamed rows x D=128, previous sub-step's 2048 scores go through fma,exp,add
template<int SHAPE, int VALU> __global__ __launch_bounds__(256,2) void mix(const u32x4* in, float* out, int iters, float scale2) {
  u32x4 res[16], f[8];
  for (int i=0;i<16;++i) res[i]=in[threadIdx.x*32+i];
  for (int i=0;i<8;++i) f[i]=in[threadIdx.x*32+16+i];
  float col[32]; for (int i=0;i<32;++i) col[i]=0;
  float prev[32]; for (int i=0;i<32;++i) prev[i]=0;
  for (int it=0; it<iters; ++it) {
    float cur[32];
    if (SHAPE==0) {
      f32x16 n0={0}, n1={0};
#pragma unroll
      for (int ks=0; ks<8; ++ks) { n0=__builtin_amdgcn_mfma_f32_32x32x16_f16(H8(res[ks]),H8(f[ks]),n0,0,0,0); n1=__builtin_amdgcn_mfma_f32_32x32x16_f16(H8(res[8+ks]),H8(f[ks]),n1,0,0,0); }
      for (int i=0;i<16;++i){cur[i]=n0[i]; cur[16+i]=n1[i];}
    } else {
      f32x4 n[8]; for (int i=0;i<8;++i) n[i]=(f32x4){0,0,0,0};
      if (SHAPE==1) {
#pragma unroll
      for (int ks=0; ks<4; ++ks)
#pragma unroll
        for (int kg=0; kg<4; ++kg)
#pragma unroll
          for (int qg=0; qg<2; ++qg)
            n[kg*2+qg]=__builtin_amdgcn_mfma_f32_16x16x32_f16(H8(res[kg*4+ks]),H8(f[qg*4+ks]),n[kg*2+qg],0,0,0);
      } else if (SHAPE==2) { // B (streamed) held fixed over 4 consecutive MFMAs
#pragma unroll
      for (int ks=0; ks<4; ++ks)
#pragma unroll
        for (int qg=0; qg<2; ++qg)
#pragma unroll
          for (int kg=0; kg<4; ++kg)
            n[kg*2+qg]=__builtin_amdgcn_mfma_f32_16x16x32_f16(H8(res[kg*4+ks]),H8(f[qg*4+ks]),n[kg*2+qg],0,0,0);
      } else if (SHAPE==3) { // operands swapped: streamed as A, resident as B
#pragma unroll
      for (int ks=0; ks<4; ++ks)
#pragma unroll
        for (int kg=0; kg<4; ++kg)
#pragma unroll
          for (int qg=0; qg<2; ++qg)
            n[kg*2+qg]=__builtin_amdgcn_mfma_f32_16x16x32_f16(H8(f[qg*4+ks]),H8(res[kg*4+ks]),n[kg*2+qg],0,0,0);
      } else { // SHAPE 4: k-steps innermost for pairs of tiles (2 chains of 4 back to back)
#pragma unroll
      for (int kg=0; kg<4; ++kg)
#pragma unroll
        for (int ks=0; ks<4; ++ks)
#pragma unroll
          for (int qg=0; qg<2; ++qg)
            n[kg*2+qg]=__builtin_amdgcn_mfma_f32_16x16x32_f16(H8(res[kg*4+ks]),H8(f[qg*4+ks]),n[kg*2+qg],0,0,0);
      }
      for (int i=0;i<8;++i) for (int r=0;r<4;++r) cur[i*4+r]=n[i][r];
    }
    if (VALU==1) {
#pragma unroll
      for (int i=0;i<32;++i) col[i]+=__builtin_amdgcn_exp2f(fmaf(prev[i],scale2,-3.0f));
    } else if (VALU==2) { // fma+exp, sum folded 4:1 (proxy for "adds done elsewhere")
#pragma unroll
      for (int i=0;i<32;i+=1) { float e=__builtin_amdgcn_exp2f(fmaf(prev[i],scale2,-3.0f)); if ((i&3)==0) col[i]+=e; else col[i]=e; }
    } else if (VALU==3) { // fma + max
#pragma unroll
      for (int i=0;i<32;++i) col[i]=fmaxf(col[i],fmaf(prev[i],scale2,-3.0f));
    } else if (VALU==4) { // exp + add only (no fma)
#pragma unroll
      for (int i=0;i<32;++i) col[i]+=__builtin_amdgcn_exp2f(prev[i]);
    } else {
#pragma unroll
      for (int i=0;i<32;++i) col[i]+=prev[i];
    }
    for (int i=0;i<32;++i) prev[i]=cur[i];
    // rotate streamed fragments so operands change like fresh data
    u32x4 t=f[0]; for (int i=0;i<7;++i) f[i]=f[i+1]; f[7]=t ^ (u32x4){1u,0u,0u,0u};
  }
  float s=0; for(int i=0;i<32;++i) s+=col[i]+prev[i];
  if (s==12345.678f) out[threadIdx.x]=s;
}
template<int S,int V> void run_mix(const char* name, const u32x4* d, float* o){
  hipEvent_t e0,e1; CHECK(hipEventCreate(&e0)); CHECK(hipEventCreate(&e1));
  mix<S,V><<<512,256>>>(d,o,500,0.1f); CHECK(hipDeviceSynchronize());
  int iters=20000;
  CHECK(hipEventRecord(e0)); mix<S,V><<<512,256>>>(d,o,iters,0.1f); CHECK(hipEventRecord(e1)); CHECK(hipEventSynchronize(e1));
  float ms; CHECK(hipEventElapsedTime(&ms,e0,e1));
  printf("%-34s %.2f ms  %.0f TFLOP/s\n", name, ms, 512.0*4*iters*16*32768.0/(ms*1e-3)/1e12);
}
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
      if (rep) printf("32x32x16 %s %s: %.2f ms  %.0f TFLOP/s\n", bf?"bf16":"f16 ", rnd?"random  ":"constant", ms, 512.0*4*iters*16*32768.0/(ms*1e-3)/1e12);
    }
    for (int rep=0; rep<2; ++rep) {
      int iters = rep? 40000: 2000;
      CHECK(hipEventRecord(e0));
      if (bf) k16<1><<<512,256>>>(d,o,iters); else k16<0><<<512,256>>>(d,o,iters);
      CHECK(hipEventRecord(e1)); CHECK(hipEventSynchronize(e1));
      float ms; CHECK(hipEventElapsedTime(&ms,e0,e1));
      if (rep) printf("16x16x32 %s %s: %.2f ms  %.0f TFLOP/s\n", bf?"bf16":"f16 ", rnd?"random  ":"constant", ms, 512.0*4*iters*32*16384.0/(ms*1e-3)/1e12);
    }
  }
  {
    int n2=256*32*8; std::vector<unsigned short> h2(n2);
    srand(1); for (int i=0;i<n2;++i){ float v=(rand()/(float)RAND_MAX + rand()/(float)RAND_MAX + rand()/(float)RAND_MAX -1.5f)*2.0f; h2[i]=f2h(v);}
    u32x4* d2; CHECK(hipMalloc(&d2,n2*2)); CHECK(hipMemcpy(d2,h2.data(),n2*2,hipMemcpyHostToDevice));
    run_mix<0,1>("mix 32x32x16 f16 + fma/exp2/add", d2,o);
    run_mix<2,1>("mix 16x16x32 f16 + fma/exp2/add", d2,o);
    run_mix<2,3>("mix 16x16x32 f16 + fma/max", d2,o);
    run_mix<2,0>("mix 16x16x32 f16 + add", d2,o);
  }
  return 0;
}

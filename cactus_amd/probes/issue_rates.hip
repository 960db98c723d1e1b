// Stand-alone probe (not part of the libraries): issue rate of the int8 MFMA forms and of a wave-wide fp32 FMA on
// the current GPU, from register-only loops of independent instructions.  bench.py runs it to report the measured
// matrix peak next to the datasheet peak; profiles/mfma_i8_and_valu_issue_rates.md holds one run's output.
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdint.h>
#define CK(x) do{hipError_t e=(x); if(e!=hipSuccess){printf("ERR %s line %d\n",hipGetErrorString(e),__LINE__); exit(1);} }while(0)
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x2 __attribute__((ext_vector_type(2)));
typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
// MODE 0: 4 independent 32x32x32 i8 accumulate chains; 1: 16x16x64 i8 x4 chains; 2: 32x32x16 i8 (legacy); 3: fma x64 independent; 4: wall clock
template<int MODE> __global__ __launch_bounds__(256) void k(int* out, int iters, long long* clk){
  i32x4 a={1+(int)threadIdx.x,2,3,4}, b={5,6,7,8};
  i32x16 c0={},c1={},c2={},c3={}; 
  typedef int i32x4v __attribute__((ext_vector_type(4)));
  i32x4v e0={},e1={},e2={},e3={};
  float f[32]; for(int i=0;i<32;i++) f[i]=i*0.5f+threadIdx.x;
  long long t0=wall_clock64(); long long s0=clock64();
  for(int it=0;it<iters;it++){
    if(MODE==0){ c0=__builtin_amdgcn_mfma_i32_32x32x32_i8(a,b,c0,0,0,0); c1=__builtin_amdgcn_mfma_i32_32x32x32_i8(a,b,c1,0,0,0); c2=__builtin_amdgcn_mfma_i32_32x32x32_i8(a,b,c2,0,0,0); c3=__builtin_amdgcn_mfma_i32_32x32x32_i8(a,b,c3,0,0,0);}
    if(MODE==1){ e0=__builtin_amdgcn_mfma_i32_16x16x64_i8(a,b,e0,0,0,0); e1=__builtin_amdgcn_mfma_i32_16x16x64_i8(a,b,e1,0,0,0); e2=__builtin_amdgcn_mfma_i32_16x16x64_i8(a,b,e2,0,0,0); e3=__builtin_amdgcn_mfma_i32_16x16x64_i8(a,b,e3,0,0,0);}
    if(MODE==2){ long la=((long)a[0]<<32)|a[1], lb=((long)b[0]<<32)|b[1]; c0=__builtin_amdgcn_mfma_i32_32x32x16_i8(la,lb,c0,0,0,0); c1=__builtin_amdgcn_mfma_i32_32x32x16_i8(la,lb,c1,0,0,0); c2=__builtin_amdgcn_mfma_i32_32x32x16_i8(la,lb,c2,0,0,0); c3=__builtin_amdgcn_mfma_i32_32x32x16_i8(la,lb,c3,0,0,0);}
    if(MODE==3){
      #pragma unroll
      for(int i=0;i<32;i++) f[i]=__builtin_fmaf(f[i],1.0001f,0.5f); }
  }
  long long s1=clock64(); long long t1=wall_clock64();
  int s=0; for(int i=0;i<16;i++) s+=c0[i]+c1[i]+c2[i]+c3[i]; for(int i=0;i<4;i++) s+=e0[i]+e1[i]+e2[i]+e3[i]; float fs=0; for(int i=0;i<32;i++) fs+=f[i];
  out[blockIdx.x*256+threadIdx.x]=s+(int)fs;
  if(blockIdx.x==0&&threadIdx.x==0){ clk[0]=s1-s0; clk[1]=t1-t0; }
}
int main(){
  int* out; CK(hipMalloc(&out,256*4096*4)); long long* clk; CK(hipMalloc(&clk,16)); long long h[2];
  hipEvent_t e0,e1; hipEventCreate(&e0); hipEventCreate(&e1);
  int wcr=0; hipDeviceGetAttribute(&wcr, hipDeviceAttributeWallClockRate, 0); printf("wall clock rate kHz %d\n",wcr);
  const int iters=20000;
  auto run=[&](const char* nm, auto kern, int wg_per_cu, double ops_per_instr, int instr_per_iter){
    int grid=256*wg_per_cu;
    hipLaunchKernelGGL(kern,dim3(grid),dim3(256),0,0,out,iters,clk); CK(hipDeviceSynchronize());
    hipEventRecord(e0); hipLaunchKernelGGL(kern,dim3(grid),dim3(256),0,0,out,iters,clk); hipEventRecord(e1); hipEventSynchronize(e1);
    float ms; hipEventElapsedTime(&ms,e0,e1); CK(hipMemcpy(h,clk,16,hipMemcpyDeviceToHost));
    double n_instr=(double)iters*instr_per_iter*wg_per_cu;   // per SIMD
    double ns_per=ms*1e6/n_instr; double total_ops=ops_per_instr*n_instr*1024; 
    printf("%-22s waves/simd %d: %8.3f ms  %6.2f ns/instr/SIMD  shader clk %lld wall ticks %lld -> %.1f clk/instr ; %8.1f Tops/s\n",nm,wg_per_cu,ms,ns_per,h[0],h[1],(double)h[0]/((double)iters*instr_per_iter*wg_per_cu), total_ops/(ms*1e-3)/1e12);
  };
  for(int w:{1,2,4}){
    run("mfma_i32_32x32x32_i8",k<0>,w,65536,4);
    run("mfma_i32_16x16x64_i8",k<1>,w,32768,4);
    run("mfma_i32_32x32x16_i8",k<2>,w,32768,4);
    run("v_fma_f32 x32",k<3>,w,64,32);
  }
}

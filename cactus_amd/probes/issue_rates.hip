// Stand-alone probe (not part of the libraries): issue rate of the int8 MFMA forms and of a wave-wide fp32 FMA on
// the current GPU, from register-only loops of independent instructions.  bench.py runs it to report the measured
// matrix peak next to the datasheet peak; profiles/mfma_i8_and_valu_issue_rates.md holds one run's output.
// The mixed modes answer how much vector work hides behind the matrix core: V fp32 FMAs after every MFMA in the same
// wave (the scaling epilogue of a block-quantized GEMM has this shape), and MFMA waves next to FMA-only waves on the
// same SIMD (a producer / consumer split).
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
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
// One wave: 4 x { MFMA ; V independent FMAs }, the order pinned with sched_group_barrier.  F16=1 uses the fp16 MFMA.
template<int V, int F16> __global__ __launch_bounds__(256) void mixed(int* out, int iters, long long* clk){
  i32x4 a={1+(int)threadIdx.x,2,3,4}, b={5,6,7,8};
  f16x8 ha, hb; for(int i=0;i<8;i++){ ha[i]=(_Float16)(i+threadIdx.x); hb[i]=(_Float16)(i*0.25f); }
  i32x16 c[4]={}; f32x16 d[4]={};
  float f[32]; for(int i=0;i<32;i++) f[i]=i*0.5f+threadIdx.x;
  long long t0=wall_clock64(); long long s0=clock64();
  for(int it=0;it<iters;it++){
    #pragma unroll
    for(int j=0;j<4;j++){
      if(F16) d[j]=__builtin_amdgcn_mfma_f32_32x32x16_f16(ha,hb,d[j],0,0,0); else c[j]=__builtin_amdgcn_mfma_i32_32x32x32_i8(a,b,c[j],0,0,0);
      #pragma unroll
      for(int i=0;i<V;i++) f[(j*V+i)%32]=__builtin_fmaf(f[(j*V+i)%32],1.0001f,0.5f);
      __builtin_amdgcn_sched_group_barrier(0x008,1,0);
      if(V>0) __builtin_amdgcn_sched_group_barrier(0x002,V,0);
    }
  }
  long long s1=clock64(); long long t1=wall_clock64();
  float s=0; for(int j=0;j<4;j++) for(int i=0;i<16;i++) s+=(float)c[j][i]+d[j][i]; for(int i=0;i<32;i++) s+=f[i];
  out[blockIdx.x*256+threadIdx.x]=(int)s;
  if(blockIdx.x==0&&threadIdx.x==0){ clk[0]=s1-s0; clk[1]=t1-t0; }
}
// Sibling waves: workgroups of 8 waves, two per SIMD (wave i runs on SIMD i % 4); waves 0-3 run MFMA only, waves 4-7 FMA
// only, `RATIO` FMAs for every MFMA of the sibling.  (Roles by workgroup would not do: consecutive workgroups go to
// different XCDs, so even and odd ones never meet on a CU.)
template<int RATIO> __global__ __launch_bounds__(512) void siblings(int* out, int iters, long long* clk){
  long long t0=wall_clock64(); long long s0=clock64();
  float s=0;
  if(threadIdx.x<256){
    i32x4 a={1+(int)threadIdx.x,2,3,4}, b={5,6,7,8}; i32x16 c[4]={};
    for(int it=0;it<iters;it++){
      #pragma unroll
      for(int j=0;j<4;j++) c[j]=__builtin_amdgcn_mfma_i32_32x32x32_i8(a,b,c[j],0,0,0);
    }
    for(int j=0;j<4;j++) for(int i=0;i<16;i++) s+=(float)c[j][i];
  } else {
    float f[32]; for(int i=0;i<32;i++) f[i]=i*0.5f+threadIdx.x;
    for(int it=0;it<iters;it++){
      #pragma unroll
      for(int i=0;i<4*RATIO;i++) f[i%32]=__builtin_fmaf(f[i%32],1.0001f,0.5f);
    }
    for(int i=0;i<32;i++) s+=f[i];
  }
  long long s1=clock64(); long long t1=wall_clock64();
  out[blockIdx.x*512+threadIdx.x]=(int)s;
  if(blockIdx.x==0&&(threadIdx.x&255)==0){ clk[threadIdx.x>>8]=s1-s0; clk[2+(threadIdx.x>>8)]=t1-t0; }
}
int main(){
  int* out; CK(hipMalloc(&out,256*4096*4)); long long* clk; CK(hipMalloc(&clk,32)); long long h[4];
  hipEvent_t e0,e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
  int wcr=0; CK(hipDeviceGetAttribute(&wcr, hipDeviceAttributeWallClockRate, 0)); printf("wall clock rate kHz %d\n",wcr);
  const int iters=20000;
  auto run=[&](const char* nm, auto kern, int wg_per_cu, double ops_per_instr, int instr_per_iter){
    int grid=256*wg_per_cu;
    hipLaunchKernelGGL(kern,dim3(grid),dim3(256),0,0,out,iters,clk); CK(hipDeviceSynchronize());
    CK(hipEventRecord(e0)); hipLaunchKernelGGL(kern,dim3(grid),dim3(256),0,0,out,iters,clk); CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
    float ms; CK(hipEventElapsedTime(&ms,e0,e1)); CK(hipMemcpy(h,clk,16,hipMemcpyDeviceToHost));
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
  // same wave: clocks per { MFMA + V FMAs } group per SIMD; alone an MFMA is 32 clocks and V FMAs are 4 V clocks
  // The whole launch is timed with events and turned into shader clocks with the clock rate the first wave saw
  // (its cycle counter over its 100 MHz wall clock).  A wave's own counter is no use with several waves per SIMD:
  // the oldest wave is served first and finishes in its uncontended time while the younger ones wait.
  auto run_mixed=[&](const char* nm, auto kern, int wg_per_cu, int v){
    int grid=256*wg_per_cu;
    hipLaunchKernelGGL(kern,dim3(grid),dim3(256),0,0,out,iters,clk); CK(hipDeviceSynchronize());
    CK(hipEventRecord(e0)); hipLaunchKernelGGL(kern,dim3(grid),dim3(256),0,0,out,iters,clk); CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
    float ms; CK(hipEventElapsedTime(&ms,e0,e1)); CK(hipMemcpy(h,clk,16,hipMemcpyDeviceToHost));
    double ghz=(double)h[0]/((double)h[1]*10.0);
    double groups_per_simd=(double)iters*4*wg_per_cu;
    double clk_per_group=ms*1e6*ghz/groups_per_simd;
    printf("%-14s MFMA + %2d FMA, waves/simd %d: %8.3f ms at %.2f GHz  %6.1f clk per group per SIMD (MFMA alone 32, FMAs alone %3d, sum %3d) -> matrix core busy %5.1f %%\n",
           nm,v,wg_per_cu,ms,ghz,clk_per_group,4*v,32+4*v,100.0*32/clk_per_group);
  };
  for(int w:{1,2,4}){
    run_mixed("same wave i8",mixed<0,0>,w,0); run_mixed("same wave i8",mixed<4,0>,w,4); run_mixed("same wave i8",mixed<8,0>,w,8);
    run_mixed("same wave i8",mixed<16,0>,w,16); run_mixed("same wave i8",mixed<32,0>,w,32);
  }
  for(int w:{1,2,4}){
    run_mixed("same wave f16",mixed<0,1>,w,0); run_mixed("same wave f16",mixed<8,1>,w,8); run_mixed("same wave f16",mixed<32,1>,w,32);
  }
  auto run_sib=[&](const char* nm, auto kern, int wg_per_cu, int ratio){
    int grid=256*wg_per_cu/2;
    hipLaunchKernelGGL(kern,dim3(grid),dim3(512),0,0,out,iters,clk); CK(hipDeviceSynchronize());
    CK(hipEventRecord(e0)); hipLaunchKernelGGL(kern,dim3(grid),dim3(512),0,0,out,iters,clk); CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
    float ms; CK(hipEventElapsedTime(&ms,e0,e1)); CK(hipMemcpy(h,clk,32,hipMemcpyDeviceToHost));
    double ghz=(double)h[0]/((double)h[2]*10.0);
    int pairs=wg_per_cu/2; double groups_per_simd=(double)iters*4*pairs;      // one group = 1 MFMA in one wave + `ratio` FMAs in its sibling
    double clk_per_group=ms*1e6*ghz/groups_per_simd;
    printf("%-14s 1 MFMA : %2d FMA, %d + %d waves/simd: %8.3f ms at %.2f GHz  %6.1f clk per group per SIMD (MFMA alone 32, FMAs alone %3d) -> matrix core busy %5.1f %%\n",
           nm,ratio,pairs,pairs,ms,ghz,clk_per_group,4*ratio,100.0*32/clk_per_group);
  };
  for(int w:{2,4}){ run_sib("sibling waves",siblings<4>,w,4); run_sib("sibling waves",siblings<8>,w,8); run_sib("sibling waves",siblings<16>,w,16); run_sib("sibling waves",siblings<32>,w,32); }
}

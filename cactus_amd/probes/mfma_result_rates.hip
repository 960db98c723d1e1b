// Measurement program: what the vector work behind an int8 MFMA costs on a gfx950 SIMD, registers only.
//   part 1: v_mfma_i32_32x32x32_i8 followed by the scaling the GEMM kernels do on its 16 results per lane - fp32 multiply-adds
//           that read the previous MFMA's result (the block-32 kernels' two operations per integer sum, with the second one as
//           v_fma_f32 or as v_fma_mix_f32 reading an fp16 scale) or 24-bit integer multiply-adds (the single-plane K-quant
//           kernel), against the same number of operations on registers the MFMA did not write;
//   part 2: the plain issue rate of v_fma_f32 and v_fma_mix_f32, alone and as dependent pairs.
// 1, 2 and 4 workgroups of 4 waves per CU = 1, 2, 4 waves per SIMD.  Times are per MFMA group (or instruction) and SIMD.
#include <hip/hip_runtime.h>
#include <stdio.h>
#define CK(x) do{hipError_t e=(x); if(e!=hipSuccess){printf("ERR %s line %d\n",hipGetErrorString(e),__LINE__); exit(1);} }while(0)
template<int MODE> __global__ __launch_bounds__(256) void k(float* out, int iters, long long* clk){
  float f[32]; for(int i=0;i<32;i++) f[i]=i*0.5f+threadIdx.x;
  float t[16];
  unsigned h = 0x3c003c00u + threadIdx.x;   // two halves ~1.0
  float dx = 1.0001f, ndx = 0.5f;
  long long s0=clock64();
  for(int it=0;it<iters;it++){
    if(MODE==0){
      #pragma unroll
      for(int i=0;i<32;i++) asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(f[i]) : "v"(dx), "v"(ndx));
    }
    if(MODE==1){
      #pragma unroll
      for(int i=0;i<32;i++) asm volatile("v_fma_mix_f32 %0, %0, %1, %2 op_sel_hi:[0,1,0]" : "+v"(f[i]) : "v"(h), "v"(ndx));
    }
    if(MODE==2){  // pairs: t = fma(f, dx, ndx); acc = fma_mix(t, h, acc), dependent back to back
      #pragma unroll
      for(int i=0;i<16;i++){
        asm volatile("v_fma_f32 %0, %1, %2, %3" : "=v"(t[i]) : "v"(f[16+i]), "v"(dx), "v"(ndx));
        asm volatile("v_fma_mix_f32 %0, %1, %2, %0 op_sel_hi:[0,1,0]" : "+v"(f[i]) : "v"(t[i]), "v"(h));
      }
    }
    if(MODE==3){  // same pairs, 16 t first then 16 acc (independent neighbours)
      #pragma unroll
      for(int i=0;i<16;i++) asm volatile("v_fma_f32 %0, %1, %2, %3" : "=v"(t[i]) : "v"(f[16+i]), "v"(dx), "v"(ndx));
      #pragma unroll
      for(int i=0;i<16;i++) asm volatile("v_fma_mix_f32 %0, %1, %2, %0 op_sel_hi:[0,1,0]" : "+v"(f[i]) : "v"(t[i]), "v"(h));
    }
    if(MODE==4){  // pairs with plain fma for the second op (scale already fp32)
      #pragma unroll
      for(int i=0;i<16;i++){
        asm volatile("v_fma_f32 %0, %1, %2, %3" : "=v"(t[i]) : "v"(f[16+i]), "v"(dx), "v"(ndx));
        asm volatile("v_fma_f32 %0, %1, %2, %0" : "+v"(f[i]) : "v"(t[i]), "v"(dx));
      }
    }
  }
  long long s1=clock64();
  float s=0; for(int i=0;i<32;i++) s+=f[i];
  out[blockIdx.x*256+threadIdx.x]=s;
  if(blockIdx.x==0&&threadIdx.x==0){ clk[0]=s1-s0; }
}
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x16 __attribute__((ext_vector_type(16)));
// MFMA + 32 vector ops per group; KIND 0: 32 independent fma, 1: 16 dependent pairs fma -> fma_mix reading the previous MFMA's result,
// 2: 16 fma (reading the MFMA result) then 16 fma_mix, 3: pairs with plain fma second
template<int KIND> __global__ __launch_bounds__(256) void grp(float* out, int iters, long long* clk){
  i32x4 a={1+(int)threadIdx.x,2,3,4}, b={5,6,7,8};
  i32x16 magic; for(int i=0;i<16;i++){ int m=0x4B400000; asm volatile("" : "+v"(m)); magic[i]=m; }
  float acc[4][16]; for(int j=0;j<4;j++) for(int i=0;i<16;i++) acc[j][i]=i+j;
  unsigned h = 0x3c003c00u + threadIdx.x; float dx=1.0001f, ndx=-12582912.f*1.0001f; asm volatile("" : "+v"(dx), "+v"(ndx), "+v"(h));
  i32x16 d_cur=__builtin_amdgcn_mfma_i32_32x32x32_i8(a,b,magic,0,0,0);
  long long s0=clock64();
  for(int it=0;it<iters;it++){
    #pragma unroll
    for(int j=0;j<4;j++){
      i32x16 d_next=__builtin_amdgcn_mfma_i32_32x32x32_i8(a,b,magic,0,0,0);
      __builtin_amdgcn_sched_barrier(0);
      if(KIND==0){
        #pragma unroll
        for(int i=0;i<16;i++){ asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(acc[j][i]) : "v"(dx), "v"(ndx)); asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(acc[(j+1)&3][i]) : "v"(dx), "v"(ndx)); }
      } else if(KIND==1){
        #pragma unroll
        for(int i=0;i<16;i++){ float t; asm volatile("v_fma_f32 %0, %1, %2, %3" : "=v"(t) : "v"(d_cur[i]), "v"(dx), "v"(ndx));
          asm volatile("v_fma_mix_f32 %0, %1, %2, %0 op_sel_hi:[0,1,0]" : "+v"(acc[j][i]) : "v"(t), "v"(h)); }
      } else if(KIND==2){
        float t[16];
        #pragma unroll
        for(int i=0;i<16;i++) asm volatile("v_fma_f32 %0, %1, %2, %3" : "=v"(t[i]) : "v"(d_cur[i]), "v"(dx), "v"(ndx));
        #pragma unroll
        for(int i=0;i<16;i++) asm volatile("v_fma_mix_f32 %0, %1, %2, %0 op_sel_hi:[0,1,0]" : "+v"(acc[j][i]) : "v"(t[i]), "v"(h));
      } else if(KIND==3) {
        float t[16];
        #pragma unroll
        for(int i=0;i<16;i++) asm volatile("v_fma_f32 %0, %1, %2, %3" : "=v"(t[i]) : "v"(d_cur[i]), "v"(dx), "v"(ndx));
        #pragma unroll
        for(int i=0;i<16;i++) asm volatile("v_fma_f32 %0, %1, %2, %0" : "+v"(acc[j][i]) : "v"(t[i]), "v"(dx));
      } else if(KIND==4) {
        #pragma unroll
        for(int i=0;i<16;i++) asm volatile("v_mad_i32_i24 %0, %1, %2, %0" : "+v"(acc[j][i]) : "v"(d_cur[i]), "v"(h));
      } else if(KIND==5) {
        #pragma unroll
        for(int i=0;i<16;i++) asm volatile("v_fma_f32 %0, %1, %2, %0" : "+v"(acc[j][i]) : "v"(d_cur[i]), "v"(dx));
      } else if(KIND==6) {
        #pragma unroll
        for(int i=0;i<16;i++) asm volatile("v_mad_i32_i24 %0, %1, %2, %0" : "+v"(acc[j][i]) : "v"(acc[(j+1)&3][i]), "v"(h));
      } else {
        #pragma unroll
        for(int i=0;i<16;i++) asm volatile("v_mad_u32_u24 %0, %1, %2, %0" : "+v"(acc[j][i]) : "v"(d_cur[i]), "v"(h));
      }
      d_cur=d_next;
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  long long s1=clock64();
  float s=0; for(int j=0;j<4;j++) for(int i=0;i<16;i++) s+=acc[j][i]; s+=d_cur[3];
  out[blockIdx.x*256+threadIdx.x]=s;
  if(blockIdx.x==0&&threadIdx.x==0){ clk[0]=s1-s0; }
}
template<int KIND> void rung(const char* name, int wg_per_cu){
  float* out; long long* clk; CK(hipMalloc(&out, 256*1024*4*8)); CK(hipMalloc(&clk,16));
  int iters=5000; int grid=256*wg_per_cu;
  grp<KIND><<<grid,256>>>(out,100,clk); CK(hipDeviceSynchronize());
  hipEvent_t e0,e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
  CK(hipEventRecord(e0)); grp<KIND><<<grid,256>>>(out,iters,clk); CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
  float ms; CK(hipEventElapsedTime(&ms,e0,e1)); long long c; CK(hipMemcpy(&c,clk,8,hipMemcpyDeviceToHost));
  double groups_per_simd = (double)iters*4*wg_per_cu;
  printf("%-52s waves/simd %d: %8.3f ms, %.1f ns per group per SIMD (%.1f clk at 2.4 GHz), wave 0 saw %.1f clk per group\n", name, wg_per_cu, ms, ms*1e6/groups_per_simd, ms*1e6/groups_per_simd*2.4, (double)c/iters/4);
  CK(hipFree(out)); CK(hipFree(clk));
}
template<int MODE> void run(const char* name, int wg_per_cu){
  float* out; long long* clk; CK(hipMalloc(&out, 256*1024*4*8)); CK(hipMalloc(&clk,16));
  int iters=20000; int grid=256*wg_per_cu;
  k<MODE><<<grid,256>>>(out,100,clk); CK(hipDeviceSynchronize());
  hipEvent_t e0,e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
  CK(hipEventRecord(e0)); k<MODE><<<grid,256>>>(out,iters,clk); CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
  float ms; CK(hipEventElapsedTime(&ms,e0,e1)); long long c; CK(hipMemcpy(&c,clk,8,hipMemcpyDeviceToHost));
  const double ns = ms * 1e6 / ((double)iters * 32.0 * wg_per_cu);   // per instruction and SIMD, from the kernel's duration
  printf("%-40s waves/simd %d: %8.3f ms, %.2f ns per instruction per SIMD (%.2f clk at 2.4 GHz); wave 0 saw %.2f clk between its own instructions\n",
         name, wg_per_cu, ms, ns, ns * 2.4, (double)c / iters / 32.0);
  CK(hipFree(out)); CK(hipFree(clk));
}
int main(){
  for(int w=1; w<=4; w*=2){ rung<0>("MFMA + 32 independent fma", w); rung<1>("MFMA + 16 dependent pairs fma->fma_mix on result", w); rung<2>("MFMA + 16 fma on result, then 16 fma_mix", w); rung<3>("MFMA + 16 fma on result, then 16 fma", w); rung<4>("MFMA + 16 mad_i32_i24 on result", w); rung<5>("MFMA + 16 fma on result", w); rung<6>("MFMA + 16 mad_i32_i24 on other regs", w); rung<7>("MFMA + 16 mad_u32_u24 on result", w); }

  for(int w=1; w<=4; w*=2){
    run<0>("v_fma_f32 x32", w); run<1>("v_fma_mix_f32 x32", w); run<2>("pairs fma -> fma_mix (dependent)", w); run<3>("16 fma then 16 fma_mix", w); run<4>("pairs fma -> fma (dependent)", w);
  }
}

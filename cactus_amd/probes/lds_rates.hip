// Stand-alone probe (not part of the libraries): LDS instruction rates per CU on the current GPU, from loops of LDS
// reads / writes with lanes at consecutive addresses, and what an LDS read between MFMAs costs a wave that has the SIMD to
// itself (the large-shape GEMM's situation).  profiles/lds_rates.md holds one run's output.
#include <hip/hip_runtime.h>
#include <cstdio>
#define CK(x) do{hipError_t e=(x); if(e!=hipSuccess){printf("ERR %s line %d\n",hipGetErrorString(e),__LINE__); exit(1);} }while(0)
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
template<int MODE> __global__ __launch_bounds__(256) void k(unsigned* out, int iters, long long* clk){
  extern __shared__ __align__(16) unsigned char lds[];
  const int tid=threadIdx.x;
  for(int i=tid;i<16384;i+=256) ((unsigned*)lds)[i]=i;
  __syncthreads();
  u32x4 acc={0,0,0,0};
  long long t0=wall_clock64(), s0=clock64();
  const u32x4* p=(const u32x4*)lds + (tid&63) + (tid>>6)*256;
  for(int it=0;it<iters;it++){
    #pragma unroll
    for(int j=0;j<8;j++){
      if(MODE==0){ u32x4 v=p[j*64]; acc+=v; }
      if(MODE==1){ u32x2 v=((const u32x2*)p)[j*64]; acc.x+=v.x; acc.y+=v.y; }
      if(MODE==2){ ((u32x4*)p)[j*64]=acc; }
      if(MODE==3){ ((u32x2*)p)[j*64]=u32x2{acc.x,acc.y}; }
      if(MODE==4){ ((unsigned*)p)[j*64]=acc.x; }
      if(MODE==5){ u32x4 v=p[j*64]; acc+=v; ((u32x4*)p)[(j^1)*64+2048]=acc; }
    }
    asm volatile("" ::: "memory");
  }
  long long s1=clock64(), t1=wall_clock64();
  out[blockIdx.x*256+tid]=acc.x+acc.y+acc.z+acc.w;
  if(blockIdx.x==0&&tid==0){clk[0]=s1-s0;clk[1]=t1-t0;}
}
// MODE 0: 16 MFMAs per step; 1: + 8 ds_read_b128 after MFMAs 8..15; 2: + a barrier every second step
template<int MODE> __global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1,1))) void m(float* out, int iters, long long* clk){
  extern __shared__ __align__(16) unsigned char lds[];
  const int tid=threadIdx.x, lane=tid&63;
  for(int i=tid;i<32768;i+=256) ((unsigned*)lds)[i]=0x3c003c00u;
  __syncthreads();
  f32x16 acc[4][4];
  for(int a=0;a<4;a++) for(int c=0;c<4;c++) for(int v=0;v<16;v++) acc[a][c][v]=0.f;
  f16x8 af[4], bf[4];
  for(int a=0;a<4;a++){ af[a]=*(const f16x8*)(lds+lane*16+a*2048); bf[a]=*(const f16x8*)(lds+65536+lane*16+a*2048); }
  long long t0=wall_clock64(), s0=clock64();
  for(int it=0;it<iters;it++){
    #pragma unroll
    for(int i=0;i<16;i++){
      const int a=i>>2,c=i&3;
      acc[a][c]=__builtin_amdgcn_mfma_f32_32x32x16_f16(af[a],bf[c],acc[a][c],0,0,0);
      if(MODE>=1){
        if(i>=8 && i<12) af[i-8]=*(const f16x8*)(lds+((it&7)*8192)+lane*16+(i-8)*2048);
        if(i>=12) bf[i-12]=*(const f16x8*)(lds+65536+((it&7)*8192)+lane*16+(i-12)*2048);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if(MODE>=2 && (it&1)) __syncthreads();
  }
  long long s1=clock64(), t1=wall_clock64();
  float s=0; for(int a=0;a<4;a++) for(int c=0;c<4;c++) for(int v=0;v<16;v++) s+=acc[a][c][v];
  out[blockIdx.x*256+tid]=s;
  if(blockIdx.x==0&&tid==0){clk[0]=s1-s0;clk[1]=t1-t0;}
}
int main(){
  unsigned* out; CK(hipMalloc(&out,1024*256*4)); long long* clk; CK(hipMalloc(&clk,16)); long long h[2];
  hipEvent_t e0,e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
  const int iters=20000;
  auto run=[&](const char* nm, auto kern, int wg_per_cu, int bytes_per_lane){
    int grid=256*wg_per_cu;
    hipLaunchKernelGGL(kern,dim3(grid),dim3(256),65536,0,out,iters,clk); CK(hipDeviceSynchronize());
    CK(hipEventRecord(e0)); hipLaunchKernelGGL(kern,dim3(grid),dim3(256),65536,0,out,iters,clk); CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
    float ms; CK(hipEventElapsedTime(&ms,e0,e1)); CK(hipMemcpy(h,clk,16,hipMemcpyDeviceToHost));
    double ghz=(double)h[0]/((double)h[1]*10.0);
    double bytes_per_cu=(double)iters*8*256*bytes_per_lane*wg_per_cu;
    printf("%-34s %d waves/CU: %.3f ms at %.2f GHz -> %6.1f B/clk/CU\n",nm,4*wg_per_cu,ms,ghz,bytes_per_cu/(ms*1e6*ghz));
  };
  for(int w:{1,2}){ run("ds_read_b128",k<0>,w,16); run("ds_read_b64",k<1>,w,8); run("ds_write_b128",k<2>,w,16); run("ds_write_b64",k<3>,w,8); run("ds_write_b32",k<4>,w,4); run("ds_read_b128 + ds_write_b128 (each)",k<5>,w,16); }
  const int mi=8192;
  auto runm=[&](const char* nm, auto kern, int grid){
    CK(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 131072));
    hipLaunchKernelGGL(kern,dim3(grid),dim3(256),131072,0,(float*)out,mi,clk); CK(hipDeviceSynchronize());
    CK(hipEventRecord(e0)); hipLaunchKernelGGL(kern,dim3(grid),dim3(256),131072,0,(float*)out,mi,clk); CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
    float ms; CK(hipEventElapsedTime(&ms,e0,e1)); CK(hipMemcpy(h,clk,16,hipMemcpyDeviceToHost));
    printf("%-34s %3d workgroups of 4 waves (one per SIMD): %.3f ms, %.2f GHz, %.1f clocks per MFMA\n",nm,grid,ms,(double)h[0]/((double)h[1]*10.0),(double)h[0]/(mi*16.0));
  };
  for(int grid:{32,256}){ runm("16 MFMA per step",m<0>,grid); runm("+ 8 ds_read_b128 per step",m<1>,grid); runm("+ a barrier every 32 MFMA",m<2>,grid); }
}

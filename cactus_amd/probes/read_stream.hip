// Stand-alone probe (not part of the libraries): what a kernel that only reads a matrix-sized buffer costs on the current
// GPU, i.e. the floor of one decode GEMV launch whatever its arithmetic.  Cold = every launch reads a different buffer
// (weights of the next layer), warm = the same buffer again.  Also the cost of an empty launch, and of a chain of reads
// in which the tail of each kernel prefetches the next buffer (the experiment behind "prefetching into the memory-side
// cache does not pay").  profiles/read_only_stream_floor.md holds one run's output.
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdint.h>
#include <stdlib.h>
#include <vector>
#define CK(x) do{hipError_t e=(x); if(e!=hipSuccess){printf("ERR %s line %d\n",hipGetErrorString(e),__LINE__); exit(1);} }while(0)
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// a wave reads 4 KB at a time (four 16-byte loads per lane in flight), waves stride over the buffer
__device__ __forceinline__ uint32_t stream_read(const uint8_t* __restrict__ p, size_t bytes, size_t wave, size_t nw, int lane){
  uint32_t acc=0; const size_t per_wave=4096;
  for(size_t base=wave*per_wave; base<bytes; base+=nw*per_wave){
    u32x4 v[4];
    #pragma unroll
    for(int j=0;j<4;j++) v[j]=*(const u32x4*)(p+base+j*1024+lane*16);
    #pragma unroll
    for(int j=0;j<4;j++) acc+=v[j].x^v[j].y^v[j].z^v[j].w;
  }
  return acc;
}
// the first G workgroups read `cur`; the other gridDim.x - G read `nxt` (the prefetch experiment)
__global__ __launch_bounds__(256) void k_read(const uint8_t* __restrict__ cur, size_t cur_bytes, const uint8_t* __restrict__ nxt, size_t nxt_bytes, int G, uint32_t* out){
  const int lane=threadIdx.x&63; uint32_t acc;
  if((int)blockIdx.x<G){ size_t wave=(size_t)blockIdx.x*4+(threadIdx.x>>6); acc=stream_read(cur,cur_bytes,wave,(size_t)G*4,lane); }
  else { size_t wave=(size_t)(blockIdx.x-G)*4+(threadIdx.x>>6); acc=stream_read(nxt,nxt_bytes,wave,(size_t)(gridDim.x-G)*4,lane); }
  if(acc==0x12345678) out[0]=acc;
}
__global__ void k_empty(uint32_t* out){ if(threadIdx.x==9999) out[0]=1; }

// How many bytes a wave keeps in flight: D loads of 16 bytes per lane and iteration (D KB per wave), and with AHEAD the next
// iteration's loads are requested before the current ones are consumed (a ring of one step, as the GEMV has it).
template<int D, bool AHEAD>
__global__ __launch_bounds__(256) void k_depth(const uint8_t* __restrict__ p, size_t bytes, uint32_t* out){
  const int lane=threadIdx.x&63; const size_t nw=(size_t)gridDim.x*4, wave=(size_t)blockIdx.x*4+(threadIdx.x>>6), per_wave=(size_t)D*1024;
  uint32_t acc=0; u32x4 v[D], w[D];
  size_t base=wave*per_wave;
  if(AHEAD && base<bytes){
    #pragma unroll
    for(int j=0;j<D;j++) v[j]=*(const u32x4*)(p+base+j*1024+lane*16);
  }
  for(; base<bytes; base+=nw*per_wave){
    if(AHEAD){
      const size_t nb=base+nw*per_wave<bytes? base+nw*per_wave: base;      // the last iteration re-reads its own chunk
      #pragma unroll
      for(int j=0;j<D;j++) w[j]=*(const u32x4*)(p+nb+j*1024+lane*16);
      #pragma unroll
      for(int j=0;j<D;j++) acc+=v[j].x^v[j].y^v[j].z^v[j].w;
      #pragma unroll
      for(int j=0;j<D;j++) v[j]=w[j];
    } else {
      #pragma unroll
      for(int j=0;j<D;j++) v[j]=*(const u32x4*)(p+base+j*1024+lane*16);
      #pragma unroll
      for(int j=0;j<D;j++) acc+=v[j].x^v[j].y^v[j].z^v[j].w;
    }
  }
  if(acc==0x12345678) out[0]=acc;
}

int main(){
  const size_t total=(size_t)6<<30; uint8_t* d; CK(hipMalloc(&d,total)); CK(hipMemset(d,1,total)); uint32_t* out; CK(hipMalloc(&out,64));
  hipEvent_t e0,e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
  auto elapsed=[&](auto fn,int reps){ fn(); CK(hipDeviceSynchronize()); CK(hipEventRecord(e0)); for(int i=0;i<reps;i++) fn(); CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1)); float ms; CK(hipEventElapsedTime(&ms,e0,e1)); return ms*1e3f/reps; };
  printf("empty kernel, back to back: %.2f us per launch\n", elapsed([&]{ hipLaunchKernelGGL(k_empty,dim3(256),dim3(256),0,0,out); },200));
  // the matrices of the Llama-3-8B Q4_K_M decode trace (wq+wk+wv, wo, gate+up, down, head) and the BASELINE single-kernel sizes
  struct Case { const char* what; double mb; };
  const Case cases[]={{"wo Q4_K 4096x4096 / config 1",9.47},{"wq+wk+wv",15.28},{"config 3 Q4_K 14336x4096",33.1},{"ffn_down Q6_K / config 2 Q8_0",48.2},
                      {"ffn_gate+ffn_up",66.2},{"output head Q6_K 128256x4096",431.5}};
  for(const Case& c: cases){
    size_t bytes=((size_t)(c.mb*1e6))/(1<<16)*(1<<16);
    float best_cold=1e9f,best_warm=1e9f; int best_g=0;
    for(int G:{512,1024,2048}){
      int idx=0; int copies=(int)(total/bytes); if(copies<2) copies=2;
      float cold=elapsed([&]{ hipLaunchKernelGGL(k_read,dim3(G),dim3(256),0,0,d+(size_t)(idx++%copies)*bytes,bytes,d,(size_t)0,G,out); }, copies<100?copies:100);
      float warm=elapsed([&]{ hipLaunchKernelGGL(k_read,dim3(G),dim3(256),0,0,d,bytes,d,(size_t)0,G,out); },50);
      if(cold<best_cold){best_cold=cold;best_g=G;} if(warm<best_warm) best_warm=warm;
    }
    printf("read %6.1f MB (%-30s): cold %7.2f us = %4.0f GB/s = %4.1f %% of 8 TB/s (best of 512/1024/2048 workgroups: %d)   warm %7.2f us = %5.0f GB/s\n",
           bytes/1e6,c.what,best_cold,bytes/best_cold/1e3,bytes/best_cold/1e3/80.0,best_g,best_warm,bytes/best_warm/1e3);
  }
  // bytes in flight: D KB per wave and iteration, plain or one iteration ahead, 2 / 4 / 8 workgroups of four waves per CU
  {
    const size_t bytes=((size_t)(48.2e6))/(1<<16)*(1<<16); const int copies=(int)(total/bytes);
    printf("48.2 MB cold, us per launch by KB per wave and iteration (plain | one iteration ahead), workgroups of 4 waves:\n");
    auto run=[&](auto kfn,int G){ int idx=0; return elapsed([&]{ hipLaunchKernelGGL(kfn,dim3(G),dim3(256),0,0,d+(size_t)(idx++%copies)*bytes,bytes,out); }, copies<100?copies:100); };
    for(int G:{512,1024,2048}){
      printf("  %4d workgroups: 1 KB %6.2f | %6.2f   2 KB %6.2f | %6.2f   4 KB %6.2f | %6.2f   8 KB %6.2f | %6.2f   16 KB %6.2f | %6.2f\n",G,
        run(k_depth<1,false>,G),run(k_depth<1,true>,G),run(k_depth<2,false>,G),run(k_depth<2,true>,G),run(k_depth<4,false>,G),run(k_depth<4,true>,G),
        run(k_depth<8,false>,G),run(k_depth<8,true>,G),run(k_depth<16,false>,G),run(k_depth<16,true>,G));
    }
  }
  // a chain of reads over rotating buffers, with P extra workgroups per kernel that already read the next buffer
  auto chain=[&](const char* name,std::vector<double> mbs,int G,int P){
    std::vector<size_t> sz,off; size_t o=0; int n=0;
    while(true){ size_t b=((size_t)(mbs[n%mbs.size()]*1e6))/(1<<16)*(1<<16); if(o+b>total) break; sz.push_back(b); off.push_back(o); o+=b; n++; }
    int N=(int)sz.size(); size_t sum=0; for(auto b:sz) sum+=b;
    auto pass=[&]{ for(int i=0;i<N;i++){ int j=(i+1)%N; hipLaunchKernelGGL(k_read,dim3(G+P),dim3(256),0,0,d+off[i],sz[i],d+off[j],P?sz[j]:(size_t)0,G,out);} };
    pass(); CK(hipDeviceSynchronize());
    CK(hipEventRecord(e0)); pass(); pass(); CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1)); float ms; CK(hipEventElapsedTime(&ms,e0,e1));
    printf("chain %-28s %4d reading + %4d prefetching workgroups: %7.2f us per kernel, %5.0f GB/s of useful bytes\n",name,G,P,ms*1e3/(2*N),2.0*sum/(ms*1e-3)/1e9);
  };
  for(int P:{0,256,1024}){
    chain("48 MB each",{48.2},1024,P);
    chain("one layer (15.3, 9.5, 66.2, 48.2)",{15.28,9.47,66.2,48.2},1024,P);
  }
  return 0;
}

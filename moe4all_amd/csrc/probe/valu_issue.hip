// Measurement aid: what one wavefront, and 2 or 4 wavefronts per SIMD, pay per instruction on gfx950 for the
// instruction mixes of the decode kernels: dependent and independent v_fma_f32, v_dot4_i32_i8 with six accumulators
// and as one chain, a dependent add fed by LDS broadcast reads, and 128-bit LDS reads with 8 / 32 / 64 active lanes.
// One workgroup of 64 .. 1024 threads; the figure is the span from the first wave's start to the last wave's end in
// ticks of s_memtime, divided by the instructions of one wave.  make -C moe4all_amd/csrc probes
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#define CK(x) do{hipError_t e_=(x); if(e_!=hipSuccess){printf("ERR %s: %s\n",#x,hipGetErrorString(e_)); exit(1);} }while(0)
__device__ __forceinline__ long long clk(){ return __builtin_readcyclecounter(); }   // s_memtime: shader clock
// 1: dependent fma chain
__global__ void k_fma_dep(float* out, long long* t, int n){ float a=out[threadIdx.x], b=1.0001f, acc=0.f; long long t0=clk();
  for(int i=0;i<n;i++){ 
#pragma unroll
    for(int k=0;k<32;k++) acc=__fmaf_rn(a,b,acc); }
  long long t1=clk(); out[threadIdx.x]=acc; if((threadIdx.x&63)==0&&blockIdx.x==0){t[threadIdx.x>>6]=t1-t0; atomicMin((unsigned long long*)&t[16],(unsigned long long)t0); atomicMax((unsigned long long*)&t[17],(unsigned long long)t1);} }
// 2: 4 independent fma chains
__global__ void k_fma_ind(float* out, long long* t, int n){ float a=out[threadIdx.x], b=1.0001f, c0=0,c1=0,c2=0,c3=0; long long t0=clk();
  for(int i=0;i<n;i++){
#pragma unroll
    for(int k=0;k<8;k++){ c0=__fmaf_rn(a,b,c0); c1=__fmaf_rn(a,b,c1); c2=__fmaf_rn(a,b,c2); c3=__fmaf_rn(a,b,c3);} }
  long long t1=clk(); out[threadIdx.x]=c0+c1+c2+c3; if((threadIdx.x&63)==0&&blockIdx.x==0){t[threadIdx.x>>6]=t1-t0; atomicMin((unsigned long long*)&t[16],(unsigned long long)t0); atomicMax((unsigned long long*)&t[17],(unsigned long long)t1);} }
// 3: dot4 with 6 independent accumulators
__global__ void k_dot(int* out, long long* t, int n){ int a=out[threadIdx.x], b=out[threadIdx.x+64]; int c[6]={0,0,0,0,0,0}; long long t0=clk();
  for(int i=0;i<n;i++){
#pragma unroll
    for(int k=0;k<5;k++){
#pragma unroll
      for(int q=0;q<6;q++) c[q]=__builtin_amdgcn_sdot4(a,b+q,c[q],false); } }
  long long t1=clk(); out[threadIdx.x]=c[0]+c[1]+c[2]+c[3]+c[4]+c[5]; if((threadIdx.x&63)==0&&blockIdx.x==0){t[threadIdx.x>>6]=t1-t0; atomicMin((unsigned long long*)&t[16],(unsigned long long)t0); atomicMax((unsigned long long*)&t[17],(unsigned long long)t1);} }
// 4: dependent dot4
__global__ void k_dot_dep(int* out, long long* t, int n){ int a=out[threadIdx.x], b=out[threadIdx.x+64]; int c=0; long long t0=clk();
  for(int i=0;i<n;i++){
#pragma unroll
    for(int k=0;k<32;k++) c=__builtin_amdgcn_sdot4(a,b,c,false); }
  long long t1=clk(); out[threadIdx.x]=c; if((threadIdx.x&63)==0&&blockIdx.x==0){t[threadIdx.x>>6]=t1-t0; atomicMin((unsigned long long*)&t[16],(unsigned long long)t0); atomicMax((unsigned long long*)&t[17],(unsigned long long)t1);} }
// 5: LDS b128 reads, strided like the chain kernel, lanes<active
__global__ void k_lds(float* out, long long* t, int n, int active, int stride){ __shared__ float s[16384]; for(int i=threadIdx.x;i<16384;i+=blockDim.x) s[i]=i; __syncthreads();
  float acc=0; long long t0=clk();
  if((int)(threadIdx.x&63)<active){ const float4* p=reinterpret_cast<const float4*>(s+(threadIdx.x&63)*stride);
    for(int i=0;i<n;i++){
#pragma unroll
      for(int k=0;k<16;k++){ float4 v=p[(i*16+k)&63]; acc+=v.x; } } }
  long long t1=clk(); out[threadIdx.x]=acc; if((threadIdx.x&63)==0&&blockIdx.x==0){t[threadIdx.x>>6]=t1-t0; atomicMin((unsigned long long*)&t[16],(unsigned long long)t0); atomicMax((unsigned long long*)&t[17],(unsigned long long)t1);} }
// 6: dependent add with LDS broadcast read
__global__ void k_addchain(float* out, long long* t, int n){ __shared__ float s[256]; s[threadIdx.x&255]=out[threadIdx.x]; __syncthreads(); float acc=0; long long t0=clk();
  for(int i=0;i<n;i++){
#pragma unroll
    for(int k=0;k<32;k++) acc=__fadd_rn(acc,s[(i*32+k)&255]); }
  long long t1=clk(); out[threadIdx.x]=acc; if((threadIdx.x&63)==0&&blockIdx.x==0){t[threadIdx.x>>6]=t1-t0; atomicMin((unsigned long long*)&t[16],(unsigned long long)t0); atomicMax((unsigned long long*)&t[17],(unsigned long long)t1);} }
int main(){ float* out; long long* t; CK(hipMalloc(&out,1<<20)); CK(hipMemset(out,0,1<<20)); CK(hipMalloc(&t,256));
  int cur_threads=64; auto rd=[&](){ long long h[18]; CK(hipDeviceSynchronize()); CK(hipMemcpy(h,t,144,hipMemcpyDeviceToHost)); long long mx=0; for(int w=0;w<cur_threads/64;w++) mx=h[w]>mx?h[w]:mx; double span=(double)(h[17]-h[16]); long long init[18]; for(int i=0;i<18;i++) init[i]=0; init[16]=0x7fffffffffffffffLL; CK(hipMemcpy(t,init,144,hipMemcpyHostToDevice)); return span; };
  { long long init[18]; for(int i=0;i<18;i++) init[i]=0; init[16]=0x7fffffffffffffffLL; CK(hipMemcpy(t,init,144,hipMemcpyHostToDevice)); }
  const int n=200;
  for(int threads: {64,256,512,1024}){ cur_threads=threads;
    hipLaunchKernelGGL(k_fma_dep,dim3(1),dim3(threads),0,0,out,t,n); double a=rd(); printf("threads %3d: dependent fma      %.2f clk/op\n",threads,a/(n*32));
    hipLaunchKernelGGL(k_fma_ind,dim3(1),dim3(threads),0,0,out,t,n); a=rd(); printf("threads %3d: 4 independent fma  %.2f clk/op\n",threads,a/(n*32));
    hipLaunchKernelGGL(k_dot,dim3(1),dim3(threads),0,0,(int*)out,t,n); a=rd(); printf("threads %3d: dot4 x6 independent %.2f clk/op\n",threads,a/(n*30));
    hipLaunchKernelGGL(k_dot_dep,dim3(1),dim3(threads),0,0,(int*)out,t,n); a=rd(); printf("threads %3d: dependent dot4     %.2f clk/op\n",threads,a/(n*32));
    hipLaunchKernelGGL(k_addchain,dim3(1),dim3(threads),0,0,out,t,n); a=rd(); printf("threads %3d: add chain from LDS  %.2f clk/op\n",threads,a/(n*32));
    for(int active: {8,32,64}) for(int stride: {260,4}){ hipLaunchKernelGGL(k_lds,dim3(1),dim3(threads),0,0,out,t,n,active,stride); a=rd(); printf("threads %3d: lds b128 active %2d stride %3d: %.2f clk/read\n",threads,active,stride,a/(n*16)); }
  }
  printf("(ticks of s_memtime per instruction of one wavefront: span of the whole workgroup / instructions per wavefront)\n");
  return 0; }

// Measurement aid: what it costs workgroups of one launch to hand a value to each other through global memory on
// gfx950.  Ping-pong between two workgroups (same XCD, different XCDs) for store / load flavours (sc1, sc0 sc1, sc0,
// atomics, nt sc1), and an all-to-all among the workgroups of a launch, whole grid or in 8 groups by blockIdx % 8
// (= one XCD each), every wait bounded by a spin limit.  make -C moe4all_amd/csrc probes
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#include <vector>
#define CK(x) do{hipError_t e=(x); if(e!=hipSuccess){printf("ERR %s: %s\n",#x,hipGetErrorString(e)); exit(1);} }while(0)
constexpr int kSpinLimit = 1 << 16;
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint32_t xcc_id(){ uint32_t v; asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(v)); return v & 0xF; }

// MODE: 0 = sc1 (agent scope) store + sc1 load; 1 = sc0 sc1 (system); 2 = sc0 only (group scope: bypasses nothing?) ; 3 = atomics
template<int MODE> __device__ __forceinline__ void pub(uint32_t* p, uint32_t v){
  if(MODE==0) asm volatile("global_store_dword %0, %1, off sc1" :: "v"(p), "v"(v) : "memory");
  else if(MODE==1) asm volatile("global_store_dword %0, %1, off sc0 sc1" :: "v"(p), "v"(v) : "memory");
  else if(MODE==2) asm volatile("global_store_dword %0, %1, off sc0" :: "v"(p), "v"(v) : "memory");
  else if(MODE==4) asm volatile("global_store_dword %0, %1, off nt sc1" :: "v"(p), "v"(v) : "memory");
  else __hip_atomic_exchange(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
template<int MODE> __device__ __forceinline__ uint32_t poll(const uint32_t* p){
  uint32_t v;
  if(MODE==0) asm volatile("global_load_dword %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(p) : "memory");
  else if(MODE==1) asm volatile("global_load_dword %0, %1, off sc0 sc1\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(p) : "memory");
  else if(MODE==2) asm volatile("global_load_dword %0, %1, off sc0\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(p) : "memory");
  else if(MODE==4) asm volatile("global_load_dword %0, %1, off nt sc1\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(p) : "memory");
  else v=__hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return v;
}
// ping-pong between block A and block B: A writes flag[0]=r, B waits for it and writes flag[64]=r, A waits ...
template<int MODE> __global__ void pingpong(uint32_t* flags, int a, int b, int rounds, uint32_t base, long long* out, uint32_t* err){
  if(threadIdx.x!=0) return;
  if((int)blockIdx.x!=a && (int)blockIdx.x!=b) return;
  const bool isA=(int)blockIdx.x==a;
  long long t0=wall_clock64();
  for(int r=1;r<=rounds;r++){
    const uint32_t ep=base+r;
    if(isA){ pub<MODE>(flags,ep); int s=0; while(poll<MODE>(flags+64)!=ep){ if(++s>kSpinLimit){ *err=1; return; } } }
    else { int s=0; while(poll<MODE>(flags)!=ep){ if(++s>kSpinLimit){ *err=1; return; } } pub<MODE>(flags+64,ep); }
  }
  long long t1=wall_clock64();
  if(isA){ out[0]=t1-t0; out[1]=xcc_id(); } else out[2]=xcc_id();
}
__global__ void xcc_map(uint32_t* out){ if(threadIdx.x==0) out[blockIdx.x]=xcc_id(); }

// all-to-all among `group` blocks: block publishes one dword record {ep}, wave 0 of every block polls all records of its group.
// groups: blocks with the same (blockIdx.x % ngroups) when by_mod, i.e. the same XCD if dispatch is round-robin.
template<int MODE> __global__ __launch_bounds__(256) void a2a(uint32_t* rec, int ngroups, int rounds, uint32_t base, uint32_t* err, long long* out){
  const int g=blockIdx.x%ngroups, m=blockIdx.x/ngroups, gsize=gridDim.x/ngroups;
  uint32_t* mine=rec+(size_t)g*1024;
  long long t0=wall_clock64();
  __shared__ int dead; if(threadIdx.x==0) dead=0; __syncthreads();
  for(int r=1;r<=rounds;r++){
    if(dead) break;
    const uint32_t ep=base+r;
    uint32_t* buf=mine+(ep&1)*512;
    if(threadIdx.x==0) pub<MODE>(buf+m,ep);
    if(threadIdx.x<64){
      int s=0; bool ok;
      do{ ok=true; for(int i=threadIdx.x;i<gsize;i+=64) if(poll<MODE>(buf+i)!=ep) ok=false; ok=__all(ok); if(++s>kSpinLimit){ if(threadIdx.x==0){*err=1; dead=1;} break; } }while(!ok);
    }
    __syncthreads();
  }
  long long t1=wall_clock64();
  if(blockIdx.x==0&&threadIdx.x==0) out[0]=t1-t0;
}

int main(){
  hipStream_t s; CK(hipStreamCreateWithFlags(&s,hipStreamNonBlocking));
  uint32_t* buf; CK(hipMalloc(&buf,1<<20)); CK(hipMemsetAsync(buf,0,1<<20,s)); CK(hipStreamSynchronize(s));
  long long* out=(long long*)(buf+65536); uint32_t* err; CK(hipMalloc(&err,256)); CK(hipMemsetAsync(err,0,256,s)); CK(hipStreamSynchronize(s)); uint32_t* flags=buf; uint32_t* map=buf+80000;
  hipLaunchKernelGGL(xcc_map,dim3(512),dim3(64),0,s,map); CK(hipStreamSynchronize(s));
  std::vector<uint32_t> hm(512); CK(hipMemcpy(hm.data(),map,2048,hipMemcpyDeviceToHost));
  printf("xcc of blocks 0..31:"); for(int i=0;i<32;i++) printf(" %u",hm[i]); printf("\n");
  int rr=0; for(int i=0;i<512;i++) if(hm[i]==(uint32_t)(i%8)) rr++; printf("blocks with xcc == id %% 8: %d of 512\n",rr);
  uint32_t base=0;
  auto pp=[&](auto kern,const char* name,int a,int b){ CK(hipMemsetAsync(buf,0,4096,s)); CK(hipMemsetAsync(err,0,4,s)); CK(hipStreamSynchronize(s)); const int rounds=2000;
    hipLaunchKernelGGL(kern,dim3(64),dim3(64),0,s,flags,a,b,rounds,base,out,err); CK(hipStreamSynchronize(s)); base+=rounds;
    long long h[3]; CK(hipMemcpy(h,out,24,hipMemcpyDeviceToHost)); uint32_t e; CK(hipMemcpy(&e,err,4,hipMemcpyDeviceToHost));
    printf("pingpong %-10s blocks %d(xcc %lld) <-> %d(xcc %lld): round trip %.0f ns%s\n",name,a,h[1],b,h[2],h[0]*10.0/rounds,e==1?"  (a wait ran into the spin limit)":""); };
  pp(pingpong<0>,"sc1",0,1); pp(pingpong<0>,"sc1",0,8); pp(pingpong<1>,"sc0sc1",0,1); pp(pingpong<1>,"sc0sc1",0,8);
  pp(pingpong<2>,"sc0",0,8); pp(pingpong<3>,"atomic",0,1); pp(pingpong<3>,"atomic",0,8); pp(pingpong<4>,"nt sc1",0,1); pp(pingpong<4>,"nt sc1",0,8);
  auto aa=[&](auto kern,const char* name,int nb,int ngroups){ CK(hipMemsetAsync(buf,0,65536,s)); CK(hipMemsetAsync(err,0,4,s)); CK(hipStreamSynchronize(s)); const int rounds=1000;
    hipLaunchKernelGGL(kern,dim3(nb),dim3(256),0,s,buf,ngroups,rounds,base,err,out); CK(hipStreamSynchronize(s)); base+=rounds;
    long long h; CK(hipMemcpy(&h,out,8,hipMemcpyDeviceToHost)); uint32_t e; CK(hipMemcpy(&e,err,4,hipMemcpyDeviceToHost));
    printf("all-to-all %-8s %d blocks in %d groups: %.0f ns per exchange%s\n",name,nb,ngroups,h*10.0/rounds,e==1?"  (a wait ran into the spin limit)":""); };
  aa(a2a<0>,"sc1",256,1); aa(a2a<0>,"sc1",256,8); aa(a2a<2>,"sc0",256,8); aa(a2a<3>,"atomic",256,1); aa(a2a<3>,"atomic",256,8); aa(a2a<1>,"sc0sc1",256,1);
  aa(a2a<0>,"sc1",128,1); aa(a2a<0>,"sc1",64,1);
  return 0;
}

// Measurement aid for the single-launch MoeFfn kernel (k_layer.hip): builds the kernel with its phase time stamps
// switched on, runs it on random banks of the config-2 layer shape (hidden 2048, 128 experts, top-8, intermediate 768,
// Q4_K gate/up, Q6_K down) and prints, per phase boundary, the minimum / median / maximum over the 256 workgroups of
// the time since the first workgroup started.  make -C moe4all_amd/csrc probes; ./moe4all_amd/csrc/probe/layer_phases
#define INFR_LAYER_TRACE 1
#include "../k_layer.hip"
#include <cstdio>
#include <cstdlib>
#include <vector>
#include <algorithm>
namespace infr { thread_local const LaunchTiming* tl_launch_timing = nullptr; }
#define CK(x) do{hipError_t e_=(x); if(e_!=hipSuccess){printf("ERR %s: %s\n",#x,hipGetErrorString(e_)); exit(1);} }while(0)
int main(){
  const int ne=2048,nff=768,E=128,K=8;
  hipStream_t s; CK(hipStreamCreateWithFlags(&s,hipStreamNonBlocking));
  const size_t gate_b=(size_t)E*nff*(ne/256)*144, down_b=(size_t)E*ne*(nff/256)*210;
  uint8_t *gate,*up,*down; float *router,*x,*dst,*logits; int32_t* ids; float* w; long long* trace; char* ws; uint32_t* fault;
  CK(hipMalloc(&gate,gate_b)); CK(hipMalloc(&up,gate_b)); CK(hipMalloc(&down,down_b));
  CK(hipMalloc(&router,(size_t)E*ne*4)); CK(hipMalloc(&x,ne*4)); CK(hipMalloc(&dst,ne*4)); CK(hipMalloc(&logits,E*4));
  CK(hipMalloc(&ids,64*4)); CK(hipMalloc(&w,64*4)); CK(hipMalloc(&trace,256*16*8)); CK(hipMemset(trace,0,256*16*8));
  const size_t wsb=infr::moe_layer_workspace_bytes(ne,nff,E); CK(hipMalloc(&ws,wsb)); CK(hipMemset(ws,0,wsb));
  CK(hipHostMalloc(&fault,64,hipHostMallocMapped)); *fault=0; uint32_t* fdev; CK(hipHostGetDevicePointer((void**)&fdev,fault,0));
  // weights: random bytes with tame f16 scales; router/x random floats
  { std::vector<uint8_t> h(gate_b); for(size_t i=0;i<gate_b;i++) h[i]=(uint8_t)(i*2654435761u>>13); for(size_t b=0;b<gate_b/144;b++){ h[b*144]=0x66;h[b*144+1]=0x0e;h[b*144+2]=0x66;h[b*144+3]=0x0e; }
    CK(hipMemcpy(gate,h.data(),gate_b,hipMemcpyHostToDevice)); CK(hipMemcpy(up,h.data(),gate_b,hipMemcpyHostToDevice)); }
  { std::vector<uint8_t> h(down_b); for(size_t i=0;i<down_b;i++) h[i]=(uint8_t)(i*2246822519u>>11); for(size_t b=0;b<down_b/210;b++){ h[b*210+208]=0x66;h[b*210+209]=0x0e; }
    CK(hipMemcpy(down,h.data(),down_b,hipMemcpyHostToDevice)); }
  { std::vector<float> h((size_t)E*ne); unsigned r=1; for(auto& v:h){ r=r*1664525u+1013904223u; v=((r>>8)/16777216.0f-0.5f)*0.1f; } CK(hipMemcpy(router,h.data(),h.size()*4,hipMemcpyHostToDevice));
    CK(hipMemcpy(x,h.data()+777,ne*4,hipMemcpyHostToDevice)); }
  infr::MoeLayerParams q{};
  q.g.x=x; q.g.ids=ids; q.g.weights=w; q.g.gate=gate; q.g.gate_stride=gate_b/E; q.g.up=up; q.g.up_stride=gate_b/E; q.g.down=down; q.g.down_stride=down_b/E;
  q.g.gate_dt=q.g.up_dt=INFR_Q4K; q.g.down_dt=INFR_Q6K; q.g.rows=1; q.g.ne=ne; q.g.nff=nff; q.g.n_used=K; q.g.n_expert=E; q.g.act=0; q.g.dst=dst; q.g.n_cu=256;
  q.g.route.n_expert=E; q.g.route.n_used=K; q.g.route.rows=1; q.g.route.gating=0; q.g.route.norm_w=1; q.g.route.scale=1.0f; q.g.route.ids=ids; q.g.route.weights=w;
  q.router=router; q.router_row_floats=ne; q.router_x=x; q.logits_out=logits;
  q.seq=(uint32_t*)ws; q.cnt=(uint32_t*)(ws+16); q.xl=(uint64_t*)(ws+256); q.xh=q.xl+(size_t)8*E; q.ypart=q.xh+(size_t)8*nff; q.fault=fdev; q.spin_limit=1<<15;
  if(!infr::moe_layer_fused_supported(q)){ printf("unsupported\n"); return 1; }
  for(int i=0;i<20;i++) infr::launch_moe_layer_fused(s,q);
  CK(hipStreamSynchronize(s));
  hipEvent_t a,b; CK(hipEventCreate(&a)); CK(hipEventCreate(&b));
  CK(hipEventRecord(a,s)); for(int i=0;i<200;i++) infr::launch_moe_layer_fused(s,q); CK(hipEventRecord(b,s)); CK(hipStreamSynchronize(s));
  float ms; CK(hipEventElapsedTime(&ms,a,b)); printf("launches without time stamps: %.2f us per launch, fault %u\n",ms*1000/200,*fault);
  q.g.y=(float*)trace;
  for(int i=0;i<3;i++){ CK(hipMemsetAsync(trace,0,256*16*8,s)); infr::launch_moe_layer_fused(s,q); }
  CK(hipStreamSynchronize(s));
  std::vector<long long> t(256*16); CK(hipMemcpy(t.data(),trace,t.size()*8,hipMemcpyDeviceToHost));
  long long t0=t[0]; for(int b2=0;b2<256;b2++) if(t[b2*16]) t0=std::min(t0,t[b2*16]);
  printf("time stamps in us after the earliest workgroup start (wall clock, 100 MHz): min / median / max over the workgroups that pass the point\n"
         "  0 start | 1 router rows and x staged | 2 logits published | 3 barrier | 4 logits gathered | 5 routed | 6 gate/up done, h published\n"
         "  7 h gathered | 8 h as cells | 9 down rows done | 10 partial published, slice counter bumped | 11 slice summed (last arriver only)\n");
  for(int i=0;i<12;i++){ std::vector<double> v; for(int b2=0;b2<256;b2++) if(t[b2*16+i]) v.push_back((t[b2*16+i]-t0)*0.01); if(v.empty()){printf("  %2d: -\n",i);continue;} std::sort(v.begin(),v.end()); printf("  %2d: %6.2f %6.2f %6.2f  (n=%zu)\n",i,v.front(),v[v.size()/2],v.back(),v.size()); }
  for(int b2: {0,9}){ printf("block %d:",b2); for(int i=0;i<12;i++) if(t[b2*16+i]) printf(" %.2f",(t[b2*16+i]-t0)*0.01); printf("\n"); }
  return 0;
}

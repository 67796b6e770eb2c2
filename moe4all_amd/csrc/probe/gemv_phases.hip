// Measurement aid for the three launches of the per-token MoeFfn path (router logits of k_route.hip; routing + gate/up
// and down + weighted sum of k_gemv.hip): builds them with their time stamps switched on, runs one token row (or a few)
// of a layer shape on random banks and prints, per phase boundary, the minimum / median / maximum over the workgroups of
// the time since the first workgroup started.  The expert kernels cycle through eight sets of logits that select
// disjoint experts, so their weights come from HBM as they do in a model with many layers.
// make -C moe4all_amd/csrc probes; ./moe4all_amd/csrc/probe/gemv_phases [c5|c2|c1] [rows]
#define INFR_GEMV_TRACE 1
#include "../k_gemv.hip"
#include "../k_route.hip"
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>
namespace infr {
thread_local const LaunchTiming* tl_launch_timing = nullptr;
// the other translation units' entry points k_gemv.hip falls back to for shapes this probe never uses
bool linear_units_supported(int, int, const void*) { return false; }
void launch_linear_units(hipStream_t, const float*, const uint8_t*, int, size_t, int, int, int, float*, const float*) {}
bool linear_float_supported(int, int, size_t, const void*, const void*) { return false; }
void launch_linear_float(hipStream_t, const float*, const uint8_t*, int, size_t, int, int, int, float*, const float*) {}
bool moe_gate_up_units_supported(const MoeGemvParams&) { return false; }
void launch_moe_gate_up_units(hipStream_t, const MoeGemvParams&) {}
}
#define CK(x) do{hipError_t e_=(x); if(e_!=hipSuccess){printf("ERR %s: %s\n",#x,hipGetErrorString(e_)); exit(1);} }while(0)

static void report(const char* name, const std::vector<long long>& t, int blocks, const std::vector<int>& order, const char* legend) {
  long long t0 = 0;
  for (int b = 0; b < blocks; b++) if (t[b * 16]) t0 = t0 ? std::min(t0, t[b * 16]) : t[b * 16];
  printf("%s: time stamps in us after the earliest workgroup start, min / median / max over %d workgroups\n  %s\n", name, blocks, legend);
  for (int i : order) {
    std::vector<double> v;
    for (int b = 0; b < blocks; b++) if (t[b * 16 + i]) v.push_back((t[b * 16 + i] - t0) * 0.01);
    if (v.empty()) { printf("  %d: -\n", i); continue; }
    std::sort(v.begin(), v.end());
    printf("  %d: %6.2f %6.2f %6.2f  (n=%zu)\n", i, v.front(), v[v.size() / 2], v.back(), v.size());
  }
}

int main(int argc, char** argv) {
  const char* shape = argc > 1 ? argv[1] : "c5";
  const int rows = argc > 2 ? atoi(argv[2]) : 1;
  const int kSets = 8;
  int ne = 4096, nff = 1536, E = 256, K = 8, gdt = INFR_Q4K, ddt = INFR_Q6K; bool shared = true;
  if (!strcmp(shape, "c2")) { ne = 2048; nff = 768; E = 128; shared = false; }
  if (!strcmp(shape, "c1")) { ne = 2048; nff = 768; E = 128; shared = false; gdt = ddt = INFR_Q8_0; }
  auto row_bytes = [](int dt, int n) { return dt == INFR_Q4K ? (size_t)n / 256 * 144 : dt == INFR_Q6K ? (size_t)n / 256 * 210 : (size_t)n / 32 * 34; };
  auto blk = [](int dt) { return dt == INFR_Q4K ? 144 : dt == INFR_Q6K ? 210 : 34; };
  hipStream_t s; CK(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
  const size_t gate_b = (size_t)E * nff * row_bytes(gdt, ne), down_b = (size_t)E * ne * row_bytes(ddt, nff);
  const size_t sg_b = (size_t)nff * row_bytes(gdt, ne), sd_b = (size_t)ne * row_bytes(ddt, nff);
  uint8_t *gate, *up, *down, *sgate, *sup, *sdown; float *x, *h, *dst, *logits, *w, *probs; int32_t* ids; long long* trace;
  CK(hipMalloc(&gate, gate_b + 64)); CK(hipMalloc(&up, gate_b + 64)); CK(hipMalloc(&down, down_b + 64));
  CK(hipMalloc(&sgate, sg_b + 64)); CK(hipMalloc(&sup, sg_b + 64)); CK(hipMalloc(&sdown, sd_b + 64));
  CK(hipMalloc(&x, (size_t)rows * ne * 4)); CK(hipMalloc(&h, (size_t)rows * (K + 1) * nff * 4)); CK(hipMalloc(&dst, (size_t)rows * ne * 4));
  CK(hipMalloc(&logits, (size_t)kSets * rows * E * 4)); CK(hipMalloc(&w, rows * 64 * 4)); CK(hipMalloc(&probs, (size_t)rows * E * 4)); CK(hipMalloc(&ids, rows * 64 * 4));
  const int max_blocks = 8192; CK(hipMalloc(&trace, (size_t)max_blocks * 128));
  auto fill = [&](uint8_t* d, size_t n, int dt, unsigned mul) {   // random codes, tame f16 scales
    std::vector<uint8_t> v(n); for (size_t i = 0; i < n; i++) v[i] = (uint8_t)(i * mul >> 13);
    const int bb = blk(dt);
    for (size_t b = 0; b < n / bb; b++) {
      if (dt == INFR_Q4K) { v[b * bb] = 0x66; v[b * bb + 1] = 0x0e; v[b * bb + 2] = 0x66; v[b * bb + 3] = 0x0e; }
      else if (dt == INFR_Q6K) { v[b * bb + 208] = 0x66; v[b * bb + 209] = 0x0e; }
      else { v[b * bb] = 0x66; v[b * bb + 1] = 0x0e; }
    }
    CK(hipMemcpy(d, v.data(), n, hipMemcpyHostToDevice));
  };
  fill(gate, gate_b, gdt, 2654435761u); fill(up, gate_b, gdt, 2246822519u); fill(down, down_b, ddt, 3266489917u);
  fill(sgate, sg_b, gdt, 668265263u); fill(sup, sg_b, gdt, 374761393u); fill(sdown, sd_b, ddt, 2654435761u);
  { std::vector<float> v((size_t)rows * std::max(ne, (K + 1) * nff)); unsigned r = 1; for (auto& q : v) { r = r * 1664525u + 1013904223u; q = ((r >> 8) / 16777216.0f - 0.5f); }
    CK(hipMemcpy(x, v.data(), (size_t)rows * ne * 4, hipMemcpyHostToDevice)); CK(hipMemcpy(h, v.data(), (size_t)rows * (K + 1) * nff * 4, hipMemcpyHostToDevice));
    // kSets sets of logits that pick disjoint experts: launches that cycle through them find their weights in HBM, not in a cache
    std::vector<float> l((size_t)kSets * rows * E); for (auto& q : l) { r = r * 1664525u + 1013904223u; q = ((r >> 8) / 16777216.0f - 0.5f) * 4.0f; }
    for (int j = 0; j < kSets; j++) for (int rr = 0; rr < rows; rr++) for (int k = 0; k < K; k++) l[((size_t)j * rows + rr) * E + ((j * rows + rr) * K + k) % E] += 8.0f + 0.1f * k;
    CK(hipMemcpy(logits, l.data(), l.size() * 4, hipMemcpyHostToDevice)); }
  int n_cu = 0; CK(hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, 0));
  infr::MoeGemvParams p{};
  p.x = x; p.ids = ids; p.weights = w; p.gate = gate; p.gate_stride = gate_b / E; p.up = up; p.up_stride = gate_b / E; p.down = down; p.down_stride = down_b / E;
  p.gate_dt = p.up_dt = gdt; p.down_dt = ddt; p.rows = rows; p.ne = ne; p.nff = nff; p.n_used = K; p.n_expert = E; p.act = 0; p.h = h; p.dst = dst; p.n_cu = n_cu;
  if (shared) { p.sh_gate = sgate; p.sh_up = sup; p.sh_down = sdown; }
  p.route_inline = infr::moe_gate_up_routes_inline(p) ? 1 : 0;
  p.route.logits = logits; p.route.n_expert = E; p.route.n_used = K; p.route.rows = rows; p.route.gating = 0; p.route.norm_w = 1; p.route.scale = 1.0f;
  p.route.ids = ids; p.route.weights = w; p.route.probs = probs;
  printf("%s: hidden %d, intermediate %d, %d experts, top-%d%s, %d row(s); routing %s\n", shape, ne, nff, E, K, shared ? " + shared expert" : "", rows,
         p.route_inline ? "inside the gate/up kernel" : "as a launch of its own");
  if (!p.route_inline) infr::launch_route(s, p.route);
  hipEvent_t a, b; CK(hipEventCreate(&a)); CK(hipEventCreate(&b));
  {   // the logits kernel on a router of its own (f32 [E, ne]), the token row normalised on the way as in the layer
    float *router, *nw, *xn; CK(hipMalloc(&router, (size_t)E * ne * 4)); CK(hipMalloc(&nw, ne * 4)); CK(hipMalloc(&xn, (size_t)rows * ne * 4));
    { std::vector<float> v((size_t)E * ne); unsigned r = 7; for (auto& q : v) { r = r * 1664525u + 1013904223u; q = ((r >> 8) / 16777216.0f - 0.5f) * 0.05f; }
      CK(hipMemcpy(router, v.data(), v.size() * 4, hipMemcpyHostToDevice)); std::vector<float> o(ne, 1.0f); CK(hipMemcpy(nw, o.data(), ne * 4, hipMemcpyHostToDevice)); }
    infr::RouterNorm nrm{}; if (rows == 1) { nrm.weight = nw; nrm.xn_out = xn; nrm.eps = 1e-6f; }
    float* lg; CK(hipMalloc(&lg, (size_t)rows * E * 4));
    auto launch = [&]() { infr::launch_router_logits(s, reinterpret_cast<const uint8_t*>(router), INFR_F32, (size_t)ne * 4, x, ne, E, rows, lg, rows == 1 ? &nrm : nullptr); };
    for (int i = 0; i < 5; i++) launch();
    CK(hipStreamSynchronize(s));
    CK(hipEventRecord(a, s)); for (int i = 0; i < 50; i++) launch(); CK(hipEventRecord(b, s)); CK(hipStreamSynchronize(s));
    float ms; CK(hipEventElapsedTime(&ms, a, b));
    printf("router logits: %.2f us per launch without time stamps (the same router every launch: it stays in the caches)\n", ms * 1000 / 50);
    CK(hipMemcpyToSymbol(HIP_SYMBOL(infr::g_logits_trace), &trace, sizeof(trace)));
    CK(hipMemsetAsync(trace, 0, (size_t)max_blocks * 128, s)); launch(); CK(hipStreamSynchronize(s));
    std::vector<long long> t((size_t)max_blocks * 16); CK(hipMemcpy(t.data(), trace, t.size() * 8, hipMemcpyDeviceToHost));
    int blocks = 0; for (int i = 0; i < max_blocks; i++) if (t[i * 16]) blocks = i + 1;
    report("router logits", t, blocks, {0, 1, 2, 3, 4, 5, 6}, "0 start | 1 operands here, squares summed per thread | 2 norm scale known | 3 operands in LDS | 4 after the barrier | 5 chains done | 6 logits stored");
    { std::vector<double> f; for (int bk = 0; bk < blocks; bk++) if (t[bk * 16 + 6] > t[bk * 16]) f.push_back((double)(t[bk * 16 + 14] - t[bk * 16 + 8]) / (double)(t[bk * 16 + 6] - t[bk * 16]) * 0.1);
      std::sort(f.begin(), f.end()); if (!f.empty()) printf("  shader clock over the kernel (clock64 ticks per wall-clock tick): median %.2f GHz\n", f[f.size() / 2]); }
    long long* none = nullptr; CK(hipMemcpyToSymbol(HIP_SYMBOL(infr::g_logits_trace), &none, sizeof(none)));
  }
  float gu_ms = 0;
  for (int which = 0; which < 2; which++) {
    int turn = 0;
    auto launch = [&]() {   // down follows a gate/up of the same set, whose routing it reads
      p.route.logits = logits + (size_t)(turn++ % kSets) * rows * E;
      if (which) { float* keep = p.y; p.y = nullptr; infr::launch_moe_gate_up(s, p); p.y = keep; infr::launch_moe_down_combine(s, p); }
      else infr::launch_moe_gate_up(s, p);
    };
    p.y = nullptr;
    for (int i = 0; i < 5; i++) launch();
    CK(hipStreamSynchronize(s));
    CK(hipEventRecord(a, s)); for (int i = 0; i < 50; i++) launch(); CK(hipEventRecord(b, s)); CK(hipStreamSynchronize(s));
    float ms; CK(hipEventElapsedTime(&ms, a, b));
    if (which) ms -= gu_ms;
    else gu_ms = ms;
    const double bytes = which ? (double)rows * (K + shared) * ne * row_bytes(ddt, nff) : (double)rows * (K + shared) * 2.0 * nff * row_bytes(gdt, ne);
    printf("%s: %.2f us per launch without time stamps (%s), %.2f TB/s\n",
           which ? "down + sum" : "routing + gate/up", ms * 1000 / 50, which ? "time of the pair of launches less the gate/up time above" : "launches cycle through expert sets", bytes / (ms / 50 * 1e-3) * 1e-12);
    p.y = reinterpret_cast<float*>(trace);
    { long long* rt = which ? nullptr : trace; CK(hipMemcpyToSymbol(HIP_SYMBOL(infr::g_route_trace), &rt, sizeof(rt))); }
    CK(hipMemsetAsync(trace, 0, (size_t)max_blocks * 128, s)); launch(); CK(hipStreamSynchronize(s));
    std::vector<long long> t((size_t)max_blocks * 16); CK(hipMemcpy(t.data(), trace, t.size() * 8, hipMemcpyDeviceToHost));
    int blocks = 0; for (int i = 0; i < max_blocks; i++) if (t[i * 16]) blocks = i + 1;
    if (which) report("down + sum", t, blocks, {0, 1, 2, 4, 5, 6, 8, 9, 10, 11, 12, 13, 14, 15}, "0 start | 1 ids here, first units requested | 2 h of every slot as cells (block barrier) | 4 wave 0 done with its units | 5 after the block barrier | 6 sums stored | 8..15: a wave of each residue class mod 8 done with its units");
    else report("routing + gate/up", t, blocks, {0, 9, 10, 11, 13, 14, 1, 2, 3, 4}, "0 start | 9 logits here, largest known | 10 exponentials in LDS | 11 their sum (wave 0; wave 1 selects meanwhile) | 13 candidates checked | 14 weights | 1 routed, x as cells (block barrier) | 2 x in registers, first items requested | 3 first round of the ring done | 4 end");
  }
  return 0;
}

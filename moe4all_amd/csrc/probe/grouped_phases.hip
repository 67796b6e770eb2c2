// Measurement aid for the grouped GEMM kernels of the batched MoeFfn path (k_grouped.hip): builds them with their time
// stamps switched on, runs gate/up (Q4_K) and down (Q6_K) of the prefill shape (hidden 2048, 128 experts, top-8,
// intermediate 768, 2048 tokens = 16384 pairs) on random banks with either equal buckets or Zipf(1.1)-like bucket sizes,
// and prints the launch time and, per row-tile height, how long the workgroups spend in each part of a work item.
// make -C moe4all_amd/csrc probes; ./moe4all_amd/csrc/probe/grouped_phases [uniform|zipf]
#define INFR_GROUPED_TRACE 1
#include "../k_grouped.hip"
#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>
namespace infr { thread_local const LaunchTiming* tl_launch_timing = nullptr; }
#define CK(x) do{hipError_t e_=(x); if(e_!=hipSuccess){printf("ERR %s: %s\n",#x,hipGetErrorString(e_)); exit(1);} }while(0)

static void report(const char* name, const std::vector<long long>& t, int blocks) {
  long long t0 = 0, t1 = 0;
  for (int b = 0; b < blocks; b++) if (t[b * 32]) { t0 = t0 ? std::min(t0, t[b * 32]) : t[b * 32]; t1 = std::max(t1, std::max(t[b * 32 + 5], t[b * 32])); }
  printf("%s: first start to last end %.1f us\n", name, (t1 - t0) * 0.01);
  printf("  rows of a tile | items | look-up | set-up | k loop | pair sum | epilogue | whole item   (median us; k loop also min / max)\n");
  for (int m = 1; m <= 4; m++) {
    std::vector<double> v[6], wl, wb, wi;
    for (int b = 0; b < blocks; b++) {
      const long long* r = &t[b * 32];
      if (!r[5] || (r[7] + 31) / 32 != m) continue;
      if (r[10]) { wl.push_back(100.0 * r[8] / r[10]); wb.push_back(100.0 * r[9] / r[10]); wi.push_back(100.0 * r[11] / r[10]); }
      for (int i = 0; i < 5; i++) v[i].push_back((r[i + 1] - r[i]) * 0.01);
      v[5].push_back((r[5] - r[0]) * 0.01);
    }
    if (v[0].empty()) continue;
    for (auto& x : v) std::sort(x.begin(), x.end());
    auto med = [](const std::vector<double>& x) { return x[x.size() / 2]; };
    printf("  %3d..%3d        | %5zu | %6.2f  | %6.2f | %6.2f (%.2f / %.2f) | %6.2f | %6.2f | %6.2f\n", 32 * m - 31, 32 * m, v[0].size(), med(v[0]),
           med(v[1]), med(v[2]), v[2].front(), v[2].back(), med(v[3]), med(v[4]), med(v[5]));
    std::sort(wl.begin(), wl.end()); std::sort(wb.begin(), wb.end());
    if (!wl.empty()) {
      printf("                    per wave (pair 0..3 first waves, then second waves), loads %% / barrier %% of the k loop:");
      for (int w = 0; w < 8; w++) {
        std::vector<double> a, c;
        for (int b = 0; b < blocks; b++) { const long long* r = &t[b * 32]; if (r[5] && (r[7] + 31) / 32 == m && r[10]) { a.push_back(100.0 * r[16 + w] / r[10]); c.push_back(100.0 * r[24 + w] / r[10]); } }
        std::sort(a.begin(), a.end()); std::sort(c.begin(), c.end());
        printf(" %.0f/%.0f", med(a), med(c));
      }
      printf("\n");
    }
    std::sort(wi.begin(), wi.end());
    if (!wl.empty()) printf("                    of the k loop (first wave): %.0f %% waiting for its loads, %.0f %% at the barrier, %.0f %% issuing loads (medians)\n", med(wl), med(wb), med(wi));
  }
  double busy = 0; int items = 0;
  for (int b = 0; b < blocks; b++) if (t[b * 32 + 5]) { busy += (t[b * 32 + 5] - t[b * 32]) * 0.01; items++; }
  printf("  %d items, sum of item times / 256 CUs = %.1f us\n", items, busy / 256);
  // per XCD (workgroup b runs on XCD b & 7): its items' time over its 32 CUs, and when its last item ends
  printf("  per XCD, sum of item times / 32 CUs | last end:");
  for (int x = 0; x < 8; x++) {
    double bx = 0; long long e = 0;
    for (int b = x; b < blocks; b += 8) if (t[b * 32 + 5]) { bx += (t[b * 32 + 5] - t[b * 32]) * 0.01; e = std::max(e, t[b * 32 + 5]); }
    printf("  %.0f | %.0f", bx / 32, (e - t0) * 0.01);
  }
  printf("\n");
}

int main(int argc, char** argv) {
  const bool zipf = argc > 1 && !strcmp(argv[1], "zipf");
  const int ne = 2048, nff = 768, E = 128, K = 8, rows = 2048, n_pairs = rows * K;
  hipStream_t s; CK(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
  // bucket sizes
  std::vector<int> cnt(E, n_pairs / E);
  if (zipf) {
    std::vector<double> w(E); for (int e = 0; e < E; e++) w[e] = 1.0 / std::pow(e + 1.0, 1.1);
    std::vector<bool> capped(E, false); int left = n_pairs; double wsum = 0; for (double x : w) wsum += x;
    for (int it = 0; it < 8; it++) {   // no expert can hold more than one pair per token
      bool again = false;
      for (int e = 0; e < E; e++) if (!capped[e] && w[e] / wsum * left > rows) { capped[e] = true; cnt[e] = rows; left -= rows; wsum -= w[e]; again = true; }
      if (!again) break;
    }
    int used = 0; for (int e = 0; e < E; e++) { if (!capped[e]) cnt[e] = (int)(w[e] / wsum * left); used += cnt[e]; }
    for (int e = E - 1; used < n_pairs; e = (e + E - 1) % E) if (!capped[e]) { cnt[e]++; used++; }
  }
  std::vector<int32_t> off(E + 1, 0); for (int e = 0; e < E; e++) off[e + 1] = off[e] + cnt[e];
  int tiles = 0, small = 0; for (int e = 0; e < E; e++) { tiles += (cnt[e] + 127) / 128; small += cnt[e] % 128 && cnt[e] % 128 <= 32; }
  printf("%s buckets: %d pairs, %d row tiles, %d of them with at most 32 rows; largest bucket %d\n", zipf ? "zipf(1.1)" : "equal", off[E], tiles, small, *std::max_element(cnt.begin(), cnt.end()));
  std::vector<int32_t> psrc(n_pairs); for (int i = 0; i < n_pairs; i++) psrc[i] = ((i * 37) % rows) * K + (i & 7);
  const size_t gate_b = (size_t)E * nff * (ne / 256) * 144, down_b = (size_t)E * ne * (nff / 256) * 210;
  uint8_t *gate, *up, *down; _Float16 *x, *h; float *xs, *hs, *gu_out; _Float16* y; int32_t *d_off, *d_psrc; long long* trace;
  CK(hipMalloc(&gate, gate_b + 64)); CK(hipMalloc(&up, gate_b + 64)); CK(hipMalloc(&down, down_b + 64));
  CK(hipMalloc(&x, (size_t)rows * ne * 2)); CK(hipMalloc(&h, (size_t)n_pairs * nff * 2)); CK(hipMalloc(&xs, rows * 4)); CK(hipMalloc(&hs, n_pairs * 4));
  CK(hipMalloc(&gu_out, (size_t)n_pairs * nff * 4)); CK(hipMalloc(&y, (size_t)n_pairs * ne * 2));
  CK(hipMalloc(&d_off, (E + 1) * 4)); CK(hipMalloc(&d_psrc, n_pairs * 4));
  const int max_blocks = 4096; CK(hipMalloc(&trace, (size_t)max_blocks * 256));
  CK(hipMemcpy(d_off, off.data(), (E + 1) * 4, hipMemcpyHostToDevice)); CK(hipMemcpy(d_psrc, psrc.data(), n_pairs * 4, hipMemcpyHostToDevice));
  { std::vector<uint8_t> v(gate_b); for (size_t i = 0; i < gate_b; i++) v[i] = (uint8_t)(i * 2654435761u >> 13);
    for (size_t b = 0; b < gate_b / 144; b++) { v[b * 144] = 0x66; v[b * 144 + 1] = 0x0e; v[b * 144 + 2] = 0x66; v[b * 144 + 3] = 0x0e; }
    CK(hipMemcpy(gate, v.data(), gate_b, hipMemcpyHostToDevice)); CK(hipMemcpy(up, v.data(), gate_b, hipMemcpyHostToDevice)); }
  { std::vector<uint8_t> v(down_b); for (size_t i = 0; i < down_b; i++) v[i] = (uint8_t)(i * 2246822519u >> 11);
    for (size_t b = 0; b < down_b / 210; b++) { v[b * 210 + 208] = 0x66; v[b * 210 + 209] = 0x0e; }
    CK(hipMemcpy(down, v.data(), down_b, hipMemcpyHostToDevice)); }
  { std::vector<_Float16> v((size_t)n_pairs * nff); unsigned r = 1; for (auto& q : v) { r = r * 1664525u + 1013904223u; q = (_Float16)(((r >> 8) / 16777216.0f - 0.5f)); }
    CK(hipMemcpy(h, v.data(), v.size() * 2, hipMemcpyHostToDevice)); CK(hipMemcpy(x, v.data(), (size_t)rows * ne * 2, hipMemcpyHostToDevice));
    std::vector<float> one(n_pairs, 1.0f); CK(hipMemcpy(xs, one.data(), rows * 4, hipMemcpyHostToDevice)); CK(hipMemcpy(hs, one.data(), n_pairs * 4, hipMemcpyHostToDevice)); }
  infr::GroupedParams g{};
  g.a = x; g.a_scale = xs; g.offsets = d_off; g.pair_src = d_psrc; g.w0 = gate; g.w0_stride = gate_b / E; g.w1 = up; g.w1_stride = gate_b / E;
  g.out = gu_out; g.K = ne; g.N = nff; g.n_expert = E; g.n_used = K; g.n_pairs = n_pairs; g.act = 0;
  infr::GroupedParams d{};
  d.a = h; d.a_scale = hs; d.offsets = d_off; d.pair_src = d_psrc; d.w0 = down; d.w0_stride = down_b / E; d.out = reinterpret_cast<float*>(y); d.out_f16 = 1;
  d.K = nff; d.N = ne; d.n_expert = E; d.n_used = K; d.n_pairs = n_pairs;
  hipEvent_t a, b; CK(hipEventCreate(&a)); CK(hipEventCreate(&b));
  for (int which = 0; which < 2; which++) {
    infr::GroupedParams& q = which ? d : g;
    auto launch = [&]() { if (which) infr::launch_grouped_down(s, INFR_Q6K, q); else infr::launch_grouped_gate_up(s, INFR_Q4K, q); };
    q.trace = nullptr;
    for (int i = 0; i < 5; i++) launch();
    CK(hipStreamSynchronize(s));
    CK(hipEventRecord(a, s)); for (int i = 0; i < 20; i++) launch(); CK(hipEventRecord(b, s)); CK(hipStreamSynchronize(s));
    float ms; CK(hipEventElapsedTime(&ms, a, b));
    const double flop = 2.0 * n_pairs * (which ? (double)ne * nff : 2.0 * nff * ne);
    printf("%s: %.1f us per launch without time stamps = %.0f TFLOP/s\n", which ? "down (Q6_K)" : "gate/up (Q4_K)", ms * 1000 / 20, flop / (ms / 20 * 1e-3) * 1e-12);
    q.trace = trace;
    CK(hipMemsetAsync(trace, 0, (size_t)max_blocks * 256, s)); launch(); CK(hipStreamSynchronize(s));
    std::vector<long long> t((size_t)max_blocks * 32); CK(hipMemcpy(t.data(), trace, t.size() * 8, hipMemcpyDeviceToHost));
    report(which ? "down" : "gate/up", t, max_blocks);
  }
  return 0;
}

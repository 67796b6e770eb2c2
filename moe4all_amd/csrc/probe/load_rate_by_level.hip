// Measurement aid: bytes per clock one CU can load, with global -> LDS direct loads and with ordinary loads, when every
// workgroup walks a window of its own that fits the L2 (64 / 128 KB), the last-level cache (512 KB) or nothing (8 MB).
// make -C moe4all_amd/csrc probes; ./moe4all_amd/csrc/probe/load_rate_by_level
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#define CK(x) do{hipError_t e_=(x); if(e_!=hipSuccess){printf("ERR %s: %s\n",#x,hipGetErrorString(e_)); exit(1);} }while(0)
template <int MODE>
__global__ __launch_bounds__(512) void k(const unsigned char* src, size_t span, unsigned* out, long long* cyc, int iters) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const unsigned lbase = (unsigned)(uintptr_t)(__attribute__((address_space(3))) void*)lds + __builtin_amdgcn_readfirstlane(wave) * 8192;
  // every CU walks its own part of the buffer; a wave-load covers 1 KB contiguous
  // a block walks a window of `span` bytes of its own (the window stays in L2 when it is small), 64 KB per iteration
  const unsigned char* base = src + (size_t)blockIdx.x * span + wave * 8192 + lane * 16;
  typedef unsigned v4u __attribute__((ext_vector_type(4)));
  v4u acc = {0, 0, 0, 0};
  const long long c0 = clock64();
  for (int i = 0; i < iters; i++) {
#pragma unroll
    for (int j = 0; j < 8; j++) {
      const unsigned char* q = base + ((size_t)i * 65536) % span + j * 1024;
      if (MODE == 0) asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(q), "s"(lbase + j * 1024) : "memory");
      else { v4u v; asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(v) : "v"(q) : "memory"); asm volatile("" : "+v"(acc) : "v"(v)); }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  }
  const long long c1 = clock64();
  if (lane == 0) cyc[blockIdx.x * 8 + wave] = c1 - c0;
  out[blockIdx.x * 512 + threadIdx.x] = acc.x + lds[threadIdx.x * 4];
}
template <int MODE> void run(const char* name, const unsigned char* src, size_t span, unsigned* out, long long* cyc, int waves) {
  const int iters = 512;
  CK(hipFuncSetAttribute((const void*)k<MODE>, hipFuncAttributeMaxDynamicSharedMemorySize, 65536));
  hipEvent_t a, b; CK(hipEventCreate(&a)); CK(hipEventCreate(&b));
  hipLaunchKernelGGL(k<MODE>, dim3(256), dim3(64 * waves), 65536, 0, src, span, out, cyc, 10);
  CK(hipEventRecord(a)); hipLaunchKernelGGL(k<MODE>, dim3(256), dim3(64 * waves), 65536, 0, src, span, out, cyc, iters); CK(hipEventRecord(b));
  CK(hipDeviceSynchronize());
  float ms; CK(hipEventElapsedTime(&ms, a, b));
  long long h[8]; CK(hipMemcpy(h, cyc, sizeof h, hipMemcpyDeviceToHost));
  const double bytes = (double)waves * iters * 8 * 1024;
  printf("%-26s span %6zu KB, %d waves: %.1f B/clk per CU, chip %.2f TB/s\n", name, span >> 10, waves, bytes / h[0], bytes * 256 / (ms * 1e-3) * 1e-12);
}
int main() {
  unsigned char* src; unsigned* out; long long* cyc; const size_t cap = (size_t)8 << 20;   // per block
  CK(hipMalloc(&src, cap * 256 + 65536 * 2)); CK(hipMemset(src, 1, cap * 256 + 65536 * 2)); CK(hipMalloc(&out, 256 * 512 * 4)); CK(hipMalloc(&cyc, 256 * 8 * 8));
  for (size_t span : {(size_t)65536, (size_t)128 << 10, (size_t)512 << 10, cap})
    for (int waves : {4, 8}) {
      run<0>("global_load_lds_dwordx4", src, span, out, cyc, waves);
      run<1>("global_load_dwordx4", src, span, out, cyc, waves);
    }
  return 0;
}

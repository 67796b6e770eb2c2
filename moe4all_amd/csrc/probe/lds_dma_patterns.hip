// Measurement aid: cost of one global -> LDS wave-load (global_load_lds_dwordx4) for the lane -> address patterns of the
// grouped GEMM's activation and weight stages, data resident in the caches: how many cycles of a CU's address / L1 path
// one such instruction takes.  make -C moe4all_amd/csrc probes; ./moe4all_amd/csrc/probe/lds_dma_patterns
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#define CK(x) do{hipError_t e_=(x); if(e_!=hipSuccess){printf("ERR %s: %s\n",#x,hipGetErrorString(e_)); exit(1);} }while(0)
__device__ __forceinline__ int rot7(int t) { return (t >> 1) & 7; }
template <int PAT>
__global__ __launch_bounds__(512) void k(const unsigned char* src, unsigned* out, long long* cyc, int iters) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const unsigned lbase = (unsigned)(uintptr_t)(__attribute__((address_space(3))) void*)lds + __builtin_amdgcn_readfirstlane(wave) * 8192;
  const unsigned char* base = src + (size_t)blockIdx.x * (1 << 20) + (size_t)wave * 65536;
  size_t off[8];
  for (int j = 0; j < 8; j++) {
    const int slot = 64 * j + lane;
    if (PAT == 0) off[j] = (size_t)slot * 16;
    else if (PAT == 1) { const int r = slot >> 3, c = slot & 7; off[j] = (size_t)r * 4096 + 16 * c; }
    else if (PAT == 2) { const int r = slot >> 3, c = (slot & 7) ^ rot7(r); off[j] = (size_t)r * 4096 + 16 * c; }
    else if (PAT == 3) { const int r = slot / 9, c = slot % 9; off[j] = (size_t)r * 4096 + 16 * (c < 8 ? c : 7); }
    else if (PAT == 4) { const int r = slot / 5, c = slot % 5; off[j] = (size_t)r * 1152 + (c ? 16 * c + 64 : 0) + 144; }
    else if (PAT == 5) { const int r = slot / 9, c = slot % 9; off[j] = (size_t)r * 1152 + 16 * c + 144; }
    else if (PAT == 6) { const int r = slot >> 3, c = slot & 7; off[j] = (size_t)r * 630 + (c < 4 ? 16 * c + 64 : c < 6 ? 128 + 16 * (c - 4) + 32 : c == 6 ? 192 : 194) + 210; }
    else { const int r = slot / 14, c = slot % 14; off[j] = (size_t)r * 630 + 16 * c + 210; }
  }
  const long long c0 = clock64();
  for (int i = 0; i < iters; i++) {
#pragma unroll
    for (int j = 0; j < 8; j++) asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(base + off[j]), "s"(lbase + j * 1024) : "memory");
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  }
  const long long c1 = clock64();
  if (lane == 0) cyc[blockIdx.x * 8 + wave] = c1 - c0;
  out[blockIdx.x * 512 + threadIdx.x] = lds[threadIdx.x * 4];
}
template <int PAT> void run(const char* name, const unsigned char* src, unsigned* out, long long* cyc, int waves) {
  const int iters = 1000;
  CK(hipFuncSetAttribute((const void*)k<PAT>, hipFuncAttributeMaxDynamicSharedMemorySize, 65536));
  hipLaunchKernelGGL(k<PAT>, dim3(256), dim3(64 * waves), 65536, 0, src, out, cyc, iters);
  CK(hipDeviceSynchronize());
  long long h[8]; CK(hipMemcpy(h, cyc, sizeof h, hipMemcpyDeviceToHost));
  printf("%-44s %d waves: %.1f cycles per wave-load on the CU (%.1f per wave)\n", name, waves, (double)h[0] / (iters * 8) / waves, (double)h[0] / (iters * 8));
}
int main() {
  unsigned char* src; unsigned* out; long long* cyc;
  CK(hipMalloc(&src, (size_t)257 << 20)); CK(hipMemset(src, 1, (size_t)257 << 20)); CK(hipMalloc(&out, 256 * 512 * 4)); CK(hipMalloc(&cyc, 256 * 8 * 8));
  for (int waves : {1, 4}) {
    run<0>("contiguous 1 KB", src, out, cyc, waves);
    run<1>("8 rows x 128 B, chunks ascending", src, out, cyc, waves);
    run<2>("8 rows x 128 B, chunks rotated", src, out, cyc, waves);
    run<3>("7 rows x 128 B + a repeated chunk each", src, out, cyc, waves);
    run<4>("Q4_K rows, header + 64 B of a half-step", src, out, cyc, waves);
    run<5>("Q4_K rows, whole 144-byte blocks", src, out, cyc, waves);
    run<6>("Q6_K rows, the parts of a half-step", src, out, cyc, waves);
    run<7>("Q6_K rows, whole 210-byte blocks", src, out, cyc, waves);
  }
  return 0;
}

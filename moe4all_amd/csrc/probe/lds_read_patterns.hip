// Measurement aid: ds_read_b128 throughput of a CU for a few lane -> address patterns (which tile layouts are free of
// LDS bank conflicts).  make -C moe4all_amd/csrc probes; ./moe4all_amd/csrc/probe/lds_read_patterns
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#define CK(x) do{hipError_t e_=(x); if(e_!=hipSuccess){printf("ERR %s: %s\n",#x,hipGetErrorString(e_)); exit(1);} }while(0)
template <int PAT>
__global__ __launch_bounds__(512) void k(unsigned* out, long long* cyc, int iters) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int i = threadIdx.x; i < 16384; i += 512) reinterpret_cast<uint4*>(lds)[i % 4096] = make_uint4(i, i, i, i);
  __syncthreads();
  const int t = lane & 31, half = lane >> 5;
  int off;
  if (PAT == 0) off = lane * 16;                                        // contiguous
  else if (PAT == 1) off = t * 128 + (((0 + 4 * half) ^ (t & 7)) * 16);   // rows of 128 B, rotation by t & 7
  else if (PAT == 2) off = t * 128 + (((0 + 4 * half) ^ ((t >> 1) & 7)) * 16);   // rotation by (t >> 1) & 7
  else if (PAT == 3) off = t * 128 + (4 * half) * 16;                      // no rotation
  else if (PAT == 4) off = t * 80 + 16 * half;                          // weight rows, pitch 80
  else off = t * 144 + 16 * half;                                       // pitch 144
  off += wave * 4096;
  uint4 acc = make_uint4(0, 0, 0, 0);
  const long long c0 = clock64();
  for (int i = 0; i < iters; i++) {
    typedef unsigned v4u __attribute__((ext_vector_type(4)));
    v4u v[8];
#pragma unroll
    for (int j = 0; j < 8; j++) asm volatile("ds_read_b128 %0, %1" : "=v"(v[j]) : "v"((unsigned)((off + j * 16384) & 65535)));
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
    for (int j = 0; j < 8; j++) { acc.x ^= v[j].x; acc.y ^= v[j].y; acc.z ^= v[j].z; acc.w ^= v[j].w; }
  }
  const long long c1 = clock64();
  if (lane == 0) cyc[blockIdx.x * 8 + wave] = c1 - c0;
  out[blockIdx.x * 512 + threadIdx.x] = acc.x ^ acc.y ^ acc.z ^ acc.w;
}
template <int PAT> void run(const char* name, unsigned* out, long long* cyc, int waves) {
  const int iters = 2000;
  CK(hipFuncSetAttribute((const void*)k<PAT>, hipFuncAttributeMaxDynamicSharedMemorySize, 65536));
  hipLaunchKernelGGL(k<PAT>, dim3(256), dim3(64 * waves), 65536, 0, out, cyc, iters);
  CK(hipDeviceSynchronize());
  long long h[8]; CK(hipMemcpy(h, cyc, sizeof h, hipMemcpyDeviceToHost));
  // bytes per clock of the CU: waves * iters * 8 reads * 1024 B / cycles
  printf("%-40s %d waves: %.1f cycles per wave-read, %.1f B/clk per CU\n", name, waves, (double)h[0] / (iters * 8), (double)waves * iters * 8 * 1024 / h[0]);
}
int main() {
  unsigned* out; long long* cyc; CK(hipMalloc(&out, 256 * 512 * 4)); CK(hipMalloc(&cyc, 256 * 8 * 8));
  for (int waves : {4, 8}) {
    run<0>("contiguous", out, cyc, waves);
    run<1>("128-B rows, rotation t & 7", out, cyc, waves);
    run<2>("128-B rows, rotation (t >> 1) & 7", out, cyc, waves);
    run<3>("128-B rows, no rotation", out, cyc, waves);
    run<4>("pitch 80", out, cyc, waves);
    run<5>("pitch 144", out, cyc, waves);
  }
  return 0;
}

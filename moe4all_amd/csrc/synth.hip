// Entry points of include/infr_synth.h: the same generator + quantiser code (synth.h) run by
// host threads or by one GPU thread per 256-element super-block.
#include <hip/hip_runtime.h>

#include <string>
#include <thread>
#include <vector>

#include "../../include/infr_synth.h"
#include "synth.h"

namespace {

SYN_HD inline size_t superblock_bytes(int dtype) {
    return dtype == INFR_Q8_0 ? 8 * 34 : dtype == INFR_Q4K ? 144 : dtype == INFR_Q6K ? 210 : dtype == INFR_MXFP4 ? 8 * 17 : 256 * 4;
}

__global__ __launch_bounds__(64) void synth_weights_kernel(uint8_t* dst, int dtype, uint64_t seed, uint64_t offset,
                                                           uint64_t n_super, double sigma) {
    const uint64_t sb = (uint64_t)blockIdx.x * 64 + threadIdx.x;
    if (sb >= n_super) return;
    const uint64_t e0 = offset + sb * 256;
    if (dtype == INFR_F32) {
        float* o = reinterpret_cast<float*>(dst) + sb * 256;
        for (int k = 0; k < 128; k++) {
            double z0, z1;
            synth::normal_pair(seed, (e0 >> 1) + (uint64_t)k, &z0, &z1);
            o[2 * k] = (float)(z0 * sigma);
            o[2 * k + 1] = (float)(z1 * sigma);
        }
        return;
    }
    uint8_t tmp[8 * 34];
    synth::synth_superblock(dtype, seed, e0, sigma, tmp);
    const size_t nb = superblock_bytes(dtype);
    uint8_t* o = dst + sb * nb;
    for (size_t i = 0; i < nb; i++) o[i] = tmp[i];
}

void host_range(int dtype, uint64_t seed, uint64_t offset, uint64_t sb0, uint64_t sb1, double sigma, uint8_t* dst) {
    const size_t nb = superblock_bytes(dtype);
    for (uint64_t sb = sb0; sb < sb1; sb++) {
        const uint64_t e0 = offset + sb * 256;
        if (dtype == INFR_F32) {
            float* o = reinterpret_cast<float*>(dst) + sb * 256;
            for (int i = 0; i < 256; i++) o[i] = synth::normal_at(seed, e0 + (uint64_t)i, sigma);
        } else {
            synth::synth_superblock(dtype, seed, e0, sigma, dst + sb * nb);
        }
    }
}

bool dtype_ok(int dtype) {
    return dtype == INFR_F32 || dtype == INFR_Q8_0 || dtype == INFR_Q4K || dtype == INFR_Q6K || dtype == INFR_MXFP4;
}

}  // namespace

extern "C" int infr_synth_normal_host(uint64_t seed, uint64_t offset, uint64_t n, double sigma, float* out) {
    if (!out && n) return -1;
    for (uint64_t i = 0; i < n; i++) out[i] = synth::normal_at(seed, offset + i, sigma);
    return 0;
}

extern "C" int64_t infr_synth_quantize_host(int32_t dtype, const float* src, uint64_t n, void* dst) {
    uint8_t* o = static_cast<uint8_t*>(dst);
    if (dtype == INFR_Q8_0) {
        if (n % 32) return -1;
        for (uint64_t b = 0; b < n / 32; b++) synth::quantize_block_q8_0(src + 32 * b, o + 34 * b);
        return (int64_t)(n / 32 * 34);
    }
    if (dtype == INFR_MXFP4) {
        if (n % 32) return -1;
        for (uint64_t b = 0; b < n / 32; b++) synth::quantize_block_mxfp4(src + 32 * b, o + 17 * b);
        return (int64_t)(n / 32 * 17);
    }
    if (n % 256) return -1;
    if (dtype == INFR_Q4K) {
        for (uint64_t b = 0; b < n / 256; b++) synth::quantize_block_q4_K(src + 256 * b, o + 144 * b);
        return (int64_t)(n / 256 * 144);
    }
    if (dtype == INFR_Q6K) {
        for (uint64_t b = 0; b < n / 256; b++) synth::quantize_block_q6_K(src + 256 * b, o + 210 * b);
        return (int64_t)(n / 256 * 210);
    }
    return -1;
}

extern "C" int64_t infr_synth_weights_host(int32_t dtype, uint64_t seed, uint64_t offset, uint64_t numel, double sigma,
                                           void* dst, int n_threads) {
    if (!dtype_ok(dtype) || numel % 256 || offset % 256 || (!dst && numel)) return -1;
    const uint64_t n_super = numel / 256;
    unsigned hw = std::thread::hardware_concurrency();
    int nt = n_threads > 0 ? n_threads : (hw ? (int)hw : 1);
    if ((uint64_t)nt > n_super) nt = n_super ? (int)n_super : 1;
    std::vector<std::thread> th;
    for (int t = 0; t < nt; t++) {
        uint64_t a = n_super * (uint64_t)t / (uint64_t)nt, b = n_super * (uint64_t)(t + 1) / (uint64_t)nt;
        th.emplace_back(host_range, dtype, seed, offset, a, b, sigma, static_cast<uint8_t*>(dst));
    }
    for (auto& t : th) t.join();
    return (int64_t)(n_super * superblock_bytes(dtype));
}

// Defined in backend.cpp: stream-ordered access to a buffer for sibling translation units.
extern "C" infr_status infr_hip_internal_buffer_span(infr_hip_backend* be, infr_hip_buffer* buf, size_t byte_offset,
                                                     size_t bytes, void** dptr, hipStream_t* stream);
extern "C" void infr_hip_internal_unlock(infr_hip_backend* be);
extern "C" infr_status infr_hip_internal_fail(infr_status st, const char* msg);

extern "C" infr_status infr_synth_weights_device(infr_hip_backend* be, infr_hip_buffer* buf, size_t byte_offset,
                                                 int32_t dtype, uint64_t seed, uint64_t offset, uint64_t numel,
                                                 double sigma) {
    if (!dtype_ok(dtype)) return infr_hip_internal_fail(INFR_ERR_UNSUPPORTED, "synth: dtype must be F32, Q8_0, Q4K, Q6K or Mxfp4");
    if (numel % 256 || offset % 256)
        return infr_hip_internal_fail(INFR_ERR_INVALID, "synth: offset and numel must be multiples of 256");
    const uint64_t n_super = numel / 256;
    void* p = nullptr;
    hipStream_t s = nullptr;
    infr_status st = infr_hip_internal_buffer_span(be, buf, byte_offset, (size_t)(n_super * superblock_bytes(dtype)), &p, &s);
    if (st != INFR_OK) return st;
    if (n_super) {
        uint64_t blocks = (n_super + 63) / 64;
        // one launch covers up to 2^31 blocks; numel here is at most a few 2^32 elements
        hipLaunchKernelGGL(synth_weights_kernel, dim3((uint32_t)blocks), dim3(64), 0, s, static_cast<uint8_t*>(p), dtype,
                           seed, offset, n_super, sigma);
    }
    infr_hip_internal_unlock(be);
    return INFR_OK;
}

// Device-side helpers shared by the gfx950 kernels: exact scalar decode of GGUF blocks,
// wave64 reductions, and an expf whose results equal the host libm's bit for bit.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/infr_hip.h"
#include "iquant.h"

namespace infr {

constexpr int kWave = 64;

// Unaligned load.  gfx950 code objects run with unaligned global access enabled, so this is
// one global_load of sizeof(T) bytes even at a 2-byte-aligned address (Q6_K blocks are 210 B,
// Q8_0 blocks 34 B).
template <class T>
__device__ __forceinline__ T ldu(const void* p) {
    T v;
    __builtin_memcpy(&v, p, sizeof(T));
    return v;
}

__device__ __forceinline__ float f16_bits_to_f32(uint32_t bits) {
    _Float16 h;
    uint16_t b = (uint16_t)bits;
    __builtin_memcpy(&h, &b, 2);
    return (float)h;  // exact, subnormals included
}

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t bits) {
    return __uint_as_float((bits & 0xFFFFu) << 16);
}

// ---------------------------------------------------------------------------------------------
// expf with the same results as glibc's expf on an FMA-capable x86-64 host (the function the
// reference's f32::exp resolves to): table of 2^(i/32) in double, degree-3 polynomial, every
// multiply-add fused, including the range reduction r = x*N/ln2 - k.  Checked against the
// host expf over every float with |x| <= 104 (zero differences).
__device__ const uint64_t kExp2Table[32] = {
    0x3ff0000000000000ull, 0x3fefd9b0d3158574ull, 0x3fefb5586cf9890full, 0x3fef9301d0125b51ull,
    0x3fef72b83c7d517bull, 0x3fef54873168b9aaull, 0x3fef387a6e756238ull, 0x3fef1e9df51fdee1ull,
    0x3fef06fe0a31b715ull, 0x3feef1a7373aa9cbull, 0x3feedea64c123422ull, 0x3feece086061892dull,
    0x3feebfdad5362a27ull, 0x3feeb42b569d4f82ull, 0x3feeab07dd485429ull, 0x3feea47eb03a5585ull,
    0x3feea09e667f3bcdull, 0x3fee9f75e8ec5f74ull, 0x3feea11473eb0187ull, 0x3feea589994cce13ull,
    0x3feeace5422aa0dbull, 0x3feeb737b0cdc5e5ull, 0x3feec49182a3f090ull, 0x3feed503b23e255dull,
    0x3feee89f995ad3adull, 0x3feeff76f2fb5e47ull, 0x3fef199bdd85529cull, 0x3fef3720dcef9069ull,
    0x3fef5818dcfba487ull, 0x3fef7c97337b9b5full, 0x3fefa4afa2a490daull, 0x3fefd0765b6e4540ull};

// T: the 32-entry table above, in global memory or a copy staged in LDS (a kernel on a latency
// critical path copies it once at start so later lookups do not wait on a global load).
__device__ __forceinline__ float expf_libm(float x, const uint64_t* T) {
    // Out-of-range and non-finite inputs: same special cases as libm.
    if (!(x == x)) return x + x;
    if (x > 0x1.62e42ep6f) return __builtin_huge_valf();
    if (x < -0x1.9fe368p6f) return 0.0f;
    const double InvLn2N = 0x1.71547652b82fep+0 * 32.0;
    const double Shift = 0x1.8p+52;
    const double C0 = 0x1.c6af84b912394p-5 / 32.0 / 32.0 / 32.0;
    const double C1 = 0x1.ebfce50fac4f3p-3 / 32.0 / 32.0;
    const double C2 = 0x1.62e42ff0c52d6p-1 / 32.0;
    double xd = (double)x;
    double z = __dmul_rn(InvLn2N, xd);
    double kd = __dadd_rn(z, Shift);
    uint64_t ki = (uint64_t)__double_as_longlong(kd);
    kd = __dsub_rn(kd, Shift);
    double r = __fma_rn(InvLn2N, xd, -kd);
    uint64_t t = T[ki & 31u] + (ki << 47);
    double s = __longlong_as_double((long long)t);
    double p = __fma_rn(C0, r, C1);
    double r2 = __dmul_rn(r, r);
    double y = __fma_rn(C2, r, 1.0);
    y = __fma_rn(p, r2, y);
    y = __dmul_rn(y, s);
    return (float)y;
}
__device__ __forceinline__ float expf_libm(float x) { return expf_libm(x, kExp2Table); }

// act_fn of the reference (crates/infr-cpu/src/kernels.rs:6664-6672), same operation order.
__device__ __forceinline__ float act_fn(int act, float g, const uint64_t* T = kExp2Table) {
    if (act == INFR_ACT_SILU) return __fdiv_rn(g, __fadd_rn(1.0f, expf_libm(-g, T)));
    if (act == INFR_ACT_GELU) {
        float g3 = __fmul_rn(__fmul_rn(__fmul_rn(0.044715f, g), g), g);
        float inner = __fmul_rn(0.7978846f, __fadd_rn(g, g3));
        float t = __fadd_rn(1.0f, tanhf(inner));
        return __fmul_rn(__fmul_rn(0.5f, g), t);
    }
    return __fdiv_rn(1.0f, __fadd_rn(1.0f, expf_libm(-g, T)));
}

// gated_act_fn (kernels.rs:6678-6683).
__device__ __forceinline__ float gated_act_fn(int act, bool has_clamp, float clamp, float gate, float up,
                                              const uint64_t* T = kExp2Table) {
    if (!has_clamp) return __fmul_rn(act_fn(act, gate, T), up);
    float gm = gate < clamp ? gate : clamp;
    float uc = up;
    if (uc < -clamp) uc = -clamp;
    if (uc > clamp) uc = clamp;
    return __fmul_rn(act_fn(act, gm, T), uc);
}

// ---------------------------------------------------------------------------------------------
// Block geometry, host and device.
__host__ __device__ inline bool block_geometry(int dtype, int* elems, int* bytes) {
    switch (dtype) {
        case INFR_F32: case INFR_I32: case INFR_U32: *elems = 1; *bytes = 4; return true;
        case INFR_F16: case INFR_BF16: *elems = 1; *bytes = 2; return true;
        case INFR_Q4_0: *elems = 32; *bytes = 18; return true;
        case INFR_Q4_1: *elems = 32; *bytes = 20; return true;
        case INFR_Q5_0: *elems = 32; *bytes = 22; return true;
        case INFR_Q5_1: *elems = 32; *bytes = 24; return true;
        case INFR_Q8_0: *elems = 32; *bytes = 34; return true;
        case INFR_Q2K: *elems = 256; *bytes = 84; return true;
        case INFR_Q3K: *elems = 256; *bytes = 110; return true;
        case INFR_Q4K: *elems = 256; *bytes = 144; return true;
        case INFR_Q5K: *elems = 256; *bytes = 176; return true;
        case INFR_Q6K: *elems = 256; *bytes = 210; return true;
        case INFR_IQ4_NL: *elems = 32; *bytes = 18; return true;
        case INFR_IQ4_XS: *elems = 256; *bytes = 136; return true;
        case INFR_TQ1_0: *elems = 256; *bytes = 54; return true;
        case INFR_TQ2_0: *elems = 256; *bytes = 66; return true;
        case INFR_Q2_0: *elems = 64; *bytes = 18; return true;
        case INFR_MXFP4: *elems = 32; *bytes = 17; return true;
        case INFR_NVFP4: *elems = 64; *bytes = 36; return true;
        // decode_spec.rs:334-347
        case INFR_IQ1_S: *elems = 256; *bytes = 50; return true;
        case INFR_IQ1_M: *elems = 256; *bytes = 56; return true;
        case INFR_IQ2_XXS: *elems = 256; *bytes = 66; return true;
        case INFR_IQ2_XS: *elems = 256; *bytes = 74; return true;
        case INFR_IQ2_S: *elems = 256; *bytes = 82; return true;
        case INFR_IQ3_XXS: *elems = 256; *bytes = 98; return true;
        case INFR_IQ3_S: *elems = 256; *bytes = 110; return true;
        default: return false;
    }
}

// The 16-entry code books (crates/infr-gguf/src/dequant.rs:407-444) as sixteen signed bytes in two
// 64-bit halves, entry i = byte i % 8 of half i / 8.
// IQ4_NL / IQ4_XS: -127 -104 -83 -65 -49 -35 -22 -10 1 13 25 38 53 69 89 113.
// MXFP4 / NVFP4 (twice the E2M1 value): 0 1 2 3 4 6 8 12 0 -1 -2 -3 -4 -6 -8 -12.
constexpr uint64_t kIq4nlLo = 0xF6EADDCFBFAD9881ull, kIq4nlHi = 0x7159453526190D01ull;
constexpr uint64_t kFp4Lo = 0x0C08060403020100ull, kFp4Hi = 0xF4F8FAFCFDFEFF00ull;
__device__ __forceinline__ int book16(uint64_t lo, uint64_t hi, uint32_t i) {
    return (int)(int8_t)(((i & 8u) ? hi : lo) >> (8u * (i & 7u)));
}

// e8m0_to_fp32_half (dequant.rs:415-421): 2^(x - 128), the two smallest as subnormals.
__device__ __forceinline__ float e8m0_half(uint32_t x) {
    return __uint_as_float(x < 2u ? 0x00200000u << x : (x - 1u) << 23);
}
// ue4m3_to_fp32 (dequant.rs:427-438): unsigned 4-bit exponent (bias 7), 3-bit mantissa, halved;
// 0x00 and 0x7F decode to zero, bit 7 is not read.
__device__ __forceinline__ float ue4m3_half(uint32_t x) {
    if (x == 0u || x == 0x7Fu) return 0.0f;
    const uint32_t e = (x >> 3) & 0xFu, m = x & 7u;
    return e == 0u ? (float)m * 0x1p-10f : __uint_as_float(((e + 119u) << 23) | (m << 20));
}

// Ternary digit n of a TQ1_0 byte (dequant.rs:938-944): 0, 1 or 2.
__device__ __forceinline__ uint32_t trit(uint32_t q, uint32_t pow3) { return (((q * pow3) & 0xFFu) * 3u) >> 8; }

// get_scale_min_k4 (crates/infr-gguf/src/dequant.rs:77-87).
__device__ __forceinline__ void k4(int j, const uint8_t* q, uint32_t& sc, uint32_t& m) {
    if (j < 4) {
        sc = q[j] & 63u;
        m = q[j + 4] & 63u;
    } else {
        sc = (uint32_t)((q[j + 4] & 0x0F) | ((q[j - 4] >> 6) << 4));
        m = (uint32_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4));
    }
}

// Exact decode of element k of a row of `dtype`, with the reference's operation order
// (crates/infr-gguf/src/dequant.rs:35-51: sc = d*f32(sc_i); mn = dmin*f32(m_i);
// out = sc*f32(code) + mn, separate multiply and add).  Slow path: used by the standalone
// decode kernel and by the shape-generic GEMV.
__device__ inline float decode_elem(int dtype, const uint8_t* row, uint32_t k) {
    switch (dtype) {
        case INFR_F32: return ldu<float>(row + 4u * k);
        case INFR_F16: return f16_bits_to_f32(ldu<uint16_t>(row + 2u * k));
        case INFR_BF16: return bf16_bits_to_f32(ldu<uint16_t>(row + 2u * k));
        case INFR_I32: return (float)ldu<int32_t>(row + 4u * k);
        case INFR_U32: return (float)ldu<uint32_t>(row + 4u * k);
        case INFR_Q8_0: {
            const uint8_t* blk = row + (size_t)(k >> 5) * 34u;
            float d = f16_bits_to_f32(ldu<uint16_t>(blk));
            int code = (int)(int8_t)blk[2 + (k & 31u)] + 128;
            float sc = __fmul_rn(d, 1.0f);
            float mn = __fmul_rn(d, -128.0f);
            return __fadd_rn(__fmul_rn(sc, (float)code), mn);
        }
        case INFR_Q4K: {
            const uint8_t* blk = row + (size_t)(k >> 8) * 144u;
            uint32_t w = k & 255u;
            uint32_t j = w >> 6, hi = (w >> 5) & 1u, l = w & 31u;
            float d = f16_bits_to_f32(ldu<uint16_t>(blk));
            float dmin = f16_bits_to_f32(ldu<uint16_t>(blk + 2));
            uint32_t sc, m;
            k4((int)(2 * j + hi), blk + 4, sc, m);
            uint8_t v = blk[16 + j * 32 + l];
            uint32_t code = hi ? (uint32_t)(v >> 4) : (uint32_t)(v & 0xF);
            float scf = __fmul_rn(d, (float)(int)sc);
            float mn = __fmul_rn(dmin, (float)(-(int)m));
            return __fadd_rn(__fmul_rn(scf, (float)code), mn);
        }
        case INFR_Q4_0: case INFR_Q4_1: case INFR_Q5_0: case INFR_Q5_1: {
            // 32-element blocks [f16 d][f16 m?][u32 qh?][16 nibble bytes] (dequant.rs:137-209): element j < 16 is
            // the low nibble of byte j, element j + 16 the high nibble; the fifth bit of element e is bit e of qh
            const bool has_m = dtype == INFR_Q4_1 || dtype == INFR_Q5_1, five = dtype == INFR_Q5_0 || dtype == INFR_Q5_1;
            const uint32_t bb = 18u + (has_m ? 2u : 0u) + (five ? 4u : 0u);
            const uint8_t* blk = row + (size_t)(k >> 5) * bb;
            const uint32_t e = k & 31u, j = e & 15u;
            const uint8_t* p = blk + 2 + (has_m ? 2 : 0);
            uint32_t code = 0;
            if (five) {
                code = ((ldu<uint32_t>(p) >> e) & 1u) << 4;
                p += 4;
            }
            code |= e < 16 ? (uint32_t)(p[j] & 0xF) : (uint32_t)(p[j] >> 4);
            const float d = f16_bits_to_f32(ldu<uint16_t>(blk));
            const float mn = has_m ? __fmul_rn(f16_bits_to_f32(ldu<uint16_t>(blk + 2)), 1.0f)
                                   : __fmul_rn(d, five ? -16.0f : -8.0f);
            return __fadd_rn(__fmul_rn(__fmul_rn(d, 1.0f), (float)code), mn);
        }
        case INFR_Q2K: {
            // [16 scale bytes][64 qs][f16 d][f16 dmin] (dequant.rs:224-250): 16-element group g = w / 16 reads the
            // 2-bit field at shift 2 * ((g % 8) / 2) of qs[32 * (g / 8) + 16 * (g % 2) + l]
            const uint8_t* blk = row + (size_t)(k >> 8) * 84u;
            const uint32_t w = k & 255u, g = w >> 4, l = w & 15u;
            const uint32_t sc = blk[g];
            const uint32_t code = ((uint32_t)blk[16 + 32 * (g >> 3) + 16 * (g & 1u) + l] >> (2u * ((g & 7u) >> 1))) & 3u;
            const float scf = __fmul_rn(f16_bits_to_f32(ldu<uint16_t>(blk + 80)), (float)(sc & 0xFu));
            const float mn = __fmul_rn(f16_bits_to_f32(ldu<uint16_t>(blk + 82)), (float)(-(int)(sc >> 4)));   // integer negation: -0 does not exist
            return __fadd_rn(__fmul_rn(scf, (float)code), mn);
        }
        case INFR_Q3K: {
            // [32 hmask][64 qs][12 scale bytes][f16 d] (dequant.rs:251-312).  6-bit scale g: low 4 bits = nibble
            // (g / 8) of scale byte g % 8, high 2 bits = field (g / 4) of scale byte 8 + g % 4; value - 32.
            // Code = 2 bits from qs as in Q2_K + bit (g / 2) of hmask[16 * (g % 2) + l] as bit 2; min = -4 * scale.
            const uint8_t* blk = row + (size_t)(k >> 8) * 110u;
            const uint32_t w = k & 255u, g = w >> 4, l = w & 15u;
            const uint32_t lo = ((uint32_t)blk[96 + (g & 7u)] >> (g >= 8u ? 4u : 0u)) & 0xFu;
            const uint32_t hi = ((uint32_t)blk[104 + (g & 3u)] >> (2u * (g >> 2))) & 3u;
            const int s = (int)(lo | (hi << 4)) - 32;
            const uint32_t low2 = ((uint32_t)blk[32 + 32 * (g >> 3) + 16 * (g & 1u) + l] >> (2u * ((g & 7u) >> 1))) & 3u;
            const uint32_t high = ((uint32_t)blk[16 * (g & 1u) + l] >> (g >> 1)) & 1u;
            const float d = f16_bits_to_f32(ldu<uint16_t>(blk + 108));
            const float scf = __fmul_rn(d, (float)s);
            const float mn = __fmul_rn(d, (float)(-4 * s));
            return __fadd_rn(__fmul_rn(scf, (float)(low2 | (high << 2))), mn);
        }
        case INFR_Q5K: {
            // Q4_K with 32 bytes of fifth bits after the scales (dequant.rs:336-363): bit (2j + hi) of qh[l]
            const uint8_t* blk = row + (size_t)(k >> 8) * 176u;
            const uint32_t w = k & 255u;
            const uint32_t j = w >> 6, hi = (w >> 5) & 1u, l = w & 31u;
            uint32_t sc, m;
            k4((int)(2 * j + hi), blk + 4, sc, m);
            const uint8_t v = blk[48 + j * 32 + l];
            const uint32_t code = (hi ? (uint32_t)(v >> 4) : (uint32_t)(v & 0xF)) + ((((uint32_t)blk[16 + l] >> (2 * j + hi)) & 1u) << 4);
            const float scf = __fmul_rn(f16_bits_to_f32(ldu<uint16_t>(blk)), (float)(int)sc);
            const float mn = __fmul_rn(f16_bits_to_f32(ldu<uint16_t>(blk + 2)), (float)(-(int)m));
            return __fadd_rn(__fmul_rn(scf, (float)code), mn);
        }
        case INFR_Q6K: {
            const uint8_t* blk = row + (size_t)(k >> 8) * 210u;
            uint32_t w = k & 255u;
            uint32_t half = w >> 7, g = (w >> 5) & 3u, l = w & 31u;
            const uint8_t* ql = blk + half * 64;
            const uint8_t* qh = blk + 128 + half * 32;
            uint32_t lo = (g & 1u) ? ql[l + 32] : ql[l];
            lo = (g & 2u) ? (lo >> 4) : (lo & 0xFu);
            uint32_t hi2 = ((uint32_t)qh[l] >> (2u * g)) & 3u;
            uint32_t code = lo | (hi2 << 4);
            int s = (int)(int8_t)blk[192 + (w >> 4)];
            float d = f16_bits_to_f32(ldu<uint16_t>(blk + 208));
            float scf = __fmul_rn(d, (float)s);
            float mn = __fmul_rn(d, (float)(-32 * s));
            return __fadd_rn(__fmul_rn(scf, (float)code), mn);
        }
        case INFR_IQ4_NL: {
            // [f16 d][16 nibble bytes] (dequant.rs:499-519): element j < 16 low nibble of byte j, j + 16 the high one
            const uint8_t* blk = row + (size_t)(k >> 5) * 18u;
            const uint32_t e = k & 31u, v = blk[2 + (e & 15u)];
            return __fmul_rn(f16_bits_to_f32(ldu<uint16_t>(blk)), (float)book16(kIq4nlLo, kIq4nlHi, e < 16u ? v & 0xFu : v >> 4));
        }
        case INFR_IQ4_XS: {
            // [f16 d][u16 scales_h][4 scales_l][128 qs] (dequant.rs:521-559): sub-block ib of 32 elements has the
            // 6-bit scale nibble ib of scales_l | field ib of scales_h << 4, minus 32; codes as in IQ4_NL
            const uint8_t* blk = row + (size_t)(k >> 8) * 136u;
            const uint32_t w = k & 255u, ib = w >> 5, e = w & 31u;
            const uint32_t lo = ((uint32_t)blk[4 + (ib >> 1)] >> (4u * (ib & 1u))) & 0xFu;
            const uint32_t hi = ((uint32_t)ldu<uint16_t>(blk + 2) >> (2u * ib)) & 3u;
            const float dl = __fmul_rn(f16_bits_to_f32(ldu<uint16_t>(blk)), (float)((int)(lo | (hi << 4)) - 32));
            const uint32_t v = blk[8 + 16u * ib + (e & 15u)];
            return __fmul_rn(dl, (float)book16(kIq4nlLo, kIq4nlHi, e < 16u ? v & 0xFu : v >> 4));
        }
        case INFR_TQ1_0: {
            // [48 qs][4 qh][f16 d] (dequant.rs:926-970): elements 0..159 = digit n of qs[m], n * 32 + m;
            // 160..239 = digit n of qs[32 + m], n * 16 + m; 240..255 = digit n of qh[j], n * 4 + j
            const uint8_t* blk = row + (size_t)(k >> 8) * 54u;
            const uint32_t w = k & 255u;
            uint32_t byte, n;
            if (w < 160u) { n = w >> 5; byte = blk[w & 31u]; }
            else if (w < 240u) { n = (w - 160u) >> 4; byte = blk[32u + (w & 15u)]; }
            else { n = (w - 240u) >> 2; byte = blk[48u + (w & 3u)]; }
            const uint32_t p3 = n == 0u ? 1u : n == 1u ? 3u : n == 2u ? 9u : n == 3u ? 27u : 81u;
            return __fmul_rn((float)((int)trit(byte, p3) - 1), f16_bits_to_f32(ldu<uint16_t>(blk + 52)));
        }
        case INFR_TQ2_0: {
            // [64 qs][f16 d] (dequant.rs:978-1000): element 128 c + 32 l + m = field l of qs[32 c + m]
            const uint8_t* blk = row + (size_t)(k >> 8) * 66u;
            const uint32_t w = k & 255u;
            const uint32_t q = ((uint32_t)blk[32u * (w >> 7) + (w & 31u)] >> (2u * ((w >> 5) & 3u))) & 3u;
            return __fmul_rn((float)((int)q - 1), f16_bits_to_f32(ldu<uint16_t>(blk + 64)));
        }
        case INFR_Q2_0: {
            // [f16 d][16 qs] (dequant.rs:1007-1022): element j = field j % 4 of qs[j / 4]
            const uint8_t* blk = row + (size_t)(k >> 6) * 18u;
            const uint32_t j = k & 63u;
            const uint32_t q = ((uint32_t)blk[2u + (j >> 2)] >> (2u * (j & 3u))) & 3u;
            return __fmul_rn((float)((int)q - 1), f16_bits_to_f32(ldu<uint16_t>(blk)));
        }
        case INFR_MXFP4: {
            // [u8 e][16 nibble bytes] (dequant.rs:1029-1045): nibble order of IQ4_NL, scale 2^(e - 128)
            const uint8_t* blk = row + (size_t)(k >> 5) * 17u;
            const uint32_t e = k & 31u, v = blk[1 + (e & 15u)];
            return __fmul_rn((float)book16(kFp4Lo, kFp4Hi, e < 16u ? v & 0xFu : v >> 4), e8m0_half(blk[0]));
        }
        case INFR_NVFP4: {
            // [4 ue4m3 scales][32 qs] (dequant.rs:1053-1073): sub-block s of 16 elements: element j < 8 low
            // nibble of qs[8 s + j], element j + 8 the high one
            const uint8_t* blk = row + (size_t)(k >> 6) * 36u;
            const uint32_t w = k & 63u, s = w >> 4, e = w & 15u, v = blk[4u + 8u * s + (e & 7u)];
            return __fmul_rn((float)book16(kFp4Lo, kFp4Hi, e < 8u ? v & 0xFu : v >> 4), ue4m3_half(blk[s]));
        }
        case INFR_IQ1_S: return decode_iq1s(row, k);
        case INFR_IQ1_M: return decode_iq1m(row, k);
        case INFR_IQ2_XXS: return decode_iq2xxs(row, k);
        case INFR_IQ2_XS: return decode_iq2xs(row, k);
        case INFR_IQ2_S: return decode_iq2s(row, k);
        case INFR_IQ3_XXS: return decode_iq3xxs(row, k);
        case INFR_IQ3_S: return decode_iq3s(row, k);
        default: return 0.0f;
    }
}

// ---------------------------------------------------------------------------------------------
// Wave64 helpers.  Cross-lane steps inside a row of 16 lanes use DPP (no LDS round trip);
// the four row results meet through readlane.
template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_u(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xF, 0xF, true);
}
// Rows selected by ROW_MASK read the DPP source, the other rows read 0 (used with
// row_bcast:15 / row_bcast:31 to carry a row's total into the following rows).
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_rows_f(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xF, false));
}
constexpr int kDppXor1 = 0xB1;        // quad_perm [1,0,3,2]
constexpr int kDppXor2 = 0x4E;        // quad_perm [2,3,0,1]
constexpr int kDppHalfMirror = 0x141; // lane i <-> 7-i inside each 8
constexpr int kDppMirror = 0x140;     // lane i <-> 15-i inside each 16

__device__ __forceinline__ float quad_sum(float v) {
    v += dpp_f<kDppXor1>(v);
    v += dpp_f<kDppXor2>(v);
    return v;
}
__device__ __forceinline__ float oct_sum(float v) {
    v = quad_sum(v);
    return v + dpp_f<kDppHalfMirror>(v);
}
__device__ __forceinline__ float row16_sum(float v) {
    v = quad_sum(v);
    v += dpp_f<kDppHalfMirror>(v);
    v += dpp_f<kDppMirror>(v);
    return v;
}
__device__ __forceinline__ float readlane_f(float v, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}
// Every lane receives the sum over the wavefront.
__device__ __forceinline__ float wave_sum(float v) {
    v = row16_sum(v);
    return (readlane_f(v, 0) + readlane_f(v, 16)) + (readlane_f(v, 32) + readlane_f(v, 48));
}
// Sum over a block of 256 threads, the same bits in every thread; red: 4 floats of LDS.
__device__ __forceinline__ float block256_sum(float v, float* red) {
    v = wave_sum(v);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    return (red[0] + red[1]) + (red[2] + red[3]);
}
// Op::RmsNorm's row scale 1 / sqrt(sum(x^2) / dim + eps) (crates/infr-cpu/src/lib.rs:1062-1063).
__device__ __forceinline__ float rms_scale(float sumsq, int dim, float eps) {
    return __fdiv_rn(1.0f, __fsqrt_rn(__fadd_rn(__fdiv_rn(sumsq, (float)dim), eps)));
}
// A thread's share of a row's sum of squares when thread t of 256 owns the float4s t, t + 256, ...
__device__ __forceinline__ float sumsq4(float acc, const float4& f) {
    acc = __fmaf_rn(f.x, f.x, acc);
    acc = __fmaf_rn(f.y, f.y, acc);
    acc = __fmaf_rn(f.z, f.z, acc);
    return __fmaf_rn(f.w, f.w, acc);
}
__device__ __forceinline__ float4 rms_apply4(const float4& x, float s, const float4& w) {
    return make_float4(__fmul_rn(__fmul_rn(x.x, s), w.x), __fmul_rn(__fmul_rn(x.y, s), w.y),
                       __fmul_rn(__fmul_rn(x.z, s), w.z), __fmul_rn(__fmul_rn(x.w, s), w.w));
}
__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, dpp_f<kDppXor1>(v));
    v = fmaxf(v, dpp_f<kDppXor2>(v));
    v = fmaxf(v, dpp_f<kDppHalfMirror>(v));
    v = fmaxf(v, dpp_f<kDppMirror>(v));
    return fmaxf(fmaxf(readlane_f(v, 0), readlane_f(v, 16)), fmaxf(readlane_f(v, 32), readlane_f(v, 48)));
}
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
    v = max(v, dpp_u<kDppXor1>(v));
    v = max(v, dpp_u<kDppXor2>(v));
    v = max(v, dpp_u<kDppHalfMirror>(v));
    v = max(v, dpp_u<kDppMirror>(v));
    uint32_t a = max((uint32_t)__builtin_amdgcn_readlane((int)v, 0), (uint32_t)__builtin_amdgcn_readlane((int)v, 16));
    uint32_t b = max((uint32_t)__builtin_amdgcn_readlane((int)v, 32), (uint32_t)__builtin_amdgcn_readlane((int)v, 48));
    return max(a, b);
}
__device__ __forceinline__ uint32_t wave_min_u32(uint32_t v) {
    v = min(v, dpp_u<kDppXor1>(v));
    v = min(v, dpp_u<kDppXor2>(v));
    v = min(v, dpp_u<kDppHalfMirror>(v));
    v = min(v, dpp_u<kDppMirror>(v));
    uint32_t a = min((uint32_t)__builtin_amdgcn_readlane((int)v, 0), (uint32_t)__builtin_amdgcn_readlane((int)v, 16));
    uint32_t b = min((uint32_t)__builtin_amdgcn_readlane((int)v, 32), (uint32_t)__builtin_amdgcn_readlane((int)v, 48));
    return min(a, b);
}

// Sum of v over each run of `seg` consecutive lanes (seg need not be a power of two); the
// total lands in the first lane of the run.  pos = lane's index inside its run.
__device__ __forceinline__ float segment_sum(float v, int seg, int pos) {
    for (int off = 1; off < seg; off <<= 1) {
        float t = __shfl_down(v, off, kWave);
        if (pos + off < seg) v += t;
    }
    return v;
}

}  // namespace infr

// Exact scalar decode of the seven grid i-quants (IQ2_XXS, IQ2_XS, IQ2_S, IQ3_XXS, IQ3_S, IQ1_S, IQ1_M):
// 256-element super-blocks whose groups of 8 (or 4) elements are entries of a lattice codebook, a sign
// byte per group and a small odd multiplier per 32 or 16 elements
// (crates/infr-gguf/src/dequant.rs:565-916).  Element k of a row: block k / 256; inside it sub-block
// ib = w / 32, group l = (w / 8) % 4, position j = w % 8.  Products are formed in the reference's order
// ((d * multiplier) * constant, then * magnitude, then * sign), one rounding each.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define IQG_QUAL static __device__ const
#include "iquant_grids.h"
#undef IQG_QUAL

namespace infr {

// entry e of a codebook with 2 (3) bits per element: the index of element j into the alphabet
__device__ __forceinline__ uint32_t grid_digit2(const uint16_t* g, uint32_t e, uint32_t j) { return ((uint32_t)g[e] >> (2u * j)) & 3u; }
__device__ __forceinline__ uint32_t grid_digit3(const uint16_t* g, uint32_t e, uint32_t j) { return ((uint32_t)g[e] >> (3u * j)) & 7u; }
// the alphabets: IQ2 {8, 25, 43}; IQ3_XXS {4, 12, ..., 52, 62}; IQ3_S {1, 3, ..., 15}; IQ1 {0, 1, -1}
__device__ __forceinline__ float iq2_value(uint32_t digit) { return (float)((0x2B1908u >> (8u * digit)) & 0xFFu); }
__device__ __forceinline__ float iq3xxs_value(uint32_t digit) { return (float)(4u + 8u * digit + (digit == 7u ? 2u : 0u)); }
__device__ __forceinline__ float iq3s_value(uint32_t digit) { return (float)(2u * digit + 1u); }
__device__ __forceinline__ float iq1_value(uint32_t digit) { return (float)((int)(digit & 1u) - (int)(digit >> 1)); }
// KSIGNS_IQ2XS (crates/infr-core/src/iquant_grids.rs): seven sign bits, the eighth makes the count of set bits even
__device__ __forceinline__ uint32_t ksigns(uint32_t i) { return i | (((uint32_t)__builtin_popcount(i) & 1u) << 7); }
__device__ __forceinline__ float signed_by(float v, uint32_t signs, uint32_t j) { return __fmul_rn(v, (signs >> j) & 1u ? -1.0f : 1.0f); }

template <class T>
__device__ __forceinline__ T iq_ldu(const void* p) {
    T v;
    __builtin_memcpy(&v, p, sizeof(T));
    return v;
}
__device__ __forceinline__ float iq_f16(const uint8_t* p) {
    _Float16 h;
    __builtin_memcpy(&h, p, 2);
    return (float)h;
}

// [f16 d][8 x (u32 four grid indices, u32 four 7-bit sign indices | scale << 28)], 66 bytes (dequant.rs:565-596)
__device__ inline float decode_iq2xxs(const uint8_t* row, uint32_t k) {
    const uint8_t* blk = row + (size_t)(k >> 8) * 66u;
    const uint32_t w = k & 255u, ib = w >> 5, l = (w >> 3) & 3u, j = w & 7u;
    const uint32_t aux0 = iq_ldu<uint32_t>(blk + 2u + 8u * ib), aux1 = iq_ldu<uint32_t>(blk + 6u + 8u * ib);
    const float db = __fmul_rn(__fmul_rn(iq_f16(blk), 0.5f + (float)(aux1 >> 28)), 0.25f);
    const float gv = iq2_value(grid_digit2(kIq2xxsGrid, (aux0 >> (8u * l)) & 0xFFu, j));
    return signed_by(__fmul_rn(db, gv), ksigns((aux1 >> (7u * l)) & 127u), j);
}

// [f16 d][32 x u16 (9-bit grid index | 7-bit sign index << 9)][8 scale bytes, a nibble per 16 elements], 74 bytes
// (dequant.rs:605-636)
__device__ inline float decode_iq2xs(const uint8_t* row, uint32_t k) {
    const uint8_t* blk = row + (size_t)(k >> 8) * 74u;
    const uint32_t w = k & 255u, ib = w >> 5, l = (w >> 3) & 3u, j = w & 7u;
    const uint32_t q = iq_ldu<uint16_t>(blk + 2u + 2u * (4u * ib + l)), sc = blk[66u + ib];
    const float db = __fmul_rn(__fmul_rn(iq_f16(blk), 0.5f + (float)(l < 2u ? sc & 0xFu : sc >> 4)), 0.25f);
    const float gv = iq2_value(grid_digit2(kIq2xsGrid, q & 511u, j));
    return signed_by(__fmul_rn(db, gv), ksigns(q >> 9), j);
}

// [f16 d][32 index bytes][32 sign bytes][8 qh: two high index bits per group][8 scale bytes], 82 bytes (dequant.rs:642-676)
__device__ inline float decode_iq2s(const uint8_t* row, uint32_t k) {
    const uint8_t* blk = row + (size_t)(k >> 8) * 82u;
    const uint32_t w = k & 255u, ib = w >> 5, l = (w >> 3) & 3u, j = w & 7u;
    const uint32_t sc = blk[74u + ib], qh = blk[66u + ib];
    const uint32_t e = (uint32_t)blk[2u + 4u * ib + l] | ((qh << (8u - 2u * l)) & 0x300u);
    const float db = __fmul_rn(__fmul_rn(iq_f16(blk), 0.5f + (float)(l < 2u ? sc & 0xFu : sc >> 4)), 0.25f);
    const float gv = iq2_value(grid_digit2(kIq2sGrid, e, j));
    return signed_by(__fmul_rn(db, gv), blk[34u + 4u * ib + l], j);
}

// [f16 d][64 index bytes, two grids of 4 per group][8 x u32 (four 7-bit sign indices | scale << 28)], 98 bytes
// (dequant.rs:685-714)
__device__ inline float decode_iq3xxs(const uint8_t* row, uint32_t k) {
    const uint8_t* blk = row + (size_t)(k >> 8) * 98u;
    const uint32_t w = k & 255u, ib = w >> 5, l = (w >> 3) & 3u, j = w & 7u;
    const uint32_t aux = iq_ldu<uint32_t>(blk + 66u + 4u * ib);
    const float db = __fmul_rn(__fmul_rn(iq_f16(blk), 0.5f + (float)(aux >> 28)), 0.5f);
    const float gv = iq3xxs_value(grid_digit3(kIq3xxsGrid, blk[2u + 8u * ib + 2u * l + (j >> 2)], j & 3u));
    return signed_by(__fmul_rn(db, gv), ksigns((aux >> (7u * l)) & 127u), j);
}

// [f16 d][64 index bytes][8 qh: ninth index bit of the eight grids of a sub-block][32 sign bytes][4 scale bytes, a
// nibble per sub-block], 110 bytes (dequant.rs:724-781)
__device__ inline float decode_iq3s(const uint8_t* row, uint32_t k) {
    const uint8_t* blk = row + (size_t)(k >> 8) * 110u;
    const uint32_t w = k & 255u, ib = w >> 5, l = (w >> 3) & 3u, j = w & 7u, half = j >> 2;
    const uint32_t sc = ((uint32_t)blk[106u + (ib >> 1)] >> (4u * (ib & 1u))) & 0xFu, qh = blk[66u + ib];
    const uint32_t e = (uint32_t)blk[2u + 8u * ib + 2u * l + half] | ((qh << (8u - 2u * l - half)) & 256u);
    const float db = __fmul_rn(iq_f16(blk), 1.0f + 2.0f * (float)sc);
    const float gv = iq3s_value(grid_digit3(kIq3sGrid, e, j & 3u));
    return signed_by(__fmul_rn(db, gv), blk[74u + 4u * ib + l], j);
}

// [f16 d][32 index bytes][8 x u16 qh: four 3-bit high index parts, 3-bit scale at 12, shift sign at 15], 50 bytes
// (dequant.rs:789-824): value = dl * (grid + delta), delta = 0.125 or -0.125
__device__ inline float decode_iq1s(const uint8_t* row, uint32_t k) {
    const uint8_t* blk = row + (size_t)(k >> 8) * 50u;
    const uint32_t w = k & 255u, ib = w >> 5, l = (w >> 3) & 3u, j = w & 7u;
    const uint32_t qh = iq_ldu<uint16_t>(blk + 34u + 2u * ib);
    const float dl = __fmul_rn(iq_f16(blk), 2.0f * (float)((qh >> 12) & 7u) + 1.0f);
    const float delta = qh & 0x8000u ? -0.125f : 0.125f;
    const uint32_t e = (uint32_t)blk[2u + 4u * ib + l] | (((qh >> (3u * l)) & 7u) << 8);
    return __fmul_rn(dl, __fadd_rn(iq1_value(grid_digit2(kIq1sGrid, e, j)), delta));
}

// [32 index bytes][16 qh: per group 3 high index bits and the shift sign in a nibble][4 x u16: four 3-bit scales and,
// in the top nibbles, the block's f16 d], 56 bytes (dequant.rs:838-916)
__device__ inline float decode_iq1m(const uint8_t* row, uint32_t k) {
    const uint8_t* blk = row + (size_t)(k >> 8) * 56u;
    const uint32_t w = k & 255u, ib = w >> 5, l = (w >> 3) & 3u, j = w & 7u;
    const uint32_t s0 = iq_ldu<uint16_t>(blk + 48), s1 = iq_ldu<uint16_t>(blk + 50), s2 = iq_ldu<uint16_t>(blk + 52),
                   s3 = iq_ldu<uint16_t>(blk + 54);
    const uint16_t dbits = (uint16_t)((s0 >> 12) | ((s1 >> 8) & 0x00F0u) | ((s2 >> 4) & 0x0F00u) | (s3 & 0xF000u));
    _Float16 dh;
    __builtin_memcpy(&dh, &dbits, 2);
    const uint32_t sc = iq_ldu<uint16_t>(blk + 48u + 2u * (ib >> 1));
    const float dl = __fmul_rn((float)dh, 2.0f * (float)((sc >> (6u * (ib & 1u) + 3u * (l >> 1))) & 7u) + 1.0f);
    const uint32_t qh = blk[32u + 2u * ib + (l >> 1)];
    const uint32_t e = (uint32_t)blk[4u * ib + l] | ((qh << (l & 1u ? 4u : 8u)) & 0x700u);
    const float delta = qh & (l & 1u ? 0x80u : 0x08u) ? -0.125f : 0.125f;
    return __fmul_rn(dl, __fadd_rn(iq1_value(grid_digit2(kIq1sGrid, e, j)), delta));
}

}  // namespace infr

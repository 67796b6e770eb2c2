// One decoder for every affine GGUF format (Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q2_K, Q3_K, Q4_K, Q5_K, Q6_K)
// and for the formats whose value is a scale times a small signed code (IQ4_NL, IQ4_XS, MXFP4, NVFP4 with
// their 16-entry books, the ternary TQ1_0, TQ2_0, Q2_0, and the lattice-codebook IQ2_XXS, IQ2_XS, IQ2_S, IQ3_XXS,
// IQ3_S, IQ1_S, IQ1_M), which become affine once the code is shifted
// to an unsigned byte: scale * code = scale * (code + bias) + (-bias * scale), every product exact.
// A row is cut into 32-element units; a unit decodes to 32 unsigned byte codes (eight dwords) plus one
// (scale, min) pair per 16 elements, value(e) = sc[e / 16] * code(e) + mn[e / 16].  The formats only differ
// in how the eight dwords and the two pairs are cut out of the block
// (crates/infr-gguf/src/dequant.rs:137-389, :499-559, :926-1073).
#pragma once

#include "device_common.h"

namespace infr {

struct Unit {
    uint32_t q[8];       // element 4k + b of the unit = byte b of q[k]
    float sc[2], mn[2];  // halves of 16 elements
};

// Every format with a unit decoder.
#define INFR_FOR_UNIT_FORMATS(X)                                                                          \
    X(INFR_Q4_0) X(INFR_Q4_1) X(INFR_Q5_0) X(INFR_Q5_1) X(INFR_Q8_0) X(INFR_Q2K) X(INFR_Q3K) X(INFR_Q4K) \
    X(INFR_Q5K) X(INFR_Q6K) X(INFR_IQ4_NL) X(INFR_IQ4_XS) X(INFR_TQ1_0) X(INFR_TQ2_0) X(INFR_Q2_0)       \
    X(INFR_MXFP4) X(INFR_NVFP4) X(INFR_IQ2_XXS) X(INFR_IQ2_XS) X(INFR_IQ2_S) X(INFR_IQ3_XXS) X(INFR_IQ3_S)       \
    X(INFR_IQ1_S) X(INFR_IQ1_M)

// Elements of one block of a unit format (a row is a whole number of blocks), 0 for any other dtype.
inline int unit_format_block(int dt) {
    switch (dt) {
        case INFR_Q4_0: case INFR_Q4_1: case INFR_Q5_0: case INFR_Q5_1: case INFR_Q8_0: case INFR_IQ4_NL: case INFR_MXFP4: return 32;
        case INFR_Q2_0: case INFR_NVFP4: return 64;
        case INFR_Q2K: case INFR_Q3K: case INFR_Q4K: case INFR_Q5K: case INFR_Q6K: case INFR_IQ4_XS: case INFR_TQ1_0:
        case INFR_TQ2_0: case INFR_IQ2_XXS: case INFR_IQ2_XS: case INFR_IQ2_S: case INFR_IQ3_XXS: case INFR_IQ3_S: case INFR_IQ1_S:
        case INFR_IQ1_M: return 256;
        default: return 0;
    }
}

constexpr uint32_t kLo4 = 0x0F0F0F0Fu, kB0 = 0x01010101u;

// bits 0..3 of t to bit 0 of bytes 0..3 (the four shifted copies of t do not overlap)
__device__ __forceinline__ uint32_t spread4(uint32_t t) { return ((t & 0xFu) * 0x00204081u) & kB0; }

// Sixteen-entry byte table applied to the four nibbles held in the low halves of w's bytes: t0..t3 hold
// entries 0-3, 4-7, 8-11, 12-15.  v_perm_b32 looks up eight entries at a time; bit 3 of the nibble picks
// between the two looks.
__device__ __forceinline__ uint32_t book4(uint32_t w, uint32_t t0, uint32_t t1, uint32_t t2, uint32_t t3) {
    const uint32_t sel = w & 0x07070707u;
    const uint32_t lo = __builtin_amdgcn_perm(t1, t0, sel), hi = __builtin_amdgcn_perm(t3, t2, sel);
    const uint32_t b3 = (w >> 3) & kB0, m = (b3 << 8) - b3;   // 0xFF in the bytes whose nibble has bit 3 set
    return lo ^ ((lo ^ hi) & m);
}
// IQ4_NL book + 127 and twice-E2M1 book + 12 as unsigned bytes.
__device__ __forceinline__ uint32_t iq4nl4(uint32_t w) { return book4(w, 0x3E2C1700u, 0x75695C4Eu, 0xA5988C80u, 0xF0D8C4B4u); }
__device__ __forceinline__ uint32_t fp4x4(uint32_t w) { return book4(w, 0x0F0E0D0Cu, 0x18141210u, 0x090A0B0Cu, 0x00040608u); }

// The four 2-bit fields of byte b of w, one per byte.
__device__ __forceinline__ uint32_t fields4(uint32_t w, int b) {
    const uint32_t x = (w >> (8 * b)) & 0xFFu;
    return (x | (x << 6) | (x << 12) | (x << 18)) & 0x03030303u;
}
// Ternary digit `pow3` of each byte of w (TQ1_0), one per byte.
__device__ __forceinline__ uint32_t trits4(uint32_t w, uint32_t pow3) {
    uint32_t r = 0;
#pragma unroll
    for (int b = 0; b < 4; b++) r |= trit((w >> (8 * b)) & 0xFFu, pow3) << (8 * b);
    return r;
}

// The lattice formats: a codebook entry is 8 (4) digits of 2 (3) bits; the digits of four elements become the byte
// selectors of one v_perm_b32 over the alphabet, then every byte is mirrored around `off` where its sign bit is set.
__device__ __forceinline__ uint32_t digits2(uint32_t x) { x &= 0xFFu; return (x | (x << 6) | (x << 12) | (x << 18)) & 0x03030303u; }
__device__ __forceinline__ uint32_t digits3(uint32_t x) {
    return (x & 7u) | ((x & 0x38u) << 5) | ((x & 0x1C0u) << 10) | ((x & 0xE00u) << 15);
}
// off + mag in the bytes whose bit of s (bits 0..3) is clear, off - mag in the others; mag <= off in every byte
__device__ __forceinline__ uint32_t mirrored4(uint32_t mag4, uint32_t off4, uint32_t s) {
    const uint32_t b = spread4(s), m = (b << 8) - b;
    return ((off4 + mag4) & ~m) | ((off4 - mag4) & m);
}
__device__ __forceinline__ uint32_t iq2_mag4(uint32_t digits8) { return __builtin_amdgcn_perm(0u, 0x002B1908u, digits2(digits8)); }
__device__ __forceinline__ uint32_t iq3xxs_mag4(uint32_t digits12) { return __builtin_amdgcn_perm(0x3E342C24u, 0x1C140C04u, digits3(digits12)); }
__device__ __forceinline__ uint32_t iq3s_mag4(uint32_t digits12) { return __builtin_amdgcn_perm(0x0F0D0B09u, 0x07050301u, digits3(digits12)); }
// IQ1: value = dl * (g + delta), g in {0, 1, -1}, delta = +-1/8, as (dl / 8) * (code - 9), code = 8 g + 8 delta + 9
__device__ __forceinline__ uint32_t iq1_code4(uint32_t digits8, bool neg_delta) {
    return __builtin_amdgcn_perm(0u, neg_delta ? 0x00001008u : 0x0002120Au, digits2(digits8));
}

// Unit u of a row that starts at `row`.
template <int DT>
__device__ __forceinline__ void load_unit(const uint8_t* __restrict__ row, int u, Unit& t) {
    if constexpr (DT == INFR_Q4_0 || DT == INFR_Q4_1 || DT == INFR_Q5_0 || DT == INFR_Q5_1) {
        constexpr bool has_m = DT == INFR_Q4_1 || DT == INFR_Q5_1, five = DT == INFR_Q5_0 || DT == INFR_Q5_1;
        constexpr int bb = 18 + (has_m ? 2 : 0) + (five ? 4 : 0);
        const uint8_t* blk = row + (size_t)u * bb;
        const uint32_t hdr = has_m ? ldu<uint32_t>(blk) : (uint32_t)ldu<uint16_t>(blk);
        const uint8_t* p = blk + (has_m ? 4 : 2);
        uint32_t qh = 0;
        if constexpr (five) {
            qh = ldu<uint32_t>(p);
            p += 4;
        }
        const uint4 qs = ldu<uint4>(p);
        const uint32_t w[4] = {qs.x, qs.y, qs.z, qs.w};
#pragma unroll
        for (int k = 0; k < 4; k++) {
            t.q[k] = w[k] & kLo4;
            t.q[4 + k] = (w[k] >> 4) & kLo4;
            if constexpr (five) {
                t.q[k] |= spread4(qh >> (4 * k)) << 4;
                t.q[4 + k] |= spread4(qh >> (16 + 4 * k)) << 4;
            }
        }
        const float d = f16_bits_to_f32(hdr & 0xFFFFu);
        t.sc[0] = t.sc[1] = d;
        t.mn[0] = t.mn[1] = has_m ? f16_bits_to_f32(hdr >> 16) : d * (five ? -16.0f : -8.0f);
    } else if constexpr (DT == INFR_Q8_0) {
        const uint8_t* blk = row + (size_t)u * 34;
        const float d = f16_bits_to_f32(ldu<uint16_t>(blk));
        const uint4 a = ldu<uint4>(blk + 2), b = ldu<uint4>(blk + 18);
        const uint32_t w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
        for (int k = 0; k < 8; k++) t.q[k] = w[k] ^ 0x80808080u;   // q + 128 as an unsigned byte
        t.sc[0] = t.sc[1] = d;
        t.mn[0] = t.mn[1] = d * -128.0f;
    } else if constexpr (DT == INFR_Q2K || DT == INFR_Q3K) {
        // unit s of a block: 16-element groups 2s, 2s+1 = the 2-bit fields at shift 2*(s%4) of qs[32*(s/4) ..+32)
        constexpr int bb = DT == INFR_Q2K ? 84 : 110;
        const uint8_t* blk = row + (size_t)(u >> 3) * bb;
        const int s = u & 7, n = s >> 2, j = s & 3;
        const uint8_t* qs = blk + (DT == INFR_Q2K ? 16 : 32) + 32 * n;
        const uint4 a = ldu<uint4>(qs), b = ldu<uint4>(qs + 16);
        const uint32_t w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
        for (int k = 0; k < 8; k++) t.q[k] = (w[k] >> (2 * j)) & 0x03030303u;
        if constexpr (DT == INFR_Q2K) {
            const uint32_t sb = ldu<uint16_t>(blk + 2 * s);
            const uint32_t dd = ldu<uint32_t>(blk + 80);
            const float d = f16_bits_to_f32(dd & 0xFFFFu), dmin = f16_bits_to_f32(dd >> 16);
            t.sc[0] = d * (float)(sb & 0xFu);
            t.mn[0] = dmin * (float)(-(int)((sb >> 4) & 0xFu));
            t.sc[1] = d * (float)((sb >> 8) & 0xFu);
            t.mn[1] = dmin * (float)(-(int)(sb >> 12));
        } else {
            const uint4 ha = ldu<uint4>(blk), hb = ldu<uint4>(blk + 16);
            const uint32_t hm[8] = {ha.x, ha.y, ha.z, ha.w, hb.x, hb.y, hb.z, hb.w};
#pragma unroll
            for (int k = 0; k < 8; k++) t.q[k] |= ((hm[k] >> (4 * n + j)) & kB0) << 2;
            const float d = f16_bits_to_f32(ldu<uint16_t>(blk + 108));
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const int g = 2 * s + h;   // 6-bit scale g: nibble g/8 of byte g%8, high bits = field g/4 of byte 8 + g%4
                const uint32_t lo = ((uint32_t)blk[96 + (g & 7)] >> (g >= 8 ? 4 : 0)) & 0xFu;
                const uint32_t hi = ((uint32_t)blk[104 + (g & 3)] >> (2 * (g >> 2))) & 3u;
                const float sc = d * (float)((int)(lo | (hi << 4)) - 32);
                t.sc[h] = sc;
                t.mn[h] = -4.0f * sc;
            }
        }
    } else if constexpr (DT == INFR_Q4K || DT == INFR_Q5K) {
        // unit s = sub-block s: nibble s%2 of qs[32*(s/2) ..+32); Q5_K adds bit s of qh[l]
        constexpr int bb = DT == INFR_Q4K ? 144 : 176;
        const uint8_t* blk = row + (size_t)(u >> 3) * bb;
        const int s = u & 7;
        const uint8_t* qs = blk + (DT == INFR_Q4K ? 16 : 48) + 32 * (s >> 1);
        const uint4 a = ldu<uint4>(qs), b = ldu<uint4>(qs + 16);
        const uint32_t w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
        for (int k = 0; k < 8; k++) t.q[k] = (w[k] >> (4 * (s & 1))) & kLo4;
        if constexpr (DT == INFR_Q5K) {
            const uint4 ha = ldu<uint4>(blk + 16), hb = ldu<uint4>(blk + 32);
            const uint32_t hq[8] = {ha.x, ha.y, ha.z, ha.w, hb.x, hb.y, hb.z, hb.w};
#pragma unroll
            for (int k = 0; k < 8; k++) t.q[k] |= ((hq[k] >> s) & kB0) << 4;
        }
        uint32_t sc, m;
        k4(s, blk + 4, sc, m);
        const uint32_t dd = ldu<uint32_t>(blk);
        t.sc[0] = t.sc[1] = f16_bits_to_f32(dd & 0xFFFFu) * (float)sc;
        t.mn[0] = t.mn[1] = f16_bits_to_f32(dd >> 16) * (float)(-(int)m);
    } else if constexpr (DT == INFR_IQ4_NL || DT == INFR_MXFP4) {
        constexpr bool fp4 = DT == INFR_MXFP4;
        const uint8_t* blk = row + (size_t)u * (fp4 ? 17 : 18);
        const uint4 qs = ldu<uint4>(blk + (fp4 ? 1 : 2));
        const uint32_t w[4] = {qs.x, qs.y, qs.z, qs.w};
#pragma unroll
        for (int k = 0; k < 4; k++) {
            t.q[k] = fp4 ? fp4x4(w[k] & kLo4) : iq4nl4(w[k] & kLo4);
            t.q[4 + k] = fp4 ? fp4x4((w[k] >> 4) & kLo4) : iq4nl4((w[k] >> 4) & kLo4);
        }
        const float d = fp4 ? e8m0_half(blk[0]) : f16_bits_to_f32(ldu<uint16_t>(blk));
        t.sc[0] = t.sc[1] = d;
        t.mn[0] = t.mn[1] = d * (fp4 ? -12.0f : -127.0f);
    } else if constexpr (DT == INFR_IQ4_XS) {
        const uint8_t* blk = row + (size_t)(u >> 3) * 136;
        const int s = u & 7;
        const uint4 qs = ldu<uint4>(blk + 8 + 16 * s);
        const uint32_t w[4] = {qs.x, qs.y, qs.z, qs.w};
#pragma unroll
        for (int k = 0; k < 4; k++) {
            t.q[k] = iq4nl4(w[k] & kLo4);
            t.q[4 + k] = iq4nl4((w[k] >> 4) & kLo4);
        }
        const uint32_t hdr = ldu<uint32_t>(blk);   // d | scales_h << 16
        const uint32_t ls = (((uint32_t)blk[4 + (s >> 1)] >> (4 * (s & 1))) & 0xFu) | (((hdr >> (16 + 2 * s)) & 3u) << 4);
        const float dl = f16_bits_to_f32(hdr & 0xFFFFu) * (float)((int)ls - 32);
        t.sc[0] = t.sc[1] = dl;
        t.mn[0] = t.mn[1] = dl * -127.0f;
    } else if constexpr (DT == INFR_NVFP4) {
        // unit = sub-blocks 2 * half, 2 * half + 1 of a 64-element block, each the low then the high nibbles of 8 bytes
        const uint8_t* blk = row + (size_t)(u >> 1) * 36;
        const int half = u & 1;
        const uint4 qs = ldu<uint4>(blk + 4 + 16 * half);
        const uint32_t w[4] = {qs.x, qs.y, qs.z, qs.w};
#pragma unroll
        for (int h = 0; h < 2; h++) {
            t.q[4 * h] = fp4x4(w[2 * h] & kLo4);
            t.q[4 * h + 1] = fp4x4(w[2 * h + 1] & kLo4);
            t.q[4 * h + 2] = fp4x4((w[2 * h] >> 4) & kLo4);
            t.q[4 * h + 3] = fp4x4((w[2 * h + 1] >> 4) & kLo4);
            const float d = ue4m3_half(blk[2 * half + h]);
            t.sc[h] = d;
            t.mn[h] = d * -12.0f;
        }
    } else if constexpr (DT == INFR_TQ2_0) {
        // unit s: field s % 4 of qs[32 * (s / 4) ..+32)
        const uint8_t* blk = row + (size_t)(u >> 3) * 66;
        const int s = u & 7;
        const uint4 a = ldu<uint4>(blk + 32 * (s >> 2)), b = ldu<uint4>(blk + 32 * (s >> 2) + 16);
        const uint32_t w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
        for (int k = 0; k < 8; k++) t.q[k] = (w[k] >> (2 * (s & 3))) & 0x03030303u;
        const float d = f16_bits_to_f32(ldu<uint16_t>(blk + 64));
        t.sc[0] = t.sc[1] = d;
        t.mn[0] = t.mn[1] = -d;
    } else if constexpr (DT == INFR_Q2_0) {
        // unit = half of a 64-element block: the four fields of each of 8 bytes, in order
        const uint8_t* blk = row + (size_t)(u >> 1) * 18;
        const uint2 qs = ldu<uint2>(blk + 2 + 8 * (u & 1));
#pragma unroll
        for (int k = 0; k < 4; k++) {
            t.q[k] = fields4(qs.x, k);
            t.q[4 + k] = fields4(qs.y, k);
        }
        const float d = f16_bits_to_f32(ldu<uint16_t>(blk));
        t.sc[0] = t.sc[1] = d;
        t.mn[0] = t.mn[1] = -d;
    } else if constexpr (DT == INFR_TQ1_0) {
        // units 0-4: digit s of qs[0..32); 5, 6: digits 2 (s - 5), 2 (s - 5) + 1 of qs[32..48); 7: digit 4 of
        // qs[32..48), then digits 0-3 of qh[0..4)
        const uint8_t* blk = row + (size_t)(u >> 3) * 54;
        const int s = u & 7;
        constexpr uint32_t p3[6] = {1, 3, 9, 27, 81, 243};
        if (s < 5) {
            const uint4 a = ldu<uint4>(blk), b = ldu<uint4>(blk + 16);
            const uint32_t w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
            const uint32_t p = s == 0 ? 1u : s == 1 ? 3u : s == 2 ? 9u : s == 3 ? 27u : 81u;
#pragma unroll
            for (int k = 0; k < 8; k++) t.q[k] = trits4(w[k], p);
        } else {
            const uint4 a = ldu<uint4>(blk + 32);
            const uint32_t w[4] = {a.x, a.y, a.z, a.w};
            const uint32_t pa = s == 5 ? 1u : s == 6 ? 9u : 81u, pb = s == 5 ? 3u : 27u;
            const uint32_t qh = ldu<uint32_t>(blk + 48);
#pragma unroll
            for (int k = 0; k < 4; k++) {
                t.q[k] = trits4(w[k], pa);
                t.q[4 + k] = s == 7 ? trits4(qh, p3[k]) : trits4(w[k], pb);
            }
        }
        const float d = f16_bits_to_f32(ldu<uint16_t>(blk + 52));
        t.sc[0] = t.sc[1] = d;
        t.mn[0] = t.mn[1] = -d;
    } else if constexpr (DT == INFR_IQ2_XXS || DT == INFR_IQ2_XS || DT == INFR_IQ2_S) {
        // unit s = sub-block s; group l of 8 elements -> q[2l], q[2l + 1] (dequant.rs:565-676)
        constexpr int bb = DT == INFR_IQ2_XXS ? 66 : DT == INFR_IQ2_XS ? 74 : 82;
        const uint8_t* blk = row + (size_t)(u >> 3) * bb;
        const int s = u & 7;
        const float d = f16_bits_to_f32(ldu<uint16_t>(blk));
        uint32_t idx[4], sg[4], m0, m1;
        if constexpr (DT == INFR_IQ2_XXS) {
            const uint2 aux = ldu<uint2>(blk + 2 + 8 * s);
#pragma unroll
            for (int l = 0; l < 4; l++) {
                idx[l] = kIq2xxsGrid[(aux.x >> (8 * l)) & 0xFFu];
                sg[l] = ksigns((aux.y >> (7 * l)) & 127u);
            }
            m0 = m1 = aux.y >> 28;
        } else if constexpr (DT == INFR_IQ2_XS) {
            const uint2 q = ldu<uint2>(blk + 2 + 8 * s);
            const uint32_t w[4] = {q.x & 0xFFFFu, q.x >> 16, q.y & 0xFFFFu, q.y >> 16};
#pragma unroll
            for (int l = 0; l < 4; l++) {
                idx[l] = kIq2xsGrid[w[l] & 511u];
                sg[l] = ksigns(w[l] >> 9);
            }
            const uint32_t sb = blk[66 + s];
            m0 = sb & 0xFu;
            m1 = sb >> 4;
        } else {
            const uint32_t qs = ldu<uint32_t>(blk + 2 + 4 * s), sn = ldu<uint32_t>(blk + 34 + 4 * s), qh = blk[66 + s];
#pragma unroll
            for (int l = 0; l < 4; l++) {
                idx[l] = kIq2sGrid[((qs >> (8 * l)) & 0xFFu) | ((qh << (8 - 2 * l)) & 0x300u)];
                sg[l] = (sn >> (8 * l)) & 0xFFu;
            }
            const uint32_t sb = blk[74 + s];
            m0 = sb & 0xFu;
            m1 = sb >> 4;
        }
#pragma unroll
        for (int l = 0; l < 4; l++) {
            t.q[2 * l] = mirrored4(iq2_mag4(idx[l]), 0x2B2B2B2Bu, sg[l]);
            t.q[2 * l + 1] = mirrored4(iq2_mag4(idx[l] >> 8), 0x2B2B2B2Bu, sg[l] >> 4);
        }
        t.sc[0] = d * (0.5f + (float)m0) * 0.25f;
        t.sc[1] = d * (0.5f + (float)m1) * 0.25f;
        t.mn[0] = -43.0f * t.sc[0];
        t.mn[1] = -43.0f * t.sc[1];
    } else if constexpr (DT == INFR_IQ3_XXS || DT == INFR_IQ3_S) {
        // two 4-element entries per group of 8 (dequant.rs:685-781)
        constexpr bool xxs = DT == INFR_IQ3_XXS;
        const uint8_t* blk = row + (size_t)(u >> 3) * (xxs ? 98 : 110);
        const int s = u & 7;
        const float d = f16_bits_to_f32(ldu<uint16_t>(blk));
        const uint2 qs = ldu<uint2>(blk + 2 + 8 * s);
        const uint32_t w[2] = {qs.x, qs.y};
        float db;
        if constexpr (xxs) {
            const uint32_t aux = ldu<uint32_t>(blk + 66 + 4 * s);
#pragma unroll
            for (int l = 0; l < 4; l++) {
                const uint32_t sg = ksigns((aux >> (7 * l)) & 127u), pair = w[l >> 1] >> (16 * (l & 1));
                t.q[2 * l] = mirrored4(iq3xxs_mag4(kIq3xxsGrid[pair & 0xFFu]), 0x3E3E3E3Eu, sg);
                t.q[2 * l + 1] = mirrored4(iq3xxs_mag4(kIq3xxsGrid[(pair >> 8) & 0xFFu]), 0x3E3E3E3Eu, sg >> 4);
            }
            db = d * (0.5f + (float)(aux >> 28)) * 0.5f;
            t.mn[0] = t.mn[1] = -62.0f * db;
        } else {
            const uint32_t qh = blk[66 + s], sn = ldu<uint32_t>(blk + 74 + 4 * s);
#pragma unroll
            for (int l = 0; l < 4; l++) {
                const uint32_t sg = (sn >> (8 * l)) & 0xFFu, pair = w[l >> 1] >> (16 * (l & 1));
                t.q[2 * l] = mirrored4(iq3s_mag4(kIq3sGrid[(pair & 0xFFu) | ((qh << (8 - 2 * l)) & 256u)]), 0x0F0F0F0Fu, sg);
                t.q[2 * l + 1] = mirrored4(iq3s_mag4(kIq3sGrid[((pair >> 8) & 0xFFu) | ((qh << (7 - 2 * l)) & 256u)]), 0x0F0F0F0Fu, sg >> 4);
            }
            db = d * (1.0f + 2.0f * (float)(((uint32_t)blk[106 + (s >> 1)] >> (4 * (s & 1))) & 0xFu));
            t.mn[0] = t.mn[1] = -15.0f * db;
        }
        t.sc[0] = t.sc[1] = db;
    } else if constexpr (DT == INFR_IQ1_S) {
        // (dequant.rs:789-824)
        const uint8_t* blk = row + (size_t)(u >> 3) * 50;
        const int s = u & 7;
        const uint32_t qs = ldu<uint32_t>(blk + 2 + 4 * s), qh = ldu<uint16_t>(blk + 34 + 2 * s);
        const bool neg = (qh & 0x8000u) != 0;
#pragma unroll
        for (int l = 0; l < 4; l++) {
            const uint32_t g = kIq1sGrid[((qs >> (8 * l)) & 0xFFu) | (((qh >> (3 * l)) & 7u) << 8)];
            t.q[2 * l] = iq1_code4(g, neg);
            t.q[2 * l + 1] = iq1_code4(g >> 8, neg);
        }
        const float sc = f16_bits_to_f32(ldu<uint16_t>(blk)) * (2.0f * (float)((qh >> 12) & 7u) + 1.0f) * 0.125f;
        t.sc[0] = t.sc[1] = sc;
        t.mn[0] = t.mn[1] = -9.0f * sc;
    } else if constexpr (DT == INFR_IQ1_M) {
        // (dequant.rs:838-916)
        const uint8_t* blk = row + (size_t)(u >> 3) * 56;
        const int s = u & 7;
        const uint32_t qs = ldu<uint32_t>(blk + 4 * s), qh = ldu<uint16_t>(blk + 32 + 2 * s);
        const uint2 scw = ldu<uint2>(blk + 48);
        const uint32_t dbits = ((scw.x >> 12) & 0xFu) | ((scw.x >> 24) & 0xF0u) | ((scw.y >> 4) & 0xF00u) | ((scw.y >> 16) & 0xF000u);
        const uint32_t word = ((s >> 1) & 1 ? (s >> 2 ? scw.y >> 16 : scw.x >> 16) : (s >> 2 ? scw.y : scw.x)) & 0xFFFFu;
#pragma unroll
        for (int l = 0; l < 4; l++) {
            const uint32_t nib = (qh >> (4 * l)) & 0xFu;    // low nibble of qh[0], high nibble, then qh[1]'s
            const uint32_t g = kIq1sGrid[((qs >> (8 * l)) & 0xFFu) | ((nib & 7u) << 8)];
            t.q[2 * l] = iq1_code4(g, (nib & 8u) != 0);
            t.q[2 * l + 1] = iq1_code4(g >> 8, (nib & 8u) != 0);
        }
        const float d8 = f16_bits_to_f32(dbits) * 0.125f;
        t.sc[0] = d8 * (2.0f * (float)((word >> (6 * (s & 1))) & 7u) + 1.0f);
        t.sc[1] = d8 * (2.0f * (float)((word >> (6 * (s & 1) + 3)) & 7u) + 1.0f);
        t.mn[0] = -9.0f * t.sc[0];
        t.mn[1] = -9.0f * t.sc[1];
    } else {   // Q6_K: unit s: half s/4, group g = s%4: ql[64*half + 32*(g&1) + l] nibble g/2, qh[32*half + l] field g
        static_assert(DT == INFR_Q6K, "format without a unit decoder");
        const uint8_t* blk = row + (size_t)(u >> 3) * 210;
        const int s = u & 7, half = s >> 2, g = s & 3;
        const uint8_t* ql = blk + 64 * half + 32 * (g & 1);
        const uint8_t* qh = blk + 128 + 32 * half;
        const uint4 a = ldu<uint4>(ql), b = ldu<uint4>(ql + 16), ha = ldu<uint4>(qh), hb = ldu<uint4>(qh + 16);
        const uint32_t w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
        const uint32_t hq[8] = {ha.x, ha.y, ha.z, ha.w, hb.x, hb.y, hb.z, hb.w};
#pragma unroll
        for (int k = 0; k < 8; k++) t.q[k] = ((w[k] >> (4 * (g >> 1))) & kLo4) | (((hq[k] >> (2 * g)) & 0x03030303u) << 4);
        const float d = f16_bits_to_f32(ldu<uint16_t>(blk + 208));
        const uint32_t sb = ldu<uint16_t>(blk + 192 + 8 * half + 2 * g);
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const float sc = d * (float)(int)(int8_t)((sb >> (8 * h)) & 0xFFu);
            t.sc[h] = sc;
            t.mn[h] = -32.0f * sc;
        }
    }
}

}  // namespace infr

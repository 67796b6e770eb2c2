// One decoder for every affine GGUF format (Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q2_K, Q3_K, Q4_K, Q5_K, Q6_K)
// and for the formats whose value is a scale times a small signed code (IQ4_NL, IQ4_XS, MXFP4, NVFP4 with
// their 16-entry books, the ternary TQ1_0, TQ2_0, Q2_0), which become affine once the code is shifted
// to an unsigned byte: scale * code = scale * (code + bias) + (-bias * scale), every product exact.  A row is cut into 32-element units; a unit decodes to 32 unsigned byte codes (eight dwords) plus one
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
    X(INFR_MXFP4) X(INFR_NVFP4)

// Elements of one block of a unit format (a row is a whole number of blocks), 0 for any other dtype.
inline int unit_format_block(int dt) {
    switch (dt) {
        case INFR_Q4_0: case INFR_Q4_1: case INFR_Q5_0: case INFR_Q5_1: case INFR_Q8_0: case INFR_IQ4_NL: case INFR_MXFP4: return 32;
        case INFR_Q2_0: case INFR_NVFP4: return 64;
        case INFR_Q2K: case INFR_Q3K: case INFR_Q4K: case INFR_Q5K: case INFR_Q6K: case INFR_IQ4_XS: case INFR_TQ1_0:
        case INFR_TQ2_0: return 256;
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

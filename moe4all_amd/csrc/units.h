// One decoder for every affine GGUF format (Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q2_K, Q3_K, Q4_K, Q5_K, Q6_K):
// a row is cut into 32-element units; a unit decodes to 32 unsigned byte codes (eight dwords) plus one
// (scale, min) pair per 16 elements, value(e) = sc[e / 16] * code(e) + mn[e / 16].  The formats only differ
// in how the eight dwords and the two pairs are cut out of the block
// (crates/infr-gguf/src/dequant.rs:137-389).
#pragma once

#include "device_common.h"

namespace infr {

struct Unit {
    uint32_t q[8];       // element 4k + b of the unit = byte b of q[k]
    float sc[2], mn[2];  // halves of 16 elements
};

constexpr uint32_t kLo4 = 0x0F0F0F0Fu, kB0 = 0x01010101u;

// bits 0..3 of t to bit 0 of bytes 0..3 (the four shifted copies of t do not overlap)
__device__ __forceinline__ uint32_t spread4(uint32_t t) { return ((t & 0xFu) * 0x00204081u) & kB0; }

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

// Inner products of the decode-regime kernels: activation rows staged as 23-bit fixed point in
// LDS cells, packed GGUF weight codes contracted against them with V_DOT4, block scales applied
// in f32 in factored form.  Shared by the register-streaming kernels (k_gemv.hip) and the
// LDS-staged single-token kernels (k_decode.hip).
#pragma once

#include "device_common.h"
#include "kernels.h"

namespace infr {

__device__ __forceinline__ int dot4i(uint32_t a, uint32_t b, int c) {
    return __builtin_amdgcn_sdot4((int)a, (int)b, c, false);
}

// ---- activation staging -------------------------------------------------------------------
// A wavefront converts the activation vector once, cooperatively, into LDS "cells" of 32
// elements (28 dwords: byte planes A, B, C of the fixed-point values, then scales and sums),
// and each lane then fetches the cells of its own K slice.  Element 4k+q of a group sits in
// byte q of dword k of each plane, the order in which byte-parallel unpacking yields codes.
//   G == 32: [A 8][B 8][C 8][scale][sum][pad 2]            one group of 32
//   G == 16: [A0 4][B0 4][C0 4][A1 4][B1 4][C1 4][k0][s0][k1][s1]   two groups of 16
// SIGNED digits (X = 65536*A + 256*B + C with every digit in [-128,127]) serve signed weight
// codes; otherwise B and C are the plain unsigned bytes of X's two's complement (A signed),
// which costs no arithmetic to extract and pairs with the unsigned dot for non-negative codes.
constexpr int kCellDwords = 28;

__device__ __forceinline__ uint32_t perm(uint32_t hi, uint32_t lo, uint32_t sel) {
    return __builtin_amdgcn_perm(hi, lo, sel);
}

// Byte `B` of four dwords -> one dword (x0's byte in byte 0).
template <int B>
__device__ __forceinline__ uint32_t gather_byte(uint32_t x0, uint32_t x1, uint32_t x2, uint32_t x3) {
    // v_perm_b32 selects bytes from {hi,lo}: selector values 0-3 = lo bytes, 4-7 = hi bytes
    const uint32_t lo = perm(x1, x0, (uint32_t)(B | ((4 + B) << 8)));          // [x0.B, x1.B, -, -]
    const uint32_t hi = perm(x3, x2, (uint32_t)(B | ((4 + B) << 8)));          // [x2.B, x3.B, -, -]
    return perm(hi, lo, 0x05040100u);                                          // [lo.0, lo.1, hi.0, hi.1]
}

// Power-of-two scaling of a group whose largest magnitude has the bit pattern `amax_bits`:
// |x| * inv < 2^21 and scale = 1 / inv.  Groups below 2^-105 are flushed to zero (inv = scale = 0);
// a group that holds a NaN or an infinity gets scale = NaN, so every output that reads the group
// becomes NaN, as an f32 dot product over it would be non-finite.
struct GroupScale { float inv, scale; };
__device__ __forceinline__ GroupScale group_scale(uint32_t amax_bits) {
    const uint32_t eb = amax_bits >> 23;  // amax in [2^(eb-127), 2^(eb-126))
    GroupScale g;
    const bool live = eb >= 22u && eb < 255u;
    g.inv = live ? __uint_as_float((274u - eb) << 23) : 0.f;   // 2^(20 - E)
    g.scale = eb == 255u ? __uint_as_float(0x7FC00000u) : live ? __uint_as_float((eb - 20u) << 23) : 0.f;  // 2^(E - 20)
    return g;
}

template <int N, bool SIGNED>
__device__ __forceinline__ void quant_to_cell(const float* x, uint32_t* a, uint32_t* b, uint32_t* c, uint32_t* ks) {
    // largest magnitude as an integer: NaN and Inf patterns order above every finite value, so a
    // group holding either is seen (fmaxf would drop a NaN)
    uint32_t amax = 0u;
#pragma unroll
    for (int i = 0; i < N; i++) amax = max(amax, __float_as_uint(x[i]) & 0x7FFFFFFFu);
    const GroupScale gs = group_scale(amax);
    const float inv = gs.inv, scale = gs.scale;
    int sx = 0;
#pragma unroll
    for (int k = 0; k < N / 4; k++) {
        int X[4];
#pragma unroll
        for (int q = 0; q < 4; q++) {
            X[q] = __float2int_rn(x[4 * k + q] * inv);  // exact scaling, |X| <= 2^21
            sx += X[q];
        }
        if (SIGNED) {
            uint32_t aw = 0, bw = 0, cw = 0;
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const int C = (int)(int8_t)(X[q] & 0xFF);
                const int R = (X[q] - C) >> 8;
                const int B = (int)(int8_t)(R & 0xFF);
                const int A = (R - B) >> 8;
                aw |= (uint32_t)(A & 0xFF) << (8 * q);
                bw |= (uint32_t)(B & 0xFF) << (8 * q);
                cw |= (uint32_t)(C & 0xFF) << (8 * q);
            }
            a[k] = aw; b[k] = bw; c[k] = cw;
        } else {
            a[k] = gather_byte<2>((uint32_t)X[0], (uint32_t)X[1], (uint32_t)X[2], (uint32_t)X[3]);
            b[k] = gather_byte<1>((uint32_t)X[0], (uint32_t)X[1], (uint32_t)X[2], (uint32_t)X[3]);
            c[k] = gather_byte<0>((uint32_t)X[0], (uint32_t)X[1], (uint32_t)X[2], (uint32_t)X[3]);
        }
    }
    ks[0] = __float_as_uint(scale);
    ks[1] = __float_as_uint((float)sx * scale);  // sum(x~); |sx| <= 2^26 rounds at 2^-24 like any f32 sum
}

// Lane L of the wave converts elements [32L, 32L+32) of x[0..n) (n <= 2048 per pass).  The
// global loads are split from the conversion so a kernel can request x early and convert it
// while later loads are in flight.
struct XLoad { float t[32]; };
__device__ __forceinline__ XLoad stage_x_load(const float* __restrict__ x, int n, int c0) {
    XLoad l;
    const float4* src = reinterpret_cast<const float4*>(x + (size_t)(c0 * 32 < n ? c0 : 0) * 32);
#pragma unroll
    for (int k = 0; k < 8; k++) {
        float4 v = src[k];
        l.t[4 * k] = v.x; l.t[4 * k + 1] = v.y; l.t[4 * k + 2] = v.z; l.t[4 * k + 3] = v.w;
    }
    return l;
}
template <int G, bool SIGNED>
__device__ __forceinline__ void stage_x_convert(const XLoad& l, int n, int c0, uint32_t* cells) {
    if (c0 * 32 >= n) return;
    uint32_t cell[kCellDwords];
    if (G == 32) {
        quant_to_cell<32, SIGNED>(l.t, cell, cell + 8, cell + 16, cell + 24);
        cell[26] = cell[27] = 0;
    } else {
        quant_to_cell<16, SIGNED>(l.t, cell, cell + 4, cell + 8, cell + 24);
        quant_to_cell<16, SIGNED>(l.t + 16, cell + 12, cell + 16, cell + 20, cell + 26);
    }
    uint4* dst = reinterpret_cast<uint4*>(cells + (size_t)c0 * kCellDwords);
#pragma unroll
    for (int k = 0; k < 7; k++) dst[k] = make_uint4(cell[4 * k], cell[4 * k + 1], cell[4 * k + 2], cell[4 * k + 3]);
}
// Whole vector, any n: first pass from an early load, further passes loaded here.
template <int G, bool SIGNED>
__device__ __forceinline__ void stage_x_finish(const XLoad& first, const float* __restrict__ x, int n, uint32_t* cells,
                                               int lane) {
    stage_x_convert<G, SIGNED>(first, n, lane, cells);
    for (int c0 = lane + kWave; c0 * 32 < n; c0 += kWave) {
        XLoad l = stage_x_load(x, n, c0);
        stage_x_convert<G, SIGNED>(l, n, c0, cells);
    }
}

// The same cells built by a whole block: a thread converts 8 consecutive elements (octet `oct` of the
// row) and the 4 (G == 32) or 2 (G == 16) threads of a group, which are adjacent lanes of a wavefront,
// agree on the group's scale and sum through DPP.  All lanes of such a lane group must be active.
template <int G, bool SIGNED>
__device__ __forceinline__ void octet_to_cell(const float4& lo, const float4& hi, int oct, uint32_t* cells) {
    const float v[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    uint32_t amax = 0u;
#pragma unroll
    for (int i = 0; i < 8; i++) amax = max(amax, __float_as_uint(v[i]) & 0x7FFFFFFFu);
    amax = max(amax, dpp_u<kDppXor1>(amax));
    if (G == 32) amax = max(amax, dpp_u<kDppXor2>(amax));
    const GroupScale gs = group_scale(amax);
    int X[8], sx = 0;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        X[i] = __float2int_rn(v[i] * gs.inv);
        sx += X[i];
    }
    sx += (int)dpp_u<kDppXor1>((uint32_t)sx);
    if (G == 32) sx += (int)dpp_u<kDppXor2>((uint32_t)sx);
    uint32_t a[2], b[2], c[2];
#pragma unroll
    for (int k = 0; k < 2; k++) {
        if (SIGNED) {
            uint32_t aw = 0, bw = 0, cw = 0;
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const int C = (int)(int8_t)(X[4 * k + q] & 0xFF);
                const int R = (X[4 * k + q] - C) >> 8;
                const int B = (int)(int8_t)(R & 0xFF);
                const int A = (R - B) >> 8;
                aw |= (uint32_t)(A & 0xFF) << (8 * q);
                bw |= (uint32_t)(B & 0xFF) << (8 * q);
                cw |= (uint32_t)(C & 0xFF) << (8 * q);
            }
            a[k] = aw; b[k] = bw; c[k] = cw;
        } else {
            const uint32_t x0 = (uint32_t)X[4 * k], x1 = (uint32_t)X[4 * k + 1], x2 = (uint32_t)X[4 * k + 2], x3 = (uint32_t)X[4 * k + 3];
            a[k] = gather_byte<2>(x0, x1, x2, x3);
            b[k] = gather_byte<1>(x0, x1, x2, x3);
            c[k] = gather_byte<0>(x0, x1, x2, x3);
        }
    }
    uint32_t* cell = cells + (size_t)(oct >> 2) * kCellDwords;
    const int qi = oct & 3;
    if (G == 32) {
        *reinterpret_cast<uint2*>(cell + 2 * qi) = make_uint2(a[0], a[1]);
        *reinterpret_cast<uint2*>(cell + 8 + 2 * qi) = make_uint2(b[0], b[1]);
        *reinterpret_cast<uint2*>(cell + 16 + 2 * qi) = make_uint2(c[0], c[1]);
        if (qi == 0) *reinterpret_cast<uint2*>(cell + 24) = make_uint2(__float_as_uint(gs.scale), __float_as_uint((float)sx * gs.scale));
    } else {
        uint32_t* grp = cell + (qi >> 1) * 12 + 2 * (qi & 1);
        *reinterpret_cast<uint2*>(grp) = make_uint2(a[0], a[1]);
        *reinterpret_cast<uint2*>(grp + 4) = make_uint2(b[0], b[1]);
        *reinterpret_cast<uint2*>(grp + 8) = make_uint2(c[0], c[1]);
        if ((qi & 1) == 0)
            *reinterpret_cast<uint2*>(cell + 24 + 2 * (qi >> 1)) = make_uint2(__float_as_uint(gs.scale), __float_as_uint((float)sx * gs.scale));
    }
}

__device__ __forceinline__ void fetch_dwords(uint32_t* dst, const uint32_t* src, int n4) {
    const uint4* s4 = reinterpret_cast<const uint4*>(src);
    for (int k = 0; k < n4; k++) {
        uint4 v = s4[k];
        dst[4 * k] = v.x; dst[4 * k + 1] = v.y; dst[4 * k + 2] = v.z; dst[4 * k + 3] = v.w;
    }
}

__device__ __forceinline__ int udot4i(uint32_t a, uint32_t b, int c) {
    return (int)__builtin_amdgcn_udot4(a, b, (uint32_t)c, false);
}

// sum(q * X) from the three exact byte-plane sums, rounded once or twice at 2^-24.
__device__ __forceinline__ float join3(int sa, int sb, int sc) {
    return fmaf((float)sa, 65536.0f, fmaf((float)sb, 256.0f, (float)sc));
}

__device__ __forceinline__ void load16(float* dst, const float* src) {
    const float4* s = reinterpret_cast<const float4*>(src);
#pragma unroll
    for (int k = 0; k < 4; k++) {
        float4 v = s[k];
        dst[4 * k + 0] = v.x; dst[4 * k + 1] = v.y; dst[4 * k + 2] = v.z; dst[4 * k + 3] = v.w;
    }
}

// ------------------------------------------------------------------------------- Q4_K
// 144 B: [f16 d][f16 dmin][12 B 6-bit scales/mins][128 B nibbles].  4 lanes per block; lane j
// owns nibble bytes [32j, 32j+32): low nibbles are elements j*64+t (sub-block 2j), high
// nibbles j*64+32+t (sub-block 2j+1), t < 32.
struct Q4KFmt {
    static constexpr int kBlockBytes = 144, kBlockElems = 256, kLPB = 4;
    static constexpr int kGroup = 32;
    static constexpr bool kSigned = false;
    struct X { uint32_t alo[8], blo[8], clo[8], ahi[8], bhi[8], chi[8]; float klo, khi, slo, shi; };
    struct Raw { uint4 hdr, qa, qb; };
    // lane j of block blk: cells 8*blk + 2j (low nibbles) and + 1 (high nibbles)
    static __device__ __forceinline__ void fetch_x(X& x, const uint32_t* cells, int blk, int j) {
        const uint32_t* lo = cells + (size_t)(8 * blk + 2 * j) * kCellDwords;
        const uint32_t* hi = lo + kCellDwords;
        uint32_t t[28];
#pragma unroll
        for (int k = 0; k < 7; k++) {
            uint4 v = reinterpret_cast<const uint4*>(lo)[k];
            t[4 * k] = v.x; t[4 * k + 1] = v.y; t[4 * k + 2] = v.z; t[4 * k + 3] = v.w;
        }
#pragma unroll
        for (int k = 0; k < 8; k++) { x.alo[k] = t[k]; x.blo[k] = t[8 + k]; x.clo[k] = t[16 + k]; }
        x.klo = __uint_as_float(t[24]); x.slo = __uint_as_float(t[25]);
#pragma unroll
        for (int k = 0; k < 7; k++) {
            uint4 v = reinterpret_cast<const uint4*>(hi)[k];
            t[4 * k] = v.x; t[4 * k + 1] = v.y; t[4 * k + 2] = v.z; t[4 * k + 3] = v.w;
        }
#pragma unroll
        for (int k = 0; k < 8; k++) { x.ahi[k] = t[k]; x.bhi[k] = t[8 + k]; x.chi[k] = t[16 + k]; }
        x.khi = __uint_as_float(t[24]); x.shi = __uint_as_float(t[25]);
    }
    static __device__ __forceinline__ Raw load(const uint8_t* blk, int j) {
        Raw r;
        r.hdr = *reinterpret_cast<const uint4*>(blk);
        r.qa = *reinterpret_cast<const uint4*>(blk + 16 + 32 * j);
        r.qb = *reinterpret_cast<const uint4*>(blk + 32 + 32 * j);
        return r;
    }
    static __device__ __forceinline__ float dot(const Raw& r, int j, const X& x) {
        const float d = f16_bits_to_f32(r.hdr.x & 0xFFFFu);
        const float dmin = f16_bits_to_f32(r.hdr.x >> 16);
        // 6-bit (scale, min) of sub-blocks 2j and 2j+1, as adjacent bytes (get_scale_min_k4)
        const uint32_t sh = (uint32_t)(j & 1) * 16u;
        const uint32_t y = r.hdr.y >> sh, z = r.hdr.z >> sh, w = r.hdr.w >> sh;
        uint32_t sc, m;
        if (j < 2) {
            sc = y & 0x3F3Fu;
            m = z & 0x3F3Fu;
        } else {
            sc = (w & 0x0F0Fu) | ((y >> 2) & 0x3030u);
            m = ((w >> 4) & 0x0F0Fu) | ((z >> 2) & 0x3030u);
        }
        const uint32_t q[8] = {r.qa.x, r.qa.y, r.qa.z, r.qa.w, r.qb.x, r.qb.y, r.qb.z, r.qb.w};
        int la = 0, lb = 0, lc = 0, ha = 0, hb = 0, hc = 0;
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const uint32_t lo = q[k] & 0x0F0F0F0Fu, hi = (q[k] >> 4) & 0x0F0F0F0Fu;
            la = dot4i(lo, x.alo[k], la);   // A signed; B, C plain unsigned bytes; codes are 0..15
            lb = udot4i(lo, x.blo[k], lb);
            lc = udot4i(lo, x.clo[k], lc);
            ha = dot4i(hi, x.ahi[k], ha);
            hb = udot4i(hi, x.bhi[k], hb);
            hc = udot4i(hi, x.chi[k], hc);
        }
        const float flo = join3(la, lb, lc) * x.klo;
        const float fhi = join3(ha, hb, hc) * x.khi;
        const float s0 = d * (float)(sc & 0xFFu), s1 = d * (float)(sc >> 8);
        const float m0 = dmin * (float)(m & 0xFFu), m1 = dmin * (float)(m >> 8);
        return (s0 * flo - m0 * x.slo) + (s1 * fhi - m1 * x.shi);
    }
};

// ------------------------------------------------------------------------------- Q6_K
// 210 B: [128 B ql][64 B qh][16 x i8 scales][f16 d].  4 lanes per block; lane i owns, in half
// h = i/2 at l0 = 16*(i&1), the bytes ql[h*64+l0 ..+16), ql[h*64+32+l0 ..+16) and
// qh[h*32+l0 ..+16): 64 elements in four 16-element scale groups g = 0..3 at
// h*128 + g*32 + l0 (scale byte h*8 + 2g + (i&1)).  Blocks are only 2-byte aligned.
struct Q6KFmt {
    static constexpr int kBlockBytes = 210, kBlockElems = 256, kLPB = 4;
    static constexpr int kGroup = 16;
    static constexpr bool kSigned = false;
    struct X { uint32_t a[4][4], b[4][4], c[4][4]; float k[4], s32[4]; };
    struct Raw { uint4 qla, qlb, qh; uint2 sc; uint32_t d; };
    // lane i of block blk: 16-groups 16*blk + 8h + 2g + (i&1), g = 0..3; a cell holds two
    static __device__ __forceinline__ void fetch_x(X& x, const uint32_t* cells, int blk, int i) {
        const int h = i >> 1, odd = i & 1;
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const int t = 16 * blk + 8 * h + 2 * g + odd;
            const uint32_t* cell = cells + (size_t)(t >> 1) * kCellDwords;
            const uint32_t* pl = cell + (t & 1) * 12;
#pragma unroll
            for (int q = 0; q < 3; q++) {
                uint4 v = reinterpret_cast<const uint4*>(pl)[q];
                uint32_t* dst = q == 0 ? x.a[g] : q == 1 ? x.b[g] : x.c[g];
                dst[0] = v.x; dst[1] = v.y; dst[2] = v.z; dst[3] = v.w;
            }
            const uint2 ks = *reinterpret_cast<const uint2*>(cell + 24 + 2 * (t & 1));
            x.k[g] = __uint_as_float(ks.x);
            x.s32[g] = 32.0f * __uint_as_float(ks.y);
        }
    }
    static __device__ __forceinline__ Raw load(const uint8_t* blk, int i) {
        const int h = i >> 1, l0 = (i & 1) * 16;
        Raw r;
        r.qla = ldu<uint4>(blk + h * 64 + l0);
        r.qlb = ldu<uint4>(blk + h * 64 + 32 + l0);
        r.qh = ldu<uint4>(blk + 128 + h * 32 + l0);
        r.sc = ldu<uint2>(blk + 192 + h * 8);
        r.d = ldu<uint16_t>(blk + 208);
        return r;
    }
    static __device__ __forceinline__ float dot(const Raw& r, int i, const X& x) {
        const uint32_t a[4] = {r.qla.x, r.qla.y, r.qla.z, r.qla.w};
        const uint32_t b[4] = {r.qlb.x, r.qlb.y, r.qlb.z, r.qlb.w};
        const uint32_t hq[4] = {r.qh.x, r.qh.y, r.qh.z, r.qh.w};
        int sa[4] = {0, 0, 0, 0}, sb[4] = {0, 0, 0, 0}, sc[4] = {0, 0, 0, 0};
#pragma unroll
        for (int k = 0; k < 4; k++) {
            uint32_t q[4];
            q[0] = (a[k] & 0x0F0F0F0Fu) | ((hq[k] << 4) & 0x30303030u);
            q[1] = (b[k] & 0x0F0F0F0Fu) | ((hq[k] << 2) & 0x30303030u);
            q[2] = ((a[k] >> 4) & 0x0F0F0F0Fu) | (hq[k] & 0x30303030u);
            q[3] = ((b[k] >> 4) & 0x0F0F0F0Fu) | ((hq[k] >> 2) & 0x30303030u);
#pragma unroll
            for (int g = 0; g < 4; g++) {
                sa[g] = dot4i(q[g], x.a[g][k], sa[g]);   // codes are 0..63
                sb[g] = udot4i(q[g], x.b[g][k], sb[g]);
                sc[g] = udot4i(q[g], x.c[g][k], sc[g]);
            }
        }
        const float d = f16_bits_to_f32(r.d);
        const uint32_t sx = (i & 1) ? (r.sc.x >> 8) : r.sc.x;
        const uint32_t sy = (i & 1) ? (r.sc.y >> 8) : r.sc.y;
        const float s[4] = {(float)(int)(int8_t)(sx & 0xFFu), (float)(int)(int8_t)((sx >> 16) & 0xFFu),
                            (float)(int)(int8_t)(sy & 0xFFu), (float)(int)(int8_t)((sy >> 16) & 0xFFu)};
        float acc = 0.f;
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const float f = join3(sa[g], sb[g], sc[g]) * x.k[g];  // sum(q*x~)
            acc += (d * s[g]) * (f - x.s32[g]);                    // d*s*sum((q-32)*x~)
        }
        return acc;
    }
};

// ------------------------------------------------------------------------------- Q8_0
// 34 B: [f16 d][32 x i8].  One lane per block; the signed codes contract directly.
struct Q80Fmt {
    static constexpr int kBlockBytes = 34, kBlockElems = 32, kLPB = 1;
    static constexpr int kGroup = 32;
    static constexpr bool kSigned = true;  // signed weight codes need signed digits throughout
    struct X { uint32_t a[8], b[8], c[8]; float k; };
    struct Raw { uint4 a, b; uint32_t d; };
    static __device__ __forceinline__ void fetch_x(X& x, const uint32_t* cells, int blk, int) {
        const uint32_t* cell = cells + (size_t)blk * kCellDwords;
        uint32_t t[28];
#pragma unroll
        for (int k = 0; k < 7; k++) {
            uint4 v = reinterpret_cast<const uint4*>(cell)[k];
            t[4 * k] = v.x; t[4 * k + 1] = v.y; t[4 * k + 2] = v.z; t[4 * k + 3] = v.w;
        }
#pragma unroll
        for (int k = 0; k < 8; k++) { x.a[k] = t[k]; x.b[k] = t[8 + k]; x.c[k] = t[16 + k]; }
        x.k = __uint_as_float(t[24]);
    }
    static __device__ __forceinline__ Raw load(const uint8_t* blk, int) {
        Raw r;
        r.d = ldu<uint16_t>(blk);
        r.a = ldu<uint4>(blk + 2);
        r.b = ldu<uint4>(blk + 18);
        return r;
    }
    static __device__ __forceinline__ float dot(const Raw& r, int, const X& x) {
        const uint32_t q[8] = {r.a.x, r.a.y, r.a.z, r.a.w, r.b.x, r.b.y, r.b.z, r.b.w};
        int sa = 0, sb = 0, sc = 0;
#pragma unroll
        for (int k = 0; k < 8; k++) {
            sa = dot4i(q[k], x.a[k], sa);
            sb = dot4i(q[k], x.b[k], sb);
            sc = dot4i(q[k], x.c[k], sc);
        }
        const float f = join3(sa, sb, sc) * x.k;
        return f16_bits_to_f32(r.d) * f;
    }
};

// Lane placement of a wavefront over weight rows of nblk blocks: a row holds lpr = nblk * LPB lanes (<= 64) and
// occupies `slot` lanes: lpr itself, or the next power of two when that leaves as many rows per wavefront (24 -> 32:
// two rows either way).  rows_per_wave = 64 / slot.  With a power-of-two slot the row's sum takes the DPP path of
// row_sum instead of cross-lane reads through the LDS.  Padding lanes of a slot and left-over lanes of the wave are
// pointed at the row's last block / the last row and flagged off: they load and compute like everyone else, so the
// code stays branch-free and every load of a round is issued back to back; their result is dropped.
template <class F>
struct Place {
    int lpr, slot, rw_count, rw, pos;  // lanes of a row, lanes a row occupies, rows per wave, my row (clamped), my lane in the slot
    bool row_on, lane_on;              // my row exists; my lane holds a block of it
    int blk, sub;                      // my block in the row and my lane inside the block
    int wpos;                          // lane-in-slot where the row's sum lands
    __device__ __forceinline__ Place(int nblk, int lane) {
        lpr = nblk * F::kLPB;
        slot = lpr;
        // (one-lane-per-block formats only: measured 4 % faster on 24-block Q8_0 rows, whose sum otherwise takes five
        // cross-lane reads per 32 elements of a lane, and 4 % slower on the 24 lanes of a six-block Q6_K row)
        if (F::kLPB == 1 && (lpr & (lpr - 1))) {
            int p2 = 16;
            while (p2 < lpr) p2 <<= 1;
            if (kWave / p2 == kWave / lpr) slot = p2;
        }
        rw_count = kWave / slot;
        const int rw_raw = lane / slot;
        pos = lane - rw_raw * slot;
        row_on = rw_raw < rw_count;
        lane_on = pos < lpr;
        rw = row_on ? rw_raw : rw_count - 1;
        const int bpos = lane_on ? pos : lpr - 1;
        blk = bpos / F::kLPB;
        sub = bpos - blk * F::kLPB;
        wpos = (slot == 64 || slot == 32 || slot == 16) ? slot - 1 : 0;
    }
    __device__ __forceinline__ bool writer() const { return row_on && pos == wpos; }
};

// LDS bytes one wave needs to stage an activation vector of n elements.
static inline size_t cells_bytes(int n) { return (size_t)((n + 31) / 32) * kCellDwords * sizeof(uint32_t); }
template <class F>
__device__ __forceinline__ typename F::Raw load_row(const Place<F>& pl, const uint8_t* row) {
    return F::load(row + (size_t)pl.blk * F::kBlockBytes, pl.sub);
}

// Sum of v over the lanes of each weight row; valid in the row's writer lane.
template <class F>
__device__ __forceinline__ float row_sum(float v, const Place<F>& pl, int nblk) {
    if (pl.slot >= 16 && (pl.slot & (pl.slot - 1)) == 0) {
        // Padding lanes add -0.0, the identity of the addition (x + -0.0 == x for every x, -0.0 included).  The DPP tree
        // then adds the same pairs as the doubling loop below, some with their operands swapped, and the sums of
        // padding-only subtrees where the loop adds nothing: the same bits.
        if (pl.slot != pl.lpr && !pl.lane_on) v = -0.0f;
        v = row16_sum(v);                                            // every lane: sum of its 16
        if (pl.slot >= 32) v += dpp_rows_f<0x142, 0xA>(v);           // rows 1,3 += lane 15 of rows 0,2
        if (pl.slot == 64) v += dpp_rows_f<0x143, 0xC>(v);           // rows 2,3 += lane 31
        return v;
    }
    // lanes of one block first (rows start at multiples of kLPB lanes, so DPP groups line up) ...
    if (F::kLPB == 4) v = quad_sum(v);
    // ... then the row's blocks, by doubling; the total lands in the row's first lane
    for (int ob = 1; ob < nblk; ob <<= 1) {
        float t = __shfl_down(v, ob * F::kLPB, kWave);
        if (pl.blk + ob < nblk) v += t;
    }
    return v;
}

}  // namespace infr

// Decode-regime expert kernels: id-indexed dequant-GEMV over the gate/up banks with the
// gated activation fused (h = act(gate.x) * (up.x)), and over the down bank with the
// rank-ordered weighted combine fused into the epilogue.
//
// Layout: a wavefront owns whole weight rows.  Every lane owns a FIXED slice of the K
// dimension (64 elements for the K-quants, 32 for Q8_0), so its slice of the activation
// vector is prepared once and stays in registers for all rows the wavefront streams; only
// packed weight blocks move from HBM, in 128-bit loads.  A row of nblk blocks occupies
// nblk*LPB consecutive lanes (LPB = lanes per block); when that is <= 32 several rows ride in
// one wavefront side by side.  All weight loads of a round are issued before the first dot.
//
// Arithmetic.  The lane's activation slice is held as 23-bit fixed point per group of 16/32
// elements, x ~ 2^k * X with |X| <= 2^21 (k from the group's largest magnitude; a power of
// two, so scaling is exact), and X is split into three signed bytes X = 65536*A + 256*B + C.
// Packed weight codes q (4, 6 or 8 bits) contract with A, B and C in V_DOT4_I32_I8; the three
// integer sums are exact and are joined in f32, which rounds the group's sum(q*x~) once at
// 2^-24 relative.  The block scales are applied in f32 in factored form,
//     (d*sc) * sum(q*x~) + (dmin*m) * sum(x~),
// so a one-hot x reads back the reference's decoded weight bit for bit
// (crates/infr-gguf/src/dequant.rs:35-51).  For general x the rounding of x to 2^-22 of its
// group's largest magnitude is of the order of f32's own 2^-24, so results track the f32
// reference as closely as a reordered f32 summation does.
#include "device_common.h"
#include "kernels.h"
#include "route.h"

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

template <int N, bool SIGNED>
__device__ __forceinline__ void quant_to_cell(const float* x, uint32_t* a, uint32_t* b, uint32_t* c, uint32_t* ks) {
    float amax = 0.f;
#pragma unroll
    for (int i = 0; i < N; i++) amax = fmaxf(amax, fabsf(x[i]));
    const uint32_t eb = (__float_as_uint(amax) >> 23) & 0xFFu;  // amax in [2^(eb-127), 2^(eb-126))
    const bool live = eb >= 22u && eb < 255u;
    const float inv = live ? __uint_as_float((274u - eb) << 23) : 0.f;  // 2^(20 - E): |x| * inv < 2^21
    const float scale = live ? __uint_as_float((eb - 20u) << 23) : 0.f; // 2^(E - 20)
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

// Lane placement of a wavefront over weight rows of nblk blocks: lanes_per_row = nblk*LPB
// (<= 64), rows_per_wave = 64 / lanes_per_row.  Left-over lanes of the wave are pointed at the
// last row and flagged off: they load and compute like everyone else, so the code stays
// branch-free and every load of a round is issued back to back; their result is dropped.
template <class F>
struct Place {
    int lpr, rw_count, rw, pos;  // lanes per row, rows per wave, my row (clamped), my lane in the row
    bool row_on;
    int blk, sub;                // my block in the row and my lane inside the block
    int wpos;                    // lane-in-row where the row's sum lands
    __device__ __forceinline__ Place(int nblk, int lane) {
        lpr = nblk * F::kLPB;
        rw_count = kWave / lpr;
        const int rw_raw = lane / lpr;
        pos = lane - rw_raw * lpr;
        row_on = rw_raw < rw_count;
        rw = row_on ? rw_raw : rw_count - 1;
        blk = pos / F::kLPB;
        sub = pos - blk * F::kLPB;
        wpos = (lpr == 64 || lpr == 32 || lpr == 16) ? lpr - 1 : 0;
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
    if (pl.lpr >= 16 && (pl.lpr & (pl.lpr - 1)) == 0) {
        v = row16_sum(v);                                            // every lane: sum of its 16
        if (pl.lpr >= 32) v += dpp_rows_f<0x142, 0xA>(v);            // rows 1,3 += lane 15 of rows 0,2
        if (pl.lpr == 64) v += dpp_rows_f<0x143, 0xC>(v);            // rows 2,3 += lane 31
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

// ------------------------------------------------------------------------------- gate/up
// grid.x = tiles of `ft` features, grid.y = token row.  A block's 4 waves share the items
// (slot, f) of its tile; x is identical for every slot of a token.  U = items a wave has in
// flight per round.  Results wait in LDS and one lane per item applies the gated activation
// after the round, so the f64 exp and the divide run once per wave, not once per item.
// One stage of a wave's work: U (gate row, up row) pairs per row lane group, loaded together.
template <class F, int U>
struct GuStage { typename F::Raw g[U], u[U]; };

struct GuTile {
    int r, f0, fcount, nitems, n_slots, wave, lane;
    size_t row_bytes;
};

// Issue every load of the stage that starts at item `base`; items past the end re-read the last.
template <class F, int U>
__device__ __forceinline__ void gu_issue(GuStage<F, U>& st, const MoeGemvParams& p, const Place<F>& pl, const GuTile& t,
                                         const int32_t* s_ids, int base) {
#pragma unroll
    for (int u = 0; u < U; u++) {
        const int it = min(base + (u * 4 + t.wave) * pl.rw_count + pl.rw, t.nitems - 1);
        const int slot = it / t.fcount, f = t.f0 + (it - slot * t.fcount);
        const int e = s_ids[slot];
        const bool routed = slot < p.n_used;
        const uint8_t* gb = routed ? p.gate + (size_t)e * p.gate_stride : p.sh_gate;
        const uint8_t* ub = routed ? p.up + (size_t)e * p.up_stride : p.sh_up;
        st.g[u] = load_row<F>(pl, gb + (size_t)f * t.row_bytes);
        st.u[u] = load_row<F>(pl, ub + (size_t)f * t.row_bytes);
    }
}

// Dot the stage's rows with x; results wait in LDS and one lane per item applies the gated
// activation, so the f64 exp and the divide run once per wave, not once per item.
template <class F, int U>
__device__ __forceinline__ void gu_finish(const GuStage<F, U>& st, const MoeGemvParams& p, const Place<F>& pl,
                                          const GuTile& t, const typename F::X& x, int nblk, int base, float (*s_g)[64],
                                          float (*s_u)[64], const float* s_w, const uint64_t* s_tab) {
#pragma unroll
    for (int u = 0; u < U; u++) {
        float gs = row_sum<F>(F::dot(st.g[u], pl.sub, x), pl, nblk);
        float us = row_sum<F>(F::dot(st.u[u], pl.sub, x), pl, nblk);
        if (pl.writer()) {
            s_g[t.wave][u * pl.rw_count + pl.rw] = gs;
            s_u[t.wave][u * pl.rw_count + pl.rw] = us;
        }
    }
    __builtin_amdgcn_wave_barrier();
    if (t.lane < U * pl.rw_count) {
        const int u = t.lane / pl.rw_count, rw = t.lane - u * pl.rw_count;
        const int it = base + (u * 4 + t.wave) * pl.rw_count + rw;
        if (it < t.nitems) {
            const int slot = it / t.fcount, f = t.f0 + (it - slot * t.fcount);
            float gs = s_g[t.wave][t.lane], us = s_u[t.wave][t.lane];
            if (p.weight_before && slot < p.n_used) {
                const float wp = s_w[slot];
                gs = __fmul_rn(wp, gs);
                us = __fmul_rn(wp, us);
            }
            p.h[((size_t)t.r * t.n_slots + slot) * p.nff + f] = gated_act_fn(p.act, p.has_clamp, p.clamp, gs, us, s_tab);
        }
    }
    __builtin_amdgcn_wave_barrier();
}

// PIPE == false: every stage is loaded, then finished (one stage is the common decode case and
// then all of the block's loads are in flight at once).  PIPE == true, for tiles of three or more
// stages: two stage buffers, the next stage's loads are issued before the current stage is
// finished, so a wave always has a stage in flight while it computes.
template <class F, int U, bool PIPE>
__global__ __launch_bounds__(256) void moe_gate_up_fast(MoeGemvParams p, int ft) {
    extern __shared__ uint32_t dyn_lds[];
    __shared__ uint64_t s_tab[32];
    __shared__ int32_t s_ids[64];
    __shared__ float s_w[64];
    __shared__ float s_g[4][64], s_u[4][64];
    GuTile t;
    t.r = blockIdx.y;
    t.f0 = blockIdx.x * ft;
    t.fcount = min(ft, p.nff - t.f0);
    t.wave = threadIdx.x >> 6;
    t.lane = threadIdx.x & 63;
    const int r = t.r, wave = t.wave, lane = t.lane;
    const int nblk = p.ne / F::kBlockElems;
    t.row_bytes = (size_t)nblk * F::kBlockBytes;
    const Place<F> pl(nblk, lane);
    const size_t cell_words = (size_t)((p.ne + 31) / 32) * kCellDwords;
    uint32_t* cells = dyn_lds + (size_t)wave * cell_words;
    // x is requested first; it does not depend on the routing
    const float* xrow = p.x + (size_t)r * p.ne;
    const XLoad xl = stage_x_load(xrow, p.ne, lane);
    if (threadIdx.x < 32) s_tab[threadIdx.x] = kExp2Table[threadIdx.x];
    if (p.route_inline) {
        // every block routes its token row itself (one wave, redundantly across blocks)
        __syncthreads();
        if (wave == 0)
            route_row_any(p.route, r, lane, reinterpret_cast<float*>(dyn_lds + 4 * cell_words), s_tab, s_ids, s_w,
                          blockIdx.x == 0);
    } else if ((int)threadIdx.x < p.n_used) {  // n_used <= 64
        s_ids[threadIdx.x] = p.ids[(size_t)r * p.n_used + threadIdx.x];
        s_w[threadIdx.x] = p.weights[(size_t)r * p.n_used + threadIdx.x];
    }
    t.n_slots = p.n_used + (p.sh_gate ? 1 : 0);   // the always-on expert is slot n_used (<= 63 then)
    if (p.sh_gate && threadIdx.x == 255) {
        s_ids[p.n_used] = 0;
        s_w[p.n_used] = 1.0f;
    }
    __syncthreads();
    __builtin_amdgcn_wave_barrier();
    t.nitems = t.fcount * t.n_slots;
    const int step = 4 * pl.rw_count * U;
    typename F::X x;
    if (!PIPE) {
        bool have_x = false;
        for (int base = 0; base < t.nitems; base += step) {
            GuStage<F, U> st;
            gu_issue<F, U>(st, p, pl, t, s_ids, base);
            if (!have_x) {
                // while the weights are in flight: the wave converts x to fixed point once, together
                stage_x_finish<F::kGroup, F::kSigned>(xl, xrow, p.ne, cells, lane);
                __builtin_amdgcn_wave_barrier();
                F::fetch_x(x, cells, pl.blk, pl.sub);
                have_x = true;
            }
            gu_finish<F, U>(st, p, pl, t, x, nblk, base, s_g, s_u, s_w, s_tab);
        }
    } else {
        GuStage<F, U> sa, sb;
        gu_issue<F, U>(sa, p, pl, t, s_ids, 0);
        gu_issue<F, U>(sb, p, pl, t, s_ids, step);
        stage_x_finish<F::kGroup, F::kSigned>(xl, xrow, p.ne, cells, lane);
        __builtin_amdgcn_wave_barrier();
        F::fetch_x(x, cells, pl.blk, pl.sub);
        gu_finish<F, U>(sa, p, pl, t, x, nblk, 0, s_g, s_u, s_w, s_tab);
        int base = step;   // the stage sb holds
        for (;;) {
            if (base + step >= t.nitems) {
                gu_finish<F, U>(sb, p, pl, t, x, nblk, base, s_g, s_u, s_w, s_tab);
                break;
            }
            gu_issue<F, U>(sa, p, pl, t, s_ids, base + step);
            gu_finish<F, U>(sb, p, pl, t, x, nblk, base, s_g, s_u, s_w, s_tab);
            base += step;
            if (base + step >= t.nitems) {
                gu_finish<F, U>(sa, p, pl, t, x, nblk, base, s_g, s_u, s_w, s_tab);
                break;
            }
            gu_issue<F, U>(sb, p, pl, t, s_ids, base + step);
            gu_finish<F, U>(sa, p, pl, t, x, nblk, base, s_g, s_u, s_w, s_tab);
            base += step;
        }
    }
}

// ------------------------------------------------------------------------------- down
// grid.x = tiles of `ot` = S * rows-per-wave output rows, grid.y = token row.  One wave per
// slot: it holds that slot's h and streams the S row groups of its expert's down matrix, all
// loads issued up front.  The per-slot results meet in LDS and are combined in rank order:
// out += w_rank * y_rank as a separate multiply and add
// (crates/infr-cpu/src/lib.rs:4290-4302).
constexpr int kMaxUsedFast = 16;
constexpr int kMaxOt = 128;

struct DownTile {
    int slot, ocount;
    size_t row_bytes;
    bool scaled;
    float ds;
};

// Issue the loads of the S row groups that start at output row `obase` of the tile; rows past
// the tile re-read its last row.
template <class F, int S>
__device__ __forceinline__ void down_issue(typename F::Raw (&raw)[S], const Place<F>& pl, const DownTile& t,
                                           const uint8_t* bank, int obase) {
#pragma unroll
    for (int st = 0; st < S; st++) {
        const int o = min(obase + st * pl.rw_count + pl.rw, t.ocount - 1);
        raw[st] = load_row<F>(pl, bank + (size_t)o * t.row_bytes);
    }
}

template <class F, int S>
__device__ __forceinline__ void down_finish(const typename F::Raw (&raw)[S], const Place<F>& pl, const DownTile& t,
                                            const typename F::X& x, int nblk, int obase, float (*ypart)[kMaxOt]) {
#pragma unroll
    for (int st = 0; st < S; st++) {
        const int o = obase + st * pl.rw_count + pl.rw;
        float y = row_sum<F>(F::dot(raw[st], pl.sub, x), pl, nblk);
        if (o < t.ocount && pl.writer()) ypart[t.slot][o] = t.scaled ? __fmul_rn(y, t.ds) : y;
    }
}

// PIPE == false: ot = S row groups, all loaded up front (single-token decode: everything in
// flight at once).  PIPE == true: the tile is any number of stages of S row groups; a wave keeps
// the next stage's loads in flight while it finishes the current one.
template <class F, int S, bool PIPE>
__global__ __launch_bounds__(512) void moe_down_combine_fast(MoeGemvParams p, int ot) {
    extern __shared__ uint32_t dyn_lds[];
    __shared__ float ypart[kMaxUsedFast][kMaxOt];
    const int r = blockIdx.y;
    const int o0 = blockIdx.x * ot;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int nwaves = blockDim.x >> 6;
    const int nblk = p.nff / F::kBlockElems;
    const Place<F> pl(nblk, lane);
    const int32_t* ids = p.ids + (size_t)r * p.n_used;
    uint32_t* cells = dyn_lds + (size_t)wave * ((p.nff + 31) / 32) * kCellDwords;
    DownTile t;
    t.ocount = min(ot, p.ne - o0);
    t.row_bytes = (size_t)nblk * F::kBlockBytes;

    const int n_slots = p.n_used + (p.sh_down ? 1 : 0);   // the always-on expert is slot n_used
    for (int slot = wave; slot < n_slots; slot += nwaves) {
        const bool routed = slot < p.n_used;
        const int e = routed ? ids[slot] : 0;  // first: every weight address below waits on it
        const float* hrow = p.h + ((size_t)r * n_slots + slot) * p.nff;
        const XLoad xl = stage_x_load(hrow, p.nff, lane);
        const uint8_t* bank = (routed ? p.down + (size_t)e * p.down_stride : p.sh_down) + (size_t)o0 * t.row_bytes;
        t.slot = slot;
        t.scaled = p.down_scale && routed;
        typename F::Raw ra[S];
        down_issue<F, S>(ra, pl, t, bank, 0);
        typename F::X x;
        if (!PIPE) {
            // while the weights are in flight: this slot's h to fixed point, once per wave
            __builtin_amdgcn_wave_barrier();
            stage_x_finish<F::kGroup, F::kSigned>(xl, hrow, p.nff, cells, lane);
            __builtin_amdgcn_wave_barrier();
            F::fetch_x(x, cells, pl.blk, pl.sub);
            t.ds = t.scaled ? p.down_scale[e] : 1.0f;
            down_finish<F, S>(ra, pl, t, x, nblk, 0, ypart);
        } else {
            const int gstep = S * pl.rw_count;
            typename F::Raw rb[S];
            down_issue<F, S>(rb, pl, t, bank, gstep);
            __builtin_amdgcn_wave_barrier();
            stage_x_finish<F::kGroup, F::kSigned>(xl, hrow, p.nff, cells, lane);
            __builtin_amdgcn_wave_barrier();
            F::fetch_x(x, cells, pl.blk, pl.sub);
            t.ds = t.scaled ? p.down_scale[e] : 1.0f;
            down_finish<F, S>(ra, pl, t, x, nblk, 0, ypart);
            int o = gstep;   // the stage rb holds
            for (;;) {
                if (o + gstep >= t.ocount) {
                    down_finish<F, S>(rb, pl, t, x, nblk, o, ypart);
                    break;
                }
                down_issue<F, S>(ra, pl, t, bank, o + gstep);
                down_finish<F, S>(rb, pl, t, x, nblk, o, ypart);
                o += gstep;
                if (o + gstep >= t.ocount) {
                    down_finish<F, S>(ra, pl, t, x, nblk, o, ypart);
                    break;
                }
                down_issue<F, S>(rb, pl, t, bank, o + gstep);
                down_finish<F, S>(ra, pl, t, x, nblk, o, ypart);
                o += gstep;
            }
            __builtin_amdgcn_wave_barrier();   // the next slot's h overwrites this wave's cells
        }
    }
    __syncthreads();
    for (int o = threadIdx.x; o < t.ocount; o += blockDim.x) {
        const float* w = p.weights + (size_t)r * p.n_used;
        float acc = 0.0f;
        for (int k = 0; k < n_slots; k++) {
            if (p.skip_zero_w && k < p.n_used && w[k] == 0.0f) continue;
            float wk = (p.weight_before || k >= p.n_used) ? 1.0f : w[k];
            if (k >= p.n_used && p.sh_logit)   // crates/infr-cpu/src/lib.rs:3336-3356: sigmoid of the row's gate logit
                wk = __fdiv_rn(1.0f, __fadd_rn(1.0f, expf_libm(-p.sh_logit[r])));
            acc = __fadd_rn(acc, __fmul_rn(wk, ypart[k][o]));
        }
        const size_t oi = (size_t)r * p.ne + o0 + o;
        p.dst[oi] = p.addend ? __fadd_rn(p.addend[oi], acc) : acc;
    }
}

// ------------------------------------------------------------------------------- generic
// Any dtype decode_elem understands and any shape: one wave per output, lanes stride over K,
// plain f32.
__global__ __launch_bounds__(256) void moe_gate_up_generic(MoeGemvParams p, size_t g_row_bytes, size_t u_row_bytes) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int f = blockIdx.x * 4 + wave;
    const int pair = blockIdx.y;
    if (f >= p.nff) return;
    const int r = pair / p.n_used;
    const int e = p.ids[pair];
    const uint8_t* grow = p.gate + (size_t)e * p.gate_stride + (size_t)f * g_row_bytes;
    const uint8_t* urow = p.up + (size_t)e * p.up_stride + (size_t)f * u_row_bytes;
    const float* x = p.x + (size_t)r * p.ne;
    float gs = 0.f, us = 0.f;
    for (int k = lane; k < p.ne; k += kWave) {
        float xv = x[k];
        gs = fmaf(decode_elem(p.gate_dt, grow, (uint32_t)k), xv, gs);
        us = fmaf(decode_elem(p.up_dt, urow, (uint32_t)k), xv, us);
    }
    gs = wave_sum(gs);
    us = wave_sum(us);
    if (lane == 0) {
        if (p.weight_before) {
            float wp = p.weights[pair];
            gs = __fmul_rn(wp, gs);
            us = __fmul_rn(wp, us);
        }
        p.h[(size_t)pair * p.nff + f] = gated_act_fn(p.act, p.has_clamp, p.clamp, gs, us);
    }
}

__global__ __launch_bounds__(256) void moe_down_combine_generic(MoeGemvParams p, size_t row_bytes) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int o = blockIdx.x * 4 + wave;
    const int r = blockIdx.y;
    if (o >= p.ne) return;
    float acc = 0.0f;
    for (int slot = 0; slot < p.n_used; slot++) {
        const int e = p.ids[(size_t)r * p.n_used + slot];
        const uint8_t* row = p.down + (size_t)e * p.down_stride + (size_t)o * row_bytes;
        const float* h = p.h + ((size_t)r * p.n_used + slot) * p.nff;
        float y = 0.f;
        for (int k = lane; k < p.nff; k += kWave) y = fmaf(decode_elem(p.down_dt, row, (uint32_t)k), h[k], y);
        y = wave_sum(y);
        if (p.down_scale) y = __fmul_rn(y, p.down_scale[e]);
        if (p.skip_zero_w && p.weights[(size_t)r * p.n_used + slot] == 0.0f) continue;
        float wk = p.weight_before ? 1.0f : p.weights[(size_t)r * p.n_used + slot];
        acc = __fadd_rn(acc, __fmul_rn(wk, y));
    }
    if (lane == 0) {
        const size_t oi = (size_t)r * p.ne + o;
        p.dst[oi] = p.addend ? __fadd_rn(p.addend[oi], acc) : acc;
    }
}

// ------------------------------------------------------------------------------- dispatch
static size_t row_bytes_of(int dt, int in_f) {
    int be = 1, bb = 4;
    block_geometry(dt, &be, &bb);
    return (size_t)(in_f / be) * bb;
}

// The fast kernels cover rows of up to 64 lanes (K-quants: in_f <= 4096, Q8_0: in_f <= 2048).
template <class F>
static bool fast_ok(int in_f) {
    if (in_f <= 0 || in_f % F::kBlockElems != 0) return false;
    return in_f / F::kBlockElems * F::kLPB <= 64;
}

static int ceil_div(int a, int b) { return (a + b - 1) / b; }

template <class F>
static bool try_gate_up(hipStream_t s, const MoeGemvParams& p) {
    if (!fast_ok<F>(p.ne) || p.n_used > 64) return false;
    const int rw = 64 / (p.ne / F::kBlockElems * F::kLPB);
    // about one block per compute unit; a block's ft * n_slots items go to 4 waves of rw rows each
    const int n_slots = p.n_used + (p.sh_gate ? 1 : 0);
    int ft = ceil_div(p.nff, p.n_cu);
    if (ft < 1) ft = 1;
    const int per_wave = ceil_div(ft * n_slots, 4 * rw);
    // tiles of three or more stages stream with the next stage in flight
    const bool pipe = per_wave > 6 && 3 * rw <= 64;
    dim3 grid(ceil_div(p.nff, ft), p.rows), block(256);
    // U * rw results per wave must fit the 64-entry staging rows
    int u = per_wave < 1 ? 1 : per_wave;
    while (u * rw > 64) u--;
    const size_t lds = 4 * cells_bytes(p.ne) +
                       (p.route_inline ? route_scratch_floats(p.route.n_expert, p.route.n_groups) * sizeof(float) : 0);
    if (pipe) INFR_LAUNCH((moe_gate_up_fast<F, 3, true>), grid, block, lds, s, p, ft);
    else if (u >= 6) INFR_LAUNCH((moe_gate_up_fast<F, 6, false>), grid, block, lds, s, p, ft);
    else if (u == 5 || u == 4) INFR_LAUNCH((moe_gate_up_fast<F, 4, false>), grid, block, lds, s, p, ft);
    else if (u == 3) INFR_LAUNCH((moe_gate_up_fast<F, 3, false>), grid, block, lds, s, p, ft);
    else if (u == 2) INFR_LAUNCH((moe_gate_up_fast<F, 2, false>), grid, block, lds, s, p, ft);
    else INFR_LAUNCH((moe_gate_up_fast<F, 1, false>), grid, block, lds, s, p, ft);
    return true;
}

bool moe_gate_up_routes_inline(const MoeGemvParams& p) {
    if (p.gate_dt != p.up_dt || p.n_used > 64) return false;
    if (p.gate_dt == INFR_Q4K) return fast_ok<Q4KFmt>(p.ne);
    if (p.gate_dt == INFR_Q6K) return fast_ok<Q6KFmt>(p.ne);
    if (p.gate_dt == INFR_Q8_0) return fast_ok<Q80Fmt>(p.ne);
    return false;
}

void launch_moe_gate_up(hipStream_t s, const MoeGemvParams& p) {
    if (p.gate_dt == p.up_dt) {
        bool done = false;
        if (p.gate_dt == INFR_Q4K) done = try_gate_up<Q4KFmt>(s, p);
        else if (p.gate_dt == INFR_Q6K) done = try_gate_up<Q6KFmt>(s, p);
        else if (p.gate_dt == INFR_Q8_0) done = try_gate_up<Q80Fmt>(s, p);
        if (done) return;
    }
    if (!p.sh_gate && moe_gate_up_units_supported(p)) {   // the other affine formats, and shapes the kernels above refuse
        launch_moe_gate_up_units(s, p);
        return;
    }
    dim3 grid((p.nff + 3) / 4, p.rows * p.n_used), block(256);
    INFR_LAUNCH(moe_gate_up_generic, grid, block, 0, s, p, row_bytes_of(p.gate_dt, p.ne),
                       row_bytes_of(p.up_dt, p.ne));
}

template <class F>
static bool try_down(hipStream_t s, const MoeGemvParams& p) {
    const int n_slots = p.n_used + (p.sh_down ? 1 : 0);
    if (!fast_ok<F>(p.nff) || n_slots > kMaxUsedFast) return false;
    const int rw = 64 / (p.nff / F::kBlockElems * F::kLPB);
    // output rows per block ~ rows * ne / n_cu
    const int want = ceil_div(p.ne, p.n_cu);
    if (p.rows >= 2) {
        // several token rows: tiles of whole stages of 2 row groups, about one block per compute
        // unit in total, streamed with the next stage in flight; one wave per slot
        const int gstep = 2 * rw;
        // tile height: whole stages; fewest rounds of blocks over the compute units, counting a
        // block's fixed cost (ids, h staging, combine) as about a dozen rows of streaming
        int ot = 0;
        long best = 0;
        for (int cand = 2 * gstep; cand <= kMaxOt; cand += gstep) {
            const long blocks = (long)p.rows * ceil_div(p.ne, cand);
            const long cost = ((blocks + p.n_cu - 1) / p.n_cu) * (cand + 12);
            if (ot == 0 || cost < best) { ot = cand; best = cost; }
        }
        if (ot >= 2 * gstep) {
            const int nwaves = n_slots < 8 ? n_slots : 8;
            dim3 grid(ceil_div(p.ne, ot), p.rows), block(64 * nwaves);
            const size_t lds = nwaves * cells_bytes(p.nff);
            INFR_LAUNCH((moe_down_combine_fast<F, 2, true>), grid, block, lds, s, p, ot);
            return true;
        }
    }
    int steps = 1;
    while (steps < 8 && steps * rw < want) steps <<= 1;
    while (steps > 1 && steps * rw > kMaxOt) steps >>= 1;
    const int ot = steps * rw;
    const int nwaves = n_slots < 8 ? n_slots : 8;
    dim3 grid(ceil_div(p.ne, ot), p.rows), block(64 * nwaves);
    const size_t lds = nwaves * cells_bytes(p.nff);
    switch (steps) {
        case 1: INFR_LAUNCH((moe_down_combine_fast<F, 1, false>), grid, block, lds, s, p, ot); break;
        case 2: INFR_LAUNCH((moe_down_combine_fast<F, 2, false>), grid, block, lds, s, p, ot); break;
        case 4: INFR_LAUNCH((moe_down_combine_fast<F, 4, false>), grid, block, lds, s, p, ot); break;
        default: INFR_LAUNCH((moe_down_combine_fast<F, 8, false>), grid, block, lds, s, p, ot); break;
    }
    return true;
}

bool moe_down_is_fast(const MoeGemvParams& p) {
    if (p.n_used + (p.sh_down ? 1 : 0) > kMaxUsedFast) return false;
    if (p.down_dt == INFR_Q4K) return fast_ok<Q4KFmt>(p.nff);
    if (p.down_dt == INFR_Q6K) return fast_ok<Q6KFmt>(p.nff);
    if (p.down_dt == INFR_Q8_0) return fast_ok<Q80Fmt>(p.nff);
    return false;
}

void launch_moe_down_combine(hipStream_t s, const MoeGemvParams& p) {
    bool done = false;
    if (p.down_dt == INFR_Q4K) done = try_down<Q4KFmt>(s, p);
    else if (p.down_dt == INFR_Q6K) done = try_down<Q6KFmt>(s, p);
    else if (p.down_dt == INFR_Q8_0) done = try_down<Q80Fmt>(s, p);
    if (done) return;
    dim3 grid((p.ne + 3) / 4, p.rows), block(256);
    INFR_LAUNCH(moe_down_combine_generic, grid, block, 0, s, p, row_bytes_of(p.down_dt, p.nff));
}

// ------------------------------------------------------------------------------- bucketed batches
// Decode batches of several token rows: grid.x = tiles of `ft` features (gate/up) or `ot` output
// rows (down), grid.y = expert, grid.z = chunk of T tokens of the expert's bucket.  A block stages
// the activations of its T tokens once (all waves share the cells), then every weight row of its
// tile is loaded once and dotted with each of them.  Same inner product as the per-token kernels,
// so the results are the same bits whichever path a batch takes.
template <class F, int T>
__device__ __forceinline__ void stage_tokens(const float* const (&rows)[T], int nt, int n, uint32_t* cells,
                                             size_t cell_words) {
    const int ncell = (n + 31) / 32;
    for (int idx = threadIdx.x; idx < T * ncell; idx += 256) {
        const int tau = idx / ncell, c0 = idx - tau * ncell;
        if (tau < nt) {
            const XLoad l = stage_x_load(rows[tau], n, c0);
            stage_x_convert<F::kGroup, F::kSigned>(l, n, c0, cells + (size_t)tau * cell_words);
        }
    }
    __syncthreads();
}

template <class F, int U, int T>
__global__ __launch_bounds__(256) void moe_gate_up_bucketed(MoeGemvParams p, int ft) {
    extern __shared__ uint32_t dyn_lds[];
    __shared__ uint64_t s_tab[32];
    __shared__ float s_g[4][T][64], s_u[4][T][64];
    const int e = blockIdx.y;
    // without tables there is one bucket holding every row in order (a dense layer)
    const int t0 = (p.bk_offsets ? p.bk_offsets[e] : 0) + blockIdx.z * T, t1 = p.bk_offsets ? p.bk_offsets[e + 1] : p.rows;
    if (t0 >= t1) return;
    const int nt = min(T, t1 - t0);
    const int f0 = blockIdx.x * ft;
    const int fcount = min(ft, p.nff - f0);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int nblk = p.ne / F::kBlockElems;
    const size_t row_bytes = (size_t)nblk * F::kBlockBytes;
    const Place<F> pl(nblk, lane);
    const size_t cell_words = (size_t)((p.ne + 31) / 32) * kCellDwords;
    if (threadIdx.x < 32) s_tab[threadIdx.x] = kExp2Table[threadIdx.x];
    int pair[T];
    const float* xrows[T];
#pragma unroll
    for (int tau = 0; tau < T; tau++) {
        pair[tau] = p.bk_pair_src ? p.bk_pair_src[t0 + min(tau, nt - 1)] : t0 + min(tau, nt - 1);
        xrows[tau] = p.x + (size_t)(pair[tau] / p.n_used) * p.ne;
    }
    const uint8_t* gbank = p.gate + (size_t)e * p.gate_stride + (size_t)f0 * row_bytes;
    const uint8_t* ubank = p.up + (size_t)e * p.up_stride + (size_t)f0 * row_bytes;
    const int per_round = 4 * pl.rw_count;
    // the first round of weight rows is requested before the activations are staged
    typename F::Raw graw[U], uraw[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
        const int f = min((u * 4 + wave) * pl.rw_count + pl.rw, fcount - 1);
        graw[u] = load_row<F>(pl, gbank + (size_t)f * row_bytes);
        uraw[u] = load_row<F>(pl, ubank + (size_t)f * row_bytes);
    }
    stage_tokens<F, T>(xrows, nt, p.ne, dyn_lds, cell_words);
    typename F::X x[T];
#pragma unroll
    for (int tau = 0; tau < T; tau++) F::fetch_x(x[tau], dyn_lds + (size_t)min(tau, nt - 1) * cell_words, pl.blk, pl.sub);
    for (int base = 0; base < fcount; base += per_round * U) {
#pragma unroll
        for (int u = 0; u < U; u++) {
#pragma unroll
            for (int tau = 0; tau < T; tau++) {
                float gs = row_sum<F>(F::dot(graw[u], pl.sub, x[tau]), pl, nblk);
                float us = row_sum<F>(F::dot(uraw[u], pl.sub, x[tau]), pl, nblk);
                if (pl.writer()) {
                    s_g[wave][tau][u * pl.rw_count + pl.rw] = gs;
                    s_u[wave][tau][u * pl.rw_count + pl.rw] = us;
                }
            }
        }
        // next round's rows are in flight while this round's activations are applied
        if (base + per_round * U < fcount) {
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int f = min(base + per_round * U + (u * 4 + wave) * pl.rw_count + pl.rw, fcount - 1);
                graw[u] = load_row<F>(pl, gbank + (size_t)f * row_bytes);
                uraw[u] = load_row<F>(pl, ubank + (size_t)f * row_bytes);
            }
        }
        __builtin_amdgcn_wave_barrier();
        if (lane < U * pl.rw_count) {
            const int u = lane / pl.rw_count, rw = lane - u * pl.rw_count;
            const int f = base + (u * 4 + wave) * pl.rw_count + rw;
            if (f < fcount) {
#pragma unroll
                for (int tau = 0; tau < T; tau++) {
                    if (tau >= nt) break;
                    float gs = s_g[wave][tau][lane], us = s_u[wave][tau][lane];
                    if (p.weight_before) {
                        const float wp = p.weights[pair[tau]];
                        gs = __fmul_rn(wp, gs);
                        us = __fmul_rn(wp, us);
                    }
                    p.h[(size_t)pair[tau] * p.nff + f0 + f] = gated_act_fn(p.act, p.has_clamp, p.clamp, gs, us, s_tab);
                }
            }
        }
        __builtin_amdgcn_wave_barrier();
    }
}

template <class F, int U, int T>
__global__ __launch_bounds__(256) void moe_down_bucketed(MoeGemvParams p, int ot) {
    extern __shared__ uint32_t dyn_lds[];
    const int e = blockIdx.y;
    const int t0 = (p.bk_offsets ? p.bk_offsets[e] : 0) + blockIdx.z * T, t1 = p.bk_offsets ? p.bk_offsets[e + 1] : p.rows;
    if (t0 >= t1) return;
    const int nt = min(T, t1 - t0);
    const int o0 = blockIdx.x * ot;
    const int ocount = min(ot, p.ne - o0);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int nblk = p.nff / F::kBlockElems;
    const size_t row_bytes = (size_t)nblk * F::kBlockBytes;
    const Place<F> pl(nblk, lane);
    const uint8_t* bank = p.down + (size_t)e * p.down_stride + (size_t)o0 * row_bytes;
    const int per_round = 4 * pl.rw_count;
    const size_t cell_words = (size_t)((p.nff + 31) / 32) * kCellDwords;
    const float ds = p.down_scale ? p.down_scale[e] : 1.0f;
    int pair[T];
    const float* xrows[T];
#pragma unroll
    for (int tau = 0; tau < T; tau++) {
        pair[tau] = p.bk_pair_src ? p.bk_pair_src[t0 + min(tau, nt - 1)] : t0 + min(tau, nt - 1);
        xrows[tau] = p.x + (size_t)pair[tau] * p.nff;   // h of the pair
    }
    typename F::Raw raw[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
        const int o = min((u * 4 + wave) * pl.rw_count + pl.rw, ocount - 1);
        raw[u] = load_row<F>(pl, bank + (size_t)o * row_bytes);
    }
    stage_tokens<F, T>(xrows, nt, p.nff, dyn_lds, cell_words);
    typename F::X x[T];
#pragma unroll
    for (int tau = 0; tau < T; tau++) F::fetch_x(x[tau], dyn_lds + (size_t)min(tau, nt - 1) * cell_words, pl.blk, pl.sub);
    for (int base = 0; base < ocount; base += per_round * U) {
        float y[U][T];
#pragma unroll
        for (int u = 0; u < U; u++)
#pragma unroll
            for (int tau = 0; tau < T; tau++) y[u][tau] = row_sum<F>(F::dot(raw[u], pl.sub, x[tau]), pl, nblk);
        const int base_next = base + per_round * U;
        typename F::Raw nxt[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int o = min(base_next + (u * 4 + wave) * pl.rw_count + pl.rw, ocount - 1);
            nxt[u] = load_row<F>(pl, bank + (size_t)o * row_bytes);
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int o = base + (u * 4 + wave) * pl.rw_count + pl.rw;
#pragma unroll
            for (int tau = 0; tau < T; tau++) {
                float v = y[u][tau];
                if (p.down_scale) v = __fmul_rn(v, ds);
                if (o < ocount && tau < nt && pl.writer()) {
                    const size_t oi = (size_t)pair[tau] * p.ne + o0 + o;
                    p.y[oi] = p.addend ? __fadd_rn(p.addend[oi], v) : v;
                }
            }
            raw[u] = nxt[u];
        }
    }
}

constexpr int kBucketT = 2;   // tokens a block of the bucketed kernels handles together

template <class F>
static void gate_up_bucketed(hipStream_t s, const MoeGemvParams& p) {
    const int rw = 64 / (p.ne / F::kBlockElems * F::kLPB);
    // about four blocks per CU if every expert had one chunk of tokens (dense: the chunks of the one bucket)
    const int groups = p.bk_offsets ? max(p.n_expert, 1) : ceil_div(p.rows, kBucketT);
    int tiles = max(1, 4 * p.n_cu / groups);
    int ft = ceil_div(p.nff, tiles);
    ft = ceil_div(ft, 4 * rw * 2) * 4 * rw * 2;   // whole rounds of 4 waves x U = 2 row groups
    dim3 grid(ceil_div(p.nff, ft), p.n_expert, ceil_div(p.max_bucket ? p.max_bucket : p.rows, kBucketT)), block(256);
    INFR_LAUNCH((moe_gate_up_bucketed<F, 2, kBucketT>), grid, block, kBucketT * cells_bytes(p.ne), s, p, ft);
}

template <class F>
static void down_bucketed(hipStream_t s, const MoeGemvParams& p) {
    const int rw = 64 / (p.nff / F::kBlockElems * F::kLPB);
    const int groups = p.bk_offsets ? max(p.n_expert, 1) : ceil_div(p.rows, kBucketT);
    int tiles = max(1, 4 * p.n_cu / groups);
    int ot = ceil_div(p.ne, tiles);
    ot = ceil_div(ot, 4 * rw * 4) * 4 * rw * 4;   // whole rounds of 4 waves x U = 4 row groups
    dim3 grid(ceil_div(p.ne, ot), p.n_expert, ceil_div(p.max_bucket ? p.max_bucket : p.rows, kBucketT)), block(256);
    INFR_LAUNCH((moe_down_bucketed<F, 4, kBucketT>), grid, block, kBucketT * cells_bytes(p.nff), s, p, ot);
}

bool bucketed_rows_supported(int dt, int k) {
    if (kBucketT * cells_bytes(k) > 48 * 1024) return false;   // the staged cells must fit the default LDS window
    if (dt == INFR_Q4K) return fast_ok<Q4KFmt>(k);
    if (dt == INFR_Q6K) return fast_ok<Q6KFmt>(k);
    if (dt == INFR_Q8_0) return fast_ok<Q80Fmt>(k);
    return false;
}

bool moe_bucketed_supported(const MoeGemvParams& p) {
    if (p.gate_dt != p.up_dt || p.fused_gate_up) return false;
    return bucketed_rows_supported(p.gate_dt, p.ne) && bucketed_rows_supported(p.down_dt, p.nff);
}

void launch_moe_gate_up_bucketed(hipStream_t s, const MoeGemvParams& p) {
    if (p.gate_dt == INFR_Q4K) gate_up_bucketed<Q4KFmt>(s, p);
    else if (p.gate_dt == INFR_Q6K) gate_up_bucketed<Q6KFmt>(s, p);
    else gate_up_bucketed<Q80Fmt>(s, p);
}

void launch_moe_down_bucketed(hipStream_t s, const MoeGemvParams& p) {
    if (p.down_dt == INFR_Q4K) down_bucketed<Q4KFmt>(s, p);
    else if (p.down_dt == INFR_Q6K) down_bucketed<Q6KFmt>(s, p);
    else down_bucketed<Q80Fmt>(s, p);
}

// ------------------------------------------------------------------------------- Op::Linear
// dst[m, out_f] = x . W^T, the dense neighbour of the expert GEMVs (shared expert).
template <class F>
__global__ __launch_bounds__(256) void linear_fast(const float* __restrict__ xin, const uint8_t* __restrict__ w,
                                                   int in_f, int out_f, float* __restrict__ dst, int ot,
                                                   const float* __restrict__ addend) {
    extern __shared__ uint32_t dyn_lds[];
    constexpr int U = 4;  // rows a wave keeps in flight
    const int r = blockIdx.y;
    const int o0 = blockIdx.x * ot;
    const int ocount = min(ot, out_f - o0);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int nblk = in_f / F::kBlockElems;
    const size_t row_bytes = (size_t)nblk * F::kBlockBytes;
    const Place<F> pl(nblk, lane);
    const uint8_t* bank = w + (size_t)o0 * row_bytes;
    const int per_round = 4 * pl.rw_count;
    uint32_t* cells = dyn_lds + (size_t)wave * ((in_f + 31) / 32) * kCellDwords;
    const float* xrow = xin + (size_t)r * in_f;
    const XLoad xl = stage_x_load(xrow, in_f, lane);
    typename F::X x;
    bool have_x = false;
    for (int base = 0; base < ocount; base += per_round * U) {
        typename F::Raw raw[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int o = min(base + (u * 4 + wave) * pl.rw_count + pl.rw, ocount - 1);
            raw[u] = load_row<F>(pl, bank + (size_t)o * row_bytes);
        }
        if (!have_x) {
            stage_x_finish<F::kGroup, F::kSigned>(xl, xrow, in_f, cells, lane);
            __builtin_amdgcn_wave_barrier();
            F::fetch_x(x, cells, pl.blk, pl.sub);
            have_x = true;
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int o = base + (u * 4 + wave) * pl.rw_count + pl.rw;
            float y = row_sum<F>(F::dot(raw[u], pl.sub, x), pl, nblk);
            if (o < ocount && pl.writer()) {
                const size_t oi = (size_t)r * out_f + o0 + o;
                dst[oi] = addend ? __fadd_rn(addend[oi], y) : y;
            }
        }
    }
}

__global__ __launch_bounds__(256) void linear_generic(const float* __restrict__ x, const uint8_t* __restrict__ w,
                                                      int dt, size_t row_bytes, int in_f, int out_f,
                                                      float* __restrict__ dst, const float* __restrict__ addend) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int o = blockIdx.x * 4 + wave;
    const int r = blockIdx.y;
    if (o >= out_f) return;
    const uint8_t* row = w + (size_t)o * row_bytes;
    const float* xr = x + (size_t)r * in_f;
    float y = 0.f;
    for (int k = lane; k < in_f; k += kWave) y = fmaf(decode_elem(dt, row, (uint32_t)k), xr[k], y);
    y = wave_sum(y);
    if (lane == 0) {
        const size_t oi = (size_t)r * out_f + o;
        dst[oi] = addend ? __fadd_rn(addend[oi], y) : y;
    }
}

template <class F>
static bool try_linear(hipStream_t s, const float* x, const uint8_t* w, int m, int in_f, int out_f, float* dst,
                       int n_cu, const float* addend) {
    if (!fast_ok<F>(in_f)) return false;
    const int rw = 64 / (in_f / F::kBlockElems * F::kLPB);
    int ot = ceil_div(out_f, n_cu);
    ot = ceil_div(ot, 4 * rw) * 4 * rw;  // whole rounds of the block's 4 waves
    dim3 grid(ceil_div(out_f, ot), m), block(256);
    INFR_LAUNCH((linear_fast<F>), grid, block, 4 * cells_bytes(in_f), s, x, w, in_f, out_f, dst, ot, addend);
    return true;
}

// Several rows: the rows are one bucket of the bucketed down kernel (two rows share each weight row).
static bool linear_rows(hipStream_t s, const float* x, const uint8_t* w, int dt, int m, int in_f, int out_f, float* dst,
                        int n_cu, const float* addend) {
    if (!bucketed_rows_supported(dt, in_f)) return false;
    MoeGemvParams q{};
    q.x = x;
    q.down = w;
    q.down_dt = dt;
    q.nff = in_f;
    q.ne = out_f;
    q.rows = m;
    q.n_expert = 1;
    q.n_used = 1;
    q.y = dst;
    q.addend = addend;
    q.n_cu = n_cu;
    launch_moe_down_bucketed(s, q);
    return true;
}

void launch_linear(hipStream_t s, const float* x, const uint8_t* w, int dt, size_t row_bytes, int m, int in_f,
                   int out_f, float* dst, int n_cu, const float* addend) {
    if (m >= 2 && linear_rows(s, x, w, dt, m, in_f, out_f, dst, n_cu, addend)) return;
    bool done = false;
    if (dt == INFR_Q4K) done = try_linear<Q4KFmt>(s, x, w, m, in_f, out_f, dst, n_cu, addend);
    else if (dt == INFR_Q6K) done = try_linear<Q6KFmt>(s, x, w, m, in_f, out_f, dst, n_cu, addend);
    else if (dt == INFR_Q8_0) done = try_linear<Q80Fmt>(s, x, w, m, in_f, out_f, dst, n_cu, addend);
    if (done) return;
    if (linear_float_supported(dt, in_f, row_bytes, x, w)) {
        launch_linear_float(s, x, w, dt, row_bytes, m, in_f, out_f, dst, addend);
        return;
    }
    if (linear_units_supported(dt, in_f, x)) {   // every other affine format, and the shapes the kernels above refuse
        launch_linear_units(s, x, w, dt, row_bytes, m, in_f, out_f, dst, addend);
        return;
    }
    dim3 grid((out_f + 3) / 4, m), block(256);
    INFR_LAUNCH(linear_generic, grid, block, 0, s, x, w, dt, row_bytes, in_f, out_f, dst, addend);
}

}  // namespace infr

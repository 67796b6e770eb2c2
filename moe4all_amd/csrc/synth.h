// Seeded synthetic workload: N(0, sigma) tensors and ggml-compatible Q8_0 / Q4_K / Q6_K
// quantisers, written once and compiled for BOTH the host and the gfx950 device so the two
// produce the same bytes.  The reference ships no weight quantiser for these formats
// (weights arrive pre-quantised in GGUF files); Q8_0 follows the reference's own test helper
// (crates/infr-metal/tests/parity.rs:271-287), Q4_K / Q6_K follow ggml's published
// quantize_row_q4_K_ref / quantize_row_q6_K_ref.
//
// Determinism: only +, -, *, /, sqrt and explicit fma are used (no libm), and FP contraction
// is off for this header, so host and device round identically.
#pragma once

#include <stdint.h>
#include <string.h>

#if defined(__HIPCC__)
#define SYN_HD __host__ __device__
#else
#define SYN_HD
#endif

#pragma clang fp contract(off)

namespace synth {

// ---- counter-based uniform stream: SplitMix64 output number k of stream `seed` ----------
SYN_HD inline uint64_t splitmix64_at(uint64_t seed, uint64_t k) {
    uint64_t z = seed + (k + 1) * 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

SYN_HD inline double u64_as_double(uint64_t u) {
    double d;
    memcpy(&d, &u, 8);
    return d;
}
SYN_HD inline uint64_t double_as_u64(double d) {
    uint64_t u;
    memcpy(&u, &d, 8);
    return u;
}

// ln(u) for u in (0, 1], |error| ~ 1e-16: u = m * 2^e, m in [sqrt(1/2), sqrt(2)),
// ln m = 2 atanh((m-1)/(m+1)) as an odd series.
SYN_HD inline double det_log(double u) {
    uint64_t b = double_as_u64(u);
    int e = (int)((b >> 52) & 0x7FF) - 1023;
    double m = u64_as_double((b & 0x000FFFFFFFFFFFFFull) | 0x3FF0000000000000ull);  // [1, 2)
    if (m > 1.4142135623730951) {
        m = m * 0.5;
        e += 1;
    }
    double s = (m - 1.0) / (m + 1.0);
    double s2 = s * s;
    double p = 1.0 / 23.0;
    p = __builtin_fma(p, s2, 1.0 / 21.0);
    p = __builtin_fma(p, s2, 1.0 / 19.0);
    p = __builtin_fma(p, s2, 1.0 / 17.0);
    p = __builtin_fma(p, s2, 1.0 / 15.0);
    p = __builtin_fma(p, s2, 1.0 / 13.0);
    p = __builtin_fma(p, s2, 1.0 / 11.0);
    p = __builtin_fma(p, s2, 1.0 / 9.0);
    p = __builtin_fma(p, s2, 1.0 / 7.0);
    p = __builtin_fma(p, s2, 1.0 / 5.0);
    p = __builtin_fma(p, s2, 1.0 / 3.0);
    p = __builtin_fma(p, s2, 1.0);
    double lnm = 2.0 * s * p;
    return __builtin_fma((double)e, 0.6931471805599453, lnm);
}

// sin and cos of 2*pi*t for t in [0, 1).
SYN_HD inline void det_sincos_turn(double t, double* sn, double* cs) {
    double t4 = t * 4.0;
    int q = (int)t4;  // quadrant 0..3
    double f = t4 - (double)q;
    double b = (f - 0.5) * 1.5707963267948966;  // [-pi/4, pi/4)
    double b2 = b * b;
    double sp = 1.0 / 355687428096000.0;  // 1/17!
    sp = __builtin_fma(sp, b2, -1.0 / 1307674368000.0);
    sp = __builtin_fma(sp, b2, 1.0 / 6227020800.0);
    sp = __builtin_fma(sp, b2, -1.0 / 39916800.0);
    sp = __builtin_fma(sp, b2, 1.0 / 362880.0);
    sp = __builtin_fma(sp, b2, -1.0 / 5040.0);
    sp = __builtin_fma(sp, b2, 1.0 / 120.0);
    sp = __builtin_fma(sp, b2, -1.0 / 6.0);
    sp = __builtin_fma(sp, b2, 1.0);
    double sb = b * sp;
    double cp = 1.0 / 20922789888000.0;  // 1/16!
    cp = __builtin_fma(cp, b2, -1.0 / 87178291200.0);
    cp = __builtin_fma(cp, b2, 1.0 / 479001600.0);
    cp = __builtin_fma(cp, b2, -1.0 / 3628800.0);
    cp = __builtin_fma(cp, b2, 1.0 / 40320.0);
    cp = __builtin_fma(cp, b2, -1.0 / 720.0);
    cp = __builtin_fma(cp, b2, 1.0 / 24.0);
    cp = __builtin_fma(cp, b2, -0.5);
    cp = __builtin_fma(cp, b2, 1.0);
    double cb = cp;
    const double r = 0.7071067811865476;
    double s0 = (sb + cb) * r;  // sin(b + pi/4)
    double c0 = (cb - sb) * r;  // cos(b + pi/4)
    switch (q & 3) {
        case 0: *sn = s0; *cs = c0; break;
        case 1: *sn = c0; *cs = -s0; break;
        case 2: *sn = -s0; *cs = -c0; break;
        default: *sn = -c0; *cs = s0; break;
    }
}

// Element pair k of stream `seed`: two independent N(0,1) deviates (Box-Muller in f64).
SYN_HD inline void normal_pair(uint64_t seed, uint64_t k, double* z0, double* z1) {
    uint64_t a = splitmix64_at(seed, 2 * k);
    uint64_t b = splitmix64_at(seed, 2 * k + 1);
    double u1 = (double)((a >> 11) + 1) * (1.0 / 9007199254740992.0);  // (0, 1]
    double u2 = (double)(b >> 11) * (1.0 / 9007199254740992.0);        // [0, 1)
    double r = __builtin_sqrt(-2.0 * det_log(u1));
    double sn, cs;
    det_sincos_turn(u2, &sn, &cs);
    *z0 = r * cs;
    *z1 = r * sn;
}

// Element i of the N(0, sigma) f32 tensor with stream `seed`.
SYN_HD inline float normal_at(uint64_t seed, uint64_t i, double sigma) {
    double z0, z1;
    normal_pair(seed, i >> 1, &z0, &z1);
    return (float)(((i & 1) ? z1 : z0) * sigma);
}

// ---- f32 -> f16 bits, round to nearest even (ggml's GGML_FP32_TO_FP16) -------------------
SYN_HD inline uint16_t f32_to_f16_bits(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t ax = x & 0x7FFFFFFFu;
    if (ax >= 0x7F800000u) return (uint16_t)(sign | (ax > 0x7F800000u ? 0x7E00u : 0x7C00u));
    if (ax >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u);  // rounds to >= 65520 -> inf
    if (ax < 0x38800000u) {                                    // subnormal half or zero
        if (ax < 0x33000000u) return (uint16_t)sign;           // < 2^-25 -> 0
        uint32_t e = ax >> 23;
        uint32_t man = (ax & 0x7FFFFFu) | 0x800000u;
        uint32_t shift = 126u - e;                             // 14..24
        uint32_t h = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1u);
        uint32_t halfway = 1u << (shift - 1u);
        if (rem > halfway || (rem == halfway && (h & 1u))) h++;
        return (uint16_t)(sign | h);
    }
    uint32_t h = ((ax - 0x38000000u) >> 13);
    uint32_t rem = ax & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h++;
    return (uint16_t)(sign | h);
}

SYN_HD inline float f16_bits_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1Fu, m = h & 0x3FFu, bits;
    if (e == 0) {
        if (m == 0) bits = sign;
        else {
            int k = -1;
            do { m <<= 1; k++; } while (!(m & 0x400u));
            bits = sign | ((uint32_t)(112 - k) << 23) | ((m & 0x3FFu) << 13);
        }
    } else if (e == 31) bits = sign | 0x7F800000u | (m << 13);
    else bits = sign | ((e + 112u) << 23) | (m << 13);
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

SYN_HD inline int nearest_int(float fval) {
    float val = fval + 12582912.f;
    int i;
    memcpy(&i, &val, 4);
    return (i & 0x007fffff) - 0x00400000;
}
SYN_HD inline float fabs_(float v) { return v < 0 ? -v : v; }
SYN_HD inline int imin(int a, int b) { return a < b ? a : b; }
SYN_HD inline int imax(int a, int b) { return a > b ? a : b; }

// ---- Q8_0: d = amax/127, q = round_half_away(v/d) clamped to +-127 -------------------------
SYN_HD inline void quantize_block_q8_0(const float* x, uint8_t* out) {
    float amax = 0.f;
    for (int i = 0; i < 32; i++) { float a = fabs_(x[i]); if (a > amax) amax = a; }
    float d = amax > 0.f ? amax / 127.0f : 0.f;
    uint16_t dh = f32_to_f16_bits(d);
    out[0] = (uint8_t)(dh & 0xFF);
    out[1] = (uint8_t)(dh >> 8);
    for (int i = 0; i < 32; i++) {
        int q = 0;
        if (d > 0.f) {
            float v = x[i] / d;
            float r = (float)(int)v;          // |v| <= 127: truncation is exact
            float frac = v - r;               // exact
            if (frac >= 0.5f) r += 1.0f;      // f32::round: half away from zero
            else if (frac <= -0.5f) r -= 1.0f;
            if (r < -127.f) r = -127.f;
            if (r > 127.f) r = 127.f;
            q = (int)r;
        }
        out[2 + i] = (uint8_t)(int8_t)q;
    }
}

// ---- Q4_K (ggml make_qkx2_quants + quantize_row_q4_K_ref) ---------------------------------
SYN_HD inline float make_qkx2_quants(int n, int nmax, const float* x, const float* weights, uint8_t* L,
                                     float* the_min, uint8_t* Laux, float rmin, float rdelta, int nstep) {
    float mn = x[0], mx = x[0];
    float sum_w = weights[0];
    float sum_x = sum_w * x[0];
    for (int i = 1; i < n; ++i) {
        if (x[i] < mn) mn = x[i];
        if (x[i] > mx) mx = x[i];
        float w = weights[i];
        sum_w += w;
        sum_x += w * x[i];
    }
    if (mn > 0) mn = 0;
    if (mx == mn) {
        for (int i = 0; i < n; ++i) L[i] = 0;
        *the_min = -mn;
        return 0.f;
    }
    float iscale = nmax / (mx - mn);
    float scale = 1 / iscale;
    float best_mad = 0;
    for (int i = 0; i < n; ++i) {
        int l = nearest_int(iscale * (x[i] - mn));
        L[i] = (uint8_t)imax(0, imin(nmax, l));
        float diff = scale * L[i] + mn - x[i];
        diff = diff * diff;
        best_mad += weights[i] * diff;
    }
    if (nstep < 1) {
        *the_min = -mn;
        return scale;
    }
    for (int is = 0; is <= nstep; ++is) {
        iscale = (rmin + rdelta * is + nmax) / (mx - mn);
        float sum_l = 0, sum_l2 = 0, sum_xl = 0;
        for (int i = 0; i < n; ++i) {
            int l = nearest_int(iscale * (x[i] - mn));
            l = imax(0, imin(nmax, l));
            Laux[i] = (uint8_t)l;
            float w = weights[i];
            sum_l += w * l;
            sum_l2 += w * l * l;
            sum_xl += w * l * x[i];
        }
        float D = sum_w * sum_l2 - sum_l * sum_l;
        if (D > 0) {
            float this_scale = (sum_w * sum_xl - sum_x * sum_l) / D;
            float this_min = (sum_l2 * sum_x - sum_l * sum_xl) / D;
            if (this_min > 0) {
                this_min = 0;
                this_scale = sum_xl / sum_l2;
            }
            float mad = 0;
            for (int i = 0; i < n; ++i) {
                float diff = this_scale * Laux[i] + this_min - x[i];
                diff = diff * diff;
                mad += weights[i] * diff;
            }
            if (mad < best_mad) {
                for (int i = 0; i < n; ++i) L[i] = Laux[i];
                best_mad = mad;
                scale = this_scale;
                mn = this_min;
            }
        }
    }
    *the_min = -mn;
    return scale;
}

SYN_HD inline void k4_get(int j, const uint8_t* q, uint8_t* d, uint8_t* m) {
    if (j < 4) {
        *d = q[j] & 63;
        *m = q[j + 4] & 63;
    } else {
        *d = (uint8_t)((q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4));
        *m = (uint8_t)((q[j + 4] >> 4) | ((q[j - 0] >> 6) << 4));
    }
}

SYN_HD inline void quantize_block_q4_K(const float* x, uint8_t* y /*144 B*/) {
    uint8_t L[256];
    uint8_t Laux[32];
    float weights[32];
    float mins[8];
    float scales[8];
    float max_scale = 0, max_min = 0;
    for (int j = 0; j < 8; ++j) {
        float sum_x2 = 0;
        for (int l = 0; l < 32; ++l) sum_x2 += x[32 * j + l] * x[32 * j + l];
        float av_x = __builtin_sqrtf(sum_x2 / 32);
        for (int l = 0; l < 32; ++l) weights[l] = av_x + fabs_(x[32 * j + l]);
        scales[j] = make_qkx2_quants(32, 15, x + 32 * j, weights, L + 32 * j, &mins[j], Laux, -1.f, 0.1f, 20);
        if (scales[j] > max_scale) max_scale = scales[j];
        if (mins[j] > max_min) max_min = mins[j];
    }
    float inv_scale = max_scale > 0 ? 63.f / max_scale : 0.f;
    float inv_min = max_min > 0 ? 63.f / max_min : 0.f;
    uint8_t* sc = y + 4;
    for (int j = 0; j < 12; j++) sc[j] = 0;
    for (int j = 0; j < 8; ++j) {
        uint8_t ls = (uint8_t)nearest_int(inv_scale * scales[j]);
        uint8_t lm = (uint8_t)nearest_int(inv_min * mins[j]);
        ls = ls < 63 ? ls : 63;
        lm = lm < 63 ? lm : 63;
        if (j < 4) {
            sc[j] = ls;
            sc[j + 4] = lm;
        } else {
            sc[j + 4] = (uint8_t)((ls & 0xF) | ((lm & 0xF) << 4));
            sc[j - 4] |= (uint8_t)((ls >> 4) << 6);
            sc[j - 0] |= (uint8_t)((lm >> 4) << 6);
        }
    }
    uint16_t dh = f32_to_f16_bits(max_scale / 63.f);
    uint16_t mh = f32_to_f16_bits(max_min / 63.f);
    y[0] = (uint8_t)(dh & 0xFF); y[1] = (uint8_t)(dh >> 8);
    y[2] = (uint8_t)(mh & 0xFF); y[3] = (uint8_t)(mh >> 8);
    const float dd = f16_bits_to_f32(dh), dmn = f16_bits_to_f32(mh);
    for (int j = 0; j < 8; ++j) {
        uint8_t s, m;
        k4_get(j, sc, &s, &m);
        const float d = dd * s;
        if (!d) continue;
        const float dm = dmn * m;
        for (int ii = 0; ii < 32; ++ii) {
            int l = nearest_int((x[32 * j + ii] + dm) / d);
            L[32 * j + ii] = (uint8_t)imax(0, imin(15, l));
        }
    }
    uint8_t* q = y + 16;
    for (int j = 0; j < 256; j += 64) {
        for (int l = 0; l < 32; ++l) q[l] = (uint8_t)(L[j + l] | (L[j + l + 32] << 4));
        q += 32;
    }
}

// ---- Q6_K (ggml make_qx_quants rmse_type 1 + quantize_row_q6_K_ref) ------------------------
SYN_HD inline float make_qx_quants(int n, int nmax, const float* x, int8_t* L) {
    float mx = 0, amax = 0;
    for (int i = 0; i < n; ++i) {
        float ax = fabs_(x[i]);
        if (ax > amax) { amax = ax; mx = x[i]; }
    }
    if (amax < 1e-15f) {
        for (int i = 0; i < n; ++i) L[i] = 0;
        return 0.f;
    }
    float iscale = -nmax / mx;
    float sumlx = 0, suml2 = 0;
    for (int i = 0; i < n; ++i) {
        int l = nearest_int(iscale * x[i]);
        l = imax(-nmax, imin(nmax - 1, l));
        L[i] = (int8_t)(l + nmax);
        float w = x[i] * x[i];
        sumlx += w * x[i] * l;
        suml2 += w * l * l;
    }
    float scale = suml2 ? sumlx / suml2 : 0.0f;
    float best = scale * sumlx;
    for (int is = -9; is <= 9; ++is) {
        if (is == 0) continue;
        iscale = -(nmax + 0.1f * is) / mx;
        sumlx = suml2 = 0;
        for (int i = 0; i < n; ++i) {
            int l = nearest_int(iscale * x[i]);
            l = imax(-nmax, imin(nmax - 1, l));
            float w = x[i] * x[i];
            sumlx += w * x[i] * l;
            suml2 += w * l * l;
        }
        if (suml2 > 0 && sumlx * sumlx > best * suml2) {
            for (int i = 0; i < n; ++i) {
                int l = nearest_int(iscale * x[i]);
                L[i] = (int8_t)(nmax + imax(-nmax, imin(nmax - 1, l)));
            }
            scale = sumlx / suml2;
            best = scale * sumlx;
        }
    }
    return scale;
}

SYN_HD inline void quantize_block_q6_K(const float* x, uint8_t* y /*210 B*/) {
    int8_t L[256];
    float scales[16];
    float max_scale = 0, max_abs_scale = 0;
    for (int ib = 0; ib < 16; ++ib) {
        const float scale = make_qx_quants(16, 32, x + 16 * ib, L + 16 * ib);
        scales[ib] = scale;
        const float a = fabs_(scale);
        if (a > max_abs_scale) { max_abs_scale = a; max_scale = scale; }
    }
    if (max_abs_scale < 1e-15f) {
        for (int i = 0; i < 210; i++) y[i] = 0;
        return;
    }
    float iscale = -128.f / max_scale;
    uint16_t dh = f32_to_f16_bits(1 / iscale);
    y[208] = (uint8_t)(dh & 0xFF);
    y[209] = (uint8_t)(dh >> 8);
    int8_t* ysc = (int8_t*)(y + 192);
    for (int ib = 0; ib < 16; ++ib) ysc[ib] = (int8_t)imin(127, nearest_int(iscale * scales[ib]));
    const float dd = f16_bits_to_f32(dh);
    for (int j = 0; j < 16; ++j) {
        float d = dd * ysc[j];
        if (!d) continue;
        for (int ii = 0; ii < 16; ++ii) {
            int l = nearest_int(x[16 * j + ii] / d);
            l = imax(-32, imin(31, l));
            L[16 * j + ii] = (int8_t)(l + 32);
        }
    }
    uint8_t* ql = y;
    uint8_t* qh = y + 128;
    for (int j = 0; j < 256; j += 128) {
        for (int l = 0; l < 32; ++l) {
            const uint8_t q1 = L[j + l + 0] & 0xF;
            const uint8_t q2 = L[j + l + 32] & 0xF;
            const uint8_t q3 = L[j + l + 64] & 0xF;
            const uint8_t q4 = L[j + l + 96] & 0xF;
            ql[l + 0] = (uint8_t)(q1 | (q3 << 4));
            ql[l + 32] = (uint8_t)(q2 | (q4 << 4));
            qh[l] = (uint8_t)((L[j + l] >> 4) | ((L[j + l + 32] >> 4) << 2) | ((L[j + l + 64] >> 4) << 4) |
                              ((L[j + l + 96] >> 4) << 6));
        }
        ql += 64;
        qh += 32;
    }
}

// ---- MXFP4: shared exponent e = floor(log2(amax)) - 2 + 127 (E8M0, so that the largest magnitude lands in
// [4, 8) of the E2M1 range 0 .. 6), each element the nearest entry of the twice-E2M1 book times 2^(e - 128)
// (first entry on a tie), low nibbles = elements 0..15, high nibbles = 16..31: ggml's quantize_row_mxfp4_ref.
SYN_HD inline void quantize_block_mxfp4(const float* x, uint8_t* out /*17 B*/) {
    const int book[16] = {0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12};
    float amax = 0.f;
    for (int i = 0; i < 32; i++) { float a = fabs_(x[i]); if (a > amax) amax = a; }
    uint32_t bits;
    memcpy(&bits, &amax, 4);
    // floor(log2(amax)) from the exponent field (a subnormal amax counts as the smallest normal)
    const int eb = amax > 0.f ? imax((int)((bits >> 23) & 0xFF), 1) - 2 : 0;
    const uint8_t e = (uint8_t)imax(eb, 0);
    const uint32_t dbits = e < 2 ? 0x00200000u << e : ((uint32_t)e - 1u) << 23;   // 2^(e - 128)
    float d;
    memcpy(&d, &dbits, 4);
    out[0] = e;
    for (int j = 0; j < 16; j++) {
        uint8_t nib[2];
        for (int h = 0; h < 2; h++) {
            const float v = x[j + 16 * h];
            int best = 0;
            float berr = fabs_((float)book[0] * d - v);
            for (int i = 1; i < 16; i++) {
                const float err = fabs_((float)book[i] * d - v);
                if (err < berr) { berr = err; best = i; }
            }
            nib[h] = (uint8_t)best;
        }
        out[1 + j] = (uint8_t)(nib[0] | (nib[1] << 4));
    }
}

// Quantise 256 consecutive elements starting at element index e0 of the N(0,sigma) tensor
// `seed` into `out` (Q8_0: 8 blocks = 272 B, Q4_K: 144 B, Q6_K: 210 B, MXFP4: 8 blocks = 136 B).
SYN_HD inline void synth_superblock(int dtype, uint64_t seed, uint64_t e0, double sigma, uint8_t* out) {
    float x[256];
    for (int k = 0; k < 128; k++) {
        double z0, z1;
        normal_pair(seed, (e0 >> 1) + (uint64_t)k, &z0, &z1);
        x[2 * k] = (float)(z0 * sigma);
        x[2 * k + 1] = (float)(z1 * sigma);
    }
    if (dtype == 9) {
        for (int b = 0; b < 8; b++) quantize_block_q8_0(x + 32 * b, out + 34 * b);
    } else if (dtype == 12) {
        quantize_block_q4_K(x, out);
    } else if (dtype == 28) {
        for (int b = 0; b < 8; b++) quantize_block_mxfp4(x + 32 * b, out + 17 * b);
    } else {
        quantize_block_q6_K(x, out);
    }
}

}  // namespace synth

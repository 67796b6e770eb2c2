/*
 * CPU oracle for the routed-expert MoE FFN path.  TEST INFRASTRUCTURE ONLY (parity checker
 * and timed CPU baseline); the HIP backend never links or calls this file.
 *
 * Plain-C restatement of the reference engine's CPU backend in its f32 "reference" numerics
 * mode.  Build with -ffp-contract=off: the reference is Rust, which performs no FP
 * contraction, so a*b+c is two roundings everywhere except where Rust wrote mul_add (fmaf).
 */
#include "infr_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------ f16 / geometry */

/* IEEE binary16 -> binary32, exact (the `half` crate's f16::to_f32 used at
 * crates/infr-gguf/src/dequant.rs:70-73). */
float orc_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: normalise */
            int e = -1;
            do { man <<= 1; e++; } while (!(man & 0x400u));
            man &= 0x3FFu;
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7F800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* crates/infr-core/src/decode_spec.rs:320 (Q8_0 2+32), :327 (Q4_K 2+2+12+128), :331 (Q6_K
 * 128+64+16+2). */
int orc_block_geometry(int dtype, int *block_elems, int *block_bytes) {
    int e, b;
    switch (dtype) {
    case ORC_F32: case ORC_I32: case ORC_U32: e = 1; b = 4; break;
    case ORC_F16: case ORC_BF16: e = 1; b = 2; break;
    case ORC_Q4_0: e = 32; b = 18; break;
    case ORC_Q4_1: e = 32; b = 20; break;
    case ORC_Q5_0: e = 32; b = 22; break;
    case ORC_Q5_1: e = 32; b = 24; break;
    case ORC_Q8_0: e = 32; b = 34; break;
    case ORC_Q2K: e = 256; b = 84; break;
    case ORC_Q3K: e = 256; b = 110; break;
    case ORC_Q4K: e = 256; b = 144; break;
    case ORC_Q5K: e = 256; b = 176; break;
    case ORC_Q6K: e = 256; b = 210; break;
    /* decode_spec.rs:349-363 */
    case ORC_IQ4_NL: e = 32; b = 18; break;
    case ORC_IQ4_XS: e = 256; b = 136; break;
    case ORC_TQ1_0: e = 256; b = 54; break;
    case ORC_TQ2_0: e = 256; b = 66; break;
    case ORC_Q2_0: e = 64; b = 18; break;
    case ORC_MXFP4: e = 32; b = 17; break;
    case ORC_NVFP4: e = 64; b = 36; break;
    /* decode_spec.rs:334-347 */
    case ORC_IQ1_S: e = 256; b = 50; break;
    case ORC_IQ1_M: e = 256; b = 56; break;
    case ORC_IQ2_XXS: e = 256; b = 66; break;
    case ORC_IQ2_XS: e = 256; b = 74; break;
    case ORC_IQ2_S: e = 256; b = 82; break;
    case ORC_IQ3_XXS: e = 256; b = 98; break;
    case ORC_IQ3_S: e = 256; b = 110; break;
    default: return -1;
    }
    if (block_elems) *block_elems = e;
    if (block_bytes) *block_bytes = b;
    return 0;
}

int64_t orc_bytes_for(int dtype, int64_t numel) {
    int e, b;
    if (orc_block_geometry(dtype, &e, &b) != 0 || numel < 0 || numel % e != 0) return -1;
    return numel / e * b;
}

/* crates/infr-gguf/src/dequant.rs:77-87 */
void orc_k4(int j, const uint8_t *q, uint32_t *sc, uint32_t *m) {
    if (j < 4) {
        *sc = q[j] & 63u;
        *m = q[j + 4] & 63u;
    } else {
        *sc = (uint32_t)((q[j + 4] & 0x0F) | ((q[j - 4] >> 6) << 4));
        *m = (uint32_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4));
    }
}

/* ------------------------------------------------------------------ dequant */

/* Factored form of one block (crates/infr-gguf/src/dequant.rs:89-108): a u8 code per element,
 * an (sc, m) i16 pair per 16 elements, one (d, dmin) f16 pair per block. */
typedef struct {
    uint8_t codes[256];
    int16_t scm[32];
    uint16_t dd[2];
} factored_block;

/* Expand exactly as dequant_block does (dequant.rs:35-51):
 *   sc = f32(d) * f32(scm_sc); mn = f32(dmin) * f32(scm_m); out = sc * f32(code) + mn
 * with a separate multiply and add. */
static void expand_block(const factored_block *f, int n, float *out) {
    float dsc = orc_f16_to_f32(f->dd[0]);
    float dmn = orc_f16_to_f32(f->dd[1]);
    for (int b16 = 0; b16 < n / 16; b16++) {
        float sc = dsc * (float)f->scm[2 * b16];
        float mn = dmn * (float)f->scm[2 * b16 + 1];
        for (int g = 0; g < 16; g++) {
            float prod = sc * (float)f->codes[b16 * 16 + g];
            out[b16 * 16 + g] = prod + mn;
        }
    }
}

static uint16_t rd_u16(const uint8_t *p) { return (uint16_t)(p[0] | (p[1] << 8)); }

/* dequant.rs:214-223 */
static void factor_q8_0(const uint8_t *blk, factored_block *f) {
    uint16_t d = rd_u16(blk);
    f->dd[0] = d;
    f->dd[1] = d;
    f->scm[0] = 1; f->scm[1] = -128;
    f->scm[2] = 1; f->scm[3] = -128;
    for (int i = 0; i < 32; i++) f->codes[i] = (uint8_t)((int16_t)(int8_t)blk[2 + i] + 128);
}

/* dequant.rs:315-335 */
static void factor_q4k(const uint8_t *blk, factored_block *f) {
    f->dd[0] = rd_u16(blk);
    f->dd[1] = rd_u16(blk + 2);
    const uint8_t *scales = blk + 4;
    const uint8_t *qs = blk + 16;
    for (int j = 0; j < 4; j++) {
        uint32_t sc1, m1, sc2, m2;
        orc_k4(2 * j, scales, &sc1, &m1);
        orc_k4(2 * j + 1, scales, &sc2, &m2);
        int b16 = j * 4;
        f->scm[2 * b16 + 0] = (int16_t)sc1; f->scm[2 * b16 + 1] = (int16_t)(-(int16_t)m1);
        f->scm[2 * b16 + 2] = (int16_t)sc1; f->scm[2 * b16 + 3] = (int16_t)(-(int16_t)m1);
        f->scm[2 * b16 + 4] = (int16_t)sc2; f->scm[2 * b16 + 5] = (int16_t)(-(int16_t)m2);
        f->scm[2 * b16 + 6] = (int16_t)sc2; f->scm[2 * b16 + 7] = (int16_t)(-(int16_t)m2);
        for (int l = 0; l < 32; l++) {
            uint8_t v = qs[j * 32 + l];
            f->codes[j * 64 + l] = v & 0xF;
            f->codes[j * 64 + 32 + l] = v >> 4;
        }
    }
}

/* dequant.rs:365-389 */
static void factor_q6k(const uint8_t *blk, factored_block *f) {
    const uint8_t *ql = blk;
    const uint8_t *qh = blk + 128;
    const uint8_t *scales = blk + 192;
    f->dd[0] = rd_u16(blk + 208);
    f->dd[1] = f->dd[0];
    for (int half = 0; half < 2; half++) {
        int qlo = half * 64, qho = half * 32, sco = half * 8, base = half * 128;
        for (int sci = 0; sci < 8; sci += 2) {
            for (int is = 0; is < 2; is++) {
                int16_t s = (int16_t)(int8_t)scales[sco + is + sci];
                int slot = base / 16 + sci + is;
                f->scm[2 * slot] = s;
                f->scm[2 * slot + 1] = (int16_t)(-32 * s);
            }
        }
        for (int l = 0; l < 32; l++) {
            f->codes[base + l] = (uint8_t)((ql[qlo + l] & 0xF) | ((qh[qho + l] & 3) << 4));
            f->codes[base + l + 32] =
                (uint8_t)((ql[qlo + l + 32] & 0xF) | (((qh[qho + l] >> 2) & 3) << 4));
            f->codes[base + l + 64] =
                (uint8_t)((ql[qlo + l] >> 4) | (((qh[qho + l] >> 4) & 3) << 4));
            f->codes[base + l + 96] =
                (uint8_t)((ql[qlo + l + 32] >> 4) | (((qh[qho + l] >> 6) & 3) << 4));
        }
    }
}

static uint32_t rd_u32(const uint8_t *p) {
    return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
}

/* The four legacy 32-element formats (dequant.rs:137-209): `nib` low nibbles are elements 0..15,
 * high nibbles 16..31; the 5-bit forms take bit j of qh for element j and bit j+16 for j+16
 * (written there as ((qh >> j) << 4) & 0x10 and (qh >> (j + 12)) & 0x10). */
static void factor_legacy(const uint8_t *blk, int has_min, int has_high, factored_block *f) {
    const uint8_t *p = blk + 2;
    f->dd[0] = rd_u16(blk);
    if (has_min) { f->dd[1] = rd_u16(p); p += 2; } else f->dd[1] = f->dd[0];
    uint32_t qh = 0;
    if (has_high) { qh = rd_u32(p); p += 4; }
    int16_t m = has_min ? 1 : (has_high ? -16 : -8);
    f->scm[0] = 1; f->scm[1] = m;
    f->scm[2] = 1; f->scm[3] = m;
    for (int j = 0; j < 16; j++) {
        uint32_t h0 = ((qh >> j) << 4) & 0x10u;
        uint32_t h1 = (qh >> (j + 12)) & 0x10u;
        f->codes[j] = (uint8_t)((p[j] & 0x0Fu) | h0);
        f->codes[j + 16] = (uint8_t)((uint32_t)(p[j] >> 4) | h1);
    }
}

/* dequant.rs:224-250: [scales 16][qs 64][d][dmin]; 16-element group g = 8n + 2j + half takes its
 * codes from qs[32n + 16*half ..][l] >> 2j and its (scale, min) nibbles from scales[g]. */
static void factor_q2k(const uint8_t *blk, factored_block *f) {
    const uint8_t *scales = blk, *qs = blk + 16;
    f->dd[0] = rd_u16(blk + 80);
    f->dd[1] = rd_u16(blk + 82);
    int g = 0;
    for (int n = 0; n < 2; n++)
        for (int j = 0; j < 4; j++)
            for (int half = 0; half < 2; half++, g++) {
                uint8_t sc = scales[g];
                f->scm[2 * g] = (int16_t)(sc & 0xF);
                f->scm[2 * g + 1] = (int16_t)(-(int16_t)(sc >> 4));
                for (int l = 0; l < 16; l++)
                    f->codes[16 * g + l] = (uint8_t)((qs[32 * n + 16 * half + l] >> (2 * j)) & 3);
            }
}

/* dequant.rs:251-312: [hmask 32][qs 64][scales 12][d]; the sixteen 6-bit scales are unpacked
 * with ggml's kmask shuffle, then each is offset by -32; the code is the 2 low bits from qs plus
 * bit (4n + j) of hmask[16*half + l] as bit 2; min = -4 * scale. */
static void factor_q3k(const uint8_t *blk, factored_block *f) {
    const uint8_t *hmask = blk, *qs = blk + 32, *sr = blk + 96;
    f->dd[0] = rd_u16(blk + 108);
    f->dd[1] = f->dd[0];
    const uint32_t k1 = 0x03030303u, k2 = 0x0f0f0f0fu;
    uint32_t a0 = rd_u32(sr), a1 = rd_u32(sr + 4), t = rd_u32(sr + 8);
    uint32_t aux[4];
    aux[2] = ((a0 >> 4) & k2) | (((t >> 4) & k1) << 4);
    aux[3] = ((a1 >> 4) & k2) | (((t >> 6) & k1) << 4);
    aux[0] = (a0 & k2) | ((t & k1) << 4);
    aux[1] = (a1 & k2) | (((t >> 2) & k1) << 4);
    int g = 0;
    for (int n = 0; n < 2; n++)
        for (int j = 0; j < 4; j++)
            for (int half = 0; half < 2; half++, g++) {
                int16_t s = (int16_t)((int16_t)(int8_t)((aux[g / 4] >> ((g % 4) * 8)) & 0xFF) - 32);
                f->scm[2 * g] = s;
                f->scm[2 * g + 1] = (int16_t)(-4 * s);
                uint8_t mbit = (uint8_t)(1u << (4 * n + j));
                for (int l = 0; l < 16; l++) {
                    uint8_t low2 = (uint8_t)((qs[32 * n + 16 * half + l] >> (2 * j)) & 3);
                    uint8_t high = (hmask[16 * half + l] & mbit) ? 1 : 0;
                    f->codes[16 * g + l] = (uint8_t)(low2 | (high << 2));
                }
            }
}

/* ------------------------------------------------------------------ scale-times-code formats
 * dequant_codebook (crates/infr-gguf/src/dequant.rs:493-1073) for the formats whose book fits in
 * sixteen entries or is arithmetic: one block in, its elements out, value = code * scale with the
 * reference's operand order. */
static const int8_t BOOK_IQ4NL[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113}; /* :442-444 */
static const int8_t BOOK_FP4[16] = {0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12};                    /* :409 */

/* e8m0_to_fp32_half (dequant.rs:415-421) */
static float e8m0_half(uint8_t x) {
    uint32_t bits = x < 2 ? 0x00200000u << x : ((uint32_t)x - 1u) << 23;
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* ue4m3_to_fp32 (dequant.rs:427-438) */
static float ue4m3_half(uint8_t x) {
    if (x == 0 || x == 0x7F) return 0.0f;
    int exp = (x >> 3) & 0xF;
    float man = (float)(x & 7);
    float raw = exp == 0 ? man * ldexpf(1.0f, -9) : (1.0f + man / 8.0f) * ldexpf(1.0f, exp - 7);
    return raw * 0.5f;
}

static int codebook_block(int dtype, const uint8_t *blk, float *out) {
    switch (dtype) {
    case ORC_IQ4_NL: { /* :499-519 */
        float d = orc_f16_to_f32(rd_u16(blk));
        for (int j = 0; j < 16; j++) {
            out[j] = d * (float)BOOK_IQ4NL[blk[2 + j] & 0xF];
            out[j + 16] = d * (float)BOOK_IQ4NL[blk[2 + j] >> 4];
        }
        return 0;
    }
    case ORC_IQ4_XS: { /* :521-559 */
        float d = orc_f16_to_f32(rd_u16(blk));
        unsigned scales_h = rd_u16(blk + 2);
        for (int ib = 0; ib < 8; ib++) {
            int ls = ((blk[4 + ib / 2] >> (4 * (ib % 2))) & 0xF) | (((scales_h >> (2 * ib)) & 3) << 4);
            float dl = d * (float)(ls - 32);
            const uint8_t *qs = blk + 8 + 16 * ib;
            for (int j = 0; j < 16; j++) {
                out[32 * ib + j] = dl * (float)BOOK_IQ4NL[qs[j] & 0xF];
                out[32 * ib + j + 16] = dl * (float)BOOK_IQ4NL[qs[j] >> 4];
            }
        }
        return 0;
    }
    case ORC_TQ1_0: { /* :926-970: five ternary digits per byte, most significant first after the multiply */
        static const uint8_t pow3[5] = {1, 3, 9, 27, 81};
        float d = orc_f16_to_f32(rd_u16(blk + 52));
        float *o = out;
        for (int n = 0; n < 5; n++)
            for (int m = 0; m < 32; m++) {
                uint8_t q = (uint8_t)(blk[m] * pow3[n]);
                *o++ = (float)((int)(((unsigned)q * 3u) >> 8) - 1) * d;
            }
        for (int n = 0; n < 5; n++)
            for (int m = 0; m < 16; m++) {
                uint8_t q = (uint8_t)(blk[32 + m] * pow3[n]);
                *o++ = (float)((int)(((unsigned)q * 3u) >> 8) - 1) * d;
            }
        for (int n = 0; n < 4; n++)
            for (int j = 0; j < 4; j++) {
                uint8_t q = (uint8_t)(blk[48 + j] * pow3[n]);
                *o++ = (float)((int)(((unsigned)q * 3u) >> 8) - 1) * d;
            }
        return 0;
    }
    case ORC_TQ2_0: { /* :978-1000 */
        float d = orc_f16_to_f32(rd_u16(blk + 64));
        float *o = out;
        for (int chunk = 0; chunk < 2; chunk++)
            for (int l = 0; l < 4; l++)
                for (int m = 0; m < 32; m++) *o++ = (float)(((blk[32 * chunk + m] >> (2 * l)) & 3) - 1) * d;
        return 0;
    }
    case ORC_Q2_0: { /* :1007-1022 */
        float d = orc_f16_to_f32(rd_u16(blk));
        for (int j = 0; j < 64; j++) out[j] = (float)(((blk[2 + j / 4] >> (2 * (j % 4))) & 3) - 1) * d;
        return 0;
    }
    case ORC_MXFP4: { /* :1029-1045 */
        float d = e8m0_half(blk[0]);
        for (int j = 0; j < 16; j++) {
            out[j] = (float)BOOK_FP4[blk[1 + j] & 0xF] * d;
            out[j + 16] = (float)BOOK_FP4[blk[1 + j] >> 4] * d;
        }
        return 0;
    }
    case ORC_NVFP4: { /* :1053-1073 */
        for (int s = 0; s < 4; s++) {
            float d = ue4m3_half(blk[s]);
            for (int j = 0; j < 8; j++) {
                out[16 * s + j] = (float)BOOK_FP4[blk[4 + 8 * s + j] & 0xF] * d;
                out[16 * s + j + 8] = (float)BOOK_FP4[blk[4 + 8 * s + j] >> 4] * d;
            }
        }
        return 0;
    }
    default: return -1;
    }
}

/* ------------------------------------------------------------------ grid i-quants */

/* The lattice codebooks (crates/infr-core/src/iquant_grids.rs) in the packed form the device library
 * uses: 2 or 3 bits per element into a small alphabet.  grid_entry() widens entry e back to the
 * reference's representation, one signed byte per element. */
#include "../moe4all_amd/csrc/iquant_grids.h"

enum { GRID_IQ2XXS, GRID_IQ2XS, GRID_IQ2S, GRID_IQ3XXS, GRID_IQ3S, GRID_IQ1S };
static const int8_t ALPHA_IQ2[3] = {8, 25, 43}, ALPHA_IQ3XXS[8] = {4, 12, 20, 28, 36, 44, 52, 62},
                    ALPHA_IQ3S[8] = {1, 3, 5, 7, 9, 11, 13, 15}, ALPHA_IQ1[3] = {0, 1, -1};

int orc_grid_entry(int grid, int e, int8_t *out) {
    const uint16_t *t;
    const int8_t *alpha;
    int n, bits, size;
    switch (grid) {
    case GRID_IQ2XXS: t = kIq2xxsGrid; size = 256; alpha = ALPHA_IQ2; n = 8; bits = 2; break;
    case GRID_IQ2XS: t = kIq2xsGrid; size = 512; alpha = ALPHA_IQ2; n = 8; bits = 2; break;
    case GRID_IQ2S: t = kIq2sGrid; size = 1024; alpha = ALPHA_IQ2; n = 8; bits = 2; break;
    case GRID_IQ3XXS: t = kIq3xxsGrid; size = 256; alpha = ALPHA_IQ3XXS; n = 4; bits = 3; break;
    case GRID_IQ3S: t = kIq3sGrid; size = 512; alpha = ALPHA_IQ3S; n = 4; bits = 3; break;
    case GRID_IQ1S: t = kIq1sGrid; size = 2048; alpha = ALPHA_IQ1; n = 8; bits = 2; break;
    default: return -1;
    }
    if (e < 0 || e >= size) return -1;
    for (int j = 0; j < n; j++) out[j] = alpha[(t[e] >> (bits * j)) & ((1 << bits) - 1)];
    return n;
}

/* KSIGNS_IQ2XS[i]: i with bit 7 set so that the number of one bits is even. */
uint8_t orc_ksigns(int i) { return (uint8_t)(i | ((__builtin_popcount((unsigned)i) & 1) << 7)); }

/* apply_signs (dequant.rs:477-488): out[j] = db * grid[j] * (bit sign_off + j of signs ? -1 : 1) */
static void apply_signs(float *out, const int8_t *grid, uint8_t signs, int sign_off, int n, float db) {
    for (int j = 0; j < n; j++) out[j] = db * (float)grid[j] * ((signs >> (sign_off + j)) & 1 ? -1.0f : 1.0f);
}

#define IQ1S_DELTA 0.125f /* dequant.rs:405 */

static int iquant_block(int dtype, const uint8_t *blk, float *out) {
    int8_t g[8], g2[8];
    switch (dtype) {
    case ORC_IQ2_XXS: { /* :565-596 */
        float d = orc_f16_to_f32(rd_u16(blk));
        const uint8_t *qs = blk + 2;
        for (int ib32 = 0; ib32 < 8; ib32++) {
            uint32_t aux0 = rd_u32(qs + 8 * ib32), aux1 = rd_u32(qs + 8 * ib32 + 4);
            float db = d * (0.5f + (float)(aux1 >> 28)) * 0.25f;
            for (int l = 0; l < 4; l++) {
                orc_grid_entry(GRID_IQ2XXS, (aux0 >> (8 * l)) & 0xFF, g);
                apply_signs(out, g, orc_ksigns((aux1 >> (7 * l)) & 127), 0, 8, db);
                out += 8;
            }
        }
        return 0;
    }
    case ORC_IQ2_XS: { /* :605-636 */
        float d = orc_f16_to_f32(rd_u16(blk));
        const uint8_t *qs = blk + 2, *scales = blk + 66;
        for (int ib32 = 0; ib32 < 8; ib32++) {
            float db0 = d * (0.5f + (float)(scales[ib32] & 0xF)) * 0.25f;
            float db1 = d * (0.5f + (float)(scales[ib32] >> 4)) * 0.25f;
            for (int l = 0; l < 4; l++) {
                unsigned q = rd_u16(qs + 2 * (4 * ib32 + l));
                orc_grid_entry(GRID_IQ2XS, q & 511, g);
                apply_signs(out, g, orc_ksigns(q >> 9), 0, 8, l < 2 ? db0 : db1);
                out += 8;
            }
        }
        return 0;
    }
    case ORC_IQ2_S: { /* :642-676 */
        float d = orc_f16_to_f32(rd_u16(blk));
        const uint8_t *qs = blk + 2, *qh = blk + 66, *scales = blk + 74;
        for (int ib32 = 0; ib32 < 8; ib32++) {
            float db0 = d * (0.5f + (float)(scales[ib32] & 0xF)) * 0.25f;
            float db1 = d * (0.5f + (float)(scales[ib32] >> 4)) * 0.25f;
            for (int l = 0; l < 4; l++) {
                int idx = qs[4 * ib32 + l] | (((unsigned)qh[ib32] << (8 - 2 * l)) & 0x300);
                orc_grid_entry(GRID_IQ2S, idx, g);
                apply_signs(out, g, qs[32 + 4 * ib32 + l], 0, 8, l < 2 ? db0 : db1);
                out += 8;
            }
        }
        return 0;
    }
    case ORC_IQ3_XXS: { /* :685-714 */
        float d = orc_f16_to_f32(rd_u16(blk));
        const uint8_t *qs = blk + 2, *sas = blk + 66;
        for (int ib32 = 0; ib32 < 8; ib32++) {
            uint32_t aux = rd_u32(sas + 4 * ib32);
            float db = d * (0.5f + (float)(aux >> 28)) * 0.5f;
            for (int l = 0; l < 4; l++) {
                uint8_t signs = orc_ksigns((aux >> (7 * l)) & 127);
                orc_grid_entry(GRID_IQ3XXS, qs[2 * l], g);
                orc_grid_entry(GRID_IQ3XXS, qs[2 * l + 1], g2);
                apply_signs(out, g, signs, 0, 4, db);
                apply_signs(out + 4, g2, signs, 4, 4, db);
                out += 8;
            }
            qs += 8;
        }
        return 0;
    }
    case ORC_IQ3_S: { /* :724-781: the reference walks pairs of sub-blocks; sub-block ib takes nibble ib % 2 of scales[ib / 2] */
        float d = orc_f16_to_f32(rd_u16(blk));
        const uint8_t *qs = blk + 2, *qh = blk + 66, *signs = blk + 74, *scales = blk + 106;
        for (int ib32 = 0; ib32 < 8; ib32++) {
            int nib = ib32 % 2 ? scales[ib32 / 2] >> 4 : scales[ib32 / 2] & 0xF;
            float db = d * (1.0f + 2.0f * (float)nib);
            for (int l = 0; l < 4; l++) {
                int i1 = qs[2 * l] | (((unsigned)qh[ib32] << (8 - 2 * l)) & 256);
                int i2 = qs[2 * l + 1] | (((unsigned)qh[ib32] << (7 - 2 * l)) & 256);
                orc_grid_entry(GRID_IQ3S, i1, g);
                orc_grid_entry(GRID_IQ3S, i2, g2);
                apply_signs(out, g, signs[l], 0, 4, db);
                apply_signs(out + 4, g2, signs[l], 4, 4, db);
                out += 8;
            }
            qs += 8;
            signs += 4;
        }
        return 0;
    }
    case ORC_IQ1_S: { /* :789-824 */
        float d = orc_f16_to_f32(rd_u16(blk));
        const uint8_t *qs = blk + 2, *qh_raw = blk + 34;
        for (int ib = 0; ib < 8; ib++) {
            unsigned qh = rd_u16(qh_raw + 2 * ib);
            float dl = d * (2.0f * (float)((qh >> 12) & 7) + 1.0f);
            float delta = qh & 0x8000 ? -IQ1S_DELTA : IQ1S_DELTA;
            for (int l = 0; l < 4; l++) {
                orc_grid_entry(GRID_IQ1S, qs[l] | (((qh >> (3 * l)) & 7) << 8), g);
                for (int j = 0; j < 8; j++) out[j] = dl * ((float)g[j] + delta);
                out += 8;
            }
            qs += 4;
        }
        return 0;
    }
    case ORC_IQ1_M: { /* :838-916 */
        const uint8_t *qs = blk, *qh = blk + 32;
        unsigned sc[4];
        for (int i = 0; i < 4; i++) sc[i] = rd_u16(blk + 48 + 2 * i);
        uint16_t d_bits = (uint16_t)((sc[0] >> 12) | ((sc[1] >> 8) & 0x00F0) | ((sc[2] >> 4) & 0x0F00) | (sc[3] & 0xF000));
        float d = orc_f16_to_f32(d_bits);
        for (int ib = 0; ib < 8; ib++) {
            float dl1 = d * (2.0f * (float)((sc[ib / 2] >> (6 * (ib % 2))) & 7) + 1.0f);
            float dl2 = d * (2.0f * (float)((sc[ib / 2] >> (6 * (ib % 2) + 3)) & 7) + 1.0f);
            int idx[4] = {qs[0] | (((unsigned)qh[0] << 8) & 0x700), qs[1] | (((unsigned)qh[0] << 4) & 0x700),
                          qs[2] | (((unsigned)qh[1] << 8) & 0x700), qs[3] | (((unsigned)qh[1] << 4) & 0x700)};
            float delta[4] = {qh[0] & 0x08 ? -IQ1S_DELTA : IQ1S_DELTA, qh[0] & 0x80 ? -IQ1S_DELTA : IQ1S_DELTA,
                              qh[1] & 0x08 ? -IQ1S_DELTA : IQ1S_DELTA, qh[1] & 0x80 ? -IQ1S_DELTA : IQ1S_DELTA};
            for (int l = 0; l < 4; l++) {
                orc_grid_entry(GRID_IQ1S, idx[l], g);
                for (int j = 0; j < 8; j++) out[j] = (l < 2 ? dl1 : dl2) * ((float)g[j] + delta[l]);
                out += 8;
            }
            qs += 4;
            qh += 2;
        }
        return 0;
    }
    default: return -1;
    }
}

/* dequant.rs:336-363: Q4_K's layout with 32 bytes of fifth bits between the scales and the
 * nibbles: bit 2j of qh[l] belongs to the low-nibble element, bit 2j+1 to the high-nibble one. */
static void factor_q5k(const uint8_t *blk, factored_block *f) {
    f->dd[0] = rd_u16(blk);
    f->dd[1] = rd_u16(blk + 2);
    const uint8_t *scales = blk + 4, *qh = blk + 16, *qs = blk + 48;
    for (int j = 0; j < 4; j++) {
        uint32_t sc1, m1, sc2, m2;
        orc_k4(2 * j, scales, &sc1, &m1);
        orc_k4(2 * j + 1, scales, &sc2, &m2);
        for (int q = 0; q < 4; q++) {
            f->scm[2 * (4 * j + q)] = (int16_t)(q < 2 ? sc1 : sc2);
            f->scm[2 * (4 * j + q) + 1] = (int16_t)(-(int16_t)(q < 2 ? m1 : m2));
        }
        for (int l = 0; l < 32; l++) {
            uint8_t v = qs[j * 32 + l];
            f->codes[j * 64 + l] = (uint8_t)((v & 0xF) + (((qh[l] >> (2 * j)) & 1) ? 16 : 0));
            f->codes[j * 64 + 32 + l] = (uint8_t)((v >> 4) + (((qh[l] >> (2 * j + 1)) & 1) ? 16 : 0));
        }
    }
}

int64_t orc_dequant(int dtype, const uint8_t *bytes, size_t nbytes, float *out) {
    int be, bb;
    if (orc_block_geometry(dtype, &be, &bb) != 0) return -1;
    if (nbytes % (size_t)bb != 0) return -1;
    size_t nblk = nbytes / (size_t)bb;
    switch (dtype) {
    case ORC_F32:
        memcpy(out, bytes, nbytes);
        return (int64_t)nblk;
    case ORC_I32: /* crates/infr-cpu/src/lib.rs:516-519: widened by value */
        for (size_t i = 0; i < nblk; i++) { int32_t v; memcpy(&v, bytes + 4 * i, 4); out[i] = (float)v; }
        return (int64_t)nblk;
    case ORC_U32:
        for (size_t i = 0; i < nblk; i++) { uint32_t v; memcpy(&v, bytes + 4 * i, 4); out[i] = (float)v; }
        return (int64_t)nblk;
    case ORC_F16:
        for (size_t i = 0; i < nblk; i++) out[i] = orc_f16_to_f32(rd_u16(bytes + 2 * i));
        return (int64_t)nblk;
    case ORC_BF16:
        for (size_t i = 0; i < nblk; i++) {
            uint32_t b = (uint32_t)rd_u16(bytes + 2 * i) << 16;
            memcpy(&out[i], &b, 4);
        }
        return (int64_t)nblk;
    default: break;
    }
    factored_block f;
    for (size_t b = 0; b < nblk; b++) {
        const uint8_t *blk = bytes + b * (size_t)bb;
        switch (dtype) {
        case ORC_Q4_0: factor_legacy(blk, 0, 0, &f); break;
        case ORC_Q4_1: factor_legacy(blk, 1, 0, &f); break;
        case ORC_Q5_0: factor_legacy(blk, 0, 1, &f); break;
        case ORC_Q5_1: factor_legacy(blk, 1, 1, &f); break;
        case ORC_Q2K: factor_q2k(blk, &f); break;
        case ORC_Q3K: factor_q3k(blk, &f); break;
        case ORC_Q5K: factor_q5k(blk, &f); break;
        case ORC_Q8_0: factor_q8_0(blk, &f); break;
        case ORC_Q4K: factor_q4k(blk, &f); break;
        case ORC_Q6K: factor_q6k(blk, &f); break;
        default:
            if (codebook_block(dtype, blk, out + b * (size_t)be) != 0 && iquant_block(dtype, blk, out + b * (size_t)be) != 0) return -1;
            continue;
        }
        expand_block(&f, be, out + b * (size_t)be);
    }
    return (int64_t)(nblk * (size_t)be);
}

/* ------------------------------------------------------------------ dot / activations */

/* crates/infr-cpu/src/kernels.rs:6568-6583 (dot_f32_scalar; the AVX2 form is asserted
 * bit-identical to it by the reference's own tests). */
float orc_dot(const float *a, const float *b, size_t n) {
    size_t chunks = n / 8;
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (size_t c = 0; c < chunks; c++) {
        size_t base = c * 8;
        for (int j = 0; j < 8; j++) acc[j] = fmaf(a[base + j], b[base + j], acc[j]);
    }
    float s = 0.0f;
    for (int j = 0; j < 8; j++) s = s + acc[j];
    for (size_t i = chunks * 8; i < n; i++) s = fmaf(a[i], b[i], s);
    return s;
}

/* crates/infr-cpu/src/kernels.rs:6664-6672 */
float orc_act(int act, float g) {
    switch (act) {
    case ORC_ACT_SILU: return g / (1.0f + expf(-g));
    case ORC_ACT_GELU: {
        float g3 = 0.044715f * g * g * g;
        float inner = 0.7978846f * (g + g3);
        float t = 1.0f + tanhf(inner);
        return 0.5f * g * t;
    }
    default: return 1.0f / (1.0f + expf(-g));
    }
}

/* crates/infr-cpu/src/kernels.rs:6678-6683 */
float orc_gated_act(int act, int has_clamp, float clamp, float gate, float up) {
    if (!has_clamp) return orc_act(act, gate) * up;
    float gmin = gate < clamp ? gate : clamp; /* f32::min */
    float uc = up;
    if (uc < -clamp) uc = -clamp;
    if (uc > clamp) uc = clamp;
    return orc_act(act, gmin) * uc;
}

/* ------------------------------------------------------------------ routing */

/* Stable sort of idx by sel DESCENDING (Rust's stable sort_by with
 * sel[b].partial_cmp(sel[a]), crates/infr-cpu/src/lib.rs:3847-3850): insertion sort keeps
 * equal keys in ascending-id order. */
static void stable_sort_desc(int32_t *idx, int n, const float *key) {
    for (int i = 1; i < n; i++) {
        int32_t v = idx[i];
        int j = i - 1;
        while (j >= 0 && key[idx[j]] < key[v]) { idx[j + 1] = idx[j]; j--; }
        idx[j + 1] = v;
    }
}

int orc_route_row(const float *logits, int n_expert, int n_used, int gating, int norm_w,
                  float scale, const float *exp_probs_b, int n_groups, int n_groups_used,
                  const float *hash_ids_row, float *probs_out, int32_t *idx_out, float *w_out) {
    if (n_expert <= 0 || n_used <= 0 || n_used > n_expert) return -1;
    float *probs = (float *)malloc(sizeof(float) * (size_t)n_expert);
    float *sel = (float *)malloc(sizeof(float) * (size_t)n_expert);
    int32_t *idx = (int32_t *)malloc(sizeof(int32_t) * (size_t)n_expert);
    int rc = 0;
    /* lib.rs:3746-3774 */
    if (gating == ORC_GATE_SOFTMAX) {
        float maxl = -INFINITY;
        for (int e = 0; e < n_expert; e++) if (logits[e] > maxl) maxl = logits[e]; /* f32::max */
        for (int e = 0; e < n_expert; e++) probs[e] = expf(logits[e] - maxl);
        float psum = 0.0f;
        for (int e = 0; e < n_expert; e++) psum = psum + probs[e];
        for (int e = 0; e < n_expert; e++) probs[e] = probs[e] / psum;
    } else if (gating == ORC_GATE_SIGMOID) {
        for (int e = 0; e < n_expert; e++) probs[e] = 1.0f / (1.0f + expf(-logits[e]));
    } else {
        for (int e = 0; e < n_expert; e++) {
            float v = logits[e];
            float sp = v > 20.0f ? v : logf(1.0f + expf(v));
            probs[e] = sqrtf(sp);
        }
    }
    for (int e = 0; e < n_expert; e++) if (isnan(probs[e])) rc = -1;
    if (hash_ids_row) { /* lib.rs:3776-3793 */
        for (int k = 0; k < n_used; k++) {
            long e = (long)hash_ids_row[k];
            if (e < 0 || e >= n_expert) { rc = -1; e = 0; }
            idx[k] = (int32_t)e;
        }
    } else {
        /* lib.rs:3797-3806 */
        for (int e = 0; e < n_expert; e++) sel[e] = exp_probs_b ? probs[e] + exp_probs_b[e] : probs[e];
        /* lib.rs:3809-3846 */
        if (n_groups > 1 && n_groups_used > 0) {
            int per = n_expert / n_groups;
            float *gscore = (float *)malloc(sizeof(float) * (size_t)n_groups);
            int32_t *gidx = (int32_t *)malloc(sizeof(int32_t) * (size_t)n_groups);
            for (int g = 0; g < n_groups; g++) {
                float best0 = -INFINITY, best1 = -INFINITY;
                for (int i = g * per; i < (g + 1) * per; i++) {
                    float s = sel[i];
                    if (s > best0) { best1 = best0; best0 = s; }
                    else if (s > best1) { best1 = s; }
                }
                gscore[g] = best0 + best1;
                gidx[g] = g;
            }
            stable_sort_desc(gidx, n_groups, gscore);
            int ngu = n_groups_used < n_groups ? n_groups_used : n_groups;
            for (int g = 0; g < n_groups; g++) {
                int chosen = 0;
                for (int k = 0; k < ngu; k++) if (gidx[k] == g) chosen = 1;
                if (!chosen) for (int i = g * per; i < (g + 1) * per; i++) sel[i] = -INFINITY;
            }
            free(gscore);
            free(gidx);
        }
        for (int e = 0; e < n_expert; e++) idx[e] = e;
        for (int e = 0; e < n_expert; e++) if (isnan(sel[e])) rc = -1;
        stable_sort_desc(idx, n_expert, sel);
    }
    /* lib.rs:3856-3861 */
    if (norm_w) {
        float wsum = 0.0f;
        for (int k = 0; k < n_used; k++) wsum = wsum + probs[idx[k]];
        if (!(wsum > 1e-20f)) wsum = 1e-20f; /* f32::max(wsum, 1e-20) */
        for (int k = 0; k < n_used; k++) {
            float q = probs[idx[k]] / wsum;
            w_out[k] = q * scale;
        }
    } else {
        for (int k = 0; k < n_used; k++) w_out[k] = probs[idx[k]] * scale;
    }
    for (int k = 0; k < n_used; k++) idx_out[k] = idx[k];
    if (probs_out) memcpy(probs_out, probs, sizeof(float) * (size_t)n_expert);
    free(probs);
    free(sel);
    free(idx);
    return rc;
}

/* ------------------------------------------------------------------ expert GEMM (Raw arm) */

/* f16 / bf16 rows dot in the same 8-lane order after an exact widening
 * (crates/infr-cpu/src/kernels.rs dot_f16/dot_bf16, tail at :6540-6552). */
static float dot_widened(const uint8_t *row, int dtype, const float *x, size_t n, float *tmp) {
    orc_dequant(dtype, row, n * 2, tmp);
    return orc_dot(tmp, x, n);
}

/* expert_gemm_range, ExpertActs::Raw arm (crates/infr-cpu/src/moe.rs:142-173): output rows
 * [o0,o1) of one bank against `count` activation rows, o-major result. */
static int gemm_range_raw(const uint8_t *wbytes, size_t wlen, int dt, int in_f, int out_f,
                          const float *xin, int count, int o0, int o1, float *out_t, float *wf) {
    size_t bpr = wlen / (size_t)out_f;
    for (int o = o0; o < o1; o++) {
        const uint8_t *row = wbytes + (size_t)o * bpr;
        float *col = out_t + (size_t)(o - o0) * (size_t)count;
        if (dt == ORC_F32) {
            for (int r = 0; r < count; r++)
                col[r] = orc_dot((const float *)(const void *)row, xin + (size_t)r * in_f, (size_t)in_f);
        } else if (dt == ORC_F16 || dt == ORC_BF16) {
            for (int r = 0; r < count; r++)
                col[r] = dot_widened(row, dt, xin + (size_t)r * in_f, (size_t)in_f, wf);
        } else {
            if (orc_dequant(dt, row, bpr, wf) != in_f) return -1;
            for (int r = 0; r < count; r++) col[r] = orc_dot(wf, xin + (size_t)r * in_f, (size_t)in_f);
        }
    }
    return 0;
}

/* ------------------------------------------------------------------ production int8 path (timed baseline only) */

/* crates/infr-cpu/src/quant.rs:27-63 */
void orc_quantize_q8(const float *x, int n, int8_t *qs, float *d, int32_t *bsums) {
    int nb = n / 256;
    for (int b = 0; b < nb; b++) {
        const float *blk = x + (size_t)b * 256;
        float amax = 0.0f;
        for (int i = 0; i < 256; i++) { float v = fabsf(blk[i]); if (v > amax) amax = v; }
        float dd = amax / 127.0f;
        float id = dd > 0.0f ? 1.0f / dd : 0.0f;
        d[b] = dd;
        for (int i = 0; i < 256; i++) {
            float r = roundf(blk[i] * id);   /* f32::round: half away from zero */
            if (r < -127.0f) r = -127.0f;
            if (r > 127.0f) r = 127.0f;
            qs[(size_t)b * 256 + i] = (int8_t)r;
        }
        for (int s8 = 0; s8 < 8; s8++) {
            int32_t acc = 0;
            for (int i = 0; i < 32; i++) acc += qs[(size_t)b * 256 + s8 * 32 + i];
            bsums[b * 8 + s8] = acc;
        }
    }
}

/* kernels.rs:151-184 */
static float vec_dot_q4k_q8(const uint8_t *row, const int8_t *qs8, const float *d8, const int32_t *bsums, int in_f) {
    float sumf = 0.0f;
    for (int b = 0; b < in_f / 256; b++) {
        const uint8_t *blk = row + (size_t)b * 144;
        float d = orc_f16_to_f32(rd_u16(blk)), dmin = orc_f16_to_f32(rd_u16(blk + 2));
        const uint8_t *scales = blk + 4, *qs = blk + 16;
        const int8_t *q8b = qs8 + (size_t)b * 256;
        int32_t sd = 0, sm = 0;
        for (int s8 = 0; s8 < 8; s8++) {
            uint32_t sc, m;
            orc_k4(s8, scales, &sc, &m);
            const uint8_t *qbyte = qs + (s8 / 2) * 32;
            int32_t iprod = 0;
            for (int l = 0; l < 32; l++) {
                int q4 = (s8 & 1) ? (qbyte[l] >> 4) : (qbyte[l] & 0xF);
                iprod += q4 * (int32_t)q8b[s8 * 32 + l];
            }
            sd += (int32_t)sc * iprod;
            sm += (int32_t)m * bsums[b * 8 + s8];
        }
        float t1 = d * (float)sd, t2 = dmin * (float)sm;
        float t = t1 - t2;
        sumf = sumf + d8[b] * t;
    }
    return sumf;
}

/* kernels.rs:487-526 */
static float vec_dot_q6k_q8(const uint8_t *row, const int8_t *qs8, const float *d8, int in_f) {
    float sumf = 0.0f;
    for (int b = 0; b < in_f / 256; b++) {
        const uint8_t *blk = row + (size_t)b * 210;
        const uint8_t *ql = blk, *qh = blk + 128;
        const int8_t *scales = (const int8_t *)(blk + 192);
        float d = orc_f16_to_f32(rd_u16(blk + 208));
        const int8_t *q8b = qs8 + (size_t)b * 256;
        int32_t sumi[16] = {0}, bsum[16] = {0};
        for (int half = 0; half < 2; half++) {
            int qlo = half * 64, qho = half * 32, sco = half * 8, base = half * 128;
            for (int l = 0; l < 32; l++) {
                int is = l / 16;
                int q[4];
                q[0] = (ql[qlo + l] & 0xF) | ((qh[qho + l] & 3) << 4);
                q[1] = (ql[qlo + l + 32] & 0xF) | (((qh[qho + l] >> 2) & 3) << 4);
                q[2] = (ql[qlo + l] >> 4) | (((qh[qho + l] >> 4) & 3) << 4);
                q[3] = (ql[qlo + l + 32] >> 4) | (((qh[qho + l] >> 6) & 3) << 4);
                for (int c = 0; c < 4; c++) {
                    int sub = sco + is + 2 * c;
                    int32_t v = q8b[base + l + 32 * c];
                    sumi[sub] += q[c] * v;
                    bsum[sub] += v;
                }
            }
        }
        int32_t isum = 0;
        for (int sub = 0; sub < 16; sub++) isum += (int32_t)scales[sub] * (sumi[sub] - 32 * bsum[sub]);
        float dd = d * d8[b];
        sumf = sumf + dd * (float)isum;
    }
    return sumf;
}

/* kernels.rs:1170-1187 */
static float vec_dot_q8_0_q8(const uint8_t *row, const int8_t *qs8, const float *d8, int in_f) {
    float sumf = 0.0f;
    for (int b = 0; b < in_f / 256; b++) {
        for (int s8 = 0; s8 < 8; s8++) {
            const uint8_t *blk = row + (size_t)(b * 8 + s8) * 34;
            float dw = orc_f16_to_f32(rd_u16(blk));
            const int8_t *qw = (const int8_t *)(blk + 2);
            const int8_t *qx = qs8 + (size_t)b * 256 + s8 * 32;
            int32_t iprod = 0;
            for (int i = 0; i < 32; i++) iprod += (int32_t)qw[i] * (int32_t)qx[i];
            float dd = d8[b] * dw;
            sumf = sumf + dd * (float)iprod;
        }
    }
    return sumf;
}

float orc_vec_dot_q8(int dtype, const uint8_t *row, const int8_t *qs, const float *d, const int32_t *bsums, int in_f) {
    switch (dtype) {
    case ORC_Q4K: return vec_dot_q4k_q8(row, qs, d, bsums, in_f);
    case ORC_Q6K: return vec_dot_q6k_q8(row, qs, d, in_f);
    case ORC_Q8_0: return vec_dot_q8_0_q8(row, qs, d, in_f);
    default: return 0.0f / 0.0f;
    }
}

/* expert_acts_kind == Super (crates/infr-cpu/src/moe.rs:42-53; Q5_K has no restatement here) */
static int acts_super(int production, int rows, int dt, int in_f) {
    return production && rows >= 2 && (dt == ORC_Q4K || dt == ORC_Q6K || dt == ORC_Q8_0) && in_f % 256 == 0;
}

/* `rows` activation rows quantised once for a stage (lib.rs:4009-4060: each row a single time) */
typedef struct { int8_t *qs; float *d; int32_t *bsums; int in_f; } q8_rows;

static q8_rows quantize_rows(const float *x, int rows, int in_f, int nthreads) {
    q8_rows q;
    int nb = in_f / 256;
    q.in_f = in_f;
    q.qs = (int8_t *)malloc((size_t)rows * in_f + 4);
    q.d = (float *)malloc(sizeof(float) * (size_t)rows * nb + 4);
    q.bsums = (int32_t *)malloc(sizeof(int32_t) * (size_t)rows * nb * 8 + 4);
#pragma omp parallel for schedule(static) num_threads(nthreads)
    for (int r = 0; r < rows; r++)
        orc_quantize_q8(x + (size_t)r * in_f, in_f, q.qs + (size_t)r * in_f, q.d + (size_t)r * nb, q.bsums + (size_t)r * nb * 8);
    return q;
}
static void free_rows(q8_rows *q) { free(q->qs); free(q->d); free(q->bsums); }

/* expert_gemm_range, ExpertActs::Super arm (moe.rs:80-115), per-row form: rows [o0,o1) x `count` activations */
static void gemm_range_q8(const uint8_t *wbytes, size_t wlen, int dt, int out_f, const q8_rows *q, int first, int count,
                          int o0, int o1, float *out_t) {
    size_t bpr = wlen / (size_t)out_f;
    int nb = q->in_f / 256;
    for (int o = o0; o < o1; o++) {
        const uint8_t *row = wbytes + (size_t)o * bpr;
        float *col = out_t + (size_t)(o - o0) * (size_t)count;
        for (int r = 0; r < count; r++) {
            size_t a = (size_t)(first + r);
            col[r] = orc_vec_dot_q8(dt, row, q->qs + a * q->in_f, q->d + a * nb, q->bsums + a * nb * 8, q->in_f);
        }
    }
}

int orc_hw_threads(void) {
#ifdef _OPENMP
    return omp_get_num_procs();
#else
    return 1;
#endif
}

static int pick_threads(int n) {
    int hw = orc_hw_threads();
    return (n <= 0 || n > hw) ? hw : n;
}

/* ------------------------------------------------------------------ Op::MoeFfn */

typedef struct { int bucket, o0, o1; } gemm_task;

int orc_moe_ffn(const orc_moe_ffn_args *a) {
    const int ne = a->ne, n_expert = a->n_expert, n_used = a->n_used, nffx = a->n_ff_exp;
    const int rows = a->rows;
    if (ne <= 0 || n_expert <= 0 || n_used <= 0 || nffx <= 0 || rows < 0) return -1;
    if (n_used > n_expert) return -1;
    /* lib.rs:3613-3629 */
    if (a->has_swiglu_clamp && (a->act == ORC_ACT_SIGMOID || a->weight_before)) return -2;
    if (a->expert_ids && (a->exp_probs_b || a->n_expert_groups > 1)) return -2;
    const int nthreads = pick_threads(a->n_threads);
    (void)nthreads;
    const size_t gst = a->gate_bytes / (size_t)n_expert;
    const size_t ust = a->fused_gate_up ? 0 : a->up_bytes / (size_t)n_expert;
    const size_t dstr = a->down_bytes / (size_t)n_expert;
    const int maxdim = ne > nffx ? ne : nffx;
    int rc = 0;

    /* ---- router logits (lib.rs:3684-3716): 8-expert chunks, o-major then transposed */
    float *logits = (float *)malloc(sizeof(float) * (size_t)rows * (size_t)n_expert);
    {
        float *lt = (float *)malloc(sizeof(float) * (size_t)rows * (size_t)n_expert);
        int nchunks = (n_expert + 7) / 8;
#pragma omp parallel for schedule(dynamic, 1) num_threads(nthreads)
        for (int c = 0; c < nchunks; c++) {
            float *wf = (float *)malloc(sizeof(float) * (size_t)maxdim);
            int o0 = c * 8, o1 = o0 + 8 < n_expert ? o0 + 8 : n_expert;
            if (gemm_range_raw(a->router, a->router_bytes, a->router_dtype, ne, n_expert, a->router_x,
                               rows, o0, o1, lt + (size_t)o0 * rows, wf) != 0) {
#pragma omp atomic write
                rc = -3;
            }
            free(wf);
        }
        for (int r = 0; r < rows; r++)
            for (int o = 0; o < n_expert; o++) logits[(size_t)r * n_expert + o] = lt[(size_t)o * rows + r];
        free(lt);
    }
    if (rc) { free(logits); return rc; }
    if (a->logits_out) memcpy(a->logits_out, logits, sizeof(float) * (size_t)rows * n_expert);

    /* ---- routing per row (lib.rs:3741-3863) */
    int32_t *ridx = (int32_t *)malloc(sizeof(int32_t) * (size_t)rows * n_used + 4);
    float *rw = (float *)malloc(sizeof(float) * (size_t)rows * n_used + 4);
    for (int r = 0; r < rows; r++) {
        int e = orc_route_row(logits + (size_t)r * n_expert, n_expert, n_used, a->gating, a->norm_w,
                              a->scale, a->exp_probs_b, a->n_expert_groups, a->n_expert_groups_used,
                              a->expert_ids ? a->expert_ids + (size_t)r * n_used : NULL,
                              a->probs_out ? a->probs_out + (size_t)r * n_expert : NULL,
                              ridx + (size_t)r * n_used, rw + (size_t)r * n_used);
        if (e) rc = -4;
    }
    if (rc) { free(logits); free(ridx); free(rw); return rc; }
    if (a->idx_out) memcpy(a->idx_out, ridx, sizeof(int32_t) * (size_t)rows * n_used);
    if (a->w_out) memcpy(a->w_out, rw, sizeof(float) * (size_t)rows * n_used);

    /* ---- bucketing (lib.rs:3874-3908): experts ascending, rows ascending inside a bucket */
    const int n_pairs = rows * n_used;
    int32_t *b_expert = (int32_t *)malloc(sizeof(int32_t) * (size_t)n_expert);
    int32_t *b_p0 = (int32_t *)malloc(sizeof(int32_t) * (size_t)n_expert);
    int32_t *b_count = (int32_t *)malloc(sizeof(int32_t) * (size_t)n_expert);
    int32_t *pair_row = (int32_t *)malloc(sizeof(int32_t) * (size_t)n_pairs + 4);
    int32_t *pair_bucket = (int32_t *)malloc(sizeof(int32_t) * (size_t)n_pairs + 4);
    int32_t *pair_local = (int32_t *)malloc(sizeof(int32_t) * (size_t)n_pairs + 4);
    float *pair_w = (float *)malloc(sizeof(float) * (size_t)n_pairs + 4);
    int32_t *slot_pair = (int32_t *)malloc(sizeof(int32_t) * (size_t)n_pairs + 4);
    int n_buckets = 0;
    {
        int np = 0;
        for (int e = 0; e < n_expert; e++) {
            int p0 = np;
            for (int r = 0; r < rows; r++)
                for (int rank = 0; rank < n_used; rank++)
                    if (ridx[(size_t)r * n_used + rank] == e) {
                        slot_pair[(size_t)r * n_used + rank] = np;
                        pair_row[np] = r;
                        pair_bucket[np] = n_buckets;
                        pair_local[np] = np - p0;
                        pair_w[np] = rw[(size_t)r * n_used + rank];
                        np++;
                    }
            if (np > p0) {
                b_expert[n_buckets] = e;
                b_p0[n_buckets] = p0;
                b_count[n_buckets] = np - p0;
                n_buckets++;
            }
        }
    }
    if (a->n_buckets_out) *a->n_buckets_out = n_buckets;
    if (a->bucket_expert_out) memcpy(a->bucket_expert_out, b_expert, sizeof(int32_t) * (size_t)n_buckets);
    if (a->bucket_p0_out) memcpy(a->bucket_p0_out, b_p0, sizeof(int32_t) * (size_t)n_buckets);
    if (a->bucket_count_out) memcpy(a->bucket_count_out, b_count, sizeof(int32_t) * (size_t)n_buckets);
    if (a->pair_row_out) memcpy(a->pair_row_out, pair_row, sizeof(int32_t) * (size_t)n_pairs);
    if (a->slot_pair_out) memcpy(a->slot_pair_out, slot_pair, sizeof(int32_t) * (size_t)n_pairs);

    const int out_gu = a->fused_gate_up ? 2 * nffx : nffx;
    size_t *gu_off = (size_t *)malloc(sizeof(size_t) * (size_t)(n_buckets + 1));
    size_t *d_off = (size_t *)malloc(sizeof(size_t) * (size_t)(n_buckets + 1));
    gu_off[0] = d_off[0] = 0;
    for (int b = 0; b < n_buckets; b++) {
        gu_off[b + 1] = gu_off[b] + (size_t)out_gu * (size_t)b_count[b];
        d_off[b + 1] = d_off[b] + (size_t)ne * (size_t)b_count[b];
    }

    /* ---- stage A (lib.rs:4030-4037): one f32 activation row per pair */
    float *xin_pairs = (float *)malloc(sizeof(float) * (size_t)n_pairs * ne + 4);
    for (int p = 0; p < n_pairs; p++)
        memcpy(xin_pairs + (size_t)p * ne, a->x + (size_t)pair_row[p] * ne, sizeof(float) * (size_t)ne);

    /* flat (bucket, 64-row chunk) task list (lib.rs:3992-4003) */
    int ntask_gu = 0, ntask_d = 0;
    gemm_task *tasks_gu = (gemm_task *)malloc(sizeof(gemm_task) * (size_t)(n_buckets * ((out_gu + 63) / 64) + 1));
    gemm_task *tasks_d = (gemm_task *)malloc(sizeof(gemm_task) * (size_t)(n_buckets * ((ne + 63) / 64) + 1));
    for (int b = 0; b < n_buckets; b++) {
        for (int o = 0; o < out_gu; o += 64) {
            gemm_task t = {b, o, o + 64 < out_gu ? o + 64 : out_gu};
            tasks_gu[ntask_gu++] = t;
        }
        for (int o = 0; o < ne; o += 64) {
            gemm_task t = {b, o, o + 64 < ne ? o + 64 : ne};
            tasks_d[ntask_d++] = t;
        }
    }

    /* ---- stage B (lib.rs:4087-4141) */
    float *gu_all = (float *)malloc(sizeof(float) * gu_off[n_buckets] + 4);
    float *up_all = a->fused_gate_up ? NULL : (float *)malloc(sizeof(float) * gu_off[n_buckets] + 4);
    const int g_q8 = acts_super(a->production, rows, a->gate_dtype, ne);
    const int u_q8 = !a->fused_gate_up && acts_super(a->production, rows, a->up_dtype, ne);
    q8_rows xq = {0};
    if (g_q8 || u_q8) xq = quantize_rows(xin_pairs, n_pairs, ne, nthreads);
#pragma omp parallel num_threads(nthreads)
    {
        float *wf = (float *)malloc(sizeof(float) * (size_t)maxdim);
#pragma omp for schedule(dynamic, 1)
        for (int t = 0; t < ntask_gu; t++) {
            int b = tasks_gu[t].bucket, o0 = tasks_gu[t].o0, o1 = tasks_gu[t].o1;
            int e = b_expert[b], count = b_count[b];
            if (g_q8) {
                gemm_range_q8(a->gate + (size_t)e * gst, gst, a->gate_dtype, out_gu, &xq, b_p0[b], count, o0, o1,
                              gu_all + gu_off[b] + (size_t)o0 * count);
                continue;
            }
            if (gemm_range_raw(a->gate + (size_t)e * gst, gst, a->gate_dtype, ne, out_gu,
                               xin_pairs + (size_t)b_p0[b] * ne, count, o0, o1,
                               gu_all + gu_off[b] + (size_t)o0 * count, wf) != 0) {
#pragma omp atomic write
                rc = -5;
            }
        }
        if (!a->fused_gate_up) {
#pragma omp for schedule(dynamic, 1)
            for (int t = 0; t < ntask_gu; t++) {
                int b = tasks_gu[t].bucket, o0 = tasks_gu[t].o0, o1 = tasks_gu[t].o1;
                int e = b_expert[b], count = b_count[b];
                if (u_q8) {
                    gemm_range_q8(a->up + (size_t)e * ust, ust, a->up_dtype, nffx, &xq, b_p0[b], count, o0, o1,
                                  up_all + gu_off[b] + (size_t)o0 * count);
                    continue;
                }
                if (gemm_range_raw(a->up + (size_t)e * ust, ust, a->up_dtype, ne, nffx,
                                   xin_pairs + (size_t)b_p0[b] * ne, count, o0, o1,
                                   up_all + gu_off[b] + (size_t)o0 * count, wf) != 0) {
#pragma omp atomic write
                    rc = -5;
                }
            }
        }
        free(wf);
    }

    /* ---- stage C (lib.rs:4149-4181): gated activation per pair */
    float *dact = (float *)malloc(sizeof(float) * (size_t)n_pairs * nffx + 4);
    for (int p = 0; p < n_pairs && !rc; p++) {
        int b = pair_bucket[p], i = pair_local[p], count = b_count[b];
        float wp = a->weight_before ? pair_w[p] : 1.0f;
        const float *gt = gu_all + gu_off[b];
        const float *ut = a->fused_gate_up ? gt + (size_t)nffx * count : up_all + gu_off[b];
        for (int f = 0; f < nffx; f++) {
            float g = wp * gt[(size_t)f * count + i];
            float u = wp * ut[(size_t)f * count + i];
            dact[(size_t)p * nffx + f] = orc_gated_act(a->act, a->has_swiglu_clamp, a->swiglu_clamp, g, u);
        }
    }

    /* ---- stage D (lib.rs:4218-4265) */
    if (g_q8 || u_q8) free_rows(&xq);
    float *down_all = (float *)malloc(sizeof(float) * d_off[n_buckets] + 4);
    const int d_q8 = acts_super(a->production, rows, a->down_dtype, nffx);
    q8_rows hq = {0};
    if (d_q8 && !rc) hq = quantize_rows(dact, n_pairs, nffx, nthreads);
#pragma omp parallel num_threads(nthreads)
    {
        float *wf = (float *)malloc(sizeof(float) * (size_t)maxdim);
#pragma omp for schedule(dynamic, 1)
        for (int t = 0; t < ntask_d; t++) {
            int b = tasks_d[t].bucket, o0 = tasks_d[t].o0, o1 = tasks_d[t].o1;
            int e = b_expert[b], count = b_count[b];
            if (d_q8 && rc == 0) {
                gemm_range_q8(a->down + (size_t)e * dstr, dstr, a->down_dtype, ne, &hq, b_p0[b], count, o0, o1,
                              down_all + d_off[b] + (size_t)o0 * count);
                continue;
            }
            if (rc == 0 &&
                gemm_range_raw(a->down + (size_t)e * dstr, dstr, a->down_dtype, nffx, ne,
                               dact + (size_t)b_p0[b] * nffx, count, o0, o1,
                               down_all + d_off[b] + (size_t)o0 * count, wf) != 0) {
#pragma omp atomic write
                rc = -6;
            }
        }
        free(wf);
    }
    if (d_q8 && hq.qs) free_rows(&hq);
    float *y_pairs = (float *)malloc(sizeof(float) * (size_t)n_pairs * ne + 4);
    for (int p = 0; p < n_pairs && !rc; p++) {
        int b = pair_bucket[p], i = pair_local[p], count = b_count[b], e = b_expert[b];
        const float *dt = down_all + d_off[b];
        if (a->down_scale) {
            float s_e = a->down_scale[e];
            for (int d = 0; d < ne; d++) y_pairs[(size_t)p * ne + d] = dt[(size_t)d * count + i] * s_e;
        } else {
            for (int d = 0; d < ne; d++) y_pairs[(size_t)p * ne + d] = dt[(size_t)d * count + i];
        }
    }

    /* ---- stage E (lib.rs:4290-4302): rank-order accumulate, separate multiply and add */
    for (int r = 0; r < rows && !rc; r++) {
        float *orow = a->dst + (size_t)r * ne;
        for (int i = 0; i < ne; i++) orow[i] = 0.0f;
        for (int rank = 0; rank < n_used; rank++) {
            int p = slot_pair[(size_t)r * n_used + rank];
            float w_e = a->weight_before ? 1.0f : rw[(size_t)r * n_used + rank];
            const float *y = y_pairs + (size_t)p * ne;
            for (int i = 0; i < ne; i++) {
                float t = w_e * y[i];
                orow[i] = orow[i] + t;
            }
        }
    }

    free(logits); free(ridx); free(rw);
    free(b_expert); free(b_p0); free(b_count);
    free(pair_row); free(pair_bucket); free(pair_local); free(pair_w); free(slot_pair);
    free(gu_off); free(d_off); free(xin_pairs); free(tasks_gu); free(tasks_d);
    free(gu_all); free(up_all); free(dact); free(down_all); free(y_pairs);
    return rc;
}

/* ------------------------------------------------------------------ neighbours of MoeFfn */

/* crates/infr-cpu/src/lib.rs:1275-1328 (reference branch :1312-1327; float dtypes take the
 * same exact dot on their production arm). */
int orc_linear(const float *x, const uint8_t *w, int w_dtype, size_t w_bytes, int64_t w_numel,
               int m, int in_f, int out_f, int64_t w_off, int n_threads, float *dst) {
    if (in_f <= 0 || out_f <= 0 || m < 0 || w_numel % in_f != 0 || w_off % in_f != 0) return -1;
    int64_t total_rows = w_numel / in_f;
    size_t bpr = w_bytes / (size_t)total_rows;
    int64_t row0 = w_off / in_f;
    if (row0 + out_f > total_rows) return -1;
    const uint8_t *wbytes = w + (size_t)row0 * bpr;
    int rc = 0;
    const int nthreads = pick_threads(n_threads);
    (void)nthreads;
    float *out_t = (float *)malloc(sizeof(float) * (size_t)out_f * (size_t)m + 4);
#pragma omp parallel num_threads(nthreads)
    {
        float *wf = (float *)malloc(sizeof(float) * (size_t)in_f);
#pragma omp for schedule(dynamic, 8)
        for (int o = 0; o < out_f; o++) {
            if (gemm_range_raw(wbytes, bpr * (size_t)out_f, w_dtype, in_f, out_f, x, m, o, o + 1,
                               out_t + (size_t)o * m, wf) != 0) {
#pragma omp atomic write
                rc = -3;
            }
        }
        free(wf);
    }
    for (int r = 0; r < m; r++)
        for (int o = 0; o < out_f; o++) dst[(size_t)r * out_f + o] = out_t[(size_t)o * m + r];
    free(out_t);
    return rc;
}

void orc_gated_act_rows(const float *gate, const float *up, int rows, int nff, int act,
                        int has_clamp, float clamp, float *dst) {
    for (int r = 0; r < rows; r++)
        for (int i = 0; i < nff; i++)
            dst[(size_t)r * nff + i] =
                orc_gated_act(act, has_clamp, clamp, gate[(size_t)r * nff + i], up[(size_t)r * nff + i]);
}

void orc_add(const float *a, const float *b, int64_t n, float *dst) {
    for (int64_t i = 0; i < n; i++) dst[i] = a[i] + b[i];
}

void orc_moe_shared_expert_add(const float *moe, const float *shexp, const float *gate,
                               int rows, int n, float *dst) {
    for (int r = 0; r < rows; r++) {
        float g = 1.0f / (1.0f + expf(-gate[r]));
        for (int c = 0; c < n; c++) {
            float t = g * shexp[(size_t)r * n + c];
            dst[(size_t)r * n + c] = moe[(size_t)r * n + c] + t;
        }
    }
}

/* Op::RmsNorm / Op::RmsNormAdd (crates/infr-cpu/src/lib.rs:1046-1093): per row the squares are
 * summed left to right in f32 (multiply, then add: rustc never contracts), divided by dim,
 * s = 1 / sqrt(ss + eps), and each element is (x * s) * w; the Add form accumulates into dst. */
void orc_rms_norm(const float *x, const float *w, int rows, int dim, float eps, int add, float *dst) {
    for (int r = 0; r < rows; r++) {
        const float *xr = x + (size_t)r * dim;
        float *d = dst + (size_t)r * dim;
        float ss = 0.0f;
        for (int i = 0; i < dim; i++) {
            float sq = xr[i] * xr[i];
            ss = ss + sq;
        }
        ss = ss / (float)dim;
        float s = 1.0f / sqrtf(ss + eps);
        for (int i = 0; i < dim; i++) {
            float t = xr[i] * s;
            t = t * w[i];
            d[i] = add ? d[i] + t : t;
        }
    }
}

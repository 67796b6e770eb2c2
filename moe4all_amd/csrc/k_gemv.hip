// Decode-regime expert kernels: id-indexed dequant-GEMV over the gate/up banks with the
// gated activation fused (h = act(gate.x) * (up.x)), and over the down bank with the
// rank-ordered weighted combine fused into the epilogue.
//
// Layout idea: a wavefront owns whole weight rows.  Every lane owns a FIXED slice of the K
// dimension, so its slice of the activation vector stays in registers for all the rows the
// wavefront streams; only packed weight blocks move from HBM, in 128-bit loads.  A row of
// nblk blocks occupies nblk*LPB consecutive lanes (LPB = lanes per block, a property of the
// format); when that is <= 32 several rows ride in one wavefront side by side.
//
// Numerics: f32 everywhere.  A block's contribution is evaluated in factored form,
//   sum_i (d*sc)*q_i*x_i + (dmin*m)*x_i  =  (d*sc) * (sum q_i x_i) + (dmin*m) * (sum x_i),
// which is exact-product arithmetic for a one-hot x, so a one-hot activation reads back the
// reference's decoded weight bit for bit (crates/infr-gguf/src/dequant.rs:35-51).
#include "device_common.h"
#include "kernels.h"

namespace infr {

__device__ __forceinline__ float ub0(uint32_t v) { return (float)(v & 0xFFu); }
__device__ __forceinline__ float ub1(uint32_t v) { return (float)((v >> 8) & 0xFFu); }
__device__ __forceinline__ float ub2(uint32_t v) { return (float)((v >> 16) & 0xFFu); }
__device__ __forceinline__ float ub3(uint32_t v) { return (float)(v >> 24); }

__device__ __forceinline__ float dot4(uint32_t packed, const float* x, float acc) {
    acc = fmaf(ub0(packed), x[0], acc);
    acc = fmaf(ub1(packed), x[1], acc);
    acc = fmaf(ub2(packed), x[2], acc);
    acc = fmaf(ub3(packed), x[3], acc);
    return acc;
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
// 144 B: [f16 d][f16 dmin][12 B 6-bit scales/mins][128 B nibbles].  8 lanes per block; lane i
// owns nibble bytes [16i, 16i+16): low nibbles are elements j*64+l0+t, high nibbles
// j*64+32+l0+t (j = i/2, l0 = 16*(i&1)), i.e. sub-blocks 2j and 2j+1.
struct Q4KFmt {
    static constexpr int kBlockBytes = 144, kBlockElems = 256, kLPB = 8;
    struct X { float lo[16], hi[16]; float slo, shi; };
    struct Raw { uint4 hdr, qs; };
    static __device__ __forceinline__ void load_x(X& x, const float* xb, int i) {
        const int j = i >> 1, l0 = (i & 1) * 16;
        load16(x.lo, xb + j * 64 + l0);
        load16(x.hi, xb + j * 64 + 32 + l0);
        float a = 0.f, b = 0.f;
#pragma unroll
        for (int t = 0; t < 16; t++) { a += x.lo[t]; b += x.hi[t]; }
        x.slo = a; x.shi = b;
    }
    static __device__ __forceinline__ void zero_x(X& x) {
#pragma unroll
        for (int t = 0; t < 16; t++) { x.lo[t] = 0.f; x.hi[t] = 0.f; }
        x.slo = 0.f; x.shi = 0.f;
    }
    static __device__ __forceinline__ Raw load(const uint8_t* blk, int i) {
        Raw r;
        r.hdr = *reinterpret_cast<const uint4*>(blk);
        r.qs = *reinterpret_cast<const uint4*>(blk + 16 + 16 * i);
        return r;
    }
    static __device__ __forceinline__ float dot(const Raw& r, int i, const X& x) {
        const int j = i >> 1;
        const float d = f16_bits_to_f32(r.hdr.x & 0xFFFFu);
        const float dmin = f16_bits_to_f32(r.hdr.x >> 16);
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
        float alo = 0.f, ahi = 0.f;
        const uint32_t q[4] = {r.qs.x, r.qs.y, r.qs.z, r.qs.w};
#pragma unroll
        for (int k = 0; k < 4; k++) {
            alo = dot4(q[k] & 0x0F0F0F0Fu, x.lo + 4 * k, alo);
            ahi = dot4((q[k] >> 4) & 0x0F0F0F0Fu, x.hi + 4 * k, ahi);
        }
        const float s0 = d * ub0(sc), s1 = d * ub1(sc);
        const float m0 = dmin * ub0(m), m1 = dmin * ub1(m);
        return (s0 * alo - m0 * x.slo) + (s1 * ahi - m1 * x.shi);
    }
};

// ------------------------------------------------------------------------------- Q6_K
// 210 B: [128 B ql][64 B qh][16 x i8 scales][f16 d].  4 lanes per block; lane i owns, in half
// h = i/2 at l0 = 16*(i&1), the bytes ql[h*64+l0 ..+16), ql[h*64+32+l0 ..+16) and
// qh[h*32+l0 ..+16): 64 elements in four 16-element scale groups g = 0..3 at
// h*128 + g*32 + l0 (scale byte h*8 + 2g + (i&1)).  Blocks are only 2-byte aligned.
struct Q6KFmt {
    static constexpr int kBlockBytes = 210, kBlockElems = 256, kLPB = 4;
    struct X { float v[4][16]; float s32[4]; };
    struct Raw { uint4 qla, qlb, qh; uint2 sc; uint32_t d; };
    static __device__ __forceinline__ void load_x(X& x, const float* xb, int i) {
        const int h = i >> 1, l0 = (i & 1) * 16;
#pragma unroll
        for (int g = 0; g < 4; g++) {
            load16(x.v[g], xb + h * 128 + g * 32 + l0);
            float a = 0.f;
#pragma unroll
            for (int t = 0; t < 16; t++) a += x.v[g][t];
            x.s32[g] = 32.0f * a;
        }
    }
    static __device__ __forceinline__ void zero_x(X& x) {
#pragma unroll
        for (int g = 0; g < 4; g++) {
#pragma unroll
            for (int t = 0; t < 16; t++) x.v[g][t] = 0.f;
            x.s32[g] = 0.f;
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
        float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const uint32_t q0 = (a[k] & 0x0F0F0F0Fu) | ((hq[k] << 4) & 0x30303030u);
            const uint32_t q1 = (b[k] & 0x0F0F0F0Fu) | ((hq[k] << 2) & 0x30303030u);
            const uint32_t q2 = ((a[k] >> 4) & 0x0F0F0F0Fu) | (hq[k] & 0x30303030u);
            const uint32_t q3 = ((b[k] >> 4) & 0x0F0F0F0Fu) | ((hq[k] >> 2) & 0x30303030u);
            acc[0] = dot4(q0, x.v[0] + 4 * k, acc[0]);
            acc[1] = dot4(q1, x.v[1] + 4 * k, acc[1]);
            acc[2] = dot4(q2, x.v[2] + 4 * k, acc[2]);
            acc[3] = dot4(q3, x.v[3] + 4 * k, acc[3]);
        }
        const float d = f16_bits_to_f32(r.d);
        const uint32_t sx = (i & 1) ? (r.sc.x >> 8) : r.sc.x;
        const uint32_t sy = (i & 1) ? (r.sc.y >> 8) : r.sc.y;
        const float s0 = (float)(int)(int8_t)(sx & 0xFFu);
        const float s1 = (float)(int)(int8_t)((sx >> 16) & 0xFFu);
        const float s2 = (float)(int)(int8_t)(sy & 0xFFu);
        const float s3 = (float)(int)(int8_t)((sy >> 16) & 0xFFu);
        return ((d * s0) * (acc[0] - x.s32[0]) + (d * s1) * (acc[1] - x.s32[1])) +
               ((d * s2) * (acc[2] - x.s32[2]) + (d * s3) * (acc[3] - x.s32[3]));
    }
};

// ------------------------------------------------------------------------------- Q8_0
// 34 B: [f16 d][32 x i8].  One lane per block.  Signed bytes are biased to unsigned
// (q+128) for the byte->float conversion and the bias leaves through 128 * sum(x).
struct Q80Fmt {
    static constexpr int kBlockBytes = 34, kBlockElems = 32, kLPB = 1;
    struct X { float v[32]; float s128; };
    struct Raw { uint4 a, b; uint32_t d; };
    static __device__ __forceinline__ void load_x(X& x, const float* xb, int) {
        load16(x.v, xb);
        load16(x.v + 16, xb + 16);
        float a = 0.f;
#pragma unroll
        for (int t = 0; t < 32; t++) a += x.v[t];
        x.s128 = 128.0f * a;
    }
    static __device__ __forceinline__ void zero_x(X& x) {
#pragma unroll
        for (int t = 0; t < 32; t++) x.v[t] = 0.f;
        x.s128 = 0.f;
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
        float acc = 0.f;
#pragma unroll
        for (int k = 0; k < 8; k++) acc = dot4(q[k] ^ 0x80808080u, x.v + 4 * k, acc);
        return f16_bits_to_f32(r.d) * (acc - x.s128);
    }
};

// Lane placement of a wavefront over weight rows of nblk blocks.
//   KS == 1: lanes_per_row = nblk*LPB <= 64, rows_per_wave = 64 / lanes_per_row.
//   KS == 2: 64 < lanes_per_row <= 128, one row per wave, two K slices per lane.
template <class F, int KS>
struct Place {
    int lpr, rw_count, rw, pos;          // lanes per row, rows per wave, my row, my lane in row
    int blk[KS], sub[KS];                // my block in the row and lane inside the block
    bool on[KS];
    __device__ __forceinline__ Place(int nblk, int lane) {
        lpr = nblk * F::kLPB;
        if (KS == 1) {
            rw_count = kWave / lpr;
            rw = lane / lpr;
            pos = lane - rw * lpr;
        } else {
            rw_count = 1;
            rw = 0;
            pos = lane;
        }
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            int id = pos + kWave * ks;
            blk[ks] = id / F::kLPB;
            sub[ks] = id - blk[ks] * F::kLPB;
            on[ks] = rw < rw_count && blk[ks] < nblk;
        }
    }
};

template <class F, int KS>
__device__ __forceinline__ void load_x_all(typename F::X (&xs)[KS], const Place<F, KS>& pl, const float* x) {
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
        if (pl.on[ks]) F::load_x(xs[ks], x + (size_t)pl.blk[ks] * F::kBlockElems, pl.sub[ks]);
        else F::zero_x(xs[ks]);
    }
}

template <class F, int KS>
__device__ __forceinline__ void load_row(typename F::Raw (&raw)[KS], const Place<F, KS>& pl, const uint8_t* row,
                                         bool valid) {
#pragma unroll
    for (int ks = 0; ks < KS; ks++)
        if (valid && pl.on[ks]) raw[ks] = F::load(row + (size_t)pl.blk[ks] * F::kBlockBytes, pl.sub[ks]);
}

template <class F, int KS>
__device__ __forceinline__ float dot_row(const typename F::Raw (&raw)[KS], const Place<F, KS>& pl,
                                         const typename F::X (&xs)[KS], bool valid) {
    float s = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ks++)
        if (valid && pl.on[ks]) s += F::dot(raw[ks], pl.sub[ks], xs[ks]);
    return s;
}

template <class F, int KS>
__device__ __forceinline__ float row_sum(float v, const Place<F, KS>& pl) {
    if (KS == 2 || pl.lpr == kWave) return wave_sum(v);
    return segment_sum(v, pl.lpr, pl.pos);
}

// ------------------------------------------------------------------------------- gate/up
// grid.x = tiles of `ft` features, grid.y = token row.  A block's 4 waves share the items
// (slot, f) of its tile round-robin; x is identical for every slot of a token.
template <class F, int KS>
__global__ __launch_bounds__(256) void moe_gate_up_fast(MoeGemvParams p, int ft) {
    const int r = blockIdx.y;
    const int f0 = blockIdx.x * ft;
    const int fcount = min(ft, p.nff - f0);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int nblk = p.ne / F::kBlockElems;
    const size_t row_bytes = (size_t)nblk * F::kBlockBytes;
    const Place<F, KS> pl(nblk, lane);
    typename F::X xs[KS];
    load_x_all<F, KS>(xs, pl, p.x + (size_t)r * p.ne);

    const int nitems = fcount * p.n_used;
    const int32_t* ids = p.ids + (size_t)r * p.n_used;
    const int stride = 4 * pl.rw_count;
    typename F::Raw graw[KS], uraw[KS];
    int it = wave * pl.rw_count + pl.rw;
    auto rows_of = [&](int item, const uint8_t*& grow, const uint8_t*& urow) {
        int slot = item / fcount, f = f0 + (item - slot * fcount);
        int e = ids[slot];
        grow = p.gate + (size_t)e * p.gate_stride + (size_t)f * row_bytes;
        urow = p.up + (size_t)e * p.up_stride + (size_t)f * row_bytes;
    };
    {
        const uint8_t *g = nullptr, *u = nullptr;
        bool v = it < nitems;
        if (v) rows_of(it, g, u);
        load_row<F, KS>(graw, pl, g, v);
        load_row<F, KS>(uraw, pl, u, v);
    }
    for (int base = wave * pl.rw_count; base < nitems; base += stride, it += stride) {
        const bool valid = it < nitems;
        typename F::Raw gn[KS], un[KS];
        {
            const uint8_t *g = nullptr, *u = nullptr;
            bool v = it + stride < nitems;
            if (v) rows_of(it + stride, g, u);
            load_row<F, KS>(gn, pl, g, v);
            load_row<F, KS>(un, pl, u, v);
        }
        float gs = dot_row<F, KS>(graw, pl, xs, valid);
        float us = dot_row<F, KS>(uraw, pl, xs, valid);
        gs = row_sum<F, KS>(gs, pl);
        us = row_sum<F, KS>(us, pl);
        if (valid && pl.pos == 0 && pl.rw < pl.rw_count) {
            int slot = it / fcount, f = f0 + (it - slot * fcount);
            if (p.weight_before) {
                float wp = p.weights[(size_t)r * p.n_used + slot];
                gs = __fmul_rn(wp, gs);
                us = __fmul_rn(wp, us);
            }
            p.h[((size_t)r * p.n_used + slot) * p.nff + f] = gated_act_fn(p.act, p.has_clamp, p.clamp, gs, us);
        }
#pragma unroll
        for (int ks = 0; ks < KS; ks++) { graw[ks] = gn[ks]; uraw[ks] = un[ks]; }
    }
}

// ------------------------------------------------------------------------------- down
// grid.x = tiles of `ot` output rows, grid.y = token row.  Wave w streams the down rows of
// slots w, w+4, ... for the block's output rows (that slot's h stays in registers), the
// per-slot results meet in LDS and are combined in rank order:
//   out += w_rank * y_rank  as a separate multiply and add (crates/infr-cpu/src/lib.rs:4290-4302).
constexpr int kMaxUsedFast = 16;
constexpr int kMaxOt = 32;

template <class F, int KS>
__global__ __launch_bounds__(256) void moe_down_combine_fast(MoeGemvParams p, int ot) {
    __shared__ float ypart[kMaxUsedFast][kMaxOt];
    const int r = blockIdx.y;
    const int o0 = blockIdx.x * ot;
    const int ocount = min(ot, p.ne - o0);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int nblk = p.nff / F::kBlockElems;
    const size_t row_bytes = (size_t)nblk * F::kBlockBytes;
    const Place<F, KS> pl(nblk, lane);
    const int32_t* ids = p.ids + (size_t)r * p.n_used;

    for (int slot = wave; slot < p.n_used; slot += 4) {
        const int e = ids[slot];
        const uint8_t* bank = p.down + (size_t)e * p.down_stride + (size_t)o0 * row_bytes;
        typename F::X xs[KS];
        load_x_all<F, KS>(xs, pl, p.h + ((size_t)r * p.n_used + slot) * p.nff);
        const float ds = p.down_scale ? p.down_scale[e] : 1.0f;
        typename F::Raw raw[KS];
        load_row<F, KS>(raw, pl, bank + (size_t)pl.rw * row_bytes, pl.rw < ocount);
        for (int oo = 0; oo < ocount; oo += pl.rw_count) {
            const int o = oo + pl.rw;
            const bool valid = o < ocount;
            typename F::Raw nx[KS];
            const int on = o + pl.rw_count;
            load_row<F, KS>(nx, pl, bank + (size_t)on * row_bytes, on < ocount);
            float y = dot_row<F, KS>(raw, pl, xs, valid);
            y = row_sum<F, KS>(y, pl);
            if (valid && pl.pos == 0 && pl.rw < pl.rw_count) ypart[slot][o] = p.down_scale ? __fmul_rn(y, ds) : y;
#pragma unroll
            for (int ks = 0; ks < KS; ks++) raw[ks] = nx[ks];
        }
    }
    __syncthreads();
    if ((int)threadIdx.x < ocount) {
        const float* w = p.weights + (size_t)r * p.n_used;
        float acc = 0.0f;
        for (int k = 0; k < p.n_used; k++) {
            float wk = p.weight_before ? 1.0f : w[k];
            acc = __fadd_rn(acc, __fmul_rn(wk, ypart[k][threadIdx.x]));
        }
        p.dst[(size_t)r * p.ne + o0 + threadIdx.x] = acc;
    }
}

// ------------------------------------------------------------------------------- generic
// Any dtype decode_elem understands and any shape: one wave per output, lanes stride over K.
__global__ __launch_bounds__(256) void moe_gate_up_generic(MoeGemvParams p, size_t g_row_bytes, size_t u_row_bytes) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int f = blockIdx.x * 4 + wave;
    const int pair = blockIdx.y;
    if (f >= p.nff) return;
    const int r = pair / p.n_used, slot = pair - r * p.n_used;
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
    (void)slot;
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
        float wk = p.weight_before ? 1.0f : p.weights[(size_t)r * p.n_used + slot];
        acc = __fadd_rn(acc, __fmul_rn(wk, y));
    }
    if (lane == 0) p.dst[(size_t)r * p.ne + o] = acc;
}

// ------------------------------------------------------------------------------- dispatch
static size_t row_bytes_of(int dt, int in_f) {
    int be = 1, bb = 4;
    block_geometry(dt, &be, &bb);
    return (size_t)(in_f / be) * bb;
}

// 0: no fast path; 1 or 2: K slices per lane.
template <class F>
static int fast_ks(int in_f) {
    if (in_f % F::kBlockElems != 0) return 0;
    int lpr = in_f / F::kBlockElems * F::kLPB;
    if (lpr <= 64) return 1;
    if (lpr <= 128) return 2;
    return 0;
}

static int tile_for(int total, int n_cu, int granule, int cap) {
    // about one block per compute unit, a multiple of the rows a wave carries at once
    int t = (total + n_cu - 1) / n_cu;
    t = (t + granule - 1) / granule * granule;
    if (t < granule) t = granule;
    if (t > cap) t = cap / granule * granule;
    if (t < 1) t = 1;
    return t;
}

template <class F>
static bool try_gate_up(hipStream_t s, const MoeGemvParams& p) {
    int ks = fast_ks<F>(p.ne);
    if (!ks) return false;
    int lpr = p.ne / F::kBlockElems * F::kLPB;
    int rw = ks == 1 ? 64 / lpr : 1;
    // items per block = ft * n_used, spread over 4 waves carrying rw rows each
    int ft = tile_for(p.nff, p.n_cu, 1, 1 << 20);
    (void)rw;
    dim3 grid((p.nff + ft - 1) / ft, p.rows), block(256);
    if (ks == 1) hipLaunchKernelGGL((moe_gate_up_fast<F, 1>), grid, block, 0, s, p, ft);
    else hipLaunchKernelGGL((moe_gate_up_fast<F, 2>), grid, block, 0, s, p, ft);
    return true;
}

void launch_moe_gate_up(hipStream_t s, const MoeGemvParams& p) {
    if (p.gate_dt == p.up_dt) {
        bool done = false;
        if (p.gate_dt == INFR_Q4K) done = try_gate_up<Q4KFmt>(s, p);
        else if (p.gate_dt == INFR_Q6K) done = try_gate_up<Q6KFmt>(s, p);
        else if (p.gate_dt == INFR_Q8_0) done = try_gate_up<Q80Fmt>(s, p);
        if (done) return;
    }
    dim3 grid((p.nff + 3) / 4, p.rows * p.n_used), block(256);
    hipLaunchKernelGGL(moe_gate_up_generic, grid, block, 0, s, p, row_bytes_of(p.gate_dt, p.ne),
                       row_bytes_of(p.up_dt, p.ne));
}

template <class F>
static bool try_down(hipStream_t s, const MoeGemvParams& p) {
    int ks = fast_ks<F>(p.nff);
    if (!ks || p.n_used > kMaxUsedFast) return false;
    int lpr = p.nff / F::kBlockElems * F::kLPB;
    int rw = ks == 1 ? 64 / lpr : 1;
    int ot = tile_for(p.ne, p.n_cu, rw, kMaxOt);
    if (ot > kMaxOt) ot = kMaxOt;
    dim3 grid((p.ne + ot - 1) / ot, p.rows), block(256);
    if (ks == 1) hipLaunchKernelGGL((moe_down_combine_fast<F, 1>), grid, block, 0, s, p, ot);
    else hipLaunchKernelGGL((moe_down_combine_fast<F, 2>), grid, block, 0, s, p, ot);
    return true;
}

void launch_moe_down_combine(hipStream_t s, const MoeGemvParams& p) {
    bool done = false;
    if (p.down_dt == INFR_Q4K) done = try_down<Q4KFmt>(s, p);
    else if (p.down_dt == INFR_Q6K) done = try_down<Q6KFmt>(s, p);
    else if (p.down_dt == INFR_Q8_0) done = try_down<Q80Fmt>(s, p);
    if (done) return;
    dim3 grid((p.ne + 3) / 4, p.rows), block(256);
    hipLaunchKernelGGL(moe_down_combine_generic, grid, block, 0, s, p, row_bytes_of(p.down_dt, p.nff));
}

// ------------------------------------------------------------------------------- Op::Linear
// dst[m, out_f] = x . W^T, the dense neighbour of the expert GEMVs (shared expert).
template <class F, int KS>
__global__ __launch_bounds__(256) void linear_fast(const float* __restrict__ x, const uint8_t* __restrict__ w,
                                                   int in_f, int out_f, float* __restrict__ dst, int ot) {
    const int r = blockIdx.y;
    const int o0 = blockIdx.x * ot;
    const int ocount = min(ot, out_f - o0);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int nblk = in_f / F::kBlockElems;
    const size_t row_bytes = (size_t)nblk * F::kBlockBytes;
    const Place<F, KS> pl(nblk, lane);
    typename F::X xs[KS];
    load_x_all<F, KS>(xs, pl, x + (size_t)r * in_f);
    const uint8_t* bank = w + (size_t)o0 * row_bytes;
    const int stride = 4 * pl.rw_count;
    typename F::Raw raw[KS];
    int o = wave * pl.rw_count + pl.rw;
    load_row<F, KS>(raw, pl, bank + (size_t)o * row_bytes, o < ocount);
    for (int base = wave * pl.rw_count; base < ocount; base += stride, o += stride) {
        const bool valid = o < ocount;
        typename F::Raw nx[KS];
        load_row<F, KS>(nx, pl, bank + (size_t)(o + stride) * row_bytes, o + stride < ocount);
        float y = dot_row<F, KS>(raw, pl, xs, valid);
        y = row_sum<F, KS>(y, pl);
        if (valid && pl.pos == 0 && pl.rw < pl.rw_count) dst[(size_t)r * out_f + o0 + o] = y;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) raw[ks] = nx[ks];
    }
}

__global__ __launch_bounds__(256) void linear_generic(const float* __restrict__ x, const uint8_t* __restrict__ w,
                                                      int dt, size_t row_bytes, int in_f, int out_f,
                                                      float* __restrict__ dst) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int o = blockIdx.x * 4 + wave;
    const int r = blockIdx.y;
    if (o >= out_f) return;
    const uint8_t* row = w + (size_t)o * row_bytes;
    const float* xr = x + (size_t)r * in_f;
    float y = 0.f;
    for (int k = lane; k < in_f; k += kWave) y = fmaf(decode_elem(dt, row, (uint32_t)k), xr[k], y);
    y = wave_sum(y);
    if (lane == 0) dst[(size_t)r * out_f + o] = y;
}

template <class F>
static bool try_linear(hipStream_t s, const float* x, const uint8_t* w, int m, int in_f, int out_f, float* dst,
                       int n_cu) {
    int ks = fast_ks<F>(in_f);
    if (!ks) return false;
    int lpr = in_f / F::kBlockElems * F::kLPB;
    int rw = ks == 1 ? 64 / lpr : 1;
    int ot = tile_for(out_f, n_cu, 4 * rw, 1 << 20);
    dim3 grid((out_f + ot - 1) / ot, m), block(256);
    if (ks == 1) hipLaunchKernelGGL((linear_fast<F, 1>), grid, block, 0, s, x, w, in_f, out_f, dst, ot);
    else hipLaunchKernelGGL((linear_fast<F, 2>), grid, block, 0, s, x, w, in_f, out_f, dst, ot);
    return true;
}

void launch_linear(hipStream_t s, const float* x, const uint8_t* w, int dt, size_t row_bytes, int m, int in_f,
                   int out_f, float* dst, int n_cu) {
    bool done = false;
    if (dt == INFR_Q4K) done = try_linear<Q4KFmt>(s, x, w, m, in_f, out_f, dst, n_cu);
    else if (dt == INFR_Q6K) done = try_linear<Q6KFmt>(s, x, w, m, in_f, out_f, dst, n_cu);
    else if (dt == INFR_Q8_0) done = try_linear<Q80Fmt>(s, x, w, m, in_f, out_f, dst, n_cu);
    if (done) return;
    dim3 grid((out_f + 3) / 4, m), block(256);
    hipLaunchKernelGGL(linear_generic, grid, block, 0, s, x, w, dt, row_bytes, in_f, out_f, dst);
}

}  // namespace infr

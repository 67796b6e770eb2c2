// Shared by the grouped-GEMM kernels of Op::MoeFfn's batched path (k_grouped.hip: byte-exact LDS layouts of Q4_K / Q6_K /
// Q8_0; k_grouped_units.hip: every other format through the unit decoder): the weight formats' f16 unpacking, the work
// item look-up and the tile epilogue.
#pragma once

#include <type_traits>

#include "device_common.h"
#include "kernels.h"

namespace infr {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float16v __attribute__((ext_vector_type(16)));

namespace {

constexpr int kBM = 128;        // token rows per tile
constexpr int kSlice = 64;      // k elements per LDS stage

// Rotation of the eight 16-byte chunks of row t in an LDS tile whose rows are 128 bytes.  The LDS has 64 banks of 4
// bytes and serves a 16-byte read of a wavefront 16 lanes at a time: rows t and t + 1 start half the banks apart, so 16
// consecutive rows reading the same chunk hit 64 distinct banks when rows 2 u and 2 u + 1 share a rotation (measured:
// 205 B/clk per CU against 139 with a rotation by t & 7, 43 without any).
__device__ __forceinline__ int rot7(int t) { return (t >> 1) & 7; }

__device__ __forceinline__ half2v as_h2(uint32_t v) { return __builtin_bit_cast(half2v, v); }
__device__ __forceinline__ uint32_t as_u32(half2v v) { return __builtin_bit_cast(uint32_t, v); }
__device__ __forceinline__ half2v splat(float v) {
    _Float16 h = (_Float16)v;
    return half2v{h, h};
}
// (1024 + code pair) -> code pair - bias, exact
__device__ __forceinline__ half2v unbias(uint32_t magic_pair, float bias) { return as_h2(magic_pair) - splat(bias); }

// --------------------------------------------------------------------------------------------
// Weight formats.  A 64-k slice of a weight row unpacks to 8 operand chunks of 8 f16; the matrix
// instruction's lane halves split them: lanes 0..31 (half 0) own chunks 0..3, lanes 32..63 own
// chunks 4..7, and k-step ks of the slice contracts chunk ks of each half.  Four slices make one
// 256-element step (a K-quant super-block); what is shared by the four slices is fetched once:
//   Blk                     per-256 part (scales, high bits) half h needs of a step
//   Q                       the code bytes half h needs of virtual slice s
//   prep(blk, q, s, h)      per-slice scale constants
//   chunk(blk, q, c, ks, s) operand chunk 4h + ks as 8 f16
//   chunk_src()             for virtual chunk c of a row, the two real offsets whose float4s feed
//                           it and whether the 4 elements of each come out in the order 0,2,1,3
struct MQ4K {
    static constexpr int kBlockElems = 256, kBlockBytes = 144;
    struct Blk {
        uint4 hdr;   // d, dmin, 12 packed 6-bit scales / mins
    };
    struct Q {
        uint4 q;
    };
    struct Prep {
        half2v s_lo, n_lo, s_hi, n_hi;
        uint32_t magic;
    };
    // scales[i] of the 12 packed bytes, i in 0..11, without branches
    static __device__ __forceinline__ uint32_t scale_byte(const uint4& hdr, int i) {
        const uint64_t lo = ((uint64_t)hdr.z << 32) | hdr.y;   // bytes 0..7
        const uint32_t w = i < 8 ? (uint32_t)(lo >> (8 * (i & 7))) : hdr.w >> (8 * (i & 3));
        return w & 0xFFu;
    }
    static __device__ __forceinline__ void scale_min(const uint4& hdr, int j, uint32_t& sc, uint32_t& m) {
        // get_scale_min_k4 (crates/infr-gguf/src/dequant.rs:77-87), both arms evaluated and selected
        const uint32_t a = scale_byte(hdr, j & 3), b = scale_byte(hdr, (j & 3) + 4), c = scale_byte(hdr, (j & 3) + 8);
        const bool low = j < 4;
        sc = low ? (a & 63u) : ((c & 0x0Fu) | ((a >> 6) << 4));
        m = low ? (b & 63u) : ((c >> 4) | ((b >> 6) << 4));
    }
    static __device__ __forceinline__ Prep prep(const Blk& blk, const Q&, int s, int) {
        const int j = s & 3;
        const float d = f16_bits_to_f32(blk.hdr.x & 0xFFFFu), dmin = f16_bits_to_f32(blk.hdr.x >> 16);
        uint32_t sc0, m0, sc1, m1;
        scale_min(blk.hdr, 2 * j, sc0, m0);
        scale_min(blk.hdr, 2 * j + 1, sc1, m1);
        uint32_t magic = 0x64006400u;
        asm volatile("" : "+v"(magic));   // keep it in a vector register (a literal cannot share an instruction with the mask)
        return Prep{splat(d * (float)sc0), splat(-(dmin * (float)m0)), splat(d * (float)sc1), splat(-(dmin * (float)m1)), magic};
    }
    // byte l of the slice holds element l (low nibble, first 32-group) and 32 + l (high nibble)
    static __device__ __forceinline__ uint4 chunk(const Blk&, const Q& f, const Prep& c, int ks, int) {
        const uint32_t v = ks == 0 ? f.q.x : ks == 1 ? f.q.y : ks == 2 ? f.q.z : f.q.w;
        const uint32_t magic = c.magic;   // 0x64006400 in a register: one v_and_or_b32 per pair
        const half2v a = unbias((v & 0x000F000Fu) | magic, 1024.f);
        const half2v b = unbias(((v >> 8) & 0x000F000Fu) | magic, 1024.f);
        const half2v g = unbias(((v >> 4) & 0x000F000Fu) | magic, 1024.f);
        const half2v e = unbias(((v >> 12) & 0x000F000Fu) | magic, 1024.f);
        return uint4{as_u32(__builtin_elementwise_fma(a, c.s_lo, c.n_lo)), as_u32(__builtin_elementwise_fma(b, c.s_lo, c.n_lo)),
                     as_u32(__builtin_elementwise_fma(g, c.s_hi, c.n_hi)), as_u32(__builtin_elementwise_fma(e, c.s_hi, c.n_hi))};
    }
    static __device__ __forceinline__ void chunk_src(int c, int& lo, int& hi, bool& swz) {
        const int i = c & 7;
        lo = (c >> 3) * 64 + 4 * i;
        hi = lo + 32;
        swz = true;
    }
};

struct MQ6K {
    static constexpr int kBlockElems = 256, kBlockBytes = 210;
    // virtual slice t of a block: t = 2*half128 + ab; ab picks ql bytes [32ab, 32ab+32) of the
    // 128-element half; their low nibbles are elements [32ab, 32ab+32), their high nibbles +64.
    // The 2-bit tops of both ab of a half share the same qh bytes.
    struct Blk {
        uint4 sc;        // 16 int8 scales
        uint4 hq0, hq1;  // qh bytes [16h, 16h+16) of 128-element half 0 / 1
        uint32_t d;      // f16
    };
    struct Q {
        uint4 l;
    };
    struct Prep {
        half2v s_lo, s_hi;
    };
    static __device__ __forceinline__ Prep prep(const Blk& blk, const Q&, int s, int h) {
        // the lane's four chunks are 16 consecutive elements: one scale for the low codes
        // (scales[8hh + 2ab + h]) and one for the high codes (+4)
        const int hh = (s >> 1) & 1, ab = s & 1;
        const uint32_t w_lo = hh ? blk.sc.z : blk.sc.x, w_hi = hh ? blk.sc.w : blk.sc.y;
        const int sh = 8 * (2 * ab + h);
        const float d = f16_bits_to_f32(blk.d);
        return Prep{splat(d * (float)(int8_t)(w_lo >> sh)), splat(d * (float)(int8_t)(w_hi >> sh))};
    }
    static __device__ __forceinline__ uint4 chunk(const Blk& blk, const Q& f, const Prep& c, int ks, int s) {
        const int sh = 2 * (s & 1);  // qh bits sh..sh+1 complete the low codes, sh+4.. the high codes
        const uint4& hq = ((s >> 1) & 1) ? blk.hq1 : blk.hq0;
        const uint32_t L = ks == 0 ? f.l.x : ks == 1 ? f.l.y : ks == 2 ? f.l.z : f.l.w;
        const uint32_t H = (ks == 0 ? hq.x : ks == 1 ? hq.y : ks == 2 ? hq.z : hq.w) >> sh;
        const uint32_t a = (L & 0x000F000Fu) | ((H & 0x00030003u) << 4) | 0x64006400u;
        const uint32_t b = ((L >> 8) & 0x000F000Fu) | (((H >> 8) & 0x00030003u) << 4) | 0x64006400u;
        const uint32_t g = ((L >> 4) & 0x000F000Fu) | (H & 0x00300030u) | 0x64006400u;
        const uint32_t e = ((L >> 12) & 0x000F000Fu) | ((H >> 8) & 0x00300030u) | 0x64006400u;
        return uint4{as_u32(unbias(a, 1056.f) * c.s_lo), as_u32(unbias(b, 1056.f) * c.s_lo), as_u32(unbias(g, 1056.f) * c.s_hi),
                     as_u32(unbias(e, 1056.f) * c.s_hi)};
    }
    static __device__ __forceinline__ void chunk_src(int c, int& lo, int& hi, bool& swz) {
        const int blk = c >> 5, t = (c >> 3) & 3, i = c & 7;
        lo = blk * 256 + 128 * (t >> 1) + 32 * (t & 1) + 4 * i;
        hi = lo + 64;
        swz = true;
    }
};

struct MQ80 {
    static constexpr int kBlockElems = 32, kBlockBytes = 34;
    struct Blk {};
    struct Q {
        uint4 qa, qb;  // the 32 codes of block h of the slice
        uint32_t d;
    };
    struct Prep {
        half2v d;
    };
    static __device__ __forceinline__ Prep prep(const Blk&, const Q& f, int, int) { return Prep{splat(f16_bits_to_f32(f.d))}; }
    static __device__ __forceinline__ uint4 chunk(const Blk&, const Q& f, const Prep& c, int ks, int) {
        const uint32_t v0 = ks == 0 ? f.qa.x : ks == 1 ? f.qa.z : ks == 2 ? f.qb.x : f.qb.z;
        const uint32_t v1 = ks == 0 ? f.qa.y : ks == 1 ? f.qa.w : ks == 2 ? f.qb.y : f.qb.w;
        // bytes (b0,b1) and (b2,b3) to the low bytes of the two halves; x ^ 0x80 = x + 128 as unsigned
        const uint32_t a = __builtin_amdgcn_perm(0u, v0, 0x0C010C00u) ^ 0x64806480u;
        const uint32_t b = __builtin_amdgcn_perm(0u, v0, 0x0C030C02u) ^ 0x64806480u;
        const uint32_t g = __builtin_amdgcn_perm(0u, v1, 0x0C010C00u) ^ 0x64806480u;
        const uint32_t e = __builtin_amdgcn_perm(0u, v1, 0x0C030C02u) ^ 0x64806480u;
        return uint4{as_u32(unbias(a, 1152.f) * c.d), as_u32(unbias(b, 1152.f) * c.d), as_u32(unbias(g, 1152.f) * c.d),
                     as_u32(unbias(e, 1152.f) * c.d)};
    }
    static __device__ __forceinline__ void chunk_src(int c, int& lo, int& hi, bool& swz) {
        lo = 8 * c;
        hi = lo + 4;
        swz = false;
    }
};

// Activation for the matrix-core path: hardware exp (about 1e-6 relative), since operands were
// already rounded to f16.  Same formulas as act_fn / gated_act_fn (crates/infr-cpu/src/kernels.rs:6664-6683).
__device__ __forceinline__ float act_fast(int act, float g) {
    if (act == INFR_ACT_SILU) return g / (1.0f + __expf(-g));
    if (act == INFR_ACT_GELU) {
        const float inner = 0.7978846f * (g + 0.044715f * g * g * g);
        return 0.5f * g * (1.0f + tanhf(inner));
    }
    return 1.0f / (1.0f + __expf(-g));
}
__device__ __forceinline__ float gated_act_fast(int act, bool has_clamp, float clamp, float gate, float up) {
    if (has_clamp) {
        gate = fminf(gate, clamp);
        up = fminf(fmaxf(up, -clamp), clamp);
    }
    return act_fast(act, gate) * up;
}

// --------------------------------------------------------------------------------------------
struct Tile {
    int e, p0, cnt;
};
// The block's work item: (expert, 128-row tile of its bucket, column tile nt), items ordered by
// expert, row tile, column tile.  Workgroups go to the chip's 8 XCDs round-robin by workgroup id
// and every XCD has its own L2, so each XCD takes a contiguous eighth of the items: the column
// tiles of one row tile, which read the same activation tile, then sit behind the same L2.
// Uniform per wave; false when the block has nothing to do (the grid is an upper bound).
__device__ __forceinline__ bool find_item(const int32_t* __restrict__ offsets, int n_expert, int n_tiles_n, int lane,
                                          Tile& t, int& nt) {
    const int epl = (n_expert + 63) >> 6;
    const int e_lo = lane * epl, e_hi = min(n_expert, e_lo + epl);
    int mine = 0;
    for (int e = e_lo; e < e_hi; e++) mine += (offsets[e + 1] - offsets[e] + kBM - 1) / kBM;
    int incl = mine;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const int o = __shfl_up(incl, d, 64);
        if (lane >= d) incl += o;
    }
    const int n_items = __shfl(incl, 63, 64) * n_tiles_n;
    const int per = (n_items + 7) >> 3;
    const int k = (int)(blockIdx.x >> 3);
    const int item = (int)(blockIdx.x & 7) * per + k;
    if (k >= per || item >= n_items) return false;
    nt = item % n_tiles_n;
    const int tile = item / n_tiles_n;
    const unsigned long long past = __ballot(incl > tile);
    if (past == 0) return false;
    const int owner = __ffsll((long long)past) - 1;
    int rem = tile - (__shfl(incl, owner, 64) - __shfl(mine, owner, 64));
    const int o_lo = owner * epl, o_hi = min(n_expert, o_lo + epl);
    for (int e = o_lo; e < o_hi; e++) {
        const int cnt = offsets[e + 1] - offsets[e];
        const int ntile = (cnt + kBM - 1) / kBM;
        if (rem < ntile) {
            t.e = e;
            t.p0 = offsets[e] + rem * kBM;
            t.cnt = min(kBM, cnt - rem * kBM);
            return true;
        }
        rem -= ntile;
    }
    return false;
}

// Epilogue of a tile whose accumulators are acc0/acc1[M] (column tiles of the wave, M 32-row
// sub-tiles): SwiGLU of (gate, up) or the scaled down-projection row, stored to p.out.
// Only the accumulator registers 4 R4LO .. 4 R4HI - 1 of every 32 x 32 tile are stored (all 16 by default): a kernel whose
// wavefronts share a tile hands each of them a part of its rows.
template <bool DOWN, int M, int R4LO = 0, int R4HI = 4>
__device__ __forceinline__ void tile_epilogue(const GroupedParams& p, const Tile& t, int n0, int wave, int lane,
                                              const float* s_scale, const float16v (&acc0)[M], const float16v (&acc1)[M]) {
    // accumulator register r of a 32x32 tile: row 8*(r/4) + 4*(lane/32) + r%4, column lane%32.
    // The epilogue variant is chosen once, outside the loops; rows below the last 32-row sub-tile
    // are all inside the tile, so only that sub-tile tests the row count.
    const int fc0 = n0 + (DOWN ? 64 : 32) * wave + (lane & 31);   // the lane's column (second column tile of DOWN: + 32)
    float* const obase = p.out + (size_t)t.p0 * p.N + fc0;
    const int mrow = 4 * (lane >> 5);
    auto for_each = [&](auto&& body) {
#pragma unroll
        for (int mi = 0; mi < M; mi++) {
#pragma unroll
            for (int r4 = R4LO; r4 < R4HI; r4++) {
                const int m0 = 32 * mi + 8 * r4 + mrow;   // rows m0 .. m0 + 3
                const float4 sc4 = *reinterpret_cast<const float4*>(s_scale + m0);
                const float scs[4] = {sc4.x, sc4.y, sc4.z, sc4.w};
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int m = m0 + i;
                    if (mi < M - 1 || m < t.cnt) body(mi, 4 * r4 + i, m, scs[i], obase + (size_t)m * p.N);
                }
            }
        }
    };
    if (DOWN && p.out_f16) {
        // f16 without the row's power-of-two scale (|acc| stays far inside the f16 range: the
        // activation rows were normalised below 1); the combine multiplies the scale back in
        const float ds = p.down_scale ? p.down_scale[t.e] : 1.0f;
        const bool ok0 = fc0 < p.N, ok1 = fc0 + 32 < p.N;
        _Float16* const hbase = reinterpret_cast<_Float16*>(p.out) + (size_t)t.p0 * p.N + fc0;
        if (ok0) {
            for_each([&](int mi, int r, int m, float, float*) {
                _Float16* o = hbase + (size_t)m * p.N;
                o[0] = (_Float16)(acc0[mi][r] * ds);
                if (ok1) o[32] = (_Float16)(acc1[mi][r] * ds);
            });
        }
    } else if (DOWN) {
        const float ds = p.down_scale ? p.down_scale[t.e] : 1.0f;
        const bool ok0 = fc0 < p.N, ok1 = fc0 + 32 < p.N;
        if (ok1) {
            for_each([&](int mi, int r, int, float sc, float* o) {
                o[0] = acc0[mi][r] * sc * ds;
                o[32] = acc1[mi][r] * sc * ds;
            });
        } else if (ok0) {
            for_each([&](int mi, int r, int, float sc, float* o) { o[0] = acc0[mi][r] * sc * ds; });
        }
    } else if (fc0 < p.N) {
        if (p.act == INFR_ACT_SILU && !p.has_clamp && !p.weight_before) {
            // silu(g) * u with the hardware exp2 and reciprocal (1 ulp each; the operands were f16)
            for_each([&](int mi, int r, int, float sc, float* o) {
                const float g = acc0[mi][r] * sc, u = acc1[mi][r] * sc;
                o[0] = g * u * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(g * -1.4426950408889634f));
            });
        } else {
            for_each([&](int mi, int r, int m, float sc, float* o) {
                float g = acc0[mi][r] * sc, u = acc1[mi][r] * sc;
                if (p.weight_before) {
                    const float wp = p.route_w[p.pair_src[t.p0 + min(m, t.cnt - 1)]];
                    g *= wp;
                    u *= wp;
                }
                o[0] = gated_act_fast(p.act, p.has_clamp, p.clamp, g, u);
            });
        }
    }
}

}  // namespace

}  // namespace infr

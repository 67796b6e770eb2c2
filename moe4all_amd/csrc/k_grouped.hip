// Batched Op::MoeFfn: token -> expert bucketing and per-expert grouped GEMMs on the matrix cores.
//
// The CPU reference groups the (token row, rank) pairs of a batch by expert, experts ascending
// and rows ascending inside a bucket (crates/infr-cpu/src/lib.rs:3874-3908), and runs one GEMM
// per bucket (crates/infr-cpu/src/moe.rs:142-173).  Here:
//
//   bucket_kernel         offsets[e] = number of pairs whose expert id is below e, and the stable
//                         scatter of the pairs into that order (one block per expert; order is
//                         an integer contract and is reproduced exactly).
//   rows_to_f16_kernel    activation rows -> f16 with one power-of-two scale per row (so any f32
//                         magnitude fits), laid out in the k order the weight format unpacks to.
//   grouped_mfma6<D,DOWN> per (expert, 128-token tile, 128/256-feature tile): the raw quantised bytes
//                         of the tile's weight rows are copied into LDS, every lane unpacks its
//                         row's codes to f16 in registers with packed 16-bit arithmetic, the
//                         contraction runs on v_mfma_f32_32x32x16_f16 with f32 accumulation;
//                         epilogue = SwiGLU (gate/up) or plain scaled store (down).
//   unbucket_combine      dst[row] = sum over ranks (rank order, separate mul and add,
//                         lib.rs:4290-4302) of w * y[pair of (row, rank)].
//
// Unpacking trick: a code c in 0..1023 or'ed into 0x6400 is the f16 number 1024 + c, so a pair of
// codes sitting in the two halves of a dword becomes a pair of f16 values with one AND/OR, an
// exact packed subtract and one packed multiply(-add) with the group's scale.  The order in
// which codes fall out of a dword is not the element order; since a dot product does not care
// about the order of its terms, the activation rows are stored in that same ("virtual") order.
#include <type_traits>

#include "device_common.h"
#include "kernels.h"
#include "units.h"

namespace infr {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float16v __attribute__((ext_vector_type(16)));

namespace {

constexpr int kBM = 128;        // token rows per tile
constexpr int kSlice = 64;      // k elements per LDS stage

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

// --------------------------------------------------------------------------------------------
// One block per row: amax -> power-of-two scale -> f16 in the virtual k order of format F.
template <class F>
__global__ __launch_bounds__(256) void rows_to_f16_kernel(const float* __restrict__ src, int n,
                                                          _Float16* __restrict__ dst, float* __restrict__ scale) {
    __shared__ float s_max[4];
    const size_t row = blockIdx.x;
    const float* x = src + row * n;
    float m = 0.0f;
    for (int k = threadIdx.x * 4; k < n; k += 1024) {
        const float4 v = *reinterpret_cast<const float4*>(x + k);
        m = fmaxf(fmaxf(m, fmaxf(fabsf(v.x), fabsf(v.y))), fmaxf(fabsf(v.z), fabsf(v.w)));
    }
    m = wave_max(m);
    if ((threadIdx.x & 63) == 0) s_max[threadIdx.x >> 6] = m;
    __syncthreads();
    m = fmaxf(fmaxf(s_max[0], s_max[1]), fmaxf(s_max[2], s_max[3]));
    int e = 0;
    if (m > 0.0f && m < __builtin_inff()) (void)frexpf(m, &e);  // m = f * 2^e, f in [0.5, 1)
    const float inv = ldexpf(1.0f, -e);
    if (threadIdx.x == 0) scale[row] = ldexpf(1.0f, e);
    uint4* out = reinterpret_cast<uint4*>(dst + row * n);
    for (int c = threadIdx.x; c < n / 8; c += 256) {
        int lo, hi;
        bool swz;
        F::chunk_src(c, lo, hi, swz);
        const float4 a = *reinterpret_cast<const float4*>(x + lo), b = *reinterpret_cast<const float4*>(x + hi);
        half2v h0, h1, h2, h3;
        if (swz) {
            h0 = half2v{(_Float16)(a.x * inv), (_Float16)(a.z * inv)};
            h1 = half2v{(_Float16)(a.y * inv), (_Float16)(a.w * inv)};
            h2 = half2v{(_Float16)(b.x * inv), (_Float16)(b.z * inv)};
            h3 = half2v{(_Float16)(b.y * inv), (_Float16)(b.w * inv)};
        } else {
            h0 = half2v{(_Float16)(a.x * inv), (_Float16)(a.y * inv)};
            h1 = half2v{(_Float16)(a.z * inv), (_Float16)(a.w * inv)};
            h2 = half2v{(_Float16)(b.x * inv), (_Float16)(b.y * inv)};
            h3 = half2v{(_Float16)(b.z * inv), (_Float16)(b.w * inv)};
        }
        out[c] = uint4{as_u32(h0), as_u32(h1), as_u32(h2), as_u32(h3)};
    }
}

// --------------------------------------------------------------------------------------------
// One block of four wavefronts per expert e in 0..n_expert; the extra one marks pairs whose id is
// out of range.  The block stages the pair ids in LDS (16-bit, chunks of 16384, sixteen 16-byte
// loads in flight per thread), counts the pairs below e (= the bucket's offset), and then scatters
// the pairs equal to e: each wavefront takes a contiguous quarter of the chunk, the quarters' hit
// counts give every wavefront its base, and inside a quarter a wave-wide prefix keeps the flat
// (row, rank) order, so buckets come out rows ascending.
constexpr int kBucketChunk = 16384;
__global__ __launch_bounds__(256) void bucket_kernel(const int32_t* __restrict__ ids, int n_pairs, int n_expert,
                                                     int32_t* __restrict__ offsets, int32_t* __restrict__ pair_src,
                                                     int32_t* __restrict__ slot_pair) {
    __shared__ uint16_t s_ids[kBucketChunk];
    __shared__ uint32_t s_cnt[4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t e = blockIdx.x;
    auto narrow = [&](int32_t v) { return (uint32_t)v < (uint32_t)n_expert ? (uint32_t)v : 0xFFFFu; };  // n_expert <= 2048
    auto stage = [&](int c0, int cn) {
        __syncthreads();  // orders the LDS reads of the previous chunk before these writes
        // full groups of four ids: sixteen unconditional (index-clamped) 16-byte loads in flight per thread
        const int full = cn & ~3;
        if (full) {
            int4 v[16];
#pragma unroll
            for (int j = 0; j < 16; j++) {
                const int i = min((j * 256 + tid) * 4, full - 4);
                v[j] = *reinterpret_cast<const int4*>(ids + c0 + i);
            }
#pragma unroll
            for (int j = 0; j < 16; j++) {
                const int i = (j * 256 + tid) * 4;
                if (i < full) {
                    const uint32_t lo = narrow(v[j].x) | (narrow(v[j].y) << 16), hi = narrow(v[j].z) | (narrow(v[j].w) << 16);
                    *reinterpret_cast<uint2*>(&s_ids[i]) = make_uint2(lo, hi);
                }
            }
        }
        // the last one to three ids, padded to a group of four with 0xFFFF
        if (tid < 4 && full < cn) s_ids[full + tid] = full + tid < cn ? (uint16_t)narrow(ids[c0 + full + tid]) : (uint16_t)0xFFFF;
        __syncthreads();
    };
    // eight ids of group g (one 128-bit LDS read); the staging filled the chunk's last partial group
    // of four with 0xFFFF, the tail of a partial group of eight is masked here
    auto ids8 = [&](int g, int cn, uint32_t (&id)[8]) {
        const uint4 v = *reinterpret_cast<const uint4*>(&s_ids[8 * g]);
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int c = 0; c < 8; c++) {
            id[c] = (w[c >> 1] >> (16 * (c & 1))) & 0xFFFFu;
            if (8 * g + c >= ((cn + 3) & ~3)) id[c] = 0xFFFFu;
        }
    };
    auto wave_total = [&](uint32_t v) {
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) v += __shfl_xor(v, d, 64);
        return v;
    };
    const bool single = n_pairs <= kBucketChunk;   // a single chunk stays staged for the second pass

    // ---- pass 0: pairs with an id below e
    uint32_t below = 0;
    for (int c0 = 0; c0 < n_pairs; c0 += kBucketChunk) {
        const int cn = min(kBucketChunk, n_pairs - c0);
        stage(c0, cn);
        const int n8 = (cn + 7) >> 3;
#pragma unroll 2
        for (int g = tid; g < n8; g += 256) {
            uint32_t id[8];
            ids8(g, cn, id);
#pragma unroll
            for (int c = 0; c < 8; c++) below += id[c] < e;
        }
    }
    below = wave_total(below);
    __syncthreads();   // (s_cnt is free: nothing has used it yet)
    if (lane == 0) s_cnt[wave] = below;
    __syncthreads();
    below = s_cnt[0] + s_cnt[1] + s_cnt[2] + s_cnt[3];
    if (tid == 0) offsets[e] = (int32_t)below;

    // ---- pass 1: scatter the pairs with id e (the extra block: mark the ids out of range)
    uint32_t run = below;
    for (int c0 = 0; c0 < n_pairs; c0 += kBucketChunk) {
        const int cn = min(kBucketChunk, n_pairs - c0);
        if (!single) stage(c0, cn);
        if (e == (uint32_t)n_expert) {
            for (int i = tid; i < cn; i += 256)
                if (s_ids[i] == 0xFFFFu) slot_pair[c0 + i] = -1;
            continue;
        }
        const int n8 = (cn + 7) >> 3;
        const int per_wave = ((n8 + 255) >> 8) << 6;   // whole steps of 64 groups
        const int g_lo = wave * per_wave, g_hi = min(n8, g_lo + per_wave);
        // hits of this wavefront's quarter
        uint32_t hits = 0;
        for (int g = g_lo + lane; g < g_hi; g += 64) {
            uint32_t id[8];
            ids8(g, cn, id);
#pragma unroll
            for (int c = 0; c < 8; c++) hits += id[c] == e;
        }
        hits = wave_total(hits);
        __syncthreads();   // the previous chunk's readers of s_cnt are done
        if (lane == 0) s_cnt[wave] = hits;
        __syncthreads();
        uint32_t base = run;
        for (int w = 0; w < wave; w++) base += s_cnt[w];
        run += s_cnt[0] + s_cnt[1] + s_cnt[2] + s_cnt[3];
        for (int g0 = g_lo; g0 < g_hi; g0 += 64) {
            const int g = g0 + lane;
            uint32_t id[8];
#pragma unroll
            for (int c = 0; c < 8; c++) id[c] = 0xFFFFu;
            if (g < g_hi) ids8(g, cn, id);
            uint32_t mine = 0;
#pragma unroll
            for (int c = 0; c < 8; c++) mine += id[c] == e;
            // inclusive prefix of the per-lane hit counts (a lane's eight pairs are consecutive)
            uint32_t incl = mine;
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) {
                const uint32_t o = __shfl_up(incl, d, 64);
                if (lane >= d) incl += o;
            }
            uint32_t pos = base + incl - mine;
#pragma unroll
            for (int c = 0; c < 8; c++) {
                if (id[c] == e) {
                    pair_src[pos] = c0 + 8 * g + c;
                    slot_pair[c0 + 8 * g + c] = (int32_t)pos;
                    pos++;
                }
            }
            base += __shfl(incl, 63, 64);
        }
    }
}

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
template <bool DOWN, int M>
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
            for (int r4 = 0; r4 < 4; r4++) {
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

// --------------------------------------------------------------------------------------------
// Grouped GEMM: 256 threads = 4 waves, one wave per SIMD (so each may use the whole 512-entry
// register file: the 128 accumulators sit in AccVGPRs).  Per 64-k slice every wave contracts the
// slice for its two 32-feature column tiles (gate w / up w, or down 2w / 2w+1) against M 32-token
// row tiles; each lane unpacks the quantised bytes of ITS weight row and k half in registers into
// exactly the operand fragments it feeds to the matrix instruction.  M is a template parameter so
// that the k loop has no branches.  Every k-loop load goes straight from global memory into LDS
// (global_load_lds_dwordx4: lane i of a wave's load deposits its 16 bytes at base + 16 i), so that
// each load instruction covers whole cache lines and nothing is staged in registers:
//   * activation stage = the tile's 128 tokens x one 64-k slice (16 KB), token-major, the eight
//     16-byte chunks of a token rotated by (token & 7) so that the operand reads of 32 consecutive
//     tokens spread over all banks; every wave loads a quarter of it, kNA stages in the ring;
//   * weight stage = the parts of the 64 weight rows of ONE wave that a half super-block (128 k,
//     two slices) needs, row-major (Q4_K: header + 4 code chunks = 80 B per row; Q6_K: 4 low-code
//     chunks, 2 high-bit chunks, scales, tail = 128 B per row, chunks rotated by the row number);
//     private to the wave, 3 stages in the ring.
// The loads are issued from inline assembly, so the compiler neither counts them nor orders LDS
// reads against them: one explicit "s_waitcnt vmcnt(n); s_barrier" per slice does both.  The issue
// order is fixed (the same number of loads in every even and in every odd slice), so the number
// of loads younger than the ones slice s needs is a compile-time constant.
// M0 carries the LDS base of the transfer.  Nothing else in these kernels uses M0 (no other LDS-direct
// load, no indirect register addressing, no message), so it is not saved around the load.
__device__ __forceinline__ void dma16(const void* gsrc, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(gsrc), "s"(lds_base) : "memory");
}
template <int N>
__device__ __forceinline__ void wait_loads_then_barrier() {
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" : : "n"(N) : "memory");
}
__device__ __forceinline__ uint32_t lds_address(const void* p) {
    return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void*)p;
}

struct D4K : MQ4K {
    static constexpr int kNC = 5, kRowStride = 80, kNA = 4, kStepBytes = 144;   // kStepBytes: a row's bytes per 256 k
    // chunk `64 j + lane` of a weight stage: which staged row, where in the super-block its 16
    // bytes start for the first half, and how far the second half's lie behind
    static __device__ __forceinline__ void lane_chunk(int j, int lane, int& row, int& off0, int& hoff) {
        const int c = 64 * j + lane;
        row = c / 5;
        const int part = c - 5 * row;   // 0: header, 1..4: code bytes of the half
        off0 = 16 * part;
        hoff = part == 0 ? 0 : 64;
    }
    static __device__ __forceinline__ Blk read_blk(const uint8_t* st, int row, int) {
        return Blk{*reinterpret_cast<const uint4*>(st + row * kRowStride)};
    }
    static __device__ __forceinline__ Q read_q(const uint8_t* st, int row, int sl, int h) {
        return Q{*reinterpret_cast<const uint4*>(st + row * kRowStride + 16 + 32 * sl + 16 * h)};
    }
};

struct D6K : MQ6K {
    static constexpr int kNC = 8, kRowStride = 128, kNA = 3, kStepBytes = 210;
    static __device__ __forceinline__ int pos(int row, int part) { return row * kRowStride + ((part + row) & 7) * 16; }
    static __device__ __forceinline__ void lane_chunk(int j, int lane, int& row, int& off0, int& hoff) {
        row = 8 * j + (lane >> 3);
        const int part = ((lane & 7) - row) & 7;   // 0..3 low codes, 4..5 high bits, 6 scales, 7 tail (d in its last 2 bytes)
        off0 = part < 4 ? 16 * part : part < 6 ? 128 + 16 * (part - 4) : part == 6 ? 192 : 194;
        hoff = part < 4 ? 64 : part < 6 ? 32 : 0;
    }
    static __device__ __forceinline__ Blk read_blk(const uint8_t* st, int row, int h) {
        const uint4 hq = *reinterpret_cast<const uint4*>(st + pos(row, 4 + h));
        return Blk{*reinterpret_cast<const uint4*>(st + pos(row, 6)), hq, hq,
                   *reinterpret_cast<const uint16_t*>(st + pos(row, 7) + 14)};
    }
    static __device__ __forceinline__ Q read_q(const uint8_t* st, int row, int sl, int h) {
        return Q{*reinterpret_cast<const uint4*>(st + pos(row, 2 * sl + h))};
    }
};

// Q8_0: a half-step is four 34-byte blocks = 136 bytes of a row: eight chunks for bytes 0..127 and a
// ninth for bytes 120..135 (the last block's upper 16 codes, so that nothing past the row is read).
struct D80 : MQ80 {
    static constexpr int kNC = 9, kRowStride = 144, kNA = 3, kStepBytes = 272;
    static __device__ __forceinline__ void lane_chunk(int j, int lane, int& row, int& off0, int& hoff) {
        const int c = 64 * j + lane;
        row = c / 9;
        const int part = c - 9 * row;
        off0 = part < 8 ? 16 * part : 120;
        hoff = 136;
    }
    static __device__ __forceinline__ Blk read_blk(const uint8_t*, int, int) { return Blk{}; }
    static __device__ __forceinline__ Q read_q(const uint8_t* st, int row, int sl, int h) {
        const int i = 2 * sl + h;   // block of the half-step
        const uint8_t* r = st + row * kRowStride;
        return Q{ldu<uint4>(r + 34 * i + 2), ldu<uint4>(r + (i == 3 ? 128 : 34 * i + 18)), ldu<uint16_t>(r + 34 * i)};
    }
};

constexpr int kNW6 = 3;                    // weight stages per wave
constexpr int kAStage6 = kBM * 128;        // bytes per activation stage
template <class D>
constexpr size_t grouped6_lds() { return (size_t)D::kNA * kAStage6 + (size_t)4 * kNW6 * 64 * D::kRowStride + kBM * 4; }

struct Grouped6Ctx {
    uint8_t* lds;             // [kNA activation stages][4 waves x kNW6 weight stages][row scales]
    const float* s_scale;
    const uint8_t* asrc[4];   // the lane's four activation chunks of slice 0
    int wave, lane, n0;
    Tile t;
};

template <class D, bool DOWN, int M>
__device__ __forceinline__ void grouped6_tile(const GroupedParams& p, const Grouped6Ctx& c, const uint8_t* const (&wsrc)[D::kNC],
                                              const int (&whoff)[D::kNC]) {
    constexpr int NA = D::kNA, NC = D::kNC, NW = kNW6;
    constexpr int kWStage = 64 * D::kRowStride;
    const int wave = c.wave, lane = c.lane, half = lane >> 5;
    float16v acc0[M], acc1[M];
#pragma unroll
    for (int i = 0; i < M; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc0[i][r] = acc1[i][r] = 0.0f;
    const int n_slices = p.K / kSlice, last = n_slices - 1, last_hs = (n_slices >> 1) - 1;
    const uint32_t lds0 = lds_address(c.lds);
    const uint32_t uwave = __builtin_amdgcn_readfirstlane(wave);
    const uint32_t a_dst = lds0 + uwave * 4096;                                   // + stage * kAStage6 + q * 1024
    const uint32_t w_dst = lds0 + NA * kAStage6 + uwave * (NW * kWStage);         // + stage * kWStage + j * 1024
    const uint8_t* const w_lds = c.lds + NA * kAStage6 + wave * (NW * kWStage);
    const uint8_t* const as0 = c.asrc[0];
    const uint8_t* const as1 = c.asrc[1];
    const uint8_t* const as2 = c.asrc[2];
    const uint8_t* const as3 = c.asrc[3];
    // Loads issued while slice s is contracted, a quarter after each k step so that the four waves
    // do not queue up at the address unit together: part ks = (on even s the weight chunks
    // 0..(NC+1)/2-1, on odd s the rest, one per k step) of half-step s/2 + NW - 1, then activation
    // quarter ks of slice s + NA - 1 (a fifth weight chunk of a slice goes with k step 0).  The last load
    // of a slice is its activation quarter 3.
    constexpr int kWEven = (NC + 1) / 2;
    auto issue_w = [&](int s, int j) {
        const int hs = (s >> 1) + NW - 1;
        if (hs < 0) return;
        const int hc = min(hs, last_hs);
        dma16(wsrc[j] + (size_t)(hc >> 1) * D::kStepBytes + ((hc & 1) ? whoff[j] : 0),
              w_dst + (uint32_t)(hs % NW) * kWStage + j * 1024);
    };
    auto issue_part = [&](int s, int odd, int ks) {   // odd = s & 1; odd and ks are constants where this is called
        const int lo = odd ? kWEven : 0, hi = odd ? NC : kWEven;
#pragma unroll
        for (int j = 0; j < NC; j++)
            if (j >= lo && j < hi && ((j - lo) & 3) == ks) issue_w(s, j);
        const int sa = s + NA - 1;
        if (sa >= 0) {
            const uint8_t* src = ks == 0 ? as0 : ks == 1 ? as1 : ks == 2 ? as2 : as3;
            dma16(src + (size_t)min(sa, last) * 128, a_dst + (uint32_t)(sa % NA) * kAStage6 + ks * 1024);
        }
    };
#pragma unroll
    for (int s = -2 * (NW - 1); s < 0; s++)
#pragma unroll
        for (int ks = 0; ks < 4; ks++) issue_part(s, s & 1, ks);

    // operand reads: token 32 mi + (lane & 31), k chunk ks + 4 half, rotated by the token's low bits
    const int x7 = lane & 7;
    const int a_lane = (lane & 31) * 128;
    int a_off[4];
#pragma unroll
    for (int ks = 0; ks < 4; ks++) a_off[ks] = a_lane + (((ks + 4 * half) ^ x7) * 16);
    const int row0 = lane & 31, row1 = 32 + (lane & 31);

    // slice s (compile-time position j4 = s & 3 inside its super-block)
    auto slice = [&](int s, auto j4c) {
        constexpr int j4 = decltype(j4c)::value;
        // loads younger than the last one this slice needs (activation quarter 3 of slice s, issued at
        // the end of slice s - NA + 1): everything issued during the NA - 2 slices since
        constexpr int kWOdd = NC - kWEven;
        constexpr int kYoung = NA == 4 ? 8 + NC : 4 + ((j4 & 1) ? kWEven : kWOdd);
        static_assert(NA == 3 || NA == 4, "the load counts above are written for these ring depths");
        wait_loads_then_barrier<kYoung>();
        const uint8_t* ap = c.lds + (s % NA) * kAStage6;
        const uint8_t* wst = w_lds + ((s >> 1) % NW) * kWStage;
        const typename D::Blk k0 = D::read_blk(wst, row0, half), k1 = D::read_blk(wst, row1, half);
        const typename D::Q f0 = D::read_q(wst, row0, j4 & 1, half), f1 = D::read_q(wst, row1, j4 & 1, half);
        uint4 a[M];
#pragma unroll
        for (int mi = 0; mi < M; mi++) a[mi] = *reinterpret_cast<const uint4*>(ap + a_off[0] + mi * 4096);
        const typename D::Prep c0 = D::prep(k0, f0, j4, half), c1 = D::prep(k1, f1, j4, half);
        uint4 b0 = D::chunk(k0, f0, c0, 0, j4), b1 = D::chunk(k1, f1, c1, 0, j4);
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
            uint4 nb0 = b0, nb1 = b1;
            if (ks < 3) {
                nb0 = D::chunk(k0, f0, c0, ks + 1, j4);
                nb1 = D::chunk(k1, f1, c1, ks + 1, j4);
            }
            issue_part(s, j4 & 1, ks);
#pragma unroll
            for (int mi = 0; mi < M; mi++) {
                acc0[mi] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, a[mi]), __builtin_bit_cast(half8, b0),
                                                                  acc0[mi], 0, 0, 0);
                acc1[mi] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, a[mi]), __builtin_bit_cast(half8, b1),
                                                                  acc1[mi], 0, 0, 0);
                if (ks < 3) a[mi] = *reinterpret_cast<const uint4*>(ap + a_off[ks + 1] + mi * 4096);
            }
            b0 = nb0;
            b1 = nb1;
        }
    };
    for (int s0 = 0; s0 < n_slices; s0 += 4) {
        slice(s0, std::integral_constant<int, 0>{});
        slice(s0 + 1, std::integral_constant<int, 1>{});
        slice(s0 + 2, std::integral_constant<int, 2>{});
        slice(s0 + 3, std::integral_constant<int, 3>{});
    }
    // nothing may still be landing in LDS when the block ends (or another block takes over the CU's LDS)
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    tile_epilogue<DOWN, M>(p, c.t, c.n0, wave, lane, c.s_scale, acc0, acc1);
}

template <class D, bool DOWN>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void grouped_mfma6(GroupedParams p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds6[];
    Grouped6Ctx c;
    c.lds = lds6;
    float* s_scale = reinterpret_cast<float*>(lds6 + grouped6_lds<D>() - kBM * 4);
    c.s_scale = s_scale;
    const int tid = threadIdx.x;
    c.wave = tid >> 6;
    c.lane = tid & 63;
    int nt;
    if (!find_item(p.offsets, p.n_expert, p.n_tiles_n, c.lane, c.t, nt)) return;
    const Tile& t = c.t;
    constexpr int kBN = DOWN ? 256 : 128;
    c.n0 = nt * kBN;
    // sources of the lane's chunks of the wave's weight stage (half-step 0)
    const size_t row_bytes = (size_t)(p.K / D::kBlockElems) * D::kBlockBytes;
    const uint8_t* wsrc[D::kNC];
    int whoff[D::kNC];
#pragma unroll
    for (int j = 0; j < D::kNC; j++) {
        int row, off0;
        D::lane_chunk(j, c.lane, row, off0, whoff[j]);
        const uint8_t* base;
        int f;
        if (DOWN) {
            base = p.w0 + (size_t)t.e * p.w0_stride;
            f = c.n0 + 64 * c.wave + row;
        } else {
            base = row < 32 ? p.w0 + (size_t)t.e * p.w0_stride : p.w1 + (size_t)t.e * p.w1_stride;
            f = c.n0 + 32 * c.wave + (row & 31);
        }
        wsrc[j] = base + (size_t)min(f, p.N - 1) * row_bytes + off0;
    }
    // the lane's activation chunks: token 32 wave + 8 q + lane / 8, chunk (lane & 7) ^ (token & 7)
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const int tok = 32 * c.wave + 8 * q + (c.lane >> 3), kg = (c.lane & 7) ^ ((c.lane >> 3) & 7);
        const int pr = t.p0 + min(tok, t.cnt - 1);
        const size_t src_row = DOWN ? (size_t)pr : (size_t)(p.pair_src[pr] / p.n_used);
        c.asrc[q] = reinterpret_cast<const uint8_t*>(p.a + src_row * p.K) + 16 * kg;
    }
    if (tid < kBM) {
        const int pr = t.p0 + min(tid, t.cnt - 1);
        s_scale[tid] = p.a_scale[DOWN ? pr : p.pair_src[pr] / p.n_used];
    }
    switch ((t.cnt + 31) >> 5) {
        case 1: grouped6_tile<D, DOWN, 1>(p, c, wsrc, whoff); break;
        case 2: grouped6_tile<D, DOWN, 2>(p, c, wsrc, whoff); break;
        case 3: grouped6_tile<D, DOWN, 3>(p, c, wsrc, whoff); break;
        default: grouped6_tile<D, DOWN, 4>(p, c, wsrc, whoff); break;
    }
}

// dst[row, :] = sum over ranks of w * y[slot_pair[row, rank], :], rank order, separate mul/add.
// Y = _Float16: y rows carry no row scale, pair_scale[pair] multiplies it back in.
template <class Y>
__global__ __launch_bounds__(256) void unbucket_combine_kernel(const Y* __restrict__ y, const int32_t* __restrict__ slot_pair,
                                                               const float* __restrict__ weights, int ne, int n_used,
                                                               int weight_before, float* dst, int identity,
                                                               const float* __restrict__ pair_scale, const float* addend,
                                                               int skip_zero_w) {
    const size_t row = blockIdx.y;
    const int i = (blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= ne) return;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int k = 0; k < n_used; k++) {
        int pr = slot_pair ? slot_pair[row * n_used + k] : 0;
        if (pr < 0) continue;
        if (identity || !slot_pair) pr = (int)(row * n_used + k);
        if (skip_zero_w && weights[row * n_used + k] == 0.0f) continue;
        const float w = weight_before ? 1.0f : weights[row * n_used + k];
        const float sc = pair_scale ? pair_scale[pr] : 1.0f;
        const Y* yr = y + (size_t)pr * ne + i;
        float v[4] = {0.f, 0.f, 0.f, 0.f};
        if (i + 3 < ne) {
            if (sizeof(Y) == 2) {
                const uint2 raw = *reinterpret_cast<const uint2*>(yr);
                const half2v a = as_h2(raw.x), b = as_h2(raw.y);
                v[0] = (float)a[0]; v[1] = (float)a[1]; v[2] = (float)b[0]; v[3] = (float)b[1];
            } else {
                const float4 f = *reinterpret_cast<const float4*>(yr);
                v[0] = f.x; v[1] = f.y; v[2] = f.z; v[3] = f.w;
            }
        } else {
            for (int q = 0; i + q < ne; q++) v[q] = (float)yr[q];
        }
        if (pair_scale) {
#pragma unroll
            for (int q = 0; q < 4; q++) v[q] *= sc;
        }
        acc.x = __fadd_rn(acc.x, __fmul_rn(w, v[0]));
        acc.y = __fadd_rn(acc.y, __fmul_rn(w, v[1]));
        acc.z = __fadd_rn(acc.z, __fmul_rn(w, v[2]));
        acc.w = __fadd_rn(acc.w, __fmul_rn(w, v[3]));
    }
    float* o = dst + row * ne + i;
    if (addend) {   // a following Op::Add folded in: the finished sum is added to the other operand
        const float* ad = addend + row * ne + i;
        if (i + 3 < ne) {
            const float4 f = *reinterpret_cast<const float4*>(ad);
            acc.x = __fadd_rn(f.x, acc.x); acc.y = __fadd_rn(f.y, acc.y);
            acc.z = __fadd_rn(f.z, acc.z); acc.w = __fadd_rn(f.w, acc.w);
        } else {
            float* a = &acc.x;
            for (int q = 0; i + q < ne; q++) a[q] = __fadd_rn(ad[q], a[q]);
        }
    }
    if (i + 3 < ne) *reinterpret_cast<float4*>(o) = acc;
    else {
        const float* a = &acc.x;
        for (int q = 0; i + q < ne; q++) o[q] = a[q];
    }
}

// The same sum for f16 pair rows whose length is a multiple of 8: eight elements (16 bytes) per lane and slot, all
// slots of the row requested before the first is used.  Same operations per element as the kernel above.
template <int K>
__global__ __launch_bounds__(256) void unbucket_combine_h8_kernel(const _Float16* __restrict__ y, const int32_t* __restrict__ slot_pair,
                                                                  const float* __restrict__ weights, int ne, int weight_before,
                                                                  float* dst, int identity, const float* __restrict__ pair_scale,
                                                                  const float* addend, int skip_zero_w) {
    const size_t row = blockIdx.y;
    const int i = (blockIdx.x * 256 + threadIdx.x) * 8;
    if (i >= ne) return;
    uint4 raw[K];
    float w[K], sc[K];
    bool live[K];
#pragma unroll
    for (int k = 0; k < K; k++) {
        int pr = slot_pair ? slot_pair[row * K + k] : 0;
        const float wk = weights[row * K + k];
        live[k] = pr >= 0 && !(skip_zero_w && wk == 0.0f);
        if (identity || !slot_pair) pr = (int)(row * K + k);
        w[k] = weight_before ? 1.0f : wk;
        sc[k] = live[k] ? pair_scale[pr] : 0.0f;
        raw[k] = live[k] ? *reinterpret_cast<const uint4*>(y + (size_t)pr * ne + i) : make_uint4(0, 0, 0, 0);
    }
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int k = 0; k < K; k++) {
        if (!live[k]) continue;
        const uint32_t d[4] = {raw[k].x, raw[k].y, raw[k].z, raw[k].w};
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const half2v h = as_h2(d[q]);
            acc[2 * q] = __fadd_rn(acc[2 * q], __fmul_rn(w[k], (float)h[0] * sc[k]));
            acc[2 * q + 1] = __fadd_rn(acc[2 * q + 1], __fmul_rn(w[k], (float)h[1] * sc[k]));
        }
    }
    float* o = dst + row * ne + i;
    if (addend) {
        const float4 a0 = *reinterpret_cast<const float4*>(addend + row * ne + i), a1 = *reinterpret_cast<const float4*>(addend + row * ne + i + 4);
        const float ad[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
#pragma unroll
        for (int q = 0; q < 8; q++) acc[q] = __fadd_rn(ad[q], acc[q]);
    }
    *reinterpret_cast<float4*>(o) = make_float4(acc[0], acc[1], acc[2], acc[3]);
    *reinterpret_cast<float4*>(o + 4) = make_float4(acc[4], acc[5], acc[6], acc[7]);
}

template <class F>
void rows_to_f16(hipStream_t s, const float* src, int rows, int n, _Float16* dst, float* scale) {
    INFR_LAUNCH(rows_to_f16_kernel<F>, dim3(rows), dim3(256), 0, s, src, n, dst, scale);
}

template <class D, bool DOWN>
void grouped6(hipStream_t s, const GroupedParams& p) {
    const int bn = DOWN ? 256 : 128;
    GroupedParams q = p;
    q.n_tiles_n = (p.N + bn - 1) / bn;
    const int max_tiles = p.n_pairs / kBM + (p.n_expert < p.n_pairs ? p.n_expert : p.n_pairs);
    static bool attr_set = false;  // per instantiation
    if (!attr_set) {
        (void)hipFuncSetAttribute((const void*)grouped_mfma6<D, DOWN>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                  (int)grouped6_lds<D>());
        attr_set = true;
    }
    INFR_LAUNCH((grouped_mfma6<D, DOWN>), dim3((unsigned)((max_tiles * q.n_tiles_n + 7) & ~7)), dim3(256), grouped6_lds<D>(), s, q);   // whole rounds of the 8 XCDs
}

// --------------------------------------------------------------------------------------------
// Grouped GEMM for every affine format through the 32-element unit decoder: the matrix-core path of banks
// that have no byte-exact LDS layout above.  Same tiles (expert, <= 128 tokens, 128 features with gate and
// up, or 256 features of down), same accumulator layout and epilogue.  Per 64-k slice a lane decodes ONE
// unit of each of its two weight rows - lanes 0..31 the slice's first 32 k, lanes 32..63 the second - into
// four 8-element f16 operand fragments (f32 sc * code + mn, rounded once), so no element is decoded
// twice; k step ks of the slice contracts elements 8 ks .. 8 ks + 7 of both units.  The activation tile
// (natural k order) goes through registers into a two-stage LDS ring with the chunk rotation of the
// kernel above; the next slice's units and activation chunks are requested before the current slice is
// contracted.
constexpr int kUStage = kBM * 128;   // 128 tokens x 64 halfs

// The 32 k of one weight row that a lane contracts in a slice, and its four 8-element f16 fragments.
template <int DT>
struct WSlice {
    Unit u;
    __device__ __forceinline__ void load(const uint8_t* __restrict__ row, int idx) { load_unit<DT>(row, idx, u); }
    __device__ __forceinline__ half8 frag(int ks) const {
        const float sc = u.sc[ks >> 1], mn = u.mn[ks >> 1];
        const uint32_t a = u.q[2 * ks], b = u.q[2 * ks + 1];
        half8 h;
        h[0] = (_Float16)fmaf(sc, (float)(a & 0xFFu), mn);
        h[1] = (_Float16)fmaf(sc, (float)((a >> 8) & 0xFFu), mn);
        h[2] = (_Float16)fmaf(sc, (float)((a >> 16) & 0xFFu), mn);
        h[3] = (_Float16)fmaf(sc, (float)(a >> 24), mn);
        h[4] = (_Float16)fmaf(sc, (float)(b & 0xFFu), mn);
        h[5] = (_Float16)fmaf(sc, (float)((b >> 8) & 0xFFu), mn);
        h[6] = (_Float16)fmaf(sc, (float)((b >> 16) & 0xFFu), mn);
        h[7] = (_Float16)fmaf(sc, (float)(b >> 24), mn);
        return h;
    }
};
// Unquantised weights: F16 rows are the fragments as they lie in memory; BF16 / F32 are rounded to f16.
template <>
struct WSlice<INFR_F16> {
    uint4 v[4];
    __device__ __forceinline__ void load(const uint8_t* __restrict__ row, int idx) {
#pragma unroll
        for (int k = 0; k < 4; k++) v[k] = ldu<uint4>(row + (size_t)idx * 64 + 16 * k);
    }
    __device__ __forceinline__ half8 frag(int ks) const { return __builtin_bit_cast(half8, v[ks]); }
};
template <>
struct WSlice<INFR_BF16> {
    uint4 v[4];
    __device__ __forceinline__ void load(const uint8_t* __restrict__ row, int idx) {
#pragma unroll
        for (int k = 0; k < 4; k++) v[k] = ldu<uint4>(row + (size_t)idx * 64 + 16 * k);
    }
    __device__ __forceinline__ half8 frag(int ks) const {
        const uint32_t d[4] = {v[ks].x, v[ks].y, v[ks].z, v[ks].w};
        half8 h;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            h[2 * k] = (_Float16)__uint_as_float(d[k] << 16);
            h[2 * k + 1] = (_Float16)__uint_as_float(d[k] & 0xFFFF0000u);
        }
        return h;
    }
};
template <>
struct WSlice<INFR_F32> {
    uint4 v[8];
    __device__ __forceinline__ void load(const uint8_t* __restrict__ row, int idx) {
#pragma unroll
        for (int k = 0; k < 8; k++) v[k] = ldu<uint4>(row + (size_t)idx * 128 + 16 * k);
    }
    __device__ __forceinline__ half8 frag(int ks) const {
        const uint4 a = v[2 * ks], b = v[2 * ks + 1];
        half8 h;
        h[0] = (_Float16)__uint_as_float(a.x); h[1] = (_Float16)__uint_as_float(a.y);
        h[2] = (_Float16)__uint_as_float(a.z); h[3] = (_Float16)__uint_as_float(a.w);
        h[4] = (_Float16)__uint_as_float(b.x); h[5] = (_Float16)__uint_as_float(b.y);
        h[6] = (_Float16)__uint_as_float(b.z); h[7] = (_Float16)__uint_as_float(b.w);
        return h;
    }
};

template <int DT, bool DOWN, int M>
__device__ __forceinline__ void grouped_units_tile(const GroupedParams& p, const Tile& t, int n0, uint8_t* lds, const float* s_scale) {
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, half = lane >> 5;
    float16v acc0[M], acc1[M];
#pragma unroll
    for (int i = 0; i < M; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc0[i][r] = acc1[i][r] = 0.0f;
    int be = 1, bb = 4;
    block_geometry(DT, &be, &bb);
    const size_t row_bytes = (size_t)(p.K / be) * bb;
    // the lane's two weight rows
    const uint8_t* w0;
    const uint8_t* w1;
    {
        const int c = lane & 31;
        if (DOWN) {
            const uint8_t* base = p.w0 + (size_t)t.e * p.w0_stride;
            w0 = base + (size_t)min(n0 + 64 * wave + c, p.N - 1) * row_bytes;
            w1 = base + (size_t)min(n0 + 64 * wave + 32 + c, p.N - 1) * row_bytes;
        } else {
            const int f = min(n0 + 32 * wave + c, p.N - 1);
            w0 = p.w0 + (size_t)t.e * p.w0_stride + (size_t)f * row_bytes;
            w1 = p.w1 + (size_t)t.e * p.w1_stride + (size_t)f * row_bytes;
        }
    }
    // the lane's four activation chunks of a slice: token 32 wave + 8 q + lane / 8, LDS position lane & 7
    const uint8_t* asrc[4];
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const int tok = 32 * wave + 8 * q + (lane >> 3), kg = (lane & 7) ^ ((lane >> 3) & 7);
        const int pr = t.p0 + min(tok, t.cnt - 1);
        const size_t src_row = DOWN ? (size_t)pr : (size_t)(p.pair_src[pr] / p.n_used);
        asrc[q] = reinterpret_cast<const uint8_t*>(p.a + src_row * p.K) + 16 * kg;
    }
    uint8_t* const a_dst = lds + wave * 4096 + lane * 16;   // + stage * kUStage + q * 1024
    const int x7 = lane & 7;
    int a_off[4];
#pragma unroll
    for (int ks = 0; ks < 4; ks++) a_off[ks] = (lane & 31) * 128 + (((ks + 4 * half) ^ x7) * 16);

    const int n_slices = p.K / kSlice;
    WSlice<DT> u0, u1;
    uint4 ar0, ar1, ar2, ar3;   // named, not an array: the array form ends up in scratch memory
    u0.load(w0, half);
    u1.load(w1, half);
    ar0 = *reinterpret_cast<const uint4*>(asrc[0]);
    ar1 = *reinterpret_cast<const uint4*>(asrc[1]);
    ar2 = *reinterpret_cast<const uint4*>(asrc[2]);
    ar3 = *reinterpret_cast<const uint4*>(asrc[3]);
    *reinterpret_cast<uint4*>(a_dst) = ar0;
    *reinterpret_cast<uint4*>(a_dst + 1024) = ar1;
    *reinterpret_cast<uint4*>(a_dst + 2048) = ar2;
    *reinterpret_cast<uint4*>(a_dst + 3072) = ar3;
    __syncthreads();
    for (int s = 0; s < n_slices; s++) {
        const bool more = s + 1 < n_slices;
        WSlice<DT> v0, v1;
        if (more) {   // requests for the next slice
            v0.load(w0, 2 * (s + 1) + half);
            v1.load(w1, 2 * (s + 1) + half);
            const size_t ao = (size_t)(s + 1) * 128;
            ar0 = *reinterpret_cast<const uint4*>(asrc[0] + ao);
            ar1 = *reinterpret_cast<const uint4*>(asrc[1] + ao);
            ar2 = *reinterpret_cast<const uint4*>(asrc[2] + ao);
            ar3 = *reinterpret_cast<const uint4*>(asrc[3] + ao);
        }
        const uint8_t* ap = lds + (s & 1) * kUStage;
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
            const half8 b0 = u0.frag(ks), b1 = u1.frag(ks);
#pragma unroll
            for (int mi = 0; mi < M; mi++) {
                const half8 a = *reinterpret_cast<const half8*>(ap + a_off[ks] + mi * 4096);
                acc0[mi] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b0, acc0[mi], 0, 0, 0);
                acc1[mi] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b1, acc1[mi], 0, 0, 0);
            }
        }
        // One wave per SIMD: the decode of the next fragments has to issue between this wave's own matrix
        // instructions, or the two pipes take turns.  Ask the scheduler for one MFMA, then a share of the VALU work.
#pragma unroll
        for (int i = 0; i < 8 * M; i++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x002, 256 / (8 * M), 0);
        }
        if (more) {
            uint8_t* d = a_dst + ((s + 1) & 1) * kUStage;
            *reinterpret_cast<uint4*>(d) = ar0;
            *reinterpret_cast<uint4*>(d + 1024) = ar1;
            *reinterpret_cast<uint4*>(d + 2048) = ar2;
            *reinterpret_cast<uint4*>(d + 3072) = ar3;
            u0 = v0;
            u1 = v1;
        }
        __syncthreads();   // the stage just written is complete; the stage just read may be overwritten
    }
    tile_epilogue<DOWN, M>(p, t, n0, wave, lane, s_scale, acc0, acc1);
}

// Weight rows through LDS.  A lane that reads its own row's unit straight from memory makes every load
// instruction of the wave touch 64 rows, one or two cache lines each: the address unit of the CU, not the
// matrix pipe, then sets the pace (measured: 93 line look-ups per load instruction, 73 % of the kernel's
// cycles).  Here each wave copies the next 256 k of its 64 rows (the window: a whole number of blocks, WB
// bytes per row) into a region of its own with consecutive lanes on consecutive 16-byte chunks of a row, and
// the units are cut out of LDS.  Row pitch 16 * odd: sixteen lanes reading the same offset of sixteen rows
// fall on distinct banks.  Windows alternate between two stages; window g + 1 is requested at the first
// slice of window g and written after its third, one barrier before its first unit is read.
template <int DT>
struct StagedW {
    static constexpr int kBlock = DT == INFR_Q4_0 || DT == INFR_Q4_1 || DT == INFR_Q5_0 || DT == INFR_Q5_1 || DT == INFR_Q8_0 ||
                                          DT == INFR_IQ4_NL || DT == INFR_MXFP4 ? 32
                                  : DT == INFR_Q2_0 || DT == INFR_NVFP4 ? 64 : 256;
    static constexpr int kBlockBytes = DT == INFR_Q4_0 ? 18 : DT == INFR_Q4_1 ? 20 : DT == INFR_Q5_0 ? 22 : DT == INFR_Q5_1 ? 24
                                       : DT == INFR_Q8_0 ? 34 : DT == INFR_Q2K ? 84 : DT == INFR_Q3K ? 110 : DT == INFR_Q4K ? 144
                                       : DT == INFR_Q5K ? 176 : DT == INFR_Q6K ? 210 : DT == INFR_IQ4_NL ? 18 : DT == INFR_IQ4_XS ? 136
                                       : DT == INFR_TQ1_0 ? 54 : DT == INFR_TQ2_0 ? 66 : DT == INFR_Q2_0 ? 18 : DT == INFR_MXFP4 ? 17
                                       : DT == INFR_NVFP4 ? 36 : DT == INFR_IQ1_S ? 50 : DT == INFR_IQ1_M ? 56 : DT == INFR_IQ2_XXS ? 66
                                       : DT == INFR_IQ2_XS ? 74 : DT == INFR_IQ2_S ? 82 : DT == INFR_IQ3_XXS ? 98 : DT == INFR_IQ3_S ? 110 : 0;
    static constexpr int kWB = kBlockBytes * (256 / kBlock);   // bytes of one row in a window of 256 k
    static constexpr int kChunks = (kWB + 15) / 16;
    static constexpr int kPitch = 16 * (kChunks | 1);
    // every block format except Q8_0 (272-byte windows: two stages of four waves would not fit beside the
    // activation ring); unquantised rows are read in whole cache lines as they are
    static constexpr bool kOn = kBlockBytes != 0 && DT != INFR_Q8_0;
    static constexpr size_t kLds = kOn ? (size_t)4 * 2 * 64 * kPitch : 0;
};

template <int DT, bool DOWN, int M>
__device__ __forceinline__ void grouped_units_tile_staged(const GroupedParams& p, const Tile& t, int n0, uint8_t* lds,
                                                          const float* s_scale, uint8_t* wlds) {
    using W = StagedW<DT>;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, half = lane >> 5;
    float16v acc0[M], acc1[M];
#pragma unroll
    for (int i = 0; i < M; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc0[i][r] = acc1[i][r] = 0.0f;
    const int row_bytes = (p.K / W::kBlock) * W::kBlockBytes;
    // chunk i of the lane: row (64 i + lane) / kChunks of the wave's 64, 16-byte chunk (64 i + lane) % kChunks
    const uint8_t* csrc[W::kChunks];
    int cdst[W::kChunks], coff[W::kChunks];
#pragma unroll
    for (int i = 0; i < W::kChunks; i++) {
        const int idx = 64 * i + lane, r = idx / W::kChunks, ch = idx - r * W::kChunks;
        const uint8_t* row;
        if (DOWN) row = p.w0 + (size_t)t.e * p.w0_stride + (size_t)min(n0 + 64 * wave + r, p.N - 1) * row_bytes;
        else row = (r < 32 ? p.w0 + (size_t)t.e * p.w0_stride : p.w1 + (size_t)t.e * p.w1_stride) +
                   (size_t)min(n0 + 32 * wave + (r & 31), p.N - 1) * row_bytes;
        csrc[i] = row + 16 * ch;
        coff[i] = 16 * ch;
        cdst[i] = r * W::kPitch + 16 * ch;
    }
    uint8_t* const wbase = wlds + wave * (2 * 64 * W::kPitch);
    const uint8_t* const u0row = wbase + (lane & 31) * W::kPitch;
    const uint8_t* const u1row = u0row + 32 * W::kPitch;
    const uint8_t* asrc[4];
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const int tok = 32 * wave + 8 * q + (lane >> 3), kg = (lane & 7) ^ ((lane >> 3) & 7);
        const int pr = t.p0 + min(tok, t.cnt - 1);
        const size_t src_row = DOWN ? (size_t)pr : (size_t)(p.pair_src[pr] / p.n_used);
        asrc[q] = reinterpret_cast<const uint8_t*>(p.a + src_row * p.K) + 16 * kg;
    }
    uint8_t* const a_dst = lds + wave * 4096 + lane * 16;
    const int x7 = lane & 7;
    int a_off[4];
#pragma unroll
    for (int ks = 0; ks < 4; ks++) a_off[ks] = (lane & 31) * 128 + (((ks + 4 * half) ^ x7) * 16);

    const int n_slices = p.K / kSlice, n_win = (n_slices + 3) >> 2;
    uint4 wreg[W::kChunks];
    uint4 ar0, ar1, ar2, ar3;   // named, not an array: the array form ends up in scratch memory
    // a chunk that starts past the row's end (last window of a row that is no whole number of windows) is not read;
    // one that starts inside may run up to 15 bytes past it, which every buffer of the backend has room for
    auto request = [&](int g) {
        const int valid = row_bytes - g * W::kWB;
        const size_t o = (size_t)g * W::kWB;
        if (valid >= W::kWB) {   // uniform: only a row's last window can be short
#pragma unroll
            for (int i = 0; i < W::kChunks; i++) wreg[i] = ldu<uint4>(csrc[i] + o);
        } else {
#pragma unroll
            for (int i = 0; i < W::kChunks; i++) wreg[i] = ldu<uint4>(csrc[i] + o - (coff[i] < valid ? 0 : coff[i]));
        }
    };
    auto deposit = [&](int g) {
        uint8_t* d = wbase + (g & 1) * (64 * W::kPitch);
#pragma unroll
        for (int i = 0; i < W::kChunks; i++)
            *reinterpret_cast<uint4*>(d + cdst[i]) = wreg[i];
    };
    request(0);
    ar0 = *reinterpret_cast<const uint4*>(asrc[0]);
    ar1 = *reinterpret_cast<const uint4*>(asrc[1]);
    ar2 = *reinterpret_cast<const uint4*>(asrc[2]);
    ar3 = *reinterpret_cast<const uint4*>(asrc[3]);
    deposit(0);
    *reinterpret_cast<uint4*>(a_dst) = ar0;
    *reinterpret_cast<uint4*>(a_dst + 1024) = ar1;
    *reinterpret_cast<uint4*>(a_dst + 2048) = ar2;
    *reinterpret_cast<uint4*>(a_dst + 3072) = ar3;
    __syncthreads();
    WSlice<DT> u0, u1;
    u0.load(u0row, half);
    u1.load(u1row, half);
    for (int s = 0; s < n_slices; s++) {
        const bool more = s + 1 < n_slices;
        const int g = s >> 2, j = s & 3;
        WSlice<DT> v0, v1;
        if (j == 0 && g + 1 < n_win) request(g + 1);
        if (more) {
            const int so = (((s + 1) >> 2) & 1) * (64 * W::kPitch), ui = 2 * ((s + 1) & 3) + half;
            v0.load(u0row + so, ui);
            v1.load(u1row + so, ui);
            const size_t ao = (size_t)(s + 1) * 128;
            ar0 = *reinterpret_cast<const uint4*>(asrc[0] + ao);
            ar1 = *reinterpret_cast<const uint4*>(asrc[1] + ao);
            ar2 = *reinterpret_cast<const uint4*>(asrc[2] + ao);
            ar3 = *reinterpret_cast<const uint4*>(asrc[3] + ao);
        }
        const uint8_t* ap = lds + (s & 1) * kUStage;
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
            const half8 b0 = u0.frag(ks), b1 = u1.frag(ks);
#pragma unroll
            for (int mi = 0; mi < M; mi++) {
                const half8 a = *reinterpret_cast<const half8*>(ap + a_off[ks] + mi * 4096);
                acc0[mi] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b0, acc0[mi], 0, 0, 0);
                acc1[mi] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b1, acc1[mi], 0, 0, 0);
            }
        }
        // One wave per SIMD: the decode of the next fragments has to issue between this wave's own matrix
        // instructions, or the two pipes take turns.  Ask the scheduler for one MFMA, then a share of the VALU work.
#pragma unroll
        for (int i = 0; i < 8 * M; i++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x002, 256 / (8 * M), 0);
        }
        if (more) {
            uint8_t* d = a_dst + ((s + 1) & 1) * kUStage;
            *reinterpret_cast<uint4*>(d) = ar0;
            *reinterpret_cast<uint4*>(d + 1024) = ar1;
            *reinterpret_cast<uint4*>(d + 2048) = ar2;
            *reinterpret_cast<uint4*>(d + 3072) = ar3;
            u0 = v0;
            u1 = v1;
        }
        if (j == 2 && g + 1 < n_win) deposit(g + 1);
        __syncthreads();
    }
    tile_epilogue<DOWN, M>(p, t, n0, wave, lane, s_scale, acc0, acc1);
}

template <int DT, bool DOWN>
__global__ __launch_bounds__(256) void grouped_units_mfma(GroupedParams p) {
    __shared__ __attribute__((aligned(16))) uint8_t lds[2 * kUStage];
    __shared__ __attribute__((aligned(16))) float s_scale[kBM];
    const int tid = threadIdx.x, lane = tid & 63;
    Tile t;
    int nt;
    if (!find_item(p.offsets, p.n_expert, p.n_tiles_n, lane, t, nt)) return;
    constexpr int kBN = DOWN ? 256 : 128;
    if (tid < kBM) {
        const int pr = t.p0 + min(tid, t.cnt - 1);
        s_scale[tid] = p.a_scale[DOWN ? pr : p.pair_src[pr] / p.n_used];
    }
    if constexpr (StagedW<DT>::kOn) {
        extern __shared__ __attribute__((aligned(16))) uint8_t wlds[];
        switch ((t.cnt + 31) >> 5) {
            case 1: grouped_units_tile_staged<DT, DOWN, 1>(p, t, nt * kBN, lds, s_scale, wlds); break;
            case 2: grouped_units_tile_staged<DT, DOWN, 2>(p, t, nt * kBN, lds, s_scale, wlds); break;
            case 3: grouped_units_tile_staged<DT, DOWN, 3>(p, t, nt * kBN, lds, s_scale, wlds); break;
            default: grouped_units_tile_staged<DT, DOWN, 4>(p, t, nt * kBN, lds, s_scale, wlds); break;
        }
    } else {
        switch ((t.cnt + 31) >> 5) {
            case 1: grouped_units_tile<DT, DOWN, 1>(p, t, nt * kBN, lds, s_scale); break;
            case 2: grouped_units_tile<DT, DOWN, 2>(p, t, nt * kBN, lds, s_scale); break;
            case 3: grouped_units_tile<DT, DOWN, 3>(p, t, nt * kBN, lds, s_scale); break;
            default: grouped_units_tile<DT, DOWN, 4>(p, t, nt * kBN, lds, s_scale); break;
        }
    }
}

template <int DT, bool DOWN>
void grouped_units(hipStream_t s, const GroupedParams& p) {
    const int bn = DOWN ? 256 : 128;
    GroupedParams q = p;
    q.n_tiles_n = (p.N + bn - 1) / bn;
    const int max_tiles = p.n_pairs / kBM + (p.n_expert < p.n_pairs ? p.n_expert : p.n_pairs);
    static bool attr_set = false;
    if (!attr_set && StagedW<DT>::kLds) {
        (void)hipFuncSetAttribute((const void*)grouped_units_mfma<DT, DOWN>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                  (int)StagedW<DT>::kLds);
        attr_set = true;
    }
    INFR_LAUNCH((grouped_units_mfma<DT, DOWN>), dim3((unsigned)((max_tiles * q.n_tiles_n + 7) & ~7)), dim3(256), StagedW<DT>::kLds,
                s, q);
}

template <bool DOWN>
void grouped_units_any(hipStream_t s, int dt, const GroupedParams& p) {
    switch (dt) {
#define INFR_UNITS(D) case D: grouped_units<D, DOWN>(s, p); break;
        INFR_FOR_UNIT_FORMATS(INFR_UNITS)
        INFR_UNITS(INFR_F16) INFR_UNITS(INFR_BF16) INFR_UNITS(INFR_F32)
#undef INFR_UNITS
        default: break;
    }
}

}  // namespace

// The unit-decoder grouped GEMM: any affine format, contraction length a whole number of 64-k slices
// (and of the format's blocks).  Its activations come from launch_rows_to_f16 in natural k order (ask it
// for a format without an LDS layout of its own, e.g. INFR_Q5K).
bool grouped_units_supported(int dt, int k) {
    if (k <= 0 || k % kSlice != 0) return false;
    if (dt == INFR_F16 || dt == INFR_BF16 || dt == INFR_F32) return true;   // rounded to f16 (weights beyond 65504 would not fit)
    const int block = unit_format_block(dt);
    return block != 0 && k % block == 0;
}
void launch_grouped_units_gate_up(hipStream_t s, int dt, const GroupedParams& p) { grouped_units_any<false>(s, dt, p); }
void launch_grouped_units_down(hipStream_t s, int dt, const GroupedParams& p) { grouped_units_any<true>(s, dt, p); }

bool grouped_supported(int dt, int k) {
    // the k loop runs in groups of four 64-element slices (one K-quant super-block)
    if (k <= 0 || (k % (kSlice * 4)) != 0) return false;
    return dt == INFR_Q4K || dt == INFR_Q6K || dt == INFR_Q8_0;
}

void launch_rows_to_f16(hipStream_t s, int weight_dt, const float* src, int rows, int n, void* dst, float* scale) {
    if (rows <= 0) return;
    _Float16* d = reinterpret_cast<_Float16*>(dst);
    if (weight_dt == INFR_Q4K) rows_to_f16<MQ4K>(s, src, rows, n, d, scale);
    else if (weight_dt == INFR_Q6K) rows_to_f16<MQ6K>(s, src, rows, n, d, scale);
    else rows_to_f16<MQ80>(s, src, rows, n, d, scale);
}

void launch_bucket(hipStream_t s, const int32_t* ids, int n_pairs, int n_expert, int32_t* offsets, int32_t* pair_src,
                   int32_t* slot_pair) {
    INFR_LAUNCH(bucket_kernel, dim3(n_expert + 1), dim3(256), 0, s, ids, n_pairs, n_expert, offsets, pair_src, slot_pair);
}

void launch_grouped_gate_up(hipStream_t s, int dt, const GroupedParams& p) {
    if (dt == INFR_Q4K) grouped6<D4K, false>(s, p);
    else if (dt == INFR_Q6K) grouped6<D6K, false>(s, p);
    else grouped6<D80, false>(s, p);
}

void launch_grouped_down(hipStream_t s, int dt, const GroupedParams& p) {
    if (dt == INFR_Q4K) grouped6<D4K, true>(s, p);
    else if (dt == INFR_Q6K) grouped6<D6K, true>(s, p);
    else grouped6<D80, true>(s, p);
}

void launch_unbucket_combine(hipStream_t s, const void* y, const int32_t* slot_pair, const float* weights, int rows,
                             int ne, int n_used, int weight_before, float* dst, int identity, const float* pair_scale,
                             const float* addend, int skip_zero_w) {
    if (rows <= 0) return;
    const dim3 grid((ne + 1023) / 1024, rows), block(256);
    if (pair_scale && ne % 8 == 0 && (((uintptr_t)y | (uintptr_t)dst | (uintptr_t)addend) & 15) == 0 &&
        (n_used == 8 || n_used == 4 || n_used == 6 || n_used == 2)) {
        const dim3 g8((ne + 2047) / 2048, rows);
#define INFR_H8(KK)                                                                                                       \
    INFR_LAUNCH(unbucket_combine_h8_kernel<KK>, g8, block, 0, s, (const _Float16*)y, slot_pair, weights, ne, weight_before, \
                dst, identity, pair_scale, addend, skip_zero_w)
        if (n_used == 8) INFR_H8(8);
        else if (n_used == 6) INFR_H8(6);
        else if (n_used == 4) INFR_H8(4);
        else INFR_H8(2);
#undef INFR_H8
        return;
    }
    if (pair_scale)
        INFR_LAUNCH(unbucket_combine_kernel<_Float16>, grid, block, 0, s, (const _Float16*)y, slot_pair, weights, ne, n_used,
                    weight_before, dst, identity, pair_scale, addend, skip_zero_w);
    else
        INFR_LAUNCH(unbucket_combine_kernel<float>, grid, block, 0, s, (const float*)y, slot_pair, weights, ne, n_used,
                    weight_before, dst, identity, pair_scale, addend, skip_zero_w);
}

}  // namespace infr

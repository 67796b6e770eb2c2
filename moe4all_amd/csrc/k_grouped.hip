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
//                         magnitude fits), laid out in the k order the weight format unpacks to
//                         (route_rows_to_f16_kernel: the same for the token rows, with the row's routing).
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
#include "grouped_common.h"
#include "route.h"

namespace infr {

namespace {

// --------------------------------------------------------------------------------------------
// One block per row: amax -> power-of-two scale -> f16 in the virtual k order of format F.
template <class F>
__device__ __forceinline__ void row_to_f16(const float* __restrict__ src, int n, _Float16* __restrict__ dst,
                                           float* __restrict__ scale, size_t row, float* s_max) {
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

template <class F>
__global__ __launch_bounds__(256) void rows_to_f16_kernel(const float* __restrict__ src, int n,
                                                          _Float16* __restrict__ dst, float* __restrict__ scale) {
    __shared__ float s_max[4];
    row_to_f16<F>(src, n, dst, scale, blockIdx.x, s_max);
}

// The routing of token row b (route_kernel's work, on the block's first wavefront) behind the f16 conversion of the same
// row for the gate/up GEMM: both are per row and both precede the bucketing, and a launch of either alone is mostly its
// dispatch (32 to 2048 rows: 5.0-7.8 us and 3.9-4.7 us as two launches).
template <class F>
__global__ __launch_bounds__(256) void route_rows_to_f16_kernel(RouteParams rp, const float* __restrict__ src, int n,
                                                                _Float16* __restrict__ dst, float* __restrict__ scale) {
    extern __shared__ float lds[];
    __shared__ float s_max[4];
    uint64_t* tab = reinterpret_cast<uint64_t*>(lds);
    if (threadIdx.x < 32) tab[threadIdx.x] = kExp2Table[threadIdx.x];
    row_to_f16<F>(src, n, dst, scale, blockIdx.x, s_max);   // (its barrier also publishes the table)
    if (threadIdx.x < 64) route_row_any(rp, blockIdx.x, threadIdx.x, lds + 64, tab);
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

// --------------------------------------------------------------------------------------------
// Grouped GEMM: 512 threads = 8 waves, two per SIMD (256 registers each, 128 of them accumulators).  Waves p and
// p + 4 form a pair that owns two 32-feature column tiles (gate p / up p, or down 2p / 2p+1) against M 32-token row
// tiles; of every 64-k slice the first wave of the pair contracts k steps 0 and 1, the second k steps 2 and 3, each
// into accumulators of its own, and the two sets are added through LDS after the k loop.  A lane unpacks the quantised
// bytes of ITS weight row and k half in registers into exactly the operand fragments it feeds to the matrix instruction.
// M is a template parameter so that the k loop has no branches.  Every k-loop load goes straight from global memory
// into LDS
// (global_load_lds_dwordx4: lane i of a wave's load deposits its 16 bytes at base + 16 i), so that
// each load instruction covers whole cache lines and nothing is staged in registers:
//   * activation stage = the tile's 128 tokens x one 64-k slice (16 KB), token-major, the eight
//     16-byte chunks of a token rotated by rot7(token) so that the operand reads of 32 consecutive
//     tokens spread over all banks; every pair loads a quarter of it, kNA stages in the ring;
//   * weight stage = the parts of the 64 weight rows of ONE pair that a half super-block (128 k,
//     two slices) needs, row-major (Q4_K: header + 4 code chunks = 80 B per row; Q6_K: 4 low-code
//     chunks, 2 high-bit chunks, scales, tail = 128 B per row, chunks rotated by the row number);
//     private to the pair, 3 stages in the ring.
// The loads are issued from inline assembly, so the compiler neither counts them nor orders LDS
// reads against them: one explicit "s_waitcnt vmcnt(n); s_barrier" per slice does both.  The issue
// order is fixed (the same number of loads in every even and in every odd slice), so the number
// of loads younger than the ones slice s needs is a compile-time constant.
// M0 carries the LDS base of the transfer.  The statement writes M0 immediately before its only use, and nothing
// else in these kernels uses M0 (no other LDS-direct load, no indirect register addressing, no message), so no
// value of the compiler's can be live in it across the statement.  M0 cannot be named as a clobber: the compiler
// reserves the register and warns that it does not honour such a clobber.
#ifndef INFR_ABLATE
#define INFR_ABLATE 0
#endif
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

// Q4_K: a weight stage holds the whole 144-byte blocks of one 256-k step (four slices), nine 16-byte chunks per row in
// memory order: a wave-load then reads runs of 144 contiguous bytes (34 cycles of the address path against 59 for a
// header and 64 code bytes per row and half-step).  Row pitch 144 = 36 banks: sixteen rows, sixteen distinct bank groups.
struct D4K : MQ4K {
    static constexpr int kNC = 9, kRowStride = 144, kNA = 4, kStepBytes = 144;   // kStepBytes: a row's bytes per 256 k
    static constexpr int kStageSlices = 4, kNW = 2;   // slices per weight stage, stages in the ring
    static constexpr bool kApart = true;   // a slice is contracted one barrier after it is unpacked (needs a fourth activation stage)
    // chunk `64 j + lane` of a weight stage: which staged row and where in the super-block its 16 bytes start
    static __device__ __forceinline__ void lane_chunk(int j, int lane, int& row, int& off0, int& hoff) {
        const int c = 64 * j + lane;
        row = c / 9;
        off0 = 16 * (c - 9 * row);
        hoff = 0;
    }
    static __device__ __forceinline__ Blk read_blk(const uint8_t* st, int row, int) {
        return Blk{*reinterpret_cast<const uint4*>(st + row * kRowStride)};
    }
    static __device__ __forceinline__ Q read_q(const uint8_t* st, int row, int sl, int h) {   // sl: slice of the stage
        return Q{*reinterpret_cast<const uint4*>(st + row * kRowStride + 16 + 32 * sl + 16 * h)};
    }
};

struct D6K : MQ6K {
    static constexpr int kNC = 8, kRowStride = 128, kNA = 4, kStepBytes = 210;
    static constexpr int kStageSlices = 2, kNW = 3;
    static constexpr bool kApart = true;
    static __device__ __forceinline__ int pos(int row, int part) { return row * kRowStride + ((part + rot7(row)) & 7) * 16; }
    static __device__ __forceinline__ void lane_chunk(int j, int lane, int& row, int& off0, int& hoff) {
        row = 8 * j + (lane >> 3);
        const int part = ((lane & 7) - rot7(row)) & 7;   // 0..3 low codes, 4..5 high bits, 6 scales, 7 tail (d in its last 2 bytes)
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
    static constexpr int kStageSlices = 2, kNW = 3;
    static constexpr bool kApart = false;   // 108 KB of weight stages leave room for three activation stages only
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

constexpr int kAStage6 = kBM * 128;        // bytes per activation stage
template <class D>
constexpr size_t grouped6_lds() { return (size_t)D::kNA * kAStage6 + (size_t)4 * D::kNW * 64 * D::kRowStride; }   // Q6_K: all 160 KB
constexpr int kScaleAt6 = 8 * 16384;      // after the k loop: the pairs' hand-over area (16 KB per wave), then the tile's row scales

// Time stamps of every workgroup for a measurement build (-DINFR_GROUPED_TRACE with a buffer in GroupedParams::trace);
// compiled out otherwise.
#ifdef INFR_GROUPED_TRACE
#define GROUPED_STAMP(i)                                                                                \
    do {                                                                                                \
        if (threadIdx.x == 0 && p.trace) p.trace[(size_t)blockIdx.x * 32 + (i)] = wall_clock64();        \
    } while (0)
#define GROUPED_NOTE(i, v)                                                                              \
    do {                                                                                                \
        if (threadIdx.x == 0 && p.trace) p.trace[(size_t)blockIdx.x * 32 + (i)] = (v);                  \
    } while (0)
#else
#define GROUPED_STAMP(i) do { } while (0)
#define GROUPED_NOTE(i, v) do { } while (0)
#endif

// measurement variants (template parameter ABL; -DINFR_ABLATE=<bits> makes one the default of a probe build):
// bit 0 = weight loads re-read half-step 0, bit 1 = activation loads re-read slice 0,
// bit 2 = no unpacking (raw bytes as fragments), bit 3 = one vector instruction in place of each matrix instruction,
// bit 4 = no k-loop loads at all, bit 5 = no weight loads, bit 6 = no activation loads.  Results are wrong in every
// case; only the time is of interest.
template <class D, int ABL>
__device__ __forceinline__ uint4 chunk_of(const typename D::Blk& k, const typename D::Q& f, const typename D::Prep& c, int ks, int j4) {
    if (ABL & 4) {
        uint4 r = *reinterpret_cast<const uint4*>(&f);
        r.x += ks;
        return r;
    }
    return D::chunk(k, f, c, ks, j4);
}
template <int ABL>
__device__ __forceinline__ float16v mma(const uint4& a, const uint4& b, float16v acc) {
    if (ABL & 8) {
        acc[0] += __uint_as_float((a.x ^ b.x) & 0x3FFFFFFFu);
        acc[1] += __uint_as_float((a.w ^ b.w) & 0x3FFFFFFFu);
        return acc;
    }
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, a), __builtin_bit_cast(half8, b), acc, 0, 0, 0);
}

struct Grouped6Ctx {
    uint8_t* lds;             // [kNA activation stages][4 pairs x kNW weight stages]
    const uint8_t* asrc[4];   // the lane's activation chunks of slice 0: quarters 0..3 of the pair's 32 tokens
    int pair, lane, n0;
    Tile t;
};

// KH = which wave of the pair: it contracts k steps 2 KH and 2 KH + 1 of every slice and stores the accumulator
// registers 8 KH .. 8 KH + 7 of every tile.  The pair's loads are all issued by its first wave: a load instruction holds
// up the wave that issues it until the address unit has taken it (with rows of 80 to 144 bytes a wave-load touches 20
// to 30 cache lines), and the first wave, being the older one on its SIMD, is served first and has time to spare before
// every barrier.
template <class D, bool DOWN, int M, int KH, int ABL>
__device__ __forceinline__ void grouped6_tile(const GroupedParams& p, const Grouped6Ctx& c, const uint8_t* const (&wsrc)[D::kNC],
                                              const int (&whoff)[D::kNC]) {
    constexpr int NA = D::kNA, NC = D::kNC, NW = D::kNW;
    constexpr bool kWhole = D::kStageSlices == 4;   // a weight stage is a whole 256-k step
    // kApart: a wave unpacks slice s after barrier s and contracts it only after barrier s + 1, next to the unpacking of
    // slice s + 1, so that its matrix and vector instructions are independent and can be interleaved one to seven, and
    // the first k step's activation fragments are read from LDS a slice before they are used.  Activation stage s is
    // then still read after barrier s + 1, so loads run one slice less ahead (kAhead) and never target it.
    constexpr bool kLate = D::kApart;
    constexpr int kAhead = kLate ? NA - 2 : NA - 1;
    constexpr int kWStage = 64 * D::kRowStride;
    const int pair = c.pair, lane = c.lane, half = lane >> 5;
    float16v acc0[M], acc1[M];
#pragma unroll
    for (int i = 0; i < M; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc0[i][r] = acc1[i][r] = 0.0f;
    const int n_slices = p.K / kSlice, last = n_slices - 1, last_hs = (n_slices >> 1) - 1;
    const uint32_t lds0 = lds_address(c.lds);
    const uint32_t upair = __builtin_amdgcn_readfirstlane(pair);
    const uint32_t a_dst = lds0 + upair * 4096;                                   // + stage * kAStage6 + q * 1024
    const uint32_t w_dst = lds0 + NA * kAStage6 + upair * (NW * kWStage);         // + stage * kWStage + j * 1024
    const uint8_t* const w_lds = c.lds + NA * kAStage6 + pair * (NW * kWStage);
    // Loads the first wave issues while slice s is contracted, in two parts i = 0, 1.  Weight chunks: with half-step
    // stages, of half-step s/2 + NW - 1 the chunks that belong to the slice's parity (even s: chunks 0..(NC+1)/2-1, odd
    // s: the rest), every second one per part; with whole-step stages, during the first three slices of a step three
    // chunks each of the NEXT step (so the last of them is two slices old when that step begins, as kAhead assumes, and
    // the stage they go to was last read before this step's first barrier).  Then the activation quarters 2 i and
    // 2 i + 1 of slice s + kAhead.  The last load of a slice is an activation quarter.
    // A pair whose 32 tokens lie beyond the tile's rows (pair >= M) loads no activations: nothing reads them.
    constexpr int kWEven = (NC + 1) / 2;
    const int last_step = (n_slices >> 2) - 1;
    const bool loads_a = pair < M;
    auto issue_part = [&](int s, int j4, int i) {   // j4 = s & 3; j4 and i are constants where this is called
        if (KH == 1 || (ABL & 16)) return;
        if (kWhole) {
            const int t = (s >> 2) + 1, tc = min(t, last_step);
#pragma unroll
            for (int j = 0; j < NC; j++)
                if (j4 < 3 && j / 3 == j4 && ((j % 3) & 1) == i && !(ABL & 32))
#ifdef INFR_W_CONTIG
                    dma16(wsrc[j] + (size_t)tc * D::kStepBytes * p.N, w_dst + (uint32_t)(t % NW) * kWStage + j * 1024);
#else
                    dma16(wsrc[j] + ((ABL & 1) ? (size_t)0 : (size_t)tc * D::kStepBytes), w_dst + (uint32_t)(t % NW) * kWStage + j * 1024);
#endif
        } else {
            const int odd = j4 & 1, lo = odd ? kWEven : 0, hi = odd ? NC : kWEven;
            const int hs = (s >> 1) + NW - 1, hc = min(hs, last_hs);
#pragma unroll
            for (int j = 0; j < NC; j++)
                if (j >= lo && j < hi && ((j - lo) & 1) == i && hs >= 0 && !(ABL & 32))
                    dma16(wsrc[j] + ((ABL & 1) ? (size_t)0 : (size_t)(hc >> 1) * D::kStepBytes + ((hc & 1) ? whoff[j] : 0)),
                          w_dst + (uint32_t)(hs % NW) * kWStage + j * 1024);
        }
        const int sa = s + kAhead;
        if (sa >= 0 && loads_a && !(ABL & 64)) {
            const size_t ao = (ABL & 2) ? (size_t)0 : (size_t)min(sa, last) * 128;
            dma16(c.asrc[2 * i] + ao, a_dst + (uint32_t)(sa % NA) * kAStage6 + (2 * i) * 1024);
            dma16(c.asrc[2 * i + 1] + ao, a_dst + (uint32_t)(sa % NA) * kAStage6 + (2 * i + 1) * 1024);
        }
    };
#pragma unroll
    for (int s = -4; s < 0; s++)
#pragma unroll
        for (int i = 0; i < 2; i++) issue_part(s, s & 3, i);

    // operand reads: token 32 mi + (lane & 31), k chunk ks + 4 half, rotated by the token's number
    const int x7 = rot7(lane & 31);
    const int a_lane = (lane & 31) * 128;
    int a_off[2];
#pragma unroll
    for (int i = 0; i < 2; i++) a_off[i] = a_lane + (((2 * KH + i + 4 * half) ^ x7) * 16);
    const int row0 = lane & 31, row1 = 32 + (lane & 31);

#ifdef INFR_GROUPED_TRACE
    long long wait_loads = 0, wait_barrier = 0, issue_time = 0;
    const long long loop_in = clock64();
#endif
    // kLate: the wave's two k steps of the previous slice: first-step fragments a0 (read a slice earlier), second-step
    // fragments from the activation stage at ap
    auto contract = [&](const uint8_t* ap, const uint4 (&a0)[M], const uint4 (&b)[4]) {
        uint4 a1[M];
#pragma unroll
        for (int mi = 0; mi < M; mi++) a1[mi] = *reinterpret_cast<const uint4*>(ap + a_off[1] + mi * 4096);
#pragma unroll
        for (int mi = 0; mi < M; mi++) {
            acc0[mi] = mma<ABL>(a0[mi], b[0], acc0[mi]);
            acc1[mi] = mma<ABL>(a0[mi], b[1], acc1[mi]);
        }
#pragma unroll
        for (int mi = 0; mi < M; mi++) {
            acc0[mi] = mma<ABL>(a1[mi], b[2], acc0[mi]);
            acc1[mi] = mma<ABL>(a1[mi], b[3], acc1[mi]);
        }
    };
    uint4 afirst[M] = {};   // kLate: the first k step's activation fragments of the previous slice
    uint4 held[4] = {};     // kLate: the unpacked weight fragments of the previous slice (k step 2 KH: rows 0, 1; 2 KH + 1: rows 0, 1)
    // slice s (compile-time position j4 = s & 3 inside its super-block)
    auto slice = [&](int s, auto j4c) {
        constexpr int j4 = decltype(j4c)::value;
        // loads of the first wave younger than the last one this slice needs (an activation quarter of slice s, issued
        // at the end of slice s - kAhead): everything it issued during the kAhead - 1 slices since
        constexpr int kWOdd = NC - kWEven;
        constexpr int kYoungW = kWhole ? (j4 == 0 ? 0 : 3) : kAhead == 3 ? NC : ((j4 & 1) ? kWEven : kWOdd);   // weight loads among them
        constexpr int kYoung = KH == 1 ? 0 : kYoungW + 4 * (kAhead - 1);
        static_assert(kAhead == 2 || (kAhead == 3 && !kWhole), "the load counts above are written for these distances");
#ifdef INFR_GROUPED_TRACE
        const long long w_in = clock64();
        if (loads_a) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" : : "n"(kYoung) : "memory");
        else asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" : : "n"(KH == 1 ? 0 : kYoungW) : "memory");
        const long long w_mid = clock64();
        asm volatile("s_barrier" ::: "memory");
        wait_loads += w_mid - w_in;
        wait_barrier += clock64() - w_mid;
#else
        if (loads_a) wait_loads_then_barrier<kYoung>();
        else wait_loads_then_barrier<(KH == 1 ? 0 : kYoungW)>();
#endif
        const uint8_t* ap = c.lds + (s % NA) * kAStage6;
        const uint8_t* wst = w_lds + (kWhole ? (s >> 2) % NW : (s >> 1) % NW) * kWStage;
        if (kLate) {
            // all of the slice's loads first: what follows is one region for the instruction scheduler
#ifdef INFR_GROUPED_TRACE
            const long long i_in = clock64();
#endif
            issue_part(s, j4, 0);
            issue_part(s, j4, 1);
#ifdef INFR_GROUPED_TRACE
            issue_time += clock64() - i_in;
#endif
            if (s > 0) contract(c.lds + ((s - 1) % NA) * kAStage6, afirst, held);
        }
        const typename D::Blk k0 = D::read_blk(wst, row0, half), k1 = D::read_blk(wst, row1, half);
        const typename D::Q f0 = D::read_q(wst, row0, j4 % D::kStageSlices, half), f1 = D::read_q(wst, row1, j4 % D::kStageSlices, half);
        const typename D::Prep c0 = D::prep(k0, f0, j4, half), c1 = D::prep(k1, f1, j4, half);
        if (kLate) {
            held[0] = chunk_of<D, ABL>(k0, f0, c0, 2 * KH, j4);
            held[1] = chunk_of<D, ABL>(k1, f1, c1, 2 * KH, j4);
            held[2] = chunk_of<D, ABL>(k0, f0, c0, 2 * KH + 1, j4);
            held[3] = chunk_of<D, ABL>(k1, f1, c1, 2 * KH + 1, j4);
#pragma unroll
            for (int mi = 0; mi < M; mi++) afirst[mi] = *reinterpret_cast<const uint4*>(ap + a_off[0] + mi * 4096);
            // one matrix instruction, then a share of the vector work
#pragma unroll
            for (int i = 0; i < 4 * M; i++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x002, (112 + 4 * M - 1) / (4 * M), 0);
            }
        } else {
            uint4 a[M];
#pragma unroll
            for (int mi = 0; mi < M; mi++) a[mi] = *reinterpret_cast<const uint4*>(ap + a_off[0] + mi * 4096);
            uint4 b0 = chunk_of<D, ABL>(k0, f0, c0, 2 * KH, j4), b1 = chunk_of<D, ABL>(k1, f1, c1, 2 * KH, j4);
#pragma unroll
            for (int i = 0; i < 2; i++) {
                uint4 nb0 = b0, nb1 = b1;
                if (i < 1) {
                    nb0 = chunk_of<D, ABL>(k0, f0, c0, 2 * KH + 1, j4);
                    nb1 = chunk_of<D, ABL>(k1, f1, c1, 2 * KH + 1, j4);
                }
                issue_part(s, j4, i);
#pragma unroll
                for (int mi = 0; mi < M; mi++) {
                    acc0[mi] = mma<ABL>(a[mi], b0, acc0[mi]);
                    acc1[mi] = mma<ABL>(a[mi], b1, acc1[mi]);
                    if (i < 1) a[mi] = *reinterpret_cast<const uint4*>(ap + a_off[1] + mi * 4096);
                }
                b0 = nb0;
                b1 = nb1;
            }
        }
    };
    for (int s0 = 0; s0 < n_slices; s0 += 4) {
        slice(s0, std::integral_constant<int, 0>{});
        slice(s0 + 1, std::integral_constant<int, 1>{});
        slice(s0 + 2, std::integral_constant<int, 2>{});
        slice(s0 + 3, std::integral_constant<int, 3>{});
    }
    if (kLate) contract(c.lds + (last % NA) * kAStage6, afirst, held);
    // nothing may still be landing in LDS when the rings are reused below or the block ends
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    GROUPED_STAMP(3);
#ifdef INFR_GROUPED_TRACE
    GROUPED_NOTE(8, wait_loads);
    GROUPED_NOTE(9, wait_barrier);
    GROUPED_NOTE(10, clock64() - loop_in);
    GROUPED_NOTE(11, issue_time);
    if (lane == 0 && p.trace) {
        p.trace[(size_t)blockIdx.x * 32 + 16 + pair + 4 * KH] = wait_loads;
        p.trace[(size_t)blockIdx.x * 32 + 24 + pair + 4 * KH] = wait_barrier;
    }
#endif

    // The pair's two partial sums: each wave hands over the accumulator registers the other one stores (this wave keeps
    // registers 8 KH .. 8 KH + 7 of every tile) through the ring memory, 4 KB per row tile and wave, in one round.
    static_assert(grouped6_lds<D>() >= kScaleAt6 + kBM * 4, "hand-over area and row scales fit the rings");
    float* const s_scale = reinterpret_cast<float*>(c.lds + kScaleAt6);
    uint8_t* const mine = c.lds + (size_t)(pair + 4 * KH) * 16384 + lane * 16;
    const uint8_t* const theirs = c.lds + (size_t)(pair + 4 * (1 - KH)) * 16384 + lane * 16;
    __syncthreads();   // the rings have been read by everyone
    if (KH == 0 && lane < 32) {   // the tile's row scales for the epilogue
        const int pr = c.t.p0 + min(32 * pair + lane, c.t.cnt - 1);
        s_scale[32 * pair + lane] = p.a_scale[DOWN ? pr : p.pair_src[pr] / p.n_used];
    }
#pragma unroll
    for (int mi = 0; mi < M; mi++) {
        constexpr int o = 8 * (1 - KH);
        *reinterpret_cast<float4*>(mine + (4 * mi + 0) * 1024) = make_float4(acc0[mi][o], acc0[mi][o + 1], acc0[mi][o + 2], acc0[mi][o + 3]);
        *reinterpret_cast<float4*>(mine + (4 * mi + 1) * 1024) = make_float4(acc0[mi][o + 4], acc0[mi][o + 5], acc0[mi][o + 6], acc0[mi][o + 7]);
        *reinterpret_cast<float4*>(mine + (4 * mi + 2) * 1024) = make_float4(acc1[mi][o], acc1[mi][o + 1], acc1[mi][o + 2], acc1[mi][o + 3]);
        *reinterpret_cast<float4*>(mine + (4 * mi + 3) * 1024) = make_float4(acc1[mi][o + 4], acc1[mi][o + 5], acc1[mi][o + 6], acc1[mi][o + 7]);
    }
    __syncthreads();
#pragma unroll
    for (int mi = 0; mi < M; mi++) {
        constexpr int o = 8 * KH;
        const float4 v0 = *reinterpret_cast<const float4*>(theirs + (4 * mi + 0) * 1024), v1 = *reinterpret_cast<const float4*>(theirs + (4 * mi + 1) * 1024);
        const float4 v2 = *reinterpret_cast<const float4*>(theirs + (4 * mi + 2) * 1024), v3 = *reinterpret_cast<const float4*>(theirs + (4 * mi + 3) * 1024);
        // first wave's part + second wave's part, whichever of the two this is
        const float t0[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w}, t1[8] = {v2.x, v2.y, v2.z, v2.w, v3.x, v3.y, v3.z, v3.w};
#pragma unroll
        for (int r = 0; r < 8; r++) {
            acc0[mi][o + r] = KH ? t0[r] + acc0[mi][o + r] : acc0[mi][o + r] + t0[r];
            acc1[mi][o + r] = KH ? t1[r] + acc1[mi][o + r] : acc1[mi][o + r] + t1[r];
        }
    }
    GROUPED_STAMP(4);
    tile_epilogue<DOWN, M, 2 * KH, 2 * KH + 2>(p, c.t, c.n0, pair, lane, s_scale, acc0, acc1);
    GROUPED_STAMP(5);
}

// ABL: measurement variants (see chunk_of); 0 in the product path
template <class D, bool DOWN, int ABL = INFR_ABLATE>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void grouped_mfma6(GroupedParams p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds6[];
    Grouped6Ctx c;
    c.lds = lds6;
    const int tid = threadIdx.x;
    const int kh = tid >> 8;
    c.pair = (tid >> 6) & 3;
    c.lane = tid & 63;
    int nt;
    GROUPED_STAMP(0);
    if (!find_item(p.offsets, p.n_expert, p.n_tiles_n, c.lane, c.t, nt)) return;
    const Tile& t = c.t;
    GROUPED_STAMP(1);
    GROUPED_NOTE(7, (long long)t.cnt);
    constexpr int kBN = DOWN ? 256 : 128;
    c.n0 = nt * kBN;
    // sources of the lane's chunks of the pair's weight stage (half-step 0)
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
            f = c.n0 + 64 * c.pair + row;
        } else {
            base = row < 32 ? p.w0 + (size_t)t.e * p.w0_stride : p.w1 + (size_t)t.e * p.w1_stride;
            f = c.n0 + 32 * c.pair + (row & 31);
        }
#ifdef INFR_W_CONTIG   // measurement builds: banks laid out [step][row][block] (timing only, the data is not re-laid)
        wsrc[j] = base + (size_t)min(f, p.N - 1) * D::kStepBytes + off0;
#else
        wsrc[j] = base + (size_t)min(f, p.N - 1) * row_bytes + off0;
#endif
    }
    // the lane's activation chunks: token 32 pair + 8 q + lane / 8, chunk (lane & 7) ^ rot7(token)
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const int tok = 32 * c.pair + 8 * q + (c.lane >> 3), kg = (c.lane & 7) ^ rot7(tok);
        const int pr = t.p0 + min(tok, t.cnt - 1);
        const size_t src_row = DOWN ? (size_t)pr : (size_t)(p.pair_src[pr] / p.n_used);
        c.asrc[q] = reinterpret_cast<const uint8_t*>(p.a + src_row * p.K) + 16 * kg;
    }
    const int m = (t.cnt + 31) >> 5;
    GROUPED_STAMP(2);
#define INFR_TILE(MM)                                                     \
    if (kh) grouped6_tile<D, DOWN, MM, 1, ABL>(p, c, wsrc, whoff);        \
    else grouped6_tile<D, DOWN, MM, 0, ABL>(p, c, wsrc, whoff)
    if (m == 1) { INFR_TILE(1); }
    else if (m == 2) { INFR_TILE(2); }
    else if (m == 3) { INFR_TILE(3); }
    else { INFR_TILE(4); }
#undef INFR_TILE
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
    const dim3 grid((unsigned)((max_tiles * q.n_tiles_n + 7) & ~7));   // whole rounds of the 8 XCDs
    INFR_LDS_LIMIT((grouped_mfma6<D, DOWN>), (int)grouped6_lds<D>());
    INFR_LDS_LIMIT((grouped_mfma6<D, DOWN, 12>), (int)grouped6_lds<D>());
    // loads_only: the measurement variant without unpacking and matrix instructions (its output is meaningless)
    if (p.loads_only) INFR_LAUNCH((grouped_mfma6<D, DOWN, 12>), grid, dim3(512), grouped6_lds<D>(), s, q);
    else INFR_LAUNCH((grouped_mfma6<D, DOWN>), grid, dim3(512), grouped6_lds<D>(), s, q);
}

}  // namespace

bool grouped_supported(int dt, int k) {
    // the k loop runs in groups of four 64-element slices (one K-quant super-block)
    if (k <= 0 || (k % (kSlice * 4)) != 0) return false;
    return dt == INFR_Q4K || dt == INFR_Q6K || dt == INFR_Q8_0;
}

void launch_route_rows_to_f16(hipStream_t s, const RouteParams& rp, int weight_dt, const float* src, int n, void* dst, float* scale) {
    if (rp.rows <= 0) return;
    _Float16* d = reinterpret_cast<_Float16*>(dst);
    const size_t lds = (64 + route_scratch_floats(rp.n_expert, rp.n_groups)) * sizeof(float);
    if (weight_dt == INFR_Q4K) INFR_LAUNCH(route_rows_to_f16_kernel<MQ4K>, dim3(rp.rows), dim3(256), lds, s, rp, src, n, d, scale);
    else if (weight_dt == INFR_Q6K) INFR_LAUNCH(route_rows_to_f16_kernel<MQ6K>, dim3(rp.rows), dim3(256), lds, s, rp, src, n, d, scale);
    else INFR_LAUNCH(route_rows_to_f16_kernel<MQ80>, dim3(rp.rows), dim3(256), lds, s, rp, src, n, d, scale);
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
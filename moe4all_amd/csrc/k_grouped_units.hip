// Batched Op::MoeFfn and large Linear ops for every affine weight format: the grouped GEMM on the matrix cores with the
// weight operand decoded by the 32-element unit decoder (units.h).  Bucketing, activation conversion and the combine are
// in k_grouped.hip.
#include "grouped_common.h"
#include "units.h"

namespace infr {

namespace {

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
        const int tok = 32 * wave + 8 * q + (lane >> 3), kg = (lane & 7) ^ rot7(tok);
        const int pr = t.p0 + min(tok, t.cnt - 1);
        const size_t src_row = DOWN ? (size_t)pr : (size_t)(p.pair_src[pr] / p.n_used);
        asrc[q] = reinterpret_cast<const uint8_t*>(p.a + src_row * p.K) + 16 * kg;
    }
    uint8_t* const a_dst = lds + wave * 4096 + lane * 16;   // + stage * kUStage + q * 1024
    const int x7 = rot7(lane & 31);
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
        const int tok = 32 * wave + 8 * q + (lane >> 3), kg = (lane & 7) ^ rot7(tok);
        const int pr = t.p0 + min(tok, t.cnt - 1);
        const size_t src_row = DOWN ? (size_t)pr : (size_t)(p.pair_src[pr] / p.n_used);
        asrc[q] = reinterpret_cast<const uint8_t*>(p.a + src_row * p.K) + 16 * kg;
    }
    uint8_t* const a_dst = lds + wave * 4096 + lane * 16;
    const int x7 = rot7(lane & 31);
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
    if (StagedW<DT>::kLds) INFR_LDS_LIMIT((grouped_units_mfma<DT, DOWN>), (int)StagedW<DT>::kLds);
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

}  // namespace infr

// Router: logits = router . x with the reference's exact f32 accumulation order, then
// gating -> top-k -> renormalised routing weights, one wavefront per token row.
//
// The selected expert ids are an integer contract, so everything that feeds the comparison
// is computed in the reference's operation order: 8 independent FMA chains over
// i = j (mod 8), chains summed 0..7 (crates/infr-cpu/src/kernels.rs:6568-6583), softmax as
// exp(l - max) / sequential sum (crates/infr-cpu/src/lib.rs:3747-3756), selection by
// (probability descending, id ascending) = Rust's stable sort (lib.rs:3847-3850).
//
// The per-row routing itself lives in route.h; the decode GEMV kernel compiles it in as well,
// so that every block routes its own token row and no separate launch is needed there.
#include "device_common.h"
#include "kernels.h"
#include "route.h"

// Time stamps of every block for a measurement build; compiled out in the library.
#ifdef INFR_GEMV_TRACE
namespace infr { __device__ long long* g_logits_trace; }
#define LOGITS_STAMP(i)                                                                                                \
    do {                                                                                                               \
        if (threadIdx.x == 0 && infr::g_logits_trace) {                                                                \
            long long* rec_ = infr::g_logits_trace + ((size_t)blockIdx.y * gridDim.x + blockIdx.x) * 16;               \
            rec_[i] = wall_clock64();                                                                                  \
            rec_[8 + (i)] = clock64();   /* the shader clock beside the 100 MHz wall clock */                          \
        }                                                                                                              \
    } while (0)
#else
#define LOGITS_STAMP(i) do { } while (0)
#endif

namespace infr {

// One wavefront per token row (n_used <= 64, n_expert <= 2048).
__global__ __launch_bounds__(64) void route_kernel(RouteParams p) {
    extern __shared__ float lds[];
    uint64_t* tab = reinterpret_cast<uint64_t*>(lds);
    if (threadIdx.x < 32) tab[threadIdx.x] = kExp2Table[threadIdx.x];
    __syncthreads();
    route_row_any(p, blockIdx.x, threadIdx.x, lds + 64, tab);
}

static size_t route_lds_bytes(const RouteParams& p) {
    return (64 + (size_t)2 * p.n_expert + (size_t)(p.n_groups > 0 ? p.n_groups : 0)) * sizeof(float);
}

void launch_route(hipStream_t s, const RouteParams& p) {
    INFR_LAUNCH(route_kernel, dim3(p.rows), dim3(64), route_lds_bytes(p), s, p);
}

// ---------------------------------------------------------------------------------------------
// Logits.  Block = 256 threads, EPB experts per block, rpb token rows per pass
// (EPB*8*rpb <= 256).  The router rows and the activation rows are staged in LDS TRANSPOSED:
// chain j of a row holds elements j, j+8, j+16, ... contiguously, so a chain thread streams
// its operands with 128-bit LDS reads.  Strides are padded so the 16 lanes of a read phase
// (2 experts x 8 chains) hit disjoint banks.
// XQ: 128-bit loads of activations a thread holds in the one-burst staging (4: up to 1024 per block; 16: four rows of
// 4096 elements, for small batches of a wide model, whose blocks would otherwise take one token row each and read the
// router rows once per token row).
template <int EPB, int XQ = 4>
__global__ __launch_bounds__(256) void router_logits_kernel(const uint8_t* __restrict__ router, int rdt,
                                                            size_t row_bytes, const float* __restrict__ x, int ne,
                                                            int n_expert, int rows, int rpb,
                                                            float* __restrict__ logits, RouterNorm nrm) {
    extern __shared__ float lds[];
    __shared__ float red[4];
    const int nc = ne >> 3;                 // full chunks of 8
    const int ntail = ne & 7;
    const int jstride = ((nc + 63) & ~63) + 4;
    const int estride = 8 * jstride;        // = 32 (mod 64) banks
    float* w = lds;                         // [EPB][8][jstride]
    float* wt = w + EPB * estride;          // [EPB][8] tail elements
    float* xs = wt + EPB * 8;               // [rpb][8][jstride]
    float* xt = xs + rpb * estride;         // [rpb][8]
    const int tid = threadIdx.x;
    const int e0 = blockIdx.x * EPB;

    // Decode-sized launch (one pass over <= 2 token rows, f32 router): every global load of the
    // block, activations included, is issued before the first LDS store, so the block pays the
    // memory latency once.
    LOGITS_STAMP(0);
    const int nv = ne >> 2;
    const int rbase = blockIdx.y * rpb;   // first token row of this block's (only) pass when one_shot
    const bool one_shot = rdt == INFR_F32 && (ne & 3) == 0 && (int)gridDim.y * rpb >= rows && EPB * nv <= 8 * 256 &&
                          rpb * nv <= XQ * 256;
    if (one_shot) {
        float4 wr[8], xr[XQ], nw[4];
#pragma unroll
        for (int i = 0; i < XQ; i++) {
            const int idx = tid + 256 * i, rr = idx / nv, v = idx - rr * nv;
            xr[i] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (rr < rpb && rbase + rr < rows) xr[i] = reinterpret_cast<const float4*>(x + (size_t)(rbase + rr) * ne)[v];
        }
        if (nrm.weight) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int idx = tid + 256 * i;
                nw[i] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (idx < nv) nw[i] = reinterpret_cast<const float4*>(nrm.weight)[idx];
            }
        }
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int idx = tid + 256 * i, e = idx / nv, v = idx - e * nv;
            wr[i] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (e < EPB && e0 + e < n_expert)
                wr[i] = reinterpret_cast<const float4*>(router + (size_t)(e0 + e) * row_bytes)[v];
        }
        if (nrm.weight) {
            // The single token row arrives raw: Op::RmsNorm is applied while it is staged, with the
            // summation tree of the standalone kernel, and the first block stores the normalised row.
            float part = 0.0f;
#pragma unroll
            for (int i = 0; i < 4; i++)
                if (tid + 256 * i < nv) part = sumsq4(part, xr[i]);
            LOGITS_STAMP(1);
            const float sc = rms_scale(block256_sum(part, red), ne, nrm.eps);
            LOGITS_STAMP(2);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int idx = tid + 256 * i;
                if (idx >= nv) continue;
                xr[i] = rms_apply4(xr[i], sc, nw[i]);
                if (blockIdx.x == 0 && blockIdx.y == 0) reinterpret_cast<float4*>(nrm.xn_out)[idx] = xr[i];
            }
        }
        // element 4v + t of a row: chain (4v + t) & 7 = 4 (v & 1) + t, step (4v + t) >> 3 = v >> 1: the four
        // elements of a 128-bit load go to four chains at one step, or all four to the tail
#pragma unroll
        for (int i = 0; i < XQ; i++) {
            const int idx = tid + 256 * i, rr = idx / nv, v = idx - rr * nv;
            if (rr >= rpb) continue;
            if ((v >> 1) < nc) {
                float* d = xs + rr * estride + 4 * (v & 1) * jstride + (v >> 1);
                d[0] = xr[i].x; d[jstride] = xr[i].y; d[2 * jstride] = xr[i].z; d[3 * jstride] = xr[i].w;
            } else {
                float* d = xt + rr * 8;
                d[0] = xr[i].x; d[1] = xr[i].y; d[2] = xr[i].z; d[3] = xr[i].w;
            }
        }
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int idx = tid + 256 * i, e = idx / nv, v = idx - e * nv;
            if (e >= EPB) continue;
            if ((v >> 1) < nc) {
                float* d = w + e * estride + 4 * (v & 1) * jstride + (v >> 1);
                d[0] = wr[i].x; d[jstride] = wr[i].y; d[2 * jstride] = wr[i].z; d[3 * jstride] = wr[i].w;
            } else {
                float* d = wt + e * 8;
                d[0] = wr[i].x; d[1] = wr[i].y; d[2] = wr[i].z; d[3] = wr[i].w;
            }
        }
    } else if (rdt == INFR_F32 && (ne & 3) == 0) {
        for (int idx = tid; idx < EPB * nv; idx += 256) {
            int e = idx / nv, v = idx - e * nv;
            float4 f = make_float4(0.f, 0.f, 0.f, 0.f);
            if (e0 + e < n_expert) f = reinterpret_cast<const float4*>(router + (size_t)(e0 + e) * row_bytes)[v];
            const float fv[4] = {f.x, f.y, f.z, f.w};
#pragma unroll
            for (int q = 0; q < 4; q++) {
                int k = 4 * v + q, c = k >> 3, j = k & 7;
                if (c < nc) w[e * estride + j * jstride + c] = fv[q];
                else wt[e * 8 + j] = fv[q];
            }
        }
    } else {
        for (int idx = tid; idx < EPB * ne; idx += 256) {
            int e = idx / ne, k = idx - e * ne;
            float v = 0.0f;
            if (e0 + e < n_expert) v = decode_elem(rdt, router + (size_t)(e0 + e) * row_bytes, (uint32_t)k);
            int c = k >> 3, j = k & 7;
            if (c < nc) w[e * estride + j * jstride + c] = v;
            else wt[e * 8 + j] = v;
        }
    }
    LOGITS_STAMP(3);
    const int rsub = tid / (EPB * 8);
    const int e = (tid >> 3) % EPB;
    const int j = tid & 7;
    const int lane = tid & 63;
    for (int r0 = blockIdx.y * rpb; r0 < rows; r0 += gridDim.y * rpb) {
        if (!one_shot) __syncthreads();
        for (int rr = 0; rr < (one_shot ? 0 : rpb); rr++) {
            const bool row_ok = r0 + rr < rows;
            const float* xr = x + (size_t)(row_ok ? r0 + rr : 0) * ne;
            for (int k = tid; k < ne; k += 256) {
                float v = row_ok ? xr[k] : 0.0f;
                int c = k >> 3, jj = k & 7;
                if (c < nc) xs[rr * estride + jj * jstride + c] = v;
                else xt[rr * 8 + jj] = v;
            }
        }
        __syncthreads();
        LOGITS_STAMP(4);
        float acc = 0.0f;
        const bool live = rsub < rpb;
        const float* wp = w + e * estride + j * jstride;
        const float* xp = xs + (live ? rsub : 0) * estride + j * jstride;
        if (live) {
            int c = 0;
#pragma unroll 8
            for (; c + 4 <= nc; c += 4) {
                float4 a = *reinterpret_cast<const float4*>(wp + c);
                float4 b = *reinterpret_cast<const float4*>(xp + c);
                acc = __fmaf_rn(a.x, b.x, acc);
                acc = __fmaf_rn(a.y, b.y, acc);
                acc = __fmaf_rn(a.z, b.z, acc);
                acc = __fmaf_rn(a.w, b.w, acc);
            }
            for (; c < nc; c++) acc = __fmaf_rn(wp[c], xp[c], acc);
        }
        LOGITS_STAMP(5);
        float s = 0.0f;
#pragma unroll
        for (int jj = 0; jj < 8; jj++) s = __fadd_rn(s, __shfl(acc, (lane & ~7) + jj, kWave));
        if (live && j == 0) {
            for (int t = 0; t < ntail; t++) s = __fmaf_rn(wt[e * 8 + t], xt[rsub * 8 + t], s);
            if (r0 + rsub < rows && e0 + e < n_expert) logits[(size_t)(r0 + rsub) * n_expert + e0 + e] = s;
        }
        LOGITS_STAMP(6);
    }
}

// ---------------------------------------------------------------------------------------------
// Logits for a batch on the matrix cores.  v_mfma_f32_16x16x1_4b_f32 computes D_b[i][j] = A_b[i] * B_b[j] + C_b[i][j]
// for four independent 16 x 16 blocks b: with one k per instruction every element is ONE fused multiply-add, so a
// chain of them over k = 8 s + c, s ascending, is the reference's chain c term by term (the same bits as __fmaf_rn;
// the parity tests compare them with the scalar restatement bit for bit).  A block b holds one chain, so two
// instructions per step cover the eight chains of a 16 (token) x 16 (expert) tile, and the two accumulator sets are
// independent, which keeps the pipe busy from one wavefront.
// Workgroup (the 2 x 2 form) = 32 tokens x 32 experts = 8 wavefronts, two per SIMD: wavefronts 0-3 contract (each a
// 16 x 16 tile), wavefronts 4-7 only move data, so that no load, LDS store or address arithmetic sits between two
// matrix instructions of a contracting wavefront.  Operands are staged per 128-k chunk transposed in LDS (layout below: reads
// and stores free of bank conflicts), double-buffered, one barrier per chunk.  A contracting
// wavefront passes the barrier in the MIDDLE of a chunk's matrix instructions and reads the next chunk's first half
// behind it, beside the second half of its instructions, so neither the barrier nor the LDS latency empties the pipe.
// The moving wavefronts load four chunks ahead in registers.
// Lane l supplies A = x[token l % 16][chain l / 16], B = w[expert l % 16][chain l / 16]; it receives, in register
// 4 b + i, the element (token 4 (l / 16) + i, expert l % 16) of chain b, so the sum over the chains is lane-local.
// Workgroups that share a token tile (one per expert tile) are given indices 8 apart: they run on one XCD and the
// tile's activations come through one L2.
// (The vector-ALU kernel this replaced, 16 x 16 tiles with a 2 x 2 patch of chain accumulators per thread, took 13-14 us
// for 32 to 512 rows x 128 experts x 2048 where the 1 x 1 form takes 10, and 28-30 us for 2048 rows where the 2 x 2
// form takes 17.)
constexpr int kLmChunk = 128;
// LDS layout of a chunk: 1 KB blocks [16-row tile: the router's, then the activations'][accumulator set][four steps], inside a block
// [chain of the set][row][step]: a contracting wavefront's 128-bit read of a block and a moving wavefront's 32-bit store
// into it are both 64 consecutive lanes on consecutive addresses.
constexpr int kLmBlock = 256;                                          // floats of a block
template <int TW, int EW>
constexpr int lm_buffer() { return (TW + EW) * 8 * kLmBlock; }          // floats of one chunk of both operands
template <int TW, int EW>
constexpr size_t lm_lds_bytes() { return (size_t)2 * lm_buffer<TW, EW>() * sizeof(float); }   // two buffers
typedef float lm_acc_t __attribute__((ext_vector_type(16)));
template <int NS>
struct LmHalf { float4 w[2][NS], x[2][NS]; };   // operands of half a chunk: [four steps][accumulator set]
// TW x EW: the workgroup's 16 x 16 tiles along the tokens and along the experts, one contracting wavefront each, and
// one moving wavefront per 16 rows of either operand: 2 x 2 (eight wavefronts) for batches that give every compute unit
// such a workgroup, 1 x 1 for smaller ones.  SPLIT: two contracting wavefronts per tile, one accumulator set (four chains)
// each; a small batch's time is the chain of dependent matrix instructions, 256 steps at hidden size 2048, and two
// instructions per step on one wavefront take twice as long as one on each of two.  The second wavefront hands its
// four chain sums over through LDS at the end; the order of the sum over the chains stays 0..7.
template <int TW, int EW, int SPLIT>
__global__ __launch_bounds__(64 * (TW * EW * (SPLIT ? 2 : 1) + TW + EW)) void router_logits_mfma_kernel(const float* __restrict__ router, size_t row_floats,
                                                                                        const float* __restrict__ x, int ne, int n_expert,
                                                                                        int rows, float* __restrict__ logits) {
    extern __shared__ float lm_lds[];
    constexpr int kLmBuffer = lm_buffer<TW, EW>(), NT = TW * EW, NC = NT * (SPLIT ? 2 : 1), NS = SPLIT ? 1 : 2;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int neb = (n_expert + 16 * EW - 1) / (16 * EW), bq = blockIdx.x >> 3;
    const int e0 = (bq % neb) * 16 * EW, r0 = ((bq / neb) * 8 + (blockIdx.x & 7)) * 16 * TW;
    if (r0 >= rows) return;
    const int nfast = (ne / kLmChunk) & ~3;   // whole chunks that run through the pipelines below, four per trip
    if (wave >= NC) {
        // ---- the moving wavefronts: the first EW of them move the router's 16-row tiles, the others the activations'.  Lane
        // (row, step) = (lane / 4, lane % 4) of a wavefront loads, for q = 4 s + c, the four chains of accumulator set s
        // at step 4 c + step of its row: chunk elements 32 c + 8 step + 4 s .. + 3, a 128-bit load; component t of it
        // goes to block (tile, s, c), place 64 t + lane.  Rows past the end repeat the last one (their results are never
        // stored), and so do loads past the end of a row (those steps are never contracted).
        const int pw = wave - NC, is_x = pw >= EW ? 1 : 0, tile = is_x ? pw - EW : pw;
        const int grow = min((is_x ? r0 : e0) + 16 * tile + (lane >> 2), (is_x ? rows : n_expert) - 1);
        const float* src = is_x ? x + (size_t)grow * ne : router + (size_t)grow * row_floats;
        const int koff = 8 * (lane & 3);
        const int dst0 = pw * 8 * kLmBlock + lane;
        auto fetch = [&](float4 (&st)[8], int k0) __attribute__((always_inline)) {
#pragma unroll
            for (int q = 0; q < 8; q++)
                st[q] = *reinterpret_cast<const float4*>(src + min(k0 + 32 * (q & 3) + koff + 4 * (q >> 2), ne - 4));
        };
        // whole chunks need no clamp: one address per lane and chunk, the eight loads at constant offsets from it
        auto fetch_whole = [&](float4 (&st)[8], int k0) __attribute__((always_inline)) {
            const float* at = src + koff + k0;
#pragma unroll
            for (int q = 0; q < 8; q++) st[q] = *reinterpret_cast<const float4*>(at + 32 * (q & 3) + 4 * (q >> 2));
        };
        auto deposit = [&](const float4 (&st)[8], int buf) __attribute__((always_inline)) {
#pragma unroll
            for (int q = 0; q < 8; q++) {
                float* d = lm_lds + buf * kLmBuffer + dst0 + q * kLmBlock;   // block (tile, s, c): q = 4 s + c
                d[0] = st[q].x;
                d[64] = st[q].y;
                d[128] = st[q].z;
                d[192] = st[q].w;
            }
        };
        if (nfast > 0) {
            // chunk c is loaded into register set c % 4 and deposited into LDS buffer c % 2 while chunk c - 1 is contracted
            // (one basic block per trip, its order pinned: the compiler otherwise sinks the loads to their deposits)
            float4 s0[8], s1[8], s2[8], s3[8];
            auto step = [&](int c, float4 (&s_free)[8], const float4 (&s_next)[8], int buf) __attribute__((always_inline)) {
                fetch_whole(s_free, min(c + 4, nfast - 1) * kLmChunk);
                __builtin_amdgcn_sched_barrier(0);
                deposit(s_next, buf ^ 1);   // past the last chunk: a repeat of it that nobody contracts
                __builtin_amdgcn_sched_barrier(0);
                __syncthreads();
                __builtin_amdgcn_sched_barrier(0);
            };
            __builtin_amdgcn_s_setprio(3);   // requests ahead of the contracting wavefronts' instructions: 17.4 -> 16.9 us
            fetch_whole(s0, 0);
            fetch_whole(s1, kLmChunk);
            fetch_whole(s2, 2 * kLmChunk);
            fetch_whole(s3, 3 * kLmChunk);
            deposit(s0, 0);
            __syncthreads();
            for (int c = 0; c < nfast; c += 4) {
                step(c, s0, s1, 0);
                step(c + 1, s1, s2, 1);
                step(c + 2, s2, s3, 0);
                step(c + 3, s3, s0, 1);
            }
        }
        for (int k0 = nfast * kLmChunk; k0 < ne; k0 += kLmChunk) {   // up to three whole chunks and a shorter one
            float4 st[8];
            fetch(st, k0);
            __syncthreads();
            deposit(st, 0);
            __syncthreads();
        }
        return;
    }
    // ---- the contracting wavefronts
    const int cw = wave % NT, set0 = wave / NT;   // (set0: the accumulator set of a wavefront that has one)
    const int tw = cw % TW, ew = cw / TW;   // the wavefront's 16 x 16 tile of the workgroup's
    // the lane's operands of accumulator set s: chain 4 s + lane / 16, row lane % 16 of the wavefront's tile
    const int wo = ew * 8 * kLmBlock + 4 * lane;
    const int xo = (EW + tw) * 8 * kLmBlock + 4 * lane;
    auto read_half = [&](LmHalf<NS>& o, int buf, int half) __attribute__((always_inline)) {
        const float* base = lm_lds + buf * kLmBuffer + 2 * half * kLmBlock;
#pragma unroll
        for (int c = 0; c < 2; c++)
#pragma unroll
            for (int s = 0; s < NS; s++) {
                o.w[c][s] = *reinterpret_cast<const float4*>(base + wo + (4 * (set0 + s) + c) * kLmBlock);
                o.x[c][s] = *reinterpret_cast<const float4*>(base + xo + (4 * (set0 + s) + c) * kLmBlock);
            }
    };
    lm_acc_t acc[NS];
#pragma unroll
    for (int s = 0; s < NS; s++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[s][i] = 0.0f;
    auto contract4 = [&](const LmHalf<NS>& o, int c) __attribute__((always_inline)) {   // four steps of the wavefront's sets
#pragma unroll
        for (int s = 0; s < NS; s++) acc[s] = __builtin_amdgcn_mfma_f32_16x16x1f32(o.x[c][s].x, o.w[c][s].x, acc[s], 0, 0, 0);
#pragma unroll
        for (int s = 0; s < NS; s++) acc[s] = __builtin_amdgcn_mfma_f32_16x16x1f32(o.x[c][s].y, o.w[c][s].y, acc[s], 0, 0, 0);
#pragma unroll
        for (int s = 0; s < NS; s++) acc[s] = __builtin_amdgcn_mfma_f32_16x16x1f32(o.x[c][s].z, o.w[c][s].z, acc[s], 0, 0, 0);
#pragma unroll
        for (int s = 0; s < NS; s++) acc[s] = __builtin_amdgcn_mfma_f32_16x16x1f32(o.x[c][s].w, o.w[c][s].w, acc[s], 0, 0, 0);
    };
    if (nfast > 0) {
        // chunk c is read from LDS buffer c % 2 half a chunk at a time: its first half beside the second half of chunk
        // c - 1's matrix instructions, its second half beside its own first half
        LmHalf<NS> h1, h2;
        __syncthreads();
        read_half(h1, 0, 0);
        for (int c = 0; c < nfast; c++) {
            const int buf = c & 1;
            contract4(h1, 0);
            contract4(h1, 1);
            read_half(h2, buf, 1);
#pragma unroll
            for (int i = 0; i < 8; i++) {   // one matrix instruction, one LDS read
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
            __syncthreads();
            __builtin_amdgcn_sched_barrier(0);
            contract4(h2, 0);
            contract4(h2, 1);
            read_half(h1, buf ^ 1, 0);
#pragma unroll
            for (int i = 0; i < 8; i++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    for (int k0 = nfast * kLmChunk; k0 < ne; k0 += kLmChunk) {   // up to three whole chunks and a shorter one, unpipelined
        __syncthreads();
        __syncthreads();
        const int steps = min(kLmChunk, ne - k0) >> 3;   // 4, 8, 12 or 16 (ne is a multiple of 32)
        LmHalf<NS> o;
        read_half(o, 0, 0);
        contract4(o, 0);
        if (steps > 4) contract4(o, 1);
        if (steps > 8) {
            read_half(o, 0, 1);
            contract4(o, 0);
            if (steps > 12) contract4(o, 1);
        }
    }
    if (SPLIT) {   // chains 4..7 to the tile's first wavefront (the moving wavefronts are through: the buffers are free)
        __syncthreads();
        if (set0 == 1) {
#pragma unroll
            for (int i = 0; i < 16; i++) lm_lds[(cw * 16 + i) * 64 + lane] = acc[0][i];
        }
        __syncthreads();
        if (set0 == 1) return;
    }
    const int e = e0 + 16 * ew + (lane & 15);
#pragma unroll
    for (int i = 0; i < 4; i++) {
        float s = 0.0f;
#pragma unroll
        for (int c = 0; c < 8; c++) {
            float a;
            if (SPLIT) a = c < 4 ? acc[0][4 * c + i] : lm_lds[(cw * 16 + 4 * (c & 3) + i) * 64 + lane];
            else a = acc[NS - 1 < (c >> 2) ? 0 : (c >> 2)][4 * (c & 3) + i];
            s = __fadd_rn(s, a);
        }
        const int r = r0 + 16 * tw + 4 * (lane >> 4) + i;
        if (e < n_expert && r < rows) logits[(size_t)r * n_expert + e] = s;
    }
}

// Experts and token rows per block of router_logits_kernel for a shape, or false when even one of each does
// not fit the LDS budget.
constexpr size_t kRouterLdsBudget = 140 * 1024;
static bool router_logits_tile(int rdt, int ne, int rows, int* epb_out, int* rpb_out) {
    // Decode and small batches of an f32 router: many small blocks of 2 experts x 2 rows, each
    // staging its operands with one burst of loads.  Otherwise: 8 experts x 4 rows per pass.
    const bool small = rows <= 2 || (rows < 32 && rdt == INFR_F32 && (ne & 3) == 0 && ne <= 4096);
    int epb = small ? 2 : 8;
    // the one-burst staging holds 1024 128-bit loads of activations, or 4096 in its wide form (up to four rows of 4096)
    int rpb = small ? (rows < 2 ? 1 : ne > 2048 ? (rows < 4 ? 2 : 4) : 2) : 4;
    const int nc = ne >> 3;
    const size_t estride = (size_t)8 * (((nc + 63) & ~63) + 4);
    auto lds_bytes = [&](int e, int r) { return ((size_t)(e + r) * (estride + 8)) * sizeof(float); };
    while (lds_bytes(epb, rpb) > kRouterLdsBudget && rpb > 1) rpb >>= 1;
    while (lds_bytes(epb, rpb) > kRouterLdsBudget && epb > 1) epb >>= 1;
    if (lds_bytes(epb, rpb) > kRouterLdsBudget) return false;
    *epb_out = epb;
    *rpb_out = rpb;
    return true;
}

bool router_logits_fits(int rdt, size_t row_bytes, int ne, int rows) {
    if (rows >= 32 && rdt == INFR_F32 && (ne & 31) == 0 && (row_bytes & 15) == 0) return true;   // the matrix-core kernel
    int epb, rpb;
    return router_logits_tile(rdt, ne, rows, &epb, &rpb);
}

// The fold needs the one-burst staging of a single row (rows = 1 gives 2 experts x 1 row per block).
bool router_logits_can_norm(int rdt, size_t row_bytes, int ne, int rows) {
    return rows == 1 && rdt == INFR_F32 && (ne & 3) == 0 && ne >= 4 && ne <= 4096 && (row_bytes & 15) == 0;
}

bool launch_router_logits(hipStream_t s, const uint8_t* router, int rdt, size_t row_bytes, const float* x, int ne,
                          int n_expert, int rows, float* logits, const RouterNorm* norm) {
    const RouterNorm nrm = norm ? *norm : RouterNorm{};
    if (nrm.weight && (!router_logits_can_norm(rdt, row_bytes, ne, rows) || !nrm.xn_out || nrm.xn_out == x ||
                       (((uintptr_t)x | (uintptr_t)nrm.weight | (uintptr_t)nrm.xn_out) & 15) != 0))
        return false;
    if (rows >= 32 && rdt == INFR_F32 && (ne & 31) == 0 && (row_bytes & 15) == 0) {
        // 32 x 32 tiles when they give every compute unit a workgroup; 16 x 16 with split chains otherwise (a workgroup's
        // time does not shrink with the batch: it is its chain length; for the large form splitting changed nothing, 16.0
        // against 16.1 us)
        const int neb = (n_expert + 31) / 32, ntb = (rows + 31) / 32;
        if ((size_t)neb * ntb >= 256) {
            dim3 grid((unsigned)(neb * ((ntb + 7) / 8) * 8));
            INFR_LDS_LIMIT((router_logits_mfma_kernel<2, 2, 0>), (int)(lm_lds_bytes<2, 2>()));
            INFR_LAUNCH((router_logits_mfma_kernel<2, 2, 0>), grid, dim3(512), (lm_lds_bytes<2, 2>()), s,
                        reinterpret_cast<const float*>(router), row_bytes / 4, x, ne, n_expert, rows, logits);
        } else {
            const int neb1 = (n_expert + 15) / 16, ntb1 = (rows + 15) / 16;
            dim3 grid((unsigned)(neb1 * ((ntb1 + 7) / 8) * 8));
            INFR_LAUNCH((router_logits_mfma_kernel<1, 1, 1>), grid, dim3(256), (lm_lds_bytes<1, 1>()), s,
                        reinterpret_cast<const float*>(router), row_bytes / 4, x, ne, n_expert, rows, logits);
        }
        return true;
    }
    int epb = 0, rpb = 0;
    if (!router_logits_tile(rdt, ne, rows, &epb, &rpb)) return false;
    // one token row and no more experts than compute units: a block per expert halves what a block stages
    if (rows == 1 && epb == 2 && n_expert <= 256) epb = 1;
    const bool small = rows <= 2 || (rows < 32 && rdt == INFR_F32 && (ne & 3) == 0 && ne <= 4096);
    const size_t budget = kRouterLdsBudget;
    const int nc = ne >> 3;
    const size_t estride = (size_t)8 * (((nc + 63) & ~63) + 4);
    auto lds_bytes = [&](int e, int r) { return ((size_t)(e + r) * (estride + 8)) * sizeof(float); };
    size_t lds = lds_bytes(epb, rpb);
    int gx = (n_expert + epb - 1) / epb;
    int passes = (rows + rpb - 1) / rpb;
    int gy = passes;
    int cap = small ? passes : (1024 + gx - 1) / gx;
    if (gy > cap) gy = cap;
    if (gy < 1) gy = 1;
    dim3 grid(gx, gy), block(256);
#define LAUNCH_RL(E)                                                                                               \
    do {                                                                                                           \
        INFR_LDS_LIMIT((router_logits_kernel<E>), (int)budget); \
        INFR_LAUNCH(router_logits_kernel<E>, grid, block, lds, s, router, rdt, row_bytes, x, ne, n_expert,  \
                           rows, rpb, logits, nrm);                                                   \
    } while (0)
    if (small && rpb * (ne >> 2) > 4 * 256 && epb <= 2) {   // the wide one-burst staging
        INFR_LDS_LIMIT((router_logits_kernel<2, 16>), (int)budget);
        if (epb == 2) INFR_LAUNCH((router_logits_kernel<2, 16>), grid, block, lds, s, router, rdt, row_bytes, x, ne, n_expert, rows, rpb, logits, nrm);
        else {
            INFR_LDS_LIMIT((router_logits_kernel<1, 16>), (int)budget);
            INFR_LAUNCH((router_logits_kernel<1, 16>), grid, block, lds, s, router, rdt, row_bytes, x, ne, n_expert, rows, rpb, logits, nrm);
        }
        return true;
    }
    switch (epb) {
        case 8: LAUNCH_RL(8); break;
        case 4: LAUNCH_RL(4); break;
        case 2: LAUNCH_RL(2); break;
        default: LAUNCH_RL(1); break;
    }
#undef LAUNCH_RL
    return true;
}

}  // namespace infr

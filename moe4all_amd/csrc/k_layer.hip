// Single-token Op::MoeFfn as ONE launch: router logits, routing, gate/up with the gated activation, down
// and the rank-ordered weighted sum, with the two hand-overs between the stages done inside the kernel
// instead of at kernel boundaries.
//
// Work split.  The grid is 256 blocks in 8 groups of 32 (group = blockIdx & 7; the dispatcher deals
// consecutive blocks to consecutive XCDs, so a group's blocks share an L2).  Group g owns rank g of the
// token's selection:
//   A  every block computes n_expert / 32 router logits (each group computes all of them, so the logits
//      never cross a group) and publishes them to its group;
//   R  every block gathers its group's logits and routes the row (the same routine as the routing
//      kernel: ids and weights are an integer / bit contract);
//   B  block m of group g computes features [m * nff / 32, +nff / 32) of gate and up of expert ids[g],
//      applies the activation and publishes its slice of h to the group; its down rows are requested
//      before, so they arrive while gate/up is computed;
//   C  every block gathers the group's h and computes output rows [m * ne / 32, +ne / 32) of
//      down(ids[g]) . h, stores them as rank g's partial result, and the last of the 8 blocks that
//      finish an output slice sums the 8 partials in rank order (+ addend) into dst.
// The inner products, the activation and the order of the final sum are those of the three-kernel path
// (moe_gate_up_fast / moe_down_combine_fast), so the result has the same bits.
//
// Hand-over.  A published value is one 64-bit record {value bits, tag} written with an agent-scope
// atomic store; the tag is the launch's sequence number, kept in device memory and advanced by the block
// that finishes last, so a record of an earlier launch is never mistaken for a current one (also under
// graph replay, where kernel arguments do not change).  A consumer polls the records it needs with
// agent-scope atomic loads.  Every wait is bounded: after `spin_limit` polls a block raises the fault
// word (host-visible) and leaves; its peers then run into their own limits, so the grid always drains.
// The host reports the fault at the next synchronisation and stops using this kernel.  Blocks only wait
// for blocks of the same launch, which are co-resident when the device has a compute unit per block.
#include "device_common.h"
#include "kernels.h"
#include "route.h"
#include "gemv_fmt.h"

#include <type_traits>

namespace infr {

namespace {

// Phase time stamps of every block for a measurement build (-DINFR_LAYER_TRACE with a buffer in g.y); compiled out otherwise.
#ifdef INFR_LAYER_TRACE
#define LAYER_STAMP(i)                                                                                         \
    do {                                                                                                       \
        if (threadIdx.x == 0 && q.g.y) reinterpret_cast<long long*>(q.g.y)[blockIdx.x * 16 + (i)] = wall_clock64(); \
    } while (0)
#else
#define LAYER_STAMP(i) do { } while (0)
#endif

constexpr int kGroups = 8, kPerGroup = 32, kLayerBlocks = kGroups * kPerGroup;
constexpr int kMaxSliceRows = 128;   // ne / 32 <= 128

__device__ __forceinline__ uint64_t rec_load(const uint64_t* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void rec_store(uint64_t* p, float v, uint32_t tag) {
    __hip_atomic_store(p, (uint64_t)__float_as_uint(v) | ((uint64_t)tag << 32), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Wave-wide: gathers the 64 * N records rec[0 .. 64 N) into out[] once all carry `tag`.  Every poll issues all of a
// lane's loads before it looks at any of them, so a poll costs one memory round trip.  False when the spin limit ran out.
template <int N>
__device__ __forceinline__ bool gather_records(const uint64_t* rec, uint32_t tag, float* out, int lane, int spin_limit) {
    uint64_t r[N];
    for (int spin = 0;; spin++) {
#pragma unroll
        for (int s = 0; s < N; s++) r[s] = rec_load(rec + s * kWave + lane);
        bool ok = true;
#pragma unroll
        for (int s = 0; s < N; s++) ok = ok && (uint32_t)(r[s] >> 32) == tag;
        if (__all(ok)) break;
        if (spin >= spin_limit) return false;
    }
#pragma unroll
    for (int s = 0; s < N; s++) out[s * kWave + lane] = __uint_as_float((uint32_t)r[s]);
    return true;
}

}  // namespace

// FG / FD: formats of the gate/up and down banks; U: gate/up items a wave has in flight; S: down row groups a wave
// has in flight; EPB: router rows per block (n_expert / 32); NH: nff / 64.
template <class FG, class FD, int U, int S, int EPB, int NH>
__global__ __launch_bounds__(256) void moe_layer_fused(MoeLayerParams q) {
    extern __shared__ __attribute__((aligned(16))) uint32_t dyn_lds[];
    __shared__ uint64_t s_tab[32];
    __shared__ int32_t s_ids[64];
    __shared__ float s_w[64];
    __shared__ float s_g[4][64], s_u[4][64];
    __shared__ float s_y[kMaxSliceRows];
    __shared__ int s_flag;
    __shared__ uint32_t s_tag;
    const MoeGemvParams& p = q.g;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int g = blockIdx.x & (kGroups - 1), m = blockIdx.x >> 3;
    const int ne = p.ne, nff = p.nff, n_expert = p.route.n_expert;

    // LDS: [x cells][stage A: router rows and x, transposed | later: logits, routing scratch, h, h cells]
    const size_t cell_words = (size_t)((ne + 31) / 32) * kCellDwords;
    uint32_t* cells = dyn_lds;
    float* stage = reinterpret_cast<float*>(dyn_lds + cell_words);

    if (tid < 32) s_tab[tid] = kExp2Table[tid];
    if (tid == 0) {
        s_flag = 0;
        s_tag = __hip_atomic_load(q.seq, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1u;   // one load per block
    }
    LAYER_STAMP(0);

    // ---- A: logits of experts [m * EPB, +EPB) with the reference's order: 8 chains over i = j (mod 8), summed 0..7
    // (crates/infr-cpu/src/kernels.rs:6568-6583).  Operands are staged transposed, chain-major, as in router_logits_kernel.
    const int nv = ne >> 2, nc = ne >> 3;
    const int jstride = ((nc + 63) & ~63) + 4, estride = 8 * jstride;
    float* wst = stage;
    float* xst = stage + EPB * estride;
    {
        constexpr int NXV = 2;   // ne <= 2048: at most 2 float4 of a row per thread
        float4 xr[NXV], wr[EPB * NXV];
        const float4* x4 = reinterpret_cast<const float4*>(q.router_x);
#pragma unroll
        for (int i = 0; i < NXV; i++) {
            const int idx = tid + 256 * i;
            xr[i] = idx < nv ? x4[idx] : make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int i = 0; i < EPB * NXV; i++) {
            const int idx = tid + 256 * i, e = idx / nv, v = idx - e * nv;
            wr[i] = e < EPB ? reinterpret_cast<const float4*>(q.router + (size_t)(m * EPB + e) * q.router_row_floats)[v]
                            : make_float4(0.f, 0.f, 0.f, 0.f);
        }
        // the token row for the expert stages, requested with the rest: waves 1-3 turn it into fixed-point cells, eight
        // elements per thread and pass (ne <= 2048: at most two passes of 192 threads), while wave 0 runs the chains
        const float4* px4 = reinterpret_cast<const float4*>(p.x);
        const int oct0 = tid - kWave, oct1 = oct0 + 3 * kWave;
        const bool own0 = wave > 0 && 8 * oct0 < ne, own1 = wave > 0 && 8 * oct1 < ne;
        float4 xo[4];
        xo[0] = own0 ? px4[2 * oct0] : make_float4(0.f, 0.f, 0.f, 0.f);
        xo[1] = own0 ? px4[2 * oct0 + 1] : make_float4(0.f, 0.f, 0.f, 0.f);
        xo[2] = own1 ? px4[2 * oct1] : make_float4(0.f, 0.f, 0.f, 0.f);
        xo[3] = own1 ? px4[2 * oct1 + 1] : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int i = 0; i < NXV; i++) {
            const int idx = tid + 256 * i;
            if (idx >= nv) continue;
            const float fv[4] = {xr[i].x, xr[i].y, xr[i].z, xr[i].w};
#pragma unroll
            for (int t = 0; t < 4; t++) {
                const int k = 4 * idx + t;
                xst[(k & 7) * jstride + (k >> 3)] = fv[t];
            }
        }
#pragma unroll
        for (int i = 0; i < EPB * NXV; i++) {
            const int idx = tid + 256 * i, e = idx / nv, v = idx - e * nv;
            if (e >= EPB) continue;
            const float fv[4] = {wr[i].x, wr[i].y, wr[i].z, wr[i].w};
#pragma unroll
            for (int t = 0; t < 4; t++) {
                const int k = 4 * v + t;
                wst[e * estride + (k & 7) * jstride + (k >> 3)] = fv[t];
            }
        }
        __syncthreads();
        const uint32_t tag = s_tag;
        LAYER_STAMP(1);
        if (wave > 0) {
            // cells of x (whole lane groups take part: ne is a multiple of 256, so is every pass's first octet)
            if (own0) octet_to_cell<FG::kGroup, FG::kSigned>(xo[0], xo[1], oct0, cells);
            if (own1) octet_to_cell<FG::kGroup, FG::kSigned>(xo[2], xo[3], oct1, cells);
        } else {
            const int e = lane >> 3, j = lane & 7;
            const bool live = e < EPB;
            float acc = 0.0f;
            if (live) {
                const float4* wp = reinterpret_cast<const float4*>(wst + e * estride + j * jstride);
                const float4* xp = reinterpret_cast<const float4*>(xst + j * jstride);
                const int n4 = nc >> 2;   // a multiple of 8
#pragma unroll 1
                for (int c = 0; c < n4; c += 8) {
                    float4 a[8], b[8];
#pragma unroll
                    for (int k = 0; k < 8; k++) { a[k] = wp[c + k]; b[k] = xp[c + k]; }
#pragma unroll
                    for (int k = 0; k < 8; k++) {
                        acc = __fmaf_rn(a[k].x, b[k].x, acc);
                        acc = __fmaf_rn(a[k].y, b[k].y, acc);
                        acc = __fmaf_rn(a[k].z, b[k].z, acc);
                        acc = __fmaf_rn(a[k].w, b[k].w, acc);
                    }
                }
            }
            float s = 0.0f;
#pragma unroll
            for (int jj = 0; jj < 8; jj++) s = __fadd_rn(s, __shfl(acc, (lane & ~7) + jj, kWave));
            if (live && j == 0) {
                rec_store(q.xl + (size_t)g * n_expert + m * EPB + e, s, tag);
                if (g == 0 && q.logits_out) q.logits_out[m * EPB + e] = s;
            }
        }
        LAYER_STAMP(2);
    }
    __syncthreads();   // stage A's LDS is free from here on
    const uint32_t tag = s_tag;
    LAYER_STAMP(3);

    float* s_logits = stage;                                   // [n_expert]
    float* route_scratch = s_logits + n_expert;                // route_scratch_floats(n_expert, n_groups)
    float* s_h = route_scratch + ((route_scratch_floats(n_expert, p.route.n_groups) + 3) & ~(size_t)3);   // [nff]
    uint32_t* hcells = reinterpret_cast<uint32_t*>(s_h + nff); // cells of h, one copy for the block (16-byte aligned: all counts are multiples of 4)

    // ---- R: gather the group's logits, route
    if (wave == 0) {
        const bool ok = gather_records<EPB / 2>(q.xl + (size_t)g * n_expert, tag, s_logits, lane, q.spin_limit);
        LAYER_STAMP(4);
        if (!ok && lane == 0) {
            s_flag = 1;
            __hip_atomic_store(q.fault, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        }
    }
    __syncthreads();
    if (s_flag) return;
    {
        // Plain softmax routing on two wavefronts.  The serial parts of the reference's routing are the left-to-right
        // sum of the exponentials and the selection rounds; wave 0 runs the sum while wave 1 selects the nine largest
        // exponentials, (value descending, id ascending).  A probability is fl(exp / sum), a non-decreasing function of
        // the exponential, so when the nine candidates' probabilities are strictly decreasing the first eight are the
        // reference's selection in its order (crates/infr-cpu/src/lib.rs:3847-3850); when two of them collide after the
        // division (exponentials an ulp apart) or anything is not a number, wave 0 runs the complete routine instead.
        constexpr int NS = EPB / 2;
        const RouteParams& rq = p.route;
        const bool plain = rq.gating == INFR_GATING_SOFTMAX && !rq.exp_probs_b && !rq.expert_ids &&
                           !(rq.n_groups > 1 && rq.n_groups_used > 0);
        __shared__ float s_psum;
        __shared__ int32_t s_cand[16];
        __shared__ float s_cand_e[16];
        float pr[NS];
        if (plain && wave < 2) {
            float mx = -__builtin_huge_valf();
#pragma unroll
            for (int t = 0; t < NS; t++) {
                pr[t] = s_logits[t * kWave + lane];
                mx = fmaxf(mx, pr[t]);
            }
            mx = wave_max(mx);
#pragma unroll
            for (int t = 0; t < NS; t++) pr[t] = expf_libm(__fsub_rn(pr[t], mx), s_tab);
            if (wave == 0) {
                float* ex = route_scratch;
#pragma unroll
                for (int t = 0; t < NS; t++) ex[t * kWave + lane] = pr[t];
                __builtin_amdgcn_wave_barrier();
                float psum = 0.0f;
                {
                    // the terms come in batches of 32 (eight 128-bit broadcast reads), the next batch requested
                    // before the current one is added, so the chain of dependent adds never waits for LDS
                    // (n_expert is a multiple of 64, ex is 16-byte aligned)
                    float4 cur[8], nxt[8];
#pragma unroll
                    for (int k = 0; k < 8; k++) cur[k] = reinterpret_cast<const float4*>(ex)[k];
                    for (int i = 0; i < n_expert; i += 32) {
                        const int ni = i + 64 <= n_expert ? i + 32 : i;   // past the end: re-read, unused
#pragma unroll
                        for (int k = 0; k < 8; k++) nxt[k] = reinterpret_cast<const float4*>(ex + ni)[k];
#pragma unroll
                        for (int k = 0; k < 8; k++) {
                            psum = __fadd_rn(psum, cur[k].x);
                            psum = __fadd_rn(psum, cur[k].y);
                            psum = __fadd_rn(psum, cur[k].z);
                            psum = __fadd_rn(psum, cur[k].w);
                        }
#pragma unroll
                        for (int k = 0; k < 8; k++) cur[k] = nxt[k];
                    }
                }
                if (lane == 0) s_psum = psum;
            } else {
                // every lane first sorts its own NS candidates, (key descending, id ascending), so a round only looks
                // at the lane's head: one reduction for the largest key, one ballot for who holds it, and the winner's
                // list moves up by one.  An exponential is not negative, so a live key has its top bit set and 0
                // marks an empty place.
                uint32_t key[NS], id[NS];
#pragma unroll
                for (int t = 0; t < NS; t++) {
                    id[t] = (uint32_t)(t * kWave + lane);
                    key[t] = order_key(pr[t]);
                }
#pragma unroll
                for (int a = 0; a + 1 < NS; a++) {
#pragma unroll
                    for (int b = 0; b + 1 < NS - a; b++) {
                        const bool swap = key[b + 1] > key[b];   // strict, adjacent: equal keys stay in id order
                        const uint32_t hk = swap ? key[b + 1] : key[b], lk = swap ? key[b] : key[b + 1];
                        const uint32_t hi = swap ? id[b + 1] : id[b], li = swap ? id[b] : id[b + 1];
                        key[b] = hk; key[b + 1] = lk;
                        id[b] = hi; id[b + 1] = li;
                    }
                }
                for (int k = 0; k < 9; k++) {
                    const uint32_t kmax = wave_max_u32(key[0]);
                    const bool match = key[0] == kmax && kmax != 0u;
                    const uint64_t holders = __ballot(match);
                    uint32_t win;
                    if (__builtin_popcountll(holders) == 1) {
                        win = (uint32_t)__builtin_amdgcn_readlane((int)id[0], __builtin_ctzll(holders));
                    } else {
                        // several lanes hold the largest key: the smallest id among their heads
                        win = wave_min_u32(match ? id[0] : 0xFFFFFFFFu);
                    }
                    if (holders == 0 && lane == 0) {   // nothing comparable left (keys of negative NaNs): the check fails
                        s_cand[k] = 0;
                        s_cand_e[k] = __uint_as_float(0x7FC00000u);
                    }
                    if (match && id[0] == win) {
                        s_cand[k] = (int32_t)win;
                        s_cand_e[k] = __uint_as_float(key[0] & 0x7FFFFFFFu);   // the exponential back from its key
#pragma unroll
                        for (int t = 0; t + 1 < NS; t++) {
                            key[t] = key[t + 1];
                            id[t] = id[t + 1];
                        }
                        key[NS - 1] = 0u;
                    }
                }
            }
        }
        if (plain) __syncthreads();
        if (wave == 0) {
            bool done = false;
            if (plain) {
                const float psum = s_psum;
                const float pc = lane < 9 ? __fdiv_rn(s_cand_e[lane], psum) : 0.0f;
                const float nxt = __shfl_down(pc, 1, kWave);
                done = __all(lane >= 8 || pc > nxt);
                if (done) {
                    // routing weights (lib.rs:3856-3861): lane k owns rank k
                    const bool mine = lane < rq.n_used;
                    int my_id = mine ? s_cand[lane] : 0;
                    const float pk = mine ? pc : 0.0f;
                    float w;
                    if (rq.norm_w) {
                        float wsum = 0.0f;
                        for (int k = 0; k < rq.n_used; k++) wsum = __fadd_rn(wsum, readlane_f(pk, k));
                        wsum = fmaxf(wsum, 1e-20f);
                        w = __fmul_rn(__fdiv_rn(pk, wsum), rq.scale);
                    } else {
                        w = __fmul_rn(pk, rq.scale);
                    }
                    if (rq.ep_n > 0) {
                        const bool own = my_id >= rq.ep_lo && my_id < rq.ep_lo + rq.ep_n;
                        my_id = own ? my_id - rq.ep_lo : 0;
                        w = own ? w : 0.0f;
                    }
                    if (mine) {
                        s_ids[lane] = my_id;
                        s_w[lane] = w;
                        if (blockIdx.x == 0) {
                            rq.ids[lane] = my_id;
                            rq.weights[lane] = w;
                        }
                    }
                    if (blockIdx.x == 0 && rq.probs) {
#pragma unroll
                        for (int t = 0; t < NS; t++) rq.probs[t * kWave + lane] = __fdiv_rn(pr[t], psum);
                    }
                }
            }
            if (!done) {
                RouteParams rp = p.route;
                rp.logits = s_logits;
                route_row_any(rp, 0, lane, route_scratch, s_tab, s_ids, s_w, blockIdx.x == 0);
            }
        }
    }
    __syncthreads();
    LAYER_STAMP(5);

    // ---- B: gate/up of expert ids[g], features [m * fpb, +fpb); the down rows of phase C are requested first
    const int e = s_ids[g];
    const int nblk_g = ne / FG::kBlockElems, nblk_d = nff / FD::kBlockElems;
    const size_t rb_g = (size_t)nblk_g * FG::kBlockBytes, rb_d = (size_t)nblk_d * FD::kBlockBytes;
    const Place<FG> pg(nblk_g, lane);
    const Place<FD> pd(nblk_d, lane);
    const int fpb = nff / kPerGroup, f0 = m * fpb;
    const int R = ne / kPerGroup, RW = (R + 3) >> 2;           // output rows of the block, of a wave
    const int ow0 = wave * RW, ocount = min(RW, R - ow0);      // may be <= 0 for the last waves of a small slice
    typename FD::Raw rd[S];
    {
        typename FG::Raw sg[U], su[U];
        const uint8_t* gb = p.gate + (size_t)e * p.gate_stride;
        const uint8_t* ub = p.up + (size_t)e * p.up_stride;
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int it = min((u * 4 + wave) * pg.rw_count + pg.rw, fpb - 1);
            sg[u] = load_row<FG>(pg, gb + (size_t)(f0 + it) * rb_g);
            su[u] = load_row<FG>(pg, ub + (size_t)(f0 + it) * rb_g);
        }
        // the down rows of phase C, requested behind the gate/up rows: they arrive while gate/up is computed
        {
            const uint8_t* bank = p.down + (size_t)e * p.down_stride + (size_t)(m * R + ow0) * rb_d;
#pragma unroll
            for (int st = 0; st < S; st++) {
                const int o = max(min(st * pd.rw_count + pd.rw, ocount - 1), -ow0);   // clamped into the block's slice
                rd[st] = load_row<FD>(pd, bank + (ptrdiff_t)o * (ptrdiff_t)rb_d);
            }
        }
        typename FG::X x;
        FG::fetch_x(x, cells, pg.blk, pg.sub);
#pragma unroll
        for (int u = 0; u < U; u++) {
            const float gs = row_sum<FG>(FG::dot(sg[u], pg.sub, x), pg, nblk_g);
            const float us = row_sum<FG>(FG::dot(su[u], pg.sub, x), pg, nblk_g);
            if (pg.writer()) {
                s_g[wave][u * pg.rw_count + pg.rw] = gs;
                s_u[wave][u * pg.rw_count + pg.rw] = us;
            }
        }
        __builtin_amdgcn_wave_barrier();
        if (lane < U * pg.rw_count) {
            const int u = lane / pg.rw_count, rw = lane - u * pg.rw_count;
            const int it = (u * 4 + wave) * pg.rw_count + rw;
            if (it < fpb) {
                float gs = s_g[wave][lane], us = s_u[wave][lane];
                if (p.weight_before) {
                    const float wp = s_w[g];
                    gs = __fmul_rn(wp, gs);
                    us = __fmul_rn(wp, us);
                }
                rec_store(q.xh + (size_t)g * nff + f0 + it, gated_act_fn(p.act, p.has_clamp, p.clamp, gs, us, s_tab), tag);
            }
        }
    }
    LAYER_STAMP(6);

    // ---- C: gather the group's h, down rows [m * R, +R) of expert ids[g]
    if (wave == 0) {
        const bool ok = gather_records<NH>(q.xh + (size_t)g * nff, tag, s_h, lane, q.spin_limit);
        LAYER_STAMP(7);
        if (!ok) {
            if (lane == 0) {
                s_flag = 1;
                __hip_atomic_store(q.fault, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            }
        } else {
            __builtin_amdgcn_wave_barrier();
            // h to fixed-point cells, eight elements per lane and pass (nff is a multiple of 64: whole lane groups)
            for (int oct = lane; oct * 8 < nff; oct += kWave) {
                const float4 lo = *reinterpret_cast<const float4*>(s_h + 8 * oct), hi = *reinterpret_cast<const float4*>(s_h + 8 * oct + 4);
                octet_to_cell<FD::kGroup, FD::kSigned>(lo, hi, oct, hcells);
            }
        }
    }
    __syncthreads();
    LAYER_STAMP(8);
    if (s_flag) return;
    {
        typename FD::X xd;
        FD::fetch_x(xd, hcells, pd.blk, pd.sub);
        const bool scaled = p.down_scale != nullptr;
        const float ds = scaled ? p.down_scale[e] : 1.0f;
#pragma unroll
        for (int st = 0; st < S; st++) {
            const int o = st * pd.rw_count + pd.rw;
            const float y = row_sum<FD>(FD::dot(rd[st], pd.sub, xd), pd, nblk_d);
            if (o < ocount && pd.writer()) s_y[ow0 + o] = scaled ? __fmul_rn(y, ds) : y;
        }
    }
    __syncthreads();
    LAYER_STAMP(9);
    // partial results travel as tagged records too, so no fence is needed anywhere: the counter only elects the block
    // that sums, the tags say when a partial has arrived
    uint64_t* part = q.ypart + (size_t)m * R;   // + rank * ne
    if (tid < R) rec_store(part + (size_t)g * ne + tid, s_y[tid], tag);
    if (tid == 0) {
        const uint32_t old = __hip_atomic_fetch_add(q.cnt + m, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        s_flag = (old & (kGroups - 1)) == kGroups - 1 ? 2 : 0;
    }
    __syncthreads();
    LAYER_STAMP(10);
    if (s_flag != 2) return;
    // the last block of the slice: out = sum over ranks of w_rank * y_rank as a separate multiply and add
    // (crates/infr-cpu/src/lib.rs:4290-4302)
    if (tid < R) {
        uint64_t yk[kGroups];
        bool ok = false;
        for (int spin = 0; !ok && spin <= q.spin_limit; spin++) {
#pragma unroll
            for (int k = 0; k < kGroups; k++) yk[k] = rec_load(part + (size_t)k * ne + tid);   // all eight requested before the first is used
            ok = true;
#pragma unroll
            for (int k = 0; k < kGroups; k++) ok = ok && (uint32_t)(yk[k] >> 32) == tag;
        }
        if (!ok) __hip_atomic_store(q.fault, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        const size_t oi = (size_t)m * R + tid;
        const float add = p.addend ? p.addend[oi] : 0.0f;
        float acc = 0.0f;
#pragma unroll
        for (int k = 0; k < kGroups; k++) {
            if (p.skip_zero_w && s_w[k] == 0.0f) continue;
            const float wk = p.weight_before ? 1.0f : s_w[k];
            acc = __fadd_rn(acc, __fmul_rn(wk, __uint_as_float((uint32_t)yk[k])));
        }
        p.dst[oi] = p.addend ? __fadd_rn(add, acc) : acc;
    }
    LAYER_STAMP(11);
    if (tid == 0) {
        const uint32_t old = __hip_atomic_fetch_add(q.cnt + kPerGroup, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if ((old & (kPerGroup - 1)) == kPerGroup - 1) __hip_atomic_store(q.seq, tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

// ---------------------------------------------------------------------------------------------
size_t moe_layer_workspace_bytes(int ne, int nff, int n_expert) {
    // [seq][cnt 32 + done][pad to 256][xl 8 * n_expert records][xh 8 * nff records][ypart 8 * ne records]
    return 256 + (size_t)kGroups * n_expert * 8 + (size_t)kGroups * nff * 8 + (size_t)kGroups * ne * 8;
}

namespace {

struct LayerShape {
    int u, s, epb, nh;
    size_t lds;
};

template <class FG, class FD>
bool layer_shape(const MoeLayerParams& q, LayerShape* out) {
    const MoeGemvParams& p = q.g;
    const int ne = p.ne, nff = p.nff, n_expert = p.route.n_expert;
    if (ne % FG::kBlockElems || nff % FD::kBlockElems || ne % 256 || ne > 2048 || nff % 64 || nff > 2048) return false;
    const int lpr_g = ne / FG::kBlockElems * FG::kLPB, lpr_d = nff / FD::kBlockElems * FD::kLPB;
    if (lpr_g > 64 || lpr_d > 64) return false;
    if (ne / kPerGroup > kMaxSliceRows || n_expert % 64 || n_expert > 512) return false;   // whole waves of logit records
    const int rwc_g = 64 / lpr_g, rwc_d = 64 / lpr_d;
    const int fpb = nff / kPerGroup, rw = (ne / kPerGroup + 3) / 4;
    out->u = (fpb + 4 * rwc_g - 1) / (4 * rwc_g);
    out->s = (rw + rwc_d - 1) / rwc_d;
    out->epb = n_expert / kPerGroup;
    out->nh = nff / 64;
    const int nc = ne >> 3, jstride = ((nc + 63) & ~63) + 4;
    const size_t stage_a = (size_t)(out->epb + 1) * 8 * jstride * 4;
    const size_t stage_b = ((size_t)n_expert + ((route_scratch_floats(n_expert, p.route.n_groups) + 3) & ~(size_t)3) + nff) * 4 + cells_bytes(nff);
    out->lds = cells_bytes(ne) + (stage_a > stage_b ? stage_a : stage_b);
    return out->lds <= 150 * 1024;
}

template <class FG, class FD, int U, int S, int EPB, int NH>
void launch_layer(hipStream_t s, const MoeLayerParams& q, size_t lds) {
    INFR_LDS_LIMIT((moe_layer_fused<FG, FD, U, S, EPB, NH>), 150 * 1024);
    INFR_LAUNCH((moe_layer_fused<FG, FD, U, S, EPB, NH>), dim3(kLayerBlocks), dim3(256), lds, s, q);
}

// The instantiated (format pair, U, S, EPB) combinations.
template <class FG, class FD>
bool dispatch_layer(hipStream_t s, const MoeLayerParams& q, bool launch) {
    LayerShape sh;
    if (!layer_shape<FG, FD>(q, &sh)) return false;
#define INFR_LAYER(UU, SS, EE, HH)                                              \
    if (sh.u == UU && sh.s == SS && sh.epb == EE && sh.nh == HH) {                 \
        if (launch) launch_layer<FG, FD, UU, SS, EE, HH>(s, q, sh.lds);            \
        return true;                                                               \
    }
    if constexpr (std::is_same<FG, Q4KFmt>::value) {
        INFR_LAYER(3, 4, 4, 12)   // ne 2048, nff 768, 128 experts
        INFR_LAYER(3, 4, 8, 12)   // ... 256 experts
    } else {
        INFR_LAYER(6, 8, 4, 12)
        INFR_LAYER(6, 8, 8, 12)
    }
#undef INFR_LAYER
    return false;
}

bool layer_any(hipStream_t s, const MoeLayerParams& q, bool launch) {
    const MoeGemvParams& p = q.g;
    if (p.rows != 1 || p.n_used != kGroups || p.n_cu < kLayerBlocks || p.sh_gate || p.sh_down || p.gate_dt != p.up_dt) return false;
    if ((((uintptr_t)q.router | (uintptr_t)q.router_x | (uintptr_t)p.x) & 15) != 0 || (q.router_row_floats & 3) != 0) return false;
    if (p.gate_dt == INFR_Q4K && p.down_dt == INFR_Q6K) return dispatch_layer<Q4KFmt, Q6KFmt>(s, q, launch);
    if (p.gate_dt == INFR_Q8_0 && p.down_dt == INFR_Q8_0) return dispatch_layer<Q80Fmt, Q80Fmt>(s, q, launch);
    return false;
}

}  // namespace

bool moe_layer_fused_supported(const MoeLayerParams& q) { return layer_any(nullptr, q, false); }
bool launch_moe_layer_fused(hipStream_t s, const MoeLayerParams& q) { return layer_any(s, q, true); }

}  // namespace infr

// Routing of one token row by one wavefront: gating -> selection -> routing weights, in the
// reference's operation order (crates/infr-cpu/src/lib.rs:3741-3863).  Shared by the
// standalone route kernel and by the decode GEMV kernel, where every block routes its own
// token row redundantly instead of waiting for a separate launch.
#pragma once

#include "device_common.h"
#include "kernels.h"

// Time stamps for a measurement build; the includer may define the macro, the library compiles it out.
#ifndef ROUTE_STAMP
#define ROUTE_STAMP(i) do { } while (0)
#endif

namespace infr {

// ---------------------------------------------------------------------------------------------
// Routing of one token row by one wavefront.  lds: 2*n floats (+ n_groups) of scratch, tab: the
// exp table staged in LDS.  NS = candidates per lane (n <= 64*NS).
__device__ __forceinline__ uint32_t order_key(float v) {
    uint32_t u = __float_as_uint(v);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// Results go to global memory (p.ids / p.weights / p.probs) when store_global is set, and to
// lds_ids / lds_w when those are non-null.  stage_tab (the LDS array `tab` points at, writable): the wave fills the
// exp table itself right after it has requested its logits, so the two memory latencies overlap.
template <int NS>
__device__ __forceinline__ void route_row(const RouteParams& p, int row, int lane, float* lds, const uint64_t* tab,
                                          int32_t* lds_ids, float* lds_w, bool store_global, uint64_t* stage_tab) {
    const int n = p.n_expert;
    float* prob = lds;
    float* sel = lds + n;
    float* gscore = sel + n;
    const float* lg = p.logits + (size_t)row * n;
    const float ninf = -__builtin_huge_valf();

    float pr[NS];
#pragma unroll
    for (int s = 0; s < NS; s++) {
        int i = s * kWave + lane;
        pr[s] = i < n ? lg[i] : ninf;
    }
    if (stage_tab) {
        if (lane < 32) stage_tab[lane] = kExp2Table[lane];
        __builtin_amdgcn_wave_barrier();
    }
    // ---- gating (lib.rs:3746-3774)
    if (p.gating == INFR_GATING_SOFTMAX) {
        float m = ninf;
#pragma unroll
        for (int s = 0; s < NS; s++) m = fmaxf(m, pr[s]);
        m = wave_max(m);
        ROUTE_STAMP(1);
#pragma unroll
        for (int s = 0; s < NS; s++) pr[s] = (s * kWave + lane < n) ? expf_libm(__fsub_rn(pr[s], m), tab) : 0.0f;
        // psum = p[0] + p[1] + ... strictly left to right (lib.rs:3752-3755).  The terms go through LDS and every
        // lane adds all of them in order (same-address reads are broadcasts): one dependent add per term, where a
        // chain over lanes would pay a cross-lane read per term as well.
#pragma unroll
        for (int s = 0; s < NS; s++)
            if (s * kWave + lane < n) prob[s * kWave + lane] = pr[s];
        __builtin_amdgcn_wave_barrier();
        ROUTE_STAMP(2);
        float psum = 0.0f;
        {
            // the terms come in batches of 32 (eight 128-bit broadcast reads), the next batch requested before the
            // current one is added, so the chain of dependent adds never waits for LDS
            int i = 0;
            if (n >= 32 && (reinterpret_cast<uintptr_t>(prob) & 15) == 0) {
                float4 cur[8], nxt[8];
#pragma unroll
                for (int k = 0; k < 8; k++) cur[k] = reinterpret_cast<const float4*>(prob)[k];
                for (; i + 32 <= n; i += 32) {
                    const int ni = i + 64 <= n ? i + 32 : i;   // past the end: re-read, unused
#pragma unroll
                    for (int k = 0; k < 8; k++) nxt[k] = reinterpret_cast<const float4*>(prob + ni)[k];
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
            for (; i < n; i++) psum = __fadd_rn(psum, prob[i]);
        }
        ROUTE_STAMP(3);
        __builtin_amdgcn_wave_barrier();   // prob is rewritten with the final probabilities below
#pragma unroll
        for (int s = 0; s < NS; s++) pr[s] = __fdiv_rn(pr[s], psum);
    } else if (p.gating == INFR_GATING_SIGMOID) {
#pragma unroll
        for (int s = 0; s < NS; s++) pr[s] = __fdiv_rn(1.0f, __fadd_rn(1.0f, expf_libm(-pr[s], tab)));
    } else {
#pragma unroll
        for (int s = 0; s < NS; s++) {
            float v = pr[s];
            float sp = v > 20.0f ? v : logf(__fadd_rn(1.0f, expf_libm(v, tab)));
            pr[s] = __fsqrt_rn(sp);
        }
    }
#pragma unroll
    for (int s = 0; s < NS; s++) {
        int i = s * kWave + lane;
        if (i < n) prob[i] = pr[s];
    }
    __builtin_amdgcn_wave_barrier();

    ROUTE_STAMP(4);
    int32_t* ids_out = p.ids + (size_t)row * p.n_used;
    float* w_out = p.weights + (size_t)row * p.n_used;
    int my_id = 0;  // lane k < n_used holds the rank-k expert
    if (p.expert_ids) {
        // Hash routing (lib.rs:3776-3793): the supplied ids are the selection, in table order.
        if (lane < p.n_used) {
            int e = p.expert_ids[(size_t)row * p.n_used + lane];
            my_id = e < 0 ? 0 : (e >= n ? n - 1 : e);
        }
    } else {
        float sl[NS];
        // lib.rs:3797-3806: bias on a selection-only copy.
#pragma unroll
        for (int s = 0; s < NS; s++) {
            int i = s * kWave + lane;
            sl[s] = (p.exp_probs_b && i < n) ? __fadd_rn(pr[s], p.exp_probs_b[i]) : pr[s];
        }
        // lib.rs:3809-3846: group-limited routing.
        if (p.n_groups > 1 && p.n_groups_used > 0) {
            const int ng = p.n_groups, per = n / ng;
#pragma unroll
            for (int s = 0; s < NS; s++) {
                int i = s * kWave + lane;
                if (i < n) sel[i] = sl[s];
            }
            __builtin_amdgcn_wave_barrier();
            for (int g = lane; g < ng; g += kWave) {
                float b0 = ninf, b1 = ninf;
                for (int i = g * per; i < (g + 1) * per; i++) {
                    float sv = sel[i];
                    if (sv > b0) { b1 = b0; b0 = sv; }
                    else if (sv > b1) { b1 = sv; }
                }
                gscore[g] = __fadd_rn(b0, b1);
            }
            __builtin_amdgcn_wave_barrier();
            // Keep the top n_groups_used groups (stable descending).  chosen: group g -> lane g%64, bit g/64.
            uint32_t chosen = 0;
            const int ngu = p.n_groups_used < ng ? p.n_groups_used : ng;
            for (int k = 0; k < ngu; k++) {
                uint32_t bk = 0, bi = 0xFFFFFFFFu;
                for (int g = lane, t = 0; g < ng; g += kWave, t++) {
                    if (chosen & (1u << t)) continue;
                    uint32_t key = order_key(gscore[g]);
                    if (bi == 0xFFFFFFFFu || key > bk) { bk = key; bi = (uint32_t)g; }
                }
                uint32_t kmax = wave_max_u32(bi == 0xFFFFFFFFu ? 0u : bk);
                uint32_t win = wave_min_u32((bi != 0xFFFFFFFFu && bk == kmax) ? bi : 0xFFFFFFFFu);
                if (win != 0xFFFFFFFFu && (int)(win & 63u) == lane) chosen |= 1u << (win >> 6);
            }
            for (int g = lane, t = 0; g < ng; g += kWave, t++) {
                if (!(chosen & (1u << t)))
                    for (int i = g * per; i < (g + 1) * per; i++) sel[i] = ninf;
            }
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int s = 0; s < NS; s++) {
                int i = s * kWave + lane;
                if (i < n) sl[s] = sel[i];
            }
        }
        // Top n_used by (sel desc, id asc).
        uint32_t taken = 0;
#pragma unroll
        for (int s = 0; s < NS; s++)
            if (s * kWave + lane >= n) taken |= 1u << s;
        uint32_t keys[NS];
#pragma unroll
        for (int s = 0; s < NS; s++) keys[s] = order_key(sl[s]);
        for (int k = 0; k < p.n_used; k++) {
            uint32_t bk = 0, bi = 0xFFFFFFFFu;
#pragma unroll
            for (int s = 0; s < NS; s++) {
                if (taken & (1u << s)) continue;
                if (bi == 0xFFFFFFFFu || keys[s] > bk) { bk = keys[s]; bi = (uint32_t)(s * kWave + lane); }
            }
            // the winner: largest key, then smallest id = smallest slot s, then smallest lane.  One reduction for the
            // key; the id comes from ballots of the lanes that hold the key, slot by slot.
            const bool has = bi != 0xFFFFFFFFu;
            const uint32_t kmax = wave_max_u32(has ? bk : 0u);
            const bool match = has && bk == kmax;
            uint32_t win = 0xFFFFFFFFu;
            const uint64_t holders = __ballot(match);
            if (__builtin_popcountll(holders) == 1) {
                // one lane holds the largest key: its candidate is the winner
                win = (uint32_t)__builtin_amdgcn_readlane((int)bi, __builtin_ctzll(holders));
            } else {
                // several lanes hold it: smallest slot first, then smallest lane
#pragma unroll
                for (int s = 0; s < NS; s++) {
                    const uint64_t mk = __ballot(match && (int)(bi >> 6) == s);
                    if (win == 0xFFFFFFFFu && mk) win = (uint32_t)(s * kWave) + (uint32_t)__builtin_ctzll(mk);
                }
            }
            if (win == 0xFFFFFFFFu) win = 0;
            if ((int)(win & 63u) == lane) taken |= 1u << (win >> 6);
            if (lane == k) my_id = (int)win;
        }
    }
    ROUTE_STAMP(5);
    // ---- routing weights (lib.rs:3856-3861): lane k owns rank k
    const bool mine = lane < p.n_used;
    float pk = mine ? prob[my_id] : 0.0f;
    float w;
    if (p.norm_w) {
        float wsum = 0.0f;
        for (int k = 0; k < p.n_used; k++) wsum = __fadd_rn(wsum, readlane_f(pk, k));
        wsum = fmaxf(wsum, 1e-20f);
        w = __fmul_rn(__fdiv_rn(pk, wsum), p.scale);
    } else {
        w = __fmul_rn(pk, p.scale);
    }
    if (p.ep_n > 0) {
        // expert-parallel band: ids become indices into the local shard, foreign selections weigh nothing
        const bool own = my_id >= p.ep_lo && my_id < p.ep_lo + p.ep_n;
        my_id = own ? my_id - p.ep_lo : 0;
        w = own ? w : 0.0f;
    }
    if (mine) {
        if (store_global) {
            ids_out[lane] = my_id;
            w_out[lane] = w;
        }
        if (lds_ids) lds_ids[lane] = my_id;
        if (lds_w) lds_w[lane] = w;
    }
    ROUTE_STAMP(6);
    if (p.probs && store_global) {
#pragma unroll
        for (int s = 0; s < NS; s++) {
            int i = s * kWave + lane;
            if (i < n) p.probs[(size_t)row * n + i] = pr[s];
        }
    }
}

__device__ __forceinline__ void route_row_any(const RouteParams& p, int row, int lane, float* lds, const uint64_t* tab,
                                              int32_t* lds_ids = nullptr, float* lds_w = nullptr,
                                              bool store_global = true, uint64_t* stage_tab = nullptr) {
    const int n = p.n_expert;
    if (n <= 128) route_row<2>(p, row, lane, lds, tab, lds_ids, lds_w, store_global, stage_tab);
    else if (n <= 256) route_row<4>(p, row, lane, lds, tab, lds_ids, lds_w, store_global, stage_tab);
    else if (n <= 512) route_row<8>(p, row, lane, lds, tab, lds_ids, lds_w, store_global, stage_tab);
    else route_row<32>(p, row, lane, lds, tab, lds_ids, lds_w, store_global, stage_tab);
}

// ---------------------------------------------------------------------------------------------
// Plain softmax routing of one token row on two wavefronts of a block.  The serial parts of the routing are the
// left-to-right sum of the exponentials and the selection rounds; wave 0 runs the sum while wave 1 selects the
// n_used + 1 largest exponentials, (value descending, id ascending).  A probability is fl(exp / sum), a non-decreasing
// function of the exponential, so when the candidates' probabilities are strictly decreasing the first n_used are the
// reference's selection in its order (crates/infr-cpu/src/lib.rs:3847-3850); when two of them collide after the
// division (exponentials an ulp apart) or anything is not a number, wave 0 runs the complete routine instead.
// Calling sequence, the same for every thread of the block: route_duo_first on waves 0 and 1, __syncthreads(),
// route_duo_second on wave 0, __syncthreads().
struct RouteDuo {
    float psum;
    int32_t cand[16];
    float cand_e[16];
};
__host__ __device__ inline bool route_duo_ok(const RouteParams& p) {
    return p.gating == INFR_GATING_SOFTMAX && !p.exp_probs_b && !p.expert_ids && !(p.n_groups > 1 && p.n_groups_used > 0) &&
           p.n_used <= 15 && p.n_expert <= 512 && p.n_expert > p.n_used;
}
template <int NS>
__device__ __forceinline__ void route_duo_first(const RouteParams& p, int row, int wave, int lane, float* lds,
                                                uint64_t* tab, RouteDuo* duo, float (&pr)[NS]) {
    const int n = p.n_expert;
    const float* lg = p.logits + (size_t)row * n;
    const float ninf = -__builtin_huge_valf();
#pragma unroll
    for (int s = 0; s < NS; s++) {
        const int i = s * kWave + lane;
        pr[s] = i < n ? lg[i] : ninf;
    }
    if (lane < 32) tab[lane] = kExp2Table[lane];   // both waves write the same values
    __builtin_amdgcn_wave_barrier();
    float m = ninf;
#pragma unroll
    for (int s = 0; s < NS; s++) m = fmaxf(m, pr[s]);
    m = wave_max(m);
    ROUTE_STAMP(1);
#pragma unroll
    for (int s = 0; s < NS; s++) pr[s] = (s * kWave + lane < n) ? expf_libm(__fsub_rn(pr[s], m), tab) : 0.0f;
    if (wave == 0) {
        float* ex = lds;
#pragma unroll
        for (int s = 0; s < NS; s++)
            if (s * kWave + lane < n) ex[s * kWave + lane] = pr[s];
        __builtin_amdgcn_wave_barrier();
        ROUTE_STAMP(2);
        float psum = 0.0f;
        int i = 0;
        if (n >= 32 && (reinterpret_cast<uintptr_t>(ex) & 15) == 0) {
            float4 cur[8], nxt[8];
#pragma unroll
            for (int k = 0; k < 8; k++) cur[k] = reinterpret_cast<const float4*>(ex)[k];
            for (; i + 32 <= n; i += 32) {
                const int ni = i + 64 <= n ? i + 32 : i;   // past the end: re-read, unused
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
        for (; i < n; i++) psum = __fadd_rn(psum, ex[i]);
        if (lane == 0) duo->psum = psum;
        ROUTE_STAMP(3);
    } else {
        // Every lane first sorts its own NS candidates, (key descending, id ascending: adjacent exchanges on a strict
        // compare keep equal keys in id order), so a round only looks at the lane's head: one reduction for the
        // largest key, one ballot for who holds it, and the winner's list moves up by one.  An exponential is not
        // negative, so a live key has its top bit set and 0 marks an empty place.
        uint32_t key[NS], id[NS];
#pragma unroll
        for (int s = 0; s < NS; s++) {
            id[s] = (uint32_t)(s * kWave + lane);
            key[s] = (s * kWave + lane < n) ? order_key(pr[s]) : 0u;
        }
#pragma unroll
        for (int a = 0; a + 1 < NS; a++) {
#pragma unroll
            for (int b = 0; b + 1 < NS - a; b++) {
                const bool swap = key[b + 1] > key[b];
                const uint32_t hk = swap ? key[b + 1] : key[b], lk = swap ? key[b] : key[b + 1];
                const uint32_t hi = swap ? id[b + 1] : id[b], li = swap ? id[b] : id[b + 1];
                key[b] = hk; key[b + 1] = lk;
                id[b] = hi; id[b + 1] = li;
            }
        }
        for (int k = 0; k <= p.n_used; k++) {
            const uint32_t kmax = wave_max_u32(key[0]);
            const bool match = key[0] == kmax && kmax != 0u;
            const uint64_t holders = __ballot(match);
            uint32_t win;
            if (__builtin_popcountll(holders) == 1) {
                win = (uint32_t)__builtin_amdgcn_readlane((int)id[0], __builtin_ctzll(holders));
            } else {
                // several lanes hold the largest key: the smallest id among their heads (a lane's own equal keys
                // are already in id order)
                win = wave_min_u32(match ? id[0] : 0xFFFFFFFFu);
            }
            if (holders == 0 && lane == 0) {   // nothing comparable left (keys of negative NaNs): the check fails
                duo->cand[k] = 0;
                duo->cand_e[k] = __uint_as_float(0x7FC00000u);
            }
            if (match && id[0] == win) {
                duo->cand[k] = (int32_t)win;
                duo->cand_e[k] = __uint_as_float(key[0] & 0x7FFFFFFFu);   // the exponential back from its key
#pragma unroll
                for (int s = 0; s + 1 < NS; s++) {
                    key[s] = key[s + 1];
                    id[s] = id[s + 1];
                }
                key[NS - 1] = 0u;
            }
        }
    }
}
// Wave 0 after the block barrier.  False: the candidates collide (or something is not a number) and the caller runs
// route_row_any.
template <int NS>
__device__ __forceinline__ bool route_duo_second(const RouteParams& p, int row, int lane, const RouteDuo* duo,
                                                 const float (&pr)[NS], int32_t* lds_ids, float* lds_w, bool store_global) {
    const int n = p.n_expert;
    const float psum = duo->psum;
    const float pc = lane <= p.n_used ? __fdiv_rn(duo->cand_e[lane], psum) : 0.0f;
    const float nxt = __shfl_down(pc, 1, kWave);
    if (!__all(lane >= p.n_used || pc > nxt)) return false;
    ROUTE_STAMP(5);
    // routing weights (lib.rs:3856-3861): lane k owns rank k
    const bool mine = lane < p.n_used;
    int my_id = mine ? duo->cand[lane] : 0;
    const float pk = mine ? pc : 0.0f;
    float w;
    if (p.norm_w) {
        float wsum = 0.0f;
        for (int k = 0; k < p.n_used; k++) wsum = __fadd_rn(wsum, readlane_f(pk, k));
        wsum = fmaxf(wsum, 1e-20f);
        w = __fmul_rn(__fdiv_rn(pk, wsum), p.scale);
    } else {
        w = __fmul_rn(pk, p.scale);
    }
    if (p.ep_n > 0) {
        const bool own = my_id >= p.ep_lo && my_id < p.ep_lo + p.ep_n;
        my_id = own ? my_id - p.ep_lo : 0;
        w = own ? w : 0.0f;
    }
    if (mine) {
        if (store_global) {
            p.ids[(size_t)row * p.n_used + lane] = my_id;
            p.weights[(size_t)row * p.n_used + lane] = w;
        }
        if (lds_ids) lds_ids[lane] = my_id;
        if (lds_w) lds_w[lane] = w;
    }
    ROUTE_STAMP(6);
    if (p.probs && store_global) {
#pragma unroll
        for (int s = 0; s < NS; s++) {
            const int i = s * kWave + lane;
            if (i < n) p.probs[(size_t)row * n + i] = __fdiv_rn(pr[s], psum);
        }
    }
    return true;
}

// ---------------------------------------------------------------------------------------------
// Plain softmax routing of one token row by one wavefront when a CANDIDATE for the selected set is known (the
// single-launch kernel has guessed it from estimates of the logits).  The probabilities are computed as always
// (crates/infr-cpu/src/lib.rs:3747-3756: exp(l - max), the left-to-right sum, one division each); then, instead of
// n_used selection rounds, one test: if every candidate's probability is strictly above every other expert's, the
// candidates ARE the reference's selection (lib.rs:3847-3850 sorts by probability descending, ties to the lower id,
// and no tie crosses the boundary), and their ranks follow from comparing the n_used candidates with each other under
// that same order.  Otherwise (a wrong candidate set, a tie across the boundary, anything not a number) the function
// returns false and the caller runs the complete routine.  Needs n_expert == 64 * NS and n_used <= 16.
// cand: n_used distinct ids in LDS; lds: 2 * n_expert floats, 16-byte aligned.
template <int NS>
__device__ __forceinline__ bool route_softmax_checked(const RouteParams& p, int row, int lane, const int32_t* cand, float* lds,
                                                      const uint64_t* tab, int32_t* lds_ids, float* lds_w, bool store_global) {
    const int n = p.n_expert;
    const float* lg = p.logits + (size_t)row * n;
    float* ex = lds;          // [n] exponentials, then probabilities
    float pr[NS];
#pragma unroll
    for (int s = 0; s < NS; s++) pr[s] = lg[s * kWave + lane];
    float m = pr[0];
#pragma unroll
    for (int s = 1; s < NS; s++) m = fmaxf(m, pr[s]);
    m = wave_max(m);
#pragma unroll
    for (int s = 0; s < NS; s++) {
        pr[s] = expf_libm(__fsub_rn(pr[s], m), tab);
        ex[s * kWave + lane] = pr[s];
    }
    // which of this lane's experts are candidates (beside the sum's dependent adds, which leave issue slots free)
    uint32_t member = 0;
    for (int k = 0; k < p.n_used; k++) {
        const int c = cand[k];
#pragma unroll
        for (int s = 0; s < NS; s++) member |= (c == s * kWave + lane ? 1u : 0u) << s;
    }
    __builtin_amdgcn_wave_barrier();
    float psum = 0.0f;
    {
        float4 cur[8], nxt[8];
#pragma unroll
        for (int k = 0; k < 8; k++) cur[k] = reinterpret_cast<const float4*>(ex)[k];
        for (int i = 0; i < n; i += 32) {
            const int ni = i + 64 <= n ? i + 32 : i;   // past the end: re-read, unused
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
    __builtin_amdgcn_wave_barrier();
    // probabilities; the smallest among the candidates against the largest among the rest
    uint32_t lo_in = 0xFFFFFFFFu, hi_out = 0u;
#pragma unroll
    for (int s = 0; s < NS; s++) {
        pr[s] = __fdiv_rn(pr[s], psum);
        ex[s * kWave + lane] = pr[s];
        const uint32_t key = order_key(pr[s]);
        const bool in = (member >> s) & 1u;
        lo_in = in ? min(lo_in, key) : lo_in;
        hi_out = in ? hi_out : max(hi_out, key);
    }
    lo_in = wave_min_u32(lo_in);
    hi_out = wave_max_u32(hi_out);
    uint32_t cnt = 0;
#pragma unroll
    for (int s = 0; s < NS; s++) cnt += (uint32_t)__builtin_popcountll(__ballot((member >> s) & 1u));
    // a NaN among the probabilities has a key above every number's: it fails one side or the other
    const bool clean = psum == psum && lo_in > hi_out && lo_in < order_key(__builtin_huge_valf()) + 1u && (int)cnt == p.n_used;
    if (!clean) return false;
    __builtin_amdgcn_wave_barrier();
    // lane k < n_used: candidate k, its rank among the candidates (probability descending, id ascending)
    const bool own = lane < p.n_used;
    const int my_cand = own ? cand[lane] : 0;
    const float my_p = own ? ex[my_cand] : 0.0f;
    int rank = 0;
    for (int k = 0; k < p.n_used; k++) {
        const float pk = readlane_f(my_p, k);
        const int ik = __builtin_amdgcn_readlane(my_cand, k);
        rank += (pk > my_p || (pk == my_p && ik < my_cand)) ? 1 : 0;
    }
    // into rank order through LDS (the exponentials' copy is no longer needed: probabilities live in ex[], this is ex + n)
    float* by_rank_p = lds + n;
    int32_t* by_rank_id = reinterpret_cast<int32_t*>(lds + n + 16);
    if (own) {
        by_rank_p[rank] = my_p;
        by_rank_id[rank] = my_cand;
    }
    __builtin_amdgcn_wave_barrier();
    int my_id = own ? by_rank_id[lane] : 0;
    const float pk = own ? by_rank_p[lane] : 0.0f;
    // routing weights (lib.rs:3856-3861): lane k owns rank k
    float w;
    if (p.norm_w) {
        float wsum = 0.0f;
        for (int k = 0; k < p.n_used; k++) wsum = __fadd_rn(wsum, readlane_f(pk, k));
        wsum = fmaxf(wsum, 1e-20f);
        w = __fmul_rn(__fdiv_rn(pk, wsum), p.scale);
    } else {
        w = __fmul_rn(pk, p.scale);
    }
    if (p.ep_n > 0) {
        const bool in_band = my_id >= p.ep_lo && my_id < p.ep_lo + p.ep_n;
        my_id = in_band ? my_id - p.ep_lo : 0;
        w = in_band ? w : 0.0f;
    }
    if (own) {
        if (store_global) {
            p.ids[(size_t)row * p.n_used + lane] = my_id;
            p.weights[(size_t)row * p.n_used + lane] = w;
        }
        if (lds_ids) lds_ids[lane] = my_id;
        if (lds_w) lds_w[lane] = w;
    }
    if (p.probs && store_global) {
#pragma unroll
        for (int s = 0; s < NS; s++) p.probs[(size_t)row * n + s * kWave + lane] = pr[s];
    }
    return true;
}

// LDS floats route_row_any needs behind the 64-float exp table.
__host__ __device__ inline size_t route_scratch_floats(int n_expert, int n_groups) {
    return (size_t)2 * n_expert + (size_t)(n_groups > 0 ? n_groups : 0);
}

}  // namespace infr

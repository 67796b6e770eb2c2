// Router: logits = router . x with the reference's exact f32 accumulation order, then
// gating -> top-k -> renormalised routing weights, one wavefront per token row.
//
// The selected expert ids are an integer contract, so everything that feeds the comparison
// is computed in the reference's operation order: 8 independent FMA chains over
// i = j (mod 8), chains summed 0..7 (crates/infr-cpu/src/kernels.rs:6568-6583), softmax as
// exp(l - max) / sequential sum (crates/infr-cpu/src/lib.rs:3747-3756), selection by
// (probability descending, id ascending) = Rust's stable sort (lib.rs:3847-3850).
#include "device_common.h"
#include "kernels.h"

namespace infr {

// Block = 256 threads, EPB experts per block, RPB token rows per pass (EPB*8*RPB <= 256).
// LDS: EPB decoded router rows (stride ne+8 floats: the 8-float pad puts the EPB rows on
// distinct banks for the 8-wide chain reads) followed by RPB activation rows.
template <int EPB>
__global__ __launch_bounds__(256) void router_logits_kernel(const uint8_t* __restrict__ router, int rdt,
                                                            size_t row_bytes, const float* __restrict__ x, int ne,
                                                            int n_expert, int rows, int rpb,
                                                            float* __restrict__ logits) {
    extern __shared__ float lds[];
    const int wstride = ne + 8;
    float* w = lds;
    float* xs = lds + EPB * wstride;
    const int tid = threadIdx.x;
    const int e0 = blockIdx.x * EPB;

    for (int idx = tid; idx < EPB * ne; idx += 256) {
        int e = idx / ne, k = idx - e * ne;
        float v = 0.0f;
        if (e0 + e < n_expert) v = decode_elem(rdt, router + (size_t)(e0 + e) * row_bytes, (uint32_t)k);
        w[e * wstride + k] = v;
    }
    const int rsub = tid / (EPB * 8);
    const int e = (tid >> 3) % EPB;
    const int j = tid & 7;
    const int lane = tid & 63;
    const int chunks = ne >> 3;
    for (int r0 = blockIdx.y * rpb; r0 < rows; r0 += gridDim.y * rpb) {
        __syncthreads();
        for (int idx = tid; idx < rpb * ne; idx += 256) {
            int rr = idx / ne, k = idx - rr * ne;
            xs[idx] = (r0 + rr < rows) ? x[(size_t)(r0 + rr) * ne + k] : 0.0f;
        }
        __syncthreads();
        float acc = 0.0f;
        const bool live = rsub < rpb;
        const float* wp = w + e * wstride;
        const float* xp = xs + (live ? rsub : 0) * ne;
        if (live) {
            for (int c = 0; c < chunks; c++) acc = __fmaf_rn(wp[8 * c + j], xp[8 * c + j], acc);
        }
        float s = 0.0f;
#pragma unroll
        for (int jj = 0; jj < 8; jj++) s = __fadd_rn(s, __shfl(acc, (lane & ~7) + jj, kWave));
        if (live && j == 0) {
            for (int i = chunks * 8; i < ne; i++) s = __fmaf_rn(wp[i], xp[i], s);
            if (r0 + rsub < rows && e0 + e < n_expert) logits[(size_t)(r0 + rsub) * n_expert + e0 + e] = s;
        }
    }
}

bool launch_router_logits(hipStream_t s, const uint8_t* router, int rdt, size_t row_bytes, const float* x, int ne,
                          int n_expert, int rows, float* logits) {
    // Decode (few rows): many small blocks.  Batches: 8 experts x 4 rows per pass.
    int epb = rows <= 2 ? 2 : 8;
    int rpb = rows <= 2 ? rows : 4;
    const size_t budget = 140 * 1024;
    auto lds_bytes = [&](int e, int r) { return ((size_t)e * (ne + 8) + (size_t)r * ne) * sizeof(float); };
    while (lds_bytes(epb, rpb) > budget && rpb > 1) rpb >>= 1;
    while (lds_bytes(epb, rpb) > budget && epb > 1) epb >>= 1;
    if (lds_bytes(epb, rpb) > budget) return false;
    size_t lds = lds_bytes(epb, rpb);
    int gx = (n_expert + epb - 1) / epb;
    int passes = (rows + rpb - 1) / rpb;
    int gy = passes;
    int cap = (1024 + gx - 1) / gx;
    if (gy > cap) gy = cap;
    if (gy < 1) gy = 1;
    dim3 grid(gx, gy), block(256);
#define LAUNCH_RL(E)                                                                                               \
    do {                                                                                                           \
        static bool attr_set = false;                                                                              \
        if (!attr_set) {                                                                                           \
            (void)hipFuncSetAttribute((const void*)router_logits_kernel<E>,                                         \
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)budget);                   \
            attr_set = true;                                                                                       \
        }                                                                                                          \
        hipLaunchKernelGGL(router_logits_kernel<E>, grid, block, lds, s, router, rdt, row_bytes, x, ne, n_expert,  \
                           rows, rpb, logits);                                                                     \
    } while (0)
    switch (epb) {
        case 8: LAUNCH_RL(8); break;
        case 4: LAUNCH_RL(4); break;
        case 2: LAUNCH_RL(2); break;
        default: LAUNCH_RL(1); break;
    }
#undef LAUNCH_RL
    return true;
}

// (value, index) ordering of the reference's stable descending sort: larger value first,
// equal values keep ascending index.
__device__ __forceinline__ bool better(float v, int i, float bv, int bi) {
    return bi < 0 || v > bv || (v == bv && i < bi);
}

__device__ __forceinline__ void wave_argbest(float& v, int& i) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        float ov = __shfl_xor(v, off, kWave);
        int oi = __shfl_xor(i, off, kWave);
        if (oi >= 0 && better(ov, oi, v, i)) {
            v = ov;
            i = oi;
        }
    }
}

// One wavefront per token row.  n_expert <= 2048 (32 candidates per lane).
__global__ __launch_bounds__(64) void route_kernel(RouteParams p) {
    extern __shared__ float lds[];
    const int n = p.n_expert;
    float* prob = lds;
    float* sel = lds + n;
    float* gscore = sel + n;  // n_groups
    const int row = blockIdx.x;
    const int lane = threadIdx.x;
    const float* lg = p.logits + (size_t)row * n;

    // ---- gating (lib.rs:3746-3774)
    if (p.gating == INFR_GATING_SOFTMAX) {
        float m = -__builtin_huge_valf();
        for (int i = lane; i < n; i += kWave) m = fmaxf(m, lg[i]);
        m = wave_max(m);
        for (int i = lane; i < n; i += kWave) prob[i] = expf_libm(__fsub_rn(lg[i], m));
        __syncthreads();
        float psum = 0.0f;
        if (lane == 0) {
            for (int i = 0; i < n; i++) psum = __fadd_rn(psum, prob[i]);
        }
        psum = __shfl(psum, 0, kWave);
        for (int i = lane; i < n; i += kWave) prob[i] = __fdiv_rn(prob[i], psum);
    } else if (p.gating == INFR_GATING_SIGMOID) {
        for (int i = lane; i < n; i += kWave) prob[i] = __fdiv_rn(1.0f, __fadd_rn(1.0f, expf_libm(-lg[i])));
    } else {
        for (int i = lane; i < n; i += kWave) {
            float v = lg[i];
            float sp = v > 20.0f ? v : logf(__fadd_rn(1.0f, expf_libm(v)));
            prob[i] = __fsqrt_rn(sp);
        }
    }
    __syncthreads();

    int32_t* ids_out = p.ids + (size_t)row * p.n_used;
    float* w_out = p.weights + (size_t)row * p.n_used;
    if (p.expert_ids) {
        // Hash routing (lib.rs:3776-3793): the supplied ids are the selection, in table order.
        if (lane < p.n_used) {
            int e = p.expert_ids[(size_t)row * p.n_used + lane];
            if (e < 0) e = 0;
            if (e >= n) e = n - 1;
            ids_out[lane] = e;
        }
    } else {
        // lib.rs:3797-3806: bias on a selection-only copy.
        for (int i = lane; i < n; i += kWave)
            sel[i] = p.exp_probs_b ? __fadd_rn(prob[i], p.exp_probs_b[i]) : prob[i];
        __syncthreads();
        // lib.rs:3809-3846: group-limited routing.
        if (p.n_groups > 1 && p.n_groups_used > 0) {
            const int ng = p.n_groups, per = n / ng;
            for (int g = lane; g < ng; g += kWave) {
                float b0 = -__builtin_huge_valf(), b1 = -__builtin_huge_valf();
                for (int i = g * per; i < (g + 1) * per; i++) {
                    float sv = sel[i];
                    if (sv > b0) { b1 = b0; b0 = sv; }
                    else if (sv > b1) { b1 = sv; }
                }
                gscore[g] = __fadd_rn(b0, b1);
            }
            __syncthreads();
            // Keep the top n_groups_used groups (stable descending), mask the others.
            // chosen flags live in a per-lane bitmask: group g -> lane g%64, bit g/64.
            uint32_t chosen = 0;
            const int ngu = p.n_groups_used < ng ? p.n_groups_used : ng;
            for (int k = 0; k < ngu; k++) {
                float bv = 0.0f;
                int bi = -1;
                for (int g = lane, t = 0; g < ng; g += kWave, t++) {
                    if (chosen & (1u << t)) continue;
                    float v = gscore[g];
                    if (better(v, g, bv, bi)) { bv = v; bi = g; }
                }
                wave_argbest(bv, bi);
                if (bi >= 0 && (bi & 63) == lane) chosen |= 1u << (bi >> 6);
            }
            for (int g = lane, t = 0; g < ng; g += kWave, t++) {
                if (!(chosen & (1u << t)))
                    for (int i = g * per; i < (g + 1) * per; i++) sel[i] = -__builtin_huge_valf();
            }
            __syncthreads();
        }
        // Top n_used by (sel desc, id asc).
        uint32_t taken = 0;
        for (int k = 0; k < p.n_used; k++) {
            float bv = 0.0f;
            int bi = -1;
            for (int i = lane, t = 0; i < n; i += kWave, t++) {
                if (taken & (1u << t)) continue;
                float v = sel[i];
                if (better(v, i, bv, bi)) { bv = v; bi = i; }
            }
            wave_argbest(bv, bi);
            if (bi < 0) bi = 0;
            if ((bi & 63) == lane) taken |= 1u << (bi >> 6);
            if (lane == 0) ids_out[k] = bi;
        }
    }
    __syncthreads();
    // ---- routing weights (lib.rs:3856-3861)
    if (lane == 0) {
        if (p.norm_w) {
            float wsum = 0.0f;
            for (int k = 0; k < p.n_used; k++) wsum = __fadd_rn(wsum, prob[ids_out[k]]);
            wsum = fmaxf(wsum, 1e-20f);
            for (int k = 0; k < p.n_used; k++) w_out[k] = __fmul_rn(__fdiv_rn(prob[ids_out[k]], wsum), p.scale);
        } else {
            for (int k = 0; k < p.n_used; k++) w_out[k] = __fmul_rn(prob[ids_out[k]], p.scale);
        }
    }
    if (p.probs) {
        for (int i = lane; i < n; i += kWave) p.probs[(size_t)row * n + i] = prob[i];
    }
}

void launch_route(hipStream_t s, const RouteParams& p) {
    size_t lds = ((size_t)2 * p.n_expert + (size_t)(p.n_groups > 0 ? p.n_groups : 0)) * sizeof(float);
    hipLaunchKernelGGL(route_kernel, dim3(p.rows), dim3(64), lds, s, p);
}

}  // namespace infr

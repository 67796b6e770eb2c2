// Dense Op::Linear GEMV for every affine GGUF format (Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q2_K, Q3_K,
// Q4_K, Q5_K, Q6_K) and the scale-times-code formats (IQ4_NL, IQ4_XS, MXFP4, NVFP4, TQ1_0, TQ2_0, Q2_0,
// their codes shifted to unsigned bytes) through one common shape: a row is cut into 32-element units; a unit decodes to
// 32 unsigned byte codes (eight dwords) plus one (scale, min) pair per 16 elements, and
//     dot(unit, x) = sum_h  sc[h] * sum_{e in half h} code[e] * x[e]  +  mn[h] * sum_{e in half h} x[e].
// The byte -> float conversion is one instruction per element (the compiler selects the
// byte-lane convert for (q >> 8b) & 0xFF), the sums of x per 16 elements are computed once per
// block while the activation row is staged in LDS, and the formats only differ in how the eight
// dwords and the two pairs are cut out of the block (crates/infr-gguf/src/dequant.rs:137-389, :499-1073).
//
// The formats with their own integer-dot kernels (Q4_K, Q6_K, Q8_0) only come here for shapes those
// kernels do not take.  Work split: a block of four waves stages up to four activation rows, each
// wave walks output rows two at a time, lanes stride over the units of a row.
#include "device_common.h"
#include "kernels.h"
#include "route.h"
#include "units.h"

namespace infr {

namespace {

constexpr int kUnitStride = 36;   // dwords between the x values of consecutive units in LDS: 16 lanes, 64 banks
constexpr int kRowsPerWave = 2;   // output rows a wave has in flight
constexpr int kRowsPerBlock = 16; // 4 waves x 2 rows x 2 rounds

// T activation rows per block (grid.y walks chunks of T); dst[r, o] = x[r] . W[o] (+ addend[r, o]).
template <int DT, int T>
__global__ __launch_bounds__(256) void linear_units_kernel(const float* __restrict__ x, const uint8_t* __restrict__ w,
                                                           size_t row_bytes, int m, int in_f, int out_f, float* dst,
                                                           const float* addend, int rows_per_block) {
    extern __shared__ float lds[];
    const int n_units = in_f >> 5;
    float* xs = lds;                                   // [T][n_units][kUnitStride]
    float* xsum = lds + (size_t)T * n_units * kUnitStride;   // [T][2 * n_units]
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int r0 = blockIdx.y * T;
    // stage: one thread per 16 elements (a half unit), which also gives that half's sum
    for (int idx = tid; idx < T * 2 * n_units; idx += 256) {
        const int tr = idx / (2 * n_units), hu = idx - tr * 2 * n_units;
        float4 v[4];
        float s = 0.0f;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            v[k] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (r0 + tr < m) v[k] = reinterpret_cast<const float4*>(x + (size_t)(r0 + tr) * in_f + 16 * hu)[k];
            s += (v[k].x + v[k].y) + (v[k].z + v[k].w);
        }
        float* d = xs + ((size_t)tr * n_units + (hu >> 1)) * kUnitStride + 16 * (hu & 1);
#pragma unroll
        for (int k = 0; k < 4; k++) reinterpret_cast<float4*>(d)[k] = v[k];
        xsum[idx] = s;
    }
    __syncthreads();
    const int row_base = blockIdx.x * rows_per_block;
    for (int round = 0; round < rows_per_block / (4 * kRowsPerWave); round++) {
        const int o0 = row_base + (round * 4 + wave) * kRowsPerWave;
        if (o0 >= out_f) break;
        float acc[kRowsPerWave][T];
#pragma unroll
        for (int a = 0; a < kRowsPerWave; a++)
#pragma unroll
            for (int tr = 0; tr < T; tr++) acc[a][tr] = 0.0f;
        for (int u = lane; u < n_units; u += kWave) {
            Unit t[kRowsPerWave];
#pragma unroll
            for (int a = 0; a < kRowsPerWave; a++) {
                const int o = o0 + a < out_f ? o0 + a : out_f - 1;   // a clamped duplicate, dropped at the store
                load_unit<DT>(w + (size_t)o * row_bytes, u, t[a]);
            }
#pragma unroll
            for (int tr = 0; tr < T; tr++) {
                const float* xu = xs + ((size_t)tr * n_units + u) * kUnitStride;
                float s[kRowsPerWave][2];
#pragma unroll
                for (int a = 0; a < kRowsPerWave; a++) s[a][0] = s[a][1] = 0.0f;
#pragma unroll
                for (int k = 0; k < 8; k++) {
                    const float4 xv = reinterpret_cast<const float4*>(xu)[k];
#pragma unroll
                    for (int a = 0; a < kRowsPerWave; a++) {
                        const uint32_t q = t[a].q[k];
                        float& sh = s[a][k >> 2];
                        sh = fmaf((float)(q & 0xFFu), xv.x, sh);
                        sh = fmaf((float)((q >> 8) & 0xFFu), xv.y, sh);
                        sh = fmaf((float)((q >> 16) & 0xFFu), xv.z, sh);
                        sh = fmaf((float)(q >> 24), xv.w, sh);
                    }
                }
                const float2 xsu = *reinterpret_cast<const float2*>(xsum + (size_t)tr * 2 * n_units + 2 * u);
#pragma unroll
                for (int a = 0; a < kRowsPerWave; a++)
                    acc[a][tr] += (t[a].sc[0] * s[a][0] + t[a].mn[0] * xsu.x) + (t[a].sc[1] * s[a][1] + t[a].mn[1] * xsu.y);
            }
        }
#pragma unroll
        for (int a = 0; a < kRowsPerWave; a++)
#pragma unroll
            for (int tr = 0; tr < T; tr++) {
                const float y = wave_sum(acc[a][tr]);
                if (lane == 0 && o0 + a < out_f && r0 + tr < m) {
                    const size_t oi = (size_t)(r0 + tr) * out_f + o0 + a;
                    dst[oi] = addend ? __fadd_rn(addend[oi], y) : y;
                }
            }
    }
}

// Op::MoeFfn's two expert GEMV stages on units, for expert banks in formats without an integer-dot
// kernel: grid.y = (row, rank) pair; the block stages that pair's activation row (x for gate/up, h for
// down) and its waves walk the selected expert's rows.  gate/up: h[pair, f] = act(gate . x) * (up . x);
// down: y[pair, o] = down . h[pair] (* down_scale[e]); the rank-ordered weighted sum is a separate
// combine launch.  An expert id outside the bank (possible with caller-given ids) yields zeros.
template <int DT, bool GATE_UP>
__global__ __launch_bounds__(256) void moe_units_kernel(MoeGemvParams p, size_t row_bytes, int kRB) {
    // output rows a wave has in flight: two rows of two matrices for gate/up (two rounds per 16-row tile), four
    // rows for down (one round; measured 11.5 -> 10.0 us on 2880 x 2880 MXFP4 banks, four rows of gate/up are slower)
    constexpr int kRW = GATE_UP ? 2 : 4;
    extern __shared__ float lds[];
    const int in_f = GATE_UP ? p.ne : p.nff, out_f = GATE_UP ? p.nff : p.ne;
    const int n_units = in_f >> 5;
    float* xs = lds;
    float* xsum = lds + (size_t)n_units * kUnitStride;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int pair = blockIdx.y, r = pair / p.n_used;
    const float* xrow = GATE_UP ? p.x + (size_t)r * p.ne : p.h + (size_t)pair * p.nff;
    float* out = GATE_UP ? p.h + (size_t)pair * p.nff : p.y + (size_t)pair * p.ne;
    const int row_base = blockIdx.x * kRB;
    // gate/up with routing folded in: the block routes its token row itself (one wave, the same routine as the
    // routing kernel) while the activation row is on its way; block column 0 of a row's first pair stores the result
    const bool routes = GATE_UP && p.route_inline;
    __shared__ uint64_t s_tab[32];
    __shared__ int32_t s_ids[64];
    __shared__ float s_w[64];
    int e = 0;
    if (!routes) {
        e = p.ids[pair];
        if (e < 0 || e >= p.n_expert) {
            for (int o = row_base + tid; o < min(row_base + kRB, out_f); o += 256) out[o] = 0.0f;
            return;
        }
    } else if (wave == 3) {
        // the last wave has the smallest share of the activation row to stage (none up to 3072 elements): it
        // routes while the others stage
        if (lane < 32) s_tab[lane] = kExp2Table[lane];
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
        __builtin_amdgcn_wave_barrier();
        const int slot0 = pair - r * p.n_used;
        route_row_any(p.route, r, lane, xsum + 2 * n_units, s_tab, s_ids, s_w, blockIdx.x == 0 && slot0 == 0);
    }
    for (int hu = tid; hu < 2 * n_units; hu += 256) {
        float4 v[4];
        float sm = 0.0f;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            v[k] = reinterpret_cast<const float4*>(xrow + 16 * hu)[k];
            sm += (v[k].x + v[k].y) + (v[k].z + v[k].w);
        }
        float* d = xs + (size_t)(hu >> 1) * kUnitStride + 16 * (hu & 1);
#pragma unroll
        for (int k = 0; k < 4; k++) reinterpret_cast<float4*>(d)[k] = v[k];
        xsum[hu] = sm;
    }
    __syncthreads();
    float w_before = 1.0f;
    if constexpr (GATE_UP) {
        if (routes) {
            const int slot = pair - r * p.n_used;
            e = s_ids[slot];
            w_before = s_w[slot];
            if (e < 0 || e >= p.n_expert) {
                for (int o = row_base + tid; o < min(row_base + kRB, out_f); o += 256) out[o] = 0.0f;
                return;
            }
        } else if (p.weight_before) {
            w_before = p.weights[pair];
        }
    }
    constexpr int M = GATE_UP ? 2 : 1;   // matrices per output row
    const uint8_t* base[M];
    base[0] = (GATE_UP ? p.gate + (size_t)e * p.gate_stride : p.down + (size_t)e * p.down_stride);
    if constexpr (GATE_UP) base[1] = p.up + (size_t)e * p.up_stride;
    for (int round = 0; round < kRB / (4 * kRW); round++) {
        const int o0 = row_base + (round * 4 + wave) * kRW;
        if (o0 >= out_f) break;
        float acc[kRW][M];
#pragma unroll
        for (int a = 0; a < kRW; a++)
#pragma unroll
            for (int mi = 0; mi < M; mi++) acc[a][mi] = 0.0f;
        for (int u = lane; u < n_units; u += kWave) {
            Unit t[kRW][M];
#pragma unroll
            for (int a = 0; a < kRW; a++) {
                const int o = o0 + a < out_f ? o0 + a : out_f - 1;
#pragma unroll
                for (int mi = 0; mi < M; mi++) load_unit<DT>(base[mi] + (size_t)o * row_bytes, u, t[a][mi]);
            }
            const float* xu = xs + (size_t)u * kUnitStride;
            float sh[kRW][M][2];
#pragma unroll
            for (int a = 0; a < kRW; a++)
#pragma unroll
                for (int mi = 0; mi < M; mi++) sh[a][mi][0] = sh[a][mi][1] = 0.0f;
#pragma unroll
            for (int k = 0; k < 8; k++) {
                const float4 xv = reinterpret_cast<const float4*>(xu)[k];
#pragma unroll
                for (int a = 0; a < kRW; a++)
#pragma unroll
                    for (int mi = 0; mi < M; mi++) {
                        const uint32_t q = t[a][mi].q[k];
                        float& v = sh[a][mi][k >> 2];
                        v = fmaf((float)(q & 0xFFu), xv.x, v);
                        v = fmaf((float)((q >> 8) & 0xFFu), xv.y, v);
                        v = fmaf((float)((q >> 16) & 0xFFu), xv.z, v);
                        v = fmaf((float)(q >> 24), xv.w, v);
                    }
            }
            const float2 xsu = *reinterpret_cast<const float2*>(xsum + 2 * u);
#pragma unroll
            for (int a = 0; a < kRW; a++)
#pragma unroll
                for (int mi = 0; mi < M; mi++)
                    acc[a][mi] += (t[a][mi].sc[0] * sh[a][mi][0] + t[a][mi].mn[0] * xsu.x) +
                                  (t[a][mi].sc[1] * sh[a][mi][1] + t[a][mi].mn[1] * xsu.y);
        }
#pragma unroll
        for (int a = 0; a < kRW; a++) {
            float v[M];
#pragma unroll
            for (int mi = 0; mi < M; mi++) v[mi] = wave_sum(acc[a][mi]);
            if (lane == 0 && o0 + a < out_f) {
                if constexpr (GATE_UP) {
                    if (p.weight_before) {
                        v[0] = __fmul_rn(w_before, v[0]);
                        v[1] = __fmul_rn(w_before, v[1]);
                    }
                    out[o0 + a] = gated_act_fn(p.act, p.has_clamp, p.clamp, v[0], v[1]);
                } else {
                    out[o0 + a] = p.down_scale ? __fmul_rn(v[0], p.down_scale[e]) : v[0];
                }
            }
        }
    }
}

// The (expert, chunk) a block works on when an expert's bucket [offsets[e], offsets[e+1]) is cut into
// chunks of `chunk` tokens and the chunks of all experts are numbered in order.  Every wave computes it
// for itself (lanes share out the experts, a prefix sum over the lanes finds the owner); false past the
// last chunk (the grid is an upper bound).
__device__ __forceinline__ bool find_chunk(const int32_t* __restrict__ offsets, int n_expert, int chunk, int item, int lane,
                                           int& e_out, int& p0, int& cnt) {
    const int epl = (n_expert + 63) >> 6;
    const int e_lo = lane * epl, e_hi = min(n_expert, e_lo + epl);
    int mine = 0;
    for (int e = e_lo; e < e_hi; e++) mine += (offsets[e + 1] - offsets[e] + chunk - 1) / chunk;
    int incl = mine;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const int o = __shfl_up(incl, d, 64);
        if (lane >= d) incl += o;
    }
    const unsigned long long past = __ballot(incl > item);
    if (past == 0) return false;
    const int owner = __ffsll((long long)past) - 1;
    int rem = item - (__shfl(incl, owner, 64) - __shfl(mine, owner, 64));
    const int o_lo = owner * epl, o_hi = min(n_expert, o_lo + epl);
    for (int e = o_lo; e < o_hi; e++) {
        const int n = offsets[e + 1] - offsets[e];
        const int nc = (n + chunk - 1) / chunk;
        if (rem < nc) {
            e_out = e;
            p0 = offsets[e] + rem * chunk;
            cnt = min(chunk, n - rem * chunk);
            return true;
        }
        rem -= nc;
    }
    return false;
}

// Batches: the same two stages over expert buckets.  A block takes one 16-row tile of one expert and up
// to T tokens of that expert's bucket: the tile's units are decoded once and dotted with each token, so an
// expert's rows are fetched once per T tokens instead of once per pair.  h and y are in bucket order
// (position t of the bucket tables), as on the matrix-core path; launch_unbucket_combine maps them back.
template <int DT, bool GATE_UP, int T>
__global__ __launch_bounds__(256) void moe_units_bucketed_kernel(MoeGemvParams p, size_t row_bytes, int n_tiles) {
    extern __shared__ float lds[];
    const int in_f = GATE_UP ? p.ne : p.nff, out_f = GATE_UP ? p.nff : p.ne;
    const int n_units = in_f >> 5;
    float* xs = lds;                                           // [T][n_units][kUnitStride]
    float* xsum = lds + (size_t)T * n_units * kUnitStride;     // [T][2 * n_units]
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int tile = (int)(blockIdx.x % (unsigned)n_tiles), item = (int)(blockIdx.x / (unsigned)n_tiles);
    int e, p0, nt;
    if (!find_chunk(p.bk_offsets, p.n_expert, T, item, lane, e, p0, nt)) return;
    for (int idx = tid; idx < T * 2 * n_units; idx += 256) {
        const int tr = idx / (2 * n_units), hu = idx - tr * 2 * n_units;
        const int pos = p0 + min(tr, nt - 1);
        const float* xrow = GATE_UP ? p.x + (size_t)(p.bk_pair_src[pos] / p.n_used) * p.ne : p.h + (size_t)pos * p.nff;
        float4 v[4];
        float sm = 0.0f;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            v[k] = reinterpret_cast<const float4*>(xrow + 16 * hu)[k];
            sm += (v[k].x + v[k].y) + (v[k].z + v[k].w);
        }
        float* d = xs + ((size_t)tr * n_units + (hu >> 1)) * kUnitStride + 16 * (hu & 1);
#pragma unroll
        for (int k = 0; k < 4; k++) reinterpret_cast<float4*>(d)[k] = v[k];
        xsum[idx] = sm;
    }
    __syncthreads();
    constexpr int M = GATE_UP ? 2 : 1;
    const uint8_t* base[M];
    base[0] = (GATE_UP ? p.gate + (size_t)e * p.gate_stride : p.down + (size_t)e * p.down_stride);
    if constexpr (GATE_UP) base[1] = p.up + (size_t)e * p.up_stride;
    const int row_base = tile * kRowsPerBlock;
    for (int round = 0; round < kRowsPerBlock / (4 * kRowsPerWave); round++) {
        const int o0 = row_base + (round * 4 + wave) * kRowsPerWave;
        if (o0 >= out_f) break;
        float acc[kRowsPerWave][M][T];
#pragma unroll
        for (int a = 0; a < kRowsPerWave; a++)
#pragma unroll
            for (int mi = 0; mi < M; mi++)
#pragma unroll
                for (int tr = 0; tr < T; tr++) acc[a][mi][tr] = 0.0f;
        for (int u = lane; u < n_units; u += kWave) {
            Unit t[kRowsPerWave][M];
#pragma unroll
            for (int a = 0; a < kRowsPerWave; a++) {
                const int o = o0 + a < out_f ? o0 + a : out_f - 1;
#pragma unroll
                for (int mi = 0; mi < M; mi++) load_unit<DT>(base[mi] + (size_t)o * row_bytes, u, t[a][mi]);
            }
#pragma unroll
            for (int tr = 0; tr < T; tr++) {
                const float* xu = xs + ((size_t)tr * n_units + u) * kUnitStride;
                float sh[kRowsPerWave][M][2];
#pragma unroll
                for (int a = 0; a < kRowsPerWave; a++)
#pragma unroll
                    for (int mi = 0; mi < M; mi++) sh[a][mi][0] = sh[a][mi][1] = 0.0f;
#pragma unroll
                for (int k = 0; k < 8; k++) {
                    const float4 xv = reinterpret_cast<const float4*>(xu)[k];
#pragma unroll
                    for (int a = 0; a < kRowsPerWave; a++)
#pragma unroll
                        for (int mi = 0; mi < M; mi++) {
                            const uint32_t q = t[a][mi].q[k];
                            float& v = sh[a][mi][k >> 2];
                            v = fmaf((float)(q & 0xFFu), xv.x, v);
                            v = fmaf((float)((q >> 8) & 0xFFu), xv.y, v);
                            v = fmaf((float)((q >> 16) & 0xFFu), xv.z, v);
                            v = fmaf((float)(q >> 24), xv.w, v);
                        }
                }
                const float2 xsu = *reinterpret_cast<const float2*>(xsum + (size_t)tr * 2 * n_units + 2 * u);
#pragma unroll
                for (int a = 0; a < kRowsPerWave; a++)
#pragma unroll
                    for (int mi = 0; mi < M; mi++)
                        acc[a][mi][tr] += (t[a][mi].sc[0] * sh[a][mi][0] + t[a][mi].mn[0] * xsu.x) +
                                          (t[a][mi].sc[1] * sh[a][mi][1] + t[a][mi].mn[1] * xsu.y);
            }
        }
#pragma unroll
        for (int a = 0; a < kRowsPerWave; a++)
#pragma unroll
            for (int tr = 0; tr < T; tr++) {
                float v[M];
#pragma unroll
                for (int mi = 0; mi < M; mi++) v[mi] = wave_sum(acc[a][mi][tr]);
                if (lane == 0 && o0 + a < out_f && tr < nt) {
                    const int pos = p0 + tr;
                    if constexpr (GATE_UP) {
                        if (p.weight_before) {
                            const float wp = p.weights[p.bk_pair_src[pos]];
                            v[0] = __fmul_rn(wp, v[0]);
                            v[1] = __fmul_rn(wp, v[1]);
                        }
                        p.h[(size_t)pos * p.nff + o0 + a] = gated_act_fn(p.act, p.has_clamp, p.clamp, v[0], v[1]);
                    } else {
                        p.y[(size_t)pos * p.ne + o0 + a] = p.down_scale ? __fmul_rn(v[0], p.down_scale[e]) : v[0];
                    }
                }
            }
    }
}

template <int DT, bool GATE_UP, int T>
void launch_moe_units_bucketed_t(hipStream_t s, const MoeGemvParams& p, int n_pairs) {
    const int in_f = GATE_UP ? p.ne : p.nff, out_f = GATE_UP ? p.nff : p.ne;
    int be = 1, bb = 4;
    block_geometry(DT, &be, &bb);
    const size_t row_bytes = (size_t)(in_f / be) * bb;
    INFR_LDS_LIMIT((moe_units_bucketed_kernel<DT, GATE_UP, T>), 160 * 1024);
    const int n_tiles = (out_f + kRowsPerBlock - 1) / kRowsPerBlock;
    // every expert with tokens has at most one ragged chunk: chunks <= pairs / T + min(experts, pairs)
    const long items = (long)n_pairs / T + (p.n_expert < n_pairs ? p.n_expert : n_pairs);
    dim3 grid((unsigned)(items * n_tiles)), block(256);
    INFR_LAUNCH((moe_units_bucketed_kernel<DT, GATE_UP, T>), grid, block, (size_t)T * (in_f >> 5) * (kUnitStride + 2) * sizeof(float),
                s, p, row_bytes, n_tiles);
}

template <int DT, bool GATE_UP>
void launch_moe_units_bucketed_dt(hipStream_t s, const MoeGemvParams& p, int n_pairs) {
    const int in_f = GATE_UP ? p.ne : p.nff;
    const size_t per_token = (size_t)(in_f >> 5) * (kUnitStride + 2) * sizeof(float), budget = 80 * 1024;
    if (8 * per_token <= budget) launch_moe_units_bucketed_t<DT, GATE_UP, 8>(s, p, n_pairs);
    else if (4 * per_token <= budget) launch_moe_units_bucketed_t<DT, GATE_UP, 4>(s, p, n_pairs);
    else launch_moe_units_bucketed_t<DT, GATE_UP, 2>(s, p, n_pairs);
}

template <bool GATE_UP>
void launch_moe_units_bucketed_any(hipStream_t s, int dt, const MoeGemvParams& p, int n_pairs) {
    switch (dt) {
#define INFR_UNITS(D) case D: launch_moe_units_bucketed_dt<D, GATE_UP>(s, p, n_pairs); break;
        INFR_FOR_UNIT_FORMATS(INFR_UNITS)
#undef INFR_UNITS
        default: break;
    }
}

// Decode: the down stage and the rank-ordered weighted sum of a token row in one launch.  grid.x = tiles of 16
// output elements, grid.y = token row; sixteen waves share out the (slot, four-row group) items of the tile, each
// dot computed exactly as moe_units_kernel<DT, false> computes it (same lane-to-unit map, same sums), so the
// result has the bits of that kernel followed by the combine kernel.  The row's n_used activation rows h are
// staged once per block.
constexpr int kDcRows = 4;
template <int DT, int kDcTile>
__global__ __launch_bounds__(1024) void moe_down_combine_units_kernel(MoeGemvParams p, size_t row_bytes) {
    extern __shared__ float lds[];
    const int n_units = p.nff >> 5, K = p.n_used;
    float* xs = lds;                                              // [K][n_units][kUnitStride]
    float* xsum = xs + (size_t)K * n_units * kUnitStride;         // [K][2 * n_units]
    float* ys = xsum + (size_t)K * 2 * n_units;                   // [K][kDcTile]
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int r = blockIdx.y, row_base = blockIdx.x * kDcTile;
    for (int idx = tid; idx < K * 2 * n_units; idx += 1024) {
        const int k = idx / (2 * n_units), hu = idx - k * 2 * n_units;
        const float* xrow = p.h + ((size_t)r * K + k) * p.nff;
        float4 v[4];
        float sm = 0.0f;
#pragma unroll
        for (int q = 0; q < 4; q++) {
            v[q] = reinterpret_cast<const float4*>(xrow + 16 * hu)[q];
            sm += (v[q].x + v[q].y) + (v[q].z + v[q].w);
        }
        float* d = xs + ((size_t)k * n_units + (hu >> 1)) * kUnitStride + 16 * (hu & 1);
#pragma unroll
        for (int q = 0; q < 4; q++) reinterpret_cast<float4*>(d)[q] = v[q];
        xsum[idx] = sm;
    }
    __syncthreads();
    constexpr int kGroups = kDcTile / kDcRows;
    for (int it = wave; it < K * kGroups; it += 16) {
        const int k = it / kGroups, o0 = row_base + (it - k * kGroups) * kDcRows;
        if (o0 >= p.ne) continue;
        const int e = p.ids[(size_t)r * K + k];
        float v[kDcRows];
#pragma unroll
        for (int a = 0; a < kDcRows; a++) v[a] = 0.0f;
        if (e >= 0 && e < p.n_expert) {   // an id outside the bank contributes zeros, as in the separate kernels
            const uint8_t* base = p.down + (size_t)e * p.down_stride;
            const float* xk = xs + (size_t)k * n_units * kUnitStride;
            const float* sk = xsum + (size_t)k * 2 * n_units;
            float acc[kDcRows];
#pragma unroll
            for (int a = 0; a < kDcRows; a++) acc[a] = 0.0f;
            for (int u = lane; u < n_units; u += kWave) {
                Unit t[kDcRows];
#pragma unroll
                for (int a = 0; a < kDcRows; a++) {
                    const int o = o0 + a < p.ne ? o0 + a : p.ne - 1;
                    load_unit<DT>(base + (size_t)o * row_bytes, u, t[a]);
                }
                const float* xu = xk + (size_t)u * kUnitStride;
                float sh[kDcRows][2];
#pragma unroll
                for (int a = 0; a < kDcRows; a++) sh[a][0] = sh[a][1] = 0.0f;
#pragma unroll
                for (int q = 0; q < 8; q++) {
                    const float4 xv = reinterpret_cast<const float4*>(xu)[q];
#pragma unroll
                    for (int a = 0; a < kDcRows; a++) {
                        const uint32_t c = t[a].q[q];
                        float& w = sh[a][q >> 2];
                        w = fmaf((float)(c & 0xFFu), xv.x, w);
                        w = fmaf((float)((c >> 8) & 0xFFu), xv.y, w);
                        w = fmaf((float)((c >> 16) & 0xFFu), xv.z, w);
                        w = fmaf((float)(c >> 24), xv.w, w);
                    }
                }
                const float2 xsu = *reinterpret_cast<const float2*>(sk + 2 * u);
#pragma unroll
                for (int a = 0; a < kDcRows; a++)
                    acc[a] += (t[a].sc[0] * sh[a][0] + t[a].mn[0] * xsu.x) + (t[a].sc[1] * sh[a][1] + t[a].mn[1] * xsu.y);
            }
#pragma unroll
            for (int a = 0; a < kDcRows; a++) {
                v[a] = wave_sum(acc[a]);
                if (p.down_scale) v[a] = __fmul_rn(v[a], p.down_scale[e]);
            }
        }
        if (lane == 0) {
#pragma unroll
            for (int a = 0; a < kDcRows; a++) ys[k * kDcTile + (o0 - row_base) + a] = v[a];
        }
    }
    __syncthreads();
    if (tid < kDcTile && row_base + tid < p.ne) {
        float acc = 0.0f;
        for (int k = 0; k < K; k++) {   // rank order, separate multiply and add (crates/infr-cpu/src/lib.rs:4290-4302)
            const float w = p.weights[(size_t)r * K + k];
            if (p.skip_zero_w && w == 0.0f) continue;
            acc = __fadd_rn(acc, __fmul_rn(p.weight_before ? 1.0f : w, ys[k * kDcTile + tid]));
        }
        const size_t oi = (size_t)r * p.ne + row_base + tid;
        p.dst[oi] = p.addend ? __fadd_rn(p.addend[oi], acc) : acc;
    }
}

// Output elements per block: as many as give every one of the sixteen waves one (slot, four-row group) item.
int down_combine_units_tile(int n_used) { return n_used <= 4 ? 16 : n_used <= 8 ? 8 : 4; }
size_t down_combine_units_lds(const MoeGemvParams& p) {
    return ((size_t)p.n_used * (p.nff >> 5) * (kUnitStride + 2) + (size_t)p.n_used * 16) * sizeof(float);
}

template <int DT, int TILE>
void launch_moe_down_combine_units_t(hipStream_t s, const MoeGemvParams& p) {
    int be = 1, bb = 4;
    block_geometry(DT, &be, &bb);
    INFR_LDS_LIMIT((moe_down_combine_units_kernel<DT, TILE>), 158 * 1024);
    dim3 grid((p.ne + TILE - 1) / TILE, p.rows), block(1024);
    INFR_LAUNCH((moe_down_combine_units_kernel<DT, TILE>), grid, block, down_combine_units_lds(p), s, p, (size_t)(p.nff / be) * bb);
}
template <int DT>
void launch_moe_down_combine_units_dt(hipStream_t s, const MoeGemvParams& p) {
    const int tile = down_combine_units_tile(p.n_used);
    if (tile == 16) launch_moe_down_combine_units_t<DT, 16>(s, p);
    else if (tile == 8) launch_moe_down_combine_units_t<DT, 8>(s, p);
    else launch_moe_down_combine_units_t<DT, 4>(s, p);
}

template <int DT, bool GATE_UP>
void launch_moe_units_dt(hipStream_t s, const MoeGemvParams& p) {
    const int in_f = GATE_UP ? p.ne : p.nff, out_f = GATE_UP ? p.nff : p.ne;
    int be = 1, bb = 4;
    block_geometry(DT, &be, &bb);
    const size_t row_bytes = (size_t)(in_f / be) * bb;
    INFR_LDS_LIMIT((moe_units_kernel<DT, GATE_UP>), 158 * 1024);
    // output rows of a block (kRB in the kernel): 16, or 8 for gate/up when that still leaves the compute units short
    // of two blocks each (one round per block instead of two serial ones; C2 shape, one row: 11.5 -> 10.1 us)
    const int blocks16 = ((out_f + kRowsPerBlock - 1) / kRowsPerBlock) * p.rows * p.n_used;
    const int rb = GATE_UP && blocks16 < 512 ? 8 : kRowsPerBlock;
    dim3 grid((out_f + rb - 1) / rb, p.rows * p.n_used), block(256);
    const size_t route_lds = GATE_UP && p.route_inline ? route_scratch_floats(p.route.n_expert, p.route.n_groups) * sizeof(float) : 0;
    INFR_LAUNCH((moe_units_kernel<DT, GATE_UP>), grid, block, (size_t)(in_f >> 5) * (kUnitStride + 2) * sizeof(float) + route_lds,
                s, p, row_bytes, rb);
}

template <bool GATE_UP>
void launch_moe_units_any(hipStream_t s, int dt, const MoeGemvParams& p) {
    switch (dt) {
#define INFR_UNITS(D) case D: launch_moe_units_dt<D, GATE_UP>(s, p); break;
        INFR_FOR_UNIT_FORMATS(INFR_UNITS)
#undef INFR_UNITS
        default: break;
    }
}

size_t units_lds_bytes(int t, int in_f) { return (size_t)t * (in_f >> 5) * (kUnitStride + 2) * sizeof(float); }

template <int DT, int T>
void launch_units(hipStream_t s, const float* x, const uint8_t* w, size_t row_bytes, int m, int in_f, int out_f, float* dst,
                  const float* addend) {
    const size_t lds = units_lds_bytes(T, in_f);
    INFR_LDS_LIMIT((linear_units_kernel<DT, T>), 160 * 1024);
    // 16 output rows per block, or 8 (one round instead of two serial ones) while the grid would be small
    const int gy = (m + T - 1) / T;
    const int rb = ((out_f + kRowsPerBlock - 1) / kRowsPerBlock) * gy < 512 ? 8 : kRowsPerBlock;
    dim3 grid((out_f + rb - 1) / rb, gy), block(256);
    INFR_LAUNCH((linear_units_kernel<DT, T>), grid, block, lds, s, x, w, row_bytes, m, in_f, out_f, dst, addend, rb);
}

template <int DT>
void launch_units_dt(hipStream_t s, const float* x, const uint8_t* w, size_t row_bytes, int m, int in_f, int out_f, float* dst,
                     const float* addend) {
    constexpr size_t budget = 144 * 1024;
    if (m >= 4 && units_lds_bytes(4, in_f) <= budget) launch_units<DT, 4>(s, x, w, row_bytes, m, in_f, out_f, dst, addend);
    else if (m >= 2 && units_lds_bytes(2, in_f) <= budget) launch_units<DT, 2>(s, x, w, row_bytes, m, in_f, out_f, dst, addend);
    else launch_units<DT, 1>(s, x, w, row_bytes, m, in_f, out_f, dst, addend);
}

}  // namespace

namespace {

// Op::Linear on unquantised weights (F16, BF16, F32): lanes read 16 bytes of a weight row at a time against
// the activation row(s) staged in LDS; the same block / wave / row split as the unit kernel.
template <int DT, int T>
__global__ __launch_bounds__(256) void linear_float_kernel(const float* __restrict__ x, const uint8_t* __restrict__ w,
                                                           size_t row_bytes, int m, int in_f, int out_f, float* dst,
                                                           const float* addend) {
    extern __shared__ float lds[];
    constexpr int E = DT == INFR_F32 ? 4 : 8;   // elements per 16-byte load
    const int n_chunks = in_f / E;
    const int pitch = in_f + 4;                  // row pitch in LDS
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int r0 = blockIdx.y * T;
    for (int idx = tid; idx < T * (in_f >> 2); idx += 256) {
        const int tr = idx / (in_f >> 2), v = idx - tr * (in_f >> 2);
        float4 f = make_float4(0.f, 0.f, 0.f, 0.f);
        if (r0 + tr < m) f = reinterpret_cast<const float4*>(x + (size_t)(r0 + tr) * in_f)[v];
        reinterpret_cast<float4*>(lds + (size_t)tr * pitch)[v] = f;
    }
    __syncthreads();
    const int row_base = blockIdx.x * kRowsPerBlock;
    for (int round = 0; round < kRowsPerBlock / (4 * kRowsPerWave); round++) {
        const int o0 = row_base + (round * 4 + wave) * kRowsPerWave;
        if (o0 >= out_f) break;
        float acc[kRowsPerWave][T];
#pragma unroll
        for (int a = 0; a < kRowsPerWave; a++)
#pragma unroll
            for (int tr = 0; tr < T; tr++) acc[a][tr] = 0.0f;
        for (int c = lane; c < n_chunks; c += kWave) {
            float wv[kRowsPerWave][E];
#pragma unroll
            for (int a = 0; a < kRowsPerWave; a++) {
                const int o = o0 + a < out_f ? o0 + a : out_f - 1;
                const uint4 raw = *reinterpret_cast<const uint4*>(w + (size_t)o * row_bytes + 16 * (size_t)c);
                const uint32_t d[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    if constexpr (DT == INFR_F32) {
                        wv[a][k] = __uint_as_float(d[k]);
                    } else if constexpr (DT == INFR_BF16) {
                        wv[a][2 * k] = __uint_as_float(d[k] << 16);
                        wv[a][2 * k + 1] = __uint_as_float(d[k] & 0xFFFF0000u);
                    } else {
                        wv[a][2 * k] = f16_bits_to_f32(d[k] & 0xFFFFu);
                        wv[a][2 * k + 1] = f16_bits_to_f32(d[k] >> 16);
                    }
                }
            }
#pragma unroll
            for (int tr = 0; tr < T; tr++) {
                const float* xr = lds + (size_t)tr * pitch + E * c;
#pragma unroll
                for (int q = 0; q < E / 4; q++) {
                    const float4 xv = reinterpret_cast<const float4*>(xr)[q];
#pragma unroll
                    for (int a = 0; a < kRowsPerWave; a++) {
                        acc[a][tr] = fmaf(wv[a][4 * q], xv.x, acc[a][tr]);
                        acc[a][tr] = fmaf(wv[a][4 * q + 1], xv.y, acc[a][tr]);
                        acc[a][tr] = fmaf(wv[a][4 * q + 2], xv.z, acc[a][tr]);
                        acc[a][tr] = fmaf(wv[a][4 * q + 3], xv.w, acc[a][tr]);
                    }
                }
            }
        }
#pragma unroll
        for (int a = 0; a < kRowsPerWave; a++)
#pragma unroll
            for (int tr = 0; tr < T; tr++) {
                const float y = wave_sum(acc[a][tr]);
                if (lane == 0 && o0 + a < out_f && r0 + tr < m) {
                    const size_t oi = (size_t)(r0 + tr) * out_f + o0 + a;
                    dst[oi] = addend ? __fadd_rn(addend[oi], y) : y;
                }
            }
    }
}

template <int DT, int T>
void launch_float(hipStream_t s, const float* x, const uint8_t* w, size_t row_bytes, int m, int in_f, int out_f, float* dst,
                  const float* addend) {
    INFR_LDS_LIMIT((linear_float_kernel<DT, T>), 160 * 1024);
    dim3 grid((out_f + kRowsPerBlock - 1) / kRowsPerBlock, (m + T - 1) / T), block(256);
    INFR_LAUNCH((linear_float_kernel<DT, T>), grid, block, (size_t)T * (in_f + 4) * sizeof(float), s, x, w, row_bytes, m, in_f,
                out_f, dst, addend);
}

template <int DT>
void launch_float_dt(hipStream_t s, const float* x, const uint8_t* w, size_t row_bytes, int m, int in_f, int out_f, float* dst,
                     const float* addend) {
    const size_t budget = 144 * 1024, row = (size_t)(in_f + 4) * sizeof(float);
    if (m >= 4 && 4 * row <= budget) launch_float<DT, 4>(s, x, w, row_bytes, m, in_f, out_f, dst, addend);
    else if (m >= 2 && 2 * row <= budget) launch_float<DT, 2>(s, x, w, row_bytes, m, in_f, out_f, dst, addend);
    else launch_float<DT, 1>(s, x, w, row_bytes, m, in_f, out_f, dst, addend);
}

}  // namespace

bool linear_units_supported(int dt, int in_f, const void* x) {
    const int block = unit_format_block(dt);
    if (block == 0 || in_f % block) return false;
    return in_f >= 32 && in_f % 32 == 0 && units_lds_bytes(1, in_f) <= 144 * 1024 && ((uintptr_t)x & 15) == 0;
}

bool moe_gate_up_units_supported(const MoeGemvParams& p) {
    return p.gate_dt == p.up_dt && p.rows * p.n_used <= 65535 && linear_units_supported(p.gate_dt, p.ne, p.x);
}
void launch_moe_gate_up_units(hipStream_t s, const MoeGemvParams& p) { launch_moe_units_any<true>(s, p.gate_dt, p); }
// The unit gate/up kernel can route a token row inside each of its blocks (p.route_inline) for as many slots as its
// LDS tables hold.
bool moe_gate_up_units_routes_inline(const MoeGemvParams& p) { return moe_gate_up_units_supported(p) && p.n_used <= 64; }
bool moe_down_units_supported(const MoeGemvParams& p) {
    return p.y != nullptr && p.rows * p.n_used <= 65535 && linear_units_supported(p.down_dt, p.nff, p.h);
}
void launch_moe_down_units(hipStream_t s, const MoeGemvParams& p) { launch_moe_units_any<false>(s, p.down_dt, p); }
// The fused form needs the row's n_used activation rows side by side in LDS.
bool moe_down_combine_units_supported(const MoeGemvParams& p) {
    return p.rows * p.n_used <= 65535 && p.n_used <= 16 && linear_units_supported(p.down_dt, p.nff, p.h) &&
           down_combine_units_lds(p) <= 144 * 1024;
}
void launch_moe_down_combine_units(hipStream_t s, const MoeGemvParams& p) {
    switch (p.down_dt) {
#define INFR_UNITS(D) case D: launch_moe_down_combine_units_dt<D>(s, p); break;
        INFR_FOR_UNIT_FORMATS(INFR_UNITS)
#undef INFR_UNITS
        default: break;
    }
}

// x and h rows must be 16-byte aligned: ne and nff are multiples of 32 here, the bases are checked by the caller.
bool moe_units_batch_supported(int gate_dt, int up_dt, int down_dt, int ne, int nff) {
    const void* aligned = nullptr;
    return gate_dt == up_dt && linear_units_supported(gate_dt, ne, aligned) && linear_units_supported(down_dt, nff, aligned) &&
           (size_t)2 * (ne >> 5) * (kUnitStride + 2) * sizeof(float) <= 144 * 1024 &&
           (size_t)2 * (nff >> 5) * (kUnitStride + 2) * sizeof(float) <= 144 * 1024;
}
void launch_moe_gate_up_units_bucketed(hipStream_t s, const MoeGemvParams& p) {
    launch_moe_units_bucketed_any<true>(s, p.gate_dt, p, p.rows * p.n_used);
}
void launch_moe_down_units_bucketed(hipStream_t s, const MoeGemvParams& p) {
    launch_moe_units_bucketed_any<false>(s, p.down_dt, p, p.rows * p.n_used);
}

// 16-byte loads of the weight rows and of x: in_f a multiple of 8, rows and bases 16-byte aligned.
bool linear_float_supported(int dt, int in_f, size_t row_bytes, const void* x, const void* w) {
    if (dt != INFR_F32 && dt != INFR_F16 && dt != INFR_BF16) return false;
    return in_f >= 8 && in_f % 8 == 0 && (row_bytes & 15) == 0 && (((uintptr_t)x | (uintptr_t)w) & 15) == 0 &&
           (size_t)(in_f + 4) * sizeof(float) <= 144 * 1024;
}

void launch_linear_float(hipStream_t s, const float* x, const uint8_t* w, int dt, size_t row_bytes, int m, int in_f,
                         int out_f, float* dst, const float* addend) {
    if (dt == INFR_F32) launch_float_dt<INFR_F32>(s, x, w, row_bytes, m, in_f, out_f, dst, addend);
    else if (dt == INFR_F16) launch_float_dt<INFR_F16>(s, x, w, row_bytes, m, in_f, out_f, dst, addend);
    else launch_float_dt<INFR_BF16>(s, x, w, row_bytes, m, in_f, out_f, dst, addend);
}

void launch_linear_units(hipStream_t s, const float* x, const uint8_t* w, int dt, size_t row_bytes, int m, int in_f,
                         int out_f, float* dst, const float* addend) {
    switch (dt) {
#define INFR_UNITS(D) case D: launch_units_dt<D>(s, x, w, row_bytes, m, in_f, out_f, dst, addend); break;
        INFR_FOR_UNIT_FORMATS(INFR_UNITS)
#undef INFR_UNITS
        default: break;
    }
}

}  // namespace infr

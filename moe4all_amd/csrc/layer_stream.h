// The streaming single-launch kernel of Op::MoeFfn (one, two or four token rows in one launch) and its launcher
// template: included by the two translation units that instantiate it (k_layer_stream.hip: any shape;
// k_layer_stream_shapes.hip: the benchmark shapes with their sizes as compile-time constants).
#pragma once

#include "device_common.h"
#include "kernels.h"
#include "route.h"
#include "gemv_fmt.h"

#include <type_traits>


namespace infr {

namespace {

// Time stamps of every workgroup for a measurement build (-DINFR_LAYER_TRACE with a buffer in g.y); compiled out otherwise.
#ifdef INFR_LAYER_TRACE
#define STAMP(i)                                                                                                   \
    do {                                                                                                           \
        if ((threadIdx.x & 63) == 0 && q.g.y) reinterpret_cast<long long*>(q.g.y)[blockIdx.x * 32 + (i)] = wall_clock64(); \
    } while (0)
#else
#define STAMP(i) do { } while (0)
#endif

constexpr int kGroups = 8, kPerGroup = 32, kBlocks = kGroups * kPerGroup;
constexpr int kThreads = 512, kWaves = 8, kSW = 7;   // wavefronts 1..7 stream
constexpr uint32_t kCodePlain = 0x1FFu;              // tag code of records that belong to no expert

__device__ __forceinline__ uint64_t rec_load(const uint64_t* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void rec_store(uint64_t* p, float v, uint32_t tag) {
    __hip_atomic_store(p, (uint64_t)__float_as_uint(v) | ((uint64_t)tag << 32), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// A record for readers on the writer's own XCD only: a plain store, which stops in that XCD's L2, where the polling
// loads (which pass the L1 but not the L2) find it: about a fifth less latency than a write-through store, and the
// polls of a group no longer travel the fabric.  `local` false: for everyone, as above.
__device__ __forceinline__ void rec_store_xcd(uint64_t* p, float v, uint32_t tag, bool local) {
    if (!local) {
        rec_store(p, v, tag);
        return;
    }
    const uint64_t r = (uint64_t)__float_as_uint(v) | ((uint64_t)tag << 32);
    asm volatile("global_store_dwordx2 %0, %1, off" ::"v"(p), "v"(r) : "memory");
}

// Wave-wide: gathers rec[0 .. n) (n a multiple of 64, n <= 64 N) into out[] once all carry `tag`.  Every poll issues
// all of a lane's loads before it looks at any of them, so a poll costs one round trip (two polls in flight half a
// round trip apart were measured slower: the polls of 256 workgroups share one path).  False: spin limit.
// Outcome of gather_activations below.
enum : int { kGathered = 0, kGatherTimeout = 1, kGatherSuperseded = 2 };
// gather_records for the activations of a group, whose records carry the expert they were computed for: a record of
// this launch with ANOTHER expert's code means that its writer has seen the exact routing name a different expert for
// the group and has started over; the records wanted here will not come, and this workgroup is about to see the same
// routing.  kGatherSuperseded then, with out[] unspecified.  first_pass false: the group is on its second and last pass,
// and a record with another code is one of the first pass that its writer has not replaced yet.
template <int N>
__device__ __forceinline__ int gather_activations(const uint64_t* rec, int n, uint32_t tag, float* out, int lane, int spin_limit,
                                                  bool first_pass) {
    uint64_t r[N];
    const int ns = n >> 6;
    int state = kGathered;
    for (int spin = 0;; spin++) {
#pragma unroll
        for (int s = 0; s < N; s++) r[s] = s < ns ? rec_load(rec + s * kWave + lane) : ((uint64_t)tag << 32);
        bool ok = true, other = false;
#pragma unroll
        for (int s = 0; s < N; s++) {
            const uint32_t t = (uint32_t)(r[s] >> 32);
            ok = ok && t == tag;
            other = other || (t != tag && (t >> 9) == (tag >> 9));
        }
        if (__all(ok)) break;
        if (first_pass && __any(other)) { state = kGatherSuperseded; break; }
        if (spin >= spin_limit) return kGatherTimeout;
    }
#pragma unroll
    for (int s = 0; s < N; s++)
        if (s < ns) out[s * kWave + lane] = __uint_as_float((uint32_t)r[s]);
    return state;
}

template <int N>
__device__ __forceinline__ bool gather_records(const uint64_t* rec, int n, uint32_t tag, float* out, int lane, int spin_limit) {
    uint64_t r[N];
    const int ns = n >> 6;
    for (int spin = 0;; spin++) {
#pragma unroll
        for (int s = 0; s < N; s++) r[s] = s < ns ? rec_load(rec + s * kWave + lane) : ((uint64_t)tag << 32);
        bool ok = true;
#pragma unroll
        for (int s = 0; s < N; s++) ok = ok && (uint32_t)(r[s] >> 32) == tag;
        if (__all(ok)) break;
        if (spin >= spin_limit) return false;
    }
#pragma unroll
    for (int s = 0; s < N; s++)
        if (s < ns) out[s * kWave + lane] = __uint_as_float((uint32_t)r[s]);
    return true;
}

// Hand-over between the wavefronts of a workgroup through a word of LDS.  A wavefront's LDS operations complete in
// order, so data written before the flag is visible to whoever has read the flag.
__device__ __forceinline__ void lds_flag_set(volatile int* f, int v) {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    *f = v;
}
__device__ __forceinline__ int lds_flag_wait(volatile int* f) {
    int v;
    while ((v = __builtin_amdgcn_readfirstlane(*f)) == 0) __builtin_amdgcn_s_sleep(1);
    asm volatile("" ::: "memory");
    return v;
}

// The guess: the n_sel indices with the largest estimates, into out[] (any fixed rule will do: every workgroup runs
// this on the same values, and a wrong guess only costs time).  Keys are made unique by putting 255 - index into the
// low byte of the order-preserving key (n <= 256): estimates that agree in all but their last 8 mantissa bits are
// ranked by index, like exact ties.  Ranks come from counting, which has no serial chain: every lane sorts its NS keys
// and counts the lanes whose largest key beats its own; a member of the top K overall lies in one of the K lanes with
// the largest heads, so those lanes' K * NS keys (<= 64) are ranked among themselves the same way and the ranks
// [skew, skew + n_sel) are the guess.  skew > 0 (tests only, <= 8) leaves the `skew` largest out, so the guess is wrong
// on purpose.  scratch: 128 words of LDS.
template <int NS>
__device__ __forceinline__ void guess_set(const float* vals, int n_sel, int skew, int lane, int32_t* out, uint32_t* scratch) {
    static_assert(NS == 1 || NS == 2 || NS == 4, "sorting network");
    uint32_t key[NS];
#pragma unroll
    for (int s = 0; s < NS; s++) {
        const int i = s * kWave + lane;
        key[s] = (order_key(vals[i]) & ~0xFFu) | (uint32_t)(255 - i);
    }
    auto order = [&](int a, int b) {
        const uint32_t hi = max(key[a], key[b]), lo = min(key[a], key[b]);
        key[a] = hi;
        key[b] = lo;
    };
    if (NS == 2) order(0, 1);
    if (NS == 4) { order(0, 1); order(2, 3); order(0, 2); order(1, 3); order(1, 2); }
    uint32_t* heads = scratch;
    uint32_t* cand = scratch + kWave;
    heads[lane] = key[0];
    cand[lane] = 0u;
    __builtin_amdgcn_wave_barrier();
    auto beaten_by = [&](const uint32_t* list, int n4, uint32_t mine) {
        int r0 = 0, r1 = 0, r2 = 0, r3 = 0;
        for (int c = 0; c < n4; c++) {
            const uint4 v = reinterpret_cast<const uint4*>(list)[c];   // the same address in every lane: a broadcast
            r0 += v.x > mine ? 1 : 0;
            r1 += v.y > mine ? 1 : 0;
            r2 += v.z > mine ? 1 : 0;
            r3 += v.w > mine ? 1 : 0;
        }
        return (r0 + r1) + (r2 + r3);
    };
    const int K = n_sel + skew;   // <= 16
    const int r = beaten_by(heads, kWave / 4, key[0]);
    if (r < K) {
#pragma unroll
        for (int s = 0; s < NS; s++) cand[r * NS + s] = key[s];
    }
    __builtin_amdgcn_wave_barrier();
    const int nc = K * NS;
    const uint32_t mine = cand[lane];   // 0 past the candidates
    const int r2 = beaten_by(cand, (nc + 3) >> 2, mine);
    if (lane < nc && r2 >= skew && r2 < K) out[r2 - skew] = 255 - (int)(mine & 0xFFu);
}

// A ring of D items in flight: `issue(slot, j)` requests item j into ring slot `slot`, `finish(slot, j)` consumes it.
// The first D items have been requested by the caller (ring_prime); items past `cn` are never finished.
template <int D, class Issue>
__device__ __forceinline__ void ring_prime(Issue issue) {
#pragma unroll
    for (int d = 0; d < D; d++) issue(d, d);
}
template <int D, class Issue, class Finish>
__device__ __forceinline__ void ring_drain(int cn, Issue issue, Finish finish) {
    const int refills = cn - D;   // steps that still have an item to request
    int j0 = 0;
    for (; j0 + D <= refills; j0 += D) {
#pragma unroll
        for (int d = 0; d < D; d++) {
            finish(d, j0 + d);
            issue(d, j0 + d + D);
        }
    }
#pragma unroll
    for (int d = 0; d < D; d++) {
        if (j0 + d >= cn) break;
        finish(d, j0 + d);
        if (j0 + d < refills) issue(d, j0 + d + D);
    }
    j0 += D;
#pragma unroll
    for (int d = 0; d < D; d++) {
        if (j0 + d >= cn) break;
        finish(d, j0 + d);
    }
}

__device__ __forceinline__ float dot8(const float4& a0, const float4& a1, const float4& b0, const float4& b1) {
    float s = a0.x * b0.x;
    s = fmaf(a0.y, b0.y, s);
    s = fmaf(a0.z, b0.z, s);
    s = fmaf(a0.w, b0.w, s);
    s = fmaf(a1.x, b1.x, s);
    s = fmaf(a1.y, b1.y, s);
    s = fmaf(a1.z, b1.z, s);
    return fmaf(a1.w, b1.w, s);
}

}  // namespace

// Down items (groups of output rows a wavefront covers at once) of a workgroup that the router's wavefront takes, the
// last ones of the n_di: an eighth when that leaves the seven streaming wavefronts equal shares.  It knows the exact
// routing first and has nothing to do while the others stream.
__host__ __device__ constexpr int router_wave_down_items(int n_di) { return n_di % 8 == 0 ? n_di / 8 : 0; }

// FG / FD: formats of the gate/up and down banks; DG / DD: ring depths (items in flight per streaming wavefront);
// EPT: router rows a thread holds while staging (rows per workgroup / (512 / (ne / 8))); NSP: n_expert / 64.
// NE, NFF, ROWS: hidden size, intermediate size and token rows when they are known at compile time (the benchmark
// shapes), 0 for any shape.  With constants the lane placement, the item counts and every index division below fold;
// with run-time values they are integer arithmetic on the critical path of a kernel that one wavefront paces.
// NORM: 1 with an Op::RmsNorm of the token row folded in (its own instantiations: the branches of a run-time switch cost
// the plain kernel a microsecond and a half of its operand staging).
template <class FG, class FD, int DG, int DD, int EPT, int NSP, int NE = 0, int NFF = 0, int ROWS = 0, int NORM = 0>
__global__ __launch_bounds__(kThreads) void moe_layer_stream(MoeLayerParams q) {
    extern __shared__ __attribute__((aligned(16))) uint32_t dyn_lds[];
    __shared__ uint64_t s_tab[32];
    __shared__ int32_t s_ids[64];
    __shared__ float s_w[64];
    __shared__ float s_g[kWaves][64], s_u[kWaves][64];
    __shared__ float s_part[kWaves][8];
    __shared__ int32_t s_spec[kGroups], s_final[kGroups], s_gor[kGroups];
    __shared__ float s_ysh[64];
    __shared__ float s_red[4];
    __shared__ uint32_t s_guess[2 * kWave];
    __shared__ int s_f_spec, s_f_route, s_fault, s_cells_done, s_h_done, s_xn_done;
    __shared__ uint32_t s_seq;
    const MoeGemvParams& p = q.g;
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;   // wave: uniform, scalar registers
    const int ne = NE ? NE : p.ne, nff = NFF ? NFF : p.nff, n_expert = 64 * NSP;
    const bool shared = p.sh_gate != nullptr;
    // One, two or four token rows per launch: a row takes 8 / rows of the XCDs (workgroups are dealt to the XCDs in turn,
    // so workgroup b sits on XCD b & 7 up to a rotation), its eight groups of mpg = 32 / rows members each lie on one XCD
    // as before, and everything below happens per row among the row's 256 / rows workgroups.
    const int b = blockIdx.x;
    const int n_rows = ROWS ? ROWS : p.rows, xpr = kGroups / n_rows, mpg = kPerGroup / n_rows, bpr = kBlocks / n_rows;
    const int xcd = b & 7, jx = b >> 3;
    const int trow = xcd / xpr;                            // this workgroup's token row
    const int g = (xcd - trow * xpr) * n_rows + jx / mpg;  // its group: the rank slot it works on
    const int m = jx % mpg;                                // its place in the group
    const int os = m * kGroups + g;                        // its place among the row's workgroups: output rows, always-on share
    {   // this row's operands and results
        MoeGemvParams& pw = q.g;
        pw.x += (size_t)trow * ne;
        pw.dst += (size_t)trow * ne;
        if (pw.addend) pw.addend += (size_t)trow * ne;
        if (pw.sh_logit) pw.sh_logit += trow;
        pw.route.ids += (size_t)trow * pw.route.n_used;
        pw.route.weights += (size_t)trow * pw.route.n_used;
        if (pw.route.probs) pw.route.probs += (size_t)trow * n_expert;
        q.router_x += (size_t)trow * ne;
        if (q.logits_out) q.logits_out += (size_t)trow * n_expert;
        q.xa += (size_t)trow * kGroups * n_expert;
        q.xl += (size_t)trow * kGroups * n_expert;
        q.xh += (size_t)trow * kGroups * nff;
        q.xs += (size_t)trow * nff;
        q.ypart += (size_t)trow * kGroups * ne;
    }

    // who computes which router logits: every group all of them (epb = n_expert / 32 rows per workgroup, published to
    // the group), or every logit once for the grid (epb rows per workgroup while they last, published to everyone)
    const int epb = q.epb;
    const bool group_local = !q.logits_once;   // logit records stay inside the group's XCD
    const int area = q.logits_once ? 0 : g;
    const int row0 = (q.logits_once ? os : m) * epb;
    const bool has_rows = row0 < n_expert;

    // LDS: [cells of x][chain operands, transposed][estimates][logits][routing scratch][h][cells of h][h, cells: always-on]
    const int oct_n = ne >> 3;                 // octets of a row: 256 or 512
    const int jstride = oct_n + 4;
    const int hsel = tid / oct_n, o = tid - hsel * oct_n;   // replica (0 or 1 when ne = 2048) and octet of this thread
    const int H = kThreads / oct_n;
    uint32_t* cells = dyn_lds;
    float* wst = reinterpret_cast<float*>(cells + (size_t)(ne >> 5) * kCellDwords);
    float* xst = wst + (size_t)epb * 8 * jstride;
    float* s_alog = xst + 8 * jstride;
    float* s_logits = s_alog + n_expert;
    float* route_scratch = s_logits + n_expert;
    float* s_h = route_scratch + ((route_scratch_floats(n_expert, p.route.n_groups) + 3) & ~(size_t)3);
    uint32_t* hcells = reinterpret_cast<uint32_t*>(s_h + nff);
    float* s_hs = reinterpret_cast<float*>(hcells + (size_t)(nff >> 5) * kCellDwords);
    uint32_t* hscells = reinterpret_cast<uint32_t*>(s_hs + nff);

    if (tid < 32) s_tab[tid] = kExp2Table[tid];
    if (tid == 0) {
        s_f_spec = s_f_route = s_fault = s_cells_done = s_h_done = s_xn_done = 0;
        // the launch's number: every workgroup keeps its own count of the launches it has run (a counter shared by all
        // would serialise 256 atomics, at the start or, worse, at the end of the kernel), read here and written back
        // with a plain store at the end; launches on a workspace never overlap, so all 256 counts agree
        s_seq = q.cnt[b] + 1u;
    }
    if (wave == 0) STAMP(0);
    // (Records written for the own group only stop in the XCD's L2.  Workgroups are dealt to the XCDs in turn by their
    // index, starting from an XCD that changes from launch to launch, so a group sits on one XCD; were it ever split, a
    // record would simply not be seen, the wait would run out and the launch be reported: a record is one 64-bit unit.)

    // ---- A: operands.  Thread (replica hsel, octet o) holds elements [8 o, 8 o + 8) of the routing row, of the token
    // row and of the router rows hsel, hsel + H, ...  The token row becomes fixed-point cells later, by the threads
    // of the last replica (with two replicas that keeps the router's and the guessing wavefront out of it).
    const bool converts = hsel == H - 1;
    constexpr bool normed = NORM != 0;   // one token row only; the token row is then the normalised row (the host checks)
    float4 cx0, cx1, nw0, nw1;
    {
        const float4* rx4 = reinterpret_cast<const float4*>(normed ? q.norm_x : q.router_x);
        float4 rx0 = rx4[2 * o], rx1 = rx4[2 * o + 1];
        if (normed) {   // the routing row and the token row are one row, raw so far
            cx0 = rx0;
            cx1 = rx1;
            const float4* nw4 = reinterpret_cast<const float4*>(q.norm_w);
            nw0 = nw4[2 * o];
            nw1 = nw4[2 * o + 1];
        } else {
            const float4* px4 = reinterpret_cast<const float4*>(p.x);
            cx0 = px4[2 * o];
            cx1 = px4[2 * o + 1];
        }
        float4 w0[EPT], w1[EPT];
#pragma unroll
        for (int i = 0; i < EPT; i++) {
            const int el = hsel + H * i;
            const bool on = has_rows && el < epb;
            const float4* row = reinterpret_cast<const float4*>(q.router + (size_t)(on ? row0 + el : 0) * q.router_row_floats);
            w0[i] = row[2 * o];
            w1[i] = row[2 * o + 1];
        }
        if (normed) {
            // An Op::RmsNorm of the single token row folded in: the row arrives raw and every workgroup normalises it.
            // The sum of squares runs exactly as in the standalone kernel - 256 threads, thread t over the 128-bit pieces
            // t, t + 256, ..., the same tree over the threads - so the scale has the same bits; it takes its own loads of
            // the row (the pieces this thread holds for the dots are two neighbours).  The scale is applied behind the
            // barrier below.  The estimates do not wait for it: a positive factor common to all of them does not change
            // their order, so they are taken from x * w without the scale.
            float part = 0.0f;
            if (tid < 256)
                for (int v = tid; v < (ne >> 2); v += 256) part = sumsq4(part, rx4[v]);
            part = wave_sum(part);
            if (lane == 0 && wave < 4) s_red[wave] = part;
            rx0 = make_float4(rx0.x * nw0.x, rx0.y * nw0.y, rx0.z * nw0.z, rx0.w * nw0.w);
            rx1 = make_float4(rx1.x * nw1.x, rx1.y * nw1.y, rx1.z * nw1.z, rx1.w * nw1.w);
        }
        // the estimate's share of this thread, summed over the wavefront
#pragma unroll
        for (int i = 0; i < EPT; i++) {
            const float part = wave_sum(dot8(w0[i], w1[i], rx0, rx1));
            if (lane == 0) s_part[wave][i] = part;
        }
        // chain operands: element 8 o + t belongs to chain t, position o
        if (hsel == 0 && !normed) {
            const float xv[8] = {rx0.x, rx0.y, rx0.z, rx0.w, rx1.x, rx1.y, rx1.z, rx1.w};
#pragma unroll
            for (int t = 0; t < 8; t++) xst[t * jstride + o] = xv[t];
        }
#pragma unroll
        for (int i = 0; i < EPT; i++) {
            const int el = hsel + H * i;
            if (el < epb) {
                const float wv[8] = {w0[i].x, w0[i].y, w0[i].z, w0[i].w, w1[i].x, w1[i].y, w1[i].z, w1[i].w};
#pragma unroll
                for (int t = 0; t < 8; t++) wst[(el * 8 + t) * jstride + o] = wv[t];
            }
        }
    }
    __syncthreads();
    const uint32_t seq_tag = (s_seq & 0x7FFFFFu) << 9;
    if (wave == 0) STAMP(1);
    const uint32_t tag = seq_tag | kCodePlain;
    const int waves_per_replica = oct_n >> 6;
    if (wave == 1 && has_rows && lane < epb) {
        // the estimate of logit row0 + lane: the shares of the wavefronts that held that row, in a fixed order
        const int hs = lane % H, i = lane / H;
        float a = 0.0f;
        for (int w = hs * waves_per_replica; w < (hs + 1) * waves_per_replica; w++) a += s_part[w][i];
        rec_store_xcd(q.xa + (size_t)area * n_expert + row0 + lane, a, tag, group_local);
    }
    // the token row as fixed-point cells, one set for the workgroup; the guessing wavefront takes its share after the guess
    const int n_conv_waves = oct_n >> 6;
    auto convert_share = [&]() {
        if (!converts) return;   // whole wavefronts
        octet_to_cell<FG::kGroup, FG::kSigned>(cx0, cx1, o, cells);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (lane == 0) __hip_atomic_fetch_add(&s_cells_done, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    };
    auto wait_cells = [&]() {
        while (__builtin_amdgcn_readfirstlane(*(volatile int*)&s_cells_done) < n_conv_waves) __builtin_amdgcn_s_sleep(1);
        asm volatile("" ::: "memory");
    };
    if (normed) {
        // the scale, the same bits in every thread; the normalised row for the cells, for the exact chains (the router's
        // wavefront waits for the wavefronts that stage it) and, from one workgroup, for the RmsNorm's dst
        const float sc = rms_scale((s_red[0] + s_red[1]) + (s_red[2] + s_red[3]), ne, q.norm_eps);
        cx0 = rms_apply4(cx0, sc, nw0);
        cx1 = rms_apply4(cx1, sc, nw1);
        if (hsel == 0) {
            const float xv[8] = {cx0.x, cx0.y, cx0.z, cx0.w, cx1.x, cx1.y, cx1.z, cx1.w};
#pragma unroll
            for (int t = 0; t < 8; t++) xst[t * jstride + o] = xv[t];
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            if (lane == 0) __hip_atomic_fetch_add(&s_xn_done, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            if (os == 0 && q.norm_out) {
                reinterpret_cast<float4*>(q.norm_out)[2 * o] = cx0;
                reinterpret_cast<float4*>(q.norm_out)[2 * o + 1] = cx1;
            }
        }
    }
    if (wave != 1) convert_share();
    if (wave == 0) STAMP(2);

    const int spin_limit = q.spin_limit;
    if (wave == 0) {
        // ================================================================ the router: exact logits, exact routing
        bool ok = true;
        {
            const int e = lane >> 3, j = lane & 7;
            const bool live = has_rows && e < epb;
            float acc = 0.0f;
            if (normed) {   // the normalised row is staged behind the barrier, by oct_n / 64 wavefronts
                while (__builtin_amdgcn_readfirstlane(*(volatile int*)&s_xn_done) < waves_per_replica) __builtin_amdgcn_s_sleep(1);
                asm volatile("" ::: "memory");
            }
            if (live) {
                // the reference's order: 8 chains over i = j (mod 8), summed 0..7 (crates/infr-cpu/src/kernels.rs:6568-6583)
                const float4* wp = reinterpret_cast<const float4*>(wst + (e * 8 + j) * jstride);
                const float4* xp = reinterpret_cast<const float4*>(xst + j * jstride);
                const int n4 = oct_n >> 2;   // a multiple of 8
#pragma unroll 1
                for (int c = 0; c < n4; c += 8) {
                    float4 a[8], bb[8];
#pragma unroll
                    for (int k = 0; k < 8; k++) { a[k] = wp[c + k]; bb[k] = xp[c + k]; }
#pragma unroll
                    for (int k = 0; k < 8; k++) {
                        acc = __fmaf_rn(a[k].x, bb[k].x, acc);
                        acc = __fmaf_rn(a[k].y, bb[k].y, acc);
                        acc = __fmaf_rn(a[k].z, bb[k].z, acc);
                        acc = __fmaf_rn(a[k].w, bb[k].w, acc);
                    }
                }
            }
            float s = 0.0f;
#pragma unroll
            for (int jj = 0; jj < 8; jj++) s = __fadd_rn(s, __shfl(acc, (lane & ~7) + jj, kWave));
            if (live && j == 0) {
                rec_store_xcd(q.xl + (size_t)area * n_expert + row0 + e, s, tag, group_local);
                if ((q.logits_once || g == 0) && q.logits_out) q.logits_out[row0 + e] = s;
            }
        }
        STAMP(16);
        ok = gather_records<NSP>(q.xl + (size_t)area * n_expert, n_expert, tag, s_logits, lane, spin_limit);
        STAMP(17);
        if (ok) {
            __builtin_amdgcn_wave_barrier();
            RouteParams rp = p.route;
            rp.logits = s_logits;
            rp.n_expert = n_expert;   // compile-time here: the routing code's loops and index arithmetic fold
            rp.n_used = kGroups;
            // the guess is the candidate for the selection: when the exact probabilities confirm it, the selection
            // rounds are not needed; else (a missed expert, a tie at the boundary, another gating) the complete routine
            const int guess_state = lds_flag_wait(&s_f_spec);
            if (guess_state != 1) ok = false;
            bool routed = false;
            if (ok && route_duo_ok(rp) && rp.n_expert == 64 * NSP)
                routed = route_softmax_checked<NSP>(rp, 0, lane, s_spec, route_scratch, s_tab, s_ids, s_w, os == 0);
            if (!routed) {
                __builtin_amdgcn_wave_barrier();
                route_row_any(rp, 0, lane, route_scratch, s_tab, s_ids, s_w, os == 0);
            }
            STAMP(18);
            __builtin_amdgcn_wave_barrier();
            // which group holds which rank; groups whose guess is outside the exact set take the missed experts
            if (ok) {
                // lane k < 8 owns rank k: the group whose guess is that expert; ranks the guess missed take the groups
                // whose guess is outside the exact set, both in ascending order
                const bool rank = lane < kGroups;
                const int id = rank ? s_ids[lane] : -1;
                int gk = -1;
#pragma unroll
                for (int gg = 0; gg < kGroups; gg++)
                    if (s_spec[gg] == id) gk = gg;
                uint32_t used = 0;
#pragma unroll
                for (int gg = 0; gg < kGroups; gg++) used |= (__ballot(rank && gk == gg) ? 1u : 0u) << gg;
                const uint32_t missed = (uint32_t)__ballot(rank && gk < 0) & 0xFFu;
                if (rank && gk < 0) {
                    const int j = __builtin_popcount(missed & ((1u << lane) - 1u));
                    int seen = 0;
#pragma unroll
                    for (int gg = 0; gg < kGroups; gg++) {
                        const bool free_g = !((used >> gg) & 1u);
                        if (free_g && seen == j) gk = gg;
                        seen += free_g ? 1 : 0;
                    }
                }
                if (rank) {
                    s_gor[lane] = gk;
                    s_final[gk] = id;
                }
                if (os == 0 && missed && lane == 0 && q.late)
                    __hip_atomic_fetch_add(q.late, (uint32_t)__builtin_popcount(missed), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            }
        }
        if (!ok && lane == 0) {
            s_fault = 1;
            __hip_atomic_store(q.fault, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        }
        lds_flag_set(&s_f_route, ok ? 1 : 2);
        STAMP(19);
    } else {
        // ================================================================ the streaming wavefronts
        const int sw = wave - 1;
        const int nblk_g = ne / FG::kBlockElems, nblk_d = nff / FD::kBlockElems;
        const size_t rb_g = (size_t)nblk_g * FG::kBlockBytes, rb_d = (size_t)nblk_d * FD::kBlockBytes;
        const Place<FG> pg(nblk_g, lane);
        const Place<FD> pd(nblk_d, lane);
        struct GuItem { typename FG::Raw g, u; };
        bool alive = true;

        // gate/up items of this wavefront: item j covers features (j * kSW + sw) * rw_count + rw of the workgroup's slice.
        // With an always-on expert the wavefronts take the items of its share [os * nff / bpr, ..), dealt like the expert's,
        // as their ring's first entries: they need no routing, so the first of them are requested before the guess is known.
        const int fpb = nff / mpg, f0 = m * fpb;
        const int n_gi = (fpb + pg.rw_count - 1) / pg.rw_count;
        const int my_gi = n_gi > sw ? (n_gi - sw + kSW - 1) / kSW : 0;
        const int sfpb = nff / bpr, sf0 = os * sfpb;
        const int n_si = shared ? (sfpb + pg.rw_count - 1) / pg.rw_count : 0;
        const int sh_n = n_si > sw ? (n_si - sw + kSW - 1) / kSW : 0;
        // down items: item j covers output rows (j * kSW + sw) * rw_count + rw of the workgroup's slice (the always-on
        // expert's down rows are the router's wavefront's: it has nothing else to do while the activations change hands)
        const int R = ne / mpg;
        const int n_di = (R + pd.rw_count - 1) / pd.rw_count;
        const int n_ds = n_di - router_wave_down_items(n_di);   // the streaming wavefronts' items: the first n_ds
        const int my_di = n_ds > sw ? (n_ds - sw + kSW - 1) / kSW : 0;

        GuItem gring[DG];
        auto sh_load = [&](GuItem& it, int j) __attribute__((always_inline)) {   // item j of this wavefront's share
            const int f = sf0 + min((j * kSW + sw) * pg.rw_count + pg.rw, sfpb - 1);
            it.g = load_row<FG>(pg, p.sh_gate + (size_t)f * rb_g);
            it.u = load_row<FG>(pg, p.sh_up + (size_t)f * rb_g);
        };
        auto sh_issue = [&]() __attribute__((always_inline)) {   // those of the first ring fill
#pragma unroll
            for (int d = 0; d < DG; d++)
                if (d < sh_n) sh_load(gring[d], d);
        };
        if (sh_n && wave != 1) sh_issue();
        if (wave == 1) {
            // the guess of the selected set, from the estimates
            bool ok = gather_records<NSP>(q.xa + (size_t)area * n_expert, n_expert, tag, s_alog, lane, spin_limit);
            STAMP(3);
            if (ok) {
                __builtin_amdgcn_wave_barrier();
                guess_set<NSP>(s_alog, kGroups, q.guess_skew, lane, s_spec, s_guess);
            } else if (lane == 0) {
                s_fault = 1;
                __hip_atomic_store(q.fault, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            }
            lds_flag_set(&s_f_spec, ok ? 1 : 2);
            STAMP(4);
            alive = ok;
            convert_share();
            if (sh_n) sh_issue();
        } else {
            alive = lds_flag_wait(&s_f_spec) == 1;
        }

        typename FD::Raw dring[DD];
        int e_cur = alive ? __builtin_amdgcn_readfirstlane(s_spec[g]) : 0;
        const uint8_t* dbank = nullptr;
        auto dn_issue = [&](int slot, int j) __attribute__((always_inline)) {   // items past the end re-read the last row
            const int orow = min((j * kSW + sw) * pd.rw_count + pd.rw, R - 1);
            dring[slot] = load_row<FD>(pd, dbank + (size_t)(m * R + orow) * rb_d);
        };
        // One pass per expert this group works on: the guessed one, and once more if the exact routing names another.
        // A pass does not wait for the routing: the group's activations carry the expert they were computed for, so
        // the members of a group meet on the guess, and the down rows' results carry it too, so nobody consumes a
        // result of an expert the routing did not select.  The routing is looked at after the pass (and, without
        // waiting, before the down stage, which is skipped when it is already known to be for nothing).
        const int chunk = nff / 6;   // records per gathering wavefront: a multiple of 64
        // (two straight-line copies of the pass instead of a loop: a loop's invariant addresses would stay in registers
        // across the whole pass and spill)
        auto run_pass = [&](const int attempt) __attribute__((always_inline)) -> bool {   // true: once more, with e_cur renewed
            const uint8_t* gb = p.gate + (size_t)e_cur * p.gate_stride + (size_t)f0 * rb_g;
            const uint8_t* ub = p.up + (size_t)e_cur * p.up_stride + (size_t)f0 * rb_g;
            dbank = p.down + (size_t)e_cur * p.down_stride;
            const int sh = attempt == 0 ? sh_n : 0;   // ring entries ahead of the expert's items
            {
                typename FG::X x;   // fetched again on a second pass: not kept alive across the hand-over
                auto gu_issue = [&](int slot, int j) __attribute__((always_inline)) {
                    if (j < sh) {   // more items of the always-on expert than the first ring fill held
                        sh_load(gring[slot], j);
                        return;
                    }
                    const int f = min(((j - sh) * kSW + sw) * pg.rw_count + pg.rw, fpb - 1);
                    gring[slot].g = load_row<FG>(pg, gb + (size_t)f * rb_g);
                    gring[slot].u = load_row<FG>(pg, ub + (size_t)f * rb_g);
                };
                auto gu_finish = [&](int slot, int j) __attribute__((always_inline)) {
                    const float gs = row_sum<FG>(FG::dot(gring[slot].g, pg.sub, x), pg, nblk_g);
                    const float us = row_sum<FG>(FG::dot(gring[slot].u, pg.sub, x), pg, nblk_g);
                    if (j < sh) {   // the always-on expert's item: its activation goes to every workgroup
                        const int fi = (j * kSW + sw) * pg.rw_count + pg.rw;
                        if (pg.writer() && fi < sfpb)
                            rec_store(q.xs + sf0 + fi, gated_act_fn(p.act, p.has_clamp, p.clamp, gs, us, s_tab), tag);
                    } else if (pg.writer()) {
                        s_g[wave][(j - sh) * pg.rw_count + pg.rw] = gs;
                        s_u[wave][(j - sh) * pg.rw_count + pg.rw] = us;
                    }
                };
#pragma unroll
                for (int d = 0; d < DG; d++)
                    if (d >= sh) gu_issue(d, d);
                if (q.early_down) ring_prime<DD>(dn_issue);
                if (wave == 3) STAMP(5);
                if (wave == 1) STAMP(20);
                if (attempt == 0) wait_cells();
                FG::fetch_x(x, cells, pg.blk, pg.sub);
                ring_drain<DG>(sh + my_gi, gu_issue, gu_finish);
            }
            if (wave == 3) STAMP(6);
            __builtin_amdgcn_wave_barrier();
            if (lane < my_gi * pg.rw_count) {
                const int j = lane / pg.rw_count, rw = lane - j * pg.rw_count;
                const int fi = (j * kSW + sw) * pg.rw_count + rw;
                if (fi < fpb)
                    rec_store_xcd(q.xh + (size_t)g * nff + f0 + fi,
                                  gated_act_fn(p.act, p.has_clamp, p.clamp, s_g[wave][lane], s_u[wave][lane], s_tab),
                                  seq_tag | (uint32_t)e_cur, true);
            }
            __builtin_amdgcn_wave_barrier();
            if (wave == 3) STAMP(7);
            if (wave == 1) STAMP(21);
            if (wave == 7) STAMP(22);
            // ---- hand-over of the group's activations: six wavefronts gather a sixth each and turn it into cells
            bool superseded = false;
            if (sw < 6) {
                const int st = gather_activations<4>(q.xh + (size_t)g * nff + sw * chunk, chunk, seq_tag | (uint32_t)e_cur,
                                                     s_h + sw * chunk, lane, spin_limit, attempt == 0);
                if (wave == 1) STAMP(9);
                superseded = st == kGatherSuperseded;
                if (st == kGathered) {
                    __builtin_amdgcn_wave_barrier();
                    if (lane * 8 < chunk) {   // whole groups of four lanes
                        const int oct = sw * (chunk >> 3) + lane;
                        const float4 lo = *reinterpret_cast<const float4*>(s_h + 8 * oct), hi = *reinterpret_cast<const float4*>(s_h + 8 * oct + 4);
                        octet_to_cell<FD::kGroup, FD::kSigned>(lo, hi, oct, hcells);
                    }
                } else if (st == kGatherTimeout && lane == 0) {
                    s_fault = 1;
                    __hip_atomic_store(q.fault, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                }
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                if (lane == 0)
                    __hip_atomic_fetch_add(&s_h_done, st == kGatherTimeout ? 0x101 : 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                if (wave == 1) STAMP(10);
            }
            // the first down rows, requested behind the polls: a poll issued behind them would not return before them
            if (!q.early_down && alive) ring_prime<DD>(dn_issue);
            {
                int v;
                while ((((v = __builtin_amdgcn_readfirstlane(*(volatile int*)&s_h_done)) & 0xFF) < 6 * (attempt + 1)) && !(v >> 8))
                    __builtin_amdgcn_s_sleep(1);
                asm volatile("" ::: "memory");
                if (v >> 8) alive = false;
            }
            // is this pass already known to be for another expert than the routing's?  (the same answer in every
            // wavefront is not needed: the down stage has no hand-over between wavefronts)
            int routed = __builtin_amdgcn_readfirstlane(*(volatile int*)&s_f_route);
            asm volatile("" ::: "memory");
            const bool in_vain = superseded || routed == 2 || (routed == 1 && __builtin_amdgcn_readfirstlane(s_final[g]) != e_cur);
            if (alive && !in_vain) {
                // ---- down: rows of the group's expert
                typename FD::X xd;
                FD::fetch_x(xd, hcells, pd.blk, pd.sub);
                const bool scaled = p.down_scale != nullptr;
                const float ds = scaled ? p.down_scale[e_cur] : 1.0f;
                uint64_t* part = q.ypart + (size_t)g * ne + (size_t)m * R;
                const uint32_t ytag = seq_tag | (uint32_t)e_cur;
                auto dn_finish = [&](int slot, int j) __attribute__((always_inline)) {
                    const int orow = (j * kSW + sw) * pd.rw_count + pd.rw;
                    const float y = row_sum<FD>(FD::dot(dring[slot], pd.sub, xd), pd, nblk_d);
                    if (pd.writer() && orow < R) rec_store(part + orow, scaled ? __fmul_rn(y, ds) : y, ytag);
                };
                ring_drain<DD>(my_di, dn_issue, dn_finish);
                if (wave == 3) STAMP(11);
            }
            if (!alive) return false;
            routed = lds_flag_wait(&s_f_route);
            if (wave == 3) STAMP(8);
            if (routed != 1) {
                alive = false;
                return false;
            }
            const int e_fin = __builtin_amdgcn_readfirstlane(s_final[g]);
            if (e_fin == e_cur) return false;
            e_cur = e_fin;   // the guess missed this group's expert: once more with the right one
            return true;
        };
        if (alive && run_pass(0)) run_pass(1);
    }
    if (wave == 0) {
        // ---- the rank-ordered sum, by the router's wavefront: workgroup (g, m) owns rows [m R + g R / 8, + R / 8) of
        // the output, which are also the rows of the always-on expert it has just computed.  out = sum over ranks of
        // w_rank * y_rank as a separate multiply and add (crates/infr-cpu/src/lib.rs:4290-4302), then the always-on
        // expert, then the residual operand.  The partial results are polled while the streaming wavefronts still work.
        const int R = ne / mpg, SR = R / kGroups;
        const int nblk_d = nff / FD::kBlockElems;
        const size_t rb_d = (size_t)nblk_d * FD::kBlockBytes;
        const Place<FD> pd(nblk_d, lane);
        typename FD::X xd;
        typename FD::Raw ring[DD];
        if (shared) {
            // ---- the always-on expert's down rows of this workgroup, [os * SR, + SR), while the streaming wavefronts wait
            // for their group's activations: nothing else is in flight then.  Its activations were written long ago by all
            // the workgroups of the row.
            bool got = gather_records<24>(q.xs, nff, tag, s_hs, lane, spin_limit);
            if (got) {
                __builtin_amdgcn_wave_barrier();
                for (int oct = lane; oct * 8 < nff; oct += kWave) {
                    const float4 lo = *reinterpret_cast<const float4*>(s_hs + 8 * oct), hi = *reinterpret_cast<const float4*>(s_hs + 8 * oct + 4);
                    octet_to_cell<FD::kGroup, FD::kSigned>(lo, hi, oct, hscells);
                }
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                __builtin_amdgcn_wave_barrier();
                FD::fetch_x(xd, hscells, pd.blk, pd.sub);
                const uint8_t* rows0 = p.sh_down + (size_t)os * SR * rb_d;
                const int n_sdi = (SR + pd.rw_count - 1) / pd.rw_count;
                auto sd_issue = [&](int slot, int j) __attribute__((always_inline)) {
                    ring[slot] = load_row<FD>(pd, rows0 + (size_t)min(j * pd.rw_count + pd.rw, SR - 1) * rb_d);
                };
                auto sd_finish = [&](int slot, int j) __attribute__((always_inline)) {
                    const int orow = j * pd.rw_count + pd.rw;
                    const float y = row_sum<FD>(FD::dot(ring[slot], pd.sub, xd), pd, nblk_d);
                    if (pd.writer() && orow < SR) s_ysh[orow] = y;
                };
                ring_prime<DD>(sd_issue);
                ring_drain<DD>(n_sdi, sd_issue, sd_finish);
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                __builtin_amdgcn_wave_barrier();
            } else if (lane == 0) {
                s_fault = 1;
                __hip_atomic_store(q.fault, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            }
        }
        const int n_di = (R + pd.rw_count - 1) / pd.rw_count, n_w0 = router_wave_down_items(n_di);
        if (n_w0 > 0 && *(volatile int*)&s_f_route == 1) {
            // ---- this wavefront's share of the down rows of the group's expert: the one the exact routing names, so
            // its rows are requested at once and contracted when the pass that gathers that expert's activations is
            // through (the first if the guess was right, the second otherwise)
            const int e_fin = __builtin_amdgcn_readfirstlane(s_final[g]);
            const int through = 6 * (__builtin_amdgcn_readfirstlane(s_spec[g]) == e_fin ? 1 : 2);
            const uint8_t* rows0 = p.down + (size_t)e_fin * p.down_stride + (size_t)m * R * rb_d;
            const int i0 = n_di - n_w0;
            auto wd_issue = [&](int slot, int j) __attribute__((always_inline)) {
                ring[slot] = load_row<FD>(pd, rows0 + (size_t)min((i0 + j) * pd.rw_count + pd.rw, R - 1) * rb_d);
            };
            ring_prime<DD>(wd_issue);
            int v;
            bool lost = false;   // a streaming wavefront that gave up has raised the fault: the count will not come
            while ((((v = __builtin_amdgcn_readfirstlane(*(volatile int*)&s_h_done)) & 0xFF) < through) && !(v >> 8) &&
                   !(lost = __builtin_amdgcn_readfirstlane(*(volatile int*)&s_fault) != 0))
                __builtin_amdgcn_s_sleep(1);
            asm volatile("" ::: "memory");
            if (!(v >> 8) && !lost) {
                FD::fetch_x(xd, hcells, pd.blk, pd.sub);
                const bool scaled = p.down_scale != nullptr;
                const float ds = scaled ? p.down_scale[e_fin] : 1.0f;
                uint64_t* part = q.ypart + (size_t)g * ne + (size_t)m * R;
                const uint32_t ytag = seq_tag | (uint32_t)e_fin;
                auto wd_finish = [&](int slot, int j) __attribute__((always_inline)) {
                    const int orow = (i0 + j) * pd.rw_count + pd.rw;
                    const float y = row_sum<FD>(FD::dot(ring[slot], pd.sub, xd), pd, nblk_d);
                    if (pd.writer() && orow < R) rec_store(part + orow, scaled ? __fmul_rn(y, ds) : y, ytag);
                };
                ring_drain<DD>(n_w0, wd_issue, wd_finish);
            }
        }
        const bool mine = lane < SR;
        const size_t oi = (size_t)m * R + (size_t)g * SR + (mine ? lane : 0);
        uint64_t yk[kGroups];
        bool ok = *(volatile int*)&s_f_route == 1;
        if (ok) {
            for (int spin = 0;; spin++) {
#pragma unroll
                for (int k = 0; k < kGroups; k++) yk[k] = rec_load(q.ypart + (size_t)s_gor[k] * ne + oi);   // rank order
                bool got = true;
#pragma unroll
                for (int k = 0; k < kGroups; k++) got = got && (uint32_t)(yk[k] >> 32) == (seq_tag | (uint32_t)s_ids[k]);
                if (__all(got || !mine)) break;
                if (spin >= spin_limit) {
                    ok = false;
                    break;
                }
            }
            if (!ok && lane == 0) {
                s_fault = 1;
                __hip_atomic_store(q.fault, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            }
        }
        STAMP(12);
        if (ok && mine && !*(volatile int*)&s_fault) {
            float acc = 0.0f;
#pragma unroll
            for (int k = 0; k < kGroups; k++) acc = __fadd_rn(acc, __fmul_rn(s_w[k], __uint_as_float((uint32_t)yk[k])));
            if (shared) {
                float ws = 1.0f;
                if (p.sh_logit)   // crates/infr-cpu/src/lib.rs:3336-3356: sigmoid of the row's gate logit
                    ws = __fdiv_rn(1.0f, __fadd_rn(1.0f, expf_libm(-p.sh_logit[0], s_tab)));   // this row's: the pointer was advanced
                acc = __fadd_rn(acc, __fmul_rn(ws, s_ysh[lane]));
            }
            p.dst[oi] = p.addend ? __fadd_rn(p.addend[oi], acc) : acc;
        }
        STAMP(13);
        if (lane == 0) q.cnt[b] = s_seq;
    }
}

// ---------------------------------------------------------------------------------------------
struct StreamShape {
    int dg, dd, ept, nsp, epb, once, early_down;
    size_t lds;
};

namespace {

template <class FG, class FD, int DG, int DD, int EPT, int NSP, int NE = 0, int NFF = 0, int ROWS = 0, int NORM = 0>
bool launch_stream(hipStream_t s, const MoeLayerParams& q, size_t lds) {
    static bool attr_ok[16] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16) return false;
    if (!attr_ok[dev]) {
        if (hipFuncSetAttribute((const void*)moe_layer_stream<FG, FD, DG, DD, EPT, NSP, NE, NFF, ROWS, NORM>,
                                hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024) != hipSuccess)
            return false;
        attr_ok[dev] = true;
    }
    INFR_LAUNCH((moe_layer_stream<FG, FD, DG, DD, EPT, NSP, NE, NFF, ROWS, NORM>), dim3(kBlocks), dim3(kThreads), lds, s, q);
    return true;
}

}  // namespace

// The instantiations with compile-time sizes (k_layer_stream_shapes.hip).  *taken: one of them matches the shape; the
// return value is then that of the launch (true without launching when `launch` is false).
bool launch_stream_fixed(hipStream_t s, const MoeLayerParams& q, const StreamShape& sh, bool launch, bool* taken);

}  // namespace infr

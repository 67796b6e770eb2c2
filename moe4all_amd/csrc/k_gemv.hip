// Decode-regime expert kernels: id-indexed dequant-GEMV over the gate/up banks with the
// gated activation fused (h = act(gate.x) * (up.x)), and over the down bank with the
// rank-ordered weighted combine fused into the epilogue.
//
// Layout: a wavefront owns whole weight rows.  Every lane owns a FIXED slice of the K
// dimension (64 elements for the K-quants, 32 for Q8_0), so its slice of the activation
// vector is prepared once and stays in registers for all rows the wavefront streams; only
// packed weight blocks move from HBM, in 128-bit loads.  A row of nblk blocks occupies
// nblk*LPB consecutive lanes (LPB = lanes per block); when that is <= 32 several rows ride in
// one wavefront side by side.  All weight loads of a round are issued before the first dot.
//
// Arithmetic.  The lane's activation slice is held as 23-bit fixed point per group of 16/32
// elements, x ~ 2^k * X with |X| <= 2^21 (k from the group's largest magnitude; a power of
// two, so scaling is exact), and X is split into three signed bytes X = 65536*A + 256*B + C.
// Packed weight codes q (4, 6 or 8 bits) contract with A, B and C in V_DOT4_I32_I8; the three
// integer sums are exact and are joined in f32, which rounds the group's sum(q*x~) once at
// 2^-24 relative.  The block scales are applied in f32 in factored form,
//     (d*sc) * sum(q*x~) + (dmin*m) * sum(x~),
// so a one-hot x reads back the reference's decoded weight bit for bit
// (crates/infr-gguf/src/dequant.rs:35-51).  For general x the rounding of x to 2^-22 of its
// group's largest magnitude is of the order of f32's own 2^-24, so results track the f32
// reference as closely as a reordered f32 summation does.
#include "device_common.h"
#include "kernels.h"
#ifdef INFR_GEMV_TRACE
// the routing's own time stamps go to slots 8..15 of the block's record
namespace infr { __device__ long long* g_route_trace; }
#define ROUTE_STAMP(i)                                                                                                 \
    do {                                                                                                               \
        if (lane == 0 && infr::g_route_trace) infr::g_route_trace[((size_t)blockIdx.y * gridDim.x + blockIdx.x) * 16 + 8 + (i)] = wall_clock64(); \
    } while (0)
#endif
#include "route.h"
#include "gemv_fmt.h"

namespace infr {

// Time stamps of every block for a measurement build (-DINFR_GEMV_TRACE with a buffer in p.y, which these kernels do
// not use otherwise); compiled out in the library.
#ifdef INFR_GEMV_TRACE
#define GEMV_STAMP(i)                                                                                                  \
    do {                                                                                                               \
        if (threadIdx.x == 0 && p.y) reinterpret_cast<long long*>(p.y)[((size_t)blockIdx.y * gridDim.x + blockIdx.x) * 16 + (i)] = wall_clock64(); \
    } while (0)
#else
#define GEMV_STAMP(i) do { } while (0)
#endif

// ------------------------------------------------------------------------------- gate/up
// grid.x = tiles of `ft` features, grid.y = token row.  A block's 4 waves share the items
// (slot, f) of its tile; x is identical for every slot of a token.  U = items a wave has in
// flight per round.  Results wait in LDS and one lane per item applies the gated activation
// after the round, so the f64 exp and the divide run once per wave, not once per item.
// One stage of a wave's work: U (gate row, up row) pairs per row lane group, loaded together.
template <class F, int U>
struct GuStage { typename F::Raw g[U], u[U]; };

struct GuTile {
    int r, f0, fcount, nitems, n_slots, wave, lane;
    size_t row_bytes;
};

// Issue every load of the stage that starts at item `base`; items past the end re-read the last.
template <class F, int U>
__device__ __forceinline__ void gu_issue(GuStage<F, U>& st, const MoeGemvParams& p, const Place<F>& pl, const GuTile& t,
                                         const int32_t* s_ids, int base) {
#pragma unroll
    for (int u = 0; u < U; u++) {
        const int it = min(base + (u * 4 + t.wave) * pl.rw_count + pl.rw, t.nitems - 1);
        const int slot = it / t.fcount, f = t.f0 + (it - slot * t.fcount);
        const int e = s_ids[slot];
        const bool routed = slot < p.n_used;
        const uint8_t* gb = routed ? p.gate + (size_t)e * p.gate_stride : p.sh_gate;
        const uint8_t* ub = routed ? p.up + (size_t)e * p.up_stride : p.sh_up;
        st.g[u] = load_row<F>(pl, gb + (size_t)f * t.row_bytes);
        st.u[u] = load_row<F>(pl, ub + (size_t)f * t.row_bytes);
    }
}

// Dot the stage's rows with x; results wait in LDS and one lane per item applies the gated
// activation, so the f64 exp and the divide run once per wave, not once per item.
template <class F, int U>
__device__ __forceinline__ void gu_finish(const GuStage<F, U>& st, const MoeGemvParams& p, const Place<F>& pl,
                                          const GuTile& t, const typename F::X& x, int nblk, int base, float (*s_g)[64],
                                          float (*s_u)[64], const float* s_w, const uint64_t* s_tab) {
#pragma unroll
    for (int u = 0; u < U; u++) {
        float gs = row_sum<F>(F::dot(st.g[u], pl.sub, x), pl, nblk);
        float us = row_sum<F>(F::dot(st.u[u], pl.sub, x), pl, nblk);
        if (pl.writer()) {
            s_g[t.wave][u * pl.rw_count + pl.rw] = gs;
            s_u[t.wave][u * pl.rw_count + pl.rw] = us;
        }
    }
    __builtin_amdgcn_wave_barrier();
    if (t.lane < U * pl.rw_count) {
        const int u = t.lane / pl.rw_count, rw = t.lane - u * pl.rw_count;
        const int it = base + (u * 4 + t.wave) * pl.rw_count + rw;
        if (it < t.nitems) {
            const int slot = it / t.fcount, f = t.f0 + (it - slot * t.fcount);
            float gs = s_g[t.wave][t.lane], us = s_u[t.wave][t.lane];
            if (p.weight_before && slot < p.n_used) {
                const float wp = s_w[slot];
                gs = __fmul_rn(wp, gs);
                us = __fmul_rn(wp, us);
            }
            p.h[((size_t)t.r * t.n_slots + slot) * p.nff + f] = gated_act_fn(p.act, p.has_clamp, p.clamp, gs, us, s_tab);
        }
    }
    __builtin_amdgcn_wave_barrier();
}

// Tiles of at most two items per wave (larger tiles go to moe_gate_up_stream): every load of the block is in flight at
// once, then the items are finished.
template <class F, int U>
__global__ __launch_bounds__(256) void moe_gate_up_fast(MoeGemvParams p, int ft) {
    extern __shared__ __attribute__((aligned(16))) uint32_t dyn_lds[];
    __shared__ uint64_t s_tab[32];
    __shared__ int32_t s_ids[64];
    __shared__ float s_w[64];
    __shared__ float s_g[4][64], s_u[4][64];
    GuTile t;
    t.r = blockIdx.y;
    t.f0 = blockIdx.x * ft;
    t.fcount = min(ft, p.nff - t.f0);
    t.wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    t.lane = threadIdx.x & 63;
    const int r = t.r, wave = t.wave, lane = t.lane;
    const int nblk = p.ne / F::kBlockElems;
    t.row_bytes = (size_t)nblk * F::kBlockBytes;
    const Place<F> pl(nblk, lane);
    const size_t cell_words = (size_t)((p.ne + 31) / 32) * kCellDwords;
    uint32_t* cells = dyn_lds + (size_t)wave * cell_words;
    GEMV_STAMP(0);
    // x is requested first; it does not depend on the routing
    const float* xrow = p.x + (size_t)r * p.ne;
    const XLoad xl = stage_x_load(xrow, p.ne, lane);
    if (threadIdx.x < 32) s_tab[threadIdx.x] = kExp2Table[threadIdx.x];
    if (p.route_inline) {
        // every block routes its token row itself (one wave, redundantly across blocks)
        __syncthreads();
        if (wave == 0)
            route_row_any(p.route, r, lane, reinterpret_cast<float*>(dyn_lds + 4 * cell_words), s_tab, s_ids, s_w,
                          blockIdx.x == 0);
    } else if ((int)threadIdx.x < p.n_used) {  // n_used <= 64
        s_ids[threadIdx.x] = p.ids[(size_t)r * p.n_used + threadIdx.x];
        s_w[threadIdx.x] = p.weights[(size_t)r * p.n_used + threadIdx.x];
    }
    t.n_slots = p.n_used + (p.sh_gate ? 1 : 0);   // the always-on expert is slot n_used (<= 63 then)
    if (p.sh_gate && threadIdx.x == 255) {
        s_ids[p.n_used] = 0;
        s_w[p.n_used] = 1.0f;
    }
    __syncthreads();
    __builtin_amdgcn_wave_barrier();
    GEMV_STAMP(1);
    t.nitems = t.fcount * t.n_slots;
    const int step = 4 * pl.rw_count * U;
    typename F::X x;
    bool have_x = false;
    for (int base = 0; base < t.nitems; base += step) {
        GuStage<F, U> st;
        gu_issue<F, U>(st, p, pl, t, s_ids, base);
        if (!have_x) {
            // while the weights are in flight: the wave converts x to fixed point once, together
            stage_x_finish<F::kGroup, F::kSigned>(xl, xrow, p.ne, cells, lane);
            __builtin_amdgcn_wave_barrier();
            F::fetch_x(x, cells, pl.blk, pl.sub);
            have_x = true;
            GEMV_STAMP(2);
        }
        gu_finish<F, U>(st, p, pl, t, x, nblk, base, s_g, s_u, s_w, s_tab);
        if (base == 0) GEMV_STAMP(3);
    }
    GEMV_STAMP(4);
}

// ------------------------------------------------------------------------------- gate/up, streamed
// The same tiles as moe_gate_up_fast, for tiles of several items per wave, on NW waves (8 to 12).  Three things differ.
// The routing and the conversion of x run side by side: waves 0 and 1 route (plain softmax: the sum on one, the
// selection on the other; anything else on wave 0 alone; or wave 0 fetches the ids) while the remaining waves turn x
// into one set of fixed-point cells for the whole block.  A wave keeps D items (a gate row and an up row each) in
// flight as a ring: it finishes the oldest item and requests the item D places ahead into the registers that just
// became free, so its dot products and its loads alternate item by item and the waves drift apart instead of all
// waiting for memory and then all computing; many waves with a shallow ring measured faster than few with a deep one.
// Results wait in LDS until the wave has finished a chunk of its items, then one lane per item applies the gated
// activation.  The second launch bound (waves per SIMD) keeps two 8-wave blocks resident on a compute unit.
// NBLK: blocks per weight row when known at compile time (the benchmark shapes), 0 for any: the lane placement and the
// index arithmetic around the dots then fold.
template <class F, int D, int NW, int NBLK = 0>
__global__ __launch_bounds__(64 * NW, NW <= 8 ? 4 : 3) void moe_gate_up_stream(MoeGemvParams p, int ft) {
    extern __shared__ __attribute__((aligned(16))) uint32_t dyn_lds[];
    __shared__ uint64_t s_tab[32];
    __shared__ int32_t s_ids[64];
    __shared__ float s_w[64];
    __shared__ float s_g[NW][64], s_u[NW][64];
    __shared__ RouteDuo s_duo;
    const int r = blockIdx.y;
    const int f0 = blockIdx.x * ft;
    const int fcount = min(ft, p.nff - f0);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;   // uniform: scalar registers
    const int nblk = NBLK ? NBLK : p.ne / F::kBlockElems;
    const size_t row_bytes = (size_t)nblk * F::kBlockBytes;
    const Place<F> pl(nblk, lane);
    const int ncell = (p.ne + 31) / 32;
    uint32_t* cells = dyn_lds;
    GEMV_STAMP(0);
    const float* xrow = p.x + (size_t)r * p.ne;
    float* route_lds = reinterpret_cast<float*>(dyn_lds + (size_t)ncell * kCellDwords);
    // plain softmax routing runs on waves 0 and 1 (sum and selection side by side), anything else on wave 0
    const int duo_ns = !(p.route_inline && route_duo_ok(p.route)) ? 0 : p.route.n_expert <= 128 ? 2 : p.route.n_expert <= 256 ? 4 : 8;
    const int first_conv = duo_ns ? 2 : 1;   // the waves from here on turn x into cells
    float pr[8];
    if (wave < first_conv) {
        if (duo_ns == 2) route_duo_first<2>(p.route, r, wave, lane, route_lds, s_tab, &s_duo, reinterpret_cast<float(&)[2]>(pr));
        else if (duo_ns == 4) route_duo_first<4>(p.route, r, wave, lane, route_lds, s_tab, &s_duo, reinterpret_cast<float(&)[4]>(pr));
        else if (duo_ns == 8) route_duo_first<8>(p.route, r, wave, lane, route_lds, s_tab, &s_duo, pr);
        else if (p.route_inline) {
            route_row_any(p.route, r, lane, route_lds, s_tab, s_ids, s_w, blockIdx.x == 0, s_tab);
        } else {
            if (lane < p.n_used) {   // n_used <= 64
                s_ids[lane] = p.ids[(size_t)r * p.n_used + lane];
                s_w[lane] = p.weights[(size_t)r * p.n_used + lane];
            }
            if (lane < 32) s_tab[lane] = kExp2Table[lane];
        }
    } else {
        for (int c0 = (int)threadIdx.x - 64 * first_conv; c0 < ncell; c0 += 64 * (NW - first_conv)) {
            const XLoad l = stage_x_load(xrow, p.ne, c0);
            stage_x_convert<F::kGroup, F::kSigned>(l, p.ne, c0, cells);
        }
    }
    const int n_slots = p.n_used + (p.sh_gate ? 1 : 0);   // the always-on expert is slot n_used (<= 63 then)
    if (p.sh_gate && threadIdx.x == 64 * NW - 1) {
        s_ids[p.n_used] = 0;
        s_w[p.n_used] = 1.0f;
    }
    __syncthreads();
    if (duo_ns) {
        if (wave == 0) {
            const bool store = blockIdx.x == 0;
            bool done;
            if (duo_ns == 2) done = route_duo_second<2>(p.route, r, lane, &s_duo, reinterpret_cast<float(&)[2]>(pr), s_ids, s_w, store);
            else if (duo_ns == 4) done = route_duo_second<4>(p.route, r, lane, &s_duo, reinterpret_cast<float(&)[4]>(pr), s_ids, s_w, store);
            else done = route_duo_second<8>(p.route, r, lane, &s_duo, pr, s_ids, s_w, store);
            if (!done) route_row_any(p.route, r, lane, route_lds, s_tab, s_ids, s_w, store);
        }
        __syncthreads();
    }
    GEMV_STAMP(1);
    typename F::X x;   // fetched once the first items are requested
    const int nitems = fcount * n_slots;
    const int per_step = NW * pl.rw_count;   // items the block's waves take per ring step
    const int n_mine = nitems > wave * pl.rw_count ? (nitems - wave * pl.rw_count + per_step - 1) / per_step : 0;
    const float inv_fcount = 1.0f / (float)fcount;
    // item j of this wave's rows: (slot, feature), exact for the few thousand items a tile can hold
    // (rows of 64 lanes: one item per wave and step, so slot, expert and row address are the same in every lane and are
    // kept in scalar registers; the loads then take a scalar base and the lane's block offset)
    const bool one_row = pl.rw_count == 1;
    auto issue = [&](GuStage<F, 1>& st, int j) {
        const int it = min((j * NW + wave) * pl.rw_count + pl.rw, nitems - 1);
        int slot = (int)(((float)it + 0.5f) * inv_fcount);
        if (one_row) slot = __builtin_amdgcn_readfirstlane(slot);
        const int f = f0 + ((one_row ? __builtin_amdgcn_readfirstlane(it) : it) - slot * fcount);
        int e = s_ids[slot];
        if (one_row) e = __builtin_amdgcn_readfirstlane(e);
        const bool routed = slot < p.n_used;
        const uint8_t* gb = routed ? p.gate + (size_t)e * p.gate_stride : p.sh_gate;
        const uint8_t* ub = routed ? p.up + (size_t)e * p.up_stride : p.sh_up;
        st.g[0] = load_row<F>(pl, gb + (size_t)f * row_bytes);
        st.u[0] = load_row<F>(pl, ub + (size_t)f * row_bytes);
    };
    const int chunk = 64 / pl.rw_count;   // items of a wave whose results fit its staging row
    for (int c0 = 0; c0 < n_mine; c0 += chunk) {
        const int cn = min(chunk, n_mine - c0);
        GuStage<F, 1> ring[D];
        auto finish = [&](const GuStage<F, 1>& st, int j) {
            const float gs = row_sum<F>(F::dot(st.g[0], pl.sub, x), pl, nblk);
            const float us = row_sum<F>(F::dot(st.u[0], pl.sub, x), pl, nblk);
            if (pl.writer()) {
                s_g[wave][j * pl.rw_count + pl.rw] = gs;
                s_u[wave][j * pl.rw_count + pl.rw] = us;
            }
        };
#pragma unroll
        for (int d = 0; d < D; d++)
            if (d < cn) issue(ring[d], c0 + d);
        if (c0 == 0) {
            F::fetch_x(x, cells, pl.blk, pl.sub);
            GEMV_STAMP(2);
        }
        // steady state: every step finishes its ring entry and refills it, no branch in between, so the waits count
        // exactly the loads that are younger than the entry
        const int refills = cn - D;   // steps that still have an item to request
        int j0 = 0;
        for (; j0 + D <= refills; j0 += D) {
#pragma unroll
            for (int d = 0; d < D; d++) {
                finish(ring[d], j0 + d);
                issue(ring[d], c0 + j0 + d + D);
            }
            if (c0 == 0 && j0 == 0) GEMV_STAMP(3);
        }
        // the last refills, then the entries still in flight
#pragma unroll
        for (int d = 0; d < D; d++) {
            if (j0 + d >= cn) break;
            finish(ring[d], j0 + d);
            if (j0 + d < refills) issue(ring[d], c0 + j0 + d + D);
        }
        j0 += D;
#pragma unroll
        for (int d = 0; d < D; d++) {
            if (j0 + d >= cn) break;
            finish(ring[d], j0 + d);
        }
        __builtin_amdgcn_wave_barrier();
        if (lane < cn * pl.rw_count) {
            const int j = lane / pl.rw_count, rw = lane - j * pl.rw_count;
            const int it = ((c0 + j) * NW + wave) * pl.rw_count + rw;
            if (it < nitems) {
                const int slot = (int)(((float)it + 0.5f) * inv_fcount), f = f0 + (it - slot * fcount);
                float gs = s_g[wave][lane], us = s_u[wave][lane];
                if (p.weight_before && slot < p.n_used) {
                    const float wp = s_w[slot];
                    gs = __fmul_rn(wp, gs);
                    us = __fmul_rn(wp, us);
                }
                p.h[((size_t)r * n_slots + slot) * p.nff + f] = gated_act_fn(p.act, p.has_clamp, p.clamp, gs, us, s_tab);
            }
        }
        __builtin_amdgcn_wave_barrier();
    }
    GEMV_STAMP(4);
}

// ------------------------------------------------------------------------------- down
// grid.x = tiles of `ot` = S * rows-per-wave output rows, grid.y = token row.  One wave per
// slot: it holds that slot's h and streams the S row groups of its expert's down matrix, all
// loads issued up front.  The per-slot results meet in LDS and are combined in rank order:
// out += w_rank * y_rank as a separate multiply and add
// (crates/infr-cpu/src/lib.rs:4290-4302).
constexpr int kMaxUsedFast = 16;
constexpr int kMaxOt = 128;

struct DownTile {
    int slot, ocount;
    size_t row_bytes;
    bool scaled;
    float ds;
};

// Issue the loads of the S row groups that start at output row `obase` of the tile; rows past
// the tile re-read its last row.
template <class F, int S>
__device__ __forceinline__ void down_issue(typename F::Raw (&raw)[S], const Place<F>& pl, const DownTile& t,
                                           const uint8_t* bank, int obase) {
#pragma unroll
    for (int st = 0; st < S; st++) {
        const int o = min(obase + st * pl.rw_count + pl.rw, t.ocount - 1);
        raw[st] = load_row<F>(pl, bank + (size_t)o * t.row_bytes);
    }
}

template <class F, int S>
__device__ __forceinline__ void down_finish(const typename F::Raw (&raw)[S], const Place<F>& pl, const DownTile& t,
                                            const typename F::X& x, int nblk, int obase, float (*ypart)[kMaxOt]) {
#pragma unroll
    for (int st = 0; st < S; st++) {
        const int o = obase + st * pl.rw_count + pl.rw;
        float y = row_sum<F>(F::dot(raw[st], pl.sub, x), pl, nblk);
        if (o < t.ocount && pl.writer()) ypart[t.slot][o] = t.scaled ? __fmul_rn(y, t.ds) : y;
    }
}

// PIPE == false: ot = S row groups, all loaded up front (single-token decode: everything in
// flight at once).  PIPE == true: the tile is any number of stages of S row groups; a wave keeps
// the next stage's loads in flight while it finishes the current one.
template <class F, int S, bool PIPE>
__global__ __launch_bounds__(512) void moe_down_combine_fast(MoeGemvParams p, int ot) {
    extern __shared__ __attribute__((aligned(16))) uint32_t dyn_lds[];
    __shared__ float ypart[kMaxUsedFast][kMaxOt];
    const int r = blockIdx.y;
    const int o0 = blockIdx.x * ot;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;   // uniform: scalar registers
    const int nwaves = blockDim.x >> 6;
    const int nblk = p.nff / F::kBlockElems;
    const Place<F> pl(nblk, lane);
    const int32_t* ids = p.ids + (size_t)r * p.n_used;
    uint32_t* cells = dyn_lds + (size_t)wave * ((p.nff + 31) / 32) * kCellDwords;
    DownTile t;
    t.ocount = min(ot, p.ne - o0);
    t.row_bytes = (size_t)nblk * F::kBlockBytes;
    GEMV_STAMP(0);

    const int n_slots = p.n_used + (p.sh_down ? 1 : 0);   // the always-on expert is slot n_used
    for (int slot = wave; slot < n_slots; slot += nwaves) {
        const bool routed = slot < p.n_used;
        const int e = routed ? ids[slot] : 0;  // first: every weight address below waits on it
        const float* hrow = p.h + ((size_t)r * n_slots + slot) * p.nff;
        const XLoad xl = stage_x_load(hrow, p.nff, lane);
        const uint8_t* bank = (routed ? p.down + (size_t)e * p.down_stride : p.sh_down) + (size_t)o0 * t.row_bytes;
        t.slot = slot;
        t.scaled = p.down_scale && routed;
        typename F::Raw ra[S];
        down_issue<F, S>(ra, pl, t, bank, 0);
        if (slot == wave) GEMV_STAMP(1);
        typename F::X x;
        if (!PIPE) {
            // while the weights are in flight: this slot's h to fixed point, once per wave
            __builtin_amdgcn_wave_barrier();
            stage_x_finish<F::kGroup, F::kSigned>(xl, hrow, p.nff, cells, lane);
            __builtin_amdgcn_wave_barrier();
            F::fetch_x(x, cells, pl.blk, pl.sub);
            if (slot == wave) GEMV_STAMP(2);
            t.ds = t.scaled ? p.down_scale[e] : 1.0f;
            down_finish<F, S>(ra, pl, t, x, nblk, 0, ypart);
            if (slot == wave) GEMV_STAMP(3);
        } else {
            const int gstep = S * pl.rw_count;
            typename F::Raw rb[S];
            down_issue<F, S>(rb, pl, t, bank, gstep);
            __builtin_amdgcn_wave_barrier();
            stage_x_finish<F::kGroup, F::kSigned>(xl, hrow, p.nff, cells, lane);
            __builtin_amdgcn_wave_barrier();
            F::fetch_x(x, cells, pl.blk, pl.sub);
            t.ds = t.scaled ? p.down_scale[e] : 1.0f;
            down_finish<F, S>(ra, pl, t, x, nblk, 0, ypart);
            int o = gstep;   // the stage rb holds
            for (;;) {
                if (o + gstep >= t.ocount) {
                    down_finish<F, S>(rb, pl, t, x, nblk, o, ypart);
                    break;
                }
                down_issue<F, S>(ra, pl, t, bank, o + gstep);
                down_finish<F, S>(rb, pl, t, x, nblk, o, ypart);
                o += gstep;
                if (o + gstep >= t.ocount) {
                    down_finish<F, S>(ra, pl, t, x, nblk, o, ypart);
                    break;
                }
                down_issue<F, S>(rb, pl, t, bank, o + gstep);
                down_finish<F, S>(ra, pl, t, x, nblk, o, ypart);
                o += gstep;
            }
            __builtin_amdgcn_wave_barrier();   // the next slot's h overwrites this wave's cells
        }
    }
    GEMV_STAMP(4);
    __syncthreads();
    GEMV_STAMP(5);
    for (int o = threadIdx.x; o < t.ocount; o += blockDim.x) {
        const float* w = p.weights + (size_t)r * p.n_used;
        float acc = 0.0f;
        for (int k = 0; k < n_slots; k++) {
            if (p.skip_zero_w && k < p.n_used && w[k] == 0.0f) continue;
            float wk = (p.weight_before || k >= p.n_used) ? 1.0f : w[k];
            if (k >= p.n_used && p.sh_logit)   // crates/infr-cpu/src/lib.rs:3336-3356: sigmoid of the row's gate logit
                wk = __fdiv_rn(1.0f, __fadd_rn(1.0f, expf_libm(-p.sh_logit[r])));
            acc = __fadd_rn(acc, __fmul_rn(wk, ypart[k][o]));
        }
        const size_t oi = (size_t)r * p.ne + o0 + o;
        p.dst[oi] = p.addend ? __fadd_rn(p.addend[oi], acc) : acc;
    }
    GEMV_STAMP(6);
}

// ------------------------------------------------------------------------------- down, streamed
// The same tiles as moe_down_combine_fast with the work cut differently: a tile's units (slot, group of rows a wave
// covers at once) are dealt to the block's NW waves in equal contiguous runs, so nine slots keep every wave equally
// busy, and a wave keeps D units in flight as a ring (finish the oldest, request the unit D places ahead into the
// registers that became free).  h of every slot is turned into fixed-point cells once, by the whole block; a wave
// fetches a slot's cells when its run crosses into that slot.
template <class F, int D, int NW, int NBLK = 0>
__global__ __launch_bounds__(64 * NW) void moe_down_combine_stream(MoeGemvParams p, int ot) {
    extern __shared__ __attribute__((aligned(16))) uint32_t dyn_lds[];
    __shared__ float ypart[kMaxUsedFast][kMaxOt];
    __shared__ int32_t s_ids[kMaxUsedFast];
    __shared__ float s_w[kMaxUsedFast], s_ds[kMaxUsedFast];
    __shared__ int s_skip[kMaxUsedFast];
    const int r = blockIdx.y;
    const int o0 = blockIdx.x * ot;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;   // uniform: scalar registers
    const int nblk = NBLK ? NBLK : p.nff / F::kBlockElems;
    const Place<F> pl(nblk, lane);
    const size_t row_bytes = (size_t)nblk * F::kBlockBytes;
    const int ocount = min(ot, p.ne - o0);
    const int n_slots = p.n_used + (p.sh_down ? 1 : 0);   // the always-on expert is slot n_used
    const int ncell = (p.nff + 31) / 32;
    const size_t cell_words = (size_t)ncell * kCellDwords;
    GEMV_STAMP(0);
    // ids and routing weights first: every weight address waits on the ids
    if ((int)threadIdx.x < n_slots) {
        const int k = threadIdx.x;
        const bool routed = k < p.n_used;
        const int e = routed ? p.ids[(size_t)r * p.n_used + k] : 0;
        const float w = routed ? p.weights[(size_t)r * p.n_used + k] : 1.0f;
        float wk = (p.weight_before || !routed) ? 1.0f : w;
        if (!routed && p.sh_logit)   // crates/infr-cpu/src/lib.rs:3336-3356: sigmoid of the row's gate logit
            wk = __fdiv_rn(1.0f, __fadd_rn(1.0f, expf_libm(-p.sh_logit[r])));
        s_ids[k] = e;
        s_w[k] = wk;
        s_skip[k] = p.skip_zero_w && routed && w == 0.0f;
        s_ds[k] = (p.down_scale && routed) ? p.down_scale[e] : 1.0f;
    }
    // h of every slot, requested before the weights so that its conversion does not wait behind them
    const int total_cells = n_slots * ncell;
    const int my_cell = threadIdx.x;   // further cells of this thread follow in the loop below
    const int slot0 = my_cell / ncell;
    const float* hbase = p.h + (size_t)r * n_slots * p.nff;
    XLoad hl;
    if (my_cell < total_cells) hl = stage_x_load(hbase + (size_t)slot0 * p.nff, p.nff, my_cell - slot0 * ncell);
    __syncthreads();
    const int G = (ocount + pl.rw_count - 1) / pl.rw_count;   // units per slot
    const int n_units = n_slots * G;
    // equal contiguous runs, the remainder one unit each to the first waves (72 units on 16 waves: 5 for eight waves and
    // 4 for eight, so every SIMD's four waves carry 18, not 20 on two SIMDs and 15 on another)
    const int base_units = n_units / NW, rem_units = n_units - base_units * NW;
    const int ub = wave * base_units + min(wave, rem_units);
    const int cn = base_units + (wave < rem_units ? 1 : 0);
    // Units are taken in order, once by the requests and once by the dots: two cursors (slot, row group) that step
    // through the run, in scalar registers (the wave's index is uniform), instead of a division per unit.
    const int slot_first = __builtin_amdgcn_readfirstlane((int)(((float)ub + 0.5f) * (1.0f / (float)G)));
    int i_slot = slot_first, i_rg = ub - slot_first * G;   // cursor of the requests
    const uint8_t* i_bank = nullptr;
    int i_bank_slot = -1;
    auto issue = [&](typename F::Raw& raw, int) {
        if (i_slot != i_bank_slot) {   // the same for the whole wave
            const int e = __builtin_amdgcn_readfirstlane(s_ids[i_slot < n_slots ? i_slot : 0]);
            i_bank = i_slot < p.n_used ? p.down + (size_t)e * p.down_stride : p.sh_down;
            i_bank_slot = i_slot;
        }
        const int o = min(i_rg * pl.rw_count + pl.rw, ocount - 1);
        raw = load_row<F>(pl, i_bank + (size_t)(o0 + o) * row_bytes);
        if (++i_rg == G) {
            i_rg = 0;
            i_slot++;
        }
    };
    typename F::Raw ring[D];
#pragma unroll
    for (int d = 0; d < D; d++)
        if (d < cn) issue(ring[d], d);
    GEMV_STAMP(1);
    // h to fixed point, once per block
    if (my_cell < total_cells)
        stage_x_convert<F::kGroup, F::kSigned>(hl, p.nff, my_cell - slot0 * ncell, dyn_lds + slot0 * cell_words);
    for (int c = my_cell + (int)blockDim.x; c < total_cells; c += blockDim.x) {
        const int sl = c / ncell;
        const XLoad l = stage_x_load(hbase + (size_t)sl * p.nff, p.nff, c - sl * ncell);
        stage_x_convert<F::kGroup, F::kSigned>(l, p.nff, c - sl * ncell, dyn_lds + sl * cell_words);
    }
    __syncthreads();
    GEMV_STAMP(2);
    typename F::X x;
    int cur_slot = -1;
    float ds = 1.0f;
    int f_slot = slot_first, f_rg = ub - slot_first * G;   // cursor of the dots
    auto finish = [&](const typename F::Raw& raw, int) {
        const int slot = f_slot, rg = f_rg;
        if (slot != cur_slot) {   // the same for the whole wave
            F::fetch_x(x, dyn_lds + slot * cell_words, pl.blk, pl.sub);
            ds = s_ds[slot];
            cur_slot = slot;
        }
        const int o = rg * pl.rw_count + pl.rw;
        const float y = row_sum<F>(F::dot(raw, pl.sub, x), pl, nblk);
        if (o < ocount && pl.writer()) ypart[slot][o] = (p.down_scale && slot < p.n_used) ? __fmul_rn(y, ds) : y;
        if (++f_rg == G) {
            f_rg = 0;
            f_slot++;
        }
    };
    const int refills = cn - D;
    int j0 = 0;
    for (; j0 + D <= refills; j0 += D) {
#pragma unroll
        for (int d = 0; d < D; d++) {
            finish(ring[d], j0 + d);
            issue(ring[d], j0 + d + D);
        }
    }
#pragma unroll
    for (int d = 0; d < D; d++) {
        if (j0 + d >= cn) break;
        finish(ring[d], j0 + d);
        if (j0 + d < refills) issue(ring[d], j0 + d + D);
    }
    j0 += D;
#pragma unroll
    for (int d = 0; d < D; d++) {
        if (j0 + d >= cn) break;
        finish(ring[d], j0 + d);
    }
#ifdef INFR_GEMV_TRACE
    if (lane == 0 && p.y) reinterpret_cast<long long*>(p.y)[((size_t)blockIdx.y * gridDim.x + blockIdx.x) * 16 + 8 + (wave & 7)] = wall_clock64();
#endif
    GEMV_STAMP(4);
    __syncthreads();
    GEMV_STAMP(5);
    for (int o = threadIdx.x; o < ocount; o += blockDim.x) {
        float acc = 0.0f;
        for (int k = 0; k < n_slots; k++) {
            if (s_skip[k]) continue;
            acc = __fadd_rn(acc, __fmul_rn(s_w[k], ypart[k][o]));
        }
        const size_t oi = (size_t)r * p.ne + o0 + o;
        p.dst[oi] = p.addend ? __fadd_rn(p.addend[oi], acc) : acc;
    }
    GEMV_STAMP(6);
}

// ------------------------------------------------------------------------------- generic
// Any dtype decode_elem understands and any shape: one wave per output, lanes stride over K,
// plain f32.
__global__ __launch_bounds__(256) void moe_gate_up_generic(MoeGemvParams p, size_t g_row_bytes, size_t u_row_bytes) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;   // uniform: scalar registers
    const int f = blockIdx.x * 4 + wave;
    const int pair = blockIdx.y;
    if (f >= p.nff) return;
    const int r = pair / p.n_used;
    const int e = p.ids[pair];
    const uint8_t* grow = p.gate + (size_t)e * p.gate_stride + (size_t)f * g_row_bytes;
    const uint8_t* urow = p.up + (size_t)e * p.up_stride + (size_t)f * u_row_bytes;
    const float* x = p.x + (size_t)r * p.ne;
    float gs = 0.f, us = 0.f;
    for (int k = lane; k < p.ne; k += kWave) {
        float xv = x[k];
        gs = fmaf(decode_elem(p.gate_dt, grow, (uint32_t)k), xv, gs);
        us = fmaf(decode_elem(p.up_dt, urow, (uint32_t)k), xv, us);
    }
    gs = wave_sum(gs);
    us = wave_sum(us);
    if (lane == 0) {
        if (p.weight_before) {
            float wp = p.weights[pair];
            gs = __fmul_rn(wp, gs);
            us = __fmul_rn(wp, us);
        }
        p.h[(size_t)pair * p.nff + f] = gated_act_fn(p.act, p.has_clamp, p.clamp, gs, us);
    }
}

__global__ __launch_bounds__(256) void moe_down_combine_generic(MoeGemvParams p, size_t row_bytes) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;   // uniform: scalar registers
    const int o = blockIdx.x * 4 + wave;
    const int r = blockIdx.y;
    if (o >= p.ne) return;
    float acc = 0.0f;
    for (int slot = 0; slot < p.n_used; slot++) {
        const int e = p.ids[(size_t)r * p.n_used + slot];
        const uint8_t* row = p.down + (size_t)e * p.down_stride + (size_t)o * row_bytes;
        const float* h = p.h + ((size_t)r * p.n_used + slot) * p.nff;
        float y = 0.f;
        for (int k = lane; k < p.nff; k += kWave) y = fmaf(decode_elem(p.down_dt, row, (uint32_t)k), h[k], y);
        y = wave_sum(y);
        if (p.down_scale) y = __fmul_rn(y, p.down_scale[e]);
        if (p.skip_zero_w && p.weights[(size_t)r * p.n_used + slot] == 0.0f) continue;
        float wk = p.weight_before ? 1.0f : p.weights[(size_t)r * p.n_used + slot];
        acc = __fadd_rn(acc, __fmul_rn(wk, y));
    }
    if (lane == 0) {
        const size_t oi = (size_t)r * p.ne + o;
        p.dst[oi] = p.addend ? __fadd_rn(p.addend[oi], acc) : acc;
    }
}

// ------------------------------------------------------------------------------- dispatch
static size_t row_bytes_of(int dt, int in_f) {
    int be = 1, bb = 4;
    block_geometry(dt, &be, &bb);
    return (size_t)(in_f / be) * bb;
}

// The fast kernels cover rows of up to 64 lanes (K-quants: in_f <= 4096, Q8_0: in_f <= 2048).
template <class F>
static bool fast_ok(int in_f) {
    if (in_f <= 0 || in_f % F::kBlockElems != 0) return false;
    return in_f / F::kBlockElems * F::kLPB <= 64;
}

static int ceil_div(int a, int b) { return (a + b - 1) / b; }

template <class F>
static bool try_gate_up(hipStream_t s, const MoeGemvParams& p) {
    if (!fast_ok<F>(p.ne) || p.n_used > 64) return false;
    const int rw = 64 / (p.ne / F::kBlockElems * F::kLPB);
    // about one block per compute unit; a block's ft * n_slots items go to 4 waves of rw rows each
    const int n_slots = p.n_used + (p.sh_gate ? 1 : 0);
    // about one block per compute unit for a single token row; with several rows about two, resident together, so
    // that a compute unit pays a block's start (routing, x) once while it streams
    int ft = p.rows >= 2 ? ceil_div(p.nff, max(1, 2 * p.n_cu / p.rows)) : ceil_div(p.nff, p.n_cu);
    if (ft < 1) ft = 1;
    const int per_wave = ceil_div(ft * n_slots, 4 * rw);
    dim3 grid(ceil_div(p.nff, ft), p.rows), block(256);
    const size_t lds = 4 * cells_bytes(p.ne) +
                       (p.route_inline ? route_scratch_floats(p.route.n_expert, p.route.n_groups) * sizeof(float) : 0);
    if (per_wave >= 3) {
        // several items per wave: streamed, one set of cells for the block
        const size_t lds_s = cells_bytes(p.ne) +
                             (p.route_inline ? route_scratch_floats(p.route.n_expert, p.route.n_groups) * sizeof(float) : 0);
        // one token row: twelve waves, each with one item in flight, cover the memory latency between them; with
        // several rows two blocks of eight waves share a compute unit
        // the benchmark shapes' rows (2048 or 4096 elements) with their block count as a constant
        constexpr int kNb0 = 2048 / F::kBlockElems, kNb1 = 4096 / F::kBlockElems;
        const int nblk = p.ne / F::kBlockElems;
        if (p.rows == 1) INFR_LAUNCH((moe_gate_up_stream<F, 1, 12>), grid, dim3(768), lds_s, s, p, ft);
        else if (nblk == kNb0) INFR_LAUNCH((moe_gate_up_stream<F, 1, 8, kNb0>), grid, dim3(512), lds_s, s, p, ft);
        else if (nblk == kNb1 && kNb1 * F::kLPB <= 64) INFR_LAUNCH((moe_gate_up_stream<F, 1, 8, (kNb1 * F::kLPB <= 64 ? kNb1 : 0)>), grid, dim3(512), lds_s, s, p, ft);
        else INFR_LAUNCH((moe_gate_up_stream<F, 1, 8>), grid, dim3(512), lds_s, s, p, ft);
        return true;
    }
    if (per_wave == 2 && 2 * rw <= 64)   // U * rw results per wave must fit the 64-entry staging rows
        INFR_LAUNCH((moe_gate_up_fast<F, 2>), grid, block, lds, s, p, ft);
    else INFR_LAUNCH((moe_gate_up_fast<F, 1>), grid, block, lds, s, p, ft);
    return true;
}

bool moe_gate_up_routes_inline(const MoeGemvParams& p) {
    if (p.gate_dt != p.up_dt || p.n_used > 64) return false;
    if (p.gate_dt == INFR_Q4K) return fast_ok<Q4KFmt>(p.ne);
    if (p.gate_dt == INFR_Q6K) return fast_ok<Q6KFmt>(p.ne);
    if (p.gate_dt == INFR_Q8_0) return fast_ok<Q80Fmt>(p.ne);
    return false;
}

void launch_moe_gate_up(hipStream_t s, const MoeGemvParams& p) {
    if (p.gate_dt == p.up_dt) {
        bool done = false;
        if (p.gate_dt == INFR_Q4K) done = try_gate_up<Q4KFmt>(s, p);
        else if (p.gate_dt == INFR_Q6K) done = try_gate_up<Q6KFmt>(s, p);
        else if (p.gate_dt == INFR_Q8_0) done = try_gate_up<Q80Fmt>(s, p);
        if (done) return;
    }
    if (!p.sh_gate && moe_gate_up_units_supported(p)) {   // the other affine formats, and shapes the kernels above refuse
        launch_moe_gate_up_units(s, p);
        return;
    }
    dim3 grid((p.nff + 3) / 4, p.rows * p.n_used), block(256);
    INFR_LAUNCH(moe_gate_up_generic, grid, block, 0, s, p, row_bytes_of(p.gate_dt, p.ne),
                       row_bytes_of(p.up_dt, p.ne));
}

template <class F>
static bool try_down(hipStream_t s, const MoeGemvParams& p) {
    const int n_slots = p.n_used + (p.sh_down ? 1 : 0);
    if (!fast_ok<F>(p.nff) || n_slots > kMaxUsedFast) return false;
    const int rw = 64 / (p.nff / F::kBlockElems * F::kLPB);
    // output rows per block ~ rows * ne / n_cu
    const int want = ceil_div(p.ne, p.n_cu);
    if (p.rows >= 2) {
        // several token rows: tiles of whole stages of 2 row groups, about one block per compute
        // unit in total, streamed with the next stage in flight; one wave per slot
        const int gstep = 2 * rw;
        // tile height: whole stages; fewest rounds of blocks over the compute units, counting a
        // block's fixed cost (ids, h staging, combine) as about a dozen rows of streaming
        int ot = 0;
        long best = 0;
        for (int cand = 2 * gstep; cand <= kMaxOt; cand += gstep) {
            const long blocks = (long)p.rows * ceil_div(p.ne, cand);
            const long cost = ((blocks + p.n_cu - 1) / p.n_cu) * (cand + 12);
            if (ot == 0 || cost < best) { ot = cand; best = cost; }
        }
        if (ot >= 2 * gstep && n_slots * cells_bytes(p.nff) <= 64 * 1024) {
            dim3 grid(ceil_div(p.ne, ot), p.rows), block(1024);
            // the benchmark shapes' rows (768 or 1536 elements) with their block count as a constant
            constexpr int kNb0 = 768 / F::kBlockElems, kNb1 = 1536 / F::kBlockElems;
            const int nblk = p.nff / F::kBlockElems;
            if (nblk == kNb0) INFR_LAUNCH((moe_down_combine_stream<F, 1, 16, kNb0>), grid, block, n_slots * cells_bytes(p.nff), s, p, ot);
            else if (nblk == kNb1) INFR_LAUNCH((moe_down_combine_stream<F, 1, 16, kNb1>), grid, block, n_slots * cells_bytes(p.nff), s, p, ot);
            else INFR_LAUNCH((moe_down_combine_stream<F, 1, 16>), grid, block, n_slots * cells_bytes(p.nff), s, p, ot);
            return true;
        }
        if (ot >= 2 * gstep) {
            const int nwaves = n_slots < 8 ? n_slots : 8;
            dim3 grid(ceil_div(p.ne, ot), p.rows), block(64 * nwaves);
            const size_t lds = nwaves * cells_bytes(p.nff);
            INFR_LAUNCH((moe_down_combine_fast<F, 2, true>), grid, block, lds, s, p, ot);
            return true;
        }
    }
    int steps = 1;
    while (steps < 8 && steps * rw < want) steps <<= 1;
    while (steps > 1 && steps * rw > kMaxOt) steps >>= 1;
    const int ot = steps * rw;
    const size_t lds_s = n_slots * cells_bytes(p.nff);
    if (n_slots * steps >= 16 && lds_s <= 64 * 1024) {
        // two or more units per slot-wave: dealt evenly to sixteen waves and streamed
        dim3 grid(ceil_div(p.ne, ot), p.rows), block(1024);
        INFR_LAUNCH((moe_down_combine_stream<F, 1, 16>), grid, block, lds_s, s, p, ot);
        return true;
    }
    const int nwaves = n_slots < 8 ? n_slots : 8;
    dim3 grid(ceil_div(p.ne, ot), p.rows), block(64 * nwaves);
    const size_t lds = nwaves * cells_bytes(p.nff);
    switch (steps) {
        case 1: INFR_LAUNCH((moe_down_combine_fast<F, 1, false>), grid, block, lds, s, p, ot); break;
        case 2: INFR_LAUNCH((moe_down_combine_fast<F, 2, false>), grid, block, lds, s, p, ot); break;
        case 4: INFR_LAUNCH((moe_down_combine_fast<F, 4, false>), grid, block, lds, s, p, ot); break;
        default: INFR_LAUNCH((moe_down_combine_fast<F, 8, false>), grid, block, lds, s, p, ot); break;
    }
    return true;
}

bool moe_down_is_fast(const MoeGemvParams& p) {
    if (p.n_used + (p.sh_down ? 1 : 0) > kMaxUsedFast) return false;
    if (p.down_dt == INFR_Q4K) return fast_ok<Q4KFmt>(p.nff);
    if (p.down_dt == INFR_Q6K) return fast_ok<Q6KFmt>(p.nff);
    if (p.down_dt == INFR_Q8_0) return fast_ok<Q80Fmt>(p.nff);
    return false;
}

void launch_moe_down_combine(hipStream_t s, const MoeGemvParams& p) {
    bool done = false;
    if (p.down_dt == INFR_Q4K) done = try_down<Q4KFmt>(s, p);
    else if (p.down_dt == INFR_Q6K) done = try_down<Q6KFmt>(s, p);
    else if (p.down_dt == INFR_Q8_0) done = try_down<Q80Fmt>(s, p);
    if (done) return;
    dim3 grid((p.ne + 3) / 4, p.rows), block(256);
    INFR_LAUNCH(moe_down_combine_generic, grid, block, 0, s, p, row_bytes_of(p.down_dt, p.nff));
}

// ------------------------------------------------------------------------------- bucketed batches
// Decode batches of several token rows: grid.x = tiles of `ft` features (gate/up) or `ot` output
// rows (down), grid.y = expert, grid.z = chunk of T tokens of the expert's bucket.  A block stages
// the activations of its T tokens once (all waves share the cells), then every weight row of its
// tile is loaded once and dotted with each of them.  Same inner product as the per-token kernels,
// so the results are the same bits whichever path a batch takes.
template <class F, int T>
__device__ __forceinline__ void stage_tokens(const float* const (&rows)[T], int nt, int n, uint32_t* cells,
                                             size_t cell_words) {
    const int ncell = (n + 31) / 32;
    for (int idx = threadIdx.x; idx < T * ncell; idx += 256) {
        const int tau = idx / ncell, c0 = idx - tau * ncell;
        if (tau < nt) {
            const XLoad l = stage_x_load(rows[tau], n, c0);
            stage_x_convert<F::kGroup, F::kSigned>(l, n, c0, cells + (size_t)tau * cell_words);
        }
    }
    __syncthreads();
}

template <class F, int U, int T>
__global__ __launch_bounds__(256) void moe_gate_up_bucketed(MoeGemvParams p, int ft) {
    extern __shared__ __attribute__((aligned(16))) uint32_t dyn_lds[];
    __shared__ uint64_t s_tab[32];
    __shared__ float s_g[4][T][64], s_u[4][T][64];
    const int e = blockIdx.y;
    // without tables there is one bucket holding every row in order (a dense layer)
    const int t0 = (p.bk_offsets ? p.bk_offsets[e] : 0) + blockIdx.z * T, t1 = p.bk_offsets ? p.bk_offsets[e + 1] : p.rows;
    if (t0 >= t1) return;
    const int nt = min(T, t1 - t0);
    const int f0 = blockIdx.x * ft;
    const int fcount = min(ft, p.nff - f0);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;   // uniform: scalar registers
    const int nblk = p.ne / F::kBlockElems;
    const size_t row_bytes = (size_t)nblk * F::kBlockBytes;
    const Place<F> pl(nblk, lane);
    const size_t cell_words = (size_t)((p.ne + 31) / 32) * kCellDwords;
    if (threadIdx.x < 32) s_tab[threadIdx.x] = kExp2Table[threadIdx.x];
    int pair[T];
    const float* xrows[T];
#pragma unroll
    for (int tau = 0; tau < T; tau++) {
        pair[tau] = p.bk_pair_src ? p.bk_pair_src[t0 + min(tau, nt - 1)] : t0 + min(tau, nt - 1);
        xrows[tau] = p.x + (size_t)(pair[tau] / p.n_used) * p.ne;
    }
    const uint8_t* gbank = p.gate + (size_t)e * p.gate_stride + (size_t)f0 * row_bytes;
    const uint8_t* ubank = p.up + (size_t)e * p.up_stride + (size_t)f0 * row_bytes;
    const int per_round = 4 * pl.rw_count;   // features the block's four waves take per round
    const int n_rounds = (fcount + per_round - 1) / per_round;
    // A wave keeps U rounds (a gate row and an up row per row lane group) in flight as a ring: it finishes the oldest
    // round against its T tokens and requests the round U places ahead into the registers that became free, so loads
    // and dots alternate round by round.  The first rounds are requested before the activations are staged.
    typename F::Raw graw[U], uraw[U];
    auto issue = [&](int u, int k) {
        const int f = min((k * 4 + wave) * pl.rw_count + pl.rw, fcount - 1);
        graw[u] = load_row<F>(pl, gbank + (size_t)f * row_bytes);
        uraw[u] = load_row<F>(pl, ubank + (size_t)f * row_bytes);
    };
#pragma unroll
    for (int u = 0; u < U; u++)
        if (u < n_rounds) issue(u, u);
    stage_tokens<F, T>(xrows, nt, p.ne, dyn_lds, cell_words);
    typename F::X x[T];
#pragma unroll
    for (int tau = 0; tau < T; tau++) F::fetch_x(x[tau], dyn_lds + (size_t)min(tau, nt - 1) * cell_words, pl.blk, pl.sub);
    const int chunk = 64 / pl.rw_count;   // rounds whose results fit a wave's staging row; the ring restarts per chunk
    for (int c0 = 0; c0 < n_rounds; c0 += chunk) {
        const int cn = min(chunk, n_rounds - c0);
        auto finish = [&](int u, int j) {
#pragma unroll
            for (int tau = 0; tau < T; tau++) {
                if (tau >= nt) break;   // a short chunk of the bucket: no dots for tokens it does not have
                const float gs = row_sum<F>(F::dot(graw[u], pl.sub, x[tau]), pl, nblk);
                const float us = row_sum<F>(F::dot(uraw[u], pl.sub, x[tau]), pl, nblk);
                if (pl.writer()) {
                    s_g[wave][tau][j * pl.rw_count + pl.rw] = gs;
                    s_u[wave][tau][j * pl.rw_count + pl.rw] = us;
                }
            }
        };
        if (c0 > 0) {
#pragma unroll
            for (int u = 0; u < U; u++)
                if (u < cn) issue(u, c0 + u);
        }
        // steady state: no branch between a round's dots and its refill, so the waits count exactly the younger loads
        const int refills = cn - U;   // steps of this chunk that still have a round to request
        int j0 = 0;
        for (; j0 + U <= refills; j0 += U) {
#pragma unroll
            for (int u = 0; u < U; u++) {
                finish(u, j0 + u);
                issue(u, c0 + j0 + u + U);
            }
        }
        for (; j0 < cn; j0 += U) {
#pragma unroll
            for (int u = 0; u < U; u++) {
                if (j0 + u >= cn) break;
                finish(u, j0 + u);
                if (j0 + u < refills) issue(u, c0 + j0 + u + U);
            }
        }
        __builtin_amdgcn_wave_barrier();
        if (lane < cn * pl.rw_count) {
            const int j = lane / pl.rw_count, rw = lane - j * pl.rw_count;
            const int f = ((c0 + j) * 4 + wave) * pl.rw_count + rw;
            if (f < fcount) {
#pragma unroll
                for (int tau = 0; tau < T; tau++) {
                    if (tau >= nt) break;
                    float gs = s_g[wave][tau][lane], us = s_u[wave][tau][lane];
                    if (p.weight_before) {
                        const float wp = p.weights[pair[tau]];
                        gs = __fmul_rn(wp, gs);
                        us = __fmul_rn(wp, us);
                    }
                    p.h[(size_t)pair[tau] * p.nff + f0 + f] = gated_act_fn(p.act, p.has_clamp, p.clamp, gs, us, s_tab);
                }
            }
        }
        __builtin_amdgcn_wave_barrier();
    }
}

template <class F, int U, int T>
__global__ __launch_bounds__(256) void moe_down_bucketed(MoeGemvParams p, int ot) {
    extern __shared__ __attribute__((aligned(16))) uint32_t dyn_lds[];
    const int e = blockIdx.y;
    const int t0 = (p.bk_offsets ? p.bk_offsets[e] : 0) + blockIdx.z * T, t1 = p.bk_offsets ? p.bk_offsets[e + 1] : p.rows;
    if (t0 >= t1) return;
    const int nt = min(T, t1 - t0);
    const int o0 = blockIdx.x * ot;
    const int ocount = min(ot, p.ne - o0);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;   // uniform: scalar registers
    const int nblk = p.nff / F::kBlockElems;
    const size_t row_bytes = (size_t)nblk * F::kBlockBytes;
    const Place<F> pl(nblk, lane);
    const uint8_t* bank = p.down + (size_t)e * p.down_stride + (size_t)o0 * row_bytes;
    const int per_round = 4 * pl.rw_count;
    const size_t cell_words = (size_t)((p.nff + 31) / 32) * kCellDwords;
    const float ds = p.down_scale ? p.down_scale[e] : 1.0f;
    int pair[T];
    const float* xrows[T];
#pragma unroll
    for (int tau = 0; tau < T; tau++) {
        pair[tau] = p.bk_pair_src ? p.bk_pair_src[t0 + min(tau, nt - 1)] : t0 + min(tau, nt - 1);
        xrows[tau] = p.x + (size_t)pair[tau] * p.nff;   // h of the pair
    }
    typename F::Raw raw[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
        const int o = min((u * 4 + wave) * pl.rw_count + pl.rw, ocount - 1);
        raw[u] = load_row<F>(pl, bank + (size_t)o * row_bytes);
    }
    stage_tokens<F, T>(xrows, nt, p.nff, dyn_lds, cell_words);
    typename F::X x[T];
#pragma unroll
    for (int tau = 0; tau < T; tau++) F::fetch_x(x[tau], dyn_lds + (size_t)min(tau, nt - 1) * cell_words, pl.blk, pl.sub);
    for (int base = 0; base < ocount; base += per_round * U) {
        float y[U][T];
#pragma unroll
        for (int u = 0; u < U; u++)
#pragma unroll
            for (int tau = 0; tau < T; tau++) y[u][tau] = row_sum<F>(F::dot(raw[u], pl.sub, x[tau]), pl, nblk);
        const int base_next = base + per_round * U;
        typename F::Raw nxt[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int o = min(base_next + (u * 4 + wave) * pl.rw_count + pl.rw, ocount - 1);
            nxt[u] = load_row<F>(pl, bank + (size_t)o * row_bytes);
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int o = base + (u * 4 + wave) * pl.rw_count + pl.rw;
#pragma unroll
            for (int tau = 0; tau < T; tau++) {
                float v = y[u][tau];
                if (p.down_scale) v = __fmul_rn(v, ds);
                if (o < ocount && tau < nt && pl.writer()) {
                    const size_t oi = (size_t)pair[tau] * p.ne + o0 + o;
                    p.y[oi] = p.addend ? __fadd_rn(p.addend[oi], v) : v;
                }
            }
            raw[u] = nxt[u];
        }
    }
}

constexpr int kBucketT = 2;   // tokens a block of the bucketed kernels handles together

template <class F>
static void gate_up_bucketed(hipStream_t s, const MoeGemvParams& p) {
    const int rw = 64 / (p.ne / F::kBlockElems * F::kLPB);
    // about eight blocks per CU if every expert had one chunk of tokens (dense: the chunks of the one bucket): about
    // two thirds of the experts have one, and finer tiles fill the last round of blocks better (128 experts, 24 rows:
    // 101 us with four, 93 with eight, 92 with twelve)
    const int groups = p.bk_offsets ? max(p.n_expert, 1) : ceil_div(p.rows, kBucketT);
    int tiles = max(1, 8 * p.n_cu / groups);
    int ft = ceil_div(p.nff, tiles);
    ft = ceil_div(ft, 4 * rw * 2) * 4 * rw * 2;   // whole rounds of 4 waves x U = 2 row groups
    dim3 grid(ceil_div(p.nff, ft), p.n_expert, ceil_div(p.max_bucket ? p.max_bucket : p.rows, kBucketT)), block(256);
    INFR_LAUNCH((moe_gate_up_bucketed<F, 2, kBucketT>), grid, block, kBucketT * cells_bytes(p.ne), s, p, ft);
}

template <class F>
static void down_bucketed(hipStream_t s, const MoeGemvParams& p) {
    const int rw = 64 / (p.nff / F::kBlockElems * F::kLPB);
    const int groups = p.bk_offsets ? max(p.n_expert, 1) : ceil_div(p.rows, kBucketT);
    int tiles = max(1, 4 * p.n_cu / groups);
    int ot = ceil_div(p.ne, tiles);
    ot = ceil_div(ot, 4 * rw * 4) * 4 * rw * 4;   // whole rounds of 4 waves x U = 4 row groups
    dim3 grid(ceil_div(p.ne, ot), p.n_expert, ceil_div(p.max_bucket ? p.max_bucket : p.rows, kBucketT)), block(256);
    INFR_LAUNCH((moe_down_bucketed<F, 4, kBucketT>), grid, block, kBucketT * cells_bytes(p.nff), s, p, ot);
}

bool bucketed_rows_supported(int dt, int k) {
    if (kBucketT * cells_bytes(k) > 48 * 1024) return false;   // the staged cells must fit the default LDS window
    if (dt == INFR_Q4K) return fast_ok<Q4KFmt>(k);
    if (dt == INFR_Q6K) return fast_ok<Q6KFmt>(k);
    if (dt == INFR_Q8_0) return fast_ok<Q80Fmt>(k);
    return false;
}

bool moe_bucketed_supported(const MoeGemvParams& p) {
    if (p.gate_dt != p.up_dt || p.fused_gate_up) return false;
    return bucketed_rows_supported(p.gate_dt, p.ne) && bucketed_rows_supported(p.down_dt, p.nff);
}

void launch_moe_gate_up_bucketed(hipStream_t s, const MoeGemvParams& p) {
    if (p.gate_dt == INFR_Q4K) gate_up_bucketed<Q4KFmt>(s, p);
    else if (p.gate_dt == INFR_Q6K) gate_up_bucketed<Q6KFmt>(s, p);
    else gate_up_bucketed<Q80Fmt>(s, p);
}

void launch_moe_down_bucketed(hipStream_t s, const MoeGemvParams& p) {
    if (p.down_dt == INFR_Q4K) down_bucketed<Q4KFmt>(s, p);
    else if (p.down_dt == INFR_Q6K) down_bucketed<Q6KFmt>(s, p);
    else down_bucketed<Q80Fmt>(s, p);
}

// ------------------------------------------------------------------------------- Op::Linear
// dst[m, out_f] = x . W^T, the dense neighbour of the expert GEMVs (shared expert).
template <class F>
__global__ __launch_bounds__(256) void linear_fast(const float* __restrict__ xin, const uint8_t* __restrict__ w,
                                                   int in_f, int out_f, float* __restrict__ dst, int ot,
                                                   const float* __restrict__ addend) {
    extern __shared__ __attribute__((aligned(16))) uint32_t dyn_lds[];
    constexpr int U = 4;  // rows a wave keeps in flight
    const int r = blockIdx.y;
    const int o0 = blockIdx.x * ot;
    const int ocount = min(ot, out_f - o0);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;   // uniform: scalar registers
    const int nblk = in_f / F::kBlockElems;
    const size_t row_bytes = (size_t)nblk * F::kBlockBytes;
    const Place<F> pl(nblk, lane);
    const uint8_t* bank = w + (size_t)o0 * row_bytes;
    const int per_round = 4 * pl.rw_count;
    uint32_t* cells = dyn_lds + (size_t)wave * ((in_f + 31) / 32) * kCellDwords;
    const float* xrow = xin + (size_t)r * in_f;
    const XLoad xl = stage_x_load(xrow, in_f, lane);
    typename F::X x;
    bool have_x = false;
    for (int base = 0; base < ocount; base += per_round * U) {
        typename F::Raw raw[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int o = min(base + (u * 4 + wave) * pl.rw_count + pl.rw, ocount - 1);
            raw[u] = load_row<F>(pl, bank + (size_t)o * row_bytes);
        }
        if (!have_x) {
            stage_x_finish<F::kGroup, F::kSigned>(xl, xrow, in_f, cells, lane);
            __builtin_amdgcn_wave_barrier();
            F::fetch_x(x, cells, pl.blk, pl.sub);
            have_x = true;
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int o = base + (u * 4 + wave) * pl.rw_count + pl.rw;
            float y = row_sum<F>(F::dot(raw[u], pl.sub, x), pl, nblk);
            if (o < ocount && pl.writer()) {
                const size_t oi = (size_t)r * out_f + o0 + o;
                dst[oi] = addend ? __fadd_rn(addend[oi], y) : y;
            }
        }
    }
}

__global__ __launch_bounds__(256) void linear_generic(const float* __restrict__ x, const uint8_t* __restrict__ w,
                                                      int dt, size_t row_bytes, int in_f, int out_f,
                                                      float* __restrict__ dst, const float* __restrict__ addend) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;   // uniform: scalar registers
    const int o = blockIdx.x * 4 + wave;
    const int r = blockIdx.y;
    if (o >= out_f) return;
    const uint8_t* row = w + (size_t)o * row_bytes;
    const float* xr = x + (size_t)r * in_f;
    float y = 0.f;
    for (int k = lane; k < in_f; k += kWave) y = fmaf(decode_elem(dt, row, (uint32_t)k), xr[k], y);
    y = wave_sum(y);
    if (lane == 0) {
        const size_t oi = (size_t)r * out_f + o;
        dst[oi] = addend ? __fadd_rn(addend[oi], y) : y;
    }
}

template <class F>
static bool try_linear(hipStream_t s, const float* x, const uint8_t* w, int m, int in_f, int out_f, float* dst,
                       int n_cu, const float* addend) {
    if (!fast_ok<F>(in_f)) return false;
    const int rw = 64 / (in_f / F::kBlockElems * F::kLPB);
    int ot = ceil_div(out_f, n_cu);
    ot = ceil_div(ot, 4 * rw) * 4 * rw;  // whole rounds of the block's 4 waves
    dim3 grid(ceil_div(out_f, ot), m), block(256);
    INFR_LAUNCH((linear_fast<F>), grid, block, 4 * cells_bytes(in_f), s, x, w, in_f, out_f, dst, ot, addend);
    return true;
}

// Several rows: the rows are one bucket of the bucketed down kernel (two rows share each weight row).
static bool linear_rows(hipStream_t s, const float* x, const uint8_t* w, int dt, int m, int in_f, int out_f, float* dst,
                        int n_cu, const float* addend) {
    if (!bucketed_rows_supported(dt, in_f)) return false;
    MoeGemvParams q{};
    q.x = x;
    q.down = w;
    q.down_dt = dt;
    q.nff = in_f;
    q.ne = out_f;
    q.rows = m;
    q.n_expert = 1;
    q.n_used = 1;
    q.y = dst;
    q.addend = addend;
    q.n_cu = n_cu;
    launch_moe_down_bucketed(s, q);
    return true;
}

void launch_linear(hipStream_t s, const float* x, const uint8_t* w, int dt, size_t row_bytes, int m, int in_f,
                   int out_f, float* dst, int n_cu, const float* addend) {
    if (m >= 2 && linear_rows(s, x, w, dt, m, in_f, out_f, dst, n_cu, addend)) return;
    bool done = false;
    if (dt == INFR_Q4K) done = try_linear<Q4KFmt>(s, x, w, m, in_f, out_f, dst, n_cu, addend);
    else if (dt == INFR_Q6K) done = try_linear<Q6KFmt>(s, x, w, m, in_f, out_f, dst, n_cu, addend);
    else if (dt == INFR_Q8_0) done = try_linear<Q80Fmt>(s, x, w, m, in_f, out_f, dst, n_cu, addend);
    if (done) return;
    if (linear_float_supported(dt, in_f, row_bytes, x, w)) {
        launch_linear_float(s, x, w, dt, row_bytes, m, in_f, out_f, dst, addend);
        return;
    }
    if (linear_units_supported(dt, in_f, x)) {   // every other affine format, and the shapes the kernels above refuse
        launch_linear_units(s, x, w, dt, row_bytes, m, in_f, out_f, dst, addend);
        return;
    }
    dim3 grid((out_f + 3) / 4, m), block(256);
    INFR_LAUNCH(linear_generic, grid, block, 0, s, x, w, dt, row_bytes, in_f, out_f, dst, addend);
}

}  // namespace infr

// Host-callable launchers of the gfx950 kernels.  Every launcher validates nothing: the
// backend checks shapes, dtypes and buffer extents before it calls one.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include <hip/hip_ext.h>

#include <atomic>

namespace infr {

// Per-kernel timing.  While a thread has tl_launch_timing set, every launch it makes through
// INFR_LAUNCH attaches the two events to the kernel's own dispatch packet: `start` is stamped
// when the kernel begins executing and `stop` when its last wave retires, so their difference
// is the kernel's execution time without the dispatch gap around it.
struct LaunchTiming {
    hipEvent_t start, stop;
};
extern thread_local const LaunchTiming* tl_launch_timing;
#define INFR_LAUNCH(kernel, grid, block, lds, stream, ...)                                                       \
    do {                                                                                                         \
        const ::infr::LaunchTiming* lt_ = ::infr::tl_launch_timing;                                              \
        if (lt_) hipExtLaunchKernelGGL(kernel, grid, block, lds, stream, lt_->start, lt_->stop, 0, __VA_ARGS__); \
        else hipLaunchKernelGGL(kernel, grid, block, lds, stream, __VA_ARGS__);                                  \
    } while (0)

// Raises a kernel's limit of dynamic LDS once per device and kernel (`done`: one bit per device ordinal).  When the
// runtime refuses, the bit stays clear and the launch that follows fails with the runtime's own error, which the
// entry point that made the launch reports.
inline void lds_limit(const void* kernel, int bytes, std::atomic<uint32_t>& done) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 32) return;
    if (done.load(std::memory_order_relaxed) >> dev & 1u) return;
    if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) == hipSuccess)
        done.fetch_or(1u << dev, std::memory_order_relaxed);
}
#define INFR_LDS_LIMIT(kernel, bytes)                                       \
    do {                                                                    \
        static std::atomic<uint32_t> lds_limit_done_{0};                    \
        ::infr::lds_limit((const void*)kernel, (bytes), lds_limit_done_);   \
    } while (0)

// An Op::RmsNorm of the single token row folded into the logits kernel: x is the raw row, every
// block normalises it while staging and the first block also stores the normalised row to xn_out.
struct RouterNorm {
    const float* weight = nullptr;   // [ne]
    float eps = 0.0f;
    float* xn_out = nullptr;         // [ne], not x
};
bool router_logits_can_norm(int rdt, size_t row_bytes, int ne, int rows);
// False when launch_router_logits would refuse the shape (its staging does not fit the LDS): asked at compile time.
bool router_logits_fits(int rdt, size_t row_bytes, int ne, int rows);
// Router logits with the reference's dot order (8 FMA lanes, lanes summed 0..7).
// logits[rows, n_expert]; router rows are `row_bytes` apart, decoded as `rdt`.
// Returns false when the shape does not fit the kernel's LDS budget (or the fold of `norm`).
bool launch_router_logits(hipStream_t s, const uint8_t* router, int rdt, size_t row_bytes, const float* x,
                          int ne, int n_expert, int rows, float* logits, const RouterNorm* norm = nullptr);

struct RouteParams {
    const float* logits;      // [rows, n_expert]
    int n_expert, n_used, rows;
    int gating, norm_w;
    float scale;
    const float* exp_probs_b; // [n_expert] or null
    int n_groups, n_groups_used;
    const int32_t* expert_ids;  // [rows, n_used] or null (hash routing)
    // expert-parallel band (crates/infr-vulkan/shaders/moe_ep_band_remap.comp): ep_n > 0 keeps the
    // selections inside [ep_lo, ep_lo + ep_n) as id - ep_lo and turns the others into id 0, weight 0
    int ep_lo, ep_n;
    int32_t* ids;             // out [rows, n_used] rank order
    float* weights;           // out [rows, n_used]
    float* probs;             // out [rows, n_expert]
};
void launch_route(hipStream_t s, const RouteParams& p);

struct MoeGemvParams {
    const float* x;           // gate/up: [rows, ne]; down: h [rows, n_used, nff]
    const int32_t* ids;       // [rows, n_used]
    const float* weights;     // [rows, n_used]
    const uint8_t* gate; size_t gate_stride;   // per-expert byte stride
    const uint8_t* up;   size_t up_stride;
    const uint8_t* down; size_t down_stride;
    const float* down_scale;  // [n_expert] or null
    int gate_dt, up_dt, down_dt;
    int rows, ne, nff, n_used, n_expert;
    int act; int has_clamp; float clamp;
    int weight_before;
    int fused_gate_up;
    float* h;                 // [rows, n_used, nff]
    float* dst;               // [rows, ne]
    const float* addend;      // down: optional [rows, ne] added to the combined result (fused residual / MoE sum)
    // optional always-on expert handled as one more slot after the n_used routed ones (same dtypes,
    // same n_ff, routing weight 1): h then has n_used + 1 slots per row
    const uint8_t* sh_gate; const uint8_t* sh_up; const uint8_t* sh_down;
    // null: the always-on expert weighs 1 (Op::Add); else [rows] gate logits, its weight is sigmoid(logit)
    // (Op::MoeSharedExpertAdd)
    const float* sh_logit;
    // bucketed kernels: the most pairs one bucket can hold (0 = rows; rows * n_used when given expert ids
    // may repeat an expert inside a row)
    int max_bucket;
    // down: ranks whose routing weight is exactly 0 are left out of the combine (pairs an
    // expert-parallel band dropped: their h rows may never have been written)
    int skip_zero_w;
    int n_cu;
    // When set, the gate/up kernel routes each token row itself from route.logits (every block
    // redundantly; block 0 of a row publishes ids / weights / probs) and no route launch is needed.
    int route_inline;
    RouteParams route;
    // bucketed decode batches (launch_moe_*_bucketed): pairs grouped by expert
    const int32_t* bk_offsets;   // [n_expert + 1]
    const int32_t* bk_pair_src;  // [rows * n_used] flat (row * n_used + rank) in bucket order
    float* y;                    // [rows * n_used, ne] per-pair down outputs, flat pair order
};
// True when launch_moe_down_combine will take the bandwidth-bound kernel.
bool moe_down_is_fast(const MoeGemvParams& p);
// True when launch_moe_gate_up will take the kernel that can route inline.
bool moe_gate_up_routes_inline(const MoeGemvParams& p);
// h = act(gate.x) * (up.x) for every (row, slot).
void launch_moe_gate_up(hipStream_t s, const MoeGemvParams& p);
// dst[row] = sum over slots (rank order) of w * (down . h).
void launch_moe_down_combine(hipStream_t s, const MoeGemvParams& p);

// Single-token Op::MoeFfn in one launch: logits, routing, gate/up, down and the weighted sum, the stages handing over
// inside the kernel.  g: as for the two-launch path (g.route filled, rows == 1); the workspace (zeroed once) holds the
// hand-over records, the per-rank partial results and the launch sequence number; *fault (host-visible) is raised when
// a bounded wait runs out.  Two kernels take these parameters:
//   moe_layer_stream (k_layer_stream.hip): requests the expert rows of a GUESSED selection (from fast estimates of the
//     logits) while the exact logits and the exact routing are computed beside the stream; plain gatings only, an
//     always-on expert may ride along (g.sh_*);
//   moe_layer_fused (k_layer.hip): the stages in order; every routing option.
struct MoeLayerParams {
    MoeGemvParams g;
    const float* router;        // [n_expert, ne] f32
    size_t router_row_floats;
    const float* router_x;      // [ne]
    float* logits_out;          // [n_expert] or null: the logits, for the plan's routing capture
    uint32_t* seq;              // workspace + 0
    uint32_t* cnt;              // in-order kernel: workspace + 16, 32 slice counters then the finished-slice counter;
                                // streaming kernel: workspace + 0, the launch count of each of its 256 workgroups
    uint64_t* xl;               // [8][n_expert] logit records
    uint64_t* xh;               // [8][nff] activation records
    uint64_t* ypart;            // [8][ne] partial-result records
    uint32_t* fault;
    int spin_limit;
    // streaming kernel only
    uint64_t* xa;               // [8][n_expert] records of the logits' estimates
    uint64_t* xs;               // [nff] activation records of the always-on expert
    uint32_t* late;             // host-visible: experts a guess missed, summed over launches (or null)
    int logits_once;            // every logit computed by one workgroup for the whole grid, not once per group
    int guess_skew;             // tests: the guess leaves out this many of the largest estimates
    int epb, early_down;        // set by the launcher
    // an Op::RmsNorm of the single token row folded in (null norm_w: none): router_x is then ignored, the routing row is
    // rmsnorm(norm_x) * norm_w, stored to norm_out by one workgroup; norm_for_x: g.x is that row too (and is not read)
    const float* norm_x = nullptr;
    const float* norm_w = nullptr;
    float* norm_out = nullptr;
    float norm_eps = 0.0f;
    int norm_for_x = 0;
};
size_t moe_layer_workspace_bytes(int ne, int nff, int n_expert);
bool moe_layer_fused_supported(const MoeLayerParams& q);
bool launch_moe_layer_fused(hipStream_t s, const MoeLayerParams& q);
size_t moe_layer_stream_workspace_bytes(int ne, int nff, int n_expert, int rows);
bool moe_layer_stream_supported(const MoeLayerParams& q);
bool launch_moe_layer_stream(hipStream_t s, const MoeLayerParams& q);

// ---- batched path: bucketing + grouped GEMMs on the matrix cores --------------------------------
struct GroupedParams {
    const _Float16* a;        // gate/up: [rows, K] activations; down: [n_pairs, K]; f16, virtual k order
    const float* a_scale;     // one power-of-two scale per row of a
    const int32_t* offsets;   // [n_expert + 1] first pair of each expert's bucket
    const int32_t* pair_src;  // [n_pairs] flat (row * n_used + rank) of the pair at each bucket position
    const uint8_t* w0; size_t w0_stride;  // gate (or down) expert slices
    const uint8_t* w1; size_t w1_stride;  // up expert slices (gate/up only)
    const float* route_w;     // [rows, n_used] routing weights, read when weight_before
    const float* down_scale;  // [n_expert] or null (down only)
    float* out;               // [n_pairs, N] f32, bucket order (down with out_f16: f16 without the row scale)
    int out_f16;              // down only: store f16(acc * down_scale); the combine applies the row's a_scale
    int K, N, n_expert, n_used, n_pairs;
    int act, has_clamp; float clamp; int weight_before;
    int n_tiles_n;            // set by the launcher
    int loads_only;           // measurement: run the GEMM's loads, LDS reads and barriers without unpacking or matrix work
#ifdef INFR_GROUPED_TRACE
    long long* trace;         // measurement builds only: 32 slots per workgroup
#endif
};
// Formats and contraction lengths the grouped kernels take.
bool grouped_supported(int dt, int k);
// rows of f32 -> f16 with a per-row power-of-two scale, in the k order weights of `weight_dt` unpack to.
void launch_rows_to_f16(hipStream_t s, int weight_dt, const float* src, int rows, int n, void* dst, float* scale);
// route_kernel and the conversion of the same rows in one launch (rp.rows rows of n floats)
void launch_route_rows_to_f16(hipStream_t s, const RouteParams& rp, int weight_dt, const float* src, int n, void* dst, float* scale);
// offsets / pair_src / slot_pair ([n_pairs], -1 for ids outside [0, n_expert)) from ids [n_pairs].
// ids with the pairs of weight exactly 0 replaced by -1 (pairs an expert-parallel band dropped).
void launch_mask_dropped_pairs(hipStream_t s, const int32_t* ids, const float* weights, int n_pairs, int32_t* out);
void launch_bucket(hipStream_t s, const int32_t* ids, int n_pairs, int n_expert, int32_t* offsets, int32_t* pair_src,
                   int32_t* slot_pair);
// The same GEMMs for any affine format through the 32-element unit decoder; activations (p.a) in natural k order.
bool grouped_units_supported(int dt, int k);
void launch_grouped_units_gate_up(hipStream_t s, int dt, const GroupedParams& p);
void launch_grouped_units_down(hipStream_t s, int dt, const GroupedParams& p);
void launch_grouped_gate_up(hipStream_t s, int dt, const GroupedParams& p);
void launch_grouped_down(hipStream_t s, int dt, const GroupedParams& p);
// identity != 0: y is in flat (row, rank) order and slot_pair only flags invalid pairs (< 0); a null slot_pair
// means flat order with every pair valid.  skip_zero_w: pairs of weight 0 are left out (expert-parallel bands).
void launch_unbucket_combine(hipStream_t s, const void* y, const int32_t* slot_pair, const float* weights, int rows,
                             int ne, int n_used, int weight_before, float* dst, int identity = 0,
                             const float* pair_scale = nullptr,   // != null: y is f16, y[pair] * pair_scale[pair]
                             const float* addend = nullptr,       // != null: dst = addend + sum ([rows, ne], may be dst)
                             int skip_zero_w = 0);

// Decode batches with weight reuse: one block per (feature tile, expert) walks the expert's bucket,
// so an expert's rows are read from HBM once however many token rows selected it.  h and y are in
// flat (row, rank) order; launch_unbucket_combine with slot_pair_is_flags sums them.
bool moe_bucketed_supported(const MoeGemvParams& p);
// One side of it: rows of k elements in format dt.  Without bucket tables (bk_offsets == nullptr)
// the bucketed kernels treat all p.rows rows as one bucket in order: a dense layer.
bool bucketed_rows_supported(int dt, int k);
void launch_moe_gate_up_bucketed(hipStream_t s, const MoeGemvParams& p);
void launch_moe_down_bucketed(hipStream_t s, const MoeGemvParams& p);

// Standalone decode: out[i] = value of element i (exact reference arithmetic).
void launch_dequant(hipStream_t s, const uint8_t* src, int dtype, uint64_t numel, float* out);

// dst[m, out_f] = x[m, in_f] . W^T (W rows start at `w`, `row_bytes` apart).
// With `addend` ([m, out_f]) the result is addend + x . W^T (a following Op::Add folded in).
void launch_linear(hipStream_t s, const float* x, const uint8_t* w, int dt, size_t row_bytes, int m, int in_f,
                   int out_f, float* dst, int n_cu, const float* addend = nullptr);
void launch_gated_act(hipStream_t s, const float* gate, const float* up, float* dst, int rows, int nff, int act,
                      int up_off, int up_stride, int gate_stride, int gate_block_width, int has_clamp, float clamp);
// GEMV over 32-element units for any affine GGUF format (k_affine.hip); x must be 16-byte aligned.
bool linear_units_supported(int dt, int in_f, const void* x);
void launch_linear_units(hipStream_t s, const float* x, const uint8_t* w, int dt, size_t row_bytes, int m, int in_f,
                         int out_f, float* dst, const float* addend);
// Op::Linear on F32 / F16 / BF16 weights with 16-byte loads (k_affine.hip).
bool linear_float_supported(int dt, int in_f, size_t row_bytes, const void* x, const void* w);
void launch_linear_float(hipStream_t s, const float* x, const uint8_t* w, int dt, size_t row_bytes, int m, int in_f,
                         int out_f, float* dst, const float* addend);
// Op::MoeFfn's expert stages on the same units, one block column per (row, rank) pair: h[pair] from x (gate/up),
// y[pair] from h (down; needs p.y).  The weighted sum over ranks is launch_unbucket_combine's.
bool moe_gate_up_units_supported(const MoeGemvParams& p);
void launch_moe_gate_up_units(hipStream_t s, const MoeGemvParams& p);
bool moe_gate_up_units_routes_inline(const MoeGemvParams& p);
bool moe_down_units_supported(const MoeGemvParams& p);
void launch_moe_down_units(hipStream_t s, const MoeGemvParams& p);
bool moe_down_combine_units_supported(const MoeGemvParams& p);
void launch_moe_down_combine_units(hipStream_t s, const MoeGemvParams& p);
// Batches on the unit kernels: an expert's rows are fetched once per chunk of tokens of its bucket
// (p.bk_offsets / p.bk_pair_src from launch_bucket); h and y are written in bucket order.
bool moe_units_batch_supported(int gate_dt, int up_dt, int down_dt, int ne, int nff);
void launch_moe_gate_up_units_bucketed(hipStream_t s, const MoeGemvParams& p);
void launch_moe_down_units_bucketed(hipStream_t s, const MoeGemvParams& p);
void launch_add(hipStream_t s, const float* a, const float* b, float* dst, uint32_t n);
// Op::RmsNorm (add = 0) / Op::RmsNormAdd (add = 1); dst may be x.
void launch_rms_norm(hipStream_t s, const float* x, const float* weight, float* dst, int rows, int dim, float eps, int add);
// Op::Copy / Op::CopyStrided on elements of `elem_bytes` (2 or 4): row r copies n elements from
// src + r * src_stride to dst + r * dst_stride (pointers already at the ops' offsets).
void launch_copy_rows(hipStream_t s, const void* src, void* dst, uint32_t rows, uint32_t n, uint32_t src_stride,
                      uint32_t dst_stride, int elem_bytes);
void launch_moe_shared_expert_add(hipStream_t s, const float* moe, const float* shexp, const float* gate, float* dst,
                                  int rows, int n);
void launch_fill_zero(hipStream_t s, void* p, size_t bytes);
// One stage of a chain of dependent reads (measurement aid): `bytes` of `pool` from a window chosen by ctl[0].
void launch_probe_dependent_read(hipStream_t s, const uint8_t* pool, uint64_t pool_bytes, uint64_t bytes, uint32_t* ctl,
                                 uint32_t salt, int n_cu);

}  // namespace infr

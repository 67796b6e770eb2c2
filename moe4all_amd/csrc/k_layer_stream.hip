// Single-token Op::MoeFfn as ONE launch in which the expert weights are requested before the routing is known.
//
// What the reference fixes for this op is the routing (ids in rank order, routing weights, bit for bit:
// crates/infr-cpu/src/lib.rs:3684-3716 for the logits' summation order, :3746-3861 for gating, selection and
// renormalisation) and the rank order of the final sum (:4290-4302).  The expert stages need much less: the SET of
// selected experts.  This kernel therefore computes every router logit twice.  A fast estimate (each thread multiplies
// the eight elements it loaded, a tree adds them up) gives a guess of the selected set a few hundred nanoseconds
// after the operands have arrived, and the expert rows of the guessed set are requested at once.  The exact logits
// (eight 256- or 512-step chains of dependent multiply-adds per logit), the exact routing routine and the check of the
// guess run on one wavefront beside the stream of weights.  Only the exact results are published, decide the ranks and
// weigh the sum.  When the guess misses an expert of the exact set (logits that differ by less than the estimate's
// rounding), the workgroups that hold an expert outside the set compute the missing one late; a record's tag carries
// the expert it belongs to, so a consumer can never take the product of a wrong guess for the one it waits for.
//
// Work split.  256 workgroups of 8 wavefronts in 8 groups of 32 (group = blockIdx & 7; consecutive workgroups go to
// consecutive XCDs, so a group shares an L2).  Group g computes one expert of the set: workgroup m of the group the
// features [m * nff / 32, +nff / 32) of gate and up, then the output rows [m * ne / 32, +ne / 32) of down.  An
// always-on expert folded into the op is spread over all 256 workgroups (features [b * nff / 256, ..), rows
// [b * ne / 256, ..)); it needs no routing, so its rows are the first bytes requested.  Wavefront 0 is the router
// (exact chains, exact routing, check of the guess), wavefronts 1..7 stream weights: each keeps a ring of items
// (a gate row and an up row, or a group of down rows) in flight, finishes the oldest and requests the one D places
// ahead.  The first down rows are requested before the group's activations have been handed over.
//
// Hand-over between workgroups: 64-bit records {value bits, tag} written and polled with agent-scope relaxed atomics,
// no fence anywhere; the tag is the launch's sequence number (kept in device memory, advanced by the workgroup that
// leaves last) and, for the activations, the expert id.  Every wait is bounded: after `spin_limit` polls a workgroup
// raises the host-visible fault word and skips to the end; its peers run into their own limits, so the grid drains.
// Inside a workgroup the wavefronts hand over through LDS flags; a flag is always set, also on the failure path.
//
// The inner products, the activation, the routing routine and the order of the final sum are those of the
// three-launch kernels (k_gemv.hip): same bits.
#include "layer_stream.h"

namespace infr {

size_t moe_layer_stream_workspace_bytes(int ne, int nff, int n_expert, int rows) {
    // [launch count of each workgroup: 1 KB], then for each of the regions one part per token row:
    // [estimates 8 * n_expert][logits 8 * n_expert][h 8 * nff][h always-on nff][partials 8 * ne]
    return 1024 + (size_t)rows * ((size_t)2 * kGroups * n_expert + (size_t)kGroups * nff + (size_t)nff + (size_t)kGroups * ne) * 8;
}

namespace {

template <class FG, class FD>
bool stream_shape(const MoeLayerParams& q, StreamShape* out) {
    const MoeGemvParams& p = q.g;
    const int ne = p.ne, nff = p.nff, n_expert = p.route.n_expert;
    const bool shared = p.sh_gate != nullptr;
    if (ne != 2048 && ne != 4096) return false;                      // 256 or 512 octets on 512 threads
    if (ne % FG::kBlockElems || nff % FD::kBlockElems || nff % 256 || nff % 384 || nff > 1536) return false;   // six gathering wavefronts
    const int lpr_g = ne / FG::kBlockElems * FG::kLPB, lpr_d = nff / FD::kBlockElems * FD::kLPB;
    if (lpr_g > 64 || lpr_d > 64) return false;
    if (n_expert % 64 || n_expert > 256 || n_expert < 64) return false;
    const int rwc_g = 64 / lpr_g, rwc_d = 64 / lpr_d;
    const int rows = p.rows;
    if (rows != 1 && rows != 2 && rows != 4 && rows != 8) return false;   // whole XCDs per token row
    // eight rows (one XCD per row, four workgroups per group): faster than the per-token kernels for the K-quant shape
    // (48.4 against 51.4 us at 2048 / 768), slower for Q8_0 banks (86.3 against 79 us)
    if (rows == 8 && std::is_same<FG, Q80Fmt>::value) return false;
    const int mpg = kPerGroup / rows, bpr = kBlocks / rows;
    if (nff % mpg || ne % bpr) return false;
    const int fpb = nff / mpg, R = ne / mpg;
    const int n_gi = (fpb + rwc_g - 1) / rwc_g, n_di = (R + rwc_d - 1) / rwc_d;
    const int my_gi = (n_gi + kSW - 1) / kSW, my_di = (n_di - router_wave_down_items(n_di) + kSW - 1) / kSW;
    if (my_gi * rwc_g > 64) return false;                            // a wavefront's results wait in one 64-float row
    if (shared) {
        if (nff % bpr) return false;
    }
    // every logit once for the grid when a group's copy of the router would be a large share of the layer's bytes
    out->once = q.logits_once;
    if (ne / bpr > 64) return false;                                  // a workgroup's output rows: one per lane of the summing wavefront
    out->epb = out->once ? (n_expert + bpr - 1) / bpr : n_expert / mpg;
    const int H = kThreads / (ne / 8);
    out->ept = (out->epb + H - 1) / H;
    out->nsp = n_expert / 64;
    // everything in flight at once when a wavefront has few items, rings otherwise
    out->dg = my_gi <= 2 ? 2 : my_gi <= 4 && std::is_same<FG, Q80Fmt>::value ? 4 : 2;
    out->early_down = my_gi <= out->dg ? 1 : 0;
    // down rows requested behind the last gate/up rows ride out the hand-over of the activations: a deep ring
    out->dd = my_di <= 2 ? 2 : my_di <= 5 && std::is_same<FD, Q80Fmt>::value ? 5 : out->early_down ? 3 : 4;
    const int jstride = ne / 8 + 4;
    const size_t floats = (size_t)(out->epb + 1) * 8 * jstride + 2 * (size_t)n_expert +
                          ((route_scratch_floats(n_expert, p.route.n_groups) + 3) & ~(size_t)3) + 2 * (size_t)nff;
    out->lds = cells_bytes(ne) + floats * 4 + 2 * cells_bytes(nff);
    return out->lds <= 150 * 1024;
}

template <class FG, class FD>
bool dispatch_stream(hipStream_t s, MoeLayerParams q, bool launch) {
    StreamShape sh;
    if (!stream_shape<FG, FD>(q, &sh)) return false;
    q.epb = sh.epb;
    q.early_down = sh.early_down;
#define INFR_STREAM(DGv, DDv, EPTv, NSPv)                                                        \
    if (sh.dg == DGv && sh.dd == DDv && sh.ept == EPTv && sh.nsp == NSPv)                           \
        return launch ? launch_stream<FG, FD, DGv, DDv, EPTv, NSPv>(s, q, sh.lds) : true;
    {   // the benchmark shapes with their sizes as constants, ahead of the instantiations for any shape
        bool taken = false;
        const bool done = launch_stream_fixed(s, q, sh, launch, &taken);
        if (taken) return done;
    }
    if (q.norm_w) return false;   // the fold of the token row's RmsNorm exists for the fixed shapes only
    if constexpr (std::is_same<FG, Q4KFmt>::value) {
        INFR_STREAM(2, 2, 2, 2)   // ne 2048, nff 768, 128 experts, a copy of the router per group
        INFR_STREAM(2, 2, 1, 2)   // ... every logit once
        INFR_STREAM(2, 2, 1, 4)   // ... 256 experts
        INFR_STREAM(2, 4, 1, 2)   // ne 2048, nff 768, 128 experts, two or four token rows
        INFR_STREAM(2, 4, 1, 4)   // ne 4096, nff 1536, 256 experts, every logit once
    } else {
        INFR_STREAM(4, 5, 2, 2)   // Q8_0: ne 2048, nff 768, 128 experts
        INFR_STREAM(4, 5, 1, 2)
        INFR_STREAM(4, 5, 1, 4)
        INFR_STREAM(2, 4, 1, 2)   // two or four token rows
    }
#undef INFR_STREAM
    return false;
}

bool stream_any(hipStream_t s, const MoeLayerParams& q, bool launch) {
    const MoeGemvParams& p = q.g;
    const RouteParams& r = p.route;
    if (p.n_used != kGroups || p.n_cu < kBlocks || p.gate_dt != p.up_dt) return false;
    if ((p.sh_gate != nullptr) != (p.sh_down != nullptr) || (p.sh_gate != nullptr) != (p.sh_up != nullptr)) return false;
    // the guess ranks the experts by their logits: gatings that are monotone in the logit, no bias, no groups, no given
    // ids; options that need the routing weights before the gate/up stage or remap ids stay on the in-order kernels
    if ((r.gating != INFR_GATING_SOFTMAX && r.gating != INFR_GATING_SIGMOID) || r.exp_probs_b || r.expert_ids ||
        (r.n_groups > 1 && r.n_groups_used > 0) || r.ep_n > 0 || p.weight_before || p.skip_zero_w)
        return false;
    if (launch && ((((uintptr_t)q.router | (uintptr_t)q.router_x | (uintptr_t)p.x) & 15) != 0 || (q.router_row_floats & 3) != 0))
        return false;
    if (p.gate_dt == INFR_Q4K && p.down_dt == INFR_Q6K) return dispatch_stream<Q4KFmt, Q6KFmt>(s, q, launch);
    if (p.gate_dt == INFR_Q8_0 && p.down_dt == INFR_Q8_0) return dispatch_stream<Q80Fmt, Q80Fmt>(s, q, launch);
    return false;
}

}  // namespace

bool moe_layer_stream_supported(const MoeLayerParams& q) { return stream_any(nullptr, q, false); }
bool launch_moe_layer_stream(hipStream_t s, const MoeLayerParams& q) { return stream_any(s, q, true); }

}  // namespace infr

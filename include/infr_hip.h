/*
 * infr_hip.h — C ABI of the MI355X (gfx950) backend for the routed-expert MoE FFN path.
 *
 * The entry points mirror, one for one, the object-safe trait `infr_core::backend::Backend`
 * of the reference engine (crates/infr-core/src/backend.rs:630-1088) together with its
 * `Buffer` (:423-452), `Plan` (:468-482), `Bindings` (:522-620) and the slice of the graph IR
 * (`Graph`/`Op`, crates/infr-core/src/graph.rs) that the MoE FFN path uses.  A Rust crate
 * implementing `Backend` binds exactly these symbols through `extern "C"`.
 *
 * Conventions
 *   - every fallible call returns an infr_status; the message is read with
 *     infr_hip_last_error() (thread-local, UTF-8, valid until the next failing call on
 *     that thread).  No exception, abort or panic crosses this boundary
 *     (reference: `Result<T, infr_core::Error>`, crates/infr-core/src/error.rs:11-31).
 *   - handles are opaque; a handle from another backend instance is an INVALID error, never
 *     undefined behaviour (reference: `as_any().downcast_ref`, backend.rs:433-436).
 *   - all entry points are thread-safe (`Backend: Send + Sync`).
 *   - work is stream-ordered on one internal HIP stream: execute() enqueues and returns;
 *     download() and sync() wait.
 */
#ifndef INFR_HIP_H
#define INFR_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* infr_core::Error variants that can occur on this path (error.rs:11-31). */
typedef enum infr_status {
    INFR_OK = 0,
    INFR_ERR_BACKEND = 1,     /* Error::Backend: HIP failure, bad binding, size mismatch */
    INFR_ERR_UNSUPPORTED = 2, /* Error::Unsupported: op / dtype / option not implemented */
    INFR_ERR_ABORTED = 3,     /* Error::Aborted: shutdown latch set (reserved: this library has no latch and never returns it) */
    INFR_ERR_INVALID = 4,     /* null / foreign handle, malformed graph */
    INFR_ERR_LOADER = 5,      /* Error::Loader: malformed or inconsistent weight file */
    INFR_ERR_IO = 6           /* Error::Io: the file could not be opened or mapped */
} infr_status;

/* infr_core::DType, same ordinal order (crates/infr-core/src/tensor.rs:7-57). */
typedef enum infr_dtype {
    INFR_F32 = 0, INFR_F16 = 1, INFR_BF16 = 2, INFR_I32 = 3, INFR_U32 = 4,
    INFR_Q4_0 = 5, INFR_Q4_1 = 6, INFR_Q5_0 = 7, INFR_Q5_1 = 8, INFR_Q8_0 = 9,
    INFR_Q2K = 10, INFR_Q3K = 11, INFR_Q4K = 12, INFR_Q5K = 13, INFR_Q6K = 14,
    /* lattice-codebook i-quants (crates/infr-gguf/src/dequant.rs:565-916) */
    INFR_IQ1_S = 15, INFR_IQ1_M = 16, INFR_IQ2_XXS = 17, INFR_IQ2_XS = 18, INFR_IQ2_S = 19, INFR_IQ3_XXS = 20,
    INFR_IQ3_S = 21,
    /* small-table codebook, ternary and fp4 formats (dequant.rs:499-559, :926-1073) */
    INFR_IQ4_NL = 22, INFR_IQ4_XS = 23, INFR_TQ1_0 = 24, INFR_TQ2_0 = 25,
    INFR_Q2_0 = 27, INFR_MXFP4 = 28, INFR_NVFP4 = 29
    /* every format above is decoded on the device.  The remaining ordinals (I2S = 26, whose scale lives outside the
     * tensor bytes, and the turbo formats from 30 on) are accepted in declarations and rejected with
     * INFR_ERR_UNSUPPORTED by any op that would decode them */
} infr_dtype;

/* infr_core::backend::BufferUsage (backend.rs:384-406). */
typedef enum infr_buffer_usage {
    INFR_USAGE_WEIGHTS = 0, INFR_USAGE_ACTIVATIONS = 1, INFR_USAGE_KV_CACHE = 2,
    INFR_USAGE_STAGING = 3, INFR_USAGE_READBACK = 4, INFR_USAGE_HOST_WEIGHTS = 5
} infr_buffer_usage;

/* infr_core::graph::TensorKind (graph.rs:119-131). */
typedef enum infr_tensor_kind {
    INFR_KIND_INPUT = 0, INFR_KIND_WEIGHT = 1, INFR_KIND_INTERNAL = 2, INFR_KIND_OUTPUT = 3
} infr_tensor_kind;

/* infr_core::graph::Activation (graph.rs:47-54), MoeGating (graph.rs:73-85). */
typedef enum infr_activation { INFR_ACT_SILU = 0, INFR_ACT_GELU = 1, INFR_ACT_SIGMOID = 2 } infr_activation;
typedef enum infr_moe_gating {
    INFR_GATING_SOFTMAX = 0, INFR_GATING_SIGMOID = 1, INFR_GATING_SQRT_SOFTPLUS = 2
} infr_moe_gating;

#define INFR_NO_TENSOR 0xFFFFFFFFu /* Option<TensorId>::None */

/* TensorDecl { desc: TensorDesc { shape, dtype }, kind } (graph.rs:133-140, tensor.rs:258-261). */
typedef struct infr_tensor_decl {
    uint32_t rank;      /* 0..4 */
    uint64_t shape[4];
    int32_t dtype;      /* infr_dtype */
    int32_t kind;       /* infr_tensor_kind */
} infr_tensor_decl;

/* Op variants on the MoE FFN path.  Every other Op of the reference IR has no encoding here:
 * a front end that meets one reports Unsupported itself, as the reference's GPU adapter does
 * for combinations it cannot lower (crates/infr-vulkan/src/adapter.rs:8936-8985). */
typedef enum infr_op_kind {
    INFR_OP_MOE_FFN = 0,               /* Op::MoeFfn              graph.rs:1259-1352 */
    INFR_OP_LINEAR = 1,                /* Op::Linear              graph.rs:200-212   */
    INFR_OP_GATED_ACT = 2,             /* Op::GatedAct            graph.rs:935-975   */
    INFR_OP_ADD = 3,                   /* Op::Add                                   */
    INFR_OP_MOE_SHARED_EXPERT_ADD = 4, /* Op::MoeSharedExpertAdd  graph.rs:1449-1463 */
    INFR_OP_COPY = 5,                  /* Op::Copy                graph.rs:1230-1237 */
    INFR_OP_COPY_STRIDED = 6,          /* Op::CopyStrided         graph.rs:1238-1251 */
    INFR_OP_RMS_NORM = 7,              /* Op::RmsNorm             graph.rs:160-169   */
    INFR_OP_RMS_NORM_ADD = 8           /* Op::RmsNormAdd          graph.rs:170-179   */
} infr_op_kind;

/* Field-for-field Op::MoeFfn.  Option<TensorId> = INFR_NO_TENSOR; Option<f32> and
 * Option<(u32,u32)> carry a has_* flag. */
typedef struct infr_op_moe_ffn {
    uint32_t x, router_x, router, gate_exps, up_exps, down_exps;
    uint32_t down_scale;           /* optional */
    uint32_t fused_gate_up;        /* bool */
    uint32_t dst;
    uint32_t ne, n_expert, n_used, n_ff_exp;
    float scale;
    int32_t act;                   /* infr_activation */
    uint32_t has_swiglu_clamp; float swiglu_clamp;
    int32_t gating;                /* infr_moe_gating */
    uint32_t norm_w;               /* bool */
    uint32_t weight_before;        /* bool */
    /* Option<(base, n_local)> (graph.rs:1307-1319): routing stays global over n_expert, the expert
     * tensors (gate/up/down, down_scale) hold only the shard [ep_base, ep_base + ep_n_local);
     * selections of other experts become (id 0, weight 0) as in moe_ep_band_remap.comp, so dst is
     * this rank's partial sum. */
    uint32_t has_ep_band; uint32_t ep_base, ep_n_local;
    uint32_t exp_probs_b;          /* optional */
    uint32_t n_expert_groups, n_expert_groups_used;
    uint32_t expert_ids;           /* optional: I32 [rows, n_used], the selection in table order (hash routing,
                                    * crates/infr-cpu/src/lib.rs:3776-3793); an id outside [0, n_expert) is clamped into
                                    * the range before use (the reference indexes with it unchecked and would panic) */
} infr_op_moe_ffn;

typedef struct infr_op_linear {
    uint32_t x, weight, dst;
    uint32_t m, in_f, out_f, w_off;
} infr_op_linear;

typedef struct infr_op_gated_act {
    uint32_t gate, up, dst;
    uint32_t rows, nff;
    int32_t act;
    uint32_t up_off, up_stride, gate_stride, gate_block_width;
    uint32_t has_swiglu_clamp; float swiglu_clamp;
} infr_op_gated_act;

typedef struct infr_op_add { uint32_t a, b, dst, n; } infr_op_add;

typedef struct infr_op_moe_shared_expert_add {
    uint32_t moe, shexp, gate, dst;
    uint32_t rows, n;
} infr_op_moe_shared_expert_add;

/* Op::Copy is the rows = 1 case (strides unused).  Offsets, strides and n count elements of the
 * tensors' common dtype (F32, I32, U32, F16 or BF16).  src may equal dst: the source window is read
 * before anything is written, as the CPU backend does (crates/infr-cpu/src/lib.rs:3532-3583). */
typedef struct infr_op_copy {
    uint32_t src, src_off, src_stride;
    uint32_t dst, dst_off, dst_stride;
    uint32_t rows, n;
} infr_op_copy;

/* Op::RmsNorm: dst = rmsnorm(x) * weight over the last `dim` of each of `rows` rows;
 * Op::RmsNormAdd: dst += rmsnorm(x) * weight (crates/infr-cpu/src/lib.rs:1046-1093).  x, dst: F32
 * [rows, dim]; weight: F32 [dim].  dst may be x. */
typedef struct infr_op_rms_norm {
    uint32_t x, weight, dst;
    uint32_t rows, dim;
    float eps;
} infr_op_rms_norm;

typedef struct infr_op {
    int32_t kind; /* infr_op_kind */
    union {
        infr_op_moe_ffn moe_ffn;
        infr_op_linear linear;
        infr_op_gated_act gated_act;
        infr_op_add add;
        infr_op_moe_shared_expert_add moe_shared_expert_add;
        infr_op_copy copy;
        infr_op_rms_norm rms_norm;
    } u;
} infr_op;

/* Graph { tensors, ops } (graph.rs:2056-2123); the inputs/weights/outputs lists are implied by
 * each declaration's kind. */
typedef struct infr_graph {
    const infr_tensor_decl *tensors; uint32_t n_tensors;
    const infr_op *ops;              uint32_t n_ops;
} infr_graph;

typedef struct infr_hip_backend infr_hip_backend;
typedef struct infr_hip_buffer infr_hip_buffer;
typedef struct infr_hip_plan infr_hip_plan;

/* One Bindings::bind(id, buf) (backend.rs:582-590). */
typedef struct infr_binding { uint32_t tensor; const infr_hip_buffer *buffer; } infr_binding;

/* Subset of Capabilities (backend.rs:45-236) a caller of this path consults. */
typedef struct infr_hip_capabilities {
    char name[64];
    uint32_t f16, bf16, i8, i8_dot;
    uint32_t subgroup_min, subgroup_max;
    uint32_t integrated, compute_units;
    uint32_t buffer_device_address;
    uint32_t max_shared_memory_bytes;
    uint32_t unified_memory, decode_replay, combined_gu, graph_input_inplace;
    uint64_t device_memory_bytes;
} infr_hip_capabilities;

typedef struct infr_hip_config {
    /* Reserved for HIP-graph replay of a plan that is re-run with identical bindings.  This build
     * always launches its kernels directly on the backend's stream; the field is ignored. */
    uint32_t disable_graph_replay;
    /* Token rows from which Op::MoeFfn takes the bucketed grouped-GEMM path on the matrix cores
     * (f16 operands, f32 accumulation) instead of the f32-accurate GEMV paths; 0 selects the
     * built-in default (32). */
    uint32_t moe_batched_min_rows;
    /* Non-zero: every op of a graph gets its own launch(es); no neighbouring ops are folded into one
     * kernel.  The escape hatch the reference's backends keep for their rewrites
     * (crates/infr-core/src/fusion.rs:49-52, `enabled`); results are bit-identical either way. */
    uint32_t disable_op_fusion;
    /* Non-zero: a single-token Op::MoeFfn always runs as three launches (logits, routing + gate/up, down + sum).
     * By default shapes that fit (8 experts per token, Q4_K / Q6_K or Q8_0 banks, hidden size 2048 or 4096, a device
     * with 256 compute units) run as ONE launch whose stages hand over inside the kernel; results are bit-identical. */
    uint32_t disable_single_launch_moe;
    /* Polls a workgroup of the single-launch kernel spends on one of its hand-overs before it gives up (the error
     * then surfaces at the next infr_hip_sync / download and the backend falls back to three launches for good).
     * 0 selects the built-in default (32768, some tens of milliseconds); 1 gives up after the first poll. */
    uint32_t single_launch_spin_limit;
    /* Single-launch kernel, router logits: 0 = built-in choice per shape, 1 = every logit is computed by one
     * workgroup and handed to all (the router is read once), 2 = every group of 32 workgroups computes all logits
     * for itself (the router is read 8 times, the hand-over stays inside a group).  Same bits either way. */
    uint32_t single_launch_logits;
    /* Tests only.  The single-launch kernel requests expert rows for a guessed selection before the exact routing is
     * known; n > 0 makes every guess leave out the n most likely experts, so the path that loads a missed expert late
     * runs on every launch.  Results are unaffected. */
    uint32_t single_launch_guess_skew;
    /* Non-zero: keep the single-launch kernel whose stages run in order (no guess) for every shape it takes. */
    uint32_t disable_single_launch_guess;
} infr_hip_config;

/* Construction of the backend object (reference: VulkanBackend::new / CpuBackend::new,
 * crates/infr-cpu/src/lib.rs:868).  cfg may be NULL.  Fails with INFR_ERR_BACKEND when no
 * gfx950 device is visible: there is no CPU fallback.
 * infr_hip_destroy drains and closes the backend's stream; buffers and plans made by it may be freed
 * afterwards in any order (each keeps the backend object alive until it is freed, as the reference's buffers
 * keep their device alive), every other call on the destroyed handle or with such a buffer is refused. */
infr_status infr_hip_create(int device_ordinal, const infr_hip_config *cfg, infr_hip_backend **out);
void infr_hip_destroy(infr_hip_backend *be);

/* Backend::name (backend.rs:631), Backend::capabilities (:632). */
const char *infr_hip_name(const infr_hip_backend *be);
infr_status infr_hip_capabilities_get(const infr_hip_backend *be, infr_hip_capabilities *out);

/* Backend::alloc — zero-initialised, max(bytes,4) (backend.rs:651-656; CPU impl
 * crates/infr-cpu/src/lib.rs:930-932).  Backend::alloc_uninit (:657-666): contents unspecified. */
infr_status infr_hip_alloc(infr_hip_backend *be, size_t bytes, int32_t usage, infr_hip_buffer **out);
infr_status infr_hip_alloc_uninit(infr_hip_backend *be, size_t bytes, int32_t usage, infr_hip_buffer **out);
/* Buffer::len_bytes (backend.rs:424-433), Buffer::device_addr (:437-451), drop. */
size_t infr_hip_buffer_len(const infr_hip_buffer *buf);
uint64_t infr_hip_buffer_device_addr(const infr_hip_buffer *buf);
void infr_hip_buffer_free(infr_hip_buffer *buf);

/* Backend::upload / download (backend.rs:759-760): copy a prefix of n bytes. */
infr_status infr_hip_upload(infr_hip_backend *be, infr_hip_buffer *dst, const void *src, size_t n);
infr_status infr_hip_download(infr_hip_backend *be, const infr_hip_buffer *src, void *dst, size_t n);
/* Backend::upload_range / download_range (backend.rs:700-748). */
infr_status infr_hip_upload_range(infr_hip_backend *be, infr_hip_buffer *dst, size_t offset, const void *src, size_t n);
infr_status infr_hip_download_range(infr_hip_backend *be, const infr_hip_buffer *src, size_t offset, void *dst, size_t n);
/* Backend::copy_buffer (backend.rs:827-837): device-to-device prefix copy. */
infr_status infr_hip_copy_buffer(infr_hip_backend *be, const infr_hip_buffer *src, infr_hip_buffer *dst, size_t n);

/* Backend::compile (backend.rs:907): validates the graph, sizes internal scratch. */
infr_status infr_hip_compile(infr_hip_backend *be, const infr_graph *graph, infr_hip_plan **out);
void infr_hip_plan_free(infr_hip_plan *plan);
/* Backend::execute (backend.rs:908): binds Input/Weight/Output handles for this call only. */
infr_status infr_hip_execute(infr_hip_backend *be, infr_hip_plan *plan, const infr_binding *bindings, uint32_t n_bindings);
/* Backend::sync (backend.rs:1006). */
infr_status infr_hip_sync(infr_hip_backend *be);

/* Thread-local message of the last failing call on this thread ("" if none). */
const char *infr_hip_last_error(void);

/* Debug taps used by the parity tests: Op::MoeFfn's routing decision and bucketing of the
 * LAST executed MoeFfn op of `plan` (the reference exposes the same facts through
 * `debug.moe_counts`, crates/infr-cpu/src/lib.rs:3919-3980).  ids/weights are
 * [rows, n_used] in rank order; any pointer may be NULL. */
infr_status infr_hip_plan_moe_routing(infr_hip_backend *be, const infr_hip_plan *plan, uint32_t op_index,
                                      int32_t *ids, float *weights, float *logits, float *probs);

/* Bucketing of the last execution of MoeFfn op `op_index` when it took the batched path
 * (reference: crates/infr-cpu/src/lib.rs:3874-3908).  offsets[n_expert + 1]: first bucket
 * position of each expert (experts ascending); pair_src[rows * n_used]: flat index
 * row * n_used + rank of the pair at each bucket position (rows ascending inside a bucket);
 * slot_pair[rows * n_used]: bucket position of pair (row, rank), -1 for an expert id outside
 * [0, n_expert).  INFR_ERR_INVALID when the op ran the per-token path.  Any pointer may be NULL. */
infr_status infr_hip_plan_moe_bucketing(infr_hip_backend *be, const infr_hip_plan *plan, uint32_t op_index,
                                        int32_t *offsets, int32_t *pair_src, int32_t *slot_pair);

/* Standalone weight decode (reference: infr_gguf::dequant::dequant_block,
 * crates/infr-gguf/src/dequant.rs:11-55): dst f32 buffer receives the decoded prefix of
 * `numel` elements of `src` interpreted as `dtype`. */
infr_status infr_hip_dequant(infr_hip_backend *be, const infr_hip_buffer *src, int32_t dtype, uint64_t numel, infr_hip_buffer *dst);

/* One Op::MoeFfn WITHOUT ANY ALLOCATION.  This entry point has no counterpart in the reference; it is for callers
 * that cannot allocate device memory: code under HIP-graph capture, tight serving loops, harnesses that forbid it.
 * It is infr_hip_compile + infr_hip_execute of a graph holding one MoeFfn in the plain qwen3moe parameterisation
 * (softmax gating, renormalised weights, scale 1, SiLU, no option tensors, f32 router; 1 to 15 token rows), except
 * that the routing results and the rows between the two expert stages live in a static device array of
 * INFR_HIP_STATIC_SCRATCH_BYTES per GPU instead of a plan's arena; the output is the bits infr_hip_execute writes.
 * Shapes that need more scratch return INFR_ERR_UNSUPPORTED (needed bytes = 2 * rows * n_expert * 4 +
 * 2 * rows * n_used * 4 + rows * n_used * (n_ff_exp + ne) * 4, each term rounded up to 256).  Every call on a GPU
 * uses that GPU's one array: calls that overlap in time on one GPU (two backends, two threads) race; a call reads
 * only what it has written itself, so nothing needs clearing between calls.  Enqueues on the backend's stream like
 * infr_hip_execute; no profiling events are recorded for it. */
#define INFR_HIP_STATIC_SCRATCH_BYTES (1u << 20)
typedef struct infr_hip_moe_ffn_static_args {
    const infr_hip_buffer *x;          /* [rows, ne] f32 */
    const infr_hip_buffer *router;     /* [n_expert, ne] f32 */
    const infr_hip_buffer *gate_exps;  /* [n_expert, n_ff_exp, ne] */
    const infr_hip_buffer *up_exps;    /* [n_expert, n_ff_exp, ne] */
    const infr_hip_buffer *down_exps;  /* [n_expert, ne, n_ff_exp] */
    infr_hip_buffer *dst;              /* [rows, ne] f32 */
    int32_t gate_dtype, up_dtype, down_dtype;   /* infr_dtype of the three banks */
    uint32_t rows, ne, n_expert, n_used, n_ff_exp;
} infr_hip_moe_ffn_static_args;
infr_status infr_hip_moe_ffn_static(infr_hip_backend *be, const infr_hip_moe_ffn_static_args *a);

#ifdef __cplusplus
}
#endif
#endif /* INFR_HIP_H */

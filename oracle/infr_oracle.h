/*
 * CPU oracle for the routed-expert MoE FFN path (Op::MoeFfn and the shared-expert ops
 * around it).  TEST INFRASTRUCTURE ONLY: this library is the parity checker and the timed
 * CPU baseline.  Nothing in the shipped HIP backend links, loads or calls it.
 *
 * It restates, in plain C, the f32 "reference mode" of the reference engine's CPU backend
 * (crates/infr-cpu/src/lib.rs:366-396 `CpuBackend::reference`), i.e. every quantised weight
 * row is decoded to f32 and dotted in f32 with the 8-lane FMA order.  Each function cites
 * the reference lines it follows.
 *
 * Arithmetic contract: compiled with -ffp-contract=off.  rustc never contracts a*b+c
 * (reference Cargo.toml:117-122), so every `a*b+c` below is two roundings unless written
 * fmaf(), which mirrors Rust's `mul_add`.
 */
#ifndef INFR_ORACLE_H
#define INFR_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Same ordinal order as infr_core::DType (crates/infr-core/src/tensor.rs:7-57). */
enum orc_dtype {
    ORC_F32 = 0, ORC_F16 = 1, ORC_BF16 = 2, ORC_I32 = 3, ORC_U32 = 4,
    ORC_Q4_0 = 5, ORC_Q4_1 = 6, ORC_Q5_0 = 7, ORC_Q5_1 = 8, ORC_Q8_0 = 9,
    ORC_Q2K = 10, ORC_Q3K = 11, ORC_Q4K = 12, ORC_Q5K = 13, ORC_Q6K = 14,
    ORC_IQ1_S = 15, ORC_IQ1_M = 16, ORC_IQ2_XXS = 17, ORC_IQ2_XS = 18, ORC_IQ2_S = 19, ORC_IQ3_XXS = 20, ORC_IQ3_S = 21,
    ORC_IQ4_NL = 22, ORC_IQ4_XS = 23, ORC_TQ1_0 = 24, ORC_TQ2_0 = 25, ORC_Q2_0 = 27, ORC_MXFP4 = 28, ORC_NVFP4 = 29
};
/* infr_core::graph::Activation (graph.rs:47-54) and MoeGating (graph.rs:73-85). */
enum orc_activation { ORC_ACT_SILU = 0, ORC_ACT_GELU = 1, ORC_ACT_SIGMOID = 2 };
enum orc_gating { ORC_GATE_SOFTMAX = 0, ORC_GATE_SIGMOID = 1, ORC_GATE_SQRT_SOFTPLUS = 2 };

/* Block geometry (crates/infr-core/src/decode_spec.rs:320,327,331).  Returns 0, or -1 for a
 * dtype this oracle does not decode.  Float dtypes report 1 element per "block". */
int orc_block_geometry(int dtype, int *block_elems, int *block_bytes);
/* Entry e of lattice codebook `grid` (0 IQ2_XXS, 1 IQ2_XS, 2 IQ2_S, 3 IQ3_XXS, 4 IQ3_S, 5 IQ1_S) as signed bytes, in the
 * representation of crates/infr-core/src/iquant_grids.rs; returns the entry's length (8 or 4), -1 out of range. */
int orc_grid_entry(int grid, int e, int8_t *out);
/* KSIGNS_IQ2XS[i] of the same file, i in 0..127. */
uint8_t orc_ksigns(int i);
/* Bytes of `numel` elements of `dtype` (numel must be a whole number of blocks); -1 on error. */
int64_t orc_bytes_for(int dtype, int64_t numel);

float orc_f16_to_f32(uint16_t h);
/* get_scale_min_k4 (crates/infr-gguf/src/dequant.rs:77-87). */
void orc_k4(int j, const uint8_t *q, uint32_t *sc, uint32_t *m);

/* dequant_block / bytes_to_f32 (crates/infr-gguf/src/dequant.rs:11-55, 214-223, 315-335,
 * 365-389; crates/infr-cpu/src/lib.rs:513-527).  Decodes nbytes of `dtype` into out; returns
 * the number of f32 written or -1. */
int64_t orc_dequant(int dtype, const uint8_t *bytes, size_t nbytes, float *out);

/* dot (crates/infr-cpu/src/kernels.rs:6556-6583): 8 FMA lanes over i = j (mod 8), lanes summed
 * 0..7 left to right, scalar FMA tail. */
float orc_dot(const float *a, const float *b, size_t n);

/* act_fn / gated_act_fn (crates/infr-cpu/src/kernels.rs:6664-6683). */
float orc_act(int act, float g);
float orc_gated_act(int act, int has_clamp, float clamp, float gate, float up);

/* One row of routing (crates/infr-cpu/src/lib.rs:3741-3863): logits[n_expert] -> probs,
 * selected ids (rank order) and routing weights.  bias/hash_ids may be NULL.  Returns 0, or
 * -1 if a NaN makes the comparison undefined (the reference panics there) or an id is out of
 * range. */
int orc_route_row(const float *logits, int n_expert, int n_used, int gating, int norm_w,
                  float scale, const float *exp_probs_b, int n_groups, int n_groups_used,
                  const float *hash_ids_row, float *probs_out, int32_t *idx_out, float *w_out);

typedef struct orc_moe_ffn_args {
    /* activations: [rows, ne] f32 */
    const float *x;
    const float *router_x;
    int rows;
    /* weights as raw GGUF bytes */
    const uint8_t *router;  int router_dtype;  size_t router_bytes;
    const uint8_t *gate;    int gate_dtype;    size_t gate_bytes;
    const uint8_t *up;      int up_dtype;      size_t up_bytes;    /* unused when fused_gate_up */
    const uint8_t *down;    int down_dtype;    size_t down_bytes;
    const float *down_scale;   /* [n_expert] or NULL */
    int fused_gate_up;
    int ne, n_expert, n_used, n_ff_exp;
    float scale;
    int act;
    int has_swiglu_clamp; float swiglu_clamp;
    int gating, norm_w, weight_before;
    const float *exp_probs_b;  /* [n_expert] or NULL */
    int n_expert_groups, n_expert_groups_used;
    const float *expert_ids;   /* [rows, n_used] ids widened to f32, or NULL */
    int n_threads;             /* <=0: all hardware threads */
    /* outputs */
    float *dst;                /* [rows, ne] */
    /* optional captures (any may be NULL) */
    float *logits_out;         /* [rows, n_expert] */
    float *probs_out;          /* [rows, n_expert] */
    int32_t *idx_out;          /* [rows, n_used], rank order */
    float *w_out;              /* [rows, n_used] */
    /* bucketing (lib.rs:3874-3908) */
    int32_t *n_buckets_out;    /* [1] */
    int32_t *bucket_expert_out;/* [n_expert] (first n_buckets valid) */
    int32_t *bucket_p0_out;    /* [n_expert] */
    int32_t *bucket_count_out; /* [n_expert] */
    int32_t *pair_row_out;     /* [rows*n_used] */
    int32_t *slot_pair_out;    /* [rows, n_used] -> flat pair index */
    /* 0: reference (f32) numerics, the parity oracle.  1: the CPU backend's production numerics for a
     * batch (crates/infr-cpu/src/lib.rs:3679 `int8_ok = rows >= 2 && !reference`): banks in Q4_K / Q6_K /
     * Q8_0 whose row length is a multiple of 256 are dotted against int8 activations
     * (crates/infr-cpu/src/moe.rs:42-53).  Only the timed CPU baseline uses it: it misses the parity bar by
     * design (activation rounding of 1/127 per 256-element block). */
    int production;
} orc_moe_ffn_args;

/* Op::MoeFfn, reference (f32) numerics (crates/infr-cpu/src/lib.rs:3584-4304).
 * Returns 0 on success, negative on invalid arguments. */
int orc_moe_ffn(const orc_moe_ffn_args *a);

/* Op::Linear in reference mode (crates/infr-cpu/src/lib.rs:1275-1328):
 * dst[m,out_f] = x[m,in_f] . W^T with W rows [w_off/in_f, +out_f) of a tensor of w_numel elems. */
int orc_linear(const float *x, const uint8_t *w, int w_dtype, size_t w_bytes, int64_t w_numel,
               int m, int in_f, int out_f, int64_t w_off, int n_threads, float *dst);
/* Op::GatedAct, tightly packed rows (crates/infr-cpu/src/lib.rs:2973-3027 with strides 0). */
void orc_gated_act_rows(const float *gate, const float *up, int rows, int nff, int act,
                        int has_clamp, float clamp, float *dst);
/* Op::Add (crates/infr-cpu/src/lib.rs:3055-3070). */
void orc_add(const float *a, const float *b, int64_t n, float *dst);
/* Op::MoeSharedExpertAdd (crates/infr-cpu/src/lib.rs:3336-3356). */
void orc_moe_shared_expert_add(const float *moe, const float *shexp, const float *gate,
                               int rows, int n, float *dst);

/* Op::RmsNorm (add = 0) and Op::RmsNormAdd (add = 1: dst += ...), crates/infr-cpu/src/lib.rs:1046-1093. */
void orc_rms_norm(const float *x, const float *w, int rows, int dim, float eps, int add, float *dst);

/* quantize_q8 (crates/infr-cpu/src/quant.rs:27-63): per 256 elements d = amax / 127, q = round half away
 * from zero of x / d clamped to +-127, bsums = sums of q per 32 elements.  n a multiple of 256. */
void orc_quantize_q8(const float *x, int n, int8_t *qs, float *d, int32_t *bsums);
/* vec_dot_q4k / q6k / q8_0, scalar forms (crates/infr-cpu/src/kernels.rs:151-184, :487-526, :1170-1187):
 * one quantised weight row against one quantize_q8 activation row. */
float orc_vec_dot_q8(int dtype, const uint8_t *row, const int8_t *qs, const float *d, const int32_t *bsums, int in_f);

/* Number of hardware threads the pool would use. */
int orc_hw_threads(void);

#ifdef __cplusplus
}
#endif
#endif

/*
 * infr_hip_probe.h — measurement entry points of libinfr_hip.so.
 *
 * Nothing here belongs to the drop-in boundary (include/infr_hip.h holds that): a host that only drives the backend
 * never includes this file.  The benchmark uses these calls to time individual kernels and to measure what the
 * device allows for a kernel chain of a given shape.
 */
#ifndef INFR_HIP_PROBE_H
#define INFR_HIP_PROBE_H

#include "infr_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Per-kernel timing, the counterpart of the reference's per-op profiler seam
 * (crates/infr-core/src/prof.rs:54-120, enabled by `prof.ops`): while enabled every kernel
 * launch is bracketed by HIP events on the backend's stream.  Reading drains and resets. */
typedef struct infr_hip_prof_entry {
    char kernel[64];
    uint64_t launches;
    double total_ms;
    double min_ms, max_ms;
} infr_hip_prof_entry;
infr_status infr_hip_prof_enable(infr_hip_backend *be, int on);
infr_status infr_hip_prof_read(infr_hip_backend *be, infr_hip_prof_entry *out, uint32_t cap, uint32_t *n_out);
/* Measurement only (no counterpart in the reference).  on != 0: from now on the grouped GEMMs of the batched
 * Op::MoeFfn / Op::Linear paths (Q4_K / Q6_K / Q8_0 weights) run their loads, LDS reads and barriers but neither
 * unpack weights nor issue matrix instructions, so their launch time is what the kernels' data movement alone takes.
 * Everything such launches write is meaningless; switch it off again before using results. */
infr_status infr_hip_probe_grouped_loads_only(infr_hip_backend *be, int on);

/* Measurement aid, no counterpart in the reference: the time a chain of DEPENDENT kernels of given sizes cannot go below
 * on this device.  Stage k is one kernel that reads stage_bytes[k] bytes of `pool` (a window whose position depends on
 * a word the previous stage wrote; windows rotate through the pool, so make it larger than the caches) with every load
 * of a block in flight at once and no arithmetic.  us_per_stage[k]: stage k alone, launched back to back `iters`
 * times; us_per_chain: the stages in order, `iters` times.  Either pointer may be NULL.  Each stage needs 1 KB up to a
 * quarter of the pool.  Allocates a control word and two events for the duration of the call. */
infr_status infr_hip_probe_dependent_reads(infr_hip_backend *be, const infr_hip_buffer *pool, const uint64_t *stage_bytes,
                                           uint32_t n_stages, uint32_t iters, double *us_per_stage, double *us_per_chain);

/* Measurement / tests, no counterpart in the reference.  The single-launch Op::MoeFfn kernel requests expert rows for a
 * guessed selection and loads an expert late when the exact routing names one the guess missed; *out receives the
 * number of such late experts over all launches of this backend so far (waits for the backend's stream). */
infr_status infr_hip_probe_late_experts(infr_hip_backend *be, uint64_t *out);

/* Tests, no counterpart in the reference.  *out receives how many calls into the allocating part of the HIP runtime
 * (device memory, host memory, events) this library has made in this process so far, over all backends: a caller
 * that must not allocate reads it before and after the calls it wants to vouch for. */
infr_status infr_hip_probe_alloc_calls(uint64_t *out);

#ifdef __cplusplus
}
#endif
#endif /* INFR_HIP_PROBE_H */

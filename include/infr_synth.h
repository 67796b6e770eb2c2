/*
 * infr_synth.h — seeded synthetic workload for the MoE FFN benchmarks and parity tests.
 *
 * No counterpart in the reference's backend interface: the reference's tests build their
 * inputs with test-local helpers (crates/infr-testkit/src/lib.rs:49-123,
 * crates/infr-metal/tests/parity.rs:271-287) and its models read real GGUF files.  These
 * entry points produce N(0, sigma) tensors from a counter-based generator and quantise them
 * to Q8_0 / Q4_K / Q6_K / MXFP4, on the host or directly into a device buffer, with identical bytes.
 */
#ifndef INFR_SYNTH_H
#define INFR_SYNTH_H

#include "infr_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* out[i] = element (offset + i) of the N(0, sigma) stream `seed`, i < n.  Host only. */
int infr_synth_normal_host(uint64_t seed, uint64_t offset, uint64_t n, double sigma, float *out);
/* Quantise n f32 values (n a whole number of blocks) to `dtype` (Q8_0, Q4K, Q6K, MXFP4) on the host.
 * Returns the number of bytes written or -1. */
int64_t infr_synth_quantize_host(int32_t dtype, const float *src, uint64_t n, void *dst);
/* dst = dtype-quantised elements [offset, offset + numel) of the N(0, sigma) stream `seed`
 * (offset and numel multiples of 256).  dtype F32 writes the floats themselves. */
int64_t infr_synth_weights_host(int32_t dtype, uint64_t seed, uint64_t offset, uint64_t numel, double sigma,
                                void *dst, int n_threads);
/* Same bytes, produced on the device into buf at byte_offset. */
infr_status infr_synth_weights_device(infr_hip_backend *be, infr_hip_buffer *buf, size_t byte_offset, int32_t dtype,
                                      uint64_t seed, uint64_t offset, uint64_t numel, double sigma);

#ifdef __cplusplus
}
#endif
#endif

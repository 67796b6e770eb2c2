/*
 * infr_gguf.h — C ABI of the GGUF weight source that feeds the MI355X backend.
 *
 * Mirrors the reference's loader `infr_gguf::Gguf` (crates/infr-gguf/src/lib.rs:82-110, its
 * `WeightSource` impl :1000-1025) as far as the routed-expert FFN path needs it: open one file or
 * a whole `gguf-split` shard set, read metadata, enumerate tensors, and hand out each tensor's raw
 * block bytes straight from the file mapping.  Quantised blocks are never decoded on the host; the
 * backend receives them as they lie in the file (`BindWeight`, crates/infr-llama/src/seam/mod.rs:597-608).
 *
 * Every fallible call returns an infr_status; the message is read with infr_gguf_last_error()
 * (thread-local).  A malformed file is an error, never a crash: every length, count and offset read
 * from the file is bounds-checked before it is used, as the reference does (lib.rs:160-196).
 */
#ifndef INFR_GGUF_H
#define INFR_GGUF_H

#include "infr_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct infr_gguf infr_gguf;

/* TensorInfo (crates/infr-core/src/loader.rs): shape in the file's order, shape[0] varies fastest.
 * dtype is the infr_dtype ordinal (F32..Q6K = 0..14, then Iq1S 15, Iq1M 16, Iq2Xxs 17, Iq2Xs 18,
 * Iq2S 19, Iq3Xxs 20, Iq3S 21, Iq4Nl 22, Iq4Xs 23, Tq1_0 24, Tq2_0 25, I2S 26, Q2_0 27, Mxfp4 28,
 * Nvfp4 29, the order of crates/infr-core/src/tensor.rs:7-57).  offset counts from the first byte of
 * the first shard (lib.rs:923-936); name stays valid until infr_gguf_close. */
typedef struct infr_gguf_tensor {
    const char *name;
    int32_t dtype;
    uint32_t ggml_type;
    uint32_t rank;
    uint64_t shape[4];
    uint64_t numel;
    uint64_t offset;
    uint64_t nbytes;
} infr_gguf_tensor;

/* Gguf::open (lib.rs:484-493): `path` may name any shard of a set; the whole set is loaded. */
infr_status infr_gguf_open(const char *path, infr_gguf **out);
void infr_gguf_close(infr_gguf *g);
const char *infr_gguf_last_error(void);

/* WeightSource::tensors (lib.rs:1011-1013), in file order (shard after shard). */
uint64_t infr_gguf_tensor_count(const infr_gguf *g);
infr_status infr_gguf_tensor_at(const infr_gguf *g, uint64_t index, infr_gguf_tensor *out);
infr_status infr_gguf_tensor_find(const infr_gguf *g, const char *name, infr_gguf_tensor *out);
/* WeightSource::tensor_bytes (lib.rs:1019-1023): pointer into the mapping of the shard that holds
 * the tensor, valid until infr_gguf_close; the byte range is checked against that shard's size. */
infr_status infr_gguf_tensor_bytes(const infr_gguf *g, const char *name, const void **data, uint64_t *nbytes);

/* Number of files backing the model (Gguf::shards, lib.rs:938-943). */
uint32_t infr_gguf_shard_count(const infr_gguf *g);

/* Metadata (first shard's KV store, lib.rs:90-93).  Integer kinds widen to 64 bits, FLOAT32 to double
 * (read_meta_value, lib.rs:281-321).  INFR_ERR_INVALID when the key is absent or of another kind. */
infr_status infr_gguf_meta_u64(const infr_gguf *g, const char *key, uint64_t *out);
infr_status infr_gguf_meta_i64(const infr_gguf *g, const char *key, int64_t *out);
infr_status infr_gguf_meta_f64(const infr_gguf *g, const char *key, double *out);
infr_status infr_gguf_meta_bool(const infr_gguf *g, const char *key, int32_t *out);
/* Pointer to the string's bytes inside the mapping (not NUL-terminated) and its length. */
infr_status infr_gguf_meta_str(const infr_gguf *g, const char *key, const char **data, uint64_t *len);
/* Length of an ARRAY value. */
infr_status infr_gguf_meta_array_len(const infr_gguf *g, const char *key, uint64_t *out);

/* block_layout / nbytes (lib.rs:378-380, :436-438; decode_spec.rs:455-504): elements and bytes of one
 * block of `dtype`; INFR_ERR_UNSUPPORTED for I2S (no block layout: numel / 4 code bytes + one f32). */
infr_status infr_gguf_block_layout(int32_t dtype, uint32_t *block_elems, uint32_t *block_bytes);

/* The weight binder's step for a device backend (crates/infr-llama/src/seam/mod.rs:597-608,
 * :6412-6431): alloc_uninit(Weights) of the tensor's size and one upload of its raw bytes from the
 * mapping.  *dtype / *numel (either may be NULL) receive what the caller declares the graph tensor
 * with.  The buffer belongs to the caller (infr_hip_buffer_free). */
infr_status infr_gguf_bind_weight(const infr_gguf *g, const char *name, infr_hip_backend *be,
                                  infr_hip_buffer **out, int32_t *dtype, uint64_t *numel);

#ifdef __cplusplus
}
#endif
#endif /* INFR_GGUF_H */

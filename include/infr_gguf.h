/*
 * infr_gguf.h - C ABI of the GGUF model-file reader that feeds the HIP backend its weights.
 *
 * The reader is host code in the same shared library as the backend (libinfr_hip.so). It maps a
 * GGUF file (or a whole `gguf-split` shard set) read-only, parses header, metadata and tensor
 * directory with the reference reader's validation rules, and hands out pointers straight into
 * the mapping, so a weight goes file -> page cache -> HBM with no intermediate copy.
 *
 * What it replaces: `infr_gguf::Gguf` and its `WeightSource` impl
 * (crates/infr-gguf/src/lib.rs:79-156, 476-1008; crates/infr-core/src/loader.rs:7-92) and the
 * shard-name helpers of crates/infr-core/src/gguf_split.rs:12-90.
 *
 * Every function that can fail returns an infr_hip_status (infr_hip.h); the message of the last
 * failure on the calling thread is infr_gguf_last_error().
 */
#ifndef INFR_GGUF_H
#define INFR_GGUF_H

#include <stddef.h>
#include <stdint.h>

#include "infr_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct infr_gguf infr_gguf_t;             /* Gguf (lib.rs:79-97)            */
typedef struct infr_gguf_value infr_gguf_value_t; /* MetaValue (loader.rs:9-16)     */

/* MetaValue's variants. The thirteen GGUF value types collapse onto these exactly as the
 * reference's reader does (lib.rs:278-316): every unsigned width -> U64, every signed width ->
 * I64, FLOAT32/FLOAT64 -> F64. */
typedef enum {
    INFR_GGUF_BOOL = 0,
    INFR_GGUF_U64 = 1,
    INFR_GGUF_I64 = 2,
    INFR_GGUF_F64 = 3,
    INFR_GGUF_STR = 4,
    INFR_GGUF_ARR = 5
} infr_gguf_kind;

/* TensorInfo (crates/infr-core/src/loader.rs; filled at lib.rs:864-870). `ggml_type` is the id
 * stored in the file (the same numbering infr_dtype uses). `shape[0]` is the fastest-varying
 * axis: a Linear weight [out_f, in_f] has shape {in_f, out_f}. `offset` is the tensor's first
 * byte in the model's concatenated file address space (shards laid end to end, lib.rs:646-664);
 * for a single file it is a file offset. `name` stays valid until infr_gguf_close. */
typedef struct {
    const char *name;
    int ggml_type;
    int n_dims;
    uint64_t shape[4];
    uint64_t numel;
    uint64_t offset;
    size_t nbytes;
} infr_gguf_tensor_t;

/* Gguf::open (lib.rs:476-486). Opens `path`; when its metadata carries split.count > 1 the rest
 * of the `<base>-NNNNN-of-MMMMM.gguf` set is opened from the same directory and every claim the
 * set makes about itself is checked (lib.rs:496-626). Rejections (INFR_HIP_ERR_LOADER unless
 * noted): wrong magic, version other than 2 or 3, a length that runs past the file, invalid
 * UTF-8, unknown metadata value type, array nesting deeper than 64, general.alignment that is
 * zero / not a power of two / above 16 MiB, more than 4 dimensions, a shape or byte count that
 * overflows, a quantised element count that is not whole blocks, duplicate tensor names, any
 * shard-set inconsistency; an unknown ggml type is INFR_HIP_ERR_UNSUPPORTED (lib.rs:363); a file
 * that cannot be opened or mapped is INFR_HIP_ERR_IO. */
int infr_gguf_open(const char *path, infr_gguf_t **out);
void infr_gguf_close(infr_gguf_t *g);
const char *infr_gguf_last_error(void);

/* WeightSource::tensors (lib.rs:992-994): directory order, shard by shard. */
size_t infr_gguf_n_tensors(const infr_gguf_t *g);
int infr_gguf_tensor(const infr_gguf_t *g, size_t index, infr_gguf_tensor_t *out);
/* Index of the tensor called `name`, or -1. */
int64_t infr_gguf_find(const infr_gguf_t *g, const char *name);

/* WeightSource::tensor_bytes / Gguf::resolve (lib.rs:942-969, 1000-1003): pointer into the
 * mapping of the shard that holds the tensor, bounds-checked against that shard's size. */
int infr_gguf_tensor_bytes(const infr_gguf_t *g, const char *name, const void **data, size_t *len);
/* Gguf::tensor_file_range (lib.rs:915-918). */
int infr_gguf_tensor_file_range(const infr_gguf_t *g, const char *name, uint64_t *offset, size_t *len);
/* Gguf::shards (lib.rs:930-935): the files in shard order with the lengths the offsets assume. */
size_t infr_gguf_n_shards(const infr_gguf_t *g);
int infr_gguf_shard(const infr_gguf_t *g, size_t index, const char **path, uint64_t *len);

/* WeightSource::metadata (lib.rs:988-990): the FIRST shard's key/value store. Keys are listed in
 * file order; a key written twice keeps its last value (HashMap::insert, lib.rs:768). */
size_t infr_gguf_n_meta(const infr_gguf_t *g);
const char *infr_gguf_meta_key(const infr_gguf_t *g, size_t index);
/* Metadata::get (loader.rs:59-61): NULL when absent. */
const infr_gguf_value_t *infr_gguf_meta_get(const infr_gguf_t *g, const char *key);
int infr_gguf_value_kind(const infr_gguf_value_t *v);
/* MetaValue::as_u64 / as_f64 / as_str / as_arr (loader.rs:20-49): return 1 and fill the output
 * when the value converts, 0 otherwise. as_u64 takes U64 and non-negative I64; as_f64 takes F64,
 * U64 and I64; the others take their own variant only. */
int infr_gguf_value_u64(const infr_gguf_value_t *v, uint64_t *out);
int infr_gguf_value_i64(const infr_gguf_value_t *v, int64_t *out);
int infr_gguf_value_f64(const infr_gguf_value_t *v, double *out);
int infr_gguf_value_bool(const infr_gguf_value_t *v, int *out);
int infr_gguf_value_str(const infr_gguf_value_t *v, const char **s, size_t *len);
int infr_gguf_value_arr_len(const infr_gguf_value_t *v, size_t *len);
const infr_gguf_value_t *infr_gguf_value_arr_at(const infr_gguf_value_t *v, size_t index);
/* WeightSource::chat_template (lib.rs:1005-1007): tokenizer.chat_template or NULL. */
const char *infr_gguf_chat_template(const infr_gguf_t *g);

/* Block geometry of every ggml type the reader accepts (lib.rs:321-365;
 * crates/infr-core/src/decode_spec.rs:305-371); returns 0 for an unknown id. I2_S reports
 * (4, 1): four 2-bit codes per byte, plus one trailing f32 scale per TENSOR that
 * infr_gguf_nbytes adds (lib.rs:387-406). */
int infr_gguf_block_layout(int ggml_type, int *elems, int *bytes);
/* infr_gguf::nbytes (lib.rs:428-430): bytes of `numel` elements, rounded UP to whole blocks;
 * 0 with *ok = 0 on an unknown type or overflow. */
size_t infr_gguf_nbytes(int ggml_type, uint64_t numel, int *ok);

/* parse_shard (gguf_split.rs:44-68): split `<base>-NNNNN-of-MMMMM.gguf`. Returns 1 for a shard
 * name (fields equal width, all digits, at most five wide, suffix matched case-insensitively),
 * else 0. `base` receives at most base_cap-1 bytes plus a NUL; *base_len is the full length. */
int infr_gguf_parse_shard(const char *fname, char *base, size_t base_cap, size_t *base_len,
                          uint32_t *index, uint32_t *total, size_t *width);
/* shard_set (gguf_split.rs:72-88): the `i`-th (0-based) file name of the set `fname` belongs
 * to, written to `out`; returns the set's size (1, and `fname` itself, when it is no shard). */
size_t infr_gguf_shard_set(const char *fname, size_t i, char *out, size_t out_cap);

/* Weight upload: allocate a INFR_USAGE_WEIGHTS buffer of the tensor's byte size on `be` and copy
 * the tensor's bytes from the mapping into it. The reference's runner does the same through
 * Backend::alloc + Backend::upload on `tensor_bytes` (crates/infr-core/src/backend.rs:387-416).
 * The buffer holds the raw blocks, ready to be an Op::Linear / Op::MoeFfn weight. */
int infr_gguf_upload(const infr_gguf_t *g, const char *name, infr_hip_t *be, infr_hip_buffer_t **out);
/* Same, for several tensors back to back in ONE buffer (the reference's concatenated weights
 * addressed through Op::Linear's w_off, crates/infr-core/src/graph.rs:177-191). Every tensor
 * must have the same ggml type; `offsets[i]` receives tensor i's byte offset in the buffer. */
int infr_gguf_upload_concat(const infr_gguf_t *g, const char *const *names, size_t n, infr_hip_t *be,
                            infr_hip_buffer_t **out, size_t *offsets);

#ifdef __cplusplus
}
#endif
#endif /* INFR_GGUF_H */

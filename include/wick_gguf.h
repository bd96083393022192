/* wick_gguf.h -- read-only GGUF v3 container access for the ROCm backend.
 *
 * Host-side counterpart of the reference's GgufFile (wick/src/gguf.rs:128-745) as far
 * as the weight path needs it: parse header, metadata and tensor infos, validate every
 * tensor's byte range, hand out absolute offsets / raw bytes, and resolve a 2-D tensor
 * to the {rows m, row length k, ggml type} a GEMV / GEMM weight is uploaded with
 * (wick/src/model/lfm2.rs:310-338).  Nothing here touches the GPU.
 *
 * Conventions:
 *   - Every call returns 0 on success or a negative wick_gguf_status; the message of
 *     the last failure on the calling thread is wick_gguf_last_error().
 *   - Offsets are ABSOLUTE byte offsets into the file image (data section start +
 *     the tensor's stored offset), like TensorInfo::offset (wick/src/gguf.rs:547-575).
 *   - GGUF dims are [ne0, ne1, ...] with ne0 the contiguous one: a weight has
 *     k = ne0 (row length) and m = ne1 (rows) (wick/src/gguf.rs:678-693).
 *   - Strings are NOT NUL-terminated in the file; getters return pointer + length into
 *     memory owned by the handle (valid until wick_gguf_close).
 */
#ifndef WICK_GGUF_H
#define WICK_GGUF_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum wick_gguf_status {
    WICK_GGUF_OK = 0,
    WICK_GGUF_ERR_INVALID_ARG = -1, /* null pointer, index out of range */
    WICK_GGUF_ERR_IO = -2,          /* open / stat / mmap failed */
    WICK_GGUF_ERR_FORMAT = -3,      /* not GGUF v3, truncated, limits exceeded, tensor beyond file */
    WICK_GGUF_ERR_NOT_FOUND = -4,   /* no such key / tensor, or the value has another type */
    WICK_GGUF_ERR_UNSUPPORTED = -5  /* tensor of a ggml type without a known block size */
} wick_gguf_status;

/* Metadata value type ids of the container (wick/src/gguf.rs:20-33). */
enum {
    WICK_GGUF_T_U8 = 0, WICK_GGUF_T_I8 = 1, WICK_GGUF_T_U16 = 2, WICK_GGUF_T_I16 = 3, WICK_GGUF_T_U32 = 4,
    WICK_GGUF_T_I32 = 5, WICK_GGUF_T_F32 = 6, WICK_GGUF_T_BOOL = 7, WICK_GGUF_T_STRING = 8, WICK_GGUF_T_ARRAY = 9,
    WICK_GGUF_T_U64 = 10, WICK_GGUF_T_I64 = 11, WICK_GGUF_T_F64 = 12
};

typedef struct wick_gguf wick_gguf;

/* Message of the last failed call on this thread ("" if none). */
const char *wick_gguf_last_error(void);

/* GgufFile::open (wick/src/gguf.rs:331-341): maps the file read-only and parses it. */
int wick_gguf_open(const char *path, wick_gguf **out);
/* GgufFile::from_bytes (wick/src/gguf.rs:352-361).  The bytes are COPIED, the caller's
 * buffer is not referenced afterwards. */
int wick_gguf_from_bytes(const void *bytes, size_t nbytes, wick_gguf **out);
void wick_gguf_close(wick_gguf *g);

/* The whole file image (GgufFile::mmap_data, wick/src/gguf.rs:640-647) and where the tensor data
 * section starts in it (data_offset, wick/src/gguf.rs:649-653). */
const void *wick_gguf_data(const wick_gguf *g, size_t *nbytes);
size_t wick_gguf_data_offset(const wick_gguf *g);
uint32_t wick_gguf_alignment(const wick_gguf *g);

/* ---- metadata (typed getters match ONLY the exact stored type, wick/src/gguf.rs:553-637) ---- */
uint64_t wick_gguf_metadata_count(const wick_gguf *g);
int wick_gguf_metadata_key(const wick_gguf *g, uint64_t index, const char **key, size_t *len);
/* Stored type of a key; for arrays also the element type and count (else 0). */
int wick_gguf_value_type(const wick_gguf *g, const char *key, int *type, int *elem_type, uint64_t *count);
int wick_gguf_get_u32(const wick_gguf *g, const char *key, uint32_t *out);
int wick_gguf_get_f32(const wick_gguf *g, const char *key, float *out);
int wick_gguf_get_bool(const wick_gguf *g, const char *key, int *out);
int wick_gguf_get_str(const wick_gguf *g, const char *key, const char **s, size_t *len);
/* Any scalar integer / bool value widened to 64 bits (signed types sign-extend). */
int wick_gguf_get_int(const wick_gguf *g, const char *key, int64_t *out);
/* Array of fixed-size scalars: pointer to `count` little-endian elements inside the file image
 * (only as aligned as the file stores them: read them with memcpy).  elem_type must equal the stored one. */
int wick_gguf_get_array(const wick_gguf *g, const char *key, int elem_type, const void **data, uint64_t *count);
/* Element `index` of a string array. */
int wick_gguf_get_array_str(const wick_gguf *g, const char *key, uint64_t index, const char **s, size_t *len);

/* ---- tensors ------------------------------------------------------------------------ */
uint64_t wick_gguf_tensor_count(const wick_gguf *g);
int wick_gguf_tensor_name(const wick_gguf *g, uint64_t index, const char **name, size_t *len);
/* TensorInfo (wick/src/gguf.rs:72-83): size_bytes is 0 for a ggml type whose block size is unknown
 * (such a tensor is listed, but the data getters below refuse it).  dims has room for 8. */
int wick_gguf_tensor_info(const wick_gguf *g, const char *name, int *ggml_type, uint32_t *n_dims, uint64_t *dims,
                          uint64_t *abs_offset, uint64_t *size_bytes);
/* tensor_data (wick/src/gguf.rs:666-676): the raw bytes. */
int wick_gguf_tensor_data(const wick_gguf *g, const char *name, const void **data, size_t *nbytes);
/* tensor_meta (wick/src/gguf.rs:678-693) / resolve_weight (wick/src/model/lfm2.rs:310-338):
 * rank 1 -> rows 1, cols ne0; rank 2 -> rows ne1, cols ne0; other ranks are rejected. */
int wick_gguf_tensor_meta(const wick_gguf *g, const char *name, uint64_t *abs_offset, uint64_t *rows, uint64_t *cols,
                          int *ggml_type);

/* tensor_data_size (wick/src/gguf.rs:297-320): bytes of a tensor of `numel` elements;
 * fails when the type is unknown, numel is not a whole number of blocks, or the product overflows. */
int wick_gguf_tensor_data_size(int ggml_type, uint64_t numel, uint64_t *nbytes);
/* ggml_type_name (wick/src/gguf.rs:273-294): "Q4_0", ..., "???" for unknown ids. */
const char *wick_gguf_type_name(int ggml_type);

#ifdef __cplusplus
}
#endif
#endif /* WICK_GGUF_H */

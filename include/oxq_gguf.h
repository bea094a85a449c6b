/*
 * oxq_gguf.h -- GGUF container reader and tensor -> HBM loader of liboxq_hip.so.
 *
 * The on-disk side of the quantized-matmul path: what the reference does between opening a
 * model file and holding a QuantTensor (crates/oxillama-gguf/src/{header,parser,reader,
 * tensor_info,loader}.rs and load_quant_linear, crates/oxillama-arch/src/llama/model.rs:805-822),
 * with the tensor bytes going from the memory-mapped file through pinned staging buffers
 * straight into HBM instead of into a host Vec (`data.to_vec()`, model.rs:819).
 *
 * Parsing follows the reference's GgufFile::parse (parser.rs:34-60) field for field, including
 * its per-version widths: counts, string lengths, dimensions and array counts are u64 in
 * version 3 and u32 before; tensor offsets are u64 from version 2 and u32 in version 1.
 * Status codes 10..16 are the GgufError variants (crates/oxillama-gguf/src/error.rs:14-60);
 * oxq_last_error() gives (a, b) = the variant's payload.
 */
#ifndef OXQ_GGUF_H
#define OXQ_GGUF_H

#include "oxq.h"

#ifdef __cplusplus
extern "C" {
#endif

#define OXQ_ERR_GGUF_INVALID_MAGIC 10          /* GgufError::InvalidMagic{magic}: a = magic */
#define OXQ_ERR_GGUF_UNSUPPORTED_VERSION 11    /* GgufError::UnsupportedVersion{version}: a = version */
#define OXQ_ERR_GGUF_UNEXPECTED_EOF 12         /* GgufError::UnexpectedEof{offset}: a = offset */
#define OXQ_ERR_GGUF_INVALID_METADATA 13       /* GgufError::InvalidMetadata{key, reason}: message */
#define OXQ_ERR_GGUF_UNSUPPORTED_QUANT_TYPE 14 /* GgufError::UnsupportedQuantType{type_id}: a = type_id */
#define OXQ_ERR_GGUF_TENSOR_NOT_FOUND 15       /* GgufError::TensorNotFound{name}: message = name */
#define OXQ_ERR_GGUF_INVALID_STRING 16         /* GgufError::InvalidString{offset}: a = offset */
#define OXQ_ERR_GGUF_IO 17                     /* GgufError::MmapError: a = errno */

/* GgufValueType, crates/oxillama-gguf/src/types.rs:15-42 */
#define OXQ_GGUF_UINT8 0u
#define OXQ_GGUF_INT8 1u
#define OXQ_GGUF_UINT16 2u
#define OXQ_GGUF_INT16 3u
#define OXQ_GGUF_UINT32 4u
#define OXQ_GGUF_INT32 5u
#define OXQ_GGUF_FLOAT32 6u
#define OXQ_GGUF_BOOL 7u
#define OXQ_GGUF_STRING 8u
#define OXQ_GGUF_ARRAY 9u
#define OXQ_GGUF_UINT64 10u
#define OXQ_GGUF_INT64 11u
#define OXQ_GGUF_FLOAT64 12u

typedef struct oxq_gguf *oxq_gguf_t;

/* GgufModel::load_mmap (loader.rs:54-69): map the file read-only and parse it.  The mapping
 * lives until oxq_gguf_close. */
int oxq_gguf_open(const char *path, oxq_gguf_t *out);
/* GgufModel::from_bytes (loader.rs:103-110): parse a file image held in memory (copied). */
int oxq_gguf_open_bytes(const uint8_t *data, size_t len, oxq_gguf_t *out);
int oxq_gguf_close(oxq_gguf_t g);

/* GgufHeader (header.rs:9-18) and the derived layout (parser.rs:41-52). */
typedef struct oxq_gguf_summary {
    uint32_t version;
    uint64_t tensor_count;      /* as the header states it */
    uint64_t metadata_kv_count; /* as the header states it */
    uint64_t n_tensors;         /* distinct tensor names (TensorStore::len) */
    uint64_t n_metadata;        /* distinct keys (MetadataStore::len) */
    uint64_t alignment;         /* general.alignment, else 32 */
    uint64_t data_offset;       /* start of the tensor data section */
    uint64_t file_size;
} oxq_gguf_summary;
int oxq_gguf_get_summary(oxq_gguf_t g, oxq_gguf_summary *out);

/* TensorInfo (tensor_info.rs:22-50).  name points into the handle and lives as long as it. */
typedef struct oxq_gguf_tensor {
    const char *name;
    uint32_t n_dims;
    uint64_t dims[4];     /* dimensions as stored (the reference takes dims[0] as rows, dims[1] as columns);
                           * a tensor of more than four dimensions parses as in the reference and shows its
                           * first four here (n_dims, n_elements and data_size cover all of them) */
    uint32_t type;        /* GgufTensorType id */
    uint64_t offset;      /* relative to the data section */
    uint64_t n_elements;  /* product of the dimensions; 0 when there are none */
    uint64_t data_size;   /* ceil(n_elements / block_size) * block_bytes */
} oxq_gguf_tensor;
/* index: 0 .. n_tensors-1 in file order.  OXQ_ERR_GGUF_TENSOR_NOT_FOUND past the end / for an
 * unknown name (TensorStore::get, tensor_info.rs:83-89). */
int oxq_gguf_tensor_at(oxq_gguf_t g, uint64_t index, oxq_gguf_tensor *out);
int oxq_gguf_find_tensor(oxq_gguf_t g, const char *name, oxq_gguf_tensor *out);

/* GgufFile::tensor_data (parser.rs:66-80): the tensor's bytes inside the mapping (host memory).
 * OXQ_ERR_GGUF_UNEXPECTED_EOF{abs_offset} when they run past the end of the file. */
int oxq_gguf_tensor_data(oxq_gguf_t g, const char *name, const uint8_t **data, size_t *len);

/* MetadataStore::get (metadata.rs): a scalar or string value, or the summary of an array.
 * Unsigned values come back in u, signed in i, floats in f, bool in u; str points into the
 * handle (not NUL-terminated: str_len bytes). */
typedef struct oxq_gguf_value {
    uint32_t type;
    uint64_t u;
    int64_t i;
    double f;
    const char *str;
    size_t str_len;
    uint32_t elem_type; /* arrays */
    uint64_t count;     /* arrays */
    /* arrays: the encoded elements (fixed-width values back to back; strings as length + bytes, the
     * length u64 in version 3, u32 before) occupy array_bytes bytes at this offset of the
     * file image; oxq_gguf_meta_array_data hands out the pointer. */
    uint64_t array_offset;
    uint64_t array_bytes;
} oxq_gguf_value;
/* OXQ_ERR_GGUF_INVALID_METADATA when the key is missing (as MetadataStore::get_string does). */
int oxq_gguf_meta_find(oxq_gguf_t g, const char *key, oxq_gguf_value *out);
int oxq_gguf_meta_at(oxq_gguf_t g, uint64_t index, const char **key, oxq_gguf_value *out);
/* The encoded elements of an array value (tokenizer.ggml.tokens, scores, merges ...), valid until
 * oxq_gguf_close; INVALID_METADATA when the key is missing or not an array. */
int oxq_gguf_meta_array_data(oxq_gguf_t g, const char *key, const uint8_t **data, size_t *len);

/* load_quant_linear (llama/model.rs:805-822) with the QuantTensor in HBM: shape = the stored
 * dimensions (rows = dims[0], columns = dims[1]), bytes copied unchanged, mmap -> pinned staging ->
 * device in overlapping pieces.  The handle is an ordinary oxq_weights_t.  Errors:
 * TENSOR_NOT_FOUND; OXQ_ERR_UNSUPPORTED_TYPE when no kernel exists for the tensor's format;
 * OXQ_ERR_UNSUPPORTED_SHAPE unless the tensor is 2-D with columns a multiple of the block size
 * (rows must be whole blocks); UNEXPECTED_EOF when the data is truncated. */
int oxq_gguf_load_weights(oxq_gguf_t g, const char *name, oxq_weights_t *handle);
/* Raw bytes of any tensor (norm weights, biases, ...) into a caller's device buffer of at least
 * data_size bytes; synchronous. */
int oxq_gguf_upload_tensor(oxq_gguf_t g, const char *name, void *d_dst, size_t dst_len);

#ifdef __cplusplus
}
#endif
#endif /* OXQ_GGUF_H */

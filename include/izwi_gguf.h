/*
 * izwi_gguf — GGUF ingress for the quantized linear-layer library: container
 * parse, tensor lookup and upload of Q8_0 / Q4_K / Q6_K tensors straight into
 * izwi_qmm weight handles.
 *
 * It replaces, for this library's device, the reference's
 *   GgufLoader            crates/izwi-core/src/models/shared/weights/gguf.rs:36-203
 *   open_gguf_reader      crates/izwi-core/src/backends/model_io.rs:123-160
 * which delegate the container format to candle-core 0.10.2
 * (`quantized::gguf_file::Content::{read, tensor}`, not shipped with the
 * reference).  The format itself is the public GGUF specification, versions
 * 1-3: little-endian; header {magic "GGUF", version, tensor count, metadata
 * count}; metadata key/value pairs; tensor infos {name, n_dims, dims
 * (innermost first), ggml type id, offset}; tensor data from the next multiple
 * of `general.alignment` (default 32), offsets relative to that point.
 *
 * Conventions are those of izwi_qmm.h: every function returns IZWI_QMM_OK or a
 * negative izwi_qmm_status, the message is read with izwi_qmm_last_error().
 * Parsing, lookup and metadata need no GPU; only the load functions touch the
 * device.  The file is mapped read-only for the lifetime of the handle (the
 * reference's default on every backend, model_io.rs:70-83, 144-157); if the
 * mapping fails, or the mode is "off" (izwi_gguf_open_with_mode, IZWI_GGUF_MMAP),
 * the file is read with buffered I/O into memory instead, as the reference falls
 * back (model_io.rs:146-160).  In that buffered mode the WHOLE file stays on the host heap for the
 * life of the handle (the returned tensor pointers point into it): as many bytes of host memory as the
 * file has, beside the device copies of the tensors that are loaded - close the handle once the
 * weights are on the device.  The reference's BufReader streams instead; it has no such pointers to keep
 * valid.  Pointers returned by this API stay valid until izwi_gguf_close.  A handle is immutable and may be shared between threads.
 * No C++ exception leaves these functions: running out of memory on a crafted
 * file is IZWI_QMM_ERR_INVALID.
 */
#ifndef IZWI_GGUF_H
#define IZWI_GGUF_H

#include <stddef.h>
#include <stdint.h>

#include "izwi_qmm.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct izwi_gguf izwi_gguf; /* opaque: GgufLoader { path, content, metadata } */

/* GGUF metadata value types (gguf_file::ValueType) */
typedef enum izwi_gguf_value_type {
    IZWI_GGUF_U8 = 0,
    IZWI_GGUF_I8 = 1,
    IZWI_GGUF_U16 = 2,
    IZWI_GGUF_I16 = 3,
    IZWI_GGUF_U32 = 4,
    IZWI_GGUF_I32 = 5,
    IZWI_GGUF_F32 = 6,
    IZWI_GGUF_BOOL = 7,
    IZWI_GGUF_STRING = 8,
    IZWI_GGUF_ARRAY = 9,
    IZWI_GGUF_U64 = 10,
    IZWI_GGUF_I64 = 11,
    IZWI_GGUF_F64 = 12
} izwi_gguf_value_type;

#define IZWI_GGUF_MAX_DIMS 8

typedef struct izwi_gguf_tensor_info {
    int32_t ggml_dtype;               /* GGUF ggml type id: F32 0, F16 1, Q8_0 8, Q4_K 12, Q6_K 14, BF16 30 ... */
    int32_t n_dims;
    int64_t dims[IZWI_GGUF_MAX_DIMS]; /* row-major (outermost first), i.e. the file's order reversed, as
                                         gguf_file::TensorInfo::read does; a linear weight is [n, k] */
    uint64_t offset;                  /* from the start of the tensor data section */
    uint64_t nbytes;                  /* elements / block_size * type_size; 0 for types whose size this
                                         library does not know */
    const void* data;                 /* the tensor's bytes in the mapping (NULL if nbytes is 0) */
} izwi_gguf_tensor_info;

/* `is_gguf_file` (gguf.rs:366-377): 1 if the file starts with the bytes "GGUF", else 0 (also
 * for files that cannot be opened or are shorter than four bytes). */
int izwi_gguf_is_gguf_file(const char* path);

/* `GgufLoader::from_path` (gguf.rs:44-70): maps the file and parses header, metadata and tensor
 * infos.  Errors (bad magic, unknown version, truncated or inconsistent file) are
 * IZWI_QMM_ERR_INVALID; the reference maps them to Error::ModelLoadError. */
int izwi_gguf_open(const char* path, izwi_gguf** out);
void izwi_gguf_close(izwi_gguf* g);

/* `GgufMmapMode` and `open_gguf_reader_with_mode` (model_io.rs:13-45, 127-160).  The mode in force
 * is the configured one, else the environment variable IZWI_GGUF_MMAP ("auto", "on" | "true" | "1" |
 * "yes", "off" | "false" | "0" | "no", case and surrounding blanks ignored; anything else is
 * ignored), else auto (`resolve_gguf_mmap_mode`, model_io.rs:63-67); auto maps.  A mapping that
 * fails falls back to buffered I/O.  `mmap_mode` = -1 means "not configured"; izwi_gguf_open is
 * izwi_gguf_open_with_mode(path, -1, out).  `parse_mmap_mode` returns the mode or -1 for a word it
 * does not know (`GgufMmapMode::parse`); `reader_kind` is `GgufReader::kind`. */
typedef enum izwi_gguf_mmap_mode { IZWI_GGUF_MMAP_AUTO = 0, IZWI_GGUF_MMAP_ON = 1, IZWI_GGUF_MMAP_OFF = 2 } izwi_gguf_mmap_mode;
typedef enum izwi_gguf_reader_kind { IZWI_GGUF_READER_BUFFERED = 0, IZWI_GGUF_READER_MAPPED = 1 } izwi_gguf_reader_kind_t;
int izwi_gguf_open_with_mode(const char* path, int mmap_mode, izwi_gguf** out);
int izwi_gguf_parse_mmap_mode(const char* raw);
int izwi_gguf_resolve_mmap_mode(int configured);
int izwi_gguf_reader_kind(const izwi_gguf* g);

/* Header fields: format version (1-3), `general.alignment` in force, offset of the tensor data
 * section in the file. */
int izwi_gguf_header(const izwi_gguf* g, uint32_t* version, uint32_t* alignment, uint64_t* data_offset);

/* `tensor_count` / `tensor_names` (gguf.rs:147-154); names in file order. */
int64_t izwi_gguf_tensor_count(const izwi_gguf* g);
int izwi_gguf_tensor_name(const izwi_gguf* g, int64_t index, const char** name);

/* `has_tensor` / `tensor_shape` (gguf.rs:100-110): IZWI_QMM_ERR_INVALID with "tensor not found"
 * if the file has no such tensor. */
int izwi_gguf_tensor_info_get(const izwi_gguf* g, const char* name, izwi_gguf_tensor_info* out);

/* Metadata (gguf.rs:157-181).  `metadata_type` returns the value type or -1 if the key is absent.
 * `metadata_string` succeeds only for STRING values (`get_metadata_string`); `metadata_u64` for
 * U64, I64 (cast) and U32 values (`get_metadata_u64`); `metadata_f64` for every scalar numeric or
 * BOOL value.  `metadata_array` gives the element type, the count and, for fixed-size element
 * types, a pointer to the packed little-endian elements (NULL for arrays of strings or arrays);
 * `metadata_array_string` reads element i of an array of strings. */
int64_t izwi_gguf_metadata_count(const izwi_gguf* g);
int izwi_gguf_metadata_key(const izwi_gguf* g, int64_t index, const char** key);
int izwi_gguf_metadata_type(const izwi_gguf* g, const char* key);
int izwi_gguf_metadata_string(const izwi_gguf* g, const char* key, const char** str, uint64_t* len);
int izwi_gguf_metadata_u64(const izwi_gguf* g, const char* key, uint64_t* value);
int izwi_gguf_metadata_f64(const izwi_gguf* g, const char* key, double* value);
int izwi_gguf_metadata_array(const izwi_gguf* g, const char* key, int32_t* elem_type, uint64_t* count,
                             const void** data);
int izwi_gguf_metadata_array_string(const izwi_gguf* g, const char* key, uint64_t index, const char** str,
                                    uint64_t* len);

/* `load_qtensor` (gguf.rs:117-124) followed by `QMatMul::from_arc` (core.rs:710-715): the
 * tensor's block bytes go from the mapping into a weight handle on the current HIP device.  The
 * tensor must have two dimensions [n, k] and type Q8_0, Q4_K or Q6_K; other quantized types are
 * IZWI_QMM_ERR_UNSUPPORTED. */
int izwi_gguf_load_weight(const izwi_gguf* g, const char* name, izwi_qmm_weight** out);

/* `packed_quantized_qmatmul` (core.rs:834-845): the named tensors, all [n_i, k] of one type,
 * concatenated along rows into one handle (q|k|v, gate|up). */
int izwi_gguf_load_packed(const izwi_gguf* g, const char* const* names, int32_t n_names,
                          izwi_qmm_weight** out);

/* `load_tensor(name, DType::F32, device)` (gguf.rs:127-144): the tensor as dense f32 in row-major
 * order, `count` = number of elements `out` holds (must equal the tensor's element count).  F32 is
 * copied, F16 / BF16 converted, Q8_0 / Q4_K / Q6_K dequantized bit-exactly as candle-core's
 * `to_float`; conversion runs on the device (`mem_space` says where `out` lives). */
int izwi_gguf_load_tensor_f32(const izwi_gguf* g, const char* name, float* out, uint64_t count,
                              int mem_space, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* IZWI_GGUF_H */

/* C ABI over the GGUF reader of libvla.so.
 *
 * Mirrors what the reference's model loaders call on `struct gguf_reader`
 * (src/gguf_reader.h:33-216: open, has, u32 / f32 / f64 / str, meta, read_raw, read_f32,
 * read_convert, fetch_rows_f32) for hosts that bind the library through FFI; the C++ class
 * itself (vla.cpp_amd/host/gguf_reader.h) keeps the reference's member names.  All functions
 * run on the host, touch no GPU state, and report failure through their return value (a
 * message goes to stderr, as in the reference); none aborts on a malformed file.
 * One handle is not safe for concurrent calls (it owns one FILE position).
 */
#ifndef VLA_GGUF_H
#define VLA_GGUF_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define VLA_GGUF_API __attribute__((visibility("default")))

typedef struct vla_gguf vla_gguf;

enum { VLA_GGUF_OK = 0, VLA_GGUF_ERR_ARG = -1, VLA_GGUF_ERR_MISSING = -2, VLA_GGUF_ERR_READ = -3 };

/* ggml tensor type numbers as stored in the file (the ones read_f32 / read_convert understand,
 * plus I8 for packed payloads). */
enum { VLA_GGUF_F32 = 0, VLA_GGUF_F16 = 1, VLA_GGUF_I8 = 24, VLA_GGUF_BF16 = 30 };

/* gguf_reader::open (src/gguf_reader.h:52-68).  NULL when the file is missing, is not GGUF
 * version 2 or 3, or any record reaches past the end of the file. */
VLA_GGUF_API vla_gguf* vla_gguf_open(const char* path);
VLA_GGUF_API void vla_gguf_close(vla_gguf* g); /* NULL is fine */
VLA_GGUF_API int32_t vla_gguf_version(const vla_gguf* g);
VLA_GGUF_API int64_t vla_gguf_data_offset(const vla_gguf* g); /* gguf_get_data_offset, src/gguf_reader.h:66 */

/* gguf_reader::has / typed getters (src/gguf_reader.h:70-104): a missing key or a key of
 * another type reads as 0 / 0.0 / -1 (string), never aborts.  vla_gguf_key_type returns the
 * stored value type number or -1. */
VLA_GGUF_API int32_t vla_gguf_has_key(const vla_gguf* g, const char* key);
VLA_GGUF_API int32_t vla_gguf_key_type(const vla_gguf* g, const char* key);
VLA_GGUF_API uint32_t vla_gguf_u32(const vla_gguf* g, const char* key);
VLA_GGUF_API float vla_gguf_f32(const vla_gguf* g, const char* key);
VLA_GGUF_API double vla_gguf_f64(const vla_gguf* g, const char* key);
/* Copies at most cap-1 bytes plus a NUL into buf (buf may be NULL); returns the string's
 * length or -1. */
VLA_GGUF_API int64_t vla_gguf_str(const vla_gguf* g, const char* key, char* buf, int64_t cap);
/* Element count of an array value (and its element type number), -1 if absent. */
VLA_GGUF_API int64_t vla_gguf_array_len(const vla_gguf* g, const char* key, int32_t* elem_type);

/* gguf_reader::meta (src/gguf_reader.h:105-107): ne[0] is the contiguous dimension, unused
 * dimensions are 1; offset is relative to the data section. */
VLA_GGUF_API int64_t vla_gguf_n_tensors(const vla_gguf* g);
VLA_GGUF_API const char* vla_gguf_tensor_name(const vla_gguf* g, int64_t i);
VLA_GGUF_API int32_t vla_gguf_tensor_info(const vla_gguf* g, const char* name, int32_t* type, int32_t* n_dims, int64_t ne[4],
                                          int64_t* offset, int64_t* nbytes);

/* gguf_reader::read_raw (src/gguf_reader.h:116-137): cap must equal the tensor's byte size. */
VLA_GGUF_API int32_t vla_gguf_read_raw(vla_gguf* g, const char* name, void* buf, int64_t cap);
/* gguf_reader::read_f32 (src/gguf_reader.h:139-149): F32 / BF16 (and F16) widened to fp32;
 * n must equal the element count. */
VLA_GGUF_API int32_t vla_gguf_read_f32(vla_gguf* g, const char* name, float* out, int64_t n);
/* gguf_reader::read_convert (src/gguf_reader.h:151-181): target F32 or BF16 converts (round to
 * nearest even; gemma_norm adds 1.0 first), any other target passes the stored bytes through
 * and refuses gemma_norm.  cap must equal the result's size. */
VLA_GGUF_API int32_t vla_gguf_read_convert(vla_gguf* g, const char* name, int32_t target_type, int32_t gemma_norm, void* out,
                                           int64_t cap);
/* gguf_reader::fetch_rows_f32 (src/gguf_reader.h:183-215): rows of a 2-D matrix with ne[0] = cols. */
VLA_GGUF_API int32_t vla_gguf_fetch_rows_f32(vla_gguf* g, const char* name, const int32_t* row_ids, int64_t n_rows, float* dst,
                                             int64_t cols);

/* Runs the checkpoint import that vla_model_load would run on a GGUF file (host only, no GPU
 * state, nothing kept) and writes the names of the GGUF tensors it read, one per line in
 * reading order, NUL-terminated: the importer's view of the reference's tensor names
 * (src/models/smolvla.cpp:648-755, src/models/pi0.cpp:427-437, src/models/pi05.cpp:459-485,
 * src/modules/dit_head.cpp:29-85, src/modules/action_expert.cpp:20-39, src/models/bitvla.cpp:640-700).
 * Returns the length, VLA_GGUF_ERR_READ when the file cannot be imported (the reason goes to
 * stderr), or a value below -16 when cap is too small. */
VLA_GGUF_API int64_t vla_gguf_import_trace(const char* path, char* out, int64_t cap);

#ifdef __cplusplus
}
#endif
#endif

/* Load-time side of the int8 path: which weights are quantized, and the checkpoint file that carries
 * them.  Host code only (no device work): the entry points below read and write files and host
 * buffers; the bytes of a Q8_0 tensor go to the device through mul_mat_q8_hip (wtype 0) or
 * q8_weight_pack_hip as they come out of the file.
 *
 * References (paths relative to the reference tree):
 *   weight selection       src/model/PPML.cpp:4426-4456 (ppml_int8_bigop_default_list,
 *                          ppml_int8_bigop_selected), 4461-4494 (shape rule of
 *                          quantize_big_weight_matrices)
 *   checkpoint file        src/model/GGUF.cpp:194-316 (save_gguf), 318-470 (load_gguf),
 *                          31-74 (fnv1a_layout_hash), include/ppml/GGUF.h
 * The reference writes every tensor as F32 and refuses quantized parameters (GGUF.cpp:203-213);
 * this library writes the same file for F32 tensors, byte for byte, and stores a Q8_0 parameter as
 * ggml type 8 (blocks of {fp16 d, int8 qs[32]}, 34 bytes per 32 elements, rows never split). */
#ifndef PPML_HIP_WEIGHTS_H
#define PPML_HIP_WEIGHTS_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PPML_GGUF_TYPE_F32 0u
#define PPML_GGUF_TYPE_Q8_0 8u

/* ---- weight selection ----------------------------------------------------------------------- */
/* ppml_int8_bigop_default_list (src/model/PPML.cpp:4431-4434): the comma-separated name fragments
 * that "1" / "on" / "all" stand for. */
const char *ppml_int8_bigop_default_list(void);
/* ppml_int8_bigop_selected (src/model/PPML.cpp:4436-4456): 1 if `name` contains one of the
 * comma-separated fragments of `env_list` (blanks and tabs around a fragment are dropped, empty
 * fragments never match); NULL, "", "0" and "off" select nothing. */
int ppml_int8_bigop_selected(const char *name, const char *env_list);
/* The shape rule of quantize_big_weight_matrices (src/model/PPML.cpp:4481-4488): a selected weight
 * is quantized only if it is 2-D and its innermost dimension dims[0] (K) and its element count are
 * multiples of 32.  Returns 1 if the tensor qualifies. */
int ppml_int8_bigop_shape_ok(uint32_t ndim, const uint64_t *dims);

/* ---- layout fingerprint --------------------------------------------------------------------- */
/* fnv1a_layout_hash (src/model/GGUF.cpp:52-74): FNV-1a over (name, 0xFF, ndim, dims..., 0xFE) of
 * every tensor in order; an empty or missing name counts as "tensor_<index>".  `dims` holds the
 * dimensions of all tensors one after the other (ndims[i] of them for tensor i); `names` may be
 * NULL. */
uint64_t ppml_gguf_layout_hash(size_t n, const char *const *names, const uint32_t *ndims,
                               const uint64_t *dims);

/* ---- writing -------------------------------------------------------------------------------- */
typedef struct ppml_gguf_tensor {
    const char *name;   /* NULL or "" -> "tensor_<index>" for parameters */
    uint32_t ndim;      /* 1..4 */
    uint64_t dims[4];   /* dims[0] innermost, as in the reference's tensors */
    uint32_t type;      /* PPML_GGUF_TYPE_F32 or PPML_GGUF_TYPE_Q8_0 */
    const void *data;   /* host memory: numel floats, or numel / 32 blocks of 34 bytes */
} ppml_gguf_tensor;

/* save_gguf (src/model/GGUF.cpp:194-316): header, float metadata, string metadata with
 * "layout_hash" (16 hex digits, over the first n_params tensors) first, tensor infos, data aligned
 * to 32 bytes.  The n_extra tensors after the parameters (optimizer state: 1-D F32, named by the
 * caller) do not enter the fingerprint.  Returns 0, or 1 with the reason in ppml_hip_last_error. */
int ppml_gguf_save(const char *path, const ppml_gguf_tensor *tensors, size_t n_params, size_t n_extra,
                   const char *const *float_keys, const float *float_values, size_t n_float,
                   const char *const *string_keys, const char *const *string_values, size_t n_string);

/* ---- reading -------------------------------------------------------------------------------- */
typedef struct ppml_gguf_file ppml_gguf_file;

/* Parses header, metadata and tensor infos as load_gguf does (src/model/GGUF.cpp:318-400): magic
 * and version 3 are required; numeric metadata of every width are kept as floats, strings as
 * strings, arrays are skipped as arrays of 4-byte elements.  NULL on failure. */
ppml_gguf_file *ppml_gguf_open(const char *path);
void ppml_gguf_close(ppml_gguf_file *f);
size_t ppml_gguf_tensor_count(const ppml_gguf_file *f);
/* Tensor i: its name (valid until close), dimensions, type, file offset and size in bytes.  Any of
 * the output pointers may be NULL.  Returns 0, or 1 if i is out of range. */
int ppml_gguf_tensor_info(const ppml_gguf_file *f, size_t i, const char **name, uint32_t *ndim,
                          uint64_t dims[4], uint32_t *type, uint64_t *offset, uint64_t *nbytes);
/* Index of the tensor called `name`, or -1. */
int64_t ppml_gguf_find_tensor(const ppml_gguf_file *f, const char *name);
/* Copies the bytes of tensor i to dst (capacity bytes, at least its size).  Returns 0 or 1. */
int ppml_gguf_read_tensor(ppml_gguf_file *f, size_t i, void *dst, size_t capacity);
/* Numeric metadata `key` as a float (integers converted, as load_gguf does); 0 if present, 1 if not. */
int ppml_gguf_meta_float(const ppml_gguf_file *f, const char *key, float *value);
/* String metadata `key` (valid until close), or NULL. */
const char *ppml_gguf_meta_string(const ppml_gguf_file *f, const char *key);
/* The checks of load_gguf against a model's parameter list (src/model/GGUF.cpp:340-343, 404-415,
 * 438-468): at least n tensors in the file, the first n with these dimension counts and
 * dimensions, and -- if the file carries "layout_hash" -- the fingerprint of (names, dims) equal to
 * it (of the file's own names when `names` is NULL).  Returns 0, or 1 with the reference's message
 * in ppml_hip_last_error. */
int ppml_gguf_check_layout(const ppml_gguf_file *f, size_t n, const char *const *names,
                           const uint32_t *ndims, const uint64_t *dims);

#ifdef __cplusplus
}
#endif
#endif /* PPML_HIP_WEIGHTS_H */

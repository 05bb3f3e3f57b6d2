/*
 * libxabe_hip, weight ingest: the GGUF v3 container and the upload of one layer's tensors to the device
 * in the formats the file stores them in.
 *
 * Replaces, for the feed-forward block's tensors, `xabe_gguf::{GgufFile, TensorInfo, GgmlType, GgufError}`
 * ("F" = crates/xabe-gguf/src/file.rs, "T" = crates/xabe-gguf/src/types.rs, "E" = crates/xabe-gguf/src/error.rs),
 * the tensor names of crates/xabe-model/src/weights.rs:170-211, `MoeLayerWeights::upload`
 * ("B" = crates/xabe-engine/src/block/moe.rs:660-756, :811-892) and `DenseFfnLayerWeights::upload`
 * ("D" = crates/xabe-engine/src/block/dense_ffn.rs:663-760).
 *
 * A file is untrusted input: every malformed case is a status, never a crash.  Statuses are the
 * `xabe_status` values of xabe_hip.h; `xabe_last_error()` gives the message.
 */
#ifndef XABE_GGUF_H
#define XABE_GGUF_H

#include <stddef.h>
#include <stdint.h>

#include "xabe_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* `enum ggml_type` ids of the types this library sizes (T:38-60); anything else fails the load. */
typedef enum xabe_ggml_type {
  XABE_GGML_F32 = 0,
  XABE_GGML_F16 = 1,
  XABE_GGML_Q4_0 = 2,
  XABE_GGML_Q8_0 = 8,
  XABE_GGML_Q4_K = 12,
  XABE_GGML_Q5_K = 13,
  XABE_GGML_Q6_K = 14,
  XABE_GGML_BF16 = 30
} xabe_ggml_type;

/* GgmlType::{block_size, type_size, name, bytes_for_elements} (T:62-119).  0 / NULL for an unknown id;
 * bytes_for_elements returns XABE_ERR_GGUF_UNALIGNED_ELEMENT_COUNT for a partial block. */
uint64_t xabe_ggml_type_block_size(int ggml_type);
uint64_t xabe_ggml_type_size(int ggml_type);
const char* xabe_ggml_type_name(int ggml_type);
int xabe_ggml_type_bytes_for_elements(int ggml_type, uint64_t n_elements, uint64_t* out_bytes);

/* `gguf_type` tags of metadata values (F:386-412). */
typedef enum xabe_gguf_value_type {
  XABE_GGUF_U8 = 0, XABE_GGUF_I8 = 1, XABE_GGUF_U16 = 2, XABE_GGUF_I16 = 3, XABE_GGUF_U32 = 4, XABE_GGUF_I32 = 5,
  XABE_GGUF_F32 = 6, XABE_GGUF_BOOL = 7, XABE_GGUF_STRING = 8, XABE_GGUF_ARRAY = 9, XABE_GGUF_U64 = 10,
  XABE_GGUF_I64 = 11, XABE_GGUF_F64 = 12
} xabe_gguf_value_type;

typedef struct xabe_gguf_file xabe_gguf_file;

/* GgufFile::open (F:93-97): memory-maps the file; tensor bytes are never copied on the host.
 * GgufFile::from_bytes (F:103-105): parses a copy of `bytes`. */
int xabe_gguf_open(const char* path, xabe_gguf_file** out);
int xabe_gguf_from_bytes(const void* bytes, size_t len, xabe_gguf_file** out);
void xabe_gguf_close(xabe_gguf_file* f);

uint32_t xabe_gguf_version(const xabe_gguf_file* f);      /* F:152-154, always 3 */
uint32_t xabe_gguf_alignment(const xabe_gguf_file* f);    /* F:157-159 */
size_t xabe_gguf_n_kv(const xabe_gguf_file* f);           /* F:162-164 */
size_t xabe_gguf_n_tensors(const xabe_gguf_file* f);      /* F:167-169 */
uint64_t xabe_gguf_data_offset(const xabe_gguf_file* f);  /* metadata end padded up to the alignment (F:366-367) */

/* One tensor directory entry (crates/xabe-gguf/src/tensor.rs:11-28).  `name` points into the handle. */
typedef struct xabe_gguf_tensor_info {
  const char* name;
  uint32_t n_dims;
  uint64_t dims[4];      /* ggml order: dims[0] is the innermost dimension */
  int ggml_type;
  uint64_t offset;       /* relative to the data section */
  uint64_t n_elements;
  uint64_t n_bytes;
} xabe_gguf_tensor_info;

/* GgufFile::tensors()[index] (F:172-174), ::tensor(name) (F:177-179): XABE_OK, or XABE_ERR_MISSING_TENSOR. */
int xabe_gguf_tensor_at(const xabe_gguf_file* f, size_t index, xabe_gguf_tensor_info* out);
int xabe_gguf_tensor(const xabe_gguf_file* f, const char* name, xabe_gguf_tensor_info* out);
/* GgufFile::tensor_bytes (F:186-191): the tensor's bytes inside the mapping, NULL when there is no such tensor. */
const void* xabe_gguf_tensor_bytes(const xabe_gguf_file* f, const char* name, size_t* len);

/* Metadata (F:194-270).  The typed getters return 1 and store the value when the key exists WITH that
 * type, else 0: no coercion, as in the reference. */
const char* xabe_gguf_key_at(const xabe_gguf_file* f, size_t index);   /* keys in file order */
/* type tag of a key's value; for arrays also the element tag and the count.  0 when the key is absent. */
int xabe_gguf_value_type_of(const xabe_gguf_file* f, const char* key, int* type, int* elem_type, uint64_t* count);
int xabe_gguf_get_u32(const xabe_gguf_file* f, const char* key, uint32_t* out);
int xabe_gguf_get_u64(const xabe_gguf_file* f, const char* key, uint64_t* out);
int xabe_gguf_get_f32(const xabe_gguf_file* f, const char* key, float* out);
const char* xabe_gguf_get_str(const xabe_gguf_file* f, const char* key, size_t* len);
/* Arrays: packed little-endian elements of a numeric or bool array whose element tag is `elem_type`
 * (bool as one byte each), or NULL; one element of a string array, or NULL. */
const void* xabe_gguf_get_array(const xabe_gguf_file* f, const char* key, int elem_type, uint64_t* count);
const char* xabe_gguf_get_string_array_item(const xabe_gguf_file* f, const char* key, uint64_t index, size_t* len);

/* ---- one layer's feed-forward tensors on the device ---- */
typedef struct xabe_moe_layer xabe_moe_layer;
typedef struct xabe_dense_ffn_layer xabe_dense_ffn_layer;

/* MoeLayerWeights::upload (B:660-756).  Reads `blk.<layer>.{post_attention_norm, ffn_gate_inp,
 * ffn_gate_inp_shexp, ffn_{gate,up,down}_exps, ffn_{gate,up,down}_shexp}.weight`; norm, router and shared
 * gate vector are widened to f32 on the host (f32 as is, bf16 by a 16-bit shift; anything else
 * XABE_ERR_UNSUPPORTED_DENSE_TYPE), the expert stacks stay in the file's format and block stride
 * (Q6_K / Q8_0; Q4_0 / Q4_K / Q5_K are recognised and refused with XABE_ERR_UNSUPPORTED_QUANT, any other
 * type likewise).  Shapes are checked against the geometry (XABE_ERR_SHAPE_MISMATCH), a tensor the file
 * lacks is XABE_ERR_MISSING_TENSOR.  Allocates; synchronises `stream` before returning. */
int xabe_moe_layer_upload(void* stream, const xabe_gguf_file* f, uint32_t layer, const xabe_moe_geometry* geometry,
                          xabe_moe_layer** out);
void xabe_moe_layer_free(xabe_moe_layer* l);
/* The argument xabe_moe_block_forward takes, pointing at this layer's device tensors (valid until _free). */
const xabe_moe_layer_weights* xabe_moe_layer_weights_of(const xabe_moe_layer* l);
uint32_t xabe_moe_layer_index(const xabe_moe_layer* l);                      /* B:759-761 */
int xabe_moe_layer_expert_quants(const xabe_moe_layer* l, int out[3]);       /* B:768-770 gate, up, down */
int xabe_moe_layer_shared_quants(const xabe_moe_layer* l, int out[3]);       /* B:773-779 */
int xabe_moe_layer_router_types(const xabe_moe_layer* l, int out[2]);        /* B:785-787 ggml types in the file */
size_t xabe_moe_layer_bytes(const xabe_moe_layer* l);                        /* B:790-800 */

/* DenseFfnLayerWeights::upload (D:663-760), quantized residency: `blk.<layer>.{post_attention_norm,
 * ffn_gate, ffn_up, ffn_down}.weight` with hidden / intermediate as given. */
int xabe_dense_ffn_layer_upload(void* stream, const xabe_gguf_file* f, uint32_t layer, size_t hidden,
                                size_t intermediate, xabe_dense_ffn_layer** out);
void xabe_dense_ffn_layer_free(xabe_dense_ffn_layer* l);
const xabe_dense_ffn_layer_weights* xabe_dense_ffn_layer_weights_of(const xabe_dense_ffn_layer* l);
int xabe_dense_ffn_layer_quants(const xabe_dense_ffn_layer* l, int out[3]);
size_t xabe_dense_ffn_layer_bytes(const xabe_dense_ffn_layer* l);

#ifdef __cplusplus
}
#endif
#endif /* XABE_GGUF_H */

/*
 * libxabe_hip, LM head: logits[t][v] = sum_h weight[v][h] * hidden_states[t][h] over a quantized or 16-bit
 * vocabulary matrix, and the device half of greedy sampling (argmax, and the softmax probability of the maximum).
 *
 * Replaces `xabe_cuda::kernels::lm_head::{LmHeadKernels, LmHeadGeometry, HeadFormat, HeadTensor, LmHeadError}`
 * ("L" = crates/xabe-cuda/src/kernels/lm_head.rs).  The same streaming machinery as the decode kernels of
 * xabe_hip.h: every 16-byte piece of the matrix is requested once, coalesced, and the fields are unpacked
 * from a wavefront-private staging slot; a pass over the weights serves up to
 * XABE_LM_HEAD_MAX_BATCH_TILE tokens.  Statuses are the `xabe_status` values of xabe_hip.h.
 */
#ifndef XABE_LM_HEAD_H
#define XABE_LM_HEAD_H

#include <stddef.h>
#include <stdint.h>

#include "xabe_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Tokens one pass over the weights serves (L:125 has 8: here a lane keeps the tile's activations in
 * registers, 32 per token, which fits four). */
#define XABE_LM_HEAD_MAX_BATCH_TILE 4
/* Length of the partial-winner buffers xabe_lm_head_argmax takes (L:169). */
#define XABE_LM_HEAD_ARGMAX_BLOCKS 512

/* HeadFormat (L:1206-1258).  Q4_0 / Q4_K / Q5_K are recognised and refused with XABE_ERR_UNSUPPORTED_QUANT. */
typedef enum xabe_head_format {
  XABE_HEAD_Q8_0 = 0,
  XABE_HEAD_BF16 = 1,
  XABE_HEAD_Q6K = 2,
  XABE_HEAD_F16 = 3,
  XABE_HEAD_Q4_0 = 4,
  XABE_HEAD_Q4K = 5,
  XABE_HEAD_Q5K = 6
} xabe_head_format;

/* HeadFormat::from_ggml (L:1243-1258): the format a ggml type id names, or -1. */
int xabe_head_format_from_ggml(int ggml_type);

/* LmHeadGeometry (L:1304-1395). */
typedef struct xabe_lm_head_geometry {
  size_t hidden;
  size_t vocab;
  size_t max_tokens;
} xabe_lm_head_geometry;

xabe_lm_head_geometry xabe_lm_head_geometry_qwen3_6(size_t max_tokens);                      /* L:1318-1324: 2048 x 248320 */
size_t xabe_lm_head_row_bytes_for(const xabe_lm_head_geometry* g, int format);               /* L:1339-1349 */
size_t xabe_lm_head_weight_bytes_for(const xabe_lm_head_geometry* g, int format);            /* L:1358-1360 */
size_t xabe_lm_head_elements(const xabe_lm_head_geometry* g);                                /* L:1363-1365 */
size_t xabe_lm_head_weight_passes(const xabe_lm_head_geometry* g, size_t tokens);            /* L:1381-1383 */
size_t xabe_lm_head_weight_bytes_read(const xabe_lm_head_geometry* g, int format, size_t tokens); /* L:1390-1392 */

typedef struct xabe_lm_head xabe_lm_head;

/* LmHeadKernels::new (L:1500-1560): hidden and vocab non-zero, hidden a multiple of 512, max_tokens non-zero;
 * else XABE_ERR_UNSUPPORTED_GEOMETRY. */
int xabe_lm_head_new(const xabe_lm_head_geometry* geometry, xabe_lm_head** out);
void xabe_lm_head_free(xabe_lm_head* h);
int xabe_lm_head_geometry_of(const xabe_lm_head* h, xabe_lm_head_geometry* out);             /* L:1680-1682 */

/* LmHeadKernels::forward (L:1694-1935).  `weight` is the tensor as the file holds it ([vocab][hidden] rows in
 * `format`), `hidden_states` [max_tokens][hidden], `logits` [max_tokens][vocab]; rows past `tokens` are
 * neither read nor written.  Checks, in the reference's order: whole blocks (XABE_ERR_RAGGED_WEIGHTS),
 * element count (XABE_ERR_WRONG_ELEMENT_COUNT), 1 <= tokens <= max_tokens (XABE_ERR_TOO_MANY_TOKENS), buffer
 * lengths (XABE_ERR_SHAPE_MISMATCH).  The weight tensor must start on a 16-byte boundary.
 * A token's logits are the same bits whatever the batch it arrives in. */
int xabe_lm_head_forward(const xabe_lm_head* h, void* stream, int format, const void* weight, size_t weight_len,
                         const float* hidden_states, size_t hidden_states_len, size_t tokens, float* logits,
                         size_t logits_len);

/* LmHeadKernels::argmax (L:1938-2010): out[0] = argmax(values[..n]), ties to the lower index, with the
 * reference's scalar semantics for NaN (a NaN never wins; a NaN at index 0 keeps index 0).  The partial
 * buffers hold XABE_LM_HEAD_ARGMAX_BLOCKS elements each and are caller-owned, so a decode step allocates nothing. */
int xabe_lm_head_argmax(const xabe_lm_head* h, void* stream, const float* values, size_t values_len, size_t n,
                        float* partial_values, size_t partial_values_len, int32_t* partial_indices,
                        size_t partial_indices_len, int32_t* out, size_t out_len);
/* LmHeadKernels::argmax_prob (L:2017-2044): out[0] = 1 / sum(exp(values[i] - max)). */
int xabe_lm_head_argmax_prob(const xabe_lm_head* h, void* stream, const float* values, size_t values_len, size_t n,
                             float* out, size_t out_len);

#ifdef __cplusplus
}
#endif
#endif /* XABE_LM_HEAD_H */

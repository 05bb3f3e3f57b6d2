/*
 * libxabe_hip: the quantized MoE feed-forward block for one MI355X (gfx950).
 *
 * C ABI that a Rust FFI crate binds in place of `xabe_cuda::kernels::moe`.
 * Each entry point names the reference item it replaces; paths are relative to
 * the reference tree, "M" = crates/xabe-cuda/src/kernels/moe.rs,
 * "B" = crates/xabe-engine/src/block/moe.rs, "D" = crates/xabe-engine/src/block/dense_ffn.rs.
 *
 * Conventions
 *   - Every function returns an `xabe_status` (0 = ok).  `xabe_last_error()` gives the
 *     message of the calling thread's last failure, worded like the reference's
 *     `MoeError` / `MoeBlockError` Display impls.
 *   - Device memory is passed as a raw pointer plus an element count, the way the
 *     reference passes `&CudaSlice<T>`; lengths are checked where the reference checks them.
 *   - `stream` is a `hipStream_t` passed as `void*` (NULL = the default stream).
 *   - Every launch is asynchronous on `stream`, sized from the geometry only, and reads the
 *     live token count from the device scalar `valid_tokens` (M:34-41): the sequence can be
 *     captured into a hipGraph.  No entry point allocates except the `_new` / `_upload` ones.
 *   - One kernels+buffers pair per pass shape per thread; calls on one buffer set must not overlap.
 */
#ifndef XABE_HIP_H
#define XABE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- status codes: MoeError (M:4602-4637) and MoeBlockError (B:494-547) ---- */
typedef enum xabe_status {
  XABE_OK = 0,
  XABE_ERR_COMPILE = 1,               /* MoeError::Compile: the code object failed to load on this device */
  XABE_ERR_DRIVER = 2,                /* MoeError::Driver: a HIP runtime call failed */
  XABE_ERR_MMA = 3,                   /* MoeError::Mma: the matrix-core path rejected its operands */
  XABE_ERR_UNSUPPORTED_GEOMETRY = 4,  /* MoeError::UnsupportedGeometry { geometry, reason } */
  XABE_ERR_RAGGED_WEIGHTS = 5,        /* MoeError::RaggedWeights { which, bytes, block_bytes } */
  XABE_ERR_WRONG_ELEMENT_COUNT = 6,   /* MoeError::WrongElementCount { which, expected, found } */
  XABE_ERR_TOO_MANY_TOKENS = 7,       /* MoeError::TooManyTokens { tokens, max_tokens } */
  XABE_ERR_SHARED_ONLY_BUFFERS = 8,   /* MoeError::SharedOnlyBuffers { entry } */
  XABE_ERR_BUFFER_LENGTH = 9,         /* MoeBlockError::BufferLength { what, expected, found } */
  XABE_ERR_INVALID_ARGUMENT = 10,     /* a NULL handle or pointer (the Rust API rules this out by type) */
  XABE_ERR_UNSUPPORTED_QUANT = 11,    /* MoeBlockError::UnsupportedExpertType: Q4_0/Q4_K/Q5_K have no kernel here */
  XABE_ERR_FFN_KIND_MISMATCH = 12,    /* MoeBlockError::FfnKindMismatch */
  XABE_ERR_MISSING_TENSOR = 13,       /* MoeBlockError::MissingTensor { role, layer } */
  XABE_ERR_UNSUPPORTED_DENSE_TYPE = 14, /* MoeBlockError::UnsupportedDenseType { name, found } */
  XABE_ERR_SHAPE_MISMATCH = 15,       /* MoeBlockError::ShapeMismatch { name, expected, found } */
  /* GgufError (crates/xabe-gguf/src/error.rs:11-108), one status per variant */
  XABE_ERR_GGUF_BAD_MAGIC = 20,
  XABE_ERR_GGUF_UNSUPPORTED_VERSION = 21,
  XABE_ERR_GGUF_UNEXPECTED_EOF = 22,
  XABE_ERR_GGUF_INVALID_UTF8 = 23,
  XABE_ERR_GGUF_NEGATIVE_COUNT = 24,
  XABE_ERR_GGUF_DUPLICATE_KEY = 25,
  XABE_ERR_GGUF_UNKNOWN_VALUE_TYPE = 26,
  XABE_ERR_GGUF_NESTED_ARRAY = 27,
  XABE_ERR_GGUF_BAD_ALIGNMENT_TYPE = 28,
  XABE_ERR_GGUF_BAD_ALIGNMENT = 29,
  XABE_ERR_GGUF_TOO_MANY_DIMENSIONS = 30,
  XABE_ERR_GGUF_ZERO_DIMENSION = 31,
  XABE_ERR_GGUF_DUPLICATE_TENSOR = 32,
  XABE_ERR_GGUF_UNSUPPORTED_GGML_TYPE = 33,
  XABE_ERR_GGUF_UNALIGNED_ELEMENT_COUNT = 34,
  XABE_ERR_GGUF_OFFSET_OVERFLOW = 35,
  XABE_ERR_GGUF_TENSOR_OUT_OF_BOUNDS = 36,
  XABE_ERR_GGUF_IO = 37
} xabe_status;

const char* xabe_last_error(void);
const char* xabe_status_name(int status);
/* Library version and the architecture the code object was built for ("gfx950"). */
const char* xabe_version(void);

/* ---- MoeGeometry (M:4523-4598) ---- */
typedef struct xabe_moe_geometry {
  size_t num_experts;
  size_t experts_per_token;
  size_t hidden;
  size_t intermediate;
  size_t block_size;
  size_t max_tokens;
} xabe_moe_geometry;

/* MoeGeometry::qwen3_6 (M:4544-4553) */
xabe_moe_geometry xabe_moe_geometry_qwen3_6(size_t block_size, size_t max_tokens);
size_t xabe_moe_geometry_max_flat_pairs(const xabe_moe_geometry* g);         /* M:4556-4558 */
size_t xabe_moe_geometry_sorted_capacity(const xabe_moe_geometry* g);        /* M:4575-4584 */
size_t xabe_moe_geometry_expert_block_capacity(const xabe_moe_geometry* g);  /* M:4587-4589 */
size_t xabe_moe_geometry_stack_elements(const xabe_moe_geometry* g);         /* M:4595-4597 */
/* crates/xabe-engine/src/forward.rs:163-165: 32 up to 1152 tokens, else 64 */
size_t xabe_moe_block_size_for(size_t tokens);

/* ---- ExpertQuant (M:298-401), QuantTensor (M:448-464), to_device_layout (M:410-444) ---- */
typedef enum xabe_expert_quant {
  XABE_QUANT_Q6K = 0,
  XABE_QUANT_Q8_0 = 1,
  XABE_QUANT_Q4_0 = 2, /* community formats: recognised, rejected with XABE_ERR_UNSUPPORTED_QUANT */
  XABE_QUANT_Q4K = 3,
  XABE_QUANT_Q5K = 4
} xabe_expert_quant;

size_t xabe_expert_quant_block_elements(int quant);   /* M:353-360 */
size_t xabe_expert_quant_file_block_bytes(int quant); /* M:366-374 */
/* M:388-400.  Equal to file_block_bytes for every format: the kernels stream the 210-byte
 * Q6_K superblock as the file stores it, so there is no 224-byte device stride. */
size_t xabe_expert_quant_block_bytes(int quant);
int xabe_expert_quant_is_community(int quant);        /* M:348-350 */

/* A quantized stack resident on the device.  `bytes` is a device pointer to `len` bytes and must lie on a
 * 16-byte boundary (any device allocation does; a sub-tensor of one must be placed accordingly): every entry
 * point that takes a stack answers XABE_ERR_INVALID_ARGUMENT otherwise.  Inside the stack, blocks sit wherever
 * their 210- or 34-byte stride puts them. */
typedef struct xabe_quant_tensor {
  const void* bytes;
  size_t len;
  int quant;
} xabe_quant_tensor;

/* M:410-444.  The identity copy: `out` (host, `len` bytes) receives `bytes` unchanged and
 * `*out_len = len`.  Kept so callers that route every upload through the hook keep working. */
int xabe_to_device_layout(int quant, const uint8_t* bytes, size_t len, uint8_t* out, size_t* out_len);

/* ---- MoeKernels (M:5033-5458) ---- */
typedef struct xabe_moe_kernels xabe_moe_kernels;
typedef struct xabe_moe_buffers xabe_moe_buffers;

typedef enum xabe_buffer_scope { XABE_SCOPE_ROUTED = 0, XABE_SCOPE_SHARED_ONLY = 1 } xabe_buffer_scope; /* M:4698-4705 */

/* MoeKernels::new (M:5038-5330): validates the geometry (same rules, same reasons) and
 * loads the gfx950 code object on the current device. */
int xabe_moe_kernels_new(const xabe_moe_geometry* geometry, xabe_moe_kernels** out);
void xabe_moe_kernels_free(xabe_moe_kernels* k);
int xabe_moe_kernels_geometry(const xabe_moe_kernels* k, xabe_moe_geometry* out); /* M:5333 */
/* M:5416-5418: force the matrix-core (MFMA) regime off; prefill widths then take the fp32 kernels. */
int xabe_moe_kernels_disable_tensor_cores(xabe_moe_kernels* k);
int xabe_moe_kernels_tensor_cores_enabled(const xabe_moe_kernels* k);             /* M:5456-5458 */
/* M:5432-5434: no community-format kernels exist here; `on != 0` is accepted and recorded only. */
int xabe_moe_kernels_force_community(xabe_moe_kernels* k, int on);
/* M:5450-5452: pin the fp32 decode kernels at any width so rows equal plain decode bit for bit. */
/* No counterpart in the reference (a test and comparison switch like force_community): which of the two
 * matrix-core grouped-GEMM kernels the routed launches of a wide pass take.  0 (default) and 1: the kernel whose
 * wavefronts all load, dequantise and multiply in turn; 2: the kernel whose wavefronts are specialised (half of them
 * multiply, half dequantise) wherever the shape allows: same bits, measured slower at every width, kept as the
 * reproducible record of that comparison. */
int xabe_moe_kernels_set_mfma_form(xabe_moe_kernels* k, int form);
int xabe_moe_kernels_set_exact_decode_regime(xabe_moe_kernels* k, int on);

/* MoeKernels::buffers (M:5338-5340) / shared_only_buffers (M:5354-5360) */
int xabe_moe_buffers_new(const xabe_moe_kernels* k, void* stream, xabe_moe_buffers** out);
int xabe_moe_shared_only_buffers_new(const xabe_moe_kernels* k, void* stream, int mma, xabe_moe_buffers** out);
void xabe_moe_buffers_free(xabe_moe_buffers* b);

/* MoeBuffers accessors (M:4768-4864): device pointer + element count. */
int xabe_moe_buffers_scope(const xabe_moe_buffers* b);
int32_t* xabe_moe_buffers_topk_ids(const xabe_moe_buffers* b, size_t* len);
float* xabe_moe_buffers_topk_weights(const xabe_moe_buffers* b, size_t* len);
int32_t* xabe_moe_buffers_sorted_token_ids(const xabe_moe_buffers* b, size_t* len);
int32_t* xabe_moe_buffers_expert_ids(const xabe_moe_buffers* b, size_t* len);
int32_t* xabe_moe_buffers_bucket_live(const xabe_moe_buffers* b, size_t* len);
int32_t* xabe_moe_buffers_num_tokens_post_pad(const xabe_moe_buffers* b, size_t* len);
int32_t* xabe_moe_buffers_valid_tokens(const xabe_moe_buffers* b, size_t* len);
float* xabe_moe_buffers_partial(const xabe_moe_buffers* b, size_t* len);
float* xabe_moe_buffers_shared_inter(const xabe_moe_buffers* b, size_t* len);
size_t xabe_moe_buffers_bytes(const xabe_moe_buffers* b);

/* MoeKernels::set_valid_tokens (M:5473-5491): one 4-byte host-to-device write, skipped when unchanged. */
int xabe_moe_set_valid_tokens(const xabe_moe_kernels* k, void* stream, xabe_moe_buffers* b, size_t tokens);

/* MoeKernels::route (M:5567-5609): softmax, top-k (probability descending, lower index on ties),
 * renormalise.  `logits` is [max_tokens][num_experts]. */
int xabe_moe_route(const xabe_moe_kernels* k, void* stream, xabe_moe_buffers* b, const float* logits, size_t logits_len);
/* MoeKernels::build_dispatch (M:5623-5714) */
int xabe_moe_build_dispatch(const xabe_moe_kernels* k, void* stream, xabe_moe_buffers* b);
/* MoeKernels::route_and_dispatch (M:5498-5558): the dispatch tables are skipped when the flat
 * per-pair kernels will run (max_tokens <= 4, or the exact decode regime). */
int xabe_moe_route_and_dispatch(const xabe_moe_kernels* k, void* stream, xabe_moe_buffers* b, const float* logits,
                                size_t logits_len);

/* MoeKernels::grouped_forward_partial (M:5727-6170): leaves partial[(t*K+k)*hidden ..] = w_{t,k} * y. */
int xabe_moe_grouped_forward_partial(const xabe_moe_kernels* k, void* stream, xabe_moe_buffers* b,
                                     xabe_quant_tensor gate, xabe_quant_tensor up, xabe_quant_tensor down,
                                     const float* hidden_states, size_t hidden_states_len);
/* One half of grouped_forward_partial on its own: stage 0 = gate/up + SwiGLU (fills the intermediate),
 * stage 1 = down (fills `partial`).  For measurement: the reference's bench times the stages of the
 * path separately (crates/xabe-cuda/src/bin/bench_moe.rs:140-334). */
int xabe_moe_grouped_forward_stage(const xabe_moe_kernels* k, void* stream, xabe_moe_buffers* b, xabe_quant_tensor gate,
                                   xabe_quant_tensor up, xabe_quant_tensor down, const float* hidden_states,
                                   size_t hidden_states_len, int stage);
/* MoeKernels::grouped_forward_partial_with_shared (M:6190-6335).  `*fused` = 1 when the shared
 * expert rode the routed launches, 0 (nothing launched) when the pass is not covered. */
int xabe_moe_grouped_forward_partial_with_shared(const xabe_moe_kernels* k, void* stream, xabe_moe_buffers* b,
                                                 xabe_quant_tensor gate, xabe_quant_tensor up, xabe_quant_tensor down,
                                                 xabe_quant_tensor shared_gate, xabe_quant_tensor shared_up,
                                                 xabe_quant_tensor shared_down, const float* hidden_states,
                                                 size_t hidden_states_len, float* out, size_t out_len, int* fused);
/* MoeKernels::grouped_forward (M:6345-6376): partial + the ascending-k sum (`moe_reduce`, M:4049-4065). */
int xabe_moe_grouped_forward(const xabe_moe_kernels* k, void* stream, xabe_moe_buffers* b, xabe_quant_tensor gate,
                             xabe_quant_tensor up, xabe_quant_tensor down, const float* hidden_states,
                             size_t hidden_states_len, float* out, size_t out_len);
/* MoeKernels::shared_expert (M:6488-6714): expert_mlp on every live token, ungated.  Also the dense
 * sibling's MLP (D:34-43): widths come from the geometry, stacks are single-expert. */
int xabe_moe_shared_expert(const xabe_moe_kernels* k, void* stream, xabe_moe_buffers* b, xabe_quant_tensor gate,
                           xabe_quant_tensor up, xabe_quant_tensor down, const float* hidden_states,
                           size_t hidden_states_len, float* out, size_t out_len);
/* MoeKernels::shared_expert_mma (M:6389-6476) with SharedExpertInt8::repack (M:4896-4938) folded in:
 * the matrix-core path reads the quantized stacks directly, so there is nothing to repack. */
int xabe_moe_shared_expert_mma(const xabe_moe_kernels* k, void* stream, xabe_moe_buffers* b, xabe_quant_tensor gate,
                               xabe_quant_tensor up, xabe_quant_tensor down, const float* hidden_states,
                               size_t hidden_states_len, float* out, size_t out_len);

/* ---- kernels the engine compiled for itself through NVRTC; here they are library entry points ---- */
/* LayerOpsKernels::rms_norm (crates/xabe-cuda/src/kernels/layer_ops.rs:777-805): every row, 1/sqrtf. */
int xabe_rms_norm(void* stream, const float* x, size_t x_len, const float* weight, size_t weight_len, float* out,
                  size_t out_len, size_t rows, size_t width, float eps);
/* moe_block_router_logits (B:301-382, launch B:1150-1184).  `router` is f32 [E][H], or Q8_0 bytes
 * dequantised in-kernel as q*d when `router_quant` is XABE_QUANT_Q8_0 (pass -1 for f32). */
int xabe_moe_router_logits(const xabe_moe_kernels* k, void* stream, const xabe_moe_buffers* b, const void* router,
                           size_t router_len, int router_quant, const float* normed, size_t normed_len, float* logits,
                           size_t logits_len);
/* moe_block_gate_and_combine (B:424-483, launch B:1297-1326) */
int xabe_moe_gate_and_combine(const xabe_moe_kernels* k, void* stream, const xabe_moe_buffers* b,
                              const float* shared_gate_inp, const float* normed, const float* shexp,
                              const float* residual, float* gate, float* routed, float* ffn_out, float* l_out);
/* dense_ffn_add_residual (D:1149-1175): l_out = ffn_out + residual on live rows. */
int xabe_dense_ffn_add_residual(const xabe_moe_kernels* k, void* stream, const xabe_moe_buffers* b,
                                const float* ffn_out, const float* residual, float* l_out);
/* Adds `bias[e]` to every live row of `logits` (a harness hook: skewed-routing workloads add a
 * per-expert bias between the router GEMV and `route`; no counterpart in the reference). */
int xabe_moe_add_logit_bias(const xabe_moe_kernels* k, void* stream, const xabe_moe_buffers* b, const float* bias,
                            float* logits);
/* Standalone dequantisation, bit-identical to the CPU reference
 * (crates/xabe-cuda/src/kernels/dequant.rs:19-27). `out` holds blocks*block_elements floats. */
int xabe_dequantize(void* stream, int quant, const void* bytes, size_t len, float* out, size_t out_len);

/* MmaKernels::quantize_rows (crates/xabe-cuda/src/kernels/mma.rs:769-811, kernel :118-157): fp32 rows [rows][k] ->
 * int8 `q` [rows][k] and one fp32 scale per 32 elements `scales` [rows][k / 32]; d = amax / 127 (1.0 for a block
 * of zeros), q = rintf(v * (127 / amax)) clamped to +-127.  Lengths are checked as "at least", as the reference
 * does; k not a multiple of 32 is XABE_ERR_MMA (MmaError::RaggedContraction).  The matrix-core path of this
 * library takes fp16 operands and does not use it. */
int xabe_mma_quantize_rows(void* stream, const float* x, size_t x_len, int8_t* q, size_t q_len, float* scales,
                           size_t scales_len, size_t rows, size_t k);

/* ---- MoeBlock / MoeLayerWeights (B:634-1330) and DenseFfnBlock (D:1047-1178): block sequencing ---- */
typedef struct xabe_moe_block xabe_moe_block;

/* Device-resident tensors of one layer (B:634-658).  The router may be f32 or Q8_0. */
typedef struct xabe_moe_layer_weights {
  const float* post_norm;       /* [hidden] */
  const void* router;           /* [num_experts][hidden] */
  int router_quant;             /* -1 = f32, XABE_QUANT_Q8_0 = quantized */
  xabe_quant_tensor gate_exps, up_exps, down_exps;
  const float* shared_gate_inp; /* [hidden] */
  xabe_quant_tensor shared_gate, shared_up, shared_down;
} xabe_moe_layer_weights;

/* MoeBlock::new (B:948-977): kernels, buffers and the normed/logits/routed/shexp/gate scratch. */
int xabe_moe_block_new(const xabe_moe_geometry* geometry, float eps, void* stream, xabe_moe_block** out);
void xabe_moe_block_free(xabe_moe_block* blk);
int xabe_moe_block_publish_tokens(xabe_moe_block* blk, void* stream, size_t tokens); /* B:1081-1089 */
/* MoeBlock::forward (B:1091-1329).  residual / ffn_out / l_out are [max_tokens][hidden];
 * `logit_bias` (may be NULL) is added to the router logits before routing.
 * From 64 tokens up the shared expert's launches go to a stream the handle owns, forked from `stream` after the
 * RMSNorm and joined to it before the combine (event record / wait only, capturable): work the caller enqueues on
 * `stream` after the call is ordered after all of it.  One handle serves one stream at a time. */
int xabe_moe_block_forward(xabe_moe_block* blk, void* stream, const xabe_moe_layer_weights* w, const float* residual,
                           size_t residual_len, size_t tokens, const float* logit_bias, float* ffn_out,
                           size_t ffn_out_len, float* l_out, size_t l_out_len);
/* The post-mixer seam between consecutive layers (the reference's seam-fusion work, docs/BENCHMARKS.md:1340-1377 and
 * the row it measured at :1761, "the next layer's RMSNorm in the MoE combine kernel's tail ... the mixer skips its
 * norm launch").  Two halves that pair up across a layer boundary:
 *   producer: with `next_norm_weight` set, the launch that finishes l_out also writes
 *             next_normed = rms_norm(l_out, next_norm_weight, next_eps) for the live rows (and, if `next_normed_h` is
 *             set, the same values rounded once to fp16, the copy the matrix-core kernels read), so the consumer of
 *             l_out launches no RMSNorm and makes no second pass over l_out;
 *   consumer: with `input_normed` nonzero, the block takes its normalised rows as given in its own `normed` buffer
 *             (xabe_moe_block_normed_mut; at matrix-core widths also the fp16 copy, xabe_moe_block_normed_h_mut)
 *             instead of normalising `residual`, which it still adds back at the end.
 * Every tensor holds the bits the unfused sequence (block, RMSNorm launch, block) produces; rows past the live
 * count of next_normed are left as they were.  next_normed may be the producing block's own normed buffer (one
 * handle serving every layer of a stack).  Hidden sizes above 2048 take the separate RMSNorm launch inside the call.
 * `ffn_out` may be NULL here (a read-back tensor the layer loop does not consume); with `skip_readback` nonzero the
 * `routed` tensor behind xabe_moe_block_routed is not written either (its contents are then stale). */
typedef struct xabe_moe_seam {
  int input_normed;
  int skip_readback;
  const float* next_norm_weight; /* [hidden] or NULL */
  float next_eps;
  float* next_normed;            /* [max_tokens][hidden] */
  size_t next_normed_len;
  void* next_normed_h;           /* fp16 [max_tokens][hidden] or NULL */
  size_t next_normed_h_len;
} xabe_moe_seam;
/* xabe_moe_block_forward with a seam on either side; `seam` NULL is xabe_moe_block_forward itself. */
int xabe_moe_block_forward_seam(xabe_moe_block* blk, void* stream, const xabe_moe_layer_weights* w, const float* residual,
                                size_t residual_len, size_t tokens, const float* logit_bias, float* ffn_out,
                                size_t ffn_out_len, float* l_out, size_t l_out_len, const xabe_moe_seam* seam);
/* Writable views of the block's normalised rows for a producer's `next_normed` / `next_normed_h` (the second is NULL
 * with length 0 below matrix-core widths, where no kernel reads an fp16 copy). */
float* xabe_moe_block_normed_mut(xabe_moe_block* blk, size_t* len);
void* xabe_moe_block_normed_h_mut(xabe_moe_block* blk, size_t* len);
/* The combine with the producer half of the seam as a step of its own, for callers that sequence the block
 * themselves (xabe_moe_gate_and_combine plus the tail; `routed` and `ffn_out` may be NULL; the next_* arguments as in
 * xabe_moe_seam, all NULL for the plain combine).  Rows of at most 2048 elements. */
int xabe_moe_gate_and_combine_seam(const xabe_moe_kernels* k, void* stream, const xabe_moe_buffers* b,
                                   const float* shared_gate_inp, const float* normed, const float* shexp,
                                   const float* residual, float* gate, float* routed, float* ffn_out, float* l_out,
                                   const float* next_norm_weight, float next_eps, float* next_normed, void* next_normed_h);
int xabe_moe_block_disable_tensor_cores(xabe_moe_block* blk);            /* B:987-989 */
int xabe_moe_block_set_exact_decode_regime(xabe_moe_block* blk, int on); /* B:1003-1005 */
/* At max_tokens <= 32 and the model shapes (hidden 2048 / intermediate 512, and the 512 / 256 test shape) the
 * block's eight steps are regrouped into three launches (logits + shared gate/up; route + gate/up; down +
 * combine) that compute the same values bit for bit.  `on` = 0 keeps one launch per step as the reference
 * has them (B:1091-1329); the switch exists for tests and measurement. */
int xabe_moe_block_set_fused_decode(xabe_moe_block* blk, int on);
int xabe_moe_block_set_mfma_form(xabe_moe_block* blk, int form); /* xabe_moe_kernels_set_mfma_form on the block's kernels */
/* Measurement hook, no counterpart in the reference: ONE of the three decode launches (0: logits + shared
 * gate/up, 1: route + gate/up, 2: down + combine) with the arguments of xabe_moe_block_forward, so that a
 * launch can be timed and profiled alone.  Stage n reads what stages < n of an earlier call left in the
 * block's buffers; the live-token count is the one last published.  From eight tokens up stage 1 is two
 * launches, the routing launch and the gate/up launch that reads its selections. */
int xabe_moe_block_forward_stage(xabe_moe_block* blk, void* stream, const xabe_moe_layer_weights* w,
                                 const float* residual, size_t residual_len, const float* logit_bias, float* ffn_out,
                                 size_t ffn_out_len, float* l_out, size_t l_out_len, int stage);
int xabe_moe_block_tensor_cores_enabled(const xabe_moe_block* blk);      /* B:1008-1010 */
/* No counterpart in the reference.  For callers that cannot allocate device memory (code that builds its launches
 * under hipGraph capture without handles, tight serving loops, harnesses that forbid hipMalloc): xabe_moe_block_forward
 * at decode widths with the block's working set (normalised rows, logits, selections, intermediates, the live-token
 * count) in a device array the library holds statically (1.4 MB per GPU, until the process ends) instead of in buffers
 * that xabe_moe_block_new allocates.  No handle, no hipMalloc/hipFree, the same three launches and the same bits.
 * Serves max_tokens <= 32, hidden <= 2048, intermediate <= 512, <= 512 experts, top-k <= 8, in the shapes and
 * formats of the three-launch decode block; anything larger is XABE_ERR_UNSUPPORTED_GEOMETRY.  The live-token count
 * is published by a one-thread kernel, so the call may be captured.  All calls on one GPU share that GPU's array:
 * calls that overlap on one GPU race.  The first call on a device resolves the array's address there; make it
 * outside a capture (a first call that arrives while `stream` is capturing is refused with
 * XABE_ERR_INVALID_ARGUMENT and records nothing). */
int xabe_moe_block_forward_noalloc(const xabe_moe_geometry* geometry, float eps, void* stream,
                                   const xabe_moe_layer_weights* w, const float* residual, size_t residual_len,
                                   size_t tokens, const float* logit_bias, float* ffn_out, size_t ffn_out_len, float* l_out,
                                   size_t l_out_len);
/* Read-back accessors (B:1023-1060): device pointer + element count. */
const float* xabe_moe_block_normed(const xabe_moe_block* blk, size_t* len);
const float* xabe_moe_block_router_logits(const xabe_moe_block* blk, size_t* len);
const float* xabe_moe_block_routed(const xabe_moe_block* blk, size_t* len);
const float* xabe_moe_block_shared_ungated(const xabe_moe_block* blk, size_t* len);
const float* xabe_moe_block_shared_gate(const xabe_moe_block* blk, size_t* len);
xabe_moe_buffers* xabe_moe_block_buffers(const xabe_moe_block* blk);
xabe_moe_kernels* xabe_moe_block_kernels(const xabe_moe_block* blk);

typedef struct xabe_dense_ffn_block xabe_dense_ffn_block;
typedef struct xabe_dense_ffn_layer_weights {
  const float* post_norm; /* [hidden] */
  xabe_quant_tensor gate, up, down;
} xabe_dense_ffn_layer_weights;
/* DenseFfnBlock::new / forward (D:1047-1178): shared-only buffers, rms_norm -> shared_expert -> residual add. */
int xabe_dense_ffn_block_new(size_t hidden, size_t intermediate, size_t max_tokens, float eps, void* stream,
                             xabe_dense_ffn_block** out);
void xabe_dense_ffn_block_free(xabe_dense_ffn_block* blk);
int xabe_dense_ffn_block_forward(xabe_dense_ffn_block* blk, void* stream, const xabe_dense_ffn_layer_weights* w,
                                 const float* residual, size_t residual_len, size_t tokens, float* ffn_out,
                                 size_t ffn_out_len, float* l_out, size_t l_out_len);
int xabe_dense_ffn_block_disable_tensor_cores(xabe_dense_ffn_block* blk);
int xabe_dense_ffn_block_tensor_cores_enabled(const xabe_dense_ffn_block* blk);
int xabe_dense_ffn_block_publish_tokens(xabe_dense_ffn_block* blk, void* stream, size_t tokens); /* D: publish_tokens */
const float* xabe_dense_ffn_block_normed(const xabe_dense_ffn_block* blk, size_t* len);

/* ---- FfnBlock / FfnLayerWeights (crates/xabe-engine/src/block/ffn.rs:27-228): which feed-forward block a layer
 * runs, chosen once from the model configuration; the pairing of block and weights is checked on every pass. ---- */
typedef enum xabe_ffn_kind { XABE_FFN_MOE = 0, XABE_FFN_DENSE = 1 } xabe_ffn_kind;
/* The fields of ModelConfig the geometry is made from (crates/xabe-model/src/config.rs:126-187): `hidden` for both
 * kinds; the MoeConfig fields for XABE_FFN_MOE, DenseFfnConfig::intermediate for XABE_FFN_DENSE. */
typedef struct xabe_ffn_config {
  int kind; /* xabe_ffn_kind */
  size_t hidden;
  size_t num_experts, experts_per_token, expert_intermediate;
  size_t dense_intermediate;
} xabe_ffn_config;
typedef struct xabe_ffn_layer_weights {
  int kind; /* xabe_ffn_kind: which of the two members below is filled in */
  xabe_moe_layer_weights moe;
  xabe_dense_ffn_layer_weights dense;
} xabe_ffn_layer_weights;
typedef struct xabe_ffn_block xabe_ffn_block;
/* FfnBlock::geometry_for (ffn.rs:92-104): dense = one expert, top-1, at the MLP's intermediate width. */
int xabe_ffn_block_geometry_for(const xabe_ffn_config* config, size_t block_size, size_t max_tokens, xabe_moe_geometry* out);
/* FfnBlock::new (ffn.rs:107-127) */
int xabe_ffn_block_new(const xabe_ffn_config* config, const xabe_moe_geometry* geometry, float eps, void* stream,
                       xabe_ffn_block** out);
void xabe_ffn_block_free(xabe_ffn_block* blk);
int xabe_ffn_block_kind(const xabe_ffn_block* blk);
int xabe_ffn_block_disable_tensor_cores(xabe_ffn_block* blk);            /* ffn.rs:130-135 */
int xabe_ffn_block_tensor_cores_enabled(const xabe_ffn_block* blk);      /* ffn.rs:138-143 */
int xabe_ffn_block_set_exact_decode_regime(xabe_ffn_block* blk, int on); /* ffn.rs:148-152: a no-op on the dense block */
int xabe_ffn_block_geometry(const xabe_ffn_block* blk, xabe_moe_geometry* out); /* ffn.rs:155-160 */
const float* xabe_ffn_block_normed(const xabe_ffn_block* blk, size_t* len);     /* ffn.rs:163-168 */
xabe_moe_block* xabe_ffn_block_as_moe(const xabe_ffn_block* blk);               /* ffn.rs:173-178: NULL on the dense path */
int xabe_ffn_block_publish_tokens(xabe_ffn_block* blk, void* stream, size_t tokens); /* ffn.rs:182-191 */
/* FfnBlock::forward (ffn.rs:199-212): XABE_ERR_FFN_KIND_MISMATCH, nothing launched, when block and weights differ in kind. */
int xabe_ffn_block_forward(xabe_ffn_block* blk, void* stream, const xabe_ffn_layer_weights* w, const float* residual,
                           size_t residual_len, size_t tokens, float* ffn_out, size_t ffn_out_len, float* l_out,
                           size_t l_out_len);

/* ---- synthetic stacks for benches (the role of crates/xabe-cuda/src/bin/bench_moe.rs:140-334) ----
 * Fills device memory with seeded values: element i belongs to chunk i/256, chunk c draws from
 * xorshift64*(splitmix64(seed + c*0x9E3779B97F4A7C15)); each value is sigma times an Irwin-Hall(12)
 * normal approximation computed in integer arithmetic; quantized with the reference's own amax
 * quantizers (crates/xabe-kernels/src/quant.rs:75-88, :495-567). */
int xabe_synth_normal_f32(void* stream, uint64_t seed, size_t n, float sigma, float* out);
int xabe_synth_quant(void* stream, int quant, uint64_t seed, size_t n_elements, float sigma, void* out, size_t out_len);

/* ---- what the part reaches, measured as the reference measures its card (no counterpart among the
 * reference's library calls; crates/xabe-cuda/src/bin/bench_dense_ffn.rs:88-111 does the read in its bench,
 * docs/BENCHMARKS.md:1022-1024 the matrix-instruction loop).  One launch per call; the caller times it. ----
 * xabe_calibrate_hbm_read: every 16-byte piece of `buffer` read once, coalesced.
 * xabe_calibrate_mfma_f16: a register-resident loop of 32x32x16 fp16 matrix instructions on every SIMD;
 *   `out` needs 512 floats per CU; `*flops` receives the floating-point operations of the launch. */
int xabe_calibrate_hbm_read(void* stream, const void* buffer, size_t bytes, void* sink);
int xabe_calibrate_mfma_f16(void* stream, float* out, size_t out_len, int iters, double* flops);

#ifdef __cplusplus
}
#endif
#endif /* XABE_HIP_H */

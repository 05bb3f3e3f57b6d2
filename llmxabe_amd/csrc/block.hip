// Block sequencing: the host-side mirror of `MoeBlock::forward`
// (crates/xabe-engine/src/block/moe.rs:1091-1329) and `DenseFfnBlock::forward`
// (crates/xabe-engine/src/block/dense_ffn.rs:1047-1178), over the C ABI above it.
#include <string.h>

#include "host_common.h"

using namespace xabe;

struct xabe_moe_block {
  xabe_moe_kernels* moe;
  xabe_moe_buffers* buffers;
  xabe_moe_geometry g;
  float eps;
  float *normed, *logits, *routed, *shexp, *gate;
  size_t n_act, n_logits;
  int fused_decode;  // decode widths: the regrouped three-launch block where the shape allows
  // matrix-core widths: the shared expert runs beside the router, the routing and the dispatch tables, on a stream
  // of the block's own that forks from the caller's after the RMSNorm and joins it before the combine
  hipStream_t side;
  hipEvent_t forked, joined;
};

static int block_alloc(float** p, size_t n, hipStream_t s) {
  XABE_HIP_TRY(hipMalloc(reinterpret_cast<void**>(p), n * sizeof(float)));
  XABE_HIP_TRY(hipMemsetAsync(*p, 0, n * sizeof(float), s));
  return XABE_OK;
}

// (default priority, like every stream this library makes)
static int block_side_stream(xabe_moe_block* blk) {
  XABE_HIP_TRY(hipStreamCreateWithFlags(&blk->side, hipStreamNonBlocking));
  XABE_HIP_TRY(hipEventCreateWithFlags(&blk->forked, hipEventDisableTiming));
  XABE_HIP_TRY(hipEventCreateWithFlags(&blk->joined, hipEventDisableTiming));
  return XABE_OK;
}

int xabe_moe_block_new(const xabe_moe_geometry* geometry, float eps, void* stream, xabe_moe_block** out) {
  if (!geometry || !out) return set_error(XABE_ERR_INVALID_ARGUMENT, "MoeBlock::new: null pointer");
  xabe_moe_block* blk = new xabe_moe_block();
  memset(blk, 0, sizeof(*blk));
  blk->g = *geometry;
  blk->eps = eps;
  blk->fused_decode = 1;
  int st = xabe_moe_kernels_new(geometry, &blk->moe);
  if (st == XABE_OK) st = xabe_moe_buffers_new(blk->moe, stream, &blk->buffers);
  blk->n_act = geometry->max_tokens * geometry->hidden;
  blk->n_logits = geometry->max_tokens * geometry->num_experts;
  hipStream_t s = as_stream(stream);
  if (st == XABE_OK) st = block_alloc(&blk->normed, blk->n_act, s);
  if (st == XABE_OK) st = block_alloc(&blk->logits, blk->n_logits, s);
  if (st == XABE_OK) st = block_alloc(&blk->routed, blk->n_act, s);
  if (st == XABE_OK) st = block_alloc(&blk->shexp, blk->n_act, s);
  if (st == XABE_OK) st = block_alloc(&blk->gate, geometry->max_tokens, s);
  if (st == XABE_OK && geometry->max_tokens >= kMfmaMinTokens) st = block_side_stream(blk);
  if (st != XABE_OK) {
    xabe_moe_block_free(blk);
    return st;
  }
  *out = blk;
  return XABE_OK;
}

void xabe_moe_block_free(xabe_moe_block* blk) {
  if (!blk) return;
  float* ptrs[] = {blk->normed, blk->logits, blk->routed, blk->shexp, blk->gate};
  for (float* p : ptrs)
    if (p) (void)hipFree(p);
  if (blk->forked) (void)hipEventDestroy(blk->forked);
  if (blk->joined) (void)hipEventDestroy(blk->joined);
  if (blk->side) (void)hipStreamDestroy(blk->side);
  xabe_moe_buffers_free(blk->buffers);
  xabe_moe_kernels_free(blk->moe);
  delete blk;
}

int xabe_moe_block_publish_tokens(xabe_moe_block* blk, void* stream, size_t tokens) {
  if (!blk) return set_error(XABE_ERR_INVALID_ARGUMENT, "publish_tokens: null handle");
  return xabe_moe_set_valid_tokens(blk->moe, stream, blk->buffers, tokens);
}

static int blk_check_len(const char* what, size_t expected, size_t found) {
  if (expected != found) return set_error(XABE_ERR_BUFFER_LENGTH, "%s holds %zu elements, expected %zu", what, found, expected);
  return XABE_OK;
}

int xabe_moe_block_forward_stage(xabe_moe_block* blk, void* stream, const xabe_moe_layer_weights* w, const float* residual,
                                 size_t residual_len, const float* logit_bias, float* ffn_out, size_t ffn_out_len,
                                 float* l_out, size_t l_out_len, int stage) {
  if (!blk || !w || !residual || !ffn_out || !l_out) return set_error(XABE_ERR_INVALID_ARGUMENT, "forward_stage: null pointer");
  if (stage < 0 || stage > 2) return set_error(XABE_ERR_INVALID_ARGUMENT, "forward_stage: stage %d is not 0, 1 or 2", stage);
  XABE_TRY(blk_check_len("residual", blk->n_act, residual_len));
  XABE_TRY(blk_check_len("ffn_out", blk->n_act, ffn_out_len));
  XABE_TRY(blk_check_len("l_out", blk->n_act, l_out_len));
  if (!decode_block_supported(blk->moe, blk->buffers, w))
    return set_error(XABE_ERR_UNSUPPORTED_GEOMETRY, "forward_stage: this geometry does not take the three-launch decode path");
  XABE_TRY(check_layer_stacks(blk->moe, w));
  return launch_decode_block(blk->moe, as_stream(stream), blk->buffers, w, residual, logit_bias, blk->eps, blk->normed,
                             blk->logits, blk->shexp, blk->gate, blk->routed, ffn_out, l_out, 1u << stage);
}

// step 2 of the forward below: router logits, (bias,) softmax + top-k + renormalise, dispatch tables
static int route_rows(xabe_moe_block* blk, void* stream, const xabe_moe_layer_weights* w, const float* logit_bias) {
  const xabe_moe_geometry& g = blk->g;
  if (!(w->router_quant < 0 || w->router_quant == XABE_QUANT_Q8_0))
    return set_error(XABE_ERR_UNSUPPORTED_QUANT, "router: only f32 and Q8_0 routers are supported, got code %d", w->router_quant);
  const size_t router_len = w->router_quant < 0
                                ? g.num_experts * g.hidden
                                : g.num_experts * g.hidden / xabe_expert_quant_block_elements(w->router_quant) *
                                      xabe_expert_quant_block_bytes(w->router_quant);
  bool bias_added = false, planes = false;
  XABE_TRY(router_logits_biased(blk->moe, stream, blk->buffers, w->router, router_len, w->router_quant, blk->normed,
                                blk->n_act, blk->logits, blk->n_logits, logit_bias, &bias_added, &planes));
  // (a split router GEMM leaves partial planes: the routing launch adds them, and the bias, as it reads them)
  if (planes) return route_planes_and_dispatch(blk->moe, stream, blk->buffers, blk->logits, blk->n_logits, logit_bias);
  if (logit_bias && !bias_added) XABE_TRY(xabe_moe_add_logit_bias(blk->moe, stream, blk->buffers, logit_bias, blk->logits));
  return xabe_moe_route_and_dispatch(blk->moe, stream, blk->buffers, blk->logits, blk->n_logits);
}

int xabe_moe_block_forward(xabe_moe_block* blk, void* stream, const xabe_moe_layer_weights* w, const float* residual,
                           size_t residual_len, size_t tokens, const float* logit_bias, float* ffn_out,
                           size_t ffn_out_len, float* l_out, size_t l_out_len) {
  if (!ffn_out) return set_error(XABE_ERR_INVALID_ARGUMENT, "MoeBlock::forward: null pointer");
  return xabe_moe_block_forward_seam(blk, stream, w, residual, residual_len, tokens, logit_bias, ffn_out, ffn_out_len, l_out,
                                     l_out_len, nullptr);
}

float* xabe_moe_block_normed_mut(xabe_moe_block* blk, size_t* len) {
  if (len) *len = blk ? blk->n_act : 0;
  return blk ? blk->normed : nullptr;
}
void* xabe_moe_block_normed_h_mut(xabe_moe_block* blk, size_t* len) {
  void* p = blk && blk->buffers ? blk->buffers->x_h : nullptr;
  if (len) *len = p ? blk->n_act : 0;
  return p;
}

int xabe_moe_block_forward_seam(xabe_moe_block* blk, void* stream, const xabe_moe_layer_weights* w, const float* residual,
                                size_t residual_len, size_t tokens, const float* logit_bias, float* ffn_out,
                                size_t ffn_out_len, float* l_out, size_t l_out_len, const xabe_moe_seam* seam) {
  if (!blk || !w || !residual || !l_out || (!ffn_out && !seam))
    return set_error(XABE_ERR_INVALID_ARGUMENT, "MoeBlock::forward: null pointer");
  const xabe_moe_geometry& g = blk->g;
  if (tokens > g.max_tokens)
    return set_error(XABE_ERR_TOO_MANY_TOKENS, "%zu tokens exceeds the %zu the block was sized for", tokens, g.max_tokens);
  XABE_TRY(blk_check_len("residual", blk->n_act, residual_len));
  if (ffn_out) XABE_TRY(blk_check_len("ffn_out", blk->n_act, ffn_out_len));
  XABE_TRY(blk_check_len("l_out", blk->n_act, l_out_len));
  const bool pre = seam && seam->input_normed;
  const bool tail = seam && seam->next_norm_weight;
  if (tail) {
    if (!seam->next_normed) return set_error(XABE_ERR_INVALID_ARGUMENT, "MoeBlock::forward: a seam with a norm weight but no next_normed");
    XABE_TRY(blk_check_len("next_normed", blk->n_act, seam->next_normed_len));
    if (seam->next_normed_h) XABE_TRY(blk_check_len("next_normed_h", blk->n_act, seam->next_normed_h_len));
  }
  XABE_TRY(xabe_moe_block_publish_tokens(blk, stream, tokens));

  // decode widths, model shapes: the eight steps below regrouped into three launches, same arithmetic
  if (blk->fused_decode && !blk->moe->exact_regime && decode_block_supported(blk->moe, blk->buffers, w)) {
    XABE_TRY(check_layer_stacks(blk->moe, w));  // (the checks the step-by-step sequence below makes call by call)
    DecodeSeam ds = {pre, tail ? seam->next_norm_weight : nullptr, tail ? seam->next_eps : 0.0f, tail ? seam->next_normed : nullptr,
                     tail ? seam->next_normed_h : nullptr};
    return launch_decode_block(blk->moe, as_stream(stream), blk->buffers, w, residual, logit_bias, blk->eps, blk->normed,
                               blk->logits, blk->shexp, blk->gate, blk->routed, ffn_out, l_out, 7u, seam ? &ds : nullptr);
  }

  const bool wide = g.max_tokens >= kMfmaMinTokens && xabe_moe_kernels_tensor_cores_enabled(blk->moe);
  // 1. post-mixer RMSNorm over every row of the buffer; at matrix-core widths the same launch writes the fp16 copy
  //    of the rows that the routed and the shared expert kernels read.  With the seam's consumer half on, the previous
  //    block's tail has left both already.
  bool normed_h = pre && wide && blk->buffers->x_h;
  if (!pre) {
    if (wide && blk->buffers->x_h)
      XABE_TRY(rms_norm_rows_with_f16(stream, residual, w->post_norm, blk->normed, blk->buffers->x_h, g.max_tokens, g.hidden,
                                      blk->eps, &normed_h));
    if (!normed_h)
      XABE_TRY(xabe_rms_norm(stream, residual, blk->n_act, w->post_norm, g.hidden, blk->normed, blk->n_act, g.max_tokens,
                             g.hidden, blk->eps));
  }
  const bool shared_mma =
      wide && mfma_supported(blk->moe, blk->buffers, w->shared_gate.quant, w->shared_up.quant, w->shared_down.quant, false);
  if (shared_mma && blk->side) {
    // Matrix-core widths: the shared expert needs the rows only, so it forks off here and runs beside steps 2 and 3,
    // whose first launches (router, routing, dispatch tables, tile lists) leave most of the device idle.
    hipStream_t s = as_stream(stream);
    if (!normed_h) XABE_TRY(mfma_convert_activations(blk->moe, s, blk->buffers, blk->normed));
    XABE_HIP_TRY(hipEventRecord(blk->forked, s));
    XABE_HIP_TRY(hipStreamWaitEvent(blk->side, blk->forked, 0));
    blk->buffers->x_h_ready = true;  // both expert paths read the fp16 copy of the rows made above
    int st = xabe_moe_shared_expert_mma(blk->moe, blk->side, blk->buffers, w->shared_gate, w->shared_up, w->shared_down,
                                        blk->normed, blk->n_act, blk->shexp, blk->n_act);
    hipError_t he = hipEventRecord(blk->joined, blk->side);
    if (st == XABE_OK) st = route_rows(blk, stream, w, logit_bias);
    if (st == XABE_OK)
      st = xabe_moe_grouped_forward_partial(blk->moe, stream, blk->buffers, w->gate_exps, w->up_exps, w->down_exps, blk->normed,
                                            blk->n_act);
    blk->buffers->x_h_ready = false;
    // (whatever happened above, the caller's stream takes the side stream back)
    if (he == hipSuccess) he = hipStreamWaitEvent(s, blk->joined, 0);
    if (st != XABE_OK) return st;
    XABE_HIP_TRY(he);
  } else {
    XABE_TRY(route_rows(blk, stream, w, logit_bias));
    // 3 + 4. routed experts (stopping at `partial`) and the ungated shared expert
    int fused = 0;
    if (!wide)
      XABE_TRY(xabe_moe_grouped_forward_partial_with_shared(blk->moe, stream, blk->buffers, w->gate_exps, w->up_exps,
                                                            w->down_exps, w->shared_gate, w->shared_up, w->shared_down,
                                                            blk->normed, blk->n_act, blk->shexp, blk->n_act, &fused));
    if (!fused) {
      // the routed and the shared matrix-core paths read the same fp16 copy of the rows: made once here
      if (normed_h) {
        blk->buffers->x_h_ready = true;
      } else if (shared_mma) {
        XABE_TRY(mfma_convert_activations(blk->moe, as_stream(stream), blk->buffers, blk->normed));
        blk->buffers->x_h_ready = true;
      }
      int st = xabe_moe_grouped_forward_partial(blk->moe, stream, blk->buffers, w->gate_exps, w->up_exps, w->down_exps,
                                                blk->normed, blk->n_act);
      if (st == XABE_OK && shared_mma)
        st = xabe_moe_shared_expert_mma(blk->moe, stream, blk->buffers, w->shared_gate, w->shared_up, w->shared_down,
                                        blk->normed, blk->n_act, blk->shexp, blk->n_act);
      else if (st == XABE_OK)
        st = xabe_moe_shared_expert(blk->moe, stream, blk->buffers, w->shared_gate, w->shared_up, w->shared_down,
                                    blk->normed, blk->n_act, blk->shexp, blk->n_act);
      blk->buffers->x_h_ready = false;
      if (st != XABE_OK) return st;
    }
  }
  // 5. routed sum, sigmoid gate, combine, residual (and, across a seam, the next layer's RMSNorm in the same launch)
  if (!seam)
    return xabe_moe_gate_and_combine(blk->moe, stream, blk->buffers, w->shared_gate_inp, blk->normed, blk->shexp, residual,
                                     blk->gate, blk->routed, ffn_out, l_out);
  float* routed = seam->skip_readback ? nullptr : blk->routed;
  if (g.hidden <= 2048)
    return xabe_moe_gate_and_combine_seam(blk->moe, stream, blk->buffers, w->shared_gate_inp, blk->normed, blk->shexp, residual,
                                          blk->gate, routed, ffn_out, l_out, tail ? seam->next_norm_weight : nullptr,
                                          tail ? seam->next_eps : 0.0f, tail ? seam->next_normed : nullptr,
                                          tail ? seam->next_normed_h : nullptr);
  // longer rows: the plain combine (which writes every tensor) and the RMSNorm as a launch of its own: the same values
  if (!ffn_out) return set_error(XABE_ERR_INVALID_ARGUMENT, "MoeBlock::forward: rows of %zu elements take the plain combine, which needs an ffn_out", g.hidden);
  XABE_TRY(xabe_moe_gate_and_combine(blk->moe, stream, blk->buffers, w->shared_gate_inp, blk->normed, blk->shexp, residual,
                                     blk->gate, blk->routed, ffn_out, l_out));
  if (!tail) return XABE_OK;
  bool with_h = false;
  if (seam->next_normed_h)
    XABE_TRY(rms_norm_rows_with_f16(stream, l_out, seam->next_norm_weight, seam->next_normed, seam->next_normed_h, g.max_tokens,
                                    g.hidden, seam->next_eps, &with_h));
  if (!with_h)
    XABE_TRY(xabe_rms_norm(stream, l_out, blk->n_act, seam->next_norm_weight, g.hidden, seam->next_normed, blk->n_act,
                           g.max_tokens, g.hidden, seam->next_eps));
  return XABE_OK;
}

int xabe_moe_block_disable_tensor_cores(xabe_moe_block* blk) {
  if (!blk) return set_error(XABE_ERR_INVALID_ARGUMENT, "disable_tensor_cores: null handle");
  return xabe_moe_kernels_disable_tensor_cores(blk->moe);
}
int xabe_moe_block_set_exact_decode_regime(xabe_moe_block* blk, int on) {
  if (!blk) return set_error(XABE_ERR_INVALID_ARGUMENT, "set_exact_decode_regime: null handle");
  return xabe_moe_kernels_set_exact_decode_regime(blk->moe, on);
}
int xabe_moe_block_set_mfma_form(xabe_moe_block* blk, int form) {
  if (!blk) return set_error(XABE_ERR_INVALID_ARGUMENT, "set_mfma_form: null handle");
  return xabe_moe_kernels_set_mfma_form(blk->moe, form);
}
int xabe_moe_block_set_fused_decode(xabe_moe_block* blk, int on) {
  if (!blk) return set_error(XABE_ERR_INVALID_ARGUMENT, "set_fused_decode: null handle");
  blk->fused_decode = on != 0;
  return XABE_OK;
}
int xabe_moe_block_tensor_cores_enabled(const xabe_moe_block* blk) {
  return blk ? xabe_moe_kernels_tensor_cores_enabled(blk->moe) : 0;
}

#define XABE_BLOCK_ACCESSOR(name, field, count)                                   \
  const float* xabe_moe_block_##name(const xabe_moe_block* blk, size_t* len) {    \
    if (!blk) { if (len) *len = 0; return nullptr; }                              \
    if (len) *len = (count);                                                      \
    return blk->field;                                                            \
  }
XABE_BLOCK_ACCESSOR(normed, normed, blk->n_act)
XABE_BLOCK_ACCESSOR(router_logits, logits, blk->n_logits)
XABE_BLOCK_ACCESSOR(routed, routed, blk->n_act)
XABE_BLOCK_ACCESSOR(shared_ungated, shexp, blk->n_act)
XABE_BLOCK_ACCESSOR(shared_gate, gate, blk->g.max_tokens)
xabe_moe_buffers* xabe_moe_block_buffers(const xabe_moe_block* blk) { return blk ? blk->buffers : nullptr; }
xabe_moe_kernels* xabe_moe_block_kernels(const xabe_moe_block* blk) { return blk ? blk->moe : nullptr; }

// ------------------------------------------------------------------ dense sibling
struct xabe_dense_ffn_block {
  xabe_moe_kernels* moe;
  xabe_moe_buffers* buffers;
  xabe_moe_geometry g;
  float eps;
  float* normed;
  size_t n_act;
};

int xabe_dense_ffn_block_new(size_t hidden, size_t intermediate, size_t max_tokens, float eps, void* stream,
                             xabe_dense_ffn_block** out) {
  if (!out) return set_error(XABE_ERR_INVALID_ARGUMENT, "DenseFfnBlock::new: null pointer");
  // DenseFfnBlock::geometry_for: one "expert", no routing (dense_ffn.rs)
  xabe_moe_geometry g = {1, 1, hidden, intermediate, xabe_moe_block_size_for(max_tokens), max_tokens};
  xabe_dense_ffn_block* blk = new xabe_dense_ffn_block();
  memset(blk, 0, sizeof(*blk));
  blk->g = g;
  blk->eps = eps;
  blk->n_act = max_tokens * hidden;
  int st = xabe_moe_kernels_new(&g, &blk->moe);
  if (st == XABE_OK) st = xabe_moe_shared_only_buffers_new(blk->moe, stream, 1, &blk->buffers);
  if (st == XABE_OK) st = block_alloc(&blk->normed, blk->n_act, as_stream(stream));
  if (st != XABE_OK) {
    xabe_dense_ffn_block_free(blk);
    return st;
  }
  *out = blk;
  return XABE_OK;
}

void xabe_dense_ffn_block_free(xabe_dense_ffn_block* blk) {
  if (!blk) return;
  if (blk->normed) (void)hipFree(blk->normed);
  xabe_moe_buffers_free(blk->buffers);
  xabe_moe_kernels_free(blk->moe);
  delete blk;
}

int xabe_dense_ffn_block_disable_tensor_cores(xabe_dense_ffn_block* blk) {
  if (!blk) return set_error(XABE_ERR_INVALID_ARGUMENT, "disable_tensor_cores: null handle");
  return xabe_moe_kernels_disable_tensor_cores(blk->moe);
}

const float* xabe_dense_ffn_block_normed(const xabe_dense_ffn_block* blk, size_t* len) {
  if (!blk) { if (len) *len = 0; return nullptr; }
  if (len) *len = blk->n_act;
  return blk->normed;
}

int xabe_dense_ffn_block_forward(xabe_dense_ffn_block* blk, void* stream, const xabe_dense_ffn_layer_weights* w,
                                 const float* residual, size_t residual_len, size_t tokens, float* ffn_out,
                                 size_t ffn_out_len, float* l_out, size_t l_out_len) {
  if (!blk || !w || !residual || !ffn_out || !l_out)
    return set_error(XABE_ERR_INVALID_ARGUMENT, "DenseFfnBlock::forward: null pointer");
  const xabe_moe_geometry& g = blk->g;
  if (tokens > g.max_tokens)
    return set_error(XABE_ERR_TOO_MANY_TOKENS, "%zu tokens exceeds the %zu the block was sized for", tokens, g.max_tokens);
  XABE_TRY(blk_check_len("residual", blk->n_act, residual_len));
  XABE_TRY(blk_check_len("ffn_out", blk->n_act, ffn_out_len));
  XABE_TRY(blk_check_len("l_out", blk->n_act, l_out_len));
  XABE_TRY(xabe_moe_set_valid_tokens(blk->moe, stream, blk->buffers, tokens));
  const bool wide = g.max_tokens >= kMfmaMinTokens && xabe_moe_kernels_tensor_cores_enabled(blk->moe) &&
                    mfma_supported(blk->moe, blk->buffers, w->gate.quant, w->up.quant, w->down.quant, false);
  // fp32 widths: norm folded into gate/up, residual into down (same values, two launches instead of four)
  if (!wide && w->post_norm) {
    bool launched = false;
    XABE_TRY(dense_fp32_fused(blk->moe, as_stream(stream), blk->buffers, w->gate, w->up, w->down, w->post_norm, blk->eps,
                              residual, blk->normed, ffn_out, l_out, &launched));
    if (launched) return XABE_OK;
  }
  XABE_TRY(xabe_rms_norm(stream, residual, blk->n_act, w->post_norm, g.hidden, blk->normed, blk->n_act, g.max_tokens,
                         g.hidden, blk->eps));
  if (wide)
    XABE_TRY(xabe_moe_shared_expert_mma(blk->moe, stream, blk->buffers, w->gate, w->up, w->down, blk->normed, blk->n_act,
                                        ffn_out, blk->n_act));
  else
    XABE_TRY(xabe_moe_shared_expert(blk->moe, stream, blk->buffers, w->gate, w->up, w->down, blk->normed, blk->n_act,
                                    ffn_out, blk->n_act));
  return xabe_dense_ffn_add_residual(blk->moe, stream, blk->buffers, ffn_out, residual, l_out);
}

int xabe_dense_ffn_block_publish_tokens(xabe_dense_ffn_block* blk, void* stream, size_t tokens) {
  if (!blk) return set_error(XABE_ERR_INVALID_ARGUMENT, "publish_tokens: null handle");
  return xabe_moe_set_valid_tokens(blk->moe, stream, blk->buffers, tokens);
}
int xabe_dense_ffn_block_tensor_cores_enabled(const xabe_dense_ffn_block* blk) {
  return blk ? xabe_moe_kernels_tensor_cores_enabled(blk->moe) : 0;
}

// ------------------------------------------------------------------ FfnBlock
// The two-variant dispatch of crates/xabe-engine/src/block/ffn.rs:27-228: one handle that is either block,
// one weights value that is either layer kind, and a pairing that is checked rather than assumed.
struct xabe_ffn_block {
  int kind;
  xabe_moe_block* moe;
  xabe_dense_ffn_block* dense;
};

static const char* ffn_kind_name(int kind) { return kind == XABE_FFN_MOE ? "moe" : kind == XABE_FFN_DENSE ? "dense" : "unknown"; }

int xabe_ffn_block_geometry_for(const xabe_ffn_config* config, size_t block_size, size_t max_tokens, xabe_moe_geometry* out) {
  if (!config || !out) return set_error(XABE_ERR_INVALID_ARGUMENT, "FfnBlock::geometry_for: null pointer");
  if (config->kind == XABE_FFN_MOE) {  // MoeBlock::geometry_for (block/moe.rs:931-945)
    *out = {config->num_experts, config->experts_per_token, config->hidden, config->expert_intermediate, block_size, max_tokens};
    return XABE_OK;
  }
  if (config->kind == XABE_FFN_DENSE) {  // DenseFfnBlock::geometry_for (block/dense_ffn.rs:836-850)
    *out = {1, 1, config->hidden, config->dense_intermediate, block_size, max_tokens};
    return XABE_OK;
  }
  return set_error(XABE_ERR_INVALID_ARGUMENT, "FfnBlock::geometry_for: unknown feed-forward kind %d", config->kind);
}

int xabe_ffn_block_new(const xabe_ffn_config* config, const xabe_moe_geometry* geometry, float eps, void* stream,
                       xabe_ffn_block** out) {
  if (!config || !geometry || !out) return set_error(XABE_ERR_INVALID_ARGUMENT, "FfnBlock::new: null pointer");
  if (config->kind != XABE_FFN_MOE && config->kind != XABE_FFN_DENSE)
    return set_error(XABE_ERR_INVALID_ARGUMENT, "FfnBlock::new: unknown feed-forward kind %d", config->kind);
  xabe_ffn_block* blk = new xabe_ffn_block();
  blk->kind = config->kind;
  blk->moe = nullptr;
  blk->dense = nullptr;
  const int st = config->kind == XABE_FFN_MOE
                     ? xabe_moe_block_new(geometry, eps, stream, &blk->moe)
                     : xabe_dense_ffn_block_new(geometry->hidden, geometry->intermediate, geometry->max_tokens, eps, stream,
                                                &blk->dense);
  if (st != XABE_OK) {
    delete blk;
    return st;
  }
  *out = blk;
  return XABE_OK;
}

void xabe_ffn_block_free(xabe_ffn_block* blk) {
  if (!blk) return;
  xabe_moe_block_free(blk->moe);
  xabe_dense_ffn_block_free(blk->dense);
  delete blk;
}

int xabe_ffn_block_kind(const xabe_ffn_block* blk) { return blk ? blk->kind : -1; }

int xabe_ffn_block_disable_tensor_cores(xabe_ffn_block* blk) {
  if (!blk) return set_error(XABE_ERR_INVALID_ARGUMENT, "disable_tensor_cores: null handle");
  return blk->kind == XABE_FFN_MOE ? xabe_moe_block_disable_tensor_cores(blk->moe)
                                   : xabe_dense_ffn_block_disable_tensor_cores(blk->dense);
}
int xabe_ffn_block_tensor_cores_enabled(const xabe_ffn_block* blk) {
  if (!blk) return 0;
  return blk->kind == XABE_FFN_MOE ? xabe_moe_block_tensor_cores_enabled(blk->moe)
                                   : xabe_dense_ffn_block_tensor_cores_enabled(blk->dense);
}
int xabe_ffn_block_set_exact_decode_regime(xabe_ffn_block* blk, int on) {
  if (!blk) return set_error(XABE_ERR_INVALID_ARGUMENT, "set_exact_decode_regime: null handle");
  // the dense block has no routed kernels and so no regime to pin (block/ffn.rs:146-153)
  return blk->kind == XABE_FFN_MOE ? xabe_moe_block_set_exact_decode_regime(blk->moe, on) : XABE_OK;
}
int xabe_ffn_block_geometry(const xabe_ffn_block* blk, xabe_moe_geometry* out) {
  if (!blk || !out) return set_error(XABE_ERR_INVALID_ARGUMENT, "geometry: null pointer");
  *out = blk->kind == XABE_FFN_MOE ? blk->moe->g : blk->dense->g;
  return XABE_OK;
}
const float* xabe_ffn_block_normed(const xabe_ffn_block* blk, size_t* len) {
  if (!blk) { if (len) *len = 0; return nullptr; }
  return blk->kind == XABE_FFN_MOE ? xabe_moe_block_normed(blk->moe, len) : xabe_dense_ffn_block_normed(blk->dense, len);
}
xabe_moe_block* xabe_ffn_block_as_moe(const xabe_ffn_block* blk) { return blk ? blk->moe : nullptr; }

int xabe_ffn_block_publish_tokens(xabe_ffn_block* blk, void* stream, size_t tokens) {
  if (!blk) return set_error(XABE_ERR_INVALID_ARGUMENT, "publish_tokens: null handle");
  return blk->kind == XABE_FFN_MOE ? xabe_moe_block_publish_tokens(blk->moe, stream, tokens)
                                   : xabe_dense_ffn_block_publish_tokens(blk->dense, stream, tokens);
}

int xabe_ffn_block_forward(xabe_ffn_block* blk, void* stream, const xabe_ffn_layer_weights* w, const float* residual,
                           size_t residual_len, size_t tokens, float* ffn_out, size_t ffn_out_len, float* l_out,
                           size_t l_out_len) {
  if (!blk || !w) return set_error(XABE_ERR_INVALID_ARGUMENT, "FfnBlock::forward: null pointer");
  if (blk->kind != w->kind)  // checked before anything is launched (block/ffn.rs:205-208)
    return set_error(XABE_ERR_FFN_KIND_MISMATCH, "a `%s` feed-forward block was handed `%s` weights", ffn_kind_name(blk->kind),
                     ffn_kind_name(w->kind));
  if (blk->kind == XABE_FFN_MOE)
    return xabe_moe_block_forward(blk->moe, stream, &w->moe, residual, residual_len, tokens, nullptr, ffn_out, ffn_out_len,
                                  l_out, l_out_len);
  return xabe_dense_ffn_block_forward(blk->dense, stream, &w->dense, residual, residual_len, tokens, ffn_out, ffn_out_len,
                                      l_out, l_out_len);
}

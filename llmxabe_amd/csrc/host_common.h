// Host-side state shared by the C-ABI translation units.
#pragma once

#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stddef.h>
#include <stdint.h>

#include <string>

#include "../../include/xabe_hip.h"

namespace xabe {

// Widths at which the regimes change hands.
//   <= kFlatMaxTokens: flat per-pair kernels, no dispatch table
//      (MOE_NARROW_DECODE_MAX, crates/xabe-cuda/src/kernels/moe.rs:213-229).
//   >= kMfmaMinTokens: matrix-core grouped GEMM.  The reference switches its int8 path in at 8
//      tokens (MMA_MIN_TOKENS); here the fp32 regime is kept through 63 so that every decode
//      batch up to 32 sequences stays bit-identical to single-stream decode.
constexpr size_t kFlatMaxTokens = 4;
constexpr size_t kMfmaMinTokens = 64;
constexpr size_t kRouteMaxExperts = 512;  // the routing wavefront holds 8 experts per lane

int set_error(int status, const char* fmt, ...);
int hip_error(hipError_t e, const char* what);
std::string geometry_debug(const xabe_moe_geometry& g);
int validate_geometry(const xabe_moe_geometry& g);  // MoeKernels::new's checks (api.hip)

#define XABE_HIP_TRY(expr)                                  \
  do {                                                      \
    hipError_t _e = (expr);                                 \
    if (_e != hipSuccess) return ::xabe::hip_error(_e, #expr); \
  } while (0)

#define XABE_TRY(expr)            \
  do {                            \
    int _s = (expr);              \
    if (_s != XABE_OK) return _s; \
  } while (0)

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }
// id of the capture `s` is recording into, 0 when it is not capturing.  A query the runtime refuses (the legacy
// stream while another stream of the process captures in global mode) is not an error of the caller's: it answers
// kCaptureUnknown, which compares unequal to every capture and to "eager", and clears the runtime's error state.
// Handles are meant for explicit streams.
constexpr unsigned long long kCaptureUnknown = ~0ull;
inline unsigned long long stream_capture_id(hipStream_t s) {
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  unsigned long long cid = 0;
  if (hipStreamGetCaptureInfo(s, &status, &cid) != hipSuccess) {
    (void)hipGetLastError();
    return kCaptureUnknown;
  }
  return status == hipStreamCaptureStatusActive ? cid : 0;
}

}  // namespace xabe

struct xabe_moe_kernels;
struct xabe_moe_buffers;

namespace xabe {
// decode-width fusions (fused.hip).  `quant` < 0 means plain fp32 rows.
int launch_flat_with_shared(const xabe_moe_kernels* k, hipStream_t s, xabe_moe_buffers* b, int nm, int routed_quant,
                            int shared_quant, const void* rw0, const void* rw1, size_t expert_bytes, const float* rx,
                            float* rout, const void* sw0, const void* sw1, const float* sx, float* sout, int K,
                            int n_rows);
// rows per workgroup for a launch with `live_units` busy work units
int pick_tile_rows(const xabe_moe_kernels* k, size_t live_units, int n_rows, int rows_per_step);

// the decode-width block in three launches (decode_block.hip)
bool decode_block_supported(const xabe_moe_kernels* k, const xabe_moe_buffers* b, const xabe_moe_layer_weights* w);
// the checks the step-by-step entry points make on a layer's six stacks (whole blocks, element counts, formats,
// 16-byte-aligned device pointers), for the block-level paths that launch without passing through them (api.hip)
int check_layer_stacks(const xabe_moe_kernels* k, const xabe_moe_layer_weights* w);
// The seam between this block and the next as the decode launches see it: `input_normed`: `normed` holds the pass's
// rows already; `next_normed` (null: the pass ends at l_out): where the third launch's last workgroup per token
// writes rms_norm(l_out, next_w, next_eps), `next_normed_h` (may be null) its fp16 copy.
size_t seam_counter_ints_per_token();  // ints of arrival counters the seam's tail needs per token (decode_block.hip)
struct DecodeSeam {
  bool input_normed;
  const float* next_w;
  float next_eps;
  float* next_normed;
  void* next_normed_h;
};
int launch_decode_block(const xabe_moe_kernels* k, hipStream_t s, xabe_moe_buffers* b, const xabe_moe_layer_weights* w,
                        const float* residual, const float* logit_bias, float eps, float* normed, float* logits,
                        float* shexp, float* gate_out, float* routed, float* ffn_out, float* l_out, unsigned launches = 7u,
                        const DecodeSeam* seam = nullptr);

// matrix-core regime (mfma.hip)
// dense block, fp32 widths, rows longer than one step: norm + gate/up, down + residual (api.hip)
// (`*launched` false and XABE_OK: not applicable, nothing launched)
int dense_fp32_fused(const xabe_moe_kernels* k, hipStream_t s, xabe_moe_buffers* b, xabe_quant_tensor gate,
                     xabe_quant_tensor up, xabe_quant_tensor down, const float* post_norm, float eps,
                     const float* residual, float* normed, float* ffn_out, float* l_out, bool* launched);
// router logits as an fp32 matrix-core GEMM at prefill widths (router_gemm.hip)
// The router GEMM from kRouterGemmMinTokens up (below it the vector kernel), its contraction split over workgroups
// while its 64-token x 128-expert tiles are fewer than four per CU: 8 parts up to 4096 tokens, 4 at 8192, 2 at
// 16384, unsplit beyond.
constexpr size_t kRouterGemmMinTokens = 256;
inline int router_gemm_splits(const xabe_moe_geometry& g) {
  const size_t tiles = (g.num_experts / 128) * ((g.max_tokens + 63) / 64);
  int splits = 1;
  while (splits < 8 && tiles * splits < 1024 && g.hidden % (size_t)(32 * splits * 2) == 0) splits *= 2;
  return splits;
}
bool router_gemm_supported(const xabe_moe_kernels* k, const xabe_moe_buffers* b, int router_quant);
int launch_router_gemm(const xabe_moe_kernels* k, hipStream_t s, const xabe_moe_buffers* b, const void* router,
                       int router_quant, const float* normed, float* logits, const float* bias = nullptr,
                       bool* bias_added = nullptr, bool* sum_deferred = nullptr);
// Router logits with the per-expert bias folded into the launch that finishes them where there is one (the split
// matrix-instruction GEMM's plane sum); `*bias_added` says whether it was (otherwise the caller adds it).
// `sum_deferred` (may be null): where the logits come out as the partial planes of a split contraction, leave them
// so and say so in *sum_deferred; the caller then routes with route_planes_and_dispatch, which adds the planes (and
// the bias) in the same order in the routing launch and writes `logits` there.
int router_logits_biased(const xabe_moe_kernels* k, void* stream, const xabe_moe_buffers* b, const void* router,
                         size_t router_len, int router_quant, const float* normed, size_t normed_len, float* logits,
                         size_t logits_len, const float* bias, bool* bias_added, bool* sum_deferred = nullptr);
int route_planes_and_dispatch(const xabe_moe_kernels* k, void* stream, xabe_moe_buffers* b, float* logits, size_t logits_len,
                              const float* bias);
// RMSNorm of `rows` rows that also writes the fp16 copy the matrix-core kernels read (rows of at most 2048
// elements, at least 64 of them); returns false in *done when the shape is not served.
int rms_norm_rows_with_f16(void* stream, const float* x, const float* weight, float* out, void* out_h, size_t rows,
                           size_t width, float eps, bool* done);
// one-time, at handle creation: LDS limits of the kernels that ask for more than the static 64 KB (mfma.hip, api.hip)
int mfma_configure();
int long_rows_configure();
bool mfma_supported(const xabe_moe_kernels* k, const xabe_moe_buffers* b, int gate_q, int up_q, int down_q, bool routed);
// token-tile heights of the routed down and gate/up launches of the pass as published, and the entries one of the two
// lists in `tile_list` holds; false when these buffers carry no lists
bool mfma_tile_plan(const xabe_moe_kernels* k, const xabe_moe_buffers* b, int* bm, int* bm_up, int* capacity);
int mfma_grouped_forward_partial(const xabe_moe_kernels* k, hipStream_t s, xabe_moe_buffers* b, xabe_quant_tensor gate,
                                 xabe_quant_tensor up, xabe_quant_tensor down, const float* x);
int mfma_shared_expert(const xabe_moe_kernels* k, hipStream_t s, xabe_moe_buffers* b, xabe_quant_tensor gate,
                       xabe_quant_tensor up, xabe_quant_tensor down, const float* x, float* out);
// fp16 copy of the activations both of the above start from; a caller that makes it once sets
// `x_h_ready` on the buffers for the calls that follow and clears it afterwards
int mfma_convert_activations(const xabe_moe_kernels* k, hipStream_t s, xabe_moe_buffers* b, const float* x);

}  // namespace xabe

struct xabe_moe_kernels {
  xabe_moe_geometry g;
  bool tensor_cores;
  bool exact_regime;
  bool force_community;
  int mfma_form;  // matrix-core regime, routed launches: 0 chosen by width, 1 k_mfma_expert, 2 k_mfma_pc (mfma.hip)
  int device;
  int num_cus;
};

struct xabe_moe_buffers {
  int scope;
  bool mma;
  xabe_moe_geometry g;
  // lengths in elements
  size_t n_topk, n_sorted, n_expert_blocks, n_inter, n_partial, n_shared_inter;
  int32_t* topk_ids;
  float* topk_weights;
  int32_t* sorted_token_ids;
  int32_t* expert_ids;
  int32_t* bucket_live;
  int32_t* expert_counts;
  int32_t* align_hist;      // [chunks of 1024 selections][num_experts], prefill widths only
  size_t n_align_chunks;
  int32_t* num_tokens_post_pad;
  int32_t* valid_tokens;
  int32_t valid_published;  // what `valid_tokens` holds (0 after allocation)
  int32_t valid_host;       // source of the host-to-device copy that publishes a new count
  float* inter;         // [slot][intermediate] fp32 (decode regimes)
  float* partial;       // [flat][hidden]
  float* shared_inter;  // [token][intermediate]
  // matrix-core regime staging
  uint16_t* x_h;        // [token][hidden] fp16 activations
  bool x_h_ready;       // the caller has converted this pass's activations already
  uint16_t* inter_h;    // [slot][intermediate] fp16
  uint16_t* shared_inter_h;
  int32_t* tile_list;   // device-built tile schedule
  size_t n_tile_list;
  // tile heights the lists were cut for by the last dispatch build (0: not built there), and the capture that
  // build was recorded into (0: launched eagerly): a forward trusts the lists only inside the same capture, or
  // eagerly after an eager build, so that a captured forward never depends on lists made outside its graph
  int tiles_bm, tiles_bm_up;
  unsigned long long tiles_capture;
  // set for good once a dispatch build on these buffers has been recorded into a capture: a replay of that graph
  // rewrites the device lists without touching the fields above, so from then on only a forward inside a capture
  // that holds its own build trusts them; eager forwards always make their own
  bool tiles_graph_owned;
  int32_t* seam_arrivals;  // decode widths: arrival counters of the seam's tail (zero between passes)
  size_t n_seam_arrivals;
  float* router_partial;  // [split][token][expert]: the router GEMM's contraction splits at mid widths
  size_t n_router_partial;
  size_t bytes;
};

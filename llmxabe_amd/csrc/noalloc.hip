// xabe_moe_block_forward_noalloc: the decode-width MoE block for callers that cannot allocate device memory
// (code under hipGraph capture that builds no handles, tight serving loops, harnesses that forbid hipMalloc).
//
// xabe_moe_block_forward keeps its working set (normalised rows, router logits, selections, the routed and shared
// intermediates, the read-back tensors, the live-token count) in buffers that xabe_moe_block_new allocates.  Here
// the same working set lives in one file-scope device array, carved up at fixed offsets for the largest pass the
// entry point serves, and the three decode launches receive pointers into it exactly as they receive the block's
// buffers: same kernels, same arithmetic, same bits.
//
// The array's name is a host-side stand-in, not a device address: host code resolves the address once per device
// with hipGetSymbolAddress and passes that pointer on.  Each GPU holds its own copy until the process ends.  Every
// call on one GPU shares that GPU's copy, which keeps the last call's contents: two calls that overlap on one GPU
// (different streams, or graphs replayed concurrently) race.  Nothing in it needs to start at zero: the kernels
// write every row they later read for a live token and drop what they compute for rows past the live count.
#include <string.h>

#include <mutex>

#include "host_common.h"

namespace xabe {

// Largest pass served: the three-launch decode block's own limits.
constexpr size_t kNaMaxTokens = 32, kNaMaxHidden = 2048, kNaMaxInter = 512, kNaMaxExperts = 512, kNaMaxTopK = 8;

// Offsets in floats; every region starts on a 256-byte boundary.
constexpr size_t na_align(size_t floats) { return (floats + 63) / 64 * 64; }
constexpr size_t kNaValid = 0;                                                        // int32 live-token count
constexpr size_t kNaGate = kNaValid + 64;                                             // [tokens]
constexpr size_t kNaTopkIds = kNaGate + na_align(kNaMaxTokens);                       // int32 [tokens][top_k]
constexpr size_t kNaTopkW = kNaTopkIds + na_align(kNaMaxTokens * kNaMaxTopK);         // [tokens][top_k]
constexpr size_t kNaLogits = kNaTopkW + na_align(kNaMaxTokens * kNaMaxTopK);          // [tokens][experts]
constexpr size_t kNaSharedInter = kNaLogits + na_align(kNaMaxTokens * kNaMaxExperts); // [tokens][intermediate]
constexpr size_t kNaInter = kNaSharedInter + na_align(kNaMaxTokens * kNaMaxInter);    // [tokens * top_k][intermediate]
constexpr size_t kNaNormed = kNaInter + na_align(kNaMaxTokens * kNaMaxTopK * kNaMaxInter);  // [tokens][hidden]
constexpr size_t kNaRouted = kNaNormed + na_align(kNaMaxTokens * kNaMaxHidden);
constexpr size_t kNaShexp = kNaRouted + na_align(kNaMaxTokens * kNaMaxHidden);
constexpr size_t kNaFloats = kNaShexp + na_align(kNaMaxTokens * kNaMaxHidden);        // 1 458 432 B in all

static __device__ __align__(256) float scratch[kNaFloats];

constexpr int kNaMaxDevices = 64;
static std::mutex g_na_mutex;
static float* g_na_ptr[kNaMaxDevices];  // the array's address on each device, resolved on first use there

// The calling thread's current device and the address of that device's copy of the array.  The address is resolved
// on the first call on a device, and that call must not arrive while `s` is capturing: resolving the symbol may load
// the code object, which a capture in progress does not survive; such a call is refused with nothing recorded.
static int na_scratch(hipStream_t s, float** out) {
  int dev = 0;
  XABE_HIP_TRY(hipGetDevice(&dev));
  if (dev < 0 || dev >= kNaMaxDevices)
    return set_error(XABE_ERR_INVALID_ARGUMENT, "block_forward_noalloc: device ordinal %d is beyond the %d this entry point tracks",
                     dev, kNaMaxDevices);
  std::lock_guard<std::mutex> lock(g_na_mutex);
  if (!g_na_ptr[dev]) {
    if (stream_capture_id(s) != 0)
      return set_error(XABE_ERR_INVALID_ARGUMENT,
                       "block_forward_noalloc: the first call on device %d arrived while the stream is capturing; make one "
                       "call on the device before the capture begins", dev);
    float* p = nullptr;
    XABE_HIP_TRY(hipGetSymbolAddress(reinterpret_cast<void**>(&p), HIP_SYMBOL(scratch)));
    if (!p) return set_error(XABE_ERR_DRIVER, "block_forward_noalloc: the scratch array has no address on device %d", dev);
    g_na_ptr[dev] = p;
  }
  *out = g_na_ptr[dev];
  return XABE_OK;
}

// The live-token count goes to the device as a kernel argument: a fill kernel, not a copy or a memset, so that a
// captured call replays with the value it was captured with.
__global__ void k_na_publish_tokens(int* valid_tokens, int tokens) {
  if (threadIdx.x == 0 && blockIdx.x == 0) *valid_tokens = tokens;
}

}  // namespace xabe

using namespace xabe;

int xabe_moe_block_forward_noalloc(const xabe_moe_geometry* geometry, float eps, void* stream,
                                   const xabe_moe_layer_weights* w, const float* residual, size_t residual_len,
                                   size_t tokens, const float* logit_bias, float* ffn_out, size_t ffn_out_len, float* l_out,
                                   size_t l_out_len) {
  if (!geometry || !w || !residual || !ffn_out || !l_out)
    return set_error(XABE_ERR_INVALID_ARGUMENT, "block_forward_noalloc: null pointer");
  const xabe_moe_geometry g = *geometry;
  XABE_TRY(validate_geometry(g));
  if (g.max_tokens > kNaMaxTokens || g.hidden > kNaMaxHidden || g.intermediate > kNaMaxInter || g.num_experts > kNaMaxExperts ||
      g.experts_per_token > kNaMaxTopK)
    return set_error(XABE_ERR_UNSUPPORTED_GEOMETRY,
                     "unsupported MoE geometry %s: block_forward_noalloc serves at most %zu tokens, hidden %zu, intermediate %zu, "
                     "%zu experts, top-%zu (its scratch array is sized for that); larger passes go through xabe_moe_block_forward",
                     geometry_debug(g).c_str(), kNaMaxTokens, kNaMaxHidden, kNaMaxInter, kNaMaxExperts, kNaMaxTopK);
  if (tokens > g.max_tokens)
    return set_error(XABE_ERR_TOO_MANY_TOKENS, "%zu tokens exceeds the %zu the pass was sized for", tokens, g.max_tokens);
  const size_t n_act = g.max_tokens * g.hidden;
  if (residual_len != n_act) return set_error(XABE_ERR_BUFFER_LENGTH, "residual holds %zu elements, expected %zu", residual_len, n_act);
  if (ffn_out_len != n_act) return set_error(XABE_ERR_BUFFER_LENGTH, "ffn_out holds %zu elements, expected %zu", ffn_out_len, n_act);
  if (l_out_len != n_act) return set_error(XABE_ERR_BUFFER_LENGTH, "l_out holds %zu elements, expected %zu", l_out_len, n_act);

  float* base = nullptr;
  XABE_TRY(na_scratch(as_stream(stream), &base));

  // host-side views over the scratch array, in the shape the launch code takes the block's buffers in
  xabe_moe_kernels k;
  memset(&k, 0, sizeof(k));
  k.g = g;
  k.tensor_cores = true;
  xabe_moe_buffers b;
  memset(&b, 0, sizeof(b));
  b.scope = XABE_SCOPE_ROUTED;
  b.g = g;
  b.valid_tokens = reinterpret_cast<int32_t*>(base + kNaValid);
  b.topk_ids = reinterpret_cast<int32_t*>(base + kNaTopkIds);
  b.topk_weights = base + kNaTopkW;
  b.inter = base + kNaInter;
  b.shared_inter = base + kNaSharedInter;
  b.n_topk = g.max_tokens * g.experts_per_token;
  b.n_inter = b.n_topk * g.intermediate;
  b.n_shared_inter = g.max_tokens * g.intermediate;
  if (!decode_block_supported(&k, &b, w))
    return set_error(XABE_ERR_UNSUPPORTED_GEOMETRY,
                     "unsupported MoE geometry %s: block_forward_noalloc serves the shapes and formats of the three-launch decode "
                     "block only (hidden 2048 / intermediate 512 or 512 / 256; Q6_K or Q8_0 stacks; f32 or Q8_0 router)",
                     geometry_debug(g).c_str());
  XABE_TRY(check_layer_stacks(&k, w));
  hipStream_t s = as_stream(stream);
  hipLaunchKernelGGL(k_na_publish_tokens, dim3(1), dim3(64), 0, s, b.valid_tokens, (int)tokens);
  XABE_HIP_TRY(hipGetLastError());
  return launch_decode_block(&k, s, &b, w, residual, logit_bias, eps, base + kNaNormed, base + kNaLogits, base + kNaShexp,
                             base + kNaGate, base + kNaRouted, ffn_out, l_out);
}

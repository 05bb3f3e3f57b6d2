// Matrix-core (MFMA) regime for prefill widths.
#include "host_common.h"

namespace xabe {

bool mfma_supported(const xabe_moe_kernels* k, const xabe_moe_buffers* b, int gate_q, int up_q, int down_q, bool routed) {
  (void)k; (void)b; (void)gate_q; (void)up_q; (void)down_q; (void)routed;
  return false;
}

int mfma_grouped_forward_partial(const xabe_moe_kernels*, hipStream_t, xabe_moe_buffers*, xabe_quant_tensor,
                                 xabe_quant_tensor, xabe_quant_tensor, const float*) {
  return set_error(XABE_ERR_MMA, "matrix-core regime not built");
}

int mfma_shared_expert(const xabe_moe_kernels*, hipStream_t, xabe_moe_buffers*, xabe_quant_tensor, xabe_quant_tensor,
                       xabe_quant_tensor, const float*, float*) {
  return set_error(XABE_ERR_MMA, "matrix-core regime not built");
}

}  // namespace xabe

// Decode-width fusion of the routed and shared experts:
//   k_expert_flat_with_shared: the shared expert's work units ride the routed experts' grid
//                              (crates/xabe-cuda/src/kernels/moe.rs:6190-6335).
// Every value is computed by the same device functions the separate launches use, so the results
// are bit-identical to them.
#include <string.h>

#include "decode_kernels.h"
#include "host_common.h"

namespace xabe {

enum Shape { kRps8, kRps4, kRps2, kKs1, kKs2, kStream };
static Shape shape_for(size_t K) {
  if (K == 256) return kRps8;
  if (K == 512) return kRps4;
  if (K == 1024) return kRps2;
  if (K <= 2048) return kKs1;
  if (K <= 4096) return kKs2;
  return kStream;
}
static int rows_per_step(Shape s) { return s == kRps8 ? 8 : s == kRps4 ? 4 : s == kRps2 ? 2 : 1; }

template <int RQ, int SQ, int NM>
static void launch_fused_shape(Shape shape, dim3 grid, hipStream_t s, const FusedArgs& a) {
  switch (shape) {
    case kRps8: hipLaunchKernelGGL((k_expert_flat_with_shared<RQ, SQ, 1, 8, NM>), grid, dim3(256), 0, s, a); break;
    case kRps4: hipLaunchKernelGGL((k_expert_flat_with_shared<RQ, SQ, 1, 4, NM>), grid, dim3(256), 0, s, a); break;
    case kRps2: hipLaunchKernelGGL((k_expert_flat_with_shared<RQ, SQ, 1, 2, NM>), grid, dim3(256), 0, s, a); break;
    case kKs1: hipLaunchKernelGGL((k_expert_flat_with_shared<RQ, SQ, 1, 1, NM>), grid, dim3(256), 0, s, a); break;
    case kKs2: hipLaunchKernelGGL((k_expert_flat_with_shared<RQ, SQ, 2, 1, NM>), grid, dim3(256), 0, s, a); break;
    default: hipLaunchKernelGGL((k_expert_flat_with_shared<RQ, SQ, 0, 1, NM>), grid, dim3(256), 0, s, a); break;
  }
}

template <int NM>
static int launch_fused_quant(int rq, int sq, Shape shape, dim3 grid, hipStream_t s, const FusedArgs& a) {
  if (rq == XABE_QUANT_Q6K && sq == XABE_QUANT_Q6K) launch_fused_shape<kQ6K, kQ6K, NM>(shape, grid, s, a);
  else if (rq == XABE_QUANT_Q6K && sq == XABE_QUANT_Q8_0) launch_fused_shape<kQ6K, kQ8_0, NM>(shape, grid, s, a);
  else if (rq == XABE_QUANT_Q8_0 && sq == XABE_QUANT_Q6K) launch_fused_shape<kQ8_0, kQ6K, NM>(shape, grid, s, a);
  else if (rq == XABE_QUANT_Q8_0 && sq == XABE_QUANT_Q8_0) launch_fused_shape<kQ8_0, kQ8_0, NM>(shape, grid, s, a);
  else return set_error(XABE_ERR_UNSUPPORTED_QUANT, "no fused kernel for quantization codes %d / %d", rq, sq);
  XABE_HIP_TRY(hipGetLastError());
  return XABE_OK;
}

int launch_flat_with_shared(const xabe_moe_kernels* k, hipStream_t s, xabe_moe_buffers* b, int nm, int routed_quant,
                            int shared_quant, const void* rw0, const void* rw1, size_t expert_bytes, const float* rx,
                            float* rout, const void* sw0, const void* sw1, const float* sx, float* sout, int K,
                            int n_rows) {
  const xabe_moe_geometry& g = k->g;
  FusedArgs a;
  memset(&a, 0, sizeof(a));
  ExpertArgs base;
  memset(&base, 0, sizeof(base));
  base.valid_tokens = b->valid_tokens;
  base.topk_ids = b->topk_ids;
  base.topk_weights = b->topk_weights;
  base.top_k = (int)g.experts_per_token;
  base.block_size = (int)g.block_size;
  base.K = K;
  base.n_rows = n_rows;
  const Shape shape = shape_for((size_t)K);
  const size_t routed_units = xabe_moe_geometry_max_flat_pairs(&g);
  const size_t shared_units = (g.max_tokens + 1) / 2;
  base.tile_rows = pick_tile_rows(k, routed_units + shared_units, n_rows, rows_per_step(shape));
  a.routed = base;
  a.routed.w0 = static_cast<const uint8_t*>(rw0);
  a.routed.w1 = static_cast<const uint8_t*>(rw1);
  a.routed.expert_bytes = expert_bytes;
  a.routed.x = rx;
  a.routed.out = rout;
  a.shared = base;
  a.shared.w0 = static_cast<const uint8_t*>(sw0);
  a.shared.w1 = static_cast<const uint8_t*>(sw1);
  a.shared.x = sx;
  a.shared.out = sout;
  a.routed_units = (int)routed_units;
  dim3 grid((unsigned)((n_rows + base.tile_rows - 1) / base.tile_rows), (unsigned)(routed_units + shared_units));
  return nm == 2 ? launch_fused_quant<2>(routed_quant, shared_quant, shape, grid, s, a)
                 : launch_fused_quant<1>(routed_quant, shared_quant, shape, grid, s, a);
}

}  // namespace xabe

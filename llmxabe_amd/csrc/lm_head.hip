// LM head: logits[t][v] = sum_h W[v][h] * x[t][h] for a [vocab][hidden] matrix in Q8_0, Q6_K, bf16 or f16,
// and the device half of greedy sampling.  Takes the place of crates/xabe-cuda/src/kernels/lm_head.rs.
//
// The matrix is read once per pass and a pass serves up to four tokens: the lane's activations of the tile
// (32 per token for a 2048-wide row) stay in registers for the whole launch, so the only stream is the
// weights.  A wavefront owns R adjacent rows at a time, requests the next R rows before it accumulates the
// current ones, and walks the vocabulary with all other wavefronts in row order, so the launch reads the
// tensor front to back.  Quantized rows go through the coalesced loader of decode_kernels.h (each 16-byte
// piece requested once, fields unpacked from a wavefront-private LDS slot); 16-bit rows are read as
// 16-byte pieces directly.
//
// Numerics: fp32, no contraction.  A lane sums its products in element order (the accumulation of the decode
// kernels), the 64 lane sums are combined by the fixed DPP tree, and nothing depends on the batch: a token's
// logits are the same bits at every batch width and position.
#include <string.h>

#include <algorithm>

#include "../../include/xabe_gguf.h"
#include "../../include/xabe_lm_head.h"
#include "decode_kernels.h"
#include "host_common.h"

namespace xabe {

struct LmHeadArgs {
  const uint8_t* w;
  const float* x;   // [*][K]
  float* out;       // [*][vocab]
  int K, vocab;
  int t0, nt;       // tokens [t0, t0 + nt) are served by this launch, 1 <= nt <= TOK
  int row_lo, row_hi;    // quantized kernels: rows [row_lo, row_hi) are served by this launch
  const uint8_t* w_end;  // TAIL launches: one past the tensor's last byte
};

// Q8_0 / Q6_K rows.  ONE: the row is a single wavefront step (K <= 2048) and the activations are hoisted out
// of the row loop; otherwise the contraction is walked step by step with the activations re-read per step.
// TAIL: the launch that serves the last row of a tensor whose length is not a multiple of 16 bytes; the one
// piece that would reach past the tensor is put together from 2-byte loads.
template <int QUANT, int R, int TOK, bool ONE, bool TAIL = false>
__global__ void __launch_bounds__(256) k_lm_head_quant(LmHeadArgs a) {
  using F = Fmt<QUANT>;
  using Raw = typename F::Raw;
  constexpr int kSlot = StageFmt<QUANT>::kSlotBytes;
  __shared__ __attribute__((aligned(16))) uint8_t s_slots[kWavesPerWg * R * kSlot];
  const LaneGeom g = lane_geom<QUANT>();
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const size_t row_bytes = (size_t)(a.K / F::kBlockElems) * F::kBlockBytes;
  const int steps = (a.K + kStepElems - 1) / kStepElems;
  const int groups = (a.row_hi - a.row_lo + R - 1) / R;
  const int stride = (int)gridDim.x * kWavesPerWg;
  uint8_t* slots = s_slots + (size_t)wave * R * kSlot;

  auto issue_w = [&](int rg, int k, Staged<QUANT> (&pend)[R]) __attribute__((always_inline)) {
    const uint32_t nbytes = (uint32_t)(min(kStepElems, a.K - k * kStepElems) / F::kBlockElems) * F::kBlockBytes;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int row = min(a.row_lo + rg * R + r, a.row_hi - 1);  // a group past the last row repeats it and stores nothing
      const uint8_t* chunk = a.w + (size_t)row * row_bytes + (size_t)k * F::kChunkBytes;
      if constexpr (TAIL) stage_load_bounded<QUANT>(chunk, nbytes, a.w_end, pend[r]);
      else stage_load<QUANT>(chunk, nbytes, pend[r]);
    }
    issue_fence();
  };
  auto load_x = [&](int k, float (&xl)[TOK][32], float (&xs)[TOK][4]) __attribute__((always_inline)) {
    const int koff = min(lane_koff<QUANT, 1>(g, k), a.K - F::kBlockElems);
    const bool act = lane_koff<QUANT, 1>(g, k) < a.K;
#pragma unroll
    for (int t = 0; t < TOK; ++t) {
      float v[32];
      lane_x_load<QUANT>(a.x + (size_t)(a.t0 + min(t, a.nt - 1)) * a.K, koff, g, v);
#pragma unroll
      for (int i = 0; i < 32; ++i) xl[t][i] = act ? v[i] : 0.0f;
      lane_x_offsets<QUANT>(xl[t], xs[t]);
    }
  };
  auto store = [&](int rg, const float (&acc)[R][TOK]) __attribute__((always_inline)) {
#pragma unroll
    for (int t = 0; t < TOK; ++t) {
      if (t >= a.nt) break;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const float tot = group_sum<64>(acc[r][t]);
        const int row = a.row_lo + rg * R + r;
        if (g.lane == 0 && row < a.row_hi) a.out[(size_t)(a.t0 + t) * a.vocab + row] = 1.0f * tot;
      }
    }
  };

  int rg = (int)blockIdx.x * kWavesPerWg + wave;
  if (rg >= groups) return;
  if constexpr (ONE) {
    float xl[TOK][32], xs[TOK][4];
    load_x(0, xl, xs);
    const bool act = lane_koff<QUANT, 1>(g, 0) < a.K;
    Staged<QUANT> pend[R];
    issue_w(rg, 0, pend);
#pragma unroll 1
    for (; rg < groups; rg += stride) {
      Raw raw[R];
#pragma unroll
      for (int r = 0; r < R; ++r) stage_pick<QUANT>(pend[r], slots + (size_t)r * kSlot, act, g, raw[r]);
      if (rg + stride < groups) issue_w(rg + stride, 0, pend);
      float acc[R][TOK];
#pragma unroll
      for (int r = 0; r < R; ++r) {
#pragma unroll
        for (int t = 0; t < TOK; ++t) acc[r][t] = 0.0f;
        accum<QUANT, TOK>(raw[r], g, xl, xs, acc[r]);
      }
      store(rg, acc);
    }
  } else {
#pragma unroll 1
    for (; rg < groups; rg += stride) {
      float acc[R][TOK];
#pragma unroll
      for (int r = 0; r < R; ++r)
#pragma unroll
        for (int t = 0; t < TOK; ++t) acc[r][t] = 0.0f;
      Staged<QUANT> pend[R];
      issue_w(rg, 0, pend);
#pragma unroll 1
      for (int k = 0; k < steps; ++k) {
        float xl[TOK][32], xs[TOK][4];
        load_x(k, xl, xs);
        const bool act = lane_koff<QUANT, 1>(g, k) < a.K;
        Raw raw[R];
#pragma unroll
        for (int r = 0; r < R; ++r) stage_pick<QUANT>(pend[r], slots + (size_t)r * kSlot, act, g, raw[r]);
        if (k + 1 < steps) issue_w(rg, k + 1, pend);
#pragma unroll
        for (int r = 0; r < R; ++r) accum<QUANT, TOK>(raw[r], g, xl, xs, acc[r]);
      }
      store(rg, acc);
    }
  }
}

// bf16 / f16 rows: lane l covers elements j*512 + 8*l .. +8 of every 512-element section j.
typedef uint32_t piece16 __attribute__((ext_vector_type(4)));

template <bool F16>
__device__ __forceinline__ void widen8(const piece16& p, float (&w)[8]) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if constexpr (F16) {
      w[2 * i] = (float)__builtin_bit_cast(_Float16, (uint16_t)(p[i] & 0xffffu));
      w[2 * i + 1] = (float)__builtin_bit_cast(_Float16, (uint16_t)(p[i] >> 16));
    } else {  // bf16 is a truncated f32: the widening is a shift
      w[2 * i] = __builtin_bit_cast(float, p[i] << 16);
      w[2 * i + 1] = __builtin_bit_cast(float, p[i] & 0xffff0000u);
    }
  }
}

// SEC > 0: K = 512 * SEC, activations in registers; SEC == 0: sections from K at run time, activations re-read.
template <bool F16, int R, int TOK, int SEC>
__global__ void __launch_bounds__(256) k_lm_head_half(LmHeadArgs a) {
  const int lane = (int)__lane_id();
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int groups = (a.vocab + R - 1) / R;
  const int stride = (int)gridDim.x * kWavesPerWg;
  const int sections = a.K / 512;
  constexpr int kHeld = SEC > 0 ? SEC : 1;
  float x[TOK][kHeld][8];
  auto load_x = [&](int j, int slot) __attribute__((always_inline)) {
#pragma unroll
    for (int t = 0; t < TOK; ++t) {
      const float4* p = reinterpret_cast<const float4*>(a.x + (size_t)(a.t0 + min(t, a.nt - 1)) * a.K + j * 512 + lane * 8);
      const float4 u = p[0], v = p[1];
      x[t][slot][0] = u.x, x[t][slot][1] = u.y, x[t][slot][2] = u.z, x[t][slot][3] = u.w;
      x[t][slot][4] = v.x, x[t][slot][5] = v.y, x[t][slot][6] = v.z, x[t][slot][7] = v.w;
    }
  };
  if constexpr (SEC > 0) {
#pragma unroll
    for (int j = 0; j < SEC; ++j) load_x(j, j);
  }
  auto row_ptr = [&](int rg, int r) __attribute__((always_inline)) {
    const int row = min(rg * R + r, a.vocab - 1);
    return reinterpret_cast<const piece16*>(a.w + (size_t)row * a.K * 2) + lane;
  };
  int rg = (int)blockIdx.x * kWavesPerWg + wave;
  if (rg >= groups) return;
  piece16 pend[R][kHeld];
  auto issue_w = [&](int g2, int j0) __attribute__((always_inline)) {
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int j = 0; j < kHeld; ++j) pend[r][j] = row_ptr(g2, r)[(j0 + j) * 64];
    issue_fence();
  };
  issue_w(rg, 0);
#pragma unroll 1
  for (; rg < groups; rg += stride) {
    float acc[R][TOK];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int t = 0; t < TOK; ++t) acc[r][t] = 0.0f;
    const int n_sec = SEC > 0 ? 1 : sections;
#pragma unroll 1
    for (int j = 0; j < n_sec; ++j) {
      piece16 cur[R][kHeld];
#pragma unroll
      for (int r = 0; r < R; ++r)
#pragma unroll
        for (int h = 0; h < kHeld; ++h) cur[r][h] = pend[r][h];
      if (SEC == 0) load_x(j, 0);
      // next pieces: the next section of this group, or the first of the next group
      if (j + 1 < n_sec) issue_w(rg, j + 1);
      else if (rg + stride < groups) issue_w(rg + stride, 0);
#pragma unroll
      for (int r = 0; r < R; ++r)
#pragma unroll
        for (int h = 0; h < kHeld; ++h) {
          float w[8];
          widen8<F16>(cur[r][h], w);
#pragma unroll
          for (int t = 0; t < TOK; ++t)
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[r][t] += w[i] * x[t][h][i];
        }
    }
#pragma unroll
    for (int t = 0; t < TOK; ++t) {
      if (t >= a.nt) break;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const float tot = group_sum<64>(acc[r][t]);
        const int row = rg * R + r;
        if (lane == 0 && row < a.vocab) a.out[(size_t)(a.t0 + t) * a.vocab + row] = tot;
      }
    }
  }
}

// ---------------------------------------------------------------------------------
// argmax with the scalar reference's semantics (crates/xabe-kernels/src/gemv.rs:103-112: `best` moves only on
// a strictly greater value, so the first maximum wins, a NaN never wins, and a NaN at index 0 is never
// displaced).  A candidate is (value, index); NaN candidates are dropped, equal values keep the lower index.
// ---------------------------------------------------------------------------------
struct Cand {
  float v;
  int i;
};
__device__ __forceinline__ Cand better(Cand a, Cand b) {
  const bool take_b = b.i >= 0 && (a.i < 0 || b.v > a.v || (b.v == a.v && b.i < a.i));
  return take_b ? b : a;
}
__device__ __forceinline__ Cand block_best(Cand c, Cand* s) {
  // wavefront: butterfly through LDS-free lane permutes, then one slot per wavefront
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) {
    Cand o;
    o.v = __shfl_xor(c.v, d, 64);
    o.i = __shfl_xor(c.i, d, 64);
    c = better(c, o);
  }
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) s[wave] = c;
  __syncthreads();
  Cand r = s[0];
  for (int w = 1; w < (int)(blockDim.x >> 6); ++w) r = better(r, s[w]);
  return r;
}

__global__ void __launch_bounds__(256) k_argmax_partial(const float* __restrict__ v, int n, float* __restrict__ pv,
                                                         int* __restrict__ pi) {
  __shared__ Cand s[4];
  Cand c{0.0f, -1};
  for (int i = blockIdx.x * 256 + threadIdx.x; i < n; i += gridDim.x * 256) {
    const float x = v[i];
    if (x == x) c = better(c, Cand{x, i});
  }
  c = block_best(c, s);
  if (threadIdx.x == 0) {
    pv[blockIdx.x] = c.v;
    pi[blockIdx.x] = c.i;
  }
}

__global__ void __launch_bounds__(256) k_argmax_final(const float* __restrict__ pv, const int* __restrict__ pi, int blocks,
                                                       const float* __restrict__ v, int* __restrict__ out) {
  __shared__ Cand s[4];
  Cand c{0.0f, -1};
  for (int b = threadIdx.x; b < blocks; b += 256) c = better(c, Cand{pv[b], pi[b]});
  c = block_best(c, s);
  if (threadIdx.x == 0) {
    const float first = v[0];
    out[0] = (first != first || c.i < 0) ? 0 : c.i;
  }
}

// 1 / sum(exp(x - max)): one workgroup, a maximum pass and a sum pass, both in a fixed order.
__global__ void __launch_bounds__(256) k_argmax_prob(const float* __restrict__ v, int n, float* __restrict__ out) {
  __shared__ float s[4];
  float m = -INFINITY;
  for (int i = threadIdx.x; i < n; i += 256) m = fmaxf(m, v[i]);
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) m = fmaxf(m, __shfl_xor(m, d, 64));
  if ((threadIdx.x & 63) == 0) s[threadIdx.x >> 6] = m;
  __syncthreads();
  m = fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3]));
  __syncthreads();
  float sum = 0.0f;
  for (int i = threadIdx.x; i < n; i += 256) sum += expf(v[i] - m);
  sum = group_sum<64>(sum);
  if ((threadIdx.x & 63) == 0) s[threadIdx.x >> 6] = sum;
  __syncthreads();
  if (threadIdx.x == 0) out[0] = 1.0f / ((s[0] + s[1]) + (s[2] + s[3]));
}

static size_t format_elements(int format, size_t bytes, size_t* block_bytes) {
  switch (format) {
    case XABE_HEAD_Q8_0: *block_bytes = kQ8Bytes; return bytes / kQ8Bytes * 32;
    case XABE_HEAD_Q6K: *block_bytes = kQ6KBytes; return bytes / kQ6KBytes * 256;
    default: *block_bytes = 2; return bytes / 2;
  }
}

}  // namespace xabe

using xabe::set_error;

struct xabe_lm_head {
  xabe_lm_head_geometry g;
  int num_cus;
};

static int bad_head(const xabe_lm_head_geometry& g, const char* reason) {
  return set_error(XABE_ERR_UNSUPPORTED_GEOMETRY, "unsupported LM head geometry LmHeadGeometry { hidden: %zu, vocab: %zu, max_tokens: %zu }: %s",
                   g.hidden, g.vocab, g.max_tokens, reason);
}

static int check_len(const char* what, size_t expected, size_t got) {
  if (got == expected) return XABE_OK;
  return set_error(XABE_ERR_SHAPE_MISMATCH, "%s: expected %zu elements, got %zu", what, expected, got);
}

extern "C" {

int xabe_head_format_from_ggml(int t) {
  switch (t) {
    case XABE_GGML_Q8_0: return XABE_HEAD_Q8_0;
    case XABE_GGML_BF16: return XABE_HEAD_BF16;
    case XABE_GGML_Q6_K: return XABE_HEAD_Q6K;
    case XABE_GGML_F16: return XABE_HEAD_F16;
    case XABE_GGML_Q4_0: return XABE_HEAD_Q4_0;
    case XABE_GGML_Q4_K: return XABE_HEAD_Q4K;
    case XABE_GGML_Q5_K: return XABE_HEAD_Q5K;
  }
  return -1;
}

xabe_lm_head_geometry xabe_lm_head_geometry_qwen3_6(size_t max_tokens) {
  xabe_lm_head_geometry g = {2048, 248320, max_tokens};
  return g;
}

size_t xabe_lm_head_row_bytes_for(const xabe_lm_head_geometry* g, int format) {
  if (!g) return 0;
  switch (format) {
    case XABE_HEAD_Q8_0: return g->hidden / 32 * 34;
    case XABE_HEAD_Q6K: return g->hidden / 256 * 210;
    case XABE_HEAD_BF16: case XABE_HEAD_F16: return g->hidden * 2;
    case XABE_HEAD_Q4_0: return g->hidden / 32 * 18;
    case XABE_HEAD_Q4K: return g->hidden / 256 * 144;
    case XABE_HEAD_Q5K: return g->hidden / 256 * 176;
  }
  return 0;
}

size_t xabe_lm_head_weight_bytes_for(const xabe_lm_head_geometry* g, int format) {
  return g ? g->vocab * xabe_lm_head_row_bytes_for(g, format) : 0;
}
size_t xabe_lm_head_elements(const xabe_lm_head_geometry* g) { return g ? g->vocab * g->hidden : 0; }
size_t xabe_lm_head_weight_passes(const xabe_lm_head_geometry*, size_t tokens) {
  return (tokens + XABE_LM_HEAD_MAX_BATCH_TILE - 1) / XABE_LM_HEAD_MAX_BATCH_TILE;
}
size_t xabe_lm_head_weight_bytes_read(const xabe_lm_head_geometry* g, int format, size_t tokens) {
  return xabe_lm_head_weight_bytes_for(g, format) * xabe_lm_head_weight_passes(g, tokens);
}

int xabe_lm_head_new(const xabe_lm_head_geometry* geometry, xabe_lm_head** out) {
  if (!geometry || !out) return set_error(XABE_ERR_INVALID_ARGUMENT, "null geometry or output pointer");
  const xabe_lm_head_geometry& g = *geometry;
  if (g.hidden == 0 || g.vocab == 0) return bad_head(g, "hidden and vocab must be non-zero");
  if (g.hidden % 512 != 0) return bad_head(g, "hidden must be a whole number of 16-block staging segments (a multiple of 512)");
  if (g.max_tokens == 0) return bad_head(g, "max_tokens must be non-zero");
  if (g.vocab > 0x7fffffffu || g.hidden > 0x7fffffffu) return bad_head(g, "vocabulary exceeds the grid.x limit");
  int dev = 0, cus = 256;
  XABE_HIP_TRY(hipGetDevice(&dev));
  XABE_HIP_TRY(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
  xabe_lm_head* h = new xabe_lm_head();
  h->g = g;
  h->num_cus = cus;
  *out = h;
  return XABE_OK;
}

void xabe_lm_head_free(xabe_lm_head* h) { delete h; }

int xabe_lm_head_geometry_of(const xabe_lm_head* h, xabe_lm_head_geometry* out) {
  if (!h || !out) return set_error(XABE_ERR_INVALID_ARGUMENT, "null handle or output pointer");
  *out = h->g;
  return XABE_OK;
}

}  // extern "C"

namespace xabe {

template <int TOK>
static void launch_pass(const xabe_lm_head* h, hipStream_t s, int format, const LmHeadArgs& a) {
  // rows per wavefront iteration: four for one token, two once the tile's activations take the registers
  constexpr int R = TOK == 1 ? 4 : 2;
  const int groups = (a.row_hi - a.row_lo + R - 1) / R;
  const unsigned grid = (unsigned)std::max(1, std::min((groups + kWavesPerWg - 1) / kWavesPerWg, h->num_cus * 4));
  const bool one = a.K <= kStepElems;
  if (a.w_end) {  // the last row of a tensor that ends inside a 16-byte piece: one wavefront, bounded loads
    if (format == XABE_HEAD_Q8_0) hipLaunchKernelGGL((k_lm_head_quant<kQ8_0, R, TOK, false, true>), dim3(1), dim3(256), 0, s, a);
    else hipLaunchKernelGGL((k_lm_head_quant<kQ6K, R, TOK, false, true>), dim3(1), dim3(256), 0, s, a);
    return;
  }
  switch (format) {
    case XABE_HEAD_Q8_0:
      if (one) hipLaunchKernelGGL((k_lm_head_quant<kQ8_0, R, TOK, true>), dim3(grid), dim3(256), 0, s, a);
      else hipLaunchKernelGGL((k_lm_head_quant<kQ8_0, R, TOK, false>), dim3(grid), dim3(256), 0, s, a);
      break;
    case XABE_HEAD_Q6K:
      if (one) hipLaunchKernelGGL((k_lm_head_quant<kQ6K, R, TOK, true>), dim3(grid), dim3(256), 0, s, a);
      else hipLaunchKernelGGL((k_lm_head_quant<kQ6K, R, TOK, false>), dim3(grid), dim3(256), 0, s, a);
      break;
    case XABE_HEAD_BF16:
      if (a.K == 2048) hipLaunchKernelGGL((k_lm_head_half<false, R, TOK, 4>), dim3(grid), dim3(256), 0, s, a);
      else hipLaunchKernelGGL((k_lm_head_half<false, R, TOK, 0>), dim3(grid), dim3(256), 0, s, a);
      break;
    default:
      if (a.K == 2048) hipLaunchKernelGGL((k_lm_head_half<true, R, TOK, 4>), dim3(grid), dim3(256), 0, s, a);
      else hipLaunchKernelGGL((k_lm_head_half<true, R, TOK, 0>), dim3(grid), dim3(256), 0, s, a);
      break;
  }
}

}  // namespace xabe

extern "C" {

int xabe_lm_head_forward(const xabe_lm_head* h, void* stream, int format, const void* weight, size_t weight_len,
                         const float* hidden_states, size_t hidden_states_len, size_t tokens, float* logits,
                         size_t logits_len) {
  if (!h || !weight || !hidden_states || !logits) return set_error(XABE_ERR_INVALID_ARGUMENT, "null handle or buffer");
  const xabe_lm_head_geometry& g = h->g;
  switch (format) {
    case XABE_HEAD_Q8_0: case XABE_HEAD_Q6K: case XABE_HEAD_BF16: case XABE_HEAD_F16: break;
    case XABE_HEAD_Q4_0: case XABE_HEAD_Q4K: case XABE_HEAD_Q5K:
      return set_error(XABE_ERR_UNSUPPORTED_QUANT, "LM head: format %d is recognised, but this library has kernels for Q8_0, Q6_K, bf16 and f16 only", format);
    default: return set_error(XABE_ERR_INVALID_ARGUMENT, "LM head: unknown format %d", format);
  }
  if (format == XABE_HEAD_Q6K && g.hidden % 256 != 0)
    return set_error(XABE_ERR_UNSUPPORTED_GEOMETRY, "the Q6_K GEMV covers 256 elements per warp step, so `hidden` must be a multiple of 256, not %zu", g.hidden);
  size_t block_bytes = 0;
  const size_t found = xabe::format_elements(format, weight_len, &block_bytes);
  if (weight_len % block_bytes != 0)
    return set_error(XABE_ERR_RAGGED_WEIGHTS, "LM head: %zu bytes is not a whole number of %zu B blocks", weight_len, block_bytes);
  if (found != g.vocab * g.hidden)
    return set_error(XABE_ERR_WRONG_ELEMENT_COUNT, "LM head: expected %zu elements for this geometry, tensor holds %zu", g.vocab * g.hidden, found);
  if (tokens == 0 || tokens > g.max_tokens)
    return set_error(XABE_ERR_TOO_MANY_TOKENS, "%zu tokens is outside 1..=%zu, the range the buffers were sized for", tokens, g.max_tokens);
  XABE_TRY(check_len("hidden states", g.max_tokens * g.hidden, hidden_states_len));
  XABE_TRY(check_len("logits", g.max_tokens * g.vocab, logits_len));
  if ((reinterpret_cast<uintptr_t>(weight) & 15u) != 0 || (reinterpret_cast<uintptr_t>(hidden_states) & 15u) != 0)
    return set_error(XABE_ERR_INVALID_ARGUMENT, "LM head: the weight tensor and the hidden states must start on 16-byte boundaries");
  // the coalesced loader reads whole 16-byte pieces.  A quantized tensor that ends inside one has its last row
  // served by a launch of its own, whose loads stop at the tensor's end; the 16-byte windows of every earlier
  // row end inside the last row.
  const bool quant = format == XABE_HEAD_Q8_0 || format == XABE_HEAD_Q6K;
  const bool ragged_end = quant && weight_len % 16 != 0;
  hipStream_t s = xabe::as_stream(stream);
  xabe::LmHeadArgs a;
  a.w = static_cast<const uint8_t*>(weight);
  a.x = hidden_states;
  a.out = logits;
  a.K = (int)g.hidden;
  a.vocab = (int)g.vocab;
  for (size_t base = 0; base < tokens; base += XABE_LM_HEAD_MAX_BATCH_TILE) {
    const int tile = (int)std::min<size_t>(XABE_LM_HEAD_MAX_BATCH_TILE, tokens - base);
    a.t0 = (int)base;
    a.nt = tile;
    for (int part = 0; part < (ragged_end ? 2 : 1); ++part) {
      a.row_lo = part == 0 ? 0 : a.vocab - 1;
      a.row_hi = ragged_end && part == 0 ? a.vocab - 1 : a.vocab;
      a.w_end = part == 0 ? nullptr : a.w + weight_len;
      if (a.row_lo >= a.row_hi) continue;  // a one-row tensor has only the bounded part
      switch (tile) {
        case 1: xabe::launch_pass<1>(h, s, format, a); break;
        case 2: xabe::launch_pass<2>(h, s, format, a); break;
        case 3: xabe::launch_pass<3>(h, s, format, a); break;
        default: xabe::launch_pass<4>(h, s, format, a); break;
      }
      XABE_HIP_TRY(hipGetLastError());
    }
  }
  return XABE_OK;
}

int xabe_lm_head_argmax(const xabe_lm_head* h, void* stream, const float* values, size_t values_len, size_t n,
                        float* partial_values, size_t partial_values_len, int32_t* partial_indices,
                        size_t partial_indices_len, int32_t* out, size_t out_len) {
  if (!h || !values || !partial_values || !partial_indices || !out) return set_error(XABE_ERR_INVALID_ARGUMENT, "null handle or buffer");
  if (n == 0 || n > values_len || n > 0x7fffffffu)
    return set_error(XABE_ERR_SHAPE_MISMATCH, "argmax length: expected %zu elements, got %zu", values_len, n);
  XABE_TRY(check_len("argmax partial values", XABE_LM_HEAD_ARGMAX_BLOCKS, partial_values_len));
  XABE_TRY(check_len("argmax partial indices", XABE_LM_HEAD_ARGMAX_BLOCKS, partial_indices_len));
  XABE_TRY(check_len("argmax output", 1, out_len));
  const unsigned blocks = (unsigned)std::min<size_t>((n + 255) / 256, XABE_LM_HEAD_ARGMAX_BLOCKS);
  hipStream_t s = xabe::as_stream(stream);
  hipLaunchKernelGGL(xabe::k_argmax_partial, dim3(blocks), dim3(256), 0, s, values, (int)n, partial_values, partial_indices);
  XABE_HIP_TRY(hipGetLastError());
  hipLaunchKernelGGL(xabe::k_argmax_final, dim3(1), dim3(256), 0, s, partial_values, partial_indices, (int)blocks, values, out);
  XABE_HIP_TRY(hipGetLastError());
  return XABE_OK;
}

int xabe_lm_head_argmax_prob(const xabe_lm_head* h, void* stream, const float* values, size_t values_len, size_t n,
                             float* out, size_t out_len) {
  if (!h || !values || !out) return set_error(XABE_ERR_INVALID_ARGUMENT, "null handle or buffer");
  if (n == 0 || n > values_len || n > 0x7fffffffu)
    return set_error(XABE_ERR_SHAPE_MISMATCH, "argmax_prob length: expected %zu elements, got %zu", values_len, n);
  XABE_TRY(check_len("argmax_prob output", 1, out_len));
  hipLaunchKernelGGL(xabe::k_argmax_prob, dim3(1), dim3(256), 0, xabe::as_stream(stream), values, (int)n, out);
  XABE_HIP_TRY(hipGetLastError());
  return XABE_OK;
}

}  // extern "C"

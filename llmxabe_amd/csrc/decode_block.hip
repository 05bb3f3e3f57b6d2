// The decode-width MoE block (max_tokens <= 32) as three launches with no intermediate passes.
//
// At a few tokens the block moves ~20 MB per token and every dependent memory access costs 1-2 us, so what
// decides the time is the number of dependent round trips and launch boundaries on the critical path, not
// bytes.  The eight steps of the block (norm, router, bias, route, gate/up, down, shared expert, combine)
// are regrouped so that each launch issues everything it needs in one or two rounds of loads:
//
//   A  k_decode_logits:  router logits (+ bias) and the shared expert's gate/up, both normalising the
//                        residual rows on load; one workgroup per token writes the normalised row and
//                        the sigmoid gate scalar.
//   B  k_decode_up:      one (token, k) pair x row tile per workgroup.  One wavefront routes the token from
//                        its logits (every workgroup of a token repeats this: a few microseconds of one
//                        wavefront is cheaper than one more launch or a device-wide handshake), then the
//                        four wavefronts stream the selected expert's gate/up rows, all loads in flight
//                        at once.
//   C  k_decode_down:    one (token, row tile) per workgroup: the eight routed down projections and the
//                        shared one for those rows, summed in registers in k order, gated, combined with
//                        the residual.  No partial buffer, no reduction pass.
//
// Every value is produced by the same per-row device functions (load_raw, accum, group_sum, rms_fold,
// route_one_token) and the same sequence of fp32 operations as the multi-launch path, so the outputs are
// bit-identical to it and to the wider regimes: the batch-invariance contract is unchanged.
#include <string.h>

#include <type_traits>

#include "decode_kernels.h"
#include "host_common.h"
#ifdef XABE_TRACE_ITEMS
namespace xabe { static __device__ long long g_route_trace[4096 * 8]; }
#define XABE_ROUTE_TRACE(slot)                                                                              \
  do {                                                                                                      \
    if ((threadIdx.x & 63) == 0 && blockIdx.x < 4096) xabe::g_route_trace[blockIdx.x * 8 + (slot)] = wall_clock64(); \
  } while (0)
#endif
#include "route_device.h"

namespace xabe {

constexpr size_t kDecodeBlockMaxTokens = 32;  // widest batch served by the three launches (at 32 tokens 198 against the dispatch-table regime's 203 us; it wins beyond)
constexpr int kMaxTopK = 8;       // contributions held in registers by k_decode_down
constexpr int kMaxInter = 512;    // intermediate width staged in LDS by k_decode_down
// Steps per wavefront of the first launch: a wavefront reads 24 KB of activation rows and norm weights for the 2-4 KB
// of weights of one step, so more steps against the same registers cut what the launch pulls out of L2, at the
// price of fewer workgroups.  Measured per width (launch A, us, depth 1 / 2 / 4): one token 5.2 / 5.3 / 6.6, three
// 7.7 / 6.5 / 8.4, eight 14.2 / 9.4 / 8.4, sixteen - / 15.7 / 11.7.
static int logits_depth(int max_tokens) { return max_tokens <= 1 ? 1 : max_tokens <= 6 ? 2 : 4; }

#ifdef XABE_TRACE_ITEMS
// measurement builds only: per-workgroup timestamps (100 MHz device clock), [kernel][workgroup][slot]
static __device__ long long g_item_trace[3 * 4096 * 4];
#define XABE_TRACE(kernel, slot)                                                                          \
  do {                                                                                                    \
    if (threadIdx.x == 0 && blockIdx.x < 4096) g_item_trace[((kernel) * 4096 + blockIdx.x) * 4 + (slot)] = wall_clock64(); \
  } while (0)
#else
#define XABE_TRACE(kernel, slot) do { } while (0)
#endif

struct DecodeArgs {
  const float* residual;
  const float* post_norm;
  const uint8_t* router;
  const uint8_t *gate, *up, *down;
  const uint8_t *sgate, *sup, *sdown;
  const float* shared_gate_inp;
  const float* logit_bias;
  const int* valid_tokens;
  float* normed;
  float* logits;
  int* topk_ids;
  float* topk_weights;
  float* inter;
  float* shared_inter;
  float* shexp;
  float* gate_out;
  float* routed;
  float* ffn_out;
  float* l_out;
  size_t expert_bytes;  // bytes of one expert's gate (= up) matrix
  size_t down_bytes;    // bytes of one expert's down matrix (its format may differ)
  float eps;
  int H, I, E, top_k, max_tokens;
  int tiles_r, tiles_s, tiles_g, tiles_d;  // row tiles: router, shared gate/up (launch A), gate/up (B), down (C)
};

// One step (RPS rows of K = 2048 / RPS elements) of a matrix, or of a gate/up pair, against TC tokens whose
// rows are normalised on load.  Issues every load before the first use.
//   NM = 2: out[t][row] = silu(gate . x_t) * (up . x_t);   NM = 1: out[t][row] = (w . x_t) (+ bias[row]).
template <int QUANT, int RPS, int TC, int NM, int D = 1>
__device__ __forceinline__ void step_normed(const uint8_t* __restrict__ w0, const uint8_t* __restrict__ w1, int K,
                                            int n_rows, int row0, const float* const (&xrow)[TC],
                                            const float* __restrict__ norm_w, float eps, float* const (&out)[TC],
                                            const float* __restrict__ bias, const int* __restrict__ valid_tokens,
                                            int token0) {
  using F = Fmt<QUANT>;
  using Raw = typename F::Raw;
  constexpr int G = 64 / RPS;
  if (row0 >= n_rows) return;
  const LaneGeom g = lane_geom<QUANT>();
  const int koff = lane_koff<QUANT, RPS>(g, 0);
  const size_t row_bytes = (size_t)(K / F::kBlockElems) * F::kBlockBytes;
  // Q8_0 / fp32 steps give lane L the elements 32L..32L+31 of the row, which is what the RMS fold takes
  // from it; Q6_K interleaves a superblock over eight lanes, so the fold needs its own copy.
  constexpr bool kOwnRms = QUANT == kQ6K;
  RmsRaw q[kOwnRms ? TC : 1];
  float x[TC][32], xs[TC][4], nw[32];
  if constexpr (kOwnRms) {
#pragma unroll
    for (int t = 0; t < TC; ++t) rms_load(xrow[t], 0, K, q[t]);
  }
#pragma unroll
  for (int t = 0; t < TC; ++t) lane_x_load<QUANT>(xrow[t], koff, g, x[t]);
  lane_x_load<QUANT>(norm_w, koff, g, nw);
  // D steps (RPS rows each) against the same activation registers: the rows' weights are all requested here
  Raw r[D][NM];
#pragma unroll
  for (int d = 0; d < D; ++d) {
    const int rd = min(row0 + d * RPS, n_rows - RPS);  // (a step past the matrix re-reads its last one: never stored)
    load_raw<QUANT, true>(w0 + (size_t)rd * row_bytes, true, g, r[d][0]);
    if constexpr (NM == 2) load_raw<QUANT, true>(w1 + (size_t)rd * row_bytes, true, g, r[d][NM - 1]);
  }
#pragma unroll
  for (int t = 0; t < TC; ++t) {
    float s = 0.0f;
    if constexpr (kOwnRms) {
      s = rms_fold(q[t], 0.0f);
    } else {
#pragma unroll
      for (int i = 0; i < 32; ++i) s = __builtin_fmaf(x[t][i], x[t][i], s);
      if (g.lane * 32 >= K) s = 0.0f;  // lanes past the row's end hold another lane's elements
    }
    const float inv = rms_finish(s, K, eps);
#pragma unroll
    for (int i = 0; i < 32; ++i) x[t][i] = x[t][i] * inv * nw[i];
    lane_x_offsets<QUANT>(x[t], xs[t]);
  }
  // the live-token count was requested first and is only needed here: rows past it were computed from
  // whatever the buffer held (in bounds, sized for max_tokens) and are dropped
  const int valid = *valid_tokens;
#pragma unroll
  for (int d = 0; d < D; ++d) {
    float tot[NM][TC];
#pragma unroll
    for (int m = 0; m < NM; ++m) {
#pragma unroll
      for (int t = 0; t < TC; ++t) tot[m][t] = 0.0f;
      accum<QUANT, TC>(r[d][m], g, x, xs, tot[m]);
#pragma unroll
      for (int t = 0; t < TC; ++t) tot[m][t] = group_sum<G>(tot[m][t]);
    }
    const int row = row0 + d * RPS + g.lane / G;
    if ((g.lane % G) == 0 && row < n_rows) {
#pragma unroll
      for (int t = 0; t < TC; ++t) {
        float v = NM == 2 ? silu_f(tot[0][t]) * tot[NM - 1][t] : 1.0f * tot[0][t];
        if (NM == 1 && bias) v += bias[row];
        if (token0 + t < valid) out[t][row] = v;
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------
// A: grid = max_tokens (norm + gate scalar) + chunks * tiles_r (router) + chunks * tiles_s (shared gate/up).
// A chunk is two tokens sharing one pass over the weights.
// ------------------------------------------------------------------------------------------------
template <int SQ, int RF, int RPS, int kLogitsDepth>
__global__ void __launch_bounds__(256) k_decode_logits(DecodeArgs a) {
  __shared__ float s_red[4];
  const int chunks = (a.max_tokens + 1) / 2;
  const int n_r = chunks * a.tiles_r;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  XABE_TRACE(0, 0);
  if ((int)blockIdx.x >= a.max_tokens) {
    int item = blockIdx.x - a.max_tokens;
    const bool router = item < n_r;
    if (!router) item -= n_r;
    const int tiles = router ? a.tiles_r : a.tiles_s;
    const int c = item / tiles, tile = item % tiles, t0 = 2 * c;
    const int row0 = (tile * kWavesPerWg + wave) * RPS * kLogitsDepth;
    const float* x0 = a.residual + (size_t)t0 * a.H;
    if (t0 + 1 < a.max_tokens) {
      const float* const xr[2] = {x0, x0 + a.H};
      if (router) {
        float* const o[2] = {a.logits + (size_t)t0 * a.E, a.logits + (size_t)(t0 + 1) * a.E};
        step_normed<RF, RPS, 2, 1, kLogitsDepth>(a.router, nullptr, a.H, a.E, row0, xr, a.post_norm, a.eps, o, a.logit_bias, a.valid_tokens, t0);
      } else {
        float* const o[2] = {a.shared_inter + (size_t)t0 * a.I, a.shared_inter + (size_t)(t0 + 1) * a.I};
        step_normed<SQ, RPS, 2, 2, kLogitsDepth>(a.sgate, a.sup, a.H, a.I, row0, xr, a.post_norm, a.eps, o, nullptr, a.valid_tokens, t0);
      }
    } else {
      const float* const xr[1] = {x0};
      if (router) {
        float* const o[1] = {a.logits + (size_t)t0 * a.E};
        step_normed<RF, RPS, 1, 1, kLogitsDepth>(a.router, nullptr, a.H, a.E, row0, xr, a.post_norm, a.eps, o, a.logit_bias, a.valid_tokens, t0);
      } else {
        float* const o[1] = {a.shared_inter + (size_t)t0 * a.I};
        step_normed<SQ, RPS, 1, 2, kLogitsDepth>(a.sgate, a.sup, a.H, a.I, row0, xr, a.post_norm, a.eps, o, nullptr, a.valid_tokens, t0);
      }
    }
    XABE_TRACE(0, 3);
    return;
  }
  // the normalised row (callers read it back) and g = sigmoid(shared_gate_inp . normed): the order of
  // operations of the stand-alone RMSNorm and gate kernels
  const int t = blockIdx.x;
  const int valid = *a.valid_tokens;
  const float* xr = a.residual + (size_t)t * a.H;
  // hidden <= 2048: eight columns per thread, every load issued before the first use
  float xv[8], nv[8], gv[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int j = threadIdx.x + 256 * i;
    const bool in = j < a.H;
    xv[i] = in ? xr[j] : 0.0f;
    nv[i] = in ? a.post_norm[j] : 0.0f;
    gv[i] = in ? a.shared_gate_inp[j] : 0.0f;
  }
  const float inv = row_inv_rms(xr, a.H, a.eps);
  if (t >= valid) return;
  float s = 0.0f;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int j = threadIdx.x + 256 * i;
    if (j < a.H) {
      const float v = xv[i] * inv * nv[i];
      a.normed[(size_t)t * a.H + j] = v;
      s = __builtin_fmaf(gv[i], v, s);
    }
  }
  s = group_sum<64>(s);
  if ((threadIdx.x & 63) == 0) s_red[wave] = s;
  __syncthreads();
  const float total = ((s_red[0] + s_red[1]) + s_red[2]) + s_red[3];
  if (threadIdx.x == 0) a.gate_out[t] = 1.0f / (1.0f + expf(-total));
  XABE_TRACE(0, 2);
}

// ------------------------------------------------------------------------------------------------
// B: grid = max_tokens * top_k * tiles_g.  A tile is 4 wavefronts x DEPTH steps x RPS rows.
// ------------------------------------------------------------------------------------------------
template <int RQ, int RPS, int DEPTH>
__global__ void __launch_bounds__(256) k_decode_up(DecodeArgs a) {
  using F = Fmt<RQ>;
  using Raw = typename F::Raw;
  constexpr int G = 64 / RPS;
  extern __shared__ float s_route[];  // num_experts floats for the routing wavefront
  __shared__ int s_expert, s_final;  // the candidate expert of this pair; the one routing settles on
  const int p = blockIdx.x / a.tiles_g, tile = blockIdx.x % a.tiles_g;
  const int t = p / a.top_k, k = p % a.top_k;
  // everything read before the live-token count is known is sized for max_tokens rows
  const int valid = *a.valid_tokens;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const LaneGeom g = lane_geom<RQ>();
  const int koff = lane_koff<RQ, RPS>(g, 0);
  XABE_TRACE(1, 0);
  // one wavefront routes the token (a different one in neighbouring workgroups, which share a CU); its
  // logits and every wavefront's copy of the normalised row are requested together
  const bool routes = wave == (int)((blockIdx.x >> 8) & 3);
  const bool few = a.E <= 256;
  float lg[kRouteMaxPerLane];
  if (routes) {
    if (few) route_load<4>(a.logits + (size_t)t * a.E, a.E, nullptr, nullptr, *reinterpret_cast<float(*)[4]>(lg));
    else route_load<kRouteMaxPerLane>(a.logits + (size_t)t * a.E, a.E, nullptr, nullptr, lg);
  }
  float x[1][32], xs[1][4];
  lane_x_load<RQ>(a.normed + (size_t)t * a.H, koff, g, x[0]);
  if (t >= valid) return;
  // Routing in two halves (route_device.h).  The first orders the experts by logit: its k-th candidate is
  // the pair's expert unless probabilities tie, and it is known ~2 us before the softmax is, so the four
  // wavefronts request the candidate's rows right away.  The routing wavefront then finishes the softmax
  // under its own loads' latency; in the rare pass where the probabilities reorder the candidates, the rows
  // are streamed again for the expert the reference's rule selects.
  const int n_cand = min(a.top_k + 1, a.E);
  int cand_i = 0;
  if (routes) {
    XABE_ROUTE_TRACE(0);
    if (few) route_order<4>(*reinterpret_cast<float(*)[4]>(lg), a.E, n_cand, cand_i);
    else route_order<kRouteMaxPerLane>(lg, a.E, n_cand, cand_i);
    if (g.lane == k) s_expert = cand_i;
  }
  lane_x_offsets<RQ>(x[0], xs[0]);
  __syncthreads();
  XABE_TRACE(1, 1);
  const size_t row_bytes = (size_t)(a.H / F::kBlockElems) * F::kBlockBytes;
  const int wave_row0 = (tile * kWavesPerWg + wave) * DEPTH * RPS;
  float* out = a.inter + (size_t)p * a.I;
  // the pair's rows of expert e: all loads, (the routing wavefront: the rest of the routing,) accumulation
  auto stream_rows = [&](int e, auto finish_c) __attribute__((always_inline)) {
    constexpr bool kFinish = decltype(finish_c)::value;
    const uint8_t* wg = a.gate + (size_t)e * a.expert_bytes;
    const uint8_t* wu = a.up + (size_t)e * a.expert_bytes;
    Raw r[DEPTH][2];
    auto request = [&](int d0, int d1) __attribute__((always_inline)) {
#pragma unroll
      for (int d = 0; d < DEPTH; ++d) {
        if (d < d0 || d >= d1) continue;
        const int row0 = wave_row0 + d * RPS;  // the tiles divide the rows exactly (checked by the host)
        load_raw<RQ, true>(wg + (size_t)row0 * row_bytes, true, g, r[d][0]);
        load_raw<RQ, true>(wu + (size_t)row0 * row_bytes, true, g, r[d][1]);
      }
    };
    // The routing wavefront finishes the softmax before it requests its own rows: its neighbours' requests
    // fill the CU's memory pipeline at this point, and a load issued now would hold the wavefront (and the
    // routing) until they drain; raised priority keeps it ahead of their arithmetic.
    if constexpr (kFinish) {
      if (routes) {
        __builtin_amdgcn_s_setprio(3);
        int sel_i;
        float sel_w;
        bool exact;
        if (few) route_finish<4>(*reinterpret_cast<float(*)[4]>(lg), a.E, a.top_k, n_cand, cand_i, s_route, sel_i, sel_w, exact);
        else route_finish<kRouteMaxPerLane>(lg, a.E, a.top_k, n_cand, cand_i, s_route, sel_i, sel_w, exact);
        XABE_ROUTE_TRACE(5);
        if (g.lane == k) s_final = sel_i;
        if (k == 0 && tile == 0 && g.lane < a.top_k) {
          a.topk_ids[(size_t)t * a.top_k + g.lane] = sel_i;
          a.topk_weights[(size_t)t * a.top_k + g.lane] = sel_w;
        }
        __builtin_amdgcn_s_setprio(0);
      }
    }
    request(0, DEPTH);  // (the other wavefronts come straight here)
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      if (d == 1) XABE_TRACE(1, 2);
      float tg[1] = {0.0f}, tu[1] = {0.0f};
      accum<RQ, 1>(r[d][0], g, x, xs, tg);
      accum<RQ, 1>(r[d][1], g, x, xs, tu);
      const float sg = group_sum<G>(tg[0]), su = group_sum<G>(tu[0]);
      const int row = wave_row0 + d * RPS + g.lane / G;
      if ((g.lane % G) == 0 && row < a.I) out[row] = silu_f(sg) * su;
    }
  };
  const int e = s_expert;
  stream_rows(e, std::true_type{});
  __syncthreads();  // s_final is there
  const int e_final = s_final;
  if (e_final != e) stream_rows(e_final, std::false_type{});  // (same rows of `inter`, written again)
  XABE_TRACE(1, 3);
}

// ------------------------------------------------------------------------------------------------
// C: grid = max_tokens * tiles_d.  A tile is 4 wavefronts x RPS rows; K = intermediate = 2048 / RPS.
// ------------------------------------------------------------------------------------------------
template <int RQ, int SQ, int RPS>
__global__ void __launch_bounds__(256) k_decode_down(DecodeArgs a) {
  using RawR = typename Fmt<RQ>::Raw;
  using RawS = typename Fmt<SQ>::Raw;
  constexpr int G = 64 / RPS;
  __shared__ __attribute__((aligned(16))) float s_x[(kMaxTopK + 1) * kMaxInter];
  const int t = blockIdx.x / a.tiles_d, tile = blockIdx.x % a.tiles_d;
  // every buffer read below is sized for max_tokens rows, so round one is issued before the live-token
  // count is known; rows past it hold an earlier pass's values or zeros, and nothing is stored for them
  const int valid = *a.valid_tokens;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int lane = __lane_id();
  const int row0 = (tile * kWavesPerWg + wave) * RPS;  // hidden is a multiple of 4 * RPS
  XABE_TRACE(2, 0);
  // round one: selections, gate scalar, the nine activation rows (into LDS), the shared expert's rows
  int my_e = 0;
  float my_w = 0.0f;
  if (lane < a.top_k) {
    my_e = a.topk_ids[(size_t)t * a.top_k + lane];
    my_w = a.topk_weights[(size_t)t * a.top_k + lane];
  }
  const float gate = a.gate_out[t];
  constexpr int kStage = ((kMaxTopK + 1) * kMaxInter / 4 + 255) / 256;  // float4 per thread
  float4 stage[kStage];
  const int n4 = a.I / 4;
  {
    const float4* src_r = reinterpret_cast<const float4*>(a.inter + (size_t)t * a.top_k * a.I);
    const float4* src_s = reinterpret_cast<const float4*>(a.shared_inter + (size_t)t * a.I);
#pragma unroll
    for (int j = 0; j < kStage; ++j) {
      const int i = threadIdx.x + 256 * j;
      stage[j] = make_float4(0.f, 0.f, 0.f, 0.f);
      if (i < (a.top_k + 1) * n4) stage[j] = i < a.top_k * n4 ? src_r[i] : src_s[i - a.top_k * n4];
    }
  }
  const LaneGeom gs = lane_geom<SQ>();
  const LaneGeom gr = lane_geom<RQ>();
  const size_t rb_s = (size_t)(a.I / Fmt<SQ>::kBlockElems) * Fmt<SQ>::kBlockBytes;
  const size_t rb_r = (size_t)(a.I / Fmt<RQ>::kBlockElems) * Fmt<RQ>::kBlockBytes;
  RawS rs;
  load_raw<SQ, true>(a.sdown + (size_t)row0 * rb_s, true, gs, rs);
  if (t >= valid) return;
  // round two: the selected experts' rows
  RawR rr[kMaxTopK];
#pragma unroll
  for (int k = 0; k < kMaxTopK; ++k) {
    const int e = min(max(__builtin_amdgcn_readlane(my_e, k), 0), a.E - 1);
    // k >= top_k reads expert 0's rows and never uses them: an unconditional load keeps all of round two
    // in one basic block, so every load is issued before the first wait
    load_raw<RQ, true>(a.down + (size_t)e * a.down_bytes + (size_t)row0 * rb_r, true, gr, rr[k]);
  }
  // the activation rows arrived before the weights (loads return in order); publish them to LDS
#pragma unroll
  for (int j = 0; j < kStage; ++j) {
    const int i = threadIdx.x + 256 * j;
    if (i < (a.top_k + 1) * n4) reinterpret_cast<float4*>(s_x)[i] = stage[j];
  }
  __syncthreads();
  XABE_TRACE(2, 1);
  float r = 0.0f;
#pragma unroll
  for (int k = 0; k < kMaxTopK; ++k) {
    if (k < a.top_k) {
      float x[1][32], xs[1][4], tot[1] = {0.0f};
      lane_x_load<RQ>(s_x + k * a.I, lane_koff<RQ, RPS>(gr, 0), gr, x[0]);
      lane_x_offsets<RQ>(x[0], xs[0]);
      accum<RQ, 1>(rr[k], gr, x, xs, tot);
      const float w = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, my_w), k));
      r += w * group_sum<G>(tot[0]);
    }
  }
  XABE_TRACE(2, 2);
  float sh;
  {
    float x[1][32], xs[1][4], tot[1] = {0.0f};
    lane_x_load<SQ>(s_x + a.top_k * a.I, lane_koff<SQ, RPS>(gs, 0), gs, x[0]);
    lane_x_offsets<SQ>(x[0], xs[0]);
    accum<SQ, 1>(rs, gs, x, xs, tot);
    sh = 1.0f * group_sum<G>(tot[0]);
  }
  const int row = row0 + lane / G;
  if ((lane % G) == 0 && row < a.H) {
    const size_t i = (size_t)t * a.H + row;
    const float v = r + sh * gate;
    a.routed[i] = r;
    a.shexp[i] = sh;
    a.ffn_out[i] = v;
    a.l_out[i] = v + a.residual[i];
  }
  XABE_TRACE(2, 3);
}

// ------------------------------------------------------------------ host side
struct Launch {
  const DecodeArgs& a;
  hipStream_t s;
  unsigned grid_a, grid_b, grid_c;
  size_t route_lds;
  unsigned launches;  // bit i: issue launch i (A, B, C); all three outside measurements
};

// Each launch is chosen by the formats it reads: A by the shared gate/up and router formats, B by the routed
// gate/up format, C by the routed and shared down formats (the shipped layers mix them: gate/up Q6_K with
// down Q8_0).
template <int RPSH, int DEPTH, int RPSI>
static bool launch_all(const Launch& l, int gq, int dq, int sgq, int sdq, int router_quant) {
  const bool g6 = gq == XABE_QUANT_Q6K, d6 = dq == XABE_QUANT_Q6K, sg6 = sgq == XABE_QUANT_Q6K, sd6 = sdq == XABE_QUANT_Q6K;
  const bool rf32 = router_quant < 0;
  if (!rf32 && router_quant != XABE_QUANT_Q8_0) return false;
  if (l.launches & 1u) {
#define XABE_A(SQ, RF)                                                                                              \
  do {                                                                                                            \
    const int da = logits_depth(l.a.max_tokens);                                                                  \
    if (da == 1) hipLaunchKernelGGL((k_decode_logits<SQ, RF, RPSH, 1>), dim3(l.grid_a), dim3(256), 0, l.s, l.a);  \
    else if (da == 2) hipLaunchKernelGGL((k_decode_logits<SQ, RF, RPSH, 2>), dim3(l.grid_a), dim3(256), 0, l.s, l.a); \
    else hipLaunchKernelGGL((k_decode_logits<SQ, RF, RPSH, 4>), dim3(l.grid_a), dim3(256), 0, l.s, l.a);          \
  } while (0)
    if (sg6 && rf32) XABE_A(kQ6K, kF32);
    else if (sg6) XABE_A(kQ6K, kQ8_0);
    else if (rf32) XABE_A(kQ8_0, kF32);
    else XABE_A(kQ8_0, kQ8_0);
#undef XABE_A
  }
  if (l.launches & 2u) {
    if (g6) hipLaunchKernelGGL((k_decode_up<kQ6K, RPSH, DEPTH>), dim3(l.grid_b), dim3(256), l.route_lds, l.s, l.a);
    else hipLaunchKernelGGL((k_decode_up<kQ8_0, RPSH, DEPTH>), dim3(l.grid_b), dim3(256), l.route_lds, l.s, l.a);
  }
  if (l.launches & 4u) {
#define XABE_C(RQ, SQ) hipLaunchKernelGGL((k_decode_down<RQ, SQ, RPSI>), dim3(l.grid_c), dim3(256), 0, l.s, l.a)
    if (d6 && sd6) XABE_C(kQ6K, kQ6K);
    else if (d6) XABE_C(kQ6K, kQ8_0);
    else if (sd6) XABE_C(kQ8_0, kQ6K);
    else XABE_C(kQ8_0, kQ8_0);
#undef XABE_C
  }
  return true;
}

static bool launch_shape(const Launch& l, int gq, int dq, int sgq, int sdq, int router_quant) {
  if (l.a.H == 2048 && l.a.I == 512) return launch_all<1, 4, 4>(l, gq, dq, sgq, sdq, router_quant);
  if (l.a.H == 512 && l.a.I == 256) return launch_all<4, 1, 8>(l, gq, dq, sgq, sdq, router_quant);
  return false;
}

bool decode_block_supported(const xabe_moe_kernels* k, const xabe_moe_buffers* b, const xabe_moe_layer_weights* w) {
  const xabe_moe_geometry& g = k->g;
  if (g.max_tokens > kDecodeBlockMaxTokens || k->force_community || b->scope != XABE_SCOPE_ROUTED) return false;
  if (!((g.hidden == 2048 && g.intermediate == 512) || (g.hidden == 512 && g.intermediate == 256))) return false;
  if (g.experts_per_token > (size_t)kMaxTopK || g.num_experts > kRouteMaxExperts || g.num_experts % 4 != 0) return false;
  auto ok = [](int q) { return q == XABE_QUANT_Q6K || q == XABE_QUANT_Q8_0; };
  if (!ok(w->gate_exps.quant) || w->gate_exps.quant != w->up_exps.quant || !ok(w->down_exps.quant)) return false;
  if (!ok(w->shared_gate.quant) || w->shared_gate.quant != w->shared_up.quant || !ok(w->shared_down.quant)) return false;
  if (!(w->router_quant < 0 || w->router_quant == XABE_QUANT_Q8_0)) return false;
  return true;
}

int launch_decode_block(const xabe_moe_kernels* k, hipStream_t s, xabe_moe_buffers* b, const xabe_moe_layer_weights* w,
                        const float* residual, const float* logit_bias, float eps, float* normed, float* logits,
                        float* shexp, float* gate_out, float* routed, float* ffn_out, float* l_out, unsigned launches) {
  const xabe_moe_geometry& g = k->g;
  DecodeArgs a;
  memset(&a, 0, sizeof(a));
  a.residual = residual;
  a.post_norm = w->post_norm;
  a.router = static_cast<const uint8_t*>(w->router);
  a.gate = static_cast<const uint8_t*>(w->gate_exps.bytes);
  a.up = static_cast<const uint8_t*>(w->up_exps.bytes);
  a.down = static_cast<const uint8_t*>(w->down_exps.bytes);
  a.sgate = static_cast<const uint8_t*>(w->shared_gate.bytes);
  a.sup = static_cast<const uint8_t*>(w->shared_up.bytes);
  a.sdown = static_cast<const uint8_t*>(w->shared_down.bytes);
  a.shared_gate_inp = w->shared_gate_inp;
  a.logit_bias = logit_bias;
  a.valid_tokens = b->valid_tokens;
  a.normed = normed;
  a.logits = logits;
  a.topk_ids = b->topk_ids;
  a.topk_weights = b->topk_weights;
  a.inter = b->inter;
  a.shared_inter = b->shared_inter;
  a.shexp = shexp;
  a.gate_out = gate_out;
  a.routed = routed;
  a.ffn_out = ffn_out;
  a.l_out = l_out;
  const int rq = w->gate_exps.quant, dq = w->down_exps.quant;
  a.expert_bytes = g.intermediate * g.hidden / xabe_expert_quant_block_elements(rq) * xabe_expert_quant_block_bytes(rq);
  a.down_bytes = g.intermediate * g.hidden / xabe_expert_quant_block_elements(dq) * xabe_expert_quant_block_bytes(dq);
  a.eps = eps;
  a.H = (int)g.hidden;
  a.I = (int)g.intermediate;
  a.E = (int)g.num_experts;
  a.top_k = (int)g.experts_per_token;
  a.max_tokens = (int)g.max_tokens;
  const int rps_h = 2048 / a.H, rps_i = 2048 / a.I;
  const int da = logits_depth(a.max_tokens);
  a.tiles_r = (a.E + kWavesPerWg * rps_h * da - 1) / (kWavesPerWg * rps_h * da);
  a.tiles_s = (a.I + kWavesPerWg * rps_h * da - 1) / (kWavesPerWg * rps_h * da);
  const int depth = a.H == 2048 ? 4 : 1;  // steps per wavefront of the gate/up launch (launch_shape)
  a.tiles_g = (a.I + kWavesPerWg * depth * rps_h - 1) / (kWavesPerWg * depth * rps_h);
  a.tiles_d = (a.H + kWavesPerWg * rps_i - 1) / (kWavesPerWg * rps_i);
  if (a.E % rps_h != 0 || a.I % (kWavesPerWg * depth * rps_h) != 0 || a.H % (kWavesPerWg * rps_i) != 0)
    return set_error(XABE_ERR_UNSUPPORTED_GEOMETRY, "decode block: %d experts / %d intermediate rows do not fill whole steps of %d rows",
                     a.E, a.I, rps_h);
  const int chunks = (a.max_tokens + 1) / 2;
  Launch l{a, s, 0, 0, 0, g.num_experts * sizeof(float), launches};
  l.grid_a = (unsigned)(chunks * (a.tiles_r + a.tiles_s) + a.max_tokens);
  l.grid_b = (unsigned)(a.max_tokens * a.top_k * a.tiles_g);
  l.grid_c = (unsigned)(a.max_tokens * a.tiles_d);
  const bool ok = launch_shape(l, w->gate_exps.quant, w->down_exps.quant, w->shared_gate.quant, w->shared_down.quant, w->router_quant);
  if (!ok) return set_error(XABE_ERR_UNSUPPORTED_GEOMETRY, "decode block: no kernels for this shape or format");
  XABE_HIP_TRY(hipGetLastError());
  return XABE_OK;
}

}  // namespace xabe

#ifdef XABE_TRACE_ITEMS
extern "C" int xabe_debug_read_route_trace(long long* out, size_t n) {
  return (int)hipMemcpyFromSymbol(out, HIP_SYMBOL(xabe::g_route_trace), n * sizeof(long long));
}
extern "C" int xabe_debug_read_item_trace(long long* out, size_t n) {
  return (int)hipMemcpyFromSymbol(out, HIP_SYMBOL(xabe::g_item_trace), n * sizeof(long long));
}
#endif

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
#include "route_device.h"

namespace xabe {

constexpr size_t kDecodeBlockMaxTokens = 32;  // widest batch served by the three launches (at 32 tokens 198 against the dispatch-table regime's 203 us; it wins beyond)
// From this width on the routing is a launch of its own between the first two (one wavefront per token) and the second
// launch reads the selections: inside the second launch every workgroup of a token repeats the token's routing, and
// past a few tokens its grid runs in several rounds per CU, each paying for it again.  Same-box, us per block, routing
// inside / routing launch: 4 tokens 38.6 / 40.5, 6: 49.8 / 51.2, 8: 61.5 / 61.1, 12: 83.3 / 79.4, 16: 101.7 / 94.9,
// 32: 181.3 / 161.5.
constexpr int kPreRouteMinTokens = 8;
// From this width on the second and third launches deal their workgroups so that the ones that read the same row
// tile (of whichever experts their pairs or tokens selected) run next to each other on one XCD: workgroup ids go
// round-robin to the eight XCDs, each with its own L2, and at these widths several pairs select the same expert
// (32 tokens: 256 pairs over ~163 experts), whose rows then come out of HBM once per XCD instead of once per pair.
// Fetched per launch at 32 tokens (FETCH_SIZE): gate/up 415 -> 342 MB, down 204 -> 151 MB.  The launches take the
// same time either way (they are bound by vector instructions at these widths, not by bytes): at 16 tokens and
// below, where fewer pairs coincide, the plain order measured 0.1-0.5 us faster and is kept.
// (Grouping the second launch by expert instead, one workgroup per (expert, row tile) running its pairs against
// one copy of the rows in registers, reads every expert exactly once and was measured slower: 109 us against 95 at
// 32 tokens with one pair at a time, 135 us two at a time (sharing the dequantisation takes ~230 registers); the
// pairs of an expert run one after the other there, and a third of the workgroups find no pair at all.)
constexpr int kXcdGroupMinTokens = 24;
// the seam's arrival counters: per token one counter and one per group of kSeamGroup workgroups, 128 bytes apart
constexpr int kSeamGroup = 16, kSeamMaxGroups = 64, kSeamCountersPerToken = 1 + kSeamMaxGroups, kSeamCounterStride = 32;
constexpr int kMaxTopK = 8;       // contributions held in registers by k_decode_down
constexpr int kMaxInter = 512;    // intermediate width staged in LDS by k_decode_down
// Steps per wavefront of the first launch: a wavefront reads 24 KB of activation rows and norm weights for the 2-4 KB
// of weights of one step, so more steps against the same registers cut what the launch pulls out of L2, at the
// price of fewer workgroups.  Measured per width (launch A, us, depth 1 / 2 / 4): one token 5.2 / 5.3 / 6.6, three
// 7.7 / 6.5 / 8.4, eight 14.2 / 9.4 / 8.4, sixteen - / 15.7 / 11.7.
// Row steps per workgroup of the third launch (two wavefronts each): two, i.e. eight rows of the 2048-wide block.
// Four (half as many workgroups, each staging the token's nine activation rows for twice as many rows) measured
// slower or equal at every width: one token 22.3 against 20.9 us per block, three 32.6 / 31.2, eight 63.8 / 61.8,
// thirty-two 195.7 / 185.6.
constexpr int kDownSteps = 2;
static int logits_depth(int max_tokens) { return max_tokens <= 1 ? 1 : max_tokens <= 6 ? 2 : 4; }


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
  // the seam to the next layer (all null / zero when the pass ends at l_out): the last workgroup of the third launch to
  // finish a token's row applies the next layer's RMSNorm to it (arrival counters: one int per token, zero between passes)
  const float* next_w;
  float* next_normed;
  _Float16* next_normed_h;
  int* arrivals;
  float next_eps;
  size_t expert_bytes;  // bytes of one expert's gate (= up) matrix
  size_t down_bytes;    // bytes of one expert's down matrix (its format may differ)
  float eps;
  int H, I, E, top_k, max_tokens;
  int tiles_r, tiles_s, tiles_g, tiles_d;  // row tiles: router, shared gate/up (launch A), gate/up (B), down (C)
};

// Row tiles of the first launch: D steps (RPS rows of K = 2048 / RPS elements each) per wavefront of a matrix, or of
// a gate/up pair, against the TC tokens of the workgroup's chunk, whose rows are normalised on the way in.
//   NM = 2: out[t][row] = silu(gate . x_t) * (up . x_t);   NM = 1: out[t][row] = (w . x_t) (+ bias[row]).
// The workgroup's four wavefronts need the same TC rows and the norm weight.  They are fetched once per workgroup, as
// consecutive 16-byte pieces, and handed to the wavefronts through LDS; each wavefront then derives the RMS scales in
// the canonical order and normalises its own elements, (x * inv) * w: the stand-alone RMSNorm kernel's values.
// (Each wavefront fetching its own copy from global memory cost 1.9 us of the launch at three tokens: a lane's 32
// elements are one cache line, so every one of its eight loads touched 64 lines, and all workgroups of the launch aim
// at the same few rows.)
// LDS rows are padded by four floats per 32, so that lanes reading 16-byte pieces 128 bytes apart take different banks.
constexpr int kXnPad = kStepElems + kStepElems / 8;  // floats per staged row
__device__ __forceinline__ int xn_at(int e) { return e + 4 * (e >> 5); }

// PRE: the rows handed over are normalised already (the previous block's tail wrote them into this block's `normed`):
// they are staged and used as they are, no norm weight, no scale.
template <int QUANT, int RPS, int TC, int NM, int D, bool PRE>
__device__ __forceinline__ void tile_normed(const uint8_t* __restrict__ w0, const uint8_t* __restrict__ w1, int K,
                                            int n_rows, int row0, const float* const (&xrow)[TC],
                                            const float* __restrict__ norm_w, float eps, float* const (&out)[TC],
                                            const float* __restrict__ bias, const int* __restrict__ valid_tokens,
                                            int token0, float* s_xn) {
  using F = Fmt<QUANT>;
  using Raw = typename F::Raw;
  constexpr int G = 64 / RPS;
  const LaneGeom g = lane_geom<QUANT>();
  const int koff = lane_koff<QUANT, RPS>(g, 0);
  const size_t row_bytes = (size_t)(K / F::kBlockElems) * F::kBlockBytes;
  // the rows' weights first: D steps against the same activation registers, all requested here
  // (a step past the matrix re-reads its last one and is never stored)
  Raw r[D][NM];
#pragma unroll
  for (int d = 0; d < D; ++d) {
    const int rd = min(row0 + d * RPS, n_rows - RPS);
    load_raw<QUANT, true>(w0 + (size_t)rd * row_bytes, true, g, r[d][0]);
    if constexpr (NM == 2) load_raw<QUANT, true>(w1 + (size_t)rd * row_bytes, true, g, r[d][NM - 1]);
  }
  // the chunk's rows and the norm weight, 16 bytes per thread and piece (K <= 2048: two pieces per thread), as they are
  const int n4 = K / 4;
  float* s_nw = s_xn + TC * kXnPad;
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int i = (int)threadIdx.x + 256 * j, ic = min(i, n4 - 1);
    float4 nq = make_float4(0.f, 0.f, 0.f, 0.f);
    if constexpr (!PRE) nq = reinterpret_cast<const float4*>(norm_w)[ic];
    float4 xq[TC];
#pragma unroll
    for (int t = 0; t < TC; ++t) xq[t] = reinterpret_cast<const float4*>(xrow[t])[ic];
    if (i < n4) {
      if constexpr (!PRE) *reinterpret_cast<float4*>(s_nw + xn_at(4 * i)) = nq;
#pragma unroll
      for (int t = 0; t < TC; ++t) *reinterpret_cast<float4*>(s_xn + t * kXnPad + xn_at(4 * i)) = xq[t];
    }
  }
  __syncthreads();
  if (row0 >= n_rows) return;
  // from here on every wavefront works for itself, out of LDS: the RMS scale of each token in the canonical order
  // (lane L folds elements 32L .. 32L+31, then the wavefront tree), its own 32 elements normalised as (x * inv) * w
  auto lds8 = [&](const float* row, int e, float (&v)[32], int at) __attribute__((always_inline)) {
    const float4* p = reinterpret_cast<const float4*>(row + xn_at(e));
    const float4 lo = p[0], hi = p[1];
    v[at + 0] = lo.x; v[at + 1] = lo.y; v[at + 2] = lo.z; v[at + 3] = lo.w;
    v[at + 4] = hi.x; v[at + 5] = hi.y; v[at + 6] = hi.z; v[at + 7] = hi.w;
  };
  float x[TC][32], xs[TC][4], nw[32];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int off = QUANT == kQ6K ? koff + g.half * 128 + j * 32 + g.l8 * 8 : koff + j * 8;
    if constexpr (!PRE) lds8(s_nw, off, nw, j * 8);
#pragma unroll
    for (int t = 0; t < TC; ++t) lds8(s_xn + t * kXnPad, off, x[t], j * 8);
  }
#pragma unroll
  for (int t = 0; t < TC; ++t) {
    if constexpr (PRE) {
      lane_x_offsets<QUANT>(x[t], xs[t]);
      continue;
    }
    float f[32];
    const int base = g.lane * 32;  // (lanes past the row's end fold zeros: fma(0, 0, s) == s)
#pragma unroll
    for (int j = 0; j < 4; ++j) lds8(s_xn + t * kXnPad, min(base, K - 32) + j * 8, f, j * 8);
    float sq = 0.0f;
#pragma unroll
    for (int i = 0; i < 32; ++i) sq = __builtin_fmaf(f[i], f[i], sq);
    if (base >= K) sq = 0.0f;
    const float inv = rms_finish(sq, K, eps);
#pragma unroll
    for (int i = 0; i < 32; ++i) x[t][i] = x[t][i] * inv * nw[i];
    lane_x_offsets<QUANT>(x[t], xs[t]);
  }
  // rows past the live-token count were computed from whatever the buffer held (in bounds, sized for max_tokens)
  // and are dropped
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
template <int SQ, int RF, int RPS, int kLogitsDepth, bool PRE = false>
__global__ void __launch_bounds__(256) k_decode_logits(DecodeArgs a) {
  __shared__ float s_red[4];
  __shared__ __attribute__((aligned(16))) float s_xn[3 * kXnPad];  // the chunk's rows and the norm weight
  const int chunks = (a.max_tokens + 1) / 2;
  const int n_r = chunks * a.tiles_r;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  if ((int)blockIdx.x >= a.max_tokens) {
    int item = blockIdx.x - a.max_tokens;
    const bool router = item < n_r;
    if (!router) item -= n_r;
    const int tiles = router ? a.tiles_r : a.tiles_s;
    const int c = item / tiles, tile = item % tiles, t0 = 2 * c;
    const int row0 = (tile * kWavesPerWg + wave) * RPS * kLogitsDepth;
    const float* x0 = (PRE ? a.normed : a.residual) + (size_t)t0 * a.H;
    if (t0 + 1 < a.max_tokens) {
      const float* const xr[2] = {x0, x0 + a.H};
      if (router) {
        float* const o[2] = {a.logits + (size_t)t0 * a.E, a.logits + (size_t)(t0 + 1) * a.E};
        tile_normed<RF, RPS, 2, 1, kLogitsDepth, PRE>(a.router, nullptr, a.H, a.E, row0, xr, a.post_norm, a.eps, o, a.logit_bias, a.valid_tokens, t0, s_xn);
      } else {
        float* const o[2] = {a.shared_inter + (size_t)t0 * a.I, a.shared_inter + (size_t)(t0 + 1) * a.I};
        tile_normed<SQ, RPS, 2, 2, kLogitsDepth, PRE>(a.sgate, a.sup, a.H, a.I, row0, xr, a.post_norm, a.eps, o, nullptr, a.valid_tokens, t0, s_xn);
      }
    } else {
      const float* const xr[1] = {x0};
      if (router) {
        float* const o[1] = {a.logits + (size_t)t0 * a.E};
        tile_normed<RF, RPS, 1, 1, kLogitsDepth, PRE>(a.router, nullptr, a.H, a.E, row0, xr, a.post_norm, a.eps, o, a.logit_bias, a.valid_tokens, t0, s_xn);
      } else {
        float* const o[1] = {a.shared_inter + (size_t)t0 * a.I};
        tile_normed<SQ, RPS, 1, 2, kLogitsDepth, PRE>(a.sgate, a.sup, a.H, a.I, row0, xr, a.post_norm, a.eps, o, nullptr, a.valid_tokens, t0, s_xn);
      }
    }
    return;
  }
  // the normalised row (callers read it back) and g = sigmoid(shared_gate_inp . normed): the order of
  // operations of the stand-alone RMSNorm and gate kernels
  const int t = blockIdx.x;
  const int valid = *a.valid_tokens;
  const float* xr = (PRE ? a.normed : a.residual) + (size_t)t * a.H;
  // hidden <= 2048: eight columns per thread, every load issued before the first use
  float xv[8], nv[8], gv[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int j = threadIdx.x + 256 * i;
    const bool in = j < a.H;
    xv[i] = in ? xr[j] : 0.0f;
    nv[i] = in && !PRE ? a.post_norm[j] : 0.0f;
    gv[i] = in ? a.shared_gate_inp[j] : 0.0f;
  }
  float inv = 1.0f;
  if constexpr (!PRE) inv = row_inv_rms(xr, a.H, a.eps);
  if (t >= valid) return;
  float s = 0.0f;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int j = threadIdx.x + 256 * i;
    if (j < a.H) {
      float v = xv[i];  // (PRE: the row is there already, written by the previous block's tail)
      if constexpr (!PRE) {
        v = xv[i] * inv * nv[i];
        a.normed[(size_t)t * a.H + j] = v;
      }
      s = __builtin_fmaf(gv[i], v, s);
    }
  }
  s = group_sum<64>(s);
  if ((threadIdx.x & 63) == 0) s_red[wave] = s;
  __syncthreads();
  const float total = ((s_red[0] + s_red[1]) + s_red[2]) + s_red[3];
  if (threadIdx.x == 0) a.gate_out[t] = 1.0f / (1.0f + expf(-total));
}

// ------------------------------------------------------------------------------------------------
// B: grid = max_tokens * top_k * tiles_g.  A tile is 4 wavefronts x DEPTH steps x RPS rows.
// ------------------------------------------------------------------------------------------------
// The routing launch of wider batches: one wavefront per token (route_one_token, the stand-alone routing kernel's
// body), one token per workgroup so that the tokens spread over the chip.
__global__ void __launch_bounds__(64) k_decode_route(DecodeArgs a) {
  extern __shared__ float s_route_one[];  // num_experts floats
  const int t = blockIdx.x;
  if (t >= *a.valid_tokens) return;
  int sel_i;
  float sel_w;
  route_one_token(a.logits + (size_t)t * a.E, a.E, a.top_k, s_route_one, sel_i, sel_w);
  if ((int)threadIdx.x < a.top_k) {
    a.topk_ids[(size_t)t * a.top_k + threadIdx.x] = sel_i;
    a.topk_weights[(size_t)t * a.top_k + threadIdx.x] = sel_w;
  }
}

// ROUTED: the token's selection was made by a routing launch between A and this one (wider batches: there a token's
// routing would otherwise be repeated by every one of its workgroups, several rounds of them per CU); the pair's
// expert then comes out of topk_ids through the scalar cache and nothing else of the routing runs here.
template <int RQ, int RPS, int DEPTH, bool ROUTED = false>
__global__ void __launch_bounds__(256) k_decode_up(DecodeArgs a) {
  using F = Fmt<RQ>;
  using Raw = typename F::Raw;
  constexpr int G = 64 / RPS;
  extern __shared__ float s_route[];  // num_experts floats for the routing wavefront
  __shared__ int s_expert, s_final;  // the candidate expert of this pair; the one routing settles on
  int p = blockIdx.x / a.tiles_g, tile = blockIdx.x % a.tiles_g;
  if (ROUTED && a.max_tokens >= kXcdGroupMinTokens && (a.tiles_g & 7) == 0) {
    // wide batches (see kXcdGroupMinTokens): all pairs of one row tile next to each other on one XCD
    const int n_pairs = a.max_tokens * a.top_k, xcd = blockIdx.x & 7, j = blockIdx.x >> 3;
    tile = xcd + 8 * (j / n_pairs);
    p = j % n_pairs;
  }
  const int t = p / a.top_k, k = p % a.top_k;
  [[maybe_unused]] int pre_e = 0;
  if constexpr (ROUTED) pre_e = a.topk_ids[p];
  // everything read before the live-token count is known is sized for max_tokens rows
  const int valid = *a.valid_tokens;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const LaneGeom g = lane_geom<RQ>();
  const int koff = lane_koff<RQ, RPS>(g, 0);
  // one wavefront routes the token (a different one in neighbouring workgroups, which share a CU); its
  // logits and every wavefront's copy of the normalised row are requested together
  const bool routes = !ROUTED && wave == (int)((blockIdx.x >> 8) & 3);
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
  // The pair's candidate is known after k + 1 selection rounds; the remaining rounds (the rest of the token's
  // selection and the k + 1-th candidate the verification needs) run after the rows have been requested.
  const int n_cand = min(a.top_k + 1, a.E);
  int cand_i = 0;
  int key[kRouteMaxPerLane];
  if (routes) {
    if (few) {
      route_keys<4>(*reinterpret_cast<float(*)[4]>(lg), a.E, *reinterpret_cast<int(*)[4]>(key));
      route_rounds<4>(*reinterpret_cast<int(*)[4]>(key), 0, k + 1, cand_i);
    } else {
      route_keys<kRouteMaxPerLane>(lg, a.E, key);
      route_rounds<kRouteMaxPerLane>(key, 0, k + 1, cand_i);
    }
    if (g.lane == k) s_expert = cand_i;
  }
  lane_x_offsets<RQ>(x[0], xs[0]);
  if constexpr (!ROUTED) __syncthreads();
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
        if (few) route_rounds<4>(*reinterpret_cast<int(*)[4]>(key), k + 1, n_cand, cand_i);
        else route_rounds<kRouteMaxPerLane>(key, k + 1, n_cand, cand_i);
        if (few) route_finish<4>(*reinterpret_cast<float(*)[4]>(lg), a.E, a.top_k, n_cand, cand_i, s_route, sel_i, sel_w, exact);
        else route_finish<kRouteMaxPerLane>(lg, a.E, a.top_k, n_cand, cand_i, s_route, sel_i, sel_w, exact);
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
      float tg[1] = {0.0f}, tu[1] = {0.0f};
      accum<RQ, 1>(r[d][0], g, x, xs, tg);
      accum<RQ, 1>(r[d][1], g, x, xs, tu);
      const float sg = group_sum<G>(tg[0]), su = group_sum<G>(tu[0]);
      const int row = wave_row0 + d * RPS + g.lane / G;
      if ((g.lane % G) == 0 && row < a.I) out[row] = silu_f(sg) * su;
    }
  };
  if constexpr (ROUTED) {
    stream_rows(min(max(pre_e, 0), a.E - 1), std::false_type{});
  } else {
    const int e = s_expert;
    stream_rows(e, std::true_type{});
    __syncthreads();  // s_final is there
    const int e_final = s_final;
    if (e_final != e) stream_rows(e_final, std::false_type{});  // (same rows of `inter`, written again)
  }
}

// ------------------------------------------------------------------------------------------------
// C: grid = max_tokens * tiles_d.  A workgroup is RS row steps (RPS rows each; K = intermediate = 2048 / RPS)
// x two wavefronts per step: the first takes the first half of the token's selections and the shared expert,
// the second the other half, so that a token's nine contractions per row step spread over twice as many
// wavefronts and every SIMD of the chip gets the same number of them (max_tokens x hidden / RPS x 2
// wavefronts: 12 per CU at three tokens).  The second wavefront hands its weighted row sums to the first
// through LDS, which adds all of them in selection order: the same operations as one wavefront would do.
// ------------------------------------------------------------------------------------------------
template <int RQ, int SQ, int RPS, int RS>
__global__ void __launch_bounds__(128 * RS) k_decode_down(DecodeArgs a) {
  using RawR = typename Fmt<RQ>::Raw;
  using RawS = typename Fmt<SQ>::Raw;
  constexpr int G = 64 / RPS;
  constexpr int kThreads = 128 * RS;
  constexpr int kHalf = kMaxTopK / 2;  // selections per wavefront
  __shared__ __attribute__((aligned(16))) float s_x[(kMaxTopK + 1) * kMaxInter];
  __shared__ float s_xs[(kMaxTopK + 1) * kMaxInter / 8];  // -32 * (sum of each run of eight), Q6_K's code offset
  __shared__ float s_part[RS][kHalf][RPS];               // the second wavefront's weighted row sums
  __shared__ int s_arrived;                              // the seam's tail: storing wavefronts of this workgroup that are done
  if (threadIdx.x == 0) s_arrived = 0;                   // (two barriers before anyone counts)
  int t = blockIdx.x / a.tiles_d, tile = blockIdx.x % a.tiles_d;
  if (a.max_tokens >= kXcdGroupMinTokens && (a.tiles_d & 7) == 0) {
    // wide batches (see kXcdGroupMinTokens): all tokens of one row tile next to each other on one XCD
    const int xcd = blockIdx.x & 7, j = blockIdx.x >> 3;
    tile = xcd + 8 * (j / a.max_tokens);
    t = j % a.max_tokens;
  }
  // every buffer read below is sized for max_tokens rows, so round one is issued before the live-token
  // count is known; rows past it hold an earlier pass's values or zeros, and nothing is stored for them
  const int valid = *a.valid_tokens;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int rs = wave >> 1, second = wave & 1;
  const int lane = __lane_id();
  const int row0 = (tile * RS + rs) * RPS;  // hidden is a multiple of RS * RPS
  // this wavefront's selections: [k0, k1)
  const int split = (a.top_k + 1) / 2;
  const int k0 = second ? split : 0, k1 = second ? a.top_k : split;
  // round one: selections (addressed uniformly, so they come through the scalar cache and arrive in the registers
  // the row addresses are formed from), gate scalar, the nine activation rows, the shared expert's rows
  int sel_e[kHalf];
  float sel_w[kHalf];
#pragma unroll
  for (int j = 0; j < kHalf; ++j) {
    const int kk = min(k0 + j, a.top_k - 1);
    sel_e[j] = a.topk_ids[(size_t)t * a.top_k + kk];
    sel_w[j] = a.topk_weights[(size_t)t * a.top_k + kk];
  }
  const float gate = a.gate_out[t];
  // a thread stages whole runs of eight consecutive activations (two 16-byte pieces): the run's sum is then
  // formed once per workgroup, in element order, instead of once per lane and selection
  constexpr int kRunsMax = (kMaxTopK + 1) * kMaxInter / 8;
  constexpr int kStage = (kRunsMax + kThreads - 1) / kThreads;
  float4 stage[kStage][2];
  const int runs_per_row = a.I / 8, n_runs = (a.top_k + 1) * runs_per_row;
  {
    const float4* src_r = reinterpret_cast<const float4*>(a.inter + (size_t)t * a.top_k * a.I);
    const float4* src_s = reinterpret_cast<const float4*>(a.shared_inter + (size_t)t * a.I);
#pragma unroll
    for (int j = 0; j < kStage; ++j) {
      const int i = threadIdx.x + kThreads * j;
      stage[j][0] = stage[j][1] = make_float4(0.f, 0.f, 0.f, 0.f);
      if (i < n_runs) {
        const float4* p = i < a.top_k * runs_per_row ? src_r + 2 * i : src_s + 2 * (i - a.top_k * runs_per_row);
        stage[j][0] = p[0];
        stage[j][1] = p[1];
      }
    }
  }
  const LaneGeom gs = lane_geom<SQ>();
  const LaneGeom gr = lane_geom<RQ>();
  const size_t rb_s = (size_t)(a.I / Fmt<SQ>::kBlockElems) * Fmt<SQ>::kBlockBytes;
  const size_t rb_r = (size_t)(a.I / Fmt<RQ>::kBlockElems) * Fmt<RQ>::kBlockBytes;
  RawS raw_s;
  if (!second) load_raw<SQ, true>(a.sdown + (size_t)row0 * rb_s, true, gs, raw_s);
  if (t >= valid) return;
  // round two: the selected experts' rows
  RawR rr[kHalf];
#pragma unroll
  for (int j = 0; j < kHalf; ++j) {
    const int e = min(max(sel_e[j], 0), a.E - 1);
    // j past this wavefront's share reads a selected expert's rows again and never uses them: an unconditional
    // load keeps all of round two in one basic block, so every load is issued before the first wait
    load_raw<RQ, true>(a.down + (size_t)e * a.down_bytes + (size_t)row0 * rb_r, true, gr, rr[j]);
  }
  // the activation rows arrived before the weights (loads return in order); publish them and their run sums
#pragma unroll
  for (int j = 0; j < kStage; ++j) {
    const int i = threadIdx.x + kThreads * j;
    if (i < n_runs) {
      reinterpret_cast<float4*>(s_x)[2 * i] = stage[j][0];
      reinterpret_cast<float4*>(s_x)[2 * i + 1] = stage[j][1];
      float sum = 0.0f;  // (the order of lane_x_offsets)
      sum += stage[j][0].x; sum += stage[j][0].y; sum += stage[j][0].z; sum += stage[j][0].w;
      sum += stage[j][1].x; sum += stage[j][1].y; sum += stage[j][1].z; sum += stage[j][1].w;
      s_xs[i] = -32.0f * sum;
    }
  }
  __syncthreads();
  // x[32] of one staged row for this lane, and (Q6_K) the four run sums that go with them
  auto lane_x = [&](auto quant_c, int slot, const LaneGeom& g, float (&x)[1][32], float (&xs)[1][4]) __attribute__((always_inline)) {
    constexpr int Q = decltype(quant_c)::value;
    const int koff = lane_koff<Q, RPS>(g, 0);
    lane_x_load<Q>(s_x + slot * a.I, koff, g, x[0]);
#pragma unroll
    for (int j = 0; j < 4; ++j)
      xs[0][j] = Q == kQ6K ? s_xs[slot * runs_per_row + (koff + g.half * 128 + j * 32 + g.l8 * 8) / 8] : 0.0f;
  };
  float part[kHalf];
#pragma unroll
  for (int j = 0; j < kHalf; ++j) {
    part[j] = 0.0f;
    if (k0 + j < k1) {
      float x[1][32], xs[1][4], tot[1] = {0.0f};
      lane_x(std::integral_constant<int, RQ>{}, k0 + j, gr, x, xs);
      accum<RQ, 1>(rr[j], gr, x, xs, tot);
      part[j] = sel_w[j] * group_sum<G>(tot[0]);
    }
  }
  const bool writes = (lane % G) == 0;
  if (second) {
    if (writes) {
#pragma unroll
      for (int j = 0; j < kHalf; ++j) s_part[rs][j][lane / G] = part[j];
    }
  }
  float sh = 0.0f;
  if (!second) {
    float x[1][32], xs[1][4], tot[1] = {0.0f};
    lane_x(std::integral_constant<int, SQ>{}, a.top_k, gs, x, xs);
    accum<SQ, 1>(raw_s, gs, x, xs, tot);
    sh = 1.0f * group_sum<G>(tot[0]);
  }
  __syncthreads();
  const int row = row0 + lane / G;
  if (!second && writes && row < a.H) {
    // the routed sum in selection order: this wavefront's share, then the other's
    float r = 0.0f;
#pragma unroll
    for (int j = 0; j < kHalf; ++j)
      if (j < k1) r += part[j];
#pragma unroll
    for (int j = 0; j < kHalf; ++j)
      if (split + j < a.top_k) r += s_part[rs][j][lane / G];
    const size_t i = (size_t)t * a.H + row;
    const float v = r + sh * gate;
    a.routed[i] = r;
    a.shexp[i] = sh;
    if (a.ffn_out) a.ffn_out[i] = v;
    const float lo = v + a.residual[i];
    // (with the seam on, another workgroup of this launch reads the row back: the store goes through to memory)
    if (a.next_normed) __hip_atomic_store(a.l_out + i, lo, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else a.l_out[i] = lo;
  }
  if (!a.next_normed) return;
  // The seam (docs/BENCHMARKS.md:1376 of the reference: the next layer's RMSNorm in the combine's tail).  A token's
  // row is finished by tiles_d workgroups, and the wavefront that finishes it last applies the norm.  Arrivals are
  // counted in three levels so that no counter sees more than a few dozen of them (atomics on one address are served
  // one after the other, ~70 ns each: 256 arrivals on one counter cost 18 us per pass at 32 tokens): the storing
  // wavefronts of a workgroup in LDS, 16 workgroups on a group counter, the groups on the token's counter, every
  // counter on a 128-byte line of its own.  A wavefront counts itself once its own stores are acknowledged (they go
  // through to memory: no fence, whose L2 write-back costs microseconds here), so whoever sees a count complete knows
  // all stores below it have landed.  No workgroup barrier: the other wavefronts are done.
  if (second) return;
  __builtin_amdgcn_s_waitcnt(0);
  int prev = 0;
  if (lane == 0) prev = __hip_atomic_fetch_add(&s_arrived, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  if (__builtin_amdgcn_readfirstlane(prev) != RS - 1) return;
  int* const token_ctr = a.arrivals + (size_t)t * kSeamCountersPerToken * kSeamCounterStride;
  const int groups = (a.tiles_d + kSeamGroup - 1) / kSeamGroup, grp = tile / kSeamGroup;
  const int in_group = min(kSeamGroup, a.tiles_d - grp * kSeamGroup);
  int* const group_ctr = token_ctr + (1 + grp) * kSeamCounterStride;
  if (lane == 0) prev = __hip_atomic_fetch_add(group_ctr, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if (__builtin_amdgcn_readfirstlane(prev) != in_group - 1) return;
  if (lane == 0) {
    __hip_atomic_store(group_ctr, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // (zero again for the next pass)
    prev = __hip_atomic_fetch_add(token_ctr, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  if (__builtin_amdgcn_readfirstlane(prev) != groups - 1) return;
  if (lane == 0) __hip_atomic_store(token_ctr, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  // the row comes in coalesced (element 64 j + lane per load) and changes hands through LDS (s_x is free now), padded
  // by four floats per 32 as the first launch pads its rows
  float* s_l = s_x;  // (free since the last barrier; one wavefront per workgroup at most gets here: a workgroup serves one token)
  const float* lrow = a.l_out + (size_t)t * a.H;
  float in[32];
#pragma unroll
  for (int j = 0; j < 32; ++j) {
    const int e = 64 * j + lane;
    in[j] = e < a.H ? __hip_atomic_load(lrow + e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0.0f;
  }
#pragma unroll
  for (int j = 0; j < 32; ++j) s_l[xn_at(64 * j + lane)] = in[j];
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  RmsRaw rowq;
#pragma unroll
  for (int j = 0; j < 8; ++j) rowq.q[j] = *reinterpret_cast<const float4*>(s_l + xn_at(32 * lane + 4 * j));
  const float inv = rms_finish(rms_fold(rowq, 0.0f), a.H, a.next_eps);
  // out the same way: element 64 j + lane, (x * inv) * w
#pragma unroll
  for (int j = 0; j < 32; ++j) {
    const int e = 64 * j + lane;
    if (e < a.H) {
      const float v = in[j] * inv * a.next_w[e];
      a.next_normed[(size_t)t * a.H + e] = v;
      if (a.next_normed_h) a.next_normed_h[(size_t)t * a.H + e] = (_Float16)v;
    }
  }
}

// ------------------------------------------------------------------ host side
struct Launch {
  const DecodeArgs& a;
  hipStream_t s;
  unsigned grid_a, grid_b, grid_c;
  bool pre_routed;  // a routing launch between A and B instead of routing inside B
  bool pre_normed;  // `normed` holds this pass's rows already (the previous block's tail): A neither normalises nor writes them
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
#define XABE_A1(SQ, RF, PRE)                                                                                        \
  do {                                                                                                            \
    const int da = logits_depth(l.a.max_tokens);                                                                  \
    if (da == 1) hipLaunchKernelGGL((k_decode_logits<SQ, RF, RPSH, 1, PRE>), dim3(l.grid_a), dim3(256), 0, l.s, l.a);  \
    else if (da == 2) hipLaunchKernelGGL((k_decode_logits<SQ, RF, RPSH, 2, PRE>), dim3(l.grid_a), dim3(256), 0, l.s, l.a); \
    else hipLaunchKernelGGL((k_decode_logits<SQ, RF, RPSH, 4, PRE>), dim3(l.grid_a), dim3(256), 0, l.s, l.a);     \
  } while (0)
#define XABE_A(SQ, RF)                  \
  do {                                  \
    if (l.pre_normed) XABE_A1(SQ, RF, true); \
    else XABE_A1(SQ, RF, false);        \
  } while (0)
    if (sg6 && rf32) XABE_A(kQ6K, kF32);
    else if (sg6) XABE_A(kQ6K, kQ8_0);
    else if (rf32) XABE_A(kQ8_0, kF32);
    else XABE_A(kQ8_0, kQ8_0);
#undef XABE_A
#undef XABE_A1
  }
  if (l.launches & 2u) {
    if (l.pre_routed) {
      hipLaunchKernelGGL(k_decode_route, dim3((unsigned)l.a.max_tokens), dim3(64), l.route_lds, l.s, l.a);
      if (g6) hipLaunchKernelGGL((k_decode_up<kQ6K, RPSH, DEPTH, true>), dim3(l.grid_b), dim3(256), 0, l.s, l.a);
      else hipLaunchKernelGGL((k_decode_up<kQ8_0, RPSH, DEPTH, true>), dim3(l.grid_b), dim3(256), 0, l.s, l.a);
    } else if (g6) hipLaunchKernelGGL((k_decode_up<kQ6K, RPSH, DEPTH>), dim3(l.grid_b), dim3(256), l.route_lds, l.s, l.a);
    else hipLaunchKernelGGL((k_decode_up<kQ8_0, RPSH, DEPTH>), dim3(l.grid_b), dim3(256), l.route_lds, l.s, l.a);
  }
  if (l.launches & 4u) {
#define XABE_C(RQ, SQ)                                                                                            \
  do {                                                                                                          \
    hipLaunchKernelGGL((k_decode_down<RQ, SQ, RPSI, kDownSteps>), dim3(l.grid_c), dim3(128 * kDownSteps), 0, l.s, l.a); \
  } while (0)
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

size_t seam_counter_ints_per_token() { return (size_t)kSeamCountersPerToken * kSeamCounterStride; }

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
                        float* shexp, float* gate_out, float* routed, float* ffn_out, float* l_out, unsigned launches,
                        const DecodeSeam* seam) {
  const xabe_moe_geometry& g = k->g;
  DecodeArgs a;
  memset(&a, 0, sizeof(a));
  if (seam && seam->next_normed) {
    if (!b->seam_arrivals || b->n_seam_arrivals < g.max_tokens * seam_counter_ints_per_token())
      return set_error(XABE_ERR_INVALID_ARGUMENT, "decode block: these buffers carry no arrival counters for the seam");
    a.next_w = seam->next_w;
    a.next_normed = seam->next_normed;
    a.next_normed_h = static_cast<_Float16*>(seam->next_normed_h);
    a.next_eps = seam->next_eps;
    a.arrivals = b->seam_arrivals;
  }
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
  const int down_steps = kDownSteps;
  a.tiles_d = (a.H + down_steps * rps_i - 1) / (down_steps * rps_i);
  if (a.E % rps_h != 0 || a.I % (kWavesPerWg * depth * rps_h) != 0 || a.H % (down_steps * rps_i) != 0)
    return set_error(XABE_ERR_UNSUPPORTED_GEOMETRY, "decode block: %d experts / %d intermediate rows do not fill whole steps of %d rows",
                     a.E, a.I, rps_h);
  const int chunks = (a.max_tokens + 1) / 2;
  const bool pre_routed = a.max_tokens >= kPreRouteMinTokens;
  Launch l{a, s, 0, 0, 0, pre_routed, seam && seam->input_normed, g.num_experts * sizeof(float), launches};
  l.grid_a = (unsigned)(chunks * (a.tiles_r + a.tiles_s) + a.max_tokens);
  l.grid_b = (unsigned)(a.max_tokens * a.top_k * a.tiles_g);
  l.grid_c = (unsigned)(a.max_tokens * a.tiles_d);
  const bool ok = launch_shape(l, w->gate_exps.quant, w->down_exps.quant, w->shared_gate.quant, w->shared_down.quant, w->router_quant);
  if (!ok) return set_error(XABE_ERR_UNSUPPORTED_GEOMETRY, "decode block: no kernels for this shape or format");
  XABE_HIP_TRY(hipGetLastError());
  return XABE_OK;
}

}  // namespace xabe

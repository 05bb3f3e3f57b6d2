/*
 * CPU oracle for the quantized MoE feed-forward block: TEST INFRASTRUCTURE ONLY.
 * See xabe_oracle.h.  Nothing shipped links this file.
 *
 * Reference paths below are relative to the reference tree's root.
 * "K" = crates/xabe-kernels/src.
 *
 * What pins each function besides this restatement (tests/test_oracle_*.py):
 *   xo_rng_*             K/rng.rs:20-55      closed form vs Python big-int arithmetic; zero-seed remap
 *   xo_to_f16_bits etc.  K/f16.rs:17-100     numpy float16 over all 65536 patterns + random f32 (RNE, subnormals)
 *   xo_dequantize_q6_k   K/quant.rs:171-202  hand-built superblock (quant.rs:689-711), independent vectorised numpy
 *                                            re-derivation from the block_q6_K struct, group-partition test
 *   xo_dequantize_q8_0   K/quant.rs:62-69    [0xFF;34] => all -1 (quant.rs:1339-1347), numpy re-derivation
 *   xo_quantize_q8_0     K/quant.rs:75-88    zero block, saturation 10 -> 127, step/2 bound (quant.rs:576-615);
 *                                            exact bytes on arbitrary input: PARITY UNPINNED (only the formula)
 *   xo_quantize_q6_k     K/quant.rs:495-567  zero block, round trip < 0.35 / cos > 0.999 on seed 2 (quant.rs:618-640),
 *                                            to_bytes layout (quant.rs:1297-1337);
 *                                            exact bytes on arbitrary input: PARITY UNPINNED (only the formula)
 *   xo_rms_norm, silu... K/norm.rs:28-143    hand values (norm.rs:152-351), float64 numpy within 1e-6
 *   xo_gemv              K/gemv.rs:44-58     [[1,2,3],[4,5,6]].[1,10,100] = [321,654]; the 2^24 accumulator test
 *   xo_route_token       K/moe/router.rs:32-76  reference vectors (router.rs:88-181); brute-force full sort;
 *                                            behaviour at exact probability ties created by libm expf rounding:
 *                                            PARITY UNPINNED (platform libm)
 *   xo_moe_align_block_size K/moe/dispatch.rs:60-131  vLLM docstring table (dispatch.rs:138-169) + invariants
 *   xo_expert_mlp, naive, grouped  K/moe/gemm.rs:25-125  grouped == naive, single expert == expert_mlp,
 *                                            zero weight => zero (gemm.rs:154-266); float64 numpy bound
 *   xo_compare           K/compare.rs:67-135 hand cases
 *   xo_sorted_capacity.. xabe-cuda kernels/moe.rs:4556-4598  reference-held values (moe.rs:6921-6989), brute force
 *   xo_quantize_rows_q8  xabe-cuda kernels/mma.rs:118-157  closed forms (exact factor, ties to even, zero and
 *                                            negative blocks), numpy restatement
 *   xo_moe_block_forward xabe-engine block/moe.rs:12-25  composition order: PARITY UNPINNED except by algebraic
 *                                            self-checks ((ffn_out-routed)/shexp == gate, l_out-ffn_out == residual);
 *                                            the reference's behavioural pin is a llama.cpp capture that is not
 *                                            in the tree
 *   xo_synth_*           no reference counterpart (this build's input definition)
 */
#include "xabe_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ===================================================================== */
/* rng.rs:20-55                                                           */
/* ===================================================================== */
void xo_rng_new(xo_rng* r, uint64_t seed) { r->state = seed == 0 ? 0x9E3779B97F4A7C15ull : seed; }

uint64_t xo_rng_next_u64(xo_rng* r) {
  uint64_t x = r->state;
  x ^= x >> 12;
  x ^= x << 25;
  x ^= x >> 27;
  r->state = x;
  return x * 0x2545F4914F6CDD1Dull;
}

float xo_rng_next_f32(xo_rng* r) { return (float)(xo_rng_next_u64(r) >> 40) / (float)(1ull << 24); }

float xo_rng_next_f32_range(xo_rng* r, float low, float high) { return low + xo_rng_next_f32(r) * (high - low); }

uint32_t xo_rng_next_u32_below(xo_rng* r, uint32_t bound) { return (uint32_t)(xo_rng_next_u64(r) % (uint64_t)bound); }

void xo_rng_vec_f32(xo_rng* r, size_t n, float low, float high, float* out) {
  for (size_t i = 0; i < n; ++i) out[i] = xo_rng_next_f32_range(r, low, high);
}

/* ===================================================================== */
/* f16.rs:17-100 (same rounding as half::f16::from_f32, the crate quant.rs uses) */
/* ===================================================================== */
static uint32_t f32_bits(float x) { uint32_t b; memcpy(&b, &x, 4); return b; }
static float bits_f32(uint32_t b) { float x; memcpy(&x, &b, 4); return x; }

uint16_t xo_to_f16_bits(float x) {
  uint32_t b = f32_bits(x);
  uint16_t sign = (uint16_t)((b >> 16) & 0x8000u);
  int32_t biased = (int32_t)((b >> 23) & 0xffu);
  uint32_t mant = b & 0x007fffffu;
  if (biased == 0xff) return (uint16_t)(sign | 0x7c00u | (mant != 0 ? 0x0200u : 0u));
  int32_t e = biased - 127 + 15;
  if (e >= 0x1f) return (uint16_t)(sign | 0x7c00u);
  if (e <= 0) {
    if (e < -10) return sign;
    uint32_t full = mant | 0x00800000u;
    uint32_t shift = (uint32_t)(14 - e);
    uint32_t half = 1u << (shift - 1);
    uint32_t sticky = full & (half - 1);
    uint32_t r = full >> shift;
    if ((full & half) != 0 && (sticky != 0 || (r & 1u) != 0)) r += 1;
    return (uint16_t)(sign | (uint16_t)r);
  }
  uint32_t half = 1u << 12;
  uint32_t sticky = mant & (half - 1);
  uint32_t m = mant >> 13;
  if ((mant & half) != 0 && (sticky != 0 || (m & 1u) != 0)) {
    m += 1;
    if (m == 0x400u) {
      m = 0;
      e += 1;
      if (e >= 0x1f) return (uint16_t)(sign | 0x7c00u);
    }
  }
  return (uint16_t)(sign | ((uint16_t)e << 10) | (uint16_t)m);
}

float xo_from_f16_bits(uint16_t h) {
  uint32_t sign = ((uint32_t)(h & 0x8000u)) << 16;
  uint32_t e = (h >> 10) & 0x1fu;
  uint32_t mant = h & 0x03ffu;
  if (e == 0) {
    if (mant == 0) return bits_f32(sign);
    uint32_t m = mant;
    int32_t ee = -1;
    while ((m & 0x400u) == 0) { m <<= 1; ee -= 1; }
    uint32_t e32 = (uint32_t)(ee + 1 - 14 + 127);
    return bits_f32(sign | (e32 << 23) | ((m & 0x3ffu) << 13));
  }
  if (e == 0x1f) return bits_f32(sign | 0x7f800000u | (mant << 13));
  return bits_f32(sign | ((e + 127 - 15) << 23) | (mant << 13));
}

/* ===================================================================== */
/* quant.rs                                                               */
/* ===================================================================== */
/* Rust `x as i8` from f32: saturating, NaN -> 0. */
static int8_t sat_i8(float v) {
  if (v != v) return 0;
  if (v <= -128.0f) return -128;
  if (v >= 127.0f) return 127;
  return (int8_t)v;
}
static float clampf(float v, float lo, float hi) { return v < lo ? lo : (v > hi ? hi : v); }

/* quant.rs:75-88 */
void xo_quantize_q8_0(const float* x, uint8_t* out) {
  float amax = 0.0f;
  for (int j = 0; j < XO_QK8_0; ++j) amax = fmaxf(amax, fabsf(x[j]));
  float d = amax / 127.0f;
  float inv_d = d != 0.0f ? 1.0f / d : 0.0f;
  uint16_t dh = xo_to_f16_bits(d);
  out[0] = (uint8_t)(dh & 0xff);
  out[1] = (uint8_t)(dh >> 8);
  for (int j = 0; j < XO_QK8_0; ++j) out[2 + j] = (uint8_t)sat_i8(roundf(x[j] * inv_d));
}

/* quant.rs:62-69, from_bytes quant.rs:762-776 */
void xo_dequantize_q8_0(const uint8_t* in, float* y) {
  float d = xo_from_f16_bits((uint16_t)(in[0] | (in[1] << 8)));
  for (int j = 0; j < XO_QK8_0; ++j) y[j] = (float)(int8_t)in[2 + j] * d;
}

/* quant.rs:171-202, from_bytes quant.rs:797-820 */
void xo_dequantize_q6_k(const uint8_t* in, float* y) {
  const uint8_t* ql_all = in;
  const uint8_t* qh_all = in + 128;
  const int8_t* sc_all = (const int8_t*)(in + 192);
  float d = xo_from_f16_bits((uint16_t)(in[208] | (in[209] << 8)));
  for (int half = 0; half < 2; ++half) {
    int y_off = half * 128;
    const uint8_t* ql = ql_all + half * 64;
    const uint8_t* qh = qh_all + half * 32;
    const int8_t* sc = sc_all + half * 8;
    for (int l = 0; l < 32; ++l) {
      int is = l / 16;
      uint8_t raw1 = (uint8_t)((ql[l] & 0xF) | ((qh[l] & 3) << 4));
      uint8_t raw2 = (uint8_t)((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4));
      uint8_t raw3 = (uint8_t)((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4));
      uint8_t raw4 = (uint8_t)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4));
      int q1 = (int)raw1 - 32, q2 = (int)raw2 - 32, q3 = (int)raw3 - 32, q4 = (int)raw4 - 32;
      /* `d * sc * q` is left-associative: (d*sc)*q, each product rounded. */
      y[y_off + l] = d * (float)sc[is] * (float)q1;
      y[y_off + l + 32] = d * (float)sc[is + 2] * (float)q2;
      y[y_off + l + 64] = d * (float)sc[is + 4] * (float)q3;
      y[y_off + l + 96] = d * (float)sc[is + 6] * (float)q4;
    }
  }
}

/* quant.rs:495-567 (group addressing quant.rs:208-217), to_bytes quant.rs:826-839 */
void xo_quantize_q6_k(const float* x, uint8_t* out) {
  float global_amax = 0.0f;
  for (int i = 0; i < XO_QK_K; ++i) global_amax = fmaxf(global_amax, fabsf(x[i]));
  float d = global_amax > 0.0f ? global_amax / (32.0f * 127.0f) : 0.0f;
  uint8_t* ql = out;
  uint8_t* qh = out + 128;
  int8_t* scales = (int8_t*)(out + 192);
  memset(out, 0, XO_BLOCK_Q6_K_BYTES);
  for (int half = 0; half < 2; ++half)
    for (int lane = 0; lane < 4; ++lane)
      for (int is = 0; is < 2; ++is) {
        int scale_index = half * 8 + lane * 2 + is;
        int y_off = half * 128 + lane * 32;
        int l_start = is * 16;
        float group_amax = 0.0f;
        for (int k = 0; k < 16; ++k) group_amax = fmaxf(group_amax, fabsf(x[y_off + l_start + k]));
        int8_t sc = 0;
        if (d > 0.0f) sc = sat_i8(clampf(roundf(group_amax / (d * 32.0f)), 0.0f, 127.0f));
        scales[scale_index] = sc;
        float denom = d * (float)sc;
        for (int k = 0; k < 16; ++k) {
          int pos = y_off + l_start + k;
          int l = l_start + k;
          int code = 0;
          if (denom != 0.0f) code = (int)clampf(roundf(x[pos] / denom), -32.0f, 31.0f);
          uint8_t raw = (uint8_t)(code + 32);
          qh[half * 32 + l] |= (uint8_t)((raw >> 4) << (lane * 2));
          int ql_index = (lane & 1) ? l + 32 : l;
          int nibble_high = lane >= 2;
          uint8_t low4 = raw & 0xF;
          if (nibble_high) ql[half * 64 + ql_index] |= (uint8_t)(low4 << 4);
          else ql[half * 64 + ql_index] |= low4;
        }
      }
  uint16_t dh = xo_to_f16_bits(d);
  out[208] = (uint8_t)(dh & 0xff);
  out[209] = (uint8_t)(dh >> 8);
}

size_t xo_block_bytes(int quant) { return quant == XO_Q6K ? XO_BLOCK_Q6_K_BYTES : XO_BLOCK_Q8_0_BYTES; }
size_t xo_block_elements(int quant) { return quant == XO_Q6K ? XO_QK_K : XO_QK8_0; }

/* quant.rs:950-983 */
int xo_dequantize_row(int quant, const uint8_t* bytes, size_t len, float* out) {
  size_t bb = xo_block_bytes(quant), be = xo_block_elements(quant);
  if (len % bb != 0) return -1;
  size_t n = len / bb;
  for (size_t b = 0; b < n; ++b) {
    if (quant == XO_Q6K) xo_dequantize_q6_k(bytes + b * bb, out + b * be);
    else xo_dequantize_q8_0(bytes + b * bb, out + b * be);
  }
  return 0;
}

int xo_quantize_row(int quant, const float* x, size_t n, uint8_t* out) {
  size_t bb = xo_block_bytes(quant), be = xo_block_elements(quant);
  if (n % be != 0) return -1;
  size_t nb = n / be;
#pragma omp parallel for schedule(static)
  for (size_t b = 0; b < nb; ++b) {
    if (quant == XO_Q6K) xo_quantize_q6_k(x + b * be, out + b * bb);
    else xo_quantize_q8_0(x + b * be, out + b * bb);
  }
  return 0;
}

/* ===================================================================== */
/* norm.rs                                                                */
/* ===================================================================== */
/* Rust's `Iterator::sum::<f32>()` folds from -0.0. */
#define XO_SUM_INIT (-0.0f)

/* norm.rs:28-43 */
void xo_rms_norm(const float* x, const float* weight, size_t n, float eps, float* y) {
  float ss = XO_SUM_INIT;
  for (size_t i = 0; i < n; ++i) ss += x[i] * x[i];
  float mean_sq = ss / (float)n;
  float inv_rms = 1.0f / sqrtf(mean_sq + eps);
  for (size_t i = 0; i < n; ++i) y[i] = x[i] * inv_rms * weight[i];
}
/* norm.rs:46-48 */
float xo_silu(float x) { return x / (1.0f + expf(-x)); }
/* norm.rs:58-60 */
float xo_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }
/* norm.rs:93-103 */
void xo_swiglu(const float* gate, const float* up, size_t n, float* out) {
  for (size_t i = 0; i < n; ++i) out[i] = xo_silu(gate[i]) * up[i];
}
/* norm.rs:119-129 */
void xo_sigmoid_gate(const float* x, const float* gate, size_t n, float* out) {
  for (size_t i = 0; i < n; ++i) out[i] = x[i] * xo_sigmoid(gate[i]);
}
/* norm.rs:136-143 */
void xo_residual_add(const float* a, const float* b, size_t n, float* out) {
  for (size_t i = 0; i < n; ++i) out[i] = a[i] + b[i];
}

/* ===================================================================== */
/* gemv.rs:44-58 and moe/gemm.rs:25-34 (same body)                         */
/* ===================================================================== */
static inline float dot_seq(const float* w, const float* x, size_t n) {
  float s = XO_SUM_INIT;
  for (size_t i = 0; i < n; ++i) s += w[i] * x[i];
  return s;
}
void xo_gemv(const float* weight, size_t out_dim, size_t in_dim, const float* x, float* out) {
  for (size_t o = 0; o < out_dim; ++o) out[o] = dot_seq(weight + o * in_dim, x, in_dim);
}
/* gemv.rs:103-112 */
size_t xo_argmax(const float* v, size_t n) {
  size_t best = 0;
  for (size_t i = 1; i < n; ++i)
    if (v[i] > v[best]) best = i;
  return best;
}

/* ===================================================================== */
/* moe/router.rs:32-81                                                    */
/* ===================================================================== */
typedef struct { uint32_t idx; float p; } ranked_t;

/* The reference sorts (index, prob) by (-prob, index) with a stable sort.
 * Insertion sort is stable and applies the same comparator, including its
 * "incomparable (NaN) counts as equal, then index" rule. */
static int ranked_less(const ranked_t* a, const ranked_t* b) {
  /* b.1.partial_cmp(&a.1).unwrap_or(Equal).then(a.0.cmp(&b.0)) == Less */
  if (b->p < a->p) return 1;  /* b.p < a.p  => Ordering::Less: a first */
  if (b->p > a->p) return 0;
  return a->idx < b->idx;    /* equal or incomparable */
}

int xo_route_token(const float* logits, size_t n, size_t k, uint32_t* expert_ids, float* weights) {
  if (n == 0 || k == 0 || k > n) return -1;
  float max_logit = -INFINITY;
  for (size_t i = 0; i < n; ++i) max_logit = fmaxf(max_logit, logits[i]);
  float* e = (float*)malloc(n * sizeof(float));
  ranked_t* ranked = (ranked_t*)malloc(n * sizeof(ranked_t));
  float sum_exp = XO_SUM_INIT;
  for (size_t i = 0; i < n; ++i) { e[i] = expf(logits[i] - max_logit); }
  for (size_t i = 0; i < n; ++i) sum_exp += e[i];
  for (size_t i = 0; i < n; ++i) { ranked[i].idx = (uint32_t)i; ranked[i].p = e[i] / sum_exp; }
  for (size_t i = 1; i < n; ++i) {
    ranked_t key = ranked[i];
    size_t j = i;
    while (j > 0 && ranked_less(&key, &ranked[j - 1])) { ranked[j] = ranked[j - 1]; --j; }
    ranked[j] = key;
  }
  float selected_sum = XO_SUM_INIT;
  for (size_t i = 0; i < k; ++i) selected_sum += ranked[i].p;
  for (size_t i = 0; i < k; ++i) {
    expert_ids[i] = ranked[i].idx;
    weights[i] = selected_sum > 0.0f ? ranked[i].p / selected_sum : 1.0f / (float)k;
  }
  free(e);
  free(ranked);
  return 0;
}

int xo_route_batch(const float* logits, size_t tokens, size_t n, size_t k, uint32_t* expert_ids, float* weights) {
  for (size_t t = 0; t < tokens; ++t)
    if (xo_route_token(logits + t * n, n, k, expert_ids + t * k, weights + t * k) != 0) return -1;
  return 0;
}

/* ===================================================================== */
/* moe/dispatch.rs:60-131                                                 */
/* ===================================================================== */
int xo_moe_align_block_size(const uint32_t* topk_ids, size_t tokens, size_t top_k, size_t block_size,
                            size_t num_experts, uint32_t* sorted_token_ids, int32_t* expert_ids,
                            size_t* num_tokens_post_pad) {
  if (block_size == 0) return -1;
  size_t numel = tokens * top_k;
  for (size_t i = 0; i < numel; ++i)
    if (topk_ids[i] >= num_experts) return -1;
  uint32_t* counts = (uint32_t*)calloc(num_experts, sizeof(uint32_t));
  uint32_t* cumsum = (uint32_t*)calloc(num_experts + 1, sizeof(uint32_t));
  uint32_t* running = (uint32_t*)calloc(num_experts, sizeof(uint32_t));
  for (size_t i = 0; i < numel; ++i) counts[topk_ids[i]] += 1;
  for (size_t e = 0; e < num_experts; ++e) {
    uint32_t padded = (uint32_t)((counts[e] + block_size - 1) / block_size * block_size);
    cumsum[e + 1] = cumsum[e] + padded;
  }
  size_t post_pad = cumsum[num_experts];
  uint32_t sentinel = (uint32_t)numel;
  for (size_t i = 0; i < post_pad; ++i) sorted_token_ids[i] = sentinel;
  for (size_t i = 0; i < numel; ++i) {
    uint32_t e = topk_ids[i];
    sorted_token_ids[cumsum[e] + running[e]] = (uint32_t)i;
    running[e] += 1;
  }
  size_t num_blocks = post_pad / block_size;
  for (size_t b = 0; b < num_blocks; ++b) expert_ids[b] = -1;
  for (size_t e = 0; e < num_experts; ++e) {
    size_t first = cumsum[e] / block_size, last = cumsum[e + 1] / block_size;
    for (size_t b = first; b < last; ++b) expert_ids[b] = (int32_t)e;
  }
  *num_tokens_post_pad = post_pad;
  free(counts);
  free(cumsum);
  free(running);
  return 0;
}

/* ===================================================================== */
/* moe/gemm.rs                                                            */
/* ===================================================================== */
/* gemm.rs:37-47 */
void xo_expert_mlp(const float* gate, const float* up, const float* down, const float* x, size_t hidden,
                   size_t intermediate, float* out) {
  float* g = (float*)malloc(intermediate * sizeof(float));
  float* u = (float*)malloc(intermediate * sizeof(float));
  xo_gemv(gate, intermediate, hidden, x, g);
  xo_gemv(up, intermediate, hidden, x, u);
  xo_swiglu(g, u, intermediate, g);
  xo_gemv(down, hidden, intermediate, g, out);
  free(g);
  free(u);
}

/* gemm.rs:102-125 */
void xo_naive_forward(const float* hidden_states, size_t tokens, const uint32_t* expert_ids, const float* weights,
                      size_t top_k, const float* gate, const float* up, const float* down, size_t hidden,
                      size_t intermediate, float* out) {
  size_t mat = hidden * intermediate;
  float* c = (float*)malloc(hidden * sizeof(float));
  for (size_t t = 0; t < tokens; ++t) {
    float* acc = out + t * hidden;
    for (size_t i = 0; i < hidden; ++i) acc[i] = 0.0f;
    for (size_t k = 0; k < top_k; ++k) {
      size_t e = expert_ids[t * top_k + k];
      float w = weights[t * top_k + k];
      xo_expert_mlp(gate + e * mat, up + e * mat, down + e * mat, hidden_states + t * hidden, hidden, intermediate, c);
      for (size_t i = 0; i < hidden; ++i) acc[i] += w * c[i];
    }
  }
  free(c);
}

/* gemm.rs:58-98 */
void xo_grouped_forward(const float* hidden_states, size_t tokens, const uint32_t* sorted_token_ids,
                        const int32_t* expert_block_ids, size_t num_blocks, size_t block_size,
                        const float* flat_weights, size_t top_k, const float* gate, const float* up,
                        const float* down, size_t hidden, size_t intermediate, float* out) {
  size_t mat = hidden * intermediate;
  uint32_t sentinel = (uint32_t)(tokens * top_k);
  float* c = (float*)malloc(hidden * sizeof(float));
  for (size_t i = 0; i < tokens * hidden; ++i) out[i] = 0.0f;
  for (size_t b = 0; b < num_blocks; ++b) {
    int32_t e = expert_block_ids[b];
    if (e == -1) continue;
    for (size_t slot = b * block_size; slot < (b + 1) * block_size; ++slot) {
      uint32_t flat = sorted_token_ids[slot];
      if (flat == sentinel) continue;
      size_t t = flat / top_k;
      float w = flat_weights[flat];
      xo_expert_mlp(gate + (size_t)e * mat, up + (size_t)e * mat, down + (size_t)e * mat, hidden_states + t * hidden,
                    hidden, intermediate, c);
      float* o = out + t * hidden;
      for (size_t i = 0; i < hidden; ++i) o[i] += w * c[i];
    }
  }
  free(c);
}

/* ===================================================================== */
/* compare.rs:67-135                                                      */
/* ===================================================================== */
int xo_compare(const float* c, const float* r, size_t n, xo_comparison* out) {
  if (n == 0) return -1;
  const float REL_EPS = 1e-6f;
  memset(out, 0, sizeof(*out));
  double dot = 0.0, nc = 0.0, nr = 0.0;
  for (size_t i = 0; i < n; ++i) {
    if (!isfinite(c[i])) { out->non_finite_count += 1; continue; }
    float abs_err = fabsf(c[i] - r[i]);
    if (abs_err > out->max_abs_error) { out->max_abs_error = abs_err; out->max_abs_error_index = i; }
    float rel = abs_err / fmaxf(fabsf(r[i]), REL_EPS);
    if (rel > out->max_rel_error) { out->max_rel_error = rel; out->max_rel_error_index = i; }
    dot += (double)c[i] * (double)r[i];
    nc += (double)c[i] * (double)c[i];
    nr += (double)r[i] * (double)r[i];
  }
  double denom = sqrt(nc) * sqrt(nr);
  if (denom > 0.0) out->cosine_similarity = (float)(dot / denom);
  else out->cosine_similarity = (nc == 0.0 && nr == 0.0) ? 1.0f : 0.0f;
  out->len = n;
  return 0;
}

/* ===================================================================== */
/* xabe-cuda kernels/moe.rs:4556-4598                                     */
/* ===================================================================== */
size_t xo_max_flat_pairs(size_t max_tokens, size_t top_k) { return max_tokens * top_k; }
size_t xo_sorted_capacity(size_t num_experts, size_t top_k, size_t block_size, size_t max_tokens) {
  size_t numel = max_tokens * top_k;
  size_t active = num_experts < numel ? num_experts : numel;
  size_t bound = numel + active * (block_size - 1);
  return (bound + block_size - 1) / block_size * block_size;
}
size_t xo_expert_block_capacity(size_t num_experts, size_t top_k, size_t block_size, size_t max_tokens) {
  return xo_sorted_capacity(num_experts, top_k, block_size, max_tokens) / block_size;
}

/* ===================================================================== */
/* xabe-cuda kernels/mma.rs:118-157                                       */
/* ===================================================================== */
void xo_quantize_rows_q8(const float* x, size_t rows, size_t k, int8_t* q, float* scales) {
  size_t blocks = k / 32;
  for (size_t r = 0; r < rows; ++r)
    for (size_t b = 0; b < blocks; ++b) {
      const float* v = x + r * k + b * 32;
      float a = 0.0f;
      for (int i = 0; i < 32; ++i) a = fmaxf(a, fabsf(v[i]));
      float d = a > 0.0f ? a / 127.0f : 1.0f;
      float inv = a > 0.0f ? 127.0f / a : 0.0f;
      for (int i = 0; i < 32; ++i) {
        int qi = (int)rintf(v[i] * inv);
        qi = qi < -127 ? -127 : (qi > 127 ? 127 : qi);
        q[r * k + b * 32 + i] = (int8_t)qi;
      }
      scales[r * blocks + b] = d;
    }
}

/* ===================================================================== */
/* Block composition: xabe-engine block/moe.rs:12-25; exercised on the    */
/* host in xabe-engine tests/moe_block.rs:981-1123                         */
/* ===================================================================== */
static double now_s(void) {
  struct timespec ts;
  clock_gettime(CLOCK_MONOTONIC, &ts);
  return (double)ts.tv_sec + 1e-9 * (double)ts.tv_nsec;
}

int xo_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

static int dequant_matrix(int quant, const uint8_t* bytes, size_t elements, float* out) {
  size_t len = elements / xo_block_elements(quant) * xo_block_bytes(quant);
  return xo_dequantize_row(quant, bytes, len, out);
}

int xo_moe_block_forward(const xo_moe_weights* w, const float* residual, size_t tokens, const float* logits_override,
                         const float* logit_bias, int threads, xo_moe_outputs* out) {
  const size_t E = w->num_experts, K = w->top_k, H = w->hidden, I = w->intermediate;
  const size_t mat = H * I;
  if (threads < 1) threads = 1;
  out->seconds_dequant = 0.0;
  out->seconds_matvec = 0.0;

  float* normed = (float*)malloc(tokens * H * sizeof(float));
  float* logits = (float*)malloc(tokens * E * sizeof(float));
  uint32_t* ids = (uint32_t*)malloc(tokens * K * sizeof(uint32_t));
  float* tw = (float*)malloc(tokens * K * sizeof(float));
  float* contrib = (float*)malloc(tokens * K * H * sizeof(float)); /* expert_mlp per (t,k) */
  float* shexp = (float*)malloc(tokens * H * sizeof(float));
  float* router = NULL;
  int rc = 0;

  /* normed = RMSNorm(input) */
  for (size_t t = 0; t < tokens; ++t) xo_rms_norm(residual + t * H, w->post_norm, H, w->eps, normed + t * H);

  /* logits = ffn_gate_inp . normed */
  if (logits_override) {
    memcpy(logits, logits_override, tokens * E * sizeof(float));
  } else {
    const float* rw = w->router_f32;
    if (!rw) {
      router = (float*)malloc(E * H * sizeof(float));
      if (dequant_matrix(XO_Q8_0, w->router_q8, E * H, router) != 0) { rc = -1; goto done; }
      rw = router;
    }
    for (size_t t = 0; t < tokens; ++t) xo_gemv(rw, E, H, normed + t * H, logits + t * E);
    if (logit_bias)
      for (size_t t = 0; t < tokens; ++t)
        for (size_t e = 0; e < E; ++e) logits[t * E + e] += logit_bias[e];
  }

  /* softmax, top-k, renormalise */
  if (xo_route_batch(logits, tokens, E, K, ids, tw) != 0) { rc = -1; goto done; }

  /* routed experts, grouped by expert so each is unpacked once; every
   * (token, k) contribution is the same expert_mlp call naive_forward makes. */
  {
    double t_deq = 0.0, t_mv = 0.0;
#pragma omp parallel num_threads(threads) reduction(+ : t_deq, t_mv)
    {
      float* g = (float*)malloc(mat * sizeof(float));
      float* u = (float*)malloc(mat * sizeof(float));
      float* d = (float*)malloc(mat * sizeof(float));
#pragma omp for schedule(dynamic, 1)
      for (size_t e = 0; e < E; ++e) {
        int used = 0;
        for (size_t i = 0; i < tokens * K && !used; ++i) used = ids[i] == e;
        if (!used) continue;
        double t0 = now_s();
        dequant_matrix(w->gate_quant, w->gate_exps + e * (mat / xo_block_elements(w->gate_quant)) * xo_block_bytes(w->gate_quant), mat, g);
        dequant_matrix(w->up_quant, w->up_exps + e * (mat / xo_block_elements(w->up_quant)) * xo_block_bytes(w->up_quant), mat, u);
        dequant_matrix(w->down_quant, w->down_exps + e * (mat / xo_block_elements(w->down_quant)) * xo_block_bytes(w->down_quant), mat, d);
        double t1 = now_s();
        for (size_t i = 0; i < tokens * K; ++i)
          if (ids[i] == e) xo_expert_mlp(g, u, d, normed + (i / K) * H, H, I, contrib + i * H);
        double t2 = now_s();
        t_deq += t1 - t0;
        t_mv += t2 - t1;
      }
      free(g);
      free(u);
      free(d);
    }
    out->seconds_dequant += t_deq;
    out->seconds_matvec += t_mv;
  }

  /* shared expert, ungated */
  {
    double t0 = now_s();
    float* g = (float*)malloc(mat * sizeof(float));
    float* u = (float*)malloc(mat * sizeof(float));
    float* d = (float*)malloc(mat * sizeof(float));
    dequant_matrix(w->sgate_quant, w->shared_gate, mat, g);
    dequant_matrix(w->sup_quant, w->shared_up, mat, u);
    dequant_matrix(w->sdown_quant, w->shared_down, mat, d);
    double t1 = now_s();
#pragma omp parallel for num_threads(threads) schedule(dynamic, 1)
    for (size_t t = 0; t < tokens; ++t) xo_expert_mlp(g, u, d, normed + t * H, H, I, shexp + t * H);
    double t2 = now_s();
    out->seconds_dequant += t1 - t0;
    out->seconds_matvec += t2 - t1;
    free(g);
    free(u);
    free(d);
  }

  /* routed = sum_k w_k * contribution_k (ascending k: gemm.rs:114-121);
   * g = sigmoid(w_sh . normed); ffn_out = routed + shexp * g; l_out = ffn_out + input */
  for (size_t t = 0; t < tokens; ++t) {
    float gate_logit;
    xo_gemv(w->shared_gate_inp, 1, H, normed + t * H, &gate_logit);
    float gsc = xo_sigmoid(gate_logit);
    if (out->gate) out->gate[t] = gsc;
    for (size_t j = 0; j < H; ++j) {
      float r = 0.0f;
      for (size_t k = 0; k < K; ++k) r += tw[t * K + k] * contrib[(t * K + k) * H + j];
      float v = r + shexp[t * H + j] * gsc;
      if (out->routed) out->routed[t * H + j] = r;
      if (out->ffn_out) out->ffn_out[t * H + j] = v;
      out->l_out[t * H + j] = v + residual[t * H + j];
    }
  }
  if (out->normed) memcpy(out->normed, normed, tokens * H * sizeof(float));
  if (out->logits) memcpy(out->logits, logits, tokens * E * sizeof(float));
  if (out->topk_ids) memcpy(out->topk_ids, ids, tokens * K * sizeof(uint32_t));
  if (out->topk_weights) memcpy(out->topk_weights, tw, tokens * K * sizeof(float));
  if (out->shexp) memcpy(out->shexp, shexp, tokens * H * sizeof(float));

done:
  free(normed);
  free(logits);
  free(ids);
  free(tw);
  free(contrib);
  free(shexp);
  free(router);
  return rc;
}

/* xabe-engine block/dense_ffn.rs:11-16 */
int xo_dense_block_forward(size_t hidden, size_t intermediate, float eps, const float* post_norm, int gate_quant,
                           int up_quant, int down_quant, const uint8_t* gate, const uint8_t* up, const uint8_t* down,
                           const float* residual, size_t tokens, int threads, float* normed_out, float* ffn_out,
                           float* l_out) {
  size_t mat = hidden * intermediate;
  if (threads < 1) threads = 1;
  float* g = (float*)malloc(mat * sizeof(float));
  float* u = (float*)malloc(mat * sizeof(float));
  float* d = (float*)malloc(mat * sizeof(float));
  float* normed = (float*)malloc(tokens * hidden * sizeof(float));
  float* gu = (float*)malloc(tokens * intermediate * 2 * sizeof(float));
  int rc = 0;
  if (dequant_matrix(gate_quant, gate, mat, g) || dequant_matrix(up_quant, up, mat, u) ||
      dequant_matrix(down_quant, down, mat, d)) { rc = -1; goto done; }
  for (size_t t = 0; t < tokens; ++t) xo_rms_norm(residual + t * hidden, post_norm, hidden, eps, normed + t * hidden);
  /* expert_mlp, with its three matvecs split over rows when threads > 1:
   * each output element is still one sequential dot product. */
  for (size_t t = 0; t < tokens; ++t) {
    float* gt = gu + t * 2 * intermediate;
    float* ut = gt + intermediate;
    const float* x = normed + t * hidden;
#pragma omp parallel for num_threads(threads) schedule(static)
    for (size_t o = 0; o < intermediate; ++o) {
      gt[o] = dot_seq(g + o * hidden, x, hidden);
      ut[o] = dot_seq(u + o * hidden, x, hidden);
    }
    for (size_t o = 0; o < intermediate; ++o) gt[o] = xo_silu(gt[o]) * ut[o];
#pragma omp parallel for num_threads(threads) schedule(static)
    for (size_t o = 0; o < hidden; ++o) {
      float v = dot_seq(d + o * intermediate, gt, intermediate);
      ffn_out[t * hidden + o] = v;
      l_out[t * hidden + o] = v + residual[t * hidden + o];
    }
  }
  if (normed_out) memcpy(normed_out, normed, tokens * hidden * sizeof(float));
done:
  free(g);
  free(u);
  free(d);
  free(normed);
  free(gu);
  return rc;
}

/* ===================================================================== */
/* Synthetic inputs (no reference counterpart)                            */
/* ===================================================================== */
static uint64_t splitmix64(uint64_t z) {
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

static void synth_chunk(uint64_t seed, size_t chunk, float sigma, float* out256) {
  xo_rng r;
  xo_rng_new(&r, splitmix64(seed + (uint64_t)chunk * 0x9E3779B97F4A7C15ull));
  for (int i = 0; i < 256; ++i) {
    uint32_t s = 0;
    for (int k = 0; k < 3; ++k) {
      uint64_t v = xo_rng_next_u64(&r);
      s += (uint32_t)(v & 0xffff) + (uint32_t)((v >> 16) & 0xffff) + (uint32_t)((v >> 32) & 0xffff) +
           (uint32_t)(v >> 48);
    }
    float z = (float)(2 * (int32_t)s - 12 * 65535) * (1.0f / 131072.0f);
    out256[i] = sigma * z;
  }
}

void xo_synth_normal_f32(uint64_t seed, size_t n, float sigma, float* out) {
  size_t chunks = (n + 255) / 256;
#pragma omp parallel for schedule(static)
  for (size_t c = 0; c < chunks; ++c) {
    float tmp[256];
    synth_chunk(seed, c, sigma, tmp);
    size_t m = n - c * 256 < 256 ? n - c * 256 : 256;
    memcpy(out + c * 256, tmp, m * sizeof(float));
  }
}

int xo_synth_quant(int quant, uint64_t seed, size_t n, float sigma, uint8_t* out) {
  if (n % 256 != 0) return -1;
  size_t chunks = n / 256;
#pragma omp parallel for schedule(static)
  for (size_t c = 0; c < chunks; ++c) {
    float tmp[256];
    synth_chunk(seed, c, sigma, tmp);
    if (quant == XO_Q6K) xo_quantize_q6_k(tmp, out + c * XO_BLOCK_Q6_K_BYTES);
    else
      for (int b = 0; b < 8; ++b) xo_quantize_q8_0(tmp + b * 32, out + (c * 8 + b) * XO_BLOCK_Q8_0_BYTES);
  }
  return 0;
}

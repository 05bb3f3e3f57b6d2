/*
 * CPU oracle for the quantized MoE feed-forward block: TEST INFRASTRUCTURE ONLY.
 *
 * A plain-C restatement of the reference's scalar fp32 CPU path
 * (crates/xabe-kernels in the reference tree).  It exists to check the HIP
 * kernels; nothing in the product library may include, link or call it.
 * Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg use it.
 *
 * Every function cites the reference file:line it follows.  Build with
 * -ffp-contract=off -fno-fast-math so that `a*b+c` rounds twice, exactly as
 * the reference's scalar Rust does.
 *
 * Parity status of each function (what pins it besides this restatement) is
 * listed at the top of xabe_oracle.c.
 */
#ifndef XABE_ORACLE_H
#define XABE_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define XO_QK_K 256
#define XO_QK8_0 32
#define XO_BLOCK_Q8_0_BYTES 34
#define XO_BLOCK_Q6_K_BYTES 210

enum { XO_Q6K = 0, XO_Q8_0 = 1 };

/* ---- rng.rs:20-55 ---------------------------------------------------- */
typedef struct { uint64_t state; } xo_rng;
void xo_rng_new(xo_rng* r, uint64_t seed);
uint64_t xo_rng_next_u64(xo_rng* r);
float xo_rng_next_f32(xo_rng* r);
float xo_rng_next_f32_range(xo_rng* r, float low, float high);
uint32_t xo_rng_next_u32_below(xo_rng* r, uint32_t bound);
/* vec_f32 on a generator that the caller keeps (state advances). */
void xo_rng_vec_f32(xo_rng* r, size_t n, float low, float high, float* out);

/* ---- f16.rs:17-100 --------------------------------------------------- */
uint16_t xo_to_f16_bits(float x);
float xo_from_f16_bits(uint16_t h);

/* ---- quant.rs -------------------------------------------------------- */
void xo_quantize_q8_0(const float* x32, uint8_t* out34);
void xo_dequantize_q8_0(const uint8_t* in34, float* y32);
void xo_quantize_q6_k(const float* x256, uint8_t* out210);
void xo_dequantize_q6_k(const uint8_t* in210, float* y256);
/* Row forms: return 0, or -1 when `len` is not a whole number of blocks. */
int xo_dequantize_row(int quant, const uint8_t* bytes, size_t len, float* out);
int xo_quantize_row(int quant, const float* x, size_t n, uint8_t* out);
size_t xo_block_bytes(int quant);
size_t xo_block_elements(int quant);

/* ---- norm.rs --------------------------------------------------------- */
void xo_rms_norm(const float* x, const float* weight, size_t n, float eps, float* y);
float xo_silu(float x);
float xo_sigmoid(float x);
void xo_swiglu(const float* gate, const float* up, size_t n, float* out);
void xo_sigmoid_gate(const float* x, const float* gate, size_t n, float* out);
void xo_residual_add(const float* a, const float* b, size_t n, float* out);

/* ---- gemv.rs --------------------------------------------------------- */
void xo_gemv(const float* weight, size_t out_dim, size_t in_dim, const float* x, float* out);
size_t xo_argmax(const float* v, size_t n);

/* ---- moe/router.rs --------------------------------------------------- */
/* Returns 0, or -1 on the conditions the reference panics on. */
int xo_route_token(const float* logits, size_t num_experts, size_t k, uint32_t* expert_ids, float* weights);
int xo_route_batch(const float* logits, size_t tokens, size_t num_experts, size_t k, uint32_t* expert_ids,
                   float* weights);

/* ---- moe/dispatch.rs ------------------------------------------------- */
/* `sorted_token_ids` needs room for tokens*top_k + num_experts*(block_size-1)
 * entries and `expert_ids` for that many / block_size.  Returns 0, or -1 on
 * the conditions the reference panics on (zero block size, id out of range). */
int xo_moe_align_block_size(const uint32_t* topk_ids, size_t tokens, size_t top_k, size_t block_size,
                            size_t num_experts, uint32_t* sorted_token_ids, int32_t* expert_ids,
                            size_t* num_tokens_post_pad);

/* ---- moe/gemm.rs ----------------------------------------------------- */
void xo_expert_mlp(const float* gate, const float* up, const float* down, const float* x, size_t hidden,
                   size_t intermediate, float* out);
/* experts: gate/up/down stacks [E][I][H], [E][I][H], [E][H][I] as f32. */
void xo_naive_forward(const float* hidden_states, size_t tokens, const uint32_t* expert_ids, const float* weights,
                      size_t top_k, const float* gate, const float* up, const float* down, size_t hidden,
                      size_t intermediate, float* out);
void xo_grouped_forward(const float* hidden_states, size_t tokens, const uint32_t* sorted_token_ids,
                        const int32_t* expert_block_ids, size_t num_blocks, size_t block_size,
                        const float* flat_weights, size_t top_k, const float* gate, const float* up,
                        const float* down, size_t hidden, size_t intermediate, float* out);

/* ---- compare.rs ------------------------------------------------------ */
typedef struct {
  float max_abs_error;
  size_t max_abs_error_index;
  float max_rel_error;
  size_t max_rel_error_index;
  float cosine_similarity;
  size_t non_finite_count;
  size_t len;
} xo_comparison;
int xo_compare(const float* candidate, const float* reference, size_t n, xo_comparison* out);

/* ---- MoeGeometry capacity arithmetic (xabe-cuda kernels/moe.rs:4556-4598) */
size_t xo_max_flat_pairs(size_t max_tokens, size_t top_k);
size_t xo_sorted_capacity(size_t num_experts, size_t top_k, size_t block_size, size_t max_tokens);
size_t xo_expert_block_capacity(size_t num_experts, size_t top_k, size_t block_size, size_t max_tokens);

/* ---- mma.rs:118-157 (activation quantisation of the reference's int8 regime) */
void xo_quantize_rows_q8(const float* x, size_t rows, size_t k, int8_t* q, float* scales);

/* ---- the block composition (xabe-engine block/moe.rs:12-25, dense_ffn.rs:11-16) */
typedef struct {
  size_t num_experts, top_k, hidden, intermediate;
  float eps;
  const float* post_norm;      /* [H] */
  const float* router_f32;     /* [E][H] f32, or NULL when router_q8 is given */
  const uint8_t* router_q8;    /* [E][H] as Q8_0 bytes, dequantised q*d, or NULL */
  int gate_quant, up_quant, down_quant;
  const uint8_t *gate_exps, *up_exps, *down_exps; /* [E][I][H], [E][I][H], [E][H][I] */
  const float* shared_gate_inp; /* [H] */
  int sgate_quant, sup_quant, sdown_quant;
  const uint8_t *shared_gate, *shared_up, *shared_down;
} xo_moe_weights;

typedef struct {
  float* normed;      /* [T][H]   or NULL */
  float* logits;      /* [T][E]   or NULL (the logits actually routed on, after bias) */
  uint32_t* topk_ids; /* [T][K]   or NULL */
  float* topk_weights;/* [T][K]   or NULL */
  float* routed;      /* [T][H]   or NULL */
  float* shexp;       /* [T][H]   or NULL */
  float* gate;        /* [T]      or NULL */
  float* ffn_out;     /* [T][H]   or NULL */
  float* l_out;       /* [T][H]   required */
  double seconds_dequant; /* time spent unpacking experts */
  double seconds_matvec;  /* time spent in expert_mlp */
} xo_moe_outputs;

/* residual: [T][H].  logits_override (may be NULL): route on these [T][E]
 * logits instead of the oracle's own router GEMV (the reference's parity
 * method: "route on the host from the device's own logits",
 * xabe-engine tests/moe_block.rs:1012-1016).  logit_bias (may be NULL): [E]
 * added to the logits before routing.  threads: 1 = the faithful scalar
 * path; >1 = OpenMP over distinct experts (same arithmetic per pair and the
 * same ascending-k sum, so the result is bit-identical to threads=1). */
int xo_moe_block_forward(const xo_moe_weights* w, const float* residual, size_t tokens, const float* logits_override,
                         const float* logit_bias, int threads, xo_moe_outputs* out);

/* Dense sibling: normed = rms_norm; ffn_out = expert_mlp(normed); l_out = ffn_out + residual. */
int xo_dense_block_forward(size_t hidden, size_t intermediate, float eps, const float* post_norm, int gate_quant,
                           int up_quant, int down_quant, const uint8_t* gate, const uint8_t* up, const uint8_t* down,
                           const float* residual, size_t tokens, int threads, float* normed, float* ffn_out,
                           float* l_out);

/* ---- synthetic inputs (this build's own definition; no reference counterpart)
 * Element i of a tensor seeded `seed` belongs to chunk c = i / 256; chunk c
 * draws from its own xorshift64* stream seeded splitmix64(seed + c * GOLDEN).
 * Each value is z * sigma with z an Irwin-Hall(12) normal approximation built
 * in integer arithmetic from twelve 16-bit fields of three next_u64 outputs,
 * so CPU and GPU generators agree bit for bit. */
void xo_synth_normal_f32(uint64_t seed, size_t n, float sigma, float* out);
int xo_synth_quant(int quant, uint64_t seed, size_t n_elements, float sigma, uint8_t* out);

int xo_num_threads(void);

#ifdef __cplusplus
}
#endif
#endif

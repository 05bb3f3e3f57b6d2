// Router logits at prefill widths: logits[t][e] = router[e] . normed[t] as a GEMM on the fp32 matrix
// instruction (v_mfma_f32_32x32x2_f32).  The decode-style kernel re-reads the router once per two tokens
// (8192 tokens: 4096 passes over it out of L2, 340 us); here a workgroup holds a 64-token x 128-expert tile
// and walks the contraction in steps of 32, so the router is read once per 64 tokens.
//
// fp32 operands on purpose: the routing decision hangs on these numbers, and fp16 operands would move a few
// selections per thousand tokens.  A Q8_0 router dequantises to exactly q * d in fp32 (the CPU reference's
// value); products and sums are fp32 inside the matrix core.  The contraction order differs from the
// decode kernels', so these logits agree with theirs to fp32 rounding, not bit for bit: as with the expert
// contractions, a token is bit-identical across batches WITHIN a regime.
// Up to 16384 tokens the tiles are too few to fill the chip with more than a workgroup or two per CU (8 x 2 at
// 512 tokens, each walking all 64 contraction steps: ~115 us whatever the width), so the contraction is split
// over workgroups (grid.z: 8 parts up to 4096 tokens, 4 at 8192), each part writing its own [token][expert] plane,
// and a second small launch adds the planes in part order: a fixed order, so a token's logits do not depend on
// its batch mates here either.
// Replaces the reference's router launch for wide passes (crates/xabe-engine/src/block/moe.rs:1150-1184).
#include <string.h>

#include "device_common.h"
#include "host_common.h"

namespace xabe {

typedef float float16v __attribute__((ext_vector_type(16)));

constexpr int kRgM = 64;        // tokens per tile
constexpr int kRgN = 128;       // experts per tile (64 while the wider tiles are fewer than the compute units)
constexpr int kRgK = 32;        // contraction step: one Q8_0 block per row
constexpr int kRgLdA = kRgM + 1;  // LDS tiles are k-major: element (k, m) at k * ld + m
constexpr int kRgLdB = kRgN + 1;
// Narrow tiles, 64 experts (each wavefront 32 x 32): twice the workgroups and half the matrix instructions in each.  At
// 512 tokens the 16 wide tiles in 8 parts are 128 workgroups of ~8 us of fp32 matrix work on 256 compute units.

struct RouterGemmArgs {
  const void* router;   // [E][H] f32, or Q8_0 blocks
  const float* normed;  // [T][H]
  float* logits;        // [T][E]; with splits > 1 the planes [split][max_tokens][E]
  const int* valid_tokens;
  int H, E;
  int splits, max_tokens;
};

// grid: (E / RN, ceil(max_tokens / 64), splits); 4 wavefronts as 2 (tokens) x 2 (experts), each 32 x RN / 2.
template <bool Q8, int RN = kRgN>
__global__ void __launch_bounds__(256) k_router_gemm(RouterGemmArgs a) {
  static_assert(RN == 128 || RN == 64, "expert tile");
  constexpr int NJ = RN / 64;      // 32-column blocks per wavefront
  constexpr int kBPer = RN / 8;    // elements of the B tile a thread stages per step
  __shared__ float sA[kRgK * kRgLdA];
  __shared__ float sB[kRgK * kRgLdB];
  const int valid = *a.valid_tokens;
  const int m0 = blockIdx.y * kRgM, n0 = blockIdx.x * RN;
  if (m0 >= valid) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  // A staging: thread -> (token row tid / 4, eight floats at (tid % 4) * 8); rows past the last live token
  // re-read the last live one (computed, never stored)
  const int am = tid >> 2, ak = (tid & 3) * 8;
  const float* arow = a.normed + (size_t)min(m0 + am, valid - 1) * a.H + ak;
  // B staging: thread -> (expert row tid / 2, sixteen elements at (tid % 2) * 16); narrow tile: row tid / 4, eight
  const int bn = tid / (32 / kBPer), bk = (tid % (32 / kBPer)) * kBPer;
  const size_t brow_bytes = Q8 ? (size_t)(a.H / 32) * kQ8Bytes : (size_t)a.H * 4;
  const uint8_t* brow = static_cast<const uint8_t*>(a.router) + (size_t)(n0 + bn) * brow_bytes;

  float16v acc[NJ];
#pragma unroll
  for (int j = 0; j < NJ; ++j) acc[j] = (float16v)(0.0f);

  const int nks_all = a.H / kRgK, ks0 = (int)blockIdx.z * (nks_all / a.splits), nks = ks0 + nks_all / a.splits;
  float* const plane = a.logits + (size_t)blockIdx.z * a.max_tokens * a.E;
  float4 ra[2];
  float rb[kBPer];
  auto load_step = [&](int ks) {
    ra[0] = reinterpret_cast<const float4*>(arow + (size_t)ks * kRgK)[0];
    ra[1] = reinterpret_cast<const float4*>(arow + (size_t)ks * kRgK)[1];
    if constexpr (Q8) {
      // block ks of the row: d (fp16) then 32 codes; this thread takes codes bk .. bk + 15 (2-byte aligned)
      const uint8_t* blk = brow + (size_t)ks * kQ8Bytes;
      const float d = f16_bits_to_f32(*reinterpret_cast<const uint16_t*>(blk));
      const uint16_t* q = reinterpret_cast<const uint16_t*>(blk + 2 + bk);
#pragma unroll
      for (int i = 0; i < kBPer / 2; ++i) {
        const uint32_t two = q[i];
        rb[2 * i] = (float)(int8_t)(two & 0xff) * d;
        rb[2 * i + 1] = (float)(int8_t)(two >> 8) * d;
      }
    } else {
      const float4* p = reinterpret_cast<const float4*>(brow + ((size_t)ks * kRgK + bk) * 4);
#pragma unroll
      for (int i = 0; i < kBPer / 4; ++i) {
        const float4 v = p[i];
        rb[4 * i] = v.x; rb[4 * i + 1] = v.y; rb[4 * i + 2] = v.z; rb[4 * i + 3] = v.w;
      }
    }
  };
  load_step(ks0);
  for (int ks = ks0; ks < nks; ++ks) {
    __syncthreads();  // the previous step's tiles have been read
    const float va[8] = {ra[0].x, ra[0].y, ra[0].z, ra[0].w, ra[1].x, ra[1].y, ra[1].z, ra[1].w};
#pragma unroll
    for (int i = 0; i < 8; ++i) sA[(ak + i) * kRgLdA + am] = va[i];
#pragma unroll
    for (int i = 0; i < kBPer; ++i) sB[(bk + i) * kRgLdB + bn] = rb[i];
    __syncthreads();
    if (ks + 1 < nks) load_step(ks + 1);  // in flight while the matrix core works
    // operand layout of the 32x32x2 instruction: lane l supplies row (column) l % 32 at k = l / 32
    const float* pa = &sA[(lane >> 5) * kRgLdA + wm * 32 + (lane & 31)];
    const float* pb = &sB[(lane >> 5) * kRgLdB + wn * (RN / 2) + (lane & 31)];
#pragma unroll
    for (int kk = 0; kk < kRgK / 2; ++kk) {
      const float av = pa[kk * 2 * kRgLdA];
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const float bv = pb[kk * 2 * kRgLdB + 32 * j];
        acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv, acc[j], 0, 0, 0);
      }
    }
  }
  // acc[j][v]: tile row (v / 4) * 8 + (lane / 32) * 4 + v % 4, column lane % 32 of column block j
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int t = m0 + wm * 32 + (v >> 2) * 8 + (lane >> 5) * 4 + (v & 3);
    if (t >= valid) continue;
#pragma unroll
    for (int j = 0; j < NJ; ++j) plane[(size_t)t * a.E + n0 + wn * (RN / 2) + j * 32 + (lane & 31)] = acc[j][v];
  }
}

// The Q8_0 router on the bf16 matrix instruction (v_mfma_f32_32x32x16_bf16), still with fp32-grade operands: an
// activation splits exactly into three bf16 pieces (x = x0 + x1 + x2, each the leading eight bits of what is
// left), a Q8_0 code is a small integer and exact in bf16, so every product code * piece is exact in the matrix
// core's fp32 and a block's sum S = sum code * (x2 + x1 + x0) is an fp32 accumulation of exact terms.  The block
// scale is applied outside: logit += d * S, one fp32 fused multiply-add per block and output element.  Six matrix
// instructions of 32 cycles per 32 x 32 x 32 block against sixteen of 64 on the fp32 instruction.
// Same tiles, grid and planes as k_router_gemm; the two agree to fp32 rounding (the order of the additions
// inside a block differs), and a token's logits do not depend on its batch mates here either.
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t rg_u32x4 __attribute__((ext_vector_type(4)));
constexpr int kRgAhead = 2;     // steps of global loads a thread keeps in flight (four: 55 us against 50 at 8192 tokens)
constexpr int kRgRowBytes = 80;  // a 32-element bf16 row padded to 80 bytes: 16-byte reads of 32 rows hit every bank once

template <int RN>
__global__ void __launch_bounds__(256) k_router_gemm_q8_bf16x3(RouterGemmArgs a) {
  static_assert(RN == 128 || RN == 64, "expert tile");
  // wavefronts: 2 (tokens) x 2 (experts), each 32 tokens x NJ blocks of 32 experts.  (A 256-expert tile on eight
  // wavefronts, which reads the activations once for the whole router, was measured: 92 us against 50 at 8192
  // tokens; its 512 workgroups are too few to cover each other's loads.)
  constexpr int kThreads = 256;
  constexpr int WN = 2;
  constexpr int NJ = RN / (32 * WN);
  constexpr int kAPer = kRgM * kRgK / kThreads;  // activations a thread stages per step (8 or 4)
  constexpr int kBPer = RN * kRgK / kThreads;    // codes of the B tile a thread stages per step (16 or 8)
  __shared__ __attribute__((aligned(16))) uint8_t sA[3 * kRgM * kRgRowBytes];
  __shared__ __attribute__((aligned(16))) uint8_t sB[RN * kRgRowBytes];
  __shared__ float sD[RN];
  const int valid = *a.valid_tokens;
  const int m0 = blockIdx.y * kRgM, n0 = blockIdx.x * RN;
  if (m0 >= valid) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;
  const int am = tid / (32 / kAPer), ak = (tid % (32 / kAPer)) * kAPer;
  const float* arow = a.normed + (size_t)min(m0 + am, valid - 1) * a.H + ak;
  const int bn = tid / (32 / kBPer), bk = (tid % (32 / kBPer)) * kBPer;
  const uint8_t* brow = static_cast<const uint8_t*>(a.router) + (size_t)(n0 + bn) * (size_t)(a.H / 32) * kQ8Bytes;

  float16v acc[NJ];
#pragma unroll
  for (int j = 0; j < NJ; ++j) acc[j] = (float16v)(0.0f);

  const int nks_all = a.H / kRgK, ks0 = (int)blockIdx.z * (nks_all / a.splits), nks = ks0 + nks_all / a.splits;
  float* const plane = a.logits + (size_t)blockIdx.z * a.max_tokens * a.E;
  // what a thread holds of one step: kRgAhead steps are in flight, so that a step's loads have that many steps' time to land
  struct Held {
    float4 ra[kAPer / 4];
    uint32_t rq[kBPer / 4 + 1];  // the aligned dwords around this thread's codes
    uint32_t rd;                 // the block's scale (fp16 bits), bk == 0 threads
  };
  auto load_step = [&](int ks, Held& h) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < kAPer / 4; ++i) h.ra[i] = reinterpret_cast<const float4*>(arow + (size_t)ks * kRgK)[i];
    // block ks of the row: d (fp16) then 32 codes; rows start on 16 bytes and a block is 34, so the codes start
    // on a dword in odd blocks and two bytes past one in even blocks (the row's block count is even: checked by
    // the host, so the dword past an even block's codes lies inside the row)
    const uint8_t* blk = brow + (size_t)ks * kQ8Bytes;
    const uint32_t* w = reinterpret_cast<const uint32_t*>(blk + (ks & 1 ? 2 : 0) + bk);
#pragma unroll
    for (int i = 0; i <= kBPer / 4; ++i) h.rq[i] = (i < kBPer / 4 || !(ks & 1)) ? w[i] : 0u;
    h.rd = 0;
    if (bk == 0) h.rd = *reinterpret_cast<const uint16_t*>(blk);
  };
  auto step = [&](int ks, Held& h) __attribute__((always_inline)) {
    const uint32_t (&rq)[kBPer / 4 + 1] = h.rq;
    const uint32_t rd = h.rd;
    __syncthreads();  // the previous step's tiles have been read
    {
      // activations: three exact bf16 pieces, kAPer elements = one 16- or 8-byte row segment per piece
      float va[kAPer];
#pragma unroll
      for (int i = 0; i < kAPer / 4; ++i) {
        va[4 * i] = h.ra[i].x; va[4 * i + 1] = h.ra[i].y; va[4 * i + 2] = h.ra[i].z; va[4 * i + 3] = h.ra[i].w;
      }
      uint32_t p0[kAPer], p1[kAPer], p2[kAPer];
#pragma unroll
      for (int i = 0; i < kAPer; ++i) {
        p0[i] = __builtin_bit_cast(uint32_t, va[i]);
        const float r1 = va[i] - __builtin_bit_cast(float, p0[i] & 0xffff0000u);
        p1[i] = __builtin_bit_cast(uint32_t, r1);
        const float r2 = r1 - __builtin_bit_cast(float, p1[i] & 0xffff0000u);
        p2[i] = __builtin_bit_cast(uint32_t, r2);
      }
      typedef uint32_t piece_t __attribute__((ext_vector_type(kAPer / 2)));
      auto pack = [&](const uint32_t (&p)[kAPer]) {
        piece_t v;
#pragma unroll
        for (int i = 0; i < kAPer / 2; ++i) v[i] = __builtin_amdgcn_perm(p[2 * i + 1], p[2 * i], 0x07060302u);  // two upper halves
        return v;
      };
      uint8_t* dst = sA + am * kRgRowBytes + ak * 2;
      *reinterpret_cast<piece_t*>(dst) = pack(p0);
      *reinterpret_cast<piece_t*>(dst + kRgM * kRgRowBytes) = pack(p1);
      *reinterpret_cast<piece_t*>(dst + 2 * kRgM * kRgRowBytes) = pack(p2);
      // codes: in even blocks they sit two bytes into the dwords that were read
      uint32_t c[kBPer / 4];
#pragma unroll
      for (int i = 0; i < kBPer / 4; ++i) c[i] = (ks & 1) ? rq[i] : __builtin_amdgcn_alignbit(rq[i + 1], rq[i], 16);
      uint8_t* bdst = sB + bn * kRgRowBytes + bk * 2;
#pragma unroll
      for (int h = 0; h < kBPer / 8; ++h) {
        rg_u32x4 v;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const uint32_t w4 = c[2 * h + (i >> 1)];
          const int sh = (i & 1) * 16;
          const float f0 = (float)(int8_t)((w4 >> sh) & 0xff), f1 = (float)(int8_t)((w4 >> (sh + 8)) & 0xff);
          v[i] = __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, f1), __builtin_bit_cast(uint32_t, f0), 0x07060302u);
        }
        *reinterpret_cast<rg_u32x4*>(bdst + 16 * h) = v;
      }
      if (bk == 0) sD[bn] = f16_bits_to_f32((uint16_t)rd);
    }
    __syncthreads();
    if (ks + kRgAhead < nks) load_step(ks + kRgAhead, h);  // in flight during the next kRgAhead steps' matrix work
    // operand layout of the 32x32x16 instruction: lane l supplies row (column) l % 32, k = (l / 32) * 8 .. + 8
    const uint8_t* pa = sA + (wm * 32 + (lane & 31)) * kRgRowBytes + (lane >> 5) * 16;
    bf16x8 fa[3][2];
#pragma unroll
    for (int p = 0; p < 3; ++p)
#pragma unroll
      for (int kh = 0; kh < 2; ++kh)
        fa[p][kh] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const rg_u32x4*>(pa + p * kRgM * kRgRowBytes + kh * 32));
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const int col = wn * (RN / WN) + j * 32 + (lane & 31);
      const uint8_t* pb = sB + col * kRgRowBytes + (lane >> 5) * 16;
      const bf16x8 fb0 = __builtin_bit_cast(bf16x8, *reinterpret_cast<const rg_u32x4*>(pb));
      const bf16x8 fb1 = __builtin_bit_cast(bf16x8, *reinterpret_cast<const rg_u32x4*>(pb + 32));
      const float d = sD[col];
      float16v blk = (float16v)(0.0f);
#pragma unroll
      for (int p = 2; p >= 0; --p) {  // the smallest pieces first
        blk = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[p][0], fb0, blk, 0, 0, 0);
        blk = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[p][1], fb1, blk, 0, 0, 0);
      }
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[j][v] = __builtin_fmaf(d, blk[v], acc[j][v]);
    }
  };
  Held held[kRgAhead];
#pragma unroll
  for (int d = 0; d < kRgAhead; ++d)
    if (ks0 + d < nks) load_step(ks0 + d, held[d]);
  for (int ks = ks0; ks < nks; ks += kRgAhead) {
#pragma unroll
    for (int d = 0; d < kRgAhead; ++d)
      if (ks + d < nks) step(ks + d, held[d]);
  }
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int t = m0 + wm * 32 + (v >> 2) * 8 + (lane >> 5) * 4 + (v & 3);
    if (t >= valid) continue;
#pragma unroll
    for (int j = 0; j < NJ; ++j) plane[(size_t)t * a.E + n0 + wn * (RN / WN) + j * 32 + (lane & 31)] = acc[j][v];
  }
}

// logits[t][e] = planes[0][t][e] + planes[1][t][e] + ... in part order, live tokens only; then (+ bias[e]): the
// add of the stand-alone bias kernel, on the finished sum
__global__ void __launch_bounds__(256) k_router_sum_planes(const float* __restrict__ planes, const int* __restrict__ valid_tokens,
                                                            int splits, int max_tokens, int E, const float* __restrict__ bias,
                                                            float* __restrict__ logits) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= (size_t)*valid_tokens * E) return;
  float s = planes[i];
  for (int z = 1; z < splits; ++z) s += planes[(size_t)z * max_tokens * E + i];
  if (bias) s += bias[i % (size_t)E];
  logits[i] = s;
}

bool router_gemm_supported(const xabe_moe_kernels* k, const xabe_moe_buffers* b, int router_quant) {
  const xabe_moe_geometry& g = k->g;
  // below 256 tokens even the split tiles are too few and the decode-style kernel wins
  if (!k->tensor_cores || k->exact_regime || k->force_community || g.max_tokens < kRouterGemmMinTokens) return false;
  if (!(router_quant < 0 || router_quant == XABE_QUANT_Q8_0)) return false;
  const int splits = router_gemm_splits(g);
  if (splits > 1 && (!b->router_partial || b->n_router_partial < (size_t)splits * g.max_tokens * g.num_experts ||
                     g.hidden % (kRgK * splits) != 0))
    return false;
  return g.hidden % kRgK == 0 && g.num_experts % kRgN == 0;
}

int launch_router_gemm(const xabe_moe_kernels* k, hipStream_t s, const xabe_moe_buffers* b, const void* router,
                       int router_quant, const float* normed, float* logits, const float* bias, bool* bias_added,
                       bool* sum_deferred) {
  if (bias_added) *bias_added = false;
  if (sum_deferred) *sum_deferred = false;
  const xabe_moe_geometry& g = k->g;
  RouterGemmArgs a;
  memset(&a, 0, sizeof(a));
  a.splits = router_gemm_splits(g);
  a.max_tokens = (int)g.max_tokens;
  a.router = router;
  a.normed = normed;
  a.logits = a.splits > 1 ? b->router_partial : logits;
  a.valid_tokens = b->valid_tokens;
  a.H = (int)g.hidden;
  a.E = (int)g.num_experts;
  const size_t m_tiles = (g.max_tokens + kRgM - 1) / kRgM;
  const bool narrow = g.num_experts / kRgN * m_tiles * a.splits < (size_t)k->num_cus;
  dim3 grid((unsigned)(g.num_experts / (narrow ? 64 : kRgN)), (unsigned)m_tiles, (unsigned)a.splits);
  // a Q8_0 router whose rows hold an even number of blocks takes the bf16x3 form (its dword loads may reach two
  // bytes past an even block, which then is still inside the row)
  const bool x3 = router_quant >= 0 && (g.hidden / 32) % 2 == 0;
  if (narrow) {
    if (router_quant < 0) hipLaunchKernelGGL((k_router_gemm<false, 64>), grid, dim3(256), 0, s, a);
    else if (x3) hipLaunchKernelGGL((k_router_gemm_q8_bf16x3<64>), grid, dim3(256), 0, s, a);
    else hipLaunchKernelGGL((k_router_gemm<true, 64>), grid, dim3(256), 0, s, a);
  } else {
    if (router_quant < 0) hipLaunchKernelGGL((k_router_gemm<false, kRgN>), grid, dim3(256), 0, s, a);
    else if (x3) hipLaunchKernelGGL((k_router_gemm_q8_bf16x3<kRgN>), grid, dim3(256), 0, s, a);
    else hipLaunchKernelGGL((k_router_gemm<true, kRgN>), grid, dim3(256), 0, s, a);
  }
  XABE_HIP_TRY(hipGetLastError());
  if (a.splits > 1 && sum_deferred) {
    *sum_deferred = true;  // the caller's routing launch adds the planes (k_route_planes)
  } else if (a.splits > 1) {
    const size_t n = g.max_tokens * g.num_experts;
    hipLaunchKernelGGL(k_router_sum_planes, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, b->router_partial,
                       b->valid_tokens, a.splits, a.max_tokens, a.E, bias, logits);
    XABE_HIP_TRY(hipGetLastError());
    if (bias && bias_added) *bias_added = true;
  }
  return XABE_OK;
}

}  // namespace xabe

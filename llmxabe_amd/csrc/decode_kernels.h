// Decode-regime expert kernels: fp32 accumulation, weights streamed once from HBM
// in their file layout (210-byte Q6_K superblocks / 34-byte Q8_0 blocks), dequantised
// in registers.  Replaces the reference's gemv / flat / tiled fp32 families
// (crates/xabe-cuda/src/kernels/moe.rs:2403-3124, :3425-3725, :4082-4227).
//
// One wavefront "step" covers 2048 contraction elements of a row: 8 Q6_K superblocks
// (1680 B) or 64 Q8_0 blocks (2176 B), 32 elements per lane.  Rows shorter than 2048
// pack RPS = 2048/K rows into a step; longer rows take KS steps, the last one masked.
// Activations for the lane's fixed element positions live in registers, so a row costs
// its own bytes and nothing else.
//
// Numerics contract: the value of (row, token) is computed by one fixed sequence of
// fp32 operations that does not depend on which other tokens are present, so a token
// decodes to the same bits alone or in a batch (tests/test_gpu_batch_invariance.py).
#pragma once

#include <type_traits>

#include "device_common.h"

namespace xabe {

constexpr int kWavesPerWg = 4;

template <int QUANT>
struct Fmt;
template <>
struct Fmt<kQ6K> {
  using Raw = Q6Raw;
  static constexpr uint32_t kChunkBytes = 8 * kQ6KBytes;
  static constexpr int kBlockElems = 256;
  static constexpr int kBlockBytes = kQ6KBytes;
};
template <>
struct Fmt<kQ8_0> {
  using Raw = Q8Raw;
  static constexpr uint32_t kChunkBytes = 64 * kQ8Bytes;
  static constexpr int kBlockElems = 32;
  static constexpr int kBlockBytes = kQ8Bytes;
};

template <>
struct Fmt<kF32> {
  using Raw = F32Raw;
  static constexpr uint32_t kChunkBytes = 2048 * 4;
  static constexpr int kBlockElems = 1;
  static constexpr int kBlockBytes = 4;
};

struct LaneGeom {
  int lane, slot, half, l8;
  uint32_t lane_off;  // byte offset of the lane's block inside a step's chunk
};

template <int QUANT>
__device__ __forceinline__ LaneGeom lane_geom() {
  LaneGeom g;
  g.lane = __lane_id();
  g.slot = g.lane >> 3;
  g.half = (g.lane >> 2) & 1;
  g.l8 = g.lane & 3;
  g.lane_off = QUANT == kQ6K ? (uint32_t)g.slot * kQ6KBytes
             : QUANT == kQ8_0 ? (uint32_t)g.lane * kQ8Bytes
                              : (uint32_t)g.lane * 128u;
  return g;
}

// Offset, within a row, of the first of the 32 elements this lane covers in step `k`.
// For Q6_K that is the start of the lane's superblock (positions inside it: q6_pos).
template <int QUANT, int RPS>
__device__ __forceinline__ int lane_koff(const LaneGeom& g, int k) {
  if (QUANT == kQ6K) return ((g.slot % (8 / RPS)) + k * 8) * 256;
  return ((g.lane % (64 / RPS)) + k * 64) * 32;
}

// How a kernel obtains its activations and publishes its outputs.
//   kXPlain: read fp32 rows as they are.
//   kXNorm:  RMS-normalise on load, (x * inv_rms) * norm_weight -- the same two products, in the same
//            order, as the stand-alone RMSNorm kernel, so the values are bit-identical to its output.
//   kXCoherent: the rows were written earlier in the SAME launch by other workgroups; read them with
//            agent-scope loads (sc1) so another XCD's writes are visible without a cache flush.
constexpr int kXPlain = 0, kXNorm = 1, kXCoherent = 2;
// kOPlain: ordinary stores.  kOCoherent: agent-scope stores (written through to the coherence point).
constexpr int kOPlain = 0, kOCoherent = 1;

struct XNorm {
  float inv;              // 1 / sqrt(mean(x^2) + eps) of this token
  const float* weight;    // norm weight, indexed like the row
};

__device__ __forceinline__ float2 load2_coherent(const float* p) {
  const unsigned long long v = __hip_atomic_load(reinterpret_cast<const unsigned long long*>(p), __ATOMIC_RELAXED,
                                                 __HIP_MEMORY_SCOPE_AGENT);
  return make_float2(__builtin_bit_cast(float, (uint32_t)v), __builtin_bit_cast(float, (uint32_t)(v >> 32)));
}
__device__ __forceinline__ void store_coherent(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Eight consecutive activations starting at xrow + off (off a multiple of 4).
template <int XMODE>
__device__ __forceinline__ void load8(const float* __restrict__ xrow, int off, const XNorm& nm, float (&v)[8]) {
  if constexpr (XMODE == kXCoherent) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float2 a = load2_coherent(xrow + off + 2 * i);
      v[2 * i] = a.x;
      v[2 * i + 1] = a.y;
    }
  } else {
    const float4 a = reinterpret_cast<const float4*>(xrow + off)[0];
    const float4 b = reinterpret_cast<const float4*>(xrow + off)[1];
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
    v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    if constexpr (XMODE == kXNorm) {
      const float4 wa = reinterpret_cast<const float4*>(nm.weight + off)[0];
      const float4 wb = reinterpret_cast<const float4*>(nm.weight + off)[1];
      const float w[8] = {wa.x, wa.y, wa.z, wa.w, wb.x, wb.y, wb.z, wb.w};
#pragma unroll
      for (int i = 0; i < 8; ++i) v[i] = v[i] * nm.inv * w[i];
    }
  }
}

template <int QUANT, int XMODE = kXPlain>
__device__ __forceinline__ void load_x(const float* __restrict__ xrow, int koff, bool active, const LaneGeom& g,
                                       float (&x)[32], float (&xs)[4], const XNorm& nm = XNorm{1.0f, nullptr}) {
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    float v[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    // Q6_K: run j of the lane's superblock unit; Q8_0 / fp32: the j-th eight of 32 consecutive elements
    const int off = QUANT == kQ6K ? koff + g.half * 128 + j * 32 + g.l8 * 8 : koff + j * 8;
    if (active) load8<XMODE>(xrow, off, nm, v);
#pragma unroll
    for (int i = 0; i < 8; ++i) x[j * 8 + i] = v[i];
    if (QUANT == kQ6K) {
      float s = 0.0f;
#pragma unroll
      for (int i = 0; i < 8; ++i) s += v[i];
      xs[j] = -32.0f * s;
    } else {
      xs[j] = 0.0f;
    }
  }
}

template <int QUANT>
__device__ __forceinline__ void raw_zero(typename Fmt<QUANT>::Raw& r);
template <>
__device__ __forceinline__ void raw_zero<kQ6K>(Q6Raw& r) {
  r.qa0 = r.qa1 = r.qb0 = r.qb1 = r.qh0 = r.qh1 = r.sc0 = r.sc1 = r.dh = 0;
}
template <>
__device__ __forceinline__ void raw_zero<kQ8_0>(Q8Raw& r) {
#pragma unroll
  for (int i = 0; i < 8; ++i) r.q[i] = 0;
  r.dh = 0;
}
template <>
__device__ __forceinline__ void raw_zero<kF32>(F32Raw& r) {
#pragma unroll
  for (int i = 0; i < 32; ++i) r.v[i] = 0.0f;
}

// Loads this lane's block of the step that starts at `chunk` (any 2-byte alignment).
// DIRECT: Q6_K fields read at their own alignment (q6_load_direct); the Raw is the same.
template <int QUANT, bool DIRECT = false>
__device__ __forceinline__ void load_raw(const uint8_t* chunk, bool active, const LaneGeom& g,
                                         typename Fmt<QUANT>::Raw& r) {
  if (!active) {
    raw_zero<QUANT>(r);
    return;
  }
  const uint32_t mis = (uint32_t)(reinterpret_cast<uintptr_t>(chunk) & 3u);
  const uint8_t* chunk4 = chunk - mis;
  if constexpr (QUANT == kQ6K && DIRECT) q6_load_direct(chunk4, g.lane_off + mis, g.half, g.l8, r);
  else if constexpr (QUANT == kQ6K) q6_load(chunk4, g.lane_off + mis, g.half, g.l8, r);
  else if constexpr (QUANT == kQ8_0) q8_load(chunk4, g.lane_off + mis, r);
  else f32_load(chunk, g.lane_off, r);
}

template <int QUANT, int TC>
__device__ __forceinline__ void accum(const typename Fmt<QUANT>::Raw& r, const LaneGeom& g, const float (&x)[TC][32],
                                      const float (&xs)[TC][4], float (&tot)[TC]) {
  if constexpr (QUANT == kQ6K) q6_accum<TC>(r, g.l8, x, xs, tot);
  else if constexpr (QUANT == kQ8_0) q8_accum<TC>(r, x, tot);
  else f32_accum<TC>(r, x, tot);
}

// ---------------------------------------------------------------------------------
// Coalesced form of load_raw.  A lane picking its own fields out of global memory touches every cache
// line of the step with every one of its seven to ten load instructions, and the vector L1 serves a
// line that is still pending by stalling; measured on this part, that halves the streaming rate
// (2.7 against 5.5 TB/s).  Instead the wavefront requests the step as consecutive 16-byte pieces (each
// line touched once), parks them in a wavefront-private LDS slot and picks the fields up from there with
// the same funnel loads, so the Raw it produces is bit for bit the one load_raw produces.
//   stage_load:  issue the global loads of one step (`nbytes` live bytes starting at `chunk`, any 2-byte
//                alignment).  The 16-byte window around them must lie inside the tensor: the host checks
//                that the tensor starts and ends on 16-byte boundaries, or uses stage_load_bounded for
//                the row at the tensor's end.
//   stage_pick:  pieces -> LDS slot -> Raw.  Slots are private to a wavefront, whose LDS operations
//                complete in program order; the fences only keep the compiler from reordering them.
// ---------------------------------------------------------------------------------
template <int QUANT>
struct StageFmt;
template <>
struct StageFmt<kQ6K> {
  static constexpr int kPieces = 2;        // 1680 (+14) bytes: up to 106 pieces
  static constexpr int kSlotBytes = 1696;
};
template <>
struct StageFmt<kQ8_0> {
  static constexpr int kPieces = 3;        // 2176 (+14) bytes: up to 137 pieces
  static constexpr int kSlotBytes = 2192;
};

typedef uint32_t stage_piece __attribute__((ext_vector_type(4)));  // a first-class vector: stays in registers

template <int QUANT>
struct Staged {
  stage_piece p[StageFmt<QUANT>::kPieces];
  uint32_t mis;  // bytes from the 16-byte boundary below `chunk` to `chunk`
  int last;      // index of the last live piece
};

template <int QUANT>
__device__ __forceinline__ void stage_load(const uint8_t* chunk, uint32_t nbytes, Staged<QUANT>& s) {
  s.mis = (uint32_t)(reinterpret_cast<uintptr_t>(chunk) & 15u);
  s.last = (int)((s.mis + nbytes + 15u) >> 4) - 1;
  const stage_piece* base = reinterpret_cast<const stage_piece*>(chunk - s.mis);
  const int lane = (int)__lane_id();
#pragma unroll
  for (int i = 0; i < StageFmt<QUANT>::kPieces; ++i) s.p[i] = base[min(lane + 64 * i, s.last)];
}

// stage_load for a step whose last piece may reach past the tensor's end (`end`, 2-byte aligned): that piece
// is put together from the 2-byte fields that exist, the rest of it reads as zero.
template <int QUANT>
__device__ __forceinline__ void stage_load_bounded(const uint8_t* chunk, uint32_t nbytes, const uint8_t* end, Staged<QUANT>& s) {
  s.mis = (uint32_t)(reinterpret_cast<uintptr_t>(chunk) & 15u);
  s.last = (int)((s.mis + nbytes + 15u) >> 4) - 1;
  const stage_piece* base = reinterpret_cast<const stage_piece*>(chunk - s.mis);
  const int lane = (int)__lane_id();
#pragma unroll
  for (int i = 0; i < StageFmt<QUANT>::kPieces; ++i) {
    const stage_piece* p = base + min(lane + 64 * i, s.last);
    if (reinterpret_cast<const uint8_t*>(p + 1) <= end) {
      s.p[i] = *p;
    } else {
      const uint16_t* h = reinterpret_cast<const uint16_t*>(p);
      const int live = (int)(end - reinterpret_cast<const uint8_t*>(p)) >> 1;
      stage_piece v = {0u, 0u, 0u, 0u};
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if (j < live) v[j >> 1] |= (uint32_t)h[j] << (16 * (j & 1));
      s.p[i] = v;
    }
  }
}

template <int QUANT>
__device__ __forceinline__ void stage_pick(const Staged<QUANT>& s, uint8_t* slot, bool active, const LaneGeom& g,
                                           typename Fmt<QUANT>::Raw& r) {
  const int lane = (int)__lane_id();
#pragma unroll
  for (int i = 0; i < StageFmt<QUANT>::kPieces; ++i)  // lanes past the last piece repeat its store
    reinterpret_cast<stage_piece*>(slot)[min(lane + 64 * i, s.last)] = s.p[i];
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  if (active) {
    if constexpr (QUANT == kQ6K) q6_load(slot, g.lane_off + s.mis, g.half, g.l8, r);
    else q8_load(slot, g.lane_off + s.mis, r);
  } else {
    raw_zero<QUANT>(r);
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
}

// ---------------------------------------------------------------------------------
// matvec_rows: the body every decode kernel shares.
//   NM = 2: out[t][row] = silu(gate_row . x_t) * (up_row . x_t)      (gate/up + SwiGLU)
//   NM = 1: out[t][row] = scale[t] * (w_row . x_t)                    (down / plain GEMV)
// `w0`/`w1` point at row 0 of the matrix (one expert).  Rows [tile0, tile0+tile_rows)
// are split over the workgroup's four wavefronts.  KS > 0: steps per row, activations
// in registers.  KS == 0: steps from K at run time, activations re-read per step.
// ---------------------------------------------------------------------------------
template <int QUANT, int KS, int RPS, int TC, int NM, int XMODE = kXPlain, int OMODE = kOPlain>
__device__ __forceinline__ void matvec_rows(const uint8_t* __restrict__ w0, const uint8_t* __restrict__ w1, int K,
                                            int n_rows, int tile0, int tile_rows,
                                            const float* const (&xrow)[TC], float* const (&out)[TC],
                                            const float (&scale)[TC], const XNorm* norm = nullptr) {
  using F = Fmt<QUANT>;
  using Raw = typename F::Raw;
  constexpr int G = 64 / RPS;
  static_assert(RPS == 1 || KS == 1, "short rows take exactly one step");
  const LaneGeom g = lane_geom<QUANT>();
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const size_t row_bytes = (size_t)(K / F::kBlockElems) * F::kBlockBytes;
  const int tile_end = min(tile0 + tile_rows, n_rows);

  if constexpr (KS > 0) {
    float x[KS][TC][32];
    float xs[KS][TC][4];
    bool active[KS];
#pragma unroll
    for (int k = 0; k < KS; ++k) {
      const int koff = lane_koff<QUANT, RPS>(g, k);
      active[k] = koff < K;
#pragma unroll
      for (int t = 0; t < TC; ++t)
        load_x<QUANT, XMODE>(xrow[t], koff, active[k], g, x[k][t], xs[k][t], XMODE == kXNorm ? norm[t] : XNorm{1.0f, nullptr});
    }
    auto load_item = [&](int row0, Raw (&r)[NM][KS]) {
#pragma unroll
      for (int k = 0; k < KS; ++k) {
        const size_t off = (size_t)row0 * row_bytes + (size_t)k * F::kChunkBytes;
        load_raw<QUANT>(w0 + off, active[k], g, r[0][k]);
        if constexpr (NM == 2) load_raw<QUANT>(w1 + off, active[k], g, r[NM - 1][k]);
      }
    };
    auto finish_item = [&](int row0, const Raw (&r)[NM][KS]) {
      float tot[NM][TC];
#pragma unroll
      for (int m = 0; m < NM; ++m) {
#pragma unroll
        for (int t = 0; t < TC; ++t) tot[m][t] = 0.0f;
#pragma unroll
        for (int k = 0; k < KS; ++k) accum<QUANT, TC>(r[m][k], g, x[k], xs[k], tot[m]);
#pragma unroll
        for (int t = 0; t < TC; ++t) tot[m][t] = group_sum<G>(tot[m][t]);
      }
      const int row = row0 + g.lane / G;
      if ((g.lane % G) == 0 && row < n_rows) {
#pragma unroll
        for (int t = 0; t < TC; ++t) {
          const float v = NM == 2 ? silu_f(tot[0][t]) * tot[NM - 1][t] : scale[t] * tot[0][t];
          if constexpr (OMODE == kOCoherent) store_coherent(&out[t][row], v);
          else out[t][row] = v;
        }
      }
    };
    int row0 = tile0 + wave * RPS;
    if constexpr (KS == 1) {
      // software pipeline: the next item's bytes are in flight while this one is reduced
      Raw cur[NM][KS], nxt[NM][KS];
      if (row0 < tile_end) load_item(row0, cur);
      for (; row0 < tile_end; row0 += kWavesPerWg * RPS) {
        const int nrow = row0 + kWavesPerWg * RPS;
        if (nrow < tile_end) load_item(nrow, nxt);
        finish_item(row0, cur);
#pragma unroll
        for (int m = 0; m < NM; ++m) cur[m][0] = nxt[m][0];
      }
    } else {
      for (; row0 < tile_end; row0 += kWavesPerWg * RPS) {
        Raw cur[NM][KS];
        load_item(row0, cur);
        finish_item(row0, cur);
      }
    }
  } else {
    // long rows: K / 2048 steps (last one masked), activations re-read each step
    const int steps = (K + kStepElems - 1) / kStepElems;
    for (int row0 = tile0 + wave; row0 < tile_end; row0 += kWavesPerWg) {
      float tot[NM][TC];
#pragma unroll
      for (int m = 0; m < NM; ++m)
#pragma unroll
        for (int t = 0; t < TC; ++t) tot[m][t] = 0.0f;
      for (int k = 0; k < steps; ++k) {
        const int koff = lane_koff<QUANT, 1>(g, k);
        const bool act = koff < K;
        float x[TC][32];
        float xs[TC][4];
#pragma unroll
        for (int t = 0; t < TC; ++t)
          load_x<QUANT, XMODE>(xrow[t], koff, act, g, x[t], xs[t], XMODE == kXNorm ? norm[t] : XNorm{1.0f, nullptr});
        const size_t off = (size_t)row0 * row_bytes + (size_t)k * F::kChunkBytes;
        Raw r0;
        load_raw<QUANT>(w0 + off, act, g, r0);
        accum<QUANT, TC>(r0, g, x, xs, tot[0]);
        if constexpr (NM == 2) {
          Raw r1;
          load_raw<QUANT>(w1 + off, act, g, r1);
          accum<QUANT, TC>(r1, g, x, xs, tot[NM - 1]);
        }
      }
#pragma unroll
      for (int m = 0; m < NM; ++m)
#pragma unroll
        for (int t = 0; t < TC; ++t) tot[m][t] = group_sum<64>(tot[m][t]);
      if (g.lane == 0) {
#pragma unroll
        for (int t = 0; t < TC; ++t) {
          const float v = NM == 2 ? silu_f(tot[0][t]) * tot[NM - 1][t] : scale[t] * tot[0][t];
          if constexpr (OMODE == kOCoherent) store_coherent(&out[t][row0], v);
          else out[t][row0] = v;
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------------
// Kernels.  grid.x tiles the output rows, grid.y enumerates work units; every grid is
// a function of the geometry, the live token count is read from `valid_tokens`.
// ---------------------------------------------------------------------------------
struct ExpertArgs {
  const uint8_t* w0;         // gate stack (NM=2) or down stack (NM=1)
  const uint8_t* w1;         // up stack (NM=2) or unused
  size_t expert_bytes;       // bytes of one expert in a stack (0 for a single-expert stack)
  const float* x;            // activations: [token][K] (gate/up: normed; down: inter rows)
  float* out;                // gate/up: inter [unit][n_rows]; down: partial/out [unit][n_rows]
  const int* valid_tokens;   // device scalar
  const int* topk_ids;       // [T][top_k]
  const float* topk_weights; // [T][top_k]
  const int* sorted_token_ids;
  const int* expert_ids;
  int K;                     // contraction length
  int n_rows;                // output rows per expert
  int top_k;
  int block_size;
  int tile_rows;             // rows per workgroup
};

// Flat regime (max_tokens <= 4, or the exact decode regime): one work unit per live
// (token, k) pair read straight from topk_ids; no dispatch table
// (crates/xabe-cuda/src/kernels/moe.rs:2525-2634, :3066-3124).
template <int QUANT, int KS, int RPS, int NM>
__device__ __forceinline__ void flat_body(const ExpertArgs& a, int p, int tile) {
  const int valid = *a.valid_tokens;
  if (p >= valid * a.top_k) return;
  const int e = a.topk_ids[p];
  const uint8_t* w0 = a.w0 + (size_t)e * a.expert_bytes;
  const uint8_t* w1 = NM == 2 ? a.w1 + (size_t)e * a.expert_bytes : nullptr;
  // gate/up reads the token's activation row; down reads the pair's own inter row
  const float* const xr[1] = {a.x + (size_t)(NM == 2 ? p / a.top_k : p) * a.K};
  float* const o[1] = {a.out + (size_t)p * a.n_rows};
  const float sc[1] = {NM == 2 ? 1.0f : a.topk_weights[p]};
  matvec_rows<QUANT, KS, RPS, 1, NM>(w0, w1, a.K, a.n_rows, tile * a.tile_rows, a.tile_rows, xr, o, sc);
}

template <int QUANT, int KS, int RPS, int NM>
__global__ void __launch_bounds__(256) k_expert_flat(ExpertArgs a) {
  flat_body<QUANT, KS, RPS, NM>(a, blockIdx.y, blockIdx.x);
}

// Dispatch-table regime: one work unit per dispatch block; the block's live slots all
// belong to one expert, whose rows are streamed once per chunk of two tokens
// (chunks after the first hit in L2).  gate/up writes inter[slot]; down reads
// inter[slot] and writes partial[flat].
template <int QUANT, int KS, int RPS, int NM>
__global__ void __launch_bounds__(256) k_expert_block(ExpertArgs a) {
  const int b = blockIdx.y;
  const int e = a.expert_ids[b];
  if (e < 0) return;
  const int valid = *a.valid_tokens;
  const int sentinel = valid * a.top_k;
  const uint8_t* w0 = a.w0 + (size_t)e * a.expert_bytes;
  const uint8_t* w1 = NM == 2 ? a.w1 + (size_t)e * a.expert_bytes : nullptr;
  const int* slots = a.sorted_token_ids + (size_t)b * a.block_size;
  for (int i = 0; i < a.block_size; i += 2) {
    const int f0 = slots[i];
    if (f0 >= sentinel) break;
    const int f1 = (i + 1 < a.block_size) ? slots[i + 1] : sentinel;
    const size_t s0 = (size_t)b * a.block_size + i;
    if (f1 < sentinel) {
      const float* const xr[2] = {a.x + (NM == 2 ? (size_t)(f0 / a.top_k) : s0) * a.K,
                                  a.x + (NM == 2 ? (size_t)(f1 / a.top_k) : s0 + 1) * a.K};
      float* const o[2] = {a.out + (NM == 2 ? s0 : (size_t)f0) * a.n_rows,
                           a.out + (NM == 2 ? s0 + 1 : (size_t)f1) * a.n_rows};
      const float sc[2] = {NM == 2 ? 1.0f : a.topk_weights[f0], NM == 2 ? 1.0f : a.topk_weights[f1]};
      matvec_rows<QUANT, KS, RPS, 2, NM>(w0, w1, a.K, a.n_rows, blockIdx.x * a.tile_rows, a.tile_rows, xr, o, sc);
    } else {
      const float* const xr[1] = {a.x + (NM == 2 ? (size_t)(f0 / a.top_k) : s0) * a.K};
      float* const o[1] = {a.out + (NM == 2 ? s0 : (size_t)f0) * a.n_rows};
      const float sc[1] = {NM == 2 ? 1.0f : a.topk_weights[f0]};
      matvec_rows<QUANT, KS, RPS, 1, NM>(w0, w1, a.K, a.n_rows, blockIdx.x * a.tile_rows, a.tile_rows, xr, o, sc);
    }
  }
}

// The same dispatch-table work unit with the weights resident: a workgroup's tile is exactly what its four
// wavefronts can hold in registers (DEPTH steps each), every weight byte is requested before the first wait,
// and the block's token chunks then run against those registers -- the weights are read once per block
// instead of once per chunk, and a wavefront's loads are all in flight together instead of one step at a
// time.  Rows of at most 2048 elements (one step); n_rows must be a multiple of 4 * DEPTH * RPS.
// The per-row arithmetic is matvec_rows', so the outputs are bit-identical to k_expert_block's.
template <int N>
struct TcC {
  static constexpr int value = N;
};

template <int QUANT, int RPS, int NM, int DEPTH>
__global__ void __launch_bounds__(256) k_expert_block_resident(ExpertArgs a) {
  using F = Fmt<QUANT>;
  using Raw = typename F::Raw;
  constexpr int G = 64 / RPS;
  const int b = blockIdx.y;
  const int* slots = a.sorted_token_ids + (size_t)b * a.block_size;
  const int e = a.expert_ids[b];
  int f0 = slots[0], f1 = a.block_size > 1 ? slots[1] : 0x7fffffff;
  const int valid = *a.valid_tokens;
  if (e < 0) return;
  const int sentinel = valid * a.top_k;
  if (f0 >= sentinel) return;
  const LaneGeom g = lane_geom<QUANT>();
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int koff = lane_koff<QUANT, RPS>(g, 0);
  const size_t row_bytes = (size_t)(a.K / F::kBlockElems) * F::kBlockBytes;
  const uint8_t* w0 = a.w0 + (size_t)e * a.expert_bytes;
  const uint8_t* w1 = NM == 2 ? a.w1 + (size_t)e * a.expert_bytes : nullptr;
  const int wave_row0 = ((int)blockIdx.x * kWavesPerWg + wave) * DEPTH * RPS;
  // a chunk's activation rows (the second repeats the first in a one-token chunk: loaded, never used)
  float x[2][32], xs[2][4];
  bool two;
  auto load_chunk = [&](int i) {
    two = f1 < sentinel;
    const size_t s0 = (size_t)b * a.block_size + i;
    load_x<QUANT>(a.x + (NM == 2 ? (size_t)(f0 / a.top_k) : s0) * a.K, koff, true, g, x[0], xs[0]);
    load_x<QUANT>(a.x + (NM == 2 ? (size_t)((two ? f1 : f0) / a.top_k) : (two ? s0 + 1 : s0)) * a.K, koff, true, g, x[1], xs[1]);
  };
  load_chunk(0);  // requested ahead of the weights, so it is there when they arrive
  Raw r[DEPTH][NM];
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) {
    const size_t off = (size_t)(wave_row0 + d * RPS) * row_bytes;
    load_raw<QUANT>(w0 + off, true, g, r[d][0]);
    if constexpr (NM == 2) load_raw<QUANT>(w1 + off, true, g, r[d][NM - 1]);
  }
  for (int i = 0;;) {
    const size_t s0 = (size_t)b * a.block_size + i;
    auto chunk = [&](auto tc_c) {
      constexpr int TC = decltype(tc_c)::value;
      const int f[2] = {f0, f1};
      const float (&xt)[TC][32] = *reinterpret_cast<const float (*)[TC][32]>(&x);
      const float (&xst)[TC][4] = *reinterpret_cast<const float (*)[TC][4]>(&xs);
      float* o[TC];
      float sc[TC];
#pragma unroll
      for (int t = 0; t < TC; ++t) {
        o[t] = a.out + (NM == 2 ? s0 + t : (size_t)f[t]) * a.n_rows;
        sc[t] = NM == 2 ? 1.0f : a.topk_weights[f[t]];
      }
#pragma unroll
      for (int d = 0; d < DEPTH; ++d) {
        float tot[NM][TC];
#pragma unroll
        for (int m = 0; m < NM; ++m) {
#pragma unroll
          for (int t = 0; t < TC; ++t) tot[m][t] = 0.0f;
          accum<QUANT, TC>(r[d][m], g, xt, xst, tot[m]);
#pragma unroll
          for (int t = 0; t < TC; ++t) tot[m][t] = group_sum<G>(tot[m][t]);
        }
        const int row = wave_row0 + d * RPS + g.lane / G;
        if ((g.lane % G) == 0) {
#pragma unroll
          for (int t = 0; t < TC; ++t) o[t][row] = NM == 2 ? silu_f(tot[0][t]) * tot[NM - 1][t] : sc[t] * tot[0][t];
        }
      }
    };
    if (two) chunk(TcC<2>{});
    else chunk(TcC<1>{});
    i += 2;
    if (i >= a.block_size) break;
    f0 = slots[i];
    f1 = (i + 1 < a.block_size) ? slots[i + 1] : sentinel;
    if (f0 >= sentinel) break;
    load_chunk(i);
  }
}

// Shared expert / dense MLP: every live token, no indirection, no routing weight
// (crates/xabe-cuda/src/kernels/moe.rs:3425-3725, :4082-4227).  One work unit per chunk of two tokens.
template <int QUANT, int KS, int RPS, int NM>
__device__ __forceinline__ void shared_body(const ExpertArgs& a, int chunk, int tile) {
  const int t0 = chunk * 2;
  const int valid = *a.valid_tokens;
  if (t0 >= valid) return;
  if (t0 + 1 < valid) {
    const float* const xr[2] = {a.x + (size_t)t0 * a.K, a.x + (size_t)(t0 + 1) * a.K};
    float* const o[2] = {a.out + (size_t)t0 * a.n_rows, a.out + (size_t)(t0 + 1) * a.n_rows};
    const float sc[2] = {1.0f, 1.0f};
    matvec_rows<QUANT, KS, RPS, 2, NM>(a.w0, a.w1, a.K, a.n_rows, tile * a.tile_rows, a.tile_rows, xr, o, sc);
  } else {
    const float* const xr[1] = {a.x + (size_t)t0 * a.K};
    float* const o[1] = {a.out + (size_t)t0 * a.n_rows};
    const float sc[1] = {1.0f};
    matvec_rows<QUANT, KS, RPS, 1, NM>(a.w0, a.w1, a.K, a.n_rows, tile * a.tile_rows, a.tile_rows, xr, o, sc);
  }
}

// The lane's 32 activations of one step from a row in global memory or LDS, raw (no arithmetic, so a
// caller can request them and other data together and do the arithmetic when they arrive).
template <int QUANT>
__device__ __forceinline__ void lane_x_load(const float* row, int koff, const LaneGeom& g, float (&v)[32]) {
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int off = QUANT == kQ6K ? koff + g.half * 128 + j * 32 + g.l8 * 8 : koff + j * 8;
    const float4 a = reinterpret_cast<const float4*>(row + off)[0];
    const float4 b = reinterpret_cast<const float4*>(row + off)[1];
    v[j * 8 + 0] = a.x; v[j * 8 + 1] = a.y; v[j * 8 + 2] = a.z; v[j * 8 + 3] = a.w;
    v[j * 8 + 4] = b.x; v[j * 8 + 5] = b.y; v[j * 8 + 6] = b.z; v[j * 8 + 7] = b.w;
  }
}

// xs[j] = -32 * (sum of the j-th eight), the Q6_K code offset folded out of the inner loop (as load_x).
template <int QUANT>
__device__ __forceinline__ void lane_x_offsets(const float (&x)[32], float (&xs)[4]) {
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) s += x[j * 8 + i];
    xs[j] = QUANT == kQ6K ? -32.0f * s : 0.0f;
  }
}

// Everything above this point in program order has been issued before anything below it is: keeps the
// compiler from sinking a batch of loads down to their first uses, which would serialise them.
__device__ __forceinline__ void issue_fence() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);
}

// Shared expert / dense MLP with rows longer than one step (the dense sibling: 5120 and 17408 elements).
// A wavefront owns R rows at a time and walks the contraction step by step with the rows inside: the step's
// weights for all R rows are requested together and the step's activations are read once per step instead
// of once per (row, step).  Per (row, token) the lane partial accumulates step after step and is reduced
// once at the end: the operation order of matvec_rows' long-row path, so the bits are the same.
// grid (row groups / wavefronts per workgroup; ceil(max_tokens / TOK)), TOK = 1 or 2 tokens per pass over
// the weights (later passes find most of them in the memory-side cache); 64 or 256 threads.
//   Software pipeline: the next step's weights are requested before this step's accumulation and its
//   activations right after it, into the registers the accumulation has just released.
//   Weights come through the coalesced loader (stage_load / stage_pick): the host takes this kernel only for
//   tensors that start and end on 16-byte boundaries.
//   RESID:  also write l_out = out + residual (the dense block's last step).
struct LongRowArgs {
  ExpertArgs m;
  const float* residual;  // RESID
  float* l_out;           // RESID
  int row_begin, row_end;  // k_long_rows_staged: the launch serves rows [row_begin, row_end); row_end 0 = all of them
};

//   XLDS:   the pass's activation rows are copied into LDS once per workgroup and every step reads its 32
//           elements per token and lane from there, just before they are used: no activation registers held
//           across a step, which is what lets a pass serve four tokens (each weight dequantised once for the
//           four) where the register form stops at two.  Workgroups of up to eight wavefronts, persistent over
//           the row groups; dynamic LDS = TOK * K floats, then the wavefronts' staging slots.
template <int QUANT, int NM, int R, int TOK, bool RESID, bool XLDS = false>
__global__ void __launch_bounds__(XLDS ? 512 : 256) k_shared_long_rows(LongRowArgs la) {
  using F = Fmt<QUANT>;
  using Raw = typename F::Raw;
  constexpr int kSlot = StageFmt<QUANT>::kSlotBytes;
  __shared__ __attribute__((aligned(16))) uint8_t s_slots_static[XLDS ? 16 : kWavesPerWg * R * NM * kSlot];
  extern __shared__ __attribute__((aligned(16))) float s_xrows[];
  const ExpertArgs& a = la.m;
  const int valid = *a.valid_tokens;
  const int t0 = blockIdx.y * TOK;
  if (t0 >= valid) return;
  const int nt = min(TOK, valid - t0);
  const LaneGeom g = lane_geom<QUANT>();
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const size_t row_bytes = (size_t)(a.K / F::kBlockElems) * F::kBlockBytes;
  const int steps = (a.K + kStepElems - 1) / kStepElems;
  const int wg_waves = (int)(blockDim.x >> 6);  // 4, or 1 for a matrix with few row groups (XLDS: up to 8)
  uint8_t* const s_slots = XLDS ? reinterpret_cast<uint8_t*>(s_xrows + (size_t)TOK * a.K) : s_slots_static;
  if constexpr (XLDS) {
    // (a token past the batch copies the last live one: computed, never stored)
    const int n4 = a.K / 4;
#pragma unroll
    for (int t = 0; t < TOK; ++t) {
      const float4* src = reinterpret_cast<const float4*>(a.x + (size_t)(t0 + min(t, nt - 1)) * a.K);
      float4* dst = reinterpret_cast<float4*>(s_xrows + (size_t)t * a.K);
      for (int i = threadIdx.x; i < n4; i += blockDim.x) dst[i] = src[i];
    }
    __syncthreads();
  }
#pragma unroll 1
  for (int rg = (int)blockIdx.x * wg_waves + wave; rg < a.n_rows / R; rg += (int)gridDim.x * wg_waves) {
    const int row0 = rg * R;
    float acc[R][NM][TOK];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int m = 0; m < NM; ++m)
#pragma unroll
        for (int t = 0; t < TOK; ++t) acc[r][m][t] = 0.0f;
    float x[XLDS ? 1 : TOK][32];
    Staged<QUANT> pend[R][NM];
    // raw activations of step k.  Unconditional loads from clamped addresses (a token past the batch reads
    // the last live one, a lane past the end of the row its last block): a select here would need the data
    // at once and stall the pipeline; lanes past the row are zeroed where the values are used.
    auto issue_x = [&](int k) __attribute__((always_inline)) {
      if constexpr (XLDS) return;
      const int koff = min(lane_koff<QUANT, 1>(g, k), a.K - F::kBlockElems);
#pragma unroll
      for (int t = 0; t < TOK; ++t) lane_x_load<QUANT>(a.x + (size_t)(t0 + min(t, nt - 1)) * a.K, koff, g, x[t]);
      issue_fence();
    };
    auto issue_w = [&](int k) __attribute__((always_inline)) {
      // live bytes of this step: whole blocks up to the end of the row
      const uint32_t nbytes = (uint32_t)(min(kStepElems, a.K - k * kStepElems) / F::kBlockElems) * F::kBlockBytes;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const size_t off = (size_t)(row0 + r) * row_bytes + (size_t)k * F::kChunkBytes;
        stage_load<QUANT>(a.w0 + off, nbytes, pend[r][0]);
        if constexpr (NM == 2) stage_load<QUANT>(a.w1 + off, nbytes, pend[r][NM - 1]);
      }
      issue_fence();
    };
    issue_x(0);
    issue_w(0);
#pragma unroll 1
    for (int k = 0; k < steps; ++k) {
      const bool act = lane_koff<QUANT, 1>(g, k) < a.K;
      float xl[TOK][32], xs[TOK][4];
      if constexpr (!XLDS) {
#pragma unroll
        for (int t = 0; t < TOK; ++t) {
#pragma unroll
          for (int i = 0; i < 32; ++i) xl[t][i] = act ? x[t][i] : 0.0f;
          lane_x_offsets<QUANT>(xl[t], xs[t]);
        }
      }
      Raw raw[R][NM];
#pragma unroll
      for (int r = 0; r < R; ++r)
#pragma unroll
        for (int m = 0; m < NM; ++m)
          stage_pick<QUANT>(pend[r][m], s_slots + (size_t)((wave * R + r) * NM + m) * kSlot, act, g, raw[r][m]);
      if (k + 1 < steps) issue_w(k + 1);
      if constexpr (XLDS) {
        // the step's activations, out of LDS, once the staging registers above have been handed back
        const int koff = min(lane_koff<QUANT, 1>(g, k), a.K - F::kBlockElems);
#pragma unroll
        for (int t = 0; t < TOK; ++t) {
          lane_x_load<QUANT>(s_xrows + (size_t)t * a.K, koff, g, xl[t]);
#pragma unroll
          for (int i = 0; i < 32; ++i) xl[t][i] = act ? xl[t][i] : 0.0f;
          lane_x_offsets<QUANT>(xl[t], xs[t]);
        }
      }
#pragma unroll
      for (int r = 0; r < R; ++r)
#pragma unroll
        for (int m = 0; m < NM; ++m) accum<QUANT, TOK>(raw[r][m], g, xl, xs, acc[r][m]);
      if (k + 1 < steps) issue_x(k + 1);
    }
#pragma unroll
    for (int t = 0; t < TOK; ++t) {
      if (t >= nt) break;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        float tot[NM];
#pragma unroll
        for (int m = 0; m < NM; ++m) tot[m] = group_sum<64>(acc[r][m][t]);
        if (g.lane == 0) {
          const size_t i = (size_t)(t0 + t) * a.n_rows + row0 + r;
          const float v = NM == 2 ? silu_f(tot[0]) * tot[NM - 1] : 1.0f * tot[0];
          a.out[i] = v;
          if constexpr (RESID) la.l_out[i] = v + la.residual[i];
        }
      }
    }
  }
}

// The long-row kernel for five to eight tokens in ONE pass over the weights (more tokens: further passes of eight).
// With a lane's 32 activations per token held in registers a pass serves two tokens, or four with the rows in LDS
// (k_shared_long_rows); the dense sibling's down projection then reads its 73 MB four times at eight tokens.  Here
// the step's activations of all eight tokens (2048 elements each) are staged in LDS, double-buffered, by
// global -> LDS DMA in the order the lanes consume them ([place j][word w][token][lane] as 16-byte slots, conflict
// free), and a wavefront runs R rows (or gate/up pairs) against them with the work ordered place-major: for one
// place j the eight tokens' four activations of word w sit in 32 registers while every row's codes of that place
// are converted once and multiplied for all eight tokens.  Per (row, token) this is q6_accum's / q8_accum's
// sequence of operations exactly (acc_j: word 0's four products, then word 1's; tot += ds_j * (acc_j + xs_j) for
// j = 0..3; Q8_0: one accumulator over the eight words, tot += d * acc), the lane partial carried step after step
// and reduced once: the bits of k_shared_long_rows and of single-token decode.
// A workgroup is eight (or ten) wavefronts (wavefront w < 8 issues the DMA of place-word w), one per CU (144 KB of
// LDS), persistent over row groups of WAVES x R rows; the (group, step) sequence is one pipeline: while a step is multiplied
// the next step's activations and raw weight bytes are in flight.  Two barriers per step: the DMA has landed
// everywhere; the run sums (-32 * sum of each eight, Q6_K's code offset) have been formed from it, and lanes past
// the end of a row's last step zeroed.
constexpr int kStagedTok = 8;
constexpr size_t kStagedLdsBytes = 2 * (8 * kStagedTok * 64 * 16 + 4 * kStagedTok * 64 * 4);

// WAVES: wavefronts per workgroup, eight or ten (ten x two rows = twenty rows per group gives the down projection's
// 5120 rows one group per CU, where eight x four leave 96 of 256 CUs without work).
template <int QUANT, int NM, int R, bool RESID, int WAVES = 8>
__global__ void __launch_bounds__(64 * WAVES, WAVES > 8 ? 3 : 2) k_long_rows_staged(LongRowArgs la) {
  using F = Fmt<QUANT>;
  using Raw = typename F::Raw;
  constexpr int TOK = kStagedTok, RW = R * NM;
  extern __shared__ __attribute__((aligned(16))) uint8_t s_staged[];
  float4* const s_xq = reinterpret_cast<float4*>(s_staged);               // [2][8][TOK][64]
  float* const s_xs = reinterpret_cast<float*>(s_xq + 2 * 8 * TOK * 64);  // [2][4][TOK][64]
  const ExpertArgs& a = la.m;
  const int valid = *a.valid_tokens;
  const int t0 = blockIdx.y * TOK;
  if (t0 >= valid) return;
  const int nt = min(TOK, valid - t0);
  const LaneGeom g = lane_geom<QUANT>();
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const size_t row_bytes = (size_t)(a.K / F::kBlockElems) * F::kBlockBytes;
  const int steps = (a.K + kStepElems - 1) / kStepElems;
  // groups of WAVES x R rows; this launch's range starts at group g0 (the host cuts ranges at group boundaries)
  const int g0 = la.row_begin / (WAVES * R);
  const int n_groups = (la.row_end ? la.row_end : a.n_rows) / (WAVES * R) - g0;
  if ((int)blockIdx.x >= n_groups) return;
  const int n_mine = (n_groups - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x;
  const int total = n_mine * steps;

  // DMA of step s into buffer b: this wavefront's place-word (j = wave >> 1, w = wave & 1) of all tokens
  const uint32_t lds_x = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)s_xq;
  auto stage = [&](int s, int b) __attribute__((always_inline)) {
    if (WAVES > 8 && wave >= 8) return;
    const int koff = min(lane_koff<QUANT, 1>(g, s), a.K - F::kBlockElems);
    const int j = wave >> 1, w = wave & 1;
    const int e = QUANT == kQ6K ? koff + g.half * 128 + j * 32 + g.l8 * 8 + w * 4 : koff + j * 8 + w * 4;
#pragma unroll
    for (int t = 0; t < TOK; ++t) {
      const uint32_t voff = (uint32_t)(((size_t)(t0 + min(t, nt - 1)) * a.K + e) * sizeof(float));
      const uint32_t dst = __builtin_amdgcn_readfirstlane(lds_x + (uint32_t)(((b * 8 + wave) * TOK + t) * 64 * 16));
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
      asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(a.x), "s"(dst) : "memory", "m0");
#pragma clang diagnostic pop
    }
  };
  // run sums of buffer b (step s), and zeros for the lanes past the end of the row: four runs per thread
  auto finish_stage = [&](int s, int b) __attribute__((always_inline)) {
    constexpr int kRuns = 4 * kStagedTok * 64, kThreads = 64 * WAVES;
#pragma unroll
    for (int i = 0; i < (kRuns + kThreads - 1) / kThreads; ++i) {
      const int r = (int)threadIdx.x + kThreads * i, ln = r & 63, t = (r >> 6) & 7, j = r >> 9;
      if (kRuns % kThreads != 0 && r >= kRuns) break;
      const int koff = QUANT == kQ6K ? ((ln >> 3) + s * 8) * 256 : (ln + s * 64) * 32;
      const bool act = koff < a.K;
      float4* p0 = s_xq + ((b * 8 + 2 * j) * TOK + t) * 64 + ln;
      float4* p1 = p0 + TOK * 64;
      float4 v0 = *p0, v1 = *p1;
      if (!act) {
        v0 = v1 = make_float4(0.f, 0.f, 0.f, 0.f);
        *p0 = v0;
        *p1 = v1;
      }
      if constexpr (QUANT == kQ6K) {
        float sum = 0.0f;  // (the order of lane_x_offsets)
        sum += v0.x; sum += v0.y; sum += v0.z; sum += v0.w;
        sum += v1.x; sum += v1.y; sum += v1.z; sum += v1.w;
        s_xs[((b * 4 + j) * TOK + t) * 64 + ln] = -32.0f * sum;
      }
    }
  };
  auto load_rows = [&](int grp, int s, Raw (&raw)[RW]) __attribute__((always_inline)) {
    const bool act = lane_koff<QUANT, 1>(g, s) < a.K;
    const int row0 = (grp * WAVES + wave) * R;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const size_t off = (size_t)(row0 + r) * row_bytes + (size_t)s * F::kChunkBytes;
      load_raw<QUANT, true>(a.w0 + off, act, g, raw[r * NM]);
      if constexpr (NM == 2) load_raw<QUANT, true>(a.w1 + off, act, g, raw[r * NM + NM - 1]);
    }
  };

  Raw raw_next[RW];
  stage(0, 0);
  load_rows(g0 + (int)blockIdx.x, 0, raw_next);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  finish_stage(0, 0);
  __syncthreads();

  float tot[RW][TOK];
#pragma unroll
  for (int rw = 0; rw < RW; ++rw)
#pragma unroll
    for (int t = 0; t < TOK; ++t) tot[rw][t] = 0.0f;
  int grp = g0 + (int)blockIdx.x, s = 0;
#pragma unroll 1
  for (int i = 0; i < total; ++i) {
    const int b = i & 1;
    Raw raw[RW];
#pragma unroll
    for (int rw = 0; rw < RW; ++rw) raw[rw] = raw_next[rw];
    const int s_n = s + 1 < steps ? s + 1 : 0, grp_n = s + 1 < steps ? grp : grp + (int)gridDim.x;
    if (i + 1 < total) {
      stage(s_n, b ^ 1);
      load_rows(grp_n, s_n, raw_next);
      issue_fence();
    }
    // ---- this step, place-major
    const float4* xq = s_xq + (size_t)b * 8 * TOK * 64 + g.lane;
    const float* xsb = s_xs + (size_t)b * 4 * TOK * 64 + g.lane;
    float accj[RW][TOK];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (QUANT == kQ6K || j == 0) {
#pragma unroll
        for (int rw = 0; rw < RW; ++rw)
#pragma unroll
          for (int t = 0; t < TOK; ++t) accj[rw][t] = 0.0f;
      }
#pragma unroll
      for (int w = 0; w < 2; ++w) {
        float4 xv[TOK];
#pragma unroll
        for (int t = 0; t < TOK; ++t) xv[t] = xq[((2 * j + w) * TOK + t) * 64];
#pragma unroll
        for (int rw = 0; rw < RW; ++rw) {
          float f0, f1, f2, f3;
          if constexpr (QUANT == kQ6K) {
            const Q6Raw& r = raw[rw];
            const uint32_t qa = w ? r.qa1 : r.qa0, qb = w ? r.qb1 : r.qb0, qh = w ? r.qh1 : r.qh0;
            const uint32_t c = j == 0   ? (qa & 0x0F0F0F0Fu) | ((qh << 4) & 0x30303030u)
                               : j == 1 ? (qb & 0x0F0F0F0Fu) | ((qh << 2) & 0x30303030u)
                               : j == 2 ? ((qa >> 4) & 0x0F0F0F0Fu) | (qh & 0x30303030u)
                                        : ((qb >> 4) & 0x0F0F0F0Fu) | ((qh >> 2) & 0x30303030u);
            f0 = ub0(c), f1 = ub1(c), f2 = ub2(c), f3 = ub3(c);
          } else {
            const uint32_t c = raw[rw].q[2 * j + w];
            f0 = sb0(c), f1 = sb1(c), f2 = sb2(c), f3 = sb3(c);
          }
#pragma unroll
          for (int t = 0; t < TOK; ++t) {
            float v = accj[rw][t];
            v = __builtin_fmaf(f0, xv[t].x, v);
            v = __builtin_fmaf(f1, xv[t].y, v);
            v = __builtin_fmaf(f2, xv[t].z, v);
            v = __builtin_fmaf(f3, xv[t].w, v);
            accj[rw][t] = v;
          }
        }
      }
      if constexpr (QUANT == kQ6K) {
        float xsj[TOK];
#pragma unroll
        for (int t = 0; t < TOK; ++t) xsj[t] = xsb[(j * TOK + t) * 64];
        const int is8 = (g.l8 >> 1) * 8;
#pragma unroll
        for (int rw = 0; rw < RW; ++rw) {
          const uint32_t sw = (j < 2 ? raw[rw].sc0 : raw[rw].sc1) >> is8;
          const float ds = f16_bits_to_f32(raw[rw].dh) * (float)(int8_t)((j & 1 ? sw >> 16 : sw) & 0xff);
#pragma unroll
          for (int t = 0; t < TOK; ++t) tot[rw][t] = __builtin_fmaf(ds, accj[rw][t] + xsj[t], tot[rw][t]);
        }
      }
    }
    if constexpr (QUANT != kQ6K) {
#pragma unroll
      for (int rw = 0; rw < RW; ++rw) {
        const float d = f16_bits_to_f32(raw[rw].dh);
#pragma unroll
        for (int t = 0; t < TOK; ++t) tot[rw][t] = __builtin_fmaf(d, accj[rw][t], tot[rw][t]);
      }
    }
    if (s == steps - 1) {
      // the group's rows are complete: reduce over the lanes once, store, start over
      const int row0 = (grp * WAVES + wave) * R;
#pragma unroll
      for (int t = 0; t < TOK; ++t) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
          float red[NM];
#pragma unroll
          for (int m = 0; m < NM; ++m) red[m] = group_sum<64>(tot[r * NM + m][t]);
          if (g.lane == 0 && t < nt) {
            const size_t o = (size_t)(t0 + t) * a.n_rows + row0 + r;
            const float v = NM == 2 ? silu_f(red[0]) * red[NM - 1] : 1.0f * red[0];
            a.out[o] = v;
            if constexpr (RESID) la.l_out[o] = v + la.residual[o];
          }
        }
      }
#pragma unroll
      for (int rw = 0; rw < RW; ++rw)
#pragma unroll
        for (int t = 0; t < TOK; ++t) tot[rw][t] = 0.0f;
    }
    // the next step's activations have landed (requested a whole step ago) and everyone is done with this buffer
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (i + 1 < total) finish_stage(s_n, b ^ 1);
    __syncthreads();
    s = s_n;
    grp = grp_n;
  }
}

template <int QUANT, int KS, int RPS, int NM>
__global__ void __launch_bounds__(256) k_expert_shared(ExpertArgs a) {
  shared_body<QUANT, KS, RPS, NM>(a, blockIdx.y, blockIdx.x);
}

// The shared expert's work units appended to the routed grid (blockIdx.y >= routed_units), each
// unit running the body its separate launch runs, so every output is bit-identical to the
// four-launch form (crates/xabe-cuda/src/kernels/moe.rs:3727-4032).
struct FusedArgs {
  ExpertArgs routed;
  ExpertArgs shared;
  int routed_units;
};

template <int RQ, int SQ, int KS, int RPS, int NM>
__global__ void __launch_bounds__(256) k_expert_flat_with_shared(FusedArgs a) {
  const int unit = blockIdx.y;
  if (unit < a.routed_units) flat_body<RQ, KS, RPS, NM>(a.routed, unit, blockIdx.x);
  else shared_body<SQ, KS, RPS, NM>(a.shared, unit - a.routed_units, blockIdx.x);
}

}  // namespace xabe

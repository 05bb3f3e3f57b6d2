// Device-side primitives shared by every kernel: 2-byte-aligned block streaming,
// in-register Q6_K / Q8_0 unpack, and the fixed-order wavefront reductions.
//
// gfx950 only: wave64, DPP row operations, v_alignbit funnel shifts.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace xabe {

constexpr int kQ6K = 0;
constexpr int kQ8_0 = 1;
constexpr int kF32 = 2;          // plain fp32 rows (the f32 router), same lane/element mapping as Q8_0
constexpr int kQ6KBytes = 210;   // ql[128] qh[64] scales[16] d (crates/xabe-kernels/src/quant.rs:729)
constexpr int kQ8Bytes = 34;     // d, qs[32]                  (crates/xabe-kernels/src/quant.rs:726)
constexpr int kStepElems = 2048; // elements one wavefront covers per step: 64 lanes x 32

__device__ __forceinline__ float f16_bits_to_f32(uint32_t h) {
  return (float)__builtin_bit_cast(_Float16, (uint16_t)h);
}

// ---------------------------------------------------------------------------------
// Wavefront reductions.  The order is part of the numerics contract: a row's value
// must not depend on which other tokens share the launch, so every kernel reduces a
// row with exactly this tree.  `G` is the number of consecutive lanes that hold one
// row's partials (8, 16, 32 or 64).
// ---------------------------------------------------------------------------------
template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
  int r = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true);
  return v + __builtin_bit_cast(float, r);
}

__device__ __forceinline__ float lane_bcast(float v, int lane) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

// After this call every lane of a G-lane group holds the group's sum.
template <int G>
__device__ __forceinline__ float group_sum(float v) {
  static_assert(G == 8 || G == 16 || G == 32 || G == 64, "group width");
  v = dpp_add<0xB1>(v);   // quad_perm [1,0,3,2]
  v = dpp_add<0x4E>(v);   // quad_perm [2,3,0,1]
  v = dpp_add<0x141>(v);  // row_half_mirror: lanes i <-> 7-i within each 8
  if (G >= 16) v = dpp_add<0x140>(v);  // row_mirror: lanes i <-> 15-i within each 16
  if (G == 32) {
    float a = lane_bcast(v, 0), b = lane_bcast(v, 16), c = lane_bcast(v, 32), d = lane_bcast(v, 48);
    float lo = a + b, hi = c + d;
    v = (__lane_id() < 32) ? lo : hi;
  }
  if (G == 64) {
    float a = lane_bcast(v, 0), b = lane_bcast(v, 16), c = lane_bcast(v, 32), d = lane_bcast(v, 48);
    v = (a + b) + (c + d);
  }
  return v;
}

// Wavefront max / min over all 64 lanes (order-free, exact): DPP within 16-lane rows, then the four row
// results through scalar broadcasts.  Every lane receives the result.
template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
template <int CTRL>
__device__ __forceinline__ int dpp_i(int v) {
  return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, true);
}
__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, dpp_f<0xB1>(v));
  v = fmaxf(v, dpp_f<0x4E>(v));
  v = fmaxf(v, dpp_f<0x141>(v));
  v = fmaxf(v, dpp_f<0x140>(v));
  return fmaxf(fmaxf(lane_bcast(v, 0), lane_bcast(v, 16)), fmaxf(lane_bcast(v, 32), lane_bcast(v, 48)));
}
__device__ __forceinline__ int wave_max_i(int v) {
  v = max(v, dpp_i<0xB1>(v));
  v = max(v, dpp_i<0x4E>(v));
  v = max(v, dpp_i<0x141>(v));
  v = max(v, dpp_i<0x140>(v));
  const int a = __builtin_amdgcn_readlane(v, 0), b = __builtin_amdgcn_readlane(v, 16);
  const int c = __builtin_amdgcn_readlane(v, 32), d = __builtin_amdgcn_readlane(v, 48);
  return max(max(a, b), max(c, d));
}
__device__ __forceinline__ int wave_min_i(int v) {
  v = min(v, dpp_i<0xB1>(v));
  v = min(v, dpp_i<0x4E>(v));
  v = min(v, dpp_i<0x141>(v));
  v = min(v, dpp_i<0x140>(v));
  const int a = __builtin_amdgcn_readlane(v, 0), b = __builtin_amdgcn_readlane(v, 16);
  const int c = __builtin_amdgcn_readlane(v, 32), d = __builtin_amdgcn_readlane(v, 48);
  return min(min(a, b), min(c, d));
}

// 1 / sqrt(mean(x^2) + eps) of one row, computed by one wavefront in a fixed order: lane L folds
// elements 32L..32L+31 of every 2048-element chunk sequentially, then the wavefront tree.  Every kernel
// that needs the RMS scale of a token goes through rms_fold / rms_finish, so they all see the same bits.
struct RmsRaw {
  float4 q[8];  // the lane's 32 elements of one chunk (zeros past the end of the row: fma(0, 0, s) == s)
};

__device__ __forceinline__ void rms_load(const float* __restrict__ x, int chunk0, int width, RmsRaw& r) {
  const int base = chunk0 + (int)__lane_id() * 32;
#pragma unroll
  for (int i = 0; i < 8; ++i)  // width is a multiple of 4
    r.q[i] = base + 4 * i < width ? reinterpret_cast<const float4*>(x + base)[i] : make_float4(0.f, 0.f, 0.f, 0.f);
}

__device__ __forceinline__ float rms_fold(const RmsRaw& r, float s) {
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    s = __builtin_fmaf(r.q[i].x, r.q[i].x, s);
    s = __builtin_fmaf(r.q[i].y, r.q[i].y, s);
    s = __builtin_fmaf(r.q[i].z, r.q[i].z, s);
    s = __builtin_fmaf(r.q[i].w, r.q[i].w, s);
  }
  return s;
}

__device__ __forceinline__ float rms_finish(float lane_sum, int width, float eps) {
  const float ss = group_sum<64>(lane_sum);
  return 1.0f / sqrtf(ss / (float)width + eps);
}

// Three chunks are requested together (a chunk past the end of the row loads nothing and folds zeros,
// which leave the sum as it is), then folded in chunk order.
__device__ __forceinline__ float row_inv_rms(const float* __restrict__ x, int width, float eps) {
  float s = 0.0f;
  for (int c = 0; c < width; c += 3 * 2048) {
    RmsRaw r[3];
#pragma unroll
    for (int i = 0; i < 3; ++i) rms_load(x, c + 2048 * i, width, r[i]);
#pragma unroll
    for (int i = 0; i < 3; ++i) s = rms_fold(r[i], s);
  }
  return rms_finish(s, width, eps);
}

// ---------------------------------------------------------------------------------
// Streaming loads.  Blocks are 210 or 34 bytes, so block fields sit at 2-byte
// alignment.  Unaligned dword loads cost about 15 % of achieved bandwidth on this
// part; instead load the covering aligned dwords and funnel-shift by 0 or 16 bits.
// `base4` must be 4-byte aligned; `off` is a byte offset (even).
// ---------------------------------------------------------------------------------
__device__ __forceinline__ void load8_funnel(const uint8_t* base4, uint32_t off, uint32_t& lo, uint32_t& hi) {
  const uint32_t a = off & ~3u, sh = (off & 2u) << 3;
  const uint32_t* p = reinterpret_cast<const uint32_t*>(base4 + a);
  const uint32_t d0 = p[0], d1 = p[1], d2 = p[2];
  lo = __builtin_amdgcn_alignbit(d1, d0, sh);
  hi = __builtin_amdgcn_alignbit(d2, d1, sh);
}
// Same, but never touches the third dword unless the field really spills into it
// (the last field of the last block of a tensor must not be over-read).  Branch-free: an aligned field
// reads its second dword twice instead; a branch here would end the basic block and make the compiler
// wait for each block's loads before issuing the next block's.
__device__ __forceinline__ void load8_funnel_tail(const uint8_t* base4, uint32_t off, uint32_t& lo, uint32_t& hi) {
  const uint32_t a = off & ~3u, sh = (off & 2u) << 3;
  const uint32_t* p = reinterpret_cast<const uint32_t*>(base4 + a);
  const uint32_t d0 = p[0], d1 = p[1];
  const uint32_t d2 = p[sh ? 2 : 1];
  lo = __builtin_amdgcn_alignbit(d1, d0, sh);
  hi = __builtin_amdgcn_alignbit(d2, d1, sh);
}
__device__ __forceinline__ uint32_t load_u16(const uint8_t* base, uint32_t off) {
  return *reinterpret_cast<const uint16_t*>(base + off);
}

// ---------------------------------------------------------------------------------
// Q6_K.  One wavefront step covers 8 consecutive superblocks (1680 bytes).  Lane L:
// superblock slot L>>3, unit u = L&7 with half = u>>2 and l8 = u&3.  The lane owns,
// for each of the four interleaved code planes j, the eight codes at
//   half*128 + j*32 + l8*8 + i,  i = 0..7
// i.e. 32 elements as four runs of eight.  Scale index = half*8 + 2*j + (l8>>1).
// ---------------------------------------------------------------------------------
struct Q6Raw {
  uint32_t qa0, qa1, qb0, qb1, qh0, qh1, sc0, sc1, dh;
};

// `chunk4`: 4-byte-aligned pointer at or just below the step's first superblock;
// `lane_off`: byte offset of this lane's superblock from chunk4.
__device__ __forceinline__ void q6_load(const uint8_t* chunk4, uint32_t lane_off, int half, int l8, Q6Raw& r) {
  load8_funnel(chunk4, lane_off + half * 64 + l8 * 8, r.qa0, r.qa1);
  load8_funnel(chunk4, lane_off + half * 64 + 32 + l8 * 8, r.qb0, r.qb1);
  load8_funnel(chunk4, lane_off + 128 + half * 32 + l8 * 8, r.qh0, r.qh1);
  load8_funnel_tail(chunk4, lane_off + 192 + half * 8, r.sc0, r.sc1);
  r.dh = load_u16(chunk4, lane_off + 208);
}
// The same fields read where they lie, at the block's own two-byte alignment (vector memory loads take any
// alignment): the same Raw, with four load instructions of eight bytes instead of eleven dwords and no shifts.
// Slower than the aligned windows where a wavefront streams long runs of consecutive blocks (dispatch-table
// and long-row kernels: 202 against 211 us per block at 32 tokens), faster where it reads a few short rows
// per request (the decode block's launches: 37.1 against 36.0 us per block at 3 tokens).
__device__ __forceinline__ void q6_load_direct(const uint8_t* chunk4, uint32_t lane_off, int half, int l8, Q6Raw& r) {
  const uint8_t* blk = chunk4 + lane_off;
  uint2 v;
  __builtin_memcpy(&v, blk + half * 64 + l8 * 8, 8);
  r.qa0 = v.x, r.qa1 = v.y;
  __builtin_memcpy(&v, blk + half * 64 + 32 + l8 * 8, 8);
  r.qb0 = v.x, r.qb1 = v.y;
  __builtin_memcpy(&v, blk + 128 + half * 32 + l8 * 8, 8);
  r.qh0 = v.x, r.qh1 = v.y;
  __builtin_memcpy(&v, blk + 192 + half * 8, 8);
  r.sc0 = v.x, r.sc1 = v.y;
  r.dh = load_u16(chunk4, lane_off + 208);
}

__device__ __forceinline__ float ub0(uint32_t v) { return (float)(v & 0xffu); }
__device__ __forceinline__ float ub1(uint32_t v) { return (float)((v >> 8) & 0xffu); }
__device__ __forceinline__ float ub2(uint32_t v) { return (float)((v >> 16) & 0xffu); }
__device__ __forceinline__ float ub3(uint32_t v) { return (float)(v >> 24); }

// Position of lane element e (0..31) inside its superblock.
__device__ __forceinline__ int q6_pos(int half, int l8, int e) { return half * 128 + (e >> 3) * 32 + l8 * 8 + (e & 7); }

// The lane's contribution to the dot product of one superblock with TC activation
// vectors, added into tot[t].  x[t][e] holds the activation at q6_pos(e);
// xs[t][j] = -32 * (x[t][8j] + ... + x[t][8j+7]) removes the code offset, so the
// inner loop is one v_cvt_f32_ubyte and one fma per weight:
//   sum_j (d*sc_j) * (sum_i raw_ji * x_ji - 32 * sum_i x_ji)
// d*sc is exact in fp32 (11-bit x 8-bit significands).
template <int TC>
__device__ __forceinline__ void q6_accum(const Q6Raw& r, int l8, const float (&x)[TC][32], const float (&xs)[TC][4],
                                         float (&tot)[TC]) {
  float acc[TC][4];
#pragma unroll
  for (int t = 0; t < TC; ++t)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[t][j] = 0.0f;
#pragma unroll
  for (int w = 0; w < 2; ++w) {
    const uint32_t a = w ? r.qa1 : r.qa0, b = w ? r.qb1 : r.qb0, h = w ? r.qh1 : r.qh0;
    uint32_t c[4];
    c[0] = (a & 0x0F0F0F0Fu) | ((h << 4) & 0x30303030u);
    c[1] = (b & 0x0F0F0F0Fu) | ((h << 2) & 0x30303030u);
    c[2] = ((a >> 4) & 0x0F0F0F0Fu) | (h & 0x30303030u);
    c[3] = ((b >> 4) & 0x0F0F0F0Fu) | ((h >> 2) & 0x30303030u);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float f0 = ub0(c[j]), f1 = ub1(c[j]), f2 = ub2(c[j]), f3 = ub3(c[j]);
#pragma unroll
      for (int t = 0; t < TC; ++t) {
        float v = acc[t][j];
        v = __builtin_fmaf(f0, x[t][j * 8 + w * 4 + 0], v);
        v = __builtin_fmaf(f1, x[t][j * 8 + w * 4 + 1], v);
        v = __builtin_fmaf(f2, x[t][j * 8 + w * 4 + 2], v);
        v = __builtin_fmaf(f3, x[t][j * 8 + w * 4 + 3], v);
        acc[t][j] = v;
      }
    }
  }
  const int is8 = (l8 >> 1) * 8;
  const uint32_t slo = r.sc0 >> is8, shi = r.sc1 >> is8;
  const float d = f16_bits_to_f32(r.dh);
  const float ds0 = d * (float)(int8_t)(slo & 0xff), ds1 = d * (float)(int8_t)((slo >> 16) & 0xff);
  const float ds2 = d * (float)(int8_t)(shi & 0xff), ds3 = d * (float)(int8_t)((shi >> 16) & 0xff);
#pragma unroll
  for (int t = 0; t < TC; ++t) {
    float v = tot[t];
    v = __builtin_fmaf(ds0, acc[t][0] + xs[t][0], v);
    v = __builtin_fmaf(ds1, acc[t][1] + xs[t][1], v);
    v = __builtin_fmaf(ds2, acc[t][2] + xs[t][2], v);
    v = __builtin_fmaf(ds3, acc[t][3] + xs[t][3], v);
    tot[t] = v;
  }
}

// ---------------------------------------------------------------------------------
// Q8_0.  One wavefront step covers 64 consecutive blocks (2176 bytes); lane L owns
// block L: elements 0..31 in order.
// ---------------------------------------------------------------------------------
struct Q8Raw {
  uint32_t q[8];
  uint32_t dh;
};

__device__ __forceinline__ void q8_load(const uint8_t* chunk4, uint32_t lane_off, Q8Raw& r) {
  // qs start at lane_off + 2.  When that is 4-byte aligned the eight dwords are the
  // codes themselves; otherwise nine aligned dwords are funnel-shifted by 16 bits.
  const uint32_t qoff = lane_off + 2;
  const uint32_t a = qoff & ~3u, sh = (qoff & 2u) << 3;
  const uint32_t* p = reinterpret_cast<const uint32_t*>(chunk4 + a);
  uint32_t e[9];
#pragma unroll
  for (int i = 0; i < 8; ++i) e[i] = p[i];
  // The ninth piece is the block's last two codes only: a dword there would read two
  // bytes past the last block of a tensor.  Unused (and aimed at the block's first bytes, no branch) when
  // the codes are dword-aligned.
  e[8] = load_u16(chunk4, lane_off + (sh ? 32u : 0u));
#pragma unroll
  for (int i = 0; i < 8; ++i) r.q[i] = __builtin_amdgcn_alignbit(e[i + 1], e[i], sh);
  r.dh = load_u16(chunk4, lane_off);
}

__device__ __forceinline__ float sb0(uint32_t v) { return (float)(int8_t)(v & 0xff); }
__device__ __forceinline__ float sb1(uint32_t v) { return (float)(int8_t)((v >> 8) & 0xff); }
__device__ __forceinline__ float sb2(uint32_t v) { return (float)(int8_t)((v >> 16) & 0xff); }
__device__ __forceinline__ float sb3(uint32_t v) { return (float)(int8_t)(v >> 24); }

template <int TC>
__device__ __forceinline__ void q8_accum(const Q8Raw& r, const float (&x)[TC][32], float (&tot)[TC]) {
  float acc[TC];
#pragma unroll
  for (int t = 0; t < TC; ++t) acc[t] = 0.0f;
#pragma unroll
  for (int w = 0; w < 8; ++w) {
    const float f0 = sb0(r.q[w]), f1 = sb1(r.q[w]), f2 = sb2(r.q[w]), f3 = sb3(r.q[w]);
#pragma unroll
    for (int t = 0; t < TC; ++t) {
      float v = acc[t];
      v = __builtin_fmaf(f0, x[t][w * 4 + 0], v);
      v = __builtin_fmaf(f1, x[t][w * 4 + 1], v);
      v = __builtin_fmaf(f2, x[t][w * 4 + 2], v);
      v = __builtin_fmaf(f3, x[t][w * 4 + 3], v);
      acc[t] = v;
    }
  }
  const float d = f16_bits_to_f32(r.dh);
#pragma unroll
  for (int t = 0; t < TC; ++t) tot[t] = __builtin_fmaf(d, acc[t], tot[t]);
}

// ---------------------------------------------------------------------------------
// fp32 rows.  One wavefront step covers 2048 floats; lane L owns floats 32L..32L+31.
// ---------------------------------------------------------------------------------
struct F32Raw {
  float v[32];
};

__device__ __forceinline__ void f32_load(const uint8_t* chunk16, uint32_t lane_off, F32Raw& r) {
  const float4* p = reinterpret_cast<const float4*>(chunk16 + lane_off);
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const float4 a = p[i];
    r.v[i * 4 + 0] = a.x; r.v[i * 4 + 1] = a.y; r.v[i * 4 + 2] = a.z; r.v[i * 4 + 3] = a.w;
  }
}

template <int TC>
__device__ __forceinline__ void f32_accum(const F32Raw& r, const float (&x)[TC][32], float (&tot)[TC]) {
#pragma unroll
  for (int t = 0; t < TC; ++t) {
    float v = 0.0f;
#pragma unroll
    for (int i = 0; i < 32; ++i) v = __builtin_fmaf(r.v[i], x[t][i], v);
    tot[t] += v;
  }
}

// silu(x) = x / (1 + exp(-x)): one division, libm-grade expf (crates/xabe-kernels/src/norm.rs:46-48).
__device__ __forceinline__ float silu_f(float x) { return x / (1.0f + expf(-x)); }

}  // namespace xabe

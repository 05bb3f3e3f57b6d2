// The small kernels around the expert contractions: RMSNorm, routing, dispatch
// tables, combine, stand-alone dequantisation and the synthetic-stack generator.
#pragma once

#include "device_common.h"
#include "route_device.h"

namespace xabe {

// Sum over a 256-thread workgroup in a fixed order: the wavefront tree, then the four
// wavefront totals ascending.  `scratch` holds 4 floats.
__device__ __forceinline__ float block_sum_256(float v, float* scratch) {
  v = group_sum<64>(v);
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) scratch[wave] = v;
  __syncthreads();
  const float total = ((scratch[0] + scratch[1]) + scratch[2]) + scratch[3];
  __syncthreads();
  return total;
}

// ---------------------------------------------------------------------------------
// rms_norm_rows (crates/xabe-cuda/src/kernels/layer_ops.rs:129-151): every row of the
// buffer, y = x * (1/sqrtf(mean(x^2) + eps)) * w.  grid = rows, 256 threads.
// ---------------------------------------------------------------------------------
__global__ void __launch_bounds__(256) k_rms_norm_rows(const float* __restrict__ x, const float* __restrict__ w,
                                                        float* __restrict__ out, int width, float eps) {
  const float* xr = x + (size_t)blockIdx.x * width;
  float* o = out + (size_t)blockIdx.x * width;
  // width is a multiple of 4; up to eight float4 columns per thread (rows up to 8192 wide) are requested
  // together with the row's RMS chunks.  The guards are uniform, so the loads stay in flight together.
  const int n4 = width / 4;
  const float4* x4 = reinterpret_cast<const float4*>(xr);
  const float4* w4 = reinterpret_cast<const float4*>(w);
  float4* o4 = reinterpret_cast<float4*>(o);
  float4 xv[8], wv[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    if (256 * i < n4) {
      const int j = min((int)threadIdx.x + 256 * i, n4 - 1);
      xv[i] = x4[j];
      wv[i] = w4[j];
    }
  }
  const float inv = row_inv_rms(xr, width, eps);  // each wavefront computes the same scale
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int j = threadIdx.x + 256 * i;
    if (j < n4)
      o4[j] = make_float4(xv[i].x * inv * wv[i].x, xv[i].y * inv * wv[i].y, xv[i].z * inv * wv[i].z, xv[i].w * inv * wv[i].w);
  }
  for (int j = threadIdx.x + 2048; j < n4; j += 256) {
    const float4 a = x4[j], b = w4[j];
    o4[j] = make_float4(a.x * inv * b.x, a.y * inv * b.y, a.z * inv * b.z, a.w * inv * b.w);
  }
}

// Rows of at most 2048 elements: one wavefront per row, four rows per workgroup.  The lane's 32 elements are the ones
// rms_fold takes from it, but a lane fetching its own 128 bytes makes every load instruction touch 64 cache lines, so
// the row comes in as consecutive 16-byte pieces and changes hands through LDS (16-byte slot q of the row at
// q + q / 8: lanes reading eight consecutive slots each then start nine slots apart and take different banks), and
// goes out the same way; the norm weight is staged once per workgroup.  Same values in the same order as before
// (8192 rows of 2048 with the fp16 copy: 63 -> 31 us).
// WITH_H: the row also goes out as fp16 (the copy the matrix-core kernels read: the fp32 value rounded once, what
// the stand-alone conversion kernel writes).
template <bool WITH_H>
__global__ void __launch_bounds__(256) k_rms_norm_short_rows(const float* __restrict__ x, const float* __restrict__ w,
                                                              float* __restrict__ out, _Float16* __restrict__ out_h, int rows,
                                                              int width, float eps) {
  constexpr int kSlots = 512 + 64;  // padded 16-byte slots of one 2048-element row
  __shared__ float4 s_w[kSlots];
  __shared__ float4 s_row[4][kSlots];
  const int wave = (int)(threadIdx.x >> 6), lane = (int)__lane_id();
  const int n4 = width / 4;
  auto slot = [](int q) { return q + (q >> 3); };
  // the norm weight: 512 pieces over 256 threads
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int q = (int)threadIdx.x + 256 * j;
    s_w[slot(q)] = q < n4 ? reinterpret_cast<const float4*>(w)[q] : make_float4(0.f, 0.f, 0.f, 0.f);
  }
  const int row = blockIdx.x * 4 + wave;
  const bool live = row < rows;
  float4* mine = s_row[wave];
  if (live) {
    const float4* x4 = reinterpret_cast<const float4*>(x + (size_t)row * width);
    float4 piece[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int q = 64 * j + lane;
      piece[j] = q < n4 ? x4[q] : make_float4(0.f, 0.f, 0.f, 0.f);
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) mine[slot(64 * j + lane)] = piece[j];
  }
  __syncthreads();  // (the weight for everyone; the row's own pieces only cross lanes of one wavefront)
  if (!live) return;
  RmsRaw r, nw;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    r.q[i] = mine[slot(8 * lane + i)];
    nw.q[i] = s_w[slot(8 * lane + i)];
  }
  const float inv = rms_finish(rms_fold(r, 0.0f), width, eps);
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();  // every lane has read its pieces before they are overwritten
#pragma unroll
  for (int i = 0; i < 8; ++i)
    mine[slot(8 * lane + i)] = make_float4(r.q[i].x * inv * nw.q[i].x, r.q[i].y * inv * nw.q[i].y, r.q[i].z * inv * nw.q[i].z,
                                           r.q[i].w * inv * nw.q[i].w);
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  float4* o4 = reinterpret_cast<float4*>(out + (size_t)row * width);
  [[maybe_unused]] uint2* h4 = reinterpret_cast<uint2*>(out_h + (WITH_H ? (size_t)row * width : 0));
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int q = 64 * j + lane;
    if (q < n4) {
      const float4 v = mine[slot(q)];
      o4[q] = v;
      if constexpr (WITH_H) {
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        const h2 lo = {(_Float16)v.x, (_Float16)v.y}, hi = {(_Float16)v.z, (_Float16)v.w};
        h4[q] = make_uint2(__builtin_bit_cast(uint32_t, lo), __builtin_bit_cast(uint32_t, hi));
      }
    }
  }
}

__global__ void __launch_bounds__(256) k_route(const float* __restrict__ logits, const int* __restrict__ valid_tokens,
                                                int num_experts, int top_k, int* __restrict__ topk_ids,
                                                float* __restrict__ topk_weights) {
  extern __shared__ float route_smem[];  // 4 x num_experts
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int t = blockIdx.x * 4 + wave;
  if (t >= *valid_tokens) return;
  int sel_i;
  float sel_w;
  route_one_token(logits + (size_t)t * num_experts, num_experts, top_k, route_smem + (size_t)wave * num_experts, sel_i,
                  sel_w);
  if (lane < top_k) {
    topk_ids[(size_t)t * top_k + lane] = sel_i;
    topk_weights[(size_t)t * top_k + lane] = sel_w;
  }
}

// route_load for logits that are still the `splits` (at most 8) partial planes of a split contraction, `plane_stride`
// floats apart: the planes are added in part order and the bias (may be null) after them, as the stand-alone sum
// does, and the finished logits are written to `lg_out`.
template <int PER>
__device__ __forceinline__ void route_load_planes(const float* planes, size_t plane_stride, int splits, int num_experts,
                                                  const float* __restrict__ bias, float* lg_out, float (&l)[PER]) {
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int idx = i * 64 + lane;
    l[i] = -INFINITY;
    if (idx < num_experts) {
      float part[8];
#pragma unroll
      for (int z = 0; z < 8; ++z) part[z] = z < splits ? planes[(size_t)z * plane_stride + idx] : 0.0f;
      float s = part[0];
#pragma unroll
      for (int z = 1; z < 8; ++z)
        if (z < splits) s += part[z];
      if (bias) s += bias[idx];
      lg_out[idx] = s;
      l[i] = s;
    }
  }
}

// The same routing for logits that a split router GEMM left as partial planes: a token's wavefront adds its row of
// the planes (and the bias) in the order of k_router_sum_planes, writes the finished logits, and routes them.
__global__ void __launch_bounds__(256) k_route_planes(const float* __restrict__ planes, size_t plane_stride, int splits,
                                                       const float* __restrict__ bias, const int* __restrict__ valid_tokens,
                                                       int num_experts, int top_k, float* __restrict__ logits,
                                                       int* __restrict__ topk_ids, float* __restrict__ topk_weights) {
  extern __shared__ float route_smem[];  // 4 x num_experts
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int t = blockIdx.x * 4 + wave;
  if (t >= *valid_tokens) return;
  int sel_i;
  float sel_w;
  const size_t row = (size_t)t * num_experts;
  float* e_all = route_smem + (size_t)wave * num_experts;
  if (num_experts <= 256) {
    float l[4];
    route_load_planes<4>(planes + row, plane_stride, splits, num_experts, bias, logits + row, l);
    route_compute<4>(l, num_experts, top_k, e_all, sel_i, sel_w);
  } else {
    float l[kRouteMaxPerLane];
    route_load_planes<kRouteMaxPerLane>(planes + row, plane_stride, splits, num_experts, bias, logits + row, l);
    route_compute<kRouteMaxPerLane>(l, num_experts, top_k, e_all, sel_i, sel_w);
  }
  if (lane < top_k) {
    topk_ids[(size_t)t * top_k + lane] = sel_i;
    topk_weights[(size_t)t * top_k + lane] = sel_w;
  }
}

// ---------------------------------------------------------------------------------
// Dispatch tables (crates/xabe-cuda/src/kernels/moe.rs:2233-2366; CPU:
// crates/xabe-kernels/src/moe/dispatch.rs:60-131).  Two launches of num_experts workgroups.
//   count:   per-expert selection counts; whole-capacity sentinel / -1 / 0 fill.
//   scatter: exclusive prefix of padded counts (recomputed per workgroup), then the
//            expert's flat ids in ascending order, by a workgroup scan: no atomics,
//            so the order is the CPU reference's.
// ---------------------------------------------------------------------------------
__global__ void __launch_bounds__(256) k_align_count(const int* __restrict__ topk_ids, const int* __restrict__ valid_tokens,
                                                      int top_k, int sorted_capacity, int expert_capacity,
                                                      int* __restrict__ sorted_token_ids, int* __restrict__ expert_ids,
                                                      int* __restrict__ bucket_live, int* __restrict__ expert_counts) {
  __shared__ int red[4];
  const int e = blockIdx.x;
  const int numel = *valid_tokens * top_k;
  int c = 0;
  for (int i = threadIdx.x; i < numel; i += 256) c += topk_ids[i] == e;
  for (int off = 32; off > 0; off >>= 1) c += __shfl_xor(c, off, 64);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = c;
  __syncthreads();
  if (threadIdx.x == 0) expert_counts[e] = red[0] + red[1] + red[2] + red[3];
  // fill this workgroup's slice of the fixed-capacity tables
  const int nb = gridDim.x;
  for (int i = e * 256 + threadIdx.x; i < sorted_capacity; i += nb * 256) sorted_token_ids[i] = numel;
  for (int i = e * 256 + threadIdx.x; i < expert_capacity; i += nb * 256) {
    expert_ids[i] = -1;
    bucket_live[i] = 0;
  }
}

__global__ void __launch_bounds__(256) k_align_scatter(const int* __restrict__ topk_ids, const int* __restrict__ valid_tokens,
                                                        const int* __restrict__ expert_counts, int top_k, int num_experts,
                                                        int block_size, int sorted_capacity, int expert_capacity,
                                                        int* __restrict__ sorted_token_ids, int* __restrict__ expert_ids,
                                                        int* __restrict__ num_tokens_post_pad, int* __restrict__ bucket_live) {
  __shared__ int s_wave[4];
  __shared__ int s_base;
  __shared__ int s_total;
  const int e = blockIdx.x;
  const int numel = *valid_tokens * top_k;
  // exclusive prefix of padded counts below e, and the grand total
  int below = 0, total = 0;
  for (int i = threadIdx.x; i < num_experts; i += 256) {
    const int padded = (expert_counts[i] + block_size - 1) / block_size * block_size;
    total += padded;
    if (i < e) below += padded;
  }
  for (int off = 32; off > 0; off >>= 1) {
    below += __shfl_xor(below, off, 64);
    total += __shfl_xor(total, off, 64);
  }
  if ((threadIdx.x & 63) == 0) s_wave[threadIdx.x >> 6] = below;
  __syncthreads();
  if (threadIdx.x == 0) s_base = s_wave[0] + s_wave[1] + s_wave[2] + s_wave[3];
  __syncthreads();
  if ((threadIdx.x & 63) == 0) s_wave[threadIdx.x >> 6] = total;
  __syncthreads();
  if (threadIdx.x == 0) s_total = s_wave[0] + s_wave[1] + s_wave[2] + s_wave[3];
  __syncthreads();
  const int base = s_base;
  if (e == 0 && threadIdx.x == 0) *num_tokens_post_pad = s_total;
  const int count = expert_counts[e];
  // this expert's blocks
  const int nblk = (count + block_size - 1) / block_size;
  for (int b = threadIdx.x; b < nblk; b += 256) {
    const int blk = base / block_size + b;
    if (blk < expert_capacity) {
      expert_ids[blk] = e;
      bucket_live[blk] = min(block_size, count - b * block_size);
    }
  }
  // ordered placement: running offset + workgroup exclusive scan of the match flags
  int running = 0;
  for (int i0 = 0; i0 < numel; i0 += 256) {
    const int i = i0 + threadIdx.x;
    const int flag = (i < numel) && (topk_ids[i] == e);
    const unsigned long long ballot = __ballot(flag);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int before = __popcll(ballot & ((1ull << lane) - 1ull));
    __syncthreads();
    if (lane == 0) s_wave[wave] = __popcll(ballot);
    __syncthreads();
    int wave_base = 0;
    for (int w = 0; w < wave; ++w) wave_base += s_wave[w];
    const int chunk_total = s_wave[0] + s_wave[1] + s_wave[2] + s_wave[3];
    if (flag) {
      const int slot = base + running + wave_base + before;
      if (slot < sorted_capacity) sorted_token_ids[slot] = i;
    }
    running += chunk_total;
  }
}

// ---------------------------------------------------------------------------------
// Token-tile lists of the matrix-core grouped GEMM, written by the dispatch kernels below that hold every expert's
// count and first slot in one workgroup (otherwise by k_build_tiles in mfma.hip, which documents the layout): one
// entry {expert, first slot, live rows, 0} per `bm`-slot piece of each active expert's run, [0] = the entry count.
// With bm_b > 0 a second list of that tile height goes to list_b.  bm = 0: no lists asked for.
// ---------------------------------------------------------------------------------
struct TileListArgs {
  int capacity;  // entries a list holds
  int bm, bm_b;
  int* list;
  int* list_b;
};
// entries of expert e (count selections from slot `base`), the first of them entry `first` of the list
__device__ __forceinline__ void write_tile_entries(int e, int count, int base, int first, int h, int capacity, int* list) {
  const int nt = (count + h - 1) / h;
  for (int i = 0; i < nt; ++i) {
    const int idx = first + i;
    if (idx >= capacity) break;
    list[4 + 4 * idx + 0] = e;
    list[4 + 4 * idx + 1] = base + i * h;
    list[4 + 4 * idx + 2] = min(h, count - i * h);
    list[4 + 4 * idx + 3] = 0;
  }
}

// ---------------------------------------------------------------------------------
// The same tables from ONE launch of one workgroup, for passes of at most 8192 selections (1024 tokens of top-8):
// the two launches above cost ~15 us at 512 tokens, nearly all of it launch and barrier latency (every expert's
// workgroup walks all selections, two barriers per 256 of them).  Sixteen wavefronts split the selections into
// sixteen consecutive ranges.  Each counts its range per expert (LDS atomics: only the totals are used), thread e
// turns the sixteen counts of expert e into first slots (prefix over the ranges, plus the expert's base from a scan of
// the padded totals), and each wavefront then ranks its selections among equals in index order, 64 at a time with
// one ballot per bit of the id, and writes them.  No result depends on the order in which atomics land.
// ---------------------------------------------------------------------------------
constexpr int kAlignFusedMaxSelections = 8192;
constexpr int kAlignFusedWaves = 16;
__global__ void __launch_bounds__(1024) k_align_fused(const int* __restrict__ topk_ids, const int* __restrict__ valid_tokens,
                                                       int top_k, int num_experts, int block_size, int sorted_capacity,
                                                       int expert_capacity, int* __restrict__ sorted_token_ids,
                                                       int* __restrict__ expert_ids, int* __restrict__ bucket_live,
                                                       int* __restrict__ expert_counts, int* __restrict__ num_tokens_post_pad,
                                                       TileListArgs tl) {
  constexpr int kMaxE = 512, kRounds = kAlignFusedMaxSelections / (kAlignFusedWaves * 64);
  __shared__ int cnt[kAlignFusedWaves][kMaxE];  // per range and expert: count, then next slot
  __shared__ int s_scan[2][3][kMaxE];           // scanned together: padded counts, tiles of either list
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int numel = min(*valid_tokens * top_k, kAlignFusedMaxSelections);
  // whole-capacity fill first: the barriers below order it before the entries written over it
  for (int i = tid; i < sorted_capacity; i += 1024) sorted_token_ids[i] = numel;
  for (int i = tid; i < expert_capacity; i += 1024) {
    expert_ids[i] = -1;
    bucket_live[i] = 0;
  }
  for (int i = tid; i < kAlignFusedWaves * kMaxE; i += 1024) (&cnt[0][0])[i] = 0;
  __syncthreads();
  const int per_range = ((numel + kAlignFusedWaves - 1) / kAlignFusedWaves + 63) / 64 * 64;
  const int r0 = wave * per_range, r1 = min(r0 + per_range, numel);
  int id[kRounds];
#pragma unroll
  for (int r = 0; r < kRounds; ++r) {
    const int i = r0 + r * 64 + lane;
    id[r] = i < r1 ? topk_ids[i] : -1;
    if (id[r] >= num_experts) id[r] = -1;  // (an id no expert has matches nothing, as in the two-launch form)
    if (id[r] >= 0) atomicAdd(&cnt[wave][id[r]], 1);
  }
  __syncthreads();
  int count = 0, padded = 0, tiles_a = 0, tiles_b = 0;
  if (tid < kMaxE) {
    if (tid < num_experts) {
#pragma unroll
      for (int w = 0; w < kAlignFusedWaves; ++w) {
        const int h = cnt[w][tid];
        cnt[w][tid] = count;  // selections of this expert in earlier ranges
        count += h;
      }
      padded = (count + block_size - 1) / block_size * block_size;
    }
    tiles_a = tl.bm > 0 ? (count + tl.bm - 1) / tl.bm : 0;
    tiles_b = tl.bm_b > 0 ? (count + tl.bm_b - 1) / tl.bm_b : 0;
    s_scan[0][0][tid] = padded;
    s_scan[0][1][tid] = tiles_a;
    s_scan[0][2][tid] = tiles_b;
  }
  __syncthreads();
  int cur = 0;
  for (int d = 1; d < kMaxE; d <<= 1) {
    if (tid < kMaxE) {
#pragma unroll
      for (int a = 0; a < 3; ++a) s_scan[cur ^ 1][a][tid] = s_scan[cur][a][tid] + (tid >= d ? s_scan[cur][a][tid - d] : 0);
    }
    cur ^= 1;
    __syncthreads();
  }
  if (tid < kMaxE) {
    const int base = s_scan[cur][0][tid] - padded;
    if (tid == kMaxE - 1) {
      *num_tokens_post_pad = s_scan[cur][0][tid];
      if (tl.bm > 0) tl.list[0] = min(s_scan[cur][1][tid], tl.capacity);
      if (tl.bm_b > 0) tl.list_b[0] = min(s_scan[cur][2][tid], tl.capacity);
    }
    if (tid < num_experts) {
      if (tl.bm > 0) write_tile_entries(tid, count, base, s_scan[cur][1][tid] - tiles_a, tl.bm, tl.capacity, tl.list);
      if (tl.bm_b > 0) write_tile_entries(tid, count, base, s_scan[cur][2][tid] - tiles_b, tl.bm_b, tl.capacity, tl.list_b);
      expert_counts[tid] = count;
#pragma unroll
      for (int w = 0; w < kAlignFusedWaves; ++w) cnt[w][tid] += base;
      const int nblk = (count + block_size - 1) / block_size;
      for (int b = 0; b < nblk; ++b) {
        const int blk = base / block_size + b;
        if (blk < expert_capacity) {
          expert_ids[blk] = tid;
          bucket_live[blk] = min(block_size, count - b * block_size);
        }
      }
    }
  }
  __syncthreads();
  int* mine = cnt[wave];
  int id_bits = 1;
  while ((1 << id_bits) < num_experts) ++id_bits;
#pragma unroll
  for (int r = 0; r < kRounds; ++r) {
    const int i = r0 + r * 64 + lane;
    const int v = id[r];
    unsigned long long same = __ballot(v >= 0);
    for (int bit = 0; bit < id_bits; ++bit) {
      const unsigned long long set = __ballot((v >> bit) & 1);
      same &= ((v >> bit) & 1) ? set : ~set;
    }
    int pos = -1;
    if (v >= 0) pos = mine[v] + __popcll(same & ((1ull << lane) - 1ull));
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();  // every lane has read its expert's slot
    if (v >= 0 && lane == __builtin_ctzll(same)) mine[v] += __popcll(same);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    if (pos >= 0 && pos < sorted_capacity) sorted_token_ids[pos] = i;
  }
}

// ---------------------------------------------------------------------------------
// The same dispatch tables for prefill widths, as a stable counting sort in three launches whose work is
// proportional to the number of selections (the two-launch form above has every expert's workgroup scan all
// of them).  A chunk is 1024 consecutive flat ids, 256 per wavefront.
//   hist:    per-chunk, per-expert counts; whole-capacity sentinel / -1 / 0 fill.
//   offsets: one workgroup: per-expert totals, the exclusive prefix of the padded totals, every chunk's
//            first slot per expert, the block tables.
//   place:   per chunk: each wavefront ranks its ids among equals in index order and writes them.
// No result depends on the order in which atomics land, so the tables are the CPU reference's.
// ---------------------------------------------------------------------------------
constexpr int kAlignChunk = 1024;
constexpr int kAlignMaxExperts = 512;

__global__ void __launch_bounds__(256) k_align_hist(const int* __restrict__ topk_ids, const int* __restrict__ valid_tokens,
                                                     int top_k, int num_experts, int sorted_capacity, int expert_capacity,
                                                     int* __restrict__ chunk_hist, int* __restrict__ sorted_token_ids,
                                                     int* __restrict__ expert_ids, int* __restrict__ bucket_live) {
  __shared__ int hist[kAlignMaxExperts];
  const int numel = *valid_tokens * top_k;
  for (int e = threadIdx.x; e < num_experts; e += 256) hist[e] = 0;
  __syncthreads();
  const int i0 = blockIdx.x * kAlignChunk;
  for (int j = threadIdx.x; j < kAlignChunk; j += 256) {
    const int i = i0 + j;
    if (i < numel) atomicAdd(&hist[topk_ids[i]], 1);
  }
  __syncthreads();
  for (int e = threadIdx.x; e < num_experts; e += 256) chunk_hist[(size_t)blockIdx.x * num_experts + e] = hist[e];
  const int nb = gridDim.x;
  for (int i = blockIdx.x * 256 + threadIdx.x; i < sorted_capacity; i += nb * 256) sorted_token_ids[i] = numel;
  for (int i = blockIdx.x * 256 + threadIdx.x; i < expert_capacity; i += nb * 256) {
    expert_ids[i] = -1;
    bucket_live[i] = 0;
  }
}

// One workgroup of 512 threads, thread e = expert e.  chunk_hist[c][e] becomes the first slot of chunk c's
// selections of expert e.  A thread's column of the histogram is fetched in one batch of independent loads and kept
// in registers for the second pass (64 chunks, 65 536 selections; beyond that the tail is walked load by load),
// and the experts' padded counts are scanned across the workgroup: walked one after the other, the 64 dependent
// loads per pass and the 256-step scan by one thread were 25 us of latency at 8192 tokens.
constexpr int kAlignCachedChunks = 64;
__global__ void __launch_bounds__(512) k_align_offsets(const int* __restrict__ valid_tokens, int top_k, int num_experts,
                                                        int block_size, int n_chunks_max, int expert_capacity,
                                                        int* __restrict__ chunk_hist, int* __restrict__ expert_counts,
                                                        int* __restrict__ expert_ids, int* __restrict__ bucket_live,
                                                        int* __restrict__ num_tokens_post_pad, TileListArgs tl) {
  static_assert(kAlignMaxExperts == 512, "one thread per expert slot of the scan");
  __shared__ int s_scan[2][3][kAlignMaxExperts];  // scanned together: padded counts, tiles of either list
  const int e = threadIdx.x;
  const int numel = *valid_tokens * top_k;
  const int n_chunks = min(n_chunks_max, (numel + kAlignChunk - 1) / kAlignChunk);
  const bool live = e < num_experts;
  int h[kAlignCachedChunks];
#pragma unroll
  for (int c = 0; c < kAlignCachedChunks; ++c) h[c] = live && c < n_chunks ? chunk_hist[(size_t)c * num_experts + e] : 0;
  int count = 0;
#pragma unroll
  for (int c = 0; c < kAlignCachedChunks; ++c) count += h[c];
  if (live)
    for (int c = kAlignCachedChunks; c < n_chunks; ++c) count += chunk_hist[(size_t)c * num_experts + e];
  const int padded = live ? (count + block_size - 1) / block_size * block_size : 0;
  const int tiles_a = tl.bm > 0 ? (count + tl.bm - 1) / tl.bm : 0;
  const int tiles_b = tl.bm_b > 0 ? (count + tl.bm_b - 1) / tl.bm_b : 0;
  // inclusive scan of the padded counts and the tile counts (nine doubling steps), then exclusive
  s_scan[0][0][e] = padded;
  s_scan[0][1][e] = tiles_a;
  s_scan[0][2][e] = tiles_b;
  __syncthreads();
  int cur = 0;
  for (int d = 1; d < kAlignMaxExperts; d <<= 1) {
#pragma unroll
    for (int a = 0; a < 3; ++a) s_scan[cur ^ 1][a][e] = s_scan[cur][a][e] + (e >= d ? s_scan[cur][a][e - d] : 0);
    cur ^= 1;
    __syncthreads();
  }
  const int base = s_scan[cur][0][e] - padded;
  if (e == kAlignMaxExperts - 1) {
    *num_tokens_post_pad = s_scan[cur][0][e];
    if (tl.bm > 0) tl.list[0] = min(s_scan[cur][1][e], tl.capacity);
    if (tl.bm_b > 0) tl.list_b[0] = min(s_scan[cur][2][e], tl.capacity);
  }
  if (!live) return;
  if (tl.bm > 0) write_tile_entries(e, count, base, s_scan[cur][1][e] - tiles_a, tl.bm, tl.capacity, tl.list);
  if (tl.bm_b > 0) write_tile_entries(e, count, base, s_scan[cur][2][e] - tiles_b, tl.bm_b, tl.capacity, tl.list_b);
  expert_counts[e] = count;
  int run = base;
#pragma unroll
  for (int c = 0; c < kAlignCachedChunks; ++c) {
    if (c < n_chunks) chunk_hist[(size_t)c * num_experts + e] = run;
    run += h[c];
  }
  for (int c = kAlignCachedChunks; c < n_chunks; ++c) {
    const size_t i = (size_t)c * num_experts + e;
    const int v = chunk_hist[i];
    chunk_hist[i] = run;
    run += v;
  }
  const int nblk = (count + block_size - 1) / block_size;
  for (int b = 0; b < nblk; ++b) {
    const int blk = base / block_size + b;
    if (blk < expert_capacity) {
      expert_ids[blk] = e;
      bucket_live[blk] = min(block_size, count - b * block_size);
    }
  }
}

__global__ void __launch_bounds__(256) k_align_place(const int* __restrict__ topk_ids, const int* __restrict__ valid_tokens,
                                                      int top_k, int num_experts, int sorted_capacity,
                                                      const int* __restrict__ chunk_first, int* __restrict__ sorted_token_ids) {
  __shared__ int cnt[4][kAlignMaxExperts];  // next slot of expert e for wavefront w
  const int numel = *valid_tokens * top_k;
  const int i0 = blockIdx.x * kAlignChunk;
  if (i0 >= numel) return;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  // pass 1: per-wavefront counts
  for (int e = threadIdx.x; e < 4 * kAlignMaxExperts; e += 256) (&cnt[0][0])[e] = 0;
  __syncthreads();
  int id[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int i = i0 + wave * 256 + r * 64 + lane;
    id[r] = i < numel ? topk_ids[i] : -1;
    if (id[r] >= 0) atomicAdd(&cnt[wave][id[r]], 1);
  }
  __syncthreads();
  // counts -> first slots: this chunk's first slot of the expert, plus the earlier wavefronts' counts
  for (int e = threadIdx.x; e < num_experts; e += 256) {
    int run = chunk_first[(size_t)blockIdx.x * num_experts + e];
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const int h = cnt[w][e];
      cnt[w][e] = run;
      run += h;
    }
  }
  __syncthreads();
  // pass 2: rank among equals in index order.  The lanes that hold the same expert as this one are found for all
  // lanes at once, one ballot per bit of the id (walking the distinct experts of the 64 ids one by one took ~57
  // rounds of ballots and LDS updates per 64 ids: 23 us at 8192 tokens); the lowest lane of each group then moves the
  // expert's next slot on.
  int* mine = cnt[wave];
  int id_bits = 1;
  while ((1 << id_bits) < num_experts) ++id_bits;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int i = i0 + wave * 256 + r * 64 + lane;
    const int v = id[r];
    unsigned long long same = __ballot(v >= 0);
    for (int bit = 0; bit < id_bits; ++bit) {
      const unsigned long long set = __ballot((v >> bit) & 1);
      same &= ((v >> bit) & 1) ? set : ~set;
    }
    int pos = -1;
    if (v >= 0) {
      const int first = mine[v];
      pos = first + __popcll(same & ((1ull << lane) - 1ull));
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();  // every lane has read its expert's slot
    if (v >= 0 && lane == __builtin_ctzll(same)) mine[v] += __popcll(same);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    if (pos >= 0 && pos < sorted_capacity) sorted_token_ids[pos] = i;
  }
}

// ---------------------------------------------------------------------------------
// moe_reduce (crates/xabe-cuda/src/kernels/moe.rs:4049-4065): out[t] = sum_k partial[t*K+k], ascending k.
// grid (max_tokens, ceil(hidden/256)).
// ---------------------------------------------------------------------------------
__global__ void __launch_bounds__(256) k_moe_reduce(const float* __restrict__ partial, const int* __restrict__ valid_tokens,
                                                     int top_k, int hidden, float* __restrict__ out) {
  const int t = blockIdx.x;
  if (t >= *valid_tokens) return;
  const int j = blockIdx.y * 256 + threadIdx.x;
  if (j >= hidden) return;
  const float* p = partial + (size_t)t * top_k * hidden + j;
  float r = 0.0f;
  for (int k = 0; k < top_k; ++k) r += p[(size_t)k * hidden];
  out[(size_t)t * hidden + j] = r;
}

// ---------------------------------------------------------------------------------
// moe_block_gate_and_combine (crates/xabe-engine/src/block/moe.rs:424-483):
//   g = 1/(1+expf(-(w . normed[t])));  r = sum_k partial (ascending k);
//   ffn_out = r + shexp*g;  l_out = ffn_out + residual.   grid (max_tokens, ceil(hidden/1024)).
// ---------------------------------------------------------------------------------
__global__ void __launch_bounds__(256) k_gate_and_combine(const float* __restrict__ w, const float* __restrict__ normed,
                                                           const float* __restrict__ partial, const float* __restrict__ shexp,
                                                           const float* __restrict__ residual, const int* __restrict__ valid_tokens,
                                                           int top_k, int hidden, float* __restrict__ gate,
                                                           float* __restrict__ routed, float* __restrict__ ffn_out,
                                                           float* __restrict__ l_out) {
  __shared__ float scratch[4];
  const int t = blockIdx.x;
  if (t >= *valid_tokens) return;
  const size_t base = (size_t)t * hidden;
  const float* xs = normed + base;
  float s = 0.0f;
  for (int j = threadIdx.x; j < hidden; j += 256) s = __builtin_fmaf(w[j], xs[j], s);
  s = block_sum_256(s, scratch);
  const float g = 1.0f / (1.0f + expf(-s));
  if (threadIdx.x == 0 && blockIdx.y == 0) gate[t] = g;
  // four consecutive columns per thread (hidden is a multiple of 128)
  const int j = (blockIdx.y * 256 + threadIdx.x) * 4;
  if (j >= hidden) return;
  const float* p = partial + (size_t)t * top_k * hidden + j;
  float4 r = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int k = 0; k < top_k; ++k) {
    const float4 v = *reinterpret_cast<const float4*>(p + (size_t)k * hidden);
    r.x += v.x; r.y += v.y; r.z += v.z; r.w += v.w;
  }
  const float4 sh = *reinterpret_cast<const float4*>(shexp + base + j);
  const float4 rs = *reinterpret_cast<const float4*>(residual + base + j);
  float4 v, lo;
  v.x = r.x + sh.x * g; v.y = r.y + sh.y * g; v.z = r.z + sh.z * g; v.w = r.w + sh.w * g;
  lo.x = v.x + rs.x; lo.y = v.y + rs.y; lo.z = v.z + rs.z; lo.w = v.w + rs.w;
  *reinterpret_cast<float4*>(routed + base + j) = r;
  *reinterpret_cast<float4*>(ffn_out + base + j) = v;
  *reinterpret_cast<float4*>(l_out + base + j) = lo;
}

// The same combine for rows of at most 2048 elements, one workgroup per token, with the post-mixer seam fusion the
// reference measured on its own card ("the next layer's RMSNorm in the MoE combine kernel's tail",
// docs/BENCHMARKS.md:1376, :1761): the workgroup holds the whole row of l_out, so it can apply the NEXT layer's
// RMSNorm to it before it leaves, and the next block starts from normalised rows (and, WITH_H, from their fp16 copy)
// without a launch of its own or a second pass over l_out.  Every value is the one the separate launches produce:
// gate, routed sum, ffn_out and l_out in k_gate_and_combine's operations and order; the RMS scale of the row in the
// canonical order (lane L of a wavefront folds elements 32L .. 32L+31, then the wavefront tree: the row changes
// hands through LDS for that, padded like k_rms_norm_short_rows'), the normalised elements as (x * inv) * w.
// `routed` and `ffn_out` may be null (read-back tensors a serving loop does not need: 16 bytes per element less
// to write); NORM = false leaves the tail out.
template <bool NORM, bool WITH_H>
__global__ void __launch_bounds__(256) k_combine_rows(const float* __restrict__ w, const float* normed,
                                                       const float* __restrict__ partial, const float* __restrict__ shexp,
                                                       const float* __restrict__ residual, const int* __restrict__ valid_tokens,
                                                       int top_k, int hidden, float* __restrict__ gate,
                                                       float* __restrict__ routed, float* __restrict__ ffn_out,
                                                       float* __restrict__ l_out, const float* __restrict__ next_w, float next_eps,
                                                       float* next_normed, _Float16* __restrict__ next_normed_h) {
  // (`next_normed` may be `normed` itself, a block that feeds the next pass through its own buffers: the row is read
  // in round one and written after the last barrier, by this workgroup only)
  constexpr int kSlots = 512 + 64;  // padded 16-byte slots of one 2048-element row
  __shared__ float scratch[4];
  __shared__ float4 s_row[NORM ? kSlots : 1];
  const int t = blockIdx.x;
  if (t >= *valid_tokens) return;
  const size_t base = (size_t)t * hidden;
  const int n4 = hidden / 4;
  // round one: everything the row needs, requested together (two 16-byte columns per thread)
  const float4* p4 = reinterpret_cast<const float4*>(partial + (size_t)t * top_k * hidden);
  float4 pv[2][8], sh[2], rs[2], nw[2];
  float wv[8], xv[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int j = min((int)threadIdx.x + 256 * i, hidden - 1);
    wv[i] = w[j];
    xv[i] = normed[base + j];
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int q = min((int)threadIdx.x + 256 * i, n4 - 1);
#pragma unroll
    for (int k = 0; k < 8; ++k) pv[i][k] = p4[(size_t)min(k, top_k - 1) * n4 + q];
    sh[i] = reinterpret_cast<const float4*>(shexp + base)[q];
    rs[i] = reinterpret_cast<const float4*>(residual + base)[q];
    if constexpr (NORM) nw[i] = reinterpret_cast<const float4*>(next_w)[q];
  }
  // selections past the eighth (top_k > 8) are added from memory in the loop below
  float s = 0.0f;
#pragma unroll
  for (int i = 0; i < 8; ++i)
    if ((int)threadIdx.x + 256 * i < hidden) s = __builtin_fmaf(wv[i], xv[i], s);
  s = block_sum_256(s, scratch);
  const float g = 1.0f / (1.0f + expf(-s));
  if (threadIdx.x == 0) gate[t] = g;
  float4 lo[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int q = (int)threadIdx.x + 256 * i;
    lo[i] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (q < n4) {
      float4 r = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
      for (int k = 0; k < 8; ++k)
        if (k < top_k) { r.x += pv[i][k].x; r.y += pv[i][k].y; r.z += pv[i][k].z; r.w += pv[i][k].w; }
      for (int k = 8; k < top_k; ++k) {
        const float4 v = p4[(size_t)k * n4 + q];
        r.x += v.x; r.y += v.y; r.z += v.z; r.w += v.w;
      }
      float4 v;
      v.x = r.x + sh[i].x * g; v.y = r.y + sh[i].y * g; v.z = r.z + sh[i].z * g; v.w = r.w + sh[i].w * g;
      lo[i].x = v.x + rs[i].x; lo[i].y = v.y + rs[i].y; lo[i].z = v.z + rs[i].z; lo[i].w = v.w + rs[i].w;
      if (routed) reinterpret_cast<float4*>(routed + base)[q] = r;
      if (ffn_out) reinterpret_cast<float4*>(ffn_out + base)[q] = v;
      reinterpret_cast<float4*>(l_out + base)[q] = lo[i];
    }
    if constexpr (NORM) s_row[q + (q >> 3)] = lo[i];  // (zeros past the end of a short row: fma(0, 0, s) == s)
  }
  if constexpr (NORM) {
    __syncthreads();
    const int lane = (int)__lane_id();
    RmsRaw r;
#pragma unroll
    for (int i = 0; i < 8; ++i) r.q[i] = s_row[8 * lane + i + lane];  // slot(8 * lane + i)
    const float inv = rms_finish(rms_fold(r, 0.0f), hidden, next_eps);  // every wavefront: the same scale
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int q = (int)threadIdx.x + 256 * i;
      if (q < n4) {
        const float4 v = make_float4(lo[i].x * inv * nw[i].x, lo[i].y * inv * nw[i].y, lo[i].z * inv * nw[i].z,
                                     lo[i].w * inv * nw[i].w);
        reinterpret_cast<float4*>(next_normed + base)[q] = v;
        if constexpr (WITH_H) {
          typedef _Float16 h2 __attribute__((ext_vector_type(2)));
          const h2 a = {(_Float16)v.x, (_Float16)v.y}, b = {(_Float16)v.z, (_Float16)v.w};
          reinterpret_cast<uint2*>(next_normed_h + base)[q] = make_uint2(__builtin_bit_cast(uint32_t, a), __builtin_bit_cast(uint32_t, b));
        }
      }
    }
  }
}

// dense_ffn_add_residual (crates/xabe-engine/src/block/dense_ffn.rs:1149-1175)
__global__ void __launch_bounds__(256) k_add_residual(const float* __restrict__ ffn_out, const float* __restrict__ residual,
                                                       const int* __restrict__ valid_tokens, int hidden,
                                                       float* __restrict__ l_out) {
  const int t = blockIdx.x;
  if (t >= *valid_tokens) return;
  const int j = blockIdx.y * 256 + threadIdx.x;
  if (j >= hidden) return;
  const size_t i = (size_t)t * hidden + j;
  l_out[i] = ffn_out[i] + residual[i];
}

__global__ void __launch_bounds__(256) k_add_logit_bias(const float* __restrict__ bias, const int* __restrict__ valid_tokens,
                                                         int num_experts, float* __restrict__ logits) {
  const int t = blockIdx.x;
  if (t >= *valid_tokens) return;
  for (int e = threadIdx.x; e < num_experts; e += 256) logits[(size_t)t * num_experts + e] += bias[e];
}

// ---------------------------------------------------------------------------------
// Stand-alone dequantisation, bit-identical to the CPU reference
// (crates/xabe-kernels/src/quant.rs:62-69, :171-202): (d*sc)*q and q*d, each product rounded.
// One thread per element.
// ---------------------------------------------------------------------------------
__global__ void __launch_bounds__(256) k_dequant_q6k(const uint8_t* __restrict__ bytes, size_t n_elems, float* __restrict__ out) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n_elems) return;
  const uint8_t* b = bytes + (i >> 8) * kQ6KBytes;
  const int n = (int)(i & 255);
  const int half = n >> 7, lane = (n & 127) >> 5, l = n & 31;
  const uint32_t qlb = b[half * 64 + (lane & 1) * 32 + l];
  const uint32_t low4 = lane >= 2 ? qlb >> 4 : qlb & 0xF;
  const uint32_t hi2 = (b[128 + half * 32 + l] >> (2 * lane)) & 3;
  const int q = (int)(low4 | (hi2 << 4)) - 32;
  const float sc = (float)(int8_t)b[192 + half * 8 + lane * 2 + (l >> 4)];
  const float d = f16_bits_to_f32((uint32_t)b[208] | ((uint32_t)b[209] << 8));
  const float dsc = d * sc;
  out[i] = dsc * (float)q;
}

__global__ void __launch_bounds__(256) k_dequant_q8_0(const uint8_t* __restrict__ bytes, size_t n_elems, float* __restrict__ out) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n_elems) return;
  const uint8_t* b = bytes + (i >> 5) * kQ8Bytes;
  const float d = f16_bits_to_f32((uint32_t)b[0] | ((uint32_t)b[1] << 8));
  out[i] = (float)(int8_t)b[2 + (i & 31)] * d;
}

// ---------------------------------------------------------------------------------
// Activation rows narrowed to int8 with one fp32 scale per 32 elements, the operand the reference's integer
// tensor-core path makes before its matmuls (crates/xabe-cuda/src/kernels/mma.rs:118-157): a = max |v| of the block,
// d = a / 127 (1.0 for a block of zeros), q = rintf(v * (127 / a)) clamped to +-127.  This library multiplies fp16
// operands instead and never calls it; it is here so that a caller that keeps the int8 form of its activations (or
// measures against it) finds the reference's values bit for bit.  Half a wavefront per block, one element per lane.
// ---------------------------------------------------------------------------------
__global__ void __launch_bounds__(256) k_quantize_rows_q8(const float* __restrict__ x, size_t n_blocks,
                                                           int8_t* __restrict__ q, float* __restrict__ scales) {
  const size_t block = (size_t)blockIdx.x * 8 + (threadIdx.x >> 5);
  if (block >= n_blocks) return;
  const int lane = threadIdx.x & 31;
  const float v = x[block * 32 + lane];
  float a = fabsf(v);
#pragma unroll
  for (int off = 16; off > 0; off >>= 1) a = fmaxf(a, __shfl_xor(a, off, 64));  // (stays inside the 32-lane half)
  const float d = a > 0.0f ? a / 127.0f : 1.0f;
  const float inv = a > 0.0f ? 127.0f / a : 0.0f;
  int qi = (int)rintf(v * inv);
  qi = qi < -127 ? -127 : (qi > 127 ? 127 : qi);
  q[block * 32 + lane] = (int8_t)qi;
  if (lane == 0) scales[block] = d;
}

// ---------------------------------------------------------------------------------
// Synthetic stacks: one thread per 256-element chunk.  Integer Irwin-Hall(12) normal
// approximation over a per-chunk xorshift64* stream, then the reference's amax
// quantizers (crates/xabe-kernels/src/quant.rs:75-88, :495-567).
// ---------------------------------------------------------------------------------
__device__ __forceinline__ uint64_t splitmix64(uint64_t z) {
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}
__device__ __forceinline__ uint64_t xorshift_next(uint64_t& s) {
  uint64_t x = s;
  x ^= x >> 12;
  x ^= x << 25;
  x ^= x >> 27;
  s = x;
  return x * 0x2545F4914F6CDD1Dull;
}
__device__ __forceinline__ uint64_t chunk_state(uint64_t seed, size_t chunk) {
  const uint64_t st = splitmix64(seed + (uint64_t)chunk * 0x9E3779B97F4A7C15ull);
  return st == 0 ? 0x9E3779B97F4A7C15ull : st;
}
__device__ __forceinline__ float synth_value(uint64_t& st, float sigma) {
  uint32_t s = 0;
#pragma unroll
  for (int k = 0; k < 3; ++k) {
    const uint64_t v = xorshift_next(st);
    s += (uint32_t)(v & 0xffff) + (uint32_t)((v >> 16) & 0xffff) + (uint32_t)((v >> 32) & 0xffff) + (uint32_t)(v >> 48);
  }
  const float z = (float)(2 * (int32_t)s - 12 * 65535) * (1.0f / 131072.0f);
  return sigma * z;
}
__device__ __forceinline__ uint16_t f32_to_f16_bits(float v) {
  return __builtin_bit_cast(uint16_t, (_Float16)v);
}
__device__ __forceinline__ float clampf(float v, float lo, float hi) { return v < lo ? lo : (v > hi ? hi : v); }

__global__ void __launch_bounds__(64) k_synth_f32(uint64_t seed, size_t n, float sigma, float* __restrict__ out) {
  const size_t c = (size_t)blockIdx.x * 64 + threadIdx.x;
  if (c * 256 >= n) return;
  uint64_t st = chunk_state(seed, c);
  const size_t m = min((size_t)256, n - c * 256);
  for (size_t i = 0; i < m; ++i) out[c * 256 + i] = synth_value(st, sigma);
}

__global__ void __launch_bounds__(64) k_synth_q6k(uint64_t seed, size_t chunks, float sigma, uint8_t* __restrict__ out) {
  const size_t c = (size_t)blockIdx.x * 64 + threadIdx.x;
  if (c >= chunks) return;
  // pass 1: group and global amax
  uint64_t st = chunk_state(seed, c);
  float gamax[16];
  float amax = 0.0f;
#pragma unroll
  for (int g = 0; g < 16; ++g) {
    float a = 0.0f;
    for (int k = 0; k < 16; ++k) a = fmaxf(a, fabsf(synth_value(st, sigma)));
    gamax[g] = a;
    amax = fmaxf(amax, a);
  }
  const float d = amax > 0.0f ? amax / (32.0f * 127.0f) : 0.0f;
  uint8_t* blk = out + c * kQ6KBytes;
  for (int i = 0; i < 192; ++i) blk[i] = 0;
  // pass 2: regenerate, quantize, pack (group g covers positions 16g..16g+15)
  st = chunk_state(seed, c);
#pragma unroll
  for (int g = 0; g < 16; ++g) {
    int sc = 0;
    if (d > 0.0f) sc = (int)clampf(roundf(gamax[g] / (d * 32.0f)), 0.0f, 127.0f);
    blk[192 + g] = (uint8_t)(int8_t)sc;
    const float denom = d * (float)sc;
    const int half = g >> 3, lane = (g >> 1) & 3, is = g & 1;
    for (int k = 0; k < 16; ++k) {
      const float v = synth_value(st, sigma);
      const int l = is * 16 + k;
      int code = 0;
      if (denom != 0.0f) code = (int)clampf(roundf(v / denom), -32.0f, 31.0f);
      const uint32_t raw = (uint32_t)(code + 32);
      blk[128 + half * 32 + l] |= (uint8_t)((raw >> 4) << (lane * 2));
      const int qi = half * 64 + (lane & 1) * 32 + l;
      blk[qi] |= (uint8_t)(lane >= 2 ? (raw & 0xF) << 4 : (raw & 0xF));
    }
  }
  const uint16_t dh = f32_to_f16_bits(d);
  blk[208] = (uint8_t)(dh & 0xff);
  blk[209] = (uint8_t)(dh >> 8);
}

__global__ void __launch_bounds__(64) k_synth_q8_0(uint64_t seed, size_t chunks, float sigma, uint8_t* __restrict__ out) {
  const size_t c = (size_t)blockIdx.x * 64 + threadIdx.x;
  if (c >= chunks) return;
  uint64_t st = chunk_state(seed, c);
  for (int b = 0; b < 8; ++b) {
    float v[32];
    float amax = 0.0f;
#pragma unroll
    for (int j = 0; j < 32; ++j) {
      v[j] = synth_value(st, sigma);
      amax = fmaxf(amax, fabsf(v[j]));
    }
    const float d = amax / 127.0f;
    const float inv_d = d != 0.0f ? 1.0f / d : 0.0f;
    uint8_t* blk = out + (c * 8 + b) * kQ8Bytes;
    const uint16_t dh = f32_to_f16_bits(d);
    blk[0] = (uint8_t)(dh & 0xff);
    blk[1] = (uint8_t)(dh >> 8);
#pragma unroll
    for (int j = 0; j < 32; ++j) {
      float q = roundf(v[j] * inv_d);
      q = clampf(q, -128.0f, 127.0f);
      blk[2 + j] = (uint8_t)(int8_t)(int)q;
    }
  }
}

}  // namespace xabe

// Routing of one token on one wavefront, shared by the stand-alone route kernel and the
// single-launch router + route kernel (so both give the same bits).
#pragma once

#include "device_common.h"


namespace xabe {

constexpr int kRouteMaxPerLane = 8;  // 64 lanes x 8 = 512 experts

// Routes one token on one wavefront, in two parts so that a caller can put other loads between them.
// route_load: the token's logits `lg` into registers, expert i*64+lane in l[i]; `bias` (may be null) is
// added first and the sums are written back to `lg_out`.  route_compute: `e_all` is num_experts floats of
// LDS private to this wavefront; lanes 0..top_k-1 return the k-th selection in (sel_i, sel_w).
// PER: experts held per lane, num_experts <= 64 * PER.
//
// The arithmetic is the reference's, operation for operation: e = (float)exp((double)(l - max)), the
// sum of e in index order, p = e / sum, the k largest p with the lower index winning a tie, weights
// p / (sum of the selected p in selection order).
template <int PER, bool COHERENT = false>
__device__ __forceinline__ void route_load(const float* lg, int num_experts, const float* __restrict__ bias,
                                           float* lg_out, float (&l)[PER]) {
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int idx = i * 64 + lane;
    l[i] = -INFINITY;
    if (idx < num_experts)
      l[i] = COHERENT ? __hip_atomic_load(lg + idx, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : lg[idx];
    if (bias && idx < num_experts) {
      l[i] += bias[idx];
      lg_out[idx] = l[i];
    }
  }
}

// One selection round over per-lane keys (kTaken = out of the running): the largest key, the lowest index
// among equals; the winner is marked taken.  Returns the winning key and index to every lane.
// Almost always exactly one (lane, slot) holds the maximum: then its index is read straight off the ballots and
// every holder (the one) is retired.  Several holders (equal keys) take the general path, which finds the lowest
// index among them and retires that one alone.
constexpr int kRouteTaken = (int)0x80000000;
template <int PER>
__device__ __forceinline__ void route_round(int (&key)[PER], int& best, int& bi) {
  const int lane = threadIdx.x & 63;
  int bp = key[0];
#pragma unroll
  for (int i = 1; i < PER; ++i) bp = max(bp, key[i]);
  best = wave_max_i(bp);
  unsigned long long holders[PER];
  int n_holders = 0;
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    holders[i] = __builtin_amdgcn_ballot_w64(key[i] == best);
    n_holders += __builtin_popcountll(holders[i]);
  }
  if (n_holders == 1) {  // (wave-uniform)
    bi = 0;
#pragma unroll
    for (int i = 0; i < PER; ++i)
      if (holders[i]) bi = i * 64 + __builtin_ctzll(holders[i]);
#pragma unroll
    for (int i = 0; i < PER; ++i) key[i] = key[i] == best ? kRouteTaken : key[i];
    return;
  }
  int li = 0x7fffffff;
#pragma unroll
  for (int i = PER - 1; i >= 0; --i)
    if (key[i] == best) li = i * 64 + lane;  // descending i: the lowest index of this lane wins
  bi = wave_min_i(li);
  if ((bi & 63) == lane) {
#pragma unroll
    for (int i = 0; i < PER; ++i)
      if (i == (bi >> 6)) key[i] = kRouteTaken;
  }
}

// First half of route_compute: the n experts with the largest LOGITS, in order (lower index first among
// equal logits); lane j < n returns the j-th in cand_i.  exp and the division by the common sum are
// monotone non-decreasing, so p orders the experts the same way except where distinct logits round to the
// same p: with n = top_k + 1 candidates, route_finish sees whether that happened anywhere it matters, and
// the candidates are then the selection itself -- known before a single exp has been evaluated.
// In two steps so that a caller who needs the j-th candidate only can act on it after j + 1 rounds:
// route_keys makes the keys, route_rounds runs rounds [j0, j1) and leaves the j-th winner in lane j's cand_i.
template <int PER>
__device__ __forceinline__ void route_keys(const float (&l)[PER], int num_experts, int (&key)[PER]) {
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int b = __builtin_bit_cast(int, l[i]);
    key[i] = i * 64 + lane < num_experts ? b ^ ((b >> 31) & 0x7fffffff) : kRouteTaken;  // int order == float order
  }
}
template <int PER>
__device__ __forceinline__ void route_rounds(int (&key)[PER], int j0, int j1, int& cand_i) {
  const int lane = threadIdx.x & 63;
  for (int j = j0; j < j1; ++j) {
    int best, bi;
    route_round<PER>(key, best, bi);
    if (lane == j) cand_i = bi;
  }
}
template <int PER>
__device__ __forceinline__ void route_order(const float (&l)[PER], int num_experts, int n, int& cand_i) {
  int key[PER];
  route_keys<PER>(l, num_experts, key);
  cand_i = 0;
  route_rounds<PER>(key, 0, n, cand_i);
}

// Second half: softmax, then the selection.  If the top_k + 1 candidates' probabilities are strictly
// decreasing (lane j against lane j + 1, j < top_k) the candidates are the reference's selection; otherwise
// some probabilities tie and the selection is redone on the probabilities themselves, the reference's way.
// `exact` (wave-uniform) tells the caller whether cand_i stood.
template <int PER>
__device__ __forceinline__ void route_finish(const float (&l)[PER], int num_experts, int top_k, int n, int cand_i,
                                             float* e_all, int& sel_i, float& sel_w, bool& exact) {
  const int lane = threadIdx.x & 63;
  float m = l[0];
#pragma unroll
  for (int i = 1; i < PER; ++i) m = fmaxf(m, l[i]);
  m = wave_max(m);
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int idx = i * 64 + lane;
    if (idx < num_experts) e_all[idx] = (float)exp((double)(l[i] - m));
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  // sequential sum in index order on lane 0 alone (a 16-byte LDS read that all 64 lanes aim at one
  // address is serialised lane by lane), 32 values per batch so that the reads are in flight together and
  // only the additions form the dependent chain
  float sum = -0.0f;
  if (lane == 0) {
    const int n32 = num_experts & ~31;
    for (int i = 0; i < n32; i += 32) {
      float4 v[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = *reinterpret_cast<const float4*>(e_all + i + 4 * j);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        sum += v[j].x;
        sum += v[j].y;
        sum += v[j].z;
        sum += v[j].w;
      }
    }
    for (int i = n32; i < num_experts; ++i) sum += e_all[i];
  }
  sum = lane_bcast(sum, 0);
  // p >= +0, so the bit patterns order like the values and comparisons run on integers
  const int pj = lane < n ? __builtin_bit_cast(int, e_all[cand_i] / sum) : 0;
  const int pn = __builtin_amdgcn_ds_bpermute(((lane + 1) & 63) * 4, pj);
  const bool strict = lane >= top_k || lane + 1 >= n || pj > pn;
  exact = __builtin_amdgcn_ballot_w64(strict) == ~0ull;
  int sel_bits = pj;
  sel_i = cand_i;
  if (!exact) {
    int p[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int idx = i * 64 + lane;
      p[i] = idx < num_experts ? __builtin_bit_cast(int, e_all[idx] / sum) : kRouteTaken;
    }
    sel_bits = 0;
    sel_i = 0;
    for (int k = 0; k < top_k; ++k) {
      int best, bi;
      route_round<PER>(p, best, bi);
      if (lane == k) { sel_bits = best; sel_i = bi; }
    }
  }
  const float sel_p = __builtin_bit_cast(float, sel_bits);
  // sum of the selected probabilities in selection order
  float ssum = -0.0f;
  for (int k = 0; k < top_k; ++k) ssum += lane_bcast(sel_p, k);
  sel_w = ssum > 0.0f ? sel_p / ssum : 1.0f / (float)top_k;
}

template <int PER>
__device__ __forceinline__ void route_compute(const float (&l)[PER], int num_experts, int top_k, float* e_all,
                                              int& sel_i, float& sel_w) {
  const int n = min(top_k + 1, num_experts);
  int cand_i;
  bool exact;
  route_order<PER>(l, num_experts, n, cand_i);
  route_finish<PER>(l, num_experts, top_k, n, cand_i, e_all, sel_i, sel_w, exact);
}

template <bool COHERENT = false>
__device__ __forceinline__ void route_one_token(const float* lg, int num_experts, int top_k, float* e_all,
                                                int& sel_i, float& sel_w, const float* __restrict__ bias = nullptr,
                                                float* lg_out = nullptr) {
  if (num_experts <= 256) {
    float l[4];
    route_load<4, COHERENT>(lg, num_experts, bias, lg_out, l);
    route_compute<4>(l, num_experts, top_k, e_all, sel_i, sel_w);
  } else {
    float l[kRouteMaxPerLane];
    route_load<kRouteMaxPerLane, COHERENT>(lg, num_experts, bias, lg_out, l);
    route_compute<kRouteMaxPerLane>(l, num_experts, top_k, e_all, sel_i, sel_w);
  }
}

}  // namespace xabe

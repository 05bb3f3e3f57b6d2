// Matrix-core regime for prefill widths: a grouped GEMM over expert-sorted tokens that
// dequantises Q6_K / Q8_0 weight tiles into LDS as fp16 and feeds v_mfma_f32_32x32x16_f16.
// Takes the place of the reference's int8 tensor-core family
// (crates/xabe-cuda/src/kernels/moe.rs:1316-1819, :2901-2943, :3152-3373) and of its
// int8 shared-expert path (moe.rs:6389-6476); one prologue per format feeds the same
// MFMA body for gate, up and down, so there is no per-format asymmetry.
//
// Work decomposition.  A workgroup (4 wavefronts, 2x2) owns a 128-token x 128-weight-row
// tile and walks the contraction in steps of 128.  For gate/up the 128 weight rows are 64
// gate rows and the matching 64 up rows, so SwiGLU happens in registers.  Token tiles come
// from a device-built list with one entry per 128-slot chunk of every *active* expert's
// run of the dispatch table: experts with no tokens cost nothing, whatever the skew.
// Workgroups are persistent and stride over (token tile, row tile) items.  (Token tiles are 64 rows while an
// expert's share of a pass is small, and 384 rows on eight wavefronts for the routed gate/up launch of wide passes:
// see k_mfma_expert's TBM.)
//
// Numerics.  Operands are fp16: activations rounded once; weights are (code - offset) exactly,
// times fp16(d * sc * 256) -- the 2^8 keeps small scales out of the fp16 subnormal range and
// is divided out in the epilogue.  Accumulation is fp32 in the MFMA.  Each output element
// depends only on its own token row and weight row in a fixed contraction order, so a token's
// row is the same bits wherever it sits in a batch of this regime.
#include <string.h>

#include <algorithm>
#include <type_traits>

#include "device_common.h"
#include "host_common.h"

namespace xabe {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kBM = 128;          // token rows per tile (64 in the narrow form: see k_mfma_expert's TBM)
constexpr int kBR = 128;          // weight rows per tile
constexpr int kBK = 128;          // contraction elements per step
// The weight tile's rows are unpadded too, its 16-byte chunks XOR-swizzled by w_swizzle(row): any eight
// consecutive rows spread one chunk over the eight 16-byte slots of a 128-byte bank line (the fragment reads:
// lanes = rows), and two neighbouring rows put chunks 4j .. 4j + 3 into disjoint halves of it (the
// dequantised stores: eight lanes = two rows x four units).  With padded rows (272 B) the reads were
// conflict-free and the stores two-way conflicted: a fifth of the LDS cycles the counters showed; the bank
// conflict counter now reads zero (the launches take the same time: LDS was not what held them).
constexpr int kLd = kBK;
// The activation tile goes from global memory straight into LDS (global_load_lds_dwordx4: no registers, no
// store instructions), which writes a wavefront's 64 pieces contiguously, so its rows are unpadded (256 B)
// and the 16-byte chunks of a row are stored XOR-swizzled by the row number instead: chunk c of row r sits at
// position c ^ (r & 15), and 16 consecutive rows reading the same chunk hit 16 different bank groups.
constexpr int kLdA = kBK;
constexpr float kWScale = 256.0f;
constexpr float kWScaleInv = 1.0f / 256.0f;

struct MfmaArgs {
  const uint8_t* w0;            // gate (NM=2) or down (NM=1) stack
  const uint8_t* w1;            // up stack (NM=2)
  size_t expert_bytes;          // bytes of one expert in a stack
  const _Float16* a;            // activations, row-major [*][K]
  void* out;                    // NM=2: fp16 [*][n_rows]; NM=1: fp32 [*][n_rows]
  const int* valid_tokens;
  const int* sorted_token_ids;
  const float* topk_weights;
  const int* tile_list;         // [0] = tile count; entry i at 4+4i: expert, first slot, live rows
  int K;                        // contraction length
  int n_rows;                   // output columns per token (rows of one weight matrix)
  int top_k;
};

// SwiGLU's gate in the matrix-core regime: x / (1 + e^-x) from the hardware's exp2 and reciprocal (a few ulp of
// fp32; the product is rounded to fp16 right after, 2^-11).  The fp32 regimes keep silu_f, whose bits they pin.
__device__ __forceinline__ float silu_fast(float x) {
  return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.44269504088896340736f * x));
}

__device__ __forceinline__ int w_swizzle(int row) {
  return (row & 8) | ((row & 1) << 2) | ((row >> 1) & 3);
}

// ---- prologues: one 32-element unit of one weight row -> 32 halfs in LDS -----------------
__device__ __forceinline__ u32x4 pack8(uint32_t c0, uint32_t c1, half2v off, half2v s) {
  // c0, c1: eight byte codes; returns eight halfs (code + 1024 - off) * s
  uint32_t p[4];
  p[0] = __builtin_amdgcn_perm(0x64646464u, c0, 0x04010400u);
  p[1] = __builtin_amdgcn_perm(0x64646464u, c0, 0x04030402u);
  p[2] = __builtin_amdgcn_perm(0x64646464u, c1, 0x04010400u);
  p[3] = __builtin_amdgcn_perm(0x64646464u, c1, 0x04030402u);
  uint32_t o[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    half2v v = __builtin_bit_cast(half2v, p[i]);
    v = (v + off) * s;
    o[i] = __builtin_bit_cast(uint32_t, v);
  }
  u32x4 r = {o[0], o[1], o[2], o[3]};
  return r;
}

// Q6_K unit (half h of a superblock, l8): codes at j*32 + l8*8 + i of that half.
__device__ __forceinline__ void q6_unit_to_lds(const Q6Raw& r, int l8, _Float16* brow, int swz) {
  const int is8 = (l8 >> 1) * 8;
  const uint32_t slo = r.sc0 >> is8, shi = r.sc1 >> is8;
  const float d = f16_bits_to_f32(r.dh) * kWScale;
  const float ds[4] = {d * (float)(int8_t)(slo & 0xff), d * (float)(int8_t)((slo >> 16) & 0xff),
                       d * (float)(int8_t)(shi & 0xff), d * (float)(int8_t)((shi >> 16) & 0xff)};
  uint32_t c[2][4];
#pragma unroll
  for (int w = 0; w < 2; ++w) {
    const uint32_t a = w ? r.qa1 : r.qa0, b = w ? r.qb1 : r.qb0, h = w ? r.qh1 : r.qh0;
    c[w][0] = (a & 0x0F0F0F0Fu) | ((h << 4) & 0x30303030u);
    c[w][1] = (b & 0x0F0F0F0Fu) | ((h << 2) & 0x30303030u);
    c[w][2] = ((a >> 4) & 0x0F0F0F0Fu) | (h & 0x30303030u);
    c[w][3] = ((b >> 4) & 0x0F0F0F0Fu) | ((h >> 2) & 0x30303030u);
  }
  const half2v off = {(_Float16)-1056.0f, (_Float16)-1056.0f};  // 1024 (perm bias) + 32 (code centre)
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const _Float16 sh = (_Float16)ds[j];
    const half2v s = {sh, sh};
    *reinterpret_cast<u32x4*>(brow + ((j * 4 + l8) ^ swz) * 8) = pack8(c[0][j], c[1][j], off, s);
  }
}

// Q8_0 unit: one 34-byte block -> the row's chunks 4 du .. 4 du + 3.
__device__ __forceinline__ void q8_unit_to_lds(const Q8Raw& r, int du, _Float16* brow, int swz) {
  const _Float16 sh = (_Float16)(f16_bits_to_f32(r.dh) * kWScale);  // exact: d is fp16, scaled by 2^8
  const half2v s = {sh, sh};
  const half2v off = {(_Float16)-1152.0f, (_Float16)-1152.0f};      // 1024 (perm bias) + 128 (sign flip)
#pragma unroll
  for (int w = 0; w < 4; ++w)
    *reinterpret_cast<u32x4*>(brow + ((du * 4 + w) ^ swz) * 8) = pack8(r.q[2 * w] ^ 0x80808080u, r.q[2 * w + 1] ^ 0x80808080u, off, s);
}

// Nothing moves across this point, in either direction, when the compiler schedules.
__device__ __forceinline__ void order_fence() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);
}

// Raw blocks in flight, in the registers the loads deliver them to.  Blocks sit at two-byte alignment (210- and
// 34-byte blocks) and the fields are read where they lie: vector memory loads on this hardware take any
// alignment, which is what the compiler itself relies on for a memcpy from a byte pointer.
// (d stays the sixteen bits the load delivers until the step that consumes it widens them: widened here, the
// compiler carries the narrow value across the item boundary and widens it right after an item's last step,
// waiting there for the loads meant to be in flight under the epilogue)
struct Q6Pend {
  uint2 qa, qb, qh, sc;
  uint16_t dh;
};
struct Q8Pend {
  u32x4 lo, hi;
  uint16_t dh;
};
template <typename T>
__device__ __forceinline__ T load_any(const uint8_t* p) {
  T v;
  __builtin_memcpy(&v, p, sizeof(T));
  return v;
}
// unit l8 of half `half` of the superblock at `blk` (field offsets: crates/xabe-kernels/src/quant.rs:725-729)
__device__ __forceinline__ void q6_issue(const uint8_t* blk, int half, int l8, Q6Pend& r) {
  r.qa = load_any<uint2>(blk + half * 64 + l8 * 8);
  r.qb = load_any<uint2>(blk + half * 64 + 32 + l8 * 8);
  r.qh = load_any<uint2>(blk + 128 + half * 32 + l8 * 8);
  r.sc = load_any<uint2>(blk + 192 + half * 8);
  r.dh = load_any<uint16_t>(blk + 208);
}
__device__ __forceinline__ void q6_finish(const Q6Pend& p, Q6Raw& r) {
  r.qa0 = p.qa.x, r.qa1 = p.qa.y;
  r.qb0 = p.qb.x, r.qb1 = p.qb.y;
  r.qh0 = p.qh.x, r.qh1 = p.qh.y;
  r.sc0 = p.sc.x, r.sc1 = p.sc.y;
  r.dh = p.dh;
}
__device__ __forceinline__ void q8_issue(const uint8_t* blk, Q8Pend& r) {
  r.dh = load_any<uint16_t>(blk);
  r.lo = load_any<u32x4>(blk + 2);
  r.hi = load_any<u32x4>(blk + 18);
}
__device__ __forceinline__ void q8_finish(const Q8Pend& p, Q8Raw& r) {
#pragma unroll
  for (int i = 0; i < 4; ++i) r.q[i] = p.lo[i], r.q[4 + i] = p.hi[i];
  r.dh = p.dh;
}

template <int QUANT, int UNITS>
struct WRaw {
  typename std::conditional<QUANT == kQ6K, Q6Pend, Q8Pend>::type u[UNITS];
};

// Global loads of one contraction step into registers: the raw blocks of this thread's weight-row units.
template <int QUANT, int UNITS>
__device__ __forceinline__ void load_unit_w(int ks, int i, const uint8_t* const (&wrow)[UNITS], int du, WRaw<QUANT, UNITS>& wreg) {
  {
    if constexpr (QUANT == kQ6K) {
      // step ks covers half (ks & 1) of superblock ks >> 1
      q6_issue(wrow[i] + (size_t)(ks >> 1) * kQ6KBytes, ks & 1, du, wreg.u[i]);
    } else {
      q8_issue(wrow[i] + (size_t)(ks * 4 + du) * kQ8Bytes, wreg.u[i]);
    }
  }
}
template <int QUANT, int UNITS>
__device__ __forceinline__ void load_step_w(int ks, const uint8_t* const (&wrow)[UNITS], int du, WRaw<QUANT, UNITS>& wreg) {
#pragma unroll
  for (int i = 0; i < UNITS; ++i) load_unit_w<QUANT, UNITS>(ks, i, wrow, du, wreg);
}


// TBM: token rows per tile, 384, 128 or 64.  The narrow form serves geometries whose experts see at most ~64 tokens
// each (up to ~2000 tokens per pass): half the matrix instructions, activation bytes and output stores per
// item, the same weight work.  A wavefront then owns 32 x 64 of the tile instead of 64 x 64; every output
// element sees the same operands in the same order, so the forms give the same bits.
// The tall form (384 token rows) is a workgroup of eight wavefronts, 4 x 2, each owning 96 x 64.  The vector
// instructions of the dequantisation cost a SIMD more time than the matrix instructions they feed (39 % against 32 %
// of the launch at 128 rows) and the two do not overlap, so what pays is dequantising a weight tile less often: at
// ~256 rows per expert one tall tile holds all of an expert's rows, one dequantisation per expert and row tile
// instead of two or three, one unit per thread and step instead of two.  A wavefront multiplies only the 32-row
// blocks that hold live rows, and only live rows' activation pieces are requested.
template <int QUANT, int NM, bool ROUTED, int TBM = 128>
__global__ void __launch_bounds__(TBM == 384 ? 512 : 256, TBM == 64 ? 3 : 2) k_mfma_expert(MfmaArgs a) {
  static_assert(TBM == 384 || TBM == 128 || TBM == 64, "token tile");
  constexpr bool kTall = TBM == 384;
  // Routed tiles are rarely full (an expert's run ends inside its last tile, and below ~1000 tokens most experts hold
  // a handful of rows): a wavefront multiplies only its 32-row blocks that hold live rows, and only live rows'
  // activation pieces are requested.  Same-box, per block: 512 tokens 304 -> 289 us, 2048: 482 -> 442, 4096: 716 -> 693.
  constexpr bool kSkip = kTall || ROUTED;
  constexpr int kThreads = kTall ? 512 : 256;
  constexpr int kUnits = 512 / kThreads;          // weight-row units (32 elements of a row) per thread and step
  constexpr int MI = kTall ? 3 : TBM / 64;        // 32-row blocks of the tile per wavefront
  // first tile row of block mi of wavefront row wm: consecutive blocks in the short forms; in the tall form block b of
  // the tile belongs to wavefront row b % 4, so that the live rows (the first `rows` of the tile) spread evenly
  constexpr int kBlockStride = kTall ? 128 : 32;  // rows between a wavefront's consecutive blocks
  constexpr int kWaveStride = kTall ? 32 : 32 * MI;  // rows between consecutive wavefront rows' first blocks
  constexpr int kAPieces = TBM * 16 / kThreads;   // 16-byte activation pieces per thread and step
  // 67.5 KB of LDS per workgroup at 128 token rows (two per CU), 137 KB at 384: dynamic, since the static limit is 64 KB
  extern __shared__ __attribute__((aligned(16))) uint8_t mfma_smem[];
  _Float16* sA = reinterpret_cast<_Float16*>(mfma_smem);
  _Float16* sB = sA + TBM * kLdA;
  // row tables, two sets (this item's and the next one's), each kTable = 3 * TBM words apart
  constexpr int kTable = 3 * TBM;
  int* sArow = reinterpret_cast<int*>(sB + kBR * kLd);  // activation row index of each tile row
  int* sOrow = sArow + TBM;                             // output row index, or -1 for a dead row
  float* sScale = reinterpret_cast<float*>(sOrow + TBM);

  const int tid = threadIdx.x, lane = tid & 63;
  // (uniform, so that the count of live blocks is a scalar and dead ones are branched around)
  const int wave = kSkip ? __builtin_amdgcn_readfirstlane(tid >> 6) : tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int valid = *a.valid_tokens;
  const int n_ntiles = a.n_rows / (NM == 2 ? 64 : 128);
  const int n_mtiles = ROUTED ? a.tile_list[0] : (valid + TBM - 1) / TBM;
  const int total = n_mtiles * n_ntiles;
  const int nks = a.K / kBK;
  const size_t row_bytes = QUANT == kQ6K ? (size_t)(a.K / 256) * kQ6KBytes : (size_t)(a.K / 32) * kQ8Bytes;

  // dequant mapping: unit u of LDS weight rows rb0 and rb0 + 64
  const int du = tid & 3, rb0 = tid >> 2;

  // Which items this workgroup takes.  Workgroup ids are dealt round-robin to the eight XCDs, each with its
  // own L2: when there is work for every workgroup, XCD x takes a contiguous eighth of the token tiles and its
  // workgroups walk that range together (token tile major), so an activation tile is fetched into one L2
  // once instead of into all eight, and the token tiles of one expert reuse its weights from that L2.
  const bool by_xcd = (gridDim.x & 7u) == 0 && total >= 2 * (int)gridDim.x && n_mtiles >= 8;
  const int xcd = blockIdx.x & 7;
  const int m_lo = by_xcd ? (int)((long long)n_mtiles * xcd / 8) : 0;
  const int m_hi = by_xcd ? (int)((long long)n_mtiles * (xcd + 1) / 8) : n_mtiles;
  const int first = by_xcd ? (int)(blockIdx.x >> 3) : (int)blockIdx.x;
  const int stride = by_xcd ? (int)(gridDim.x >> 3) : (int)gridDim.x;
  const int local_total = (m_hi - m_lo) * n_ntiles;
  if (first >= local_total) return;

  // One item = (token tile, weight-row tile).  Items are pipelined: the row tables, pointers and first loads of
  // item i + 1 are set up inside the last contraction step of item i, so its epilogue and the latency of the
  // next item's first loads overlap instead of adding up (the weight loads of a short contraction, 4 steps
  // for the down projection, otherwise wait ~8 us per item with nothing to hide behind).
  struct Item { int e, m0, rows, nt; };
  auto decode = [&](int item) __attribute__((always_inline)) {
    const int mt = m_lo + item / n_ntiles;
    Item it{0, mt * TBM, min(TBM, valid - mt * TBM), item % n_ntiles};
    if (ROUTED) {
      // The tile's entry through the scalar unit: a vector load here would be waited for with a count of zero,
      // i.e. together with every store the previous item's epilogue has just issued.
      typedef int int4v __attribute__((ext_vector_type(4)));
      int4v ent;
      const int* p = a.tile_list + 4 + 4 * mt;  // 16-byte aligned: the list starts on an allocation boundary
      asm volatile("s_load_dwordx4 %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(ent) : "s"(p));
      it.e = ent.x;
      it.m0 = ent.y;
      it.rows = ent.z;
    }
    return it;
  };
  // table entry of tile row `tid` (threads below TBM): activation row, output row (-1: dead), output scale.
  // In two parts, so that nothing waits for a load it has just issued: the row's flat selection index is
  // requested when the item is decoded, the entry is derived from it steps later.
  auto table_flat = [&](const Item& it) __attribute__((always_inline)) {
    // (an address that is always valid rather than a select on the loaded value, which would wait for it here)
    return ROUTED ? a.sorted_token_ids[it.m0 + min(tid, it.rows - 1)] : 0;
  };
  auto table_scale = [&](const Item& it, int flat) __attribute__((always_inline)) {
    return ROUTED && NM == 1 ? a.topk_weights[flat] : 1.0f;
  };
  auto table_entry = [&](const Item& it, int flat, int& arow, int& orow) __attribute__((always_inline)) {
    arow = 0, orow = -1;
    if (tid < it.rows) {
      if (ROUTED) {
        const int slot = it.m0 + tid;
        if (NM == 2) { arow = flat / a.top_k; orow = slot; }
        else { arow = slot; orow = flat; }
      } else {
        arow = orow = it.m0 + tid;
      }
    }
  };
  const ptrdiff_t up_minus_gate = NM == 2 ? a.w1 - a.w0 : 0;
  const uint8_t* wrow[kUnits];   // weight rows this thread dequantises
  uint32_t arow_off[kAPieces];   // activation chunks this thread moves, 16 bytes each per step: element offsets
  [[maybe_unused]] uint32_t arow_live = ~0u;  // routed forms: bit i set when piece i belongs to a live row
  auto set_wrow = [&](const Item& it) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < kUnits; ++i) {
      const int rb = rb0 + 64 * i;
      const uint8_t* base = a.w0;
      int wr;
      if (NM == 2) {
        const int half_n = rb >> 6, which = (rb >> 5) & 1, c = rb & 31;
        // (arithmetic, not a select of the two pointers: the compiler turns that into a per-lane load from the
        // kernel arguments, a memory operation in the middle of the steps)
        base += which ? up_minus_gate : (ptrdiff_t)0;
        wr = it.nt * 64 + half_n * 32 + c;
      } else {
        wr = it.nt * 128 + rb;
      }
      wrow[i] = base + (size_t)it.e * a.expert_bytes + (size_t)wr * row_bytes;
    }
  };
  auto set_arow = [&](int buf, [[maybe_unused]] int live_rows) __attribute__((always_inline)) {
    if constexpr (kSkip) arow_live = 0u;
#pragma unroll
    for (int i = 0; i < kAPieces; ++i) {
      const int c = tid + kThreads * i;
      // piece c of the tile lands at LDS byte 16 c: row c >> 4, position c & 15, which holds chunk pos ^ (row & 15)
      const int row = c >> 4, chunk = (c & 15) ^ (row & 15);
      arow_off[i] = (uint32_t)sArow[buf * kTable + row] * (uint32_t)a.K + (uint32_t)chunk * 8u;
      if constexpr (kSkip) arow_live |= row < live_rows ? 1u << i : 0u;
    }
  };

  // this step's activation tile: 1 KB pieces (eight per wavefront for 128 rows), global memory -> LDS.
  // Written as assembly on purpose: the compiler's wait bookkeeping treats the instruction as one that may
  // complete out of order with everything else, and answers any later wait for a weight register with "wait
  // for all of memory", which stalls every other step on the pieces it has just requested.  Unseen by that
  // bookkeeping, the pieces are covered by the step's second barrier (written by hand below), and the waits
  // the compiler computes for the weight registers only ever come out too strict, by the pieces it did not count.
  const uint32_t lds_a = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)sA + (uint32_t)wave * 1024u;
  auto move_a = [&](int ks) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < kAPieces; ++i) {
      if constexpr (kSkip) {
        if (!(arow_live & (1u << i))) continue;  // (a dead row's slot in LDS keeps whatever it held: its products are dropped)
      }
      // (the tile's base in scalar registers plus a 32-bit byte offset per lane: one address register instead of two)
      const uint32_t voff = (arow_off[i] + (uint32_t)ks * (uint32_t)kBK) * 2u;
      const uint32_t dst = __builtin_amdgcn_readfirstlane(lds_a + (uint32_t)(kThreads * 16) * i);  // + 16 * lane, by the hardware
      // (m0 is named as clobbered so that the compiler sets it again before any use of its own; it warns that it
      // does not preserve the register across the statement, which is what is wanted here)
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
      asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(a.a), "s"(dst) : "memory", "m0");
#pragma clang diagnostic pop
    }
  };

  // In flight per step: the raw weight bytes of the next two steps (the HBM-cold ones), in w[ks & 1]; the
  // activation tile (L2-warm) is moved during the step's own write phase, behind the dequantisation.  The contraction has an even
  // number of steps (whole superblocks), so the step pairs are unrolled and no register is copied.
  // (The down launch, NM = 1, has no registers to spare for the second step and keeps one in flight.)
  // (tall form: one step ahead; its steps are long enough, and a second set of raw registers does not fit)
  constexpr int kWDepth = kTall ? 1 : 2;
  // load instructions one step's two units issue at the very least, one per separately addressed piece: Q6_K ql
  // low, ql high, qh, scales, d; Q8_0 the two 16-byte halves of the codes and d.  (No two pieces of a unit
  // are adjacent in memory except the scales and d, ten bytes that no single load covers, so the compiler cannot
  // issue fewer; issuing more only makes the barrier's wait stricter.)
  constexpr int kWLoadsAtLeast = (QUANT == kQ6K ? 5 : 3) * kUnits;
  WRaw<QUANT, kUnits> w[kWDepth];

  Item cur = decode(first);
  {
    int arow, orow;
    if (tid < TBM) {
      const int flat = table_flat(cur);
      table_entry(cur, flat, arow, orow);
      sArow[tid] = arow;
      sOrow[tid] = orow;
      sScale[tid] = table_scale(cur, flat);
    }
    __syncthreads();
    set_wrow(cur);
    set_arow(0, cur.rows);
    // (fenced apart: the waits the compiler places in the steps are the strictest any path into them needs, and
    // with these two sets of loads interleaved here it would make every step wait for its newest loads)
    order_fence();
    load_step_w<QUANT, kUnits>(0, wrow, du, w[0]);
    order_fence();
    if constexpr (kWDepth == 2) load_step_w<QUANT, kUnits>(1, wrow, du, w[kWDepth - 1]);
    order_fence();
  }
  int buf = 0;
  // (routed down launch: the output scales requested during the previous item, stored to this item's table at its
  // start, by which time the load is many requests old and waiting for it waits for nothing else)
  float carried_sc = 1.0f;
  for (int item = first;; item += stride) {
    if constexpr (ROUTED && NM == 1) {
      if (item != first && tid < TBM) sScale[buf * kTable + tid] = carried_sc;
    }
    const bool has_next = item + stride < local_total;
    const Item nxt = has_next ? decode(item + stride) : cur;
    // (materialised here: a load sunk into the steps would put a full wait on one of their paths)
    asm volatile("" ::"s"(nxt.e), "s"(nxt.m0), "s"(nxt.rows), "s"(nxt.nt));
    // the next item's table entries: the flat index requested now, the scale two steps before the end, both
    // stored to the other table in the last step
    int n_flat = 0;
    if (has_next && tid < TBM) n_flat = table_flat(nxt);

    float16v acc[MI][2];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    auto step = [&](auto p_c, int ks) __attribute__((always_inline)) {
      constexpr int P = decltype(p_c)::value % kWDepth;
      // first barrier of the step: everyone has finished reading the previous step's tiles (LDS reads only: the
      // weight loads in flight stay in flight)
      order_fence();
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
      order_fence();
      if constexpr (ROUTED && NM == 1) {
        // the next item's output scales, two steps before they are stored.  (First thing in the step: the
        // compiler waits for everything in flight before it uses the flat index, and at this point that is the
        // previous step's weight loads, a whole step old, and not yet this step's activation pieces.)
        if (ks + kWDepth == nks && has_next && tid < TBM) {
          int flat = n_flat;
          asm volatile("" : "+v"(flat));
          carried_sc = table_scale(nxt, flat);
        }
      }
      move_a(ks);
#pragma unroll
      for (int i = 0; i < kUnits; ++i) {
        const int rb = rb0 + 64 * i;
        if constexpr (QUANT == kQ6K) {
          Q6Raw r;
          q6_finish(w[P].u[i], r);
          q6_unit_to_lds(r, du, &sB[rb * kLd], w_swizzle(rb));
        } else {
          Q8Raw r;
          q8_finish(w[P].u[i], r);
          q8_unit_to_lds(r, du, &sB[rb * kLd], w_swizzle(rb));
        }
      }
      if (ks == nks - 1 && has_next && tid < TBM) {
        // (the other table's last reader, the previous item's epilogue, finished before this item's first barrier)
        int n_arow, n_orow, flat = n_flat;
        asm volatile("" : "+v"(flat));  // (pins the entry's arithmetic here: hoisted to the item's start it would wait for the load there)
        table_entry(nxt, flat, n_arow, n_orow);
        sArow[(buf ^ 1) * kTable + tid] = n_arow;
        sOrow[(buf ^ 1) * kTable + tid] = n_orow;
        if constexpr (!(ROUTED && NM == 1)) sScale[(buf ^ 1) * kTable + tid] = 1.0f;
      }
      // The raw weight bytes of the step after next (past the end of this item: the first steps of the next one),
      // into the registers the dequantisation above has just released.  Issued after the activation pieces, so
      // that the wait for those at the barrier leaves these in flight: they have two whole steps to arrive.
      // (every step issues the same loads, so that the compiler's count of what is in flight is exact on every
      // path: the last two steps of a workgroup's last item re-read two of its own steps and drop them)
      const int ks_w = ks + kWDepth < nks ? ks + kWDepth : ks + kWDepth - nks;
      if (ks + kWDepth == nks && has_next) set_wrow(nxt);
      load_step_w<QUANT, kUnits>(ks_w, wrow, du, w[P]);
      // Second barrier of the step, by hand: this wavefront's LDS stores and its activation pieces must have
      // landed, the weight loads just issued need not.  Memory operations retire in order, so "all but the last
      // kWLoadsAtLeast" covers the pieces; the count is a lower bound of the load instructions a step issues
      // (one per field of each unit), so a miscount can only wait for more, never for less.
      order_fence();
      asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(kWLoadsAtLeast) : "memory");
      order_fence();
      if (ks + 1 == nks && has_next) set_arow(buf ^ 1, nxt.rows);
      const _Float16* pa = &sA[(wm * kWaveStride + (lane & 31)) * kLdA];
      // 32-row blocks of this wavefront that hold live rows (all of them in the unrouted forms)
      const int nb = kSkip ? min(max((cur.rows - wm * kWaveStride + kBlockStride - 1) / kBlockStride, 0), MI) : MI;
      const int swz = lane & 15, khalf = lane >> 5;  // (the row's low four bits are the lane's)
      const _Float16* pb = &sB[(wn * 64 + (lane & 31)) * kLd];
      const int wswz = w_swizzle(lane & 15);  // (the rows' low four bits are the lane's)
      // Operand fragments one sub-step ahead, in two register sets: the four LDS reads of sub-step kk + 1 are
      // issued before the four matrix instructions of sub-step kk, so their latency hides behind 128 cycles of
      // matrix work instead of standing between every group of four.
      // (tall form: one register set for the activation fragments, read at the start of their sub-step: a second set
      // does not fit beside 96 accumulators, and the SIMD's other wavefront multiplies while this one waits for LDS)
      constexpr int kASets = kTall ? 1 : 2;
      half8 fa[kASets][MI], fb[2][2];
      auto frags_a = [&](int kk, int set) __attribute__((always_inline)) {
        const int apos = ((kk * 2 + khalf) ^ swz) * 8;
#pragma unroll
        for (int mi = 0; mi < MI; ++mi)
          if (mi < nb) fa[set][mi] = *reinterpret_cast<const half8*>(pa + mi * kBlockStride * kLdA + apos);
      };
      auto frags_b = [&](int kk, int set) __attribute__((always_inline)) {
        const int bpos = ((kk * 2 + khalf) ^ wswz) * 8;
        fb[set][0] = *reinterpret_cast<const half8*>(pb + bpos);
        fb[set][1] = *reinterpret_cast<const half8*>(pb + 32 * kLd + bpos);
      };
      if (nb > 0) {
        frags_a(0, 0);
        frags_b(0, 0);
#pragma unroll
        for (int kk = 0; kk < kBK / 16; ++kk) {
          const int c = kk & 1;
          if (kk + 1 < kBK / 16) {
            if constexpr (kASets == 2) frags_a(kk + 1, c ^ 1);
            frags_b(kk + 1, c ^ 1);
          }
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int mi = 0; mi < MI; ++mi) {
            if (mi < nb) {
              acc[mi][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[c % kASets][mi], fb[c][0], acc[mi][0], 0, 0, 0);
              acc[mi][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[c % kASets][mi], fb[c][1], acc[mi][1], 0, 0, 0);
            }
          }
          __builtin_amdgcn_sched_barrier(0);
          if constexpr (kASets == 1) {
            if (kk + 1 < kBK / 16) frags_a(kk + 1, 0);
          }
        }
      }
    };
    if constexpr (kWDepth == 2) {
      // (at least one pair of steps, and written so: a path around the loop would count for the compiler's waits
      // after it, and on that path the loads issued just before the loop are the newest)
      int ks = 0;
      do {
        step(std::integral_constant<int, 0>{}, ks);
        step(std::integral_constant<int, 1>{}, ks + 1);
        ks += 2;
      } while (ks < nks);
    } else {
#pragma unroll 1
      for (int ks = 0; ks < nks; ++ks) step(std::integral_constant<int, 0>{}, ks);
    }

    // epilogue.  acc[mi][ni][v]: tile row (v/4)*8 + (lane/32)*4 + v%4, tile column lane%32
    // (transposing the tile through LDS so that every lane stores 16 bytes of a row was measured: two more
    // barriers per item and the extra registers cost more than the 48 fewer store instructions gave; so was
    // the transposed product, weights as the first operand, whose lanes hold four consecutive columns of one
    // token row: a quarter of the store instructions, but each touches 32 rows' cache lines with 32 bytes
    // instead of two rows' with 128, and the block took 1365 against 1333 us at 8192 tokens)
    // (the rows' table entries are all read first: one LDS round trip for the item instead of one per row)
    // (tall form: one 32-row block at a time, skipping blocks without live rows: all three blocks' entries at once
    // do not fit the registers beside 96 accumulators)
    auto store_blocks = [&](auto first_c, auto count_c) __attribute__((always_inline)) {
      constexpr int M0 = decltype(first_c)::value, MN = decltype(count_c)::value;
      int orows[MN][16];
      [[maybe_unused]] float scs[MN][16];
#pragma unroll
      for (int mi = 0; mi < MN; ++mi) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int r = wm * kWaveStride + (M0 + mi) * kBlockStride + (v >> 2) * 8 + (lane >> 5) * 4 + (v & 3);
          orows[mi][v] = sOrow[buf * kTable + r];
          if (NM == 1) scs[mi][v] = sScale[buf * kTable + r];
        }
      }
#pragma unroll
      for (int mi = 0; mi < MN; ++mi) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int orow = orows[mi][v];
          if (orow < 0) continue;
          if (NM == 2) {
            const int col = cur.nt * 64 + wn * 32 + (lane & 31);
            const float g = acc[M0 + mi][0][v] * kWScaleInv, u = acc[M0 + mi][1][v] * kWScaleInv;
            static_cast<_Float16*>(a.out)[(size_t)orow * a.n_rows + col] = (_Float16)(silu_fast(g) * u);
          } else {
            const float sc = scs[mi][v];
#pragma unroll
            for (int ni = 0; ni < 2; ++ni) {
              const int col = cur.nt * 128 + wn * 64 + ni * 32 + (lane & 31);
              static_cast<float*>(a.out)[(size_t)orow * a.n_rows + col] = sc * (acc[M0 + mi][ni][v] * kWScaleInv);
            }
          }
        }
      }
    };
    if constexpr (kTall) {
      const int nb = min(max((cur.rows - wm * kWaveStride + kBlockStride - 1) / kBlockStride, 0), MI);
      if (nb > 0) store_blocks(std::integral_constant<int, 0>{}, std::integral_constant<int, 1>{});
      if (nb > 1) store_blocks(std::integral_constant<int, 1>{}, std::integral_constant<int, 1>{});
      if (nb > 2) store_blocks(std::integral_constant<int, 2>{}, std::integral_constant<int, 1>{});
    } else if constexpr (kSkip) {
      const int nb = min(max((cur.rows - wm * kWaveStride + kBlockStride - 1) / kBlockStride, 0), MI);
      if (nb == MI) store_blocks(std::integral_constant<int, 0>{}, std::integral_constant<int, MI>{});
      else if (MI == 2 && nb == 1) store_blocks(std::integral_constant<int, 0>{}, std::integral_constant<int, 1>{});
    } else {
      store_blocks(std::integral_constant<int, 0>{}, std::integral_constant<int, MI>{});
    }
    if (!has_next) break;
    cur = nxt;
    buf ^= 1;
  }
}

// ------------------------------------------------------------------------------------------------------------
// The same grouped GEMM with the wavefronts of a workgroup specialised: an alternative form of the routed launches,
// selected with xabe_moe_kernels_set_mfma_form(k, 2).  Same bits as k_mfma_expert; measured within 0-7 % of it and
// never ahead (8192 tokens: gate/up 461 against 421 us, down 333 against 308), so it is not the default.  It is kept
// because it is the measured answer to "would wavefronts that only dequantise beside wavefronts that only multiply
// overlap the two kinds of work": they do not.  On a SIMD the producers' vector instructions and the consumers'
// matrix instructions take turns,
// so what decides the time is the sum of the two per token row, and that sum is smallest for the tallest token tile
// (one dequantisation per expert), whose accumulators only fit a few fat wavefronts: k_mfma_expert's 384-row form.
//
// A workgroup is sixteen wavefronts with two jobs:
//   consumers (wavefronts 0-7, 2 row halves x 4 column quarters): request the activation tile three steps ahead
//     (global memory -> LDS, no registers) and multiply THIS step's tiles: 64 token rows x 64 weight rows each;
//   producers (wavefronts 8-15): keep the raw weight bytes of the next two 128-element blocks of the contraction in
//     flight and dequantise the next step's weight tile into LDS.
// A step is 64 contraction elements; the weight tile is double-buffered and the activation tile sits in a ring of
// four, so there is ONE barrier per step and nobody waits inside a step for memory it has just asked for: a
// consumer's pieces were requested three steps earlier, a producer's raw bytes two to four steps earlier, and each
// kind of wavefront counts only its own loads (the wait counters are per wavefront).
//
// The tile is 128 token rows x 256 weight rows (gate/up: 128 + 128): twice k_mfma_expert's weight rows per
// activation byte (with 128 weight rows and a one-step-ahead activation tile the consumers waited for L2 every step:
// 623 us).
// Per output element the operands and the order of the matrix instructions are k_mfma_expert's (ascending
// contraction index, 16 elements per instruction), so the bits are the same.
// A Q6_K unit (32 codes of one row: 8 at each of four places 32 elements apart) spans two steps: its raw registers
// are loaded once per 128-element block and dequantised a half at a time.
// LDS: rows of 64 halfs (128 bytes: two rows to a 256-byte line of the 64 banks), 16-byte chunks XOR-swizzled by
// pc_swizzle(row) in both tiles.  Fragment reads are served sixteen lanes at a time (sixteen rows, one chunk each): the
// eight rows of either parity must put the chunk at eight different positions, hence a permutation of (row >> 1) & 7;
// the dequantised stores (lanes = rows x the four chunks 4 jj .. 4 jj + 3) need rows two apart to differ in the
// position's high bit, hence the bit order.  (With row & 7 the bank-conflict counter showed every fragment read taking
// twice its cycles.)
constexpr int kPK = 64;        // contraction elements per step
constexpr int kPM = 128;       // token rows per tile
constexpr int kPR = 256;       // weight rows per tile
constexpr int kPARing = 4;     // activation tiles in LDS
constexpr int kPAhead = 3;     // steps between an activation tile's request and its use
constexpr int kPCWaves = 8;    // consumer wavefronts (as many producers)
constexpr int kPAInstr = kPM / (8 * kPCWaves);  // activation-piece instructions per consumer wavefront and step (1 KB = 8 rows each)

__device__ __forceinline__ int pc_swizzle(int row) { return (((row >> 1) & 1) << 2) | ((row >> 2) & 3); }

constexpr size_t mfma_pc_lds_bytes() {
  return (size_t)kPARing * kPM * kPK * sizeof(_Float16) + (size_t)2 * kPR * kPK * sizeof(_Float16) + (size_t)2 * 3 * kPM * sizeof(int);
}

// half HH (codes at places 2 HH and 2 HH + 1) of a Q6_K unit -> chunks (jj * 4 + l8) of the row's 64-element tile row
template <int HH>
__device__ __forceinline__ void q6_half_unit_to_lds(const Q6Pend& r, int l8, _Float16* brow, int swz) {
  const int is8 = (l8 >> 1) * 8;
  const uint32_t sw = (HH ? r.sc.y : r.sc.x) >> is8;
  const float d = f16_bits_to_f32(r.dh) * kWScale;
  const float ds[2] = {d * (float)(int8_t)(sw & 0xff), d * (float)(int8_t)((sw >> 16) & 0xff)};
  uint32_t c[2][2];
#pragma unroll
  for (int w = 0; w < 2; ++w) {
    const uint32_t a = w ? r.qa.y : r.qa.x, b = w ? r.qb.y : r.qb.x, h = w ? r.qh.y : r.qh.x;
    if (HH == 0) {
      c[w][0] = (a & 0x0F0F0F0Fu) | ((h << 4) & 0x30303030u);
      c[w][1] = (b & 0x0F0F0F0Fu) | ((h << 2) & 0x30303030u);
    } else {
      c[w][0] = ((a >> 4) & 0x0F0F0F0Fu) | (h & 0x30303030u);
      c[w][1] = ((b >> 4) & 0x0F0F0F0Fu) | ((h >> 2) & 0x30303030u);
    }
  }
  const half2v off = {(_Float16)-1056.0f, (_Float16)-1056.0f};  // 1024 (perm bias) + 32 (code centre)
#pragma unroll
  for (int jj = 0; jj < 2; ++jj) {
    const _Float16 sh = (_Float16)ds[jj];
    const half2v s = {sh, sh};
    *reinterpret_cast<u32x4*>(brow + ((jj * 4 + l8) ^ swz) * 8) = pack8(c[0][jj], c[1][jj], off, s);
  }
}
// a Q8_0 block -> chunks 4 blk .. 4 blk + 3 of the row's 64-element tile row
__device__ __forceinline__ void q8_block_to_lds(const Q8Pend& r, int blk, _Float16* brow, int swz) {
  const _Float16 sh = (_Float16)(f16_bits_to_f32(r.dh) * kWScale);
  const half2v s = {sh, sh};
  const half2v off = {(_Float16)-1152.0f, (_Float16)-1152.0f};
  const uint32_t q[8] = {r.lo[0], r.lo[1], r.lo[2], r.lo[3], r.hi[0], r.hi[1], r.hi[2], r.hi[3]};
#pragma unroll
  for (int w = 0; w < 4; ++w)
    *reinterpret_cast<u32x4*>(brow + ((blk * 4 + w) ^ swz) * 8) = pack8(q[2 * w] ^ 0x80808080u, q[2 * w + 1] ^ 0x80808080u, off, s);
}

template <int QUANT, int NM>
__global__ void __launch_bounds__(1024, 4) k_mfma_pc(MfmaArgs a) {
  constexpr int kTable = 3 * kPM;
  extern __shared__ __attribute__((aligned(16))) uint8_t mfma_smem[];
  _Float16* sA = reinterpret_cast<_Float16*>(mfma_smem);          // [kPARing][128][64]
  _Float16* sB = sA + kPARing * kPM * kPK;                        // [2][256][64]
  int* sArow = reinterpret_cast<int*>(sB + 2 * kPR * kPK);        // [2][3 x 128]: activation row, output row (-1: dead), scale
  int* sOrow = sArow + kPM;
  float* sScale = reinterpret_cast<float*>(sOrow + kPM);

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const bool producer = wave >= kPCWaves;
  const int n_ntiles = a.n_rows / (NM == 2 ? kPR / 2 : kPR);
  const int n_mtiles = a.tile_list[0];
  const int total = n_mtiles * n_ntiles;
  const int nks = a.K / kPK;  // a multiple of four (whole superblocks), at least eight (checked by the host)
  const size_t row_bytes = QUANT == kQ6K ? (size_t)(a.K / 256) * kQ6KBytes : (size_t)(a.K / 32) * kQ8Bytes;

  // which items this workgroup takes: k_mfma_expert's dealing (an XCD walks a contiguous eighth of the token tiles)
  const bool by_xcd = (gridDim.x & 7u) == 0 && total >= 2 * (int)gridDim.x && n_mtiles >= 8;
  const int xcd = blockIdx.x & 7;
  const int m_lo = by_xcd ? (int)((long long)n_mtiles * xcd / 8) : 0;
  const int m_hi = by_xcd ? (int)((long long)n_mtiles * (xcd + 1) / 8) : n_mtiles;
  const int first = by_xcd ? (int)(blockIdx.x >> 3) : (int)blockIdx.x;
  const int stride = by_xcd ? (int)(gridDim.x >> 3) : (int)gridDim.x;
  const int local_total = (m_hi - m_lo) * n_ntiles;
  if (first >= local_total) return;
  const int n_items = (local_total - first + stride - 1) / stride;
  const int n_steps = n_items * nks;  // a multiple of four

  struct Item { int e, m0, rows, nt; };
  auto decode = [&](int item) __attribute__((always_inline)) {
    const int mt = m_lo + item / n_ntiles;
    typedef int int4v __attribute__((ext_vector_type(4)));
    int4v ent;
    const int* p = a.tile_list + 4 + 4 * mt;
    asm volatile("s_load_dwordx4 %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(ent) : "s"(p));
    return Item{ent.x, ent.y, ent.z, item % n_ntiles};
  };

  // ---- the first item's row tables, by the consumers' threads; everyone meets at one barrier before the steps
  if (tid < kPM) {
    const Item it = decode(first);
    int arow = 0, orow = -1;
    float sc = 1.0f;
    if (tid < it.rows) {
      const int slot = it.m0 + tid, flat = a.sorted_token_ids[slot];
      if (NM == 2) { arow = flat / a.top_k; orow = slot; }
      else { arow = slot; orow = flat; sc = a.topk_weights[flat]; }
    }
    sArow[tid] = arow;
    sOrow[tid] = orow;
    sScale[tid] = sc;
  }
  __syncthreads();

  if (producer) {
    // ================================================================= producers
    const int ptid = tid - 64 * kPCWaves;
    // Q6_K: units (row rb0 + 128 i, place l8) of the 256-row tile, two per thread, raw registers per 128-element block
    // Q8_0: one 34-byte block per thread and step: row q8row, block q8blk of the step's two
    constexpr int kUnits = QUANT == kQ6K ? 2 : 1;
    const int du = ptid & 3, rb0 = ptid >> 2;
    const int q8row = ptid & 255, q8blk = ptid >> 8;
    const ptrdiff_t up_minus_gate = NM == 2 ? a.w1 - a.w0 : 0;
    const uint8_t* wrow[kUnits];
    auto tile_row = [&](int i) __attribute__((always_inline)) { return QUANT == kQ6K ? rb0 + 128 * i : q8row; };
    auto set_wrow = [&](const Item& it) __attribute__((always_inline)) {
#pragma unroll
      for (int i = 0; i < kUnits; ++i) {
        const int rb = tile_row(i);
        const uint8_t* base = a.w0;
        int wr;
        if (NM == 2) {
          // tile rows in groups of 32: gate columns, the matching up columns, the next 32 gate columns, ...
          const int grp = rb >> 6, which = (rb >> 5) & 1, c = rb & 31;
          base += which ? up_minus_gate : (ptrdiff_t)0;
          wr = it.nt * (kPR / 2) + grp * 32 + c;
        } else {
          wr = it.nt * kPR + rb;
        }
        wrow[i] = base + (size_t)it.e * a.expert_bytes + (size_t)wr * row_bytes;
      }
    };
    // raw bytes in flight: Q6_K two blocks of 128 (sets by block parity), Q8_0 four steps (sets by step & 3)
    constexpr int kSets = QUANT == kQ6K ? 2 : 4;
    typename std::conditional<QUANT == kQ6K, Q6Pend, Q8Pend>::type raw[kSets][kUnits];
    // the load stream runs ahead of the dequantisation, across item boundaries: its own item counter and pointers
    int ld_item = 0, ld_k = 0;  // next load: item index (0 .. n_items), and block (Q6_K) or step (Q8_0) within it
    const int ld_per_item = QUANT == kQ6K ? nks / 2 : nks;
    set_wrow(decode(first));
    auto issue = [&](auto set_c) __attribute__((always_inline)) {
      constexpr int S = decltype(set_c)::value;
      // (past the last item the stream re-reads the last item's first blocks and drops them: every fill issues
      // the same loads, so the compiler's count of what is in flight is exact on every path)
#pragma unroll
      for (int i = 0; i < kUnits; ++i) {
        if constexpr (QUANT == kQ6K) {
          // block ld_k covers superblock ld_k >> 1, half ld_k & 1
          q6_issue(wrow[i] + (size_t)(ld_k >> 1) * kQ6KBytes, ld_k & 1, du, raw[S][i]);
        } else {
          q8_issue(wrow[i] + (size_t)(ld_k * 2 + q8blk) * kQ8Bytes, raw[S][i]);
        }
      }
      if (++ld_k == ld_per_item) {
        ld_k = 0;
        if (++ld_item < n_items) set_wrow(decode(first + ld_item * stride));
      }
    };
    // fill of the weight tile of global step T (T & 3 == P): into buffer T & 1
    auto fill = [&](auto p_c) __attribute__((always_inline)) {
      constexpr int P = decltype(p_c)::value;
      _Float16* dst = sB + (P & 1) * kPR * kPK;
      if constexpr (QUANT == kQ6K) {
        constexpr int S = P >> 1, HH = P & 1;
#pragma unroll
        for (int i = 0; i < kUnits; ++i) {
          const int rb = tile_row(i);
          q6_half_unit_to_lds<HH>(raw[S][i], du, dst + rb * kPK, pc_swizzle(rb));
        }
        if constexpr (HH == 1) issue(std::integral_constant<int, S>{});  // the block after next, into the registers just released
      } else {
#pragma unroll
        for (int i = 0; i < kUnits; ++i) {
          const int rb = tile_row(i);
          q8_block_to_lds(raw[P][i], q8blk, dst + rb * kPK, pc_swizzle(rb));
        }
        issue(std::integral_constant<int, P>{});
      }
    };
    order_fence();
    issue(std::integral_constant<int, 0>{});
    order_fence();
    issue(std::integral_constant<int, 1>{});
    order_fence();
    if constexpr (QUANT != kQ6K) {
      issue(std::integral_constant<int, 2>{});
      order_fence();
      issue(std::integral_constant<int, 3>{});
      order_fence();
    }
    fill(std::integral_constant<int, 0>{});
    for (int T = 0; T < n_steps; T += 4) {
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
      fill(std::integral_constant<int, 1>{});
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
      fill(std::integral_constant<int, 2>{});
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
      fill(std::integral_constant<int, 3>{});
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
      if (T + 4 < n_steps) fill(std::integral_constant<int, 0>{});
    }
    return;
  }

  // ================================================================= consumers
  const int wm = wave >> 2, wq = wave & 3;  // row half (blocks b % 2 == wm), column quarter (64 weight rows)
  // piece q = i * kPCWaves + wave of the tile: rows 8 q .. 8 q + 7; lane: row 8 q + (lane >> 3), position lane & 7, which holds
  // chunk (lane & 7) ^ pc_swizzle(row).  Every piece is requested, dead rows' too (from the tile's first row): the count of
  // requests in flight is then the same at every step, which is what the waits below rely on.
  uint32_t arow_off[kPAInstr], arow_nxt[kPAInstr];
  auto set_arow = [&](int tb, uint32_t (&dst)[kPAInstr]) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < kPAInstr; ++i) {
      const int row = 8 * (i * kPCWaves + wave) + (lane >> 3), chunk = (lane & 7) ^ pc_swizzle(row);
      dst[i] = (uint32_t)sArow[tb * kTable + row] * (uint32_t)a.K + (uint32_t)chunk * 8u;
    }
  };
  const uint32_t lds_a = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)sA;
  auto move_a = [&](int slot, int ks, const uint32_t (&off)[kPAInstr]) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < kPAInstr; ++i) {
      const int q = i * kPCWaves + wave;
      const uint32_t voff = (off[i] + (uint32_t)ks * (uint32_t)kPK) * 2u;
      const uint32_t dst = __builtin_amdgcn_readfirstlane(lds_a + (uint32_t)(slot * kPM * kPK * 2) + (uint32_t)q * 1024u);
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
      asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(a.a), "s"(dst) : "memory", "m0");
#pragma clang diagnostic pop
    }
  };

  Item cur = decode(first);
  set_arow(0, arow_off);
#pragma unroll
  for (int i = 0; i < kPAInstr; ++i) arow_nxt[i] = arow_off[i];
  // the first kPAhead tiles (an item has at least eight steps)
#pragma unroll
  for (int t = 0; t < kPAhead; ++t) move_a(t, t, arow_off);
  int step = 0;
  for (int idx = 0; idx < n_items; ++idx) {
    const bool has_next = idx + 1 < n_items;
    const Item nxt = has_next ? decode(first + (idx + 1) * stride) : cur;
    asm volatile("" ::"s"(nxt.e), "s"(nxt.m0), "s"(nxt.rows), "s"(nxt.nt));
    const int tb = idx & 1;
    int n_flat = 0;
    float n_sc = 1.0f;

    float16v acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;
    // live 32-row blocks of this consumer row: block b = 2 mi + wm holds rows 32 b ..
    const int nb = min(max((cur.rows - 32 * wm + 63) / 64, 0), 2);

#pragma unroll 1
    for (int ks = 0; ks < nks; ++ks, ++step) {
      // this step's tiles are there: my own pieces of it (requested three steps ago; memory operations retire in
      // order, so all but the two newer tiles' requests covers them) have landed, and past the barrier so have
      // everyone else's and the producers' weight tile.  Near the end of the workgroup's work fewer requests follow.
      order_fence();
      if (step + kPAhead <= n_steps) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"((kPAhead - 1) * kPAInstr) : "memory");
      else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
      order_fence();
      // the next item's row tables, in three parts spread over this item's steps so that nothing waits for a load
      // it has just issued: flat selection index, output scale, the table itself
      if (has_next && tid < kPM) {
        if (ks == 0) n_flat = a.sorted_token_ids[nxt.m0 + min(tid, nxt.rows - 1)];
        if (NM == 1 && ks == 2) n_sc = a.topk_weights[n_flat];
        if (ks == nks - kPAhead - 2) {
          int arow = 0, orow = -1;
          if (tid < nxt.rows) {
            const int slot = nxt.m0 + tid;
            if (NM == 2) { arow = n_flat / a.top_k; orow = slot; }
            else { arow = slot; orow = n_flat; }
          }
          sArow[(tb ^ 1) * kTable + tid] = arow;
          sOrow[(tb ^ 1) * kTable + tid] = orow;
          sScale[(tb ^ 1) * kTable + tid] = n_sc;
        }
      }
      if (has_next && ks == nks - kPAhead - 1) set_arow(tb ^ 1, arow_nxt);  // (the table was written a step ago)
      // the activation tile of three steps on, into the ring slot everyone finished reading before the barrier above
      if (step + kPAhead < n_steps) {
        const int slot = (step + kPAhead) & (kPARing - 1);
        if (ks + kPAhead < nks) move_a(slot, ks + kPAhead, arow_off);
        else move_a(slot, ks + kPAhead - nks, arow_nxt);
      }
      if (nb > 0) {
        const _Float16* pa = sA + (step & (kPARing - 1)) * kPM * kPK + (32 * wm + (lane & 31)) * kPK;
        const _Float16* pb = sB + (step & 1) * kPR * kPK + (wq * 64 + (lane & 31)) * kPK;
        const int aswz = pc_swizzle(lane), khalf = lane >> 5;    // (block rows start at multiples of 32: the row's low bits are the lane's)
        const int wswz = aswz;
        half8 fa[2][2], fb[2][2];
        auto frags = [&](int kk, int set) __attribute__((always_inline)) {
          const int apos = ((kk * 2 + khalf) ^ aswz) * 8, bpos = ((kk * 2 + khalf) ^ wswz) * 8;
#pragma unroll
          for (int mi = 0; mi < 2; ++mi)
            if (mi < nb) fa[set][mi] = *reinterpret_cast<const half8*>(pa + mi * 64 * kPK + apos);
#pragma unroll
          for (int ni = 0; ni < 2; ++ni) fb[set][ni] = *reinterpret_cast<const half8*>(pb + ni * 32 * kPK + bpos);
        };
        frags(0, 0);
#pragma unroll
        for (int kk = 0; kk < kPK / 16; ++kk) {
          const int c = kk & 1;
          if (kk + 1 < kPK / 16) frags(kk + 1, c ^ 1);
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int mi = 0; mi < 2; ++mi) {
            if (mi < nb) {
#pragma unroll
              for (int ni = 0; ni < 2; ++ni)
                acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[c][mi], fb[c][ni], acc[mi][ni], 0, 0, 0);
            }
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }

    // epilogue: acc[mi][ni][v] is tile row 32 (2 mi + wm) + (v / 4) * 8 + (lane / 32) * 4 + v % 4, column lane % 32 of
    // the wavefront's column block ni
#pragma unroll
    for (int mi = 0; mi < 2; ++mi) {
      if (mi >= nb) break;
      int orows[16];
      [[maybe_unused]] float scs[16];
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int r = 32 * (2 * mi + wm) + (v >> 2) * 8 + (lane >> 5) * 4 + (v & 3);
        orows[v] = sOrow[tb * kTable + r];
        if (NM == 1) scs[v] = sScale[tb * kTable + r];
      }
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int orow = orows[v];
        if (orow < 0) continue;
        if (NM == 2) {
          // column blocks 0 and 1: gate and the matching up columns
          const int col = cur.nt * (kPR / 2) + wq * 32 + (lane & 31);
          const float g = acc[mi][0][v] * kWScaleInv, u = acc[mi][1][v] * kWScaleInv;
          static_cast<_Float16*>(a.out)[(size_t)orow * a.n_rows + col] = (_Float16)(silu_fast(g) * u);
        } else {
#pragma unroll
          for (int ni = 0; ni < 2; ++ni) {
            const int col = cur.nt * kPR + wq * 64 + ni * 32 + (lane & 31);
            static_cast<float*>(a.out)[(size_t)orow * a.n_rows + col] = scs[v] * (acc[mi][ni][v] * kWScaleInv);
          }
        }
      }
    }
    cur = nxt;
#pragma unroll
    for (int i = 0; i < kPAInstr; ++i) arow_off[i] = arow_nxt[i];
  }
}

// fp32 -> fp16 activations for live rows; rows past `valid` are left alone.
__global__ void __launch_bounds__(256) k_to_f16_rows(const float* __restrict__ x, const int* __restrict__ valid_tokens,
                                                      int width, _Float16* __restrict__ out) {
  const int t = blockIdx.x;
  if (t >= *valid_tokens) return;
  const float4* src = reinterpret_cast<const float4*>(x + (size_t)t * width);
  uint2* dst = reinterpret_cast<uint2*>(out + (size_t)t * width);
  for (int j = threadIdx.x; j < width / 4; j += 256) {
    const float4 v = src[j];
    const half2v lo = {(_Float16)v.x, (_Float16)v.y}, hi = {(_Float16)v.z, (_Float16)v.w};
    dst[j] = make_uint2(__builtin_bit_cast(uint32_t, lo), __builtin_bit_cast(uint32_t, hi));
  }
}

// Token-tile list: one entry per `bm`-slot chunk of each active expert's run.  One workgroup.  With bm_b > 0 a second
// list of that tile height goes to tile_list_b in the same launch (the routed gate/up launch's, where it differs).
__global__ void __launch_bounds__(256) k_build_tiles(const int* __restrict__ expert_counts, int num_experts, int block_size,
                                                      int capacity, int bm, int* __restrict__ tile_list, int bm_b,
                                                      int* __restrict__ tile_list_b) {
  __shared__ int s_base[513], s_tiles[513];
  // exclusive prefixes of the padded run lengths and of the tile counts (num_experts <= 512): every thread
  // takes two experts, the pair sums are scanned across the workgroup in eight doubling steps
  __shared__ int s_scan[2][2][256];
  const int t = threadIdx.x;
  for (int pass = 0; pass < (bm_b > 0 ? 2 : 1); ++pass) {
    const int h = pass ? bm_b : bm;
    int* list = pass ? tile_list_b : tile_list;
    int pad[2], til[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int e = 2 * t + j;
      const int c = e < num_experts ? expert_counts[e] : 0;
      pad[j] = (c + block_size - 1) / block_size * block_size;
      til[j] = (c + h - 1) / h;
    }
    __syncthreads();  // (the previous pass has read its tables)
    s_scan[0][0][t] = pad[0] + pad[1];
    s_scan[0][1][t] = til[0] + til[1];
    __syncthreads();
    int cur = 0;
    for (int d = 1; d < 256; d <<= 1) {
#pragma unroll
      for (int a = 0; a < 2; ++a) s_scan[cur ^ 1][a][t] = s_scan[cur][a][t] + (t >= d ? s_scan[cur][a][t - d] : 0);
      cur ^= 1;
      __syncthreads();
    }
    {
      const int base = s_scan[cur][0][t] - (pad[0] + pad[1]), tiles = s_scan[cur][1][t] - (til[0] + til[1]);
      if (2 * t < num_experts) s_base[2 * t] = base, s_tiles[2 * t] = tiles;
      if (2 * t + 1 < num_experts) s_base[2 * t + 1] = base + pad[0], s_tiles[2 * t + 1] = tiles + til[0];
      if (t == 255) list[0] = min(s_scan[cur][1][t], capacity);
    }
    __syncthreads();
    for (int e = threadIdx.x; e < num_experts; e += 256) {
      const int c = expert_counts[e];
      const int nt = (c + h - 1) / h;
      for (int i = 0; i < nt; ++i) {
        const int idx = s_tiles[e] + i;
        if (idx >= capacity) break;
        list[4 + 4 * idx + 0] = e;
        list[4 + 4 * idx + 1] = s_base[e] + i * h;
        list[4 + 4 * idx + 2] = min(h, c - i * h);
        list[4 + 4 * idx + 3] = 0;
      }
    }
  }
}

// ------------------------------------------------------------------ host side
static size_t stack_row_bytes(int quant, size_t K) {
  return K / xabe_expert_quant_block_elements(quant) * xabe_expert_quant_block_bytes(quant);
}

bool mfma_supported(const xabe_moe_kernels* k, const xabe_moe_buffers* b, int gate_q, int up_q, int down_q, bool routed) {
  const xabe_moe_geometry& g = k->g;
  if (!k->tensor_cores || k->exact_regime || g.max_tokens < kMfmaMinTokens) return false;
  if (!b->x_h || !b->shared_inter_h) return false;
  if (routed && (!b->inter_h || !b->tile_list)) return false;
  if (routed && g.num_experts > 512) return false;  // k_build_tiles scans two experts per thread of one 256-thread workgroup
  auto ok = [](int q) { return q == XABE_QUANT_Q6K || q == XABE_QUANT_Q8_0; };
  if (!ok(gate_q) || !ok(down_q) || gate_q != up_q) return false;
  // contraction in steps of 128 (whole Q6_K superblocks: 256); gate/up tiles 64 columns, down tiles 128
  if (g.hidden % 256 != 0 || g.intermediate % 256 != 0) return false;
  // an activation piece is addressed by a 32-bit byte offset from its tensor's base (fp16 rows of either width, as
  // many as the sorted table has slots)
  const size_t rows = g.max_tokens * g.experts_per_token + g.num_experts * g.block_size;
  if (rows * std::max(g.hidden, g.intermediate) >= ((size_t)1 << 31)) return false;
  return true;
}

// Token-tile height for a geometry: the narrow tile while an expert's share of a full pass usually fits in it
// (an average of 48 selections per expert; at 64 every second expert overflows into a second tile, measured
// 702 against 695 us at 2048 tokens).
// `tokens`: pass_tokens() below.
static int routed_tile_rows(const xabe_moe_geometry& g, size_t tokens) {
  return tokens * g.experts_per_token <= 48 * g.num_experts ? 64 : kBM;
}
// The specialised form (k_mfma_pc) serves both routed launches for contractions of whole superblocks and at least
// eight steps, when asked for: `mfma_form` 2 (0 and 1: k_mfma_expert everywhere; it is the faster at every width
// measured, see k_mfma_pc).
static bool pc_shape_ok(const xabe_moe_geometry& g) {
  return g.hidden % 256 == 0 && g.intermediate % 256 == 0 && g.hidden >= 512 && g.intermediate >= 512;
}
static bool pc_form(const xabe_moe_kernels* k, size_t) { return k->mfma_form == 2 && pc_shape_ok(k->g); }
// The tokens a pass is known to hold when its launches are chosen: the live count last published to the device
// scalar (a 512-token chunk run in buffers sized for 8192 should get the tiles of a 512-token pass), the buffers'
// size before any was.  Every tile height serves any live count and gives the same bits, so a graph captured at one
// count and replayed after another was published is slower at worst.
static size_t pass_tokens(const xabe_moe_kernels* k, const xabe_moe_buffers* b) {
  return b->valid_published > 0 ? std::min<size_t>((size_t)b->valid_published, k->g.max_tokens) : k->g.max_tokens;
}
// Token-tile height of the routed gate/up launch: the tall tile once an expert's share of a full pass fills most of it
// (an average of 192 selections per expert: 6144 tokens of the model's shape).  Same-box, per block: 8192 tokens 1323
// -> 1263 us (the launch itself 503 -> ~415), 6144 tokens 1081 -> 1043; at 4096 tokens (128 per expert) the tall tile
// loses (778 against 767).  The down launch keeps the short tiles at every width: its contraction is four steps, its
// items are mostly epilogue, and with tall tiles the block measured 1279 us against 1263.
static int routed_up_tile_rows(const xabe_moe_kernels* k, size_t tokens) {
  const xabe_moe_geometry& g = k->g;
  if (pc_form(k, tokens)) return kPM;
  if (tokens * g.experts_per_token >= 192 * g.num_experts) return 384;
  return routed_tile_rows(g, tokens);
}
// The shared expert's launches are short of workgroups below a few thousand tokens: the narrow tile while all
// of its items still start at once (two workgroups per compute unit), so that twice as many units share the work.
static int shared_tile_rows(const xabe_moe_kernels* k, size_t tokens, size_t row_tiles) {
  return (tokens + 63) / 64 * row_tiles <= (size_t)k->num_cus * 2 ? 64 : kBM;
}

bool mfma_tile_plan(const xabe_moe_kernels* k, const xabe_moe_buffers* b, int* bm, int* bm_up, int* capacity) {
  if (!b->tile_list || b->n_tile_list < 16 || !k->tensor_cores || k->exact_regime) return false;
  const size_t tokens = pass_tokens(k, b);
  *bm = routed_tile_rows(k->g, tokens);
  if (pc_form(k, tokens)) *bm = kPM;  // (both specialised launches: 128-row tiles, one list)
  *bm_up = routed_up_tile_rows(k, tokens);
  *capacity = (int)((b->n_tile_list / 2 - 4) / 4);
  return true;
}

// LDS a workgroup of the kernel asks for (dynamic: above the static limit).  The limit is raised per function,
// once, when a kernels handle is created (mfma_configure): nothing on the launch path but the launch.
template <int TBM>
constexpr size_t mfma_lds_bytes() {
  return (size_t)(TBM * kLdA + kBR * kLd) * sizeof(_Float16) + 2 * 3 * TBM * sizeof(int);
}
template <int NM, bool ROUTED, int TBM>
static int configure_one() {
  const void* fns[2] = {reinterpret_cast<const void*>(k_mfma_expert<kQ6K, NM, ROUTED, TBM>),
                        reinterpret_cast<const void*>(k_mfma_expert<kQ8_0, NM, ROUTED, TBM>)};
  for (const void* f : fns)
    XABE_HIP_TRY(hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, (int)mfma_lds_bytes<TBM>()));
  return XABE_OK;
}
template <int NM>
static int configure_pc() {
  const void* fns[2] = {reinterpret_cast<const void*>(k_mfma_pc<kQ6K, NM>), reinterpret_cast<const void*>(k_mfma_pc<kQ8_0, NM>)};
  for (const void* f : fns)
    XABE_HIP_TRY(hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, (int)mfma_pc_lds_bytes()));
  return XABE_OK;
}
template <int NM>
static int launch_pc(const xabe_moe_kernels* k, int quant, const MfmaArgs& a, size_t max_items, hipStream_t s) {
  const unsigned grid = (unsigned)std::max<size_t>(1, std::min<size_t>(max_items, (size_t)k->num_cus));  // one workgroup per CU
  constexpr size_t smem = mfma_pc_lds_bytes();
  if (quant == XABE_QUANT_Q6K) hipLaunchKernelGGL((k_mfma_pc<kQ6K, NM>), dim3(grid), dim3(1024), smem, s, a);
  else hipLaunchKernelGGL((k_mfma_pc<kQ8_0, NM>), dim3(grid), dim3(1024), smem, s, a);
  XABE_HIP_TRY(hipGetLastError());
  return XABE_OK;
}

int mfma_configure() {
  static bool done = false;  // (one device per process)
  if (done) return XABE_OK;
  XABE_TRY((configure_pc<2>()));
  XABE_TRY((configure_pc<1>()));
  XABE_TRY((configure_one<1, false, 64>()));
  XABE_TRY((configure_one<1, false, 128>()));
  XABE_TRY((configure_one<1, true, 64>()));
  XABE_TRY((configure_one<1, true, 128>()));
  XABE_TRY((configure_one<2, false, 64>()));
  XABE_TRY((configure_one<2, false, 128>()));
  XABE_TRY((configure_one<2, true, 64>()));
  XABE_TRY((configure_one<2, true, 128>()));
  XABE_TRY((configure_one<2, true, 384>()));
  done = true;
  return XABE_OK;
}

template <int NM, bool ROUTED, int TBM>
static int launch_mfma(const xabe_moe_kernels* k, int quant, const MfmaArgs& a, size_t max_items, hipStream_t s) {
  // workgroups resident per CU: the narrow tile's registers (about 150) and LDS (49.5 KB) leave room for a third
  // (the tall tile: eight wavefronts and 137 KB of LDS, one workgroup per CU)
  const size_t per_cu = TBM == 64 ? 3 : TBM == 128 ? 2 : 1;
  const unsigned grid = (unsigned)std::max<size_t>(1, std::min<size_t>(max_items, (size_t)k->num_cus * per_cu));
  constexpr size_t smem = mfma_lds_bytes<TBM>();
  constexpr unsigned threads = TBM == 384 ? 512 : 256;
  if (quant == XABE_QUANT_Q6K) hipLaunchKernelGGL((k_mfma_expert<kQ6K, NM, ROUTED, TBM>), dim3(grid), dim3(threads), smem, s, a);
  else hipLaunchKernelGGL((k_mfma_expert<kQ8_0, NM, ROUTED, TBM>), dim3(grid), dim3(threads), smem, s, a);
  XABE_HIP_TRY(hipGetLastError());
  return XABE_OK;
}

static int to_f16(const xabe_moe_kernels* k, hipStream_t s, const xabe_moe_buffers* b, const float* x) {
  hipLaunchKernelGGL(k_to_f16_rows, dim3((unsigned)k->g.max_tokens), dim3(256), 0, s, x, b->valid_tokens, (int)k->g.hidden,
                     reinterpret_cast<_Float16*>(b->x_h));
  XABE_HIP_TRY(hipGetLastError());
  return XABE_OK;
}

int mfma_convert_activations(const xabe_moe_kernels* k, hipStream_t s, xabe_moe_buffers* b, const float* x) {
  return to_f16(k, s, b, x);
}

int mfma_grouped_forward_partial(const xabe_moe_kernels* k, hipStream_t s, xabe_moe_buffers* b, xabe_quant_tensor gate,
                                 xabe_quant_tensor up, xabe_quant_tensor down, const float* x) {
  const xabe_moe_geometry& g = k->g;
  if (!b->x_h_ready) XABE_TRY(to_f16(k, s, b, x));
  // (the allocation holds two lists of the same capacity: the down launch's, and the gate/up launch's where its tile
  // height differs)
  const size_t list_ints = b->n_tile_list / 2;
  int bm = 0, bm_up = 0, cap = 0;
  if (!mfma_tile_plan(k, b, &bm, &bm_up, &cap))
    return set_error(XABE_ERR_INVALID_ARGUMENT, "grouped_forward: these buffers hold no token-tile lists");
  int* list_up = bm_up == bm ? b->tile_list : b->tile_list + list_ints;
  // (the dispatch build has usually left the lists, cut for these heights)
  // trusted only when nothing can have rewritten them since: inside the capture that holds the build, or eagerly
  // after an eager build on buffers no graph has ever recorded a build on
  const unsigned long long capture = stream_capture_id(s);
  const bool trusted = b->tiles_bm == bm && b->tiles_bm_up == bm_up && capture != kCaptureUnknown &&
                       b->tiles_capture == capture && (capture != 0 || !b->tiles_graph_owned);
  if (!trusted) {
    hipLaunchKernelGGL(k_build_tiles, dim3(1), dim3(256), 0, s, b->expert_counts, (int)g.num_experts, (int)g.block_size, cap,
                       bm, b->tile_list, bm_up != bm ? bm_up : 0, list_up);
    XABE_HIP_TRY(hipGetLastError());
  }
  MfmaArgs a;
  memset(&a, 0, sizeof(a));
  a.valid_tokens = b->valid_tokens;
  a.sorted_token_ids = b->sorted_token_ids;
  a.topk_weights = b->topk_weights;
  a.tile_list = list_up;
  a.top_k = (int)g.experts_per_token;
  const size_t max_mtiles = (size_t)cap;
  // gate/up + SwiGLU -> inter_h[slot][I]
  a.w0 = static_cast<const uint8_t*>(gate.bytes);
  a.w1 = static_cast<const uint8_t*>(up.bytes);
  a.expert_bytes = g.intermediate * stack_row_bytes(gate.quant, g.hidden);
  a.a = reinterpret_cast<const _Float16*>(b->x_h);
  a.out = b->inter_h;
  a.K = (int)g.hidden;
  a.n_rows = (int)g.intermediate;
  const bool pc = pc_form(k, pass_tokens(k, b));
  if (pc && bm_up == kPM) XABE_TRY((launch_pc<2>(k, gate.quant, a, max_mtiles * (g.intermediate / (kPR / 2)), s)));
  else if (bm_up == 64) XABE_TRY((launch_mfma<2, true, 64>(k, gate.quant, a, max_mtiles * (g.intermediate / 64), s)));
  else if (bm_up == 384) XABE_TRY((launch_mfma<2, true, 384>(k, gate.quant, a, max_mtiles * (g.intermediate / 64), s)));
  else XABE_TRY((launch_mfma<2, true, 128>(k, gate.quant, a, max_mtiles * (g.intermediate / 64), s)));
  // down -> partial[flat][H], scaled by the routing weight
  a.tile_list = b->tile_list;
  a.w0 = static_cast<const uint8_t*>(down.bytes);
  a.w1 = nullptr;
  a.expert_bytes = g.hidden * stack_row_bytes(down.quant, g.intermediate);
  a.a = reinterpret_cast<const _Float16*>(b->inter_h);
  a.out = b->partial;
  a.K = (int)g.intermediate;
  a.n_rows = (int)g.hidden;
  if (pc && bm == kPM) XABE_TRY((launch_pc<1>(k, down.quant, a, max_mtiles * (g.hidden / kPR), s)));
  else if (bm == 64) XABE_TRY((launch_mfma<1, true, 64>(k, down.quant, a, max_mtiles * (g.hidden / 128), s)));
  else XABE_TRY((launch_mfma<1, true, 128>(k, down.quant, a, max_mtiles * (g.hidden / 128), s)));
  return XABE_OK;
}

int mfma_shared_expert(const xabe_moe_kernels* k, hipStream_t s, xabe_moe_buffers* b, xabe_quant_tensor gate,
                       xabe_quant_tensor up, xabe_quant_tensor down, const float* x, float* out) {
  const xabe_moe_geometry& g = k->g;
  if (!b->x_h_ready) XABE_TRY(to_f16(k, s, b, x));
  MfmaArgs a;
  memset(&a, 0, sizeof(a));
  a.valid_tokens = b->valid_tokens;
  a.top_k = 1;
  a.w0 = static_cast<const uint8_t*>(gate.bytes);
  a.w1 = static_cast<const uint8_t*>(up.bytes);
  a.a = reinterpret_cast<const _Float16*>(b->x_h);
  a.out = b->shared_inter_h;
  a.K = (int)g.hidden;
  a.n_rows = (int)g.intermediate;
  {
    const size_t row_tiles = g.intermediate / 64;
    const int bm = shared_tile_rows(k, pass_tokens(k, b), row_tiles);
    const size_t items = (g.max_tokens + bm - 1) / bm * row_tiles;
    if (bm == 64) XABE_TRY((launch_mfma<2, false, 64>(k, gate.quant, a, items, s)));
    else XABE_TRY((launch_mfma<2, false, 128>(k, gate.quant, a, items, s)));
  }
  a.w0 = static_cast<const uint8_t*>(down.bytes);
  a.w1 = nullptr;
  a.a = reinterpret_cast<const _Float16*>(b->shared_inter_h);
  a.out = out;
  a.K = (int)g.intermediate;
  a.n_rows = (int)g.hidden;
  {
    const size_t row_tiles = g.hidden / 128;
    const int bm = shared_tile_rows(k, pass_tokens(k, b), row_tiles);
    const size_t items = (g.max_tokens + bm - 1) / bm * row_tiles;
    if (bm == 64) XABE_TRY((launch_mfma<1, false, 64>(k, down.quant, a, items, s)));
    else XABE_TRY((launch_mfma<1, false, 128>(k, down.quant, a, items, s)));
  }
  return XABE_OK;
}

}  // namespace xabe

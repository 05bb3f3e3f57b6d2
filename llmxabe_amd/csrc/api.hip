// C-ABI host side of libxabe_hip: geometry, buffers, routing, dispatch and the
// decode-regime launches.  Mirrors `MoeKernels` and friends
// (crates/xabe-cuda/src/kernels/moe.rs in the reference).
#include <stdio.h>
#include <string.h>

#include <algorithm>

#include "decode_kernels.h"
#include "host_common.h"
#include "small_kernels.h"

namespace xabe {

// ------------------------------------------------------------------ errors
static thread_local char g_err[1024] = "";

int set_error(int status, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return status;
}

int hip_error(hipError_t e, const char* what) {
  // clear the sticky error so that the next call reports its own
  (void)hipGetLastError();
  return set_error(XABE_ERR_DRIVER, "HIP runtime error: %s (%s)", hipGetErrorString(e), what);
}

std::string geometry_debug(const xabe_moe_geometry& g) {
  char buf[256];
  snprintf(buf, sizeof(buf),
           "MoeGeometry { num_experts: %zu, experts_per_token: %zu, hidden: %zu, intermediate: %zu, block_size: %zu, "
           "max_tokens: %zu }",
           g.num_experts, g.experts_per_token, g.hidden, g.intermediate, g.block_size, g.max_tokens);
  return buf;
}

static int bad_geometry(const xabe_moe_geometry& g, const char* reason) {
  return set_error(XABE_ERR_UNSUPPORTED_GEOMETRY, "unsupported MoE geometry %s: %s", geometry_debug(g).c_str(), reason);
}

// ------------------------------------------------------------------ quant helpers
static bool quant_known(int q) { return q >= XABE_QUANT_Q6K && q <= XABE_QUANT_Q5K; }

static int check_stack(const char* which, const xabe_quant_tensor& t, size_t expected) {
  if (!quant_known(t.quant)) return set_error(XABE_ERR_UNSUPPORTED_QUANT, "%s: unknown quantization code %d", which, t.quant);
  const size_t bb = xabe_expert_quant_block_bytes(t.quant);
  if (t.len % bb != 0)
    return set_error(XABE_ERR_RAGGED_WEIGHTS, "%s: %zu bytes is not a whole number of %zu B blocks", which, t.len, bb);
  const size_t found = t.len / bb * xabe_expert_quant_block_elements(t.quant);
  if (found != expected)
    return set_error(XABE_ERR_WRONG_ELEMENT_COUNT, "%s: expected %zu elements for this geometry, stack holds %zu", which,
                     expected, found);
  if (xabe_expert_quant_is_community(t.quant))
    return set_error(XABE_ERR_UNSUPPORTED_QUANT, "%s: community formats (Q4_0/Q4_K/Q5_K) have no kernel in this library",
                     which);
  if (!t.bytes) return set_error(XABE_ERR_INVALID_ARGUMENT, "%s: null device pointer", which);
  if (reinterpret_cast<uintptr_t>(t.bytes) % 16 != 0)
    return set_error(XABE_ERR_INVALID_ARGUMENT, "%s: device pointer must be 16-byte aligned", which);
  return XABE_OK;
}

static int check_len(const char* what, size_t expected, size_t found) {
  if (expected != found)
    return set_error(XABE_ERR_BUFFER_LENGTH, "%s holds %zu elements, expected %zu", what, found, expected);
  return XABE_OK;
}

static int require_routed(const xabe_moe_buffers* b, const char* entry) {
  if (b->scope != XABE_SCOPE_ROUTED)
    return set_error(XABE_ERR_SHARED_ONLY_BUFFERS,
                     "`%s` needs the routed dispatch tables, but these buffers were allocated for the shared-expert path only",
                     entry);
  return XABE_OK;
}

// A contraction of length K in format `quant` needs whole blocks per row.
static int check_contraction(const xabe_moe_geometry& g, int quant, size_t K, const char* which) {
  const size_t be = xabe_expert_quant_block_elements(quant);
  if (K % be != 0) {
    static thread_local char reason[160];
    snprintf(reason, sizeof(reason), "%s: rows of %zu elements are not whole %zu-element blocks", which, K, be);
    return bad_geometry(g, reason);
  }
  return XABE_OK;
}

// ------------------------------------------------------------------ shape dispatch
enum Shape { kRps8, kRps4, kRps2, kKs1, kKs2, kStream };
static Shape shape_for(size_t K) {
  if (K == 256) return kRps8;
  if (K == 512) return kRps4;
  if (K == 1024) return kRps2;
  if (K <= 2048) return kKs1;
  if (K <= 4096) return kKs2;
  return kStream;
}
static int rows_per_step(Shape s) { return s == kRps8 ? 8 : s == kRps4 ? 4 : s == kRps2 ? 2 : 1; }

enum Mode { kFlat, kBlock, kShared };

template <int QUANT, int KS, int RPS, int NM>
static void launch_mode(Mode mode, dim3 grid, hipStream_t s, const ExpertArgs& a) {
  if (mode == kFlat) hipLaunchKernelGGL((k_expert_flat<QUANT, KS, RPS, NM>), grid, dim3(256), 0, s, a);
  else if (mode == kBlock) hipLaunchKernelGGL((k_expert_block<QUANT, KS, RPS, NM>), grid, dim3(256), 0, s, a);
  else hipLaunchKernelGGL((k_expert_shared<QUANT, KS, RPS, NM>), grid, dim3(256), 0, s, a);
}

template <int QUANT, int NM>
static void launch_shape(Shape shape, Mode mode, dim3 grid, hipStream_t s, const ExpertArgs& a) {
  switch (shape) {
    case kRps8: launch_mode<QUANT, 1, 8, NM>(mode, grid, s, a); break;
    case kRps4: launch_mode<QUANT, 1, 4, NM>(mode, grid, s, a); break;
    case kRps2: launch_mode<QUANT, 1, 2, NM>(mode, grid, s, a); break;
    case kKs1: launch_mode<QUANT, 1, 1, NM>(mode, grid, s, a); break;
    case kKs2: launch_mode<QUANT, 2, 1, NM>(mode, grid, s, a); break;
    default: launch_mode<QUANT, 0, 1, NM>(mode, grid, s, a); break;
  }
}

// Dispatch-table regime, rows of one step: the weights-resident kernel where its tile divides the rows.
template <int QUANT, int NM>
static bool launch_block_resident(Shape shape, const ExpertArgs& a, size_t units, hipStream_t s) {
  if (shape == kKs2 || shape == kStream || a.K * rows_per_step(shape) != 2048) return false;
  const int rps = rows_per_step(shape);
  // steps per wavefront: as many as keep the raw bytes of a tile within ~36 registers per lane
  const int want = NM == 2 ? 2 : 4;
  const int depth = a.n_rows % (kWavesPerWg * want * rps) == 0 ? want : a.n_rows % (kWavesPerWg * 2 * rps) == 0 ? 2 : 0;
  if (!depth) return false;
  const unsigned tiles = (unsigned)(a.n_rows / (kWavesPerWg * depth * rps));
  if (tiles > 65535u || units > 65535u) return false;
  dim3 grid(tiles, (unsigned)units);
#define XABE_RESIDENT(RPS)                                                                                         \
  do {                                                                                                             \
    if (depth == 4) hipLaunchKernelGGL((k_expert_block_resident<QUANT, RPS, NM, 4>), grid, dim3(256), 0, s, a);    \
    else hipLaunchKernelGGL((k_expert_block_resident<QUANT, RPS, NM, 2>), grid, dim3(256), 0, s, a);               \
  } while (0)
  switch (shape) {
    case kRps8: XABE_RESIDENT(8); break;
    case kRps4: XABE_RESIDENT(4); break;
    case kRps2: XABE_RESIDENT(2); break;
    default: XABE_RESIDENT(1); break;
  }
#undef XABE_RESIDENT
  return true;
}

constexpr size_t kLongRowsLdsMax = 159 * 1024;  // what a workgroup of the LDS-activation form may ask for
template <int Q, int NM, int R, int TOK, bool RESID>
static bool launch_long_rows_lds(const LongRowArgs& la, dim3 grid, dim3 block, size_t smem, hipStream_t s) {
  hipLaunchKernelGGL((k_shared_long_rows<Q, NM, R, TOK, RESID, true>), grid, block, smem, s, la);
  return true;
}
int long_rows_configure() {
  static bool done = false;  // (one device per process)
  if (done) return XABE_OK;
  const void* fns[2] = {reinterpret_cast<const void*>(k_shared_long_rows<kQ6K, 2, 2, 4, false, true>),
                        reinterpret_cast<const void*>(k_shared_long_rows<kQ8_0, 2, 2, 4, false, true>)};
  for (const void* f : fns)
    XABE_HIP_TRY(hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLongRowsLdsMax));
  const void* staged[8] = {reinterpret_cast<const void*>(k_long_rows_staged<kQ6K, 2, 2, false>),
                           reinterpret_cast<const void*>(k_long_rows_staged<kQ8_0, 2, 2, false>),
                           reinterpret_cast<const void*>(k_long_rows_staged<kQ6K, 2, 1, false>),
                           reinterpret_cast<const void*>(k_long_rows_staged<kQ8_0, 2, 1, false>),
                           reinterpret_cast<const void*>(k_long_rows_staged<kQ6K, 1, 4, false>),
                           reinterpret_cast<const void*>(k_long_rows_staged<kQ8_0, 1, 4, false>),
                           reinterpret_cast<const void*>(k_long_rows_staged<kQ6K, 1, 4, true>),
                           reinterpret_cast<const void*>(k_long_rows_staged<kQ8_0, 1, 4, true>)};
  const void* staged10[4] = {reinterpret_cast<const void*>(k_long_rows_staged<kQ6K, 1, 2, false, 10>),
                             reinterpret_cast<const void*>(k_long_rows_staged<kQ8_0, 1, 2, false, 10>),
                             reinterpret_cast<const void*>(k_long_rows_staged<kQ6K, 1, 2, true, 10>),
                             reinterpret_cast<const void*>(k_long_rows_staged<kQ8_0, 1, 2, true, 10>)};
  for (const void* f : staged10)
    XABE_HIP_TRY(hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kStagedLdsBytes));
  for (const void* f : staged)
    XABE_HIP_TRY(hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kStagedLdsBytes));
  done = true;
  return XABE_OK;
}

// Rows longer than one step, no expert indirection (dense sibling, wide shared experts): the step-outer
// kernel, R rows per wavefront (2 for a gate/up pair, 4 for one matrix).  `la.l_out` set: add the residual
// in the epilogue.
bool launch_long_rows(const xabe_moe_kernels* k, int quant, int nm, const LongRowArgs& la, hipStream_t s) {
  const ExpertArgs& a = la.m;
  if (k->force_community || a.K <= 2048 || !(quant == XABE_QUANT_Q6K || quant == XABE_QUANT_Q8_0)) return false;
  // rows per wavefront: 2 gate/up pairs or 4 single rows (the step's activations are read once for all of
  // them).  Wavefronts are independent, so a matrix with few row groups is launched as one-wavefront
  // workgroups, which spread evenly over the CUs.
  const int tok = k->g.max_tokens == 1 ? 1 : 2;  // tokens per pass over the weights
  const int r = nm == 2 ? 2 : 4;
  if (a.n_rows % (kWavesPerWg * r) != 0) return false;
  const unsigned passes = (unsigned)((k->g.max_tokens + tok - 1) / tok);
  const int groups = a.n_rows / r;
  const unsigned waves = (size_t)groups / kWavesPerWg * passes < (size_t)4 * k->num_cus ? 1 : kWavesPerWg;
  if (groups / waves > 0x7fffffffu / 64) return false;
  dim3 grid((unsigned)groups / waves, passes), block(64 * waves);
  const bool resid = la.l_out != nullptr;
  // the coalesced loader reads whole 16-byte pieces: the tensors must start and end on 16-byte boundaries
  const size_t row_bytes = (size_t)a.K / xabe_expert_quant_block_elements(quant) * xabe_expert_quant_block_bytes(quant);
  auto on16 = [&](const uint8_t* w) { return !w || (reinterpret_cast<uintptr_t>(w) % 16 == 0 && ((size_t)a.n_rows * row_bytes) % 16 == 0); };
  if (!(on16(a.w0) && on16(a.w1))) return false;
  // Five tokens or more: eight tokens per pass, the step's activations staged in LDS for the whole workgroup
  // (k_long_rows_staged); one workgroup of eight wavefronts per CU, persistent over groups of 8 r rows.
  if (k->g.max_tokens >= 5 && a.n_rows % (8 * r) == 0 && a.K % 256 == 0 &&
      (size_t)k->g.max_tokens * (size_t)a.K * sizeof(float) < ((size_t)1 << 32) && reinterpret_cast<uintptr_t>(a.x) % 16 == 0) {
    const unsigned pass8 = (unsigned)((k->g.max_tokens + kStagedTok - 1) / kStagedTok);
    const unsigned groups8 = (unsigned)(a.n_rows / (8 * r));
    dim3 grid8(std::min<unsigned>(groups8, (unsigned)k->num_cus), pass8), block8(512);
    // a single matrix whose groups of 32 rows leave CUs idle while groups of 20 fill them (the dense sibling's down
    // projection: 5120 rows, 160 against 256 groups): ten wavefronts of two rows
    const bool ten = nm == 1 && a.n_rows % 20 == 0 && groups8 < (unsigned)k->num_cus && (unsigned)(a.n_rows / 20) >= groups8 * 3 / 2;
    const dim3 grid10(std::min<unsigned>((unsigned)(a.n_rows / 20), (unsigned)k->num_cus), pass8), block10(640);
    // gate/up whose groups do not divide evenly over the CUs (17408 row pairs: 1088 groups of 16 on 256 CUs, a fifth
    // round for a quarter of them): whole rounds in the main launch, the left-over rows as half-size groups (one row
    // pair per wavefront) spread over twice as many CUs in a second launch
    LongRowArgs la_main = la, la_rest = la;
    unsigned rest_groups = 0;
    if (nm == 2 && groups8 > (unsigned)k->num_cus && groups8 % (unsigned)k->num_cus != 0 &&
        2 * (groups8 % (unsigned)k->num_cus) <= (unsigned)k->num_cus) {
      const unsigned whole = groups8 / (unsigned)k->num_cus * (unsigned)k->num_cus;
      la_main.row_begin = 0;
      la_main.row_end = (int)(whole * 8 * r);
      la_rest.row_begin = la_main.row_end;
      la_rest.row_end = a.n_rows;
      rest_groups = (groups8 - whole) * 2;
    }
#define XABE_STAGED(Q)                                                                                                          \
  do {                                                                                                                          \
    if (nm == 2) {                                                                                                              \
      hipLaunchKernelGGL((k_long_rows_staged<Q, 2, 2, false>), grid8, block8, kStagedLdsBytes, s, la_main);                     \
      if (rest_groups)                                                                                                          \
        hipLaunchKernelGGL((k_long_rows_staged<Q, 2, 1, false>), dim3(rest_groups, pass8), block8, kStagedLdsBytes, s, la_rest); \
    }                                                                                                                           \
    else if (ten && resid) hipLaunchKernelGGL((k_long_rows_staged<Q, 1, 2, true, 10>), grid10, block10, kStagedLdsBytes, s, la); \
    else if (ten) hipLaunchKernelGGL((k_long_rows_staged<Q, 1, 2, false, 10>), grid10, block10, kStagedLdsBytes, s, la);        \
    else if (resid) hipLaunchKernelGGL((k_long_rows_staged<Q, 1, 4, true>), grid8, block8, kStagedLdsBytes, s, la);             \
    else hipLaunchKernelGGL((k_long_rows_staged<Q, 1, 4, false>), grid8, block8, kStagedLdsBytes, s, la);                       \
  } while (0)
    if (quant == XABE_QUANT_Q6K) XABE_STAGED(kQ6K);
    else XABE_STAGED(kQ8_0);
#undef XABE_STAGED
    return true;
  }
  // Three tokens or more, gate/up: four tokens per pass with the activation rows in LDS (the kernel's XLDS form),
  // where four rows and eight wavefronts' staging slots fit; eight wavefronts per workgroup, one workgroup per
  // CU and pass, persistent over the row groups.  (Down's rows are too long for four of them to fit.)
  if (nm == 2 && k->g.max_tokens >= 3 && a.K % 4 == 0) {
    const int tokx = 4;
    const unsigned wv = 8;
    const size_t slot = (size_t)r * nm * (quant == XABE_QUANT_Q6K ? StageFmt<kQ6K>::kSlotBytes : StageFmt<kQ8_0>::kSlotBytes);
    const size_t smem = (size_t)tokx * a.K * sizeof(float) + wv * slot;
    if (smem <= kLongRowsLdsMax) {
      const unsigned passx = (unsigned)((k->g.max_tokens + tokx - 1) / tokx);
      dim3 gridx((unsigned)std::min<size_t>(((size_t)groups + wv - 1) / wv, (size_t)k->num_cus), passx), blockx(64 * wv);
      if (quant == XABE_QUANT_Q6K) return launch_long_rows_lds<kQ6K, 2, 2, 4, false>(la, gridx, blockx, smem, s);
      return launch_long_rows_lds<kQ8_0, 2, 2, 4, false>(la, gridx, blockx, smem, s);
    }
  }
#define XABE_LONG4(Q, TOK, R)                                                                                    \
  do {                                                                                                            \
    if (nm == 2) hipLaunchKernelGGL((k_shared_long_rows<Q, 2, R, TOK, false>), grid, block, 0, s, la);            \
    else if (resid) hipLaunchKernelGGL((k_shared_long_rows<Q, 1, R, TOK, true>), grid, block, 0, s, la);          \
    else hipLaunchKernelGGL((k_shared_long_rows<Q, 1, R, TOK, false>), grid, block, 0, s, la);                    \
  } while (0)
#define XABE_LONG3(Q, TOK)                              \
  do {                                                  \
    if (nm == 2) XABE_LONG4(Q, TOK, 2);                 \
    else XABE_LONG4(Q, TOK, 4);                         \
  } while (0)
#define XABE_LONG(Q)                  \
  do {                                \
    if (tok == 1) XABE_LONG3(Q, 1);   \
    else XABE_LONG3(Q, 2);            \
  } while (0)
  if (quant == XABE_QUANT_Q6K) XABE_LONG(kQ6K);
  else XABE_LONG(kQ8_0);
#undef XABE_LONG4
#undef XABE_LONG3
#undef XABE_LONG
  return true;
}

int pick_tile_rows(const xabe_moe_kernels* k, size_t live_units, int n_rows, int rps) {
  // aim for ~12 wavefronts per CU across the launch
  const size_t items = std::max<size_t>(1, live_units) * (size_t)n_rows / rps;
  const size_t target_waves = (size_t)k->num_cus * 12;
  const size_t per_wave = (items + target_waves - 1) / target_waves;
  size_t pw = 1;
  while (pw < per_wave && pw < 16) pw <<= 1;
  return (int)(pw * kWavesPerWg * rps);
}

// `units`: grid.y work units (pairs, dispatch blocks, token chunks); `live_units`: how many
// of them a typical step actually uses, for sizing the row tile.
static int launch_expert(const xabe_moe_kernels* k, Mode mode, int quant, int nm, ExpertArgs a, size_t units,
                         size_t live_units, hipStream_t s) {
  const Shape shape = shape_for((size_t)a.K);
  const int rps = rows_per_step(shape);
  if (mode == kBlock && !k->force_community) {
    bool done = false;
    if (quant == XABE_QUANT_Q6K) done = nm == 2 ? launch_block_resident<kQ6K, 2>(shape, a, units, s) : launch_block_resident<kQ6K, 1>(shape, a, units, s);
    else if (quant == XABE_QUANT_Q8_0) done = nm == 2 ? launch_block_resident<kQ8_0, 2>(shape, a, units, s) : launch_block_resident<kQ8_0, 1>(shape, a, units, s);
    if (done) {
      XABE_HIP_TRY(hipGetLastError());
      return XABE_OK;
    }
  }
  if (mode == kShared && a.expert_bytes == 0) {
    LongRowArgs la;
    memset(&la, 0, sizeof(la));
    la.m = a;
    if (launch_long_rows(k, quant, nm, la, s)) {
      XABE_HIP_TRY(hipGetLastError());
      return XABE_OK;
    }
  }
  a.tile_rows = pick_tile_rows(k, live_units, a.n_rows, rps);
  const unsigned tiles = (unsigned)((a.n_rows + a.tile_rows - 1) / a.tile_rows);
  if (tiles > 65535) return set_error(XABE_ERR_UNSUPPORTED_GEOMETRY, "row-tile count %u exceeds the grid.y limit", tiles);
  dim3 grid(tiles, (unsigned)units);  // x = row tile (fast), y = unit
  if (units > 65535) {
    return set_error(XABE_ERR_UNSUPPORTED_GEOMETRY, "%zu work units exceed the 65535 grid.y limit of the fp32 regime", units);
  }
  if (quant == XABE_QUANT_Q6K) {
    if (nm == 2) launch_shape<kQ6K, 2>(shape, mode, grid, s, a);
    else launch_shape<kQ6K, 1>(shape, mode, grid, s, a);
  } else if (quant == XABE_QUANT_Q8_0) {
    if (nm == 2) launch_shape<kQ8_0, 2>(shape, mode, grid, s, a);
    else launch_shape<kQ8_0, 1>(shape, mode, grid, s, a);
  } else if (quant < 0 && nm == 1 && mode == kShared) {  // plain fp32 rows
    launch_shape<kF32, 1>(shape, mode, grid, s, a);
  } else {
    return set_error(XABE_ERR_UNSUPPORTED_QUANT, "no kernel for quantization code %d", quant);
  }
  XABE_HIP_TRY(hipGetLastError());
  return XABE_OK;
}

// the reference's checks on a geometry, in its order, with its reasons (kernels/moe.rs:5043-5111)
int validate_geometry(const xabe_moe_geometry& g) {
  if (g.block_size == 0) return bad_geometry(g, "block_size must be non-zero");
  if (g.experts_per_token == 0) return bad_geometry(g, "experts_per_token must be non-zero");
  if (g.experts_per_token > g.num_experts) return bad_geometry(g, "experts_per_token must not exceed num_experts");
  if (g.max_tokens == 0) return bad_geometry(g, "max_tokens must be non-zero");
  if (g.hidden == 0 || g.intermediate == 0) return bad_geometry(g, "hidden and intermediate must be non-zero");
  if (g.hidden % 128 != 0) return bad_geometry(g, "hidden must be a multiple of the 128-element tile");
  if (g.intermediate % 128 != 0) return bad_geometry(g, "intermediate must be a multiple of the 128-element tile");
  if (g.block_size > 64) return bad_geometry(g, "block_size exceeds the slots the tensor-core tile stages");
  if (xabe_moe_geometry_expert_block_capacity(&g) > 65535)
    return bad_geometry(g, "dispatch-block capacity exceeds the 65535 grid.y limit");
  if (g.max_tokens > 65535) return bad_geometry(g, "max_tokens exceeds the 65535 grid limit");
  return XABE_OK;
}

}  // namespace xabe

using namespace xabe;

// ==================================================================== C ABI
// (every function below is declared extern "C" in include/xabe_hip.h)

const char* xabe_last_error(void) { return g_err; }

const char* xabe_status_name(int s) {
  switch (s) {
    case XABE_OK: return "Ok";
    case XABE_ERR_COMPILE: return "Compile";
    case XABE_ERR_DRIVER: return "Driver";
    case XABE_ERR_MMA: return "Mma";
    case XABE_ERR_UNSUPPORTED_GEOMETRY: return "UnsupportedGeometry";
    case XABE_ERR_RAGGED_WEIGHTS: return "RaggedWeights";
    case XABE_ERR_WRONG_ELEMENT_COUNT: return "WrongElementCount";
    case XABE_ERR_TOO_MANY_TOKENS: return "TooManyTokens";
    case XABE_ERR_SHARED_ONLY_BUFFERS: return "SharedOnlyBuffers";
    case XABE_ERR_BUFFER_LENGTH: return "BufferLength";
    case XABE_ERR_INVALID_ARGUMENT: return "InvalidArgument";
    case XABE_ERR_UNSUPPORTED_QUANT: return "UnsupportedExpertType";
    case XABE_ERR_FFN_KIND_MISMATCH: return "FfnKindMismatch";
    case XABE_ERR_MISSING_TENSOR: return "MissingTensor";
    case XABE_ERR_UNSUPPORTED_DENSE_TYPE: return "UnsupportedDenseType";
    case XABE_ERR_SHAPE_MISMATCH: return "ShapeMismatch";
    case XABE_ERR_GGUF_BAD_MAGIC: return "BadMagic";
    case XABE_ERR_GGUF_UNSUPPORTED_VERSION: return "UnsupportedVersion";
    case XABE_ERR_GGUF_UNEXPECTED_EOF: return "UnexpectedEof";
    case XABE_ERR_GGUF_INVALID_UTF8: return "InvalidUtf8";
    case XABE_ERR_GGUF_NEGATIVE_COUNT: return "NegativeCount";
    case XABE_ERR_GGUF_DUPLICATE_KEY: return "DuplicateKey";
    case XABE_ERR_GGUF_UNKNOWN_VALUE_TYPE: return "UnknownValueType";
    case XABE_ERR_GGUF_NESTED_ARRAY: return "NestedArray";
    case XABE_ERR_GGUF_BAD_ALIGNMENT_TYPE: return "BadAlignmentType";
    case XABE_ERR_GGUF_BAD_ALIGNMENT: return "BadAlignment";
    case XABE_ERR_GGUF_TOO_MANY_DIMENSIONS: return "TooManyDimensions";
    case XABE_ERR_GGUF_ZERO_DIMENSION: return "ZeroDimension";
    case XABE_ERR_GGUF_DUPLICATE_TENSOR: return "DuplicateTensor";
    case XABE_ERR_GGUF_UNSUPPORTED_GGML_TYPE: return "UnsupportedGgmlType";
    case XABE_ERR_GGUF_UNALIGNED_ELEMENT_COUNT: return "UnalignedElementCount";
    case XABE_ERR_GGUF_OFFSET_OVERFLOW: return "OffsetOverflow";
    case XABE_ERR_GGUF_TENSOR_OUT_OF_BOUNDS: return "TensorOutOfBounds";
    case XABE_ERR_GGUF_IO: return "Io";
  }
  return "Unknown";
}

const char* xabe_version(void) { return "xabe_hip 0.1 (gfx950)"; }

// ------------------------------------------------------------------ geometry
xabe_moe_geometry xabe_moe_geometry_qwen3_6(size_t block_size, size_t max_tokens) {
  xabe_moe_geometry g = {256, 8, 2048, 512, block_size, max_tokens};
  return g;
}
size_t xabe_moe_geometry_max_flat_pairs(const xabe_moe_geometry* g) { return g->max_tokens * g->experts_per_token; }
size_t xabe_moe_geometry_sorted_capacity(const xabe_moe_geometry* g) {
  const size_t numel = xabe_moe_geometry_max_flat_pairs(g);
  const size_t active = g->num_experts < numel ? g->num_experts : numel;
  const size_t bound = numel + active * (g->block_size - 1);
  return (bound + g->block_size - 1) / g->block_size * g->block_size;
}
size_t xabe_moe_geometry_expert_block_capacity(const xabe_moe_geometry* g) {
  return xabe_moe_geometry_sorted_capacity(g) / g->block_size;
}
size_t xabe_moe_geometry_stack_elements(const xabe_moe_geometry* g) {
  return g->num_experts * g->intermediate * g->hidden;
}
size_t xabe_moe_block_size_for(size_t tokens) { return tokens <= 1152 ? 32 : 64; }

// ------------------------------------------------------------------ quant
size_t xabe_expert_quant_block_elements(int q) {
  switch (q) {
    case XABE_QUANT_Q6K: case XABE_QUANT_Q4K: case XABE_QUANT_Q5K: return 256;
    case XABE_QUANT_Q8_0: case XABE_QUANT_Q4_0: return 32;
  }
  return 0;
}
size_t xabe_expert_quant_file_block_bytes(int q) {
  switch (q) {
    case XABE_QUANT_Q6K: return 210;
    case XABE_QUANT_Q8_0: return 34;
    case XABE_QUANT_Q4_0: return 18;
    case XABE_QUANT_Q4K: return 144;
    case XABE_QUANT_Q5K: return 176;
  }
  return 0;
}
size_t xabe_expert_quant_block_bytes(int q) { return xabe_expert_quant_file_block_bytes(q); }
int xabe_expert_quant_is_community(int q) { return q == XABE_QUANT_Q4_0 || q == XABE_QUANT_Q4K || q == XABE_QUANT_Q5K; }

int xabe_to_device_layout(int quant, const uint8_t* bytes, size_t len, uint8_t* out, size_t* out_len) {
  if (!quant_known(quant)) return set_error(XABE_ERR_UNSUPPORTED_QUANT, "unknown quantization code %d", quant);
  if ((!bytes && len) || !out_len) return set_error(XABE_ERR_INVALID_ARGUMENT, "to_device_layout: null pointer");
  *out_len = len;
  if (out && out != bytes) memcpy(out, bytes, len);
  return XABE_OK;
}

// ------------------------------------------------------------------ MoeKernels
int xabe_moe_kernels_new(const xabe_moe_geometry* geometry, xabe_moe_kernels** out) {
  if (!geometry || !out) return set_error(XABE_ERR_INVALID_ARGUMENT, "MoeKernels::new: null pointer");
  const xabe_moe_geometry g = *geometry;
  XABE_TRY(validate_geometry(g));

  int dev = 0;
  XABE_HIP_TRY(hipGetDevice(&dev));
  hipDeviceProp_t prop;
  XABE_HIP_TRY(hipGetDeviceProperties(&prop, dev));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return set_error(XABE_ERR_COMPILE, "kernel load failed: this library holds gfx950 code only, device %d is %s", dev,
                     prop.gcnArchName);
  // a code object that does not load shows up here rather than at the first launch
  hipFuncAttributes attr;
  hipError_t e = hipFuncGetAttributes(&attr, reinterpret_cast<const void*>(&k_rms_norm_rows));
  if (e != hipSuccess) {
    (void)hipGetLastError();
    return set_error(XABE_ERR_COMPILE, "kernel load failed: %s", hipGetErrorString(e));
  }
  xabe_moe_kernels* k = new xabe_moe_kernels();
  k->g = g;
  k->tensor_cores = true;
  k->exact_regime = false;
  k->force_community = false;
  k->device = dev;
  k->num_cus = prop.multiProcessorCount;
  // everything one-time happens here, none of it on the launch path (launches are captured into graphs)
  int st = mfma_configure();
  if (st == XABE_OK) st = long_rows_configure();
  if (st != XABE_OK) {
    delete k;
    return st;
  }
  *out = k;
  return XABE_OK;
}

void xabe_moe_kernels_free(xabe_moe_kernels* k) { delete k; }

int xabe_moe_kernels_geometry(const xabe_moe_kernels* k, xabe_moe_geometry* out) {
  if (!k || !out) return set_error(XABE_ERR_INVALID_ARGUMENT, "geometry: null pointer");
  *out = k->g;
  return XABE_OK;
}
int xabe_moe_kernels_disable_tensor_cores(xabe_moe_kernels* k) {
  if (!k) return set_error(XABE_ERR_INVALID_ARGUMENT, "disable_tensor_cores: null handle");
  k->tensor_cores = false;
  return XABE_OK;
}
int xabe_moe_kernels_tensor_cores_enabled(const xabe_moe_kernels* k) { return k && k->tensor_cores ? 1 : 0; }
int xabe_moe_kernels_force_community(xabe_moe_kernels* k, int on) {
  if (!k) return set_error(XABE_ERR_INVALID_ARGUMENT, "force_community: null handle");
  k->force_community = on != 0;
  return XABE_OK;
}
int xabe_moe_kernels_set_mfma_form(xabe_moe_kernels* k, int form) {
  if (!k) return set_error(XABE_ERR_INVALID_ARGUMENT, "set_mfma_form: null handle");
  if (form < 0 || form > 2) return set_error(XABE_ERR_INVALID_ARGUMENT, "set_mfma_form: form %d is not 0 (by width), 1 or 2", form);
  k->mfma_form = form;
  return XABE_OK;
}
int xabe_moe_kernels_set_exact_decode_regime(xabe_moe_kernels* k, int on) {
  if (!k) return set_error(XABE_ERR_INVALID_ARGUMENT, "set_exact_decode_regime: null handle");
  k->exact_regime = on != 0;
  return XABE_OK;
}

// ------------------------------------------------------------------ MoeBuffers
template <typename T>
static int alloc_zeros(T** p, size_t n, hipStream_t s, size_t* total) {
  *p = nullptr;
  if (n == 0) return XABE_OK;
  XABE_HIP_TRY(hipMalloc(reinterpret_cast<void**>(p), n * sizeof(T)));
  XABE_HIP_TRY(hipMemsetAsync(*p, 0, n * sizeof(T), s));
  *total += n * sizeof(T);
  return XABE_OK;
}

static int alloc_buffers(const xabe_moe_kernels* k, void* stream, int scope, bool mma, xabe_moe_buffers** out) {
  if (!k || !out) return set_error(XABE_ERR_INVALID_ARGUMENT, "buffers: null pointer");
  const xabe_moe_geometry& g = k->g;
  hipStream_t s = as_stream(stream);
  xabe_moe_buffers* b = new xabe_moe_buffers();
  memset(b, 0, sizeof(*b));
  b->scope = scope;
  b->mma = mma;
  b->g = g;
  const bool routed = scope == XABE_SCOPE_ROUTED;
  const size_t flat = xabe_moe_geometry_max_flat_pairs(&g);
  const size_t sorted = xabe_moe_geometry_sorted_capacity(&g);
  const size_t eb = xabe_moe_geometry_expert_block_capacity(&g);
  b->n_topk = routed ? flat : 0;
  b->n_sorted = routed ? sorted : 0;
  b->n_expert_blocks = routed ? eb : 0;
  b->n_inter = routed ? sorted * g.intermediate : 0;
  b->n_partial = routed ? flat * g.hidden : 0;
  b->n_shared_inter = g.max_tokens * g.intermediate;
  const bool wide = g.max_tokens >= kMfmaMinTokens;
  int st = XABE_OK;
  size_t total = 0;
  auto A = [&](auto** p, size_t n) {
    if (st == XABE_OK) st = alloc_zeros(p, n, s, &total);
  };
  A(&b->topk_ids, b->n_topk);
  A(&b->topk_weights, b->n_topk);
  A(&b->sorted_token_ids, b->n_sorted);
  A(&b->expert_ids, b->n_expert_blocks);
  A(&b->bucket_live, b->n_expert_blocks);
  A(&b->expert_counts, routed ? g.num_experts : 0);
  // the counting-sort form of the dispatch tables, from 8192 selections up
  b->n_align_chunks = (routed && flat >= 8192 && g.num_experts <= 512) ? (flat + 1023) / 1024 : 0;
  A(&b->align_hist, b->n_align_chunks * g.num_experts);
  A(&b->num_tokens_post_pad, routed ? 1 : 0);
  A(&b->valid_tokens, 1);
  A(&b->inter, b->n_inter);
  A(&b->partial, b->n_partial);
  A(&b->shared_inter, b->n_shared_inter);
  // matrix-core staging: only passes wide enough to take that regime pay for it
  A(&b->x_h, (wide && mma) ? g.max_tokens * g.hidden : 0);
  A(&b->inter_h, (wide && mma && routed) ? sorted * g.intermediate : 0);
  A(&b->shared_inter_h, (wide && mma) ? g.max_tokens * g.intermediate : 0);
  b->n_tile_list = (wide && mma && routed) ? 2 * (4 * (eb + 1) + 4) : 0;  // two lists (mfma_grouped_forward_partial)
  A(&b->tile_list, b->n_tile_list);
  b->n_router_partial = (mma && routed && g.max_tokens >= kRouterGemmMinTokens && router_gemm_splits(g) > 1)
                            ? (size_t)router_gemm_splits(g) * g.max_tokens * g.num_experts
                            : 0;
  A(&b->router_partial, b->n_router_partial);
  // decode widths: one arrival counter per token for the seam's tail in the third launch (decode_block.hip)
  b->n_seam_arrivals = (routed && g.max_tokens <= 32) ? g.max_tokens * seam_counter_ints_per_token() : 0;
  A(&b->seam_arrivals, b->n_seam_arrivals);
  b->bytes = total;
  b->valid_published = 0;
  if (st != XABE_OK) {
    xabe_moe_buffers_free(b);
    return st;
  }
  *out = b;
  return XABE_OK;
}

int xabe_moe_buffers_new(const xabe_moe_kernels* k, void* stream, xabe_moe_buffers** out) {
  return alloc_buffers(k, stream, XABE_SCOPE_ROUTED, true, out);
}
int xabe_moe_shared_only_buffers_new(const xabe_moe_kernels* k, void* stream, int mma, xabe_moe_buffers** out) {
  return alloc_buffers(k, stream, XABE_SCOPE_SHARED_ONLY, mma != 0, out);
}
void xabe_moe_buffers_free(xabe_moe_buffers* b) {
  if (!b) return;
  void* ptrs[] = {b->topk_ids, b->topk_weights, b->sorted_token_ids, b->expert_ids, b->bucket_live, b->expert_counts,
                  b->num_tokens_post_pad, b->valid_tokens, b->align_hist, b->inter, b->partial, b->shared_inter, b->x_h, b->inter_h,
                  b->shared_inter_h, b->tile_list, b->router_partial, b->seam_arrivals};
  for (void* p : ptrs)
    if (p) (void)hipFree(p);
  delete b;
}

int xabe_moe_buffers_scope(const xabe_moe_buffers* b) { return b ? b->scope : -1; }
#define XABE_ACCESSOR(name, type, field, count)                                  \
  type* xabe_moe_buffers_##name(const xabe_moe_buffers* b, size_t* len) {        \
    if (!b) { if (len) *len = 0; return nullptr; }                               \
    if (len) *len = (count);                                                     \
    return b->field;                                                             \
  }
XABE_ACCESSOR(topk_ids, int32_t, topk_ids, b->n_topk)
XABE_ACCESSOR(topk_weights, float, topk_weights, b->n_topk)
XABE_ACCESSOR(sorted_token_ids, int32_t, sorted_token_ids, b->n_sorted)
XABE_ACCESSOR(expert_ids, int32_t, expert_ids, b->n_expert_blocks)
XABE_ACCESSOR(bucket_live, int32_t, bucket_live, b->n_expert_blocks)
XABE_ACCESSOR(num_tokens_post_pad, int32_t, num_tokens_post_pad, b->scope == XABE_SCOPE_ROUTED ? 1 : 0)
XABE_ACCESSOR(valid_tokens, int32_t, valid_tokens, 1)
XABE_ACCESSOR(partial, float, partial, b->n_partial)
XABE_ACCESSOR(shared_inter, float, shared_inter, b->n_shared_inter)
size_t xabe_moe_buffers_bytes(const xabe_moe_buffers* b) { return b ? b->bytes : 0; }

int xabe_moe_set_valid_tokens(const xabe_moe_kernels* k, void* stream, xabe_moe_buffers* b, size_t tokens) {
  if (!k || !b) return set_error(XABE_ERR_INVALID_ARGUMENT, "set_valid_tokens: null handle");
  if (tokens > k->g.max_tokens)
    return set_error(XABE_ERR_TOO_MANY_TOKENS, "%zu tokens exceeds the %zu the buffers were sized for", tokens,
                     k->g.max_tokens);
  if (b->valid_published == (int32_t)tokens) return XABE_OK;
  // A change of the count is a host-to-device copy, and a copy recorded into a graph would publish, on every replay,
  // whatever the source holds then.  Like the reference (kernels/moe.rs:5473-5491: "callable outside graph capture"),
  // the count is set before a capture begins; a call that would change it inside one is refused, with nothing recorded.
  // (a query the runtime refuses is read as "not capturing": the copy below then reports what it has to)
  if (stream_capture_id(as_stream(stream)) != 0 && stream_capture_id(as_stream(stream)) != kCaptureUnknown)
    return set_error(XABE_ERR_INVALID_ARGUMENT,
                     "set_valid_tokens: the stream is capturing and the live-token count would change from %d to %zu; "
                     "publish the count before the capture begins",
                     (int)b->valid_published, tokens);
  // the source is a slot the buffers own, so it outlives the copy however the runtime stages it
  b->valid_host = (int32_t)tokens;
  XABE_HIP_TRY(hipMemcpyAsync(b->valid_tokens, &b->valid_host, sizeof(b->valid_host), hipMemcpyHostToDevice, as_stream(stream)));
  b->valid_published = b->valid_host;
  return XABE_OK;
}

// ------------------------------------------------------------------ routing and dispatch
int xabe_moe_route(const xabe_moe_kernels* k, void* stream, xabe_moe_buffers* b, const float* logits, size_t logits_len) {
  if (!k || !b || !logits) return set_error(XABE_ERR_INVALID_ARGUMENT, "route: null pointer");
  XABE_TRY(require_routed(b, "route"));
  const xabe_moe_geometry& g = k->g;
  if (g.num_experts > kRouteMaxExperts)
    return bad_geometry(g, "the routing wavefront holds 8 experts per lane, so at most 512 experts");
  if (g.experts_per_token > 64) return bad_geometry(g, "the routing wavefront keeps one selection per lane, so at most top-64");
  XABE_TRY(check_len("logits", g.max_tokens * g.num_experts, logits_len));
  const unsigned grid = (unsigned)((g.max_tokens + 3) / 4);
  const size_t smem = 4 * g.num_experts * sizeof(float);
  hipLaunchKernelGGL(k_route, dim3(grid), dim3(256), smem, as_stream(stream), logits, b->valid_tokens,
                     (int)g.num_experts, (int)g.experts_per_token, b->topk_ids, b->topk_weights);
  XABE_HIP_TRY(hipGetLastError());
  return XABE_OK;
}

int xabe_moe_build_dispatch(const xabe_moe_kernels* k, void* stream, xabe_moe_buffers* b) {
  if (!k || !b) return set_error(XABE_ERR_INVALID_ARGUMENT, "build_dispatch: null handle");
  XABE_TRY(require_routed(b, "build_dispatch"));
  const xabe_moe_geometry& g = k->g;
  hipStream_t s = as_stream(stream);
  // the matrix-core grouped GEMM's token-tile lists come out of the same launch where one workgroup holds every
  // expert's count and first slot; the heights they were cut for are noted for the launch that reads them
  TileListArgs tl;
  memset(&tl, 0, sizeof(tl));
  b->tiles_bm = b->tiles_bm_up = 0;
  b->tiles_capture = stream_capture_id(s);
  if (b->tiles_capture != 0) b->tiles_graph_owned = true;
  int bm = 0, bm_up = 0, cap = 0;
  const bool lists = mfma_tile_plan(k, b, &bm, &bm_up, &cap) && g.num_experts <= 512;
  if (lists) {
    tl.capacity = cap;
    tl.bm = bm;
    tl.list = b->tile_list;
    tl.bm_b = bm_up != bm ? bm_up : 0;
    tl.list_b = b->tile_list + b->n_tile_list / 2;
  }
  if (b->n_align_chunks) {
    const unsigned chunks = (unsigned)b->n_align_chunks;
    hipLaunchKernelGGL(k_align_hist, dim3(chunks), dim3(256), 0, s, b->topk_ids, b->valid_tokens, (int)g.experts_per_token,
                       (int)g.num_experts, (int)b->n_sorted, (int)b->n_expert_blocks, b->align_hist, b->sorted_token_ids,
                       b->expert_ids, b->bucket_live);
    hipLaunchKernelGGL(k_align_offsets, dim3(1), dim3(512), 0, s, b->valid_tokens, (int)g.experts_per_token,
                       (int)g.num_experts, (int)g.block_size, (int)chunks, (int)b->n_expert_blocks, b->align_hist,
                       b->expert_counts, b->expert_ids, b->bucket_live, b->num_tokens_post_pad, tl);
    hipLaunchKernelGGL(k_align_place, dim3(chunks), dim3(256), 0, s, b->topk_ids, b->valid_tokens, (int)g.experts_per_token,
                       (int)g.num_experts, (int)b->n_sorted, b->align_hist, b->sorted_token_ids);
    XABE_HIP_TRY(hipGetLastError());
    if (lists) b->tiles_bm = bm, b->tiles_bm_up = bm_up;
    return XABE_OK;
  }
  if (g.max_tokens * g.experts_per_token <= (size_t)kAlignFusedMaxSelections && g.num_experts <= 512) {
    hipLaunchKernelGGL(k_align_fused, dim3(1), dim3(1024), 0, s, b->topk_ids, b->valid_tokens, (int)g.experts_per_token,
                       (int)g.num_experts, (int)g.block_size, (int)b->n_sorted, (int)b->n_expert_blocks, b->sorted_token_ids,
                       b->expert_ids, b->bucket_live, b->expert_counts, b->num_tokens_post_pad, tl);
    XABE_HIP_TRY(hipGetLastError());
    if (lists) b->tiles_bm = bm, b->tiles_bm_up = bm_up;
    return XABE_OK;
  }
  hipLaunchKernelGGL(k_align_count, dim3((unsigned)g.num_experts), dim3(256), 0, s, b->topk_ids, b->valid_tokens,
                     (int)g.experts_per_token, (int)b->n_sorted, (int)b->n_expert_blocks, b->sorted_token_ids,
                     b->expert_ids, b->bucket_live, b->expert_counts);
  hipLaunchKernelGGL(k_align_scatter, dim3((unsigned)g.num_experts), dim3(256), 0, s, b->topk_ids, b->valid_tokens,
                     b->expert_counts, (int)g.experts_per_token, (int)g.num_experts, (int)g.block_size, (int)b->n_sorted,
                     (int)b->n_expert_blocks, b->sorted_token_ids, b->expert_ids, b->num_tokens_post_pad, b->bucket_live);
  XABE_HIP_TRY(hipGetLastError());
  return XABE_OK;
}

static bool flat_regime(const xabe_moe_kernels* k) { return k->g.max_tokens <= kFlatMaxTokens || k->exact_regime; }

int xabe_moe_route_and_dispatch(const xabe_moe_kernels* k, void* stream, xabe_moe_buffers* b, const float* logits,
                                size_t logits_len) {
  if (!k || !b) return set_error(XABE_ERR_INVALID_ARGUMENT, "route_and_dispatch: null handle");
  XABE_TRY(require_routed(b, "route_and_dispatch"));
  XABE_TRY(xabe_moe_route(k, stream, b, logits, logits_len));
  if (flat_regime(k)) return XABE_OK;  // the flat kernels read topk_ids directly
  return xabe_moe_build_dispatch(k, stream, b);
}

int xabe::route_planes_and_dispatch(const xabe_moe_kernels* k, void* stream, xabe_moe_buffers* b, float* logits,
                                    size_t logits_len, const float* bias) {
  if (!k || !b || !logits) return set_error(XABE_ERR_INVALID_ARGUMENT, "route: null pointer");
  XABE_TRY(require_routed(b, "route"));
  const xabe_moe_geometry& g = k->g;
  if (g.num_experts > kRouteMaxExperts)
    return bad_geometry(g, "the routing wavefront holds 8 experts per lane, so at most 512 experts");
  if (g.experts_per_token > 64) return bad_geometry(g, "the routing wavefront keeps one selection per lane, so at most top-64");
  XABE_TRY(check_len("logits", g.max_tokens * g.num_experts, logits_len));
  const int splits = router_gemm_splits(g);
  if (!b->router_partial || splits < 2 || splits > 8 || b->n_router_partial < (size_t)splits * g.max_tokens * g.num_experts)
    return set_error(XABE_ERR_INVALID_ARGUMENT, "route: no partial logit planes to route from");
  const unsigned grid = (unsigned)((g.max_tokens + 3) / 4);
  const size_t smem = 4 * g.num_experts * sizeof(float);
  hipLaunchKernelGGL(k_route_planes, dim3(grid), dim3(256), smem, as_stream(stream), b->router_partial,
                     g.max_tokens * g.num_experts, splits, bias, b->valid_tokens, (int)g.num_experts, (int)g.experts_per_token,
                     logits, b->topk_ids, b->topk_weights);
  XABE_HIP_TRY(hipGetLastError());
  if (flat_regime(k)) return XABE_OK;
  return xabe_moe_build_dispatch(k, stream, b);
}

// ------------------------------------------------------------------ expert contractions
static ExpertArgs base_args(const xabe_moe_kernels* k, const xabe_moe_buffers* b) {
  ExpertArgs a;
  memset(&a, 0, sizeof(a));
  a.valid_tokens = b->valid_tokens;
  a.topk_ids = b->topk_ids;
  a.topk_weights = b->topk_weights;
  a.sorted_token_ids = b->sorted_token_ids;
  a.expert_ids = b->expert_ids;
  a.top_k = (int)k->g.experts_per_token;
  a.block_size = (int)k->g.block_size;
  return a;
}

static int check_routed_stacks(const xabe_moe_kernels* k, xabe_quant_tensor gate, xabe_quant_tensor up,
                               xabe_quant_tensor down) {
  const xabe_moe_geometry& g = k->g;
  const size_t stack = xabe_moe_geometry_stack_elements(&g);
  XABE_TRY(check_stack("gate", gate, stack));
  XABE_TRY(check_stack("up", up, stack));
  XABE_TRY(check_stack("down", down, stack));
  if (gate.quant != up.quant)
    return set_error(XABE_ERR_UNSUPPORTED_QUANT,
                     "gate and up stacks differ in format; the reference serves that pair with its community kernels, "
                     "which this library does not have");
  XABE_TRY(check_contraction(g, gate.quant, g.hidden, "gate/up"));
  XABE_TRY(check_contraction(g, down.quant, g.intermediate, "down"));
  return XABE_OK;
}

// stages: bit 0 = gate/up + SwiGLU, bit 1 = down
static int routed_fp32(const xabe_moe_kernels* k, hipStream_t s, xabe_moe_buffers* b, xabe_quant_tensor gate,
                       xabe_quant_tensor up, xabe_quant_tensor down, const float* x, int stages = 3) {
  const xabe_moe_geometry& g = k->g;
  const bool flat = flat_regime(k);
  const size_t units = flat ? xabe_moe_geometry_max_flat_pairs(&g) : b->n_expert_blocks;
  const size_t live = std::min(units, std::min(g.num_experts, xabe_moe_geometry_max_flat_pairs(&g)));
  const size_t expert_elems = g.intermediate * g.hidden;
  ExpertArgs a = base_args(k, b);
  a.w0 = static_cast<const uint8_t*>(gate.bytes);
  a.w1 = static_cast<const uint8_t*>(up.bytes);
  a.expert_bytes = expert_elems / xabe_expert_quant_block_elements(gate.quant) * xabe_expert_quant_block_bytes(gate.quant);
  a.x = x;
  a.out = b->inter;
  a.K = (int)g.hidden;
  a.n_rows = (int)g.intermediate;
  if (stages & 1) XABE_TRY(launch_expert(k, flat ? kFlat : kBlock, gate.quant, 2, a, units, flat ? units : live, s));
  if (!(stages & 2)) return XABE_OK;
  a.w0 = static_cast<const uint8_t*>(down.bytes);
  a.w1 = nullptr;
  a.expert_bytes = expert_elems / xabe_expert_quant_block_elements(down.quant) * xabe_expert_quant_block_bytes(down.quant);
  a.x = b->inter;
  a.out = b->partial;
  a.K = (int)g.intermediate;
  a.n_rows = (int)g.hidden;
  XABE_TRY(launch_expert(k, flat ? kFlat : kBlock, down.quant, 1, a, units, flat ? units : live, s));
  return XABE_OK;
}

int xabe_moe_grouped_forward_partial(const xabe_moe_kernels* k, void* stream, xabe_moe_buffers* b, xabe_quant_tensor gate,
                                     xabe_quant_tensor up, xabe_quant_tensor down, const float* hidden_states,
                                     size_t hidden_states_len) {
  if (!k || !b || !hidden_states) return set_error(XABE_ERR_INVALID_ARGUMENT, "grouped_forward_partial: null pointer");
  XABE_TRY(require_routed(b, "grouped_forward_partial"));
  XABE_TRY(check_routed_stacks(k, gate, up, down));
  XABE_TRY(check_len("hidden_states", k->g.max_tokens * k->g.hidden, hidden_states_len));
  if (!flat_regime(k) && mfma_supported(k, b, gate.quant, up.quant, down.quant, true))
    return mfma_grouped_forward_partial(k, as_stream(stream), b, gate, up, down, hidden_states);
  return routed_fp32(k, as_stream(stream), b, gate, up, down, hidden_states);
}

int xabe_moe_grouped_forward_stage(const xabe_moe_kernels* k, void* stream, xabe_moe_buffers* b, xabe_quant_tensor gate,
                                   xabe_quant_tensor up, xabe_quant_tensor down, const float* hidden_states,
                                   size_t hidden_states_len, int stage) {
  if (!k || !b || !hidden_states) return set_error(XABE_ERR_INVALID_ARGUMENT, "grouped_forward_stage: null pointer");
  if (stage != 0 && stage != 1) return set_error(XABE_ERR_INVALID_ARGUMENT, "grouped_forward_stage: stage must be 0 or 1");
  XABE_TRY(require_routed(b, "grouped_forward_stage"));
  XABE_TRY(check_routed_stacks(k, gate, up, down));
  XABE_TRY(check_len("hidden_states", k->g.max_tokens * k->g.hidden, hidden_states_len));
  if (!flat_regime(k) && mfma_supported(k, b, gate.quant, up.quant, down.quant, true))
    return set_error(XABE_ERR_MMA, "grouped_forward_stage: the matrix-core regime has no separable stages");
  return routed_fp32(k, as_stream(stream), b, gate, up, down, hidden_states, stage == 0 ? 1 : 2);
}

static int check_shared_stacks(const xabe_moe_kernels* k, xabe_quant_tensor gate, xabe_quant_tensor up,
                               xabe_quant_tensor down) {
  const xabe_moe_geometry& g = k->g;
  const size_t one = g.intermediate * g.hidden;
  XABE_TRY(check_stack("shared gate", gate, one));
  XABE_TRY(check_stack("shared up", up, one));
  XABE_TRY(check_stack("shared down", down, one));
  if (gate.quant != up.quant)
    return set_error(XABE_ERR_UNSUPPORTED_QUANT, "shared gate and up differ in format; no kernel serves that pair here");
  XABE_TRY(check_contraction(g, gate.quant, g.hidden, "shared gate/up"));
  XABE_TRY(check_contraction(g, down.quant, g.intermediate, "shared down"));
  return XABE_OK;
}

int xabe::check_layer_stacks(const xabe_moe_kernels* k, const xabe_moe_layer_weights* w) {
  XABE_TRY(check_routed_stacks(k, w->gate_exps, w->up_exps, w->down_exps));
  XABE_TRY(check_shared_stacks(k, w->shared_gate, w->shared_up, w->shared_down));
  if (!w->router || !w->post_norm || !w->shared_gate_inp)
    return set_error(XABE_ERR_INVALID_ARGUMENT, "layer weights: null router, norm or shared-gate pointer");
  if (reinterpret_cast<uintptr_t>(w->router) % 16 != 0)
    return set_error(XABE_ERR_INVALID_ARGUMENT, "router: device pointer must be 16-byte aligned");
  return XABE_OK;
}

static int shared_fp32(const xabe_moe_kernels* k, hipStream_t s, xabe_moe_buffers* b, xabe_quant_tensor gate,
                       xabe_quant_tensor up, xabe_quant_tensor down, const float* x, float* out) {
  const xabe_moe_geometry& g = k->g;
  const size_t units = (g.max_tokens + 1) / 2;
  ExpertArgs a = base_args(k, b);
  a.w0 = static_cast<const uint8_t*>(gate.bytes);
  a.w1 = static_cast<const uint8_t*>(up.bytes);
  a.expert_bytes = 0;
  a.x = x;
  a.out = b->shared_inter;
  a.K = (int)g.hidden;
  a.n_rows = (int)g.intermediate;
  XABE_TRY(launch_expert(k, kShared, gate.quant, 2, a, units, units, s));
  a.w0 = static_cast<const uint8_t*>(down.bytes);
  a.w1 = nullptr;
  a.x = b->shared_inter;
  a.out = out;
  a.K = (int)g.intermediate;
  a.n_rows = (int)g.hidden;
  XABE_TRY(launch_expert(k, kShared, down.quant, 1, a, units, units, s));
  return XABE_OK;
}

// The dense block's fp32 path on the long-row kernel, the residual folded into down: three launches.
// Returns false (nothing launched) where the long-row kernel does not apply.
static int check_shared_stacks(const xabe_moe_kernels* k, xabe_quant_tensor gate, xabe_quant_tensor up,
                               xabe_quant_tensor down);

int xabe::dense_fp32_fused(const xabe_moe_kernels* k, hipStream_t s, xabe_moe_buffers* b, xabe_quant_tensor gate,
                           xabe_quant_tensor up, xabe_quant_tensor down, const float* post_norm, float eps,
                           const float* residual, float* normed, float* ffn_out, float* l_out, bool* launched) {
  const xabe_moe_geometry& g = k->g;
  *launched = false;
  XABE_TRY(check_shared_stacks(k, gate, up, down));  // the checks xabe_moe_shared_expert makes
  LongRowArgs la;
  memset(&la, 0, sizeof(la));
  la.m = base_args(k, b);
  la.m.w0 = static_cast<const uint8_t*>(gate.bytes);
  la.m.w1 = static_cast<const uint8_t*>(up.bytes);
  // (normalising on load was tried: with thousands of wavefronts each re-deriving the RMS scale of every
  // token it costs more than the stand-alone RMSNorm launch it saves)
  XABE_TRY(xabe_rms_norm(s, residual, g.max_tokens * g.hidden, post_norm, g.hidden, normed, g.max_tokens * g.hidden,
                         g.max_tokens, g.hidden, eps));
  la.m.x = normed;
  la.m.out = b->shared_inter;
  la.m.K = (int)g.hidden;
  la.m.n_rows = (int)g.intermediate;
  LongRowArgs ld;
  memset(&ld, 0, sizeof(ld));
  ld.m = base_args(k, b);
  ld.m.w0 = static_cast<const uint8_t*>(down.bytes);
  ld.m.x = b->shared_inter;
  ld.m.out = ffn_out;
  ld.m.K = (int)g.intermediate;
  ld.m.n_rows = (int)g.hidden;
  ld.residual = residual;
  ld.l_out = l_out;
  // both or neither: check the second shape before launching the first
  const int r_up = 2, r_down = 4;
  if (k->force_community || g.hidden <= 2048 || g.intermediate <= 2048) return XABE_OK;
  if (g.intermediate % (kWavesPerWg * r_up) != 0 || g.hidden % (kWavesPerWg * r_down) != 0) return XABE_OK;
  auto ok = [](int q) { return q == XABE_QUANT_Q6K || q == XABE_QUANT_Q8_0; };
  if (!ok(gate.quant) || !ok(down.quant)) return XABE_OK;
  if (!launch_long_rows(k, gate.quant, 2, la, s) || !launch_long_rows(k, down.quant, 1, ld, s))
    return set_error(XABE_ERR_UNSUPPORTED_GEOMETRY, "dense block: the long-row kernel refused a shape it was checked for");
  XABE_HIP_TRY(hipGetLastError());
  *launched = true;
  return XABE_OK;
}

int xabe_moe_shared_expert(const xabe_moe_kernels* k, void* stream, xabe_moe_buffers* b, xabe_quant_tensor gate,
                           xabe_quant_tensor up, xabe_quant_tensor down, const float* hidden_states,
                           size_t hidden_states_len, float* out, size_t out_len) {
  if (!k || !b || !hidden_states || !out) return set_error(XABE_ERR_INVALID_ARGUMENT, "shared_expert: null pointer");
  XABE_TRY(check_shared_stacks(k, gate, up, down));
  XABE_TRY(check_len("hidden_states", k->g.max_tokens * k->g.hidden, hidden_states_len));
  XABE_TRY(check_len("out", k->g.max_tokens * k->g.hidden, out_len));
  return shared_fp32(k, as_stream(stream), b, gate, up, down, hidden_states, out);
}

int xabe_moe_shared_expert_mma(const xabe_moe_kernels* k, void* stream, xabe_moe_buffers* b, xabe_quant_tensor gate,
                               xabe_quant_tensor up, xabe_quant_tensor down, const float* hidden_states,
                               size_t hidden_states_len, float* out, size_t out_len) {
  if (!k || !b || !hidden_states || !out) return set_error(XABE_ERR_INVALID_ARGUMENT, "shared_expert_mma: null pointer");
  XABE_TRY(check_shared_stacks(k, gate, up, down));
  XABE_TRY(check_len("hidden_states", k->g.max_tokens * k->g.hidden, hidden_states_len));
  XABE_TRY(check_len("out", k->g.max_tokens * k->g.hidden, out_len));
  if (!k->tensor_cores)
    return set_error(XABE_ERR_UNSUPPORTED_GEOMETRY, "unsupported MoE geometry %s: the matrix cores are disabled on this instance",
                     geometry_debug(k->g).c_str());
  if (!mfma_supported(k, b, gate.quant, up.quant, down.quant, false))
    return set_error(XABE_ERR_MMA, "the matrix-core path needs buffers allocated with mma staging and max_tokens >= %zu",
                     kMfmaMinTokens);
  return mfma_shared_expert(k, as_stream(stream), b, gate, up, down, hidden_states, out);
}

int xabe_moe_grouped_forward_partial_with_shared(const xabe_moe_kernels* k, void* stream, xabe_moe_buffers* b,
                                                 xabe_quant_tensor gate, xabe_quant_tensor up, xabe_quant_tensor down,
                                                 xabe_quant_tensor shared_gate, xabe_quant_tensor shared_up,
                                                 xabe_quant_tensor shared_down, const float* hidden_states,
                                                 size_t hidden_states_len, float* out, size_t out_len, int* fused) {
  if (!k || !b || !hidden_states || !out || !fused)
    return set_error(XABE_ERR_INVALID_ARGUMENT, "grouped_forward_partial_with_shared: null pointer");
  XABE_TRY(require_routed(b, "grouped_forward_partial_with_shared"));
  *fused = 0;
  const xabe_moe_geometry& g = k->g;
  // covered: decode width, tuned formats on both sides (kernels/moe.rs:6204-6220)
  const bool covered = g.max_tokens <= kFlatMaxTokens && !k->force_community && gate.quant == up.quant &&
                       !xabe_expert_quant_is_community(gate.quant) && !xabe_expert_quant_is_community(down.quant) &&
                       shared_gate.quant == shared_up.quant && !xabe_expert_quant_is_community(shared_gate.quant) &&
                       !xabe_expert_quant_is_community(shared_down.quant);
  if (!covered) return XABE_OK;
  XABE_TRY(check_routed_stacks(k, gate, up, down));
  XABE_TRY(check_shared_stacks(k, shared_gate, shared_up, shared_down));
  XABE_TRY(check_len("hidden_states", g.max_tokens * g.hidden, hidden_states_len));
  XABE_TRY(check_len("out", g.max_tokens * g.hidden, out_len));
  // The shared expert's units ride the routed grid: two launches instead of four.  Same bodies as the
  // separate entry points, so the outputs are bit-identical to them.
  {
    const size_t expert_elems = g.intermediate * g.hidden;
    hipStream_t s = as_stream(stream);
    const size_t gate_eb = expert_elems / xabe_expert_quant_block_elements(gate.quant) * xabe_expert_quant_block_bytes(gate.quant);
    const size_t down_eb = expert_elems / xabe_expert_quant_block_elements(down.quant) * xabe_expert_quant_block_bytes(down.quant);
    XABE_TRY(launch_flat_with_shared(k, s, b, 2, gate.quant, shared_gate.quant, gate.bytes, up.bytes, gate_eb, hidden_states,
                                     b->inter, shared_gate.bytes, shared_up.bytes, hidden_states, b->shared_inter,
                                     (int)g.hidden, (int)g.intermediate));
    XABE_TRY(launch_flat_with_shared(k, s, b, 1, down.quant, shared_down.quant, down.bytes, nullptr, down_eb, b->inter,
                                     b->partial, shared_down.bytes, nullptr, b->shared_inter, out, (int)g.intermediate,
                                     (int)g.hidden));
  }
  *fused = 1;
  return XABE_OK;
}

int xabe_moe_grouped_forward(const xabe_moe_kernels* k, void* stream, xabe_moe_buffers* b, xabe_quant_tensor gate,
                             xabe_quant_tensor up, xabe_quant_tensor down, const float* hidden_states,
                             size_t hidden_states_len, float* out, size_t out_len) {
  if (!k || !b || !out) return set_error(XABE_ERR_INVALID_ARGUMENT, "grouped_forward: null pointer");
  XABE_TRY(require_routed(b, "grouped_forward"));
  XABE_TRY(check_len("out", k->g.max_tokens * k->g.hidden, out_len));
  XABE_TRY(xabe_moe_grouped_forward_partial(k, stream, b, gate, up, down, hidden_states, hidden_states_len));
  const xabe_moe_geometry& g = k->g;
  dim3 grid((unsigned)g.max_tokens, (unsigned)((g.hidden + 255) / 256));
  hipLaunchKernelGGL(k_moe_reduce, grid, dim3(256), 0, as_stream(stream), b->partial, b->valid_tokens,
                     (int)g.experts_per_token, (int)g.hidden, out);
  XABE_HIP_TRY(hipGetLastError());
  return XABE_OK;
}

// ------------------------------------------------------------------ glue kernels
int xabe_rms_norm(void* stream, const float* x, size_t x_len, const float* weight, size_t weight_len, float* out,
                  size_t out_len, size_t rows, size_t width, float eps) {
  if (!x || !weight || !out) return set_error(XABE_ERR_INVALID_ARGUMENT, "rms_norm: null pointer");
  XABE_TRY(check_len("x", rows * width, x_len));
  XABE_TRY(check_len("weight", width, weight_len));
  XABE_TRY(check_len("out", rows * width, out_len));
  if (rows == 0 || width == 0) return XABE_OK;
  if (width % 4 != 0) return set_error(XABE_ERR_INVALID_ARGUMENT, "rms_norm: width %zu is not a multiple of 4", width);
  if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(weight) | reinterpret_cast<uintptr_t>(out)) % 16 != 0)
    return set_error(XABE_ERR_INVALID_ARGUMENT, "rms_norm: x, weight and out must be 16-byte aligned");
  if (width <= 2048 && rows >= 64)  // (a handful of rows: one workgroup per row finishes sooner)
    hipLaunchKernelGGL(k_rms_norm_short_rows<false>, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, as_stream(stream), x, weight, out,
                       static_cast<_Float16*>(nullptr), (int)rows, (int)width, eps);
  else
    hipLaunchKernelGGL(k_rms_norm_rows, dim3((unsigned)rows), dim3(256), 0, as_stream(stream), x, weight, out, (int)width, eps);
  XABE_HIP_TRY(hipGetLastError());
  return XABE_OK;
}

int xabe::rms_norm_rows_with_f16(void* stream, const float* x, const float* weight, float* out, void* out_h, size_t rows,
                                 size_t width, float eps, bool* done) {
  *done = false;
  if (!out_h || width > 2048 || width % 4 != 0 || rows < 64) return XABE_OK;
  if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(weight) | reinterpret_cast<uintptr_t>(out) |
       reinterpret_cast<uintptr_t>(out_h)) % 16 != 0)
    return XABE_OK;
  hipLaunchKernelGGL(k_rms_norm_short_rows<true>, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, as_stream(stream), x, weight, out,
                     static_cast<_Float16*>(out_h), (int)rows, (int)width, eps);
  XABE_HIP_TRY(hipGetLastError());
  *done = true;
  return XABE_OK;
}

int xabe_moe_router_logits(const xabe_moe_kernels* k, void* stream, const xabe_moe_buffers* b, const void* router,
                           size_t router_len, int router_quant, const float* normed, size_t normed_len, float* logits,
                           size_t logits_len) {
  return router_logits_biased(k, stream, b, router, router_len, router_quant, normed, normed_len, logits, logits_len, nullptr,
                              nullptr);
}

int xabe::router_logits_biased(const xabe_moe_kernels* k, void* stream, const xabe_moe_buffers* b, const void* router,
                               size_t router_len, int router_quant, const float* normed, size_t normed_len, float* logits,
                               size_t logits_len, const float* bias, bool* bias_added, bool* sum_deferred) {
  if (bias_added) *bias_added = false;
  if (sum_deferred) *sum_deferred = false;
  if (!k || !b || !router || !normed || !logits) return set_error(XABE_ERR_INVALID_ARGUMENT, "router_logits: null pointer");
  const xabe_moe_geometry& g = k->g;
  const size_t elems = g.num_experts * g.hidden;
  int fmt;
  if (router_quant < 0) {
    XABE_TRY(check_len("router", elems, router_len));
    fmt = -1;
  } else if (router_quant == XABE_QUANT_Q8_0) {
    xabe_quant_tensor t = {router, router_len, router_quant};
    XABE_TRY(check_stack("router", t, elems));
    XABE_TRY(check_contraction(g, router_quant, g.hidden, "router"));
    fmt = XABE_QUANT_Q8_0;
  } else {
    return set_error(XABE_ERR_UNSUPPORTED_QUANT, "router: only f32 and Q8_0 routers are supported, got code %d", router_quant);
  }
  XABE_TRY(check_len("normed", g.max_tokens * g.hidden, normed_len));
  XABE_TRY(check_len("logits", g.max_tokens * g.num_experts, logits_len));
  if (router_gemm_supported(k, b, fmt))
    return launch_router_gemm(k, as_stream(stream), b, router, fmt, normed, logits, bias, bias_added, sum_deferred);
  ExpertArgs a = base_args(k, b);
  a.w0 = static_cast<const uint8_t*>(router);
  a.x = normed;
  a.out = logits;
  a.K = (int)g.hidden;
  a.n_rows = (int)g.num_experts;
  const size_t units = (g.max_tokens + 1) / 2;
  return launch_expert(k, kShared, fmt, 1, a, units, units, as_stream(stream));
}

int xabe_moe_gate_and_combine(const xabe_moe_kernels* k, void* stream, const xabe_moe_buffers* b,
                              const float* shared_gate_inp, const float* normed, const float* shexp,
                              const float* residual, float* gate, float* routed, float* ffn_out, float* l_out) {
  if (!k || !b || !shared_gate_inp || !normed || !shexp || !residual || !gate || !routed || !ffn_out || !l_out)
    return set_error(XABE_ERR_INVALID_ARGUMENT, "gate_and_combine: null pointer");
  XABE_TRY(require_routed(b, "gate_and_combine"));
  const xabe_moe_geometry& g = k->g;
  dim3 grid((unsigned)g.max_tokens, (unsigned)((g.hidden + 1023) / 1024));
  hipLaunchKernelGGL(k_gate_and_combine, grid, dim3(256), 0, as_stream(stream), shared_gate_inp, normed, b->partial, shexp,
                     residual, b->valid_tokens, (int)g.experts_per_token, (int)g.hidden, gate, routed, ffn_out, l_out);
  XABE_HIP_TRY(hipGetLastError());
  return XABE_OK;
}

int xabe_moe_gate_and_combine_seam(const xabe_moe_kernels* k, void* stream, const xabe_moe_buffers* b,
                                   const float* shared_gate_inp, const float* normed, const float* shexp,
                                   const float* residual, float* gate, float* routed, float* ffn_out, float* l_out,
                                   const float* next_norm_weight, float next_eps, float* next_normed, void* next_normed_h) {
  if (!k || !b || !shared_gate_inp || !normed || !shexp || !residual || !gate || !l_out)
    return set_error(XABE_ERR_INVALID_ARGUMENT, "gate_and_combine_seam: null pointer");
  XABE_TRY(require_routed(b, "gate_and_combine_seam"));
  const xabe_moe_geometry& g = k->g;
  if (g.hidden > 2048)
    return set_error(XABE_ERR_UNSUPPORTED_GEOMETRY, "gate_and_combine_seam: rows of %zu elements; the one-workgroup-per-row combine serves at most 2048", g.hidden);
  if (next_norm_weight && !next_normed)
    return set_error(XABE_ERR_INVALID_ARGUMENT, "gate_and_combine_seam: a norm weight for the next layer but nowhere to write its rows");
  const uintptr_t align = reinterpret_cast<uintptr_t>(normed) | reinterpret_cast<uintptr_t>(shexp) | reinterpret_cast<uintptr_t>(residual) |
                          reinterpret_cast<uintptr_t>(routed) | reinterpret_cast<uintptr_t>(ffn_out) | reinterpret_cast<uintptr_t>(l_out) |
                          reinterpret_cast<uintptr_t>(next_norm_weight) | reinterpret_cast<uintptr_t>(next_normed) |
                          reinterpret_cast<uintptr_t>(next_normed_h);
  if (align % 16 != 0) return set_error(XABE_ERR_INVALID_ARGUMENT, "gate_and_combine_seam: tensors must be 16-byte aligned");
  const dim3 grid((unsigned)g.max_tokens);
  hipStream_t s = as_stream(stream);
  _Float16* nh = static_cast<_Float16*>(next_normed_h);
#define XABE_COMBINE(NORM, WITH_H)                                                                                          \
  hipLaunchKernelGGL((k_combine_rows<NORM, WITH_H>), grid, dim3(256), 0, s, shared_gate_inp, normed, b->partial, shexp,     \
                     residual, b->valid_tokens, (int)g.experts_per_token, (int)g.hidden, gate, routed, ffn_out, l_out,        \
                     next_norm_weight, next_eps, next_normed, nh)
  if (!next_norm_weight) XABE_COMBINE(false, false);
  else if (nh) XABE_COMBINE(true, true);
  else XABE_COMBINE(true, false);
#undef XABE_COMBINE
  XABE_HIP_TRY(hipGetLastError());
  return XABE_OK;
}

int xabe_dense_ffn_add_residual(const xabe_moe_kernels* k, void* stream, const xabe_moe_buffers* b, const float* ffn_out,
                                const float* residual, float* l_out) {
  if (!k || !b || !ffn_out || !residual || !l_out)
    return set_error(XABE_ERR_INVALID_ARGUMENT, "dense_ffn_add_residual: null pointer");
  const xabe_moe_geometry& g = k->g;
  dim3 grid((unsigned)g.max_tokens, (unsigned)((g.hidden + 255) / 256));
  hipLaunchKernelGGL(k_add_residual, grid, dim3(256), 0, as_stream(stream), ffn_out, residual, b->valid_tokens,
                     (int)g.hidden, l_out);
  XABE_HIP_TRY(hipGetLastError());
  return XABE_OK;
}

int xabe_moe_add_logit_bias(const xabe_moe_kernels* k, void* stream, const xabe_moe_buffers* b, const float* bias,
                            float* logits) {
  if (!k || !b || !bias || !logits) return set_error(XABE_ERR_INVALID_ARGUMENT, "add_logit_bias: null pointer");
  hipLaunchKernelGGL(k_add_logit_bias, dim3((unsigned)k->g.max_tokens), dim3(256), 0, as_stream(stream), bias,
                     b->valid_tokens, (int)k->g.num_experts, logits);
  XABE_HIP_TRY(hipGetLastError());
  return XABE_OK;
}

int xabe_dequantize(void* stream, int quant, const void* bytes, size_t len, float* out, size_t out_len) {
  if (!bytes || !out) return set_error(XABE_ERR_INVALID_ARGUMENT, "dequantize: null pointer");
  if (quant != XABE_QUANT_Q6K && quant != XABE_QUANT_Q8_0)
    return set_error(XABE_ERR_UNSUPPORTED_QUANT, "dequantize: no kernel for quantization code %d", quant);
  const size_t bb = xabe_expert_quant_block_bytes(quant);
  if (len % bb != 0)
    return set_error(XABE_ERR_RAGGED_WEIGHTS, "dequantize: %zu bytes is not a whole number of %zu B blocks", len, bb);
  const size_t n = len / bb * xabe_expert_quant_block_elements(quant);
  XABE_TRY(check_len("out", n, out_len));
  if (n == 0) return XABE_OK;
  const unsigned grid = (unsigned)((n + 255) / 256);
  if (quant == XABE_QUANT_Q6K)
    hipLaunchKernelGGL(k_dequant_q6k, dim3(grid), dim3(256), 0, as_stream(stream), static_cast<const uint8_t*>(bytes), n, out);
  else
    hipLaunchKernelGGL(k_dequant_q8_0, dim3(grid), dim3(256), 0, as_stream(stream), static_cast<const uint8_t*>(bytes), n, out);
  XABE_HIP_TRY(hipGetLastError());
  return XABE_OK;
}

int xabe_mma_quantize_rows(void* stream, const float* x, size_t x_len, int8_t* q, size_t q_len, float* scales,
                           size_t scales_len, size_t rows, size_t k) {
  if (!x || !q || !scales) return set_error(XABE_ERR_INVALID_ARGUMENT, "quantize_rows: null pointer");
  if (k % 32 != 0)
    return set_error(XABE_ERR_MMA, "contraction length %zu is not a multiple of 32, the elements one scale covers", k);
  // (at least, as the reference checks them: a caller may quantise the live rows of a larger buffer)
  const struct { const char* what; size_t have, need; } lens[] = {
      {"quantize x", x_len, rows * k}, {"quantize q", q_len, rows * k}, {"quantize scales", scales_len, rows * k / 32}};
  for (const auto& l : lens)
    if (l.have < l.need)
      return set_error(XABE_ERR_BUFFER_LENGTH, "%s holds %zu elements, the shape implies %zu", l.what, l.have, l.need);
  const size_t n_blocks = rows * k / 32;
  if (n_blocks == 0) return XABE_OK;
  hipLaunchKernelGGL(k_quantize_rows_q8, dim3((unsigned)((n_blocks + 7) / 8)), dim3(256), 0, as_stream(stream), x, n_blocks, q,
                     scales);
  XABE_HIP_TRY(hipGetLastError());
  return XABE_OK;
}

// ------------------------------------------------------------------ synthetic stacks
int xabe_synth_normal_f32(void* stream, uint64_t seed, size_t n, float sigma, float* out) {
  if (!out) return set_error(XABE_ERR_INVALID_ARGUMENT, "synth_normal_f32: null pointer");
  if (n == 0) return XABE_OK;
  const size_t chunks = (n + 255) / 256;
  hipLaunchKernelGGL(k_synth_f32, dim3((unsigned)((chunks + 63) / 64)), dim3(64), 0, as_stream(stream), seed, n, sigma, out);
  XABE_HIP_TRY(hipGetLastError());
  return XABE_OK;
}

int xabe_synth_quant(void* stream, int quant, uint64_t seed, size_t n_elements, float sigma, void* out, size_t out_len) {
  if (!out) return set_error(XABE_ERR_INVALID_ARGUMENT, "synth_quant: null pointer");
  if (quant != XABE_QUANT_Q6K && quant != XABE_QUANT_Q8_0)
    return set_error(XABE_ERR_UNSUPPORTED_QUANT, "synth_quant: no generator for quantization code %d", quant);
  if (n_elements % 256 != 0)
    return set_error(XABE_ERR_RAGGED_WEIGHTS, "synth_quant: %zu elements is not a whole number of 256-element chunks", n_elements);
  const size_t need = n_elements / xabe_expert_quant_block_elements(quant) * xabe_expert_quant_block_bytes(quant);
  XABE_TRY(check_len("out", need, out_len));
  const size_t chunks = n_elements / 256;
  if (chunks == 0) return XABE_OK;
  const unsigned grid = (unsigned)((chunks + 63) / 64);
  if (quant == XABE_QUANT_Q6K)
    hipLaunchKernelGGL(k_synth_q6k, dim3(grid), dim3(64), 0, as_stream(stream), seed, chunks, sigma, static_cast<uint8_t*>(out));
  else
    hipLaunchKernelGGL(k_synth_q8_0, dim3(grid), dim3(64), 0, as_stream(stream), seed, chunks, sigma, static_cast<uint8_t*>(out));
  XABE_HIP_TRY(hipGetLastError());
  return XABE_OK;
}

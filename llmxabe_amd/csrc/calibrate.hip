// What the part can do, measured the way the reference measures its card (a pure coalesced 16-byte-per-lane
// read with a sink the compiler cannot prove dead, crates/xabe-cuda/src/bin/bench_dense_ffn.rs:88-111; a
// register-resident matrix-instruction loop, docs/BENCHMARKS.md:1022-1024): the figures reported beside
// the nominal 8 TB/s and 2.5 PFLOP/s.  One launch per call on the caller's stream; the caller times it.
#include "device_common.h"
#include "host_common.h"

namespace xabe {

typedef _Float16 cal_half8 __attribute__((ext_vector_type(8)));
typedef float cal_float16 __attribute__((ext_vector_type(16)));

// Every 16-byte piece of [p, p + n16) read once; four pieces per lane in flight.
__global__ void __launch_bounds__(256) k_calibrate_read(const uint4* __restrict__ p, size_t n16, uint32_t* __restrict__ sink) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  uint32_t acc = 0;
  for (; i + 3 * stride < n16; i += 4 * stride) {
    uint4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) v[u] = p[i + u * stride];
#pragma unroll
    for (int u = 0; u < 4; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  }
  for (; i < n16; i += stride) {
    const uint4 v = p[i];
    acc ^= v.x ^ v.y ^ v.z ^ v.w;
  }
  if (acc == 0x12345678u) sink[0] = acc;  // (never true for the caller's data: keeps the loads)
}

// `iters` rounds of eight independent 32x32x16 fp16 matrix instructions per wavefront, operands in registers.
__global__ void __launch_bounds__(256) k_calibrate_mfma(float* __restrict__ out, int iters) {
  cal_half8 a, b;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = (_Float16)(float)((threadIdx.x + i) & 7);
    b[i] = (_Float16)(float)(i & 3);
  }
  cal_float16 acc[8];
#pragma unroll
  for (int j = 0; j < 8; ++j)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[j][v] = 0.0f;
  for (int i = 0; i < iters; ++i) {
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[j], 0, 0, 0);
  }
  float s = 0.0f;
#pragma unroll
  for (int j = 0; j < 8; ++j) s += acc[j][0] + acc[j][7] + acc[j][15];
  out[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = s;
}

}  // namespace xabe

using namespace xabe;

extern "C" int xabe_calibrate_hbm_read(void* stream, const void* buffer, size_t bytes, void* sink) {
  if (!buffer || !sink) return set_error(XABE_ERR_INVALID_ARGUMENT, "calibrate_hbm_read: null pointer");
  if (reinterpret_cast<uintptr_t>(buffer) % 16 != 0 || bytes % 16 != 0 || bytes == 0)
    return set_error(XABE_ERR_INVALID_ARGUMENT, "calibrate_hbm_read: buffer and size must be multiples of 16 bytes");
  int dev = 0, cus = 0;
  XABE_HIP_TRY(hipGetDevice(&dev));
  XABE_HIP_TRY(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
  hipLaunchKernelGGL(k_calibrate_read, dim3((unsigned)cus * 8), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const uint4*>(buffer), bytes / 16, static_cast<uint32_t*>(sink));
  XABE_HIP_TRY(hipGetLastError());
  return XABE_OK;
}

extern "C" int xabe_calibrate_mfma_f16(void* stream, float* out, size_t out_len, int iters, double* flops) {
  if (!out || !flops || iters <= 0) return set_error(XABE_ERR_INVALID_ARGUMENT, "calibrate_mfma_f16: bad argument");
  int dev = 0, cus = 0;
  XABE_HIP_TRY(hipGetDevice(&dev));
  XABE_HIP_TRY(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
  const unsigned grid = (unsigned)cus * 2;  // two workgroups of four wavefronts per CU: two wavefronts per SIMD
  if (out_len < (size_t)grid * 256) return set_error(XABE_ERR_INVALID_ARGUMENT, "calibrate_mfma_f16: out needs %zu floats", (size_t)grid * 256);
  hipLaunchKernelGGL(k_calibrate_mfma, dim3(grid), dim3(256), 0, static_cast<hipStream_t>(stream), out, iters);
  XABE_HIP_TRY(hipGetLastError());
  *flops = (double)grid * 4 * iters * 8 * (2.0 * 32 * 32 * 16);
  return XABE_OK;
}

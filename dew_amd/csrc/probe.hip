// Measurement aids for the roofline report: what this chip sustains, measured in the same run as the kernels.
//   dew_moe_probe_mfma  back-to-back v_mfma_f32_32x32x16_bf16 on caller-supplied operands, nothing else in
//                       the loop. With operands of random sign, exponent and mantissa the matrix cores draw
//                       more power than with constants and the clock settles lower: the sustained rate the
//                       GEMM kernels can approach on real data.
//   dew_moe_probe_copy  a plain 16-byte-per-lane copy: the HBM rate a streaming kernel sustains, and the known
//                       traffic the FETCH_SIZE / WRITE_SIZE counters are scaled by.
#include "common.h"

namespace dew {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;

constexpr int kProbeBlocks = 1024;  // four blocks a CU's worth of work, one wavefront per SIMD at a time

__global__ __launch_bounds__(256) void probe_mfma_kernel(const u32x4_t* __restrict__ operands, float* __restrict__ sink, int iters) {
  f32x16_t acc[16];
#pragma unroll
  for (int a = 0; a < 16; ++a)
#pragma unroll
    for (int q = 0; q < 16; ++q) acc[a][q] = 0.0f;
  bf16x8_t x[4], y[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    x[i] = __builtin_bit_cast(bf16x8_t, operands[i * 256 + threadIdx.x]);
    y[i] = __builtin_bit_cast(bf16x8_t, operands[(4 + i) * 256 + threadIdx.x]);
  }
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int a = 0; a < 16; ++a) acc[a] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(x[a / 4], y[a % 4], acc[a], 0, 0, 0);
  }
  float total = 0.0f;
#pragma unroll
  for (int a = 0; a < 16; ++a)
#pragma unroll
    for (int q = 0; q < 16; ++q) total += acc[a][q];
  sink[blockIdx.x * 256 + threadIdx.x] = total;
}

__global__ __launch_bounds__(256) void probe_copy_kernel(const u32x4_t* __restrict__ src, u32x4_t* __restrict__ dst, size_t chunks) {
  for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < chunks; i += static_cast<size_t>(gridDim.x) * blockDim.x)
    dst[i] = src[i];
}

}  // namespace dew

extern "C" int dew_moe_probe_mfma(const void* operands, int32_t iters, float* sink, double* flops, void* stream) {
  using namespace dew;
  DEW_REQUIRE(operands && sink && iters >= 1, "dew_moe_probe_mfma: operands (32 KiB), sink (1 MiB) and iters >= 1");
  DEW_REQUIRE(aligned16(operands), "dew_moe_probe_mfma: operands must be 16-byte aligned");
  hipLaunchKernelGGL(probe_mfma_kernel, dim3(kProbeBlocks), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const u32x4_t*>(operands), sink, iters);
  if (flops) *flops = static_cast<double>(kProbeBlocks) * 4 * iters * 16 * (2.0 * 32 * 32 * 16);
  return launched("probe_mfma_kernel");
}

extern "C" int dew_moe_probe_copy(const void* src, void* dst, size_t bytes, void* stream) {
  using namespace dew;
  DEW_REQUIRE(src && dst && bytes % 16 == 0 && aligned16(src) && aligned16(dst), "dew_moe_probe_copy: 16-byte aligned buffers and size");
  hipLaunchKernelGGL(probe_copy_kernel, dim3(256 * 32), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const u32x4_t*>(src), static_cast<u32x4_t*>(dst), bytes / 16);
  return launched("probe_copy_kernel");
}

// Measurement aids for the roofline report: what this chip sustains, measured in the same run as the kernels.
//   dew_bench_probe_mfma back-to-back v_mfma_f32_32x32x16_bf16 on caller-supplied operands, nothing else in
//                       the loop. With operands of random sign, exponent and mantissa the matrix cores draw
//                       more power than with constants and the clock settles lower: the sustained rate the
//                       GEMM kernels can approach on real data.
//   dew_bench_probe_copy a plain 16-byte-per-lane copy: the HBM rate a streaming kernel sustains, and the known
//                       traffic the FETCH_SIZE / WRITE_SIZE counters are scaled by.
//   dew_bench_probe_read a read-only stream issued as the decode tiles issue their weight loads: what HBM delivers to
//                       that access pattern with no arithmetic behind it.
//
// Built into its own small library (libdew_bench_probes.so) beside the benchmarks that use it: it is no part of the
// MoE kernels' C ABI.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace dew_bench {

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

// A read-only stream issued the way the decode tiles read their weights: every wavefront walks 64 KiB segments (a
// 32-column strip's depth), 1 KiB a load, eight non-temporal loads in flight a lane.
__global__ __launch_bounds__(256) void probe_read_kernel(const u32x4_t* __restrict__ src, size_t chunks, uint32_t* __restrict__ sink) {
  const size_t waves = static_cast<size_t>(gridDim.x) * 4, wave = static_cast<size_t>(blockIdx.x) * 4 + threadIdx.x / 64;
  const int lane = threadIdx.x % 64;
  constexpr size_t kSegment = 65536 / 16;
  u32x4_t seen = {0, 0, 0, 0};
  for (size_t segment = wave; (segment + 1) * kSegment <= chunks; segment += waves) {
    const u32x4_t* mine = src + segment * kSegment + lane;
    for (int i = 0; i < static_cast<int>(kSegment / 64); i += 8) {
      u32x4_t held[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) held[u] = __builtin_nontemporal_load(mine + (i + u) * 64);
#pragma unroll
      for (int u = 0; u < 8; ++u) seen ^= held[u];
    }
  }
  if ((seen.x ^ seen.y ^ seen.z ^ seen.w) == 0x9E3779B9u) sink[0] = 1;  // (keeps the loads; practically never true)
}

}  // namespace dew_bench

// All return 0, 1 for arguments that do not fit (null or misaligned pointers, sizes that are not whole 16 bytes), or 3
// for a failed launch.
extern "C" int dew_bench_probe_mfma(const void* operands /* 32 KiB of bf16 */, int32_t iters, float* sink /* 1 MiB */,
                                    double* flops /* host, nullable */, void* stream) {
  using namespace dew_bench;
  if (!operands || !sink || iters < 1 || (reinterpret_cast<uintptr_t>(operands) & 15u) != 0) return 1;
  hipLaunchKernelGGL(probe_mfma_kernel, dim3(kProbeBlocks), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const u32x4_t*>(operands), sink, iters);
  if (flops) *flops = static_cast<double>(kProbeBlocks) * 4 * iters * 16 * (2.0 * 32 * 32 * 16);
  return hipGetLastError() == hipSuccess ? 0 : 3;
}

extern "C" int dew_bench_probe_copy(const void* src, void* dst, size_t bytes, void* stream) {
  using namespace dew_bench;
  if (!src || !dst || bytes % 16 != 0 || ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15u) != 0) return 1;
  hipLaunchKernelGGL(probe_copy_kernel, dim3(256 * 32), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const u32x4_t*>(src), static_cast<u32x4_t*>(dst), bytes / 16);
  return hipGetLastError() == hipSuccess ? 0 : 3;
}

extern "C" int dew_bench_probe_read(const void* src, size_t bytes /* whole 64 KiB segments are read */, void* sink /* 4 bytes */, void* stream) {
  using namespace dew_bench;
  if (!src || !sink || bytes % 65536 != 0 || (reinterpret_cast<uintptr_t>(src) & 15u) != 0) return 1;
  hipLaunchKernelGGL(probe_read_kernel, dim3(256 * 8), dim3(256), 0, static_cast<hipStream_t>(stream), static_cast<const u32x4_t*>(src),
                     bytes / 16, static_cast<uint32_t*>(sink));
  return hipGetLastError() == hipSuccess ? 0 : 3;
}

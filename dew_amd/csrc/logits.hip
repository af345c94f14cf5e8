// Router gate logits: logits[t, e] = sum_d f32(x[t, d]) * kernel[d, e] in IEEE fp32
// (reference src/dew/nn/moe.py:526-534: tokens widened to fp32, Precision.HIGHEST), and group offsets.
// A 64-token x 64-expert tile per 256-thread block, 4 x 4 outputs a thread, 16-deep LDS steps, fp32 FMA.
#include "common.h"

namespace dew {

constexpr int LT = 64, LE = 64, LK = 16;

__global__ __launch_bounds__(256) void router_logits_kernel(const bf16_t* __restrict__ x, const float* __restrict__ kernel,
                                                            const float* __restrict__ bias, float* __restrict__ logits,
                                                            int tokens, int depth, int experts) {
  __shared__ float xs[LK][LT + 1];
  __shared__ float ks[LK][LE + 1];
  const int t0 = blockIdx.x * LT, e0 = blockIdx.y * LE;
  const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;  // thread owns tokens ty*4.., experts tx*4..
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.0f;
  for (int d0 = 0; d0 < depth; d0 += LK) {
    for (int item = threadIdx.x; item < LT * LK; item += 256) {
      const int t = item / LK, d = item % LK;
      xs[d][t] = (t0 + t < tokens && d0 + d < depth) ? bf16_to_f32(x[static_cast<size_t>(t0 + t) * depth + d0 + d]) : 0.0f;
    }
    for (int item = threadIdx.x; item < LK * LE; item += 256) {
      const int d = item / LE, e = item % LE;
      ks[d][e] = (d0 + d < depth && e0 + e < experts) ? kernel[static_cast<size_t>(d0 + d) * experts + e0 + e] : 0.0f;
    }
    __syncthreads();
#pragma unroll
    for (int d = 0; d < LK; ++d) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = xs[d][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = ks[d][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int t = t0 + ty * 4 + i, e = e0 + tx * 4 + j;
      // a biased router (GPT-OSS's, src/dew/nn/gpt_oss.py:163-165) adds its fp32 bias to the finished sum
      if (t < tokens && e < experts) logits[static_cast<size_t>(t) * experts + e] = bias ? acc[i][j] + bias[e] : acc[i][j];
    }
}

// offsets[0] = 0, offsets[e + 1] = offsets[e] + sizes[e]; one wavefront, serial over the experts.
__global__ void group_offsets_kernel(const int32_t* __restrict__ sizes, int32_t* __restrict__ offsets, int experts) {
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    int running = 0;
    offsets[0] = 0;
    for (int e = 0; e < experts; ++e) {
      running += sizes[e];
      offsets[e + 1] = running;
    }
  }
}

}  // namespace dew

extern "C" int dew_moe_router_logits(const void* x, const float* kernel, const float* bias, float* logits, int32_t tokens,
                                     int32_t depth, int32_t experts, void* stream) {
  using namespace dew;
  DEW_REQUIRE(tokens >= 0 && depth >= 1 && experts >= 1, "dew_moe_router_logits: tokens %d depth %d experts %d", tokens, depth, experts);
  if (tokens == 0) return DEW_MOE_OK;
  DEW_REQUIRE(x && kernel && logits, "dew_moe_router_logits: x, kernel and logits must not be null");
  const dim3 grid((tokens + LT - 1) / LT, (experts + LE - 1) / LE);
  hipLaunchKernelGGL(router_logits_kernel, grid, dim3(256), 0, static_cast<hipStream_t>(stream), static_cast<const bf16_t*>(x),
                     kernel, bias, logits, tokens, depth, experts);
  return launched("router_logits_kernel");
}

extern "C" int dew_moe_group_offsets(const int32_t* sizes, int32_t experts, int32_t* offsets, void* stream) {
  using namespace dew;
  DEW_REQUIRE(sizes && offsets && experts >= 1, "dew_moe_group_offsets: sizes, offsets must not be null, experts %d", experts);
  hipLaunchKernelGGL(group_offsets_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream), sizes, offsets, experts);
  return launched("group_offsets_kernel");
}

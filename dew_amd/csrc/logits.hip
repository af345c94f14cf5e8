// Router gate logits: logits[t, e] = sum_d f32(x[t, d]) * kernel[d, e] in IEEE fp32
// (reference src/dew/nn/moe.py:526-534: tokens widened to fp32, Precision.HIGHEST), and group offsets.
// Depths in whole 16s run on the fp32 matrix instruction (v_mfma_f32_32x32x2_f32: fp32 operands, exact products, fp32
// sums): a block takes 32 (or 64) tokens and up to four 32-expert tiles, its wavefronts a share of the depth each; the
// partial sums of a tile meet in LDS in wavefront order, so the result does not depend on timing. A decode step's few
// tokens take 16 x 16 tiles (v_mfma_f32_16x16x4_f32), four times the blocks. Measured: 64 tokens of GPT-OSS's 2880 x 32
// gate in about 5 us of kernel and 8192 tokens of a 7168 x 256 gate in 319 us (94 TFLOP/s), where the
// plain kernel below (a 64-token x 64-expert tile, 16-deep LDS steps, fp32 FMA; depths in no whole 16s still take it)
// needed 550 us and 1.3 ms.
#include "common.h"

namespace dew {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// WAVES wavefronts a block split the depth: 4 where the tokens alone fill the chip, 16 for the few tokens of a decode step
// (64 tokens are two blocks: their latency is the depth a wavefront walks).
template <int TILES, int WAVES, int ROWS = 1>
__global__ __launch_bounds__(64 * WAVES) void router_logits_mfma_kernel(const bf16_t* __restrict__ x, const float* __restrict__ kernel,
                                                                        const float* __restrict__ bias, float* __restrict__ logits,
                                                                        int tokens, int depth, int experts) {
  __shared__ float partial[WAVES][16][64];  // a tile's partial sums, [wavefront][register][lane]
  const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
  const int t0 = blockIdx.x * 32 * ROWS;  // ROWS tiles of 32 tokens a block (2 where the tokens are many: a weight load serves both)
  int row[ROWS];
#pragma unroll
  for (int r = 0; r < ROWS; ++r) row[r] = min(t0 + 32 * r + lane % 32, tokens - 1);  // (rows past the tokens repeat the last one; they are not stored)
  const int chunks = depth / 16;                    // 16 depths a chunk: the lane's 8 are 8 (lane / 32) .. + 7 of them
  const int first = static_cast<int>(static_cast<long long>(chunks) * wave / WAVES);
  const int last = static_cast<int>(static_cast<long long>(chunks) * (wave + 1) / WAVES);
  const bf16_t* a_src[ROWS];
#pragma unroll
  for (int r = 0; r < ROWS; ++r) a_src[r] = x + static_cast<size_t>(row[r]) * depth + 8 * (lane / 32);
  int column[TILES];
  const int tile0 = blockIdx.y * TILES;  // (a decode step's blocks take one tile each: the gate kernel's bytes spread over the CUs)
#pragma unroll
  for (int c = 0; c < TILES; ++c) column[c] = min(32 * (tile0 + c) + lane % 32, experts - 1);
  f32x16 acc[ROWS][TILES];
#pragma unroll
  for (int r = 0; r < ROWS; ++r)
#pragma unroll
    for (int c = 0; c < TILES; ++c)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[r][c][i] = 0.0f;
  // A chunk's operands are loaded while the chunk before it multiplies (a block may be alone on its CU: nothing else
  // would hide the loads).
  u32x4 a_words[2][ROWS];
  float b[2][TILES][8];
  auto load = [&](int buffer, int chunk) __attribute__((always_inline)) {
#pragma unroll
    for (int r = 0; r < ROWS; ++r) a_words[buffer][r] = *reinterpret_cast<const u32x4*>(a_src[r] + chunk * 16);
    const float* b_src = kernel + static_cast<size_t>(chunk * 16 + 8 * (lane / 32)) * experts;
#pragma unroll
    for (int c = 0; c < TILES; ++c)
#pragma unroll
      for (int j = 0; j < 8; ++j) b[buffer][c][j] = b_src[static_cast<size_t>(j) * experts + column[c]];
  };
  auto multiply = [&](int buffer) __attribute__((always_inline)) {
    float a[ROWS][8];
#pragma unroll
    for (int r = 0; r < ROWS; ++r)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        a[r][2 * i] = __uint_as_float(a_words[buffer][r][i] << 16);
        a[r][2 * i + 1] = __uint_as_float(a_words[buffer][r][i] & 0xFFFF0000u);
      }
#pragma unroll
    for (int c = 0; c < TILES; ++c)
#pragma unroll
      for (int r = 0; r < ROWS; ++r)
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[r][c] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[r][j], b[buffer][c][j], acc[r][c], 0, 0, 0);
  };
  if constexpr (WAVES == 16) {  // a decode step's wavefronts walk a few chunks each (loads kept further ahead changed nothing: the matrix pipe is the limit)
    for (int chunk = first; chunk < last; ++chunk) {
      load(0, chunk);
      multiply(0);
    }
  } else {
    if (first < last) load(0, first);
    for (int chunk = first; chunk < last; chunk += 2) {
      load(1, min(chunk + 1, last - 1));
      multiply(0);
      load(0, min(chunk + 2, last - 1));
      if (chunk + 1 < last) multiply(1);
    }
  }
  // register i of lane l is the sum of token 8 (i / 4) + 4 (l / 32) + i % 4, expert column l % 32 of the tile. A tile's
  // partial sums go through LDS; every thread then finishes its share of the tile's 1024 sums, adding the wavefronts'
  // partial sums in wavefront order.
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
#pragma unroll
    for (int c = 0; c < TILES; ++c) {
      if (32 * (tile0 + c) >= experts) continue;  // (the same for every wavefront of the block: the barriers below stay matched)
      __syncthreads();
#pragma unroll
      for (int i = 0; i < 16; ++i) partial[wave][i][lane] = acc[r][c][i];
      __syncthreads();
#pragma unroll
      for (int k = 0; k < 16 / WAVES; ++k) {
        const int i = wave + WAVES * k;
        float sum = partial[0][i][lane];
#pragma unroll
        for (int w = 1; w < WAVES; ++w) sum += partial[w][i][lane];
        const int t = t0 + 32 * r + 8 * (i / 4) + 4 * (lane / 32) + i % 4, e = 32 * (tile0 + c) + lane % 32;
        // a biased router (GPT-OSS's, src/dew/nn/gpt_oss.py:163-165) adds its fp32 bias to the finished sum
        if (t < tokens && e < experts) logits[static_cast<size_t>(t) * experts + e] = bias ? sum + bias[e] : sum;
      }
    }
  }
}

// The few tokens of a decode step on finer tiles: 16 tokens x 16 experts a block (v_mfma_f32_16x16x4_f32, the same
// rate a CU as the 32 x 32 form), sixteen wavefronts a share of the depth each. A 32 x 32 tile's block keeps its whole
// product on one CU's four matrix pipes (64 tokens of a 2880 x 32 gate: two blocks, 20 us); four times the blocks
// finish in a quarter of that. Lane l multiplies token l % 16 and expert l % 16 over the depths 4 (l / 16) .. + 3 of a
// 16-deep chunk, one depth an instruction; its four sums are tokens 4 (l / 16) + i of expert column l % 16.
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

__global__ __launch_bounds__(1024) void router_logits_fine_kernel(const bf16_t* __restrict__ x, const float* __restrict__ kernel,
                                                                  const float* __restrict__ bias, float* __restrict__ logits,
                                                                  int tokens, int depth, int experts) {
  constexpr int kWaves = 16;
  __shared__ float partial[kWaves][4][64];
  const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
  const int t0 = blockIdx.x * 16, e0 = blockIdx.y * 16;
  const int chunks = depth / 16;
  const int first = static_cast<int>(static_cast<long long>(chunks) * wave / kWaves);
  const int last = static_cast<int>(static_cast<long long>(chunks) * (wave + 1) / kWaves);
  const bf16_t* a_src = x + static_cast<size_t>(min(t0 + lane % 16, tokens - 1)) * depth + 4 * (lane / 16);
  const float* b_src = kernel + static_cast<size_t>(4 * (lane / 16)) * experts + min(e0 + lane % 16, experts - 1);
  f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
  // four chunks' loads are in flight while the four before them multiply (a wavefront's walk is a chain of round trips
  // otherwise: 28 chunks of a 7168-deep gate)
  constexpr int kAhead = 4;
  u32x2 words[2][kAhead];
  float b[2][kAhead][4];
  auto load = [&](int set, int chunk) __attribute__((always_inline)) {
#pragma unroll
    for (int ahead = 0; ahead < kAhead; ++ahead) {
      const int at = min(chunk + ahead, last - 1);  // (past the share: the last chunk again, which multiplies nothing)
      words[set][ahead] = *reinterpret_cast<const u32x2*>(a_src + at * 16);
#pragma unroll
      for (int j = 0; j < 4; ++j) b[set][ahead][j] = b_src[static_cast<size_t>(at * 16 + j) * experts];
    }
  };
  auto multiply = [&](int set, int chunk) __attribute__((always_inline)) {
#pragma unroll
    for (int ahead = 0; ahead < kAhead; ++ahead) {
      if (chunk + ahead >= last) continue;
      const u32x2 w = words[set][ahead];
      const float a[4] = {__uint_as_float(w[0] << 16), __uint_as_float(w[0] & 0xFFFF0000u), __uint_as_float(w[1] << 16),
                          __uint_as_float(w[1] & 0xFFFF0000u)};
#pragma unroll
      for (int j = 0; j < 4; ++j) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[j], b[set][ahead][j], acc, 0, 0, 0);
    }
  };
  if (first < last) load(0, first);
  for (int chunk = first; chunk < last; chunk += 2 * kAhead) {
    if (chunk + kAhead < last) load(1, chunk + kAhead);
    multiply(0, chunk);
    if (chunk + 2 * kAhead < last) load(0, chunk + 2 * kAhead);
    if (chunk + kAhead < last) multiply(1, chunk + kAhead);
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) partial[wave][i][lane] = acc[i];
  __syncthreads();
  if (wave < 4) {  // wavefront i finishes register i of every lane, adding the wavefronts' partial sums in wavefront order
    float sum = partial[0][wave][lane];
#pragma unroll
    for (int w = 1; w < kWaves; ++w) sum += partial[w][wave][lane];
    const int t = t0 + 4 * (lane / 16) + wave, e = e0 + lane % 16;
    if (t < tokens && e < experts) logits[static_cast<size_t>(t) * experts + e] = bias ? sum + bias[e] : sum;
  }
}

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
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int tiles = (experts + 31) / 32;
  if (depth % 16 == 0 && depth >= 64 && (reinterpret_cast<uintptr_t>(x) & 15u) == 0) {
    if (static_cast<long long>((tokens + 31) / 32) * tiles < 64) {  // a decode step: finer tiles, four times the blocks
      hipLaunchKernelGGL(router_logits_fine_kernel, dim3((tokens + 15) / 16, (experts + 15) / 16), dim3(1024), 0, s,
                         static_cast<const bf16_t*>(x), kernel, bias, logits, tokens, depth, experts);
      return launched("router_logits_fine_kernel");
    }
    if (tokens <= 2048) {  // at most 64 token blocks: a block takes one tile, its sixteen wavefronts share the depth
      hipLaunchKernelGGL((router_logits_mfma_kernel<1, 16>), dim3((tokens + 31) / 32, tiles), dim3(1024), 0, s, static_cast<const bf16_t*>(x),
                         kernel, bias, logits, tokens, depth, experts);
      return launched("router_logits_mfma_kernel");
    }
    // (more than four tiles: blocks of four tiles beside each other, 64 accumulators a lane, several blocks a CU)
    auto launch = [&](auto routine, int tiles_a_block, int rows_a_block) {
      hipLaunchKernelGGL(routine, dim3((tokens + 32 * rows_a_block - 1) / (32 * rows_a_block), (tiles + tiles_a_block - 1) / tiles_a_block),
                         dim3(256), 0, s, static_cast<const bf16_t*>(x), kernel, bias, logits, tokens, depth, experts);
    };
    if (tiles == 1) launch(router_logits_mfma_kernel<1, 4>, 1, 1);
    else if (tiles == 2) launch(router_logits_mfma_kernel<2, 4>, 2, 1);
    else if (static_cast<long long>(tokens / 64) * ((tiles + 3) / 4) >= 256) launch(router_logits_mfma_kernel<4, 4, 2>, 4, 2);  // still a block a CU
    else launch(router_logits_mfma_kernel<4, 4>, 4, 1);
    return launched("router_logits_mfma_kernel");
  }
  const dim3 grid((tokens + LT - 1) / LT, (experts + LE - 1) / LE);
  hipLaunchKernelGGL(router_logits_kernel, grid, dim3(256), 0, s, static_cast<const bf16_t*>(x), kernel, bias, logits, tokens, depth,
                     experts);
  return launched("router_logits_kernel");
}

extern "C" int dew_moe_group_offsets(const int32_t* sizes, int32_t experts, int32_t* offsets, void* stream) {
  using namespace dew;
  DEW_REQUIRE(sizes && offsets && experts >= 1, "dew_moe_group_offsets: sizes, offsets must not be null, experts %d", experts);
  hipLaunchKernelGGL(group_offsets_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream), sizes, offsets, experts);
  return launched("group_offsets_kernel");
}

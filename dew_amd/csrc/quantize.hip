// Activation rows quantized for the blockwise FP8 recipe (DeepSeek-V3's): e4m3 codes a 1 x 128 tile at a time
// along the depth under one power-of-two scale a tile (reference src/dew/nn/kernels/projections.py:176-182 over
// src/dew/nn/fake_quant.py:117-128, 48-76): amax floored at 1e-4, scale = the least power of two >= amax * f32(1 / 448)
// (read off the product's fp32 bits: its exponent, plus one where any fraction bit is set), code = e4m3(x / scale),
// ties to even; the quotient by a power of two is exact and lies within +-448 by the scale's choice.
// The codes are written in the order the scaled matrix instruction reads its 8-bit operand, so that the grouped
// GEMM copies rows into the LDS as they are: of each 128 depths, byte 16 (4 g + 2 t + h) + b holds depth
// 64 t + 32 h + 16 g + b (t the 64-deep half, g the instruction's lane group, h the half of the group's 32 bytes).
// The scales are kept as their e8m0 bytes, block_scale_pitch(depth) a row (one byte per 128 depths, padded to 16).
// HBM-bound: 2 bytes read and 1 written per element.
#include "common.h"

namespace dew {

typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2_t;

constexpr int kQuantizeWaves = 4;  // rows per 256-thread block

__global__ __launch_bounds__(64 * kQuantizeWaves) void quantize_rows_fp8_kernel(const bf16_t* __restrict__ x, uint8_t* __restrict__ codes,
                                                                              uint8_t* __restrict__ scales, int rows, int depth,
                                                                              int pitch) {
  const int lane = threadIdx.x % 64;
  const int row = blockIdx.x * kQuantizeWaves + threadIdx.x / 64;
  if (row >= rows) return;
  const bf16_t* source = x + static_cast<size_t>(row) * depth;
  uint8_t* target = codes + static_cast<size_t>(row) * depth;
  // a lane takes 8 consecutive depths, 16 lanes a tile of 128, four tiles a pass of the wavefront
  for (int chunk = lane; chunk < depth / 8; chunk += 64) {
    const u32x4_t words = *reinterpret_cast<const u32x4_t*>(source + chunk * 8);
    float v[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[2 * i] = __uint_as_float(words[i] << 16);
      v[2 * i + 1] = __uint_as_float(words[i] & 0xFFFF0000u);
    }
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(v[i]));
#pragma unroll
    for (int offset = 1; offset < 16; offset <<= 1) amax = fmaxf(amax, __shfl_xor(amax, offset, 64));
    const uint32_t bits = __float_as_uint(fmaxf(amax, 1e-4f) * 0x1.24924ap-9f);  // f32(1 / 448)
    const uint32_t field = min(max((bits >> 23) + ((bits & 0x7FFFFFu) != 0u ? 1u : 0u), 1u), 253u);
    const float inverse = __uint_as_float((254u - field) << 23);  // 1 / scale, exactly
    uint32_t packed[2];
#pragma unroll
    for (int w = 0; w < 2; ++w) {
      packed[w] = __builtin_amdgcn_cvt_pk_fp8_f32(v[4 * w] * inverse, v[4 * w + 1] * inverse, 0, false);
      packed[w] = __builtin_amdgcn_cvt_pk_fp8_f32(v[4 * w + 2] * inverse, v[4 * w + 3] * inverse, packed[w], true);
    }
    // depths 8 chunk .. 8 chunk + 7 of the row: eighth `within` of their 128-deep tile's sixteen
    const int within = chunk % 16, half = within / 8, piece = (within % 8) / 4, group = (within % 4) / 2, low = within % 2;
    *reinterpret_cast<u32x2_t*>(target + (chunk / 16) * 128 + 16 * (4 * group + 2 * half + piece) + 8 * low) = u32x2_t{packed[0], packed[1]};
    if (within == 0) scales[static_cast<size_t>(row) * pitch + chunk / 16] = static_cast<uint8_t>(field);
  }
}

// The MXFP8 recipe's rows (OCP MX; reference src/dew/nn/kernels/formats.py:186-229): e4m3 codes under one E8M0 scale
// every 32 depths, the scale 2 to the largest magnitude's binary exponent less 8 (its fp32 exponent field less 8 is
// the byte; a block of zeros, or one whose largest magnitude lies under 2^-119, takes byte 0), each value over its
// scale rounded to e4m3, ties to even, saturating at +-448. Codes in the same operand order as above; the scale
// bytes in depth order, depth / 32 a row (a 128-deep step's four bytes are one aligned dword).
__global__ __launch_bounds__(64 * kQuantizeWaves) void quantize_rows_mxfp8_kernel(const bf16_t* __restrict__ x, uint8_t* __restrict__ codes,
                                                                                uint8_t* __restrict__ scales, int rows, int depth) {
  const int lane = threadIdx.x % 64;
  const int row = blockIdx.x * kQuantizeWaves + threadIdx.x / 64;
  if (row >= rows) return;
  const bf16_t* source = x + static_cast<size_t>(row) * depth;
  uint8_t* target = codes + static_cast<size_t>(row) * depth;
  for (int chunk = lane; chunk < depth / 8; chunk += 64) {  // 8 depths a lane, 4 lanes a block of 32
    const u32x4_t words = *reinterpret_cast<const u32x4_t*>(source + chunk * 8);
    float v[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[2 * i] = __uint_as_float(words[i] << 16);
      v[2 * i + 1] = __uint_as_float(words[i] & 0xFFFF0000u);
    }
    float largest = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) largest = fmaxf(largest, fabsf(v[i]));
    largest = fmaxf(largest, __shfl_xor(largest, 1, 64));
    largest = fmaxf(largest, __shfl_xor(largest, 2, 64));
    const int field = static_cast<int>(__float_as_uint(largest) >> 23);  // 0 for a zero or subnormal magnitude
    const uint32_t byte = static_cast<uint32_t>(min(max(field - 8, 0), 254));
    const float inverse = __uint_as_float((254u - byte) << 23);  // 2^(127 - byte), exactly (byte <= 247 for finite rows)
    uint32_t packed[2];
#pragma unroll
    for (int w = 0; w < 2; ++w) {
      float q[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) q[i] = fminf(fmaxf(v[4 * w + i] * inverse, -448.0f), 448.0f);
      packed[w] = __builtin_amdgcn_cvt_pk_fp8_f32(q[0], q[1], 0, false);
      packed[w] = __builtin_amdgcn_cvt_pk_fp8_f32(q[2], q[3], packed[w], true);
    }
    const int within = chunk % 16, half = within / 8, piece = (within % 8) / 4, group = (within % 4) / 2, low = within % 2;
    *reinterpret_cast<u32x2_t*>(target + (chunk / 16) * 128 + 16 * (4 * group + 2 * half + piece) + 8 * low) = u32x2_t{packed[0], packed[1]};
    if (chunk % 4 == 0) scales[static_cast<size_t>(row) * (depth / 32) + chunk / 4] = static_cast<uint8_t>(byte);
  }
}

// The NVFP4 recipe's rows (reference src/dew/nn/kernels/formats.py:263-274 over src/dew/algebra/bits.py:941-982):
// E2M1 codes under an E4M3 scale every 16 depths and one tensor scale over the whole operand. The scaled matrix
// instruction takes power-of-two scales of 32 depths only, so this operand goes to the bf16 instruction: each value is
// written as what it stands for short of the tensor scale, code x block scale, which bf16 holds exactly (5 significant
// bits), and the product applies the tensor scale to its fp32 sums with the bank's.
// Two passes, because the tensor scale needs the whole operand's largest magnitude first.
__global__ __launch_bounds__(256) void absmax_clear_kernel(uint32_t* __restrict__ largest) { *largest = 0u; }

__global__ __launch_bounds__(256) void absmax_kernel(const bf16_t* __restrict__ x, long long chunks, uint32_t* __restrict__ largest) {
  uint32_t mine = 0;  // magnitudes of bf16 values order as their bit patterns do
  const long long stride = static_cast<long long>(gridDim.x) * blockDim.x;
  long long chunk = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
  for (; chunk + 3 * stride < chunks; chunk += 4 * stride) {  // four loads in flight a lane
    u32x4_t words[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) words[k] = reinterpret_cast<const u32x4_t*>(x)[chunk + k * stride];
#pragma unroll
    for (int k = 0; k < 4; ++k)
#pragma unroll
      for (int i = 0; i < 4; ++i) mine = max(mine, max(words[k][i] & 0x7FFFu, (words[k][i] >> 16) & 0x7FFFu));
  }
  for (; chunk < chunks; chunk += stride) {
    const u32x4_t words = reinterpret_cast<const u32x4_t*>(x)[chunk];
#pragma unroll
    for (int i = 0; i < 4; ++i) mine = max(mine, max(words[i] & 0x7FFFu, (words[i] >> 16) & 0x7FFFu));
  }
#pragma unroll
  for (int offset = 32; offset >= 1; offset >>= 1) mine = max(mine, static_cast<uint32_t>(__shfl_xor(static_cast<int>(mine), offset, 64)));
  if (threadIdx.x % 64 == 0 && mine != 0) atomicMax(largest, mine);
}

__device__ __forceinline__ float e2m1_nearest(float magnitude) {
  // ties to the even code: 0.25 -> 0, 0.75 -> 1, 1.25 -> 1, 1.75 -> 2, 2.5 -> 2, 3.5 -> 4, 5 -> 4
  float value = magnitude > 0.25f ? 0.5f : 0.0f;
  value = magnitude >= 0.75f ? 1.0f : value;
  value = magnitude > 1.25f ? 1.5f : value;
  value = magnitude >= 1.75f ? 2.0f : value;
  value = magnitude > 2.5f ? 3.0f : value;
  value = magnitude >= 3.5f ? 4.0f : value;
  return magnitude > 5.0f ? 6.0f : value;
}

// The same choice times the block scale, without the quotient: for y = x / tensor and the block scale `each` (an e4m3
// value, four significant bits), fl(y / each) > t exactly where y > t each, and >= likewise, for each of the seven
// thresholds t (at most three significant bits, so t each is exact): a y above t each lies at least one ulp of t each
// above it, which is more than half an ulp of t above t in the quotient (their ratio is 1 / m or 2 / m for each's
// significand m < 2), so the quotient rounds past t; at or below, it cannot round above. One IEEE division an element
// instead of two.
__device__ __forceinline__ float e2m1_scaled(float magnitude, float each) {
  float value = magnitude > 0.25f * each ? 0.5f * each : 0.0f;
  value = magnitude >= 0.75f * each ? each : value;
  value = magnitude > 1.25f * each ? 1.5f * each : value;
  value = magnitude >= 1.75f * each ? 2.0f * each : value;
  value = magnitude > 2.5f * each ? 3.0f * each : value;
  value = magnitude >= 3.5f * each ? 4.0f * each : value;
  return magnitude > 5.0f * each ? 6.0f * each : value;
}

__global__ __launch_bounds__(64 * kQuantizeWaves) void quantize_rows_nvfp4_kernel(const bf16_t* __restrict__ x, const uint32_t* __restrict__ largest,
                                                                                bf16_t* __restrict__ out, float* __restrict__ tensor_scale,
                                                                                int rows, int depth) {
  const float top = __uint_as_float(*largest << 16);
  // largest / (6 * 448), fp32's least normal at least; 1 for an operand of zeros
  const float tensor = top > 0.0f ? fmaxf(top / 2688.0f, 1.17549435e-38f) : 1.0f;
  if (blockIdx.x == 0 && threadIdx.x == 0) *tensor_scale = tensor;
  const int lane = threadIdx.x % 64;
  const int row = blockIdx.x * kQuantizeWaves + threadIdx.x / 64;
  if (row >= rows) return;
  const bf16_t* source = x + static_cast<size_t>(row) * depth;
  bf16_t* target = out + static_cast<size_t>(row) * depth;
  for (int chunk = lane; chunk < depth / 8; chunk += 64) {  // 8 depths a lane, 2 lanes a block of 16
    const u32x4_t words = *reinterpret_cast<const u32x4_t*>(source + chunk * 8);
    float v[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[2 * i] = __uint_as_float(words[i] << 16);
      v[2 * i + 1] = __uint_as_float(words[i] & 0xFFFF0000u);
    }
    float block = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) block = fmaxf(block, fabsf(v[i]));
    block = fmaxf(block, __shfl_xor(block, 1, 64));
    // the least e4m3 at or above blockmax / tensor / 6: the nearest one, and the next where that lies below
    const float ratio = (block / tensor) / 6.0f;
    uint32_t byte = __builtin_amdgcn_cvt_pk_fp8_f32(fminf(ratio, 448.0f), 0.0f, 0, false) & 0xFFu;
    if (__builtin_amdgcn_cvt_f32_fp8(byte, 0) < ratio) byte = min(byte + 1u, 0x7Eu);
    const float each = __builtin_amdgcn_cvt_f32_fp8(byte, 0);
    u32x4_t packed;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float pair[2];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const float source_value = v[2 * i + h];
        const float over_tensor = each > 0.0f ? source_value / tensor : 0.0f;
        pair[h] = copysignf(e2m1_scaled(fabsf(over_tensor), each), over_tensor);  // code x block scale: exact in bf16
      }
      packed[i] = (__float_as_uint(pair[0]) >> 16) | (__float_as_uint(pair[1]) & 0xFFFF0000u);
    }
    *reinterpret_cast<u32x4_t*>(target + chunk * 8) = packed;
  }
}

// A kernel gradient's operands: x [tokens, dim] quantized ALONG THE TOKENS and written transposed, for the product
// that contracts each group's tokens (reference src/dew/nn/kernels/projections.py:211-224 `rows_quantized(x.T)`, and
// :263-275 `MxFp8.quantized(x.T)`). MX false: the blockwise FP8 recipe's 1 x 128 tiles (128 tokens of one column under
// the scale rule of quantize_rows_fp8_kernel, its byte written for each of the tile's four 32-token blocks); MX true: OCP
// MX blocks of 32 tokens (quantize_rows_mxfp8_kernel's rule). BANK false writes the lhs_t operand: codes [dim, tokens]
// in the row operand's order within each 128 tokens (see the head of this file) and scales [dim, tokens / 32]. BANK true
// writes the rhs_t operand as a prepared MXFP8 bank of one expert, depth = tokens, width = dim: codes as 32 column x 32
// token atoms [dim / 32][tokens / 32][64 lanes][16 bytes] (lane 32 g + c holds tokens 16 g .. 16 g + 15 of column c) and
// scales [dim / 32][tokens / 128][32 columns][4 bytes].
// A block takes 128 tokens x 64 columns through the LDS: thread (column c, quarter a) owns the 32 tokens of block a.
// HBM-bound: 2 bytes read and 1 written per element.
template <bool MX, bool BANK>
__global__ __launch_bounds__(256) void quantize_columns_kernel(const bf16_t* __restrict__ x, uint8_t* __restrict__ codes,
                                                               uint32_t* __restrict__ scales, int tokens, int dim) {
  __shared__ uint32_t tile[128][33];     // 128 tokens x 64 columns of bf16, a dword of padding a row
  __shared__ float quarter_amax[4][64];
  __shared__ uint32_t scale_word[64];    // a column's four scale bytes
  __shared__ u32x4_t staged[64][8];      // the lhs_t operand's 64 rows of 128 bytes, chunk xor-swizzled by the row
  const int tid = threadIdx.x;
  const int t0 = blockIdx.x * 128, d0 = blockIdx.y * 64;
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int item = tid + 256 * k, row = item / 8, chunk = item % 8;
    const u32x4_t words = *reinterpret_cast<const u32x4_t*>(x + static_cast<size_t>(t0 + row) * dim + d0 + chunk * 8);
#pragma unroll
    for (int i = 0; i < 4; ++i) tile[row][chunk * 4 + i] = words[i];
  }
  if (tid < 64) scale_word[tid] = 0;
  __syncthreads();
  const int c = tid % 64, quarter = tid / 64;
  float v[32];
  float largest = 0.0f;
#pragma unroll
  for (int i = 0; i < 32; ++i) {
    const uint32_t word = tile[32 * quarter + i][c / 2];
    v[i] = __uint_as_float(c % 2 ? word & 0xFFFF0000u : word << 16);
    largest = fmaxf(largest, fabsf(v[i]));
  }
  uint32_t byte;
  if constexpr (MX) {
    const int field = static_cast<int>(__float_as_uint(largest) >> 23);
    byte = static_cast<uint32_t>(min(max(field - 8, 0), 254));
  } else {
    quarter_amax[quarter][c] = largest;
    __syncthreads();
    const float amax = fmaxf(fmaxf(quarter_amax[0][c], quarter_amax[1][c]), fmaxf(quarter_amax[2][c], quarter_amax[3][c]));
    const uint32_t bits = __float_as_uint(fmaxf(amax, 1e-4f) * 0x1.24924ap-9f);  // f32(1 / 448)
    byte = min(max((bits >> 23) + ((bits & 0x7FFFFFu) != 0u ? 1u : 0u), 1u), 253u);
  }
  const float inverse = __uint_as_float((254u - byte) << 23);
  uint32_t packed[8];
#pragma unroll
  for (int w = 0; w < 8; ++w) {
    float q[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) q[i] = MX ? fminf(fmaxf(v[4 * w + i] * inverse, -448.0f), 448.0f) : v[4 * w + i] * inverse;
    packed[w] = __builtin_amdgcn_cvt_pk_fp8_f32(q[0], q[1], 0, false);
    packed[w] = __builtin_amdgcn_cvt_pk_fp8_f32(q[2], q[3], packed[w], true);
  }
  atomicOr(&scale_word[c], byte << (8 * quarter));
  const u32x4_t low = {packed[0], packed[1], packed[2], packed[3]}, high = {packed[4], packed[5], packed[6], packed[7]};
  if constexpr (BANK) {
    uint8_t* atom = codes + ((static_cast<size_t>((d0 + c) / 32) * (tokens / 32) + t0 / 32 + quarter) * 64 + c % 32) * 16;
    *reinterpret_cast<u32x4_t*>(atom) = low;
    *reinterpret_cast<u32x4_t*>(atom + 512) = high;
    __syncthreads();
    if (tid < 64) scales[(static_cast<size_t>((d0 + tid) / 32) * (tokens / 128) + t0 / 128) * 32 + tid % 32] = scale_word[tid];
  } else {
    // tokens 32 a + 16 g + b of the 128 sit at byte 16 (4 g + a) + b
    staged[c][quarter ^ (c & 7)] = low;
    staged[c][(4 + quarter) ^ (c & 7)] = high;
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const int item = tid + 256 * k, row = item / 8, chunk = item % 8;
      *reinterpret_cast<u32x4_t*>(codes + static_cast<size_t>(d0 + row) * tokens + t0 + chunk * 16) = staged[row][chunk ^ (row & 7)];
    }
    if (tid < 64) scales[static_cast<size_t>(d0 + tid) * (tokens / 128) + t0 / 128] = scale_word[tid];
  }
}

// A kernel gradient's bf16 operands: x [tokens, dim] written transposed, as it is (`gemm_t`'s operands, reference
// src/dew/nn/kernels/gemm.py:418-431) or, NVFP4 true, quantized ALONG THE TOKENS to the NVFP4 recipe's values (E2M1
// codes under an E4M3 scale every 16 tokens, the tensor scale left to the product: quantize_rows_nvfp4_kernel's
// arithmetic, reference src/dew/nn/kernels/projections.py:330-335). BANK false: rows [dim, tokens] bf16. BANK true: a
// prepared DEW_MOE_W_BF16 bank of one expert, depth = tokens, width = dim: atoms [dim / 32][tokens / 16][64 lanes][8
// bf16], lane 32 g + c holding tokens 8 g .. 8 g + 7 of column c. The same 128-token x 64-column tile and thread
// ownership as quantize_columns_kernel.
// With `offsets` (groups + 1 of them) the groups are ragged: each is written from a whole 64-token step on, its last
// step filled with zeros, so that the product's windows need no mask; `tokens` is then the padded extent (at least
// the rows plus 64 a group, in whole 128s), the tokens past the last group are zeros, and `padded` receives the
// groups' offsets in the written order. Every block scans the group sizes itself (at most 4096 of them).
constexpr int kMaxPaddedGroups = 4096;

template <bool NVFP4, bool BANK>
__global__ __launch_bounds__(256) void transpose_columns_kernel(const bf16_t* __restrict__ x, const uint32_t* __restrict__ largest,
                                                                uint8_t* __restrict__ out, float* __restrict__ tensor_scale,
                                                                int tokens, int dim, const int32_t* __restrict__ offsets, int groups,
                                                                int32_t* __restrict__ padded, int rows) {
  __shared__ uint32_t tile[128][33];
  __shared__ u32x4_t staged[64][16];  // the rows operand's 64 rows of 256 bytes, chunk xor-swizzled by the row
  __shared__ int source_row[128];     // the row of x each of the block's tokens is, -1 for a token of padding
  __shared__ int starts[kMaxPaddedGroups + 1];
  __shared__ int partial[256];
  const int tid = threadIdx.x;
  const int t0 = blockIdx.x * 128, d0 = blockIdx.y * 64;
  if (offsets == nullptr) {
    if (tid < 128) source_row[tid] = t0 + tid;
  } else {
    // padded start of every group: an exclusive scan of the sizes rounded up to whole 64s
    const int each = (groups + 255) / 256;
    int sum = 0;
    for (int g = tid * each; g < min((tid + 1) * each, groups); ++g) sum += (offsets[g + 1] - offsets[g] + 63) / 64 * 64;
    partial[tid] = sum;
    __syncthreads();
    for (int offset = 1; offset < 256; offset <<= 1) {
      const int other = tid >= offset ? partial[tid - offset] : 0;
      __syncthreads();
      partial[tid] += other;
      __syncthreads();
    }
    int running = partial[tid] - sum;
    for (int g = tid * each; g < min((tid + 1) * each, groups); ++g) {
      starts[g] = running;
      running += (offsets[g + 1] - offsets[g] + 63) / 64 * 64;
    }
    if (tid == 255) starts[groups] = partial[255];
    __syncthreads();
    if (blockIdx.x == 0 && blockIdx.y == 0)
      for (int g = tid; g <= groups; g += 256) padded[g] = starts[g];
    if (tid < 128) {
      const int token = t0 + tid;
      int low = 0, high = groups;  // the last group that starts at or before the token
      while (high - low > 1) {
        const int middle = (low + high) / 2;
        if (starts[middle] <= token) low = middle; else high = middle;
      }
      const int within = token - starts[low];
      const int source = offsets[low] + within;  // (offsets that leave x's rows read nothing)
      source_row[tid] = (token < starts[groups] && within < offsets[low + 1] - offsets[low] && source >= 0 && source < rows) ? source : -1;
    }
  }
  __syncthreads();
  float tensor = 1.0f;
  if constexpr (NVFP4) {
    const float top = __uint_as_float(*largest << 16);
    tensor = top > 0.0f ? fmaxf(top / 2688.0f, 1.17549435e-38f) : 1.0f;
    if (blockIdx.x == 0 && blockIdx.y == 0 && tid == 0) *tensor_scale = tensor;
  }
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int item = tid + 256 * k, row = item / 8, chunk = item % 8;
    const int source = source_row[row];
    u32x4_t words = {0, 0, 0, 0};
    if (source >= 0) words = *reinterpret_cast<const u32x4_t*>(x + static_cast<size_t>(source) * dim + d0 + chunk * 8);
#pragma unroll
    for (int i = 0; i < 4; ++i) tile[row][chunk * 4 + i] = words[i];
  }
  __syncthreads();
  const int c = tid % 64, quarter = tid / 64;
  uint32_t bits[32];  // the thread's 32 tokens of column c as bf16 patterns
#pragma unroll
  for (int i = 0; i < 32; ++i) {
    const uint32_t word = tile[32 * quarter + i][c / 2];
    bits[i] = c % 2 ? word >> 16 : word & 0xFFFFu;
  }
  if constexpr (NVFP4) {
#pragma unroll
    for (int block = 0; block < 2; ++block) {
      float largest_of_block = 0.0f;
#pragma unroll
      for (int i = 0; i < 16; ++i) largest_of_block = fmaxf(largest_of_block, fabsf(__uint_as_float(bits[16 * block + i] << 16)));
      const float ratio = (largest_of_block / tensor) / 6.0f;
      uint32_t byte = __builtin_amdgcn_cvt_pk_fp8_f32(fminf(ratio, 448.0f), 0.0f, 0, false) & 0xFFu;
      if (__builtin_amdgcn_cvt_f32_fp8(byte, 0) < ratio) byte = min(byte + 1u, 0x7Eu);
      const float each = __builtin_amdgcn_cvt_f32_fp8(byte, 0);
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float value = __uint_as_float(bits[16 * block + i] << 16);
        const float over_tensor = each > 0.0f ? value / tensor : 0.0f;
        bits[16 * block + i] = __float_as_uint(copysignf(e2m1_scaled(fabsf(over_tensor), each), over_tensor)) >> 16;
      }
    }
  }
  u32x4_t pieces[4];  // 8 tokens each
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int i = 0; i < 4; ++i) pieces[j][i] = bits[8 * j + 2 * i] | (bits[8 * j + 2 * i + 1] << 16);
  if constexpr (BANK) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {  // piece j: atom 2 quarter + j / 2 of the tile's eight, lane group j % 2
      const size_t atom = static_cast<size_t>((d0 + c) / 32) * (tokens / 16) + t0 / 16 + 2 * quarter + j / 2;
      *reinterpret_cast<u32x4_t*>(out + (atom * 64 + 32 * (j % 2) + c % 32) * 16) = pieces[j];
    }
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j) staged[c][(4 * quarter + j) ^ (c & 15)] = pieces[j];
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int item = tid + 256 * k, row = item / 16, chunk = item % 16;
      *reinterpret_cast<u32x4_t*>(out + (static_cast<size_t>(d0 + row) * tokens + t0) * 2 + chunk * 16) = staged[row][chunk ^ (row & 15)];
    }
  }
}

static int transpose_columns(const char* who, bool nvfp4, const void* x, void* out, float* tensor_scale, uint32_t* workspace, int tokens,
                             int dim, int as_bank, void* stream, int rows = -1, const int32_t* offsets = nullptr, int groups = 0,
                             int32_t* padded = nullptr) {
  if (rows < 0) rows = tokens;  // (ragged groups: `rows` of x are written into `tokens` padded ones)
  DEW_REQUIRE(tokens >= 0 && tokens % 128 == 0, "%s: %d tokens are not whole 128s", who, tokens);
  if (offsets) {
    DEW_REQUIRE(groups >= 1 && groups <= kMaxPaddedGroups && padded, "%s: %d groups (at most %d) and their padded offsets", who, groups, kMaxPaddedGroups);
    DEW_REQUIRE(rows >= 0 && static_cast<long long>(tokens) >= static_cast<long long>(rows) + 64ll * groups,
                "%s: %d padded tokens do not hold %d rows in %d groups of whole 64s", who, tokens, rows, groups);
  }
  DEW_REQUIRE(dim >= 128 && dim % 128 == 0, "%s: %d columns (whole 128s)", who, dim);
  DEW_REQUIRE(!nvfp4 || (tensor_scale && workspace), "%s: tensor_scale and the 4-byte workspace must not be null", who);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (nvfp4) {
    hipLaunchKernelGGL(absmax_clear_kernel, dim3(1), dim3(1), 0, s, workspace);
    if (int rc = launched("absmax_clear_kernel")) return rc;
  }
  if (tokens == 0) {
    if (nvfp4) {  // an operand of no tokens: the unit scale
      hipLaunchKernelGGL(quantize_rows_nvfp4_kernel, dim3(1), dim3(64 * kQuantizeWaves), 0, s, static_cast<const bf16_t*>(nullptr), workspace,
                         static_cast<bf16_t*>(nullptr), tensor_scale, 0, 0);
      return launched("quantize_rows_nvfp4_kernel");
    }
    return DEW_MOE_OK;
  }
  DEW_REQUIRE(tokens / 128 <= 65535 * 32, "%s: %d tokens", who, tokens);
  DEW_REQUIRE(x && out && aligned16(x) && aligned16(out), "%s: x and out must not be null and must be 16-byte aligned", who);
  if (nvfp4) {
    const long long chunks = static_cast<long long>(rows) * dim / 8;
    const int blocks = static_cast<int>(min((chunks + 255) / 256, 256ll * 16));
    hipLaunchKernelGGL(absmax_kernel, dim3(blocks), dim3(256), 0, s, static_cast<const bf16_t*>(x), chunks, workspace);
    if (int rc = launched("absmax_kernel")) return rc;
  }
  const dim3 grid(tokens / 128, dim / 64);
  auto launch = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, grid, dim3(256), 0, s, static_cast<const bf16_t*>(x), workspace, static_cast<uint8_t*>(out), tensor_scale, tokens, dim,
                       offsets, groups, padded, rows);
  };
  if (nvfp4 && as_bank) launch(transpose_columns_kernel<true, true>);
  else if (nvfp4) launch(transpose_columns_kernel<true, false>);
  else if (as_bank) launch(transpose_columns_kernel<false, true>);
  else launch(transpose_columns_kernel<false, false>);
  return launched("transpose_columns_kernel");
}

static int quantize_columns(const char* who, bool mx, const void* x, void* codes, void* scales, int tokens, int dim, int as_bank,
                            void* stream) {
  DEW_REQUIRE(tokens >= 0 && tokens % 128 == 0, "%s: %d tokens are not whole 128-token blocks", who, tokens);
  DEW_REQUIRE(dim >= 128 && dim % 128 == 0, "%s: %d columns (whole 128s)", who, dim);
  if (tokens == 0) return DEW_MOE_OK;
  DEW_REQUIRE(tokens / 128 <= 65535 * 32, "%s: %d tokens", who, tokens);
  DEW_REQUIRE(x && codes && scales, "%s: x, codes and scales must not be null", who);
  DEW_REQUIRE(aligned16(x) && aligned16(codes) && aligned16(scales), "%s: x, codes and scales must be 16-byte aligned", who);
  const dim3 grid(tokens / 128, dim / 64);
  hipStream_t s = static_cast<hipStream_t>(stream);
  auto launch = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, grid, dim3(256), 0, s, static_cast<const bf16_t*>(x), static_cast<uint8_t*>(codes),
                       static_cast<uint32_t*>(scales), tokens, dim);
  };
  if (mx && as_bank) launch(quantize_columns_kernel<true, true>);
  else if (mx) launch(quantize_columns_kernel<true, false>);
  else if (as_bank) launch(quantize_columns_kernel<false, true>);
  else launch(quantize_columns_kernel<false, false>);
  return launched("quantize_columns_kernel");
}

}  // namespace dew

extern "C" int dew_moe_transpose_columns(const void* x, void* out, int32_t tokens, int32_t dim, int32_t as_bank, void* stream) {
  return dew::transpose_columns("dew_moe_transpose_columns", false, x, out, nullptr, nullptr, tokens, dim, as_bank, stream);
}

extern "C" int dew_moe_transpose_groups(const void* x, const int32_t* offsets, void* out, int32_t* padded_offsets, int32_t rows,
                                        int32_t padded_tokens, int32_t dim, int32_t groups, int32_t as_bank, void* stream) {
  using namespace dew;
  DEW_REQUIRE(offsets, "dew_moe_transpose_groups: offsets must not be null");
  return transpose_columns("dew_moe_transpose_groups", false, x, out, nullptr, nullptr, padded_tokens, dim, as_bank, stream, rows, offsets, groups,
                           padded_offsets);
}

extern "C" int dew_moe_quantize_columns_nvfp4(const void* x, void* values, float* tensor_scale, uint32_t* workspace, int32_t tokens,
                                              int32_t dim, int32_t as_bank, void* stream) {
  return dew::transpose_columns("dew_moe_quantize_columns_nvfp4", true, x, values, tensor_scale, workspace, tokens, dim, as_bank, stream);
}

extern "C" int dew_moe_quantize_columns_fp8(const void* x, void* codes, void* scales, int32_t tokens, int32_t dim, int32_t as_bank,
                                            void* stream) {
  return dew::quantize_columns("dew_moe_quantize_columns_fp8", false, x, codes, scales, tokens, dim, as_bank, stream);
}

extern "C" int dew_moe_quantize_columns_mxfp8(const void* x, void* codes, void* scales, int32_t tokens, int32_t dim, int32_t as_bank,
                                              void* stream) {
  return dew::quantize_columns("dew_moe_quantize_columns_mxfp8", true, x, codes, scales, tokens, dim, as_bank, stream);
}

extern "C" int dew_moe_quantize_rows_nvfp4(const void* x, void* values, float* tensor_scale, uint32_t* workspace, int32_t rows,
                                           int32_t depth, void* stream) {
  using namespace dew;
  DEW_REQUIRE(rows >= 0 && depth >= 16 && depth % 16 == 0, "dew_moe_quantize_rows_nvfp4: rows %d, depth %d (whole 16s)", rows, depth);
  DEW_REQUIRE(tensor_scale && workspace, "dew_moe_quantize_rows_nvfp4: tensor_scale and the 4-byte workspace must not be null");
  DEW_REQUIRE(rows == 0 || (x && values), "dew_moe_quantize_rows_nvfp4: x and values must not be null");
  DEW_REQUIRE(depth % 8 == 0 && aligned16(x) && aligned16(values), "dew_moe_quantize_rows_nvfp4: x and values must be 16-byte aligned");
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipLaunchKernelGGL(absmax_clear_kernel, dim3(1), dim3(1), 0, s, workspace);
  if (int rc = launched("absmax_clear_kernel")) return rc;
  const long long chunks = static_cast<long long>(rows) * depth / 8;
  if (chunks > 0) {
    const int blocks = static_cast<int>(min((chunks + 255) / 256, 256ll * 16));
    hipLaunchKernelGGL(absmax_kernel, dim3(blocks), dim3(256), 0, s, static_cast<const bf16_t*>(x), chunks, workspace);
    if (int rc = launched("absmax_kernel")) return rc;
  }
  hipLaunchKernelGGL(quantize_rows_nvfp4_kernel, dim3(max(1, (rows + kQuantizeWaves - 1) / kQuantizeWaves)), dim3(64 * kQuantizeWaves), 0, s,
                     static_cast<const bf16_t*>(x), workspace, static_cast<bf16_t*>(values), tensor_scale, rows, depth);
  return launched("quantize_rows_nvfp4_kernel");
}

extern "C" int dew_moe_quantize_rows_mxfp8(const void* x, void* codes, uint8_t* scales, int32_t rows, int32_t depth, void* stream) {
  using namespace dew;
  DEW_REQUIRE(rows >= 0 && depth >= 128 && depth % 128 == 0, "dew_moe_quantize_rows_mxfp8: rows %d, depth %d (whole 128s)", rows, depth);
  if (rows == 0) return DEW_MOE_OK;
  DEW_REQUIRE(x && codes && scales, "dew_moe_quantize_rows_mxfp8: x, codes and scales must not be null");
  DEW_REQUIRE(aligned16(x) && aligned16(codes) && aligned16(scales), "dew_moe_quantize_rows_mxfp8: x, codes and scales must be 16-byte aligned");
  hipLaunchKernelGGL(quantize_rows_mxfp8_kernel, dim3((rows + kQuantizeWaves - 1) / kQuantizeWaves), dim3(64 * kQuantizeWaves), 0,
                     static_cast<hipStream_t>(stream), static_cast<const bf16_t*>(x), static_cast<uint8_t*>(codes), scales, rows, depth);
  return launched("quantize_rows_mxfp8_kernel");
}

extern "C" int dew_moe_quantize_rows_fp8(const void* x, void* codes, uint8_t* scales, int32_t rows, int32_t depth, void* stream) {
  using namespace dew;
  DEW_REQUIRE(rows >= 0 && depth >= 128 && depth % 128 == 0, "dew_moe_quantize_rows_fp8: rows %d, depth %d (whole 128s)", rows, depth);
  if (rows == 0) return DEW_MOE_OK;
  DEW_REQUIRE(x && codes && scales, "dew_moe_quantize_rows_fp8: x, codes and scales must not be null");
  DEW_REQUIRE(aligned16(x) && aligned16(codes) && aligned16(scales), "dew_moe_quantize_rows_fp8: x, codes and scales must be 16-byte aligned");
  const int pitch = (depth / 128 + 15) / 16 * 16;
  hipLaunchKernelGGL(quantize_rows_fp8_kernel, dim3((rows + kQuantizeWaves - 1) / kQuantizeWaves), dim3(64 * kQuantizeWaves), 0,
                     static_cast<hipStream_t>(stream), static_cast<const bf16_t*>(x), static_cast<uint8_t*>(codes), scales, rows, depth,
                     pitch);
  return launched("quantize_rows_fp8_kernel");
}

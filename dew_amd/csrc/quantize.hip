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

}  // namespace dew

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

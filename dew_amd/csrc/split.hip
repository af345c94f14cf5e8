// Activation rows as two FP8 terms for the scaled matrix instructions.
// A bf16 value has 8 significant bits; hi = e4m3(x / s) keeps the first four and lo = e4m3(16 (x / s - hi)) the
// other four, so x = s (hi + lo / 16) exactly, s one power of two per row chosen so that the row's largest
// magnitude lands in [128, 256). e4m3 spans 2^-9 .. 448, so the identity holds for every element within 2^-11 of
// its row's maximum; a smaller one loses bits worth at most 2^-21 of that maximum. The grouped GEMM multiplies the
// two terms by the FP4 codes with v_mfma_scale_f32_32x32x64_f8f6f4. Measured on gfx950: of the instruction's 64
// depths, an 8-bit A operand's lane group g (lanes 32 g .. 32 g + 31) holds depths 16 g .. 16 g + 15 in its first
// 16 bytes and 32 + 16 g .. 47 + 16 g in its last 16 (a 4-bit B operand's holds 32 g .. 32 g + 31). Each 64 depths
// of a row are therefore stored as four 32-byte pieces, [group 0 hi][group 0 lo][group 1 hi][group 1 lo], each in
// its lane's operand order: the same 2 bytes per element and the same row pitch as the bf16 source.
#include "common.h"

namespace dew {

typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2_t;

constexpr int kSplitWaves = 4;  // rows per 256-thread block

__global__ __launch_bounds__(64 * kSplitWaves) void split_rows_kernel(const bf16_t* __restrict__ x, uint8_t* __restrict__ split,
                                                                     uint8_t* __restrict__ scale, int rows, int depth) {
  const int lane = threadIdx.x % 64;
  const int row = blockIdx.x * kSplitWaves + threadIdx.x / 64;
  if (row >= rows) return;
  const bf16_t* source = x + static_cast<size_t>(row) * depth;
  // the row's largest exponent field (the sign bit dropped; NaN and infinity count as the largest finite one)
  uint32_t largest = 0;
  for (int chunk = lane; chunk < depth / 8; chunk += 64) {
    const u32x4_t words = *reinterpret_cast<const u32x4_t*>(source + chunk * 8);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      largest = max(largest, (words[i] >> 7) & 0xFFu);
      largest = max(largest, (words[i] >> 23) & 0xFFu);
    }
  }
#pragma unroll
  for (int offset = 32; offset >= 1; offset >>= 1) largest = max(largest, static_cast<uint32_t>(__shfl_xor(static_cast<int>(largest), offset, 64)));
  // largest magnitude in [2^(field - 127), 2^(field - 126)): dividing by 2^(field - 134) brings it to [128, 256)
  const int field = min(max(static_cast<int>(largest), 16), 254);
  const int hi_byte = field - 7;  // e8m0 of the hi term's scale 2^(field - 134); the lo term's is 4 less
  if (lane == 0) scale[row] = static_cast<uint8_t>(hi_byte);
  const float inverse = __uint_as_float(static_cast<uint32_t>(254 - hi_byte) << 23);  // 2^-(hi_byte - 127)
  uint8_t* target = split + static_cast<size_t>(row) * depth * 2;
  for (int chunk = lane; chunk < depth / 8; chunk += 64) {
    const u32x4_t words = *reinterpret_cast<const u32x4_t*>(source + chunk * 8);
    float v[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[2 * i] = __uint_as_float(words[i] << 16) * inverse;
      v[2 * i + 1] = __uint_as_float(words[i] & 0xFFFF0000u) * inverse;
    }
    uint32_t hi[2], lo[2];
    float rest[8];
#pragma unroll
    for (int w = 0; w < 2; ++w) {  // four values a word
      hi[w] = __builtin_amdgcn_cvt_pk_fp8_f32(v[4 * w], v[4 * w + 1], 0, false);
      hi[w] = __builtin_amdgcn_cvt_pk_fp8_f32(v[4 * w + 2], v[4 * w + 3], hi[w], true);
      const auto first = __builtin_amdgcn_cvt_pk_f32_fp8(hi[w], false), second = __builtin_amdgcn_cvt_pk_f32_fp8(hi[w], true);
      rest[4 * w] = (v[4 * w] - first[0]) * 16.0f;
      rest[4 * w + 1] = (v[4 * w + 1] - first[1]) * 16.0f;
      rest[4 * w + 2] = (v[4 * w + 2] - second[0]) * 16.0f;
      rest[4 * w + 3] = (v[4 * w + 3] - second[1]) * 16.0f;
      lo[w] = __builtin_amdgcn_cvt_pk_fp8_f32(rest[4 * w], rest[4 * w + 1], 0, false);
      lo[w] = __builtin_amdgcn_cvt_pk_fp8_f32(rest[4 * w + 2], rest[4 * w + 3], lo[w], true);
    }
    // depths 8 chunk .. 8 chunk + 7: eighth `within` of their 64; halves 0-31 / 32-63, sixteenths 16 g .. 16 g + 15
    const int within = chunk % 8, half = within / 4, group = (within % 4) / 2, piece = within % 2;
    uint8_t* block = target + (chunk / 8) * 128 + group * 64 + half * 16 + piece * 8;
    *reinterpret_cast<u32x2_t*>(block) = u32x2_t{hi[0], hi[1]};
    *reinterpret_cast<u32x2_t*>(block + 32) = u32x2_t{lo[0], lo[1]};
  }
}

}  // namespace dew

extern "C" int dew_moe_split_rows(const void* x, void* split, uint8_t* scale, int32_t rows, int32_t depth, void* stream) {
  using namespace dew;
  DEW_REQUIRE(rows >= 0 && depth >= 64 && depth % 64 == 0, "dew_moe_split_rows: rows %d, depth %d (whole 64s)", rows, depth);
  if (rows == 0) return DEW_MOE_OK;
  DEW_REQUIRE(x && split && scale, "dew_moe_split_rows: x, split and scale must not be null");
  DEW_REQUIRE(aligned16(x) && aligned16(split), "dew_moe_split_rows: x and split must be 16-byte aligned");
  hipLaunchKernelGGL(split_rows_kernel, dim3((rows + kSplitWaves - 1) / kSplitWaves), dim3(64 * kSplitWaves), 0,
                     static_cast<hipStream_t>(stream), static_cast<const bf16_t*>(x), static_cast<uint8_t*>(split), scale, rows, depth);
  return launched("split_rows_kernel");
}

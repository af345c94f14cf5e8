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

// HELD = the 16-byte chunks a lane holds of its row (depth = 512 HELD, up to 4096): the row is then read once, with
// loads that leave nothing in the caches (nothing reads it again), and converted from registers; 0 = any depth, the row
// read twice (the second time from the cache).
template <int HELD>
__global__ __launch_bounds__(64 * kSplitWaves) void split_rows_kernel(const bf16_t* __restrict__ x, uint8_t* __restrict__ split,
                                                                     uint8_t* __restrict__ scale, int rows, int depth) {
  const int lane = threadIdx.x % 64;
  const int row = blockIdx.x * kSplitWaves + threadIdx.x / 64;
  if (row >= rows) return;
  const bf16_t* source = x + static_cast<size_t>(row) * depth;
  // the row's largest exponent field (the sign bit dropped; NaN and infinity count as the largest finite one)
  uint32_t largest = 0;
  u32x4_t held[HELD > 0 ? HELD : 1];
  if constexpr (HELD > 0) {
#pragma unroll
    for (int c = 0; c < HELD; ++c) held[c] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(source + (lane + 64 * c) * 8));
#pragma unroll
    for (int c = 0; c < HELD; ++c) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        largest = max(largest, (held[c][i] >> 7) & 0xFFu);
        largest = max(largest, (held[c][i] >> 23) & 0xFFu);
      }
    }
  } else {
    for (int chunk = lane; chunk < depth / 8; chunk += 64) {
      const u32x4_t words = *reinterpret_cast<const u32x4_t*>(source + chunk * 8);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        largest = max(largest, (words[i] >> 7) & 0xFFu);
        largest = max(largest, (words[i] >> 23) & 0xFFu);
      }
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
  auto convert = [&](int chunk, const u32x4_t words) __attribute__((always_inline)) {
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
  };
  if constexpr (HELD > 0) {
#pragma unroll
    for (int c = 0; c < HELD; ++c) convert(lane + 64 * c, held[c]);
  } else {
    for (int chunk = lane; chunk < depth / 8; chunk += 64) convert(chunk, *reinterpret_cast<const u32x4_t*>(source + chunk * 8));
  }
}

// The same rows with the second term in FP6: x = s hi + t lo, hi = e4m3(x / s) under the row's scale s as above and
// lo = e2m3((x - s hi) / t) under t, one power of two for every 32 depths: the least that brings the block's largest
// remainder within e2m3's range (7.5). A remainder is a multiple of its element's bf16 spacing; e2m3 holds it exactly
// where that spacing is at least t / 8, that is for the elements within two binades of their block's largest
// magnitude, and to within t / 16 (2^-10 of the block's largest magnitude, or less) for the smaller ones. A lane
// converts one block: v_cvt_scalef32_2xpk16_fp6_f32 packs its 32 remainders (the even depths in its first operand,
// the odd ones in its second: it interleaves them). A row's 64 depths are 128 bytes, [group 0: 32 bytes of hi codes,
// 24 of lo codes, the lo scale's e8m0 byte in a dword, 4 unused][group 1 alike]; the hi codes of lane group g are depths
// 16 g .. 16 g + 15 and 32 + 16 g .. 47 + 16 g, its lo codes depths 32 g .. 32 g + 31 (the instruction's own orders).
typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef __attribute__((ext_vector_type(6))) uint32_t u32x6_t;

__global__ __launch_bounds__(64 * kSplitWaves) void split_rows_fp6_kernel(const bf16_t* __restrict__ x, uint8_t* __restrict__ split,
                                                                         uint8_t* __restrict__ scale, int rows, int depth) {
  const int lane = threadIdx.x % 64;
  const int row = blockIdx.x * kSplitWaves + threadIdx.x / 64;
  if (row >= rows) return;
  const bf16_t* source = x + static_cast<size_t>(row) * depth;
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
  const int field = min(max(static_cast<int>(largest), 16), 254);
  const int hi_byte = field - 7;
  if (lane == 0) scale[row] = static_cast<uint8_t>(hi_byte);
  const float inverse = __uint_as_float(static_cast<uint32_t>(254 - hi_byte) << 23);  // 1 / s
  uint8_t* target = split + static_cast<size_t>(row) * depth * 2;
  for (int block = lane; block < depth / 32; block += 64) {
    float rest[32];
    uint32_t hi[8];
    float most = 0.0f;
#pragma unroll
    for (int piece = 0; piece < 4; ++piece) {  // 8 depths a piece
      const u32x4_t words = *reinterpret_cast<const u32x4_t*>(source + block * 32 + piece * 8);
      float v[8];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        v[2 * i] = __uint_as_float(words[i] << 16) * inverse;
        v[2 * i + 1] = __uint_as_float(words[i] & 0xFFFF0000u) * inverse;
      }
#pragma unroll
      for (int w = 0; w < 2; ++w) {
        uint32_t codes = __builtin_amdgcn_cvt_pk_fp8_f32(v[4 * w], v[4 * w + 1], 0, false);
        codes = __builtin_amdgcn_cvt_pk_fp8_f32(v[4 * w + 2], v[4 * w + 3], codes, true);
        hi[2 * piece + w] = codes;
        const auto first = __builtin_amdgcn_cvt_pk_f32_fp8(codes, false), second = __builtin_amdgcn_cvt_pk_f32_fp8(codes, true);
        rest[8 * piece + 4 * w] = v[4 * w] - first[0];
        rest[8 * piece + 4 * w + 1] = v[4 * w + 1] - first[1];
        rest[8 * piece + 4 * w + 2] = v[4 * w + 2] - second[0];
        rest[8 * piece + 4 * w + 3] = v[4 * w + 3] - second[1];
      }
    }
#pragma unroll
    for (int i = 0; i < 32; ++i) most = fmaxf(most, fabsf(rest[i]));
    // t / s = the least power of two with most / (t / s) <= 7.5 = 1.875 * 4: most's exponent less 2, one more where its
    // significand is above 1.875 (a NaN or infinite element leaves NaN remainders: the codes are then whatever the
    // conversion makes of them, as the first term's are)
    const uint32_t bits = __float_as_uint(most);
    int power = static_cast<int>(bits >> 23) - 127 - 2 + ((bits & 0x7FFFFFu) > 0x700000u ? 1 : 0);
    power = max(power, max(-126, 1 - hi_byte));  // (t and t / s stay normal powers of two; a block of zero remainders lands here)
    const float t_over_s = __uint_as_float(static_cast<uint32_t>(power + 127) << 23);
    f32x16_t even, odd;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      even[i] = rest[2 * i];
      odd[i] = rest[2 * i + 1];
    }
    const u32x6_t lo = __builtin_amdgcn_cvt_scalef32_2xpk16_fp6_f32(even, odd, t_over_s);
    const int lo_byte = min(max(hi_byte + power, 1), 254);  // e8m0 of t = s * 2^power
    const int half = block % 2;                                    // which 32 of the step's 64 depths
    uint8_t* step = target + (block / 2) * 128;
    // hi: the block's first 16 depths go to lane group 0's codes, its last 16 to group 1's, each at 16 * half
    *reinterpret_cast<u32x4_t*>(step + 16 * half) = u32x4_t{hi[0], hi[1], hi[2], hi[3]};
    *reinterpret_cast<u32x4_t*>(step + 64 + 16 * half) = u32x4_t{hi[4], hi[5], hi[6], hi[7]};
    uint8_t* lo_at = step + 64 * half + 32;
    *reinterpret_cast<u32x4_t*>(lo_at) = u32x4_t{lo[0], lo[1], lo[2], lo[3]};
    *reinterpret_cast<u32x4_t*>(lo_at + 16) = u32x4_t{lo[4], lo[5], static_cast<uint32_t>(lo_byte), 0u};
  }
}

// Both terms in FP6: x = s hi + t lo with hi = e2m3(x / s) and lo = e2m3((x - s hi) / t), s and t each one power of two for
// every 32 depths: the least that brings the block's largest magnitude (s), then its largest remainder (t), within
// e2m3's range (7.5). Two FP6 x FP4 instructions take the time of one FP8 x FP4 instruction, half of what the two e4m3
// terms take. e2m3 holds four significant bits in its upper three binades and steps of an eighth of its scale below, so
// an element within two binades of its block's largest is held exactly (four bits in each term) and any other to within
// 2^-10 of that largest magnitude. There is no scale a row: both terms' scales lie with their codes. A row's 64 depths are
// 128 bytes, [group 0: 24 bytes of hi codes, hi's e8m0 byte in a dword, 4 unused, 24 bytes of lo codes, lo's, 4 unused]
// [group 1 alike], lane group g holding depths 32 g .. 32 g + 31 (the 6-bit operand's own order).
typedef __attribute__((ext_vector_type(32))) float f32x32_t;

__device__ __forceinline__ float e2m3_block_scale(float most) {
  // the least power of two t with most / t <= 7.5 = 1.875 * 4: most's exponent less 2, one more where its significand is
  // above 1.875; kept a normal power of two whose e8m0 byte is 1 .. 254 (a block of zeros lands on the least)
  const uint32_t bits = __float_as_uint(most);
  int power = static_cast<int>(bits >> 23) - 127 - 2 + ((bits & 0x7FFFFFu) > 0x700000u ? 1 : 0);
  power = min(max(power, -126), 127);
  return __uint_as_float(static_cast<uint32_t>(power + 127) << 23);
}

__global__ __launch_bounds__(64 * kSplitWaves) void split_rows_e2m3_pair_kernel(const bf16_t* __restrict__ x, uint8_t* __restrict__ split,
                                                                               int rows, int depth) {
  const int lane = threadIdx.x % 64;
  const int row = blockIdx.x * kSplitWaves + threadIdx.x / 64;
  if (row >= rows) return;
  const bf16_t* source = x + static_cast<size_t>(row) * depth;
  uint8_t* target = split + static_cast<size_t>(row) * depth * 2;
  for (int block = lane; block < depth / 32; block += 64) {
    float rest[32];
#pragma unroll
    for (int piece = 0; piece < 4; ++piece) {  // 8 depths a piece
      const u32x4_t words = *reinterpret_cast<const u32x4_t*>(source + block * 32 + piece * 8);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        rest[8 * piece + 2 * i] = __uint_as_float(words[i] << 16);
        rest[8 * piece + 2 * i + 1] = __uint_as_float(words[i] & 0xFFFF0000u);
      }
    }
    uint8_t* at = target + (block / 2) * 128 + (block % 2) * 64;  // the step's 128 bytes, the lane group's 64 of them
#pragma unroll
    for (int term = 0; term < 2; ++term) {
      float most = 0.0f;
#pragma unroll
      for (int i = 0; i < 32; ++i) most = fmaxf(most, fabsf(rest[i]));
      const float scale = e2m3_block_scale(most);
      f32x16_t even, odd;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        even[i] = rest[2 * i];
        odd[i] = rest[2 * i + 1];
      }
      const u32x6_t codes = __builtin_amdgcn_cvt_scalef32_2xpk16_fp6_f32(even, odd, scale);
      if (term == 0) {  // what the first term holds, as the matrix instruction will read it, leaves the remainder
        const f32x32_t held = __builtin_amdgcn_cvt_scalef32_pk32_f32_fp6(codes, scale);
#pragma unroll
        for (int i = 0; i < 32; ++i) rest[i] -= held[i];
      }
      *reinterpret_cast<u32x4_t*>(at + 32 * term) = u32x4_t{codes[0], codes[1], codes[2], codes[3]};
      *reinterpret_cast<u32x4_t*>(at + 32 * term + 16) = u32x4_t{codes[4], codes[5], __float_as_uint(scale) >> 23, 0u};
    }
  }
}

// Activation rows as f16 for the f16 matrix instruction (general NVFP4 banks, whose code x e4m3-scale products are exact in
// f16 and cost the vector unit half of what their bf16 form costs): x = 2^s f, one power of two per row chosen so that the
// row's largest magnitude lands in [2^15, 2^16), under f16's largest finite value. A bf16 value has 8 significant bits and
// f16 holds 11, so f is exact for every element within 2^-29 of its row's largest magnitude (f16's normal range) and loses
// bits only below that, at most 2^-40 of the largest magnitude. The row's scale is stored as the e8m0 byte of 2^s. Same
// two bytes an element and the same row pitch as the bf16 source.
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));

__global__ __launch_bounds__(64 * kSplitWaves) void rows_f16_kernel(const bf16_t* __restrict__ x, uint16_t* __restrict__ halves,
                                                                   uint8_t* __restrict__ scale, int rows, int depth) {
  const int lane = threadIdx.x % 64;
  const int row = blockIdx.x * kSplitWaves + threadIdx.x / 64;
  if (row >= rows) return;
  const bf16_t* source = x + static_cast<size_t>(row) * depth;
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
  // largest magnitude in [2^(field - 127), 2^(field - 126)): times 2^(142 - field) it lies in [2^15, 2^16). The byte
  // (field - 15: the e8m0 of 2^s) and its inverse stay normal powers of two; NaN and infinity count as the largest finite.
  const int field = min(max(static_cast<int>(largest), 16), 254);
  const int byte = field - 15;
  if (lane == 0) scale[row] = static_cast<uint8_t>(byte);
  const float inverse = __uint_as_float(static_cast<uint32_t>(254 - byte) << 23);  // 2^-s
  uint16_t* target = halves + static_cast<size_t>(row) * depth;
  for (int chunk = lane; chunk < depth / 8; chunk += 64) {
    const u32x4_t words = *reinterpret_cast<const u32x4_t*>(source + chunk * 8);
    u32x4_t packed;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const f16x2_t pair = {static_cast<_Float16>(__uint_as_float(words[i] << 16) * inverse),
                            static_cast<_Float16>(__uint_as_float(words[i] & 0xFFFF0000u) * inverse)};
      packed[i] = __builtin_bit_cast(uint32_t, pair);
    }
    *reinterpret_cast<u32x4_t*>(target + chunk * 8) = packed;
  }
}

}  // namespace dew

extern "C" int dew_moe_split_rows_fp6(const void* x, void* split, uint8_t* scale, int32_t rows, int32_t depth, void* stream) {
  using namespace dew;
  DEW_REQUIRE(rows >= 0 && depth >= 64 && depth % 64 == 0, "dew_moe_split_rows_fp6: rows %d, depth %d (whole 64s)", rows, depth);
  if (rows == 0) return DEW_MOE_OK;
  DEW_REQUIRE(x && split && scale, "dew_moe_split_rows_fp6: x, split and scale must not be null");
  DEW_REQUIRE(aligned16(x) && aligned16(split), "dew_moe_split_rows_fp6: x and split must be 16-byte aligned");
  hipLaunchKernelGGL(split_rows_fp6_kernel, dim3((rows + kSplitWaves - 1) / kSplitWaves), dim3(64 * kSplitWaves), 0,
                     static_cast<hipStream_t>(stream), static_cast<const bf16_t*>(x), static_cast<uint8_t*>(split), scale, rows, depth);
  return launched("split_rows_fp6_kernel");
}

extern "C" int dew_moe_split_rows(const void* x, void* split, uint8_t* scale, int32_t rows, int32_t depth, void* stream) {
  using namespace dew;
  DEW_REQUIRE(rows >= 0 && depth >= 64 && depth % 64 == 0, "dew_moe_split_rows: rows %d, depth %d (whole 64s)", rows, depth);
  if (rows == 0) return DEW_MOE_OK;
  DEW_REQUIRE(x && split && scale, "dew_moe_split_rows: x, split and scale must not be null");
  DEW_REQUIRE(aligned16(x) && aligned16(split), "dew_moe_split_rows: x and split must be 16-byte aligned");
  auto launch = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, dim3((rows + kSplitWaves - 1) / kSplitWaves), dim3(64 * kSplitWaves), 0,
                       static_cast<hipStream_t>(stream), static_cast<const bf16_t*>(x), static_cast<uint8_t*>(split), scale, rows, depth);
  };
  switch (depth) {
    case 1024: launch(split_rows_kernel<2>); break;
    case 2048: launch(split_rows_kernel<4>); break;
    case 4096: launch(split_rows_kernel<8>); break;
    default: launch(split_rows_kernel<0>); break;
  }
  return launched("split_rows_kernel");
}

extern "C" int dew_moe_rows_f16(const void* x, void* halves, uint8_t* scale, int32_t rows, int32_t depth, void* stream) {
  using namespace dew;
  DEW_REQUIRE(rows >= 0 && depth >= 64 && depth % 64 == 0, "dew_moe_rows_f16: rows %d, depth %d (whole 64s)", rows, depth);
  if (rows == 0) return DEW_MOE_OK;
  DEW_REQUIRE(x && halves && scale, "dew_moe_rows_f16: x, halves and scale must not be null");
  DEW_REQUIRE(aligned16(x) && aligned16(halves), "dew_moe_rows_f16: x and halves must be 16-byte aligned");
  hipLaunchKernelGGL(rows_f16_kernel, dim3((rows + kSplitWaves - 1) / kSplitWaves), dim3(64 * kSplitWaves), 0,
                     static_cast<hipStream_t>(stream), static_cast<const bf16_t*>(x), static_cast<uint16_t*>(halves), scale, rows, depth);
  return launched("rows_f16_kernel");
}

extern "C" int dew_moe_split_rows_e2m3_pair(const void* x, void* split, int32_t rows, int32_t depth, void* stream) {
  using namespace dew;
  DEW_REQUIRE(rows >= 0 && depth >= 64 && depth % 64 == 0, "dew_moe_split_rows_e2m3_pair: rows %d, depth %d (whole 64s)", rows, depth);
  if (rows == 0) return DEW_MOE_OK;
  DEW_REQUIRE(x && split, "dew_moe_split_rows_e2m3_pair: x and split must not be null");
  DEW_REQUIRE(aligned16(x) && aligned16(split), "dew_moe_split_rows_e2m3_pair: x and split must be 16-byte aligned");
  hipLaunchKernelGGL(split_rows_e2m3_pair_kernel, dim3((rows + kSplitWaves - 1) / kSplitWaves), dim3(64 * kSplitWaves), 0,
                     static_cast<hipStream_t>(stream), static_cast<const bf16_t*>(x), static_cast<uint8_t*>(split), rows, depth);
  return launched("split_rows_e2m3_pair_kernel");
}

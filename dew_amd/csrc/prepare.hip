// One-time re-layout of a quantized expert bank from the reference's storage layout into MFMA-fragment
// order ("atoms"): every 16-byte piece a lane feeds the matrix cores is contiguous, and a wavefront's 64
// pieces are one coalesced 1 KiB read. The re-layout is a permutation of the codes and is exact.
//
//   FP8 atom  : 32 n x 32 k bytes. Lane l = 32 g + n holds k = 16 g .. 16 g + 15 of column n.
//   FP4 atom  : 32 n x 64 k nibbles. Lane l = 32 g + n holds k = 32 g .. 32 g + 31 (byte j: low nibble
//               k = 32 g + 2 j, high nibble k = 32 g + 2 j + 1) - one MX block, two NVFP4 blocks.
//   FP4 scales: per atom 64 lanes x 2 e4m3 bytes: the scales of the lane's two 16-deep blocks.
//   Atom order: [E][N / 32][K / atom_k], so one 32-column strip's whole depth is contiguous.
//
// The NVFP4 source words are K-major, in the staged depth order (word w of a 128-deep group holds depths
// 128 G + 16 j + w, j = 0..7; reference src/dew/nn/kernels/templates/gemm/packed.py:27-33) and passed
// through a GF(2) encoder; they are decoded with the 8-step form of src/dew/algebra/bits.py:696-700.
#include "common.h"

namespace dew {

__global__ __launch_bounds__(256) void prepare_fp8_kernel(const uint8_t* __restrict__ codes, uint8_t* __restrict__ out,
                                                          int experts, int depth, int width) {
  const int k_atoms = depth / 32, n_atoms = width / 32;
  const long long total = static_cast<long long>(experts) * n_atoms * k_atoms * 64;
  for (long long item = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x; item < total;
       item += static_cast<long long>(gridDim.x) * blockDim.x) {
    const int lane = static_cast<int>(item % 64);
    const long long atom = item / 64;
    const int ka = static_cast<int>(atom % k_atoms);
    const int na = static_cast<int>((atom / k_atoms) % n_atoms);
    const int e = static_cast<int>(atom / (static_cast<long long>(k_atoms) * n_atoms));
    const int n = na * 32 + lane % 32;
    const int k0 = ka * 32 + 16 * (lane / 32);
    const uint8_t* src = codes + (static_cast<size_t>(e) * depth + k0) * width + n;
    uint32_t words[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      uint32_t word = 0;
#pragma unroll
      for (int b = 0; b < 4; ++b) word |= static_cast<uint32_t>(src[static_cast<size_t>(4 * q + b) * width]) << (8 * b);
      words[q] = word;
    }
    *reinterpret_cast<uint4*>(out + item * 16) = make_uint4(words[0], words[1], words[2], words[3]);
  }
}

// bf16 matrices [E][K][N] -> atoms of 32 n x 16 k: lane 32 g + n holds depths 8 g .. 8 g + 7 of column n, the 16 bytes
// the bf16 matrix instruction takes from it for one 16-deep slice. Atom order [E][N / 32][K / 16].
__global__ __launch_bounds__(256) void prepare_bf16_kernel(const uint16_t* __restrict__ weights, uint8_t* __restrict__ out,
                                                           int experts, int depth, int width) {
  const int k_atoms = depth / 16, n_atoms = width / 32;
  const long long total = static_cast<long long>(experts) * n_atoms * k_atoms * 64;
  for (long long item = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x; item < total;
       item += static_cast<long long>(gridDim.x) * blockDim.x) {
    const int lane = static_cast<int>(item % 64);
    const long long atom = item / 64;
    const int ka = static_cast<int>(atom % k_atoms);
    const int na = static_cast<int>((atom / k_atoms) % n_atoms);
    const int e = static_cast<int>(atom / (static_cast<long long>(k_atoms) * n_atoms));
    const uint16_t* src = weights + (static_cast<size_t>(e) * depth + ka * 16 + 8 * (lane / 32)) * width + na * 32 + lane % 32;
    uint32_t words[4];
#pragma unroll
    for (int q = 0; q < 4; ++q)
      words[q] = static_cast<uint32_t>(src[static_cast<size_t>(2 * q) * width]) |
                 (static_cast<uint32_t>(src[static_cast<size_t>(2 * q + 1) * width]) << 16);
    *reinterpret_cast<uint4*>(out + item * 16) = make_uint4(words[0], words[1], words[2], words[3]);
  }
}

// The same atoms from matrices held K-major, [E][N][K] (a bf16 bank read as its transpose): a lane's 8 depths are 16
// contiguous bytes of its column's row.
__global__ __launch_bounds__(256) void prepare_bf16_kmajor_kernel(const uint16_t* __restrict__ weights, uint8_t* __restrict__ out,
                                                                  int experts, int depth, int width) {
  const int k_atoms = depth / 16, n_atoms = width / 32;
  const long long total = static_cast<long long>(experts) * n_atoms * k_atoms * 64;
  for (long long item = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x; item < total;
       item += static_cast<long long>(gridDim.x) * blockDim.x) {
    const int lane = static_cast<int>(item % 64);
    const long long atom = item / 64;
    const int ka = static_cast<int>(atom % k_atoms);
    const int na = static_cast<int>((atom / k_atoms) % n_atoms);
    const int e = static_cast<int>(atom / (static_cast<long long>(k_atoms) * n_atoms));
    const uint16_t* src = weights + (static_cast<size_t>(e) * width + na * 32 + lane % 32) * depth + ka * 16 + 8 * (lane / 32);
    *reinterpret_cast<uint4*>(out + item * 16) = *reinterpret_cast<const uint4*>(src);
  }
}

// The eight E2M1 nibbles of a stored word (sign in bit 3), code j at bits 4 j of the result.
__device__ __forceinline__ uint32_t nvfp4_natural_word(uint32_t s) {
  const uint32_t mask = 0x81C081C0u;
  const uint32_t v1 = (s >> 6) | (s << 26);
  const uint32_t regs[4] = {(s ^ v1) & mask, (s ^ (s << 6)) & mask, (s ^ (v1 << 2)) & mask, (s << 2) & mask};
  uint32_t natural = 0;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint32_t low = regs[i] & 0xFFFFu, high = regs[i] >> 16;
    natural |= (((low >> 6) & 7u) | ((low >> 15) << 3)) << (8 * i);
    natural |= (((high >> 6) & 7u) | ((high >> 15) << 3)) << (8 * i + 4);
  }
  return natural;
}

// One thread per (expert, column, 128-deep group): 16 words in, 4 runs of 32 natural-order nibbles out.
__global__ __launch_bounds__(256) void prepare_nvfp4_codes_kernel(const uint32_t* __restrict__ words,
                                                                  uint8_t* __restrict__ out, int experts, int depth,
                                                                  int width) {
  const int groups = depth / 128, n_atoms = width / 32, k_atoms = depth / 64;
  const long long total = static_cast<long long>(experts) * width * groups;
  for (long long item = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x; item < total;
       item += static_cast<long long>(gridDim.x) * blockDim.x) {
    // consecutive threads take consecutive columns, so their 16-byte writes fill an atom's lanes in order
    const int n = static_cast<int>(item % width);
    const int group = static_cast<int>((item / width) % groups);
    const int e = static_cast<int>(item / (static_cast<long long>(width) * groups));
    const uint32_t* src = words + (static_cast<size_t>(e) * width + n) * (depth / 8) + group * 16;
    uint32_t natural[16];  // natural[w] holds code j of word w at bits 4 j: depth 16 j + w of the group
#pragma unroll
    for (int w = 0; w < 16; ++w) natural[w] = nvfp4_natural_word(src[w]);
#pragma unroll
    for (int h = 0; h < 4; ++h) {  // run h = depths 32 h .. 32 h + 31 of the group
      uint32_t packed[4] = {0, 0, 0, 0};
#pragma unroll
      for (int b = 0; b < 16; ++b) {  // byte b: depths 32 h + 2 b (low), + 1 (high); depth = 16 j + w
        const int j = 2 * h + b / 8;
        const int w = 2 * (b % 8);
        const uint32_t low = (natural[w] >> (4 * j)) & 15u, high = (natural[w + 1] >> (4 * j)) & 15u;
        packed[b / 4] |= (low | (high << 4)) << (8 * (b % 4));
      }
      const int ka = 2 * group + h / 2;
      const int lane = 32 * (h % 2) + n % 32;
      const size_t atom = (static_cast<size_t>(e) * n_atoms + n / 32) * k_atoms + ka;
      *reinterpret_cast<uint4*>(out + atom * kAtomBytes + lane * 16) = make_uint4(packed[0], packed[1], packed[2], packed[3]);
    }
  }
}

// MXFP8 (K-major codes [E][N][K], scales [E][N][K / 32]): the same 32 n x 32 k atoms as the FP8 banks', a lane's 16
// bytes contiguous in its column's row of the source; the scales as [E][N / 32][K / 128][32 columns][4 bytes], so that
// a 32-column tile's scales of one 128-deep step are one 128-byte line.
__global__ __launch_bounds__(256) void prepare_mxfp8_kernel(const uint8_t* __restrict__ codes, const uint8_t* __restrict__ scales,
                                                            uint8_t* __restrict__ out, uint32_t* __restrict__ scales_out, int experts,
                                                            int depth, int width) {
  const int k_atoms = depth / 32, n_atoms = width / 32;
  const long long total = static_cast<long long>(experts) * n_atoms * k_atoms * 64;
  for (long long item = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x; item < total;
       item += static_cast<long long>(gridDim.x) * blockDim.x) {
    const int lane = static_cast<int>(item % 64);
    const long long atom = item / 64;
    const int ka = static_cast<int>(atom % k_atoms);
    const int na = static_cast<int>((atom / k_atoms) % n_atoms);
    const int e = static_cast<int>(atom / (static_cast<long long>(k_atoms) * n_atoms));
    const int n = na * 32 + lane % 32;
    const size_t column = static_cast<size_t>(e) * width + n;
    *reinterpret_cast<uint4*>(out + item * 16) = *reinterpret_cast<const uint4*>(codes + column * depth + ka * 32 + 16 * (lane / 32));
    if (ka % 4 == 0 && lane < 32)  // the column's four scale bytes of this 128-deep step
      scales_out[((static_cast<size_t>(e) * n_atoms + na) * (depth / 128) + ka / 4) * 32 + lane] =
          *reinterpret_cast<const uint32_t*>(scales + column * (depth / 32) + ka);
  }
}

// Also notes in *general whether any scale is not a normal power of two (mantissa bits set, or a zero or
// subnormal exponent).
__global__ __launch_bounds__(256) void prepare_nvfp4_scales_kernel(const uint8_t* __restrict__ scales,
                                                                   uint16_t* __restrict__ out, int experts, int depth,
                                                                   int width, uint32_t* __restrict__ general) {
  const int n_atoms = width / 32, k_atoms = depth / 64;
  const long long total = static_cast<long long>(experts) * n_atoms * k_atoms * 64;
  for (long long item = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x; item < total;
       item += static_cast<long long>(gridDim.x) * blockDim.x) {
    const int lane = static_cast<int>(item % 64);
    const long long atom = item / 64;
    const int ka = static_cast<int>(atom % k_atoms);
    const int na = static_cast<int>((atom / k_atoms) % n_atoms);
    const int e = static_cast<int>(atom / (static_cast<long long>(k_atoms) * n_atoms));
    const int n = na * 32 + lane % 32;
    const uint8_t* src = scales + (static_cast<size_t>(e) * width + n) * (depth / 16) + ka * 4 + 2 * (lane / 32);
    out[item] = static_cast<uint16_t>(src[0]) | (static_cast<uint16_t>(src[1]) << 8);
    if ((src[0] & 7) || (src[1] & 7) || !(src[0] & 0x78) || !(src[1] & 0x78)) atomicOr(general, 1u);
  }
}

// FP8 codes held K-major, [E][N][K], as a DeepSeek-style checkpoint stores each expert's `weight [out, in]`
// (src/dew/interop/codecs.py:670-703): the same 32 n x 32 k atoms, a lane's 16 bytes contiguous in the source.
__global__ __launch_bounds__(256) void prepare_fp8_kmajor_kernel(const uint8_t* __restrict__ codes, uint8_t* __restrict__ out,
                                                                 int experts, int depth, int width) {
  const int k_atoms = depth / 32, n_atoms = width / 32;
  const long long total = static_cast<long long>(experts) * n_atoms * k_atoms * 64;
  for (long long item = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x; item < total;
       item += static_cast<long long>(gridDim.x) * blockDim.x) {
    const int lane = static_cast<int>(item % 64);
    const long long atom = item / 64;
    const int ka = static_cast<int>(atom % k_atoms);
    const int na = static_cast<int>((atom / k_atoms) % n_atoms);
    const int e = static_cast<int>(atom / (static_cast<long long>(k_atoms) * n_atoms));
    const size_t column = static_cast<size_t>(e) * width + na * 32 + lane % 32;
    *reinterpret_cast<uint4*>(out + item * 16) = *reinterpret_cast<const uint4*>(codes + column * depth + ka * 32 + 16 * (lane / 32));
  }
}

// The 128 x 128 block scales into the prepared buffer as [E][K / 128][N / 128] fp32, from that layout or, `kmajor`,
// from a checkpoint's `weight_scale_inv [E][N / 128][K / 128]`.
__global__ __launch_bounds__(256) void prepare_block_scales_kernel(const float* __restrict__ scales, float* __restrict__ out,
                                                                   int experts, int depth_blocks, int width_blocks, int kmajor) {
  const int total = experts * depth_blocks * width_blocks;
  for (int item = blockIdx.x * blockDim.x + threadIdx.x; item < total; item += gridDim.x * blockDim.x) {
    const int nb = item % width_blocks, kb = (item / width_blocks) % depth_blocks, e = item / (width_blocks * depth_blocks);
    out[item] = kmajor ? scales[(static_cast<size_t>(e) * width_blocks + nb) * depth_blocks + kb] : scales[item];
  }
}

__global__ void fill_words_kernel(uint32_t* __restrict__ words, int count, uint32_t value) {
  for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < count; i += gridDim.x * blockDim.x) words[i] = value;
}

// ---- An MXFP4 checkpoint's own tensors (`*_blocks [E][N][K / 32][16]` bytes, low nibble the even element, and
// `*_scales [E][N][K / 32]` E8M0 bytes, src/dew/interop/codecs.py:193-224) straight to the prepared FP4 bank, with
// the arithmetic of the reference's `mxfp4_tensor_powers` / `mxfp4_as_nvfp4` (src/dew/interop/codecs.py:238-284) and
// no value decoded: an expert's tensor scale is 2^k with k its largest group power (of the groups that hold a nonzero
// magnitude) less 8, a group's E4M3 block scale 2^(its power - k), twice, and 2^8 for a group of zeros.
// summary[e] = {largest scale byte + 1 of the groups holding a magnitude (0: none), least such byte}; flags[1] is
// set by a 0xff scale byte.
struct Mxfp4Survey {
  uint32_t top_plus_one, bottom;
};

__device__ __forceinline__ bool holds_magnitude(const uint4& block) {
  return ((block.x | block.y | block.z | block.w) & 0x77777777u) != 0u;
}

__global__ void mxfp4_survey_start_kernel(Mxfp4Survey* __restrict__ summary, int experts) {
  const int e = blockIdx.x * blockDim.x + threadIdx.x;
  if (e < experts) summary[e] = Mxfp4Survey{0u, 0xFFFFFFFFu};
}

__global__ __launch_bounds__(256) void mxfp4_survey_kernel(const uint4* __restrict__ blocks, const uint8_t* __restrict__ scales,
                                                           Mxfp4Survey* __restrict__ summary, uint32_t* __restrict__ flags,
                                                           int experts, long long per_expert) {
  // per_expert (= N * K / 32) is a multiple of 64: a wavefront's 64 groups belong to one expert
  const long long total = static_cast<long long>(experts) * per_expert;
  for (long long base = (static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x) & ~63ll; base < total;
       base += static_cast<long long>(gridDim.x) * blockDim.x) {
    const long long item = base + threadIdx.x % 64;
    const uint32_t byte = scales[item];
    const bool held = holds_magnitude(blocks[item]);
    uint32_t top = held ? byte + 1u : 0u, bottom = held ? byte : 0xFFFFFFFFu, nan = byte == 255u ? 1u : 0u;
#pragma unroll
    for (int offset = 32; offset >= 1; offset >>= 1) {
      top = max(top, static_cast<uint32_t>(__shfl_xor(static_cast<int>(top), offset, 64)));
      bottom = min(bottom, static_cast<uint32_t>(__shfl_xor(static_cast<int>(bottom), offset, 64)));
      nan |= static_cast<uint32_t>(__shfl_xor(static_cast<int>(nan), offset, 64));
    }
    if (threadIdx.x % 64 == 0) {
      const int e = static_cast<int>(base / per_expert);
      if (top != 0u) {
        atomicMax(&summary[e].top_plus_one, top);
        atomicMin(&summary[e].bottom, bottom);
      }
      if (nan) atomicOr(flags + 1, 1u);
    }
  }
}

// One thread an expert: its power k and tensor scale 2^k; flags[1] set where the bank cannot be one NVFP4 bank (its
// group powers spread past E4M3's 17 binades, or 2^k leaves fp32's normal range). summary[e].bottom then holds k.
__global__ void mxfp4_powers_kernel(Mxfp4Survey* __restrict__ summary, float* __restrict__ tensor_scale, uint32_t* __restrict__ flags,
                                    int experts) {
  const int e = blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= experts) return;
  const bool any = summary[e].top_plus_one != 0u;
  const int top = any ? static_cast<int>(summary[e].top_plus_one) - 1 - 127 : 8;
  const int bottom = any ? static_cast<int>(summary[e].bottom) - 127 : 8;
  const int power = top - 8;
  if (top - bottom > 17 || power < -126 || power > 127) atomicOr(flags + 1, 1u);
  tensor_scale[e] = __uint_as_float(static_cast<uint32_t>(min(max(power, -126), 127) + 127) << 23);
  summary[e].bottom = static_cast<uint32_t>(power);
}

// One thread per (expert, column, 32-deep group): its 16 bytes are a lane's piece of an FP4 atom as they are, and its
// scale the lane's two equal E4M3 bytes. flags[0] is set by a block scale below E4M3's normal range (2^-7 .. 2^-9),
// which the scaled conversions cannot take as an exponent: the bank is then multiplied as a general NVFP4 bank.
__global__ __launch_bounds__(256) void prepare_mxfp4_blocks_kernel(const uint4* __restrict__ blocks, const uint8_t* __restrict__ scales,
                                                                   const Mxfp4Survey* __restrict__ summary, uint8_t* __restrict__ codes_out,
                                                                   uint16_t* __restrict__ scales_out, uint32_t* __restrict__ flags,
                                                                   int experts, int depth, int width) {
  const int groups = depth / 32, n_atoms = width / 32, k_atoms = depth / 64;
  const long long total = static_cast<long long>(experts) * width * groups;
  for (long long item = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x; item < total;
       item += static_cast<long long>(gridDim.x) * blockDim.x) {
    // consecutive threads take consecutive columns of one group, so their 16-byte writes fill an atom's lanes in order
    const int n = static_cast<int>(item % width);
    const int group = static_cast<int>((item / width) % groups);
    const int e = static_cast<int>(item / (static_cast<long long>(width) * groups));
    const size_t source = (static_cast<size_t>(e) * width + n) * groups + group;
    const uint4 block = blocks[source];
    const int local = holds_magnitude(block) ? static_cast<int>(scales[source]) - 127 - static_cast<int>(summary[e].bottom) : 8;
    const int clamped = min(max(local, -9), 8);
    const uint32_t e4m3 = clamped >= -6 ? static_cast<uint32_t>(clamped + 7) << 3 : 1u << (clamped + 9);
    if (clamped < -6) atomicOr(flags, 1u);
    const size_t atom = (static_cast<size_t>(e) * n_atoms + n / 32) * k_atoms + group / 2;
    const int lane = 32 * (group % 2) + n % 32;
    *reinterpret_cast<uint4*>(codes_out + atom * kAtomBytes + lane * 16) = block;
    scales_out[atom * 64 + lane] = static_cast<uint16_t>(e4m3 | (e4m3 << 8));
  }
}

static size_t codes_bytes(int format, int experts, int depth, int width) {
  const size_t elements = static_cast<size_t>(experts) * depth * width;
  return (format == DEW_MOE_W_NVFP4 || format == DEW_MOE_W_MXFP4_BLOCKS) ? elements / 2 : format == DEW_MOE_W_BF16 ? elements * 2 : elements;
}

// Behind an FP4 bank's codes and scales: 256 bytes of flag words, then (a checkpoint's MXFP4 tensors) the experts'
// tensor scales and the survey's two words an expert.
static size_t fp4_scales_bytes(int experts, int depth, int width) { return static_cast<size_t>(experts) * width * (depth / 16); }

}  // namespace dew

extern "C" size_t dew_moe_prepared_bytes(int32_t format, int32_t experts, int32_t depth, int32_t width) {
  if (experts <= 0 || depth <= 0 || width <= 0) return 0;
  size_t bytes = dew::codes_bytes(format, experts, depth, width);
  if (format == DEW_MOE_W_NVFP4) bytes += dew::fp4_scales_bytes(experts, depth, width) + 256;  // + a flag word
  if (format == DEW_MOE_W_MXFP4_BLOCKS)  // + flag words, tensor scales, the survey
    bytes += dew::fp4_scales_bytes(experts, depth, width) + 256 + (static_cast<size_t>(experts) * 12 + 255) / 256 * 256;
  if (format == DEW_MOE_W_FP8_BLOCK) bytes += static_cast<size_t>(experts) * (depth / 128) * (width / 128) * sizeof(float);  // its block scales
  if (format == DEW_MOE_W_MXFP8) bytes += static_cast<size_t>(experts) * width * (depth / 32);
  return bytes;
}

extern "C" int dew_moe_prepare_bank(const dew_moe_bank* ref, void* prepared, dew_moe_bank* out, void* stream) {
  using namespace dew;
  DEW_REQUIRE(ref && prepared && out, "dew_moe_prepare_bank: bank, prepared buffer and out must not be null");
  DEW_REQUIRE(ref->layout == DEW_MOE_LAYOUT_REFERENCE ||
                  (ref->layout == DEW_MOE_LAYOUT_REFERENCE_KMAJOR && (ref->format == DEW_MOE_W_BF16 || ref->format == DEW_MOE_W_FP8_BLOCK)),
              "dew_moe_prepare_bank: the bank is already prepared, or K-major in a format held one way only (layout %d, format %d)",
              ref->layout, ref->format);
  DEW_REQUIRE(ref->format == DEW_MOE_W_FP8_BLOCK || ref->format == DEW_MOE_W_FP8_CHANNEL || ref->format == DEW_MOE_W_NVFP4 ||
                  ref->format == DEW_MOE_W_MXFP8 || ref->format == DEW_MOE_W_BF16 || ref->format == DEW_MOE_W_MXFP4_BLOCKS,
              "dew_moe_prepare_bank: unknown weight format %d", ref->format);
  DEW_REQUIRE(ref->experts >= 1 && ref->depth >= 1 && ref->width >= 1, "dew_moe_prepare_bank: bank [%d, %d, %d]",
              ref->experts, ref->depth, ref->width);
  DEW_REQUIRE(ref->codes && (ref->scales || ref->format == DEW_MOE_W_BF16), "dew_moe_prepare_bank: codes and scales must not be null");
  // unquantized matrices as the reference holds them take any width in whole 32-column atoms and any depth in whole 64-deep steps
  // (so does an MXFP4 checkpoint's bank, whose groups are 32 deep: its atoms are 64 deep and 32 columns wide)
  const bool plain_bf16 = ref->format == DEW_MOE_W_BF16 && ref->layout == DEW_MOE_LAYOUT_REFERENCE;
  const bool in_atoms = plain_bf16 || ref->format == DEW_MOE_W_MXFP4_BLOCKS;
  DEW_REQUIRE(ref->width % (in_atoms ? 32 : 128) == 0, "dew_moe_prepare_bank: width %d is not a multiple of %d", ref->width, in_atoms ? 32 : 128);
  DEW_REQUIRE((reinterpret_cast<uintptr_t>(prepared) & 255u) == 0, "dew_moe_prepare_bank: prepared buffer must be 256-byte aligned");
  hipStream_t s = static_cast<hipStream_t>(stream);
  *out = *ref;
  out->layout = DEW_MOE_LAYOUT_PREPARED;
  out->codes = prepared;
  const int grid = 256 * 16;
  if (ref->format == DEW_MOE_W_NVFP4) {
    DEW_REQUIRE(ref->depth % 256 == 0, "dew_moe_prepare_bank: an NVFP4 bank's depth is whole 256s, not %d", ref->depth);
    DEW_REQUIRE(ref->tensor_scale, "dew_moe_prepare_bank: an NVFP4 bank needs its tensor scales");
    DEW_REQUIRE(aligned16(ref->codes), "dew_moe_prepare_bank: words must be 16-byte aligned");
    uint8_t* codes_out = static_cast<uint8_t*>(prepared);
    uint8_t* scales_out = codes_out + codes_bytes(ref->format, ref->experts, ref->depth, ref->width);
    hipLaunchKernelGGL(prepare_nvfp4_codes_kernel, dim3(grid), dim3(256), 0, s, static_cast<const uint32_t*>(ref->codes),
                       codes_out, ref->experts, ref->depth, ref->width);
    if (int rc = launched("prepare_nvfp4_codes_kernel")) return rc;
    uint32_t* general = reinterpret_cast<uint32_t*>(scales_out + static_cast<size_t>(ref->experts) * ref->width * (ref->depth / 16));
    hipLaunchKernelGGL(fill_words_kernel, dim3(1), dim3(64), 0, s, general, 1, 0u);  // (a kernel, not a memset node: a caller may capture this)
    if (int rc = launched("fill_words_kernel")) return rc;
    hipLaunchKernelGGL(prepare_nvfp4_scales_kernel, dim3(grid), dim3(256), 0, s, static_cast<const uint8_t*>(ref->scales),
                       reinterpret_cast<uint16_t*>(scales_out), ref->experts, ref->depth, ref->width, general);
    if (int rc = launched("prepare_nvfp4_scales_kernel")) return rc;
    out->scales = scales_out;
    uint32_t found = 1;
    if (hipMemcpyAsync(&found, general, sizeof(found), hipMemcpyDeviceToHost, s) != hipSuccess || hipStreamSynchronize(s) != hipSuccess)
      return fail(DEW_MOE_ELAUNCH, "dew_moe_prepare_bank: reading the scale summary back failed: %s", hipGetErrorString(hipGetLastError()));
    if (!found) out->format = DEW_MOE_W_MXFP4;
  } else if (ref->format == DEW_MOE_W_MXFP4_BLOCKS) {
    DEW_REQUIRE(ref->depth % 64 == 0 && ref->depth >= 128, "dew_moe_prepare_bank: an MXFP4 checkpoint bank's depth is whole 64s, not %d", ref->depth);
    DEW_REQUIRE(aligned16(ref->codes), "dew_moe_prepare_bank: blocks must be 16-byte aligned");
    uint8_t* codes_out = static_cast<uint8_t*>(prepared);
    uint8_t* scales_out = codes_out + codes_bytes(ref->format, ref->experts, ref->depth, ref->width);
    uint32_t* flags = reinterpret_cast<uint32_t*>(scales_out + fp4_scales_bytes(ref->experts, ref->depth, ref->width));
    float* tensor_scale = reinterpret_cast<float*>(flags + 64);
    Mxfp4Survey* summary = reinterpret_cast<Mxfp4Survey*>(tensor_scale + ref->experts);
    const uint4* blocks = static_cast<const uint4*>(ref->codes);
    const uint8_t* bytes = static_cast<const uint8_t*>(ref->scales);
    const long long per_expert = static_cast<long long>(ref->width) * (ref->depth / 32);
    hipLaunchKernelGGL(fill_words_kernel, dim3(1), dim3(64), 0, s, flags, 2, 0u);
    if (int rc = launched("fill_words_kernel")) return rc;
    hipLaunchKernelGGL(mxfp4_survey_start_kernel, dim3((ref->experts + 255) / 256), dim3(256), 0, s, summary, ref->experts);
    hipLaunchKernelGGL(mxfp4_survey_kernel, dim3(grid), dim3(256), 0, s, blocks, bytes, summary, flags, ref->experts, per_expert);
    if (int rc = launched("mxfp4_survey_kernel")) return rc;
    hipLaunchKernelGGL(mxfp4_powers_kernel, dim3((ref->experts + 255) / 256), dim3(256), 0, s, summary, tensor_scale, flags, ref->experts);
    hipLaunchKernelGGL(prepare_mxfp4_blocks_kernel, dim3(grid), dim3(256), 0, s, blocks, bytes, summary, codes_out,
                       reinterpret_cast<uint16_t*>(scales_out), flags, ref->experts, ref->depth, ref->width);
    if (int rc = launched("prepare_mxfp4_blocks_kernel")) return rc;
    uint32_t found[2] = {1, 1};
    if (hipMemcpyAsync(found, flags, sizeof(found), hipMemcpyDeviceToHost, s) != hipSuccess || hipStreamSynchronize(s) != hipSuccess)
      return fail(DEW_MOE_ELAUNCH, "dew_moe_prepare_bank: reading the scale summary back failed: %s", hipGetErrorString(hipGetLastError()));
    DEW_REQUIRE(!found[1], "dew_moe_prepare_bank: this MXFP4 bank is no one NVFP4 bank (an expert's group powers spread past 17 binades, "
                           "a tensor scale leaves float32's normal range, or a scale byte is 0xff): it stays dense");
    out->format = found[0] ? DEW_MOE_W_NVFP4 : DEW_MOE_W_MXFP4;
    out->scales = scales_out;
    out->tensor_scale = tensor_scale;
  } else if (ref->format == DEW_MOE_W_BF16) {
    DEW_REQUIRE(ref->depth % (plain_bf16 ? 64 : 128) == 0, "dew_moe_prepare_bank: a bf16 bank's depth is whole %ds, not %d", plain_bf16 ? 64 : 128, ref->depth);
    if (ref->layout == DEW_MOE_LAYOUT_REFERENCE_KMAJOR) {
      DEW_REQUIRE(aligned16(ref->codes), "dew_moe_prepare_bank: K-major bf16 matrices must be 16-byte aligned");
      hipLaunchKernelGGL(prepare_bf16_kmajor_kernel, dim3(grid), dim3(256), 0, s, static_cast<const uint16_t*>(ref->codes),
                         static_cast<uint8_t*>(prepared), ref->experts, ref->depth, ref->width);
    } else {
      hipLaunchKernelGGL(prepare_bf16_kernel, dim3(grid), dim3(256), 0, s, static_cast<const uint16_t*>(ref->codes),
                         static_cast<uint8_t*>(prepared), ref->experts, ref->depth, ref->width);
    }
    if (int rc = launched("prepare_bf16_kernel")) return rc;
    out->scales = nullptr;
  } else if (ref->format == DEW_MOE_W_MXFP8) {
    DEW_REQUIRE(ref->depth % 128 == 0, "dew_moe_prepare_bank: an MXFP8 bank's depth is whole 128s, not %d", ref->depth);
    DEW_REQUIRE(aligned16(ref->codes) && (reinterpret_cast<uintptr_t>(ref->scales) & 3u) == 0,
                "dew_moe_prepare_bank: MXFP8 codes must be 16-byte and scales 4-byte aligned");
    uint8_t* scales_out = static_cast<uint8_t*>(prepared) + codes_bytes(ref->format, ref->experts, ref->depth, ref->width);
    hipLaunchKernelGGL(prepare_mxfp8_kernel, dim3(grid), dim3(256), 0, s, static_cast<const uint8_t*>(ref->codes),
                       static_cast<const uint8_t*>(ref->scales), static_cast<uint8_t*>(prepared), reinterpret_cast<uint32_t*>(scales_out),
                       ref->experts, ref->depth, ref->width);
    if (int rc = launched("prepare_mxfp8_kernel")) return rc;
    out->scales = scales_out;
  } else {
    DEW_REQUIRE(ref->depth % 128 == 0, "dew_moe_prepare_bank: an FP8 bank's depth is whole 128s, not %d", ref->depth);
    const bool kmajor = ref->layout == DEW_MOE_LAYOUT_REFERENCE_KMAJOR;
    if (kmajor) {
      DEW_REQUIRE(aligned16(ref->codes), "dew_moe_prepare_bank: K-major FP8 codes must be 16-byte aligned");
      hipLaunchKernelGGL(prepare_fp8_kmajor_kernel, dim3(grid), dim3(256), 0, s, static_cast<const uint8_t*>(ref->codes),
                         static_cast<uint8_t*>(prepared), ref->experts, ref->depth, ref->width);
    } else {
      hipLaunchKernelGGL(prepare_fp8_kernel, dim3(grid), dim3(256), 0, s, static_cast<const uint8_t*>(ref->codes),
                         static_cast<uint8_t*>(prepared), ref->experts, ref->depth, ref->width);
    }
    if (int rc = launched("prepare_fp8_kernel")) return rc;
    if (ref->format == DEW_MOE_W_FP8_BLOCK) {  // the block scales travel with the codes, in the order the products read
      float* scales_out = reinterpret_cast<float*>(static_cast<uint8_t*>(prepared) + codes_bytes(ref->format, ref->experts, ref->depth, ref->width));
      hipLaunchKernelGGL(prepare_block_scales_kernel, dim3(64), dim3(256), 0, s, static_cast<const float*>(ref->scales), scales_out,
                         ref->experts, ref->depth / 128, ref->width / 128, kmajor ? 1 : 0);
      if (int rc = launched("prepare_block_scales_kernel")) return rc;
      out->scales = scales_out;
    }
  }
  return DEW_MOE_OK;
}

extern "C" int dew_moe_prepared_view(int32_t format, int32_t experts, int32_t depth, int32_t width, const void* prepared,
                                     const void* external_scales, const float* tensor_scale, dew_moe_bank* out) {
  using namespace dew;
  const char* who = "dew_moe_prepared_view";
  DEW_REQUIRE(prepared && out, "%s: the prepared buffer and out must not be null", who);
  DEW_REQUIRE(experts >= 1 && depth >= 1 && width >= 1, "%s: bank [%d, %d, %d]", who, experts, depth, width);
  const uint8_t* base = static_cast<const uint8_t*>(prepared);
  *out = dew_moe_bank{format, DEW_MOE_LAYOUT_PREPARED, experts, depth, width, base, nullptr, nullptr};
  switch (format) {
    case DEW_MOE_W_FP8_BLOCK:
    case DEW_MOE_W_MXFP8:
      out->scales = base + codes_bytes(format, experts, depth, width);
      break;
    case DEW_MOE_W_NVFP4:
    case DEW_MOE_W_MXFP4:
      DEW_REQUIRE(tensor_scale, "%s: an FP4 bank needs its tensor scales", who);
      out->scales = base + codes_bytes(DEW_MOE_W_NVFP4, experts, depth, width);
      out->tensor_scale = tensor_scale;
      break;
    case DEW_MOE_W_FP8_CHANNEL:
      DEW_REQUIRE(external_scales, "%s: a per-channel FP8 bank's scales [E, N] stay outside the prepared buffer", who);
      out->scales = external_scales;
      break;
    case DEW_MOE_W_BF16:
      break;
    default:
      return fail(DEW_MOE_EINVAL, "%s: %d is no format a prepared bank has", who, format);
  }
  return DEW_MOE_OK;
}

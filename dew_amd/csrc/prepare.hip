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

static size_t codes_bytes(int format, int experts, int depth, int width) {
  const size_t elements = static_cast<size_t>(experts) * depth * width;
  return format == DEW_MOE_W_NVFP4 ? elements / 2 : format == DEW_MOE_W_BF16 ? elements * 2 : elements;
}

}  // namespace dew

extern "C" size_t dew_moe_prepared_bytes(int32_t format, int32_t experts, int32_t depth, int32_t width) {
  if (experts <= 0 || depth <= 0 || width <= 0) return 0;
  size_t bytes = dew::codes_bytes(format, experts, depth, width);
  if (format == DEW_MOE_W_NVFP4) bytes += static_cast<size_t>(experts) * width * (depth / 16) + 256;  // + a flag word
  if (format == DEW_MOE_W_MXFP8) bytes += static_cast<size_t>(experts) * width * (depth / 32);
  return bytes;
}

extern "C" int dew_moe_prepare_bank(const dew_moe_bank* ref, void* prepared, dew_moe_bank* out, void* stream) {
  using namespace dew;
  DEW_REQUIRE(ref && prepared && out, "dew_moe_prepare_bank: bank, prepared buffer and out must not be null");
  DEW_REQUIRE(ref->layout == DEW_MOE_LAYOUT_REFERENCE || (ref->layout == DEW_MOE_LAYOUT_REFERENCE_KMAJOR && ref->format == DEW_MOE_W_BF16),
              "dew_moe_prepare_bank: the bank is already prepared (layout %d)", ref->layout);
  DEW_REQUIRE(ref->format == DEW_MOE_W_FP8_BLOCK || ref->format == DEW_MOE_W_FP8_CHANNEL || ref->format == DEW_MOE_W_NVFP4 ||
                  ref->format == DEW_MOE_W_MXFP8 || ref->format == DEW_MOE_W_BF16,
              "dew_moe_prepare_bank: unknown weight format %d", ref->format);
  DEW_REQUIRE(ref->experts >= 1 && ref->depth >= 1 && ref->width >= 1, "dew_moe_prepare_bank: bank [%d, %d, %d]",
              ref->experts, ref->depth, ref->width);
  DEW_REQUIRE(ref->codes && (ref->scales || ref->format == DEW_MOE_W_BF16), "dew_moe_prepare_bank: codes and scales must not be null");
  DEW_REQUIRE(ref->width % 128 == 0, "dew_moe_prepare_bank: width %d is not a multiple of 128", ref->width);
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
    if (hipMemsetAsync(general, 0, sizeof(uint32_t), s) != hipSuccess) return fail(DEW_MOE_ELAUNCH, "dew_moe_prepare_bank: memset failed");
    hipLaunchKernelGGL(prepare_nvfp4_scales_kernel, dim3(grid), dim3(256), 0, s, static_cast<const uint8_t*>(ref->scales),
                       reinterpret_cast<uint16_t*>(scales_out), ref->experts, ref->depth, ref->width, general);
    if (int rc = launched("prepare_nvfp4_scales_kernel")) return rc;
    out->scales = scales_out;
    uint32_t found = 1;
    if (hipMemcpyAsync(&found, general, sizeof(found), hipMemcpyDeviceToHost, s) != hipSuccess || hipStreamSynchronize(s) != hipSuccess)
      return fail(DEW_MOE_ELAUNCH, "dew_moe_prepare_bank: reading the scale summary back failed: %s", hipGetErrorString(hipGetLastError()));
    if (!found) out->format = DEW_MOE_W_MXFP4;
  } else if (ref->format == DEW_MOE_W_BF16) {
    DEW_REQUIRE(ref->depth % 128 == 0, "dew_moe_prepare_bank: a bf16 bank's depth is whole 128s, not %d", ref->depth);
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
    hipLaunchKernelGGL(prepare_fp8_kernel, dim3(grid), dim3(256), 0, s, static_cast<const uint8_t*>(ref->codes),
                       static_cast<uint8_t*>(prepared), ref->experts, ref->depth, ref->width);
    if (int rc = launched("prepare_fp8_kernel")) return rc;
  }
  return DEW_MOE_OK;
}

// Shared host/device helpers of libdew_moe_hip.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/dew_moe_hip.h"

namespace dew {

// ---- error reporting (thread-local message, reference convention: a `why` string per refusal) ----
void set_error(const char* fmt, ...);
int fail(int code, const char* fmt, ...);
int launched(const char* kernel);  // hipGetLastError() after a launch -> DEW_MOE_OK / DEW_MOE_ELAUNCH

#define DEW_REQUIRE(cond, ...)                                \
  do {                                                        \
    if (!(cond)) return ::dew::fail(DEW_MOE_EINVAL, __VA_ARGS__); \
  } while (0)

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ---- bf16 <-> f32 on the device ----
typedef uint16_t bf16_t;

__device__ __forceinline__ float bf16_to_f32(bf16_t v) { return __uint_as_float(static_cast<uint32_t>(v) << 16); }

// Round to nearest, ties to even (finite inputs and infinities; NaN stays NaN by the quiet bit).
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<bf16_t>((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return static_cast<bf16_t>(u >> 16);
}

__device__ __forceinline__ float bf16_round(float f) { return bf16_to_f32(f32_to_bf16(f)); }

// ---- prepared bank geometry (fragment-native atoms) ----
// FP8 atom: 32 n x 32 k bytes = 1 KiB; lane l = (g = l / 32, n = l % 32) holds k = 16 g .. 16 g + 15.
// FP4 atom: 32 n x 64 k nibbles = 1 KiB; lane l holds k = 32 g .. 32 g + 31 (byte j: low nibble k = 32 g + 2 j).
// Atoms are ordered [E][N / 32][K / atom_k]; FP4 scale atoms [E][N / 32][K / 64][64 lanes][2 e4m3 bytes].
constexpr int kAtomBytes = 1024;

}  // namespace dew

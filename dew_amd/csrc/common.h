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

// Round to nearest, ties to even: the hardware conversion (v_cvt_pk_bf16_f32), one instruction, no branch.
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
  return __builtin_bit_cast(bf16_t, static_cast<__bf16>(f));
}

__device__ __forceinline__ float bf16_round(float f) { return bf16_to_f32(f32_to_bf16(f)); }

// Round to nearest even on the host (the device has the hardware conversion): a finite value as the bf16 it becomes.
static inline float bf16_round_host(float value) {
  uint32_t bits;
  __builtin_memcpy(&bits, &value, 4);
  bits += 0x7FFFu + ((bits >> 16) & 1u);
  bits &= 0xFFFF0000u;
  __builtin_memcpy(&value, &bits, 4);
  return value;
}

// SwiGLU on the fp32 sums of the gate and up products with the reference's roundings
// (src/dew/nn/activations.py:267-278): g = bf16(gate), u = bf16(up), a = bf16(g * logistic(g)), h = bf16(a * u).
// logistic(g) = 1 / (1 + e^-g) uses the hardware exp2 and reciprocal (each within 1 ulp of fp32): the
// activation is rounded to 8 significant bits right after, so about one result in 2^12 differs by one bf16
// ulp from a correctly rounded logistic, the same order as the spread between two libraries' expf.
__device__ __forceinline__ bf16_t swiglu_rounded(float gate_sum, float up_sum) {
  const float g = bf16_round(gate_sum), u = bf16_round(up_sum);
  const float e = __builtin_amdgcn_exp2f(g * -1.44269504088896340736f);
  const float sig = __builtin_amdgcn_rcpf(1.0f + e);
  const float activated = bf16_round(g * sig);
  return f32_to_bf16(activated * u);
}

// GeGLU with the tanh GELU (`gated_product('geglu')` over `gelu_tanh`, src/dew/nn/activations.py:57-69, 267-278): the
// activation g * logistic(sqrt(8 / pi) (g + 0.044715 g^3)) in fp32 in that order of operations, rounded to bf16, then the
// product with the up projection rounded again. Compile with contraction off: the reference's fp32 steps each round.
__device__ __forceinline__ bf16_t geglu_rounded(float gate_sum, float up_sum) {
  const float g = bf16_round(gate_sum), u = bf16_round(up_sum);
  const float cube = (g * g) * g;
  const float inner = 1.5957691216057308f * (g + 0.044715f * cube);
  const float e = __builtin_amdgcn_exp2f(inner * -1.44269504088896340736f);
  const float sig = __builtin_amdgcn_rcpf(1.0f + e);
  const float activated = bf16_round(g * sig);
  return f32_to_bf16(activated * u);
}

// Either gate on the fp32 sums of a paired launch, with the clamp the stand-alone gating kernel applies (`swiglu_clamped`,
// src/dew/nn/activations.py:327-333): both sums rounded to bf16 first, then the gate clamped from above and the up
// projection both ways by `limit` (> 0, already the bf16 it is compared in; 0: no clamp), then the gated product.
__device__ __forceinline__ bf16_t gated_rounded(float gate_sum, float up_sum, float limit, int activation) {
  float g = bf16_round(gate_sum), u = bf16_round(up_sum);
  if (limit > 0.0f) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
  }
  return activation == DEW_MOE_GATE_GELU_TANH ? geglu_rounded(g, u) : swiglu_rounded(g, u);
}

// GPT-OSS's gating of one (gate, up) pair already rounded to bf16 (src/dew/nn/gpt_oss.py:120-121 over
// src/dew/nn/activations.py:72-74,327-333): gate clamped from above and up both ways by `limit`, then
// (up + 1) * gate * logistic(1.702 gate) with every operation rounded to bf16 as an array of that dtype
// rounds it; 1.702 enters as the bf16 it is multiplied in, 1.703125.
__device__ __forceinline__ bf16_t gated_pair_rounded(float gate, float up, float limit) {
  const float g = fminf(gate, limit), u = fminf(fmaxf(up, -limit), limit);
  const float t = bf16_round(g * 1.703125f);
  const float sig = bf16_round(__builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(t * -1.44269504088896340736f)));
  const float q = bf16_round(g * sig);
  const float u1 = bf16_round(u + 1.0f);
  return f32_to_bf16(u1 * q);
}

// e^x by Cody-Waite reduction and a degree-7 Taylor sum in Horner form, times 2^n in two exact steps
// (the reference's portable exp, src/dew/nn/precision.py:470-488). The CPU oracle runs the same sequence, so a file that uses
// it is compiled with contraction off (-ffp-contract=off): a fused multiply-add would round differently.
__device__ __forceinline__ float exp_f32(float x) {
  x = fminf(fmaxf(x, -104.0f), 90.0f);
  const float n = rintf(x * 0x1.715476p+0f);
  const float r = (x - n * 0x1.62e4p-1f) - n * 0x1.7f7d1cp-20f;
  float p = 0x1.a01a02p-13f;               // 1/5040 ... 1/6 rounded to fp32
  p = p * r + 0x1.6c16c2p-10f;
  p = p * r + 0x1.111112p-7f;
  p = p * r + 0x1.555556p-5f;
  p = p * r + 0x1.555556p-3f;
  p = p * r + 0.5f;
  p = p * r + 1.0f;
  p = p * r + 1.0f;
  const int ni = static_cast<int>(n);
  const int half = ni >> 1;  // floor(n / 2)
  const float first = __uint_as_float(static_cast<uint32_t>(half + 127) << 23);
  const float second = __uint_as_float(static_cast<uint32_t>(ni - half + 127) << 23);
  return (p * first) * second;
}

// ---- prepared bank geometry (fragment-native atoms) ----
// FP8 atom: 32 n x 32 k bytes = 1 KiB; lane l = (g = l / 32, n = l % 32) holds k = 16 g .. 16 g + 15.
// FP4 atom: 32 n x 64 k nibbles = 1 KiB; lane l holds k = 32 g .. 32 g + 31 (byte j: low nibble k = 32 g + 2 j).
// Atoms are ordered [E][N / 32][K / atom_k]; FP4 scale atoms [E][N / 32][K / 64][64 lanes][2 e4m3 bytes].
constexpr int kAtomBytes = 1024;

}  // namespace dew

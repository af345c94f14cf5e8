// Weighted combine of a token's k expert outputs, and the stand-alone SwiGLU product.
// Both are HBM-bound elementwise kernels: 16-byte loads and stores, fp32 arithmetic, explicit roundings.
#include "common.h"

#pragma clang fp contract(off)

namespace dew {

struct alignas(16) Bf16x8 {
  bf16_t v[8];
};

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// A slot row's 16 bytes. STREAM: read once and never again, the load bypasses the caches' retention (slots beyond what
// the last-level cache holds: 6.0 against 5.3 TB/s on 8192 tokens x 8 slots x 7168; slots the down launch has just
// left in that cache read 15 % slower that way, so those take the plain load).
template <bool STREAM>
__device__ __forceinline__ Bf16x8 slot_chunk(const bf16_t* from) {
  const u32x4 words = STREAM ? __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(from)) : *reinterpret_cast<const u32x4*>(from);
  Bf16x8 values;
  __builtin_memcpy(&values, &words, sizeof(values));
  return values;
}

// out[t, :] = bf16( sum_j f32(slots[t, j, :]) * weights[t, j] ): the products and the running sum each
// round to fp32 in slot order, then one rounding to bf16 (reference src/dew/nn/moe.py:1328-1333). With an
// addend, out = bf16(f32(out) + f32(addend)), the shared expert's bf16 add (src/dew/nn/moe.py:1503).
// K = the slots a token has when that is 1, 2, 4, 6 or 8 (all k loads of a lane are then in flight before the
// first sum), 0 = any number, one after another.
template <int K, bool STREAM>
__global__ __launch_bounds__(256) void combine_kernel(const bf16_t* __restrict__ slots,
                                                      const float* __restrict__ weights,
                                                      const bf16_t* __restrict__ addend, bf16_t* __restrict__ out,
                                                      int tokens, int top_k, int width) {
  const int chunks = width / 8;
  const long long total = static_cast<long long>(tokens) * chunks;
  for (long long item = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x; item < total;
       item += static_cast<long long>(gridDim.x) * blockDim.x) {
    const int token = static_cast<int>(item / chunks);
    const int chunk = static_cast<int>(item % chunks);
    float sum[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) sum[i] = 0.0f;
    const bf16_t* base = slots + (static_cast<size_t>(token) * top_k) * width + static_cast<size_t>(chunk) * 8;
    const float* w = weights + static_cast<size_t>(token) * top_k;
    if constexpr (K > 0) {
      Bf16x8 y[K];
#pragma unroll
      for (int j = 0; j < K; ++j) y[j] = slot_chunk<STREAM>(base + static_cast<size_t>(j) * width);
#pragma unroll
      for (int j = 0; j < K; ++j) {
        const float wj = w[j];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const float product = bf16_to_f32(y[j].v[i]) * wj;
          sum[i] = sum[i] + product;
        }
      }
    } else {
      for (int j = 0; j < top_k; ++j) {
        const float wj = w[j];
        const Bf16x8 y = slot_chunk<STREAM>(base + static_cast<size_t>(j) * width);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const float product = bf16_to_f32(y.v[i]) * wj;
          sum[i] = sum[i] + product;
        }
      }
    }
    Bf16x8 result;
    if (addend != nullptr) {
      const Bf16x8 a = slot_chunk<STREAM>(addend + static_cast<size_t>(token) * width + static_cast<size_t>(chunk) * 8);
#pragma unroll
      for (int i = 0; i < 8; ++i) result.v[i] = f32_to_bf16(bf16_round(sum[i]) + bf16_to_f32(a.v[i]));
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) result.v[i] = f32_to_bf16(sum[i]);
    }
    *reinterpret_cast<Bf16x8*>(out + static_cast<size_t>(token) * width + static_cast<size_t>(chunk) * 8) = result;
  }
}

// Llama 4's placement of the routing weight (src/dew/nn/moe.py:1124-1126): sorted position i holds token gather[i]'s
// row times the weight of its slot, weights[slots[i]], both in bf16, the product rounded once.
__global__ __launch_bounds__(256) void scale_rows_kernel(const bf16_t* __restrict__ x, const int32_t* __restrict__ gather,
                                                         const int32_t* __restrict__ slots, const float* __restrict__ weights,
                                                         bf16_t* __restrict__ out, int rows, int depth) {
  const int chunks = depth / 8;
  const long long total = static_cast<long long>(rows) * chunks;
  for (long long item = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x; item < total;
       item += static_cast<long long>(gridDim.x) * blockDim.x) {
    const int row = static_cast<int>(item / chunks), chunk = static_cast<int>(item % chunks);
    const float w = bf16_round(weights[slots[row]]);
    const Bf16x8 source = *reinterpret_cast<const Bf16x8*>(x + static_cast<size_t>(gather[row]) * depth + static_cast<size_t>(chunk) * 8);
    Bf16x8 scaled;
#pragma unroll
    for (int i = 0; i < 8; ++i) scaled.v[i] = f32_to_bf16(bf16_to_f32(source.v[i]) * w);
    *reinterpret_cast<Bf16x8*>(out + static_cast<size_t>(row) * depth + static_cast<size_t>(chunk) * 8) = scaled;
  }
}

// Qwen2-MoE's gate on the shared expert (`shared_gate`, src/dew/nn/moe.py:1497-1503: `shared * logistic(Dense(1)(x))` in
// the compute dtype): one wavefront a token forms the gate's logit, the fp32 sum of the token times the gate's kernel
// (each rounded to bf16, as the layer's promotion casts it), rounded to bf16; its logistic, rounded to bf16; and the
// token's row of the shared expert's output times it, each product rounded once.
__global__ __launch_bounds__(256) void gate_rows_kernel(const bf16_t* __restrict__ x, const float* __restrict__ kernel,
                                                        const bf16_t* rows_in, bf16_t* out /* may be rows_in */, int tokens,
                                                        int depth, int width) {
  const int lane = threadIdx.x % 64;
  const int token = blockIdx.x * 4 + threadIdx.x / 64;
  if (token >= tokens) return;
  // The logit's sum in float64 (each product of two bf16 values is exact there, and their sum is exact to 2^-53 of its
  // terms whatever the order), rounded to fp32 and then to bf16, which is what the CPU oracle's float64 dot product gives;
  // the logistic by the library's fixed-sequence exponential and an IEEE division, the oracle's own steps.
  double sum = 0.0;
  for (int chunk = lane; chunk < depth / 8; chunk += 64) {
    const Bf16x8 values = *reinterpret_cast<const Bf16x8*>(x + static_cast<size_t>(token) * depth + static_cast<size_t>(chunk) * 8);
#pragma unroll
    for (int i = 0; i < 8; ++i) sum += static_cast<double>(bf16_to_f32(values.v[i])) * static_cast<double>(bf16_round(kernel[chunk * 8 + i]));
  }
#pragma unroll
  for (int offset = 32; offset >= 1; offset >>= 1) sum += __shfl_xor(sum, offset, 64);
  const float logit = bf16_round(static_cast<float>(sum));
  const float gate = bf16_round(1.0f / (1.0f + exp_f32(-logit)));
  for (int chunk = lane; chunk < width / 8; chunk += 64) {
    const size_t at = static_cast<size_t>(token) * width + static_cast<size_t>(chunk) * 8;
    const Bf16x8 values = *reinterpret_cast<const Bf16x8*>(rows_in + at);
    Bf16x8 gated;
#pragma unroll
    for (int i = 0; i < 8; ++i) gated.v[i] = f32_to_bf16(bf16_to_f32(values.v[i]) * gate);
    *reinterpret_cast<Bf16x8*>(out + at) = gated;
  }
}

// The same gate where the layer states no compute dtype (src/dew/nn/moe.py:1469-1475, 1497-1503): the gate's `Dense(1)` then
// promotes the bf16 token to its fp32 kernel, so the logit, its logistic and the product with the shared expert's bf16 row
// are fp32, and so is the layer's output, routed + shared: out[t, :] = f32(routed[t, :]) + f32(shared[t, :]) * g[t], each
// operation rounded once in fp32. One wavefront a token.
__global__ __launch_bounds__(256) void gate_rows_add_f32_kernel(const bf16_t* __restrict__ x, const float* __restrict__ kernel,
                                                                const bf16_t* __restrict__ shared, const bf16_t* __restrict__ routed,
                                                                float* __restrict__ out, int tokens, int depth, int width) {
  const int lane = threadIdx.x % 64;
  const int token = blockIdx.x * 4 + threadIdx.x / 64;
  if (token >= tokens) return;
  // (the logit's sum in float64, rounded once to fp32: every product of a bf16 and an fp32 value is exact there)
  double sum = 0.0;
  for (int chunk = lane; chunk < depth / 8; chunk += 64) {
    const Bf16x8 values = *reinterpret_cast<const Bf16x8*>(x + static_cast<size_t>(token) * depth + static_cast<size_t>(chunk) * 8);
#pragma unroll
    for (int i = 0; i < 8; ++i) sum += static_cast<double>(bf16_to_f32(values.v[i])) * static_cast<double>(kernel[chunk * 8 + i]);
  }
#pragma unroll
  for (int offset = 32; offset >= 1; offset >>= 1) sum += __shfl_xor(sum, offset, 64);
  const float gate = 1.0f / (1.0f + exp_f32(-static_cast<float>(sum)));
  for (int chunk = lane; chunk < width / 8; chunk += 64) {
    const size_t at = static_cast<size_t>(token) * width + static_cast<size_t>(chunk) * 8;
    const Bf16x8 mine = *reinterpret_cast<const Bf16x8*>(shared + at), theirs = *reinterpret_cast<const Bf16x8*>(routed + at);
    float sums[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float gated = bf16_to_f32(mine.v[i]) * gate;
      sums[i] = bf16_to_f32(theirs.v[i]) + gated;
    }
    float4* to = reinterpret_cast<float4*>(out + at);
    to[0] = float4{sums[0], sums[1], sums[2], sums[3]};
    to[1] = float4{sums[4], sums[5], sums[6], sums[7]};
  }
}

// `limit` > 0: the gate clamped from above and the up projection both ways before their product (`swiglu_clamped`,
// src/dew/nn/activations.py:327-333); the limit enters as the bf16 the operands' dtype rounds it to.
__global__ __launch_bounds__(256) void swiglu_kernel(const bf16_t* __restrict__ gate, const bf16_t* __restrict__ up,
                                                     bf16_t* __restrict__ hidden, long long chunks, float limit, int activation) {
  for (long long item = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x; item < chunks;
       item += static_cast<long long>(gridDim.x) * blockDim.x) {
    const Bf16x8 g = reinterpret_cast<const Bf16x8*>(gate)[item];
    Bf16x8 u;  // without an up projection (a plain SiLU) every up value is one: bf16(bf16(g * logistic(g)) * 1) is the SiLU's one rounding
#pragma unroll
    for (int i = 0; i < 8; ++i) u.v[i] = 0x3F80;
    if (up != nullptr) u = reinterpret_cast<const Bf16x8*>(up)[item];
    Bf16x8 h;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      float gi = bf16_to_f32(g.v[i]), ui = bf16_to_f32(u.v[i]);
      if (limit > 0.0f) {
        gi = fminf(gi, limit);
        ui = fminf(fmaxf(ui, -limit), limit);
      }
      if (activation == DEW_MOE_ACT_RELU2)
        h.v[i] = f32_to_bf16(fmaxf(gi, 0.0f) * fmaxf(gi, 0.0f));  // (the square of a bf16 value, rounded once)
      else
        h.v[i] = activation == DEW_MOE_GATE_GELU_TANH ? geglu_rounded(gi, ui) : swiglu_rounded(gi, ui);
    }
    reinterpret_cast<Bf16x8*>(hidden)[item] = h;
  }
}

}  // namespace dew

extern "C" int dew_moe_combine(const void* slots, const float* weights, const void* addend, void* out,
                               int32_t tokens, int32_t top_k, int32_t width, void* stream) {
  using namespace dew;
  DEW_REQUIRE(tokens >= 0 && top_k >= 1 && width >= 8, "dew_moe_combine: tokens %d top_k %d width %d", tokens, top_k,
              width);
  DEW_REQUIRE(width % 8 == 0, "dew_moe_combine: width %d is not a multiple of 8 (16-byte rows)", width);
  if (tokens == 0) return DEW_MOE_OK;
  DEW_REQUIRE(slots && weights && out, "dew_moe_combine: slots, weights and out must not be null");
  DEW_REQUIRE(aligned16(slots) && aligned16(out) && aligned16(addend), "dew_moe_combine: buffers must be 16-byte aligned");
  const long long total = static_cast<long long>(tokens) * (width / 8);
  const int blocks = static_cast<int>(min((total + 255) / 256, 256ll * 64));
  auto launch = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const bf16_t*>(slots), weights, static_cast<const bf16_t*>(addend),
                       static_cast<bf16_t*>(out), tokens, top_k, width);
  };
  const bool stream_slots = static_cast<long long>(tokens) * top_k * width * 2 > (192ll << 20);
  switch (top_k) {
    case 1: stream_slots ? launch(combine_kernel<1, true>) : launch(combine_kernel<1, false>); break;
    case 2: stream_slots ? launch(combine_kernel<2, true>) : launch(combine_kernel<2, false>); break;
    case 4: stream_slots ? launch(combine_kernel<4, true>) : launch(combine_kernel<4, false>); break;
    case 6: stream_slots ? launch(combine_kernel<6, true>) : launch(combine_kernel<6, false>); break;
    case 8: stream_slots ? launch(combine_kernel<8, true>) : launch(combine_kernel<8, false>); break;
    default: stream_slots ? launch(combine_kernel<0, true>) : launch(combine_kernel<0, false>); break;
  }
  return launched("combine_kernel");
}

extern "C" int dew_moe_scale_rows(const void* x, const int32_t* gather, const int32_t* slots, const float* weights, void* out,
                                  int32_t rows, int32_t depth, void* stream) {
  using namespace dew;
  DEW_REQUIRE(rows >= 0 && depth >= 8 && depth % 8 == 0, "dew_moe_scale_rows: rows %d, depth %d (whole 8s)", rows, depth);
  if (rows == 0) return DEW_MOE_OK;
  DEW_REQUIRE(x && gather && slots && weights && out, "dew_moe_scale_rows: x, gather, slots, weights and out must not be null");
  DEW_REQUIRE(aligned16(x) && aligned16(out), "dew_moe_scale_rows: x and out must be 16-byte aligned");
  const long long total = static_cast<long long>(rows) * (depth / 8);
  const int blocks = static_cast<int>(min((total + 255) / 256, 256ll * 64));
  hipLaunchKernelGGL(scale_rows_kernel, dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream), static_cast<const bf16_t*>(x), gather,
                     slots, weights, static_cast<bf16_t*>(out), rows, depth);
  return launched("scale_rows_kernel");
}

extern "C" int dew_moe_gate_rows(const void* x, const float* kernel, const void* rows_in, void* out, int32_t tokens, int32_t depth,
                                 int32_t width, void* stream) {
  using namespace dew;
  DEW_REQUIRE(tokens >= 0 && depth > 0 && depth % 8 == 0 && width > 0 && width % 8 == 0,
              "dew_moe_gate_rows: tokens %d, depth %d and width %d (whole 8s)", tokens, depth, width);
  if (tokens == 0) return DEW_MOE_OK;
  DEW_REQUIRE(x && kernel && rows_in && out, "dew_moe_gate_rows: x, kernel, rows and out must not be null");
  DEW_REQUIRE(aligned16(x) && aligned16(rows_in) && aligned16(out), "dew_moe_gate_rows: x, rows and out must be 16-byte aligned");
  hipLaunchKernelGGL(gate_rows_kernel, dim3((tokens + 3) / 4), dim3(256), 0, static_cast<hipStream_t>(stream), static_cast<const bf16_t*>(x),
                     kernel, static_cast<const bf16_t*>(rows_in), static_cast<bf16_t*>(out), tokens, depth, width);
  return launched("gate_rows_kernel");
}

extern "C" int dew_moe_gate_rows_add_f32(const void* x, const float* kernel, const void* shared, const void* routed, float* out,
                                         int32_t tokens, int32_t depth, int32_t width, void* stream) {
  using namespace dew;
  DEW_REQUIRE(tokens >= 0 && depth > 0 && depth % 8 == 0 && width > 0 && width % 8 == 0,
              "dew_moe_gate_rows_add_f32: tokens %d, depth %d and width %d (whole 8s)", tokens, depth, width);
  if (tokens == 0) return DEW_MOE_OK;
  DEW_REQUIRE(x && kernel && shared && routed && out, "dew_moe_gate_rows_add_f32: x, kernel, both row buffers and out must not be null");
  DEW_REQUIRE(aligned16(x) && aligned16(shared) && aligned16(routed) && aligned16(out),
              "dew_moe_gate_rows_add_f32: x, both row buffers and out must be 16-byte aligned");
  hipLaunchKernelGGL(gate_rows_add_f32_kernel, dim3((tokens + 3) / 4), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const bf16_t*>(x), kernel, static_cast<const bf16_t*>(shared), static_cast<const bf16_t*>(routed), out, tokens,
                     depth, width);
  return launched("gate_rows_add_f32_kernel");
}

extern "C" int dew_moe_swiglu(const void* gate, const void* up, void* hidden, int64_t count, void* stream) {
  return dew_moe_swiglu_clamped(gate, up, 0.0f, hidden, count, stream);
}

extern "C" int dew_moe_silu(const void* x, void* out, int64_t count, void* stream) {
  using namespace dew;
  DEW_REQUIRE(count >= 0 && count % 8 == 0, "dew_moe_silu: count %lld is not a multiple of 8", static_cast<long long>(count));
  if (count == 0) return DEW_MOE_OK;
  DEW_REQUIRE(x && out && aligned16(x) && aligned16(out), "dew_moe_silu: x and out must not be null and must be 16-byte aligned");
  const long long chunks = count / 8;
  const int blocks = static_cast<int>(min((chunks + 255) / 256, 256ll * 64));
  hipLaunchKernelGGL(swiglu_kernel, dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream), static_cast<const bf16_t*>(x),
                     static_cast<const bf16_t*>(nullptr), static_cast<bf16_t*>(out), chunks, 0.0f, DEW_MOE_GATE_SILU);
  return launched("swiglu_kernel");
}

extern "C" int dew_moe_relu2(const void* x, void* out, int64_t count, void* stream) {
  using namespace dew;
  DEW_REQUIRE(count >= 0 && count % 8 == 0, "dew_moe_relu2: count %lld is not a multiple of 8", static_cast<long long>(count));
  if (count == 0) return DEW_MOE_OK;
  DEW_REQUIRE(x && out && aligned16(x) && aligned16(out), "dew_moe_relu2: x and out must not be null and must be 16-byte aligned");
  const long long chunks = count / 8;
  const int blocks = static_cast<int>(min((chunks + 255) / 256, 256ll * 64));
  hipLaunchKernelGGL(swiglu_kernel, dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream), static_cast<const bf16_t*>(x),
                     static_cast<const bf16_t*>(nullptr), static_cast<bf16_t*>(out), chunks, 0.0f, DEW_MOE_ACT_RELU2);
  return launched("swiglu_kernel");
}

extern "C" int dew_moe_swiglu_clamped(const void* gate, const void* up, float limit, void* hidden, int64_t count, void* stream) {
  return dew_moe_gated_product(gate, up, DEW_MOE_GATE_SILU, limit, hidden, count, stream);
}

extern "C" int dew_moe_gated_product(const void* gate, const void* up, int32_t activation, float limit, void* hidden, int64_t count,
                                     void* stream) {
  using namespace dew;
  DEW_REQUIRE(activation == DEW_MOE_GATE_SILU || activation == DEW_MOE_GATE_GELU_TANH,
              "dew_moe_gated_product: the gate's activation %d is neither silu (0: swiglu) nor the tanh gelu (1: geglu)", activation);
  DEW_REQUIRE(limit >= 0.0f, "dew_moe_swiglu: the clamp limit %g must be positive (0: none)", static_cast<double>(limit));
  DEW_REQUIRE(count >= 0 && count % 8 == 0, "dew_moe_swiglu: count %lld is not a multiple of 8", static_cast<long long>(count));
  if (count == 0) return DEW_MOE_OK;
  DEW_REQUIRE(gate && up && hidden, "dew_moe_swiglu: gate, up and hidden must not be null");
  DEW_REQUIRE(aligned16(gate) && aligned16(up) && aligned16(hidden), "dew_moe_swiglu: buffers must be 16-byte aligned");
  const long long chunks = count / 8;
  const int blocks = static_cast<int>(min((chunks + 255) / 256, 256ll * 64));
  hipLaunchKernelGGL(swiglu_kernel, dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const bf16_t*>(gate), static_cast<const bf16_t*>(up), static_cast<bf16_t*>(hidden),
                     chunks, bf16_round_host(limit), activation);
  return launched("swiglu_kernel");
}

// XLA FFI handlers over libdew_moe_hip.so's C ABI: what jax.ffi registers for platform "ROCM", in the place the
// reference's CUTLASS wheel has for "CUDA" (kernels/cutlass/ffi.cu:180-277, registered by
// kernels/cutlass/dew_cutlass/__init__.py:63-82). Each handler checks ranks and dtypes, forms the plain-pointer call and
// turns a refusal into ffi::Error(kInvalidArgument, "<target>: <why>") as the reference's `failed` does (ffi.cu:93-95).
//
// Built only where XLA's FFI headers are (they ship with jaxlib: `python -c "import jax; print(jax.ffi.include_dir())"`);
// `make ffi XLA_FFI_INCLUDE=<dir>` in ../csrc compiles this file against them. The kernels stay testable without JAX
// through the C ABI itself.
//
// Conventions of the operands:
//  * an absent optional operand (a selection bias, gather/scatter indices, an epilogue bias, an addend, a bank's external
//    scales or tensor scales) is passed as an array of no elements;
//  * a prepared bank is three arrays, `prepared u8[dew_moe_prepared_bytes]`, `scales` (a per-channel FP8 bank's f32 [E, N],
//    else empty) and `tensor_scale` (an FP4 bank's f32 [E], else empty), with its format tag and extents as attributes;
//  * groups arrive as `group_sizes s32[E]`, the operand of jax.lax.ragged_dot and of dew_cutlass_grouped_gemm
//    (ffi.cu:185-198): the launches form the prefix on the device.
#include <cstdint>
#include <optional>
#include <string>

#include <hip/hip_runtime.h>

#include "xla/ffi/api/ffi.h"

#include "../../include/dew_moe_hip.h"

namespace ffi = xla::ffi;

namespace {

ffi::Error refused(const char* target) {
  return ffi::Error(ffi::ErrorCode::kInvalidArgument, std::string(target) + ": " + dew_moe_last_error());
}

ffi::Error misshaped(const char* target, const char* what) {
  return ffi::Error(ffi::ErrorCode::kInvalidArgument, std::string(target) + ": " + what);
}

// An optional operand's pointer: null for an array of no elements.
template <class Pointer = const void*>
Pointer present(const ffi::AnyBuffer& buffer) {
  return buffer.element_count() == 0 ? nullptr : static_cast<Pointer>(buffer.untyped_data());
}

bool is(const ffi::AnyBuffer& buffer, ffi::DataType type, size_t rank) {
  return buffer.element_type() == type && buffer.dimensions().size() == rank;
}

// Scratch aligned to 256 bytes. XLA's FFI refuses an alignment past 16, so the allocation is longer and its start
// rounded up (the reference does the same for 128, ffi.cu:83-91).
void* scratch_of(ffi::ScratchAllocator& scratch, size_t bytes) {
  std::optional<void*> memory = scratch.Allocate(bytes + 240, 16);
  if (!memory.has_value()) return nullptr;
  return reinterpret_cast<void*>((reinterpret_cast<uintptr_t>(*memory) + 255) / 256 * 256);
}

ffi::Error bank_of(const char* target, int32_t format, int32_t experts, int32_t depth, int32_t width, const ffi::AnyBuffer& prepared,
                   const ffi::AnyBuffer& scales, const ffi::AnyBuffer& tensor_scale, dew_moe_bank* bank) {
  if (prepared.element_type() != ffi::U8 || prepared.element_count() < dew_moe_prepared_bytes(format, experts, depth, width))
    return misshaped(target, "a prepared bank is u8[dew_moe_prepared_bytes(format, experts, depth, width)]");
  if (dew_moe_prepared_view(format, experts, depth, width, prepared.untyped_data(), present(scales),
                            present<const float*>(tensor_scale), bank))
    return refused(target);
  return ffi::Error::Success();
}

// ---- dew_moe_route_ffi: logits f32[T, E], bias f32[E] | f32[0] -> weights f32[T, k], indices s32[T, k] ----
ffi::Error Route(hipStream_t stream, ffi::AnyBuffer logits, ffi::AnyBuffer bias, ffi::Result<ffi::AnyBuffer> weights,
                 ffi::Result<ffi::AnyBuffer> indices, int32_t score_function, bool normalize, float scaling,
                 int32_t expert_groups, int32_t groups_per_token, int32_t group_score) {
  constexpr const char* kTarget = "dew_moe_route";
  if (!is(logits, ffi::F32, 2) || !is(*weights, ffi::F32, 2) || !is(*indices, ffi::S32, 2) || bias.element_type() != ffi::F32)
    return misshaped(kTarget, "logits f32[T, E], bias f32[E] or f32[0], weights f32[T, k], indices s32[T, k]");
  const int64_t tokens = logits.dimensions()[0], experts = logits.dimensions()[1], top_k = weights->dimensions()[1];
  if (weights->dimensions()[0] != tokens || indices->dimensions()[0] != tokens || indices->dimensions()[1] != top_k ||
      (bias.element_count() != 0 && static_cast<int64_t>(bias.element_count()) != experts))
    return misshaped(kTarget, "the extents of logits, bias, weights and indices do not agree");
  const dew_moe_router router{static_cast<int32_t>(experts), static_cast<int32_t>(top_k), score_function, normalize ? 1 : 0,
                              scaling, expert_groups, groups_per_token, group_score,
                              /* the switches this target leaves at the router's defaults */ 0, DEW_MOE_WEIGHT_SUM_EPSILON, 0.0f, 0, 0.0f, 0.0f};
  if (dew_moe_route_with(&router, static_cast<const float*>(logits.untyped_data()), present<const float*>(bias),
                         static_cast<int32_t>(tokens), static_cast<float*>(weights->untyped_data()),
                         static_cast<int32_t*>(indices->untyped_data()), nullptr, nullptr, stream))
    return refused(kTarget);
  return ffi::Error::Success();
}

// ---- dew_moe_permute_ffi: indices s32[T, k] -> sizes s32[G], offsets s32[G + 1], order s32[R + S], rows s32[R + S];
// G = experts (+ 1 with shared_rows S > 0, the always-on expert as one more group). Workspace from XLA's scratch. ----
ffi::Error Permute(hipStream_t stream, ffi::ScratchAllocator scratch, ffi::AnyBuffer indices, ffi::Result<ffi::AnyBuffer> sizes,
                   ffi::Result<ffi::AnyBuffer> offsets, ffi::Result<ffi::AnyBuffer> order, ffi::Result<ffi::AnyBuffer> rows,
                   int32_t experts, int32_t shared_rows) {
  constexpr const char* kTarget = "dew_moe_permute";
  if (!is(indices, ffi::S32, 2) || !is(*sizes, ffi::S32, 1) || !is(*offsets, ffi::S32, 1) || !is(*order, ffi::S32, 1) || !is(*rows, ffi::S32, 1))
    return misshaped(kTarget, "indices s32[T, k]; sizes s32[G], offsets s32[G + 1], order and rows s32[T * k + shared_rows]");
  const int64_t tokens = indices.dimensions()[0], top_k = indices.dimensions()[1];
  const int64_t groups = experts + (shared_rows > 0 ? 1 : 0), slots = tokens * top_k + shared_rows;
  if (sizes->dimensions()[0] != groups || offsets->dimensions()[0] != groups + 1 || order->dimensions()[0] != slots || rows->dimensions()[0] != slots)
    return misshaped(kTarget, "the extents of sizes, offsets, order and rows do not fit the slots and groups");
  const size_t bytes = dew_moe_permute_workspace_bytes(static_cast<int32_t>(slots), static_cast<int32_t>(groups));
  void* workspace = scratch_of(scratch, bytes);
  if (workspace == nullptr) return misshaped(kTarget, "XLA's scratch allocator has no room for the sort's counts");
  auto* out_sizes = static_cast<int32_t*>(sizes->untyped_data());
  auto* out_offsets = static_cast<int32_t*>(offsets->untyped_data());
  auto* out_order = static_cast<int32_t*>(order->untyped_data());
  auto* out_rows = static_cast<int32_t*>(rows->untyped_data());
  const auto* ids = static_cast<const int32_t*>(indices.untyped_data());
  const int status = shared_rows > 0
      ? dew_moe_permute_shared(ids, static_cast<int32_t>(tokens), static_cast<int32_t>(top_k), experts, shared_rows, out_sizes,
                               out_offsets, out_order, out_rows, workspace, bytes, stream)
      : dew_moe_permute(ids, static_cast<int32_t>(tokens), static_cast<int32_t>(top_k), experts, out_sizes, out_offsets, out_order,
                        out_rows, workspace, bytes, stream);
  if (status) return refused(kTarget);
  return ffi::Error::Success();
}

// ---- dew_moe_prepare_bank_ffi (load time; it waits for the stream once for FP4 banks): a bank in the reference's or the
// checkpoint's own layout -> prepared u8[bytes], tensor_scale f32[E] (an FP4 bank's: copied, or computed for a checkpoint's
// MXFP4 tensors; else untouched), tag s32[1] = the prepared bank's format, which the launches take as their attribute. ----
ffi::Error PrepareBank(hipStream_t stream, ffi::AnyBuffer codes, ffi::AnyBuffer scales, ffi::AnyBuffer tensor_scale,
                       ffi::Result<ffi::AnyBuffer> prepared, ffi::Result<ffi::AnyBuffer> prepared_tensor_scale,
                       ffi::Result<ffi::AnyBuffer> tag, int32_t format, int32_t layout, int32_t experts, int32_t depth, int32_t width) {
  constexpr const char* kTarget = "dew_moe_prepare_bank";
  if (prepared->element_type() != ffi::U8 || prepared->element_count() < dew_moe_prepared_bytes(format, experts, depth, width) ||
      !is(*tag, ffi::S32, 1) || tag->dimensions()[0] != 1)
    return misshaped(kTarget, "prepared u8[dew_moe_prepared_bytes(format, experts, depth, width)], tag s32[1]");
  const dew_moe_bank reference{format, layout, experts, depth, width, codes.untyped_data(), present(scales), present<const float*>(tensor_scale)};
  dew_moe_bank out{};
  if (dew_moe_prepare_bank(&reference, prepared->untyped_data(), &out, stream)) return refused(kTarget);
  if (out.tensor_scale != nullptr) {
    if (!is(*prepared_tensor_scale, ffi::F32, 1) || prepared_tensor_scale->dimensions()[0] != experts)
      return misshaped(kTarget, "an FP4 bank's prepared_tensor_scale is f32[E]");
    if (hipMemcpyAsync(prepared_tensor_scale->untyped_data(), out.tensor_scale, sizeof(float) * experts, hipMemcpyDeviceToDevice, stream) != hipSuccess)
      return misshaped(kTarget, "copying the tensor scales failed");
  }
  const int32_t found = out.format;  // (pageable host memory: the copy has read it when the call returns)
  if (hipMemcpyAsync(tag->untyped_data(), &found, sizeof(found), hipMemcpyHostToDevice, stream) != hipSuccess || hipStreamSynchronize(stream) != hipSuccess)
    return misshaped(kTarget, "writing the format tag failed");
  return ffi::Error::Success();
}

// ---- dew_moe_grouped_gemm_ffi: x bf16[M, K], a prepared bank, group_sizes s32[E], gather / scatter s32[rows] | s32[0],
// bias f32[E, N] | f32[0] -> out bf16[rows, N] (the place of dew_cutlass_grouped_gemm, ffi.cu:180-220) ----
ffi::Error GroupedGemm(hipStream_t stream, ffi::AnyBuffer x, ffi::AnyBuffer prepared, ffi::AnyBuffer scales, ffi::AnyBuffer tensor_scale,
                       ffi::Buffer<ffi::S32> group_sizes, ffi::AnyBuffer gather, ffi::AnyBuffer scatter, ffi::AnyBuffer bias,
                       ffi::Result<ffi::AnyBuffer> out, int32_t format, int32_t experts, int32_t depth, int32_t width) {
  constexpr const char* kTarget = "dew_moe_grouped_gemm";
  if (!is(x, ffi::BF16, 2) || !is(*out, ffi::BF16, 2) || group_sizes.dimensions().size() != 1 || group_sizes.dimensions()[0] != experts)
    return misshaped(kTarget, "x bf16[M, K], group_sizes s32[E], out bf16[rows, N]");
  const int64_t rows = out->dimensions()[0];
  if (x.dimensions()[1] != depth || out->dimensions()[1] != width || (gather.element_count() == 0 && rows > x.dimensions()[0]) ||
      (gather.element_count() != 0 && (gather.element_type() != ffi::S32 || static_cast<int64_t>(gather.element_count()) < rows)) ||
      (scatter.element_count() != 0 && (scatter.element_type() != ffi::S32 || static_cast<int64_t>(scatter.element_count()) < rows)) ||
      (bias.element_count() != 0 && (bias.element_type() != ffi::F32 || static_cast<int64_t>(bias.element_count()) != int64_t{experts} * width)))
    return misshaped(kTarget, "the extents of x, the bank, gather, scatter, bias and out do not chain");
  dew_moe_bank bank{};
  if (ffi::Error error = bank_of(kTarget, format, experts, depth, width, prepared, scales, tensor_scale, &bank); error.failure()) return error;
  if (dew_moe_grouped_gemm_sizes(x.untyped_data(), present<const int32_t*>(gather), group_sizes.typed_data(), &bank,
                                 present<const float*>(bias), present<const int32_t*>(scatter), out->untyped_data(),
                                 static_cast<int32_t>(rows), stream))
    return refused(kTarget);
  return ffi::Error::Success();
}

// ---- dew_moe_gateup_swiglu_ffi: x bf16[M, K], the gate's and the up projection's prepared banks, group_sizes s32[E],
// gather s32[rows] | s32[0] -> hidden bf16[rows, F] (paired_projections + gated_product in one launch; `activation` =
// DEW_MOE_GATE_*, `limit` > 0 = swiglu_clamped's clamp before the gate, 0 = none) ----
ffi::Error GateUpSwiglu(hipStream_t stream, ffi::AnyBuffer x, ffi::AnyBuffer gate_prepared, ffi::AnyBuffer gate_scales,
                        ffi::AnyBuffer gate_tensor_scale, ffi::AnyBuffer up_prepared, ffi::AnyBuffer up_scales,
                        ffi::AnyBuffer up_tensor_scale, ffi::Buffer<ffi::S32> group_sizes, ffi::AnyBuffer gather,
                        ffi::Result<ffi::AnyBuffer> hidden, int32_t format, int32_t experts, int32_t depth, int32_t width,
                        int32_t activation, float limit) {
  constexpr const char* kTarget = "dew_moe_gateup_swiglu";
  if (!is(x, ffi::BF16, 2) || !is(*hidden, ffi::BF16, 2) || group_sizes.dimensions().size() != 1 || group_sizes.dimensions()[0] != experts)
    return misshaped(kTarget, "x bf16[M, K], group_sizes s32[E], hidden bf16[rows, F]");
  const int64_t rows = hidden->dimensions()[0];
  if (x.dimensions()[1] != depth || hidden->dimensions()[1] != width || (gather.element_count() == 0 && rows > x.dimensions()[0]) ||
      (gather.element_count() != 0 && (gather.element_type() != ffi::S32 || static_cast<int64_t>(gather.element_count()) < rows)))
    return misshaped(kTarget, "the extents of x, the banks, gather and hidden do not chain");
  dew_moe_bank gate{}, up{};
  if (ffi::Error error = bank_of(kTarget, format, experts, depth, width, gate_prepared, gate_scales, gate_tensor_scale, &gate); error.failure()) return error;
  if (ffi::Error error = bank_of(kTarget, format, experts, depth, width, up_prepared, up_scales, up_tensor_scale, &up); error.failure()) return error;
  if (dew_moe_gateup_gated(x.untyped_data(), present<const int32_t*>(gather), nullptr, group_sizes.typed_data(), &gate, &up, activation,
                           limit, hidden->untyped_data(), static_cast<int32_t>(rows), stream))
    return refused(kTarget);
  return ffi::Error::Success();
}

// ---- dew_moe_swiglu_mlp_ffi: the routed experts' whole SwiGLU MLP (`ExpertMLP._project`, src/dew/nn/moe.py:1305-1326):
// x bf16[T, D], the gate's, up's and down's prepared banks, group_sizes s32[E], gather s32[rows] | s32[0],
// scatter s32[rows] | s32[0] -> out bf16[rows, D_out]. Where the library's rule says so (dew_moe_prefers_split_rows:
// MXFP4 banks, groups of hundreds of rows) the rows run as two e4m3 terms on the scaled matrix instruction
// (dew_moe_swiglu_mlp_split, its intermediates in XLA's scratch); else the paired launch and the down launch on bf16
// operands, the hidden rows in scratch. `second_term` = DEW_MOE_SECOND_TERM_* for the split form; `activation` and `limit`
// as the gate/up handler takes them. ----
ffi::Error SwigluMlp(hipStream_t stream, ffi::ScratchAllocator scratch, ffi::AnyBuffer x, ffi::AnyBuffer gate_prepared,
                     ffi::AnyBuffer gate_scales, ffi::AnyBuffer gate_tensor_scale, ffi::AnyBuffer up_prepared, ffi::AnyBuffer up_scales,
                     ffi::AnyBuffer up_tensor_scale, ffi::AnyBuffer down_prepared, ffi::AnyBuffer down_scales,
                     ffi::AnyBuffer down_tensor_scale, ffi::Buffer<ffi::S32> group_sizes, ffi::AnyBuffer gather, ffi::AnyBuffer scatter,
                     ffi::Result<ffi::AnyBuffer> out, int32_t format, int32_t experts, int32_t depth, int32_t hidden_width,
                     int32_t width, int32_t second_term, int32_t activation, float limit) {
  constexpr const char* kTarget = "dew_moe_swiglu_mlp";
  if (!is(x, ffi::BF16, 2) || !is(*out, ffi::BF16, 2) || group_sizes.dimensions().size() != 1 || group_sizes.dimensions()[0] != experts)
    return misshaped(kTarget, "x bf16[T, D], group_sizes s32[E], out bf16[rows, D_out]");
  const int64_t tokens = x.dimensions()[0], rows = out->dimensions()[0];
  auto indices_fit = [rows](const ffi::AnyBuffer& index) {
    return index.element_count() == 0 || (index.element_type() == ffi::S32 && static_cast<int64_t>(index.element_count()) >= rows);
  };
  if (x.dimensions()[1] != depth || out->dimensions()[1] != width || (gather.element_count() == 0 && rows > tokens) ||
      !indices_fit(gather) || !indices_fit(scatter))
    return misshaped(kTarget, "the extents of x, the banks, gather, scatter and out do not chain");
  dew_moe_bank gate{}, up{}, down{};
  if (ffi::Error error = bank_of(kTarget, format, experts, depth, hidden_width, gate_prepared, gate_scales, gate_tensor_scale, &gate); error.failure()) return error;
  if (ffi::Error error = bank_of(kTarget, format, experts, depth, hidden_width, up_prepared, up_scales, up_tensor_scale, &up); error.failure()) return error;
  if (ffi::Error error = bank_of(kTarget, format, experts, hidden_width, width, down_prepared, down_scales, down_tensor_scale, &down); error.failure()) return error;
  if (dew_moe_prefers_split_rows(&gate, &up, &down, static_cast<int32_t>(rows))) {
    const size_t bytes = dew_moe_swiglu_mlp_split_workspace_bytes(static_cast<int32_t>(tokens), static_cast<int32_t>(rows), depth, hidden_width, experts);
    void* workspace = scratch_of(scratch, bytes);
    if (workspace == nullptr) return misshaped(kTarget, "XLA's scratch allocator has no room for the split rows");
    if (dew_moe_gated_mlp_split(x.untyped_data(), static_cast<int32_t>(tokens), present<const int32_t*>(gather), nullptr,
                                group_sizes.typed_data(), &gate, &up, &down, activation, limit, present<const int32_t*>(scatter),
                                out->untyped_data(), static_cast<int32_t>(rows), second_term, workspace, bytes, stream))
      return refused(kTarget);
    return ffi::Error::Success();
  }
  void* hidden = scratch_of(scratch, static_cast<size_t>(rows) * hidden_width * 2);
  if (hidden == nullptr) return misshaped(kTarget, "XLA's scratch allocator has no room for the hidden rows");
  if (dew_moe_gateup_gated(x.untyped_data(), present<const int32_t*>(gather), nullptr, group_sizes.typed_data(), &gate, &up, activation,
                           limit, hidden, static_cast<int32_t>(rows), stream) ||
      dew_moe_grouped_gemm_sizes(hidden, nullptr, group_sizes.typed_data(), &down, nullptr, present<const int32_t*>(scatter),
                                 out->untyped_data(), static_cast<int32_t>(rows), stream))
    return refused(kTarget);
  return ffi::Error::Success();
}

// ---- dew_moe_combine_ffi: slots bf16[T, k, D], weights f32[T, k], addend bf16[T, D] | bf16[0] -> out bf16[T, D] ----
ffi::Error Combine(hipStream_t stream, ffi::AnyBuffer slots, ffi::AnyBuffer weights, ffi::AnyBuffer addend, ffi::Result<ffi::AnyBuffer> out) {
  constexpr const char* kTarget = "dew_moe_combine";
  if (!is(slots, ffi::BF16, 3) || !is(weights, ffi::F32, 2) || !is(*out, ffi::BF16, 2) || addend.element_type() != ffi::BF16)
    return misshaped(kTarget, "slots bf16[T, k, D], weights f32[T, k], addend bf16[T, D] or bf16[0], out bf16[T, D]");
  const int64_t tokens = slots.dimensions()[0], top_k = slots.dimensions()[1], width = slots.dimensions()[2];
  if (weights.dimensions()[0] != tokens || weights.dimensions()[1] != top_k || out->dimensions()[0] != tokens || out->dimensions()[1] != width ||
      (addend.element_count() != 0 && static_cast<int64_t>(addend.element_count()) != tokens * width))
    return misshaped(kTarget, "the extents of slots, weights, addend and out do not agree");
  if (dew_moe_combine(slots.untyped_data(), static_cast<const float*>(weights.untyped_data()), present(addend), out->untyped_data(),
                      static_cast<int32_t>(tokens), static_cast<int32_t>(top_k), static_cast<int32_t>(width), stream))
    return refused(kTarget);
  return ffi::Error::Success();
}

}  // namespace

XLA_FFI_DEFINE_HANDLER_SYMBOL(dew_moe_route_ffi, Route,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>()
                                  .Attr<int32_t>("score_function")
                                  .Attr<bool>("normalize")
                                  .Attr<float>("scaling")
                                  .Attr<int32_t>("expert_groups")
                                  .Attr<int32_t>("groups_per_token")
                                  .Attr<int32_t>("group_score"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(dew_moe_permute_ffi, Permute,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Ctx<ffi::ScratchAllocator>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>()
                                  .Attr<int32_t>("experts")
                                  .Attr<int32_t>("shared_rows"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(dew_moe_prepare_bank_ffi, PrepareBank,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>()
                                  .Attr<int32_t>("format")
                                  .Attr<int32_t>("layout")
                                  .Attr<int32_t>("experts")
                                  .Attr<int32_t>("depth")
                                  .Attr<int32_t>("width"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(dew_moe_grouped_gemm_ffi, GroupedGemm,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::Buffer<ffi::S32>>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>()
                                  .Attr<int32_t>("format")
                                  .Attr<int32_t>("experts")
                                  .Attr<int32_t>("depth")
                                  .Attr<int32_t>("width"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(dew_moe_gateup_swiglu_ffi, GateUpSwiglu,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::Buffer<ffi::S32>>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>()
                                  .Attr<int32_t>("format")
                                  .Attr<int32_t>("experts")
                                  .Attr<int32_t>("depth")
                                  .Attr<int32_t>("width")
                                  .Attr<int32_t>("activation")
                                  .Attr<float>("limit"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(dew_moe_swiglu_mlp_ffi, SwigluMlp,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Ctx<ffi::ScratchAllocator>()
                                  .Arg<ffi::AnyBuffer>()   // x
                                  .Arg<ffi::AnyBuffer>()   // gate: prepared, scales, tensor_scale
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>()   // up
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>()   // down
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::Buffer<ffi::S32>>()   // group_sizes
                                  .Arg<ffi::AnyBuffer>()   // gather
                                  .Arg<ffi::AnyBuffer>()   // scatter
                                  .Ret<ffi::AnyBuffer>()
                                  .Attr<int32_t>("format")
                                  .Attr<int32_t>("experts")
                                  .Attr<int32_t>("depth")
                                  .Attr<int32_t>("hidden_width")
                                  .Attr<int32_t>("width")
                                  .Attr<int32_t>("second_term")
                                  .Attr<int32_t>("activation")
                                  .Attr<float>("limit"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(dew_moe_combine_ffi, Combine,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>());

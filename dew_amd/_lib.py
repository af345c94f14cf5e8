"""Loader of libdew_moe_hip.so and its C ABI (include/dew_moe_hip.h) through ctypes.

The library is the only compute path: nothing here falls back to PyTorch or the CPU. A missing library
raises on first use, naming the build command."""

import ctypes
import os
from pathlib import Path

LIBRARY = Path(__file__).resolve().parent / "libdew_moe_hip.so"

W_FP8_BLOCK, W_FP8_CHANNEL, W_NVFP4, W_MXFP4, W_MXFP8, W_BF16, W_MXFP4_BLOCKS = 1, 2, 3, 4, 5, 6, 7
LAYOUT_REFERENCE, LAYOUT_PREPARED, LAYOUT_REFERENCE_KMAJOR = 0, 1, 2
SCORE_SOFTMAX, SCORE_SIGMOID, SCORE_SQRTSOFTPLUS = 0, 1, 2
SECOND_TERM_E4M3, SECOND_TERM_E2M3, TERMS_E2M3_PAIR = 0, 1, 2
GATE_SILU, GATE_GELU_TANH = 0, 1
GROUP_TOP2, GROUP_MAX = 0, 1

EXPORTS = (
    "dew_moe_last_error", "dew_moe_architecture", "dew_moe_kernels", "dew_moe_kernel_fields",
    "dew_moe_device_check", "dew_moe_route", "dew_moe_router_logits", "dew_moe_group_offsets", "dew_moe_permute_workspace_bytes", "dew_moe_permute", "dew_moe_permute_static", "dew_moe_permute_shared",
    "dew_moe_prepared_bytes", "dew_moe_prepare_bank", "dew_moe_prepared_view", "dew_moe_tile_rows", "dew_moe_grouped_gemm", "dew_moe_grouped_gemm_bias", "dew_moe_grouped_gemm_sizes", "dew_moe_grouped_gemm_param_bias", "dew_moe_gateup_swiglu_sizes",
    "dew_moe_gateup_interleaved", "dew_moe_split_rows", "dew_moe_grouped_gemm_split", "dew_moe_gateup_swiglu_split", "dew_moe_gateup_swiglu_split_out", "dew_moe_split_rows_fp6", "dew_moe_gateup_swiglu_split_fp6_out", "dew_moe_grouped_gemm_split_blocks", "dew_moe_route_sown", "dew_moe_balance_bias", "dew_moe_quantize_rows_nvfp4", "dew_moe_quantize_columns_fp8", "dew_moe_quantize_columns_mxfp8", "dew_moe_kernel_gradient_mxfp8", "dew_moe_transpose_columns", "dew_moe_transpose_groups", "dew_moe_quantize_columns_nvfp4", "dew_moe_kernel_gradient_bf16", "dew_moe_quantize_rows_mxfp8", "dew_moe_grouped_gemm_mxfp8_rows", "dew_moe_quantize_rows_fp8", "dew_moe_grouped_gemm_fp8_rows", "dew_moe_gateup_swiglu", "dew_moe_swiglu", "dew_moe_swiglu_clamped", "dew_moe_gated_product", "dew_moe_scale_rows", "dew_moe_gate_rows", "dew_moe_gate_rows_add_f32", "dew_moe_gateup_gated", "dew_moe_silu", "dew_moe_relu2", "dew_moe_prefers_split_rows", "dew_moe_swiglu_mlp_split_workspace_bytes", "dew_moe_swiglu_mlp_split", "dew_moe_gated_mlp_split", "dew_moe_capacity_admit", "dew_moe_route_with", "dew_moe_route_call", "dew_moe_route_blocks_workspace_bytes", "dew_moe_route_blocks", "dew_moe_combine",
    "dew_moe_rows_f16", "dew_moe_gateup_gated_f16", "dew_moe_split_rows_e2m3_pair", "dew_moe_gateup_swiglu_split_e2m3_pair_out",
)
"""Every symbol include/dew_moe_hip.h declares."""


class Bank(ctypes.Structure):
    """`dew_moe_bank` of include/dew_moe_hip.h."""

    _fields_ = [("format", ctypes.c_int32), ("layout", ctypes.c_int32), ("experts", ctypes.c_int32),
                ("depth", ctypes.c_int32), ("width", ctypes.c_int32), ("codes", ctypes.c_void_p),
                ("scales", ctypes.c_void_p), ("tensor_scale", ctypes.c_void_p)]


class Router(ctypes.Structure):
    """`dew_moe_router` of include/dew_moe_hip.h."""

    _fields_ = [("experts", ctypes.c_int32), ("top_k", ctypes.c_int32), ("score_function", ctypes.c_int32),
                ("normalize", ctypes.c_int32), ("scaling", ctypes.c_float), ("expert_groups", ctypes.c_int32),
                ("groups_per_token", ctypes.c_int32), ("group_score", ctypes.c_int32),
                ("bias_in_weights", ctypes.c_int32), ("weight_sum_epsilon", ctypes.c_float), ("weight_sum_min", ctypes.c_float),
                ("fill_excluded", ctypes.c_int32), ("excluded_group_score", ctypes.c_float), ("logit_softcap", ctypes.c_float)]


class KernelError(RuntimeError):
    """An entry point refused its arguments or a launch failed; the message is the library's own."""


_handle = None


def library() -> ctypes.CDLL:
    """The loaded library, its prototypes declared. Raises if it has not been built."""
    global _handle
    if _handle is not None:
        return _handle
    path = Path(os.environ.get("DEW_MOE_HIP_LIBRARY", LIBRARY))
    if not path.exists():
        raise KernelError(f"{path} is not built: run `make -C {LIBRARY.parent / 'csrc'}` (or "
                          f"`python -c 'import __graft_entry__ as g; g.build()'` at the repository root). "
                          f"There is no CPU or PyTorch fallback for the MoE kernels.")
    lib = ctypes.CDLL(str(path))
    c = ctypes
    ptr, i32, i64, f32, size = c.c_void_p, c.c_int32, c.c_int64, c.c_float, c.c_size_t
    bank = c.POINTER(Bank)
    prototypes = {
        "dew_moe_last_error": (c.c_char_p, []),
        "dew_moe_architecture": (c.c_char_p, []),
        "dew_moe_kernels": (c.c_char_p, []),
        "dew_moe_kernel_fields": (c.c_char_p, []),
        "dew_moe_device_check": (i32, []),
        "dew_moe_route": (i32, [ptr, ptr, i32, i32, i32, i32, i32, f32, i32, i32, ptr, ptr, ptr]),
        "dew_moe_route_sown": (i32, [ptr, ptr, i32, i32, i32, i32, i32, f32, i32, i32, ptr, ptr, ptr, ptr, ptr]),
        "dew_moe_balance_bias": (i32, [ptr, ptr, f32, i32, ptr]),
        "dew_moe_router_logits": (i32, [ptr, ptr, ptr, ptr, i32, i32, i32, ptr]),
        "dew_moe_group_offsets": (i32, [ptr, i32, ptr, ptr]),
        "dew_moe_permute_workspace_bytes": (size, [i32, i32]),
        "dew_moe_permute": (i32, [ptr, i32, i32, i32, ptr, ptr, ptr, ptr, ptr, size, ptr]),
        "dew_moe_permute_shared": (i32, [ptr, i32, i32, i32, i32, ptr, ptr, ptr, ptr, ptr, size, ptr]),
        "dew_moe_permute_static": (i32, [ptr, i32, i32, i32, ptr, ptr, ptr, ptr, ptr]),
        "dew_moe_prepared_bytes": (size, [i32, i32, i32, i32]),
        "dew_moe_prepare_bank": (i32, [bank, ptr, bank, ptr]),
        "dew_moe_prepared_view": (i32, [i32, i32, i32, i32, ptr, ptr, ptr, bank]),
        "dew_moe_tile_rows": (i32, [i32]),
        "dew_moe_grouped_gemm": (i32, [ptr, ptr, ptr, bank, ptr, ptr, i32, ptr]),
        "dew_moe_grouped_gemm_bias": (i32, [ptr, ptr, ptr, bank, ptr, ptr, ptr, i32, ptr]),
        "dew_moe_grouped_gemm_sizes": (i32, [ptr, ptr, ptr, bank, ptr, ptr, ptr, i32, ptr]),
        "dew_moe_grouped_gemm_param_bias": (i32, [ptr, ptr, ptr, ptr, bank, ptr, ptr, ptr, i32, ptr]),
        "dew_moe_gateup_swiglu_sizes": (i32, [ptr, ptr, ptr, bank, bank, ptr, i32, ptr]),
        "dew_moe_gateup_interleaved": (i32, [ptr, ptr, ptr, bank, ptr, f32, ptr, i32, ptr]),
        "dew_moe_split_rows": (i32, [ptr, ptr, ptr, i32, i32, ptr]),
        "dew_moe_grouped_gemm_split": (i32, [ptr, ptr, ptr, ptr, bank, ptr, ptr, ptr, i32, ptr]),
        "dew_moe_gateup_swiglu_split": (i32, [ptr, ptr, ptr, ptr, bank, bank, ptr, i32, ptr]),
        "dew_moe_gateup_swiglu_split_out": (i32, [ptr, ptr, ptr, ptr, bank, bank, ptr, ptr, i32, ptr]),
        "dew_moe_split_rows_fp6": (i32, [ptr, ptr, ptr, i32, i32, ptr]),
        "dew_moe_gateup_swiglu_split_fp6_out": (i32, [ptr, ptr, ptr, ptr, bank, bank, ptr, ptr, i32, ptr]),
        "dew_moe_grouped_gemm_split_blocks": (i32, [ptr, ptr, ptr, ptr, bank, ptr, ptr, ptr, i32, ptr]),
        "dew_moe_quantize_rows_fp8": (i32, [ptr, ptr, ptr, i32, i32, ptr]),
        "dew_moe_quantize_rows_mxfp8": (i32, [ptr, ptr, ptr, i32, i32, ptr]),
        "dew_moe_quantize_columns_fp8": (i32, [ptr, ptr, ptr, i32, i32, i32, ptr]),
        "dew_moe_quantize_columns_mxfp8": (i32, [ptr, ptr, ptr, i32, i32, i32, ptr]),
        "dew_moe_kernel_gradient_mxfp8": (i32, [ptr, ptr, bank, ptr, ptr, i32, i32, i32, ptr]),
        "dew_moe_transpose_columns": (i32, [ptr, ptr, i32, i32, i32, ptr]),
        "dew_moe_transpose_groups": (i32, [ptr, ptr, ptr, ptr, i32, i32, i32, i32, i32, ptr]),
        "dew_moe_quantize_columns_nvfp4": (i32, [ptr, ptr, ptr, ptr, i32, i32, i32, ptr]),
        "dew_moe_kernel_gradient_bf16": (i32, [ptr, bank, ptr, ptr, ptr, ptr, i32, i32, i32, ptr]),
        "dew_moe_quantize_rows_nvfp4": (i32, [ptr, ptr, ptr, ptr, i32, i32, ptr]),
        "dew_moe_grouped_gemm_mxfp8_rows": (i32, [ptr, ptr, ptr, ptr, bank, ptr, ptr, ptr, i32, ptr]),
        "dew_moe_grouped_gemm_fp8_rows": (i32, [ptr, ptr, ptr, ptr, bank, ptr, ptr, ptr, i32, ptr]),
        "dew_moe_gateup_swiglu": (i32, [ptr, ptr, ptr, bank, bank, ptr, i32, ptr]),
        "dew_moe_swiglu": (i32, [ptr, ptr, ptr, i64, ptr]),
        "dew_moe_swiglu_clamped": (i32, [ptr, ptr, f32, ptr, i64, ptr]),
        "dew_moe_silu": (i32, [ptr, ptr, i64, ptr]),
        "dew_moe_relu2": (i32, [ptr, ptr, i64, ptr]),
        "dew_moe_gate_rows": (i32, [ptr, ptr, ptr, ptr, i32, i32, i32, ptr]),
        "dew_moe_gate_rows_add_f32": (i32, [ptr, ptr, ptr, ptr, ptr, i32, i32, i32, ptr]),
        "dew_moe_gated_product": (i32, [ptr, ptr, i32, f32, ptr, i64, ptr]),
        "dew_moe_scale_rows": (i32, [ptr, ptr, ptr, ptr, ptr, i32, i32, ptr]),
        "dew_moe_gateup_gated": (i32, [ptr, ptr, ptr, ptr, bank, bank, i32, f32, ptr, i32, ptr]),
        "dew_moe_rows_f16": (i32, [ptr, ptr, ptr, i32, i32, ptr]),
        "dew_moe_split_rows_e2m3_pair": (i32, [ptr, ptr, i32, i32, ptr]),
        "dew_moe_gateup_swiglu_split_e2m3_pair_out": (i32, [ptr, ptr, ptr, bank, bank, ptr, ptr, i32, ptr]),
        "dew_moe_gateup_gated_f16": (i32, [ptr, ptr, ptr, ptr, ptr, bank, bank, i32, f32, ptr, i32, ptr]),
        "dew_moe_prefers_split_rows": (i32, [bank, bank, bank, i32]),
        "dew_moe_swiglu_mlp_split_workspace_bytes": (size, [i32, i32, i32, i32, i32]),
        "dew_moe_swiglu_mlp_split": (i32, [ptr, i32, ptr, ptr, ptr, bank, bank, bank, ptr, ptr, i32, i32, ptr, size, ptr]),
        "dew_moe_gated_mlp_split": (i32, [ptr, i32, ptr, ptr, ptr, bank, bank, bank, i32, f32, ptr, ptr, i32, i32, ptr, size, ptr]),
        "dew_moe_capacity_admit": (i32, [ptr, i32, i32, i32, i32, i32, ptr, ptr]),
        "dew_moe_route_with": (i32, [c.POINTER(Router), ptr, ptr, i32, ptr, ptr, ptr, ptr, ptr]),
        "dew_moe_route_blocks_workspace_bytes": (size, [i32, i32, i32]),
        "dew_moe_route_blocks": (i32, [c.POINTER(Router), ptr, ptr, ptr, i32, i32, i32, ptr, size, ptr, ptr, ptr, ptr, ptr]),
        "dew_moe_route_call": (i32, [c.POINTER(Router), ptr, ptr, ptr, ptr, ptr, ptr, i32, ptr, ptr, ptr, ptr, ptr]),
        "dew_moe_combine": (i32, [ptr, ptr, ptr, ptr, i32, i32, i32, ptr]),
    }
    for name, (restype, argtypes) in prototypes.items():
        function = getattr(lib, name)
        function.restype, function.argtypes = restype, argtypes
    _handle = lib
    return lib


def check(code: int, what: str) -> None:
    """Raise `KernelError` with the library's message unless `code` is 0."""
    if code != 0:
        raise KernelError(f"{what}: {library().dew_moe_last_error().decode()} (code {code})")

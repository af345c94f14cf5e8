"""A quantized checkpoint's expert banks taken to the kernels' formats at load time, without decoding a value:
the host-side mirror of the reference's `packed_banks` / `with_banks` (src/dew/interop/quantized_loads.py:106-168)
for MXFP4 sources (gpt-oss's `*_blocks` / `*_scales`), and the same service for FP8 128 x 128 block sources
(`weight` / `weight_scale_inv`, which the reference decodes at load, src/dew/interop/codecs.py:638-648) and for
DeepSeek-V4's FP4 routed experts (`weight` nibbles / E8M0 `scale`, MXFP4's own storage).

Tensors may live on the host or the device; every step is a torch index or bit operation, so a bank loaded to the
GPU is re-laid there. The banks go into the `'quantization'` collection at the path their parameter had.
"""

import dataclasses
import logging
from collections.abc import Mapping

import torch

from . import codecs, formats

_log = logging.getLogger(__name__)

MXFP4_SUFFIXES = ("_blocks", "_scales")
"""The two tensors an MXFP4 weight is stored as (src/dew/interop/codecs.py:463)."""
FP8_SUFFIXES = (".weight", ".weight_scale_inv")


@dataclasses.dataclass(frozen=True)
class Unread:
    """The shape and dtype of a leaf whose values are held elsewhere (the reference's `unread.Unread`)."""

    shape: tuple
    dtype: torch.dtype


def source_quantization(config: Mapping) -> str | None:
    found = config.get("quantization_config") or {}
    return found.get("quant_method")


def packed_banks(tensors: Mapping[str, torch.Tensor], config: Mapping, *, device_codec: bool | None = None) -> tuple[dict, dict]:
    """`tensors` with each MXFP4 expert bank taken out of the source's decoding, and those banks by their source
    names; in each one's place an `Unread` of its decoded shape. A bank whose depth is no whole NVFP4 stages, whose
    experts' group powers span past one tensor scale's reach, or that holds no experts stays as the source states it
    and is named in the log.

    A bank is the reference's `formats.NvFp4` (exactly the MXFP4 values: `codecs.mxfp4_as_nvfp4` then `NvFp4.of`, torch
    index and bit operations wherever the tensors live), or, with `device_codec` (the default for tensors on the GPU),
    `formats.Mxfp4Blocks`: the checkpoint's own two tensors, which the device re-layout takes straight to the same
    prepared bank (`dew_moe_prepare_bank` on `DEW_MOE_W_MXFP4_BLOCKS`) with no NvFp4 words formed in between."""
    if source_quantization(config) != "mxfp4":
        raise ValueError("packed_experts serves an MXFP4 source's expert banks (gpt-oss's quant_method mxfp4); "
                         f"this source's quantization is {config.get('quantization_config')!r}")
    tensors, banks = dict(tensors), {}
    names = sorted(name[:-len(MXFP4_SUFFIXES[0])] for name in tensors
                   if name.endswith(MXFP4_SUFFIXES[0]) and name[:-len(MXFP4_SUFFIXES[0])] + MXFP4_SUFFIXES[1] in tensors)
    for name in names:
        blocks, scales = (tensors[name + suffix] for suffix in MXFP4_SUFFIXES)
        on_device = blocks.is_cuda if device_codec is None else device_codec
        powers = None
        depth = blocks.shape[2] * codecs.GROUP if blocks.ndim == 4 else 0
        if blocks.ndim != 4:
            reason = "it holds no experts"
        elif depth % formats.NVFP4_STAGE and not (on_device and depth % 64 == 0 and depth >= 128 and blocks.shape[1] % 32 == 0):
            # (the reference's rule: its NvFp4 words are staged 256 deep. The device re-layout takes the checkpoint's own
            # tensors in atoms 64 deep and 32 wide, so there gpt-oss's 2880-deep banks stay packed)
            reason = f"its depth {depth} is no whole {formats.NVFP4_STAGE}-deep stages"
        elif on_device:
            # the device re-layout itself finds an expert whose group powers spread too far, and refuses the bank by name
            from . import gemm, ops

            bank = formats.Mxfp4Blocks(blocks.view(torch.uint8).contiguous(), scales.view(torch.uint8).contiguous())
            try:
                gemm.prepared(bank)
                powers = True
            except ops.KernelError as refusal:
                reason = str(refusal)
        else:
            powers = codecs.mxfp4_tensor_powers(blocks, scales)
            reason = "its experts' group powers span past one tensor scale's reach"
            bank = None if powers is None else formats.NvFp4.of(*codecs.mxfp4_as_nvfp4(blocks, scales, powers))
        if powers is None:
            _log.warning("packed_experts: %s stays dense: %s", name, reason)
            continue
        experts, outputs, groups, _ = blocks.shape
        banks[name] = bank
        for suffix in MXFP4_SUFFIXES:
            del tensors[name + suffix]
        tensors[name] = Unread((experts, groups * codecs.GROUP, outputs), torch.float32)
    return tensors, banks


def dense_bank(blocks: torch.Tensor, scales: torch.Tensor) -> formats.Bf16:
    """An MXFP4 expert bank that `packed_banks` left as the source states it (a depth in no whole NVFP4 stages:
    gpt-oss's 2880; group powers past one tensor scale's reach), decoded as the reference's load decodes it
    (`dequantize_mxfp4`, src/dew/interop/codecs.py:193-224) into the unquantized bank the grouped launches multiply:
    bf16 `[E, in, out]`, every MXFP4 value exactly."""
    return formats.Bf16(codecs.dequantize_mxfp4(blocks, scales, torch.bfloat16))


def fp8_block_bank(weights, scale_invs, *, device_codec: bool | None = None) -> formats.Fp8Blocks:
    """One projection's experts, each stored `[out, in]` e4m3 with `[out/128, in/128]` fp32 inverse scales
    (DeepSeek-V3 / Qwen3-FP8 checkpoints), as the bank the kernels multiply, still quantized: `[E, in, out]` codes
    transposed here, or, with `device_codec` (the default for tensors on the GPU), the tensors stacked as they are
    (`Fp8Blocks(kmajor=True)`), which the device re-layout reads where they lie."""
    weights, scale_invs = list(weights), list(scale_invs)
    on_device = weights[0].is_cuda if device_codec is None else device_codec
    if on_device:
        codes = torch.stack([weight.view(torch.uint8) for weight in weights]).contiguous()
        scales = torch.stack([scale.to(torch.float32) for scale in scale_invs]).contiguous()
        experts, width, depth = codes.shape
        expected = (experts, width // 128, depth // 128)
    else:
        codes = torch.stack([weight.view(torch.uint8).transpose(0, 1) for weight in weights]).contiguous()
        scales = torch.stack([scale.to(torch.float32).transpose(0, 1) for scale in scale_invs]).contiguous()
        experts, depth, width = codes.shape
        expected = (experts, depth // 128, width // 128)
    if depth % 128 or width % 128 or tuple(scales.shape) != expected:
        raise ValueError(f"an FP8 block bank is [E, in, out] in whole 128s with [E, in/128, out/128] scales, got codes "
                         f"{tuple(codes.shape)} and scales {tuple(scales.shape)}")
    return formats.Fp8Blocks(codes, scales, kmajor=on_device)


def fp8_expert_banks(tensors: Mapping[str, torch.Tensor], prefix: str, experts: int,
                     projections=("gate_proj", "up_proj", "down_proj")) -> tuple[dict, dict]:
    """`tensors` without `prefix.{e}.{projection}.weight[_scale_inv]` for e < experts, and the stacked FP8 block
    banks by projection name."""
    tensors, banks = dict(tensors), {}
    for projection in projections:
        names = [f"{prefix}.{e}.{projection}" for e in range(experts)]
        banks[projection] = fp8_block_bank([tensors[name + FP8_SUFFIXES[0]] for name in names],
                                           [tensors[name + FP8_SUFFIXES[1]] for name in names])
        for name in names:
            for suffix in FP8_SUFFIXES:
                del tensors[name + suffix]
    return tensors, banks


FP4_SUFFIXES = (".weight", ".scale")
"""The two tensors a DeepSeek-V4 FP4 routed expert is stored as (src/dew/interop/codecs.py `deepseek_v4(fp4_experts=True)`)."""


def fp4_expert_bank(weights, scales) -> formats.Mxfp4Blocks:
    """One projection's DeepSeek-V4 FP4 experts, each stored `[out, in / 2]` bytes of two E2M1 codes (the lower input in
    the low nibble) with `[out, in / 32]` E8M0 scales, as the MXFP4 bank the kernels multiply, still packed. The storage
    is MXFP4's own (an E2M1 code times `2 ** (scale - 127)` per 32 inputs), so the bytes are stacked and viewed as
    `[E, out, in / 32, 16]` blocks, not decoded (the reference's load decodes them dense, src/dew/interop/codecs.py
    `DeepseekV4.decode`); `codecs.dequantize_mxfp4` of the bank is the release's own reading of the expert in every value."""
    weights, scales = list(weights), list(scales)
    codes = torch.stack([weight.view(torch.uint8) for weight in weights]).contiguous()
    powers = torch.stack([scale.view(torch.uint8) for scale in scales]).contiguous()
    experts, width, half = codes.shape
    if half % 16 or tuple(powers.shape) != (experts, width, half // 16):
        raise ValueError(f"an FP4 expert is [out, in / 2] bytes in whole groups of 32 inputs with [out, in / 32] E8M0 scales, got "
                         f"{tuple(codes.shape)} and {tuple(powers.shape)}")
    return formats.Mxfp4Blocks(codes.reshape(experts, width, half // 16, 16), powers)


def fp4_expert_banks(tensors: Mapping[str, torch.Tensor], prefix: str, experts: int,
                     projections=("w1", "w3", "w2")) -> tuple[dict, dict]:
    """`tensors` without `prefix.{e}.{projection}.weight` / `.scale` for e < experts, and the stacked packed banks by
    projection name (the release's w1, w3, w2 are the gate, up and down projections)."""
    tensors, banks = dict(tensors), {}
    for projection in projections:
        names = [f"{prefix}.{e}.{projection}" for e in range(experts)]
        banks[projection] = fp4_expert_bank([tensors[name + FP4_SUFFIXES[0]] for name in names],
                                            [tensors[name + FP4_SUFFIXES[1]] for name in names])
        for name in names:
            for suffix in FP4_SUFFIXES:
                del tensors[name + suffix]
    return tensors, banks


def with_banks(variables: Mapping, paths: Mapping[str, tuple], banks: Mapping) -> dict:
    """`variables` with each bank in `'quantization'` under the path its source name binds (`paths[name]`, a
    path into `'params'`), the leaf there taken out of `'params'`; a name that binds no path is refused
    (src/dew/interop/quantized_loads.py:146-168)."""
    if not banks:
        return dict(variables)
    params = _copied(variables.get("params", {}))
    held = _copied(variables.get("quantization", {}))
    for name, bank in banks.items():
        path = paths.get(name)
        if not path:
            raise ValueError(f"{name} binds no path, which a packed bank does not take: it holds a whole "
                             "[experts, in, out] matrix at one path")
        node = params
        for key in path[:-1]:
            node = node.get(key, {})
        node.pop(path[-1], None)
        node = held
        for key in path[:-1]:
            node = node.setdefault(key, {})
        node[path[-1]] = bank
    return {**variables, "params": params, "quantization": held}


def _copied(tree):
    return {key: _copied(value) if isinstance(value, dict) else value for key, value in tree.items()}

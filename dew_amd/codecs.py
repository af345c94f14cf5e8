"""Quantizers and checkpoint codecs for the expert banks the MoE path multiplies: FP8 e4m3 with 128x128
block or per-output-channel fp32 scales, MXFP4 (E2M1 codes, one E8M0 scale per 32 inputs) and NVFP4 (E2M1
codes, one E4M3 scale per 16 inputs, one fp32 scale per expert). They follow the reference's rules
byte for byte (cited per function) and run as torch tensor programs on whichever device holds the weight,
so a full-size bank is quantized on the GPU without a host copy.

Layouts (E experts, K = depth = inputs, N = width = outputs):
  FP8 block     codes uint8 [E, K, N]      scale_inv fp32 [E, ceil(K/128), ceil(N/128)]
  FP8 channel   codes uint8 [E, K, N]      scales    fp32 [E, N]
  MXFP4         blocks uint8 [E, N, K/32, 16] (low nibble first)   scales uint8 [E, N, K/32] (E8M0)
  NVFP4 parts   nibbles uint8 [E, K, N]    block scales e4m3 bytes [E, K/16, N]   tensor scale fp32 [E]
"""

import torch

E4M3_MAX = 448.0
E2M1_MAX = 6.0
AMAX_FLOOR = 1e-4
GROUP = 32
E4M3_POWERS = (-9, 8)
"""The powers of two float8_e4m3fn holds exactly (reference src/dew/interop/codecs.py:226)."""

_E2M1_VALUES = (0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0)
_E2M1_MIDPOINTS = (0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0)


def e2m1_values(device=None) -> torch.Tensor:
    """Value of each E2M1 nibble, sign in bit 3."""
    positive = torch.tensor(_E2M1_VALUES, dtype=torch.float32, device=device)
    return torch.cat([positive, -positive])


def e4m3_bytes(x: torch.Tensor) -> torch.Tensor:
    """fp32 values within +-448 rounded to float8_e4m3fn (ties to even), as their bytes."""
    return x.to(torch.float32).to(torch.float8_e4m3fn).view(torch.uint8)


def e4m3_values(codes: torch.Tensor) -> torch.Tensor:
    """fp32 value of float8_e4m3fn bytes."""
    return codes.view(torch.float8_e4m3fn).to(torch.float32)


# ---- FP8 --------------------------------------------------------------------------------------------


def fp8_block_cast(weight: torch.Tensor, block=(128, 128)):
    """DeepGEMM's `per_block_cast_to_fp8` (reference src/dew/nn/fake_quant.py:250-262): zero-pad to whole
    blocks; per block `amax = max(|x|, 1e-4)`, `scale_inv = amax / 448` (IEEE fp32 division), codes =
    e4m3(x * (1 / scale_inv)) with one reciprocal per block. `weight [..., rows, cols]`; returns
    (codes uint8 `[..., rows, cols]`, scale_inv fp32 `[..., ceil(rows/br), ceil(cols/bc)]`)."""
    br, bc = (block, block) if isinstance(block, int) else block
    values = weight.to(torch.float32)
    *lead, rows, cols = values.shape
    pad_r, pad_c = -rows % br, -cols % bc
    padded = torch.nn.functional.pad(values, (0, pad_c, 0, pad_r))
    tiles = padded.reshape(*lead, (rows + pad_r) // br, br, (cols + pad_c) // bc, bc)
    amax = tiles.abs().amax(dim=(-3, -1)).clamp_min(torch.tensor(AMAX_FLOOR, dtype=torch.float32, device=values.device))
    scale_inv = amax / torch.tensor(E4M3_MAX, dtype=torch.float32, device=values.device)
    reciprocal = torch.tensor(1.0, dtype=torch.float32, device=values.device) / scale_inv
    codes = e4m3_bytes(tiles * reciprocal[..., :, None, :, None])
    codes = codes.reshape(*lead, rows + pad_r, cols + pad_c)[..., :rows, :cols].contiguous()
    return codes, scale_inv


def fp8_channel_cast(weight: torch.Tensor):
    """One fp32 scale per output channel: the block cast with a `(K, 1)` block on the `[K, N]` matrix (the
    reference's frozen row-scaled rule, src/dew/quantization.py:505-525, is this cast with `(1, K)` blocks
    on the `[N, K]` view). Returns (codes uint8 `[..., K, N]`, scales fp32 `[..., N]`)."""
    depth = weight.shape[-2]
    codes, scale_inv = fp8_block_cast(weight, (depth, 1))
    return codes, scale_inv[..., 0, :].contiguous()


def dequantize_fp8_blocks(codes: torch.Tensor, scale_inv: torch.Tensor, block=(128, 128)) -> torch.Tensor:
    """`f32(code) * scale_inv[block]` (reference src/dew/interop/codecs.py:670-703)."""
    br, bc = block
    rows, cols = codes.shape[-2:]
    each = scale_inv.repeat_interleave(br, dim=-2).repeat_interleave(bc, dim=-1)[..., :rows, :cols]
    return e4m3_values(codes) * each


# ---- MXFP4 ------------------------------------------------------------------------------------------


def quantize_mxfp4(weight: torch.Tensor):
    """The released GPT-OSS encoder (reference src/dew/interop/codecs.py:287-310): `weight [E, K, N]`
    rounded to bf16; each 32 inputs' scale byte is `amax / 6` rounded up to a power of two on the fp32 bits
    (`(bits + 0x007fffff) >> 23`, an all-zero group byte 0); codes round to the nearest E2M1 with ties away
    from zero. Returns (blocks uint8 `[E, N, K/32, 16]`, scales uint8 `[E, N, K/32]`)."""
    if weight.ndim != 3 or weight.shape[1] % GROUP:
        raise ValueError(f"MXFP4 takes an [expert, input, output] weight with inputs in 32s, got {tuple(weight.shape)}")
    values = weight.to(torch.bfloat16).to(torch.float32).transpose(1, 2)
    experts, outs, depth = values.shape
    groups = values.reshape(experts, outs, depth // GROUP, GROUP)
    ratio = groups.abs().amax(dim=-1) / torch.tensor(E2M1_MAX, dtype=torch.float32, device=values.device)
    bits = ratio.contiguous().view(torch.int32).to(torch.int64)
    exponents = ((bits + 0x007FFFFF) >> 23).to(torch.uint8)
    scale = torch.ldexp(torch.ones((), dtype=torch.float32, device=values.device), exponents.to(torch.int32) - 127)
    quotients = groups / scale[..., None]
    midpoints = torch.tensor(_E2M1_MIDPOINTS, dtype=torch.float32, device=values.device)
    magnitudes = torch.searchsorted(midpoints, quotients.abs().contiguous(), right=True).to(torch.uint8)
    codes = magnitudes | (torch.signbit(quotients).to(torch.uint8) << 3)
    packed = codes[..., 0::2] | (codes[..., 1::2] << 4)
    return packed.contiguous(), exponents


def dequantize_mxfp4(blocks: torch.Tensor, scales: torch.Tensor, dtype=torch.bfloat16) -> torch.Tensor:
    """Packed `[expert, output, group, 16]` blocks and E8M0 scales `[expert, output, group]` to `[expert, input, output]`
    in `dtype` (reference src/dew/interop/codecs.py:193-224, transformers' `convert_moe_packed_tensors`): the low nibble
    precedes the high one, a group of 32 inputs under the scale `2^(byte - 127)`; every value is exact in bf16. What a
    load does with a bank that stays dense (src/dew/interop/quantized_loads.py:126-136), wherever the tensors live."""
    codes = blocks.view(torch.uint8)
    experts, outputs, groups, packed = codes.shape
    if packed * 2 != GROUP or tuple(scales.shape) != (experts, outputs, groups):
        raise ValueError(f"MXFP4 blocks [E, N, K / 32, 16] with scales [E, N, K / 32], not {tuple(codes.shape)} with {tuple(scales.shape)}")
    nibbles = torch.stack([codes & 0xF, codes >> 4], dim=-1).reshape(experts, outputs, groups, GROUP)
    values = e2m1_values(codes.device)[nibbles.long()]
    decoded = torch.ldexp(values, (scales.view(torch.uint8).to(torch.int32) - 127)[..., None])
    return decoded.reshape(experts, outputs, groups * GROUP).transpose(1, 2).to(dtype).contiguous()


def mxfp4_tensor_powers(blocks: torch.Tensor, scales: torch.Tensor):
    """Each expert's power `k` that takes its E8M0 group powers into E4M3's range
    (reference src/dew/interop/codecs.py:238-262): the largest power of a group holding a nonzero code,
    less 8. None where an expert's powers spread past 17 binades, `2^k` leaves fp32's normals, or a scale
    byte is 0xff: such a bank stays dense."""
    if (scales == 255).any():
        return None
    held = (((blocks & 7) != 0) | (((blocks >> 4) & 7) != 0)).any(dim=-1)
    exponents = scales.to(torch.int32) - 127
    low, high = E4M3_POWERS
    any_held = held.flatten(1).any(dim=1)
    big = torch.iinfo(torch.int32)
    top = torch.where(held, exponents, torch.full_like(exponents, big.min)).flatten(1).amax(dim=1)
    bottom = torch.where(held, exponents, torch.full_like(exponents, big.max)).flatten(1).amin(dim=1)
    top = torch.where(any_held, top, torch.full_like(top, high))
    bottom = torch.where(any_held, bottom, torch.full_like(bottom, high))
    power = top - high
    if ((top - bottom) > high - low).any() or (power < -126).any() or (power > 127).any():
        return None
    return power.to(torch.int32)


def mxfp4_as_nvfp4(blocks: torch.Tensor, scales: torch.Tensor, powers: torch.Tensor):
    """An MXFP4 bank as NVFP4's parts, exactly and with no value decoded
    (reference src/dew/interop/codecs.py:265-284): nibbles `[E, K, N]`, each 16 inputs' E4M3 block scale
    bytes `[E, K/16, N]` (its group's power less its expert's, twice; a group of zeros takes 2^8), and each
    expert's fp32 tensor scale `2^k`."""
    experts, outs, groups, _ = blocks.shape
    nibbles = torch.stack([blocks & 15, blocks >> 4], dim=-1).reshape(experts, outs, groups * GROUP)
    held = (((blocks & 7) != 0) | (((blocks >> 4) & 7) != 0)).any(dim=-1)
    local = torch.where(held, scales.to(torch.int32) - 127 - powers[:, None, None].to(torch.int32),
                        torch.full_like(scales, E4M3_POWERS[1], dtype=torch.int32))
    one = torch.ones((), dtype=torch.float32, device=blocks.device)
    block = e4m3_bytes(torch.ldexp(one, local)).transpose(1, 2)
    tensor = torch.ldexp(one, powers.to(torch.int32)).to(torch.float32)
    return (nibbles.transpose(1, 2).contiguous(), block.repeat_interleave(GROUP // 16, dim=1).contiguous(), tensor)


# ---- NVFP4 ------------------------------------------------------------------------------------------


def _e2m1_rne(quotients: torch.Tensor) -> torch.Tensor:
    """fp32 values to E2M1 nibbles, nearest with ties to even, saturating at +-6, sign kept on zero."""
    midpoints = torch.tensor(_E2M1_MIDPOINTS, dtype=torch.float32, device=quotients.device)
    magnitude = quotients.abs().contiguous()
    above = torch.searchsorted(midpoints, magnitude, right=True)       # ties go up
    below = torch.searchsorted(midpoints, magnitude, right=False)      # ties go down
    # A tie (above != below) goes to the even code: codes 0, 2, 4, 6 have a zero mantissa bit.
    chosen = torch.where((above != below) & (above % 2 == 1), below, above).to(torch.uint8)
    return chosen | (torch.signbit(quotients).to(torch.uint8) << 3)


def nvfp4_coded(x: torch.Tensor):
    """One `[K, N]` fp32 matrix as NVFP4 (reference src/dew/algebra/bits.py:941-982; closed form stated by
    its tests/test_algebra_bits.py:510-528): tensor scale `amax / (6 * 448)` (at least fp32's least normal;
    1 for a zero tile); block scale the least e4m3 at or above `blockamax / tensor / 6`; codes
    `RNE_e2m1(x / tensor / block)`, a zero block's codes zero. Every quotient is an IEEE fp32 division of
    the values divided down, never a division by a product of scales.
    Returns (nibbles uint8 `[K, N]`, block scales e4m3 bytes `[K/16, N]`, tensor scale fp32 scalar)."""
    x = x.to(torch.float32)
    depth, width = x.shape
    if depth % 16:
        raise ValueError(f"NVFP4 blocks are 16 deep, got depth {depth}")
    f32 = dict(dtype=torch.float32, device=x.device)
    magnitude = x.abs()
    largest = magnitude.max()
    tiny = torch.tensor(torch.finfo(torch.float32).tiny, **f32)
    tensor = torch.where(largest > 0, torch.maximum(largest / torch.tensor(E2M1_MAX * E4M3_MAX, **f32), tiny),
                         torch.ones((), **f32))
    blocks = magnitude.reshape(depth // 16, 16, width).amax(dim=1)
    ratio = (blocks / tensor) / torch.tensor(E2M1_MAX, **f32)
    nearest = e4m3_bytes(ratio.clamp(max=E4M3_MAX)).to(torch.int32)
    bumped = torch.where(e4m3_values(nearest.to(torch.uint8)) < ratio, (nearest + 1).clamp(max=0x7E), nearest)
    codes = bumped.to(torch.uint8)
    each = e4m3_values(codes).repeat_interleave(16, dim=0)
    positive = each > 0
    scaled = torch.where(positive, (x / tensor) / torch.where(positive, each, torch.ones_like(each)),
                         torch.zeros_like(x))
    return _e2m1_rne(scaled), codes, tensor

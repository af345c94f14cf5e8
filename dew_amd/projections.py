"""The blockwise FP8 recipe's projection, forward only, shaped as the reference's
(`src/dew/nn/kernels/projections.py:50-60,96-204`: `blockwise_fp8_projection`, `recipe_projection`,
`rows_quantized`, `blocks_quantized`; product `gemm.blockwise_fp8_product` `src/dew/nn/kernels/gemm.py:764-793`).

DeepSeek-V3's recipe: activations quantized to E4M3 a 1 x 128 tile at a time along the depth, weights a
128 x 128 block at a time, both under power-of-two scales; each 128-deep block's partial, exact, times its
row's and its block's scale, summed in fp32, rounded once. On gfx950 both operands enter
`v_mfma_scale_f32_32x32x64_f8f6f4` as stored, codes and scales: the rows' quantizer is one HBM-bound launch
(`ops.quantize_rows_fp8`) and the product one grouped launch (`ops.grouped_gemm_fp8_rows`). A group's rows need
no padding to whole 128-row blocks here (the launch finds its tiles from the group offsets), so
`recipe_projection` takes ragged groups as they are; the zero rows the reference pads with add nothing there.
The recipe's gradients (its own FP8 products of requantized operands) are not part of this package.
"""

import dataclasses

import torch

from . import formats, gemm, ops

SCALE_DEPTH = 128
"""The recipe's block: activations 1 x 128, weights 128 x 128 (`templates.product.SCALE_DEPTH`)."""

_E4M3_MAX = 448.0
_AMAX_FLOOR = 1e-4


def _power_of_two_ceil(value: torch.Tensor) -> torch.Tensor:
    """The least power of two >= `value`, off its fp32 bits (src/dew/nn/fake_quant.py:48-57)."""
    bits = value.contiguous().view(torch.int32)
    field = ((bits >> 23) & 0xFF) + ((bits & 0x7FFFFF) != 0).to(torch.int32)
    return (field << 23).view(torch.float32)


def blocks_quantized(w: torch.Tensor) -> formats.Fp8Blocks:
    """`w [groups, depth, width]` as E4M3 codes a 128 x 128 block at a time, each block's scale the least power
    of two >= max(amax, 1e-4) * f32(1 / 448) (src/dew/nn/kernels/projections.py:185-196 over
    src/dew/nn/fake_quant.py:117-128): the bank the recipe's product multiplies, made once where the weights are
    held fixed."""
    values = w.to(torch.float32)
    groups, depth, width = values.shape
    if depth % SCALE_DEPTH or width % SCALE_DEPTH:
        raise ValueError(f"a {depth} x {width} matrix holds no whole {SCALE_DEPTH}-wide blocks")
    edge = SCALE_DEPTH
    tiles = values.reshape(groups, depth // edge, edge, width // edge, edge)
    amax = tiles.abs().amax(dim=(2, 4)).clamp_min(torch.tensor(_AMAX_FLOOR, dtype=torch.float32, device=values.device))
    scale = _power_of_two_ceil(amax * torch.tensor(1 / _E4M3_MAX, dtype=torch.float32, device=values.device))
    quotient = (tiles / scale[:, :, None, :, None]).clamp(-_E4M3_MAX, _E4M3_MAX)
    codes = quotient.to(torch.float8_e4m3fn).view(torch.uint8).reshape(groups, depth, width).contiguous()
    return formats.Fp8Blocks(codes, scale.contiguous())


@dataclasses.dataclass(frozen=True)
class QuantizedRows:
    """Rows as `ops.quantize_rows_fp8` writes them: `codes [rows, K]` uint8, each 128 depths in the scaled matrix
    instruction's operand order, and `scales [rows, P]` their tiles' e8m0 bytes."""

    codes: torch.Tensor
    scales: torch.Tensor

    def values(self) -> tuple[torch.Tensor, torch.Tensor]:
        """(codes in depth order `[rows, K]` uint8, scales fp32 `[rows, K / 128]`): the reference's `rows_quantized`."""
        blocks = self.codes.shape[1] // SCALE_DEPTH
        scales = (self.scales[:, :blocks].to(torch.int32) << 23).view(torch.float32)
        return ops.depth_order_fp8(self.codes), scales


def rows_quantized(x: torch.Tensor) -> QuantizedRows:
    """`x [rows, K]` bf16 as E4M3 codes a 1 x 128 tile at a time along the depth and each tile's power-of-two scale
    (src/dew/nn/kernels/projections.py:176-182), on the device."""
    return QuantizedRows(*ops.quantize_rows_fp8(x.contiguous()))


def _offsets(group_sizes, rows: int, device) -> torch.Tensor:
    if group_sizes is None:
        return torch.tensor([0, rows], dtype=torch.int32, device=device)
    return gemm.GroupSizes.of(group_sizes).offsets


def blockwise_fp8_product(lhs: QuantizedRows, kernel, group_sizes, *, out_dtype=torch.bfloat16, bias=None,
                          gather=None, scatter=None) -> torch.Tensor:
    """Each group's quantized rows times its matrix of the FP8 block bank `kernel` (`formats.Fp8Blocks` with
    power-of-two scales, or its prepared form), each 128-deep block's exact partial under its rows' and its block's
    scales, fp32 sums (+ `bias [groups, width]`), one rounding (src/dew/nn/kernels/gemm.py:764-793). Scales that
    are not powers of two have no place in the instruction: the launch writes NaN where it meets one."""
    if out_dtype != torch.bfloat16:
        raise ValueError(f"the launch writes bfloat16, not {out_dtype}")
    bank = gemm.prepared(kernel)
    rows = lhs.codes.shape[0] if gather is None else gather.numel()
    return ops.grouped_gemm_fp8_rows(lhs.codes, lhs.scales, bank, _offsets(group_sizes, rows, lhs.codes.device),
                                     gather=gather, scatter=scatter, bias=bias)


def blockwise_fp8_projection(x: torch.Tensor, w, group_blocks, *, out_dtype=torch.bfloat16) -> torch.Tensor:
    """Each group's rows of `x [rows, depth]` times its matrix of `w [groups, depth, width]` in the blockwise FP8
    recipe; group `g` holds `group_blocks[g]` whole 128-row blocks, in order (src/dew/nn/kernels/projections.py:
    50-60). `w` is the weights (quantized here, `blocks_quantized`) or a bank already quantized."""
    bank = w if isinstance(w, (formats.Fp8Blocks, ops.PreparedBank)) else blocks_quantized(w)
    sizes = (torch.as_tensor(group_blocks, device=x.device).to(torch.int32) * SCALE_DEPTH).contiguous()
    return blockwise_fp8_product(rows_quantized(x), bank, sizes, out_dtype=out_dtype)


def recipe_projection(rows: torch.Tensor, matrix, group_sizes=None, *, out_dtype=torch.bfloat16, bias=None,
                      recipe: str = "blockwise_fp8"):
    """`rows @ matrix` in a low-precision recipe (`'blockwise_fp8'`, `'mxfp8'` or `'nvfp4'`: the reference reads the
    run's, `recipe_role`; here the caller names it): a dense projection's (`matrix [in, out]`, every row its one
    group's) or experts' (`[groups, in, out]`, `group_sizes` counting each group's leading rows, any past their sum
    zero), `bias [groups, out]` added to the fp32 sums before the one rounding
    (src/dew/nn/kernels/projections.py:96-140). The reference pads each group with zero rows to whole 128-row blocks
    for its launches; a zero row changes no other row's quantization and adds nothing, and these launches take ragged
    groups as they are. None where the widths hold no whole 128-wide blocks (`recipe_refusal`'s 'block_shape',
    :62-83): the caller then keeps the projection in the run's dtypes."""
    if recipe not in ("blockwise_fp8", "mxfp8", "nvfp4"):
        raise ValueError(f"no recipe {recipe!r}: 'blockwise_fp8', 'mxfp8' or 'nvfp4'")
    if recipe != "blockwise_fp8":
        if isinstance(matrix, (formats.MxFp8, formats.NvFp4, ops.PreparedBank)):
            bank = matrix
        else:
            stacked = matrix if matrix.dim() == 3 else matrix[None]
            if stacked.shape[1] % SCALE_DEPTH or stacked.shape[2] % SCALE_DEPTH or (recipe == "nvfp4" and stacked.shape[1] % 256):
                return None  # (an NVFP4 bank's depth is whole 256s)
            bank = formats.MxFp8.quantized(stacked) if recipe == "mxfp8" else nvfp4_matrices(stacked)
        if bias is not None:
            bias = bias.reshape(bank.shape[0], bank.shape[2]).to(torch.float32).contiguous()
        if group_sizes is None:
            group_sizes = torch.tensor([rows.shape[0]], dtype=torch.int32, device=rows.device)
        if recipe == "mxfp8":
            return mxfp8_product(mxfp8_rows(rows), bank, group_sizes, out_dtype=out_dtype, bias=bias)
        return nvfp4_block_product(nvfp4_rows(rows), bank, group_sizes, out_dtype=out_dtype, bias=bias)
    if isinstance(matrix, (formats.Fp8Blocks, ops.PreparedBank)):
        bank = matrix
    else:
        stacked = matrix if matrix.dim() == 3 else matrix[None]
        if stacked.shape[1] % SCALE_DEPTH or stacked.shape[2] % SCALE_DEPTH:
            return None
        bank = blocks_quantized(stacked)
    if bias is not None:
        bias = bias.reshape(bank.shape[0], bank.shape[2]).to(torch.float32).contiguous()  # widened as it is stored (:141)
    return blockwise_fp8_product(rows_quantized(rows), bank, group_sizes, out_dtype=out_dtype, bias=bias)


# ---- the MXFP8 recipe (OCP MX) ---------------------------------------------------------------------------


@dataclasses.dataclass(frozen=True)
class MxFp8Rows:
    """Rows as `ops.quantize_rows_mxfp8` writes them: `codes [rows, K]` uint8, each 128 depths in the scaled matrix
    instruction's operand order, and `scales [rows, K / 32]` E8M0 bytes in depth order."""

    codes: torch.Tensor
    scales: torch.Tensor

    def values(self) -> tuple[torch.Tensor, torch.Tensor]:
        """(codes in depth order, scales): the reference's `MxFp8.quantized(x)` fields."""
        return ops.depth_order_fp8(self.codes), self.scales


def mxfp8_rows(x: torch.Tensor) -> MxFp8Rows:
    """`MxFp8.quantized(x)` for rows `[rows, K]` bf16 (src/dew/nn/kernels/formats.py:195-229), on the device."""
    return MxFp8Rows(*ops.quantize_rows_mxfp8(x.contiguous()))


def mxfp8_product(lhs: MxFp8Rows, matrices, group_sizes, *, out_dtype=torch.bfloat16, bias=None, gather=None,
                  scatter=None) -> torch.Tensor:
    """Each group's MXFP8 rows times its matrix of the MXFP8 bank `matrices` (`formats.MxFp8`, or its prepared form):
    every (code x scale) product exact, fp32 sums (+ `bias [groups, width]`), one rounding
    (src/dew/nn/kernels/gemm.py:882-892, with its `gather`)."""
    if out_dtype != torch.bfloat16:
        raise ValueError(f"the launch writes bfloat16, not {out_dtype}")
    bank = gemm.prepared(matrices)
    rows = lhs.codes.shape[0] if gather is None else gather.numel()
    return ops.grouped_gemm_mxfp8_rows(lhs.codes, lhs.scales, bank, _offsets(group_sizes, rows, lhs.codes.device),
                                       gather=gather, scatter=scatter, bias=bias)


def mxfp8_projection(x: torch.Tensor, w, group_blocks, *, out_dtype=torch.bfloat16) -> torch.Tensor:
    """Each group's rows of `x [rows, depth]` times its matrix of `w [groups, depth, width]` in the MXFP8 recipe, both
    quantized along the depth (src/dew/nn/kernels/projections.py:231-258); group `g` holds `group_blocks[g]` whole
    128-row blocks. `w` is the weights (quantized here) or an MXFP8 bank already quantized."""
    bank = w if isinstance(w, (formats.MxFp8, ops.PreparedBank)) else formats.MxFp8.quantized(w)
    sizes = (torch.as_tensor(group_blocks, device=x.device).to(torch.int32) * SCALE_DEPTH).contiguous()
    return mxfp8_product(mxfp8_rows(x), bank, sizes, out_dtype=out_dtype)


# ---- the NVFP4 recipe ------------------------------------------------------------------------------------


@dataclasses.dataclass(frozen=True)
class NvFp4Rows:
    """Rows quantized to NVFP4 (`ops.quantize_rows_nvfp4`): `values [rows, K]` bf16, each its E2M1 code times its 16
    depths' E4M3 scale (exact), and the operand's tensor `scale [1]` fp32."""

    values: torch.Tensor
    scale: torch.Tensor


def nvfp4_rows(x: torch.Tensor) -> NvFp4Rows:
    """`NvFp4Block.quantized(x)` for rows `[rows, K]` bf16 (src/dew/nn/kernels/formats.py:263-274), on the device."""
    return NvFp4Rows(*ops.quantize_rows_nvfp4(x.contiguous()))


def nvfp4_matrices(w: torch.Tensor) -> formats.NvFp4:
    """`w [groups, depth, width]` as the recipe quantizes its matrices: NVFP4 along the depth, all of them under one
    tensor scale (`NvFp4Block.quantized(swapaxes(w, 1, 2))` flattens the groups into one operand,
    src/dew/nn/kernels/projections.py:243-247), packed as the bank the kernels multiply."""
    from . import codecs

    groups, depth, width = w.shape
    together = w.to(torch.float32).permute(1, 0, 2).reshape(depth, groups * width)
    codes, scales, tensor = codecs.nvfp4_coded(together)
    codes = codes.reshape(depth, groups, width).permute(1, 0, 2).contiguous()
    scales = scales.reshape(depth // 16, groups, width).permute(1, 0, 2).contiguous()
    return formats.NvFp4.of(codes, scales, tensor.reshape(1).expand(groups).contiguous())


def nvfp4_block_product(lhs: NvFp4Rows, matrices, group_sizes, *, out_dtype=torch.bfloat16, bias=None, gather=None,
                        scatter=None) -> torch.Tensor:
    """Each group's NVFP4 rows times its matrix of the NVFP4 bank `matrices`: every (code x block scale) product exact,
    fp32 sums, times both tensor scales, one rounding (src/dew/nn/kernels/gemm.py:937-947). The rows' values are
    exact in bf16, so this is the bank's bf16-operand launch with the rows' tensor scale folded into the bank's."""
    if out_dtype != torch.bfloat16:
        raise ValueError(f"the launch writes bfloat16, not {out_dtype}")
    bank = gemm.prepared(matrices).scaled(lhs.scale)
    rows = lhs.values.shape[0] if gather is None else gather.numel()
    return ops.grouped_gemm(lhs.values, bank, _offsets(group_sizes, rows, lhs.values.device), gather=gather, scatter=scatter, bias=bias)


def nvfp4_projection(x: torch.Tensor, w, group_blocks, *, out_dtype=torch.bfloat16) -> torch.Tensor:
    """Each group's rows of `x [rows, depth]` times its matrix of `w [groups, depth, width]` in the NVFP4 recipe, both
    quantized along the depth (src/dew/nn/kernels/projections.py:261-275); group `g` holds `group_blocks[g]` whole
    128-row blocks. `w` is the weights (quantized here, `nvfp4_matrices`) or an NVFP4 bank already quantized."""
    bank = w if isinstance(w, (formats.NvFp4, ops.PreparedBank)) else nvfp4_matrices(w)
    sizes = (torch.as_tensor(group_blocks, device=x.device).to(torch.int32) * SCALE_DEPTH).contiguous()
    return nvfp4_block_product(nvfp4_rows(x), bank, sizes, out_dtype=out_dtype)


# ---- the recipes' gradients ------------------------------------------------------------------------------


def _group_offsets(group_blocks, device) -> torch.Tensor:
    sizes = torch.as_tensor(group_blocks, device=device).to(torch.int64) * SCALE_DEPTH
    return torch.cat([sizes.new_zeros(1), sizes.cumsum(0)]).to(torch.int32).contiguous()


def kernel_gradient(x: torch.Tensor, cotangent: torch.Tensor, group_blocks, *, mx: bool, out_dtype=torch.bfloat16) -> torch.Tensor:
    """A recipe's gradient for the matrices, `[groups, depth, width]`: each group's tokens of `x [tokens, depth]` and
    `cotangent [tokens, width]` contracted after both are quantized ALONG THE TOKENS: the blockwise FP8 recipe's
    1 x 128 tiles (`rows_quantized(x.T)`, `blockwise_fp8_kernel_gradient`, src/dew/nn/kernels/projections.py:220-223)
    or, `mx`, MXFP8's blocks of 32 tokens (src/dew/nn/kernels/projections.py:268-274). Group `g` holds
    `group_blocks[g]` whole 128-token blocks; an empty group's gradient is zero."""
    codes, scales = ops.quantize_columns(x.contiguous(), mx=mx, as_bank=False)
    bank = ops.quantize_columns(cotangent.contiguous(), mx=mx, as_bank=True)
    return ops.kernel_gradient_mxfp8(codes, scales, bank, _group_offsets(group_blocks, x.device), out_dtype=out_dtype)


def blockwise_fp8_gradients(x: torch.Tensor, w: torch.Tensor, cotangent: torch.Tensor, group_blocks, *, out_dtype=torch.bfloat16):
    """`_projection_backward` (src/dew/nn/kernels/projections.py:211-224) -> (d_x, d_w). The input's gradient is the
    recipe's own product of the requantized cotangent and the matrices' blocks transposed (a 128 x 128 block and its
    scale transpose as they are); the matrices' is `kernel_gradient`."""
    d_x = blockwise_fp8_projection(cotangent, w.transpose(1, 2).contiguous(), group_blocks, out_dtype=x.dtype)
    return d_x, kernel_gradient(x, cotangent, group_blocks, mx=False, out_dtype=out_dtype)


def mxfp8_gradients(x: torch.Tensor, w: torch.Tensor, cotangent: torch.Tensor, group_blocks, *, out_dtype=torch.bfloat16):
    """`_mx_backward` (src/dew/nn/kernels/projections.py:263-275) -> (d_x, d_w): the MXFP8 product of the cotangent and
    the matrices, both quantized along the width, and `kernel_gradient` with a scale every 32 tokens."""
    d_x = mxfp8_projection(cotangent, w.transpose(1, 2).contiguous(), group_blocks, out_dtype=x.dtype)
    return d_x, kernel_gradient(x, cotangent, group_blocks, mx=True, out_dtype=out_dtype)


def nvfp4_gradients(x: torch.Tensor, w: torch.Tensor, cotangent: torch.Tensor, group_blocks, *, out_dtype=torch.bfloat16):
    """`_nvfp4_backward` (src/dew/nn/kernels/projections.py:322-337) -> (d_x, d_w): the NVFP4 product of the cotangent
    and the matrices, both quantized along the width; and each group's tokens contracted over `x` and the cotangent
    quantized along the tokens, every 16 a scale. The decoded operands short of their tensor scales are exact in bf16,
    so the contraction is the bf16 kernel gradient with both tensor scales applied to its fp32 sums."""
    d_x = nvfp4_projection(cotangent, w.transpose(1, 2).contiguous(), group_blocks, out_dtype=x.dtype)
    rows, rows_scale = ops.transpose_columns(x.contiguous(), nvfp4=True, as_bank=False)
    bank, bank_scale = ops.transpose_columns(cotangent.contiguous(), nvfp4=True, as_bank=True)
    d_w = ops.kernel_gradient_bf16(rows, bank, _group_offsets(group_blocks, x.device), lhs_scale=rows_scale, rhs_scale=bank_scale,
                                   out_dtype=out_dtype)
    return d_x, d_w


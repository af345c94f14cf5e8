"""The grouped-product front the MoE layer calls, shaped as the reference's GEMM template front
(`gemm.gemm(lhs, rhs, group_sizes, *, paired, gather, scatter, epilogue, out_dtype, compute, ...)`,
src/dew/nn/kernels/gemm.py:84-198), forward semantics only: every call is decided by the `GROUPED`
selector (src/dew/nn/kernels/grouped_matmul.py:2206; selection.py) and runs the gfx950 HIP launch.

A product's law (src/dew/nn/moe.py:675-677; docs/design/kernel-templates.md:876 of the reference): operands
in the compute dtype (bf16), fp32 sums, one rounding; rows past `sum(group_sizes)` are zero; empty groups
are allowed; an NVFP4 bank's deferred factor multiplies the sums before the rounding
(src/dew/nn/kernels/gemm.py:655-662).
"""

import dataclasses

import torch

from . import formats, ops, selection
from .selection import Kernel, Op, Requirement

GROUPED_MATMUL = "grouped_matmul"
"""The selector's choice name (`generation.Choice.GROUPED_MATMUL` in the reference)."""


@dataclasses.dataclass(frozen=True)
class GroupSizes:
    """Group sizes `[E]` with their exclusive prefix `[E + 1]`, both int32 on the device: what the dispatch
    sort produces, so no product recomputes the prefix. A plain int32 sizes tensor is accepted wherever this
    is, at the price of one tiny prefix launch."""

    sizes: torch.Tensor
    offsets: torch.Tensor

    @classmethod
    def of(cls, group_sizes) -> "GroupSizes":
        if isinstance(group_sizes, GroupSizes):
            return group_sizes
        sizes = group_sizes.to(torch.int32).contiguous()
        return cls(sizes, ops.group_offsets(sizes))

    @staticmethod
    def operands(group_sizes) -> dict:
        """The groups as a product's keywords: the prefix where the caller holds it (`GroupSizes`), else the plain
        `group_sizes [E]` as the reference's FFI takes them, the prefix then formed inside the launch."""
        if isinstance(group_sizes, GroupSizes):
            return dict(offsets=group_sizes.offsets)
        return dict(offsets=None, sizes=group_sizes.to(torch.int32).contiguous())


@dataclasses.dataclass(frozen=True)
class GroupedCase:
    """The facts of one grouped call the selector's requirements read."""

    lhs: torch.Tensor
    rhs: object
    paired: object = None
    epilogue: object = None
    out_dtype: torch.dtype = torch.bfloat16
    compute: torch.dtype = torch.bfloat16
    epilogue_operands: tuple = ()


_BANKS = (formats.NvFp4, formats.Fp8Blocks, formats.Fp8Channels, formats.Bf16, formats.Mxfp4Blocks, formats.Layered, ops.PreparedBank)
# (formats.MxFp8 multiplies MXFP8 rows only: projections.mxfp8_product)


def _shape(bank):
    return tuple(bank.shape)


def _is_bank(matrices) -> bool:
    """A bank the kernels multiply: one of the formats, or the reference's plain operand, bf16 `[E, K, N]`."""
    return isinstance(matrices, _BANKS) or (torch.is_tensor(matrices) and matrices.dtype == torch.bfloat16 and matrices.ndim == 3)


def _bias_fits(case, bias) -> bool:
    return bias is None or (torch.is_tensor(bias) and bias.dtype == torch.float32
                            and tuple(bias.shape) == (_shape(case.rhs)[0], _shape(case.rhs)[2]))


def _extent_units(bank) -> tuple[int, int]:
    """(depth, width) granules of a bank: the 64-deep steps and 32-column atoms of an unquantized bank or an MXFP4
    checkpoint's, else the 128 of the block scales and tiles."""
    in_atoms = torch.is_tensor(bank) or (isinstance(bank, formats.Bf16) and not bank.transposed) or isinstance(bank, formats.Mxfp4Blocks) or (
        isinstance(bank, ops.PreparedBank) and bank.descriptor.format in (ops._lib.W_BF16, ops._lib.W_MXFP4, ops._lib.W_NVFP4))
    return (64, 32) if in_atoms else (128, 128)


def _is_clamp(operands) -> bool:
    return not operands or (len(operands) == 1 and (operands[0] is None or float(operands[0]) > 0))


_EPILOGUES = {
    None: lambda c: not c.epilogue_operands,
    # the gated product of a paired launch (`gated_product`, src/dew/nn/activations.py:336-356); one operand, where
    # given, is `swiglu_clamped`'s limit (:327-333), applied to both products before the gate
    "swiglu": lambda c: c.paired is not None and _is_clamp(c.epilogue_operands),
    "geglu": lambda c: c.paired is not None and _is_clamp(c.epilogue_operands),
    # the reference's `_plus_bias` (src/dew/nn/moe.py:729-747): each expert's bias on its rows' fp32 sums
    "plus_bias": lambda c: c.paired is None and len(c.epilogue_operands) == 1 and c.epilogue_operands[0] is not None
                           and _bias_fits(c, c.epilogue_operands[0]),
    # GPT-OSS's interleaved gate/up with its clamped gating (src/dew/nn/gpt_oss.py:111-121)
    "gpt_oss_gated": lambda c: c.paired is None and len(c.epilogue_operands) == 2 and _bias_fits(c, c.epilogue_operands[0])
                               and float(c.epilogue_operands[1]) > 0 and _shape(c.rhs)[2] % (2 * _extent_units(c.rhs)[1]) == 0,
}


HIP = Kernel("hip", (
    Requirement("device", lambda c: c.lhs.is_cuda, "the rows are not on the GPU; the HIP kernels have no CPU path"),
    Requirement("quantized-bank", lambda c: _is_bank(c.rhs) and (c.paired is None or _is_bank(c.paired)),
                lambda c: f"the matrices are {type(c.rhs).__name__}; the kernels multiply NvFp4, Fp8Blocks, Fp8Channels "
                          f"and Bf16 banks", row="matrices of other dtypes"),
    Requirement("bf16", lambda c: c.lhs.dtype == torch.bfloat16 and c.compute == torch.bfloat16 and c.out_dtype == torch.bfloat16,
                lambda c: f"rows {c.lhs.dtype}, compute {c.compute}, out {c.out_dtype}; the kernels compute and write bfloat16",
                row="fp32 outputs"),
    # (unquantized matrices: whole 64-deep steps and 32-column atoms, so GPT-OSS's 2880-wide experts run as they are; the
    # reference's own grouped kernel takes extents in whole 8s, `_Cutlass.in_contract`, src/dew/nn/kernels/grouped_matmul.py:1874-1887)
    Requirement("depth", lambda c: _shape(c.rhs)[1] % _extent_units(c.rhs)[0] == 0 and _shape(c.rhs)[1] >= 128
                                   and c.lhs.shape[-1] == _shape(c.rhs)[1],
                lambda c: f"depth {_shape(c.rhs)[1]} against rows {c.lhs.shape[-1]} deep; depths are whole {_extent_units(c.rhs)[0]}s, 128 at least",
                row="ragged depth"),
    Requirement("width", lambda c: _shape(c.rhs)[2] % _extent_units(c.rhs)[1] == 0 and _shape(c.rhs)[2] >= 128,
                lambda c: f"width {_shape(c.rhs)[2]} is not a multiple of {_extent_units(c.rhs)[1]}, 128 at least", row="ragged width"),
    Requirement("pair", lambda c: c.paired is None or (_shape(c.paired) == _shape(c.rhs) and type(c.paired) is type(c.rhs)),
                "a paired product's matrices share one shape and format"),
    Requirement("epilogue", lambda c: _EPILOGUES.get(c.epilogue, lambda c: False)(c),
                lambda c: f"epilogue {c.epilogue!r} with {len(c.epilogue_operands)} operands"
                          f"{' over a pair' if c.paired is not None else ''}; the kernels fuse 'swiglu' over a pair, "
                          f"'plus_bias' [E, N] on one bank and 'gpt_oss_gated' (bias [E, N] or None, limit) on one "
                          f"interleaved bank", row="other epilogues"),
))

GROUPED = Op(GROUPED_MATMUL, (HIP,), preferred=lambda case: "hip",
             foreign=("xla", "pallas", "mosaic", "triton", "cutlass"))
"""The grouped product's selector. `chosen(grouped_matmul='hip')` names the HIP launch; the reference's other
names are refused as unlowerable."""


SPLIT_ROWS = True
"""Whether an expert MLP of MXFP4 banks with groups of 384 rows or more (`ops.prefers_split`) runs on rows split into two e4m3
terms and the scaled matrix instruction (`swiglu_mlp_on_split_rows`). The products are the same exact ones (an
element loses bits only below 2^-11 of the largest of its 128 neighbours); measured on 16384 tokens of
4096 -> 14336 -> 4096 over 8 experts the two launches take 5.45 + 2.48 ms against 5.75 + 2.54 ms on bf16
operands, the whole step 8.35 against 8.70 ms. False keeps every product on the bf16 instructions."""


SPLIT_SECOND_TERM = "e4m3"
"""How the rows of the expert MLP's first product (two thirds of the MLP's work) are held on the scaled matrix instruction:
'e4m3' (two FP8 terms: every element's bf16 value exactly, within 2^-11 of its row's largest; the default), or one of two
EXPERIMENTAL options that are not exact: 'e2m3' (the second term in FP6 under one power-of-two scale every 32 depths: its
instruction takes half the first term's cycles) and 'e2m3x2' (both terms in FP6, each under its own scale every 32 depths: two
instructions in the time of one FP8-rate instruction). Either option holds an element exactly within two binades of its
32-deep block's largest magnitude and to 2^-10 of that magnitude below. Measured on 16384 tokens of 4096 -> 14336 over 8 experts
in one run: the gate/up launch 5.07 ms ('e4m3'), 4.54 ('e2m3'), 4.32 ('e2m3x2'); against the CPU oracle all three are within
4.3e-3 of the largest output, but 91 % / 56 % / 55.5 % of the outputs are bit-identical to the oracle's and the element-wise figure
is 7.8e-3 / 1.3e-2 / 1.3e-2; on a narrower MLP (512 -> 768) the options' element-wise figure reaches 2.1e-2, past the 2e-2 bar. The
second product (hidden rows, whose blocks span more binades) keeps two e4m3 terms whichever is chosen."""


def prepared(bank) -> ops.PreparedBank:
    """The bank's one-time device re-layout, cached on the bank object."""
    if isinstance(bank, ops.PreparedBank):
        return bank
    if torch.is_tensor(bank):  # the reference's plain operand: re-laid at every call, since a parameter may have changed
        if not bank.is_contiguous() and bank.transpose(1, 2).is_contiguous():
            return ops.prepare(formats.Bf16(bank.transpose(1, 2), transposed=True))  # `w.transpose(1, 2)`: read where it lies
        return ops.prepare(formats.Bf16(bank.contiguous()))
    if isinstance(bank, formats.Layered):  # the layer's matrices where they lie in the stack
        return prepared(bank.stack).layer(int(bank.layer), int(bank.layers))
    held = getattr(bank, "_prepared", None)
    if held is None:
        held = ops.prepare(bank)
        object.__setattr__(bank, "_prepared", held)
    return held


def gemm(lhs: torch.Tensor, rhs, group_sizes, *, paired=None, gather: torch.Tensor | None = None,
         scatter: torch.Tensor | None = None, epilogue: str | None = None, epilogue_operands: tuple = (),
         out_dtype=torch.bfloat16, compute=torch.bfloat16, implementation: str | None = None):
    """Each group's rows of `lhs` (read at `gather` where given) times its matrix of the bank `rhs`, written
    at `scatter` where given. With `paired`, a second bank multiplied by the same rows in the same launch:
    returns both products, or, with `epilogue='swiglu'` (or `'geglu'`; `epilogue_operands = (limit,)` clamps both
    products first), their gated product alone. On one bank,
    `epilogue='plus_bias'` adds `epilogue_operands = (bias [E, N],)` to the fp32 sums before the rounding, and
    `epilogue='gpt_oss_gated'` with `(bias or None, limit)` returns GPT-OSS's gated `[rows, N / 2]`."""
    case = GroupedCase(lhs, rhs, paired, epilogue, out_dtype, compute, tuple(epilogue_operands))
    named = None if implementation in (None, "auto") else implementation
    selection.select(GROUPED, case, named)
    first = prepared(rhs)
    if epilogue == "gpt_oss_gated":
        if scatter is not None:
            raise selection.KernelRefused(GROUPED_MATMUL, "hip", selection.Refusal("gated-scatter", "the gated product writes sorted rows"), iter(()))
        return ops.gateup_interleaved(lhs, first, GroupSizes.of(group_sizes).offsets, bias=epilogue_operands[0],
                                      limit=float(epilogue_operands[1]), gather=gather)
    groups = GroupSizes.operands(group_sizes)    # no prefix launch where the caller holds sizes only
    offsets = groups.pop("offsets")
    if paired is None:
        bias = epilogue_operands[0] if epilogue == "plus_bias" else None   # (`_plus_bias`'s operand: rounded to the compute dtype, in the launch)
        return ops.grouped_gemm(lhs, first, offsets, gather=gather, scatter=scatter, bias=bias, round_bias=True, **groups)
    second = prepared(paired)
    if scatter is not None:
        raise selection.KernelRefused(GROUPED_MATMUL, "hip", selection.Refusal("pair-scatter", "a paired product writes sorted rows"), iter(()))
    if epilogue in ("swiglu", "geglu"):
        limit = epilogue_operands[0] if epilogue_operands else None
        return ops.gateup_swiglu(lhs, first, second, offsets, gather=gather, activation=epilogue, limit=limit, **groups)
    return (ops.grouped_gemm(lhs, first, offsets, gather=gather, **groups),
            ops.grouped_gemm(lhs, second, offsets, gather=gather, **groups))


def gemm_t(lhs: torch.Tensor, rhs: torch.Tensor, group_sizes, *, out_dtype=torch.bfloat16, whole_steps: bool = False) -> torch.Tensor:
    """Each group's rows of `lhs [rows, depth]` transposed times its rows of `rhs [rows, width]`: `[groups, depth,
    width]` in `out_dtype`, an empty group's zero, exact bf16 products summed in fp32 (the reference's `gemm_t`,
    src/dew/nn/kernels/gemm.py:418-431: a grouped product's kernel gradient). Both operands are written transposed
    first (one pass each) so that the contraction runs along contiguous tokens, each group from a whole 64-token step
    on with zeros filling its last step, so the groups are of any sizes and rows past them add nothing. A caller whose
    groups are whole 64-row steps and whose rows whole 128s (a recipe pads them so) says `whole_steps` and saves the
    padding."""
    groups = GroupSizes.of(group_sizes)
    if whole_steps:
        rows_t, _ = ops.transpose_columns(lhs.contiguous(), as_bank=False)
        bank, _ = ops.transpose_columns(rhs.contiguous(), as_bank=True)
        return ops.kernel_gradient_bf16(rows_t, bank, groups.offsets, out_dtype=out_dtype)
    rows_t, padded = ops.transpose_groups(lhs.contiguous(), groups.offsets, as_bank=False)
    bank, _ = ops.transpose_groups(rhs.contiguous(), groups.offsets, as_bank=True)
    return ops.kernel_gradient_bf16(rows_t, bank, padded, out_dtype=out_dtype)


def swiglu_mlp_on_split_rows(lhs: torch.Tensor, gate, up, down, group_sizes, *, gather: torch.Tensor | None = None,
                             scatter: torch.Tensor | None = None, implementation: str | None = None,
                             activation: str = "swiglu", limit: float | None = None):
    """`gemm(gemm(lhs, gate, paired=up, epilogue='swiglu'), down, scatter=scatter)` as two launches on the scaled
    matrix instruction, where that is the faster form, else None (the caller then makes the two `gemm` calls).
    The rows are split into two e4m3 terms under one power-of-two scale a row (`ops.split_rows`); the gate/up
    launch writes its SwiGLU rows already split, one scale per row and 128 columns, and the down launch reads
    them, so no bf16 hidden rows are written at all. The same selector decides the call. `activation` ('swiglu' or
    'geglu') and `limit` (the clamp before the gate) are the gate/up launch's epilogue, as `gemm`'s."""
    if not SPLIT_ROWS or not (torch.is_tensor(lhs) and lhs.is_cuda and lhs.dtype == torch.bfloat16):
        return None
    if any(torch.is_tensor(bank) or isinstance(bank, formats.Bf16) for bank in (gate, up, down)):
        return None  # unquantized matrices have no FP4 codes for the scaled instruction (and a plain tensor is not re-laid to find out)
    named = None if implementation in (None, "auto") else implementation
    selection.select(GROUPED, GroupedCase(lhs, gate, up, activation, epilogue_operands=() if limit is None else (limit,)), named)
    first, second, third = prepared(gate), prepared(up), prepared(down)
    rows = lhs.shape[0] if gather is None else gather.numel()
    if not ops.prefers_split_pair(first, second, third, rows):
        return None
    groups = GroupSizes.operands(group_sizes)   # a caller's plain group sizes go in as they are: the call forms their prefix
    return ops.swiglu_mlp_split(lhs, first, second, third, groups["offsets"], sizes=groups.get("sizes"), gather=gather,
                                scatter=scatter, terms=SPLIT_SECOND_TERM, activation=activation, limit=limit)

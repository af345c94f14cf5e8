"""The kernels as functions of torch tensors: each checks what only the host can (devices, dtypes,
contiguity), allocates its outputs with torch (device memory and streams are torch's here; the arithmetic is
the library's) and calls the C ABI on torch's current stream. No function reads a device value on the host."""

import contextlib
import dataclasses

import torch

from . import _lib, formats
from ._lib import KernelError


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _device(tensor: torch.Tensor, name: str, dtype=None) -> torch.Tensor:
    if not tensor.is_cuda:
        raise KernelError(f"{name} must be on the GPU: the MoE kernels have no CPU path")
    if dtype is not None and tensor.dtype != dtype:
        raise KernelError(f"{name} must be {dtype}, got {tensor.dtype}")
    if not tensor.is_contiguous():
        raise KernelError(f"{name} must be contiguous")
    return tensor


def _ptr(tensor):
    return None if tensor is None else tensor.data_ptr()


def device_check() -> None:
    """Refuse a device the kernels were not built for, by name."""
    _lib.check(_lib.library().dew_moe_device_check(), "dew_moe_device_check")


# ---- router -------------------------------------------------------------------------------------------


WEIGHT_SUM_EPSILON = 1e-20
"""What a renormalization adds to the chosen weights' sum (`WEIGHT_SUM_EPSILON`, src/dew/nn/moe.py:181)."""


def route(logits: torch.Tensor, top_k: int, *, score_function: str = "softmax", normalize_weights: bool = True,
          bias: torch.Tensor | None = None, routed_scaling_factor: float = 1.0, expert_groups: int = 1,
          groups_per_token: int = 1, group_score: str = "top2", sown: bool = False, bias_in_weights: bool = False,
          weight_sum_epsilon: float = WEIGHT_SUM_EPSILON, weight_sum_min: float = 0.0, excluded_group_score: float | None = None,
          logit_softcap: float | None = None, given: torch.Tensor | None = None, covered: torch.Tensor | None = None,
          media: torch.Tensor | None = None, media_bias: torch.Tensor | None = None):
    """(weights fp32 `[..., k]`, indices int32 `[..., k]`) of router `logits [..., E]` (fp32); with `sown`, also what
    the router sows for the balance statistics: (weights, indices, scores fp32 `[..., E]`, log_z fp32 `[...]`). The
    five switches after `sown` are `Router`'s of the same names (src/dew/nn/moe.py:361-384). `given` (int32 `[..., k]`) are
    experts to use in place of the router's own choice (a replayed record, a hash table's rows), for the tokens `covered`
    (bool `[...]`) marks, all of them where it is None; the weights are the router's for those experts. `media` (bool
    `[...]`) marks the tokens whose experts are chosen by `media_bias [E]` in place of `bias`."""
    scores = {"softmax": _lib.SCORE_SOFTMAX, "sigmoid": _lib.SCORE_SIGMOID, "sqrtsoftplus": _lib.SCORE_SQRTSOFTPLUS}
    group_scores = {"top2": _lib.GROUP_TOP2, "max": _lib.GROUP_MAX}
    if score_function not in scores:
        raise KernelError(f"score_function must be one of {list(scores)}, got {score_function!r}")
    if group_score not in group_scores:
        raise KernelError(f"group_score must be one of {list(group_scores)}, got {group_score!r}")
    _device(logits, "logits", torch.float32)
    if bias is not None:
        _device(bias, "bias", torch.float32)
        if bias.shape != logits.shape[-1:]:
            raise KernelError(f"bias {tuple(bias.shape)} does not match {logits.shape[-1]} experts")
    experts = logits.shape[-1]
    tokens = logits.numel() // experts
    if given is not None:
        _device(given, "given", torch.int32)
        if tuple(given.shape) != (*logits.shape[:-1], top_k):
            raise KernelError(f"replayed routing is {tuple(given.shape)} for {tuple(logits.shape[:-1])} tokens choosing {top_k} experts each")
    if covered is not None:
        if given is None:
            raise KernelError("a replay's coverage comes with the experts it covers")
        _device(covered, "covered", torch.bool)
        if covered.shape != logits.shape[:-1]:
            raise KernelError(f"replay coverage is {tuple(covered.shape)} for {tuple(logits.shape[:-1])} tokens")
    if (media is None) != (media_bias is None):
        raise KernelError("the media tokens and the bias that chooses for them come together")
    if media is not None:
        _device(media, "media", torch.bool), _device(media_bias, "media_bias", torch.float32)
        if media.shape != logits.shape[:-1] or media_bias.shape != logits.shape[-1:]:
            raise KernelError(f"media {tuple(media.shape)} marks {tuple(logits.shape[:-1])} tokens and media_bias "
                              f"{tuple(media_bias.shape)} biases {logits.shape[-1]} experts")
    weights = torch.empty((*logits.shape[:-1], top_k), dtype=torch.float32, device=logits.device)
    indices = torch.empty((*logits.shape[:-1], top_k), dtype=torch.int32, device=logits.device)
    activated = torch.empty_like(logits) if sown else None
    log_z = torch.empty(logits.shape[:-1], dtype=torch.float32, device=logits.device) if sown else None
    router = _lib.Router(experts, top_k, scores[score_function], int(bool(normalize_weights)), float(routed_scaling_factor),
                         expert_groups, groups_per_token, group_scores[group_score], int(bool(bias_in_weights)),
                         float(weight_sum_epsilon), float(weight_sum_min), int(excluded_group_score is not None),
                         float(excluded_group_score or 0.0), float(logit_softcap or 0.0))
    _lib.check(_lib.library().dew_moe_route_call(router, _ptr(logits), _ptr(bias), _ptr(media_bias), _ptr(media), _ptr(given), _ptr(covered),
                                                 tokens, _ptr(weights), _ptr(indices), _ptr(activated), _ptr(log_z), _stream()), "dew_moe_route")
    return (weights, indices, activated, log_z) if sown else (weights, indices)


def route_blocks(logits: torch.Tensor, top_k: int, blocks: torch.Tensor, block_experts: int, *, score_function: str = "softmax",
                 normalize_weights: bool = True, bias: torch.Tensor | None = None, routed_scaling_factor: float = 1.0,
                 sown: bool = False, bias_in_weights: bool = False, weight_sum_epsilon: float = WEIGHT_SUM_EPSILON,
                 weight_sum_min: float = 0.0, logit_softcap: float | None = None):
    """`route` under LLaDA2.2's block routing: `logits [rows, length, E]`, `blocks [rows, length]` int32 numbering each
    token's block within its row from 0 (negative: padding); a token chooses among the `block_experts` experts its block
    scores best, a block's score for an expert being its best token's selection (the reference's `Router.block_mask`)."""
    scores = {"softmax": _lib.SCORE_SOFTMAX, "sigmoid": _lib.SCORE_SIGMOID, "sqrtsoftplus": _lib.SCORE_SQRTSOFTPLUS}
    if score_function not in scores:
        raise KernelError(f"score_function must be one of {list(scores)}, got {score_function!r}")
    _device(logits, "logits", torch.float32), _device(blocks, "blocks", torch.int32)
    if logits.dim() != 3 or blocks.shape != logits.shape[:2]:
        raise KernelError(f"block routing takes logits [rows, length, E] and blocks [rows, length], got {tuple(logits.shape)} and {tuple(blocks.shape)}")
    if bias is not None:
        _device(bias, "bias", torch.float32)
        if bias.shape != logits.shape[-1:]:
            raise KernelError(f"bias {tuple(bias.shape)} does not match {logits.shape[-1]} experts")
    rows, length, experts = logits.shape
    weights = torch.empty((rows, length, top_k), dtype=torch.float32, device=logits.device)
    indices = torch.empty((rows, length, top_k), dtype=torch.int32, device=logits.device)
    activated = torch.empty_like(logits) if sown else None
    log_z = torch.empty((rows, length), dtype=torch.float32, device=logits.device) if sown else None
    router = _lib.Router(experts, top_k, scores[score_function], int(bool(normalize_weights)), float(routed_scaling_factor), 1, 1,
                         _lib.GROUP_TOP2, int(bool(bias_in_weights)), float(weight_sum_epsilon), float(weight_sum_min), 0, 0.0,
                         float(logit_softcap or 0.0))
    library = _lib.library()
    workspace = torch.empty(max(library.dew_moe_route_blocks_workspace_bytes(rows, length, experts), 4) // 4 + 1, dtype=torch.int32, device=logits.device)
    _lib.check(library.dew_moe_route_blocks(router, _ptr(logits), _ptr(bias), _ptr(blocks), rows, length, block_experts, _ptr(workspace),
                                            workspace.numel() * 4, _ptr(weights), _ptr(indices), _ptr(activated), _ptr(log_z), _stream()),
               "dew_moe_route_blocks")
    return (weights, indices, activated, log_z) if sown else (weights, indices)


def capacity_admitted(indices: torch.Tensor, num_experts: int, capacity_factor: float) -> torch.Tensor:
    """`indices [..., length, k]` with every slot past its expert's queue in its sequence replaced by the sentinel id
    `num_experts` (the reference's `capacity_positions` and the drop it decides, src/dew/nn/moe.py:832-855, 914-919);
    the capacity is `int(max(ceil(length * k / E) * capacity_factor, capacity_factor))`."""
    import math

    _device(indices, "indices", torch.int32)
    if indices.dim() < 2:
        raise KernelError("capacity dropping takes indices [..., length, top_k]")
    *leading, length, top_k = indices.shape
    capacity = int(max(math.ceil(length * top_k / num_experts) * capacity_factor, capacity_factor))
    admitted = torch.empty_like(indices)
    _lib.check(_lib.library().dew_moe_capacity_admit(_ptr(indices), math.prod(leading), length, top_k, num_experts, capacity,
                                                     _ptr(admitted), _stream()), "dew_moe_capacity_admit")
    return admitted


def balance_bias(bias: torch.Tensor, counts: torch.Tensor, rate: float) -> torch.Tensor:
    """The aux-loss-free balancing step, in place: `bias[e] += rate * direction(counts)[e]` (the reference's
    `load_balance_update`), `counts` the int32 slots each expert took (`sort_by_expert(...).sizes`)."""
    _device(bias, "bias", torch.float32), _device(counts, "counts", torch.int32)
    if bias.shape != counts.shape or bias.dim() != 1:
        raise KernelError(f"bias {tuple(bias.shape)} and counts {tuple(counts.shape)} are one value per expert")
    _lib.check(_lib.library().dew_moe_balance_bias(_ptr(counts), _ptr(bias), float(rate), bias.numel(), _stream()), "dew_moe_balance_bias")
    return bias


def router_logits(x: torch.Tensor, kernel: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
    """fp32 gate logits `[..., E]` of bf16 tokens `[..., D]` and the fp32 gate kernel `[D, E]`, plus the
    router's fp32 `bias [E]` where it has one."""
    _device(x, "x", torch.bfloat16), _device(kernel, "kernel", torch.float32)
    depth, experts = kernel.shape
    if x.shape[-1] != depth:
        raise KernelError(f"tokens are {x.shape[-1]} wide, the gate kernel {depth}")
    if bias is not None:
        _device(bias, "bias", torch.float32)
        if bias.numel() != experts:
            raise KernelError(f"the router bias holds {bias.numel()} values for {experts} experts")
    logits = torch.empty((*x.shape[:-1], experts), dtype=torch.float32, device=x.device)
    _lib.check(_lib.library().dew_moe_router_logits(_ptr(x), _ptr(kernel), _ptr(bias), _ptr(logits), x.numel() // depth, depth,
                                                    experts, _stream()), "dew_moe_router_logits")
    return logits


def group_offsets(sizes: torch.Tensor) -> torch.Tensor:
    """`[0, cumsum(sizes)]` int32 `[E + 1]`."""
    _device(sizes, "group_sizes", torch.int32)
    offsets = torch.empty(sizes.numel() + 1, dtype=torch.int32, device=sizes.device)
    _lib.check(_lib.library().dew_moe_group_offsets(_ptr(sizes), sizes.numel(), _ptr(offsets), _stream()), "dew_moe_group_offsets")
    return offsets


# ---- dispatch -----------------------------------------------------------------------------------------


@dataclasses.dataclass(frozen=True)
class Plan:
    """The sort of routed slots by expert: `order [R]` (slot of each sorted position), `rows [R]` (its
    token), `sizes [E]`, `offsets [E + 1]`, all int32 on the device."""

    order: torch.Tensor
    rows: torch.Tensor
    sizes: torch.Tensor
    offsets: torch.Tensor


def sort_by_expert(indices: torch.Tensor, num_experts: int, shared_rows: int = 0) -> Plan:
    """The stable sort of the routed slots by expert. With `shared_rows` (the tokens, where every token also takes one
    always-on expert) that expert is group `num_experts` of the plan: `shared_rows` more sorted positions behind the
    routed ones, position i of them reading token i and writing row `slots + i`; `sizes` and `offsets` grow by one."""
    _device(indices, "indices", torch.int32)
    top_k = indices.shape[-1]
    tokens = indices.numel() // top_k
    slots = tokens * top_k + shared_rows
    groups = num_experts + (1 if shared_rows else 0)
    device = indices.device
    lib = _lib.library()
    workspace = torch.empty(lib.dew_moe_permute_workspace_bytes(slots, groups), dtype=torch.uint8, device=device)
    sizes = torch.empty(groups, dtype=torch.int32, device=device)
    offsets = torch.empty(groups + 1, dtype=torch.int32, device=device)
    order = torch.empty(slots, dtype=torch.int32, device=device)
    rows = torch.empty(slots, dtype=torch.int32, device=device)
    if shared_rows:
        _lib.check(lib.dew_moe_permute_shared(_ptr(indices), tokens, top_k, num_experts, shared_rows, _ptr(sizes), _ptr(offsets),
                                              _ptr(order), _ptr(rows), _ptr(workspace), workspace.numel(), _stream()),
                   "dew_moe_permute_shared")
    else:
        _lib.check(lib.dew_moe_permute(_ptr(indices), tokens, top_k, num_experts, _ptr(sizes), _ptr(offsets), _ptr(order),
                                       _ptr(rows), _ptr(workspace), workspace.numel(), _stream()), "dew_moe_permute")
    return Plan(order, rows, sizes, offsets)


def sort_by_expert_into(indices: torch.Tensor, num_experts: int, plan: Plan) -> Plan:
    """`sort_by_expert` written into a `Plan` the caller already holds, through `dew_moe_permute_static`: no device
    memory is allocated (the sort's scratch is the library's own array), for steps that run where nothing may
    allocate. Sorts within `dew_moe_permute_static`'s limit only; calls that overlap on one GPU race."""
    _device(indices, "indices", torch.int32)
    top_k = indices.shape[-1]
    tokens = indices.numel() // top_k
    for name, tensor, count in (("sizes", plan.sizes, num_experts), ("offsets", plan.offsets, num_experts + 1),
                                ("order", plan.order, tokens * top_k), ("rows", plan.rows, tokens * top_k)):
        _device(tensor, name, torch.int32)
        if tensor.numel() < count:
            raise KernelError(f"plan.{name} holds {tensor.numel()} values, the sort writes {count}")
    _lib.check(_lib.library().dew_moe_permute_static(_ptr(indices), tokens, top_k, num_experts, _ptr(plan.sizes), _ptr(plan.offsets),
                                                     _ptr(plan.order), _ptr(plan.rows), _stream()), "dew_moe_permute_static")
    return plan


# ---- banks ----------------------------------------------------------------------------------------------


@dataclasses.dataclass(frozen=True)
class PreparedBank:
    """A bank re-laid for the matrix cores (`dew_moe_prepare_bank`); holds the buffers it points into."""

    descriptor: _lib.Bank
    shape: tuple
    keep: tuple
    first: int = 0
    """The bank's first expert within the buffers `keep` holds (a layer of a stack starts inside them)."""

    @property
    def experts(self):
        return self.shape[0]

    def scaled(self, by: torch.Tensor) -> "PreparedBank":
        """The same NVFP4 bank with every expert's tensor scale times `by` (a one-element device tensor): how a
        product of two NVFP4 operands owes both tensor scales to its fp32 sums."""
        held = self.descriptor
        if held.format not in (_lib.W_NVFP4, _lib.W_MXFP4):
            raise KernelError("only an NVFP4 bank carries tensor scales")
        own = self.keep[2].reshape(-1)[self.first:self.first + self.experts]  # a layer's experts within its stack's scales
        scales = (own.to(torch.float32) * by.to(torch.float32)).contiguous()
        view = _lib.Bank(held.format, held.layout, held.experts, held.depth, held.width, held.codes, held.scales, _ptr(scales))
        return PreparedBank(view, self.shape, (self.keep[0], self.keep[1], scales), 0)

    def layer(self, index: int, layers: int) -> "PreparedBank":
        """Layer `index` of a bank that stacks `layers` layers' experts along its expert axis (`[layers * E, K, N]`),
        read where it lies: the same buffers, the descriptor's pointers moved to the layer's first expert (the
        reference's `Layered` read, src/dew/nn/moe.py:595-606 and `gemm._grouped`'s `first`,
        src/dew/nn/kernels/gemm.py:1763-1778), so no layer is copied out of the stack."""
        total, depth, width = self.shape
        if layers < 1 or total % layers or not 0 <= index < layers:
            raise KernelError(f"layer {index} of {layers} in a bank of {total} matrices")
        experts = total // layers
        first = index * experts
        held = self.descriptor
        fp4 = held.format in (_lib.W_NVFP4, _lib.W_MXFP4)
        codes = depth * width // 2 if fp4 else depth * width
        codes = depth * width * 2 if held.format == _lib.W_BF16 else codes
        strides = {_lib.W_FP8_BLOCK: (depth // 128) * (width // 128) * 4, _lib.W_FP8_CHANNEL: width * 4,
                   _lib.W_NVFP4: width * (depth // 16), _lib.W_MXFP4: width * (depth // 16), _lib.W_MXFP8: width * (depth // 32),
                   _lib.W_BF16: 0}
        if held.format not in strides:
            raise KernelError(f"no layer stride is known for a prepared bank of format {held.format}")
        scales = strides[held.format]
        view = _lib.Bank(held.format, held.layout, experts, depth, width, held.codes + first * codes,
                         None if not held.scales else held.scales + first * scales,
                         None if not held.tensor_scale else held.tensor_scale + first * 4)
        return PreparedBank(view, (experts, depth, width), self.keep, self.first + first)


def prepare(bank) -> PreparedBank:
    """The one-time re-layout of a `formats.NvFp4`, `formats.Fp8Blocks` (either way round), `formats.Fp8Channels`,
    `formats.MxFp8`, `formats.Bf16` or `formats.Mxfp4Blocks` bank. An MXFP4 checkpoint's bank that is no one NVFP4
    bank (the reference keeps it dense) raises `KernelError`."""
    if isinstance(bank, PreparedBank):
        return bank
    if isinstance(bank, formats.NvFp4):
        bank.checked()
        fmt, codes, scales, tensor = _lib.W_NVFP4, bank.words, bank.scales, bank.scale
        _device(codes, "NvFp4.words", torch.int32), _device(scales, "NvFp4.scales", torch.uint8)
        _device(tensor, "NvFp4.scale", torch.float32)
    elif isinstance(bank, formats.Fp8Blocks):
        fmt, codes, scales, tensor = _lib.W_FP8_BLOCK, bank.codes, bank.scale_inv, None
        _device(codes, "Fp8Blocks.codes", torch.uint8), _device(scales, "Fp8Blocks.scale_inv", torch.float32)
        blocks = tuple(-(-extent // 128) for extent in ((bank.shape[2], bank.shape[1]) if bank.kmajor else bank.shape[1:]))
        if tuple(scales.shape) != (bank.shape[0], *blocks):
            raise KernelError(f"Fp8Blocks.scale_inv is {tuple(scales.shape)}, the bank's blocks {(bank.shape[0], *blocks)}")
    elif isinstance(bank, formats.Mxfp4Blocks):
        fmt, codes, scales, tensor = _lib.W_MXFP4_BLOCKS, bank.blocks, bank.scales, None
        _device(codes, "Mxfp4Blocks.blocks", torch.uint8), _device(scales, "Mxfp4Blocks.scales", torch.uint8)
    elif isinstance(bank, formats.Fp8Channels):
        fmt, codes, scales, tensor = _lib.W_FP8_CHANNEL, bank.codes, bank.scales, None
        _device(codes, "Fp8Channels.codes", torch.uint8), _device(scales, "Fp8Channels.scales", torch.float32)
    elif isinstance(bank, formats.MxFp8):
        fmt, codes, scales, tensor = _lib.W_MXFP8, bank.codes, bank.scales, None
        _device(codes, "MxFp8.codes", torch.uint8), _device(scales, "MxFp8.scales", torch.uint8)
    elif isinstance(bank, formats.Bf16):
        fmt, codes, scales, tensor = _lib.W_BF16, bank.weights, None, None
        _device(codes, "Bf16.weights", torch.bfloat16)
    else:
        raise KernelError(f"no HIP kernel multiplies a {type(bank).__name__} bank")
    experts, depth, width = bank.shape
    lib = _lib.library()
    kmajor = (isinstance(bank, formats.Bf16) and bank.transposed) or (isinstance(bank, formats.Fp8Blocks) and bank.kmajor)
    layout = _lib.LAYOUT_REFERENCE_KMAJOR if kmajor else _lib.LAYOUT_REFERENCE
    reference = _lib.Bank(fmt, layout, experts, depth, width, _ptr(codes), _ptr(scales), _ptr(tensor))
    buffer = torch.empty(lib.dew_moe_prepared_bytes(fmt, experts, depth, width), dtype=torch.uint8, device=codes.device)
    out = _lib.Bank()
    _lib.check(lib.dew_moe_prepare_bank(reference, _ptr(buffer), out, _stream()), "dew_moe_prepare_bank")
    if isinstance(bank, formats.Mxfp4Blocks):  # its tensor scales were written into the prepared buffer
        at = out.tensor_scale - buffer.data_ptr()
        tensor = buffer[at:at + 4 * experts].view(torch.float32)
    return PreparedBank(out, (experts, depth, width), (buffer, scales, tensor))


# ---- products -----------------------------------------------------------------------------------------


def _expert_bias(bias: torch.Tensor | None, experts: int, width: int) -> torch.Tensor | None:
    """An epilogue bias `[E, N]`: values of the compute dtype (bf16) held in fp32, as the reference's `_biased`."""
    if bias is None:
        return None
    _device(bias, "bias", torch.float32)
    if tuple(bias.shape) != (experts, width):
        raise KernelError(f"the bias is {tuple(bias.shape)}, the bank's outputs ({experts}, {width})")
    return bias


def _product_rows(operand: torch.Tensor, name: str, offsets: torch.Tensor, experts: int, gather, scatter, rows, sizes=None) -> int:
    """What every grouped product's launch trusts and only the host can see, checked before any pointer leaves: the
    row operand on the device and contiguous, `offsets` int32 `[E + 1]` on the device, `gather` / `scatter` int32,
    contiguous, on the device and covering every row, and no more rows asked than the operand (without a gather)
    holds. Returns the rows of the launch."""
    _device(operand, name)
    if offsets is None and sizes is not None:   # the groups as `group_sizes [E]`: the launch forms the prefix itself
        _device(sizes, "group_sizes", torch.int32)
        if sizes.numel() != experts:
            raise KernelError(f"group_sizes has {sizes.numel()} entries, the bank {experts} experts")
    else:
        if offsets is None:
            raise KernelError("a grouped product takes the groups' offsets [E + 1] or their sizes [E]")
        _device(offsets, "offsets", torch.int32)
        if offsets.numel() != experts + 1:
            raise KernelError(f"offsets has {offsets.numel()} entries, the bank {experts} experts")
    for label, index in (("gather", gather), ("scatter", scatter)):
        if index is not None:
            _device(index, label, torch.int32)
    rows = (gather.numel() if gather is not None else operand.shape[0]) if rows is None else int(rows)
    if rows < 0:
        raise KernelError(f"{rows} rows asked")
    if gather is None and rows > operand.shape[0]:
        raise KernelError(f"{rows} rows asked of {name} of {operand.shape[0]}")
    if (gather is not None and gather.numel() < rows) or (scatter is not None and scatter.numel() < rows):
        raise KernelError("gather and scatter must cover every row")
    return rows


def grouped_gemm(x: torch.Tensor, bank: PreparedBank, offsets: torch.Tensor | None, *, gather: torch.Tensor | None = None,
                 scatter: torch.Tensor | None = None, rows: int | None = None,
                 bias: torch.Tensor | None = None, sizes: torch.Tensor | None = None, round_bias: bool = False) -> torch.Tensor:
    """`out[scatter[i]] = x[gather[i]] @ W[expert of sorted position i] (+ bias[expert])`, bf16 `[rows, N]`. The groups
    are `offsets [E + 1]`, or, where that is None, `sizes [E]` (the launch then forms the prefix on the device). The
    bias meets the fp32 sums as it is given, or, with `round_bias` (an expert layer's parameter), rounded to bf16 as the
    launch reads it."""
    _device(x, "x", torch.bfloat16)
    experts, depth, width = bank.shape
    if x.shape[-1] != depth:
        raise KernelError(f"x rows are {x.shape[-1]} deep, the bank {depth}")
    rows = _product_rows(x, "x", offsets, experts, gather, scatter, rows, sizes)
    bias = _expert_bias(bias, experts, width)
    out = torch.empty((rows, width), dtype=torch.bfloat16, device=x.device)
    if round_bias and bias is not None:
        _lib.check(_lib.library().dew_moe_grouped_gemm_param_bias(_ptr(x), _ptr(gather), _ptr(offsets), _ptr(None if offsets is not None else sizes),
                                                                  bank.descriptor, _ptr(bias), _ptr(scatter), _ptr(out), rows, _stream()),
                   "dew_moe_grouped_gemm_param_bias")
        return out
    if offsets is None:
        _lib.check(_lib.library().dew_moe_grouped_gemm_sizes(_ptr(x), _ptr(gather), _ptr(sizes), bank.descriptor, _ptr(bias),
                                                             _ptr(scatter), _ptr(out), rows, _stream()), "dew_moe_grouped_gemm_sizes")
        return out
    _lib.check(_lib.library().dew_moe_grouped_gemm_bias(_ptr(x), _ptr(gather), _ptr(offsets), bank.descriptor, _ptr(bias),
                                                        _ptr(scatter), _ptr(out), rows, _stream()), "dew_moe_grouped_gemm")
    return out


def gateup_interleaved(x: torch.Tensor, gate_up: PreparedBank, offsets: torch.Tensor, *, limit: float = 7.0,
                       bias: torch.Tensor | None = None, gather: torch.Tensor | None = None,
                       rows: int | None = None) -> torch.Tensor:
    """GPT-OSS's fused projection and gating, one launch: `p = x[gather[i]] @ W[e] + bias[e]` with gate in the even
    columns and up in the odd ones, `hidden = (clip(up) + 1) * min(gate, limit) * logistic(1.702 min(gate, limit))`,
    bf16 `[rows, N / 2]`."""
    _device(x, "x", torch.bfloat16)
    experts, depth, width = gate_up.shape
    if x.shape[-1] != depth:
        raise KernelError(f"x rows are {x.shape[-1]} deep, the bank {depth}")
    rows = _product_rows(x, "x", offsets, experts, gather, None, rows)
    bias = _expert_bias(bias, experts, width)
    hidden = torch.empty((rows, width // 2), dtype=torch.bfloat16, device=x.device)
    _lib.check(_lib.library().dew_moe_gateup_interleaved(_ptr(x), _ptr(gather), _ptr(offsets), gate_up.descriptor, _ptr(bias),
                                                         float(limit), _ptr(hidden), rows, _stream()),
               "dew_moe_gateup_interleaved")
    return hidden


def gateup_swiglu(x: torch.Tensor, gate: PreparedBank, up: PreparedBank, offsets: torch.Tensor | None, *,
                  gather: torch.Tensor | None = None, rows: int | None = None, sizes: torch.Tensor | None = None,
                  activation: str = "swiglu", limit: float | None = None) -> torch.Tensor:
    """`hidden[i] = swiglu(x[gather[i]] @ Wg[e], x[gather[i]] @ Wu[e])`, bf16 `[rows, F]`, one launch. The groups are
    `offsets [E + 1]`, or, where that is None, `sizes [E]`. `activation` 'geglu' gates by the tanh GELU instead, and
    `limit` clamps the gate from above and the up projection both ways first (`gated_product`'s arithmetic, as the
    launch's epilogue)."""
    if activation not in GATES:
        raise KernelError(f"the gate's activation is one of {list(GATES)}, got {activation!r}")
    if limit is not None and not limit > 0:
        raise KernelError(f"the clamp limit {limit} must be positive")
    _device(x, "x", torch.bfloat16)
    experts, depth, width = gate.shape
    if x.shape[-1] != depth:
        raise KernelError(f"x rows are {x.shape[-1]} deep, the banks {depth}")
    if up.shape != gate.shape:
        raise KernelError(f"gate {gate.shape} and up {up.shape} differ")
    rows = _product_rows(x, "x", offsets, experts, gather, None, rows, sizes)
    hidden = torch.empty((rows, width), dtype=torch.bfloat16, device=x.device)
    if prefers_f16_rows(gate, up, rows):
        # general NVFP4 banks, groups tall enough to be bound by the matrix cores: the rows as f16 under a scale a row and
        # the f16 matrix instruction, which halves the vector work of decoding the banks; the same bits
        halves, scales = rows_f16(x)
        _lib.check(_lib.library().dew_moe_gateup_gated_f16(_ptr(halves), _ptr(scales), _ptr(gather), _ptr(offsets),
                                                           _ptr(None if offsets is not None else sizes), gate.descriptor, up.descriptor,
                                                           GATES[activation], 0.0 if limit is None else float(limit), _ptr(hidden), rows,
                                                           _stream()), "dew_moe_gateup_gated_f16")
        return hidden
    if activation != "swiglu" or limit is not None:
        _lib.check(_lib.library().dew_moe_gateup_gated(_ptr(x), _ptr(gather), _ptr(offsets), _ptr(None if offsets is not None else sizes),
                                                       gate.descriptor, up.descriptor, GATES[activation], 0.0 if limit is None else float(limit),
                                                       _ptr(hidden), rows, _stream()), "dew_moe_gateup_gated")
        return hidden
    if offsets is None:
        _lib.check(_lib.library().dew_moe_gateup_swiglu_sizes(_ptr(x), _ptr(gather), _ptr(sizes), gate.descriptor, up.descriptor,
                                                              _ptr(hidden), rows, _stream()), "dew_moe_gateup_swiglu_sizes")
        return hidden
    _lib.check(_lib.library().dew_moe_gateup_swiglu(_ptr(x), _ptr(gather), _ptr(offsets), gate.descriptor, up.descriptor,
                                                    _ptr(hidden), rows, _stream()), "dew_moe_gateup_swiglu")
    return hidden


F16_ROWS = True
"""Whether a paired launch on general NVFP4 banks (block scales with mantissas) whose groups average F16_ROWS_FROM rows or
more runs on f16 rows and the f16 matrix instruction (`prefers_f16_rows`). Bit-identical to the bf16-operand launch either
way: every product is the same exact one times a power of two. False keeps the bf16 instruction."""
F16_ROWS_FROM = 64


def prefers_f16_rows(gate: PreparedBank, up: PreparedBank, rows: int) -> bool:
    return (F16_ROWS and gate.descriptor.format == _lib.W_NVFP4 and up.descriptor.format == _lib.W_NVFP4
            and rows >= F16_ROWS_FROM * gate.experts)


def rows_f16(x: torch.Tensor):
    """(`halves [rows, depth]` float16, `scale [rows]` e8m0 bytes): each bf16 row as f16 values times one power of two, chosen
    so that the row's largest magnitude lies in [2^15, 2^16) (`dew_moe_rows_f16`)."""
    _device(x, "x", torch.bfloat16)
    if x.dim() != 2 or x.shape[1] % 64:
        raise KernelError(f"x is {tuple(x.shape)}: rows of whole 64s")
    halves = torch.empty(x.shape, dtype=torch.float16, device=x.device)
    scale = torch.empty((x.shape[0],), dtype=torch.uint8, device=x.device)
    _lib.check(_lib.library().dew_moe_rows_f16(_ptr(x), _ptr(halves), _ptr(scale), x.shape[0], x.shape[1], _stream()), "dew_moe_rows_f16")
    return halves, scale


GATES = {"swiglu": _lib.GATE_SILU, "geglu": _lib.GATE_GELU_TANH}
"""The gated activations the kernels compute (the reference's `gated_product`; its erf form 'geglu_exact' is not one)."""


def gated_product(gate: torch.Tensor, up: torch.Tensor, activation: str = "swiglu", limit: float | None = None) -> torch.Tensor:
    """`bf16(bf16(act(gate)) * up)` for `activation` 'swiglu' (silu) or 'geglu' (the tanh GELU); with `limit`, the gate
    first clamped from above and up both ways by it (the reference's `swiglu_clamped`)."""
    if activation not in GATES:
        raise KernelError(f"the gate's activation is one of {list(GATES)}, got {activation!r}")
    _device(gate, "gate", torch.bfloat16), _device(up, "up", torch.bfloat16)
    if gate.shape != up.shape:
        raise KernelError(f"gate {tuple(gate.shape)} and up {tuple(up.shape)} differ")
    hidden = torch.empty_like(gate)
    _lib.check(_lib.library().dew_moe_gated_product(_ptr(gate), _ptr(up), GATES[activation], 0.0 if limit is None else float(limit),
                                                    _ptr(hidden), gate.numel(), _stream()), "dew_moe_gated_product")
    return hidden


def scale_rows(x: torch.Tensor, gather: torch.Tensor, slots: torch.Tensor, weights: torch.Tensor) -> torch.Tensor:
    """The rows Llama 4's input-scaled experts multiply: sorted position i holds `bf16(x[gather[i]] * bf16(weights.ravel()[slots[i]]))`,
    bf16 `[len(gather), D]` (`gather`, `slots` = the dispatch sort's `rows` and `order`)."""
    _device(x, "x", torch.bfloat16), _device(weights, "weights", torch.float32)
    for name, index in (("gather", gather), ("slots", slots)):
        _device(index, name, torch.int32)
    if x.dim() != 2 or gather.numel() != slots.numel() or slots.numel() > weights.numel():
        raise KernelError(f"{gather.numel()} rows of x {tuple(x.shape)} under {slots.numel()} slots of {weights.numel()} weights")
    out = torch.empty((gather.numel(), x.shape[1]), dtype=torch.bfloat16, device=x.device)
    _lib.check(_lib.library().dew_moe_scale_rows(_ptr(x), _ptr(gather), _ptr(slots), _ptr(weights), _ptr(out), gather.numel(), x.shape[1],
                                                 _stream()), "dew_moe_scale_rows")
    return out


def swiglu(gate: torch.Tensor, up: torch.Tensor, limit: float | None = None) -> torch.Tensor:
    """`gated_product` of 'swiglu'."""
    return gated_product(gate, up, "swiglu", limit)


def silu(x: torch.Tensor) -> torch.Tensor:
    """`bf16(x * logistic(x))`, formed in fp32 and rounded once (the reference's `silu`)."""
    _device(x, "x", torch.bfloat16)
    out = torch.empty_like(x)
    _lib.check(_lib.library().dew_moe_silu(_ptr(x), _ptr(out), x.numel(), _stream()), "dew_moe_silu")
    return out


def gate_rows(x: torch.Tensor, kernel: torch.Tensor, rows: torch.Tensor) -> torch.Tensor:
    """`rows [T, W]` (bf16) with each token's row times its gate, `bf16(logistic(bf16(x[t] . bf16(kernel))))`: the
    reference's `shared_gate` on a shared expert's output under a bf16 compute dtype. `kernel` is the gate's fp32 `[D]`
    (or `[D, 1]`) parameter."""
    _device(x, "x", torch.bfloat16), _device(kernel, "kernel", torch.float32), _device(rows, "rows", torch.bfloat16)
    if x.dim() != 2 or rows.dim() != 2 or rows.shape[0] != x.shape[0] or kernel.numel() != x.shape[1]:
        raise KernelError(f"gate_rows takes x [T, D], a kernel of D values and rows [T, W], got {tuple(x.shape)}, {tuple(kernel.shape)} "
                          f"and {tuple(rows.shape)}")
    out = torch.empty_like(rows)
    _lib.check(_lib.library().dew_moe_gate_rows(_ptr(x), _ptr(kernel), _ptr(rows), _ptr(out), x.shape[0], x.shape[1], rows.shape[1],
                                                _stream()), "dew_moe_gate_rows")
    return out


def gate_rows_add_f32(x: torch.Tensor, kernel: torch.Tensor, shared: torch.Tensor, routed: torch.Tensor) -> torch.Tensor:
    """`routed + shared * logistic(x @ kernel)` in fp32, `[T, W]`: the reference's `shared_gate` where the layer states no
    compute dtype (its gate then runs in the fp32 of its kernel and widens the layer's output). `kernel` is the gate's
    fp32 `[D]` (or `[D, 1]`) parameter; `shared` and `routed` are the bf16 rows of the shared and the routed experts."""
    _device(x, "x", torch.bfloat16), _device(kernel, "kernel", torch.float32)
    _device(shared, "shared", torch.bfloat16), _device(routed, "routed", torch.bfloat16)
    if x.dim() != 2 or shared.dim() != 2 or shared.shape != routed.shape or shared.shape[0] != x.shape[0] or kernel.numel() != x.shape[1]:
        raise KernelError(f"gate_rows_add_f32 takes x [T, D], a kernel of D values and two [T, W] row buffers, got {tuple(x.shape)}, "
                          f"{tuple(kernel.shape)}, {tuple(shared.shape)} and {tuple(routed.shape)}")
    out = torch.empty(shared.shape, dtype=torch.float32, device=x.device)
    _lib.check(_lib.library().dew_moe_gate_rows_add_f32(_ptr(x), _ptr(kernel), _ptr(shared), _ptr(routed), _ptr(out), x.shape[0], x.shape[1],
                                                        shared.shape[1], _stream()), "dew_moe_gate_rows_add_f32")
    return out


def relu2(x: torch.Tensor) -> torch.Tensor:
    """`bf16(max(x, 0)^2)`: the squared ReLU of Nemotron-H's ungated experts (the reference's `relu2`)."""
    _device(x, "x", torch.bfloat16)
    out = torch.empty_like(x)
    _lib.check(_lib.library().dew_moe_relu2(_ptr(x), _ptr(out), x.numel(), _stream()), "dew_moe_relu2")
    return out


def combine(slots: torch.Tensor, weights: torch.Tensor, addend: torch.Tensor | None = None) -> torch.Tensor:
    """`out[t] = bf16(sum_j f32(slots[t, j]) * weights[t, j])` (+ the shared expert's `addend`)."""
    _device(slots, "slots", torch.bfloat16), _device(weights, "weights", torch.float32)
    tokens, top_k, width = slots.shape
    if weights.shape != (tokens, top_k):
        raise KernelError(f"routing {tuple(weights.shape)} does not describe slots {tuple(slots.shape)}")
    if addend is not None:
        _device(addend, "addend", torch.bfloat16)
        if addend.shape != (tokens, width):
            raise KernelError(f"addend {tuple(addend.shape)} is not [{tokens}, {width}]")
    out = torch.empty((tokens, width), dtype=torch.bfloat16, device=slots.device)
    _lib.check(_lib.library().dew_moe_combine(_ptr(slots), _ptr(weights), _ptr(addend), _ptr(out), tokens, top_k, width,
                                              _stream()), "dew_moe_combine")
    return out


def split_rows(x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """bf16 rows `[rows, depth]` as two e4m3 terms per element: (`split` uint8 `[rows, depth * 2]`, each 64 depths as
    four 32-byte pieces in the scaled matrix instruction's operand order; `scale` uint8 `[rows]`, e8m0) with
    `x = 2^(scale - 127) * (hi + lo / 16)`."""
    _device(x, "x", torch.bfloat16)
    rows, depth = x.shape
    split = torch.empty((rows, depth * 2), dtype=torch.uint8, device=x.device)
    scale = torch.empty((rows,), dtype=torch.uint8, device=x.device)
    _lib.check(_lib.library().dew_moe_split_rows(_ptr(x), _ptr(split), _ptr(scale), rows, depth, _stream()), "dew_moe_split_rows")
    return split, scale


def split_rows_fp6(x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """`split_rows` with the second term in FP6 (e2m3) under one power-of-two scale every 32 depths, which lies with
    the codes: the same shapes, for `gateup_swiglu_split_out(..., fp6=True)`. The FP6 term's instruction takes half the
    first term's cycles; an element more than two binades below its 32-deep block's largest is then held to within 2^-10
    of that largest magnitude, not exactly."""
    _device(x, "x", torch.bfloat16)
    rows, depth = x.shape
    split = torch.empty((rows, depth * 2), dtype=torch.uint8, device=x.device)
    scale = torch.empty((rows,), dtype=torch.uint8, device=x.device)
    _lib.check(_lib.library().dew_moe_split_rows_fp6(_ptr(x), _ptr(split), _ptr(scale), rows, depth, _stream()), "dew_moe_split_rows_fp6")
    return split, scale


def split_rows_e2m3_pair(x: torch.Tensor) -> tuple[torch.Tensor, None]:
    """`split_rows` with both terms in FP6 (e2m3), each under one power-of-two scale every 32 depths that lies with its
    codes: (`split` uint8 `[rows, depth * 2]`, None: there is no scale a row), for `gateup_swiglu_split_out(..., terms=
    'e2m3x2')`. The two instructions of a product take the time of one FP8-rate instruction; the rows are held as exactly
    as `split_rows_fp6` holds them (exactly within two binades of a 32-deep block's largest magnitude, to 2^-10 of it below)."""
    _device(x, "x", torch.bfloat16)
    rows, depth = x.shape
    split = torch.empty((rows, depth * 2), dtype=torch.uint8, device=x.device)
    _lib.check(_lib.library().dew_moe_split_rows_e2m3_pair(_ptr(x), _ptr(split), rows, depth, _stream()), "dew_moe_split_rows_e2m3_pair")
    return split, None


SPLIT_TERMS = {"e4m3": _lib.SECOND_TERM_E4M3, "e2m3": _lib.SECOND_TERM_E2M3, "e2m3x2": _lib.TERMS_E2M3_PAIR}
"""How split rows are held: two e4m3 terms (exact; the default), an e4m3 and an e2m3 term, or two e2m3 terms."""


def split_rows_as(x: torch.Tensor, terms: str = "e4m3"):
    """`x` split as `terms` names (SPLIT_TERMS): the (split, scale) pair `gateup_swiglu_split_out(..., terms=terms)` reads."""
    if terms not in SPLIT_TERMS:
        raise KernelError(f"split rows are held as one of {list(SPLIT_TERMS)}, got {terms!r}")
    return {"e4m3": split_rows, "e2m3": split_rows_fp6, "e2m3x2": split_rows_e2m3_pair}[terms](x)


@contextlib.contextmanager
def tile_rows(rows: int):
    """Within the block every grouped product uses block tiles of `rows` rows (32, 64, 128, 256) instead of the
    per-launch choice: for tuning, and for tests that must reach one tile's code whatever the problem's size."""
    _lib.check(_lib.library().dew_moe_tile_rows(rows), "dew_moe_tile_rows")
    try:
        yield
    finally:
        _lib.check(_lib.library().dew_moe_tile_rows(0), "dew_moe_tile_rows")


def prefers_split(bank: PreparedBank, rows: int) -> bool:
    """Whether a product of `rows` rows through `bank` is better run on split rows (`split_rows` then the `_split`
    launches): an MXFP4 bank of whole 256-column strips whose groups average 384 rows or more. (Measured on ragged
    groups of 4096 x 14336 x 4096 MLPs against the bf16 launches with their own best tiles: 1.20 times faster at 900
    rows a group, 1.05 at 512 to 768, 1.08 at 384, 0.975 at 256, where the 256-row tiles are half empty.)"""
    experts, depth, width = bank.shape
    return bank.descriptor.format == _lib.W_MXFP4 and depth % 128 == 0 and width % 256 == 0 and rows // experts >= SPLIT_ROWS_FROM


SPLIT_ROWS_FROM = 384
"""The average rows a group from which `prefers_split` takes the split-row launches."""


MAX_BLOCK_SCALE_DEPTH = 24576
"""`grouped_gemm_split_blocks` keeps a tile's rows' block scales in the LDS: 256 rows of 192 bytes at most."""


def prefers_split_pair(gate: PreparedBank, up: PreparedBank, down: PreparedBank, rows: int) -> bool:
    """Whether a SwiGLU expert MLP of `rows` rows is better run as `gateup_swiglu_split_out` then
    `grouped_gemm_split_blocks`: all three banks as `prefers_split` wants them, the down bank's depth the gate's width
    and within the LDS's room for its scales. The library's own rule (`dew_moe_prefers_split_rows`), so that a caller
    through the C ABI alone decides the same way."""
    return bool(_lib.library().dew_moe_prefers_split_rows(gate.descriptor, up.descriptor, down.descriptor, rows))


def swiglu_mlp_split(x: torch.Tensor, gate: PreparedBank, up: PreparedBank, down: PreparedBank, offsets: torch.Tensor | None, *,
                     sizes: torch.Tensor | None = None, gather: torch.Tensor | None = None, scatter: torch.Tensor | None = None,
                     rows: int | None = None, fp6: bool = False, activation: str = "swiglu", limit: float | None = None,
                     terms: str | None = None) -> torch.Tensor:
    """The gated expert MLP on split rows as one call (`dew_moe_gated_mlp_split`): `split_rows`, `gateup_swiglu_split_out`
    and `grouped_gemm_split_blocks` with their intermediates in one workspace. The groups as `offsets` or as `sizes`;
    `activation` and `limit` as `gateup_swiglu` takes them; `terms` (SPLIT_TERMS; `fp6=True` is 'e2m3') how x is split."""
    terms = ("e2m3" if fp6 else "e4m3") if terms is None else terms
    if terms not in SPLIT_TERMS:
        raise KernelError(f"split rows are held as one of {list(SPLIT_TERMS)}, got {terms!r}")
    if activation not in GATES:
        raise KernelError(f"the gate's activation is one of {list(GATES)}, got {activation!r}")
    if limit is not None and not limit > 0:
        raise KernelError(f"the clamp limit {limit} must be positive")
    _device(x, "x", torch.bfloat16)
    experts, depth, width = gate.shape
    if x.dim() != 2 or x.shape[1] != depth:
        raise KernelError(f"x {tuple(x.shape)} does not match the gate bank's depth {depth}")
    rows = _product_rows(x, "x", offsets, experts, gather, scatter, rows, sizes)
    tokens = x.shape[0]
    lib = _lib.library()
    workspace = torch.empty(lib.dew_moe_swiglu_mlp_split_workspace_bytes(tokens, rows, depth, width, experts), dtype=torch.uint8, device=x.device)
    out = torch.empty((rows, down.shape[2]), dtype=torch.bfloat16, device=x.device)
    _lib.check(lib.dew_moe_gated_mlp_split(_ptr(x), tokens, _ptr(gather), _ptr(offsets), _ptr(None if offsets is not None else sizes),
                                           gate.descriptor, up.descriptor, down.descriptor, GATES[activation],
                                           0.0 if limit is None else float(limit), _ptr(scatter), _ptr(out), rows,
                                           SPLIT_TERMS[terms], _ptr(workspace), workspace.numel(),
                                           _stream()), "dew_moe_gated_mlp_split")
    return out


def grouped_gemm_split(split: torch.Tensor, scale: torch.Tensor, bank: PreparedBank, offsets: torch.Tensor, *,
                       gather: torch.Tensor | None = None, scatter: torch.Tensor | None = None, rows: int | None = None,
                       bias: torch.Tensor | None = None) -> torch.Tensor:
    """`grouped_gemm` on rows already split into two e4m3 terms (`split_rows`), for an MXFP4 bank."""
    experts, depth, width = bank.shape
    if split.dtype != torch.uint8 or split.shape[-1] != 2 * depth or scale.dtype != torch.uint8 or scale.numel() != split.shape[0]:
        raise KernelError(f"split rows are uint8 [rows, {2 * depth}] with one uint8 scale a row")
    _device(scale, "scale", torch.uint8)
    rows = _product_rows(split, "split", offsets, experts, gather, scatter, rows)
    bias = _expert_bias(bias, experts, width)
    out = torch.empty((rows, width), dtype=torch.bfloat16, device=split.device)
    _lib.check(_lib.library().dew_moe_grouped_gemm_split(_ptr(split), _ptr(scale), _ptr(gather), _ptr(offsets), bank.descriptor,
                                                         _ptr(bias), _ptr(scatter), _ptr(out), rows, _stream()),
               "dew_moe_grouped_gemm_split")
    return out


def gateup_swiglu_split(split: torch.Tensor, scale: torch.Tensor, gate: PreparedBank, up: PreparedBank, offsets: torch.Tensor, *,
                        gather: torch.Tensor | None = None, rows: int | None = None) -> torch.Tensor:
    """`gateup_swiglu` on rows already split into two e4m3 terms (`split_rows`), for MXFP4 banks."""
    experts, depth, width = gate.shape
    if split.dtype != torch.uint8 or split.shape[-1] != 2 * depth or scale.dtype != torch.uint8 or scale.numel() != split.shape[0]:
        raise KernelError(f"split rows are uint8 [rows, {2 * depth}] with one uint8 scale a row")
    _device(scale, "scale", torch.uint8)
    if up.shape != gate.shape:
        raise KernelError(f"gate {gate.shape} and up {up.shape} differ")
    rows = _product_rows(split, "split", offsets, experts, gather, None, rows)
    hidden = torch.empty((rows, width), dtype=torch.bfloat16, device=split.device)
    _lib.check(_lib.library().dew_moe_gateup_swiglu_split(_ptr(split), _ptr(scale), _ptr(gather), _ptr(offsets), gate.descriptor,
                                                          up.descriptor, _ptr(hidden), rows, _stream()),
               "dew_moe_gateup_swiglu_split")
    return hidden


def block_scale_pitch(elements: int) -> int:
    """Bytes of one row's block scales: one for 128 elements, padded to whole 16-byte loads."""
    return (elements // 128 + 15) // 16 * 16


def gateup_swiglu_split_out(split: torch.Tensor, scale: torch.Tensor, gate: PreparedBank, up: PreparedBank,
                            offsets: torch.Tensor, *, gather: torch.Tensor | None = None,
                            rows: int | None = None, fp6: bool = False, terms: str | None = None) -> tuple[torch.Tensor, torch.Tensor]:
    """`gateup_swiglu_split` whose hidden rows leave already split: (`hidden_split` uint8 `[rows, F * 2]`,
    `hidden_scales` uint8 `[rows, block_scale_pitch(F)]`), one scale per row and 128 columns (byte b of a row scales its
    columns 128 b .. 128 b + 127; the pad bytes are not written), for `grouped_gemm_split_blocks`. `terms` (SPLIT_TERMS;
    `fp6=True` is 'e2m3'): how the rows were split (`split_rows_as`); two e2m3 terms come without a scale a row."""
    terms = ("e2m3" if fp6 else "e4m3") if terms is None else terms
    if terms not in SPLIT_TERMS:
        raise KernelError(f"split rows are held as one of {list(SPLIT_TERMS)}, got {terms!r}")
    experts, depth, width = gate.shape
    if split.dtype != torch.uint8 or split.shape[-1] != 2 * depth:
        raise KernelError(f"split rows are uint8 [rows, {2 * depth}]")
    if terms != "e2m3x2":
        if scale is None or scale.dtype != torch.uint8 or scale.numel() != split.shape[0]:
            raise KernelError("split rows of an e4m3 first term come with one uint8 scale a row")
        _device(scale, "scale", torch.uint8)
    if up.shape != gate.shape:
        raise KernelError(f"gate {gate.shape} and up {up.shape} differ")
    rows = _product_rows(split, "split", offsets, experts, gather, None, rows)
    hidden = torch.empty((rows, width * 2), dtype=torch.uint8, device=split.device)
    scales = torch.empty((rows, block_scale_pitch(width)), dtype=torch.uint8, device=split.device)
    if terms == "e2m3x2":
        _lib.check(_lib.library().dew_moe_gateup_swiglu_split_e2m3_pair_out(_ptr(split), _ptr(gather), _ptr(offsets), gate.descriptor, up.descriptor,
                                                                            _ptr(hidden), _ptr(scales), rows, _stream()),
                   "dew_moe_gateup_swiglu_split_e2m3_pair_out")
        return hidden, scales
    name = "dew_moe_gateup_swiglu_split_fp6_out" if terms == "e2m3" else "dew_moe_gateup_swiglu_split_out"
    _lib.check(getattr(_lib.library(), name)(_ptr(split), _ptr(scale), _ptr(gather), _ptr(offsets), gate.descriptor, up.descriptor, _ptr(hidden),
                                             _ptr(scales), rows, _stream()), name)
    return hidden, scales


def grouped_gemm_split_blocks(split: torch.Tensor, scales: torch.Tensor, bank: PreparedBank, offsets: torch.Tensor, *,
                              gather: torch.Tensor | None = None, scatter: torch.Tensor | None = None, rows: int | None = None,
                              bias: torch.Tensor | None = None) -> torch.Tensor:
    """`grouped_gemm` on rows split with one scale per row and 128 depths (`gateup_swiglu_split_out`'s), MXFP4 bank."""
    experts, depth, width = bank.shape
    if split.dtype != torch.uint8 or split.shape[-1] != 2 * depth or scales.dtype != torch.uint8 or \
            tuple(scales.shape) != (split.shape[0], block_scale_pitch(depth)) or not scales.is_contiguous():
        raise KernelError(f"split rows are uint8 [rows, {2 * depth}] with uint8 scales [rows, {block_scale_pitch(depth)}]")
    _device(scales, "scales", torch.uint8)
    rows = _product_rows(split, "split", offsets, experts, gather, scatter, rows)
    bias = _expert_bias(bias, experts, width)
    out = torch.empty((rows, width), dtype=torch.bfloat16, device=split.device)
    _lib.check(_lib.library().dew_moe_grouped_gemm_split_blocks(_ptr(split), _ptr(scales), _ptr(gather), _ptr(offsets),
                                                                bank.descriptor, _ptr(bias), _ptr(scatter), _ptr(out), rows, _stream()),
               "dew_moe_grouped_gemm_split_blocks")
    return out


def quantize_rows_fp8(x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """bf16 rows `[rows, K]` as the blockwise FP8 recipe quantizes them (1 x 128 tiles, power-of-two scales):
    (`codes` uint8 `[rows, K]`, each 128 depths in the scaled matrix instruction's operand order; `scales` uint8
    `[rows, block_scale_pitch(K)]`, the scales' e8m0 bytes)."""
    _device(x, "x", torch.bfloat16)
    rows, depth = x.shape
    codes = torch.empty((rows, depth), dtype=torch.uint8, device=x.device)
    scales = torch.empty((rows, block_scale_pitch(depth)), dtype=torch.uint8, device=x.device)
    _lib.check(_lib.library().dew_moe_quantize_rows_fp8(_ptr(x), _ptr(codes), _ptr(scales), rows, depth, _stream()),
               "dew_moe_quantize_rows_fp8")
    return codes, scales


def quantize_rows_nvfp4(x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """bf16 rows `[rows, K]` quantized to NVFP4 along the depth (E2M1 under an E4M3 scale every 16 depths and one tensor
    scale): (`values` bf16 `[rows, K]`, each what its code times its block's scale stands for, exactly; `scale` fp32
    `[1]`, the tensor scale the product owes)."""
    _device(x, "x", torch.bfloat16)
    rows, depth = x.shape
    values = torch.empty_like(x)
    scale = torch.empty(1, dtype=torch.float32, device=x.device)
    workspace = torch.empty(1, dtype=torch.int32, device=x.device)
    _lib.check(_lib.library().dew_moe_quantize_rows_nvfp4(_ptr(x), _ptr(values), _ptr(scale), _ptr(workspace), rows, depth, _stream()),
               "dew_moe_quantize_rows_nvfp4")
    return values, scale


def quantize_rows_mxfp8(x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """bf16 rows `[rows, K]` as MXFP8 (OCP MX: one E8M0 scale every 32 depths): (`codes` uint8 `[rows, K]`, each 128
    depths in the scaled matrix instruction's operand order; `scales` uint8 `[rows, K / 32]` in depth order)."""
    _device(x, "x", torch.bfloat16)
    rows, depth = x.shape
    codes = torch.empty((rows, depth), dtype=torch.uint8, device=x.device)
    scales = torch.empty((rows, depth // 32), dtype=torch.uint8, device=x.device)
    _lib.check(_lib.library().dew_moe_quantize_rows_mxfp8(_ptr(x), _ptr(codes), _ptr(scales), rows, depth, _stream()),
               "dew_moe_quantize_rows_mxfp8")
    return codes, scales


def grouped_gemm_mxfp8_rows(codes: torch.Tensor, scales: torch.Tensor, bank: PreparedBank, offsets: torch.Tensor, *,
                            gather: torch.Tensor | None = None, scatter: torch.Tensor | None = None, rows: int | None = None,
                            bias: torch.Tensor | None = None) -> torch.Tensor:
    """The MXFP8 recipe's product: `quantize_rows_mxfp8`'s rows times a prepared `formats.MxFp8` bank, every product of
    (code x scale) values exact, fp32 sums, one rounding to bf16 `[rows, N]`."""
    experts, depth, width = bank.shape
    if codes.dtype != torch.uint8 or codes.shape[-1] != depth or scales.dtype != torch.uint8 or \
            tuple(scales.shape) != (codes.shape[0], depth // 32) or not scales.is_contiguous():
        raise KernelError(f"MXFP8 rows are uint8 [rows, {depth}] with uint8 scales [rows, {depth // 32}]")
    if bank.descriptor.format != _lib.W_MXFP8:
        raise KernelError("MXFP8 rows multiply an MXFP8 bank")
    _device(scales, "scales", torch.uint8)
    rows = _product_rows(codes, "codes", offsets, experts, gather, scatter, rows)
    bias = _expert_bias(bias, experts, width)
    out = torch.empty((rows, width), dtype=torch.bfloat16, device=codes.device)
    _lib.check(_lib.library().dew_moe_grouped_gemm_mxfp8_rows(_ptr(codes), _ptr(scales), _ptr(gather), _ptr(offsets), bank.descriptor,
                                                              _ptr(bias), _ptr(scatter), _ptr(out), rows, _stream()),
               "dew_moe_grouped_gemm_mxfp8_rows")
    return out


def quantize_columns(x: torch.Tensor, *, mx: bool, as_bank: bool):
    """bf16 `[tokens, dim]` quantized along the tokens and written transposed, a kernel gradient's operand
    (`dew_moe_quantize_columns_fp8` for the blockwise FP8 recipe's 1 x 128 tiles, `_mxfp8` for MX blocks of 32 tokens).
    The lhs_t operand (`as_bank` false): (`codes` uint8 `[dim, tokens]`, each 128 tokens in the row operand's order;
    `scales` uint8 `[dim, tokens / 32]`). The rhs_t operand (`as_bank`): a `PreparedBank` of one MXFP8 matrix, depth
    the tokens, width `dim`."""
    _device(x, "x", torch.bfloat16)
    tokens, dim = x.shape
    call = _lib.library().dew_moe_quantize_columns_mxfp8 if mx else _lib.library().dew_moe_quantize_columns_fp8
    name = "dew_moe_quantize_columns_mxfp8" if mx else "dew_moe_quantize_columns_fp8"
    if as_bank:
        buffer = torch.empty(max(tokens * dim + tokens // 32 * dim, 16), dtype=torch.uint8, device=x.device)
        codes, scales = buffer[:tokens * dim], buffer[tokens * dim:tokens * dim + tokens // 32 * dim]
    else:
        codes = torch.empty((dim, tokens), dtype=torch.uint8, device=x.device)
        scales = torch.empty((dim, tokens // 32), dtype=torch.uint8, device=x.device)
    _lib.check(call(_ptr(x), _ptr(codes), _ptr(scales), tokens, dim, int(as_bank), _stream()), name)
    if not as_bank:
        return codes, scales
    view = _lib.Bank(_lib.W_MXFP8, _lib.LAYOUT_PREPARED, 1, tokens, dim, _ptr(codes), _ptr(scales), None)
    return PreparedBank(view, (1, tokens, dim), (buffer,))


def kernel_gradient_mxfp8(codes: torch.Tensor, scales: torch.Tensor, rhs_t: PreparedBank, offsets: torch.Tensor, *,
                          out_dtype=torch.bfloat16) -> torch.Tensor:
    """Each group's tokens contracted: `out[g] = lhs_t[:, tokens of g] @ rhs_t[:, tokens of g]^T`, `[groups, depth,
    width]` in bf16 or fp32, from `quantize_columns`' operands (`codes [depth, tokens]`, `scales [depth, tokens / 32]`,
    the bank `[width, tokens]`); `offsets` int32 `[groups + 1]` in whole 128-token blocks; an empty group's is zero."""
    _, tokens, width = rhs_t.shape
    depth = codes.shape[0]
    if codes.dtype != torch.uint8 or tuple(codes.shape) != (depth, tokens) or scales.dtype != torch.uint8 or \
            tuple(scales.shape) != (depth, tokens // 32) or not codes.is_contiguous() or not scales.is_contiguous():
        raise KernelError(f"the lhs_t operand is uint8 [depth, {tokens}] with uint8 scales [depth, {tokens // 32}]")
    if out_dtype not in (torch.bfloat16, torch.float32):
        raise KernelError(f"a kernel gradient is written in bfloat16 or float32, not {out_dtype}")
    _device(offsets, "offsets", torch.int32)
    groups = offsets.numel() - 1
    out = torch.empty((groups, depth, width), dtype=out_dtype, device=codes.device)
    _lib.check(_lib.library().dew_moe_kernel_gradient_mxfp8(_ptr(codes), _ptr(scales), rhs_t.descriptor, _ptr(offsets), _ptr(out),
                                                            int(out_dtype == torch.float32), depth, groups, _stream()),
               "dew_moe_kernel_gradient_mxfp8")
    return out


def transpose_columns(x: torch.Tensor, *, nvfp4: bool = False, as_bank: bool):
    """bf16 `[tokens, dim]` written transposed, a bf16 kernel gradient's operand (`dew_moe_transpose_columns`), or, `nvfp4`,
    its NVFP4 values along the tokens short of the tensor scale (`dew_moe_quantize_columns_nvfp4`). The lhs_t operand
    (`as_bank` false) is bf16 `[dim, tokens]`; the rhs_t operand a `PreparedBank` of one bf16 matrix, depth the tokens,
    width `dim`. Returns (operand, tensor scale f32 `[1]` or None)."""
    _device(x, "x", torch.bfloat16)
    tokens, dim = x.shape
    out = torch.empty((dim, tokens) if not as_bank else (max(tokens * dim, 8),), dtype=torch.bfloat16, device=x.device)
    scale = None
    if nvfp4:
        scale = torch.empty(1, dtype=torch.float32, device=x.device)
        workspace = torch.empty(1, dtype=torch.int32, device=x.device)
        _lib.check(_lib.library().dew_moe_quantize_columns_nvfp4(_ptr(x), _ptr(out), _ptr(scale), _ptr(workspace), tokens, dim,
                                                                 int(as_bank), _stream()), "dew_moe_quantize_columns_nvfp4")
    else:
        _lib.check(_lib.library().dew_moe_transpose_columns(_ptr(x), _ptr(out), tokens, dim, int(as_bank), _stream()),
                   "dew_moe_transpose_columns")
    if not as_bank:
        return out, scale
    view = _lib.Bank(_lib.W_BF16, _lib.LAYOUT_PREPARED, 1, tokens, dim, _ptr(out), None, None)
    return PreparedBank(view, (1, tokens, dim), (out,)), scale


def transpose_groups(x: torch.Tensor, offsets: torch.Tensor, *, as_bank: bool):
    """`transpose_columns` for ragged groups (`dew_moe_transpose_groups`): each group of `x [rows, dim]`'s rows is written
    from a whole 64-token step on, zeros filling its last step. Returns (operand over the padded tokens, the groups'
    padded offsets int32 `[groups + 1]`, which are `kernel_gradient_bf16`'s)."""
    _device(x, "x", torch.bfloat16), _device(offsets, "offsets", torch.int32)
    rows, dim = x.shape
    groups = offsets.numel() - 1
    tokens = (rows + 64 * groups + 127) // 128 * 128
    out = torch.empty((dim, tokens) if not as_bank else (tokens * dim,), dtype=torch.bfloat16, device=x.device)
    padded = torch.empty(groups + 1, dtype=torch.int32, device=x.device)
    _lib.check(_lib.library().dew_moe_transpose_groups(_ptr(x), _ptr(offsets), _ptr(out), _ptr(padded), rows, tokens, dim, groups,
                                                       int(as_bank), _stream()), "dew_moe_transpose_groups")
    if not as_bank:
        return out, padded
    view = _lib.Bank(_lib.W_BF16, _lib.LAYOUT_PREPARED, 1, tokens, dim, _ptr(out), None, None)
    return PreparedBank(view, (1, tokens, dim), (out,)), padded


def kernel_gradient_bf16(lhs_t: torch.Tensor, rhs_t: PreparedBank, offsets: torch.Tensor, *, lhs_scale: torch.Tensor | None = None,
                         rhs_scale: torch.Tensor | None = None, out_dtype=torch.bfloat16) -> torch.Tensor:
    """Each group's tokens contracted over bf16 operands: `out[g] = lhs_t[:, tokens of g] @ rhs_t[:, tokens of g]^T` times
    the two scales, `[groups, depth, width]` in bf16 or fp32; `lhs_t [depth, tokens]` bf16 and the bank `[width, tokens]`
    from `transpose_columns`; `offsets` int32 `[groups + 1]` in whole 64-token steps; an empty group's is zero."""
    _, tokens, width = rhs_t.shape
    _device(lhs_t, "lhs_t", torch.bfloat16), _device(offsets, "offsets", torch.int32)
    depth = lhs_t.shape[0]
    if tuple(lhs_t.shape) != (depth, tokens) or rhs_t.descriptor.format != _lib.W_BF16:
        raise KernelError(f"the lhs_t operand is bfloat16 [depth, {tokens}] and the rhs_t a bf16 bank")
    if out_dtype not in (torch.bfloat16, torch.float32):
        raise KernelError(f"a kernel gradient is written in bfloat16 or float32, not {out_dtype}")
    for name, scale in (("lhs_scale", lhs_scale), ("rhs_scale", rhs_scale)):
        if scale is not None:
            _device(scale, name, torch.float32)
    groups = offsets.numel() - 1
    out = torch.empty((groups, depth, width), dtype=out_dtype, device=lhs_t.device)
    _lib.check(_lib.library().dew_moe_kernel_gradient_bf16(_ptr(lhs_t), rhs_t.descriptor, _ptr(offsets), _ptr(lhs_scale), _ptr(rhs_scale),
                                                           _ptr(out), int(out_dtype == torch.float32), depth, groups, _stream()),
               "dew_moe_kernel_gradient_bf16")
    return out


def operand_order_fp8(codes: torch.Tensor) -> torch.Tensor:
    """e4m3 codes `[rows, K]` in depth order -> the order `quantize_rows_fp8` writes and `grouped_gemm_fp8_rows`
    reads: of each 128 depths, byte 16 (4 g + 2 t + h) + b holds depth 64 t + 32 h + 16 g + b."""
    rows, depth = codes.shape
    return codes.view(rows, depth // 128, 2, 2, 2, 16).permute(0, 1, 4, 2, 3, 5).contiguous().view(rows, depth)


def depth_order_fp8(codes: torch.Tensor) -> torch.Tensor:
    """The inverse of `operand_order_fp8`."""
    rows, depth = codes.shape
    return codes.view(rows, depth // 128, 2, 2, 2, 16).permute(0, 1, 3, 4, 2, 5).contiguous().view(rows, depth)


def grouped_gemm_fp8_rows(codes: torch.Tensor, scales: torch.Tensor, bank: PreparedBank, offsets: torch.Tensor, *,
                          gather: torch.Tensor | None = None, scatter: torch.Tensor | None = None, rows: int | None = None,
                          bias: torch.Tensor | None = None) -> torch.Tensor:
    """The blockwise FP8 recipe's product: `quantize_rows_fp8`'s rows times an FP8 128 x 128 block bank whose scales
    are powers of two, each 128-deep block's exact partial under its row's and its block's scale, fp32 sums, one
    rounding to bf16 `[rows, N]`."""
    experts, depth, width = bank.shape
    if codes.dtype != torch.uint8 or codes.shape[-1] != depth or scales.dtype != torch.uint8 or \
            tuple(scales.shape) != (codes.shape[0], block_scale_pitch(depth)) or not scales.is_contiguous():
        raise KernelError(f"quantized rows are uint8 [rows, {depth}] with uint8 scales [rows, {block_scale_pitch(depth)}]")
    if bank.descriptor.format != _lib.W_FP8_BLOCK:
        raise KernelError("quantized rows multiply an FP8 128 x 128 block bank")
    _device(scales, "scales", torch.uint8)
    rows = _product_rows(codes, "codes", offsets, experts, gather, scatter, rows)
    bias = _expert_bias(bias, experts, width)
    out = torch.empty((rows, width), dtype=torch.bfloat16, device=codes.device)
    _lib.check(_lib.library().dew_moe_grouped_gemm_fp8_rows(_ptr(codes), _ptr(scales), _ptr(gather), _ptr(offsets), bank.descriptor,
                                                            _ptr(bias), _ptr(scatter), _ptr(out), rows, _stream()),
               "dew_moe_grouped_gemm_fp8_rows")
    return out

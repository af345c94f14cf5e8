"""Every grouped product's wrapper refuses, on the host and before any pointer reaches a kernel, what a launch would
trust blindly: operands off the device, index tensors of another dtype, short gathers, offsets of the wrong length.
The CPU half needs no GPU (a host tensor is the first thing refused); the GPU half hands device tensors with one
defect each and still launches nothing."""

import pytest
import torch

from dew_amd import _lib, ops
from dew_amd.ops import KernelError


def fake_bank(fmt, experts=2, depth=256, width=256):
    return ops.PreparedBank(_lib.Bank(fmt, _lib.LAYOUT_PREPARED, experts, depth, width, None, None, None), (experts, depth, width), ())


def products(device):
    """(name, call) for each product wrapper with well-formed operands on `device`; `call(**changes)` swaps operands."""
    rows, depth, width, experts = 6, 256, 256, 2
    pitch = ops.block_scale_pitch(depth)
    make = lambda shape, dtype: torch.zeros(shape, dtype=dtype, device=device)
    base = dict(offsets=make((experts + 1,), torch.int32), gather=make((rows,), torch.int32), scatter=make((rows,), torch.int32))
    x = make((rows, depth), torch.bfloat16)
    split, scale, scales = make((rows, 2 * depth), torch.uint8), make((rows,), torch.uint8), make((rows, pitch), torch.uint8)
    codes, mx_scales = make((rows, depth), torch.uint8), make((rows, depth // 32), torch.uint8)
    mx4, fp8, mx8 = fake_bank(_lib.W_MXFP4), fake_bank(_lib.W_FP8_BLOCK), fake_bank(_lib.W_MXFP8)

    def bound(function, *operands, scattered=True):
        def call(**changes):
            arguments = {**base, **changes}
            offsets = arguments.pop("offsets")
            if not scattered:
                arguments.pop("scatter")
            return function(*operands, offsets, **arguments)
        return call

    return [
        ("grouped_gemm", bound(ops.grouped_gemm, x, mx4)),
        ("gateup_swiglu", bound(ops.gateup_swiglu, x, mx4, mx4, scattered=False)),
        ("gateup_interleaved", bound(ops.gateup_interleaved, x, mx4, scattered=False)),
        ("grouped_gemm_split", bound(ops.grouped_gemm_split, split, scale, mx4)),
        ("gateup_swiglu_split", bound(ops.gateup_swiglu_split, split, scale, mx4, mx4, scattered=False)),
        ("gateup_swiglu_split_out", bound(ops.gateup_swiglu_split_out, split, scale, mx4, mx4, scattered=False)),
        ("grouped_gemm_split_blocks", bound(ops.grouped_gemm_split_blocks, split, scales, mx4)),
        ("grouped_gemm_mxfp8_rows", bound(ops.grouped_gemm_mxfp8_rows, codes, mx_scales, mx8)),
        ("grouped_gemm_fp8_rows", bound(ops.grouped_gemm_fp8_rows, codes, scales, fp8)),
    ]


SCATTERED = ("grouped_gemm", "grouped_gemm_split", "grouped_gemm_split_blocks", "grouped_gemm_mxfp8_rows", "grouped_gemm_fp8_rows")


@pytest.mark.parametrize("name", [name for name, _ in products("cpu")])
def test_a_host_operand_is_refused_before_any_launch(name):
    call = dict(products("cpu"))[name]
    with pytest.raises(KernelError, match="must be on the GPU"):
        call()


@pytest.mark.gpu
@pytest.mark.parametrize("name", [name for name, _ in products("cpu")])
def test_defective_index_tensors_are_refused_on_the_device_side_too(name):
    call = dict(products("cuda"))[name]
    device = torch.device("cuda")
    with pytest.raises(KernelError, match="gather must be torch.int32"):
        call(gather=torch.zeros(6, dtype=torch.int64, device=device))
    with pytest.raises(KernelError, match="cover every row"):
        call(gather=torch.zeros(3, dtype=torch.int32, device=device), rows=6)
    with pytest.raises(KernelError, match="offsets has 5 entries"):
        call(offsets=torch.zeros(5, dtype=torch.int32, device=device))
    with pytest.raises(KernelError, match="offsets must be torch.int32"):
        call(offsets=torch.zeros(3, dtype=torch.int64, device=device))
    with pytest.raises(KernelError, match="gather must be on the GPU"):
        call(gather=torch.zeros(6, dtype=torch.int32))
    with pytest.raises(KernelError, match="gather must be contiguous"):
        call(gather=torch.zeros(12, dtype=torch.int32, device=device)[::2])
    with pytest.raises(KernelError, match="rows asked of"):
        call(gather=None, rows=7)
    if name in SCATTERED:   # (the paired and gated products write sorted rows: they take no scatter)
        with pytest.raises(KernelError, match="scatter must be torch.int32"):
            call(scatter=torch.zeros(6, dtype=torch.int64, device=device))


def test_the_float32_gate_and_a_latent_layers_projections_refuse_on_the_host():
    """`gate_rows_add_f32` takes device tensors only; a latent layer's dense projection refuses a kernel of another shape,
    and a float32 kernel where the layer states no compute dtype (the reference would then run the projection in float32)."""
    from dew_amd import moe

    x, rows = torch.zeros((4, 64), dtype=torch.bfloat16), torch.zeros((4, 32), dtype=torch.bfloat16)
    with pytest.raises(KernelError, match="must be on the GPU"):
        ops.gate_rows_add_f32(x, torch.zeros(64), rows, rows)
    layer = moe.SparseMLP(num_experts=4, top_k=2, hidden_features=64, out_features=64, latent_features=32)
    assert layer._bound({}, ()).experts.out_features == 32
    variables = {"params": {"routed_expert_down_proj": {"kernel": torch.zeros((64, 32))}}}
    with pytest.raises(ValueError, match="states no compute dtype"):
        layer._bound(variables, ())._dense(x, "routed_expert_down_proj", 64, 32)
    with pytest.raises(ValueError, match=r"the layer's is \(64, 16\)"):
        layer._bound(variables, ())._dense(x, "routed_expert_down_proj", 64, 16)
    with pytest.raises(KeyError, match="routed_expert_up_proj"):
        layer._bound(variables, ())._dense(x, "routed_expert_up_proj", 32, 64)

"""The kernel selector's behaviour without a GPU: preference, naming, refusal."""

import pytest
import torch

from dew_amd import formats, gemm, selection


def bank(depth=256, width=128):
    return formats.Fp8Blocks(torch.zeros((2, depth, width), dtype=torch.uint8), torch.ones((2, depth // 128, width // 128)))


def test_a_cpu_call_is_refused_with_its_first_requirement():
    case = gemm.GroupedCase(torch.zeros((4, 256), dtype=torch.bfloat16), bank())
    with pytest.raises(ValueError, match="no grouped_matmul kernel takes this call"):
        selection.select(gemm.GROUPED, case)
    with pytest.raises(selection.KernelRefused) as refused, selection.chosen(grouped_matmul="hip"):
        selection.select(gemm.GROUPED, case)
    assert refused.value.first.code == "device" and refused.value.kernel == "hip"
    assert [r.code for r in refused.value.refusals] == ["device"]


def test_requirements_are_reported_in_order():
    case = gemm.GroupedCase(torch.zeros((4, 100)), torch.zeros((2, 100, 60)), epilogue="gelu")
    codes = [refusal.code for refusal in gemm.HIP.refusals(case)]
    assert codes[:3] == ["device", "quantized-bank", "bf16"]


def test_foreign_kernel_names_are_unlowerable_and_unknown_ones_are_errors():
    case = gemm.GroupedCase(torch.zeros((4, 256), dtype=torch.bfloat16), bank())
    for name in ("xla", "cutlass", "mosaic", "triton", "pallas"):
        with pytest.raises(selection.Unlowerable, match=name):
            selection.select(gemm.GROUPED, case, named=name)
    with pytest.raises(ValueError, match="has no kernel"):
        selection.select(gemm.GROUPED, case, named="cublas")


def test_chosen_is_scoped():
    assert selection.forced("grouped_matmul") is None
    with selection.chosen(grouped_matmul="hip"):
        assert selection.forced("grouped_matmul") == "hip"
    assert selection.forced("grouped_matmul") is None

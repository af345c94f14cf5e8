"""Checkpoint banks taken to the kernels' formats at load (dew_amd/loads.py), on the CPU: no value is decoded,
and what the banks stand for is exactly what the source's own decoding yields."""

import numpy as np
import pytest
import torch
from conftest import golden

from dew_amd import codecs, formats, loads
from oracle import moe_oracle as oracle

MXFP4 = {"quantization_config": {"quant_method": "mxfp4"}}


def test_an_mxfp4_bank_is_served_packed_and_stands_for_the_sources_values():
    rng = np.random.default_rng(4)
    weight = torch.from_numpy((rng.standard_normal((3, 256, 64)) * 0.05).astype(np.float32))
    blocks, scales = codecs.quantize_mxfp4(weight)
    tensors = {"mlp.experts.down_proj_blocks": blocks, "mlp.experts.down_proj_scales": scales,
               "mlp.router.weight": torch.zeros(3, 64)}
    left, banks = loads.packed_banks(tensors, MXFP4)
    assert set(banks) == {"mlp.experts.down_proj"} and "mlp.experts.down_proj_blocks" not in left
    assert left["mlp.experts.down_proj"] == loads.Unread((3, 256, 64), torch.float32) and "mlp.router.weight" in left
    bank = banks["mlp.experts.down_proj"].checked()
    decoded = oracle.nvfp4_bank_decoded(bank.words.numpy().view(np.uint32), bank.scales.numpy())
    factor = oracle.nvfp4_bank_factor(bank.scale.numpy())
    want = oracle.decode_mxfp4(blocks.numpy(), scales.numpy())          # [E, K, N], the source's own decoding
    assert np.array_equal(decoded * factor[:, None, None], want)


def test_a_bank_of_no_whole_stages_stays_as_the_source_states_it(caplog):
    held = golden("gpt_oss/mxfp4.npz")                                   # depth 64: no whole 256-deep stage
    tensors = {"w_blocks": torch.from_numpy(held["blocks"]), "w_scales": torch.from_numpy(held["scales"])}
    with caplog.at_level("WARNING"):
        left, banks = loads.packed_banks(tensors, MXFP4)
    assert not banks and set(left) == {"w_blocks", "w_scales"} and "no whole 256-deep stages" in caplog.text
    with pytest.raises(ValueError, match="mxfp4"):
        loads.packed_banks(tensors, {"quantization_config": {"quant_method": "fp8"}})


def test_fp8_block_checkpoints_stay_quantized():
    rng = np.random.default_rng(5)
    experts, depth, width = 2, 256, 128
    tensors = {}
    for e in range(experts):
        for projection, (k, n) in {"gate_proj": (depth, width), "up_proj": (depth, width), "down_proj": (width, depth)}.items():
            codes, scale_inv = codecs.fp8_block_cast(torch.from_numpy((rng.standard_normal((n, k)) * 0.1).astype(np.float32)))
            tensors[f"mlp.experts.{e}.{projection}.weight"] = codes
            tensors[f"mlp.experts.{e}.{projection}.weight_scale_inv"] = scale_inv
    left, banks = loads.fp8_expert_banks(tensors, "mlp.experts", experts)
    assert not left and set(banks) == {"gate_proj", "up_proj", "down_proj"}
    gate = banks["gate_proj"]
    assert gate.shape == (experts, depth, width)
    for e in range(experts):
        want = oracle.dequantize_fp8_blocks(tensors[f"mlp.experts.{e}.gate_proj.weight"].view(torch.uint8).numpy(),
                                            tensors[f"mlp.experts.{e}.gate_proj.weight_scale_inv"].numpy())
        got = oracle.dequantize_fp8_blocks(gate.codes[e].numpy(), gate.scale_inv[e].numpy())
        assert np.array_equal(got, want.T)


def test_banks_take_their_parameters_place_in_the_quantization_collection():
    bank = object()
    variables = {"params": {"experts": {"down_proj": "unread", "down_proj_bias": 1}, "router": {"kernel": 2}}}
    placed = loads.with_banks(variables, {"w": ("experts", "down_proj")}, {"w": bank})
    assert placed["quantization"]["experts"]["down_proj"] is bank
    assert placed["params"] == {"experts": {"down_proj_bias": 1}, "router": {"kernel": 2}}
    assert variables["params"]["experts"]["down_proj"] == "unread"       # the caller's tree is untouched
    with pytest.raises(ValueError, match="binds no path"):
        loads.with_banks(variables, {}, {"w": bank})

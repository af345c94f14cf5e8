"""The product's quantizers and bank packers against the bytes the reference's tests hold, and against the
oracle's independent decoders (encode here, decode there)."""

import numpy as np
import pytest
import torch
from conftest import golden

from dew_amd import codecs, formats
from oracle import moe_oracle as oracle


@pytest.mark.parametrize("case,block", [("random/256x384/128", 128), ("random/130x259/128", 128),
                                        ("random/5x7/128", 128), ("random/48x32/16", 16), ("random/7x3/2", 2),
                                        ("edge", 1)])
def test_fp8_block_cast_reproduces_deepgemm_bytes(case, block):
    held = golden("codecs/deepgemm_fp8.npz")
    weight = torch.from_numpy(held[f"{case}/weight"])
    codes, scales = codecs.fp8_block_cast(weight, block)
    assert np.array_equal(scales.numpy().view(np.uint32), held[f"{case}/scales"].view(np.uint32))
    assert np.array_equal(codes.numpy(), held[f"{case}/codes"])


def test_fp8_channel_cast_scales_each_output_column():
    rng = np.random.default_rng(0)
    weight = torch.from_numpy((rng.standard_normal((3, 64, 5)) * 0.02).astype(np.float32))
    codes, scales = codecs.fp8_channel_cast(weight)
    assert codes.shape == (3, 64, 5) and scales.shape == (3, 5)
    amax = weight.abs().amax(dim=1).clamp_min(1e-4)
    assert torch.equal(scales, amax / 448)
    back = oracle.dequantize_fp8_channels(codes.numpy(), scales.numpy())
    assert np.abs(back - weight.numpy()).max() <= (amax.max().item() / 448) * 16 + 1e-9
    # the column's largest magnitude takes the largest code
    assert ((codes & 0x7F).amax(dim=1) == 0x7E).all()


@pytest.mark.parametrize("name", ["midpoints", "random_bf16", "mixed", "trained", "every_bf16_magnitude"])
def test_mxfp4_encoder_reproduces_the_released_bytes(name):
    held = golden("gpt_oss/mxfp4_encoder.npz")
    blocks, scales = codecs.quantize_mxfp4(torch.from_numpy(held[f"{name}_weight"]))
    assert np.array_equal(scales.numpy(), held[f"{name}_scales"])
    assert np.array_equal(blocks.numpy(), held[f"{name}_blocks"])


def test_mxfp4_decodes_to_the_references_dense_bank():
    """`dequantize_mxfp4` (what a load does with a bank that stays dense: gpt-oss's 2880-deep experts) on the reference's
    own vector (tests/fixtures/gpt_oss/mxfp4.npz: blocks, scales, decoded output), bit for bit, and on a seeded bank
    against the oracle's decoder; every value survives the bf16 it is held in."""
    held = golden("gpt_oss/mxfp4.npz")
    blocks, scales = torch.from_numpy(held["blocks"]), torch.from_numpy(held["scales"])
    assert np.array_equal(codecs.dequantize_mxfp4(blocks, scales, torch.float32).numpy(), held["output"])
    assert np.array_equal(codecs.dequantize_mxfp4(blocks, scales).float().numpy(), held["output"])
    rng = np.random.default_rng(5)
    weight = torch.from_numpy((rng.standard_normal((2, 320, 96)) * 0.02).astype(np.float32))     # 320 deep: no whole 256-deep stage
    blocks, scales = codecs.quantize_mxfp4(weight)
    dense = codecs.dequantize_mxfp4(blocks, scales)
    assert dense.shape == (2, 320, 96) and dense.dtype == torch.bfloat16 and dense.is_contiguous()
    assert np.array_equal(dense.float().numpy(), oracle.decode_mxfp4(blocks.numpy(), scales.numpy()))
    with pytest.raises(ValueError, match="MXFP4 blocks"):
        codecs.dequantize_mxfp4(blocks, scales[:, :, :1])


def test_mxfp4_bank_as_nvfp4_holds_every_value_exactly():
    rng = np.random.default_rng(1)
    weight = torch.from_numpy((rng.standard_normal((3, 256, 6)) * 0.02).astype(np.float32))
    weight[1, 32:64, 2] = 0                                           # an all-zero group
    blocks, scales = codecs.quantize_mxfp4(weight)
    dense = oracle.decode_mxfp4(blocks.numpy(), scales.numpy())      # [E, K, N]
    powers = codecs.mxfp4_tensor_powers(blocks, scales)
    assert powers is not None
    bank = formats.NvFp4.of(*codecs.mxfp4_as_nvfp4(blocks, scales, powers)).checked()
    assert bank.shape == (3, 256, 6) and bank.words.shape == (3, 6, 32) and bank.scales.shape == (3, 6, 16)
    decoded = oracle.nvfp4_bank_decoded(bank.words.numpy().view(np.uint32), bank.scales.numpy())
    values = decoded * oracle.nvfp4_bank_factor(bank.scale.numpy())[:, None, None]
    assert np.array_equal(values, dense)
    # both 16-blocks of a 32-group share one power-of-two scale
    block_scales = oracle.E4M3[bank.scales.numpy()]
    assert np.array_equal(block_scales[..., 0::2], block_scales[..., 1::2])
    assert (np.log2(block_scales) % 1 == 0).all()


def test_mxfp4_powers_refuse_a_bank_spread_past_e4m3():
    blocks = torch.full((1, 1, 2, 16), 0x22, dtype=torch.uint8)
    assert codecs.mxfp4_tensor_powers(blocks, torch.tensor([[[100, 118]]], dtype=torch.uint8)) is None
    assert codecs.mxfp4_tensor_powers(blocks, torch.tensor([[[100, 117]]], dtype=torch.uint8)).tolist() == [-18]
    assert codecs.mxfp4_tensor_powers(blocks, torch.tensor([[[100, 255]]], dtype=torch.uint8)) is None


def test_nvfp4_quantizer_is_the_closed_form_the_reference_states():
    rng = np.random.default_rng(5)
    x = rng.standard_normal((256, 64)).astype(np.float32)
    x[16:32, 3] = 0
    codes, scales, tensor = codecs.nvfp4_coded(torch.from_numpy(x))
    codes, scales, tensor = codes.numpy(), scales.numpy(), tensor.numpy()
    largest = np.float32(np.abs(x).max())                             # tests/test_algebra_bits.py:510-528
    assert tensor == largest / np.float32(6 * 448)
    table = oracle.E4M3[:0x7F]
    blocks = np.abs(x).reshape(16, 16, 64).max(axis=1)
    ratio = blocks / tensor / np.float32(6)
    least = table[np.minimum(np.searchsorted(table, ratio), table.size - 1)]
    assert np.array_equal(oracle.E4M3[scales], least)
    each = np.repeat(least, 16, axis=0)
    quotient = np.where(each > 0, x / tensor / np.where(each > 0, each, 1), 0).astype(np.float32)
    # nearest E2M1 with ties to even, by brute force over the eight magnitudes
    grid = oracle.E2M1[:8].astype(np.float64)
    distance = np.abs(np.abs(quotient.astype(np.float64))[..., None] - grid)
    nearest = distance.argmin(-1)
    tie = np.isclose(np.sort(distance, -1)[..., 0], np.sort(distance, -1)[..., 1], rtol=0, atol=0)
    upper = np.minimum(nearest + 1, 7)
    nearest = np.where(tie & (nearest % 2 == 1), upper, nearest)
    assert np.array_equal(codes & 7, nearest)
    assert np.array_equal((codes >> 3).astype(bool), np.signbit(quotient))
    assert not (codes[16:32, 3] & 7).any()


def test_e2m1_rounding_ties_to_even():
    q = torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 7.0, -0.25, -0.0, 0.2499, 0.2501])
    assert codecs._e2m1_rne(q).tolist() == [0, 2, 2, 4, 4, 6, 6, 7, 8, 8, 0, 1]


def test_nvfp4_bank_words_are_staged_and_encoded_and_read_back():
    rng = np.random.default_rng(6)
    weight = torch.from_numpy(rng.standard_normal((2, 256, 8)).astype(np.float32))
    bank = formats.NvFp4.quantized(weight).checked()
    assert formats.FORM_HEX == "7fb7f1b609cea47a" == oracle.nvfp4_form_digest()
    assert formats.staged_rows(256)[8 * 3 + 5] == 16 * 5 + 3 and formats.staged_rows(256)[128] == 128
    for e in range(2):
        codes, scales, tensor = codecs.nvfp4_coded(weight[e])
        assert np.array_equal(oracle.nvfp4_bank_codes(bank.words.numpy().view(np.uint32))[e], codes.numpy())
        assert np.array_equal(bank.scales[e].numpy().T, scales.numpy())
        assert bank.scale[e] == tensor
    decoded = oracle.nvfp4_bank_decoded(bank.words.numpy().view(np.uint32), bank.scales.numpy())
    values = decoded * oracle.nvfp4_bank_factor(bank.scale.numpy())[:, None, None]
    # each value is within half an E2M1 step of the weight, under its block's scale
    assert np.abs(values - weight.numpy()).max() < np.abs(weight.numpy()).max() * 0.26


def test_a_bank_packed_by_another_encoder_is_refused():
    bank = formats.NvFp4(torch.zeros((1, 1, 32), dtype=torch.int32), torch.zeros((1, 1, 16), dtype=torch.uint8),
                         torch.ones(1), torch.zeros(8, dtype=torch.uint8))
    with pytest.raises(ValueError, match="form version"):
        bank.checked()
    with pytest.raises(ValueError, match="whole 256s"):
        formats.NvFp4.of(torch.zeros((1, 128, 4), dtype=torch.uint8), torch.zeros((1, 8, 4), dtype=torch.uint8),
                         torch.ones(1))


@pytest.mark.parametrize("release", ["v4", "v4_1"])
def test_a_deepseek_v4_fp4_expert_is_an_mxfp4_bank_as_stored(release):
    """The FP4 routed expert of the reference's tests/fixtures/codecs/deepseek_v4_release.npz (each release's own
    conversion over a tiny checkpoint, tests/test_codecs.py:219-237 there): stacked as it is stored
    (`loads.fp4_expert_bank`, no value decoded), the bank's MXFP4 decoding is the release's dense reading of the expert in
    every value, by the product's decoder and by the oracle's."""
    from dew_amd import loads
    held = golden("codecs/deepseek_v4_fp4_expert.npz")
    weight, scale, dense = (held[f"{release}/{name}"] for name in ("weight", "scale", "dense"))
    bank = loads.fp4_expert_bank([torch.from_numpy(weight.copy())] * 2, [torch.from_numpy(scale.copy())] * 2)
    outputs, inputs = dense.shape
    assert isinstance(bank, formats.Mxfp4Blocks) and bank.shape == (2, inputs, outputs)
    assert np.array_equal(bank.blocks.numpy().reshape(2, outputs, inputs // 2), np.stack([weight.view(np.uint8)] * 2))   # the bytes themselves
    decoded = codecs.dequantize_mxfp4(bank.blocks, bank.scales, torch.float32).numpy()
    assert np.array_equal(decoded[0], dense.T) and np.array_equal(decoded[1], dense.T)
    assert np.array_equal(oracle.decode_mxfp4(bank.blocks.numpy(), bank.scales.numpy())[0], dense.T)
    tensors = {f"ffn.experts.{e}.{p}{suffix}": torch.from_numpy((weight if suffix == ".weight" else scale).copy())
               for e in range(2) for p in ("w1", "w3", "w2") for suffix in loads.FP4_SUFFIXES}
    tensors["ffn.gate.weight"] = torch.zeros(2, 4)
    left, banks = loads.fp4_expert_banks(tensors, "ffn.experts", 2)
    assert list(left) == ["ffn.gate.weight"] and sorted(banks) == ["w1", "w2", "w3"]
    assert all(torch.equal(found.blocks, bank.blocks) and torch.equal(found.scales, bank.scales) for found in banks.values())
    with pytest.raises(ValueError, match="whole groups of 32"):
        loads.fp4_expert_bank([torch.from_numpy(weight[:, :24].copy())], [torch.from_numpy(scale.copy())])

"""The checkpoint codecs on the device: `dew_moe_prepare_bank` takes an MXFP4 checkpoint's `*_blocks` / `*_scales` and
an FP8 checkpoint's `weight [out, in]` / `weight_scale_inv` as they are stored, and the prepared bank is, byte for
byte, the one the reference's own chain yields (`mxfp4_tensor_powers` -> `mxfp4_as_nvfp4` -> `NvFp4.of`, or the
transposed `[E, in, out]` bank, then the re-layout); products through either are bit-identical."""

import numpy as np
import pytest
import torch
from conftest import golden

from dew_amd import _lib, codecs, formats, loads
from oracle import moe_oracle as oracle

pytestmark = pytest.mark.gpu

MXFP4 = {"quantization_config": {"quant_method": "mxfp4"}}


@pytest.fixture(scope="module")
def ops():
    from dew_amd import ops

    ops.device_check()
    return ops


def prepared_parts(bank):
    """(format, codes bytes, scale bytes, tensor scales) of a prepared FP4 bank."""
    experts, depth, width = bank.shape
    buffer = bank.keep[0]
    codes, scales = experts * depth * width // 2, experts * width * (depth // 16)
    assert bank.descriptor.codes == buffer.data_ptr() and bank.descriptor.scales == buffer.data_ptr() + codes
    return bank.descriptor.format, buffer[:codes].cpu(), buffer[codes:codes + scales].cpu(), bank.keep[2].cpu()


def both_ways(ops, blocks, scales):
    """The bank prepared from the checkpoint's bytes on the device, and through the reference's chain."""
    powers = codecs.mxfp4_tensor_powers(blocks, scales)
    assert powers is not None
    chain = ops.prepare(formats.NvFp4.of(*codecs.mxfp4_as_nvfp4(blocks, scales, powers)).to("cuda"))
    direct = ops.prepare(formats.Mxfp4Blocks(blocks.cuda(), scales.cuda()))
    return direct, chain


def assert_same_bank(ops, direct, chain, seed):
    for got, want in zip(prepared_parts(direct), prepared_parts(chain), strict=True):
        assert torch.equal(got, want) if torch.is_tensor(got) else got == want
    experts, depth, width = direct.shape
    rng = np.random.default_rng(seed)
    sizes = rng.integers(0, 70, size=experts)
    offsets = torch.tensor(np.concatenate([[0], np.cumsum(sizes)]).astype(np.int32)).cuda()
    x = torch.from_numpy(rng.standard_normal((int(sizes.sum()) + 3, depth)).astype(np.float32)).to(torch.bfloat16).cuda()
    assert torch.equal(ops.grouped_gemm(x, direct, offsets), ops.grouped_gemm(x, chain, offsets))


def test_an_mxfp4_checkpoints_bytes_become_the_reference_chains_prepared_bank(ops):
    rng = np.random.default_rng(11)
    weight = torch.from_numpy((rng.standard_normal((3, 512, 256)) * 0.05).astype(np.float32))
    weight[0, :64, :5] = 0.0                       # groups of zeros
    weight[1, 32:64, 7] = -0.0                     # ... and of signed zeros
    weight[2] *= 2.0 ** 20                         # an expert far from the others: its own tensor scale
    blocks, scales = codecs.quantize_mxfp4(weight)
    direct, chain = both_ways(ops, blocks, scales)
    assert direct.descriptor.format == _lib.W_MXFP4
    assert_same_bank(ops, direct, chain, seed=1)


def test_group_powers_below_e4m3s_normals_make_a_general_nvfp4_bank_both_ways(ops):
    rng = np.random.default_rng(12)
    weight = torch.from_numpy((rng.standard_normal((2, 256, 128)) * 0.05).astype(np.float32))
    weight[0, :32, :16] *= 2.0 ** -15              # block scales 2^-7 .. 2^-9 of the expert's largest: subnormal in E4M3
    weight[1, 64:96, 3] *= 2.0 ** -16
    blocks, scales = codecs.quantize_mxfp4(weight)
    direct, chain = both_ways(ops, blocks, scales)
    assert direct.descriptor.format == _lib.W_NVFP4 == chain.descriptor.format
    assert_same_bank(ops, direct, chain, seed=2)


def test_the_reference_held_mxfp4_blocks_prepare_alike_both_ways(ops):
    """The bytes of the reference's own MXFP4 fixture (2 experts x 8 columns x 64 depths), tiled to the least bank the
    kernels take (128 columns, 256 depths). Its scale bytes span 30 binades an expert, so the whole fixture is a bank
    the reference keeps dense, and the device refuses it alike; each expert's columns whose scales lie within 17
    binades (real checkpoint scale bytes and codes, cycled across the 128 columns) prepare alike both ways."""
    held = golden("gpt_oss/mxfp4.npz")
    blocks, scales = torch.from_numpy(held["blocks"]), torch.from_numpy(held["scales"])
    whole = (blocks.repeat(1, 16, 4, 1).contiguous(), scales.repeat(1, 16, 4).contiguous())
    assert codecs.mxfp4_tensor_powers(*whole) is None
    with pytest.raises(ops.KernelError, match="stays dense"):
        ops.prepare(formats.Mxfp4Blocks(whole[0].cuda(), whole[1].cuda()))
    chosen_blocks, chosen_scales = [], []
    for expert in range(blocks.shape[0]):
        top = int(scales[expert].max())
        columns = [n for n in range(blocks.shape[1]) if int(scales[expert, n].min()) >= top - 17]
        assert len(columns) >= 2
        cycle = torch.tensor([columns[i % len(columns)] for i in range(128)])
        chosen_blocks.append(blocks[expert, cycle].repeat(1, 4, 1))
        chosen_scales.append(scales[expert, cycle].repeat(1, 4))
    direct, chain = both_ways(ops, torch.stack(chosen_blocks).contiguous(), torch.stack(chosen_scales).contiguous())
    assert direct.shape == (2, 256, 128)
    assert_same_bank(ops, direct, chain, seed=3)


def test_a_bank_the_reference_keeps_dense_is_refused_by_name(ops, caplog):
    rng = np.random.default_rng(13)
    weight = torch.from_numpy((rng.standard_normal((2, 256, 128)) * 0.05).astype(np.float32))
    weight[1, :32, 0] *= 2.0 ** -30                # one expert's group powers spread past 17 binades
    blocks, scales = codecs.quantize_mxfp4(weight)
    assert codecs.mxfp4_tensor_powers(blocks, scales) is None
    with pytest.raises(ops.KernelError, match="stays dense"):
        ops.prepare(formats.Mxfp4Blocks(blocks.cuda(), scales.cuda()))
    poisoned = scales.clone()
    poisoned[0, 5, 1] = 255                        # the NaN scale byte
    with pytest.raises(ops.KernelError, match="stays dense"):
        ops.prepare(formats.Mxfp4Blocks(blocks.cuda(), poisoned.cuda()))
    tensors = {"w_blocks": blocks.cuda(), "w_scales": scales.cuda()}
    with caplog.at_level("WARNING"):
        left, banks = loads.packed_banks(tensors, MXFP4)
    assert not banks and set(left) == {"w_blocks", "w_scales"} and "stays dense" in caplog.text


def test_a_bank_that_stays_dense_decodes_on_the_device_and_multiplies_as_the_references_does(ops, caplog):
    """gpt-oss's experts in small: 320 deep (no whole 256-deep NVFP4 stage) and 352 wide. By the reference's rule
    `packed_banks` leaves the bank as the source states it; `dense_bank` decodes it on the device as the reference's load does
    (`dequantize_mxfp4`) and the unquantized bank's launch multiplies it, against the oracle's product over the
    oracle's own decoding."""
    from dew_amd import gemm

    rng = np.random.default_rng(17)
    experts, depth, width, sizes = 3, 320, 352, [60, 0, 41]
    weight = torch.from_numpy((rng.standard_normal((experts, depth, width)) * 0.05).astype(np.float32))
    blocks, scales = codecs.quantize_mxfp4(weight)
    tensors = {"w_blocks": blocks.cuda(), "w_scales": scales.cuda()}
    with caplog.at_level("WARNING"):
        left, banks = loads.packed_banks(tensors, MXFP4, device_codec=False)   # the reference's own chain: NvFp4 words, staged 256 deep
    assert not banks and "no whole 256-deep stages" in caplog.text
    kept, _ = loads.packed_banks(tensors, MXFP4)                                # (the device re-layout keeps this bank packed)
    assert isinstance(_["w"], formats.Mxfp4Blocks) and set(kept) == {"w"}
    bank = loads.dense_bank(left["w_blocks"], left["w_scales"])
    assert bank.shape == (experts, depth, width) and bank.weights.is_cuda
    dense = oracle.decode_mxfp4(blocks.numpy(), scales.numpy())
    assert np.array_equal(bank.weights.float().cpu().numpy(), dense)
    x = torch.from_numpy(rng.standard_normal((int(np.sum(sizes)), depth)).astype(np.float32)).to(torch.bfloat16)
    got = gemm.gemm(x.cuda(), bank, torch.tensor(sizes, dtype=torch.int32).cuda()).float().cpu().numpy()
    want = oracle.grouped_matmul(x.float().numpy(), dense, sizes)
    assert got.shape == want.shape and np.abs(got - want).max() <= 2 ** -7 * np.abs(want).max() and (got == want).mean() > 0.97


def test_packed_banks_on_the_device_hands_over_the_checkpoints_own_tensors(ops):
    from dew_amd import gemm

    rng = np.random.default_rng(14)
    weight = torch.from_numpy((rng.standard_normal((4, 256, 256)) * 0.05).astype(np.float32))
    blocks, scales = codecs.quantize_mxfp4(weight)
    left, banks = loads.packed_banks({"e.down_proj_blocks": blocks.cuda(), "e.down_proj_scales": scales.cuda()}, MXFP4)
    bank = banks["e.down_proj"]
    assert isinstance(bank, formats.Mxfp4Blocks) and bank.shape == (4, 256, 256) and left["e.down_proj"].shape == (4, 256, 256)
    _, host = loads.packed_banks({"e.down_proj_blocks": blocks, "e.down_proj_scales": scales}, MXFP4)
    sizes = torch.tensor([5, 0, 130, 64], dtype=torch.int32).cuda()
    x = torch.from_numpy(rng.standard_normal((199, 256)).astype(np.float32)).to(torch.bfloat16).cuda()
    assert torch.equal(gemm.gemm(x, bank, sizes), gemm.gemm(x, host["e.down_proj"].to("cuda"), sizes))


def test_an_fp8_checkpoints_tensors_are_read_where_they_lie(ops):
    rng = np.random.default_rng(15)
    experts, depth, width = 3, 384, 256
    weights, inverses = [], []
    for _ in range(experts):   # each expert's `weight [out, in]` and `weight_scale_inv [out / 128, in / 128]`
        codes, scale_inv = codecs.fp8_block_cast(torch.from_numpy((rng.standard_normal((width, depth)) * 0.1).astype(np.float32)))
        weights.append(codes.cuda()), inverses.append(scale_inv.cuda())
    direct_bank = loads.fp8_block_bank(weights, inverses)
    chain_bank = loads.fp8_block_bank(weights, inverses, device_codec=False)
    assert direct_bank.kmajor and not chain_bank.kmajor and direct_bank.shape == chain_bank.shape == (experts, depth, width)
    direct, chain = ops.prepare(direct_bank), ops.prepare(chain_bank)
    assert torch.equal(direct.keep[0], chain.keep[0])          # codes and block scales, byte for byte
    sizes = [70, 0, 133]
    offsets = torch.tensor(np.concatenate([[0], np.cumsum(sizes)]).astype(np.int32)).cuda()
    x = torch.from_numpy(rng.standard_normal((sum(sizes), depth)).astype(np.float32)).to(torch.bfloat16).cuda()
    assert torch.equal(ops.grouped_gemm(x, direct, offsets), ops.grouped_gemm(x, chain, offsets))
    assert torch.equal(ops.gateup_swiglu(x, direct, direct, offsets), ops.gateup_swiglu(x, chain, chain, offsets))


@pytest.mark.parametrize("release", ["v4", "v4_1"])
def test_a_deepseek_v4_fp4_expert_multiplies_packed_as_the_releases_dense_reading_does(ops, release):
    """The FP4 routed expert the reference's tests hold (tests/fixtures/codecs/deepseek_v4_release.npz: the releases' own
    conversion), stacked as stored (`loads.fp4_expert_bank`) and multiplied on the device without a dense copy, against
    the oracle's product over the release's dense reading of that expert. V4.1's tiny expert is 96 deep and 64 wide,
    below the launches' least extents, so its bytes are tiled to 192 x 128; its scale bytes were drawn over 21 binades,
    past what one expert's packed bank spans (17), so the re-layout refuses it by name and it multiplies as the decoded
    bank (`loads.dense_bank`), as such a bank of gpt-oss's would."""
    from dew_amd import gemm

    held = golden("codecs/deepseek_v4_fp4_expert.npz")
    weight, scale, dense = (held[f"{release}/{name}"] for name in ("weight", "scale", "dense"))
    if release == "v4_1":
        weight, scale, dense = (np.tile(array, (2, 2)) for array in (weight, scale, dense))
    sizes = [37, 0, 70]
    bank = loads.fp4_expert_bank([torch.from_numpy(weight.copy()).cuda()] * 3, [torch.from_numpy(scale.copy()).cuda()] * 3)
    outputs, inputs = dense.shape
    assert bank.shape == (3, inputs, outputs) and bank.blocks.is_cuda
    if release == "v4_1":
        with pytest.raises(ops.KernelError, match="stays dense"):
            gemm.prepared(bank)
        bank = loads.dense_bank(bank.blocks, bank.scales)
    rng = np.random.default_rng(inputs)
    x = torch.from_numpy(rng.standard_normal((sum(sizes), inputs)).astype(np.float32)).to(torch.bfloat16)
    got = gemm.gemm(x.cuda(), bank, torch.tensor(sizes, dtype=torch.int32).cuda()).float().cpu().numpy()
    want = oracle.grouped_matmul(x.float().numpy(), np.stack([dense.T] * 3), sizes)
    assert got.shape == want.shape and np.abs(got - want).max() <= 2 ** -7 * np.abs(want).max() and (got == want).mean() > 0.97

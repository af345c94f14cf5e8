"""The blockwise FP8 recipe's forward product on the device (rows quantized 1 x 128, weights 128 x 128, power-of-two
scales, both operands through the scaled matrix instruction) against the CPU oracle.

Bars: the rows' quantizer bit for bit (codes and scales are byte work); the product within one bf16 ulp of the
largest output (kernel and oracle multiply the same codes exactly and differ in the order of the fp32 sums alone)."""

import numpy as np
import pytest
import torch

from oracle import moe_oracle as oracle

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from dew_amd import ops

    return ops


def bf16_np(tensor):
    return tensor.float().cpu().numpy()


def rows_case(rows, depth, seed):
    """Rows with the quantizer's corner tiles among ordinary ones."""
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((rows, depth)).astype(np.float32) * rng.choice([1e-3, 0.1, 1.0, 30.0], size=(rows, 1)).astype(np.float32)
    x[0, :128] = 0.0                                   # an all-zero tile: the 1e-4 floor sets its scale
    x[1, :128] = np.linspace(-1e-5, 1e-5, 128)         # under the floor: tiny codes, negative ones rounding to -0
    x[2, :128] = np.clip(x[2, :128], -0.875, 0.875)
    x[2, 5] = 0.875                                    # amax = 448 * 2^-9: amax * f32(1 / 448) decides the scale
    x[3, :128] = np.clip(x[3, :128], -448.0, 448.0)
    x[3, 77] = -448.0                                  # amax = 448 exactly
    x[4, 128:256] *= 1e30                              # a huge tile beside ordinary ones
    x[5, :128] = 2.0 ** -130                           # bf16 subnormals
    return torch.from_numpy(x).to(torch.bfloat16)


@pytest.mark.parametrize("rows,depth", [(7, 128), (33, 384), (260, 4096)])
def test_rows_are_quantized_bit_for_bit(ops, rows, depth):
    x = rows_case(rows, depth, seed=rows)
    codes, scales = ops.quantize_rows_fp8(x.cuda())
    want_values, want_scales = oracle.rows_quantized(bf16_np(x))
    want_codes = oracle.e4m3_bytes(want_values)
    got_codes = ops.depth_order_fp8(codes).cpu().numpy()
    got_scales = scales.cpu().numpy()[:, :depth // 128]
    assert np.array_equal(np.ldexp(np.float32(1), got_scales.astype(np.int32) - 127), want_scales)
    assert np.array_equal(got_codes, want_codes)
    assert np.array_equal(ops.operand_order_fp8(ops.depth_order_fp8(codes)).cpu().numpy(), codes.cpu().numpy())


def weights_case(groups, depth, width, seed):
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((groups, depth, width)) * 0.02).astype(np.float32)
    w[0, :128, :128] *= 50.0                           # blocks of different scales
    w[-1, -128:, -128:] = 0.0                          # an all-zero block
    return w


SIZES = [("ragged", [130, 0, 1, 257, 64, 0, 127, 5]), ("single", [3]), ("blocks", [256, 128, 0, 384])]


@pytest.mark.parametrize("label,sizes", SIZES, ids=[s[0] for s in SIZES])
@pytest.mark.parametrize("depth,width", [(256, 128), (1152, 384)])
def test_the_recipes_product_matches_the_oracle(ops, label, sizes, depth, width):
    from dew_amd import projections

    groups, rows = len(sizes), int(np.sum(sizes))
    rng = np.random.default_rng(depth + rows)
    x = torch.from_numpy(rng.standard_normal((rows + 6, depth)).astype(np.float32)).to(torch.bfloat16)   # 6 rows past the groups
    w = weights_case(groups, depth, width, seed=depth)
    bias = torch.from_numpy(rng.standard_normal((groups, width)).astype(np.float32) * 0.1)
    sizes_device = torch.tensor(sizes, dtype=torch.int32).cuda()
    bank = projections.blocks_quantized(torch.from_numpy(w)).to("cuda")
    for with_bias in (None, bias):
        got = bf16_np(projections.recipe_projection(x.cuda(), bank, sizes_device, bias=None if with_bias is None else with_bias.cuda()))
        padded = list(sizes) + [0]
        want = oracle.blockwise_fp8_projection(bf16_np(x), w, sizes, bias=None if with_bias is None else with_bias.numpy())
        assert np.all(got[rows:] == 0) and np.all(want[rows:] == 0)
        scale = np.abs(want).max()
        assert np.abs(got - want).max() <= 2.0 ** -7 * scale
        assert (got == want).mean() > 0.97
    # the product alone from the quantized operands, against the float64 sum of the dequantized blocks (the
    # reference's own truth, tests/blockwise_matrix.py): what one bf16 rounding of an fp32 sum allows
    values, scales = oracle.rows_quantized(bf16_np(x))
    blocks, block_scales = oracle.blocks_quantized(w)
    truth = np.zeros((rows + 6, width))
    start = 0
    for group, size in enumerate(sizes):
        lhs = (values[start:start + size].reshape(size, depth // 128, 128) * scales[start:start + size, :, None]).reshape(size, depth)
        rhs = blocks[group] * np.repeat(np.repeat(block_scales[group], 128, axis=0), 128, axis=1)
        truth[start:start + size] = lhs.astype(np.float64) @ rhs.astype(np.float64)
        start += size
    got = bf16_np(projections.recipe_projection(x.cuda(), bank, sizes_device))
    assert np.abs(got - truth).max() <= 2.0 ** -8 * np.abs(truth).max() * 1.01


def test_gathered_rows_and_scattered_outputs(ops):
    from dew_amd import projections

    sizes, depth, width = [200, 56, 300], 512, 256
    rows = sum(sizes)
    rng = np.random.default_rng(9)
    x = torch.from_numpy(rng.standard_normal((400, depth)).astype(np.float32)).to(torch.bfloat16)
    gather = rng.integers(0, 400, size=rows).astype(np.int32)
    scatter = rng.permutation(rows).astype(np.int32)
    w = weights_case(len(sizes), depth, width, seed=4)
    bank = projections.blocks_quantized(torch.from_numpy(w)).to("cuda")
    quantized = projections.rows_quantized(x.cuda())
    got = bf16_np(projections.blockwise_fp8_product(quantized, bank, torch.tensor(sizes, dtype=torch.int32).cuda(),
                                                    gather=torch.from_numpy(gather).cuda(), scatter=torch.from_numpy(scatter).cuda()))
    want = oracle.blockwise_fp8_projection(bf16_np(x)[gather], w, sizes)
    placed = np.zeros_like(want)
    placed[scatter] = want
    assert np.abs(got - placed).max() <= 2.0 ** -7 * np.abs(want).max() and (got == placed).mean() > 0.97


def test_group_blocks_count_whole_128_row_blocks(ops):
    from dew_amd import projections

    blocks, depth, width = [2, 0, 1], 256, 128
    rng = np.random.default_rng(2)
    x = torch.from_numpy(rng.standard_normal((384, depth)).astype(np.float32)).to(torch.bfloat16)
    w = weights_case(3, depth, width, seed=8)
    got = bf16_np(projections.blockwise_fp8_projection(x.cuda(), torch.from_numpy(w).cuda(), blocks))
    want = oracle.blockwise_fp8_projection(bf16_np(x), w, [256, 0, 128])
    assert np.abs(got - want).max() <= 2.0 ** -7 * np.abs(want).max() and (got == want).mean() > 0.97


def test_a_block_scale_that_is_no_power_of_two_is_not_multiplied_silently(ops):
    from dew_amd import formats, projections

    depth, width = 256, 256
    rng = np.random.default_rng(3)
    x = torch.from_numpy(rng.standard_normal((40, depth)).astype(np.float32)).to(torch.bfloat16)
    bank = projections.blocks_quantized(torch.from_numpy(weights_case(1, depth, width, seed=5)))
    scales = bank.scale_inv.clone()
    scales[0, 1, 1] *= 1.5                              # a checkpoint's fp32 block scale, not the recipe's
    spoiled = formats.Fp8Blocks(bank.codes, scales).to("cuda")
    got = bf16_np(projections.recipe_projection(x.cuda(), spoiled, torch.tensor([40], dtype=torch.int32).cuda()))
    assert np.isnan(got[:, 128:]).all() and np.isfinite(got[:, :128]).all()


# ---- the MXFP8 recipe -----------------------------------------------------------------------------------------


@pytest.mark.parametrize("rows,depth", [(7, 128), (33, 384), (260, 4096)])
def test_mxfp8_rows_are_quantized_bit_for_bit(ops, rows, depth):
    x = rows_case(rows, depth, seed=rows + 1)
    codes, scales = ops.quantize_rows_mxfp8(x.cuda())
    want_values, want_scales = oracle.mxfp8_quantized(bf16_np(x))
    assert np.array_equal(scales.cpu().numpy(), want_scales)
    assert np.array_equal(ops.depth_order_fp8(codes).cpu().numpy(), oracle.e4m3_bytes(want_values))


@pytest.mark.parametrize("label,sizes", SIZES, ids=[s[0] for s in SIZES])
@pytest.mark.parametrize("depth,width", [(256, 128), (1152, 384), (512, 512)])
def test_the_mxfp8_product_matches_the_oracle(ops, label, sizes, depth, width):
    """Every scale differs by row, column and 32-deep block here, so a lane that handed the instruction another
    block's or another row's scale would be off by powers of two."""
    from dew_amd import formats, projections

    groups, rows = len(sizes), int(np.sum(sizes))
    rng = np.random.default_rng(depth + rows + 1)
    spread = np.exp2(rng.integers(-6, 7, size=(rows + 6, depth // 32))).repeat(32, axis=1)
    x = torch.from_numpy((rng.standard_normal((rows + 6, depth)) * spread).astype(np.float32)).to(torch.bfloat16)
    w = weights_case(groups, depth, width, seed=depth + 1) * np.exp2(rng.integers(-4, 5, size=(groups, depth // 32, width))).repeat(32, axis=1)
    w = w.astype(np.float32)
    bias = torch.from_numpy(rng.standard_normal((groups, width)).astype(np.float32) * 0.1)
    sizes_device = torch.tensor(sizes, dtype=torch.int32).cuda()
    bank = formats.MxFp8.quantized(torch.from_numpy(w)).to("cuda")
    quantized = projections.mxfp8_rows(x.cuda())
    for with_bias in (None, bias):
        got = bf16_np(projections.mxfp8_product(quantized, bank, sizes_device, bias=None if with_bias is None else with_bias.cuda()))
        want = oracle.mxfp8_projection(bf16_np(x), w, sizes, bias=None if with_bias is None else with_bias.numpy())
        assert np.all(got[rows:] == 0) and np.all(want[rows:] == 0)
        scale = np.abs(want).max()
        assert np.abs(got - want).max() <= 2.0 ** -7 * scale
        assert (got == want).mean() > 0.97


def test_mxfp8_gathered_rows_scattered_outputs_and_whole_blocks(ops):
    from dew_amd import formats, projections

    sizes, depth, width = [200, 56, 300], 512, 256
    rows = sum(sizes)
    rng = np.random.default_rng(19)
    x = torch.from_numpy(rng.standard_normal((400, depth)).astype(np.float32)).to(torch.bfloat16)
    gather = rng.integers(0, 400, size=rows).astype(np.int32)
    scatter = rng.permutation(rows).astype(np.int32)
    w = weights_case(len(sizes), depth, width, seed=14)
    bank = formats.MxFp8.quantized(torch.from_numpy(w)).to("cuda")
    got = bf16_np(projections.mxfp8_product(projections.mxfp8_rows(x.cuda()), bank, torch.tensor(sizes, dtype=torch.int32).cuda(),
                                            gather=torch.from_numpy(gather).cuda(), scatter=torch.from_numpy(scatter).cuda()))
    want = oracle.mxfp8_projection(bf16_np(x)[gather], w, sizes)
    placed = np.zeros_like(want)
    placed[scatter] = want
    assert np.abs(got - placed).max() <= 2.0 ** -7 * np.abs(want).max() and (got == placed).mean() > 0.97
    blocks = [2, 0, 1]
    x = torch.from_numpy(rng.standard_normal((384, depth)).astype(np.float32)).to(torch.bfloat16)
    got = bf16_np(projections.mxfp8_projection(x.cuda(), torch.from_numpy(w).cuda(), blocks))
    want = oracle.mxfp8_projection(bf16_np(x), w, [256, 0, 128])
    assert np.abs(got - want).max() <= 2.0 ** -7 * np.abs(want).max() and (got == want).mean() > 0.97


def test_an_mxfp8_bank_is_refused_by_the_bf16_products(ops):
    from dew_amd import formats

    bank = ops.prepare(formats.MxFp8.quantized(torch.from_numpy(weights_case(1, 256, 128, seed=2))).to("cuda"))
    x = torch.zeros((8, 256), dtype=torch.bfloat16).cuda()
    with pytest.raises(Exception, match="MXFP8"):
        ops.grouped_gemm(x, bank, torch.tensor([0, 8], dtype=torch.int32).cuda())


# ---- the NVFP4 recipe -----------------------------------------------------------------------------------------


@pytest.mark.parametrize("rows,depth", [(7, 128), (33, 384), (260, 4096)])
def test_nvfp4_rows_are_quantized_bit_for_bit(ops, rows, depth):
    rng = np.random.default_rng(rows)
    x = (rng.standard_normal((rows, depth)) * rng.choice([1e-3, 0.1, 1.0, 30.0], size=(rows, 1))).astype(np.float32)
    x[0, :16] = 0.0                                   # a zero block: zero codes
    x[1, :16] = np.linspace(-1e-5, 1e-5, 16)          # far under the tensor's largest: the least scales, tiny codes
    x = torch.from_numpy(x).to(torch.bfloat16)
    values, scale = ops.quantize_rows_nvfp4(x.cuda())
    want_values, want_scales, want_tensor = oracle.nvfp4_quantized(bf16_np(x))
    assert scale.item() == want_tensor
    assert np.array_equal(bf16_np(values), want_values * np.repeat(want_scales, 16, axis=1))
    zeros, one = ops.quantize_rows_nvfp4(torch.zeros((3, 64), dtype=torch.bfloat16).cuda())
    assert one.item() == 1.0 and not zeros.any()


@pytest.mark.parametrize("label,sizes", SIZES, ids=[s[0] for s in SIZES])
def test_the_nvfp4_product_matches_the_oracle(ops, label, sizes):
    from dew_amd import projections

    depth, width = 512, 256
    groups, rows = len(sizes), int(np.sum(sizes))
    rng = np.random.default_rng(rows + 3)
    x = torch.from_numpy(rng.standard_normal((rows + 6, depth)).astype(np.float32)).to(torch.bfloat16)
    w = weights_case(groups, depth, width, seed=21)
    bank = projections.nvfp4_matrices(torch.from_numpy(w)).to("cuda")
    got = bf16_np(projections.nvfp4_block_product(projections.nvfp4_rows(x.cuda()), bank, torch.tensor(sizes, dtype=torch.int32).cuda()))
    want = oracle.nvfp4_projection(bf16_np(x), w, sizes)
    assert np.all(got[rows:] == 0) and np.all(want[rows:] == 0)
    scale = np.abs(want).max()
    assert np.abs(got - want).max() <= 2.0 ** -7 * scale and (got == want).mean() > 0.97


@pytest.mark.parametrize("recipe", ["mxfp8", "nvfp4"])
@pytest.mark.parametrize("label,sizes", SIZES, ids=[s[0] for s in SIZES])
def test_recipe_projection_takes_every_recipe_with_ragged_groups_and_a_bias(ops, recipe, label, sizes):
    """`recipe_projection` from the weights themselves: ragged groups as they are (the reference pads them with zero
    rows, which change nothing), rows past the groups zero, the bias on the fp32 sums; and a dense projection's one
    group."""
    from dew_amd import projections

    depth, width = 512, 256
    groups, rows = len(sizes), int(np.sum(sizes))
    rng = np.random.default_rng(rows + len(recipe))
    x = torch.from_numpy(rng.standard_normal((rows + 6, depth)).astype(np.float32)).to(torch.bfloat16)
    w = weights_case(groups, depth, width, seed=31)
    bias = torch.from_numpy(rng.standard_normal((groups, width)).astype(np.float32) * 0.1)
    sizes_device = torch.tensor(sizes, dtype=torch.int32).cuda()
    truth = oracle.mxfp8_projection if recipe == "mxfp8" else oracle.nvfp4_projection
    for with_bias in (None, bias):
        got = bf16_np(projections.recipe_projection(x.cuda(), torch.from_numpy(w).cuda(), sizes_device, recipe=recipe,
                                                    bias=None if with_bias is None else with_bias.cuda()))
        want = truth(bf16_np(x), w, sizes, bias=None if with_bias is None else with_bias.numpy())
        assert np.all(got[rows:] == 0) and np.all(want[rows:] == 0)
        assert np.abs(got - want).max() <= 2.0 ** -7 * np.abs(want).max() and (got == want).mean() > 0.97
    dense = bf16_np(projections.recipe_projection(x.cuda(), torch.from_numpy(w[0]).cuda(), recipe=recipe))
    want = truth(bf16_np(x), w[:1], [rows + 6])
    assert np.abs(dense - want).max() <= 2.0 ** -7 * np.abs(want).max() and (dense == want).mean() > 0.97
    assert projections.recipe_projection(x.cuda(), torch.zeros((192, 128), device="cuda"), recipe=recipe) is None
    with pytest.raises(ValueError):
        projections.recipe_projection(x.cuda(), torch.from_numpy(w).cuda(), sizes_device, recipe="int8")


def test_the_nvfp4_quantizers_choose_the_oracles_codes_over_millions_of_elements(ops):
    """The device compares x / tensor with (threshold x block scale) where the oracle, as the reference, rounds
    (x / tensor) / scale and compares with the threshold: the same choice for every element (rows over 17 binades of
    scale, so block scales and quotients of every size meet), along the depth and along the tokens."""
    rng = np.random.default_rng(12)
    x = (rng.standard_normal((2048, 2048)) * np.exp2(rng.integers(-8, 9, size=(2048, 1)))).astype(np.float32)
    x = torch.from_numpy(x).to(torch.bfloat16)
    for transposed in (False, True):
        source = bf16_np(x).T if transposed else bf16_np(x)
        values, scales, tensor = oracle.nvfp4_quantized(source)
        want = values * np.repeat(scales, 16, axis=1)
        got, scale = ops.transpose_columns(x.cuda(), nvfp4=True, as_bank=False) if transposed else ops.quantize_rows_nvfp4(x.cuda())
        assert scale.item() == tensor and np.array_equal(bf16_np(got), want)

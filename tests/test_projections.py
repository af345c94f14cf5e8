"""The blockwise FP8 recipe on the CPU: what pins the oracle's restatement (no byte fixture of the reference covers
it, so each piece is held to what the arithmetic fixes), and the host mirror's weight quantizer against the oracle."""

import pathlib

import numpy as np
import torch

from oracle import moe_oracle as oracle

GOLDEN = pathlib.Path(__file__).parent / "golden"


def test_e4m3_rounding_is_nearest_with_ties_to_the_even_code():
    """Brute force over every grid point, every midpoint between neighbours, and random values: the nearest E4M3FN
    magnitude, a tie going to the even code."""
    magnitudes = oracle.E4M3[:0x7F].astype(np.float64)
    rng = np.random.default_rng(0)
    values = np.concatenate([magnitudes, -magnitudes, (magnitudes[1:] + magnitudes[:-1]) / 2, rng.uniform(-448, 448, 5000),
                             rng.standard_normal(5000) * 0.01, [2.0 ** -10, -2.0 ** -10, 3 * 2.0 ** -10, 447.9, -448.0]]).astype(np.float32)
    got = oracle.e4m3_rounded(values)
    distance = np.abs(magnitudes[None, :] - np.abs(values.astype(np.float64))[:, None])
    best = distance.min(axis=1, keepdims=True)
    tied = distance == best
    index = np.where(tied.sum(axis=1) == 1, tied.argmax(axis=1), (tied & (np.arange(127) % 2 == 0)).argmax(axis=1))
    assert np.array_equal(np.abs(got), magnitudes[index].astype(np.float32))
    assert np.array_equal(np.signbit(got), np.signbit(values))                 # -2^-10 rounds to -0
    assert np.array_equal(oracle.E4M3[oracle.e4m3_bytes(got)], got)


def test_the_scale_is_the_least_power_of_two_at_or_above_amax_over_448():
    assert np.array_equal(oracle.power_of_two_ceil(np.array([1, np.nextafter(np.float32(1), 2), 0.5, 0.75, 3, 4, 2.0 ** -20], np.float32)),
                          np.array([1, 2, 0.5, 1, 4, 4, 2.0 ** -20], np.float32))
    block = np.zeros((6, 128), np.float32)
    block[0, 3] = 448.0                     # 448 * f32(1 / 448) rounds to 1 exactly: scale 1, code 448
    block[1, 3] = 449.0                     # just above: scale 2
    block[2, 3] = 0.875                     # 448 * 2^-9
    block[3, 3] = 1e-5                      # under the floor: the floor's scale, 2^-22 (1e-4 / 448 = 2.2e-7 < 2^-22 = 2.4e-7)
    block[5, 3] = -3.0
    values, scales = oracle.rows_quantized(block)
    assert scales[:, 0].tolist() == [1.0, 2.0, 2.0 ** -9, 2.0 ** -22, 2.0 ** -22, 2.0 ** -7]
    assert values[0, 3] == 448.0 and values[1, 3] == 224.0 and values[2, 3] == 448.0 and values[5, 3] == -384.0
    assert values[3, 3] == oracle.e4m3_rounded(np.float32(1e-5) / np.float32(2.0 ** -22))
    # what a tile stands for is within half a code step of its source, 2^-4 of the tile's largest magnitude at most
    rng = np.random.default_rng(1)
    x = rng.standard_normal((50, 256)).astype(np.float32)
    values, scales = oracle.rows_quantized(x)
    rebuilt = (values.reshape(50, 2, 128) * scales[:, :, None]).reshape(50, 256)
    assert np.abs(rebuilt - x).max() <= 2.0 ** -4 * np.abs(x).max()
    assert np.abs(values).max() <= 448 and (np.abs(values).reshape(50, 2, 128).max(axis=2) >= 224).all()  # the least such scale


def test_the_weight_blocks_agree_with_deepgemms_ue8m0_cast_where_the_rules_coincide():
    """DeepGEMM's ue8m0 cast (the reference's fixture) takes the ceiling power of two of amax / 448, the recipe of
    amax * f32(1 / 448): the same scale unless the two roundings of the quotient straddle a power of two, and then
    the same codes."""
    with np.load(GOLDEN / "codecs" / "deepgemm_fp8.npz") as held:
        for name in ("random/256x384/128",):
            weight = held[f"{name}/weight"]
            values, scales = oracle.blocks_quantized(weight[None])
            assert np.array_equal(scales[0], held[f"{name}/scales/ue8m0"])
            assert np.array_equal(oracle.e4m3_bytes(values[0]), held[f"{name}/codes/ue8m0"])


def test_the_product_scales_each_blocks_partial_before_it_is_added():
    """Against the float64 sum of the dequantized operands (the reference's own truth for this product,
    tests/test_gemm_blockwise.py:20-40): fp32's accuracy, with general (not power-of-two) scales as its test
    draws them; rows past the groups are zero; swapping the two scale operands' roles changes the result."""
    rng = np.random.default_rng(2)
    sizes, depth, width = [40, 0, 25], 384, 256
    rows = sum(sizes) + 3
    lhs = oracle.e4m3_rounded(np.clip(rng.standard_normal((rows, depth)) * 100, -448, 448).astype(np.float32))
    kernel = oracle.e4m3_rounded(np.clip(rng.standard_normal((3, depth, width)) * 100, -448, 448).astype(np.float32))
    row_scales = rng.uniform(0.5, 2.0, size=(depth // 128, rows)).astype(np.float32)
    column_scales = rng.uniform(0.5, 2.0, size=(3, depth // 128, width // 128)).astype(np.float32)
    got = oracle.blockwise_fp8_product(lhs, kernel, sizes, row_scales, column_scales, dtype="float32")
    truth = np.zeros((rows, width))
    start = 0
    for group, size in enumerate(sizes):
        for block in range(depth // 128):
            span = slice(128 * block, 128 * block + 128)
            partial = lhs[start:start + size, span].astype(np.float64) @ kernel[group, span].astype(np.float64)
            truth[start:start + size] += partial * row_scales[block, start:start + size, None] * np.repeat(column_scales[group, block], 128)[None, :]
        start += size
    assert np.all(got[sum(sizes):] == 0)
    assert np.abs(got - truth).max() <= 4 * 2.0 ** -24 * np.abs(truth).max()
    swapped = oracle.blockwise_fp8_product(lhs, kernel, sizes, row_scales[::-1], column_scales, dtype="float32")
    assert np.abs(swapped - truth).max() > 1e-3 * np.abs(truth).max()
    # scaling twice keeps extreme scales in range whichever comes first (src/dew/nn/precision.py:1782-1791)
    assert oracle.twice_scaled(np.float32(2.0 ** 100), np.float32(2.0 ** 100), np.float32(2.0 ** -120)) == np.float32(2.0 ** 80)
    assert oracle.twice_scaled(np.float32(2.0 ** -100), np.float32(2.0 ** -100), np.float32(2.0 ** 120)) == np.float32(2.0 ** -80)


def weights_case(groups, depth, width, seed):
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((groups, depth, width)) * 0.02).astype(np.float32)
    w[0, :128, :128] *= 50.0
    w[-1, -128:, -128:] = 0.0
    return w


def test_the_host_mirror_quantizes_weight_blocks_as_the_oracle_does():
    from dew_amd import projections

    w = weights_case(3, 384, 256, seed=1)
    bank = projections.blocks_quantized(torch.from_numpy(w))
    want_values, want_scales = oracle.blocks_quantized(w)
    assert np.array_equal(bank.scale_inv.numpy(), want_scales)
    assert np.array_equal(bank.codes.numpy(), oracle.e4m3_bytes(want_values))


def test_shapes_without_whole_blocks_are_left_to_the_caller():
    from dew_amd import projections

    assert projections.recipe_projection(torch.zeros((4, 192), dtype=torch.bfloat16), torch.zeros((192, 128))) is None


def test_mxfp8_quantizes_by_the_ocp_rule():
    """A block's largest magnitude over its scale lies in [256, 512), so its code is 256 .. 448 (448 .. 512 saturates);
    the scale byte is that magnitude's fp32 exponent field less 8; zeros and magnitudes under 2^-119 take byte 0."""
    rng = np.random.default_rng(7)
    x = (rng.standard_normal((64, 256)) * rng.choice([1e-4, 1.0, 3e4], size=(64, 1))).astype(np.float32)
    x[0, :32] = 0.0
    x[1, :32] = np.float32(2.0 ** -130)
    x[2, :32] = 0.0
    x[2, 5] = 511.0                                   # 511 / 2 = 255.5 -> code 256; under its own scale 2^0 it would saturate
    x[3, :32] = 0.0
    x[3, 7] = -480.0                                  # scale 2^0: -480 saturates to -448
    values, scales = oracle.mxfp8_quantized(x)
    top = np.abs(values).reshape(64, 8, 32).max(axis=2)
    nonzero = np.abs(x).reshape(64, 8, 32).max(axis=2) >= 2.0 ** -118
    assert ((top >= 256) & (top <= 448))[nonzero].all()
    field = (np.abs(x).reshape(64, 8, 32).max(axis=2).astype(np.float32).view(np.uint32) >> 23).astype(np.int32)
    assert np.array_equal(scales, np.clip(field - 8, 0, 254).astype(np.uint8))
    assert scales[0, 0] == 0 and values[0, :32].max() == 0 and scales[1, 0] == 0 and values[1, 0] == 0.125
    assert scales[2, 0] == 127 and values[2, 5] == 448.0 and scales[3, 0] == 127 and values[3, 7] == -448.0
    decoded = oracle.mxfp8_decoded(values, scales)
    unsaturated = np.abs(values) < 448
    assert (np.abs(decoded - x)[unsaturated] <= np.repeat(np.ldexp(1.0, scales.astype(np.int32) - 127 + 4), 32, axis=1)[unsaturated]).all()


def test_the_host_mirror_quantizes_an_mxfp8_bank_as_the_oracle_does():
    from dew_amd import formats

    w = weights_case(2, 256, 128, seed=3)
    bank = formats.MxFp8.quantized(torch.from_numpy(w))
    want_values, want_scales = oracle.mxfp8_quantized(np.swapaxes(w, 1, 2))
    assert bank.shape == (2, 256, 128)
    assert np.array_equal(bank.scales.numpy(), want_scales)
    assert np.array_equal(bank.codes.numpy(), oracle.e4m3_bytes(want_values))


def test_the_nvfp4_operand_follows_the_bank_quantizers_closed_form():
    """The recipe's operand rule is the bank quantizer's (tests/test_codecs.py pins that one against the reference's own
    statement); here the oracle's restatement against it, the zero block, and the decoded operand within half a code
    step of its source."""
    from dew_amd import codecs

    rng = np.random.default_rng(11)
    x = (rng.standard_normal((40, 256)) * rng.choice([0.01, 1.0, 50.0], size=(40, 1))).astype(np.float32)
    x[3, 16:32] = 0.0
    values, scales, tensor = oracle.nvfp4_quantized(x)
    codes, held, scale = codecs.nvfp4_coded(torch.from_numpy(x.T.copy()))
    assert tensor == scale.item() == np.float32(np.abs(x).max()) / np.float32(6 * 448)
    assert np.array_equal(oracle.E4M3[held.numpy()].T, scales) and np.array_equal(oracle.E2M1[codes.numpy()].T, values)
    assert not values[3, 16:32].any() and np.abs(values).max() <= 6
    decoded = values * np.repeat(scales, 16, axis=1) * tensor
    assert (np.abs(decoded - x) <= 0.5 * np.repeat(scales, 16, axis=1) * tensor * 2.0 + 1e-30).all()   # the widest step is 2
    assert oracle.nvfp4_quantized(np.zeros((2, 32), np.float32))[2] == 1.0


def test_rows_as_two_e2m3_terms_keep_what_their_bound_says():
    """`split_rows_e2m3_pair` (the oracle of `dew_moe_split_rows_e2m3_pair`; no counterpart in the reference) by what its
    definition fixes: every element within two binades of its 32-deep block's largest magnitude is held exactly (four
    significant bits in each term), any other within 2^-10 of that magnitude; each term lies within e2m3's range under its
    scale; a block of three binades is exact; a zero block holds zeros under the least scale."""
    from oracle import moe_oracle as oracle

    rng = np.random.default_rng(2)
    x = oracle.bf16_round(rng.standard_normal((40, 256)).astype(np.float32) * 10.0 ** rng.uniform(-3, 3, size=(40, 1)).astype(np.float32))
    x[3] = 0.0
    x[4] = oracle.bf16_round((np.exp2(rng.integers(0, 3, size=256)) * (1 + rng.integers(0, 128, size=256) / 128)).astype(np.float32))
    held, scales = oracle.split_rows_e2m3_pair(x)
    blocks, kept = np.abs(x).reshape(40, 8, 32), held.reshape(40, 8, 32)
    largest = blocks.max(axis=-1, keepdims=True)
    binade = np.where(largest > 0, np.exp2(np.floor(np.log2(np.maximum(largest, 1e-45)))), 0.0)
    near = blocks >= binade / 4
    assert near.mean() > 0.6 and np.array_equal(kept[near], x.reshape(40, 8, 32)[near])
    assert (np.abs(kept - x.reshape(40, 8, 32)) <= largest * 2.0 ** -10).all()
    assert np.array_equal(held[4], x[4]) and not held[3].any() and (scales[3] == 1).all()
    first = np.ldexp(np.float32(1), scales[..., 0].astype(np.int32) - 127)[..., None]
    assert (largest <= 7.5 * first).all() and (largest[largest > 0] > 3.75 * first[largest > 0]).all()   # the least such power of two

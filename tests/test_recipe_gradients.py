"""The oracle's restatement of the recipes' gradients (src/dew/nn/kernels/projections.py:211-224, 263-275) pinned on
the CPU: the kernel gradient against the definition the reference's own test writes out block by block
(tests/test_gemm_blockwise.py:97-107) with its operand shapes and scale ranges, and both gradients against the exact
derivative on operands the formats hold exactly (where quantization changes nothing, d_x = dy @ w^T and
d_w[g] = x_g^T @ dy_g to the last bit)."""

import numpy as np

from oracle import moe_oracle as oracle

BLOCKS = (1, 0, 2, 1)   # the reference test's groups: an empty one among them (tests/test_gemm_blockwise.py:66)


def test_the_kernel_gradient_is_the_blocked_sum_the_reference_tests():
    rng = np.random.default_rng(0)
    depth = width = 256
    rows = 128 * sum(BLOCKS)
    lhs_t = oracle.fp8_codes(rng.normal(size=(depth, rows)).astype(np.float32))
    rhs_t = oracle.fp8_codes(rng.normal(size=(width, rows)).astype(np.float32))
    row_scales = rng.uniform(0.5, 2.0, size=(rows // 128, depth)).astype(np.float32)
    column_scales = rng.uniform(0.5, 2.0, size=(rows // 128, width)).astype(np.float32)
    got = oracle.blockwise_fp8_kernel_gradient(lhs_t, rhs_t, BLOCKS, row_scales, column_scales, dtype="float32")
    want = np.zeros((len(BLOCKS), depth, width), np.float64)
    owners = np.repeat(np.arange(len(BLOCKS)), BLOCKS)
    for block, owner in enumerate(owners):
        span = slice(128 * block, 128 * (block + 1))
        partial = lhs_t[:, span].astype(np.float64) @ rhs_t[:, span].astype(np.float64).T
        want[owner] += partial * row_scales[block, :, None] * column_scales[block, None, :]
    assert not got[1].any()
    assert np.abs(got - want).max() <= 2.0 ** -22 * np.abs(want).max()


def _exact_case(seed):
    """Operands every format here holds exactly: small integers times one power of two a 128-block."""
    rng = np.random.default_rng(seed)
    depth, width, tokens = 128, 256, 128 * sum(BLOCKS)
    x = rng.integers(-8, 9, size=(tokens, depth)).astype(np.float32)
    dy = rng.integers(-8, 9, size=(tokens, width)).astype(np.float32) * 0.25
    w = rng.integers(-8, 9, size=(len(BLOCKS), depth, width)).astype(np.float32) * 0.5
    for each in (x, dy):
        each[0, :], each[:, 0] = 8, 8          # every tile's and block's largest magnitude the same power of two
    w[:, 0, :], w[:, :, 0] = 4.0, 4.0
    return x, w, dy


def _exact_gradients(x, w, dy):
    d_x, d_w, start = np.zeros_like(x), np.zeros_like(w), 0
    for group, blocks in enumerate(BLOCKS):
        span = slice(start, start + 128 * blocks)
        d_x[span] = dy[span] @ w[group].T
        d_w[group] = x[span].T @ dy[span]
        start += 128 * blocks
    return d_x, d_w


def test_the_blockwise_fp8_gradients_are_exact_where_the_format_is():
    x, w, dy = _exact_case(1)
    d_x, d_w = oracle.blockwise_fp8_gradients(x, w, dy, BLOCKS, dtype="float32")
    want_x, want_w = _exact_gradients(x, w, dy)
    assert np.array_equal(d_x, want_x) and np.array_equal(d_w, want_w)


def test_the_mxfp8_gradients_are_exact_where_the_format_is():
    x, w, dy = _exact_case(2)
    d_x, d_w = oracle.mxfp8_gradients(x, w, dy, BLOCKS, dtype="float32")
    want_x, want_w = _exact_gradients(x, w, dy)
    assert np.array_equal(d_x, want_x) and np.array_equal(d_w, want_w)


def test_the_nvfp4_gradients_are_exact_where_the_format_is():
    """E2M1 holds {0, .5, 1, 1.5, 2, 3, 4, 6}: operands drawn from them with every operand's largest magnitude 6 (the
    tensor scale is then 1 / 448 and every block scale 448 or, for blocks whose largest is 3, 224)."""
    rng = np.random.default_rng(3)
    grid = np.array([0, 0.5, 1, 1.5, 2, 3, 4, 6, -0.5, -1, -1.5, -2, -3, -4, -6], np.float32)
    depth, width, tokens = 128, 256, 128 * sum(BLOCKS)
    x, dy = rng.choice(grid, size=(tokens, depth)), rng.choice(grid, size=(tokens, width))
    w = rng.choice(grid, size=(len(BLOCKS), depth, width))
    for each in (x, dy):
        each[::16, :], each[:, ::16] = 6.0, 6.0     # every block of 16, along either axis, holds a 6
    w[:, ::16, :], w[:, :, ::16] = 6.0, 6.0
    d_x, d_w = oracle.nvfp4_gradients(x, w, dy, BLOCKS, dtype="float32")
    want_x, want_w = _exact_gradients(x, w, dy)
    assert np.abs(d_x - want_x).max() <= 2.0 ** -21 * np.abs(want_x).max()      # (448 x 1 / 448 rounds in fp32)
    assert np.abs(d_w - want_w).max() <= 2.0 ** -21 * np.abs(want_w).max()

"""The recipes' gradients on the device against the CPU oracle: the quantizer along the tokens bit for bit in both of
its layouts (codes and scales are byte work); the kernel gradient within 2^-13 of the largest output where it is
written in fp32 and within one bf16 ulp of it in bf16; the input's gradient through the forward's own kernels.
Kernel and oracle multiply the same codes exactly and differ in the fp32 sums alone: the oracle's are exact, the
matrix instruction's align each 64-deep dot's products to the largest of them before adding (measured: 2^-15 of the
largest output on operands whose blocks span 2^10 in magnitude, 2^-19 of an element's summed magnitudes on unit-range
ones, where fp32 additions in order reach 2^-23 and 2^-26)."""

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


def tokens_case(tokens, dim, seed):
    """Activations whose scale differs by token block and column, with the quantizers' corner tiles among them."""
    rng = np.random.default_rng(seed)
    spread = np.exp2(rng.integers(-5, 6, size=(tokens // 32, dim))).repeat(32, axis=0)
    x = (rng.standard_normal((tokens, dim)) * spread).astype(np.float32)
    x[:128, 0] = 0.0                                    # an all-zero tile: the 1e-4 floor (FP8), the least scale (MX)
    x[:128, 1] = np.linspace(-1e-5, 1e-5, 128)          # under the floor
    x[:128, 2] = np.clip(x[:128, 2], -448.0, 448.0)
    x[77, 2] = -448.0                                   # amax = 448 exactly
    x[-128:, 3] *= 1e30                                 # a huge tile
    return torch.from_numpy(x).to(torch.bfloat16)


def bank_codes(bank, tokens, dim):
    """A `quantize_columns(as_bank=True)` bank's (codes `[dim, tokens]` in token order, scales `[dim, tokens / 32]`)."""
    buffer = bank.keep[0].cpu()
    codes = buffer[:tokens * dim].view(dim // 32, tokens // 32, 2, 32, 16).permute(0, 3, 1, 2, 4).reshape(dim, tokens)
    scales = buffer[tokens * dim:tokens * dim + tokens // 32 * dim].view(dim // 32, tokens // 128, 32, 4).permute(0, 2, 1, 3)
    return codes.numpy(), scales.reshape(dim, tokens // 32).numpy()


@pytest.mark.parametrize("tokens,dim", [(128, 128), (384, 256), (1024, 640)])
@pytest.mark.parametrize("mx", [False, True], ids=["fp8", "mxfp8"])
def test_tokens_are_quantized_bit_for_bit_in_both_layouts(ops, tokens, dim, mx):
    x = tokens_case(tokens, dim, seed=tokens + dim)
    if mx:
        want_values, want_scales = oracle.mxfp8_quantized(bf16_np(x).T)
    else:
        want_values, scales = oracle.rows_quantized(bf16_np(x).T)
        want_scales = (np.frexp(scales)[1] - 1 + 127).astype(np.uint8).repeat(4, axis=1)      # each tile's byte for its four 32s
    want_codes = oracle.e4m3_bytes(want_values)
    codes, scales = ops.quantize_columns(x.cuda(), mx=mx, as_bank=False)
    assert np.array_equal(scales.cpu().numpy(), want_scales)
    assert np.array_equal(ops.depth_order_fp8(codes).cpu().numpy(), want_codes)
    got_codes, got_scales = bank_codes(ops.quantize_columns(x.cuda(), mx=mx, as_bank=True), tokens, dim)
    assert np.array_equal(got_scales, want_scales)
    assert np.array_equal(got_codes, want_codes)


GROUPS = [("reference", (1, 0, 2, 1)), ("single", (3,)), ("ragged", (5, 1, 0, 0, 2))]


@pytest.mark.parametrize("label,blocks", GROUPS, ids=[g[0] for g in GROUPS])
@pytest.mark.parametrize("depth,width", [(256, 256), (384, 384), (128, 512)])
@pytest.mark.parametrize("mx", [False, True], ids=["fp8", "mxfp8"])
def test_the_kernel_gradient_matches_the_oracle(ops, label, blocks, depth, width, mx):
    from dew_amd import projections

    tokens = 128 * sum(blocks)
    x = tokens_case(tokens, depth, seed=depth + tokens)
    dy = tokens_case(tokens, width, seed=width + tokens + 1)
    x[-128:, 3] = 1.0
    dy[-128:, 3] = 1.0                                  # (the huge tiles' products would overflow fp32)
    w = np.zeros((len(blocks), depth, width), np.float32)
    gradients = oracle.mxfp8_gradients if mx else oracle.blockwise_fp8_gradients
    _, want = gradients(bf16_np(x), w, bf16_np(dy), blocks, dtype="float32")
    scale = np.abs(want).max()
    got = projections.kernel_gradient(x.cuda(), dy.cuda(), blocks, mx=mx, out_dtype=torch.float32).cpu().numpy()
    for group, count in enumerate(blocks):
        if count == 0:
            assert not got[group].any()
    assert np.abs(got - want).max() <= 2.0 ** -13 * scale
    rounded = bf16_np(projections.kernel_gradient(x.cuda(), dy.cuda(), blocks, mx=mx))
    assert np.abs(rounded - oracle.bf16_round(want)).max() <= 2.0 ** -7 * scale
    assert (rounded == oracle.bf16_round(want)).mean() > 0.95


@pytest.mark.parametrize("mx", [False, True], ids=["fp8", "mxfp8"])
def test_the_input_gradient_is_the_recipes_own_product(ops, mx):
    from dew_amd import projections

    blocks, depth, width = (1, 0, 2, 1), 256, 384
    tokens = 128 * sum(blocks)
    rng = np.random.default_rng(5)
    x = torch.from_numpy(rng.standard_normal((tokens, depth)).astype(np.float32)).to(torch.bfloat16)
    dy = torch.from_numpy(rng.standard_normal((tokens, width)).astype(np.float32)).to(torch.bfloat16)
    w = torch.from_numpy((rng.standard_normal((len(blocks), depth, width)) * 0.05).astype(np.float32)).to(torch.bfloat16)
    gradients = oracle.mxfp8_gradients if mx else oracle.blockwise_fp8_gradients
    want_x, want_w = gradients(bf16_np(x), bf16_np(w), bf16_np(dy), blocks)
    mirror = projections.mxfp8_gradients if mx else projections.blockwise_fp8_gradients
    d_x, d_w = mirror(x.cuda(), w.cuda(), dy.cuda(), blocks)
    assert d_x.shape == x.shape and d_w.shape == w.shape
    assert np.abs(bf16_np(d_x) - want_x).max() <= 2.0 ** -7 * np.abs(want_x).max()
    assert np.abs(bf16_np(d_w) - want_w).max() <= 2.0 ** -7 * np.abs(want_w).max()
    assert (bf16_np(d_x) == want_x).mean() > 0.97 and (bf16_np(d_w) == want_w).mean() > 0.97


# ---- bf16 operands: the reference's gemm_t, and the NVFP4 recipe's kernel gradient ------------------------------


def bf16_bank_rows(bank, tokens, dim):
    """A `transpose_columns(as_bank=True)` bank's matrix `[dim, tokens]`."""
    atoms = bank.keep[0][:tokens * dim].cpu().view(dim // 32, tokens // 16, 2, 32, 8)
    return atoms.permute(0, 3, 1, 2, 4).reshape(dim, tokens)


@pytest.mark.parametrize("tokens,dim", [(128, 128), (384, 256), (1024, 640)])
def test_tokens_are_transposed_bit_for_bit_in_both_layouts(ops, tokens, dim):
    x = tokens_case(tokens, dim, seed=tokens + dim + 3)
    rows, none = ops.transpose_columns(x.cuda(), as_bank=False)
    assert none is None and torch.equal(rows.cpu(), x.T)
    bank, _ = ops.transpose_columns(x.cuda(), as_bank=True)
    assert torch.equal(bf16_bank_rows(bank, tokens, dim), x.T)
    # the NVFP4 values along the tokens: the oracle's quantizer on the transpose
    want_values, want_scales, want_tensor = oracle.nvfp4_quantized(bf16_np(x).T)
    want = want_values * np.repeat(want_scales, 16, axis=1)
    rows, scale = ops.transpose_columns(x.cuda(), nvfp4=True, as_bank=False)
    assert scale.item() == want_tensor and np.array_equal(bf16_np(rows), want)
    bank, scale = ops.transpose_columns(x.cuda(), nvfp4=True, as_bank=True)
    assert scale.item() == want_tensor and np.array_equal(bf16_np(bf16_bank_rows(bank, tokens, dim)), want)


@pytest.mark.parametrize("label,blocks", GROUPS, ids=[g[0] for g in GROUPS])
@pytest.mark.parametrize("depth,width", [(256, 256), (384, 384), (128, 512)])
def test_gemm_t_matches_the_oracle(ops, label, blocks, depth, width):
    from dew_amd import gemm

    tokens = 128 * sum(blocks)
    rng = np.random.default_rng(depth + tokens)
    x = torch.from_numpy(rng.standard_normal((tokens, depth)).astype(np.float32)).to(torch.bfloat16)
    dy = torch.from_numpy(rng.standard_normal((tokens, width)).astype(np.float32)).to(torch.bfloat16)
    sizes = np.asarray(blocks) * 128
    want = oracle.kernel_gradient(bf16_np(x).T, bf16_np(dy).T, sizes, dtype="float32")
    scale = np.abs(want).max()
    device_sizes = torch.tensor(sizes, dtype=torch.int32).cuda()
    got = gemm.gemm_t(x.cuda(), dy.cuda(), device_sizes, out_dtype=torch.float32).cpu().numpy()
    for group, count in enumerate(blocks):
        if count == 0:
            assert not got[group].any()
    assert np.abs(got - want).max() <= 2.0 ** -18 * scale
    rounded = bf16_np(gemm.gemm_t(x.cuda(), dy.cuda(), device_sizes))
    assert np.abs(rounded - oracle.bf16_round(want)).max() <= 2.0 ** -7 * scale
    assert (rounded == oracle.bf16_round(want)).mean() > 0.99


RAGGED = [("ragged", [130, 0, 1, 257, 64, 0, 127, 5]), ("single", [3]), ("steps", [64, 192, 0, 128]), ("tail", [100, 30])]


@pytest.mark.parametrize("label,sizes", RAGGED, ids=[r[0] for r in RAGGED])
def test_gemm_t_takes_groups_of_any_sizes(ops, label, sizes):
    """Each group padded to whole 64-token steps by the transposer: every boundary inside a step, empty groups, rows
    past the last group (which belong to no group and add nothing), and the same groups as whole steps."""
    from dew_amd import gemm

    sizes = np.asarray(sizes)
    rows = int(sizes.sum()) + 9                         # nine rows no group owns
    rng = np.random.default_rng(rows)
    x = torch.from_numpy(rng.standard_normal((rows, 128)).astype(np.float32)).to(torch.bfloat16)
    dy = torch.from_numpy(rng.standard_normal((rows, 256)).astype(np.float32)).to(torch.bfloat16)
    want = oracle.kernel_gradient(bf16_np(x).T, bf16_np(dy).T, sizes, dtype="float32")
    device_sizes = torch.tensor(sizes, dtype=torch.int32).cuda()
    got = gemm.gemm_t(x.cuda(), dy.cuda(), device_sizes, out_dtype=torch.float32).cpu().numpy()
    assert np.abs(got - want).max() <= 2.0 ** -18 * np.abs(want).max()
    for group, size in enumerate(sizes):
        if size == 0:
            assert not got[group].any()
    rows_t, padded = ops.transpose_groups(x.cuda(), torch.tensor(np.concatenate([[0], np.cumsum(sizes)]), dtype=torch.int32).cuda(), as_bank=False)
    starts = np.concatenate([[0], np.cumsum((sizes + 63) // 64 * 64)])
    assert padded.cpu().tolist() == starts.tolist()
    held = bf16_np(rows_t)
    for group, size in enumerate(sizes):
        first = int(np.sum(sizes[:group]))
        assert np.array_equal(held[:, starts[group]:starts[group] + size], bf16_np(x)[first:first + size].T)
        assert not held[:, starts[group] + size:starts[group + 1]].any()
    assert not held[:, starts[-1]:].any()
    if label == "steps":
        whole = gemm.gemm_t(x[:384].cuda(), dy[:384].cuda(), device_sizes, out_dtype=torch.float32, whole_steps=True).cpu().numpy()
        assert np.array_equal(whole, got)


def test_the_nvfp4_gradients_match_the_oracle(ops):
    from dew_amd import projections

    blocks, depth, width = (1, 0, 2, 1), 256, 512        # (an NVFP4 bank's depth, here also the width, is whole 256s)
    tokens = 128 * sum(blocks)
    rng = np.random.default_rng(6)
    x = torch.from_numpy(rng.standard_normal((tokens, depth)).astype(np.float32)).to(torch.bfloat16)
    dy = torch.from_numpy(rng.standard_normal((tokens, width)).astype(np.float32)).to(torch.bfloat16)
    w = torch.from_numpy((rng.standard_normal((len(blocks), depth, width)) * 0.05).astype(np.float32)).to(torch.bfloat16)
    want_x, want_w = oracle.nvfp4_gradients(bf16_np(x), bf16_np(w), bf16_np(dy), blocks)
    d_x, d_w = projections.nvfp4_gradients(x.cuda(), w.cuda(), dy.cuda(), blocks)
    assert d_x.shape == x.shape and d_w.shape == w.shape
    assert np.abs(bf16_np(d_x) - want_x).max() <= 2.0 ** -7 * np.abs(want_x).max()
    assert np.abs(bf16_np(d_w) - want_w).max() <= 2.0 ** -7 * np.abs(want_w).max()
    assert (bf16_np(d_x) == want_x).mean() > 0.97 and (bf16_np(d_w) == want_w).mean() > 0.97
    wide = projections.nvfp4_gradients(x.cuda(), w.cuda(), dy.cuda(), blocks, out_dtype=torch.float32)[1].cpu().numpy()
    exact = oracle.nvfp4_gradients(bf16_np(x), bf16_np(w), bf16_np(dy), blocks, dtype="float32")[1]
    assert np.abs(wide - exact).max() <= 2.0 ** -18 * np.abs(exact).max()


def test_the_gradients_entry_points_refuse_what_they_cannot_run(ops):
    from dew_amd._lib import KernelError

    odd = torch.zeros((100, 128), dtype=torch.bfloat16, device="cuda")
    whole = torch.zeros((128, 128), dtype=torch.bfloat16, device="cuda")
    narrow = torch.zeros((128, 64), dtype=torch.bfloat16, device="cuda")
    offsets = torch.tensor([0, 128], dtype=torch.int32, device="cuda")
    for call in (lambda x: ops.quantize_columns(x, mx=False, as_bank=False), lambda x: ops.quantize_columns(x, mx=True, as_bank=True),
                 lambda x: ops.transpose_columns(x, as_bank=False), lambda x: ops.transpose_columns(x, nvfp4=True, as_bank=True)):
        with pytest.raises(KernelError, match="whole 128"):
            call(odd)                                   # tokens in whole 128s (ragged groups go through transpose_groups)
        with pytest.raises(KernelError, match="whole 128"):
            call(narrow)                                # columns in whole 128s
        with pytest.raises(KernelError, match="GPU"):
            call(whole.cpu())
    codes, scales = ops.quantize_columns(whole, mx=True, as_bank=False)
    fp8_bank, (bf16_bank, _) = ops.quantize_columns(whole, mx=True, as_bank=True), ops.transpose_columns(whole, as_bank=True)
    with pytest.raises(KernelError, match="MXFP8"):
        ops._lib.check(ops._lib.library().dew_moe_kernel_gradient_mxfp8(codes.data_ptr(), scales.data_ptr(), bf16_bank.descriptor, offsets.data_ptr(),
                                                                        whole.data_ptr(), 0, 128, 1, None), "dew_moe_kernel_gradient_mxfp8")
    with pytest.raises(KernelError, match="bf16"):
        ops.kernel_gradient_bf16(whole, fp8_bank, offsets)
    with pytest.raises(KernelError, match="float32"):
        ops.kernel_gradient_mxfp8(codes, scales, fp8_bank, offsets, out_dtype=torch.float16)
    # an operand of no tokens: nothing to contract, every group's gradient zero
    none = torch.zeros((0, 128), dtype=torch.bfloat16, device="cuda")
    rows_t, _ = ops.transpose_columns(none, as_bank=False)
    empty_bank, _ = ops.transpose_columns(none, as_bank=True)
    zero = ops.kernel_gradient_bf16(rows_t, empty_bank, torch.zeros(3, dtype=torch.int32, device="cuda"), out_dtype=torch.float32)
    assert zero.shape == (2, 128, 128) and not zero.any()


@pytest.mark.parametrize("kind", ["mxfp8", "bf16"])
def test_kernel_gradients_over_more_groups_than_a_block_has_threads(ops, kind):
    """300 groups of 0 .. 2 blocks each (the tile search scans the groups 256 at a time; the padded transposer scans
    them in runs): every group's gradient against the oracle's, the empty ones zero."""
    from dew_amd import gemm, projections

    rng = np.random.default_rng(300)
    blocks = rng.integers(0, 3, size=300)
    depth, width, tokens = 128, 256, 128 * int(blocks.sum())
    x = torch.from_numpy(rng.standard_normal((tokens, depth)).astype(np.float32)).to(torch.bfloat16)
    dy = torch.from_numpy(rng.standard_normal((tokens, width)).astype(np.float32)).to(torch.bfloat16)
    if kind == "mxfp8":
        want = oracle.mxfp8_gradients(bf16_np(x), np.zeros((300, depth, width), np.float32), bf16_np(dy), blocks, dtype="float32")[1]
        got = projections.kernel_gradient(x.cuda(), dy.cuda(), blocks, mx=True, out_dtype=torch.float32).cpu().numpy()
        bar = 2.0 ** -13
    else:
        want = oracle.kernel_gradient(bf16_np(x).T, bf16_np(dy).T, blocks * 128, dtype="float32")
        got = gemm.gemm_t(x.cuda(), dy.cuda(), torch.tensor(blocks * 128, dtype=torch.int32).cuda(), out_dtype=torch.float32).cpu().numpy()
        bar = 2.0 ** -18
    assert np.abs(got - want).max() <= bar * np.abs(want).max()
    assert not got[blocks == 0].any()

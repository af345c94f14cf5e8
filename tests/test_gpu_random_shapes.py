"""Seeded random grouped products against the oracle: formats, depths, widths, group-size distributions (empty and
one-row groups included), gathers, scatters, biases and every tile height, each case small enough for the CPU oracle."""

import numpy as np
import pytest
import torch
from bench_aids.workloads import quantize
from oracle.banks import dequantized

from oracle import moe_oracle as oracle

pytestmark = pytest.mark.gpu

FORMATS = ("fp8_channel", "fp8_block", "mxfp4", "nvfp4")


def drawn(seed):
    rng = np.random.default_rng(1000 + seed)
    quant = FORMATS[seed % 4]
    fp4 = quant in ("mxfp4", "nvfp4")
    experts = int(rng.integers(1, 24))
    depth = int(rng.integers(1, 5)) * (256 if fp4 else 128)
    width = int(rng.integers(1, 5)) * 128
    kind = seed % 5
    if kind == 0:
        sizes = rng.integers(0, 6, size=experts)                     # decode-like
    elif kind == 1:
        sizes = rng.integers(20, 90, size=experts)
    elif kind == 2:
        sizes = (rng.integers(0, 2, size=experts) * rng.integers(1, 300, size=experts))   # many idle experts
    elif kind == 3:
        sizes = rng.integers(100, 400, size=experts)
    else:
        sizes = np.zeros(experts, np.int64)
        sizes[rng.integers(0, experts)] = int(rng.integers(1, 1200))  # one busy expert
    tile = (0, 32, 64, 128, 256)[int(rng.integers(0, 5))]
    return rng, quant, experts, depth, width, [int(v) for v in sizes], tile


@pytest.mark.parametrize("seed", range(40))
def test_random_grouped_products(seed):
    from dew_amd import ops

    rng, quant, experts, depth, width, sizes, tile = drawn(seed)
    rows = int(np.sum(sizes))
    weight = torch.from_numpy((rng.standard_normal((experts, depth, width)) * 0.05).astype(np.float32))
    bank = quantize(weight, quant)
    pool = max(rows, 1) + int(rng.integers(0, 50))
    x = torch.from_numpy(rng.standard_normal((pool, depth)).astype(np.float32)).to(torch.bfloat16)
    gather = rng.integers(0, pool, size=rows).astype(np.int32)
    padded = rows + int(rng.integers(0, 40))                       # sorted positions past the last group: zero rows
    scatter = rng.permutation(padded).astype(np.int32)
    bias = torch.from_numpy(rng.standard_normal((experts, width)).astype(np.float32)).to(torch.bfloat16).float()
    offsets = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int32)
    values, factor = dequantized(bank)
    want = oracle._biased_matmul(x.float().numpy()[gather], values, sizes, bias.numpy(), dtype="bfloat16", factor=factor)
    prepared = ops.prepare(bank.to("cuda"))
    full_gather = np.concatenate([gather, np.zeros(padded - rows, np.int32)])
    with ops.tile_rows(tile):
        got = ops.grouped_gemm(x.cuda(), prepared, torch.from_numpy(offsets).cuda(), gather=torch.from_numpy(full_gather).cuda(),
                               scatter=torch.from_numpy(scatter).cuda(), bias=bias.cuda(), rows=padded)
    got = got.float().cpu().numpy()[scatter]
    assert np.all(got[rows:] == 0)
    if rows:
        scale = max(np.abs(want).max(), 1e-6)
        # one bf16 ulp at the largest magnitude is at most 2^-7 of it
        assert np.abs(got[:rows] - want).max() <= 2 ** -7 * scale, (quant, experts, depth, width, sizes, tile)
        assert (got[:rows] == want).mean() > 0.97


@pytest.mark.parametrize("seed", range(40, 60))
def test_random_gate_up_products(seed):
    from dew_amd import ops

    rng, quant, experts, depth, width, sizes, tile = drawn(seed)
    rows = int(np.sum(sizes))
    if rows == 0:
        sizes[0], rows = 3, 3
    gate = quantize(torch.from_numpy((rng.standard_normal((experts, depth, width)) * 0.05).astype(np.float32)), quant)
    up = quantize(torch.from_numpy((rng.standard_normal((experts, depth, width)) * 0.05).astype(np.float32)), quant)
    x = torch.from_numpy(rng.standard_normal((rows, depth)).astype(np.float32)).to(torch.bfloat16)
    offsets = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int32)
    gate_values, gate_factor = dequantized(gate)
    up_values, up_factor = dequantized(up)
    rows_np = x.float().numpy()
    want = oracle.swiglu(oracle.grouped_matmul(rows_np, gate_values, sizes, factor=gate_factor),
                         oracle.grouped_matmul(rows_np, up_values, sizes, factor=up_factor))
    pg, pu = ops.prepare(gate.to("cuda")), ops.prepare(up.to("cuda"))
    od = torch.from_numpy(offsets).cuda()
    with ops.tile_rows(tile):
        fused = ops.gateup_swiglu(x.cuda(), pg, pu, od)
        apart = ops.swiglu(ops.grouped_gemm(x.cuda(), pg, od), ops.grouped_gemm(x.cuda(), pu, od))
    assert torch.equal(fused, apart)
    fused = fused.float().cpu().numpy()
    scale = max(np.abs(want).max(), 1e-6)
    assert np.abs(fused - want).max() <= 2 ** -6 * scale and (fused == want).mean() > 0.9

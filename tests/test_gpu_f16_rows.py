"""General NVFP4 banks on f16 rows (`dew_moe_rows_f16`, `dew_moe_gateup_gated_f16`): the conversion's exactness, and the
paired launch against the bf16-operand launch, bit for bit (every product is the same exact one times a power of two),
and against the oracle, on every tile height, ragged and empty groups, gathers, the clamp and the GeGLU gate."""

import numpy as np
import pytest
import torch

from bench_aids.workloads import quantize
from oracle import moe_oracle as oracle
from oracle.banks import dequantized

pytestmark = pytest.mark.gpu


def test_rows_as_f16_under_a_scale_a_row_are_the_rows():
    from dew_amd import ops

    rng = np.random.default_rng(5)
    x = rng.standard_normal((300, 512)).astype(np.float32)
    x[1] *= 1e-30            # a row of tiny magnitudes
    x[2] *= 1e30             # a row of huge ones
    x[3] = 0.0               # a zero row
    x[4, :] = 0.0
    x[4, 7] = -3.0           # one element
    x[5, ::2] *= 2.0 ** -20  # twenty binades inside a row: still exact (f16's normal range spans 29 below the largest)
    x[6, 0], x[6, 1] = 1.0, 2.0 ** -45   # past f16's range below the largest: rounded away
    rows = torch.from_numpy(x).to(torch.bfloat16).cuda()
    halves, scale = ops.rows_f16(rows)
    assert halves.dtype == torch.float16 and scale.dtype == torch.uint8
    back = np.ldexp(halves.cpu().numpy().astype(np.float64), scale.cpu().numpy().astype(np.int32)[:, None] - 127)
    wide = rows.double().cpu().numpy()
    most = np.abs(wide).max(axis=1, keepdims=True)
    within = np.abs(wide) >= most * 2.0 ** -29                   # f16's normal range under the row's largest magnitude
    assert np.array_equal(back[within], wide[within])            # exact there
    assert (np.abs(back - wide) <= most * 2.0 ** -40).all()      # and rounded to f16's subnormal step below it
    assert back[6, 0] == 1.0 and within[5].mean() > 0.99 and not within[6, 1]
    largest = halves.abs().amax(dim=1)
    nonzero = rows.abs().amax(dim=1) > 0
    assert bool(((largest[nonzero] >= 2.0 ** 15) & (largest[nonzero] < 2.0 ** 16)).all()) and bool(torch.isfinite(halves).all())


@pytest.mark.parametrize("tile", [0, 32, 64, 128, 256])
@pytest.mark.parametrize("gating", [("swiglu", None), ("geglu", None), ("swiglu", 0.75)])
def test_the_f16_launch_returns_the_bf16_launchs_bits(tile, gating, monkeypatch):
    from dew_amd import ops

    activation, limit = gating
    rng = np.random.default_rng(17 + tile)
    experts, depth, width = 7, 768, 384
    sizes = [0, 150, 1, 333, 64, 0, 97]
    rows = sum(sizes)
    gate, up = (quantize(torch.from_numpy((rng.standard_normal((experts, depth, width)) * 0.05).astype(np.float32)), "nvfp4") for _ in range(2))
    pool = rows + 31
    x = rng.standard_normal((pool, depth)).astype(np.float32)
    x[::5] *= 37.0           # rows of different magnitudes: the scales differ by row
    x[3::7] *= 2.0 ** -12
    x = torch.from_numpy(x).to(torch.bfloat16)
    gather = rng.integers(0, pool, size=rows).astype(np.int32)
    padded = rows + 9        # sorted positions past the last group: zero rows
    full_gather = torch.from_numpy(np.concatenate([gather, np.zeros(padded - rows, np.int32)])).cuda()
    offsets = torch.from_numpy(np.concatenate([[0], np.cumsum(sizes)]).astype(np.int32)).cuda()
    banks = [ops.prepare(bank.to("cuda")) for bank in (gate, up)]
    assert banks[0].descriptor.format == ops._lib.W_NVFP4          # block scales with mantissas: not an MX bank
    monkeypatch.setattr(ops, "F16_ROWS_FROM", 0)
    assert ops.prefers_f16_rows(*banks, padded)
    with ops.tile_rows(tile):
        got = ops.gateup_swiglu(x.cuda(), *banks, offsets, gather=full_gather, rows=padded, activation=activation, limit=limit)
        by_sizes = ops.gateup_swiglu(x.cuda(), *banks, None, sizes=torch.tensor(sizes, dtype=torch.int32).cuda(), gather=full_gather,
                                     rows=padded, activation=activation, limit=limit)
        monkeypatch.setattr(ops, "F16_ROWS", False)
        assert not ops.prefers_f16_rows(*banks, padded)
        plain = ops.gateup_swiglu(x.cuda(), *banks, offsets, gather=full_gather, rows=padded, activation=activation, limit=limit)
    assert torch.equal(got, plain) and torch.equal(by_sizes, plain)
    assert not bool(got[rows:].any())
    (gate_values, gate_factor), (up_values, up_factor) = dequantized(gate), dequantized(up)
    sorted_x = x.float().numpy()[gather]
    product = oracle.GATED_PRODUCTS[activation]
    want = product(oracle.grouped_matmul(sorted_x, gate_values, sizes, factor=gate_factor),
                   oracle.grouped_matmul(sorted_x, up_values, sizes, factor=up_factor), limit=limit)
    by_max, by_element = oracle.relative_errors(got[:rows].float().cpu().numpy(), want)
    assert by_max <= 2e-2 and by_element <= 2e-2, (by_max, by_element)
    assert (got[:rows].float().cpu().numpy() == want).mean() >= 0.97


def test_f16_rows_are_for_general_nvfp4_banks_only():
    from dew_amd import ops

    rng = np.random.default_rng(3)
    weight = torch.from_numpy((rng.standard_normal((2, 256, 128)) * 0.05).astype(np.float32))
    mx = ops.prepare(quantize(weight, "mxfp4").to("cuda"))
    assert mx.descriptor.format == ops._lib.W_MXFP4 and not ops.prefers_f16_rows(mx, mx, 4096)
    x = torch.from_numpy(rng.standard_normal((8, 256)).astype(np.float32)).to(torch.bfloat16).cuda()
    halves, scale = ops.rows_f16(x)
    hidden = torch.empty((8, 128), dtype=torch.bfloat16, device="cuda")
    offsets = torch.tensor([0, 4, 8], dtype=torch.int32, device="cuda")
    status = ops._lib.library().dew_moe_gateup_gated_f16(ops._ptr(halves), ops._ptr(scale), None, ops._ptr(offsets), None, mx.descriptor,
                                                         mx.descriptor, 0, 0.0, ops._ptr(hidden), 8, None)
    assert status != 0 and b"NVFP4 banks whose block scales carry mantissas" in ops._lib.library().dew_moe_last_error()

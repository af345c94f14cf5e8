"""Whole layers on seeded random settings against the CPU oracle: every bank format, every router variant, capacity
dropping, the clamp, GeGLU, input-scaled experts, a shared expert. Forty fixed seeds (one test each, so `-x` stops at the
first that fails), then the layers that run on split rows (MXFP4 banks, groups of hundreds of rows: two e4m3 terms a row
on the scaled matrix instruction), which have a bar of their own.

The bars. Every path holds the reference's metric, `max|d| / max|ref| <= 2e-2` (tools/benchmark_kernels.py:143-144). The
element-wise figure `|d| / max(|ref|, rms(ref))` is this repository's own, stricter one: the bf16-operand launches hold
2e-2 on it; the split-row launches hold ELEMENTWISE_ON_SPLIT_ROWS = 3e-2, because their sums come from another matrix
instruction (one bf16 ulp apart from the bf16 instruction's in about 1 % of outputs) and their hidden rows carry one
scale per 128 columns, and where a routed and a shared output nearly cancel two such ulps have been seen to add up to
2.05e-2 .. 2.45e-2 of the difference. `gemm.SPLIT_ROWS = False` keeps such a layer on the bf16 instruction and its 2e-2.

What the element-wise figure cannot promise, on any path: it divides by the output's rms, and one bf16 ulp of a slot (an expert's
output row, before the combine weighs it) is 2^-8 of that slot, so a single flipped rounding on a slot five times the output's
rms is 2e-2 of it. Of 4 700 further seeds of this generator five did that (2.00e-2 .. 2.2e-2; the split-row layers among them
stayed under their 3e-2, at 2.87e-2 at most; the reference's metric never passed 5.3e-3). The two largest are kept here
(ONE_ULP_SEEDS: 2.2e-2 and 2.05e-2, each one ulp of one slot of 0.17 .. 0.25 under an output rms of 0.03 .. 0.05, 99.94 % of the
outputs bit-identical) under the bar that names the case, ONE_ULP_OF_A_LARGE_SLOT."""

import numpy as np
import pytest
import torch

from bench_aids.workloads import Case, inputs
from oracle import moe_oracle as oracle
from oracle.banks import dequantized

pytestmark = pytest.mark.gpu

BAR = 2e-2
ELEMENTWISE_ON_SPLIT_ROWS = 3e-2

ONE_ULP_OF_A_LARGE_SLOT = 2.5e-2
ONE_ULP_SEEDS = (30955, 30992)

SEEDS = tuple(range(7000, 7036)) + (5051, 5085, 5086, 5127)
"""Thirty-six consecutive seeds and four that earlier, longer runs of the same generator singled out (5086: a capacity-dropped
sigmoid router over MXFP4 banks on split rows that read 2.3e-2 element-wise; 5051: a one-token layer that once produced a NaN)."""


def drawn(seed):
    """The layer a seed stands for: (case, layer settings)."""
    rng = np.random.default_rng(seed)
    experts = int(rng.choice([4, 8, 16, 32, 64]))
    groups = int(rng.choice([g for g in (1, 2, 4, 8) if experts % g == 0 and experts // g >= 2]))
    per_token = int(rng.integers(1, groups + 1))
    k = int(rng.integers(1, min(8, per_token * (experts // groups)) + 1))
    score = str(rng.choice(["softmax", "sigmoid", "sqrtsoftplus"]))
    router = dict(score_function=score, normalize_weights=bool(rng.integers(0, 2)), routed_scaling_factor=float(rng.choice([1.0, 2.5])),
                  expert_groups=groups, groups_per_token=per_token, group_score=str(rng.choice(["top2", "max"])))
    quant = str(rng.choice(["fp8_channel", "fp8_block", "mxfp4", "nvfp4", "bf16"]))
    unit = 256 if quant in ("mxfp4", "nvfp4") else 128
    tokens = int(rng.choice([1, 3, 17, 64, 200, 513, 1500, 3000]))
    case = Case(f"s{seed}", tokens, int(rng.integers(1, 5)) * unit, int(rng.integers(1, 5)) * unit, experts, k, quant, router,
                logit_bias_std=float(rng.choice([0.0, 0.5, 2.0])), shared=bool(rng.integers(0, 2)))
    settings = dict(capacity_factor=None if rng.integers(0, 3) else float(rng.choice([0.5, 1.0, 1.5])),
                    swiglu_limit=None if rng.integers(0, 3) else float(rng.choice([0.5, 3.0])),
                    activation=str(rng.choice(["swiglu", "swiglu", "geglu"])), scale_inputs=bool(rng.integers(0, 3) == 0))
    return case, settings


def layer_against_the_oracle(case, settings, seed):
    """(max|d| / max|ref|, element-wise figure, whether the routed experts ran on split rows); routing compared bit for bit."""
    from dew_amd import gemm, moe

    data = inputs(case, seed)
    layer = moe.SparseMLP(num_experts=case.experts, top_k=case.top_k, hidden_features=case.d_ff, out_features=case.d_model,
                          expert_bias=data["bias"] is not None, shared=case.d_ff if case.shared else None, **settings, **case.router)
    variables = {"params": {}, "quantization": {"experts": {f"{n}_proj": {"kernel": bank.to("cuda")} for n, bank in data["banks"].items()}}}
    if data["bias"] is not None:
        variables["moe"] = {"gate": {"e_score_correction_bias": data["bias"].cuda()}}
    if case.shared:
        variables["quantization"]["shared_experts"] = {f"{n}_proj": {"kernel": bank.to("cuda")} for n, bank in data["shared"].items()}
    x, logits = data["x"].cuda(), data["logits"].cuda()
    taken, found = [], gemm.swiglu_mlp_on_split_rows      # the layer's own decision, as it makes it
    gemm.swiglu_mlp_on_split_rows = lambda *a, **k: taken.append(found(*a, **k)) or taken[-1]
    try:
        got = layer.apply(variables, x, logits=logits).float().cpu().numpy()
    finally:
        gemm.swiglu_mlp_on_split_rows = found
    mats, factors = zip(*(dequantized(data["banks"][n]) for n in ("gate", "up", "down")), strict=True)
    bias = None if data["bias"] is None else data["bias"].numpy()
    weights, indices = oracle.route(data["logits"].numpy(), case.top_k, bias=bias, **case.router)
    want, _ = oracle.expert_mlp(data["x"].float().numpy(), weights, indices, *mats, factors=factors, limit=settings["swiglu_limit"],
                                capacity_factor=settings["capacity_factor"], activation=settings["activation"],
                                scale_inputs=settings["scale_inputs"])
    if case.shared:
        shared = [dequantized(data["shared"][n]) for n in ("gate", "up", "down")]
        xs, everyone = data["x"].float().numpy(), [case.tokens]
        hidden = oracle.swiglu(oracle.grouped_matmul(xs, shared[0][0], everyone, factor=shared[0][1]),
                               oracle.grouped_matmul(xs, shared[1][0], everyone, factor=shared[1][1]))
        want = oracle.bf16_round(want + oracle.grouped_matmul(hidden, shared[2][0], everyone, factor=shared[2][1]))
    device_weights, device_indices = layer._bound(variables, ()).gate.routed(logits)
    assert np.array_equal(device_indices.cpu().numpy(), indices)
    assert np.array_equal(device_weights.cpu().numpy().view(np.uint32), weights.view(np.uint32))
    assert np.isfinite(got).all()
    on_split_rows = any(out is not None for out in taken)
    if not want.any():      # (a capacity that drops every slot of a few tokens: the layer's output is zero, and so must the device's be)
        assert not got.any()
        return 0.0, 0.0, on_split_rows
    return (*oracle.relative_errors(got, want), on_split_rows)


@pytest.mark.parametrize("seed", SEEDS)
def test_a_seeded_layer_matches_the_oracle(seed):
    case, settings = drawn(seed)
    print(f"seed {seed}: {case} {settings}", flush=True)
    by_max, by_element, on_split_rows = layer_against_the_oracle(case, settings, seed)
    assert by_max <= BAR, (by_max, by_element)
    assert by_element <= (ELEMENTWISE_ON_SPLIT_ROWS if on_split_rows else BAR), (by_max, by_element, on_split_rows)


@pytest.mark.parametrize("seed", ONE_ULP_SEEDS)
def test_one_ulp_of_a_large_slot_is_all_that_differs(seed):
    """The two seeds whose element-wise figure passes 2e-2 on the bf16 instruction: the reference's metric holds with a wide
    margin, and the figure stays under the bar one flipped bf16 rounding of a slot several times the output's rms explains."""
    case, settings = drawn(seed)
    by_max, by_element, on_split_rows = layer_against_the_oracle(case, settings, seed)
    assert not on_split_rows
    assert by_max <= 5e-3 and by_element <= ONE_ULP_OF_A_LARGE_SLOT, (by_max, by_element)


SPLIT_ROW_LAYERS = [
    # (seed, tokens, d_model, d_ff, experts, k, routed_scaling_factor): MXFP4, >= 384 rows a group, a shared expert
    (11, 1600, 512, 768, 4, 2, 2.5), (12, 3000, 256, 1024, 8, 2, 2.5), (13, 2048, 1024, 512, 4, 1, 2.5),
    (14, 1800, 768, 768, 8, 3, 2.5), (15, 2500, 512, 256, 4, 2, 1.0), (16, 1536, 256, 768, 2, 1, 2.5),
]


@pytest.mark.parametrize("seed,tokens,d_model,d_ff,experts,k,scaling", SPLIT_ROW_LAYERS)
def test_a_split_row_layer_with_a_shared_expert_holds_its_bars(seed, tokens, d_model, d_ff, experts, k, scaling):
    """The setting in which the split rows' element-wise figure has been seen past 2e-2: MXFP4 banks, groups of 384 rows or
    more (so the routed experts run on the scaled instruction), a shared expert whose output meets the routed one, router
    weights scaled by 2.5. The reference's metric holds its 2e-2 with a wide margin; the element-wise figure holds the split
    rows' own bar; and the same layer kept on the bf16 instruction (`gemm.SPLIT_ROWS = False`) holds 2e-2 on both."""
    from dew_amd import gemm

    router = dict(score_function="sigmoid", normalize_weights=True, routed_scaling_factor=scaling)
    case = Case(f"split{seed}", tokens, d_model, d_ff, experts, k, "mxfp4", router, shared=True)
    settings = dict(capacity_factor=None, swiglu_limit=None, activation="swiglu", scale_inputs=False)
    by_max, by_element, on_split_rows = layer_against_the_oracle(case, settings, seed)
    assert on_split_rows
    assert by_max <= 1e-2 and by_element <= ELEMENTWISE_ON_SPLIT_ROWS, (by_max, by_element)
    held, gemm.SPLIT_ROWS = gemm.SPLIT_ROWS, False
    try:
        by_max, by_element, on_split_rows = layer_against_the_oracle(case, settings, seed)
    finally:
        gemm.SPLIT_ROWS = held
    assert not on_split_rows
    assert by_max <= 1e-2 and by_element <= BAR, (by_max, by_element)

"""The whole layer (SparseMLP: route, sort, gate/up + SwiGLU, down, combine, shared expert) on the device,
through the reference-shaped API, against the CPU oracle on the same seeded inputs.

Bars: routing indices, group sizes/offsets and the permutation bit-exact; router weights bit-exact; outputs
within max relative error 2e-2 (measured both as max|d| / max|ref| and element-wise as |d| / max(|ref|,
rms(ref))). The bf16-exact kernels land near 2^-8, far inside the bar; the observed figures are printed."""

from dataclasses import replace as dataclasses_replace

import numpy as np
import pytest
import torch
from bench_aids.workloads import CONFIGS, inputs
from oracle.banks import dequantized

from oracle import moe_oracle as oracle

pytestmark = pytest.mark.gpu

TOLERANCE = 2e-2
ELEMENTWISE_ON_FP6_OPTIONS = 4e-2
"""The element-wise bar of the two experimental FP6 forms of split rows (`gemm.SPLIT_SECOND_TERM` 'e2m3', 'e2m3x2'): twice the
default paths' 2e-2. They are not exact and are off by default; the reference's own metric is held to 1e-2 on them."""

CASES = {
    "c1-full": CONFIGS["c1"],
    "c2-reduced": CONFIGS["c2"].scaled(tokens=640, d_model=1024, d_ff=1792),
    "c3-reduced": CONFIGS["c3"].scaled(d_model=1024, d_ff=384 + 128),
    "c3-one-token": CONFIGS["c3"].scaled(tokens=1, d_model=512, d_ff=256, experts=16, top_k=4),
    "c4-reduced": CONFIGS["c4"].scaled(tokens=384, d_model=1024, d_ff=512),
    "c5-reduced": CONFIGS["c5"].scaled(tokens=300, d_model=1024, d_ff=1792),
}


def layer_and_variables(case, data):
    from dew_amd import moe

    router = dict(case.router)
    layer = moe.SparseMLP(num_experts=case.experts, top_k=case.top_k, hidden_features=case.d_ff,
                          out_features=case.d_model, expert_bias=data["bias"] is not None,
                          shared=case.d_ff if case.shared else None, **router)
    banks = {name: {"kernel": bank.to("cuda")} for name, bank in data["banks"].items()}
    variables = {"params": {}, "quantization": {"experts": {f"{n}_proj": v for n, v in banks.items()}}}
    if data["bias"] is not None:
        variables["moe"] = {"gate": {"e_score_correction_bias": data["bias"].cuda()}}
    if case.shared:
        variables["quantization"]["shared_experts"] = {f"{n}_proj": {"kernel": b.to("cuda")} for n, b in data["shared"].items()}
    return layer, variables


def oracle_output(case, data):
    mats, factors = zip(*(dequantized(data["banks"][name]) for name in ("gate", "up", "down")), strict=True)
    shared = None
    if case.shared:
        shared = [dequantized(data["shared"][name])[0][0] for name in ("gate", "up", "down")]
    return oracle.sparse_mlp(data["x"].float().numpy(), data["logits"].numpy(), *mats, top_k_count=case.top_k,
                             shared=shared, factors=factors, bias=None if data["bias"] is None else data["bias"].numpy(),
                             **case.router)


@pytest.mark.parametrize("name", list(CASES))
def test_layer_matches_the_oracle(name):
    from dew_amd import ops

    case = CASES[name]
    data = inputs(case, seed=0)
    layer, variables = layer_and_variables(case, data)
    x, logits = data["x"].cuda(), data["logits"].cuda()
    got = layer.apply(variables, x, logits=logits).float().cpu().numpy()
    want, trace = oracle_output(case, data)

    # routing: bit-exact
    weights, indices = layer._bound(variables, ()).gate.routed(logits)
    assert np.array_equal(indices.cpu().numpy(), trace["indices"])
    assert np.array_equal(weights.cpu().numpy().view(np.uint32), trace["weights"].view(np.uint32))
    plan = ops.sort_by_expert(indices, case.experts)
    for field in ("order", "rows", "sizes", "offsets"):
        assert np.array_equal(getattr(plan, field).cpu().numpy(), trace[field]), field

    by_max, by_element = oracle.relative_errors(got, want)
    print(f"\n{name}: max|d|/max|ref| = {by_max:.3e}, element-wise max rel = {by_element:.3e}, "
          f"identical = {(got == want).mean():.4f}")
    assert by_max <= TOLERANCE and by_element <= TOLERANCE

    # the unfused arrangement (paired product, then the SwiGLU kernel) is the fused one bit for bit
    import dataclasses
    unfused = dataclasses.replace(layer, fused=False).apply(variables, x, logits=logits).float().cpu().numpy()
    assert np.array_equal(unfused, got)
    if case.shared:
        # the shared expert as group #E of the routed launches (the default) is the reference's arrangement, a dense
        # MLP of its own whose output the combine adds, bit for bit
        from dew_amd import moe
        calls = []
        found = moe.with_shared_expert
        moe.with_shared_expert = lambda *a: calls.append(1) or found(*a)
        try:
            assert np.array_equal(layer.apply(variables, x, logits=logits).float().cpu().numpy(), got) and calls == [1]
            apart = dataclasses.replace(layer, fuse_shared=False).apply(variables, x, logits=logits).float().cpu().numpy()
            assert calls == [1]
        finally:
            moe.with_shared_expert = found
        assert np.array_equal(apart, got)


def test_large_groups_on_mxfp4_banks_run_on_split_rows_and_agree_with_the_bf16_launches(monkeypatch):
    """Groups of a thousand rows on MXFP4 banks take the two launches on the scaled matrix instruction (rows as two
    e4m3 terms); the layer's output is within the bar of the oracle either way and nearly all of it is identical."""
    from dew_amd import gemm, ops

    case = CONFIGS["c2"].scaled(tokens=4608, d_model=512, d_ff=768)       # 9216 routed rows over 8 experts
    data = inputs(case, seed=3)
    layer, variables = layer_and_variables(case, data)
    x, logits = data["x"].cuda(), data["logits"].cuda()
    calls = []
    on_split_rows = ops.swiglu_mlp_split
    monkeypatch.setattr(ops, "swiglu_mlp_split", lambda *a, **k: calls.append(1) or on_split_rows(*a, **k))
    assert gemm.SPLIT_ROWS and gemm.SPLIT_SECOND_TERM == "e4m3"
    got = layer.apply(variables, x, logits=logits).float().cpu().numpy()            # two e4m3 terms: the rows' bf16 values exactly
    assert calls == [1]
    monkeypatch.setattr(gemm, "SPLIT_SECOND_TERM", "e2m3")
    with_fp6 = layer.apply(variables, x, logits=logits).float().cpu().numpy()       # an experimental option: an e4m3 and an e2m3 term
    monkeypatch.setattr(gemm, "SPLIT_SECOND_TERM", "e2m3x2")
    with_two_fp6 = layer.apply(variables, x, logits=logits).float().cpu().numpy()   # the other: two e2m3 terms
    assert calls == [1, 1, 1]
    monkeypatch.setattr(gemm, "SPLIT_ROWS", False)
    plain = layer.apply(variables, x, logits=logits).float().cpu().numpy()
    assert calls == [1, 1, 1]
    want, _ = oracle_output(case, data)
    for name, value in (("split rows, two e4m3", got), ("bf16 operands", plain)):
        by_max, by_element = oracle.relative_errors(value, want)
        print(f"\n{name}: max|d|/max|ref| = {by_max:.3e}, element-wise max rel = {by_element:.3e}, identical = {(value == want).mean():.4f}")
        assert by_max <= TOLERANCE and by_element <= TOLERANCE
    assert (got == plain).mean() > 0.9 and np.abs(got - plain).max() <= 2.0 ** -6 * np.abs(plain).max()
    # The FP6 terms are experimental options, not the default, because of what they cost here: inside 1e-2 of the largest
    # output (the reference's own measure, which every path holds to 2e-2), but element-wise they pass this repository's
    # 2e-2 bar on an MLP this narrow (512 deep), so they are held to a bar of their own, stated as such in the header.
    for name, value in (("e4m3 + e2m3", with_fp6), ("e2m3 + e2m3", with_two_fp6)):
        by_max, by_element = oracle.relative_errors(value, want)
        print(f"\nsplit rows, {name} (experimental option): max|d|/max|ref| = {by_max:.3e}, element-wise max rel = {by_element:.3e}, "
              f"identical = {(value == want).mean():.4f}")
        assert by_max <= 1e-2 and by_element <= ELEMENTWISE_ON_FP6_OPTIONS


def test_layer_multiplies_its_own_gate_kernel_when_no_logits_are_given():
    from dew_amd import moe

    case = CASES["c3-one-token"].scaled(tokens=37)
    data = inputs(case, seed=3)
    rng = np.random.default_rng(4)
    kernel = torch.from_numpy((rng.standard_normal((case.d_model, case.experts)) * 0.05).astype(np.float32))
    layer, variables = layer_and_variables(case, data)
    variables["params"]["gate"] = {"kernel": kernel.cuda()}
    x = data["x"].cuda()
    logits = layer._bound(variables, ()).gate.logits(x).cpu().numpy()
    want_logits = oracle.router_logits(data["x"].float().numpy(), kernel.numpy())
    assert np.abs(logits - want_logits).max() <= 1e-5 * np.abs(want_logits).max()
    got = layer.apply(variables, x)
    again = layer.apply(variables, x, logits=torch.from_numpy(logits).cuda())
    assert torch.equal(got, again)


def test_idle_experts_change_nothing():
    """Adding experts no token is routed to leaves the output unchanged (the reference's
    tests/test_moe.py:356-368)."""
    from dew_amd import formats, moe, ops

    case = CASES["c3-one-token"].scaled(tokens=50, experts=4, top_k=2)
    data = inputs(case, seed=5)
    x, logits = data["x"].cuda(), data["logits"].cuda()
    layer, variables = layer_and_variables(case, data)
    got = layer.apply(variables, x, logits=logits)
    wide = case.scaled(experts=8)

    def widened(bank):
        return formats.Fp8Blocks(torch.cat([bank.codes, torch.full_like(bank.codes, 0x55)]),
                                 torch.cat([bank.scale_inv, bank.scale_inv]))

    wide_data = dict(data, banks={n: widened(b) for n, b in data["banks"].items()})
    wide_logits = torch.cat([logits, torch.full_like(logits, -1e4)], dim=-1)
    wide_layer, wide_variables = layer_and_variables(wide, wide_data)
    assert torch.equal(wide_layer.apply(wide_variables, x, logits=wide_logits), got)


def test_a_named_kernel_that_cannot_run_is_refused_by_name():
    from dew_amd import moe, selection

    case = CASES["c3-one-token"]
    data = inputs(case, seed=1)
    layer, variables = layer_and_variables(case, data)
    x, logits = data["x"].cuda(), data["logits"].cuda()
    with selection.chosen(grouped_matmul="hip"):
        layer.apply(variables, x, logits=logits)
    assert any(route.kernel == "hip" and route.forced == "hip" for route in selection.routes())
    with pytest.raises(selection.Unlowerable, match="xla"), selection.chosen(grouped_matmul="xla"):
        layer.apply(variables, x, logits=logits)
    with pytest.raises(selection.KernelRefused, match="bf16"), selection.chosen(grouped_matmul="hip"):
        layer.apply(variables, x.float(), logits=logits)


def test_no_tokens_give_no_rows_and_no_launch_fails():
    """An empty batch goes through every entry point and the whole layer and comes back empty."""
    from dew_amd import ops

    case = CASES["c3-one-token"]
    data = inputs(case, seed=2)
    layer, variables = layer_and_variables(case, data)
    x = data["x"][:0].cuda()
    logits = data["logits"][:0].cuda()
    weights, indices = ops.route(logits, case.top_k, **case.router)
    assert weights.shape == (0, case.top_k) and indices.shape == (0, case.top_k)
    plan = ops.sort_by_expert(indices, case.experts)
    assert plan.sizes.tolist() == [0] * case.experts and plan.offsets.tolist() == [0] * (case.experts + 1)
    assert plan.order.numel() == 0 and plan.rows.numel() == 0
    out = layer.apply(variables, x, logits=logits)
    assert out.shape == (0, case.d_model) and out.dtype == torch.bfloat16


def test_more_experts_than_one_scan_round_and_every_expert_chosen():
    """512 experts (the tile search scans them 256 at a time) of which most are idle, and a router whose top-k is
    all of its experts."""
    from dew_amd import ops

    rng = np.random.default_rng(8)
    experts, depth, width = 512, 256, 128
    sizes = np.zeros(experts, np.int64)
    sizes[[3, 255, 256, 300, 511]] = [40, 1, 130, 7, 64]
    from test_gpu_kernels import grouped_case, bf16_np
    bank, x, offsets = grouped_case("fp8_block", experts, depth, width, sizes.tolist(), seed=4)
    values, factor = dequantized(bank)
    want = oracle.grouped_matmul(bf16_np(x), values, sizes.tolist(), factor=factor)
    got = bf16_np(ops.grouped_gemm(x.cuda(), ops.prepare(bank.to("cuda")), torch.from_numpy(offsets).cuda()))
    assert np.abs(got - want).max() <= 2 ** -7 * np.abs(want).max() and (got == want).mean() > 0.97
    logits = torch.from_numpy(rng.standard_normal((33, 8)).astype(np.float32))
    weights, indices = ops.route(logits.cuda(), 8, score_function="softmax", normalize_weights=True)
    want_weights, want_indices = oracle.route(logits.numpy(), 8, score_function="softmax", normalize_weights=True)
    assert np.array_equal(indices.cpu().numpy(), want_indices) and np.array_equal(weights.cpu().numpy(), want_weights)
    assert np.array_equal(np.sort(indices.cpu().numpy(), -1), np.tile(np.arange(8), (33, 1)))


@pytest.mark.parametrize("score_function,experts,top_k,groups", [("softmax", 8, 2, (1, 1)), ("sigmoid", 256, 8, (8, 4)), ("softmax", 130, 4, (1, 1))])
def test_the_router_sows_its_scores_and_log_partition_and_the_bias_balances(score_function, experts, top_k, groups):
    """The launch that routes also writes what the reference's router sows for the balance statistics; the choices
    are the plain launch's bit for bit, scores and log partition within 1e-6 of the oracle's, and one balancing
    step of the selection bias from the dispatch's own counts is the oracle's bit for bit."""
    from dew_amd import moe, ops

    rng = np.random.default_rng(experts)
    logits = torch.from_numpy((rng.standard_normal((500, experts)) * 2).astype(np.float32)).cuda()
    bias = torch.from_numpy((rng.standard_normal(experts) * 0.1).astype(np.float32)).cuda() if score_function == "sigmoid" else None
    options = dict(score_function=score_function, bias=bias, expert_groups=groups[0], groups_per_token=groups[1])
    weights, indices = ops.route(logits, top_k, **options)
    sown_weights, sown_indices, scores, log_z = ops.route(logits, top_k, sown=True, **options)
    assert torch.equal(weights, sown_weights) and torch.equal(indices, sown_indices)
    want_scores, want_log_z = oracle.router_statistics(logits.cpu().numpy(), score_function=score_function)
    assert np.abs(scores.cpu().numpy() - want_scores).max() <= 1e-6
    assert np.abs(log_z.cpu().numpy() - want_log_z).max() <= 1e-6 * max(1.0, np.abs(want_log_z).max())
    counts = moe.router_counts(indices, experts)
    assert np.array_equal(counts.cpu().numpy(), np.bincount(indices.cpu().numpy().ravel(), minlength=experts))
    start = torch.zeros(experts, dtype=torch.float32).cuda() if bias is None else bias
    stepped = moe.updated_bias(start, counts, 0.001)
    want = start.cpu().numpy() + oracle.load_balance_update(counts.cpu().numpy(), 0.001)
    assert np.array_equal(stepped.cpu().numpy(), want.astype(np.float32))
    assert np.array_equal(moe.load_balance_update(counts, 0.25).cpu().numpy(), oracle.load_balance_update(counts.cpu().numpy(), 0.25))


def test_unquantized_bf16_experts_run_through_the_layer_as_plain_tensors():
    """The reference's own operand: bf16 `[E, K, N]` parameters handed to the layer as tensors (re-laid at every call)
    give the products of the same matrices wrapped as `formats.Bf16` (re-laid once), bit for bit, and match the
    oracle's layer on the decoded (here: identical) weights."""
    from dew_amd import formats, gemm

    rng = np.random.default_rng(77)
    experts, depth, width, sizes = 4, 256, 384, [70, 0, 129, 33]
    rows = int(np.sum(sizes))
    x = torch.from_numpy(rng.standard_normal((rows, depth)).astype(np.float32)).to(torch.bfloat16).cuda()
    gate, up = (torch.from_numpy((rng.standard_normal((experts, depth, width)) * 0.05).astype(np.float32)).to(torch.bfloat16).cuda()
                for _ in range(2))
    group_sizes = torch.tensor(sizes, dtype=torch.int32).cuda()
    plain = gemm.gemm(x, gate, group_sizes, paired=up, epilogue="swiglu")
    kept = gemm.gemm(x, formats.Bf16(gate), group_sizes, paired=formats.Bf16(up), epilogue="swiglu")
    assert torch.equal(plain, kept)
    want = oracle.swiglu(oracle.grouped_matmul(x.float().cpu().numpy(), gate.float().cpu().numpy(), sizes),
                         oracle.grouped_matmul(x.float().cpu().numpy(), up.float().cpu().numpy(), sizes))
    got = plain.float().cpu().numpy()
    assert np.abs(got - want).max() <= 2.0 ** -6 * np.abs(want).max() and (got == want).mean() > 0.9
    # an input gradient's matrices: the transposed view is read where it lies, no copy of the transpose is made
    dy = torch.from_numpy(rng.standard_normal((rows, width)).astype(np.float32)).to(torch.bfloat16).cuda()
    copied = gemm.gemm(dy, gate.transpose(1, 2).contiguous(), group_sizes)
    assert torch.equal(gemm.gemm(dy, gate.transpose(1, 2), group_sizes), copied)
    assert torch.equal(gemm.gemm(dy, formats.Bf16(gate).T, group_sizes), copied)
    want = oracle.grouped_matmul(dy.float().cpu().numpy(), gate.float().cpu().numpy().transpose(0, 2, 1), sizes)
    assert np.abs(copied.float().cpu().numpy() - want).max() <= 2.0 ** -7 * np.abs(want).max()



def test_the_clamped_experts_reproduce_the_references_deepseek_v4_output_and_capacity_drops_rows():
    """DeepSeek V4's experts (`swiglu_limit` 1.0) on the reference's own fixture: its fp32 matrices held as bf16 banks,
    the recorded routing, against the oracle in bf16 and (within bf16's grain) the recorded fp32 output. Then the same
    experts with a capacity factor: the dropped slots' rows come back zero, as the oracle's."""
    from conftest import golden

    from dew_amd import formats, moe

    tensors = golden("moe/deepseek_v4.npz")
    hidden = torch.from_numpy(tensors["hidden"].reshape(-1, 16))
    pad = lambda m: np.pad(m, [(0, 0), (0, 128 - m.shape[1]), (0, 128 - m.shape[2])])   # the kernels' least matrix is 128 x 128
    mats = [pad(np.stack([tensors[f"mlp.experts.{e}.{p}.weight"].T for e in range(8)])) for p in ("gate_proj", "up_proj", "down_proj")]
    banks = [formats.Bf16(torch.from_numpy(m).to(torch.bfloat16).cuda()) for m in mats]
    decoded = [bank.weights.float().cpu().numpy() for bank in banks]
    x = torch.nn.functional.pad(hidden, (0, 112)).to(torch.bfloat16)
    weights, indices = torch.from_numpy(tensors["router_weights"]), torch.from_numpy(tensors["router_indices"]).to(torch.int32)
    variables = {"params": {}, "quantization": {f"{n}_proj": {"kernel": bank} for n, bank in zip(("gate", "up", "down"), banks)}}
    experts = moe.ExpertMLP(8, 128, 128, swiglu_limit=1.0)
    got = experts.apply(variables, x.cuda(), weights.cuda(), indices.cuda()).float().cpu().numpy()
    want, _ = oracle.expert_mlp(x.float().numpy(), weights.numpy(), indices.numpy(), *decoded, limit=1.0)
    by_max, by_element = oracle.relative_errors(got, want)
    assert by_max <= TOLERANCE and by_element <= TOLERANCE
    recorded = tensors["experts_output"].reshape(-1, 16)
    assert np.abs(got[:, :16] - recorded).max() <= 2e-2 * np.abs(recorded).max()       # bf16 operands against the fp32 record
    unclamped = moe.ExpertMLP(8, 128, 128).apply(variables, x.cuda(), weights.cuda(), indices.cuda()).float().cpu().numpy()
    assert np.abs(unclamped[:, :16] - recorded).max() > 1.0

    dropping = moe.ExpertMLP(8, 128, 128, swiglu_limit=1.0, capacity_factor=0.5)
    shaped = indices.reshape(1, *indices.shape)                                        # one sequence
    got = dropping.apply(variables, x.cuda().reshape(1, *x.shape), weights.cuda().reshape(1, *weights.shape), shaped.cuda())
    want, trace = oracle.expert_mlp(x.float().numpy(), weights.numpy(), shaped.numpy(), *decoded, limit=1.0, capacity_factor=0.5)
    assert trace["sizes"].sum() < indices.numel()                                      # something was dropped
    by_max, by_element = oracle.relative_errors(got.float().cpu().numpy().reshape(want.shape), want)
    assert by_max <= TOLERANCE and by_element <= TOLERANCE


@pytest.mark.parametrize("quant", ["bf16", "fp8_block", "mxfp4"])
def test_geglu_experts_run_through_the_layer(quant):
    """Gemma's experts gate by the tanh GELU (`activation='geglu'`, src/dew/nn/gemma4_moe.py:84): the paired product, the
    stand-alone gating kernel and the down product against the oracle's `expert_mlp(activation='geglu')`; a SwiGLU layer
    on the same banks is far from it."""
    from bench_aids.workloads import quantize

    from dew_amd import moe, ops

    rng = np.random.default_rng(17)
    tokens, experts, top_k, width, hidden = 200, 8, 2, 256, 512
    x = torch.from_numpy(rng.standard_normal((tokens, width)).astype(np.float32)).to(torch.bfloat16)
    banks = {name: quantize(torch.from_numpy((rng.standard_normal((experts, d, w)) * 0.08).astype(np.float32)), quant)
             for name, (d, w) in (("gate", (width, hidden)), ("up", (width, hidden)), ("down", (hidden, width)))}
    logits = rng.standard_normal((tokens, experts)).astype(np.float32)
    weights, indices = ops.route(torch.from_numpy(logits).cuda(), top_k)
    variables = {"params": {}, "quantization": {f"{n}_proj": {"kernel": bank.to("cuda")} for n, bank in banks.items()}}
    got = moe.ExpertMLP(experts, hidden, width, activation="geglu").apply(variables, x.cuda(), weights, indices).float().cpu().numpy()
    mats, factors = zip(*(dequantized(banks[name]) for name in ("gate", "up", "down")), strict=True)
    want, _ = oracle.expert_mlp(x.float().numpy(), weights.cpu().numpy(), indices.cpu().numpy(), *mats, factors=factors, activation="geglu")
    by_max, by_element = oracle.relative_errors(got, want)
    assert by_max <= 6e-3 and by_element <= TOLERANCE, (by_max, by_element)
    assert (got == want).mean() > 0.97
    swiglu = moe.ExpertMLP(experts, hidden, width).apply(variables, x.cuda(), weights, indices).float().cpu().numpy()
    assert np.abs(swiglu - want).max() > 0.05 * np.abs(want).max()
    with pytest.raises(ValueError, match="gate by one of"):
        moe.ExpertMLP(experts, hidden, width, activation="geglu_exact")


@pytest.mark.parametrize("gating", [dict(swiglu_limit=0.5), dict(activation="geglu")])
def test_a_shared_expert_keeps_its_own_gating_beside_clamped_or_geglu_experts(gating):
    """The shared expert is a dense SwiGLU MLP of its own (src/dew/nn/moe.py:1497-1503, nn/mlp.py:139-144), whatever gates
    the routed experts: beside a clamp or a GeGLU gate it does not ride the routed launches, whose gating it would take."""
    import dataclasses

    from dew_amd import moe

    case = CASES["c4-reduced"].scaled(tokens=96)
    data = inputs(case, seed=4)
    layer, variables = layer_and_variables(case, data)
    layer = dataclasses.replace(layer, **gating)
    calls = []
    found = moe.with_shared_expert
    moe.with_shared_expert = lambda *a: calls.append(1) or found(*a)
    try:
        got = layer.apply(variables, data["x"].cuda(), logits=data["logits"].cuda()).float().cpu().numpy()
    finally:
        moe.with_shared_expert = found
    assert calls == []
    mats, factors = zip(*(dequantized(data["banks"][name]) for name in ("gate", "up", "down")), strict=True)
    x = data["x"].float().numpy()
    weights, indices = oracle.route(data["logits"].numpy(), case.top_k, bias=data["bias"].numpy(), **case.router)
    routed, _ = oracle.expert_mlp(x, weights, indices, *mats, factors=factors, limit=gating.get("swiglu_limit"),
                                  activation=gating.get("activation", "swiglu"))
    shared = [dequantized(data["shared"][name])[0][0] for name in ("gate", "up", "down")]
    want = oracle.bf16_round(routed + oracle.gated_mlp(x, *shared))
    by_max, by_element = oracle.relative_errors(got, want)
    assert by_max <= 6e-3 and by_element <= TOLERANCE, (by_max, by_element)


def test_llama_4s_input_scaled_experts_on_the_references_fixture_and_a_seeded_layer():
    """`scale_inputs` (src/dew/nn/moe.py:1124-1126, 1256-1259): the routing weight on each expert's input, the outputs
    summed unweighted. The reference's own vector (tests/fixtures/llama4/moe.npz: 32-wide tokens, 48-wide experts) padded
    with zeros to the launches' extents and held in bf16: the layer's output is the fixture's within bf16 arithmetic, and
    weighting the outputs instead is far from it. Then a seeded layer of kernel-sized FP8 banks against the oracle."""
    import dataclasses

    from conftest import golden
    from dew_amd import formats, moe

    tensors = golden("llama4/moe.npz")
    hidden = tensors["hidden"].reshape(-1, 32)
    gate_up = tensors["feed_forward.experts.gate_up_proj"]
    D, F = 128, 128

    def padded(matrix, rows, cols):      # [..., r, c] -> [..., rows, cols], zeros around
        out = np.zeros((*matrix.shape[:-2], rows, cols), np.float32)
        out[..., :matrix.shape[-2], :matrix.shape[-1]] = matrix
        return torch.from_numpy(out).to(torch.bfloat16)

    def bank(matrix, rows, cols):
        return {"kernel": formats.Bf16(padded(matrix, rows, cols)).to("cuda")}

    experts = {"gate_proj": bank(gate_up[..., :48], D, F), "up_proj": bank(gate_up[..., 48:], D, F),
               "down_proj": bank(tensors["feed_forward.experts.down_proj"], F, D)}
    shared = {name: bank(tensors[f"feed_forward.shared_expert.{name}.weight"].T[None], *((D, F) if name != "down_proj" else (F, D)))
              for name in ("gate_proj", "up_proj", "down_proj")}
    variables = {"params": {"gate": {"kernel": padded(tensors["feed_forward.router.weight"].T, D, 4).float().cuda()}},
                 "quantization": {"experts": experts, "shared_experts": shared}}
    x = padded(hidden, hidden.shape[0], D).cuda()
    layer = moe.SparseMLP(num_experts=4, top_k=2, hidden_features=F, out_features=D, score_function="sigmoid", normalize_weights=False,
                          shared=F, scale_inputs=True)
    got = layer.apply(variables, x).float().cpu().numpy()
    want = tensors["output"]
    assert not got[:, 32:].any()
    scale = np.abs(want).max()
    assert np.abs(got[:, :32] - want).max() <= 2e-2 * scale
    other = dataclasses.replace(layer, scale_inputs=False).apply(variables, x).float().cpu().numpy()
    assert np.abs(other[:, :32] - want).max() > 4 * np.abs(got[:, :32] - want).max()

    # a seeded layer at kernel sizes against the oracle: the same routing, rows scaled in bf16, unweighted sum
    case = CASES["c4-reduced"].scaled(tokens=200, shared=False)
    data = inputs(case, seed=8)
    layer, variables = layer_and_variables(case, data)
    layer = dataclasses.replace(layer, scale_inputs=True)
    got = layer.apply(variables, data["x"].cuda(), logits=data["logits"].cuda()).float().cpu().numpy()
    mats, factors = zip(*(dequantized(data["banks"][name]) for name in ("gate", "up", "down")), strict=True)
    want, _ = oracle.sparse_mlp(data["x"].float().numpy(), data["logits"].numpy(), *mats, top_k_count=case.top_k, factors=factors,
                                bias=data["bias"].numpy(), scale_inputs=True, **case.router)
    by_max, by_element = oracle.relative_errors(got, want)
    assert by_max <= 6e-3 and by_element <= TOLERANCE, (by_max, by_element)
    assert (got == want).mean() > 0.95


def test_nemotron_hs_ungated_relu2_experts():
    """`activation='relu2'` (src/dew/nn/moe.py:1250-1252, 1319-1322): up_proj, squared ReLU, down_proj. The
    reference's known answer (tests/test_moe_precision.py:652-674: experts answering 1 and -1 under weights 1/2 +- 2^-11
    give 2^-10), padded with zeros to the launches' extents; the activation on every bf16; a seeded layer of FP8 banks
    against the oracle."""
    from dew_amd import formats, moe, ops

    def one_hot(values):   # [E, 128, 128] bf16 banks whose [e, 0, 0] entries are `values`
        bank = torch.zeros((len(values), 128, 128), dtype=torch.bfloat16)
        bank[:, 0, 0] = torch.tensor(values, dtype=torch.bfloat16)
        return {"kernel": formats.Bf16(bank).to("cuda")}

    variables = {"params": {}, "quantization": {"up_proj": one_hot([1.0, 1.0]), "down_proj": one_hot([1.0, -1.0])}}
    x = torch.zeros((1, 128), dtype=torch.bfloat16)
    x[0, 0] = 1.0
    weights = torch.tensor([[0.5 + 2.0 ** -11, 0.5 - 2.0 ** -11]], dtype=torch.float32).cuda()
    indices = torch.tensor([[0, 1]], dtype=torch.int32).cuda()
    out = moe.ExpertMLP(2, 128, 128, activation="relu2").apply(variables, x.cuda(), weights, indices)
    assert out.dtype == torch.bfloat16 and float(out[0, 0]) == 2.0 ** -10 and not bool(out[0, 1:].any())

    every = (torch.arange(1 << 16, dtype=torch.int32) << 16).view(torch.float32)
    every = every[torch.isfinite(every)].to(torch.bfloat16)
    every = every[: every.numel() // 8 * 8]
    got = ops.relu2(every.cuda()).float().cpu().numpy()
    want = oracle.relu2(every.float().numpy())
    finite = np.isfinite(want)
    assert np.array_equal(got[finite], want[finite]) and np.all(np.isinf(got[~finite]))

    rng = np.random.default_rng(21)
    tokens, experts, top_k, width, hidden = 300, 8, 2, 256, 512
    from bench_aids.workloads import quantize
    xs = torch.from_numpy(rng.standard_normal((tokens, width)).astype(np.float32)).to(torch.bfloat16)
    banks = {name: quantize(torch.from_numpy((rng.standard_normal((experts, d, w)) * 0.08).astype(np.float32)), "fp8_block")
             for name, (d, w) in (("up", (width, hidden)), ("down", (hidden, width)))}
    logits = rng.standard_normal((tokens, experts)).astype(np.float32)
    weights, indices = ops.route(torch.from_numpy(logits).cuda(), top_k)
    variables = {"params": {}, "quantization": {f"{n}_proj": {"kernel": bank.to("cuda")} for n, bank in banks.items()}}
    got = moe.ExpertMLP(experts, hidden, width, activation="relu2").apply(variables, xs.cuda(), weights, indices).float().cpu().numpy()
    (up_values, _), (down_values, _) = dequantized(banks["up"]), dequantized(banks["down"])
    want, _ = oracle.expert_mlp(xs.float().numpy(), weights.cpu().numpy(), indices.cpu().numpy(), None, up_values, down_values, activation="relu2")
    by_max, by_element = oracle.relative_errors(got, want)
    assert by_max <= 6e-3 and by_element <= TOLERANCE, (by_max, by_element)
    assert (got == want).mean() > 0.97
    with pytest.raises(ValueError, match="relu2 experts have none"):
        moe.ExpertMLP(experts, hidden, width, activation="relu2", swiglu_limit=1.0)


@pytest.mark.parametrize("switches", [dict(weight_sum_min=7.5), dict(bias_in_weights=True), dict(excluded_group_score=0.9),
                                      dict(weight_sum_epsilon=0.5)],
                         ids=["ernie-sum-floor", "llada-bias-in-weights", "filled-groups", "wide-epsilon"])
def test_the_layer_hands_the_routers_further_switches_to_its_router(switches):
    """ERNIE 4.5's floor under the chosen weights' sum, LLaDA-MoE's biased weights, a fill for excluded groups (A.X-K2's switch)
    and a sum epsilon of the caller's (`SparseMLP`'s fields of src/dew/nn/moe.py:1391-1396): the whole layer against
    the oracle under the same switches, the routing bit for bit."""
    import dataclasses

    case = CASES["c4-reduced"].scaled(tokens=160, shared=False)
    data = inputs(case, seed=12)
    layer, variables = layer_and_variables(case, data)
    layer = dataclasses.replace(layer, **switches)
    sown = {}
    weights, indices = layer._bound(variables, ()).gate.routed(data["logits"].cuda(), sown)
    want_w, want_i = oracle.route(data["logits"].numpy(), case.top_k, bias=data["bias"].numpy(), **case.router, **switches)
    assert np.array_equal(indices.cpu().numpy(), want_i)
    assert np.array_equal(weights.cpu().numpy().view(np.uint32), want_w.view(np.uint32))
    plain_w, plain_i = oracle.route(data["logits"].numpy(), case.top_k, bias=data["bias"].numpy(), **case.router)
    assert not (np.array_equal(plain_w, want_w) and np.array_equal(plain_i, want_i))      # the switch switches something
    got = layer.apply(variables, data["x"].cuda(), logits=data["logits"].cuda()).float().cpu().numpy()
    mats, factors = zip(*(dequantized(data["banks"][name]) for name in ("gate", "up", "down")), strict=True)
    want, _ = oracle.sparse_mlp(data["x"].float().numpy(), data["logits"].numpy(), *mats, top_k_count=case.top_k, factors=factors,
                                bias=data["bias"].numpy(), **case.router, **switches)
    by_max, by_element = oracle.relative_errors(got, want)
    assert by_max <= 6e-3 and by_element <= TOLERANCE, (by_max, by_element)


def test_the_layers_router_softcap_is_its_routers_logit_softcap():
    from dew_amd import moe
    layer = moe.SparseMLP(num_experts=8, top_k=2, hidden_features=128, out_features=128, router_softcap=30.0)
    assert layer._bound({}, ()).gate.logit_softcap == 30.0
    with pytest.raises(ValueError, match="positive cap"):
        moe.Router(8, 128, 2, logit_softcap=0.0)
    with pytest.raises(ValueError, match="expert_bias holds"):
        moe.Router(8, 128, 2, bias_in_weights=True)


@pytest.mark.parametrize("fuse_shared", [True, False])
def test_qwen2_moes_gate_on_the_shared_expert(fuse_shared):
    """`shared_gate` (src/dew/nn/moe.py:1469-1475, 1499-1502) under the bf16 compute dtype: the kernel alone against the
    oracle, bit for bit on a few thousand tokens (the logit's sum in float64 on both sides, the same fixed-sequence
    exponential and IEEE division), the oracle's hand case on the device, and the whole layer with the shared expert inside
    the routed launches and beside them."""
    import dataclasses

    from dew_amd import ops
    rng = np.random.default_rng(41)
    x = torch.from_numpy(rng.standard_normal((4333, 512)).astype(np.float32)).to(torch.bfloat16)
    kernel = (rng.standard_normal(512) * 0.05).astype(np.float32)
    rows = torch.from_numpy(rng.standard_normal((4333, 256)).astype(np.float32)).to(torch.bfloat16)
    got = ops.gate_rows(x.cuda(), torch.from_numpy(kernel).cuda(), rows.cuda()).float().cpu().numpy()
    want = oracle.gated_rows(x.float().numpy(), kernel, rows.float().numpy())
    assert np.array_equal(got, want)
    hand_x = torch.zeros((1, 8), dtype=torch.bfloat16)
    hand_x[0, 0] = 1.0
    hand = ops.gate_rows(hand_x.cuda(), torch.full((8,), 0.3).cuda(), torch.tensor([[3.0, -1.0, 0, 0, 0, 0, 0, 0]], dtype=torch.bfloat16).cuda())
    assert hand[0, :2].float().cpu().tolist() == [1.71875, -0.57421875]

    case = CASES["c4-reduced"].scaled(tokens=200)
    data = inputs(case, seed=13)
    layer, variables = layer_and_variables(case, data)
    gate = (rng.standard_normal(case.d_model) * 0.05).astype(np.float32)
    variables["params"]["shared_expert_gate"] = {"kernel": torch.from_numpy(gate).reshape(-1, 1).cuda()}
    layer = dataclasses.replace(layer, shared_gate=True, fuse_shared=fuse_shared, dtype=torch.bfloat16)
    got = layer.apply(variables, data["x"].cuda(), logits=data["logits"].cuda()).float().cpu().numpy()
    mats, factors = zip(*(dequantized(data["banks"][name]) for name in ("gate", "up", "down")), strict=True)
    shared = [dequantized(data["shared"][name])[0][0] for name in ("gate", "up", "down")]
    want, _ = oracle.sparse_mlp(data["x"].float().numpy(), data["logits"].numpy(), *mats, top_k_count=case.top_k, factors=factors,
                                bias=data["bias"].numpy(), shared=shared, shared_gate=gate, **case.router)
    ungated, _ = oracle.sparse_mlp(data["x"].float().numpy(), data["logits"].numpy(), *mats, top_k_count=case.top_k, factors=factors,
                                   bias=data["bias"].numpy(), shared=shared, **case.router)
    by_max, by_element = oracle.relative_errors(got, want)
    assert by_max <= 6e-3 and by_element <= TOLERANCE, (by_max, by_element)
    assert oracle.relative_errors(got, ungated)[0] > 10 * by_max                 # the gate gates
    widened = dataclasses.replace(layer, dtype=None).apply(variables, data["x"].cuda(), logits=data["logits"].cuda())
    assert widened.dtype == torch.float32                                        # (no compute dtype: the gate's fp32, see the next test)
    with pytest.raises(ValueError, match="requires a shared expert"):
        dataclasses.replace(layer, shared=None).apply(variables, data["x"].cuda(), logits=data["logits"].cuda())


def test_qwen2_moes_gate_in_float32_widens_the_layers_output():
    """`shared_gate` where the layer states no compute dtype (src/dew/nn/moe.py:1469-1475, 1497-1503): the gate's `Dense(1)`
    runs in the fp32 of its kernel, and routed + shared * gate comes back fp32. The kernel alone against the oracle, bit for
    bit (the logit's sum in float64 on both sides, then the same fp32 steps) and against float64 within two fp32 roundings;
    then the whole layer, whose routed and shared rows are the bf16 layer's."""
    import dataclasses

    from dew_amd import ops
    rng = np.random.default_rng(43)
    x = torch.from_numpy(rng.standard_normal((1777, 512)).astype(np.float32)).to(torch.bfloat16)
    kernel = (rng.standard_normal(512) * 0.05).astype(np.float32)
    shared, routed = (torch.from_numpy(rng.standard_normal((1777, 256)).astype(np.float32)).to(torch.bfloat16) for _ in range(2))
    got = ops.gate_rows_add_f32(x.cuda(), torch.from_numpy(kernel).cuda(), shared.cuda(), routed.cuda())
    assert got.dtype == torch.float32
    got = got.cpu().numpy()
    want = oracle.gated_rows_added_f32(x.float().numpy(), kernel, shared.float().numpy(), routed.float().numpy())
    assert np.array_equal(got, want)
    exact = routed.double().numpy() + shared.double().numpy() / (1.0 + np.exp(-(x.double().numpy() @ kernel.astype(np.float64))))[:, None]
    assert np.abs(got - exact).max() <= 4e-7 * np.abs(exact).max()

    case = CASES["c4-reduced"].scaled(tokens=200)
    data = inputs(case, seed=14)
    layer, variables = layer_and_variables(case, data)
    gate = (rng.standard_normal(case.d_model) * 0.05).astype(np.float32)
    variables["params"]["shared_expert_gate"] = {"kernel": torch.from_numpy(gate).reshape(-1, 1).cuda()}
    layer = dataclasses.replace(layer, shared_gate=True)        # no dtype
    out = layer.apply(variables, data["x"].cuda(), logits=data["logits"].cuda())
    assert out.dtype == torch.float32 and out.shape == data["x"].shape
    mats, factors = zip(*(dequantized(data["banks"][name]) for name in ("gate", "up", "down")), strict=True)
    apart = oracle.gated_mlp(data["x"].float().numpy(), *(dequantized(data["shared"][name])[0][0] for name in ("gate", "up", "down")))
    alone, _ = oracle.sparse_mlp(data["x"].float().numpy(), data["logits"].numpy(), *mats, top_k_count=case.top_k, factors=factors,
                                 bias=data["bias"].numpy(), **case.router)
    want = oracle.gated_rows_added_f32(data["x"].float().numpy(), gate, apart, alone)
    by_max, by_element = oracle.relative_errors(out.cpu().numpy(), want)
    assert by_max <= 6e-3 and by_element <= TOLERANCE, (by_max, by_element)
    with pytest.raises(ValueError, match="runs in bfloat16"):
        dataclasses.replace(layer, dtype=torch.float16).apply(variables, data["x"].cuda(), logits=data["logits"].cuda())


@pytest.mark.parametrize("with_norm,shared_gate", [(False, False), (True, False), (True, True)])
def test_kimis_latent_experts(with_norm, shared_gate):
    """`latent_features` (src/dew/nn/moe.py:1379-1385, 1458-1467, 1491-1496): the router reads the full width, a dense down
    projection narrows the tokens to the experts' width, their combined rows go through the norm and a dense up projection,
    and the shared expert, which reads the full width, is added behind it. Against the oracle's pieces in that order."""
    from dew_amd import moe
    full_width = 1536
    narrow = CASES["c4-reduced"].scaled(tokens=200)                        # the experts: latent width 1024
    data = inputs(narrow, seed=15)
    full = inputs(narrow.scaled(d_model=full_width), seed=16)              # the tokens and the shared expert at the full width
    rng = np.random.default_rng(44)
    down = torch.from_numpy((rng.standard_normal((full_width, narrow.d_model)) * 0.03).astype(np.float32)).to(torch.bfloat16)
    up = torch.from_numpy((rng.standard_normal((narrow.d_model, full_width)) * 0.03).astype(np.float32)).to(torch.bfloat16)
    scale = torch.from_numpy(rng.uniform(0.5, 2.0, narrow.d_model).astype(np.float32))
    norm = (lambda params, rows: (rows.float() * params["scale"]).to(torch.bfloat16)) if with_norm else None
    layer = moe.SparseMLP(num_experts=narrow.experts, top_k=narrow.top_k, hidden_features=narrow.d_ff, out_features=full_width,
                          expert_bias=True, shared=narrow.d_ff, latent_features=narrow.d_model, latent_norm=norm, shared_gate=shared_gate,
                          dtype=torch.bfloat16, **narrow.router)
    variables = {"params": {"routed_expert_down_proj": {"kernel": down.cuda()}, "routed_expert_up_proj": {"kernel": up.cuda()},
                            "routed_expert_norm": {"scale": scale.cuda()}},
                 "quantization": {"experts": {f"{n}_proj": {"kernel": b.to("cuda")} for n, b in data["banks"].items()},
                                  "shared_experts": {f"{n}_proj": {"kernel": b.to("cuda")} for n, b in full["shared"].items()}},
                 "moe": {"gate": {"e_score_correction_bias": data["bias"].cuda()}}}
    gate = (rng.standard_normal(full_width) * 0.05).astype(np.float32)
    if shared_gate:
        variables["params"]["shared_expert_gate"] = {"kernel": torch.from_numpy(gate).reshape(-1, 1).cuda()}
    got = layer.apply(variables, full["x"].cuda(), logits=data["logits"].cuda())
    assert got.dtype == torch.bfloat16 and got.shape == full["x"].shape
    assert layer._bound(variables, ()).experts.out_features == narrow.d_model

    x = full["x"].float().numpy()
    everyone = [x.shape[0]]
    narrowed = oracle.grouped_matmul(x, down.float().numpy()[None], everyone)
    mats, factors = zip(*(dequantized(data["banks"][name]) for name in ("gate", "up", "down")), strict=True)
    weights, indices = oracle.route(data["logits"].numpy(), narrow.top_k, bias=data["bias"].numpy(), **narrow.router)
    routed, _ = oracle.expert_mlp(narrowed, weights, indices, *mats, factors=factors)
    if with_norm:
        routed = oracle.bf16_round(routed * scale.numpy())
    widened = oracle.grouped_matmul(routed, up.float().numpy()[None], everyone)
    apart = oracle.gated_mlp(x, *(dequantized(full["shared"][name])[0][0] for name in ("gate", "up", "down")))
    if shared_gate:
        apart = oracle.gated_rows(x, gate, apart)
    want = oracle.bf16_round(widened + apart)
    by_max, by_element = oracle.relative_errors(got.float().cpu().numpy(), want)
    # (five chained roundings: one bf16 ulp of the largest output is up to 7.8e-3 of it)
    assert by_max <= 8e-3 and by_element <= TOLERANCE, (by_max, by_element)
    without = dataclasses_replace(layer, shared=None, shared_gate=False).apply(variables, full["x"].cuda(), logits=data["logits"].cuda())
    assert oracle.relative_errors(without.float().cpu().numpy(), widened)[1] <= TOLERANCE
    with pytest.raises(ValueError, match="states no compute dtype"):
        float_kernels = {**variables, "params": {**variables["params"], "routed_expert_down_proj": {"kernel": down.float().cuda()}}}
        dataclasses_replace(layer, dtype=None).apply(float_kernels, full["x"].cuda(), logits=data["logits"].cuda())


def test_a_captured_layer_replays_to_the_eager_result():
    """The whole layer (gate GEMM, router, sort, the grouped launches, combine, the shared expert's gate) and a block
    router's four launches recorded into one HIP graph: every replay, on new inputs and with eager work and
    synchronizations between the replays, returns the eager call's bits. (Nothing in these paths clears memory with a
    memset node: the counters and keys that start at zero are cleared by kernels.)"""
    import dataclasses

    from dew_amd import moe, ops
    case = CASES["c4-reduced"].scaled(tokens=48)
    data = inputs(case, seed=21)
    layer, variables = layer_and_variables(case, data)
    rng = np.random.default_rng(5)
    variables["params"]["gate"] = {"kernel": torch.from_numpy((rng.standard_normal((case.d_model, case.experts)) * 0.05).astype(np.float32)).cuda()}
    variables["params"]["shared_expert_gate"] = {"kernel": torch.from_numpy((rng.standard_normal((case.d_model, 1)) * 0.05).astype(np.float32)).cuda()}
    layer = dataclasses.replace(layer, shared_gate=True, dtype=torch.bfloat16)
    block_router = moe.Router(case.experts, case.d_model, case.top_k, score_function="sigmoid", routing_block=8, block_experts=24)._bound(variables, ("gate",))
    blocks = (torch.arange(48, dtype=torch.int32) // 8).reshape(1, 48).cuda()
    xs = [torch.from_numpy(rng.standard_normal((48, case.d_model)).astype(np.float32)).to(torch.bfloat16).cuda() for _ in range(3)]

    def step(x):
        out = layer.apply(variables, x)
        weights, indices = block_router.chosen(block_router.logits(x)[None], blocks=blocks)
        return out, weights, indices

    eager = [tuple(t.clone() for t in step(x)) for x in xs]
    held = xs[0].clone()
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        step(held)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            recorded = step(held)
    torch.cuda.synchronize()
    for turn in (0, 1, 2, 1, 0):
        held.copy_(xs[turn])
        graph.replay()
        torch.cuda.synchronize()
        for got, want in zip(recorded, eager[turn], strict=True):
            assert torch.equal(got, want), turn
        step(xs[(turn + 1) % 3])                     # the program's own eager work between the replays
        torch.cuda.synchronize()


@pytest.mark.parametrize("name,tokens", [("c2-reduced", 2048), ("c5-reduced", 300), ("c1-full", 256)])
def test_captured_layers_of_the_other_formats_replay_to_the_eager_result(name, tokens):
    """The MXFP4 layer on split rows (its workspace comes from the caller's allocator, here the graph's pool), the NVFP4
    and the per-channel FP8 layers: recorded once, replayed on new inputs between eager calls, the eager bits each time."""
    case = CASES[name].scaled(tokens=tokens)
    data = inputs(case, seed=22)
    layer, variables = layer_and_variables(case, data)
    rng = np.random.default_rng(6)
    xs = [torch.from_numpy(rng.standard_normal((tokens, case.d_model)).astype(np.float32)).to(torch.bfloat16).cuda() for _ in range(2)]
    logits = [torch.from_numpy(rng.standard_normal((tokens, case.experts)).astype(np.float32)).cuda() for _ in range(2)]
    eager = [layer.apply(variables, x, logits=l).clone() for x, l in zip(xs, logits, strict=True)]
    held_x, held_l = xs[0].clone(), logits[0].clone()
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        layer.apply(variables, held_x, logits=held_l)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            recorded = layer.apply(variables, held_x, logits=held_l)
    torch.cuda.synchronize()
    for turn in (0, 1, 1, 0):
        held_x.copy_(xs[turn]), held_l.copy_(logits[turn])
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(recorded, eager[turn]), turn
        layer.apply(variables, xs[1 - turn], logits=logits[1 - turn])
        torch.cuda.synchronize()

"""The benchmark configurations at their full sizes, where the CPU oracle cannot follow the whole layer: checked
through properties that do not depend on size (the sort's invariants, the router on a sample of tokens, the combine
recomputed from the slots, bit-identical repeats) and against the oracle on a bounded sample of rows at full width:
the first and last rows of three experts (the busiest, the median, the least non-empty one), and c3 whole. Inputs are generated on the device exactly as the benchmark generates them."""

import numpy as np
import pytest
import torch
from bench_aids.workloads import CONFIGS

import bench
from oracle import moe_oracle as oracle

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("name", ["c2", "c3", "c4", "c5"])
def test_full_size_configuration(name):
    case = CONFIGS[name]
    device = torch.device("cuda:0")
    data = bench.build_workload(case, device)
    stepper = bench.Stepper(case, data)
    out, plan = stepper()
    again, _ = stepper()
    assert torch.equal(out, again)                                  # no atomics, no order left to chance
    tokens, k, experts = case.tokens, case.top_k, case.experts
    routed = tokens * k

    # the router, bit for bit, on the first 256 tokens
    from dew_amd import ops
    weights, indices = ops.route(data["logits"], k, bias=data["bias"], **case.router)
    sample = slice(0, min(256, tokens))
    want_weights, want_indices = oracle.route(data["logits"][sample].cpu().numpy(), k,
                                              bias=None if data["bias"] is None else data["bias"].cpu().numpy(), **case.router)
    assert np.array_equal(indices[sample].cpu().numpy(), want_indices)
    assert np.array_equal(weights[sample].cpu().numpy(), want_weights)
    assert int(indices.min()) >= 0 and int(indices.max()) < experts
    ordered = torch.sort(indices, dim=-1).values
    assert bool((ordered[:, 1:] != ordered[:, :-1]).all())          # a token's experts are distinct

    # the stable sort by expert: a permutation, experts non-decreasing, slots ascending inside an expert
    flat = indices.reshape(-1)
    shared_rows = tokens if stepper.fused_shared else 0
    assert stepper.fused_shared == case.shared                      # c4's shared expert rides the routed launches as group #E
    order = plan.order.long()
    assert torch.equal(torch.sort(order).values, torch.arange(routed + shared_rows, device=device))
    if shared_rows:   # the shared group: behind the routed slots, one row a token in token order
        assert torch.equal(order[routed:], torch.arange(routed, routed + tokens, device=device))
        assert torch.equal(plan.rows[routed:].long(), torch.arange(tokens, device=device))
        assert int(plan.sizes[experts]) == tokens and int(plan.offsets[experts + 1]) == routed + tokens
        plan = type(plan)(plan.order[:routed], plan.rows[:routed], plan.sizes[:experts], plan.offsets[:experts + 1])
        order = plan.order.long()
    sorted_experts = flat[order]
    assert bool((sorted_experts[1:] >= sorted_experts[:-1]).all())
    same = sorted_experts[1:] == sorted_experts[:-1]
    assert bool((order[1:][same] > order[:-1][same]).all())
    assert torch.equal(plan.sizes.long(), torch.bincount(flat.long(), minlength=experts))
    assert torch.equal(plan.offsets.long(), torch.cat([torch.zeros(1, dtype=torch.long, device=device), torch.cumsum(plan.sizes.long(), 0)]))
    assert torch.equal(plan.rows.long(), order // k)

    # first and last rows of the busiest, the median and the least non-empty expert through all three projections against the
    # oracle (a group's last rows are the ones a partial last tile, or c4's second launch of 64-row tiles, multiplies); c3,
    # whose experts hold 1 to 10 rows, is followed whole: every routed row, the routing and the layer's output
    _, whole_plan = stepper()
    slots = stepper.project(whole_plan)                             # c2: on split rows, the library's rule for its groups
    assert stepper.on_split_rows() == (name == "c2")
    if name in bench.WHOLE_ON_CPU:
        _, (want_out_oracle, trace) = bench.oracle_whole(case, data)
        assert np.array_equal(indices.cpu().numpy(), trace["indices"]) and np.array_equal(weights.cpu().numpy(), trace["weights"])
        got_down, want_down = slots[:routed].float().cpu().numpy(), trace["slots"].reshape(routed, case.d_model)
        sampled_experts = list(range(experts))
        peak, elementwise = oracle.relative_errors(out.float().cpu().numpy(), want_out_oracle)
        assert peak <= 6e-3 and elementwise <= 2e-2, (peak, elementwise)
    else:
        _, (sampled_slots, want_down, sampled_experts) = bench.oracle_sample(case, data, plan, budget_rows=64)
        got_down = slots[torch.from_numpy(sampled_slots).to(device).long()].float().cpu().numpy()
        assert len(sampled_experts) == 3
    assert len(want_down) >= 64
    peak, elementwise = oracle.relative_errors(got_down, want_down)
    assert peak <= 2e-2 and elementwise <= 2e-2, (peak, elementwise)
    assert peak <= 6e-3
    total = torch.zeros((tokens, case.d_model), dtype=torch.float32, device=device)
    view = slots[:routed].view(tokens, k, case.d_model)
    for j in range(k):
        total = total + view[:, j, :].float() * weights[:, j, None]
    want_out = total.to(torch.bfloat16)
    if case.shared:
        # the shared expert's rows (group #E of the same launches) against the oracle's dense SwiGLU MLP on a sample of tokens
        from oracle.banks import dequantized
        sampled = np.arange(0, tokens, tokens // 24)[:24]
        matrices = [dequantized(data["shared"][n].to("cpu"))[0][0] for n in ("gate", "up", "down")]
        want_shared = oracle.gated_mlp(data["x"][torch.from_numpy(sampled).to(device)].float().cpu().numpy(), *matrices)
        got_shared = slots[routed:][torch.from_numpy(sampled).to(device)].float().cpu().numpy()
        peak, elementwise = oracle.relative_errors(got_shared, want_shared)
        assert peak <= 6e-3 and elementwise <= 2e-2, (peak, elementwise)
        want_out = (want_out.float() + slots[routed:].float()).to(torch.bfloat16)
    assert torch.equal(out, want_out)


@pytest.mark.parametrize("recipe", ["blockwise_fp8", "mxfp8", "bf16"])
def test_full_size_kernel_gradient_partitions_its_tokens(recipe):
    """Mixtral-8x7B's gate projection at the benchmark's routed rows (32768 x 4096 x 14336), where no CPU sum follows:
    the gradient of one group holding every token is the sum of the eight groups' gradients (the same products in
    other windows: fp32 rounding of the sums apart), a group's gradient does not depend on its neighbours, and a
    sample of its elements is the oracle's exact sum of the same quantized operands."""
    from dew_amd import gemm, ops, projections

    device = torch.device("cuda:0")
    generator = torch.Generator(device=device).manual_seed(0)
    tokens, depth, width, groups = 32768, 4096, 14336, 8
    x = torch.randn((tokens, depth), device=device, generator=generator).to(torch.bfloat16)
    dy = torch.randn((tokens, width), device=device, generator=generator).to(torch.bfloat16)
    each = tokens // groups // 128
    if recipe == "bf16":
        gradient = lambda blocks: gemm.gemm_t(x, dy, torch.tensor(blocks, dtype=torch.int32, device=device) * 128,
                                              out_dtype=torch.float32, whole_steps=True)
    else:
        gradient = lambda blocks: projections.kernel_gradient(x, dy, blocks, mx=recipe == "mxfp8", out_dtype=torch.float32)
    apart = gradient([each] * groups)
    whole = gradient([each * groups])[0]
    scale = float(whole.abs().max())
    assert float((apart.sum(dim=0) - whole).abs().max()) <= 2.0 ** -12 * scale
    uneven = gradient([each, 0, 2 * each, each] + [each] * (groups - 4))
    assert torch.equal(uneven[0], apart[0]) and not bool(uneven[1].any()) and torch.equal(uneven[3], apart[3])
    # group 5's first 64 x 64 elements against the exact sums of the same operands
    span = slice(5 * each * 128, 6 * each * 128)
    left, right = x[span, :64].float().cpu().numpy(), dy[span, :64].float().cpu().numpy()
    if recipe == "bf16":
        want = oracle.kernel_gradient(left.T, right.T, [each * 128], dtype="float32")[0]
    elif recipe == "mxfp8":
        want = oracle.kernel_gradient(oracle.mxfp8_decoded(*oracle.mxfp8_quantized(left.T)), oracle.mxfp8_decoded(*oracle.mxfp8_quantized(right.T)),
                                      [each * 128], dtype="float32")[0]
    else:
        (lv, ls), (rv, rs) = oracle.rows_quantized(left.T), oracle.rows_quantized(right.T)
        want = oracle.blockwise_fp8_kernel_gradient(lv, rv, [each], ls.T, rs.T, dtype="float32")[0]
    got = apart[5, :64, :64].cpu().numpy()
    assert np.abs(got - want).max() <= 2.0 ** -12 * np.abs(want).max()

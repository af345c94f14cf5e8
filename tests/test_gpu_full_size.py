"""The benchmark configurations at their full sizes, where the CPU oracle cannot follow the whole layer: checked
through properties that do not depend on size (the sort's invariants, the router on a sample of tokens, the combine
recomputed from the slots, bit-identical repeats) and against the oracle on a bounded sample of rows of the busiest
expert at full width. Inputs are generated on the device exactly as the benchmark generates them."""

import numpy as np
import pytest
import torch
from moe_cases import CONFIGS

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
    order = plan.order.long()
    assert torch.equal(torch.sort(order).values, torch.arange(routed, device=device))
    sorted_experts = flat[order]
    assert bool((sorted_experts[1:] >= sorted_experts[:-1]).all())
    same = sorted_experts[1:] == sorted_experts[:-1]
    assert bool((order[1:][same] > order[:-1][same]).all())
    assert torch.equal(plan.sizes.long(), torch.bincount(flat.long(), minlength=experts))
    assert torch.equal(plan.offsets.long(), torch.cat([torch.zeros(1, dtype=torch.long, device=device), torch.cumsum(plan.sizes.long(), 0)]))
    assert torch.equal(plan.rows.long(), order // k)

    # the busiest expert's first rows through all three projections against the oracle, and the combine from the slots
    _, (sampled_slots, want_down) = bench.cpu_baseline(case, data, out, plan, budget_rows=48)
    slots = stepper.project(plan)                                   # c2: on split rows, the library's rule for its groups
    assert stepper.on_split_rows() == (name == "c2")
    got_down = slots[torch.from_numpy(sampled_slots).to(device).long()].float().cpu().numpy()
    peak, elementwise = oracle.relative_errors(got_down, want_down)
    assert peak <= 2e-2 and elementwise <= 2e-2, (peak, elementwise)
    assert peak <= 6e-3
    total = torch.zeros((tokens, case.d_model), dtype=torch.float32, device=device)
    view = slots.view(tokens, k, case.d_model)
    for j in range(k):
        total = total + view[:, j, :].float() * weights[:, j, None]
    want_out = total.to(torch.bfloat16)
    if case.shared:
        dense = ops.gateup_swiglu(data["x"], stepper.shared[0], stepper.shared[1], stepper.dense_offsets)
        want_out = (want_out.float() + ops.grouped_gemm(dense, stepper.shared[2], stepper.dense_offsets).float()).to(torch.bfloat16)
    assert torch.equal(out, want_out)

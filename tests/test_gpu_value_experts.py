"""Routed value experts (`dew_amd.value_experts.RoutedValues`, the reference's src/dew/nn/value_experts.py) on the device
against the CPU oracle: the router and the sort bit for bit, the stand-alone SiLU bit for bit on every bf16, the layer's
output within the bars of the expert MLP's tests."""

import numpy as np
import pytest
import torch
from bench_aids.workloads import quantize
from oracle.banks import dequantized

from oracle import moe_oracle as oracle

pytestmark = pytest.mark.gpu


def test_the_silu_kernel_matches_the_oracle_on_every_bf16():
    from dew_amd import ops

    every = oracle.bf16_from_bits(np.arange(65536, dtype=np.uint16))
    every = every[np.isfinite(every)]
    every = np.concatenate([every, np.zeros(-every.size % 8, np.float32)])
    got = ops.silu(torch.from_numpy(every).to(torch.bfloat16).cuda()).float().cpu().numpy()
    want = oracle.silu(every)
    mismatched = got != want
    # the hardware's exp2 and reciprocal against NumPy's exp: a last bf16 bit, rarely (the stand-alone SwiGLU's own bar)
    assert mismatched.mean() < 2e-3
    assert np.abs(got - want)[mismatched].max(initial=0) <= 2 ** -7 * np.abs(want)[mismatched].max(initial=1)
    assert np.array_equal(got, ops.swiglu(torch.from_numpy(every).to(torch.bfloat16).cuda(),
                                          torch.ones(every.size, dtype=torch.bfloat16, device="cuda")).float().cpu().numpy())
    assert torch.equal(ops.silu(torch.zeros(8, dtype=torch.bfloat16, device="cuda")), torch.zeros(8, dtype=torch.bfloat16, device="cuda"))


@pytest.mark.parametrize("quant,experts,top_k,tokens,score_function,bias", [
    ("bf16", 4, 2, 77, "sigmoid", True),          # K2 Horizon MoVA's own router: sigmoid scores, a selection bias, renormalized
    ("fp8_block", 8, 2, 300, "sigmoid", False),
    ("mxfp4", 16, 4, 129, "softmax", False),
    ("bf16", 4, 4, 1, "sigmoid", True),           # one token that takes every expert
])
def test_routed_values_match_the_oracle(quant, experts, top_k, tokens, score_function, bias):
    from dew_amd import value_experts

    rng = np.random.default_rng(experts * 100 + tokens)
    in_features, features = 256, 128 if quant != "mxfp4" else 256
    x = torch.from_numpy(rng.standard_normal((tokens, in_features)).astype(np.float32)).to(torch.bfloat16)
    router_kernel = (rng.standard_normal((in_features, experts)) * 0.1).astype(np.float32)
    selection_bias = (rng.standard_normal(experts) * 0.05).astype(np.float32) if bias else None
    weight = torch.from_numpy((rng.standard_normal((experts, in_features, features)) * 0.05).astype(np.float32))
    bank = quantize(weight, quant)
    spec = value_experts.ValueExperts(experts, top_k, score_function=score_function, norm_topk_prob=True, scaling=1.5, bias=bias)
    layer = value_experts.RoutedValues(spec, in_features, features)
    variables = {"params": {"v_router": {"kernel": torch.from_numpy(router_kernel).cuda()}},
                 "quantization": {"v_proj": {"kernel": bank.to("cuda")}}}
    if bias:
        variables["moe"] = {"v_router": {"e_score_correction_bias": torch.from_numpy(selection_bias).cuda()}}
    got = layer.apply(variables, x.cuda()).float().cpu().numpy()

    logits = oracle.router_logits(x.float().numpy(), router_kernel)
    weights, indices = oracle.route(logits, top_k, score_function=score_function, normalize_weights=True, bias=selection_bias,
                                    routed_scaling_factor=1.5)
    values, factor = dequantized(bank)
    want, _ = oracle.routed_values(x.float().numpy(), weights, indices, values, factor=factor)
    assert got.shape == (tokens, features)
    by_max, by_element = oracle.relative_errors(got, want)
    assert by_max <= 6e-3 and by_element <= 2e-2, (by_max, by_element)
    assert (got == want).mean() > 0.97


def test_value_experts_refuse_a_top_k_outside_their_experts():
    from dew_amd import value_experts

    with pytest.raises(ValueError, match="top_k"):
        value_experts.ValueExperts(4, 5)

"""Pins the CPU oracle against the golden vectors the reference's own tests hold, and against what the
mathematics fixes, so that a dropped term, a wrong sign or a transposed operand fails here."""

import numpy as np
import pytest
from conftest import golden

from oracle import moe_oracle as oracle

ROUTER_TOLERANCE = 1e-6      # tests/test_moe.py:37 of the reference
OUTPUT_TOLERANCE = 2e-5      # tests/test_moe.py:40


def by_expert(indices, weights):
    order = np.argsort(indices, axis=-1, kind="stable")
    return np.take_along_axis(indices, order, -1), np.take_along_axis(weights, order, -1)


def stacked(tensors, projection, experts):
    return np.stack([tensors[f"mlp.experts.{e}.{projection}.weight"].T for e in range(experts)])


ROUTERS = {
    "mixtral": dict(score_function="softmax", normalize_weights=True),
    "deepseek": dict(score_function="sigmoid", normalize_weights=True, routed_scaling_factor=2.5,
                     expert_groups=4, groups_per_token=2, biased=True),
    "deepseek_v2": dict(score_function="softmax", normalize_weights=False, routed_scaling_factor=2.5,
                        expert_groups=4, groups_per_token=2, group_score="max"),
    "deepseek_v4": dict(score_function="sqrtsoftplus", normalize_weights=True, routed_scaling_factor=2.5,
                        biased=True),
}


def routed(name):
    tensors = golden(f"moe/{name}.npz")
    settings = dict(ROUTERS[name])
    bias = tensors["mlp.gate.e_score_correction_bias"] if settings.pop("biased", False) else None
    hidden = tensors["hidden"].reshape(-1, tensors["hidden"].shape[-1])
    logits = oracle.router_logits(hidden, tensors["mlp.gate.weight"].T)
    k = tensors["router_indices"].shape[-1]
    return tensors, hidden, logits, k, dict(settings, bias=bias)


@pytest.mark.parametrize("name", list(ROUTERS))
def test_router_reproduces_the_recorded_choice_and_gate_values(name):
    tensors, _, logits, k, settings = routed(name)
    weights, indices = oracle.route(logits, k, **settings)
    theirs_i, theirs_w = by_expert(tensors["router_indices"], tensors["router_weights"])
    ours_i, ours_w = by_expert(indices, weights)
    assert np.array_equal(ours_i, theirs_i)
    assert np.abs(ours_w - theirs_w).max() < ROUTER_TOLERANCE


def test_fp32_block_reproduces_the_mixtral_block_output():
    tensors, hidden, logits, k, settings = routed("mixtral")
    mats = [stacked(tensors, p, 8) for p in ("gate_proj", "up_proj", "down_proj")]
    out, _ = oracle.sparse_mlp(hidden, logits, *mats, top_k_count=k, dtype="float32", **settings)
    assert np.abs(out - tensors["block_output"].reshape(out.shape)).max() < OUTPUT_TOLERANCE


def test_fp32_block_reproduces_the_deepseek_block_output_with_its_shared_expert():
    tensors, hidden, logits, k, settings = routed("deepseek")
    mats = [stacked(tensors, p, 8) for p in ("gate_proj", "up_proj", "down_proj")]
    shared = [tensors[f"mlp.shared_experts.{p}.weight"].T for p in ("gate_proj", "up_proj", "down_proj")]
    out, _ = oracle.sparse_mlp(hidden, logits, *mats, top_k_count=k, dtype="float32", shared=shared,
                               **settings)
    assert np.abs(out - tensors["block_output"].reshape(out.shape)).max() < OUTPUT_TOLERANCE
    without, _ = oracle.sparse_mlp(hidden, logits, *mats, top_k_count=k, dtype="float32", **settings)
    assert np.abs(without - tensors["block_output"].reshape(out.shape)).max() > 1e-2


def test_fp32_experts_reproduce_the_deepseek_v4_clamped_output():
    tensors = golden("moe/deepseek_v4.npz")
    hidden = tensors["hidden"].reshape(-1, 16)
    mats = [stacked(tensors, p, 8) for p in ("gate_proj", "up_proj", "down_proj")]
    out, _ = oracle.expert_mlp(hidden, tensors["router_weights"], tensors["router_indices"], *mats,
                               dtype="float32", limit=1.0)
    assert np.abs(out - tensors["experts_output"]).max() < OUTPUT_TOLERANCE
    unclamped, _ = oracle.expert_mlp(hidden, tensors["router_weights"], tensors["router_indices"], *mats,
                                     dtype="float32")
    assert np.abs(unclamped - tensors["experts_output"]).max() > 1.0


def test_fp32_block_reproduces_llama_4s_input_scaled_experts():
    """`Llama4TextMoe` (tests/fixtures/llama4/moe.npz, the reference's own check tests/test_llama4.py:162-191): the
    sigmoid of the top-2 logits scales each token's input to its experts, the outputs are summed unweighted, the shared
    expert adds. Tolerance 1e-5 as there; weighting the outputs instead misses by more than 1e-3."""
    tensors = golden("llama4/moe.npz")
    hidden = tensors["hidden"].reshape(-1, tensors["hidden"].shape[-1])
    gate_up = tensors["feed_forward.experts.gate_up_proj"]
    width = gate_up.shape[-1] // 2
    mats = [gate_up[..., :width], gate_up[..., width:], tensors["feed_forward.experts.down_proj"]]
    shared = [tensors[f"feed_forward.shared_expert.{name}.weight"].T for name in ("gate_proj", "up_proj", "down_proj")]
    logits = oracle.router_logits(hidden, tensors["feed_forward.router.weight"].T)
    settings = dict(top_k_count=2, dtype="float32", shared=shared, score_function="sigmoid", normalize_weights=False)
    out, _ = oracle.sparse_mlp(hidden, logits, *mats, scale_inputs=True, **settings)
    assert np.abs(out - tensors["output"]).max() < 1e-5
    other, _ = oracle.sparse_mlp(hidden, logits, *mats, scale_inputs=False, **settings)
    assert np.abs(other - tensors["output"]).max() > 1e-3


def test_relu2_experts_reproduce_the_references_known_answer():
    """tests/test_moe_precision.py:652-674 is stated on an ungated relu2 layer: two experts answer 1 and -1 (up = 1,
    relu2(1) = 1, down = +-1), weighted 1/2 +- 2^-11: the bf16 output is 2^-10. And the activation on every bf16."""
    x = np.ones((1, 1), np.float32)
    weights = np.array([[0.5 + 2.0 ** -11, 0.5 - 2.0 ** -11]], np.float32)
    indices = np.array([[0, 1]], np.int32)
    up, down = np.ones((2, 1, 1), np.float32), np.array([[[1.0]], [[-1.0]]], np.float32)
    out, _ = oracle.expert_mlp(x, weights, indices, None, up, down, activation="relu2")
    assert out.shape == (1, 1) and out[0, 0] == 2.0 ** -10
    every = (np.arange(1 << 16, dtype=np.uint32) << 16).view(np.float32)
    every = every[np.isfinite(every)]
    got = oracle.relu2(every)
    truth = np.where(every > 0, every.astype(np.float64) ** 2, 0.0)
    finite = truth < 3.3e38
    assert np.array_equal(got[finite], oracle.bf16_round(truth[finite].astype(np.float32))) and not got[every < 0].any()


def test_top_k_takes_the_lower_index_on_ties_in_descending_order():
    values = np.array([[1.0, 3.0, 3.0, -np.inf, 2.0, 3.0]], np.float32)
    got_values, got = oracle.top_k(values, 4)
    assert got.tolist() == [[1, 2, 5, 4]] and got_values.tolist() == [[3.0, 3.0, 3.0, 2.0]]


def test_exp_matches_float64_to_two_ulp_and_is_exact_at_zero():
    x = np.linspace(-87, 88, 200001).astype(np.float32)
    got = oracle.exp_f32(x).astype(np.float64)
    want = np.exp(x.astype(np.float64))
    assert np.max(np.abs(got - want) / want) < 2.5e-7
    assert oracle.exp_f32(np.float32(0.0)) == 1.0
    assert oracle.exp_f32(np.float32(-104.0)) < 1e-44 and np.isfinite(oracle.exp_f32(np.float32(88.0)))


def test_softmax_sums_to_one_and_orders_as_its_logits():
    rng = np.random.default_rng(0)
    logits = rng.standard_normal((512, 128)).astype(np.float32)
    scores = oracle.expert_softmax(logits)
    assert np.abs(scores.astype(np.float64).sum(-1) - 1).max() < 1e-6
    want = np.exp(logits.astype(np.float64))
    want /= want.sum(-1, keepdims=True)
    assert np.abs(scores - want).max() < 2e-8
    assert np.array_equal(np.argsort(-scores, -1, kind="stable")[:, :8], np.argsort(-logits, -1, kind="stable")[:, :8])


# ---- dispatch ------------------------------------------------------------------------------------


def test_sort_by_expert_is_the_stable_counting_sort():
    rng = np.random.default_rng(1)
    for tokens, k, experts in ((1, 1, 1), (7, 2, 4), (64, 8, 128), (300, 3, 5)):
        indices = rng.integers(0, experts, size=(tokens, k)).astype(np.int32)
        plan = oracle.sorted_by_expert(indices, experts)
        flat = indices.reshape(-1)
        brute = sorted(range(flat.size), key=lambda slot: (flat[slot], slot))       # brute force
        assert plan["order"].tolist() == brute
        assert plan["sizes"].tolist() == [int((flat == e).sum()) for e in range(experts)]
        assert plan["offsets"][0] == 0 and np.array_equal(np.diff(plan["offsets"]), plan["sizes"])
        assert np.array_equal(plan["rows"], plan["order"] // k)
        assert (np.diff(flat[plan["order"]]) >= 0).all()


# ---- formats --------------------------------------------------------------------------------------


def test_bf16_rounding_ties_to_even():
    x = np.array([1.0, 1.0 + 2 ** -8, 1.0 + 3 * 2 ** -8, 1.0 + 2 ** -8 + 2 ** -20, -3.3895e38], np.float32)
    want = np.array([1.0, 1.0, 1.0 + 2 ** -6, 1.0 + 2 ** -7, -3.3895314e38], np.float32)
    got = oracle.bf16_round(x)
    assert np.array_equal(got[:4], want[:4]) and np.isfinite(got[4])
    assert np.array_equal(oracle.bf16_from_bits(oracle.bf16_bits(x)), got)


def test_e4m3_table_known_values():
    table = oracle.E4M3
    assert table[0x00] == 0 and table[0x01] == 2.0 ** -9 and table[0x08] == 2.0 ** -6
    assert table[0x38] == 1.0 and table[0x7E] == 448.0 and np.isnan(table[0x7F]) and table[0xFE] == -448.0
    import torch
    theirs = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float().numpy()
    assert np.array_equal(np.nan_to_num(table, nan=7.0), np.nan_to_num(theirs, nan=7.0))


@pytest.mark.parametrize("shape", ["256x384", "130x259", "5x7"])
def test_fp8_block_dequantize_reproduces_the_deepseek_kernels_bytes(shape):
    held = golden("codecs/deepseek_kernels.npz")
    got = oracle.dequantize_fp8_blocks(held[f"v3/{shape}/codes"], held[f"v3/{shape}/scales"])
    assert np.array_equal(got.view(np.uint32), held[f"v3/{shape}/dequantized"].view(np.uint32))


def test_fp8_channel_dequantize_is_the_block_rule_with_one_column_blocks():
    rng = np.random.default_rng(2)
    codes = rng.integers(0, 0x7E, size=(3, 8, 5)).astype(np.uint8)
    scales = rng.uniform(0.5, 2, size=(3, 5)).astype(np.float32)
    got = oracle.dequantize_fp8_channels(codes, scales)
    want = oracle.dequantize_fp8_blocks(codes, scales[:, None, :], block=(8, 1))
    assert np.array_equal(got, want)


def test_mxfp4_decode_reproduces_the_gpt_oss_fixture():
    held = golden("gpt_oss/mxfp4.npz")
    got = oracle.decode_mxfp4(held["blocks"], held["scales"])
    assert np.array_equal(got.view(np.uint32), held["output"].view(np.uint32))


def natural_word(codes):
    return sum(int(c) << (4 * j) for j, c in enumerate(codes))


def encode_word(natural):
    return sum((bin(natural & mask).count("1") & 1) << i for i, mask in enumerate(oracle.NVFP4_ENCODER))


def test_nvfp4_decode_form_inverts_the_encoder_masks_on_every_basis_word_and_every_code():
    assert oracle.nvfp4_form_digest() == "7fb7f1b609cea47a"
    # GF(2)-linear: the 32 basis words and zero fix the map; every code in every position besides.
    naturals = [0] + [1 << bit for bit in range(32)] + [natural_word([c] * 8) for c in range(16)]
    rng = np.random.default_rng(3)
    naturals += [int(v) for v in rng.integers(0, 2 ** 32, size=4000, dtype=np.uint64)]
    stored = np.array([encode_word(n) for n in naturals], np.uint32)
    codes = oracle.nvfp4_words_to_codes(stored)
    want = np.array([[(n >> (4 * j)) & 15 for j in range(8)] for n in naturals], np.uint8)
    assert np.array_equal(codes, want)
    halves = oracle.nvfp4_words_to_halves(stored)
    values = oracle.bf16_from_bits(halves).astype(np.float64) * 2.0 ** 126
    assert np.array_equal(values, oracle.E2M1[want].astype(np.float64))


def test_nvfp4_staged_order_known_answers():
    order = oracle.nvfp4_staged_depths(256)          # tests/test_gemm_nvfp4.py:37-38
    assert sorted(order.tolist()) == list(range(256))
    assert order[8 * 3 + 5] == 16 * 5 + 3 and order[128] == 128


def test_nvfp4_bank_decodes_to_code_times_scale_over_256():
    rng = np.random.default_rng(4)
    experts, depth, width = 2, 256, 3
    codes = rng.integers(0, 16, size=(experts, depth, width)).astype(np.uint8)
    scales = rng.integers(0x20, 0x50, size=(experts, width, depth // 16)).astype(np.uint8)
    staged = codes[:, oracle.nvfp4_staged_depths(depth), :].swapaxes(1, 2).reshape(experts, width, depth // 8, 8)
    words = np.array([[[encode_word(natural_word(w)) for w in column] for column in bank] for bank in staged],
                     np.uint32)
    assert np.array_equal(oracle.nvfp4_bank_codes(words), codes)
    decoded = oracle.nvfp4_bank_decoded(words, scales)
    want = oracle.E2M1[codes] * np.repeat(oracle.E4M3[scales].swapaxes(1, 2), 16, axis=1) / 256
    assert np.array_equal(decoded, want.astype(np.float32))
    assert oracle.nvfp4_bank_factor(np.float32(0.25)) == 64.0


# ---- products --------------------------------------------------------------------------------------


def test_grouped_matmul_is_the_float64_per_group_product_on_small_integers():
    rng = np.random.default_rng(5)
    sizes = [3, 0, 5, 1]
    x = rng.integers(-3, 4, size=(12, 16)).astype(np.float32)       # 3 rows past the routed ones
    w = rng.integers(-2, 3, size=(4, 16, 8)).astype(np.float32)
    got = oracle.grouped_matmul(x, w, sizes)
    want = np.zeros((12, 8))
    start = 0
    for group, size in enumerate(sizes):                             # tools/grouped_oracle.py:20-27
        want[start:start + size] = x[start:start + size].astype(np.float64) @ w[group].astype(np.float64)
        start += size
    assert np.array_equal(got.astype(np.float64), want) and not got[9:].any()
    scaled = oracle.grouped_matmul(x, w, sizes, factor=np.array([2, 2, .5, 4], np.float32))
    assert np.array_equal(scaled[:3], got[:3] * 2) and np.array_equal(scaled[3:8], got[3:8] * .5)


def test_grouped_matmul_rounds_operands_to_bf16_and_the_sum_once():
    x = np.array([[1 + 2 ** -9, 1.0]], np.float32)                    # first rounds to 1 in bf16
    w = np.array([[[1.0], [2 ** -9]]], np.float32)
    assert oracle.grouped_matmul(x, w, [1])[0, 0] == 1.0              # 1 + 2^-9 rounds once to 1
    assert oracle.grouped_matmul(x, w, [1], dtype="float32")[0, 0] == np.float32(1 + 2 ** -9 + 2 ** -9)


def test_swiglu_rounds_after_the_activation_and_again_after_the_product():
    gate = np.array([1.0, -2.0, 0.0, 20.0], np.float32)
    up = np.array([3.0, 1.5, 5.0, 1.0 + 2 ** -7], np.float32)
    got = oracle.swiglu(gate, up)
    for g, u, h in zip(gate.tolist(), up.tolist(), got.tolist(), strict=True):
        silu = np.float32(g / (1 + np.exp(-np.float64(g))))
        activated = oracle.bf16_round(np.array([silu], np.float32))[0]
        assert h == oracle.bf16_round(np.array([activated * np.float32(u)], np.float32))[0]
    # Two roundings differ from one: silu(1)=0.7310586 -> bf16 0.73046875; times 3 = 2.19140625 -> 2.1875
    assert got[0] == 2.1875 and oracle.bf16_round(np.array([0.7310586 * 3], np.float32))[0] == 2.1875
    assert oracle.swiglu(gate, up, dtype="float32")[0] == np.float32(np.float32(0.7310586) * 3)


def test_bf16_combine_weighs_in_fp32_and_rounds_once():
    slots = np.array([[[1.0], [-1.0]]], np.float32)                   # tests/test_moe_precision.py:652-674
    weights = np.array([[0.5 + 2 ** -11, 0.5 - 2 ** -11]], np.float32)
    assert oracle.combine(slots, weights)[0, 0] == 2.0 ** -10


def test_gpt_oss_mlp_matches_the_reference_fixture():
    """tests/fixtures/gpt_oss/moe.npz of the reference, at its own test's tolerance (tests/test_gpt_oss.py:45-66)."""
    held = golden("gpt_oss/moe.npz")

    def run(down_bias):
        out, _ = oracle.gpt_oss_mlp(held["hidden"], held["router.weight"].T, held["router.bias"], held["experts.gate_up_proj"],
                                    held["experts.gate_up_proj_bias"], held["experts.down_proj"], down_bias,
                                    top_k_count=2, dtype="float32")
        return out

    np.testing.assert_allclose(run(held["experts.down_proj_bias"]), held["output"], atol=1.6e-4, rtol=0)
    assert np.abs(run(np.zeros_like(held["experts.down_proj_bias"])) - held["output"]).max() > 0.5


def test_gpt_oss_gating_rounds_every_operation_in_bf16():
    """Hand-followed cases: gate 1, up 0.5 -> t = bf16(1.703125) ; s = bf16(logistic(1.703125)) = 0.84765625;
    q = bf16(1 * s); u1 = 1.5; out = bf16(1.5 * 0.84765625) = 1.2734375 (1.271484375 rounds to 8 bits). Clamps: gate
    9 -> 7, up -9 -> -7 gives (1 - 7) * bf16(7 * bf16(logistic(bf16(7 * 1.703125))))."""
    out = oracle.gpt_oss_gating(np.array([[1.0, 0.5, 9.0, -9.0]], np.float32))
    s = oracle.bf16_round(np.float32(1.0) / (np.float32(1.0) + np.exp(np.float32(-1.703125))))
    assert s == np.float32(0.84765625)
    assert out[0, 0] == oracle.bf16_round(np.float32(1.5) * s) == np.float32(1.2734375)
    t = oracle.bf16_round(np.float32(7.0 * 1.703125))
    s7 = oracle.bf16_round(np.float32(1.0) / (np.float32(1.0) + np.exp(-t)))
    assert out[0, 1] == oracle.bf16_round(np.float32(-6.0) * oracle.bf16_round(np.float32(7.0) * s7))
    # fp32 mode rounds nowhere and uses 1.702 itself
    exact = oracle.gpt_oss_gating(np.array([[1.0, 0.5]], np.float32), dtype="float32")
    assert abs(exact[0, 0] - 1.5 / (1 + np.exp(-1.702))) < 1e-6


def test_the_balance_update_pushes_against_the_busy_experts():
    """The reference's own known answer (tests/test_moe.py:326-336): over four experts, three slots on expert 0 and
    one on expert 1 average one each, so expert 0 loses bias, expert 1 holds and the idle two gain."""
    assert np.array_equal(oracle.load_balance_update([3, 1, 0, 0], 0.001), np.array([-0.001, 0.0, 0.001, 0.001], np.float32))
    # a remainder tips the experts at the floor of the average upwards
    assert np.array_equal(oracle.load_balance_update([2, 1, 1, 1], 0.5), np.array([-0.5, 0.5, 0.5, 0.5], np.float32))
    assert np.array_equal(oracle.load_balance_update([2, 2, 2, 2], 0.5), np.zeros(4, np.float32))


def test_the_sown_statistics_are_the_scores_and_the_log_partition():
    rng = np.random.default_rng(5)
    logits = (rng.standard_normal((40, 24)) * 3).astype(np.float32)
    scores, log_z = oracle.router_statistics(logits)
    wide = logits.astype(np.float64)
    truth = np.log(np.exp(wide - wide.max(axis=1, keepdims=True)).sum(axis=1)) + wide.max(axis=1)
    assert np.abs(log_z - truth).max() <= 1e-6 * np.abs(truth).max()
    assert np.abs(scores - np.exp(wide - truth[:, None])).max() <= 1e-6            # softmax = exp(logit - log_z)
    shifted = oracle.router_statistics(logits + np.float32(8.0))[1]
    assert np.abs(shifted - (log_z + 8.0)).max() <= 1e-5
    sigmoid, same = oracle.router_statistics(logits, score_function="sigmoid")
    assert np.array_equal(same, log_z) and np.abs(sigmoid - 1 / (1 + np.exp(-wide))).max() <= 1e-6


def test_a_nan_selection_competes_as_minus_infinity():
    """The router's rule for a NaN selection (a NaN bias entry): never preferred, and every choice an expert in range."""
    rng = np.random.default_rng(3)
    logits = rng.standard_normal((9, 16)).astype(np.float32)
    bias = np.zeros(16, np.float32)
    bias[[2, 7]] = np.nan
    _, indices = oracle.route(logits, 4, score_function="sigmoid", bias=bias)
    assert not np.isin(indices, [2, 7]).any() and indices.min() >= 0 and indices.max() < 16
    bias[:] = np.nan
    _, indices = oracle.route(logits, 4, score_function="sigmoid", bias=bias)
    assert np.array_equal(indices, np.tile(np.arange(4, dtype=np.int32), (9, 1)))


def test_the_sort_with_a_shared_expert_by_brute_force():
    """Tiny case by hand: 3 tokens, top-2, 3 experts, one dropped slot; the shared expert's three rows form group 3."""
    indices = np.array([[2, 0], [0, 3], [1, 0]], np.int32)            # id 3: a dropped slot
    got = oracle.sorted_with_shared(indices, 3, 3)
    assert got["sizes"].tolist() == [3, 1, 1, 3] and got["offsets"].tolist() == [0, 3, 4, 5, 8]
    assert got["order"].tolist() == [1, 2, 5, 4, 0, 6, 7, 8, 3]       # experts 0, 1, 2, the shared rows, the dropped slot
    assert got["rows"].tolist() == [0, 1, 2, 2, 0, 0, 1, 2, 1]
    plain = oracle.sorted_by_expert(np.array([[2, 0], [0, 1], [1, 0]], np.int32), 3)
    with_shared = oracle.sorted_with_shared(np.array([[2, 0], [0, 1], [1, 0]], np.int32), 3, 3)
    assert with_shared["order"][:6].tolist() == plain["order"].tolist() and with_shared["sizes"][:3].tolist() == plain["sizes"].tolist()


def test_capacity_dropping_is_the_references_argsort_arithmetic():
    """`capacity_admitted` is written as the definition (a queue per sequence and expert, in slot order); the
    reference computes the same places by a stable argsort, a bincount and a cumsum (src/dew/nn/moe.py:845-855).
    Restated here with NumPy's own stable sort, the two agree on random routings, and a hand case pins both."""
    import math

    def by_argsort(indices, experts, factor):
        *_, length, top_k = indices.shape
        capacity = int(max(math.ceil(length * top_k / experts) * factor, factor))
        flat = indices.reshape(-1, length * top_k)
        order = np.argsort(flat, axis=-1, kind="stable")
        queued = np.take_along_axis(flat, order, axis=-1)
        counts = np.stack([np.bincount(row, minlength=experts)[:experts] for row in flat])
        starts = np.cumsum(counts, axis=-1) - counts
        places = np.arange(length * top_k) - np.take_along_axis(starts, queued, axis=-1)
        positions = np.zeros_like(flat)
        np.put_along_axis(positions, order, places, axis=-1)
        return np.where(positions.reshape(indices.shape) < capacity, indices, experts), capacity

    hand = np.array([[[0, 1], [0, 2], [0, 1], [1, 0]]], np.int32)       # expert 0 is asked for four times, capacity 2
    admitted, capacity = oracle.capacity_admitted(hand, 4, 1.0)
    assert capacity == 2 and admitted.tolist() == [[[0, 1], [0, 2], [4, 1], [4, 4]]]
    rng = np.random.default_rng(8)
    for sequences, length, k, experts, factor in ((2, 50, 2, 8, 1.0), (3, 17, 3, 5, 0.5), (1, 200, 4, 16, 1.5)):
        indices = np.stack([np.stack([rng.choice(experts, size=k, replace=False) for _ in range(length)]) for _ in range(sequences)]).astype(np.int32)
        ours, ours_capacity = oracle.capacity_admitted(indices, experts, factor)
        theirs, theirs_capacity = by_argsort(indices, experts, factor)
        assert ours_capacity == theirs_capacity and np.array_equal(ours, theirs)


def test_silu_is_the_activation_of_swiglu_with_its_one_rounding():
    """`silu` against the three things that fix it: `swiglu` with an up projection of one (the same activation, then
    a product by 1 that changes nothing), a float64 `x / (1 + e^-x)` rounded once, on every finite bf16; and the fp32
    mode, which rounds nowhere."""
    every = oracle.bf16_from_bits(np.arange(65536, dtype=np.uint16))
    every = every[np.isfinite(every)]
    got = oracle.silu(every)
    assert np.array_equal(got, oracle.swiglu(every, np.ones_like(every)))
    # (below -87 fp32's e^-x overflows and the reference's 1 / (1 + e^-x) is zero there, src/dew/nn/precision.py:568-575)
    inside = every > -87
    wide = every[inside].astype(np.float64)
    truth = wide / (1.0 + np.exp(-wide))
    rounded = oracle.bf16_round(truth.astype(np.float32))
    # one rounding of the fp32 product: at most one bf16 step from the float64 value's rounding, and equal almost everywhere
    steps = np.abs(oracle.bf16_bits(got[inside]).astype(np.int64) - oracle.bf16_bits(rounded).astype(np.int64))
    assert steps.max() <= 1 and (steps == 0).mean() > 0.999
    assert np.all(np.abs(got[~inside]) < 1e-35) and np.all(got[every < -89] == 0)
    assert oracle.silu(np.float32([1.0]), dtype="float32")[0] == np.float32(np.float32(0.7310586) * 1)
    assert oracle.silu(np.float32([0.0, -0.0]))[0] == 0


def test_routed_values_are_each_tokens_weighted_sum_of_its_chosen_experts_activated_projections():
    """Integer operands small enough that every fp32 sum is exact: the layer against a token-by-token float64 sum,
    with weights that are powers of two. A wrong gather, scatter, weight pairing or a missing activation fails it."""
    rng = np.random.default_rng(11)
    tokens, experts, k, depth, width = 13, 5, 2, 16, 8
    x = rng.integers(-3, 4, size=(tokens, depth)).astype(np.float32)
    kernel = rng.integers(-2, 3, size=(experts, depth, width)).astype(np.float32)
    indices = np.stack([rng.permutation(experts)[:k] for _ in range(tokens)]).astype(np.int32)
    weights = np.exp2(rng.integers(-2, 2, size=(tokens, k))).astype(np.float32)
    out, slots = oracle.routed_values(x, weights, indices, kernel)
    for t in range(tokens):
        total = np.zeros(width, np.float64)
        for j in range(k):
            projected = x[t].astype(np.float64) @ kernel[indices[t, j]].astype(np.float64)       # small integers: exact in bf16
            activated = oracle.silu(projected.astype(np.float32)).astype(np.float64)
            assert np.array_equal(slots[t, j], activated.astype(np.float32))
            total += activated * float(weights[t, j])
        assert np.array_equal(out[t], oracle.bf16_round(total.astype(np.float32))), t


def test_geglu_is_the_tanh_gelu_with_the_two_roundings():
    """The logistic form the reference computes against the textbook tanh form in float64, on every finite bf16 gate;
    then the product's second rounding, the fp32 mode and the clamp."""
    every = oracle.bf16_from_bits(np.arange(65536, dtype=np.uint16))
    every = every[np.isfinite(every) & (np.abs(every) < 1e12)]            # (beyond, x^3 overflows fp32: the reference's too)
    got = oracle.geglu(every, np.ones_like(every))
    wide = every.astype(np.float64)
    z = np.sqrt(2.0 / np.pi) * (wide + 0.044715 * wide ** 3)
    # the textbook form where float64's 1 + tanh keeps its digits (x > -4); below, the tail the tanh form cancels is held
    # to the same function written x / (1 + e^(-2 z)) in float64, down to where fp32's e^(-2 z) overflows (x near -10)
    with np.errstate(over="ignore"):
        truth = np.where(wide > -4, 0.5 * wide * (1.0 + np.tanh(z)), wide / (1.0 + np.exp(-2.0 * z)))
    inside = np.abs(truth) > 1e-30
    rounded = oracle.bf16_round(truth.astype(np.float32))
    steps = np.abs(oracle.bf16_bits(got[inside]).astype(np.int64) - oracle.bf16_bits(rounded[inside]).astype(np.int64))
    assert steps.max() <= 1 and (steps == 0).mean() > 0.995
    assert np.all(np.abs(got[~inside]) <= 1e-30)
    # gelu(1) = 0.841192 -> bf16 0.83984375 (a bf16 step is 2^-8 there); times up = 3 -> 2.51953125 -> bf16 2.515625
    assert oracle.geglu(np.float32([1.0]), np.float32([1.0]))[0] == np.float32(0.83984375)
    assert oracle.geglu(np.float32([1.0]), np.float32([3.0]))[0] == np.float32(2.515625)
    assert abs(oracle.geglu(np.float32([1.0]), np.float32([3.0]), dtype="float32")[0] - 3 * 0.8411919906082768) < 1e-6
    assert oracle.geglu(np.float32([5.0]), np.float32([-9.0]), limit=2.0)[0] == oracle.geglu(np.float32([2.0]), np.float32([-2.0]))[0]


# ---- the router's further switches (src/dew/nn/moe.py:361-384): each pinned by what its definition fixes ----


@pytest.mark.parametrize("fill", [0.0, None], ids=["axk2-zero", "deepseek-inf"])
def test_an_expert_outside_the_best_groups_is_chosen_by_the_score_filled_in(fill):
    """The reference's own case (tests/test_moe.py:265-292): eight experts in four groups, two groups a token's best,
    every selection below zero (sigmoid scores under a bias of -5). Filled at 0.0 the four experts outside those groups
    outrank the groups' own and are the choice; at -inf they never are."""
    rng = np.random.default_rng(0x3080)
    logits = rng.standard_normal((6, 8)).astype(np.float32)
    bias = np.full(8, -5.0, np.float32)
    _, indices = oracle.route(logits, 4, score_function="sigmoid", bias=bias, expert_groups=4, groups_per_token=2,
                              excluded_group_score=fill)
    scores = 1.0 / (1.0 + np.exp(-logits.astype(np.float64))) - 5.0
    pairs = scores.reshape(6, 4, 2)
    best_groups = np.argsort(-pairs.sum(-1), axis=-1, kind="stable")[:, :2]          # two experts a group: top2 is the sum
    for token in range(6):
        inside = sorted(int(g) * 2 + j for g in best_groups[token] for j in range(2))
        outside = sorted(set(range(8)) - set(inside))
        assert sorted(indices[token].tolist()) == (outside if fill is not None else inside)


def test_a_weight_sum_floor_divides_small_sums_by_itself_and_moves_a_softmax_to_its_scores():
    rng = np.random.default_rng(11)
    logits = (rng.standard_normal((50, 16)) * 2 - 3).astype(np.float32)        # sigmoid scores mostly small
    plain, chosen = oracle.route(logits, 2, score_function="sigmoid", normalize_weights=False)
    sums = plain.astype(np.float64).sum(-1)
    floor = float(np.median(sums))
    weights, indices = oracle.route(logits, 2, score_function="sigmoid", weight_sum_min=floor)
    assert np.array_equal(indices, chosen)
    truth = plain.astype(np.float64) / np.maximum(sums + 1e-20, floor)[:, None]
    assert np.abs(weights - truth).max() <= ROUTER_TOLERANCE
    small = sums < floor
    assert small.any() and (~small).any()
    assert np.abs(weights[small].astype(np.float64).sum(-1) - sums[small] / floor).max() <= ROUTER_TOLERANCE   # they sum to less than one
    assert np.abs(weights[~small].astype(np.float64).sum(-1) - 1.0).max() <= ROUTER_TOLERANCE
    # a softmax router under a floor gathers its scores and divides them (:483-494); a floor below every sum changes
    # nothing but the roundings on the way
    renormalized, _ = oracle.route(logits, 2)
    floored, _ = oracle.route(logits, 2, weight_sum_min=1e-12)
    assert np.abs(floored - renormalized).max() <= ROUTER_TOLERANCE
    wide, _ = oracle.route(logits, 2, weight_sum_epsilon=1.0, score_function="sigmoid")
    assert np.abs(wide - plain.astype(np.float64) / (sums + 1.0)[:, None]).max() <= ROUTER_TOLERANCE


def test_bias_in_weights_makes_the_biased_scores_the_weights():
    rng = np.random.default_rng(12)
    logits = rng.standard_normal((30, 12)).astype(np.float32)
    bias = (rng.standard_normal(12) * 0.3).astype(np.float32)
    for normalize in (False, True):
        weights, indices = oracle.route(logits, 3, bias=bias, bias_in_weights=True, normalize_weights=normalize)
        wide = logits.astype(np.float64)
        softmax = np.exp(wide - wide.max(-1, keepdims=True))
        biased = softmax / softmax.sum(-1, keepdims=True) + bias
        assert np.array_equal(indices, np.argsort(-biased, axis=-1, kind="stable")[:, :3])
        truth = np.take_along_axis(biased, indices, -1)
        if normalize:
            truth = truth / (truth.sum(-1, keepdims=True) + 1e-20)
        assert np.abs(weights - truth).max() <= ROUTER_TOLERANCE
    unbiased_weights, _ = oracle.route(logits, 3, bias=bias, normalize_weights=False)
    assert np.abs(unbiased_weights - (np.take_along_axis(biased, indices, -1) - bias[indices])).max() <= ROUTER_TOLERANCE


def test_a_logit_softcap_bounds_the_logits_and_keeps_their_order():
    rng = np.random.default_rng(13)
    logits = (rng.standard_normal((40, 16)) * 20).astype(np.float32)
    capped = oracle.capped_logits(logits, 30.0)
    assert np.abs(capped).max() < 30.0
    assert np.abs(capped - 30.0 * np.tanh(logits.astype(np.float64) / 30.0)).max() <= 4e-6
    assert oracle.capped_logits(logits, None) is not None and np.array_equal(oracle.capped_logits(logits, None), logits)
    # tanh is increasing: a softmax router without a bias chooses the same experts, by weights that are the capped logits'
    weights, indices = oracle.route(logits, 4, logit_softcap=30.0)
    assert np.array_equal(indices, oracle.route(logits, 4)[1])
    assert np.array_equal(weights, oracle.route(capped, 4)[0])
    chosen = np.take_along_axis(capped.astype(np.float64), indices, -1)
    truth = np.exp(chosen - chosen.max(-1, keepdims=True))
    assert np.abs(weights - truth / truth.sum(-1, keepdims=True)).max() <= ROUTER_TOLERANCE


def test_the_gated_products_are_torchs_recorded_bf16_outputs():
    """tests/fixtures/gated_product/bf16.npz of the reference: Torch's bf16 `silu(gate) * up` and tanh-`gelu(gate) * up`
    on 2048 drawn bf16 pairs, the arm the reference's own gated product is held to
    (tests/test_causal_transformer.py:1290-1340). The rounding after the activation and the one after the product are
    Torch's bf16 arithmetic; dropping either moves hundreds of these outputs."""
    held = golden("gated_product/bf16.npz")
    gate, up, output = held["swiglu/gate"], held["swiglu/up"], held["swiglu/output"]
    assert np.array_equal(oracle.swiglu(gate, up), output)
    once = oracle.bf16_round(gate.astype(np.float64) / (1.0 + np.exp(-gate.astype(np.float64))) * up)   # one rounding only
    assert (once != output).sum() > 100
    gate, up, output = held["geglu/gate"], held["geglu/up"], held["geglu/output"]
    got = oracle.geglu(gate, up)
    differs = got != output
    assert differs.sum() < 40 and np.all(output[differs] == 0) and np.abs(got[differs]).max() < 1e-16   # Torch's tanh at -1


def test_given_experts_take_the_routers_weights_for_them():
    """Replayed routes and a hash table's rows (`chosen_experts`, src/dew/nn/moe.py:202-224, 500-507): the router's own
    choice given back is its own routing; a reordering of it reorders the weights; a token the record does not cover
    keeps the router's choice; arbitrary experts weigh by their scores, gathered and normalized."""
    rng = np.random.default_rng(14)
    logits = (rng.standard_normal((60, 16)) * 2).astype(np.float32)
    for settings in (dict(score_function="softmax"), dict(score_function="sigmoid", routed_scaling_factor=2.5),
                     dict(score_function="softmax", normalize_weights=False), dict(score_function="sqrtsoftplus")):
        weights, indices = oracle.route(logits, 4, **settings)
        again_w, again_i = oracle.route(logits, 4, given=indices, **settings)
        assert np.array_equal(again_i, indices) and np.array_equal(again_w, weights)
        flipped_w, flipped_i = oracle.route(logits, 4, given=indices[:, ::-1], **settings)
        assert np.array_equal(flipped_i, indices[:, ::-1]) and np.abs(flipped_w - weights[:, ::-1]).max() <= ROUTER_TOLERANCE
        table = rng.integers(0, 16, size=(60, 4)).astype(np.int32)
        covered = rng.integers(0, 2, size=60).astype(bool)
        mixed_w, mixed_i = oracle.route(logits, 4, given=table, covered=covered, **settings)
        assert np.array_equal(mixed_i[covered], table[covered]) and np.array_equal(mixed_i[~covered], indices[~covered])
        assert np.array_equal(mixed_w[~covered], weights[~covered])
        wide = logits.astype(np.float64)
        if settings["score_function"] == "softmax":
            scores = np.exp(wide - wide.max(-1, keepdims=True))
            scores /= scores.sum(-1, keepdims=True)
        elif settings["score_function"] == "sigmoid":
            scores = 1 / (1 + np.exp(-wide))
        else:
            scores = np.sqrt(np.logaddexp(0.0, wide))
        truth = np.take_along_axis(scores, table.astype(np.int64), -1)
        if settings.get("normalize_weights", True):
            truth = truth / (truth.sum(-1, keepdims=True) + 1e-20)
        truth = truth * settings.get("routed_scaling_factor", 1.0)
        assert np.abs(mixed_w[covered] - truth[covered]).max() <= 2 * ROUTER_TOLERANCE
        # an id outside the experts (a dropped slot's sentinel, src/dew/nn/moe.py:1101-1128) passes through with weight zero,
        # and the token's other slots weigh as if the record had held them alone
        dropped = table.copy()
        dropped[::2, 1], dropped[1::4, 3] = 16, -1
        dropped_w, dropped_i = oracle.route(logits, 4, given=dropped, **settings)
        outside = (dropped < 0) | (dropped >= 16)
        assert np.array_equal(dropped_i, dropped) and not dropped_w[outside].any()
        kept = np.where(outside, 0.0, np.take_along_axis(scores, np.clip(dropped, 0, 15).astype(np.int64), -1))
        if settings.get("normalize_weights", True):
            kept = kept / (kept.sum(-1, keepdims=True) + 1e-20)
        assert np.abs(dropped_w - kept * settings.get("routed_scaling_factor", 1.0)).max() <= 2 * ROUTER_TOLERANCE


def test_media_tokens_are_routed_by_their_own_bias():
    """`selection` (src/dew/nn/moe.py:516-524): a media token's experts are chosen by scores + media_bias, the others' by
    scores + bias; the weights stay the unbiased scores'."""
    rng = np.random.default_rng(15)
    logits = rng.standard_normal((40, 32)).astype(np.float32)
    bias, media_bias = (rng.standard_normal(32) * 0.5).astype(np.float32), (rng.standard_normal(32) * 0.5).astype(np.float32)
    media = rng.integers(0, 2, size=40).astype(bool)
    settings = dict(score_function="sigmoid", expert_groups=4, groups_per_token=2, routed_scaling_factor=2.5)
    weights, indices = oracle.route(logits, 4, bias=bias, media=media, media_bias=media_bias, **settings)
    text_w, text_i = oracle.route(logits, 4, bias=bias, **settings)
    image_w, image_i = oracle.route(logits, 4, bias=media_bias, **settings)
    assert np.array_equal(indices, np.where(media[:, None], image_i, text_i))
    assert np.array_equal(weights, np.where(media[:, None], image_w, text_w))
    assert not np.array_equal(indices, text_i) and not np.array_equal(indices, image_i)
    unbiased_w, unbiased_i = oracle.route(logits, 4, media=media, media_bias=media_bias, **settings)      # a router with the media bias alone
    plain_w, plain_i = oracle.route(logits, 4, **settings)
    assert np.array_equal(unbiased_i, np.where(media[:, None], image_i, plain_i))


def test_block_routing_limits_a_token_to_its_blocks_best_experts():
    """`Router.block_mask` (src/dew/nn/moe.py:566-585): a hand case; blocks of one token (each token's own best); one
    block a row with every expert allowed (no limit); a relabelling of the blocks; padding as a block of its own."""
    selection = np.array([[[0.9, 0.1, 0.5, 0.2],       # block 0: best per expert over its two tokens = [0.9, 0.8, 0.5, 0.2]
                           [0.3, 0.8, 0.4, 0.1],
                           [0.1, 0.2, 0.3, 0.4],       # block 1 alone: best two are experts 3, 2
                           [0.7, 0.6, 0.1, 0.0]]], np.float32)   # padding: a block of its own, best two 0, 1
    mask = oracle.block_mask(selection, np.array([[0, 0, 1, -1]]), 2)
    assert np.array_equal(mask[0], np.array([[1, 1, 0, 0], [1, 1, 0, 0], [0, 0, 1, 1], [1, 1, 0, 0]], bool))
    rng = np.random.default_rng(16)
    logits = rng.standard_normal((3, 24, 16)).astype(np.float32)
    alone = np.tile(np.arange(24), (3, 1))
    _, selection = oracle.selection_scores(logits, score_function="sigmoid")
    mask = oracle.block_mask(selection, alone, 5)
    assert np.array_equal(mask, selection >= -np.sort(-selection, axis=-1)[..., 4:5])
    for settings in (dict(score_function="sigmoid"), dict(score_function="softmax", normalize_weights=False)):
        free_w, free_i = oracle.route(logits, 3, **settings)
        whole_w, whole_i = oracle.route(logits, 3, blocks=np.zeros((3, 24), np.int64), block_experts=16, **settings)
        assert np.array_equal(whole_i, free_i) and np.array_equal(whole_w, free_w)
        blocks = np.tile(np.arange(24) // 4, (3, 1))
        blocks[1, 20:] = -1
        weights, indices = oracle.route(logits, 3, blocks=blocks, block_experts=4, **settings)
        assert not np.array_equal(indices, free_i)
        relabelled = np.where(blocks < 0, -1, 5 - blocks)
        again_w, again_i = oracle.route(logits, 3, blocks=relabelled, block_experts=4, **settings)
        assert np.array_equal(again_i, indices) and np.array_equal(again_w, weights)
        for row in range(3):                       # every block uses at most block_experts experts, and the same shortlist
            for block in np.unique(blocks[row]):
                assert np.unique(indices[row, blocks[row] == block]).size <= 4


def test_the_shared_experts_gate_rounds_its_logit_its_logistic_and_its_product():
    """`gated_rows` (`shared_gate` under a bf16 compute dtype). By hand: x = (1, 0, ...), kernel = (0.3, ...): the kernel
    rounds to bf16 0.30078125, which is the logit; logistic(0.30078125) = 0.574633..., bf16 0.57421875 (the neighbours
    are 0.57421875 and 0.578125); a row value of 3.0 gives 1.72265625, which lies between the bf16 neighbours 1.71875
    and 1.7265625, nearer the former. Unrounded, 3 * sigmoid(0.3) = 1.7233... would round to 1.7265625."""
    x = np.zeros((1, 8), np.float32)
    x[0, 0] = 1.0
    kernel = np.full(8, 0.3, np.float32)
    assert oracle.gated_rows(x, kernel, np.array([[3.0, -1.0]], np.float32)).tolist() == [[1.71875, -0.57421875]]
    assert oracle.bf16_round(np.float32(3.0 / (1.0 + np.exp(-0.3)))) == np.float32(1.7265625)
    rng = np.random.default_rng(17)
    x = oracle.bf16_round(rng.standard_normal((50, 64)).astype(np.float32))
    kernel = (rng.standard_normal(64) * 0.2).astype(np.float32)
    rows = oracle.bf16_round(rng.standard_normal((50, 24)).astype(np.float32))
    truth = rows.astype(np.float64) / (1.0 + np.exp(-(x.astype(np.float64) @ kernel.astype(np.float64))))[:, None]
    got = oracle.gated_rows(x, kernel, rows)
    assert np.abs(got - truth).max() <= 3 * 2.0 ** -8 * np.abs(truth).max()          # three bf16 roundings and the kernel's own
    assert np.abs(got - truth).max() > 0
    # the layer: the shared expert's output gated, then added
    logits = rng.standard_normal((50, 4)).astype(np.float32)
    banks = [oracle.bf16_round((rng.standard_normal(shape) * 0.1).astype(np.float32)) for shape in ((4, 64, 32), (4, 64, 32), (4, 32, 64))]
    shared = [bank[0] for bank in banks]
    gate = (rng.standard_normal(64) * 0.2).astype(np.float32)
    gated, _ = oracle.sparse_mlp(x, logits, *banks, top_k_count=2, shared=shared, shared_gate=gate)
    routed, _ = oracle.sparse_mlp(x, logits, *banks, top_k_count=2)
    apart = oracle.gated_rows(x, gate, oracle.gated_mlp(x, *shared))
    assert np.array_equal(gated, oracle.bf16_round(routed + apart))

"""Parity of each HIP kernel, called through the C ABI, with the CPU oracle on the same seeded inputs.
Integer outputs (indices, sizes, offsets, order, rows) and router weights must match bit for bit; products
are compared with the tolerance stated beside each check."""

import dataclasses

import numpy as np
import pytest
import torch
from bench_aids.workloads import CONFIGS, inputs, quantize
from oracle.banks import dequantized

from oracle import moe_oracle as oracle

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from dew_amd import ops

    ops.device_check()
    return ops


def dev(t):
    return None if t is None else t.cuda()


def bf16_np(t):
    return t.float().cpu().numpy()


ROUTERS = [
    ("sqrtsoftplus-64-top6", 64, 6, dict(score_function="sqrtsoftplus", normalize_weights=True, routed_scaling_factor=2.5), True, 301),
    ("sqrtsoftplus-256-top8-raw", 256, 8, dict(score_function="sqrtsoftplus", normalize_weights=False), False, 77),
    ("softmax-64-top4-groups-by-max", 64, 4, dict(score_function="softmax", normalize_weights=False, routed_scaling_factor=2.5,
                                                  expert_groups=4, groups_per_token=2, group_score="max"), False, 500),
    ("sigmoid-32-top2-single-expert-groups", 32, 2, dict(score_function="sigmoid", normalize_weights=True, expert_groups=32,
                                                         groups_per_token=4, group_score="max"), True, 40),
    ("softmax-8-top2", 8, 2, dict(score_function="softmax", normalize_weights=True), False, 1000),
    ("softmax-128-top8", 128, 8, dict(score_function="softmax", normalize_weights=True), False, 777),
    ("softmax-128-top8-raw", 128, 8, dict(score_function="softmax", normalize_weights=False), False, 130),
    ("softmax-5-top5", 5, 5, dict(score_function="softmax", normalize_weights=True), False, 9),
    ("sigmoid-256-top8-groups", 256, 8, dict(score_function="sigmoid", normalize_weights=True, routed_scaling_factor=2.5,
                                             expert_groups=8, groups_per_token=4), True, 1111),
    ("sigmoid-64-top6-raw", 64, 6, dict(score_function="sigmoid", normalize_weights=False, routed_scaling_factor=1.5), True, 65),
    ("softmax-320-top4-groups", 320, 4, dict(score_function="softmax", normalize_weights=True, expert_groups=5,
                                             groups_per_token=2), False, 33),
    ("sigmoid-64-top6-bias-in-weights", 64, 6, dict(score_function="sigmoid", normalize_weights=True, bias_in_weights=True), True, 200),
    ("softmax-32-top4-bias-in-weights-raw", 32, 4, dict(score_function="softmax", normalize_weights=False, bias_in_weights=True,
                                                        routed_scaling_factor=2.0), True, 100),
    ("sigmoid-128-top8-sum-floor", 128, 8, dict(score_function="sigmoid", normalize_weights=True, weight_sum_min=7.5), False, 300),
    ("softmax-64-top4-sum-floor-and-epsilon", 64, 4, dict(score_function="softmax", normalize_weights=True, weight_sum_min=0.5,
                                                          weight_sum_epsilon=1e-6), False, 150),
    ("sigmoid-256-top8-wide-epsilon", 256, 8, dict(score_function="sigmoid", normalize_weights=True, weight_sum_epsilon=0.25), True, 90),
]


@pytest.mark.parametrize("name,experts,k,settings,biased,tokens", ROUTERS, ids=[r[0] for r in ROUTERS])
def test_router_matches_the_oracle_bit_for_bit(ops, name, experts, k, settings, biased, tokens):
    import zlib
    rng = np.random.default_rng(zlib.crc32(name.encode()))
    logits = (rng.standard_normal((tokens, experts)) * 2).astype(np.float32)
    logits[0, :] = 0.25                                   # an all-ties row: the lower indices win
    logits[1, : experts // 2] = logits[1, experts // 2: 2 * (experts // 2)]   # pairwise ties
    bias = (rng.standard_normal(experts) * 0.1).astype(np.float32) if biased else None
    want_w, want_i = oracle.route(logits, k, bias=bias, **settings)
    got_w, got_i = ops.route(torch.from_numpy(logits).cuda(), k, bias=None if bias is None else torch.from_numpy(bias).cuda(),
                             **settings)
    assert np.array_equal(got_i.cpu().numpy(), want_i)
    assert np.array_equal(got_w.cpu().numpy().view(np.uint32), want_w.view(np.uint32))


@pytest.mark.parametrize("fill", [0.0, 0.3, None])
@pytest.mark.parametrize("experts,groups,kept,k,group_score", [(64, 8, 2, 8, "top2"), (256, 8, 1, 8, "top2"), (32, 4, 2, 6, "max")])
def test_an_excluded_groups_experts_compete_at_the_score_filled_in(ops, experts, groups, kept, k, group_score, fill):
    """A.X-K2's fill for the experts outside a token's best groups (`excluded_group_score`): under a bias that puts most
    of the selections below the fill, those experts outrank the kept groups' weaker ones."""
    rng = np.random.default_rng(experts + groups)
    logits = (rng.standard_normal((333, experts)) * 2).astype(np.float32)
    bias = (rng.standard_normal(experts) * 0.1 - 0.8).astype(np.float32)
    settings = dict(score_function="sigmoid", normalize_weights=True, routed_scaling_factor=2.5, expert_groups=groups,
                    groups_per_token=kept, group_score=group_score, excluded_group_score=fill)
    want_w, want_i = oracle.route(logits, k, bias=bias, **settings)
    got_w, got_i = ops.route(torch.from_numpy(logits).cuda(), k, bias=torch.from_numpy(bias).cuda(), **settings)
    assert np.array_equal(got_i.cpu().numpy(), want_i)
    assert np.array_equal(got_w.cpu().numpy().view(np.uint32), want_w.view(np.uint32))
    if fill is not None:    # the case means something: some chosen experts sit outside their token's kept groups
        _, limited = oracle.route(logits, k, bias=bias, **{**settings, "excluded_group_score": None})
        assert not np.array_equal(np.sort(limited, -1), np.sort(want_i, -1))


@pytest.mark.parametrize("score_function,experts,k,cap", [("softmax", 64, 4, 30.0), ("sigmoid", 256, 8, 5.0), ("softmax", 128, 8, 2.0)])
def test_a_logit_softcap_caps_what_every_reader_of_the_logits_reads(ops, score_function, experts, k, cap):
    """`logit_softcap`: scores, choices, weights and the sown log partition all read `cap * tanh(logit / cap)`. The
    hyperbolic tangent is the device library's and the oracle's NumPy's (the reference's is XLA's: no one's bits are
    pinned), so the weights are compared at the reference's router tolerance, 1e-6, and the choices exactly wherever the
    oracle's own margin between the last expert chosen and the first left out exceeds a few fp32 spacings."""
    rng = np.random.default_rng(int(cap * 10) + experts)
    logits = (rng.standard_normal((400, experts)) * 4).astype(np.float32)
    settings = dict(score_function=score_function, normalize_weights=True, logit_softcap=cap)
    want_w, want_i = oracle.route(logits, k, **settings)
    got = ops.route(torch.from_numpy(logits).cuda(), k, sown=True, **settings)
    got_w, got_i = got[0].cpu().numpy(), got[1].cpu().numpy()
    _, selection = oracle.selection_scores(oracle.capped_logits(logits, cap), score_function=score_function)
    ranked = -np.sort(-selection, axis=-1)
    clear = (ranked[:, :-1] - ranked[:, 1:])[:, :k].min(-1) > 8 * np.spacing(np.abs(ranked[:, 0]))   # no two of the first k + 1 within a few spacings
    assert clear.mean() > 0.9
    assert np.array_equal(got_i[clear], want_i[clear])
    assert np.abs(got_w[clear] - want_w[clear]).max() <= 1e-6
    want_scores, want_log_z = oracle.router_statistics(oracle.capped_logits(logits, cap), score_function=score_function)
    assert np.abs(got[2].cpu().numpy() - want_scores).max() <= 1e-6
    assert np.abs(got[3].cpu().numpy() - want_log_z).max() <= 1e-5
    assert np.abs(got[3].cpu().numpy()).max() <= cap + np.log(experts) + 1e-3


@pytest.mark.parametrize("score_function,experts,k,extra", [("softmax", 64, 4, {}), ("sigmoid", 256, 8, dict(routed_scaling_factor=2.5)),
                                                            ("sqrtsoftplus", 128, 6, {}), ("softmax", 32, 2, dict(normalize_weights=False)),
                                                            ("sigmoid", 64, 8, dict(expert_groups=8, groups_per_token=3))])
def test_given_experts_weigh_as_the_router_weighs_them(ops, score_function, experts, k, extra):
    """A replayed record's or a hash table's experts (`dew_moe_route_call`): every token covered, and some; ids
    outside the experts (a dropped slot's sentinel) come back as given with weight zero and the sort drops their slots; the
    router's own choice given back is its own routing."""
    rng = np.random.default_rng(experts * 7 + k)
    tokens = 271
    logits = (rng.standard_normal((tokens, experts)) * 2).astype(np.float32)
    biased = score_function == "sigmoid"
    bias = (rng.standard_normal(experts) * 0.1).astype(np.float32) if biased else None
    settings = dict(score_function=score_function, **extra)
    table = rng.integers(0, experts, size=(tokens, k)).astype(np.int32)
    covered = rng.integers(0, 2, size=tokens).astype(bool)
    on_device = dict(bias=None if bias is None else torch.from_numpy(bias).cuda())
    for given, covers in ((table, None), (table, covered)):
        want_w, want_i = oracle.route(logits, k, bias=bias, given=given, covered=covers, **settings)
        got_w, got_i = ops.route(torch.from_numpy(logits).cuda(), k, given=torch.from_numpy(given).cuda(),
                                 covered=None if covers is None else torch.from_numpy(covers).cuda(), **on_device, **settings)
        assert np.array_equal(got_i.cpu().numpy(), want_i)
        assert np.array_equal(got_w.cpu().numpy().view(np.uint32), want_w.view(np.uint32))
    own_w, own_i = ops.route(torch.from_numpy(logits).cuda(), k, **on_device, **settings)
    again_w, again_i = ops.route(torch.from_numpy(logits).cuda(), k, given=own_i, **on_device, **settings)
    assert torch.equal(again_i, own_i) and torch.equal(again_w, own_w)
    wild = table.copy()
    wild[::3, 0], wild[1::3, -1], wild[5] = experts, experts + 9, -5       # the sentinel itself, a corrupt id, a token with no expert at all
    got_w, got_i = ops.route(torch.from_numpy(logits).cuda(), k, given=torch.from_numpy(wild).cuda(), **on_device, **settings)
    want_w, want_i = oracle.route(logits, k, bias=bias, given=wild, **settings)
    assert np.array_equal(want_i, wild) and np.array_equal(got_i.cpu().numpy(), want_i)
    assert np.array_equal(got_w.cpu().numpy().view(np.uint32), want_w.view(np.uint32))
    outside = (wild < 0) | (wild >= experts)
    assert not got_w.cpu().numpy()[outside].any() and not got_w.cpu().numpy()[5].any()
    plan = ops.sort_by_expert(got_i, experts)                                # the sort drops those slots: they belong to no group
    assert int(plan.sizes.sum()) == int((~outside).sum()) and int(plan.offsets[-1]) == int((~outside).sum())
    with pytest.raises(ops.KernelError, match="replayed routing"):
        ops.route(torch.from_numpy(logits).cuda(), k, given=torch.from_numpy(table[:, :1].copy()).cuda(), **settings)
    with pytest.raises(ops.KernelError, match="coverage"):
        ops.route(torch.from_numpy(logits).cuda(), k, covered=torch.from_numpy(covered).cuda(), **settings)


@pytest.mark.parametrize("experts,k,groups,kept,biased", [(256, 8, 8, 4, True), (64, 6, 1, 1, True), (32, 2, 4, 2, False)])
def test_media_tokens_are_chosen_for_by_the_media_bias(ops, experts, k, groups, kept, biased):
    """DeepSeek-V4.1's image-span bias (`media_bias`, src/dew/nn/moe.py:342-344, 516-524) in the route kernel, against the
    oracle bit for bit, through the kernel's wrapper and through the `Router` mirror's `media` argument."""
    from dew_amd import moe
    rng = np.random.default_rng(experts + k)
    tokens = 300
    logits = (rng.standard_normal((tokens, experts)) * 1.5).astype(np.float32)
    bias = (rng.standard_normal(experts) * 0.3).astype(np.float32) if biased else None
    media_bias = (rng.standard_normal(experts) * 0.3).astype(np.float32)
    media = rng.integers(0, 2, size=tokens).astype(bool)
    settings = dict(score_function="sigmoid", routed_scaling_factor=2.5, expert_groups=groups, groups_per_token=kept)
    want_w, want_i = oracle.route(logits, k, bias=bias, media=media, media_bias=media_bias, **settings)
    got_w, got_i = ops.route(torch.from_numpy(logits).cuda(), k, bias=None if bias is None else torch.from_numpy(bias).cuda(),
                             media=torch.from_numpy(media).cuda(), media_bias=torch.from_numpy(media_bias).cuda(), **settings)
    assert np.array_equal(got_i.cpu().numpy(), want_i) and np.array_equal(got_w.cpu().numpy().view(np.uint32), want_w.view(np.uint32))
    variables = {"params": {}, "moe": {"media_bias": torch.from_numpy(media_bias).cuda()}}
    if biased:
        variables["moe"]["e_score_correction_bias"] = torch.from_numpy(bias).cuda()
    router = moe.Router(experts, 128, k, expert_bias=biased, media_bias=True, **settings)._bound(variables, ())
    mirror_w, mirror_i = router.routed(torch.from_numpy(logits).cuda(), media=torch.from_numpy(media).cuda())
    assert torch.equal(mirror_i, got_i) and torch.equal(mirror_w, got_w)
    with pytest.raises(ValueError, match="only a router with a media bias"):
        moe.Router(experts, 128, k, **settings)._bound(variables, ()).routed(torch.from_numpy(logits).cuda(), media=torch.from_numpy(media).cuda())
    with pytest.raises(ops.KernelError, match="come together"):
        ops.route(torch.from_numpy(logits).cuda(), k, media=torch.from_numpy(media).cuda(), **settings)


@pytest.mark.parametrize("score_function,experts,k,allowed,rows,length,block,biased",
                         [("sigmoid", 64, 4, 8, 3, 50, 8, True), ("softmax", 256, 8, 16, 2, 129, 32, False),
                          ("sigmoid", 128, 6, 6, 5, 17, 4, True), ("sqrtsoftplus", 32, 2, 32, 1, 64, 16, False),
                          ("softmax", 8, 2, 3, 4, 9, 1, True), ("sigmoid", 512, 8, 24, 1, 40, 8, False)])
def test_block_routing_chooses_within_each_blocks_shortlist(ops, score_function, experts, k, allowed, rows, length, block, biased):
    """LLaDA2.2's block routing (`dew_moe_route_blocks`) against the oracle's `block_mask`, bit for bit: whole and partial
    blocks, padding inside and behind a row (a block of its own), a shortlist as short as the top-k and as long as the
    experts, and the `Router` mirror's `blocks` argument."""
    from dew_amd import moe
    rng = np.random.default_rng(experts + length)
    logits = (rng.standard_normal((rows, length, experts)) * 1.5).astype(np.float32)
    bias = (rng.standard_normal(experts) * 0.2).astype(np.float32) if biased else None
    blocks = np.tile(np.arange(length) // block, (rows, 1)).astype(np.int32)
    blocks[0, length - 3:] = -1                       # padding behind the row
    if rows > 1:
        blocks[1, 2] = -1                             # ... and inside one
    settings = dict(score_function=score_function, routed_scaling_factor=1.5)
    want_w, want_i = oracle.route(logits, k, bias=bias, blocks=blocks, block_experts=allowed, **settings)
    got_w, got_i = ops.route_blocks(torch.from_numpy(logits).cuda(), k, torch.from_numpy(blocks).cuda(), allowed,
                                    bias=None if bias is None else torch.from_numpy(bias).cuda(), **settings)
    assert np.array_equal(got_i.cpu().numpy(), want_i)
    assert np.array_equal(got_w.cpu().numpy().view(np.uint32), want_w.view(np.uint32))
    if allowed < experts:
        assert not np.array_equal(want_i, oracle.route(logits, k, bias=bias, **settings)[1])
    variables = {"params": {}, "moe": {} if bias is None else {"e_score_correction_bias": torch.from_numpy(bias).cuda()}}
    router = moe.Router(experts, 128, k, expert_bias=biased, routing_block=block, block_experts=allowed, **settings)._bound(variables, ())
    mirror_w, mirror_i = router.chosen(torch.from_numpy(logits).cuda(), blocks=torch.from_numpy(blocks).cuda())
    assert torch.equal(mirror_i, got_i) and torch.equal(mirror_w, got_w)
    with pytest.raises(ValueError, match="only a block router reads them"):
        moe.Router(experts, 128, k, **settings)._bound(variables, ()).chosen(torch.from_numpy(logits).cuda(), blocks=torch.from_numpy(blocks).cuda())
    with pytest.raises(ValueError, match="from the blocks its caller numbers"):
        router.chosen(torch.from_numpy(logits).cuda())
    with pytest.raises(ops.KernelError, match="block_experts"):
        ops.route_blocks(torch.from_numpy(logits).cuda(), k, torch.from_numpy(blocks).cuda(), k - 1, **settings)


def test_a_hash_router_takes_its_experts_from_the_token_table(ops):
    """DeepSeek V4's hash router (`hash_vocab`, src/dew/nn/moe.py:337-341, 500-507): the experts are `tid2eid[token id]`,
    weighted by the learned gate; a replayed record covers some tokens over it; only a hash router reads token ids."""
    from dew_amd import moe
    rng = np.random.default_rng(31)
    vocab, experts, k, width = 50, 16, 3, 128
    kernel = (rng.standard_normal((width, experts)) * 0.2).astype(np.float32)
    table = rng.integers(0, experts, size=(vocab, k)).astype(np.int32)
    x = torch.from_numpy(rng.standard_normal((2, 9, width)).astype(np.float32)).to(torch.bfloat16)
    ids = rng.integers(0, vocab, size=(2, 9))
    variables = {"params": {"kernel": torch.from_numpy(kernel).cuda()}, "moe": {"tid2eid": torch.from_numpy(table).cuda()}}
    router = moe.Router(experts, width, k, score_function="sqrtsoftplus", routed_scaling_factor=1.5, hash_vocab=vocab)
    weights, indices = router.apply(variables, x.cuda(), torch.from_numpy(ids).cuda())
    logits = oracle.router_logits(x.float().numpy().reshape(-1, width), kernel)
    want_w, want_i = oracle.route(logits, k, score_function="sqrtsoftplus", routed_scaling_factor=1.5, given=table[ids.reshape(-1)])
    assert indices.shape == (2, 9, k) and np.array_equal(indices.cpu().numpy().reshape(-1, k), table[ids.reshape(-1)])
    assert np.abs(weights.cpu().numpy().reshape(-1, k) - want_w).max() <= 1e-6
    replayed = rng.integers(0, experts, size=(2, 9, k)).astype(np.uint8)          # engines ship the narrowest unsigned type
    covers = rng.integers(0, 2, size=(2, 9)).astype(bool)
    _, mixed = router.apply(variables, x.cuda(), torch.from_numpy(ids).cuda(), routes=(torch.from_numpy(replayed).cuda(), torch.from_numpy(covers).cuda()))
    assert np.array_equal(mixed.cpu().numpy(), np.where(covers[..., None], replayed.astype(np.int32), table[ids]))
    with pytest.raises(ValueError, match="token ids, which the caller passes"):
        router.apply(variables, x.cuda())
    with pytest.raises(ValueError, match="only a hash router"):
        moe.Router(experts, width, k).apply(variables, x.cuda(), torch.from_numpy(ids).cuda())
    with pytest.raises(ValueError, match="expert ids"):
        moe.Router(experts, width, k).apply(variables, x.cuda(), routes=(torch.zeros(2, 9, k).cuda(), None))


def test_router_refuses_bounds_that_bound_nothing(ops):
    logits = torch.zeros(4, 8, device="cuda")
    with pytest.raises(ops.KernelError, match="bias_in_weights"):
        ops.route(logits, 2, bias_in_weights=True)
    with pytest.raises(ops.KernelError, match="weight_sum"):
        ops.route(logits, 2, weight_sum_min=-1.0)
    with pytest.raises(ops.KernelError, match="logit_softcap"):
        ops.route(logits, 2, logit_softcap=-3.0)


def test_a_nan_selection_bias_is_never_chosen_and_every_choice_stays_in_range(ops):
    """A NaN in the selection bias makes that expert's selection NaN for every token. It competes as -inf: never
    chosen while k others remain, and when fewer remain the lowest remaining indices fill in, all within range."""
    rng = np.random.default_rng(3)
    experts, k, tokens = 64, 6, 257
    logits = rng.standard_normal((tokens, experts)).astype(np.float32)
    settings = dict(score_function="sigmoid", normalize_weights=True, routed_scaling_factor=1.5)
    for poisoned in ([5], list(range(60)), list(range(64))):
        bias = (rng.standard_normal(experts) * 0.1).astype(np.float32)
        bias[poisoned] = np.nan
        want_w, want_i = oracle.route(logits, k, bias=bias, **settings)
        got_w, got_i = ops.route(torch.from_numpy(logits).cuda(), k, bias=torch.from_numpy(bias).cuda(), **settings)
        got_i = got_i.cpu().numpy()
        assert got_i.min() >= 0 and got_i.max() < experts
        assert np.array_equal(got_i, want_i)
        assert np.array_equal(got_w.cpu().numpy().view(np.uint32), want_w.view(np.uint32))
        if len(poisoned) <= experts - k:
            assert not np.isin(got_i, poisoned).any()


def test_router_reproduces_the_reference_fixtures_on_the_device(ops):
    from conftest import golden
    for name, settings in (("mixtral", dict(score_function="softmax", normalize_weights=True)),
                           ("deepseek", dict(score_function="sigmoid", normalize_weights=True, routed_scaling_factor=2.5,
                                             expert_groups=4, groups_per_token=2)),
                           ("deepseek_v2", dict(score_function="softmax", normalize_weights=False, routed_scaling_factor=2.5,
                                                expert_groups=4, groups_per_token=2, group_score="max")),
                           ("deepseek_v4", dict(score_function="sqrtsoftplus", normalize_weights=True, routed_scaling_factor=2.5))):
        held = golden(f"moe/{name}.npz")
        hidden = held["hidden"].reshape(-1, 16)
        logits = oracle.router_logits(hidden, held["mlp.gate.weight"].T)
        bias = held.get("mlp.gate.e_score_correction_bias") if name in ("deepseek", "deepseek_v4") else None
        k = held["router_indices"].shape[-1]
        weights, indices = ops.route(torch.from_numpy(logits).cuda(), k,
                                     bias=None if bias is None else torch.from_numpy(bias).cuda(), **settings)
        order_theirs = np.argsort(held["router_indices"], -1, kind="stable")
        order_ours = np.argsort(indices.cpu().numpy(), -1, kind="stable")
        assert np.array_equal(np.take_along_axis(indices.cpu().numpy(), order_ours, -1),
                              np.take_along_axis(held["router_indices"], order_theirs, -1))
        assert np.abs(np.take_along_axis(weights.cpu().numpy(), order_ours, -1)
                      - np.take_along_axis(held["router_weights"], order_theirs, -1)).max() < 1e-6


@pytest.mark.parametrize("tokens,k,experts", [(1, 1, 1), (7, 2, 4), (64, 8, 128), (300, 3, 5), (2048, 2, 8),
                                               (1025, 2, 8), (16384, 2, 8), (8192, 8, 256), (3000, 6, 512), (1024, 8, 128), (1025, 8, 64),
                                               (512, 8, 960), (100, 4, 1000), (700, 4, 1000), (2049, 2, 8)])
def test_permute_is_the_stable_sort_by_expert(ops, tokens, k, experts):
    rng = np.random.default_rng(tokens * 31 + experts)
    indices = rng.integers(0, experts, size=(tokens, k)).astype(np.int32)
    if experts > 2:
        indices[indices == 1] = 2                          # an empty expert
    want = oracle.sorted_by_expert(indices, experts)
    got = ops.sort_by_expert(torch.from_numpy(indices).cuda(), experts)
    for field in ("sizes", "offsets", "order", "rows"):
        assert np.array_equal(getattr(got, field).cpu().numpy(), want[field]), field


@pytest.mark.parametrize("tokens,k,experts", [(1, 1, 1), (7, 2, 4), (64, 8, 128), (300, 3, 5), (1025, 2, 8), (8192, 8, 256), (3000, 6, 511)])
def test_permute_with_a_shared_expert_as_one_more_group(ops, tokens, k, experts):
    rng = np.random.default_rng(tokens * 31 + experts)
    indices = rng.integers(0, experts, size=(tokens, k)).astype(np.int32)
    if experts > 2:
        indices[indices == 1] = 2                          # an empty expert
    if tokens > 5:
        indices[3, 0] = experts                            # a dropped slot: it sorts behind the shared group
    want = oracle.sorted_with_shared(indices, experts, tokens)
    got = ops.sort_by_expert(torch.from_numpy(indices).cuda(), experts, shared_rows=tokens)
    for field in ("sizes", "offsets", "order", "rows"):
        assert np.array_equal(getattr(got, field).cpu().numpy(), want[field]), field


def test_permute_sorts_dropped_slots_last_and_outside_every_group(ops):
    indices = np.array([[0, 3], [3, 1], [2, 3], [0, 0]], np.int32)      # id 3 = the sentinel of 3 experts
    got = ops.sort_by_expert(torch.from_numpy(indices).cuda(), 3)
    assert got.sizes.tolist() == [3, 1, 1] and got.offsets.tolist() == [0, 3, 4, 5]
    assert got.order.tolist() == [0, 6, 7, 3, 4, 1, 2, 5]


def grouped_case(quant, experts, depth, width, sizes, seed):
    rng = np.random.default_rng(seed)
    weight = torch.from_numpy((rng.standard_normal((experts, depth, width)) * 0.02).astype(np.float32))
    bank = quantize(weight, quant)
    rows = int(np.sum(sizes))
    x = torch.from_numpy(rng.standard_normal((rows, depth)).astype(np.float32)).to(torch.bfloat16)
    offsets = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int32)
    return bank, x, offsets


SIZES = [("ragged", [130, 0, 1, 257, 64, 0, 127, 5]), ("single", [3]), ("even", [128, 128, 128, 128])]


@pytest.mark.parametrize("tile", [0, 32, 64, 128])
@pytest.mark.parametrize("quant", ["fp8_channel", "fp8_block", "mxfp4", "nvfp4", "bf16"])
@pytest.mark.parametrize("label,sizes", SIZES, ids=[s[0] for s in SIZES])
def test_grouped_gemm_matches_the_dequantized_fp32_sum(ops, quant, label, sizes, tile):
    """bf16 x decoded-weight products are exact in fp32, so kernel and oracle differ by summation order
    alone before the one bf16 rounding: allow one bf16 ulp of the largest output (at most 2^-7 of it)."""
    bank, x, offsets = grouped_case(quant, len(sizes), 512, 256, sizes, seed=len(sizes) * 7 + len(quant))
    values, factor = dequantized(bank)
    want = oracle.grouped_matmul(bf16_np(x), values, sizes, factor=factor)
    with ops.tile_rows(tile):
        got = bf16_np(ops.grouped_gemm(x.cuda(), ops.prepare(bank.to("cuda")), torch.from_numpy(offsets).cuda()))
    scale = np.abs(want).max()
    assert np.abs(got - want).max() <= 2 ** -7 * scale
    assert (np.abs(got - want) <= 2 ** -7 * np.abs(want) + 1e-5 * scale).all()
    assert (got == want).mean() > 0.97                     # nearly every element rounds identically


def test_grouped_gemm_is_exact_on_small_integers(ops):
    """Known answer: integer rows times an MXFP4 bank of small powers of two sum exactly in fp32
    (the reference's tests/test_gemm_nvfp4.py:41-52 states the same for its product)."""
    rng = np.random.default_rng(11)
    sizes = [40, 0, 100, 3]
    weight = torch.from_numpy(rng.choice([-1.0, -0.5, 0.0, 0.5, 1.0, 2.0], size=(4, 256, 128)).astype(np.float32))
    bank = quantize(weight, "mxfp4")
    x = torch.from_numpy(rng.integers(-3, 4, size=(143, 256)).astype(np.float32)).to(torch.bfloat16)
    offsets = torch.tensor(np.concatenate([[0], np.cumsum(sizes)]), dtype=torch.int32)
    got = bf16_np(ops.grouped_gemm(x.cuda(), ops.prepare(bank.to("cuda")), offsets.cuda()))
    want = np.zeros((143, 128))
    start = 0
    for e, size in enumerate(sizes):
        want[start:start + size] = bf16_np(x)[start:start + size].astype(np.float64) @ weight[e].numpy().astype(np.float64)
        start += size
    assert np.array_equal(got.astype(np.float64), oracle.bf16_round(want.astype(np.float32)).astype(np.float64))


def test_grouped_gemm_gathers_scatters_and_zeroes_unrouted_rows(ops):
    rng = np.random.default_rng(5)
    sizes = [70, 0, 130]
    bank, _, offsets = grouped_case("fp8_block", 3, 256, 128, sizes, seed=3)
    tokens = torch.from_numpy(rng.standard_normal((50, 256)).astype(np.float32)).to(torch.bfloat16)
    rows = 210                                              # 10 sorted positions past sum(sizes)
    gather = rng.integers(0, 50, size=rows).astype(np.int32)
    scatter = rng.permutation(rows).astype(np.int32)
    values, _ = dequantized(bank)
    want_sorted = oracle.grouped_matmul(bf16_np(tokens)[gather], values, sizes)
    want = np.zeros_like(want_sorted)
    want[scatter] = want_sorted
    got = bf16_np(ops.grouped_gemm(tokens.cuda(), ops.prepare(bank.to("cuda")), torch.from_numpy(offsets).cuda(),
                                   gather=torch.from_numpy(gather).cuda(), scatter=torch.from_numpy(scatter).cuda(), rows=rows))
    assert not got[scatter[200:]].any()
    assert np.abs(got - want).max() <= 2 ** -7 * np.abs(want).max()


@pytest.mark.parametrize("tile", [0, 32, 64, 128])
@pytest.mark.parametrize("quant", ["fp8_channel", "fp8_block", "mxfp4", "nvfp4", "bf16"])
def test_gateup_swiglu_matches_the_two_products_and_the_rounded_epilogue(ops, quant, tile):
    sizes = [100, 0, 37, 200]
    rng = np.random.default_rng(21)
    gate, x, offsets = grouped_case(quant, 4, 512, 256, sizes, seed=1)
    up, _, _ = grouped_case(quant, 4, 512, 256, sizes, seed=2)
    gather = rng.integers(0, x.shape[0], size=x.shape[0]).astype(np.int32)
    gate_values, gate_factor = dequantized(gate)
    up_values, up_factor = dequantized(up)
    rows = bf16_np(x)[gather]
    want_gate = oracle.grouped_matmul(rows, gate_values, sizes, factor=gate_factor)
    want_up = oracle.grouped_matmul(rows, up_values, sizes, factor=up_factor)
    want = oracle.swiglu(want_gate, want_up)
    xd, od, gd = x.cuda(), torch.from_numpy(offsets).cuda(), torch.from_numpy(gather).cuda()
    pg, pu = ops.prepare(gate.to("cuda")), ops.prepare(up.to("cuda"))
    with ops.tile_rows(tile):
        fused = bf16_np(ops.gateup_swiglu(xd, pg, pu, od, gather=gd))
        apart = ops.swiglu(ops.grouped_gemm(xd, pg, od, gather=gd), ops.grouped_gemm(xd, pu, od, gather=gd))
    assert np.array_equal(fused, bf16_np(apart))           # the fused epilogue is the unfused arithmetic
    scale = np.abs(want).max()
    # a one-ulp difference in gate or up moves the product by up to ~3 ulp of the result
    assert np.abs(fused - want).max() <= 2 ** -6 * scale
    assert (fused == want).mean() > 0.9


@pytest.mark.parametrize("tokens,depth,experts,biased", [(1, 64, 8, False), (37, 512, 16, True), (64, 2880, 32, True), (100, 2048, 128, False),
                                                         (257, 1024, 160, True), (96, 7168, 256, False), (33, 768, 384, True),
                                                         (8200, 256, 160, True), (3000, 128, 40, False), (50, 520, 60, True), (70, 72, 600, False)])
def test_gate_logits_are_fp32_products_summed_in_fp32(ops, tokens, depth, experts, biased):
    """`Router.logits` (src/dew/nn/moe.py:526-534): bf16 tokens widened to fp32 times the fp32 gate kernel, IEEE fp32.
    Against the float64 product: within a few fp32 roundings of the summed magnitudes, on the matrix-instruction kernel
    (depths in whole 16s, up to 512 experts) and the plain one (the last two shapes); tokens in no whole 32s, experts in
    no whole 32s, a bias on the finished sums."""
    rng = np.random.default_rng(tokens + depth + experts)
    x = torch.from_numpy(rng.standard_normal((tokens, depth)).astype(np.float32)).to(torch.bfloat16)
    kernel = torch.from_numpy((rng.standard_normal((depth, experts)) * depth ** -0.5).astype(np.float32))
    bias = torch.from_numpy(rng.standard_normal(experts).astype(np.float32)) if biased else None
    guard = torch.full((tokens + 1, experts), 7.0, dtype=torch.float32, device="cuda")
    got = ops.router_logits(x.cuda(), kernel.cuda(), None if bias is None else bias.cuda())
    assert got.shape == (tokens, experts) and got.dtype == torch.float32 and bool(guard.eq(7.0).all())
    exact = x.double().numpy() @ kernel.double().numpy()
    magnitudes = np.abs(x.double().numpy()) @ np.abs(kernel.double().numpy())
    if biased:
        exact = exact + bias.double().numpy()
        magnitudes = magnitudes + np.abs(bias.double().numpy())
    assert np.all(np.abs(got.cpu().numpy() - exact) <= 2.0 ** -19 * magnitudes + 1e-30)
    want = oracle.router_logits(x.float().numpy(), kernel.numpy())
    if biased:
        want = want + bias.numpy()
    assert np.abs(got.cpu().numpy() - want).max() <= 1e-5 * np.abs(want).max()
    assert torch.equal(got, ops.router_logits(x.cuda(), kernel.cuda(), None if bias is None else bias.cuda()))   # the same bits every time


@pytest.mark.parametrize("tile", [0, 32, 128])
@pytest.mark.parametrize("activation,limit", [("swiglu", 0.25), ("geglu", None), ("geglu", 0.5)])
@pytest.mark.parametrize("quant", ["fp8_channel", "fp8_block", "mxfp4", "nvfp4", "bf16"])
def test_a_clamp_or_the_geglu_gate_as_the_paired_launchs_epilogue(ops, quant, activation, limit, tile):
    """`dew_moe_gateup_gated`: the launch's epilogue clamps and gates as the stand-alone gating kernel does over the two
    products, bit for bit, and agrees with the oracle's `swiglu_clamped` / `gated_product` of its own products; the
    groups arrive as offsets or as sizes."""
    sizes = [100, 0, 37, 200]
    rng = np.random.default_rng(23)
    gate, x, offsets = grouped_case(quant, 4, 512, 256, sizes, seed=5)
    up, _, _ = grouped_case(quant, 4, 512, 256, sizes, seed=6)
    gather = rng.integers(0, x.shape[0], size=x.shape[0]).astype(np.int32)
    gate_values, gate_factor = dequantized(gate)
    up_values, up_factor = dequantized(up)
    rows = bf16_np(x)[gather]
    want = oracle.GATED_PRODUCTS[activation](oracle.grouped_matmul(rows, gate_values, sizes, factor=gate_factor),
                                             oracle.grouped_matmul(rows, up_values, sizes, factor=up_factor), dtype="bfloat16", limit=limit)
    xd, od, gd = x.cuda(), torch.from_numpy(offsets).cuda(), torch.from_numpy(gather).cuda()
    pg, pu = ops.prepare(gate.to("cuda")), ops.prepare(up.to("cuda"))
    with ops.tile_rows(tile):
        fused = bf16_np(ops.gateup_swiglu(xd, pg, pu, od, gather=gd, activation=activation, limit=limit))
        by_sizes = bf16_np(ops.gateup_swiglu(xd, pg, pu, None, gather=gd, sizes=torch.tensor(sizes, dtype=torch.int32).cuda(),
                                             activation=activation, limit=limit))
        apart = ops.gated_product(ops.grouped_gemm(xd, pg, od, gather=gd), ops.grouped_gemm(xd, pu, od, gather=gd), activation, limit)
        plain = bf16_np(ops.gateup_swiglu(xd, pg, pu, od, gather=gd))
    assert np.array_equal(fused, bf16_np(apart)) and np.array_equal(by_sizes, fused)
    assert not np.array_equal(plain, fused)                 # (the clamp bites and the gates differ on these inputs)
    scale = np.abs(want).max()
    assert np.abs(fused - want).max() <= 2 ** -6 * scale
    assert (fused == want).mean() > 0.9


def test_the_gated_launch_refuses_what_it_cannot_run(ops):
    gate, x, offsets = grouped_case("bf16", 2, 128, 128, [8, 8], seed=1)
    pg = ops.prepare(gate.to("cuda"))
    xd, od = x.cuda(), torch.from_numpy(offsets).cuda()
    with pytest.raises(ops.KernelError, match="one of"):
        ops.gateup_swiglu(xd, pg, pg, od, activation="geglu_exact")
    with pytest.raises(ops.KernelError, match="positive"):
        ops.gateup_swiglu(xd, pg, pg, od, limit=0.0)


def test_swiglu_kernel_matches_the_oracle_on_every_bf16_gate(ops):
    gate_bits = np.arange(65536, dtype=np.uint16)
    gate = oracle.bf16_from_bits(gate_bits)
    keep = np.isfinite(gate)
    gate = gate[keep]
    gate = np.concatenate([gate, np.zeros(-gate.size % 8, np.float32)])
    up = np.resize(np.array([1.0, -0.75, 3.140625, 1e-3, 100.0, 2 ** -20, -7.0, 0.5], np.float32), gate.shape)
    want = oracle.swiglu(gate, up)
    got = bf16_np(ops.swiglu(torch.from_numpy(gate).to(torch.bfloat16).cuda(), torch.from_numpy(up).to(torch.bfloat16).cuda()))
    mismatched = (got != want) & ~(np.isnan(got) & np.isnan(want))
    # exp differs in the last fp32 place between libraries; after two bf16 roundings that flips at most a
    # handful of results by one ulp
    assert mismatched.mean() < 2e-3
    assert np.abs(got - want)[mismatched].max(initial=0) <= 2 ** -7 * np.abs(want)[mismatched].max(initial=1)


def test_geglu_kernel_matches_the_oracle_on_every_bf16_gate(ops):
    gate = oracle.bf16_from_bits(np.arange(65536, dtype=np.uint16))
    gate = gate[np.isfinite(gate) & (np.abs(gate) < 1e12)]     # (beyond, the gate's cube overflows fp32: inf - inf on both sides)
    gate = np.concatenate([gate, np.zeros(-gate.size % 8, np.float32)])
    up = np.resize(np.array([1.0, -0.75, 3.140625, 1e-3, 100.0, 2 ** -20, -7.0, 0.5], np.float32), gate.shape)
    for limit in (None, 2.0):
        want = oracle.geglu(gate, up, limit=limit)
        got = bf16_np(ops.gated_product(torch.from_numpy(gate).to(torch.bfloat16).cuda(), torch.from_numpy(up).to(torch.bfloat16).cuda(),
                                        "geglu", limit))
        mismatched = (got != want) & ~(np.isnan(got) & np.isnan(want))
        assert mismatched.mean() < 2e-3                    # the hardware exponential against the library's: a last bf16 bit, rarely
        assert np.abs(got - want)[mismatched].max(initial=0) <= 2 ** -7 * np.abs(want)[mismatched].max(initial=1)
    with pytest.raises(ops.KernelError, match="activation"):
        ops.gated_product(torch.zeros(8, dtype=torch.bfloat16, device="cuda"), torch.zeros(8, dtype=torch.bfloat16, device="cuda"), "reglu")


def test_the_gating_kernels_reproduce_torchs_recorded_bf16_products(ops):
    """The reference's tests/fixtures/gated_product/bf16.npz (Torch's bf16 `silu(gate) * up` and tanh-GELU product on 2048
    drawn pairs, the arm the reference's own product is held to): SwiGLU bit for bit; GeGLU bit for bit but where the
    hardware exponential moves a last bf16 bit, and where Torch's tanh has saturated (its 0 against a product below 1e-16)."""
    from conftest import golden
    held = golden("gated_product/bf16.npz")

    def on_device(name):
        return torch.from_numpy(held[name]).to(torch.bfloat16).cuda()

    got = bf16_np(ops.gated_product(on_device("swiglu/gate"), on_device("swiglu/up"), "swiglu"))
    assert np.array_equal(got, held["swiglu/output"])
    got = bf16_np(ops.gated_product(on_device("geglu/gate"), on_device("geglu/up"), "geglu"))
    want = held["geglu/output"]
    differs = got != want
    saturated = differs & (want == 0)
    assert np.abs(got[saturated]).max(initial=0) < 1e-16
    assert (differs & ~saturated).sum() <= 4 and np.all(np.abs(got - want)[differs & ~saturated] <= 2 ** -7 * np.abs(want[differs & ~saturated]))


def test_combine_weighs_in_fp32_and_rounds_once(ops):
    slots = torch.tensor([[[1.0] * 8, [-1.0] * 8]], dtype=torch.bfloat16)     # tests/test_moe_precision.py:652-674
    weights = torch.tensor([[0.5 + 2 ** -11, 0.5 - 2 ** -11]], dtype=torch.float32)
    assert (ops.combine(slots.cuda(), weights.cuda()).float().cpu() == 2.0 ** -10).all()
    rng = np.random.default_rng(8)
    slots = torch.from_numpy(rng.standard_normal((333, 8, 512)).astype(np.float32)).to(torch.bfloat16)
    weights = torch.from_numpy(rng.uniform(0, 1, size=(333, 8)).astype(np.float32))
    addend = torch.from_numpy(rng.standard_normal((333, 512)).astype(np.float32)).to(torch.bfloat16)
    want = oracle.combine(bf16_np(slots), weights.numpy())
    assert np.array_equal(bf16_np(ops.combine(slots.cuda(), weights.cuda())), want)
    with_shared = oracle.bf16_round(want + bf16_np(addend))
    assert np.array_equal(bf16_np(ops.combine(slots.cuda(), weights.cuda(), addend.cuda())), with_shared)


def test_entry_points_refuse_what_they_cannot_run(ops):
    from dew_amd._lib import KernelError
    with pytest.raises(KernelError, match="top_k"):
        ops.route(torch.zeros((4, 8), device="cuda"), 9)
    with pytest.raises(KernelError, match="multiple of 128"):
        ops.prepare(quantize(torch.zeros((1, 128, 64)), "fp8_block").to("cuda"))
    with pytest.raises(KernelError, match="GPU"):
        ops.route(torch.zeros((4, 8)), 2)
    bank = ops.prepare(quantize(torch.zeros((2, 128, 128)), "fp8_block").to("cuda"))
    with pytest.raises(KernelError, match="deep"):
        ops.grouped_gemm(torch.zeros((4, 256), dtype=torch.bfloat16, device="cuda"), bank,
                         torch.zeros(3, dtype=torch.int32, device="cuda"))


@pytest.mark.parametrize("quant", ["mxfp4", "nvfp4", "bf16"])
def test_large_tile_kernels_match_the_oracle(ops, quant):
    """The 256-row tiles (paired 256 x 2 x 128, one bank 256 x 256), which launches take for FP4 banks whose groups
    average 1024 rows or more; forced here so that a small problem reaches them."""
    sizes = [1100, 700]
    gate, x, offsets = grouped_case(quant, 2, 256, 256, sizes, seed=31)
    up, _, _ = grouped_case(quant, 2, 256, 256, sizes, seed=32)
    gate_values, gate_factor = dequantized(gate)
    up_values, up_factor = dequantized(up)
    rows = bf16_np(x)
    want_gate = oracle.grouped_matmul(rows, gate_values, sizes, factor=gate_factor)
    want = oracle.swiglu(want_gate, oracle.grouped_matmul(rows, up_values, sizes, factor=up_factor))
    xd, od = x.cuda(), torch.from_numpy(offsets).cuda()
    pg, pu = ops.prepare(gate.to("cuda")), ops.prepare(up.to("cuda"))
    with ops.tile_rows(256):
        got_gate = bf16_np(ops.grouped_gemm(xd, pg, od))
        fused = bf16_np(ops.gateup_swiglu(xd, pg, pu, od))
    assert np.abs(got_gate - want_gate).max() <= 2 ** -7 * np.abs(want_gate).max() and (got_gate == want_gate).mean() > 0.97
    assert np.abs(fused - want).max() <= 2 ** -6 * np.abs(want).max() and (fused == want).mean() > 0.9


def test_an_mxfp4_bank_is_recognized_at_preparation_and_a_general_bank_is_not(ops):
    from dew_amd import _lib
    weight = torch.from_numpy((np.random.default_rng(3).standard_normal((2, 256, 128)) * 0.02).astype(np.float32))
    assert ops.prepare(quantize(weight, "mxfp4").to("cuda")).descriptor.format == _lib.W_MXFP4
    assert ops.prepare(quantize(weight, "nvfp4").to("cuda")).descriptor.format == _lib.W_NVFP4


def test_the_benchmarks_probes_run_and_the_copy_probe_copies():
    from bench_aids import probes

    src = torch.arange(1 << 20, dtype=torch.int32, device="cuda")
    dst = torch.zeros_like(src)
    assert probes.probe_copy(src, dst) == 4 << 20 and torch.equal(src, dst)
    assert probes.probe_mfma(torch.randn(16384, device="cuda").to(torch.bfloat16), 10) == 1024 * 4 * 10 * 16 * 32768.0


@pytest.mark.parametrize("quant", ["fp8_channel", "fp8_block", "mxfp4", "nvfp4", "bf16"])
@pytest.mark.parametrize("depth", [128, 384, 640, 896])
@pytest.mark.parametrize("label,sizes,tile", [("decode", [3, 0, 9], 32), ("small", [40, 70, 1], 64), ("medium", [150, 70, 1], 128),
                                               ("large", [800], 256)])
def test_depths_that_leave_steps_after_the_unrolled_loop(ops, quant, depth, label, sizes, tile):
    """Depth / 64 steps that are not a multiple of the main loop's unroll (3 or 4) end in separately compiled
    steps; both launches must still agree with the oracle and with each other. Each tile height is forced, since
    problems this small would all be given 32-row tiles."""
    if quant in ("mxfp4", "nvfp4"):
        depth = 2 * depth  # an NvFp4 bank's depth is whole 256s
    gate, x, offsets = grouped_case(quant, len(sizes), depth, 256, sizes, seed=depth + len(quant))
    up, _, _ = grouped_case(quant, len(sizes), depth, 256, sizes, seed=depth + 50)
    gate_values, gate_factor = dequantized(gate)
    rows = bf16_np(x)
    want_gate = oracle.grouped_matmul(rows, gate_values, sizes, factor=gate_factor)
    xd, od = x.cuda(), torch.from_numpy(offsets).cuda()
    pg, pu = ops.prepare(gate.to("cuda")), ops.prepare(up.to("cuda"))
    with ops.tile_rows(tile):
        fused = bf16_np(ops.gateup_swiglu(xd, pg, pu, od))
        got_gate = ops.grouped_gemm(xd, pg, od)
        apart = bf16_np(ops.swiglu(got_gate, ops.grouped_gemm(xd, pu, od)))
    assert np.array_equal(fused, apart)
    got_gate = bf16_np(got_gate)
    assert np.abs(got_gate - want_gate).max() <= 2 ** -7 * np.abs(want_gate).max() + 1e-6
    assert (got_gate == want_gate).mean() > 0.97


def test_split_rows_is_exact_within_eleven_binades_of_the_row_maximum(ops):
    rng = np.random.default_rng(17)
    rows, depth = 64, 512
    x = rng.standard_normal((rows, depth)).astype(np.float32)
    x[8:16] *= 10.0 ** rng.uniform(-4, 4, size=(8, depth)).astype(np.float32)     # twenty-six binades in a row
    x[16] = 0.0
    x[17, 5] = 3.0e4                                                                # one outlier over a row of ~1
    x[18] *= 1e-30
    xb = torch.from_numpy(x).to(torch.bfloat16)
    split, scale = ops.split_rows(xb.cuda())
    # each 64 depths: [group][term][half][16] with depth = 32 half + 16 group + j
    split, scale = split.cpu().numpy().reshape(rows, depth // 64, 2, 2, 2, 16), scale.cpu().numpy()
    table = oracle._e4m3_table()
    s = np.ldexp(np.float64(1), scale.astype(np.int64) - 127)[:, None]
    terms = table[split].astype(np.float64)                                        # [rows, 64s, group, term, half, 16]
    values = terms[:, :, :, 0] + terms[:, :, :, 1] / 16                            # [rows, 64s, group, half, 16]
    rebuilt = values.transpose(0, 1, 3, 2, 4).reshape(rows, depth) * s             # depth order: half, group, j
    want = xb.float().numpy().astype(np.float64)
    largest = np.abs(want).max(axis=1, keepdims=True)
    near = np.abs(want) >= largest * 2.0 ** -11
    assert np.array_equal(rebuilt[near], want[near])
    assert (np.abs(rebuilt - want) <= largest * 2.0 ** -21).all()
    assert np.all((largest[:, 0] == 0) | ((largest[:, 0] / s[:, 0] >= 128) & (largest[:, 0] / s[:, 0] < 256)))


@pytest.mark.parametrize("depth", [256, 768, 1280])
def test_split_activations_give_the_bf16_products_on_mxfp4_banks(ops, depth):
    """Two e4m3 terms times the stored FP4 codes under power-of-two scales are the exact bf16 x weight products:
    the scaled-instruction kernels agree with the bf16 kernels up to the order of the fp32 sums."""
    sizes = [700, 0, 290, 5]
    gate, x, offsets = grouped_case("mxfp4", len(sizes), depth, 256, sizes, seed=depth + 1)
    up, _, _ = grouped_case("mxfp4", len(sizes), depth, 256, sizes, seed=depth + 2)
    gate_values, gate_factor = dequantized(gate)
    up_values, up_factor = dequantized(up)
    rng = np.random.default_rng(depth)
    gather = rng.integers(0, x.shape[0], size=x.shape[0]).astype(np.int32)
    scatter = rng.permutation(x.shape[0]).astype(np.int32)
    rows = bf16_np(x)[gather]
    want_gate = oracle.grouped_matmul(rows, gate_values, sizes, factor=gate_factor)
    want = oracle.swiglu(want_gate, oracle.grouped_matmul(rows, up_values, sizes, factor=up_factor))
    xd, od, gd, sd = x.cuda(), torch.from_numpy(offsets).cuda(), torch.from_numpy(gather).cuda(), torch.from_numpy(scatter).cuda()
    pg, pu = ops.prepare(gate.to("cuda")), ops.prepare(up.to("cuda"))
    split, scale = ops.split_rows(xd)
    got_gate = bf16_np(ops.grouped_gemm_split(split, scale, pg, od, gather=gd, scatter=sd))[scatter]
    plain_gate = bf16_np(ops.grouped_gemm(xd, pg, od, gather=gd))
    assert np.abs(got_gate - want_gate).max() <= 2 ** -7 * np.abs(want_gate).max()
    assert (got_gate == want_gate).mean() > 0.97 and (got_gate == plain_gate).mean() > 0.97
    fused = bf16_np(ops.gateup_swiglu_split(split, scale, pg, pu, od, gather=gd))
    assert np.abs(fused - want).max() <= 2 ** -6 * np.abs(want).max() and (fused == want).mean() > 0.9


@pytest.mark.parametrize("depth,width", [(256, 512), (768, 2304)])     # 4 and 18 blocks of scales a row: one and two 16-byte pieces
def test_the_expert_mlp_stays_on_split_rows_without_a_pass_between_its_products(ops, depth, width):
    """gate/up writes its SwiGLU rows already split (one scale per row and 128 columns), down reads them: the hidden
    rows are the bf16 ones exactly, and the output agrees with the bf16 kernels and the oracle."""
    sizes = [700, 0, 290, 5]
    gate, x, offsets = grouped_case("mxfp4", len(sizes), depth, width, sizes, seed=depth + 11)
    up, _, _ = grouped_case("mxfp4", len(sizes), depth, width, sizes, seed=depth + 12)
    down, _, _ = grouped_case("mxfp4", len(sizes), width, 256, sizes, seed=depth + 13)
    rng = np.random.default_rng(depth)
    padded = x.shape[0] + 9                                            # unrouted sorted positions past the last group
    gather = np.concatenate([rng.integers(0, x.shape[0], size=x.shape[0]), np.zeros(9)]).astype(np.int32)
    xd, od, gd = x.cuda(), torch.from_numpy(offsets).cuda(), torch.from_numpy(gather).cuda()
    pg, pu, pd = (ops.prepare(bank.to("cuda")) for bank in (gate, up, down))
    hidden = ops.gateup_swiglu(xd, pg, pu, od, gather=gd, rows=padded)
    hidden_split, hidden_scales = ops.gateup_swiglu_split_out(*ops.split_rows(xd), pg, pu, od, gather=gd, rows=padded)
    # the split rows rebuilt on the host are the bf16 hidden rows
    rows = padded
    pieces = hidden_split.cpu().numpy().reshape(rows, width // 64, 2, 2, 2, 16)
    terms = oracle._e4m3_table()[pieces].astype(np.float64)
    values = (terms[:, :, :, 0] + terms[:, :, :, 1] / 16).transpose(0, 1, 3, 2, 4).reshape(rows, width // 128, 128)
    assert tuple(hidden_scales.shape) == (rows, ops.block_scale_pitch(width))
    s = np.ldexp(np.float64(1), hidden_scales.cpu().numpy()[:, :width // 128].astype(np.int64) - 127)[:, :, None]
    rebuilt = (values * s).reshape(rows, width)
    want_hidden = bf16_np(hidden).astype(np.float64)
    largest = np.abs(want_hidden.reshape(rows, width // 128, 128)).max(axis=2, keepdims=True)
    near = (np.abs(want_hidden.reshape(rows, width // 128, 128)) >= largest * 2.0 ** -11).reshape(rows, width)
    split_hidden_matches = (rebuilt == want_hidden)
    assert (split_hidden_matches | ~near).mean() > 0.97          # up to fp32 summation order in the two kernels' products
    assert np.abs(rebuilt - want_hidden).max() <= 2 ** -6 * np.abs(want_hidden).max()
    assert np.all(rebuilt[x.shape[0]:] == 0)
    out = bf16_np(ops.grouped_gemm_split_blocks(hidden_split, hidden_scales, pd, od, rows=padded))
    plain = bf16_np(ops.grouped_gemm(hidden, pd, od, rows=padded))
    down_values, down_factor = dequantized(down)
    want = oracle.grouped_matmul(bf16_np(hidden)[:x.shape[0]], down_values, sizes, factor=down_factor)
    assert np.all(out[x.shape[0]:] == 0)
    scale = np.abs(want).max()
    assert np.abs(out[:x.shape[0]] - want).max() <= 2 ** -5 * scale and np.abs(out - plain).max() <= 2 ** -5 * scale
    assert (out == plain).mean() > 0.9


@pytest.mark.parametrize("fp6", [False, True])
def test_the_expert_mlp_on_split_rows_as_one_call_is_its_three_launches(ops, fp6):
    """`dew_moe_swiglu_mlp_split`: the split of the rows, the gate/up launch and the down launch with their intermediates
    in one workspace, given the groups' offsets or their plain sizes: the bits of the three calls, rows past the groups
    zero, the scatter honoured."""
    sizes = [700, 0, 290, 5]
    depth, width, out_width = 512, 768, 256
    gate, x, offsets = grouped_case("mxfp4", len(sizes), depth, width, sizes, seed=31)
    up, _, _ = grouped_case("mxfp4", len(sizes), depth, width, sizes, seed=32)
    down, _, _ = grouped_case("mxfp4", len(sizes), width, out_width, sizes, seed=33)
    rng = np.random.default_rng(7)
    padded = x.shape[0] + 9
    gather = torch.from_numpy(np.concatenate([rng.integers(0, x.shape[0], size=x.shape[0]), np.zeros(9)]).astype(np.int32)).cuda()
    scatter = torch.from_numpy(rng.permutation(padded).astype(np.int32)).cuda()
    xd, od, sd = x.cuda(), torch.from_numpy(offsets).cuda(), torch.tensor(sizes, dtype=torch.int32).cuda()
    pg, pu, pd = (ops.prepare(bank.to("cuda")) for bank in (gate, up, down))
    pieces = ops.split_rows_fp6(xd) if fp6 else ops.split_rows(xd)
    hidden = ops.gateup_swiglu_split_out(*pieces, pg, pu, od, gather=gather, rows=padded, fp6=fp6)
    apart = ops.grouped_gemm_split_blocks(*hidden, pd, od, scatter=scatter, rows=padded)
    with_offsets = ops.swiglu_mlp_split(xd, pg, pu, pd, od, gather=gather, scatter=scatter, rows=padded, fp6=fp6)
    with_sizes = ops.swiglu_mlp_split(xd, pg, pu, pd, None, sizes=sd, gather=gather, scatter=scatter, rows=padded, fp6=fp6)
    assert with_offsets.shape == (padded, out_width)
    assert torch.equal(with_offsets, apart) and torch.equal(with_sizes, apart)
    assert not bool(apart[scatter[x.shape[0]:].long()].any())
    # no gather: the rows as they lie
    straight = ops.swiglu_mlp_split(xd, pg, pu, pd, od, fp6=fp6)
    assert torch.equal(straight, ops.grouped_gemm_split_blocks(*ops.gateup_swiglu_split_out(*pieces, pg, pu, od, fp6=fp6), pd, od))
    with pytest.raises(ops.KernelError, match="asked of x"):
        ops.swiglu_mlp_split(xd, pg, pu, pd, od, rows=padded)


@pytest.mark.parametrize("activation,limit", [("swiglu", 0.25), ("geglu", None), ("geglu", 0.5)])
def test_clamped_and_geglu_experts_stay_on_split_rows(ops, activation, limit):
    """`dew_moe_gated_mlp_split`: the clamp and the GeGLU gate in the split-row gate/up launch's epilogue, against the
    oracle's MLP with that gating and against the bf16-operand launches with the same epilogue (nearly all outputs
    identical: the gated rows are what the bf16 launch would write wherever two e4m3 terms hold them)."""
    sizes = [700, 0, 290, 5]
    depth, width, out_width = 512, 768, 256
    gate, x, offsets = grouped_case("mxfp4", len(sizes), depth, width, sizes, seed=41)
    up, _, _ = grouped_case("mxfp4", len(sizes), depth, width, sizes, seed=42)
    down, _, _ = grouped_case("mxfp4", len(sizes), width, out_width, sizes, seed=43)
    xd, od = x.cuda(), torch.from_numpy(offsets).cuda()
    pg, pu, pd = (ops.prepare(bank.to("cuda")) for bank in (gate, up, down))
    on_split = bf16_np(ops.swiglu_mlp_split(xd, pg, pu, pd, od, activation=activation, limit=limit))
    on_bf16 = bf16_np(ops.grouped_gemm(ops.gateup_swiglu(xd, pg, pu, od, activation=activation, limit=limit), pd, od))
    plain = bf16_np(ops.swiglu_mlp_split(xd, pg, pu, pd, od))
    (gv, gf), (uv, uf), (dv, df) = (dequantized(bank) for bank in (gate, up, down))
    rows = bf16_np(x)
    hidden = oracle.GATED_PRODUCTS[activation](oracle.grouped_matmul(rows, gv, sizes, factor=gf),
                                               oracle.grouped_matmul(rows, uv, sizes, factor=uf), dtype="bfloat16", limit=limit)
    want = oracle.grouped_matmul(hidden, dv, sizes, factor=df)
    scale = np.abs(want).max()
    assert np.abs(on_split - want).max() <= 2 ** -6 * scale and np.abs(on_split - on_bf16).max() <= 2 ** -6 * scale
    assert (on_split == on_bf16).mean() > 0.9 and (on_split == want).mean() > 0.9
    assert np.abs(plain - want).max() > 2 ** -4 * scale      # (the gating matters on these inputs)


def test_rows_that_are_not_finite_stay_their_own_on_split_rows_as_on_bf16_operands(ops):
    """A row holding an infinity, a NaN or a magnitude whose products overflow comes back NaN from the split-row MLP as
    from the bf16-operand launches; zero rows and rows far below the formats' range come back zero; the rows beside
    them are untouched."""
    rng = np.random.default_rng(0)
    experts, depth, width, out_width = 2, 256, 256, 256
    banks = [ops.prepare(quantize(torch.from_numpy((rng.standard_normal((experts, d, w)) * 0.05).astype(np.float32)), "mxfp4").to("cuda"))
             for d, w in ((depth, width), (depth, width), (width, out_width))]
    x = torch.from_numpy(rng.standard_normal((7, depth)).astype(np.float32)).to(torch.bfloat16)
    clean = x.clone()
    x[1, 5], x[2, 7], x[4, 9] = float("inf"), float("nan"), 3e38
    x[3, :], x[5, :] = 0, 1e-38
    offsets = torch.tensor([0, 3, 7], dtype=torch.int32).cuda()
    on_split = ops.swiglu_mlp_split(x.cuda(), *banks, offsets).float().cpu().numpy()
    on_bf16 = ops.grouped_gemm(ops.gateup_swiglu(x.cuda(), banks[0], banks[1], offsets), banks[2], offsets).float().cpu().numpy()
    untouched = ops.swiglu_mlp_split(clean.cuda(), *banks, offsets).float().cpu().numpy()
    for got in (on_split, on_bf16):
        assert np.isnan(got[[1, 2, 4]]).all() and not got[[3, 5]].any() and np.isfinite(got[[0, 6]]).all()
    assert np.array_equal(on_split[[0, 6]], untouched[[0, 6]])


@pytest.mark.parametrize("quant", ["fp8_block", "fp8_channel", "mxfp4", "nvfp4", "bf16"])
def test_a_layer_of_a_stacked_bank_is_read_where_it_lies(ops, quant):
    """`Layered(stack, layer)`: the grouped product of one layer's experts out of a bank stacking three layers', from
    the stack's own buffers, is the product of that layer's bank prepared alone, bit for bit."""
    from dew_amd import gemm, moe

    layers, experts, depth, width = 3, 4, 512, 256
    sizes = [70, 0, 33, 129]
    banks = [grouped_case(quant, experts, depth, width, sizes, seed=17 + layer) for layer in range(layers)]
    x, offsets = banks[0][1].cuda(), torch.from_numpy(banks[0][2]).cuda()
    first = banks[0][0]
    joined = {field.name: torch.cat([getattr(bank, field.name) for bank, _, _ in banks]) for field in dataclasses.fields(first)
              if torch.is_tensor(getattr(first, field.name)) and field.name != "form"}
    stacked = type(first)(**joined)
    stack = ops.prepare(stacked.to("cuda"))
    assert stack.shape == (layers * experts, depth, width)
    for layer in range(layers):
        alone = ops.grouped_gemm(x, ops.prepare(banks[layer][0].to("cuda")), offsets)
        assert torch.equal(ops.grouped_gemm(x, stack.layer(layer, layers), offsets), alone)
        through = gemm.gemm(x, moe.Layered(stack, layer, layers), gemm.GroupSizes(torch.tensor(sizes, dtype=torch.int32).cuda(), offsets))
        assert torch.equal(through, alone)
    with pytest.raises(Exception):
        stack.layer(3, layers)


def test_a_layer_of_a_stacked_mxfp8_bank_and_a_scaled_layer_are_read_where_they_lie(ops):
    """The two reads of a stack that move more than the codes: an MXFP8 bank's scale lines (one byte every 32 depths,
    half an NVFP4 bank's stride) and `layer(i).scaled(by)`, which owes layer i's own tensor scales, not the stack's
    first ones. Both against the layer's bank prepared alone, bit for bit."""
    from dew_amd import formats

    layers, experts, depth, width = 4, 3, 512, 256
    sizes = [70, 0, 129]
    rng = np.random.default_rng(23)
    offsets = torch.tensor(np.concatenate([[0], np.cumsum(sizes)]).astype(np.int32)).cuda()
    x = torch.from_numpy(rng.standard_normal((sum(sizes), depth)).astype(np.float32)).to(torch.bfloat16).cuda()
    spread = np.exp2(rng.integers(-4, 5, size=(layers * experts, depth // 32, width))).repeat(32, axis=1)
    weights = torch.from_numpy((rng.standard_normal((layers * experts, depth, width)) * 0.02 * spread).astype(np.float32))
    stack = ops.prepare(formats.MxFp8.quantized(weights).to("cuda"))
    codes, scales = ops.quantize_rows_mxfp8(x)
    for layer in range(layers):
        alone = ops.prepare(formats.MxFp8.quantized(weights[layer * experts:(layer + 1) * experts]).to("cuda"))
        want = ops.grouped_gemm_mxfp8_rows(codes, scales, alone, offsets)
        assert torch.equal(ops.grouped_gemm_mxfp8_rows(codes, scales, stack.layer(layer, layers), offsets), want), layer

    banks = [grouped_case("nvfp4", experts, depth, width, sizes, seed=50 + layer)[0] for layer in range(layers)]
    first = banks[0]
    joined = {field.name: torch.cat([getattr(bank, field.name) for bank in banks]) for field in dataclasses.fields(first)
              if torch.is_tensor(getattr(first, field.name)) and field.name != "form"}
    stack = ops.prepare(type(first)(**joined).to("cuda"))
    by = torch.tensor([0.375], device="cuda")
    for layer in range(layers):
        want = ops.grouped_gemm(x, ops.prepare(banks[layer].to("cuda")).scaled(by), offsets)
        assert torch.equal(ops.grouped_gemm(x, stack.layer(layer, layers).scaled(by), offsets), want), layer


@pytest.mark.parametrize("quant", ["fp8_block", "fp8_channel", "mxfp4", "nvfp4", "bf16"])
def test_last_tiles_of_at_most_64_rows_go_to_a_launch_of_their_own(ops, quant):
    """With 32 groups over 8 strips the 128-row tiles' launch leaves each group's last rows, where they are at most
    64, to a launch of 64-row tiles: every remainder from none to a full tile, both products and the paired one, are
    the single launch's bit for bit (a row's sum does not depend on the tile it sits in), and rows past the groups
    are zero."""
    remainders = [0, 1, 2, 31, 63, 64, 65, 100, 127, 128, 129, 192, 193, 255, 256, 257]
    sizes = [remainders[i % 16] + 128 * (i % 3) for i in range(32)]
    depth, width = 256, 1024
    bank, x, offsets = grouped_case(quant, len(sizes), depth, width, sizes, seed=41)
    up, _, _ = grouped_case(quant, len(sizes), depth, width, sizes, seed=42)
    rows = int(np.sum(sizes))
    rng = np.random.default_rng(5)
    padded = rows + 37
    gather = np.concatenate([rng.integers(0, rows, size=rows), np.zeros(37)]).astype(np.int32)
    scatter = rng.permutation(padded).astype(np.int32)
    xd, od = x.cuda(), torch.from_numpy(offsets).cuda()
    gd, sd = torch.from_numpy(gather).cuda(), torch.from_numpy(scatter).cuda()
    pb, pu = ops.prepare(bank.to("cuda")), ops.prepare(up.to("cuda"))
    shared = ops.grouped_gemm(xd, pb, od, gather=gd, scatter=sd, rows=padded)
    hidden = ops.gateup_swiglu(xd, pb, pu, od, gather=gd, rows=padded)
    with ops.tile_rows(128):
        single = ops.grouped_gemm(xd, pb, od, gather=gd, scatter=sd, rows=padded)
        single_hidden = ops.gateup_swiglu(xd, pb, pu, od, gather=gd, rows=padded)
    assert torch.equal(shared, single) and torch.equal(hidden, single_hidden)
    values, factor = dequantized(bank)
    want = oracle.grouped_matmul(bf16_np(x)[gather[:rows]], values, sizes, factor=factor)
    got = bf16_np(shared)
    assert np.all(got[scatter[rows:]] == 0)
    assert np.abs(got[scatter[:rows]] - want).max() <= 2 ** -7 * np.abs(want).max()


@pytest.mark.parametrize("quant", ["fp8_block", "mxfp4", "bf16"])
def test_group_sizes_in_place_of_their_prefix_give_the_same_products(ops, quant):
    """The reference's FFI operand is `group_sizes [E]` (kernels/cutlass/ffi.cu:185-198): handed in as they are, the
    launch forms the prefix in its tile search. Same bits as with the prefix, for both entry points, every tile
    height, ragged and empty groups, rows past the groups zero; more than 256 groups walk the search's second round."""
    from dew_amd import gemm

    for sizes, depth, width in (([130, 0, 1, 257, 64, 0, 127, 5], 256, 256), ([3] * 150 + [0] * 60 + [7] * 90, 256, 128)):
        bank, x, offsets = grouped_case(quant, len(sizes), depth, width, sizes, seed=len(sizes))
        up, _, _ = grouped_case(quant, len(sizes), depth, width, sizes, seed=len(sizes) + 1)
        rows = int(np.sum(sizes))
        padded = rows + 9
        gather = torch.from_numpy(np.concatenate([np.random.default_rng(1).integers(0, rows, size=rows), np.zeros(9)]).astype(np.int32)).cuda()
        scatter = torch.from_numpy(np.random.default_rng(2).permutation(padded).astype(np.int32)).cuda()
        xd, od, sd = x.cuda(), torch.from_numpy(offsets).cuda(), torch.tensor(sizes, dtype=torch.int32).cuda()
        pb, pu = ops.prepare(bank.to("cuda")), ops.prepare(up.to("cuda"))
        for tile in (0, 32, 64, 128):
            with ops.tile_rows(tile):
                want = ops.grouped_gemm(xd, pb, od, gather=gather, scatter=scatter, rows=padded)
                got = ops.grouped_gemm(xd, pb, None, sizes=sd, gather=gather, scatter=scatter, rows=padded)
                assert torch.equal(got, want), (quant, tile, len(sizes))
                want = ops.gateup_swiglu(xd, pb, pu, od, gather=gather, rows=padded)
                assert torch.equal(ops.gateup_swiglu(xd, pb, pu, None, sizes=sd, gather=gather, rows=padded), want)
        assert torch.equal(gemm.gemm(xd, pb, sd, gather=gather[:rows]), ops.grouped_gemm(xd, pb, od, gather=gather[:rows]))
        assert torch.equal(gemm.gemm(xd, pb, sd, paired=pu, epilogue="swiglu"), ops.gateup_swiglu(xd, pb, pu, od, rows=rows))



def test_the_clamped_swiglu_kernel_matches_the_oracle(ops):
    """`swiglu_clamped`: the gate from above and the up projection both ways, on every bf16 gate against a few ups, for
    a limit that is a bf16 (1.0) and one that is not (0.3, which enters as the bf16 nearest it)."""
    gate = oracle.bf16_from_bits(np.arange(65536, dtype=np.uint16))
    gate = gate[np.isfinite(gate)]
    gate = np.concatenate([gate, np.zeros(-gate.size % 8, np.float32)])
    up = np.resize(np.array([1.0, -0.75, 3.140625, 1e-3, 100.0, 2 ** -20, -7.0, 0.5], np.float32), gate.shape)
    for limit in (1.0, 0.3):
        rounded = float(torch.tensor(limit).to(torch.bfloat16))
        want = oracle.swiglu(gate, up, limit=rounded)
        got = bf16_np(ops.swiglu(torch.from_numpy(gate).to(torch.bfloat16).cuda(), torch.from_numpy(up).to(torch.bfloat16).cuda(), limit))
        mismatched = (got != want) & ~(np.isnan(got) & np.isnan(want))
        assert mismatched.mean() < 2e-3                    # the hardware exponential against the library's: a last bf16 bit, rarely
        assert np.abs(got - want)[mismatched].max(initial=0) <= 2 ** -7 * np.abs(want)[mismatched].max(initial=1)
        assert np.abs(got).max() <= rounded * 100.0 + 1.0  # |silu(min(g, limit)) * clip(u)| is bounded by limit * max|u|


@pytest.mark.parametrize("sequences,length,k,experts,factor", [(1, 64, 2, 8, 1.0), (3, 100, 4, 16, 0.5), (2, 700, 8, 64, 1.25),
                                                               (5, 33, 2, 4, 2.0), (1, 3000, 6, 512, 1.0), (4, 1, 2, 8, 1.0)])
def test_capacity_dropping_keeps_each_queues_first_places(ops, sequences, length, k, experts, factor):
    rng = np.random.default_rng(sequences * 7 + length)
    skew = rng.random(experts) ** 3
    indices = np.stack([np.stack([rng.choice(experts, size=k, replace=False, p=skew / skew.sum()) for _ in range(length)])
                        for _ in range(sequences)]).astype(np.int32)
    want, capacity = oracle.capacity_admitted(indices, experts, factor)
    got = ops.capacity_admitted(torch.from_numpy(indices).cuda(), experts, factor).cpu().numpy()
    assert np.array_equal(got, want)
    kept = got != experts
    assert kept.any() and (factor > 1.0 or length == 1 or (~kept).any())   # at factors up to 1 the skewed routing overflows some queue


def test_split_rows_with_an_fp6_second_term_hold_what_the_oracle_says(ops):
    """`split_rows_fp6`: the device's bytes decoded on the host are the oracle's values, bit for bit, on rows of many
    shapes (twenty-six binades in a row, a zero row, an outlier, a tiny row); an element within two binades of its
    32-deep block's largest (and within 2^-13 of its row's, where the e4m3 term keeps four bits) is held exactly, any
    other within 2^-10 of its block's largest."""
    rng = np.random.default_rng(17)
    rows, depth = 64, 512
    x = rng.standard_normal((rows, depth)).astype(np.float32)
    x[8:16] *= 10.0 ** rng.uniform(-4, 4, size=(8, depth)).astype(np.float32)
    x[16] = 0.0
    x[17, 5] = 3.0e4
    x[18] *= 1e-30
    x[19] = np.exp2(rng.integers(0, 3, size=depth)) * rng.choice([-1.0, 1.0], size=depth) * (1 + rng.integers(0, 128, size=depth) / 128)  # three binades
    xb = torch.from_numpy(x).to(torch.bfloat16)
    split, scale = ops.split_rows_fp6(xb.cuda())
    want_values, want_scale = oracle.split_rows_fp6(bf16_np(xb))
    got = oracle.split_rows_fp6_decoded(split.cpu().numpy(), scale.cpu().numpy())
    assert np.array_equal(scale.cpu().numpy(), want_scale) and np.array_equal(got, want_values)
    exact = bf16_np(xb)
    blocks = np.abs(exact).reshape(rows, depth // 32, 32)
    largest = blocks.max(axis=-1, keepdims=True)
    binade = np.where(largest > 0, np.exp2(np.floor(np.log2(np.maximum(largest, 1e-45)))), 0.0)
    row_largest = np.abs(exact).max(axis=1, keepdims=True)
    row_binade = np.where(row_largest > 0, np.exp2(np.floor(np.log2(np.maximum(row_largest, 1e-45)))), 0.0)
    # exact: within two binades of the block's largest, where the first term has its four bits (2^-13 of the row's binade)
    near = (blocks >= binade / 4).reshape(rows, depth) & (np.abs(exact) >= row_binade * 2.0 ** -13)
    assert near.mean() > 0.5 and np.array_equal(got[near], exact[near])
    # any element: within 2^-10 of its block's largest (or, in a block that lies below the e4m3 term's four bits, 2^-22 of the row's binade)
    bound = np.maximum(largest * 2.0 ** -10, (row_binade * 2.0 ** -22)[:, :, None])
    assert (np.abs(got - exact).reshape(rows, depth // 32, 32) <= bound).all()
    assert np.array_equal(got[19], exact[19])                                        # a row within three binades is held exactly


@pytest.mark.parametrize("depth", [256, 1280])
def test_the_gateup_launch_on_an_fp6_second_term_multiplies_the_values_the_rows_hold(ops, depth):
    """The FP6 second term changes the rows' values (to the oracle's `split_rows_fp6`), not the product's arithmetic:
    against the float64 sums of those values through the decoded banks the hidden rows agree as the two-e4m3 launch's
    do with the bf16 rows' (fp32 summation order apart), at both tile heights; and rows that the FP6 term holds
    exactly (three binades a row) give the two-e4m3 launch's hidden rows bit for bit."""
    sizes = [700, 0, 290, 5]
    width = 256
    gate, x, offsets = grouped_case("mxfp4", len(sizes), depth, width, sizes, seed=depth + 21)
    up, _, _ = grouped_case("mxfp4", len(sizes), depth, width, sizes, seed=depth + 22)
    (gate_values, gate_factor), (up_values, up_factor) = dequantized(gate), dequantized(up)
    rng = np.random.default_rng(depth)
    rows = x.shape[0]
    gather = rng.integers(0, rows, size=rows).astype(np.int32)
    od, gd = torch.from_numpy(offsets).cuda(), torch.from_numpy(gather).cuda()
    pg, pu = ops.prepare(gate.to("cuda")), ops.prepare(up.to("cuda"))

    def hidden_rows(split, scales):     # the split hidden rows rebuilt on the host
        pieces = split.cpu().numpy().reshape(rows, width // 64, 2, 2, 2, 16)
        terms = oracle._e4m3_table()[pieces].astype(np.float64)
        values = (terms[:, :, :, 0] + terms[:, :, :, 1] / 16).transpose(0, 1, 3, 2, 4).reshape(rows, width // 128, 128)
        s = np.ldexp(np.float64(1), scales.cpu().numpy()[:, :width // 128].astype(np.int64) - 127)[:, :, None]
        return (values * s).reshape(rows, width)

    held, _ = oracle.split_rows_fp6(bf16_np(x))
    bounds = np.concatenate([[0], np.cumsum(sizes)])
    want = np.zeros((rows, width))
    for e in range(len(sizes)):
        span = slice(bounds[e], bounds[e + 1])
        operand = held[gather[span]].astype(np.float64)
        g = oracle.bf16_round((operand @ gate_values[e].astype(np.float64) * (1.0 if gate_factor is None else gate_factor[e])).astype(np.float32))
        u = oracle.bf16_round((operand @ up_values[e].astype(np.float64) * (1.0 if up_factor is None else up_factor[e])).astype(np.float32))
        want[span] = oracle.swiglu(g, u)
    pieces = ops.split_rows_fp6(x.cuda())
    for tile in (0, 256):
        with ops.tile_rows(tile):
            got = hidden_rows(*ops.gateup_swiglu_split_out(*pieces, pg, pu, od, gather=gd, fp6=True))
        assert np.abs(got - want).max() <= 2 ** -6 * np.abs(want).max() and (got == want).mean() > 0.9, tile
    # against the bf16 rows' own products: the representation's price, far inside the layer's 2e-2
    exact = oracle.swiglu(oracle.grouped_matmul(bf16_np(x)[gather], gate_values, sizes, factor=gate_factor),
                          oracle.grouped_matmul(bf16_np(x)[gather], up_values, sizes, factor=up_factor))
    assert np.abs(got - exact).max() <= 1e-2 * np.abs(exact).max()
    # rows of three binades: nothing is lost, and the two launches agree bit for bit
    narrow = np.exp2(rng.integers(-1, 2, size=x.shape)) * rng.choice([-1.0, 1.0], size=x.shape) * (1 + rng.integers(0, 128, size=x.shape) / 128)
    xn = torch.from_numpy(narrow.astype(np.float32)).to(torch.bfloat16).cuda()
    six = ops.gateup_swiglu_split_out(*ops.split_rows_fp6(xn), pg, pu, od, gather=gd, fp6=True)
    eight = ops.gateup_swiglu_split_out(*ops.split_rows(xn), pg, pu, od, gather=gd)
    assert torch.equal(six[0], eight[0]) and torch.equal(six[1][:, :width // 128], eight[1][:, :width // 128])


def test_split_rows_as_two_e2m3_terms_hold_what_the_oracle_says(ops):
    """`split_rows_e2m3_pair`: the device's bytes decoded on the host are the oracle's values and scale bytes, bit for bit,
    on rows of many shapes; an element within two binades of its 32-deep block's largest magnitude is held exactly, any
    other within 2^-10 of that magnitude; blocks of three binades are held exactly."""
    rng = np.random.default_rng(18)
    rows, depth = 64, 512
    x = rng.standard_normal((rows, depth)).astype(np.float32)
    x[8:16] *= 10.0 ** rng.uniform(-4, 4, size=(8, depth)).astype(np.float32)
    x[16] = 0.0
    x[17, 5] = 3.0e4
    x[18] *= 1e-30
    x[19] = np.exp2(rng.integers(0, 3, size=depth)) * rng.choice([-1.0, 1.0], size=depth) * (1 + rng.integers(0, 128, size=depth) / 128)  # three binades
    x[20] *= 1e30
    xb = torch.from_numpy(x).to(torch.bfloat16)
    split, none = ops.split_rows_e2m3_pair(xb.cuda())
    assert none is None and split.shape == (rows, 2 * depth)
    want_values, want_scales = oracle.split_rows_e2m3_pair(bf16_np(xb))
    got, got_scales = oracle.split_rows_e2m3_pair_decoded(split.cpu().numpy())
    assert np.array_equal(got_scales, want_scales) and np.array_equal(got, want_values)
    exact = bf16_np(xb)
    blocks = np.abs(exact).reshape(rows, depth // 32, 32)
    largest = blocks.max(axis=-1, keepdims=True)
    binade = np.where(largest > 0, np.exp2(np.floor(np.log2(np.maximum(largest, 1e-45)))), 0.0)
    near = (blocks >= binade / 4).reshape(rows, depth)
    assert near.mean() > 0.5 and np.array_equal(got[near], exact[near])
    assert (np.abs(got - exact).reshape(rows, depth // 32, 32) <= largest * 2.0 ** -10).all()
    assert np.array_equal(got[19], exact[19]) and not got[16].any()
    assert ops.split_rows_as(xb.cuda(), "e2m3x2")[1] is None and torch.equal(ops.split_rows_as(xb.cuda(), "e2m3x2")[0], split)


@pytest.mark.parametrize("depth", [256, 1280])
def test_the_gateup_launch_on_two_e2m3_terms_multiplies_the_values_the_rows_hold(ops, depth):
    """Two FP6 terms change the rows' values (to the oracle's `split_rows_e2m3_pair`), not the product's arithmetic: against
    the float64 sums of those values through the decoded banks the hidden rows agree as the two-e4m3 launch's do with the
    bf16 rows', at both tile heights; and rows both forms hold exactly (three binades a row) give the two-e4m3 launch's
    hidden rows bit for bit."""
    sizes = [700, 0, 290, 5]
    width = 256
    gate, x, offsets = grouped_case("mxfp4", len(sizes), depth, width, sizes, seed=depth + 31)
    up, _, _ = grouped_case("mxfp4", len(sizes), depth, width, sizes, seed=depth + 32)
    (gate_values, gate_factor), (up_values, up_factor) = dequantized(gate), dequantized(up)
    rng = np.random.default_rng(depth + 1)
    rows = x.shape[0]
    gather = rng.integers(0, rows, size=rows).astype(np.int32)
    od, gd = torch.from_numpy(offsets).cuda(), torch.from_numpy(gather).cuda()
    pg, pu = ops.prepare(gate.to("cuda")), ops.prepare(up.to("cuda"))

    def hidden_rows(split, scales):     # the split hidden rows rebuilt on the host
        pieces = split.cpu().numpy().reshape(rows, width // 64, 2, 2, 2, 16)
        terms = oracle._e4m3_table()[pieces].astype(np.float64)
        values = (terms[:, :, :, 0] + terms[:, :, :, 1] / 16).transpose(0, 1, 3, 2, 4).reshape(rows, width // 128, 128)
        s = np.ldexp(np.float64(1), scales.cpu().numpy()[:, :width // 128].astype(np.int64) - 127)[:, :, None]
        return (values * s).reshape(rows, width)

    held, _ = oracle.split_rows_e2m3_pair(bf16_np(x))
    bounds = np.concatenate([[0], np.cumsum(sizes)])
    want = np.zeros((rows, width))
    for e in range(len(sizes)):
        span = slice(bounds[e], bounds[e + 1])
        operand = held[gather[span]].astype(np.float64)
        g = oracle.bf16_round((operand @ gate_values[e].astype(np.float64) * (1.0 if gate_factor is None else gate_factor[e])).astype(np.float32))
        u = oracle.bf16_round((operand @ up_values[e].astype(np.float64) * (1.0 if up_factor is None else up_factor[e])).astype(np.float32))
        want[span] = oracle.swiglu(g, u)
    pieces = ops.split_rows_e2m3_pair(x.cuda())
    for tile in (0, 256):
        with ops.tile_rows(tile):
            got = hidden_rows(*ops.gateup_swiglu_split_out(*pieces, pg, pu, od, gather=gd, terms="e2m3x2"))
        assert np.abs(got - want).max() <= 2 ** -6 * np.abs(want).max() and (got == want).mean() > 0.9, tile
    exact = oracle.swiglu(oracle.grouped_matmul(bf16_np(x)[gather], gate_values, sizes, factor=gate_factor),
                          oracle.grouped_matmul(bf16_np(x)[gather], up_values, sizes, factor=up_factor))
    assert np.abs(got - exact).max() <= 1e-2 * np.abs(exact).max()
    narrow = np.exp2(rng.integers(-1, 2, size=x.shape)) * rng.choice([-1.0, 1.0], size=x.shape) * (1 + rng.integers(0, 128, size=x.shape) / 128)
    xn = torch.from_numpy(narrow.astype(np.float32)).to(torch.bfloat16).cuda()
    six = ops.gateup_swiglu_split_out(*ops.split_rows_e2m3_pair(xn), pg, pu, od, gather=gd, terms="e2m3x2")
    eight = ops.gateup_swiglu_split_out(*ops.split_rows(xn), pg, pu, od, gather=gd)
    assert torch.equal(six[0], eight[0]) and torch.equal(six[1][:, :width // 128], eight[1][:, :width // 128])
    # the whole MLP as one call on the same rows' terms
    down, _, _ = grouped_case("mxfp4", len(sizes), width, 256, sizes, seed=depth + 33)
    pd = ops.prepare(down.to("cuda"))
    whole = ops.swiglu_mlp_split(x.cuda(), pg, pu, pd, od, gather=gd, terms="e2m3x2")
    apart = ops.grouped_gemm_split_blocks(*ops.gateup_swiglu_split_out(*pieces, pg, pu, od, gather=gd, terms="e2m3x2"), pd, od)
    assert torch.equal(whole, apart)

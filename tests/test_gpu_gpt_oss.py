"""GPT-OSS's experts on the HIP kernels against the oracle: the bias epilogue, the interleaved clamped gating,
and the whole layer (biased router, top-k of the logits, softmax of the chosen, experts, weighted sum)."""

import numpy as np
import pytest
import torch

from bench_aids.workloads import quantize
from oracle.banks import dequantized
from oracle import moe_oracle as oracle

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from dew_amd import ops
    ops.device_check()
    return ops


def bf16_np(tensor):
    return tensor.detach().float().cpu().numpy()


def bank_case(quant, experts, depth, width, sizes, seed, scale=0.02):
    rng = np.random.default_rng(seed)
    weight = torch.from_numpy((rng.standard_normal((experts, depth, width)) * scale).astype(np.float32))
    bank = quantize(weight, quant)
    x = torch.from_numpy(rng.standard_normal((int(np.sum(sizes)), depth)).astype(np.float32)).to(torch.bfloat16)
    bias = torch.from_numpy(rng.standard_normal((experts, width)).astype(np.float32))
    offsets = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int32)
    return bank, x, bias, offsets


SIZES = [("decode", [3, 0, 9, 1]), ("medium", [150, 70, 0, 1]), ("wide", [700, 4, 20, 300]), ("large", [900, 800])]


@pytest.mark.parametrize("quant", ["fp8_channel", "fp8_block", "mxfp4", "nvfp4"])
@pytest.mark.parametrize("label,sizes", SIZES, ids=[s[0] for s in SIZES])
def test_the_bias_meets_the_fp32_sums_before_their_one_rounding(ops, quant, label, sizes):
    bank, x, bias, offsets = bank_case(quant, len(sizes), 256, 512, sizes, seed=len(label) + len(quant))
    held = bias.to(torch.bfloat16).float()          # rounded to the compute dtype, held in fp32
    values, factor = dequantized(bank)
    want = oracle._biased_matmul(bf16_np(x), values, sizes, bias.numpy(), dtype="bfloat16", factor=factor)
    scatter = torch.from_numpy(np.random.default_rng(5).permutation(x.shape[0]).astype(np.int32))
    prepared = ops.prepare(bank.to("cuda"))
    got = ops.grouped_gemm(x.cuda(), prepared, torch.from_numpy(offsets).cuda(), bias=held.cuda(), scatter=scatter.cuda())
    # with `round_bias` the launch rounds the bias to the compute dtype as it reads it: the fp32 parameter itself gives the same bits
    assert torch.equal(got, ops.grouped_gemm(x.cuda(), prepared, torch.from_numpy(offsets).cuda(), bias=bias.cuda(), scatter=scatter.cuda(),
                                             round_bias=True))
    assert torch.equal(got, ops.grouped_gemm(x.cuda(), prepared, None, sizes=torch.tensor(sizes, dtype=torch.int32).cuda(), bias=bias.cuda(),
                                             scatter=scatter.cuda(), round_bias=True))
    got = bf16_np(got)[scatter.numpy()]
    assert np.abs(got - want).max() <= 2 ** -7 * np.abs(want).max()
    assert (got == want).mean() > 0.97
    # a product whose rounding comes before the bias would differ: the bias is of the outputs' size
    late = oracle.bf16_round(oracle.grouped_matmul(bf16_np(x), values, sizes, factor=factor) + held.numpy()[np.repeat(
        np.arange(len(sizes)), sizes)])
    assert (late != want).mean() > 0.01


@pytest.mark.parametrize("tile", [0, 64, 128])
@pytest.mark.parametrize("quant", ["fp8_channel", "fp8_block", "mxfp4", "nvfp4"])
@pytest.mark.parametrize("label,sizes", SIZES, ids=[s[0] for s in SIZES])
def test_interleaved_gate_up_with_the_clamped_gating(ops, quant, label, sizes, tile):
    # weights large enough that some sums pass the clamp at 7
    bank, x, bias, offsets = bank_case(quant, len(sizes), 256, 512, sizes, seed=3 * len(label) + len(quant), scale=0.2)
    held = bias.to(torch.bfloat16).float()
    values, factor = dequantized(bank)
    projected = oracle._biased_matmul(bf16_np(x), values, sizes, bias.numpy(), dtype="bfloat16", factor=factor)
    assert (projected > 7).mean() > 0.005 and (projected < -7).mean() > 0.005
    want = oracle.gpt_oss_gating(projected)
    rng = np.random.default_rng(9)
    gather = rng.integers(0, x.shape[0], size=x.shape[0]).astype(np.int32)
    want_gathered = oracle.gpt_oss_gating(oracle._biased_matmul(bf16_np(x)[gather], values, sizes, bias.numpy(), dtype="bfloat16",
                                                                factor=factor))
    prepared = ops.prepare(bank.to("cuda"))
    od = torch.from_numpy(offsets).cuda()
    with ops.tile_rows(tile):
        got = bf16_np(ops.gateup_interleaved(x.cuda(), prepared, od, bias=held.cuda(), limit=7.0))
        own = bf16_np(ops.grouped_gemm(x.cuda(), prepared, od, bias=held.cuda()))
    assert got.shape == (x.shape[0], 256)
    # the kernel's own projection is within one bf16 ulp of the oracle's; gate it with the oracle's arithmetic
    assert np.array_equal(got, oracle.gpt_oss_gating(own)) or (got == oracle.gpt_oss_gating(own)).mean() > 0.999
    scale = np.abs(want).max()
    assert np.abs(got - want).max() <= 2e-2 * scale
    assert (got == want).mean() > 0.9
    got_gathered = bf16_np(ops.gateup_interleaved(x.cuda(), prepared, od, bias=held.cuda(), gather=torch.from_numpy(gather).cuda()))
    assert np.abs(got_gathered - want_gathered).max() <= 2e-2 * scale and (got_gathered == want_gathered).mean() > 0.9


def test_unrouted_tail_rows_of_the_gated_product_are_zero(ops):
    bank, x, bias, offsets = bank_case("mxfp4", 2, 256, 256, [5, 6], seed=2)
    rows = 40
    xs = torch.cat([x, torch.ones((rows - x.shape[0], 256), dtype=torch.bfloat16)]).cuda()
    got = bf16_np(ops.gateup_interleaved(xs, ops.prepare(bank.to("cuda")), torch.from_numpy(offsets).cuda(),
                                         bias=bias.to(torch.bfloat16).float().cuda(), rows=rows))
    assert got.shape == (rows, 128) and np.all(got[11:] == 0) and np.any(got[:11] != 0)


@pytest.mark.parametrize("quant", ["mxfp4", "fp8_block"])
def test_gpt_oss_layer_matches_the_oracle(quant):
    from dew_amd import gpt_oss

    tokens, hidden, intermediate, experts, top_k = 96, 256, 256, 8, 4
    rng = np.random.default_rng(11)
    x = torch.from_numpy(rng.standard_normal((2, tokens // 2, hidden)).astype(np.float32)).to(torch.bfloat16)
    router_kernel = torch.from_numpy((rng.standard_normal((hidden, experts)) * hidden ** -0.5).astype(np.float32))
    router_bias = torch.from_numpy((rng.standard_normal(experts) * 0.1).astype(np.float32))
    gate_up = quantize(torch.from_numpy((rng.standard_normal((experts, hidden, 2 * intermediate)) * hidden ** -0.5).astype(np.float32)), quant)
    down = quantize(torch.from_numpy((rng.standard_normal((experts, intermediate, hidden)) * intermediate ** -0.5).astype(np.float32)), quant)
    gate_bias = torch.from_numpy(rng.standard_normal((experts, 2 * intermediate)).astype(np.float32))
    down_bias = torch.from_numpy(rng.standard_normal((experts, hidden)).astype(np.float32))
    gate_up_values, gate_up_factor = dequantized(gate_up)
    down_values, down_factor = dequantized(down)
    want, trace = oracle.gpt_oss_mlp(bf16_np(x), router_kernel.numpy(), router_bias.numpy(), gate_up_values, gate_bias.numpy(),
                                     down_values, down_bias.numpy(), top_k_count=top_k, factors=(gate_up_factor, down_factor))
    variables = {"params": {"router": {"kernel": router_kernel.cuda(), "bias": router_bias.cuda()},
                            "experts": {"gate_up_proj_bias": gate_bias.cuda(), "down_proj_bias": down_bias.cuda()}},
                 "quantization": {"experts": {"gate_up_proj": gate_up.to("cuda"), "down_proj": down.to("cuda")}}}
    layer = gpt_oss.GptOssMLP(hidden, intermediate, experts, top_k)
    got = layer.apply(variables, x.cuda())
    assert got.shape == x.shape and got.dtype == torch.bfloat16
    logits = bf16_np(layer._bound(variables, ()).logits(x.cuda())).reshape(-1, experts)
    assert np.abs(logits - trace["logits"]).max() <= 1e-5 * max(1.0, np.abs(trace["logits"]).max())
    peak_error, elementwise = oracle.relative_errors(bf16_np(got).reshape(want.shape), want)
    assert peak_error <= 2e-2 and elementwise <= 2e-2          # max|got - want| / max|want| and element-wise with an rms floor
    assert peak_error <= 8e-3
    # recorded into a HIP graph (its gate GEMM, biased router, sort, both biased launches, its own combine), the layer
    # replays to the eager bits on new tokens
    others = [torch.from_numpy(rng.standard_normal(x.shape).astype(np.float32)).to(torch.bfloat16).cuda() for _ in range(2)]
    eager = [layer.apply(variables, other).clone() for other in others]
    held = others[0].clone()
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        layer.apply(variables, held)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            recorded = layer.apply(variables, held)
    torch.cuda.synchronize()
    for turn in (1, 0, 1):
        held.copy_(others[turn])
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(recorded, eager[turn])
        layer.apply(variables, others[1 - turn])
        torch.cuda.synchronize()


def test_gpt_oss_requirements_are_refused_by_name(ops):
    from dew_amd import gemm, selection

    bank, x, bias, offsets = bank_case("mxfp4", 2, 256, 256, [5, 6], seed=2)
    sizes = gemm.GroupSizes.of(torch.tensor([5, 6], dtype=torch.int32, device="cuda"))
    with pytest.raises(selection.KernelRefused, match="epilogue"):
        gemm.gemm(x.cuda(), bank.to("cuda"), sizes, epilogue="plus_bias", epilogue_operands=(bias[:, :8].cuda(),),
                  implementation="hip")
    with pytest.raises(selection.KernelRefused, match="epilogue"):
        gemm.gemm(x.cuda(), bank.to("cuda"), sizes, epilogue="gpt_oss_gated", epilogue_operands=(None, -1.0), implementation="hip")
    out = gemm.gemm(x.cuda(), bank.to("cuda"), sizes, epilogue="gpt_oss_gated", epilogue_operands=(None, 7.0))
    assert out.shape == (11, 128)


@pytest.mark.parametrize("tile", [0, 32, 64, 128, 256])
@pytest.mark.parametrize("depth,width", [(192, 160), (320, 352), (2880, 2880)])
def test_unquantized_banks_take_depths_in_whole_steps_and_widths_in_whole_atoms(ops, depth, width, tile):
    """GPT-OSS's experts are 2880 wide (45 steps of 64 depths, 90 atoms of 32 columns, no whole 128s) and the reference keeps
    such banks unquantized (`packed_banks`, src/dew/interop/quantized_loads.py:130-131): the bf16 bank's launches take
    those extents as they are, the last strip's columns past the width neither stored nor biased from out of bounds."""
    sizes = [150, 0, 37, 70] if depth < 2000 else [40, 0, 9]
    bank, x, bias, offsets = bank_case("bf16", len(sizes), depth, width, sizes, seed=depth + width)
    rows = x.shape[0] + 5                                    # five sorted positions past the groups
    rng = np.random.default_rng(3)
    scatter = torch.from_numpy(rng.permutation(rows).astype(np.int32)).cuda()
    gather = torch.from_numpy(np.concatenate([np.arange(x.shape[0]), np.zeros(5)]).astype(np.int32)).cuda()
    values, _ = dequantized(bank)
    held = bias.to(torch.bfloat16).float()
    want = oracle._biased_matmul(bf16_np(x), values, sizes, bias.numpy(), dtype="bfloat16", factor=None)
    prepared = ops.prepare(bank.to("cuda"))
    with ops.tile_rows(tile):
        got = ops.grouped_gemm(x.cuda(), prepared, torch.from_numpy(offsets).cuda(), bias=held.cuda(), gather=gather, scatter=scatter, rows=rows)
    assert got.shape == (rows, width)
    got = bf16_np(got)
    order = scatter.cpu().numpy()
    assert not got[order[x.shape[0]:]].any()
    assert np.abs(got[order[:x.shape[0]]] - want).max() <= 2 ** -7 * np.abs(want).max()
    assert (got[order[:x.shape[0]]] == want).mean() > 0.97


@pytest.mark.parametrize("tile", [0, 64, 128])
def test_ragged_unquantized_banks_through_the_paired_and_the_interleaved_launches(ops, tile):
    sizes = [150, 0, 37, 70]
    depth, width = 320, 224
    gate, x, _, offsets = bank_case("bf16", len(sizes), depth, width, sizes, seed=5)
    up, _, _, _ = bank_case("bf16", len(sizes), depth, width, sizes, seed=6)
    xd, od = x.cuda(), torch.from_numpy(offsets).cuda()
    pg, pu = ops.prepare(gate.to("cuda")), ops.prepare(up.to("cuda"))
    with ops.tile_rows(tile):
        fused = ops.gateup_swiglu(xd, pg, pu, od)
        apart = ops.swiglu(ops.grouped_gemm(xd, pg, od), ops.grouped_gemm(xd, pu, od))
    assert fused.shape == (x.shape[0], width) and torch.equal(fused, apart)
    want = oracle.swiglu(oracle.grouped_matmul(bf16_np(x), dequantized(gate)[0], sizes), oracle.grouped_matmul(bf16_np(x), dequantized(up)[0], sizes))
    assert np.abs(bf16_np(fused) - want).max() <= 2 ** -6 * np.abs(want).max()
    # the interleaved bank: 2 x 224 columns, gate even and up odd, GPT-OSS's clamped gating, a bias on the sums
    both, x, bias, offsets = bank_case("bf16", len(sizes), depth, 2 * width, sizes, seed=7, scale=0.05)
    values, _ = dequantized(both)
    projected = oracle._biased_matmul(bf16_np(x), values, sizes, bias.numpy(), dtype="bfloat16", factor=None)
    want = oracle.gpt_oss_gating(projected, limit=7.0)
    with ops.tile_rows(tile):
        got = ops.gateup_interleaved(x.cuda(), ops.prepare(both.to("cuda")), torch.from_numpy(offsets).cuda(),
                                     bias=bias.to(torch.bfloat16).float().cuda(), limit=7.0)
    assert got.shape == (x.shape[0], width)
    got = bf16_np(got)
    assert np.abs(got - want).max() <= 2 ** -6 * np.abs(want).max() and (got == want).mean() > 0.9


@pytest.mark.parametrize("held", ["dense", "packed"])
def test_a_gpt_oss_layer_of_the_models_own_width(held):
    """hidden 2880, intermediate 2880 (gpt-oss-20b's config): the banks as the reference's load keeps them (dense bf16)
    and as the device re-layout keeps them (the checkpoint's MXFP4 blocks, still 4-bit): the layer through the
    selector, against the oracle."""
    from dew_amd import codecs, formats, gpt_oss

    tokens, hidden, intermediate, experts, top_k = 48, 2880, 2880, 4, 2
    rng = np.random.default_rng(13)
    x = torch.from_numpy(rng.standard_normal((tokens, hidden)).astype(np.float32)).to(torch.bfloat16)
    router_kernel = torch.from_numpy((rng.standard_normal((hidden, experts)) * hidden ** -0.5).astype(np.float32))
    router_bias = torch.from_numpy((rng.standard_normal(experts) * 0.1).astype(np.float32))
    gate_up = torch.from_numpy((rng.standard_normal((experts, hidden, 2 * intermediate)) * hidden ** -0.5).astype(np.float32))
    down = torch.from_numpy((rng.standard_normal((experts, intermediate, hidden)) * intermediate ** -0.5).astype(np.float32))
    if held == "packed":
        gate_up, down = (formats.Mxfp4Blocks(*codecs.quantize_mxfp4(weight)) for weight in (gate_up, down))
    else:
        gate_up, down = formats.Bf16(gate_up.to(torch.bfloat16)), formats.Bf16(down.to(torch.bfloat16))
    gate_bias = torch.from_numpy(rng.standard_normal((experts, 2 * intermediate)).astype(np.float32))
    down_bias = torch.from_numpy(rng.standard_normal((experts, hidden)).astype(np.float32))
    want, _ = oracle.gpt_oss_mlp(bf16_np(x), router_kernel.numpy(), router_bias.numpy(), dequantized(gate_up)[0], gate_bias.numpy(),
                                 dequantized(down)[0], down_bias.numpy(), top_k_count=top_k, factors=(None, None))
    variables = {"params": {"router": {"kernel": router_kernel.cuda(), "bias": router_bias.cuda()},
                            "experts": {"gate_up_proj_bias": gate_bias.cuda(), "down_proj_bias": down_bias.cuda()}},
                 "quantization": {"experts": {"gate_up_proj": gate_up.to("cuda"), "down_proj": down.to("cuda")}}}
    got = gpt_oss.GptOssMLP(hidden, intermediate, experts, top_k).apply(variables, x.cuda())
    assert got.shape == x.shape
    peak_error, elementwise = oracle.relative_errors(bf16_np(got).reshape(want.shape), want)
    assert peak_error <= 8e-3 and elementwise <= 2e-2


@pytest.mark.parametrize("tile", [0, 32, 128])
def test_an_mxfp4_checkpoint_bank_of_gpt_oss_extents_stays_packed_on_the_device(ops, tile):
    """The reference keeps a 2880-deep MXFP4 bank dense because its NvFp4 words are staged 256 deep
    (src/dew/interop/quantized_loads.py:130-131). The device re-layout takes the checkpoint's own blocks and scales in
    atoms 64 deep and 32 columns wide, so here such a bank stays 4-bit: its products are those of the dense bank the
    reference would hold (`dequantize_mxfp4`) in the plain and the gated launches, to the last bit in nearly every output."""
    from dew_amd import codecs, formats, gemm, loads

    rng = np.random.default_rng(19)
    experts, depth, width, sizes = 3, 320, 352, [150, 0, 41]
    weight = torch.from_numpy((rng.standard_normal((experts, depth, 2 * width)) * 0.05).astype(np.float32))
    blocks, scales = codecs.quantize_mxfp4(weight)
    tensors = {"mlp.experts.gate_up_proj_blocks": blocks.cuda(), "mlp.experts.gate_up_proj_scales": scales.cuda()}
    left, banks = loads.packed_banks(tensors, {"quantization_config": {"quant_method": "mxfp4"}})
    packed = banks["mlp.experts.gate_up_proj"]
    assert isinstance(packed, formats.Mxfp4Blocks) and packed.shape == (experts, depth, 2 * width)
    dense = loads.dense_bank(blocks.cuda(), scales.cuda())
    x = torch.from_numpy(rng.standard_normal((int(np.sum(sizes)), depth)).astype(np.float32)).to(torch.bfloat16).cuda()
    bias = torch.from_numpy(rng.standard_normal((experts, 2 * width)).astype(np.float32)).to(torch.bfloat16).float().cuda()
    group_sizes = torch.tensor(sizes, dtype=torch.int32).cuda()
    assert gemm.prepared(packed).descriptor.format == ops._lib.W_MXFP4
    def alike(mine, theirs):   # the same exact products, summed in fp32 in the two banks' own depth orders
        mine, theirs = bf16_np(mine), bf16_np(theirs)
        return mine.shape == theirs.shape and (mine == theirs).mean() > 0.99 and np.abs(mine - theirs).max() <= 2 ** -7 * np.abs(theirs).max()

    with ops.tile_rows(tile):
        assert alike(gemm.gemm(x, packed, group_sizes, epilogue="plus_bias", epilogue_operands=(bias,)),
                     gemm.gemm(x, dense, group_sizes, epilogue="plus_bias", epilogue_operands=(bias,)))
        gated = gemm.gemm(x, packed, group_sizes, epilogue="gpt_oss_gated", epilogue_operands=(bias, 7.0))
        assert gated.shape == (x.shape[0], width)
        assert alike(gated, gemm.gemm(x, dense, group_sizes, epilogue="gpt_oss_gated", epilogue_operands=(bias, 7.0)))
    values = oracle.decode_mxfp4(blocks.numpy(), scales.numpy())
    want = oracle.gpt_oss_gating(oracle._biased_matmul(bf16_np(x), values, sizes, bias.cpu().numpy(), dtype="bfloat16", factor=None), limit=7.0)
    got = bf16_np(gated)
    assert np.abs(got - want).max() <= 2 ** -6 * np.abs(want).max() and (got == want).mean() > 0.9


@pytest.mark.parametrize("quant", ["mxfp4", "nvfp4"])
def test_a_decode_step_on_many_fp4_experts_of_a_ragged_width(ops, quant):
    """Enough experts and columns that a decode step's one-bank launches take their 256-column blocks (experts x strips of
    256 >= 640) on a width that is no whole 256s (2688 = 10 strips and 128 columns): the plain product with its bias and
    GPT-OSS's gated one, a few rows an expert and several experts empty, against the oracle."""
    from dew_amd import codecs, formats, gemm
    from bench_aids.workloads import quantize
    from oracle.banks import dequantized

    rng = np.random.default_rng(23)
    experts, depth, width = 64, 256, 2688
    sizes = rng.integers(0, 9, size=experts)
    sizes[rng.integers(0, experts, size=6)] = 0
    weight = torch.from_numpy((rng.standard_normal((experts, depth, width)) * 0.05).astype(np.float32))
    bank = formats.Mxfp4Blocks(*codecs.quantize_mxfp4(weight)) if quant == "mxfp4" else quantize(weight, "nvfp4")
    values, factor = dequantized(bank)
    x = torch.from_numpy(rng.standard_normal((int(sizes.sum()) + 5, depth)).astype(np.float32)).to(torch.bfloat16)
    bias = torch.from_numpy(rng.standard_normal((experts, width)).astype(np.float32)).to(torch.bfloat16).float()
    group_sizes = torch.tensor(sizes, dtype=torch.int32).cuda()
    got = bf16_np(gemm.gemm(x.cuda(), bank.to("cuda"), group_sizes, epilogue="plus_bias", epilogue_operands=(bias.cuda(),)))
    want = oracle._biased_matmul(bf16_np(x), values, sizes.tolist(), bias.numpy(), dtype="bfloat16", factor=factor)
    assert got.shape == want.shape and not got[int(sizes.sum()):].any()
    assert np.abs(got - want).max() <= 2 ** -7 * np.abs(want).max() and (got == want).mean() > 0.97
    if quant == "nvfp4":      # (the interleaved gated launch is GPT-OSS's: MXFP4 and unquantized banks)
        return
    gated = bf16_np(gemm.gemm(x.cuda(), bank.to("cuda"), group_sizes, epilogue="gpt_oss_gated", epilogue_operands=(bias.cuda(), 7.0)))
    sums = oracle._biased_matmul(bf16_np(x), values, sizes.tolist(), bias.numpy(), dtype="bfloat16", factor=factor)
    want = oracle.gpt_oss_gating(sums, limit=7.0)
    assert gated.shape == (x.shape[0], width // 2)
    assert np.abs(gated - want).max() <= 2 ** -6 * np.abs(want).max() and (gated == want).mean() > 0.9

"""Benchmark of the quantized MoE expert path on one MI355X.

A step is one pass of the hot path over one batch of synthetic input already resident in HBM: route ->
sort by expert -> gate/up grouped GEMM with the SwiGLU epilogue -> down grouped GEMM scattered to slot
order -> weighted combine (+ shared expert where the config has one). Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c2] [--only] [--no-cpu-baseline]

The line's top level is the `--config` workload (default c2, the one the metric is quoted on). `value` is
algorithmic TFLOP/s of the whole step: 6 * R * D * F (+ 6 * T * D * F_shared), the reference's own convention of
three projections per dispatched row (src/dew/nn/moe.py:1275-1281), over the measured step time. `roofline` is
the dominant kernel alone (the paired gate/up launch: two thirds of the FLOPs), timed with HIP events recorded on
the launch stream around every one of its launches in the timed region. `cpu_baseline` is the CPU oracle on a
bounded sample of the same workload, on this box's host cores. `configs` holds the same measurement for each of
the five workloads c1 .. c5 (step time, the dominant kernel against its roofline, parity of a full-size sample
against the CPU oracle, and the least top-k margin of the routing); `--only` leaves it out.
"""

import argparse
import gc
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

PEAKS = {"bf16_mfma": 2500.0, "fp8_mfma": 5000.0, "fp4_mfma": 10100.0, "hbm_gbs": 8000.0}
"""MI355X published dense peaks, TFLOP/s and GB/s."""

ALL_CONFIGS = ("c1", "c2", "c3", "c4", "c5")
TERM_RATES = {"e4m3": ("e4m3", "e4m3"), "e2m3": ("e4m3", "e2m3"), "e2m3x2": ("e2m3", "e2m3")}
"""The two terms a split row is held as, by the library's setting (an e4m3 term's instruction runs at the fp8 rate, an
e2m3 term's at the fp6/fp4 rate)."""
GRAPHED = ("c1", "c3")
"""The launch-bound workloads: their step is replayed as one captured HIP graph."""
DECODE = ("c3",)
"""The workloads whose dominant kernel is bound by HBM bandwidth, not by the matrix cores."""


def build_workload(case, device, seed=0):
    """Synthetic tensors of `case` on the device: bf16 activations ~N(0,1), fp32 router logits ~N(0,1) (+ a
    per-expert bias), banks ~N(0,0.02) quantized on the device one expert matrix at a time."""
    import torch
    from bench_aids.workloads import quantize

    from dew_amd import formats, gemm

    generator = torch.Generator(device=device)
    generator.manual_seed(seed)
    x = torch.randn((case.tokens, case.d_model), generator=generator, device=device, dtype=torch.float32).to(torch.bfloat16)
    logits = torch.randn((case.tokens, case.experts), generator=generator, device=device, dtype=torch.float32)
    if case.logit_bias_std:
        logits = logits + case.logit_bias_std * torch.randn(case.experts, generator=generator, device=device)
    bias = None
    if case.router.get("score_function") == "sigmoid":
        bias = 0.05 * torch.randn(case.experts, generator=generator, device=device)

    def bank(depth, width, experts):
        parts = []
        for _ in range(experts):
            weight = 0.02 * torch.randn((1, depth, width), generator=generator, device=device, dtype=torch.float32)
            parts.append(quantize(weight, case.quant))
        first = parts[0]
        if isinstance(first, formats.NvFp4):
            held = formats.NvFp4(torch.cat([p.words for p in parts]), torch.cat([p.scales for p in parts]),
                                 torch.cat([p.scale for p in parts]))
        elif isinstance(first, formats.Fp8Blocks):
            held = formats.Fp8Blocks(torch.cat([p.codes for p in parts]), torch.cat([p.scale_inv for p in parts]))
        else:
            held = formats.Fp8Channels(torch.cat([p.codes for p in parts]), torch.cat([p.scales for p in parts]))
        gemm.prepared(held)      # the one-time re-layout, outside the timed region (done at load)
        return held

    banks = {"gate": bank(case.d_model, case.d_ff, case.experts), "up": bank(case.d_model, case.d_ff, case.experts),
             "down": bank(case.d_ff, case.d_model, case.experts)}
    shared = None
    if case.shared:
        shared = {"gate": bank(case.d_model, case.d_ff, 1), "up": bank(case.d_model, case.d_ff, 1),
                  "down": bank(case.d_ff, case.d_model, 1)}
    torch.cuda.synchronize()
    return dict(x=x, logits=logits.contiguous(), bias=bias, banks=banks, shared=shared)


class Stepper:
    """One step of the hot path, launch by launch, with optional HIP events around the gate/up launch."""

    def __init__(self, case, data, split=True, fuse_shared=True):
        import torch

        from dew_amd import gemm, moe, ops

        self.torch, self.ops, self.case, self.data = torch, ops, case, data
        names = ("gate", "up", "down")
        # a shared expert of the routed experts' shape and format rides the routed launches as their group #E (the layer's
        # own rule, moe.with_shared_expert); else it is a dense MLP of its own and the combine adds its output
        stack = None
        if data["shared"] is not None and fuse_shared:
            stack = moe.with_shared_expert(tuple(data["banks"][n] for n in names), tuple(data["shared"][n] for n in names))
        self.fused_shared = stack is not None
        if self.fused_shared:
            self.gate, self.up, self.down = (gemm.prepared(bank) for bank in stack)
            self.shared = None
        else:
            self.gate, self.up, self.down = (gemm.prepared(data["banks"][n]) for n in names)
            self.shared = None if data["shared"] is None else tuple(gemm.prepared(data["shared"][n]) for n in names)
        tokens = case.tokens
        self.dense_offsets = torch.tensor([0, tokens], dtype=torch.int32, device=data["x"].device)
        self.events = []
        self.split = split
        self.terms = gemm.SPLIT_SECOND_TERM           # the library's setting for how split rows are held ('e4m3': two e4m3 terms)

    def __call__(self, timed: bool = False):
        torch, ops, case, data = self.torch, self.ops, self.case, self.data
        weights, indices = ops.route(data["logits"], case.top_k, bias=data["bias"], **case.router)
        plan = ops.sort_by_expert(indices, case.experts, case.tokens if self.fused_shared else 0)
        if timed:
            start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
        slots = self.project(plan, (start, stop) if timed else None)
        routed = case.tokens * case.top_k
        addend = slots[routed:] if self.fused_shared else None
        if self.shared is not None:
            shared_hidden = ops.gateup_swiglu(data["x"], self.shared[0], self.shared[1], self.dense_offsets)
            addend = ops.grouped_gemm(shared_hidden, self.shared[2], self.dense_offsets)
        return ops.combine(slots[:routed].view(case.tokens, case.top_k, case.d_model), weights, addend), plan

    def on_split_rows(self):
        """Whether the routed experts run on split rows and the scaled matrix instruction (the library's rule)."""
        return self.split and self.ops.prefers_split_pair(self.gate, self.up, self.down, self.case.tokens * self.case.top_k)

    def project(self, plan, events=None):
        """The routed experts' two launches: [T * k, D] rows at their slots. `events` bracket the gate/up launch."""
        ops, data = self.ops, self.data
        if self.on_split_rows():
            # MXFP4 banks and groups of hundreds of rows: the rows as two e4m3 terms and the scaled matrix instruction;
            # the gate/up launch writes its hidden rows already split, so the only extra pass is the split of x
            pieces = ops.split_rows_as(data["x"], self.terms)
            if events:
                events[0].record()
            hidden = ops.gateup_swiglu_split_out(*pieces, self.gate, self.up, plan.offsets, gather=plan.rows, terms=self.terms)
            if events:
                events[1].record()
                self.events.append(events)
            return ops.grouped_gemm_split_blocks(*hidden, self.down, plan.offsets, scatter=plan.order)
        hidden = ops.gateup_swiglu(data["x"], self.gate, self.up, plan.offsets, gather=plan.rows)
        if events:
            events[1].record()
            self.events.append(events)
        return ops.grouped_gemm(hidden, self.down, plan.offsets, scatter=plan.order)

    def gateup_ms(self):
        return sum(start.elapsed_time(stop) for start, stop in self.events) / max(1, len(self.events))


def sampled_groups(sizes, budget_rows, first_budget=None):
    """Which sorted rows the CPU oracle follows: of the busiest expert, the one of median size and the least non-empty one
    (as many of them as differ), each group's first and last rows, `budget_rows` a group in all (`first_budget` for the
    busiest: the timed baseline's larger sample). A group's last rows are the ones a launch's partial last tile, or a
    second launch of shorter tiles, multiplies. Returns [(expert, positions within the group)]."""
    import numpy as np

    filled = np.flatnonzero(sizes > 0)
    by_size = filled[np.argsort(sizes[filled], kind="stable")]
    chosen = []
    for expert in (int(by_size[-1]), int(by_size[len(by_size) // 2]), int(by_size[0])):
        if expert not in chosen:
            chosen.append(expert)
    groups = []
    for place, expert in enumerate(chosen):
        size, budget = int(sizes[expert]), int(first_budget if place == 0 and first_budget else budget_rows)
        if size <= budget:
            positions = np.arange(size)
        else:
            positions = np.concatenate([np.arange(budget - budget // 2), np.arange(size - budget // 2, size)])
        groups.append((expert, positions))
    return groups


def oracle_sample(case, data, plan, budget_rows=64, first_budget=None):
    """The CPU oracle (dequantize -> bf16-exact fp32 GEMMs -> SwiGLU -> down) on a bounded sample of the workload: first
    and last sorted rows of up to three experts (`sampled_groups`), all three projections at full width. Returns the
    timing as the `cpu_baseline` object and (the slots of those rows, the oracle's down-projection rows for them, the
    experts sampled)."""
    import numpy as np
    import torch

    from dew_amd import formats
    from oracle import moe_oracle as oracle
    from oracle.banks import dequantized

    sizes = plan.sizes.cpu().numpy()[:case.experts]      # (a fused shared expert is group #E of the plan: not sampled here)
    offsets = plan.offsets.cpu().numpy()
    sorted_rows_all, order_all = plan.rows.cpu().numpy(), plan.order.cpu().numpy()

    def one(bank, expert):
        if isinstance(bank, formats.NvFp4):
            return formats.NvFp4(bank.words[expert:expert + 1].cpu(), bank.scales[expert:expert + 1].cpu(), bank.scale[expert:expert + 1].cpu())
        if isinstance(bank, formats.Fp8Blocks):
            return formats.Fp8Blocks(bank.codes[expert:expert + 1].cpu(), bank.scale_inv[expert:expert + 1].cpu())
        return formats.Fp8Channels(bank.codes[expert:expert + 1].cpu(), bank.scales[expert:expert + 1].cpu())

    threads = os.cpu_count() or 1
    dequant_s = gemm_s = 0.0
    all_slots, all_down, described, total_rows = [], [], [], 0
    for expert, positions in sampled_groups(sizes, budget_rows, first_budget):
        at = offsets[expert] + positions
        x = data["x"][torch.from_numpy(sorted_rows_all[at]).to(data["x"].device).long()].float().cpu().numpy()
        held = [one(data["banks"][n], expert) for n in ("gate", "up", "down")]
        began = time.perf_counter()
        mats, factors = zip(*(dequantized(bank) for bank in held), strict=True)
        dequant_s += time.perf_counter() - began
        began = time.perf_counter()
        rows = len(positions)
        gate = oracle.grouped_matmul(x, mats[0], [rows], factor=factors[0])
        up = oracle.grouped_matmul(x, mats[1], [rows], factor=factors[1])
        hidden = oracle.swiglu(gate, up)
        all_down.append(oracle.grouped_matmul(hidden, mats[2], [rows], factor=factors[2]))
        gemm_s += time.perf_counter() - began
        all_slots.append(order_all[at])
        described.append(f"{rows} of expert {expert}'s {int(sizes[expert])}")
        total_rows += rows
        del mats
    flops = 6.0 * total_rows * case.d_model * case.d_ff
    baseline = {"value": round(flops / (dequant_s + gemm_s) / 1e12, 5), "unit": "TFLOP/s", "cores": threads, "kind": "port",
                "sample": f"first and last sorted rows of the busiest, the median and the least non-empty expert ({', '.join(described)}), "
                          f"3 projections at full width: dequantize {dequant_s:.2f} s + fp32 GEMMs/SwiGLU {gemm_s:.2f} s "
                          "(NumPy/OpenBLAS on bf16-exact fp32 operands)",
                "gemm_only_tflops": round(flops / gemm_s / 1e12, 5)}
    return baseline, (np.concatenate(all_slots), np.concatenate(all_down), [expert for expert, _ in sampled_groups(sizes, budget_rows, first_budget)])


WHOLE_ON_CPU = ("c1", "c3")
"""The workloads small enough for the CPU oracle to run whole (seconds): their baseline is no sample and no extrapolation,
and their parity is every element of the layer's output."""


def oracle_whole(case, data):
    """The CPU oracle on the whole workload (router, sort, three projections of every expert, combine), timed; returns the
    `cpu_baseline` object and (the oracle's layer output, its routing trace)."""
    from oracle import moe_oracle as oracle
    from oracle.banks import dequantized

    threads = os.cpu_count() or 1
    x, logits = data["x"].float().cpu().numpy(), data["logits"].cpu().numpy()
    began = time.perf_counter()
    mats, factors = zip(*(dequantized(data["banks"][n].to("cpu")) for n in ("gate", "up", "down")), strict=True)
    dequant_s = time.perf_counter() - began
    began = time.perf_counter()
    want, trace = oracle.sparse_mlp(x, logits, *mats, top_k_count=case.top_k, factors=factors,
                                    bias=None if data["bias"] is None else data["bias"].cpu().numpy(), **case.router)
    layer_s = time.perf_counter() - began
    flops = 6.0 * case.tokens * case.top_k * case.d_model * case.d_ff
    return {"value": round(flops / (dequant_s + layer_s) / 1e12, 5), "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "sample": f"the whole workload, no extrapolation: dequantize every expert {dequant_s:.2f} s + route, sort, 3 grouped "
                      f"projections, SwiGLU, combine {layer_s:.2f} s (NumPy/OpenBLAS on bf16-exact fp32 operands)"}, (want, trace)


# HBM bytes one launch of the dominant (gate/up) kernel moved, from rocprofv3 --pmc FETCH_SIZE and --pmc WRITE_SIZE (KiB per
# dispatch, two runs of `bench.py --config cN --only` per workload), each scaled by what the same counter reads for the plain
# copy probe of known size (--calibrate-copy). The counters cannot be read from inside this process: the figures are parsed,
# at every run, from the rocprofv3 summaries committed under profiles/ (the files named here), so the line cannot drift from
# them; `roofline.traffic_source` names the file. A workload whose summary is missing or has no such row reports null.
COUNTED_FROM = {"c1": "profiles/grouped_gemm_c1_small_fp8_channel.txt", "c2": "profiles/grouped_gemm_c2_prefill_mxfp4.txt",
                "c3": "profiles/grouped_gemm_c3_decode_fp8.txt", "c4": "profiles/grouped_gemm_c4_prefill_fp8_blocks.txt",
                "c5": "profiles/grouped_gemm_c5_prefill_nvfp4.txt"}
CALIBRATION = "profiles/probe_copy_counter_calibration.txt"
PAIRED_MODES = (1, 3)
"""Second template argument of grouped_gemm_kernel<FORMAT, MODE, ...> for the paired gate/up launches: SwiGLU of two banks,
and the same leaving its rows split."""


def counter_scales():
    """{counter: factor} of the copy calibration: known bytes over what the counter read."""
    import re

    text = (ROOT / CALIBRATION).read_text()
    return {name: float(factor) for name, factor in re.findall(r"^\s*(FETCH_SIZE|WRITE_SIZE)\s.*scale factor ([0-9.]+)\s*$", text, re.M)}


def counted_kib(config):
    """{counter: KiB per step} summed over the paired gate/up launches of a step (a workload whose groups' last rows go to a
    second launch of shorter tiles has two), read from section 2 of the workload's committed summary; None without one."""
    import re

    path = ROOT / COUNTED_FROM.get(config, "")
    if not path.is_file():
        return None
    section = path.read_text().split("2. HBM traffic", 1)
    if len(section) < 2:
        return None
    totals = {"FETCH_SIZE": 0.0, "WRITE_SIZE": 0.0}
    found = False
    for line in section[1].splitlines():
        row = re.match(r"^dew::grouped_gemm_kernel<\d+, (\d+), [^>]*>(?: grid \d+)?\s+\d+\s+([0-9.]+)\s+([0-9.]+)\s", line)
        if row and int(row.group(1)) in PAIRED_MODES:
            totals["FETCH_SIZE"] += float(row.group(2))
            totals["WRITE_SIZE"] += float(row.group(3))
            found = True
    return totals if found else None


def measured_traffic(config):
    counted = counted_kib(config)
    if counted is None:
        return None
    scales = counter_scales()
    return round(sum(counted[name] * scales[name] for name in counted) * 1024.0)


def sustained_rates(device):
    """What the chip sustains in this run: bf16 MFMA on random operands (TFLOP/s), a plain copy (GB/s of bytes read
    plus bytes written) and a read-only stream issued as the decode tiles issue their weight loads (GB/s), each timed
    with HIP events over several launches after a warm-up."""
    import torch

    from bench_aids import probes

    operands = torch.randn(16384, device=device).to(torch.bfloat16)
    probes.probe_mfma(operands, 2000)
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    flops = sum(probes.probe_mfma(operands, 20000) for _ in range(3))
    stop.record()
    torch.cuda.synchronize()
    mfma = flops / (start.elapsed_time(stop) * 1e-3) / 1e12
    src = torch.empty(1 << 30, dtype=torch.uint8, device=device).random_()
    dst = torch.empty_like(src)
    probes.probe_copy(src, dst)
    start.record()
    moved = sum(2 * probes.probe_copy(src, dst) for _ in range(5))
    stop.record()
    torch.cuda.synchronize()
    copied = moved / (start.elapsed_time(stop) * 1e-3) / 1e9
    probes.probe_read(src)
    start.record()
    fetched = sum(probes.probe_read(src) for _ in range(5))
    stop.record()
    torch.cuda.synchronize()
    return round(mfma, 1), round(copied, 1), round(fetched / (start.elapsed_time(stop) * 1e-3) / 1e9, 1)


def measure(config, args, device, sustained, with_cpu_baseline):
    """One workload, measured: its part of the line (ms_per_step, value, config, roofline, sample_parity,
    min_topk_margin and, where asked, cpu_baseline)."""
    import torch
    from bench_aids.workloads import CONFIGS

    from bench_aids import probes
    from oracle import moe_oracle as oracle

    case = CONFIGS[config]
    data = build_workload(case, device)
    stepper = Stepper(case, data, split=not args.bf16_operands, fuse_shared=not args.separate_shared)
    graphed = args.graph == "on" or (args.graph == "auto" and config in GRAPHED)
    for _ in range(args.warmup):
        stepper()
    torch.cuda.synchronize()
    if graphed:
        # A step is a handful of short launches. The timed steps are captured back to back as one graph, the way a
        # model's decode graph holds one such step for every MoE layer, and replayed once: no host work between
        # kernels, and the replay's own start-up (about 17 us a replay on this stack, whatever the graph holds) is paid
        # once, not once a step. The launches themselves are the same C-ABI calls on the capture stream.
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for _ in range(args.steps):
                out, plan = stepper()
        graph.replay()
        torch.cuda.synchronize()
        began = time.perf_counter()
        graph.replay()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - began
        # The dominant kernel's duration: HIP events around its launch inside eager steps on the same inputs. A
        # millisecond of queued work ahead of each step lets the host run ahead, so the step's launches follow each
        # other on the device as they do in the graph and the events bracket the kernel, not the host's launch path.
        operands = torch.randn(16384, device=device).to(torch.bfloat16)
        for _ in range(args.steps):
            probes.probe_mfma(operands, 1200)
            stepper(timed=True)
        torch.cuda.synchronize()
    else:
        began = time.perf_counter()
        for _ in range(args.steps):
            out, plan = stepper(timed=True)
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - began
    ms_per_step = 1e3 * elapsed / args.steps

    routed_rows = case.tokens * case.top_k
    flops = 6.0 * routed_rows * case.d_model * case.d_ff + (6.0 * case.tokens * case.d_model * case.d_ff if case.shared else 0.0)
    gateup_rows = routed_rows + (case.tokens if stepper.fused_shared else 0)   # the launch multiplies a fused shared expert's rows too
    gateup_flops = 4.0 * gateup_rows * case.d_model * case.d_ff
    gateup_ms = stepper.gateup_ms()
    achieved = gateup_flops / (gateup_ms * 1e-3) / 1e12
    decode = config in DECODE
    bytes_per_weight = 0.5 if case.quant in ("mxfp4", "nvfp4") else 1.0
    touched = int((plan.sizes[:case.experts] > 0).sum().item())
    # bandwidth view: the touched experts' gate and up codes read once + activations in, hidden out
    gateup_bytes = (touched + (1 if stepper.fused_shared else 0)) * 2 * case.d_model * case.d_ff * bytes_per_weight + case.tokens * case.d_model * 2 + gateup_rows * case.d_ff * 2
    gateup_gbs = gateup_bytes / (gateup_ms * 1e-3) / 1e9
    sustained_mfma, sustained_copy, sustained_read = sustained
    if decode:
        roofline = {"bound": "hbm", "achieved": round(gateup_gbs, 1), "peak": PEAKS["hbm_gbs"], "unit": "GB/s"}
    else:
        roofline = {"bound": "mfma", "achieved": round(achieved, 1), "peak": PEAKS["bf16_mfma"], "unit": "TFLOP/s",
                    "peak_note": ("the kernel multiplies each bf16 activation as two terms by the stored FP4 codes "
                                  "(v_mfma_scale_f32_32x32x64_f8f6f4: the e4m3 term at the dense fp8 rate, 5.0 PFLOP/s published, the "
                                  "second term at that rate (e4m3) or at the fp6/fp4 rate, 10.1 (e2m3)): two instructions per "
                                  "algorithmic product; priced against the dense bf16 peak, 2.5 PFLOP/s, the ceiling of two fp8-rate "
                                  "instructions; achieved counts algorithmic flops only") if stepper.on_split_rows() else
                                 ("dense bf16 MFMA: the kernel multiplies bf16 activations by weights dequantized exactly to "
                                  "bf16 (v_mfma_f32_32x32x16_bf16)"),
                    "frac_of_fp8_peak": round(achieved / PEAKS["fp8_mfma"], 4), "frac_of_fp4_peak": round(achieved / PEAKS["fp4_mfma"], 4),
                    "hbm_view": {"algorithmic_bytes": gateup_bytes, "gbs": round(gateup_gbs, 1),
                                 "frac_of_hbm_peak": round(gateup_gbs / PEAKS["hbm_gbs"], 4)}}
    roofline["frac"] = round(roofline["achieved"] / roofline["peak"], 4)
    if not decode:   # the fractions of the narrower formats' published peaks right beside it
        roofline["frac_of_fp8_peak"], roofline["frac_of_fp4_peak"] = roofline.pop("frac_of_fp8_peak"), roofline.pop("frac_of_fp4_peak")
    if not decode and stepper.on_split_rows():
        roofline["executed"] = {"tflops": round(2 * achieved, 1), "frac_of_fp8_peak": round(2 * achieved / PEAKS["fp8_mfma"], 4),
                                "note": "instruction flops: both terms' products",
                                "issue_time_frac": round(achieved / (1.0 / sum(1.0 / PEAKS["fp8_mfma" if term == "e4m3" else "fp4_mfma"]
                                                                               for term in TERM_RATES[stepper.terms])), 4),
                                "issue_time_note": "achieved over the rate at which the two instructions of a product issue back to back at "
                                                   "their published peaks (fp8 + fp8: 2.5 PFLOP/s; fp8 + fp6: 3.34; fp6 + fp6: 5.05)"}
    roofline["traffic"] = measured_traffic(config)
    roofline["traffic_source"] = (f"parsed from {COUNTED_FROM[config]}: rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE of this command's "
                                  f"gate/up launch(es), scaled by {CALIBRATION}; counters of an earlier run of the same command, "
                                  "not of this one") if roofline["traffic"] is not None else None
    roofline["algorithmic"] = {"per_launch": gateup_bytes if decode else gateup_flops, "unit": "bytes" if decode else "flop"}
    roofline["sustained"] = {"bf16_mfma_random_operands_tflops": sustained_mfma, "plain_copy_gbs": sustained_copy,
                             "read_stream_gbs": sustained_read,
                             "frac_of_sustained": round(roofline["achieved"] / (sustained_read if decode else sustained_mfma), 4),
                             "note": "measured in this run by bench_aids' probes: the MFMA rate the chip holds on random data at "
                                     "its power limit, a plain copy, and a read-only stream of non-temporal loads issued as the "
                                     "decode tiles issue theirs (the reference for an HBM-bound launch)"}
    roofline["kernel"] = "grouped_gemm_kernel<paired gate/up + SwiGLU>" + (
        f" on split rows (v_mfma_scale_f32_32x32x64_f8f6f4, {' + '.join(TERM_RATES[stepper.terms])} terms x FP4)" if stepper.on_split_rows() else "")
    roofline["kernel_ms"] = round(gateup_ms, 4)

    result = {
        "value": round(flops / (ms_per_step * 1e-3) / 1e12, 2), "unit": "TFLOP/s", "ms_per_step": round(ms_per_step, 4),
        "config": {"workload": f"{config}: T={case.tokens} D={case.d_model} F={case.d_ff} E={case.experts} k={case.top_k} "
                               f"{case.quant} weights, {case.router['score_function']} router"
                               + (" + shared expert" if case.shared else ""),
                   "routed_rows": routed_rows, "experts_touched": touched,
                   **({"shared_expert": "group #E of the routed launches" if stepper.fused_shared else "two launches of its own"} if case.shared else {}), "launch": "hip graph replay (the timed steps captured back to back as one graph)" if graphed else "eager",
                   "algorithmic_flops": flops},
        "roofline": roofline,
    }
    # The router's own GEMM (x @ gate kernel in fp32): outside the step, whose logits are synthetic as the benchmark defines
    # them; what a layer that multiplies its own gate kernel adds to the step.
    gate_kernel = torch.randn((case.d_model, case.experts), device=device, dtype=torch.float32) * case.d_model ** -0.5
    stepper.ops.router_logits(data["x"], gate_kernel)
    first, last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    first.record()
    for _ in range(5):
        stepper.ops.router_logits(data["x"], gate_kernel)
    last.record()
    torch.cuda.synchronize()
    gate_us = first.elapsed_time(last) / 5 * 1e3
    result["router_logits"] = {"us": round(gate_us, 1), "tflops_fp32": round(2.0 * case.tokens * case.d_model * case.experts / gate_us / 1e6, 2),
                               "note": "x @ gate kernel [D, E] in fp32 (dew_moe_router_logits), launched eagerly; not part of ms_per_step"}
    del gate_kernel
    # the routing's least top-k margin: how close the last chosen selection comes to the best one left out
    router = {k: v for k, v in case.router.items() if k in ("score_function", "expert_groups", "groups_per_token")}
    _, selection = oracle.selection_scores(data["logits"].cpu().numpy(), bias=None if data["bias"] is None else data["bias"].cpu().numpy(),
                                           **router)
    gap, spacings, token = oracle.top_k_margin(selection, case.top_k)
    finite = gap != float("inf")
    result["min_topk_margin"] = {"value": gap if finite else None, "fp32_spacings": round(spacings, 1) if finite else None, "token": token,
                                 "note": "least gap over the tokens between the k-th selection and the best one left out; 0 is an "
                                         "exact tie (the lower index wins everywhere)"}
    if config in WHOLE_ON_CPU and not args.no_parity:
        # small enough for the CPU oracle to follow whole: the baseline is the whole workload, and parity is every routed
        # row's down projection, the routing itself and the layer's output
        import numpy as np

        baseline, (want, trace) = oracle_whole(case, data)
        result["cpu_baseline"] = baseline
        weights, indices = stepper.ops.route(data["logits"], case.top_k, bias=data["bias"], **case.router)
        routing_identical = bool(np.array_equal(indices.cpu().numpy(), trace["indices"]) and np.array_equal(weights.cpu().numpy(), trace["weights"]))
        got = stepper.project(plan).float().cpu().numpy()[:routed_rows]
        want_slots = trace["slots"].reshape(routed_rows, case.d_model)
        by_max, by_element = oracle.relative_errors(got, want_slots)
        out_max, out_element = oracle.relative_errors(out.float().cpu().numpy(), want)
        result["sample_parity"] = {"max_abs_over_max_ref": round(float(by_max), 6), "elementwise": round(float(by_element), 6),
                                   "identical_frac": round(float((got == want_slots).mean()), 5), "rows": int(routed_rows),
                                   "experts": f"all {touched} touched experts, every routed row", "routing_identical": routing_identical,
                                   "layer_output": {"max_abs_over_max_ref": round(float(out_max), 6), "elementwise": round(float(out_element), 6),
                                                    "identical_frac": round(float((out.float().cpu().numpy() == want).mean()), 5)},
                                   "bar": 2e-2}
    elif with_cpu_baseline or not args.no_parity:
        # the timed CPU baseline takes a larger sample of the busiest expert (about ten seconds of host work, most of it the
        # GEMMs, not the dequantization); the other configs' parity samples stay small so that the default run takes minutes
        baseline, (slots, want, experts) = oracle_sample(case, data, plan, budget_rows=64, first_budget=4096 if with_cpu_baseline else None)
        if with_cpu_baseline:
            result["cpu_baseline"] = baseline
        # parity on the sample at full size: the device's down-projection rows for those slots
        got = stepper.project(plan).float().cpu().numpy()[slots]
        by_max, by_element = oracle.relative_errors(got, want)
        result["sample_parity"] = {"max_abs_over_max_ref": round(float(by_max), 6), "elementwise": round(float(by_element), 6),
                                   "identical_frac": round(float((got == want).mean()), 5), "rows": int(len(slots)),
                                   "experts": [int(e) for e in experts],
                                   "rows_note": "first and last sorted rows of the busiest, the median and the least non-empty expert",
                                   "bar": 2e-2}
    del stepper, data, out, plan
    gc.collect()
    torch.cuda.empty_cache()
    return result


def main():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=20)
    parser.add_argument("--warmup", type=int, default=3)
    parser.add_argument("--config", default="c2", choices=list(ALL_CONFIGS), help="the workload of the line's top level")
    parser.add_argument("--only", action="store_true", help="measure the --config workload alone (no `configs` object)")
    parser.add_argument("--no-cpu-baseline", action="store_true")
    parser.add_argument("--no-parity", action="store_true", help="skip the CPU oracle's sample (profiling runs)")
    parser.add_argument("--calibrate-copy", action="store_true",
                        help="only run the plain copy probe (1 GiB read + 1 GiB written, 5 launches): the known traffic "
                             "that rocprofv3's FETCH_SIZE / WRITE_SIZE are scaled by")
    parser.add_argument("--bf16-operands", action="store_true",
                        help="keep MXFP4 banks with groups of hundreds of rows on the bf16 matrix instruction too (the default "
                             "there: rows split into two e4m3 terms and the scaled instruction, the library's own choice)")
    parser.add_argument("--second-term", choices=["e4m3", "e2m3", "e2m3x2"], default=None,
                        help="how the split rows of the first product are held: two e4m3 terms, an e4m3 and an e2m3 term, or two "
                             "e2m3 terms (default: the library's, gemm.SPLIT_SECOND_TERM)")
    parser.add_argument("--separate-shared", action="store_true",
                        help="compute a shared expert as a dense MLP of its own (two more launches), as the reference does, instead "
                             "of as group #E of the routed launches")
    parser.add_argument("--graph", choices=["auto", "on", "off"], default="auto",
                        help="replay the step as one captured HIP graph (auto: for the launch-bound configs c1 and c3)")
    args = parser.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (the path would shard by expert over "
                 "an all-to-all each way; that is designed, not built). Run with --gpus 1.")

    import torch

    from dew_amd import gemm, ops

    if args.second_term is not None:
        gemm.SPLIT_SECOND_TERM = args.second_term
    ops.device_check()
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    sustained = sustained_rates(device)
    if args.calibrate_copy:
        print(json.dumps({"probe_copy_bytes_read_per_launch": 1 << 30, "probe_copy_bytes_written_per_launch": 1 << 30,
                          "sustained_copy_gbs": sustained[1], "sustained_bf16_mfma_tflops": sustained[0]}))
        return
    top = measure(args.config, args, device, sustained, with_cpu_baseline=not args.no_cpu_baseline)
    result = {
        "metric": "grouped-GEMM TFLOP/s & % MFMA peak (prefill); HBM GB/s & % peak (decode)",
        "value": top["value"], "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": top["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic", "config": top["config"], "roofline": top["roofline"],
    }
    for name in ("cpu_baseline", "sample_parity", "min_topk_margin", "router_logits"):
        if name in top:
            result[name] = top[name]
    if not args.only:
        per_config = {}
        for config in ALL_CONFIGS:
            if config == args.config:
                measured = {k: v for k, v in top.items() if k != "cpu_baseline" or config in WHOLE_ON_CPU}
            else:
                print(f"[bench] measuring {config}", file=sys.stderr, flush=True)
                measured = measure(config, args, device, sustained, with_cpu_baseline=False)
            per_config[config] = measured
        # the same c2 workload with the split rows' terms in FP6 (gemm.SPLIT_SECOND_TERM = 'e2m3': the second; 'e2m3x2': both):
        # the faster, less exact options, measured in the same run beside the default so that their price in parity stands
        # next to their gain
        for option, label in (("e2m3", "c2_option_e2m3_second_term"), ("e2m3x2", "c2_option_two_e2m3_terms")):
            if gemm.SPLIT_SECOND_TERM != option:
                print(f"[bench] measuring c2 with {label}", file=sys.stderr, flush=True)
                held, gemm.SPLIT_SECOND_TERM = gemm.SPLIT_SECOND_TERM, option
                try:
                    per_config[label] = measure("c2", args, device, sustained, with_cpu_baseline=False)
                finally:
                    gemm.SPLIT_SECOND_TERM = held
        result["configs"] = per_config
    print(json.dumps(result))


if __name__ == "__main__":
    main()

"""bench.py's command line, as far as a machine without a GPU can check it."""

import pathlib
import subprocess
import sys

ROOT = pathlib.Path(__file__).resolve().parent.parent


def test_more_than_one_gpu_is_refused_with_a_message():
    done = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert done.returncode != 0
    assert "one GPU" in done.stderr and "--gpus 1" in done.stderr and done.stdout == ""


def test_the_default_workload_is_the_metrics_configuration():
    done = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--help"], capture_output=True, text=True, timeout=120)
    assert done.returncode == 0
    for flag in ("--gpus", "--steps", "--warmup", "--config", "--bf16-operands"):
        assert flag in done.stdout


def test_the_lines_traffic_is_what_the_committed_summaries_hold():
    """`roofline.traffic` is parsed from the rocprofv3 summaries under profiles/: every workload has its rows there, the
    paired gate/up launches counted are the ones the same file's kernel trace times, and the figure in bytes is the
    summary's own scaled columns."""
    import re

    sys.path.insert(0, str(ROOT))
    import bench

    scales = bench.counter_scales()
    assert set(scales) == {"FETCH_SIZE", "WRITE_SIZE"} and all(0.5 <= factor <= 4.0 for factor in scales.values())
    for config in bench.ALL_CONFIGS:
        counted = bench.counted_kib(config)
        assert counted is not None and counted["FETCH_SIZE"] > 0 and counted["WRITE_SIZE"] > 0, config
        text = (ROOT / bench.COUNTED_FROM[config]).read_text()
        trace, traffic = text.split("2. HBM traffic", 1)
        assert f"--config {config} --only" in trace                      # the summary is of this workload's command
        paired = re.findall(r"^(dew::grouped_gemm_kernel<\d+, (?:1|3), [^>]*>(?: grid \d+)?)\s", traffic, re.M)
        assert paired and all(name in trace for name in paired), (config, paired)
        scaled = 0.0
        for line in traffic.splitlines():
            if any(line.startswith(name + " ") for name in paired):
                read, written = line.split()[-2:]
                scaled += float(read) + float(written)
        assert abs(bench.measured_traffic(config) - scaled) <= 2e-3 * scaled, (config, bench.measured_traffic(config), scaled)
    assert bench.counted_kib("c9") is None

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

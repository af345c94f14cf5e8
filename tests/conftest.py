"""Shared test plumbing: the `gpu` marker, the repo root on sys.path, golden-vector loading."""

import json
import sys
from pathlib import Path

import numpy as np
import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

GOLDEN = Path(__file__).resolve().parent / "golden"


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def moe_config():
    return json.loads((GOLDEN / "moe" / "config.json").read_text())


def golden(relative):
    """A golden .npz (data the reference's own tests hold, copied as data) as a dict of arrays."""
    with np.load(GOLDEN / relative, allow_pickle=False) as archive:
        return {name: archive[name] for name in archive.files}

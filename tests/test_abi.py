"""The C-ABI library loads and exports every symbol include/dew_moe_hip.h declares (no compute: no GPU)."""

import re
from pathlib import Path

from dew_amd import _lib

HEADER = Path(__file__).resolve().parent.parent / "include" / "dew_moe_hip.h"


def declared_symbols():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(dew_moe_\w+)\s*\(", text)))


def test_the_library_exports_every_declared_symbol():
    lib = _lib.library()
    names = declared_symbols()
    assert names == sorted(_lib.EXPORTS)
    for name in names:
        assert getattr(lib, name) is not None


def test_introspection_strings_and_size_queries():
    lib = _lib.library()
    assert lib.dew_moe_architecture() == b"gfx950"
    fields = lib.dew_moe_kernel_fields().decode().split(",")
    for line in lib.dew_moe_kernels().decode().strip().splitlines():
        assert len(line.split(",")) == len(fields)
    assert lib.dew_moe_prepared_bytes(_lib.W_FP8_BLOCK, 2, 256, 128) == 2 * 256 * 128 + 2 * 2 * 1 * 4   # codes + block scales
    assert lib.dew_moe_prepared_bytes(_lib.W_FP8_CHANNEL, 2, 256, 128) == 2 * 256 * 128
    assert lib.dew_moe_prepared_bytes(_lib.W_NVFP4, 2, 256, 128) == 2 * 256 * 128 // 2 + 2 * 128 * 16 + 256
    assert lib.dew_moe_permute_workspace_bytes(4096, 8) >= 2 * 2 * 9 * 4


def test_argument_errors_are_named_without_a_gpu():
    lib = _lib.library()
    assert lib.dew_moe_route(None, None, 4, 8, 2, 0, 1, 1.0, 1, 1, None, None, None) == 1
    assert b"must not be null" in lib.dew_moe_last_error()
    assert lib.dew_moe_combine(None, None, None, None, 4, 2, 12, None) == 1
    assert b"multiple of 8" in lib.dew_moe_last_error()

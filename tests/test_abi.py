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


def test_the_split_row_rule_is_the_librarys_and_its_workspace_holds_the_intermediates():
    """`dew_moe_prefers_split_rows` on descriptors alone (no device memory is read): three chaining MXFP4 banks of whole
    256-column strips from DEW_MOE_SPLIT_ROWS_FROM rows a group; the host mirror's constant is the header's."""
    from dew_amd import ops

    lib = _lib.library()
    assert int(re.search(r"#define DEW_MOE_SPLIT_ROWS_FROM (\d+)", HEADER.read_text()).group(1)) == ops.SPLIT_ROWS_FROM

    def bank(fmt, experts, depth, width, layout=_lib.LAYOUT_PREPARED):
        return _lib.Bank(fmt, layout, experts, depth, width, None, None, None)

    gate, down = bank(_lib.W_MXFP4, 8, 4096, 14336), bank(_lib.W_MXFP4, 8, 14336, 4096)
    assert lib.dew_moe_prefers_split_rows(gate, gate, down, 8 * ops.SPLIT_ROWS_FROM) == 1
    assert lib.dew_moe_prefers_split_rows(gate, gate, down, 8 * ops.SPLIT_ROWS_FROM - 1) == 0
    assert lib.dew_moe_prefers_split_rows(gate, gate, bank(_lib.W_MXFP4, 8, 4096, 4096), 32768) == 0           # does not chain
    assert lib.dew_moe_prefers_split_rows(gate, bank(_lib.W_NVFP4, 8, 4096, 14336), down, 32768) == 0           # general block scales
    assert lib.dew_moe_prefers_split_rows(bank(_lib.W_MXFP4, 8, 4096, 14336 + 128), gate, down, 32768) == 0     # no whole 256-column strips
    assert lib.dew_moe_prefers_split_rows(gate, gate, bank(_lib.W_MXFP4, 8, 14336, 4096, _lib.LAYOUT_REFERENCE), 32768) == 0
    assert lib.dew_moe_prefers_split_rows(None, gate, down, 32768) == 0
    deep = bank(_lib.W_MXFP4, 8, 4096, 24576 + 256)
    assert lib.dew_moe_prefers_split_rows(deep, deep, bank(_lib.W_MXFP4, 8, 24576 + 256, 4096), 32768) == 0     # a tile's scales would not fit the LDS
    tokens, rows, depth, width, experts = 16384, 32768, 4096, 14336, 8
    need = lib.dew_moe_swiglu_mlp_split_workspace_bytes(tokens, rows, depth, width, experts)
    assert need >= tokens * depth * 2 + tokens + rows * width * 2 + rows * ops.block_scale_pitch(width) + (experts + 1) * 4
    assert need <= tokens * depth * 2 + tokens + rows * width * 2 + rows * ops.block_scale_pitch(width) + (experts + 1) * 4 + 6 * 256
    assert lib.dew_moe_swiglu_mlp_split(None, 4, None, None, None, gate, gate, down, None, None, 4, 0, None, 0, None) == 1
    assert b"gate bank codes and scales must not be null" in lib.dew_moe_last_error()   # descriptors without memory are refused first

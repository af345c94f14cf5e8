"""The benchmarks' measurement probes (bench_aids/probe.hip, built into libdew_bench_probes.so): what the chip
sustains, measured in the same run as the kernels. No part of the MoE library or its C ABI."""

import ctypes
from pathlib import Path

import torch

LIBRARY = Path(__file__).resolve().parent / "libdew_bench_probes.so"
_handle = None


def _library():
    global _handle
    if _handle is None:
        if not LIBRARY.exists():
            raise RuntimeError(f"{LIBRARY} is not built: run `make -C {LIBRARY.parent}`")
        lib = ctypes.CDLL(str(LIBRARY))
        c = ctypes
        lib.dew_bench_probe_mfma.restype, lib.dew_bench_probe_mfma.argtypes = c.c_int32, [c.c_void_p, c.c_int32, c.c_void_p, c.POINTER(c.c_double), c.c_void_p]
        lib.dew_bench_probe_copy.restype, lib.dew_bench_probe_copy.argtypes = c.c_int32, [c.c_void_p, c.c_void_p, c.c_size_t, c.c_void_p]
        lib.dew_bench_probe_read.restype, lib.dew_bench_probe_read.argtypes = c.c_int32, [c.c_void_p, c.c_size_t, c.c_void_p, c.c_void_p]
        _handle = lib
    return _handle


def probe_mfma(operands: torch.Tensor, iters: int) -> float:
    """Launch back-to-back v_mfma_f32_32x32x16_bf16 on `operands` (bf16, 16384 values, on the device); returns the
    launch's FLOP count."""
    if not operands.is_cuda or operands.dtype != torch.bfloat16 or operands.numel() < 16384 or not operands.is_contiguous():
        raise ValueError("the MFMA probe reads 16384 contiguous bf16 operands on the device")
    sink = torch.empty(1024 * 256, dtype=torch.float32, device=operands.device)
    flops = ctypes.c_double(0.0)
    code = _library().dew_bench_probe_mfma(operands.data_ptr(), iters, sink.data_ptr(), ctypes.byref(flops), torch.cuda.current_stream().cuda_stream)
    if code != 0:
        raise RuntimeError(f"dew_bench_probe_mfma returned {code}")
    return flops.value


def probe_copy(src: torch.Tensor, dst: torch.Tensor) -> int:
    """Launch the plain copy `dst = src`; returns the bytes copied (read once, written once)."""
    size = src.numel() * src.element_size()
    if not (src.is_cuda and dst.is_cuda and src.is_contiguous() and dst.is_contiguous()) or size != dst.numel() * dst.element_size() or size % 16:
        raise ValueError("the copy probe takes two contiguous device buffers of one size, a multiple of 16 bytes")
    code = _library().dew_bench_probe_copy(src.data_ptr(), dst.data_ptr(), size, torch.cuda.current_stream().cuda_stream)
    if code != 0:
        raise RuntimeError(f"dew_bench_probe_copy returned {code}")
    return size


def probe_read(src: torch.Tensor) -> int:
    """Launch the read-only stream over `src` (a contiguous device buffer of whole 64 KiB); returns the bytes read."""
    size = src.numel() * src.element_size()
    if not (src.is_cuda and src.is_contiguous()) or size % 65536:
        raise ValueError("the read probe takes a contiguous device buffer of whole 64 KiB segments")
    sink = torch.zeros(1, dtype=torch.int32, device=src.device)
    code = _library().dew_bench_probe_read(src.data_ptr(), size, sink.data_ptr(), torch.cuda.current_stream().cuda_stream)
    if code != 0:
        raise RuntimeError(f"dew_bench_probe_read returned {code}")
    return size

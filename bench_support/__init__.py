"""Calibration kernels of the benchmark, kept out of the product library: ``bench_support/libmase_bench.so`` built from
``bench_support/probes.hip`` (a plain streaming copy and the matrix-core issue-rate probes).  ``bench.py`` loads it for
the ``copy`` and ``mfma_*_rate_*`` workloads; nothing in ``mase_amd`` uses it."""
from __future__ import annotations

import ctypes
import os
import subprocess
from ctypes import c_int, c_size_t, c_void_p

DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(DIR, "libmase_bench.so")
SOURCE = os.path.join(DIR, "probes.hip")

SIGNATURES = {
    "bench_copy_bytes": (c_int, [c_void_p, c_void_p, c_size_t, c_void_p]),
    "bench_probe_mfma_bf16": (c_int, [c_void_p, c_size_t, c_int, c_int, c_int, c_int, c_void_p]),
    "bench_probe_mfma_bf16_16x16": (c_int, [c_void_p, c_size_t, c_int, c_int, c_int, c_int, c_void_p]),
    "bench_probe_mfma_f8f4": (c_int, [c_void_p, c_size_t, c_int, c_int, c_int, c_int, c_void_p]),
    "bench_constant_rate_counter_khz": (c_int, []),
}

_lib = None


def build(verbose: bool = False) -> str:
    """compiles the library for gfx950 with the product library's flags"""
    from mase_amd.build import COMMON_FLAGS, HIPCC

    cmd = [HIPCC, *COMMON_FLAGS, "-shared", SOURCE, "-o", LIB_PATH]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for {SOURCE}:\n{res.stderr}")
    return LIB_PATH


def load() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} not found: build it with `python -c 'import bench_support; bench_support.build()'`")
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib

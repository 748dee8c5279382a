"""Builds ``mase_amd/lib/libmase_amd.so`` (the C-ABI library) from ``mase_amd/csrc/*.hip`` with hipcc for gfx950.

Usage:  python -m mase_amd.build [-j N] [-i]
The library is built in-tree so that it travels with the source tree; nothing is installed.
"""
from __future__ import annotations

import argparse
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
SRC_DIR = os.path.join(PKG_DIR, "csrc")
LIB_DIR = os.path.join(PKG_DIR, "lib")
OBJ_DIR = os.path.join(LIB_DIR, "obj")
LIB_PATH = os.path.join(LIB_DIR, "libmase_amd.so")

HIPCC = os.environ.get("HIPCC") or shutil.which("hipcc") or "/opt/rocm/bin/hipcc"

# packed-fp32 VALU forms are switched off for every kernel in this library
COMMON_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-gpu-rdc",
    "-ffp-contract=off",  # the reference rounds after every op; no fused multiply-add behind its back
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-function",
]


# extra compiler flags for experiments, e.g. MASE_EXTRA_HIPCC_FLAGS="-DMASE_RUN_THREADS=64"
COMMON_FLAGS += os.environ.get("MASE_EXTRA_HIPCC_FLAGS", "").split()


def sources() -> list[str]:
    return sorted(os.path.join(SRC_DIR, f) for f in os.listdir(SRC_DIR) if f.endswith(".hip"))


def _headers_mtime() -> float:
    hs = [os.path.join(SRC_DIR, f) for f in os.listdir(SRC_DIR) if f.endswith(".hpp")]
    hs.append(os.path.join(os.path.dirname(PKG_DIR), "include", "mase_amd.h"))
    return max(os.path.getmtime(h) for h in hs)


def _compile(src: str, verbose: bool, incremental: bool = False) -> str:
    obj = os.path.join(OBJ_DIR, os.path.basename(src)[:-4] + ".o")
    if incremental and os.path.exists(obj) and os.path.getmtime(obj) > max(os.path.getmtime(src), _headers_mtime()):
        return obj
    cmd = [HIPCC, *COMMON_FLAGS, "-c", src, "-o", obj]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    # hipcc's host pass warns that it does not know the packed-fp32 feature: harmless, filtered out
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l and l.strip())
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{res.stderr}")
    if err and verbose:
        print(err, file=sys.stderr)
    return obj


def build_library(jobs: int = 8, verbose: bool = True, incremental: bool = False) -> str:
    """compiles every source (``incremental``: only those newer than their object) and links the library"""
    os.makedirs(OBJ_DIR, exist_ok=True)
    srcs = sources()
    with ThreadPoolExecutor(max_workers=max(1, min(jobs, len(srcs)))) as ex:
        objs = list(ex.map(lambda s: _compile(s, verbose, incremental), srcs))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", *objs, "-o", LIB_PATH]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    return LIB_PATH


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("-j", type=int, default=8)
    ap.add_argument("-q", action="store_true")
    ap.add_argument("-i", "--incremental", action="store_true", help="recompile only sources newer than their objects")
    a = ap.parse_args()
    path = build_library(a.j, not a.q, a.incremental)
    print("built", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()

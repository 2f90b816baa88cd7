"""Compile the gfx950 kernels into libatorch_amd_fp8.so (in-tree, next to the sources).

    python -m atorch_amd.csrc.build          # or: python atorch_amd/csrc/build.py

hipcc cross-compiles for gfx950 without a GPU present.  Packed-FP32 instruction selection is
switched off for all device code.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
SOURCES = ["capi.hip", "quant.hip", "permute.hip", "gemm.hip", "probe.hip"]
LIB = os.path.join(HERE, "libatorch_amd_fp8.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]  # fmt: skip


def _compile(src: str, extra) -> str:
    obj = os.path.join(HERE, src.replace(".hip", ".o"))
    subprocess.check_call([HIPCC, *FLAGS, *extra, "-c", os.path.join(HERE, src), "-o", obj])
    return obj


def build(verbose: bool = False, extra_flags=()) -> str:
    with ThreadPoolExecutor(max_workers=5) as ex:
        objs = list(ex.map(lambda s: _compile(s, list(extra_flags)), SOURCES))
    subprocess.check_call([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs])
    if verbose:
        print("built", LIB)
    return LIB


if __name__ == "__main__":
    build(verbose=True, extra_flags=sys.argv[1:])

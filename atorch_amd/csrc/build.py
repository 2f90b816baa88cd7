"""Compile the gfx950 kernels, in-tree, next to the sources:

    libatorch_amd_fp8.so      the product library (include/atorch_amd_fp8.h)
    libatorch_amd_probes.so   measurement aids for the benchmark and the tests (include/atorch_amd_probes.h):
                              probes, and the grouped GEMMs with their launch choices pinned per call

    python -m atorch_amd.csrc.build          # or: python atorch_amd/csrc/build.py

hipcc cross-compiles for gfx950 without a GPU present.  Packed-FP32 instruction selection is
switched off for all device code.  Symbols other than the C entry points stay local to each library.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
SOURCES = ["capi.hip", "tile_offsets.hip", "quant.hip", "permute.hip", "gemm.hip"]
PROBE_SOURCES = ["capi.hip", "tile_offsets.hip", "gemm.hip", "probe.hip"]  # compiled with -DAAMD_TUNING
LIB = os.path.join(HERE, "libatorch_amd_fp8.so")
PROBES_LIB = os.path.join(HERE, "libatorch_amd_probes.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]  # fmt: skip
LINK = ["--offload-arch=gfx950", "-shared", "-fPIC", "-Wl,-Bsymbolic"]


def _compile(job) -> str:
    src, suffix, extra = job
    obj = os.path.join(HERE, src.replace(".hip", suffix + ".o"))
    subprocess.check_call([HIPCC, *FLAGS, *extra, "-c", os.path.join(HERE, src), "-o", obj])
    return obj


def build(verbose: bool = False, extra_flags=()) -> str:
    extra = list(extra_flags)
    jobs = [(s, "", extra) for s in SOURCES] + [(s, ".probes", extra + ["-DAAMD_TUNING"]) for s in PROBE_SOURCES]
    with ThreadPoolExecutor(max_workers=8) as ex:
        objs = list(ex.map(_compile, jobs))
    subprocess.check_call([HIPCC, *LINK, "-o", LIB, *objs[: len(SOURCES)]])
    subprocess.check_call([HIPCC, *LINK, "-o", PROBES_LIB, *objs[len(SOURCES) :]])
    if verbose:
        print("built", LIB)
        print("built", PROBES_LIB)
    return LIB


if __name__ == "__main__":
    build(verbose=True, extra_flags=sys.argv[1:])

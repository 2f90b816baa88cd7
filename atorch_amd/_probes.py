"""ctypes binding of libatorch_amd_probes.so (include/atorch_amd_probes.h): measurement aids for the
benchmark and the tests.  Nothing in the product path imports this module."""
import ctypes
import os
from typing import Optional

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libatorch_amd_probes.so")

_i64, _vp, _int = ctypes.c_int64, ctypes.c_void_p, ctypes.c_int
_opts = ctypes.POINTER(ctypes.c_int)

# name -> (restype, argtypes); one entry per symbol of include/atorch_amd_probes.h
SIGNATURES = {
    "aamd_probes_last_error": (ctypes.c_char_p, []),
    "aamd_tuning_grouped_gemm_fp8_nt": (
        _int,
        [_vp, _i64, _vp, _vp, _vp, _int, _vp, _int, _vp, _i64, _i64, _i64, _vp, _int, _i64, _vp, _int, _opts, _vp],
    ),
    "aamd_tuning_grouped_gemm_fp8_wgrad": (
        _int,
        [_vp, _vp, _vp, _vp, _i64, _int, _vp, _int, _vp, _i64, _i64, _vp, _int, _i64, _int, _opts, _vp],
    ),
    "aamd_clock_probe": (_int, [_vp, _i64, _vp]),
    "aamd_stream_probe": (_int, [_vp, _vp, _int, _int, _i64, _i64, _vp]),
    "aamd_mfma_probe": (_int, [_vp, _int, _int, _int, _vp, _vp, _vp]),
    "aamd_loop_probe": (_int, [_vp, _i64, _int, _int, _vp, _vp, _vp]),
}

OPTION_NAMES = ("tile", "group_r", "gl", "ls_batch")

_lib: Optional[ctypes.CDLL] = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} not found: build it with `python -m atorch_amd.csrc.build`")
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def check(rc: int):
    if rc != 0:
        msg = lib().aamd_probes_last_error().decode("utf-8", "replace")
        if rc == 1:
            raise ValueError(msg)
        raise RuntimeError(msg)


def options_array(opts: dict):
    """{tile, group_r, gl, ls_batch} -> the int[4] the pinned GEMM entry points take (-1 = library's choice)."""
    unknown = set(opts) - set(OPTION_NAMES)
    if unknown:
        raise ValueError(f"unknown GEMM launch option(s) {sorted(unknown)}; known: {OPTION_NAMES}")
    return (ctypes.c_int * 4)(*[int(opts.get(k, -1)) for k in OPTION_NAMES])

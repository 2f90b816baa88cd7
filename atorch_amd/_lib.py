"""ctypes binding of libatorch_amd_fp8.so (the C ABI declared in include/atorch_amd_fp8.h).

There is no fallback: if the HIP library has not been built, every op raises.
"""
import ctypes
import os
from typing import Optional

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libatorch_amd_fp8.so")

OK, ERR_ARG, ERR_HIP = 0, 1, 2
NONE, BF16, F32, F16 = -1, 0, 1, 2
QT_ROWS, QT_BLOCKED = 0, 1  # layouts of the transposed codes
ABI_VERSION = 4

_lib: Optional[ctypes.CDLL] = None

_i64, _i32, _f32, _vp, _int = ctypes.c_int64, ctypes.c_int32, ctypes.c_float, ctypes.c_void_p, ctypes.c_int

# name -> (restype, argtypes); one entry per symbol of include/atorch_amd_fp8.h
SIGNATURES = {
    "aamd_abi_version": (_int, []),
    "aamd_last_error": (ctypes.c_char_p, []),
    "aamd_quant_1x128": (_int, [_vp, _int, _i64, _i64, _i64, _vp, _vp, _f32, _vp]),
    "aamd_permute_quant_1x128": (_int, [_vp, _int, _i64, _i64, _i64, _vp, _int, _i64, _vp, _vp, _f32, _vp]),
    "aamd_permute_rows": (_int, [_vp, _int, _i64, _i64, _vp, _int, _i64, _vp, _vp]),
    "aamd_quant_1x128_dual_grouped": (
        _int,
        [_vp, _int, _i64, _i64, _i64, _vp, _int, _vp, _vp, _vp, _vp, _vp, _i64, _int, _f32, _vp],
    ),
    "aamd_permute_quant_1x128_dual_grouped": (
        _int,
        [_vp, _int, _i64, _i64, _i64, _vp, _int, _i64, _vp, _int, _vp, _vp, _vp, _vp, _vp, _i64, _int, _f32, _vp],
    ),
    "aamd_swiglu_quant_1x128": (_int, [_vp, _i64, _i64, _i64, _vp, _vp, _vp, _vp]),
    "aamd_swiglu_quant_1x128_dual_grouped": (
        _int,
        [_vp, _i64, _i64, _i64, _vp, _int, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _int, _vp],
    ),
    "aamd_swiglu_bwd_quant_1x128_dual_grouped": (
        _int,
        [_vp, _i64, _vp, _i64, _i64, _i64, _vp, _int, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _int, _vp],
    ),
    "aamd_gelu_quant_1x128": (_int, [_vp, _i64, _i64, _i64, _vp, _vp, _vp, _vp]),
    "aamd_gelu_quant_1x128_dual_grouped": (
        _int,
        [_vp, _vp, _i64, _i64, _i64, _vp, _int, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _int, _vp],
    ),
    "aamd_bias_gather_add": (_int, [_vp, _vp, _vp, _int, _i64, _i64, _int, _int, _vp, _vp]),
    "aamd_bias_gather_add_bgrad": (_int, [_vp, _vp, _int, _i64, _i64, _int, _int, _vp, _vp]),
    "aamd_quant_128x128": (_int, [_vp, _int, _i64, _i64, _i64, _i64, _vp, _vp, _vp, _vp, _f32, _vp]),
    "aamd_dequant": (_int, [_vp, _vp, _i64, _i64, _int, _vp, _int, _vp]),
    "aamd_grouped_gemm_fp8_nt": (
        _int,
        [_vp, _i64, _vp, _vp, _vp, _int, _vp, _int, _vp, _i64, _i64, _i64, _vp, _int, _i64, _vp, _int, _vp],
    ),
    "aamd_grouped_gemm_fp8_wgrad": (
        _int,
        [_vp, _vp, _vp, _vp, _i64, _int, _vp, _int, _vp, _i64, _i64, _vp, _int, _i64, _int, _vp],
    ),
    "aamd_grouped_gemm_fp8_nt_static": (
        _int,
        [_vp, _i64, _vp, _vp, _vp, _int, _vp, _int, _i64, _i64, _i64, _vp, _int, _i64, _vp, _int, _vp],
    ),
    "aamd_unpermute_combine": (_int, [_vp, _int, _i64, _i64, _vp, _vp, _int, _i64, _int, _vp, _vp]),
    "aamd_permute_rows_scaled": (_int, [_vp, _int, _i64, _i64, _vp, _int, _vp, _int, _i64, _vp, _int, _vp]),
    "aamd_unpermute_probs_grad": (_int, [_vp, _int, _vp, _int, _i64, _i64, _vp, _i64, _int, _vp, _vp]),
    "aamd_moe_preprocess_ws_ints": (_i64, [_i64, _int]),
    "aamd_moe_preprocess": (_int, [_vp, _int, _i64, _int, _vp, _vp, _vp, _vp, _vp]),
    "aamd_invert_permutation": (_int, [_vp, _i64, _i64, _vp, _vp]),
}


class HipLibraryMissing(RuntimeError):
    pass


def lib() -> ctypes.CDLL:
    """The loaded library.  Raises HipLibraryMissing when it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise HipLibraryMissing(
                f"{LIB_PATH} not found: build it with `python -m atorch_amd.csrc.build` "
                "(atorch_amd has no CPU or eager fallback)"
            )
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        if L.aamd_abi_version() != ABI_VERSION:
            raise HipLibraryMissing(f"{LIB_PATH}: ABI version {L.aamd_abi_version()} != {ABI_VERSION}, rebuild it")
        _lib = L
    return _lib


def check(rc: int):
    if rc != OK:
        msg = lib().aamd_last_error().decode("utf-8", "replace")
        if rc == ERR_ARG:
            raise ValueError(msg)
        raise RuntimeError(msg)


def dtype_code(dt: torch.dtype, quantiser_input: bool = False) -> int:
    if dt == torch.bfloat16:
        return BF16
    if dt == torch.float32:
        return F32
    if dt == torch.float16 and quantiser_input:
        return F16
    raise ValueError(f"atorch_amd: unsupported dtype {dt} (bf16 and fp32 are supported; fp16 as quantiser input)")


def ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    if t is None:
        return None
    if not t.is_cuda:
        raise ValueError("atorch_amd ops need tensors on the GPU (there is no CPU path)")
    return t.data_ptr()


def stream() -> int:
    return torch.cuda.current_stream().cuda_stream

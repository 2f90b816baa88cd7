"""The operator module the reference loads by name for its dense FP8 path.

``atorch/modules/fp8/cuda_kernel.py:7-11`` imports the module named by the environment variable
``FP8_GEMM_MODULE_OPS`` (default ``kitchen.ops``) and calls, on it,

    quantize_vector_blockwise(x, dtype, block_size, return_transpose=, eps=, pow_2_scale=, backend=)   (:30-38)
    quantize_square_blockwise(x, dtype, block_size, return_transpose=, eps=, pow_2_scale=, backend=)   (:53-61)
    fp8_gemm_blockwise / cutlass_gemm_fp8_blockwise(a, a_s, b, b_s, dtype, out=, accumulate=,
        use_split_accumulator=, is_a_1d_scaled=, is_b_1d_scaled=)                                       (:69-81)
    Backend.CUBLAS / Backend.CUTLASS

Setting ``FP8_GEMM_MODULE_OPS=atorch_amd.ops`` therefore routes the reference's ``tile_quant``,
``block_quant`` and ``fp8_gemm`` wrappers (and through them ``ScaledLinear``'s tile/block recipe)
onto the HIP kernels of this package without touching the reference's code.  Both backends name
the same kernels here.
"""
import enum
from typing import Optional

import torch

from . import kernels

TILE = kernels.TILE


class Backend(enum.Enum):
    CUTLASS = 0
    CUBLAS = 1


def _check_common(dtype, block_size, pow_2_scale):
    if dtype != torch.float8_e4m3fn:
        raise NotImplementedError("only torch.float8_e4m3fn is supported")
    if block_size != TILE:
        raise NotImplementedError("only block_size 128 is supported")
    if pow_2_scale:
        raise NotImplementedError("power-of-two scales are not implemented; scales are amax/448 in fp32")


def quantize_vector_blockwise(x, dtype=torch.float8_e4m3fn, block_size=TILE, return_transpose=False, eps=0.0,
                              pow_2_scale=False, backend=None):  # fmt: skip
    """1x128 quantisation; returns ``(qx, sx, qx_t, sx_t)`` with the last two ``None`` unless
    ``return_transpose`` (then ``qx_t`` is ``[K, M]`` and ``sx_t`` ``[K, ceil(M/128)]``, contiguous)."""
    _check_common(dtype, block_size, pow_2_scale)
    x = x.contiguous()
    if not return_transpose:
        q, s = kernels.tile_quant(x, eps=eps)
        return q, s, None, None
    x2 = x.view(-1, x.size(-1))
    q, s, q_t, s_t = kernels.tile_quant(x2, eps=eps, return_transpose=True)
    return q.view(x.shape), s.view(*x.shape[:-1], -1), q_t.contiguous(), s_t.contiguous()


def quantize_square_blockwise(x, dtype=torch.float8_e4m3fn, block_size=TILE, return_transpose=False, eps=0.0,
                              pow_2_scale=False, backend=None):  # fmt: skip
    """128x128 quantisation of a 2-D tensor; returns ``(qx, sx, qx_t, sx_t)``."""
    _check_common(dtype, block_size, pow_2_scale)
    out = kernels.block_quant(x.contiguous(), eps=eps, return_transpose=return_transpose)
    if return_transpose:
        return out
    return out[0], out[1], None, None


def fp8_gemm_blockwise(a, a_s, b, b_s, dtype=torch.bfloat16, out: Optional[torch.Tensor] = None, accumulate=False,
                       use_split_accumulator=True, is_a_1d_scaled=True, is_b_1d_scaled=False):  # fmt: skip
    """``C = A @ B^T`` for K-major fp8 ``A [M, K]`` (1x128 scales) and ``B [N, K]`` (128x128 or 1x128
    scales); fp32 accumulation per 128-K block with the scales applied to each block's product."""
    if not is_a_1d_scaled:
        raise NotImplementedError("A must carry 1x128 scales")
    if accumulate:
        raise NotImplementedError("accumulate is only offered by the grouped wgrad entry point")
    want_b_rows = b.size(0) if is_b_1d_scaled else b.size(0) // TILE
    assert b_s.size(0) == want_b_rows, "scale shape of B does not match is_b_1d_scaled"
    c = kernels.fp8_gemm(a.contiguous(), a_s.contiguous(), b.contiguous(), b_s.contiguous(), dtype=dtype)
    if out is not None:
        out.copy_(c)
        return out
    return c


cutlass_gemm_fp8_blockwise = fp8_gemm_blockwise

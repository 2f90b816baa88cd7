"""Functional ops over the C ABI.

The first four functions keep the names, argument meaning and error behaviour of the
reference's functional surface (atorch/modules/fp8/triton_kernel.py:40,80,127,198 and the
``return_transpose`` form of atorch/modules/fp8/cuda_kernel.py:18-61); the rest are the fused /
grouped forms the grouped linear uses.  Every function enqueues HIP kernels on the current
stream and returns torch tensors it allocated; nothing here computes on the CPU.
"""
import threading
from typing import List, Optional, Sequence, Tuple

import torch

from . import _lib
from ._lib import check, dtype_code, lib, ptr, stream

TILE = 128
FP8 = torch.float8_e4m3fn


def _require_fp8(dtype):
    if dtype != FP8:
        raise ValueError(f"only torch.float8_e4m3fn is supported, got {dtype}")


def padded_total(splits: Sequence[int]) -> int:
    return sum((int(m) + TILE - 1) // TILE * TILE for m in splits)


def padded_bound(rows: int, num_groups: int) -> int:
    """Upper bound of sum_g ceil(M_g/128)*128 that needs no knowledge of the splits."""
    return (rows // TILE + num_groups) * TILE


def group_offsets_from_splits(splits: Sequence[int], device) -> torch.Tensor:
    off = [0]
    for m in splits:
        off.append(off[-1] + int(m))
    return torch.tensor(off, dtype=torch.int64, device=device)


# ------------------------------------------------------------------------------------------
# reference-named functional surface
# ------------------------------------------------------------------------------------------
def tile_quant(
    x: torch.Tensor,
    dtype=FP8,
    block_size: int = TILE,
    eps: float = 0.0,
    return_transpose: bool = False,
):
    """1x128 quantisation along the last dim (triton_kernel.py:127-140).

    Returns ``(y, s)``; with ``return_transpose`` (cuda_kernel.py:18-38) returns
    ``(y, s, y_t, s_t)`` for a 2-D ``x`` where ``y_t`` is ``[K, M]`` (a view of a buffer whose
    rows are padded to a multiple of 128) and ``s_t`` is ``[K, ceil(M/128)]``.
    """
    _require_fp8(dtype)
    assert block_size == TILE, "only block_size 128 is supported"
    assert x.is_contiguous()
    assert x.size(-1) % block_size == 0
    cols = x.size(-1)
    rows = x.numel() // cols if cols else 0
    if return_transpose:
        assert x.dim() == 2, "return_transpose needs a 2-D input"
        if rows == 0:  # an empty group: nothing to launch
            return (
                torch.empty((0, cols), dtype=FP8, device=x.device),
                torch.empty((0, cols // TILE), dtype=torch.float32, device=x.device),
                torch.empty((cols, 0), dtype=FP8, device=x.device),
                torch.empty((cols, 0), dtype=torch.float32, device=x.device),
            )
        goff = torch.tensor([0, rows], dtype=torch.int64, device=x.device)
        y, s, y_t, s_t = tile_quant_dual_grouped(x, goff, 1, eps=eps, ld_t=padded_total([rows]))
        return y, s, y_t[:, :rows], s_t.t()
    y = torch.empty(x.shape, dtype=FP8, device=x.device)
    s = torch.empty(*x.shape[:-1], cols // TILE, dtype=torch.float32, device=x.device)
    check(lib().aamd_quant_1x128(ptr(x), dtype_code(x.dtype, True), rows, cols, cols, ptr(y), ptr(s), eps, stream()))
    return y, s


def block_quant(
    x: torch.Tensor,
    dtype=FP8,
    block_size: int = TILE,
    eps: float = 0.0,
    return_transpose: bool = False,
):
    """128x128 block quantisation of a 2-D tensor (triton_kernel.py:40-46).
    Returns ``(y, s)`` or ``(y, s, y_t, s_t)`` (cuda_kernel.py:41-61)."""
    _require_fp8(dtype)
    assert block_size == TILE, "only block_size 128 is supported"
    assert x.dim() == 2
    q, s, q_t, s_t = block_quant_batched(x.unsqueeze(0), eps=eps, return_transpose=return_transpose)
    if return_transpose:
        return q[0], s[0], q_t[0], s_t[0]
    return q[0], s[0]


def dequant(x: torch.Tensor, s: torch.Tensor, dtype=torch.float32, block_size: int = TILE) -> torch.Tensor:
    """y = x * s with tile scales when ``s.size(0) == x.size(0)``, else block scales
    (triton_kernel.py:80-91)."""
    assert x.is_contiguous() and s.is_contiguous(), "Input tensors must be contiguous"
    assert x.dim() == 2 and s.dim() == 2, "Input tensors must have 2 dimensions"
    assert block_size == TILE
    M, N = x.size()
    y = torch.empty((M, N), dtype=dtype, device=x.device)
    tile_scale = s.size(0) == x.size(0)
    check(lib().aamd_dequant(ptr(x), ptr(s), M, N, int(tile_scale), ptr(y), dtype_code(dtype), stream()))
    return y


def fp8_gemm(a: torch.Tensor, a_s: torch.Tensor, b: torch.Tensor, b_s: torch.Tensor, dtype=torch.bfloat16):
    """C = A @ B^T with 1x128 scales on A and 128x128 (or 1x128) scales on B
    (triton_kernel.py:198-210)."""
    assert a.is_contiguous() and b.is_contiguous()
    assert a_s.is_contiguous() and b_s.is_contiguous()
    K = a.size(-1)
    M = a.numel() // K
    N = b.size(0)
    c = torch.empty(*a.size()[:-1], N, dtype=dtype, device=a.device)
    b_tile_scale = b_s.size(0) == b.size(0)
    args = (ptr(a), K, ptr(a_s), ptr(b), ptr(b_s), int(b_tile_scale), None, 1, None, M, N, K,
            ptr(c), dtype_code(dtype), N, None, _lib.NONE)  # fmt: skip
    pinned = _pinned_options()
    if pinned:
        from . import _probes

        _probes.check(_probes.lib().aamd_tuning_grouped_gemm_fp8_nt(*args, _probes.options_array(pinned), stream()))
    else:
        check(lib().aamd_grouped_gemm_fp8_nt(*args, stream()))
    return c


# ------------------------------------------------------------------------------------------
# fused / grouped forms
# ------------------------------------------------------------------------------------------
def permute_tile_quant(
    x: torch.Tensor, row_map: torch.Tensor, topk: int, num_out_rows: int, eps: float = 0.0
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Quantise every token row once (1x128) and write it to its ``topk`` permuted rows.
    ``row_map`` [T*topk] int32: permuted row of flat index ``token*topk+slot`` (-1 = dropped)."""
    assert x.dim() == 2 and x.is_contiguous()
    T, cols = x.shape
    assert cols % TILE == 0
    assert row_map.dtype == torch.int32 and row_map.numel() == T * topk and row_map.is_contiguous()
    q = torch.empty((num_out_rows, cols), dtype=FP8, device=x.device)
    s = torch.empty((num_out_rows, cols // TILE), dtype=torch.float32, device=x.device)
    check(
        lib().aamd_permute_quant_1x128(
            ptr(x), dtype_code(x.dtype, True), T, cols, cols, ptr(row_map), topk, num_out_rows, ptr(q), ptr(s), eps, stream()
        )
    )
    return q, s


def permute_rows(x: torch.Tensor, row_map: torch.Tensor, topk: int, num_out_rows: int) -> torch.Tensor:
    """out[row_map[t*topk+j]] = x[t]: the un-quantised token permute, each source row read once."""
    assert x.dim() == 2 and x.is_contiguous()
    T, cols = x.shape
    assert row_map.dtype == torch.int32 and row_map.numel() == T * topk and row_map.is_contiguous()
    out = torch.empty((num_out_rows, cols), dtype=x.dtype, device=x.device)
    check(
        lib().aamd_permute_rows(ptr(x), dtype_code(x.dtype), T, cols, ptr(row_map), topk, num_out_rows, ptr(out), stream())
    )
    return out


def _alloc_qt(rows: int, ld_t: int, blocked: bool, dev) -> torch.Tensor:
    """The transposed codes of ``rows`` columns and ``ld_t`` padded tokens: ``[rows, ld_t]``, or, blocked,
    ``[ld_t/128, rows, 128]`` (token-block-major: every 128 x 128 tile is 16 KB of consecutive bytes)."""
    shape = (ld_t // TILE, rows, TILE) if blocked else (rows, ld_t)
    return torch.empty(shape, dtype=FP8, device=dev)


def qt_ld(q_t: torch.Tensor) -> int:
    """Padded token count ``ld_t`` of transposed codes in either layout."""
    return q_t.shape[0] * TILE if q_t.dim() == 3 else q_t.shape[1]


def qt_rows(q_t: torch.Tensor) -> torch.Tensor:
    """Transposed codes of either layout as ``[rows, ld_t]`` (a copy for the blocked layout)."""
    return q_t.permute(1, 0, 2).reshape(q_t.shape[1], -1) if q_t.dim() == 3 else q_t


def tile_quant_dual_grouped(
    x: torch.Tensor,
    group_offsets: torch.Tensor,
    num_groups: int,
    eps: float = 0.0,
    ld_t: Optional[int] = None,
    rowwise: bool = True,
    blocked: bool = False,
):
    """Row-wise and transposed 1x128 quantisation of ragged row groups in one pass.

    Returns ``(q [M,K], s [M,K/128], q_t [K, ld_t], s_t [ld_t/128, K])``; group g's transposed
    codes start at column ``sum_{j<g} ceil(M_j/128)*128`` and its partial last tile is zero
    padded.  ``ld_t`` defaults to a bound that needs no host knowledge of the splits.
    With ``rowwise=False`` q and s are None.  With ``blocked=True`` q_t is ``[ld_t/128, K, 128]`` (the layout
    the training path uses: the quantiser writes, and the weight-gradient GEMM reads, whole 16 KB tiles);
    ``grouped_gemm_wgrad`` takes either.
    """
    assert x.dim() == 2 and x.is_contiguous()
    M, cols = x.shape
    assert cols % TILE == 0
    assert group_offsets.dtype == torch.int64 and group_offsets.numel() == num_groups + 1
    if ld_t is None:
        ld_t = padded_bound(M, num_groups)
    dev = x.device
    q = torch.empty((M, cols), dtype=FP8, device=dev) if rowwise else None
    s = torch.empty((M, cols // TILE), dtype=torch.float32, device=dev) if rowwise else None
    q_t = _alloc_qt(cols, ld_t, blocked, dev)
    s_t = torch.empty((ld_t // TILE, cols), dtype=torch.float32, device=dev)
    ws = torch.empty(num_groups + 1, dtype=torch.int32, device=dev)
    check(
        lib().aamd_quant_1x128_dual_grouped(
            ptr(x), dtype_code(x.dtype, True), M, cols, cols, ptr(group_offsets), num_groups, ptr(ws),
            ptr(q), ptr(s), ptr(q_t), ptr(s_t), ld_t, int(blocked), eps, stream(),
        )
    )  # fmt: skip
    return q, s, q_t, s_t


def permute_tile_quant_dual_grouped(
    x: torch.Tensor,
    sorted_idx: torch.Tensor,
    topk: int,
    group_offsets: torch.Tensor,
    num_groups: int,
    eps: float = 0.0,
    ld_t: Optional[int] = None,
    rowwise: bool = True,
    blocked: bool = False,
):
    """``tile_quant_dual_grouped`` of the permuted rows without materialising them: ``x [T, K]`` is in token
    order, permuted row j is token ``sorted_idx[j] // topk`` (``sorted_idx`` int64 ``[M]`` from
    ``moe_preprocess``).  Returns ``(q [M,K], s [M,K/128], q_t [K, ld_t], s_t [ld_t/128, K])``, bit-equal to
    ``tile_quant_dual_grouped(permute_rows(x, ...), ...)``."""
    assert x.dim() == 2 and x.is_contiguous()
    T, cols = x.shape
    assert cols % TILE == 0
    assert sorted_idx.dtype == torch.int64 and sorted_idx.dim() == 1 and sorted_idx.is_contiguous()
    M = sorted_idx.numel()
    assert group_offsets.dtype == torch.int64 and group_offsets.numel() == num_groups + 1
    if ld_t is None:
        ld_t = padded_bound(M, num_groups)
    dev = x.device
    q = torch.empty((M, cols), dtype=FP8, device=dev) if rowwise else None
    s = torch.empty((M, cols // TILE), dtype=torch.float32, device=dev) if rowwise else None
    q_t = _alloc_qt(cols, ld_t, blocked, dev)
    s_t = torch.empty((ld_t // TILE, cols), dtype=torch.float32, device=dev)
    ws = torch.empty(num_groups + 1, dtype=torch.int32, device=dev)
    check(
        lib().aamd_permute_quant_1x128_dual_grouped(
            ptr(x), dtype_code(x.dtype, True), T, cols, cols, ptr(sorted_idx), topk, M, ptr(group_offsets), num_groups,
            ptr(ws), ptr(q), ptr(s), ptr(q_t), ptr(s_t), ld_t, int(blocked), eps, stream(),
        )
    )  # fmt: skip
    return q, s, q_t, s_t


def swiglu_tile_quant(fc1: torch.Tensor, return_activation: bool = False):
    """``h = silu(fc1[..., :F]) * fc1[..., F:]`` (SwiGLUActivatition, grouped_gemm_moe.py:331-334)
    quantised 1x128 along the last dim without writing ``h``.  Returns ``(q, s)`` or
    ``(q, s, h)`` (``h`` bf16) with ``return_activation``."""
    assert fc1.dtype == torch.bfloat16 and fc1.stride(-1) == 1 and fc1.is_contiguous()
    two_f = fc1.size(-1)
    assert two_f % (2 * TILE) == 0, "the gated width must be a multiple of 128"
    F = two_f // 2
    rows = fc1.numel() // two_f if two_f else 0
    dev = fc1.device
    q = torch.empty(*fc1.shape[:-1], F, dtype=FP8, device=dev)
    s = torch.empty(*fc1.shape[:-1], F // TILE, dtype=torch.float32, device=dev)
    h = torch.empty(*fc1.shape[:-1], F, dtype=torch.bfloat16, device=dev) if return_activation else None
    check(lib().aamd_swiglu_quant_1x128(ptr(fc1), rows, F, two_f, ptr(h), ptr(q), ptr(s), stream()))
    return (q, s, h) if return_activation else (q, s)


def swiglu_tile_quant_dual_grouped(
    fc1: torch.Tensor,
    group_offsets: torch.Tensor,
    num_groups: int,
    ld_t: Optional[int] = None,
    rowwise: bool = True,
    blocked: bool = False,
    return_activation: bool = False,
):
    """SwiGLU fused into ``tile_quant_dual_grouped``: row-wise and transposed 1x128 quantisation of
    ``h = silu(a) * b`` for rows ``[a | b]`` of ``fc1 [M, 2F]``.  Returns ``(q, s, q_t, s_t)`` (plus
    ``h`` with ``return_activation``), layouts as ``tile_quant_dual_grouped``."""
    assert fc1.dim() == 2 and fc1.is_contiguous() and fc1.dtype == torch.bfloat16
    M, two_f = fc1.shape
    assert two_f % (2 * TILE) == 0
    F = two_f // 2
    assert group_offsets.dtype == torch.int64 and group_offsets.numel() == num_groups + 1
    if ld_t is None:
        ld_t = padded_bound(M, num_groups)
    dev = fc1.device
    q = torch.empty((M, F), dtype=FP8, device=dev) if rowwise else None
    s = torch.empty((M, F // TILE), dtype=torch.float32, device=dev) if rowwise else None
    q_t = _alloc_qt(F, ld_t, blocked, dev)
    s_t = torch.empty((ld_t // TILE, F), dtype=torch.float32, device=dev)
    h = torch.empty((M, F), dtype=torch.bfloat16, device=dev) if return_activation else None
    ws = torch.empty(num_groups + 1, dtype=torch.int32, device=dev)
    check(
        lib().aamd_swiglu_quant_1x128_dual_grouped(
            ptr(fc1), M, F, two_f, ptr(group_offsets), num_groups, ptr(ws), ptr(h),
            ptr(q), ptr(s), ptr(q_t), ptr(s_t), ld_t, int(blocked), stream(),
        )
    )  # fmt: skip
    return (q, s, q_t, s_t, h) if return_activation else (q, s, q_t, s_t)


def swiglu_bwd_tile_quant_dual_grouped(
    dh: torch.Tensor,
    fc1: torch.Tensor,
    group_offsets: torch.Tensor,
    num_groups: int,
    ld_t: Optional[int] = None,
    rowwise: bool = True,
    blocked: bool = False,
    return_grad: bool = False,
):
    """Backward of ``h = silu(a) * b`` (rows ``[a | b]`` of ``fc1 [M, 2F]``) for the gradient
    ``dh [M, F]``, fused into ``tile_quant_dual_grouped`` of the result ``[da | db]``: what autograd
    makes of SwiGLUActivatition (grouped_gemm_moe.py:331-334) followed by the quantisation of the
    first grouped linear's output gradient.  Returns ``(q [M,2F], s, q_t [2F, ld_t], s_t)`` (plus
    the bf16 gradient ``[M, 2F]`` with ``return_grad``)."""
    assert fc1.dim() == 2 and fc1.is_contiguous() and fc1.dtype == torch.bfloat16
    assert dh.dim() == 2 and dh.is_contiguous() and dh.dtype == torch.bfloat16
    M, two_f = fc1.shape
    assert two_f % (2 * TILE) == 0
    F = two_f // 2
    assert dh.shape == (M, F), "dh must be [M, F]"
    assert group_offsets.dtype == torch.int64 and group_offsets.numel() == num_groups + 1
    if ld_t is None:
        ld_t = padded_bound(M, num_groups)
    dev = fc1.device
    q = torch.empty((M, two_f), dtype=FP8, device=dev) if rowwise else None
    s = torch.empty((M, two_f // TILE), dtype=torch.float32, device=dev) if rowwise else None
    q_t = _alloc_qt(two_f, ld_t, blocked, dev)
    s_t = torch.empty((ld_t // TILE, two_f), dtype=torch.float32, device=dev)
    g = torch.empty((M, two_f), dtype=torch.bfloat16, device=dev) if return_grad else None
    ws = torch.empty(num_groups + 1, dtype=torch.int32, device=dev)
    check(
        lib().aamd_swiglu_bwd_quant_1x128_dual_grouped(
            ptr(dh), F, ptr(fc1), two_f, M, F, ptr(group_offsets), num_groups, ptr(ws), ptr(g),
            ptr(q), ptr(s), ptr(q_t), ptr(s_t), ld_t, int(blocked), stream(),
        )
    )  # fmt: skip
    return (q, s, q_t, s_t, g) if return_grad else (q, s, q_t, s_t)


def gelu_tile_quant(x: torch.Tensor, return_activation: bool = False):
    """``h = gelu(x)`` (torch.nn.functional.gelu, the expert MLP's default activation,
    grouped_gemm_moe.py:449) quantised 1x128 along the last dim without writing ``h``.
    Returns ``(q, s)`` or ``(q, s, h)``."""
    assert x.dtype == torch.bfloat16 and x.is_contiguous()
    F = x.size(-1)
    assert F % TILE == 0
    rows = x.numel() // F if F else 0
    dev = x.device
    q = torch.empty(x.shape, dtype=FP8, device=dev)
    s = torch.empty(*x.shape[:-1], F // TILE, dtype=torch.float32, device=dev)
    h = torch.empty(x.shape, dtype=torch.bfloat16, device=dev) if return_activation else None
    check(lib().aamd_gelu_quant_1x128(ptr(x), rows, F, F, ptr(h), ptr(q), ptr(s), stream()))
    return (q, s, h) if return_activation else (q, s)


def gelu_tile_quant_dual_grouped(
    x: torch.Tensor,
    group_offsets: torch.Tensor,
    num_groups: int,
    dh: Optional[torch.Tensor] = None,
    ld_t: Optional[int] = None,
    rowwise: bool = True,
    blocked: bool = False,
    return_activation: bool = False,
):
    """GELU fused into ``tile_quant_dual_grouped``: quantises ``h = gelu(x)`` for ``x [M, F]`` bf16, or,
    with ``dh [M, F]``, the gradient ``g = dh * gelu'(x)`` (what autograd computes for the activation).
    Returns ``(q, s, q_t, s_t)`` (plus ``h`` / ``g`` in bf16 with ``return_activation``)."""
    assert x.dim() == 2 and x.is_contiguous() and x.dtype == torch.bfloat16
    M, F = x.shape
    assert F % TILE == 0
    if dh is not None:
        assert dh.shape == x.shape and dh.is_contiguous() and dh.dtype == torch.bfloat16
    assert group_offsets.dtype == torch.int64 and group_offsets.numel() == num_groups + 1
    if ld_t is None:
        ld_t = padded_bound(M, num_groups)
    dev = x.device
    q = torch.empty((M, F), dtype=FP8, device=dev) if rowwise else None
    s = torch.empty((M, F // TILE), dtype=torch.float32, device=dev) if rowwise else None
    q_t = _alloc_qt(F, ld_t, blocked, dev)
    s_t = torch.empty((ld_t // TILE, F), dtype=torch.float32, device=dev)
    h = torch.empty((M, F), dtype=torch.bfloat16, device=dev) if return_activation else None
    ws = torch.empty(num_groups + 1, dtype=torch.int32, device=dev)
    check(
        lib().aamd_gelu_quant_1x128_dual_grouped(
            ptr(x), ptr(dh), M, F, F, ptr(group_offsets), num_groups, ptr(ws), ptr(h),
            ptr(q), ptr(s), ptr(q_t), ptr(s_t), ld_t, int(blocked), stream(),
        )
    )  # fmt: skip
    return (q, s, q_t, s_t, h) if return_activation else (q, s, q_t, s_t)


def block_quant_batched(w: torch.Tensor, eps: float = 0.0, return_transpose: bool = False):
    """128x128 block quantisation of ``w [E, N, K]`` in one launch.
    Returns ``(q [E,N,K], s [E,N/128,K/128], q_t [E,K,N] | None, s_t [E,K/128,N/128] | None)``."""
    assert w.dim() == 3 and w.stride(2) == 1 and w.stride(1) == w.size(2), "rows of w must be dense"
    E, N, K = w.shape
    dev = w.device
    q = torch.empty((E, N, K), dtype=FP8, device=dev)
    s = torch.empty((E, N // TILE, K // TILE), dtype=torch.float32, device=dev)
    q_t = torch.empty((E, K, N), dtype=FP8, device=dev) if return_transpose else None
    s_t = torch.empty((E, K // TILE, N // TILE), dtype=torch.float32, device=dev) if return_transpose else None
    estride = w.stride(0) if E > 1 else N * K
    check(
        lib().aamd_quant_128x128(
            ptr(w), dtype_code(w.dtype, True), E, N, K, estride, ptr(q), ptr(s), ptr(q_t), ptr(s_t), eps, stream()
        )
    )
    return q, s, q_t, s_t


def grouped_gemm_nt(
    a: torch.Tensor,
    a_s: torch.Tensor,
    b: torch.Tensor,
    b_s: torch.Tensor,
    group_offsets: torch.Tensor,
    out: Optional[torch.Tensor] = None,
    out_dtype=torch.bfloat16,
    bias: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """out[m] = a[m] @ b[g(m)]^T with block scales, for rows m of group g (device offsets).
    a [M,K] fp8, a_s [M,K/128], b [E,N,K] fp8, b_s [E,N/128,K/128] or [E,N,K/128]."""
    M, K = a.shape
    E, N, Kb = b.shape
    assert Kb == K and a.stride(1) == 1 and b.is_contiguous() and a_s.is_contiguous() and b_s.is_contiguous()
    assert group_offsets.dtype == torch.int64 and group_offsets.numel() == E + 1
    if out is None:
        out = torch.empty((M, N), dtype=out_dtype, device=a.device)
    assert out.shape == (M, N) and out.stride(1) == 1
    b_tile_scaled = b_s.size(1) == N
    ws = torch.empty(E + 1, dtype=torch.int32, device=a.device)
    if bias is not None:
        assert bias.shape == (E, N) and bias.is_contiguous()
    args = (ptr(a), a.stride(0), ptr(a_s), ptr(b), ptr(b_s), int(b_tile_scaled), ptr(group_offsets), E, ptr(ws),
            M, N, K, ptr(out), dtype_code(out.dtype), out.stride(0),
            ptr(bias), dtype_code(bias.dtype) if bias is not None else _lib.NONE)  # fmt: skip
    pinned = _pinned_options()
    if pinned:
        from . import _probes

        _probes.check(_probes.lib().aamd_tuning_grouped_gemm_fp8_nt(*args, _probes.options_array(pinned), stream()))
    else:
        check(lib().aamd_grouped_gemm_fp8_nt(*args, stream()))
    return out


def grouped_gemm_wgrad(
    dy_t: torch.Tensor,
    sdy_t: torch.Tensor,
    x_t: torch.Tensor,
    sx_t: torch.Tensor,
    group_offsets: torch.Tensor,
    out: Optional[torch.Tensor] = None,
    out_dtype=torch.float32,
    accumulate: bool = False,
) -> torch.Tensor:
    """dW[g] (+)= dY_g^T X_g from the transposed 1x128-quantised operands of
    ``tile_quant_dual_grouped``: dy_t [N, ld_t], sdy_t [ld_t/128, N], x_t [K, ld_t], sx_t [ld_t/128, K], or
    both code operands blocked, dy_t [ld_t/128, N, 128] and x_t [ld_t/128, K, 128]."""
    blocked = dy_t.dim() == 3
    assert x_t.dim() == dy_t.dim(), "both operands must be in the same layout"
    N, K = (dy_t.shape[1], x_t.shape[1]) if blocked else (dy_t.shape[0], x_t.shape[0])
    ld_t = qt_ld(dy_t)
    E = group_offsets.numel() - 1
    assert qt_ld(x_t) == ld_t and dy_t.is_contiguous() and x_t.is_contiguous()
    assert sdy_t.shape == (ld_t // TILE, N) and sx_t.shape == (ld_t // TILE, K)
    assert sdy_t.is_contiguous() and sx_t.is_contiguous()
    if out is None:
        assert not accumulate
        out = torch.empty((E, N, K), dtype=out_dtype, device=dy_t.device)
    assert out.shape == (E, N, K) and out.stride(2) == 1 and out.stride(1) == K
    ws = torch.empty(E + 1, dtype=torch.int32, device=dy_t.device)
    estride = out.stride(0) if E > 1 else N * K
    args = (ptr(dy_t), ptr(sdy_t), ptr(x_t), ptr(sx_t), ld_t, int(blocked), ptr(group_offsets), E, ptr(ws), N, K,
            ptr(out), dtype_code(out.dtype), estride, int(accumulate))  # fmt: skip
    pinned = _pinned_options()
    if pinned:
        from . import _probes

        _probes.check(_probes.lib().aamd_tuning_grouped_gemm_fp8_wgrad(*args, _probes.options_array(pinned), stream()))
    else:
        check(lib().aamd_grouped_gemm_fp8_wgrad(*args, stream()))
    return out


def moe_preprocess(expert_ids: torch.Tensor, num_experts: int, want_sorted: bool = True):
    """Stable counting sort of the flattened expert ids on the device.
    Returns ``(sorted_indices int64 [n] | None, row_map int32 [n], group_offsets int64 [E+1])``."""
    flat = expert_ids.reshape(-1)
    assert flat.is_contiguous() and flat.dtype in (torch.int64, torch.int32)
    n = flat.numel()
    dev = flat.device
    sorted_idx = torch.empty(n, dtype=torch.int64, device=dev) if want_sorted else None
    row_map = torch.empty(n, dtype=torch.int32, device=dev)
    goff = torch.empty(num_experts + 1, dtype=torch.int64, device=dev)
    ws = torch.empty(max(1, lib().aamd_moe_preprocess_ws_ints(n, num_experts)), dtype=torch.int32, device=dev)
    check(
        lib().aamd_moe_preprocess(
            ptr(flat), int(flat.dtype == torch.int64), n, num_experts, ptr(sorted_idx), ptr(row_map), ptr(goff),
            ptr(ws), stream(),
        )
    )
    return sorted_idx, row_map, goff


def invert_permutation(sorted_indices: torch.Tensor, n_flat: int) -> torch.Tensor:
    si = sorted_indices.to(torch.int64).contiguous()
    row_map = torch.empty(n_flat, dtype=torch.int32, device=si.device)
    check(lib().aamd_invert_permutation(ptr(si), si.numel(), n_flat, ptr(row_map), stream()))
    return row_map


def unpermute_combine(
    y: torch.Tensor, row_map: torch.Tensor, probs: Optional[torch.Tensor], num_tokens: int, topk: int
) -> torch.Tensor:
    """out[t] = sum_j probs[t,j] * y[row_map[t*topk+j]] in one gather-reduce pass (bf16 or fp32 rows;
    the result has the promoted dtype of rows and probs, as the reference's multiply gives it)."""
    assert y.dim() == 2 and y.is_contiguous() and y.dtype in (torch.bfloat16, torch.float32)
    M, H = y.shape
    assert row_map.dtype == torch.int32 and row_map.numel() == num_tokens * topk
    if probs is None:
        pd, out_dtype = _lib.NONE, y.dtype
    else:
        assert probs.shape == (num_tokens, topk)
        probs = probs.contiguous()
        pd = dtype_code(probs.dtype)
        out_dtype = torch.promote_types(y.dtype, probs.dtype)
    out = torch.empty((num_tokens, H), dtype=out_dtype, device=y.device)
    check(
        lib().aamd_unpermute_combine(
            ptr(y), dtype_code(y.dtype), M, H, ptr(row_map), ptr(probs), pd, num_tokens, topk, ptr(out), stream()
        )
    )
    return out


def permute_rows_scaled(
    x: torch.Tensor, row_map: torch.Tensor, topk: int, num_out_rows: int, probs: Optional[torch.Tensor], out_dtype
) -> torch.Tensor:
    """out[row_map[t*topk+j]] = (out_dtype)(x[t] * probs[t, j]): the combine's gradient with respect to
    the permuted rows (rows that no map entry points to are zero)."""
    assert x.dim() == 2 and x.is_contiguous()
    T, cols = x.shape
    assert row_map.dtype == torch.int32 and row_map.numel() == T * topk and row_map.is_contiguous()
    alloc = torch.empty if num_out_rows == T * topk else torch.zeros  # dropped copies leave rows unwritten
    out = alloc((num_out_rows, cols), dtype=out_dtype, device=x.device)
    pd = _lib.NONE if probs is None else dtype_code(probs.dtype)
    if probs is not None:
        probs = probs.contiguous()
    check(
        lib().aamd_permute_rows_scaled(
            ptr(x), dtype_code(x.dtype), T, cols, ptr(row_map), topk, ptr(probs), pd, num_out_rows, ptr(out),
            dtype_code(out_dtype), stream(),
        )
    )  # fmt: skip
    return out


def unpermute_probs_grad(dout: torch.Tensor, y: torch.Tensor, row_map: torch.Tensor, topk: int) -> torch.Tensor:
    """d_probs[t, j] = <dout[t], y[row_map[t*topk+j]]> in fp32."""
    assert dout.dim() == 2 and dout.is_contiguous() and y.dim() == 2 and y.is_contiguous()
    T, H = dout.shape
    assert y.shape[1] == H and row_map.dtype == torch.int32 and row_map.numel() == T * topk
    dp = torch.empty((T, topk), dtype=torch.float32, device=dout.device)
    check(
        lib().aamd_unpermute_probs_grad(
            ptr(dout), dtype_code(dout.dtype), ptr(y), dtype_code(y.dtype), y.shape[0], H, ptr(row_map), T, topk,
            ptr(dp), stream(),
        )
    )  # fmt: skip
    return dp


def split_views(t: torch.Tensor, splits: Sequence[int]) -> List[torch.Tensor]:
    return list(torch.split(t, list(splits)))


_pinned = threading.local()  # launch options pinned by gemm_options on this thread


def _pinned_options() -> Optional[dict]:
    stack = getattr(_pinned, "stack", None)
    return stack[-1] if stack else None


class gemm_options:
    """Context manager for tests and tuning runs: inside it the grouped GEMMs of this thread go through the
    measurement library's entry points (include/atorch_amd_probes.h), which take the launch choices as
    per-call arguments: ``with gemm_options(tile=1): ...``.  Nested uses add to the enclosing one's options
    and restore them on exit; nothing process-wide is changed and the product library is not involved."""

    def __init__(self, **opts):
        from . import _probes

        _probes.options_array(opts)  # validates the names
        self.opts = opts

    def __enter__(self):
        if not hasattr(_pinned, "stack"):
            _pinned.stack = []
        outer = _pinned.stack[-1] if _pinned.stack else {}
        _pinned.stack.append({**outer, **self.opts})
        return self

    def __exit__(self, *exc):
        _pinned.stack.pop()
        return False

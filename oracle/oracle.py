"""CPU oracle for the FP8 grouped-linear MoE expert path (Python side).

TEST INFRASTRUCTURE ONLY.  Nothing under ``atorch_amd/`` may import this
module; it is the checker used by ``tests/``, by the smoke check and by the
CPU-baseline leg of ``bench.py``.

Two independent restatements live here:

* ``c_*`` / the un-prefixed functions call ``libfp8_moe_oracle.so`` (scalar C,
  integer-arithmetic e4m3fn encoder, see ``fp8_moe_oracle.c``);
* ``torch_*`` functions restate the same reference lines with plain torch CPU
  ops, using torch's own ``.to(torch.float8_e4m3fn)`` as the library cast.

The tests require the two to agree bit for bit, which is what pins the C
encoder, and both to reproduce the known answers the reference's own tests
describe.  All paths cited are relative to the reference tree root.
"""
import ctypes
import os
import subprocess
from typing import List, Optional, Sequence, Tuple

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libfp8_moe_oracle.so")
_lib = None

FP8_MAX = 448.0
TILE = 128


def build(force: bool = False) -> str:
    """Compile the C oracle with gcc (a few hundred ms)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        i64, f32, vp, ci = ctypes.c_int64, ctypes.c_float, ctypes.c_void_p, ctypes.c_int
        L.oracle_f32_to_e4m3fn_array.argtypes = [vp, i64, vp]
        L.oracle_e4m3fn_to_f32_array.argtypes = [vp, i64, vp]
        L.oracle_bf16_to_f32_array.argtypes = [vp, i64, vp]
        L.oracle_f32_to_bf16_array.argtypes = [vp, i64, vp]
        L.oracle_tile_quant.argtypes = [vp, i64, i64, f32, vp, vp]
        L.oracle_block_quant.argtypes = [vp, i64, i64, f32, vp, vp]
        L.oracle_tile_quant_t_grouped.argtypes = [vp, i64, i64, vp, i64, f32, vp, vp, i64]
        L.oracle_fp8_gemm.argtypes = [vp, i64, vp, i64, i64, vp, i64, vp, i64, i64, i64, i64, i64, i64, vp, i64, ci]
        L.oracle_permute_indices.argtypes = [vp, i64, i64, vp, vp]
        L.oracle_unpermute_combine.argtypes = [vp, i64, i64, vp, vp, ci, i64, i64, vp, vp]
        L.oracle_swiglu_bf16.argtypes = [vp, i64, i64, i64, vp]
        L.oracle_swiglu_bwd_bf16.argtypes = [vp, vp, i64, i64, i64, vp]
        L.oracle_bias_gather_add.argtypes = [vp, vp, vp, i64, i64, ci, ci, vp]
        L.oracle_bias_gather_bgrad.argtypes = [vp, vp, i64, i64, ci, ci, vp]
        for name in (
            "oracle_tile_quant",
            "oracle_block_quant",
            "oracle_tile_quant_t_grouped",
            "oracle_fp8_gemm",
            "oracle_permute_indices",
            "oracle_unpermute_combine",
        ):
            getattr(L, name).restype = ci
        _lib = L
    return _lib


def _p(t: torch.Tensor) -> int:
    assert t.device.type == "cpu" and t.is_contiguous()
    return t.data_ptr()


def _chk(rc: int, what: str):
    if rc != 0:
        raise ValueError(f"oracle {what} failed with status {rc}")


def _f32c(x: torch.Tensor) -> torch.Tensor:
    # the reference kernels cast their input to fp32 first (triton_kernel.py:30,105)
    return x.detach().to("cpu", torch.float32).contiguous()


def as_fp8(codes_u8: torch.Tensor) -> torch.Tensor:
    return codes_u8.view(torch.float8_e4m3fn)


def as_u8(t: torch.Tensor) -> torch.Tensor:
    return t.view(torch.uint8) if t.dtype != torch.uint8 else t


# ----------------------------------------------------------------------------
# C oracle wrappers
# ----------------------------------------------------------------------------
def f32_to_e4m3fn(x: torch.Tensor) -> torch.Tensor:
    x = _f32c(x)
    out = torch.empty(x.shape, dtype=torch.uint8)
    lib().oracle_f32_to_e4m3fn_array(_p(x), x.numel(), _p(out))
    return out


def e4m3fn_to_f32(c: torch.Tensor) -> torch.Tensor:
    c = as_u8(c).contiguous()
    out = torch.empty(c.shape, dtype=torch.float32)
    lib().oracle_e4m3fn_to_f32_array(_p(c), c.numel(), _p(out))
    return out


def f32_to_bf16(x: torch.Tensor) -> torch.Tensor:
    x = _f32c(x)
    out = torch.empty(x.shape, dtype=torch.int16)
    lib().oracle_f32_to_bf16_array(_p(x), x.numel(), _p(out))
    return out.view(torch.bfloat16)


def tile_quant(x: torch.Tensor, eps: float = 0.0) -> Tuple[torch.Tensor, torch.Tensor]:
    """triton_kernel.py:94-140.  Returns (codes uint8 same shape, scales fp32 [..., K/128])."""
    xf = _f32c(x)
    cols = xf.shape[-1]
    rows = xf.numel() // cols if cols else 0
    q = torch.empty(xf.shape, dtype=torch.uint8)
    s = torch.empty(*xf.shape[:-1], cols // TILE, dtype=torch.float32)
    _chk(lib().oracle_tile_quant(_p(xf), rows, cols, eps, _p(q), _p(s)), "tile_quant")
    return q, s


def block_quant(x: torch.Tensor, eps: float = 0.0) -> Tuple[torch.Tensor, torch.Tensor]:
    """triton_kernel.py:21-46.  x [N, K]; returns (codes [N,K] uint8, scales [N/128, K/128])."""
    xf = _f32c(x)
    assert xf.dim() == 2
    N, K = xf.shape
    q = torch.empty((N, K), dtype=torch.uint8)
    s = torch.empty((N // TILE, K // TILE), dtype=torch.float32)
    _chk(lib().oracle_block_quant(_p(xf), N, K, eps, _p(q), _p(s)), "block_quant")
    return q, s


def padded_offsets(splits: Sequence[int]) -> List[int]:
    po = [0]
    for m in splits:
        po.append(po[-1] + (int(m) + TILE - 1) // TILE * TILE)
    return po


def tile_quant_t_grouped(
    x: torch.Tensor, splits: Sequence[int], eps: float = 0.0, ld_t: Optional[int] = None
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Transposed 1x128 quantisation along the token dim inside each ragged group
    (scaled_linear.py:402-414 applied per group, zero padded partial tiles).

    Returns q_t [R, ld_t] uint8 (columns beyond the padded total stay 0) and
    s_t [ld_t/128, R] fp32 (rows beyond the padded total stay 1).
    """
    xf = _f32c(x)
    M, R = xf.shape
    po = padded_offsets(splits)
    if ld_t is None:
        ld_t = max(po[-1], TILE)
    q_t = torch.zeros((R, ld_t), dtype=torch.uint8)
    s_t = torch.ones((ld_t // TILE, R), dtype=torch.float32)
    sp = torch.tensor(list(splits), dtype=torch.int64)
    _chk(
        lib().oracle_tile_quant_t_grouped(_p(xf), M, R, _p(sp), len(splits), eps, _p(q_t), _p(s_t), ld_t),
        "tile_quant_t_grouped",
    )
    return q_t, s_t


def swiglu(fc1: torch.Tensor) -> torch.Tensor:
    """grouped_gemm_moe.py:331-334 on bf16 rows [a | b]: bf16(bf16(silu(a)) * b)."""
    assert fc1.dtype == torch.bfloat16 and fc1.dim() == 2
    x = fc1.contiguous().view(torch.int16)
    rows, two_f = x.shape
    h = torch.empty((rows, two_f // 2), dtype=torch.int16)
    _chk(lib().oracle_swiglu_bf16(_p(x), rows, two_f // 2, two_f, _p(h)), "swiglu")
    return h.view(torch.bfloat16)


def swiglu_bwd(dh: torch.Tensor, fc1: torch.Tensor) -> torch.Tensor:
    """Gradient of ``swiglu`` w.r.t. ``fc1`` for the output gradient ``dh`` (bf16): rows ``[da | db]``."""
    assert fc1.dtype == torch.bfloat16 and dh.dtype == torch.bfloat16 and fc1.dim() == 2
    x = fc1.contiguous().view(torch.int16)
    d = dh.contiguous().view(torch.int16)
    rows, two_f = x.shape
    assert d.shape == (rows, two_f // 2)
    out = torch.empty((rows, two_f), dtype=torch.int16)
    _chk(lib().oracle_swiglu_bwd_bf16(_p(d), _p(x), rows, two_f // 2, two_f, _p(out)), "swiglu_bwd")
    return out.view(torch.bfloat16)


def bias_gather_add(inp: torch.Tensor, bias: torch.Tensor, bin_ids: torch.Tensor) -> torch.Tensor:
    """bias_gather_add.py:50-66: ``inp + bias[bin_ids]`` in the tensors' dtype (bf16 or fp32)."""
    assert inp.dtype == bias.dtype and inp.dtype in (torch.bfloat16, torch.float32)
    bf = inp.dtype == torch.bfloat16
    a = inp.contiguous().view(torch.int16) if bf else inp.contiguous()
    b = bias.contiguous().view(torch.int16) if bf else bias.contiguous()
    ids = bin_ids.to(torch.int64).contiguous()
    out = torch.empty_like(a)
    T, H = a.shape
    _chk(lib().oracle_bias_gather_add(_p(a), _p(b), _p(ids), T, H, bias.shape[0], int(bf), _p(out)), "bias_gather_add")
    return out.view(torch.bfloat16) if bf else out


def bias_gather_bgrad(grad: torch.Tensor, bin_ids: torch.Tensor, num_experts: int) -> torch.Tensor:
    """bias_gather_add.py:101-127: fp32 sums of the rows of each expert (row order), ``[E, H]`` fp32."""
    bf = grad.dtype == torch.bfloat16
    g = grad.contiguous().view(torch.int16) if bf else grad.contiguous()
    ids = bin_ids.to(torch.int64).contiguous()
    T, H = g.shape
    out = torch.empty((num_experts, H), dtype=torch.float32)
    _chk(lib().oracle_bias_gather_bgrad(_p(g), _p(ids), T, H, num_experts, int(bf), _p(out)), "bias_gather_bgrad")
    return out


def gelu(x: torch.Tensor) -> torch.Tensor:
    """The expert MLP's default activation, ``torch.nn.functional.gelu`` (grouped_gemm_moe.py:449, applied
    at :849), on a bf16 tensor: the reference's own op evaluated on the CPU (fp32 inside, one rounding)."""
    assert x.dtype == torch.bfloat16
    return torch.nn.functional.gelu(x.detach())


def gelu_bwd(dh: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
    """What autograd runs for that op: ``dh * (cdf(x) + x * pdf(x))`` in fp32, rounded to bf16."""
    assert x.dtype == torch.bfloat16 and dh.dtype == torch.bfloat16
    leaf = x.detach().clone().requires_grad_(True)
    torch.nn.functional.gelu(leaf).backward(dh)
    return leaf.grad


def torch_swiglu(fc1: torch.Tensor) -> torch.Tensor:
    """The reference's own two torch ops (CPU)."""
    a, b = torch.chunk(fc1, 2, dim=-1)
    return torch.nn.functional.silu(a) * b


def dequant(q: torch.Tensor, s: torch.Tensor) -> torch.Tensor:
    """triton_kernel.py:49-91: tile scales if s.size(0)==q.size(0) (:85) else block scales."""
    v = e4m3fn_to_f32(q)
    M, N = v.shape
    if s.shape[0] == M:
        return v * s.repeat_interleave(TILE, 1)[:, :N]
    return v * s.repeat_interleave(TILE, 0)[:M].repeat_interleave(TILE, 1)[:, :N]


def fp8_gemm(
    a: torch.Tensor,
    a_s: torch.Tensor,
    b: torch.Tensor,
    b_s: torch.Tensor,
    out: Optional[torch.Tensor] = None,
    accumulate: bool = False,
) -> torch.Tensor:
    """triton_kernel.py:151-210 blockwise accumulate, fp32 result (no output cast).
    a [M,K] codes, a_s [M,K/128]; b [N,K] codes, b_s [N/128,K/128] (block) or [N,K/128] (tile)."""
    a, b = as_u8(a), as_u8(b)
    M, K = a.shape
    N = b.shape[0]
    assert b.shape[1] == K
    b_div = 1 if b_s.shape[0] == N else TILE  # :205,208
    if K == 0 or M == 0 or N == 0:
        c = torch.zeros((M, N), dtype=torch.float32)
        return c if out is None or not accumulate else out
    if out is None:
        out = torch.zeros((M, N), dtype=torch.float32)
        accumulate = False
    assert out.dtype == torch.float32 and out.is_contiguous()
    a_s, b_s = a_s.float(), b_s.float()
    _chk(
        lib().oracle_fp8_gemm(
            a.data_ptr(), a.stride(0), a_s.data_ptr(), a_s.stride(0), a_s.stride(1),
            b.data_ptr(), b.stride(0), b_s.data_ptr(), b_s.stride(0), b_s.stride(1),
            b_div, M, N, K, _p(out), out.stride(0), int(accumulate),
        ),
        "fp8_gemm",
    )  # fmt: skip
    return out


def grouped_gemm_nt(
    qa: torch.Tensor, sa: torch.Tensor, qb: torch.Tensor, sb: torch.Tensor, splits: Sequence[int]
) -> torch.Tensor:
    """E independent block-scaled GEMMs over ragged row splits (the fwd / dgrad
    grouped_qgemm of quantized_grouped_linear.py:141-151, 214-223).
    qa [M,K], sa [M,K/128], qb [E,N,K], sb [E,N/128,K/128] -> fp32 [M,N]."""
    M, K = qa.shape
    E, N, _ = qb.shape
    out = torch.zeros((M, N), dtype=torch.float32)
    off = 0
    for e, m in enumerate(splits):
        if m:
            out[off : off + m] = fp8_gemm(
                as_u8(qa)[off : off + m], sa[off : off + m].contiguous(), as_u8(qb)[e], sb[e].contiguous()
            )
        off += m
    return out


def grouped_gemm_wgrad(
    qdy_t: torch.Tensor,
    sdy_t: torch.Tensor,
    qx_t: torch.Tensor,
    sx_t: torch.Tensor,
    splits: Sequence[int],
    out: Optional[torch.Tensor] = None,
    accumulate: bool = False,
) -> torch.Tensor:
    """wgrad grouped_qgemm (quantized_grouped_linear.py:243-253): dW_i = dY_i^T X_i with both
    operands 1x128-scaled along the tokens of group i.  Layouts as tile_quant_t_grouped:
    qdy_t [N, ld], sdy_t [ld/128, N], qx_t [K, ld], sx_t [ld/128, K] -> fp32 [E, N, K].
    An empty group gives zeros (or leaves ``out`` untouched when accumulating)."""
    N, K = qdy_t.shape[0], qx_t.shape[0]
    E = len(splits)
    po = padded_offsets(splits)
    if out is None:
        out = torch.zeros((E, N, K), dtype=torch.float32)
        accumulate = False
    for e in range(E):
        p0, p1 = po[e], po[e + 1]
        if p1 == p0:
            if not accumulate:
                out[e].zero_()
            continue
        a = as_u8(qdy_t)[:, p0:p1]
        b = as_u8(qx_t)[:, p0:p1]
        a_s = sdy_t[p0 // TILE : p1 // TILE].t()  # [N, nb] strided view
        b_s = sx_t[p0 // TILE : p1 // TILE].t()  # [K, nb]
        c = out[e]
        _chk(
            lib().oracle_fp8_gemm(
                a.data_ptr(), a.stride(0), a_s.data_ptr(), a_s.stride(0), a_s.stride(1),
                b.data_ptr(), b.stride(0), b_s.data_ptr(), b_s.stride(0), b_s.stride(1),
                1, N, K, p1 - p0, c.data_ptr(), c.stride(0), int(accumulate),
            ),
            "fp8_gemm(wgrad)",
        )  # fmt: skip
    return out


def permute_indices(indices: torch.Tensor, num_experts: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """token_dispatcher.py:107-112 (+ histc :310): returns (sorted_indices [T*k] int64, counts [E] int64)."""
    flat = indices.reshape(-1).to(torch.int64).contiguous()
    sorted_idx = torch.empty_like(flat)
    counts = torch.empty(num_experts, dtype=torch.int64)
    _chk(lib().oracle_permute_indices(_p(flat), flat.numel(), num_experts, _p(sorted_idx), _p(counts)), "permute")
    return sorted_idx, counts


def permute(tokens: torch.Tensor, indices: torch.Tensor, num_experts: int):
    """token_dispatcher.py:89-116."""
    topk = 1 if indices.dim() == 1 else indices.size(1)
    sorted_idx, counts = permute_indices(indices, num_experts)
    return tokens.index_select(0, sorted_idx // topk), sorted_idx, counts


def unpermute(permuted: torch.Tensor, sorted_idx: torch.Tensor, probs: Optional[torch.Tensor] = None) -> torch.Tensor:
    """token_dispatcher.py:119-161 for bf16 rows; probs bf16 -> bf16 out, probs fp32 -> fp32 out."""
    assert permuted.dtype == torch.bfloat16
    y = permuted.contiguous().view(torch.int16)
    n_perm, H = y.shape
    si = sorted_idx.to(torch.int64).contiguous()
    if probs is None:
        T, k = n_perm, 1
        out = torch.empty((T, H), dtype=torch.int16)
        _chk(lib().oracle_unpermute_combine(_p(y), n_perm, H, _p(si), None, 1, T, k, _p(out), None), "unpermute")
        return out.view(torch.bfloat16)
    T, k = probs.shape
    if probs.dtype == torch.bfloat16:
        pr = probs.contiguous().view(torch.int16)
        out = torch.empty((T, H), dtype=torch.int16)
        _chk(lib().oracle_unpermute_combine(_p(y), n_perm, H, _p(si), _p(pr), 1, T, k, _p(out), None), "unpermute")
        return out.view(torch.bfloat16)
    pr = probs.float().contiguous()
    out = torch.empty((T, H), dtype=torch.float32)
    _chk(lib().oracle_unpermute_combine(_p(y), n_perm, H, _p(si), _p(pr), 0, T, k, None, _p(out)), "unpermute")
    return out


def grouped_linear_fwd_bwd(
    x: torch.Tensor,
    weights: Sequence[torch.Tensor],
    m_splits: Sequence[int],
    dy: Optional[torch.Tensor] = None,
    biases: Optional[Sequence[torch.Tensor]] = None,
    eps: float = 0.0,
):
    """quantized_grouped_linear.py:53-270 with the 1x128 / 128x128 e4m3fn recipe
    (tests/common_tests/fp8/test_quantized_grouped_linear.py:164-175).
    Returns dict(out, dgrad, wgrad[list], bgrad[list]) as fp32 (callers round to the output dtype)."""
    K = x.shape[-1]
    x2 = x.reshape(-1, K)
    E = len(m_splits)
    N = weights[0].shape[0]
    qx, sx = tile_quant(x2, eps)
    qw = torch.stack([block_quant(w, eps)[0] for w in weights])
    sw = torch.stack([block_quant(w, eps)[1] for w in weights])
    out = grouped_gemm_nt(qx, sx, qw, sw, m_splits)
    if biases is not None:
        off = 0
        for e, m in enumerate(m_splits):
            out[off : off + m] += biases[e].float()
            off += m
    res = {"out": out}
    if dy is None:
        return res
    dy2 = dy.reshape(-1, N)
    qdy, sdy = tile_quant(dy2, eps)
    # W^T block quant == transpose of codes and of the scale grid (scaled_linear.py:359-365)
    qw_t = qw.transpose(1, 2).contiguous()
    sw_t = sw.transpose(1, 2).contiguous()
    res["dgrad"] = grouped_gemm_nt(qdy, sdy, qw_t, sw_t, m_splits)
    qdy_t, sdy_t = tile_quant_t_grouped(dy2, m_splits, eps)
    qx_t, sx_t = tile_quant_t_grouped(x2, m_splits, eps)
    wg = grouped_gemm_wgrad(qdy_t, sdy_t, qx_t, sx_t, m_splits)
    res["wgrad"] = [wg[e] for e in range(E)]
    off = 0
    bg = []
    for m in m_splits:
        bg.append(dy2[off : off + m].float().sum(0))  # :201
        off += m
    res["bgrad"] = bg
    return res


# ----------------------------------------------------------------------------
# torch restatements (independent of the C code; also the CPU baseline that
# bench.py times: "dequantize + per-expert matmul")
# ----------------------------------------------------------------------------
def torch_tile_quant(x: torch.Tensor, eps: float = 0.0):
    """triton_kernel.py:103-124 with torch CPU ops."""
    xf = x.float()
    shp = xf.shape
    t = xf.reshape(-1, TILE)
    amax = t.abs().amax(dim=1, keepdim=True)
    s = torch.clamp(amax, min=eps) / FP8_MAX
    s = torch.where(s == 0, torch.ones_like(s), s)
    q = (t / s).to(torch.float8_e4m3fn)
    return q.view(shp).view(torch.uint8), s.view(*shp[:-1], shp[-1] // TILE)


def torch_block_quant(x: torch.Tensor, eps: float = 0.0):
    """triton_kernel.py:21-37 with torch CPU ops."""
    xf = x.float()
    N, K = xf.shape
    b = xf.view(N // TILE, TILE, K // TILE, TILE)
    amax = b.abs().amax(dim=(1, 3), keepdim=True)
    s = torch.clamp(amax, min=eps) / FP8_MAX
    s = torch.where(s == 0, torch.ones_like(s), s)
    q = (b / s).to(torch.float8_e4m3fn).view(N, K)
    return q.view(torch.uint8), s.view(N // TILE, K // TILE)


def torch_dequant_tile(q: torch.Tensor, s: torch.Tensor) -> torch.Tensor:
    return as_fp8(as_u8(q)).float() * s.repeat_interleave(TILE, -1)


def torch_dequant_block(q: torch.Tensor, s: torch.Tensor) -> torch.Tensor:
    return as_fp8(as_u8(q)).float() * s.repeat_interleave(TILE, -2).repeat_interleave(TILE, -1)


def torch_grouped_gemm_dequant(qa, sa, qb, sb, splits, out_dtype=torch.bfloat16) -> torch.Tensor:
    """The reference's PyTorch CPU path: dequantize + per-expert matmul."""
    M = qa.shape[0]
    N = qb.shape[1]
    out = torch.zeros((M, N), dtype=out_dtype)
    off = 0
    for e, m in enumerate(splits):
        if m:
            a = torch_dequant_tile(qa[off : off + m], sa[off : off + m])
            b = torch_dequant_block(qb[e], sb[e])
            out[off : off + m] = (a @ b.t()).to(out_dtype)
        off += m
    return out


def torch_permute(tokens: torch.Tensor, indices: torch.Tensor):
    """token_dispatcher.py:89-116 restated."""
    topk = 1 if indices.dim() == 1 else indices.size(1)
    sorted_indices = torch.argsort(indices.reshape(-1), stable=True)
    return tokens.index_select(0, sorted_indices // topk), sorted_indices


def torch_unpermute(permuted: torch.Tensor, sorted_indices: torch.Tensor, probs: Optional[torch.Tensor] = None):
    """token_dispatcher.py:119-161 restated."""
    if probs is not None:
        n, topk = probs.numel(), probs.size(1)
    else:
        n, topk = permuted.size(0), 1
    buf = torch.zeros([n, permuted.shape[-1]], dtype=permuted.dtype)
    buf.index_copy_(0, sorted_indices, permuted)
    buf = buf.reshape(-1, topk, permuted.size(-1))
    if probs is not None:
        buf = buf * probs.unsqueeze(-1)
    return buf.sum(dim=1)


# ----------------------------------------------------------------------------
# exact rational e4m3fn rounder (slow, for pinning the encoders on small sets)
# ----------------------------------------------------------------------------
def exact_e4m3fn_code(value: float) -> int:
    """Round a finite python float to e4m3fn with exact rational arithmetic
    (nearest representable value, ties to the even code, NaN above the 448/480 midpoint)."""
    from fractions import Fraction

    if value != value or value in (float("inf"), float("-inf")):
        return 0x7F | (0x80 if str(value).startswith("-") else 0)
    neg = np.signbit(value)
    v = abs(Fraction(value))
    # all non-negative finite codes and their values
    vals = []
    for c in range(0x7F):
        e, m = c >> 3, c & 7
        vals.append(Fraction(m, 512) if e == 0 else Fraction(8 + m, 8) * Fraction(2) ** (e - 7))
    best = None
    for c in range(0x7F):
        d = abs(vals[c] - v)
        if best is None or d < best[0] or (d == best[0] and c % 2 == 0 and best[1] % 2 == 1):
            best = (d, c)
    code = best[1]
    if code == 0x7E:
        # beyond the midpoint to the next (non-existent) value 480 -> NaN; the tie goes to 448 (even)
        if v - vals[0x7E] > Fraction(16):
            code = 0x7F
    return code | (0x80 if neg else 0)

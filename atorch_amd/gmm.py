"""``gmm(a, b, batch_sizes, trans_b)`` on the fp8 grouped GEMM.

Same call shape as the grouped-GEMM binding the reference's MoE layer uses
(atorch/kernels/extensions/grouped_gemm_exts/grouped_gemm_gmm.py:10-52, called from
atorch/modules/moe/grouped_gemm_moe.py:841-850): ``a [M, K]``, ``b [E, K, N]`` (or ``[E, N, K]``
with ``trans_b``), ``batch_sizes`` int64 ``[E]`` rows per expert -> ``[M, N]``.  Operands are
quantised on the fly (1x128 for ``a`` and the incoming gradient, 128x128 for ``b``) and the
three GEMMs of forward and backward run on the grouped fp8 kernels.
"""
from typing import Optional

import torch

from . import kernels
from .quantization import WeightCodeCache

TILE = kernels.TILE


def _offsets(batch_sizes: torch.Tensor, device) -> torch.Tensor:
    """Exclusive prefix [E+1] on the device; computed where ``batch_sizes`` lives (the reference
    passes a CPU tensor, grouped_gemm_moe.py:837), so a device tensor costs no host round trip."""
    bs = batch_sizes.to(torch.int64)
    off = torch.zeros(bs.numel() + 1, dtype=torch.int64, device=bs.device)
    off[1:] = torch.cumsum(bs, 0)
    return off.to(device)


class _Fp8Gmm(torch.autograd.Function):
    @staticmethod
    def forward(ctx, a, b, batch_sizes, trans_b, is_first_microbatch, weight_cache):
        assert a.dim() == 2 and b.dim() == 3
        E = b.shape[0]
        goff = _offsets(batch_sizes, a.device)
        need_grad = any(ctx.needs_input_grad[:2])  # all False under no_grad
        # weight as [E, N, K]: block quantisation commutes with the transpose, so for
        # trans_b == False the transposed output of the quantiser is the [N, K] operand.
        # Under no_grad only the orientation the forward GEMM reads is needed when that is the stored one.
        both = need_grad or not trans_b
        quantise = lambda t: kernels.block_quant_batched(b.detach().contiguous(), return_transpose=t)  # noqa: E731
        if weight_cache is None:
            qb, sb, qb_t, sb_t = quantise(both)
        else:
            qb, sb, qb_t, sb_t = weight_cache.codes("b", (b,), is_first_microbatch, both, quantise)
        if trans_b:
            w_q, w_s, wt_q, wt_s = qb, sb, qb_t, sb_t
        else:
            w_q, w_s, wt_q, wt_s = qb_t, sb_t, qb, sb
        a_c = a.detach().contiguous()
        if need_grad:
            qa, sa, qa_t, sa_t = kernels.tile_quant_dual_grouped(a_c, goff, E, blocked=True)
        else:
            qa, sa = kernels.tile_quant(a_c)
            qa_t = sa_t = None
        out = kernels.grouped_gemm_nt(qa, sa, w_q, w_s, goff, out_dtype=a.dtype)
        ctx.trans_b = trans_b
        ctx.b_dtype = b.dtype
        if need_grad:
            ctx.save_for_backward(goff, wt_q, wt_s, qa_t, sa_t)
        return out

    @staticmethod
    def backward(ctx, dy):
        goff, wt_q, wt_s, qa_t, sa_t = ctx.saved_tensors
        E = goff.numel() - 1
        dy = dy.contiguous()
        qdy, sdy, qdy_t, sdy_t = kernels.tile_quant_dual_grouped(dy, goff, E, ld_t=kernels.qt_ld(qa_t), blocked=True)
        da = kernels.grouped_gemm_nt(qdy, sdy, wt_q, wt_s, goff, out_dtype=dy.dtype)
        # dW[g] = dY_g^T A_g -> [E, N, K]; for trans_b == False the parameter is [E, K, N]
        if ctx.trans_b:
            db = kernels.grouped_gemm_wgrad(qdy_t, sdy_t, qa_t, sa_t, goff, out_dtype=ctx.b_dtype)
        else:
            db = kernels.grouped_gemm_wgrad(qa_t, sa_t, qdy_t, sdy_t, goff, out_dtype=ctx.b_dtype)
        return da, db, None, None, None, None


def gmm(a: torch.Tensor, b: torch.Tensor, batch_sizes: torch.Tensor, trans_b: bool = False, *,
        is_first_microbatch: Optional[bool] = None, weight_cache: Optional[WeightCodeCache] = None) -> torch.Tensor:
    """``is_first_microbatch`` / ``weight_cache`` (not in the reference's binding): with a ``WeightCodeCache`` the
    codes of ``b`` are kept between the microbatches of a step under the grouped linear's rule
    (quantized_grouped_linear.py:103-134); without one ``b`` is quantised in every call."""
    if torch.is_autocast_enabled():
        dt = torch.get_autocast_gpu_dtype()
        a, b = a.to(dt), b.to(dt)
    return _Fp8Gmm.apply(a, b, batch_sizes, trans_b, is_first_microbatch, weight_cache)

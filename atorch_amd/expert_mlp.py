"""The expert MLP of an MoE layer on the fp8 grouped kernels, SwiGLU fused into the quantiser.

Mirrors the body of ``Grouped_GEMM_MoE.compute_moe`` for the merged gate/up weight with SwiGLU
(atorch/modules/moe/grouped_gemm_moe.py:836-855 with ``use_swiglu`` and ``merge_w1_v1``):

    fc1 = gmm(hidden_states, w1, tokens_per_expert, trans_b=transpose_w1)   # [M, 2F]
    intermediate = F.silu(fc1[:, :F]) * fc1[:, F:]                           # :331-334
    fc2 = gmm(intermediate, w2, tokens_per_expert, trans_b=False)           # [M, H]

with weights ``w1 [E, 2F, H]`` (``transpose_w1=True``, the default) or ``[E, H, 2F]`` and
``w2 [E, F, H]`` (:473-488).  The intermediate activation never exists in memory on the way
forward: the first GEMM's output is read once by a kernel that applies SwiGLU and writes the fp8
codes and scales the second GEMM (and, under autograd, its weight-gradient GEMM) consume.

Backward: the gradient through SwiGLU is computed from the saved first-GEMM output by the kernel
that quantises it (same fusion, autograd's bf16 arithmetic), and the four gradient GEMMs run on
the fp8 kernels.
"""
import torch

from . import kernels
from .gmm import _offsets


class _Fp8SwigluMlp(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, w1, w2, batch_sizes, transpose_w1):
        assert x.dim() == 2 and w1.dim() == 3 and w2.dim() == 3
        E = w1.shape[0]
        goff = _offsets(batch_sizes, x.device)
        train = x.requires_grad or w1.requires_grad or w2.requires_grad
        # first weight as [E, 2F, H] (rows = outputs), second as [E, H, F]: block quantisation
        # commutes with the transpose, so both orientations come out of one launch each
        q1, s1, q1_t, s1_t = kernels.block_quant_batched(w1.detach().contiguous(), return_transpose=True)
        if not transpose_w1:
            q1, s1, q1_t, s1_t = q1_t, s1_t, q1, s1
        q2, s2, q2_t, s2_t = kernels.block_quant_batched(w2.detach().contiguous(), return_transpose=True)
        xc = x.detach().contiguous()
        if train:
            qx, sx, qx_t, sx_t = kernels.tile_quant_dual_grouped(xc, goff, E)
        else:
            qx, sx = kernels.tile_quant(xc)
        fc1 = kernels.grouped_gemm_nt(qx, sx, q1, s1, goff, out_dtype=torch.bfloat16)
        if train:
            qh, sh, qh_t, sh_t = kernels.swiglu_tile_quant_dual_grouped(fc1, goff, E)
        else:
            qh, sh = kernels.swiglu_tile_quant(fc1)
        out = kernels.grouped_gemm_nt(qh, sh, q2_t, s2_t, goff, out_dtype=x.dtype)
        if train:
            ctx.transpose_w1 = transpose_w1
            ctx.dtypes = (x.dtype, w1.dtype, w2.dtype)
            ctx.save_for_backward(goff, fc1, qx_t, sx_t, qh_t, sh_t, q1_t, s1_t, q2, s2)
        return out

    @staticmethod
    def backward(ctx, dy):
        goff, fc1, qx_t, sx_t, qh_t, sh_t, q1_t, s1_t, q2, s2 = ctx.saved_tensors
        E = goff.numel() - 1
        x_dtype, w1_dtype, w2_dtype = ctx.dtypes
        dy = dy.contiguous().to(torch.bfloat16)
        qdy, sdy, qdy_t, sdy_t = kernels.tile_quant_dual_grouped(dy, goff, E)
        # through the second linear: dh = dy @ w2^T ([M, F]); dw2[f, h] = sum_m h[m, f] dy[m, h]
        dh = kernels.grouped_gemm_nt(qdy, sdy, q2, s2, goff, out_dtype=torch.bfloat16)
        dw2 = kernels.grouped_gemm_wgrad(qh_t, sh_t, qdy_t, sdy_t, goff, out_dtype=w2_dtype)
        # through SwiGLU: [da | db] is quantised by the kernel that computes it and never written
        qg, sg, qg_t, sg_t = kernels.swiglu_bwd_tile_quant_dual_grouped(dh, fc1, goff, E)
        # through the first linear: dx = dfc1 @ w1 ([M, H]); dw1[n, h] = sum_m dfc1[m, n] x[m, h]
        dx = kernels.grouped_gemm_nt(qg, sg, q1_t, s1_t, goff, out_dtype=x_dtype)
        if ctx.transpose_w1:
            dw1 = kernels.grouped_gemm_wgrad(qg_t, sg_t, qx_t, sx_t, goff, out_dtype=w1_dtype)
        else:
            dw1 = kernels.grouped_gemm_wgrad(qx_t, sx_t, qg_t, sg_t, goff, out_dtype=w1_dtype)
        return dx, dw1, dw2, None, None


def grouped_mlp_swiglu(hidden_states: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor,
                       tokens_per_expert: torch.Tensor, transpose_w1: bool = True) -> torch.Tensor:
    """``gmm -> SwiGLU -> gmm`` of an expert MLP on already permuted tokens.

    ``hidden_states [M, H]`` bf16 rows grouped by expert, ``tokens_per_expert`` int64 ``[E]`` (CPU or
    device), ``w1 [E, 2F, H]`` (or ``[E, H, 2F]`` with ``transpose_w1=False``), ``w2 [E, F, H]``;
    H and F multiples of 128.  Returns ``[M, H]``."""
    assert hidden_states.dtype == torch.bfloat16, "the fused SwiGLU kernel reads bf16"
    return _Fp8SwigluMlp.apply(hidden_states, w1, w2, tokens_per_expert, transpose_w1)

"""The expert MLP of an MoE layer on the fp8 grouped kernels, the activation fused into the quantiser.

Mirrors every body of ``Grouped_GEMM_MoE.compute_moe`` (atorch/modules/moe/grouped_gemm_moe.py:836-855):

    merged SwiGLU      fc1 = gmm(x, w1 [E, 2F, H]);  h = F.silu(fc1[:, :F]) * fc1[:, F:]          # :845-849, :331-334
    separate SwiGLU    x1 = gmm(x, w1 [E, F, H]);  x2 = gmm(x, v1 [E, F, H]);  h = F.silu(x1) * x2   # :840-843
    GELU (default)     fc1 = gmm(x, w1 [E, F, H]);  h = F.gelu(fc1)                                  # :449, :849
    use_bias           fc1 = bias_gather_add(fc1, b1, bin_ids) before the activation, and           # :846-848
                       fc2 = bias_gather_add(gmm(h, w2), b2, bin_ids)                               # :850-853

with ``trans_b=transpose_w1`` for the first weight(s) (``[E, H, *]`` when False) and ``w2 [E, F, H]``
(:473-488).  The intermediate activation never exists in memory on the way forward: the first GEMM's
output is read once by a kernel that applies the activation and writes the fp8 codes and scales the
second GEMM (and, under autograd, its weight-gradient GEMM) consume.  Rows are grouped by expert, so
the per-expert bias of ``bias_gather_add`` is the bias epilogue of the grouped GEMM (added to the fp32
accumulator, one rounding instead of the reference's two).  Separate gate / up weights are quantised
separately and their codes laid side by side, which makes the rest the merged case.

Backward: the gradient through the activation is computed from the saved first-GEMM output by the
kernel that quantises it (same fusion, autograd's bf16 arithmetic), and the four gradient GEMMs run
on the fp8 kernels; bias gradients are per-expert fp32 row sums.

Fused dispatch: with a ``TokenDispatch`` the hidden states come in token order and the permute of
atorch/modules/moe/token_dispatcher.py:89-116 happens inside the quantiser of the first GEMM's operand
(each permuted row is quantised straight from its token's row); the gradient of the hidden states goes
back to token order through the sum over the top-k copies that ``index_select``'s backward makes there.
The permuted bf16 rows are then neither written nor read, forward or backward.
"""
from typing import NamedTuple, Optional

import torch

from . import kernels
from .bias_gather_add import bias_gather_add_bw
from .gmm import _offsets
from .quantization import WeightCodeCache


class TokenDispatch(NamedTuple):
    """The routing of one batch as the device-side preprocess leaves it (``kernels.moe_preprocess``)."""

    sorted_indices: torch.Tensor  # int64 [M]: flat (token * topk + slot) index of permuted row j
    row_map: torch.Tensor  # int32 [T * topk]: permuted row of flat index i (-1: dropped copy)
    topk: int
    group_offsets: torch.Tensor  # int64 [E + 1]: exclusive prefix of permuted rows per expert


def _quant_first_weight(w1, v1, transpose_w1, need_transpose=True):
    """Codes and scales of the first layer as the logical ``[E, N1, H]`` operand (N1 = 2F with SwiGLU) and
    its transpose ``[E, H, N1]``, from ``w1`` (and ``v1``) in either storage orientation."""
    q, s, q_t, s_t = kernels.block_quant_batched(w1.detach().contiguous(), return_transpose=True)
    if v1 is not None:
        qv, sv, qv_t, sv_t = kernels.block_quant_batched(v1.detach().contiguous(), return_transpose=True)
        if transpose_w1:  # stored [E, F, H]: gate rows on top of up rows
            q, s = torch.cat([q, qv], dim=1), torch.cat([s, sv], dim=1)
            q_t, s_t = torch.cat([q_t, qv_t], dim=2), torch.cat([s_t, sv_t], dim=2)
        else:  # stored [E, H, F]
            q, s = torch.cat([q, qv], dim=2), torch.cat([s, sv], dim=2)
            q_t, s_t = torch.cat([q_t, qv_t], dim=1), torch.cat([s_t, sv_t], dim=1)
    if not transpose_w1:
        q, s, q_t, s_t = q_t, s_t, q, s
    return q, s, q_t, s_t


class _Fp8ExpertMlp(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, w1, w2, v1, b1, b2, batch_sizes, transpose_w1, activation, dispatch, is_first_microbatch,
                weight_cache):
        assert x.dim() == 2 and w1.dim() == 3 and w2.dim() == 3
        E = w1.shape[0]
        goff = dispatch.group_offsets if dispatch is not None else _offsets(batch_sizes, x.device)
        train = any(ctx.needs_input_grad)  # all False under no_grad
        glu = activation == "swiglu"
        # first weight(s) as [E, N1, H] (rows = outputs), second as [E, H, F]: block quantisation
        # commutes with the transpose, so both orientations come out of one launch each
        quant1 = lambda t: _quant_first_weight(w1, v1, transpose_w1)  # noqa: E731
        quant2 = lambda t: kernels.block_quant_batched(w2.detach().contiguous(), return_transpose=True)  # noqa: E731
        if weight_cache is None:
            (q1, s1, q1_t, s1_t), (q2, s2, q2_t, s2_t) = quant1(True), quant2(True)
        else:
            q1, s1, q1_t, s1_t = weight_cache.codes("w1", (w1, v1), is_first_microbatch, True, quant1)
            q2, s2, q2_t, s2_t = weight_cache.codes("w2", (w2,), is_first_microbatch, True, quant2)
        xc = x.detach().contiguous()
        if dispatch is not None:
            M = dispatch.sorted_indices.numel()
            if train:
                qx, sx, qx_t, sx_t = kernels.permute_tile_quant_dual_grouped(
                    xc, dispatch.sorted_indices, dispatch.topk, goff, E, blocked=True
                )
            else:  # every token quantised once, its codes written to its top-k rows
                qx, sx = kernels.permute_tile_quant(xc, dispatch.row_map, dispatch.topk, M)
        elif train:
            qx, sx, qx_t, sx_t = kernels.tile_quant_dual_grouped(xc, goff, E, blocked=True)
        else:
            qx, sx = kernels.tile_quant(xc)
        fc1 = kernels.grouped_gemm_nt(qx, sx, q1, s1, goff, out_dtype=torch.bfloat16,
                                      bias=b1.detach().contiguous() if b1 is not None else None)  # fmt: skip
        if train:
            quant = kernels.swiglu_tile_quant_dual_grouped if glu else kernels.gelu_tile_quant_dual_grouped
            qh, sh, qh_t, sh_t = quant(fc1, goff, E, ld_t=kernels.qt_ld(qx_t), blocked=True)
        else:
            qh, sh = kernels.swiglu_tile_quant(fc1) if glu else kernels.gelu_tile_quant(fc1)
        out = kernels.grouped_gemm_nt(qh, sh, q2_t, s2_t, goff, out_dtype=x.dtype,
                                      bias=b2.detach().contiguous() if b2 is not None else None)  # fmt: skip
        if train:
            ctx.transpose_w1, ctx.glu, ctx.has_v1 = transpose_w1, glu, v1 is not None
            ctx.has_b1, ctx.has_b2 = b1 is not None, b2 is not None
            ctx.dtypes = (x.dtype, w1.dtype, w2.dtype)
            ctx.dispatch_topk = dispatch.topk if dispatch is not None else 0
            ctx.num_tokens = x.shape[0]
            row_map = dispatch.row_map if dispatch is not None else goff
            ctx.save_for_backward(goff, fc1, qx_t, sx_t, qh_t, sh_t, q1_t, s1_t, q2, s2, row_map)
        return out

    @staticmethod
    def backward(ctx, dy):
        goff, fc1, qx_t, sx_t, qh_t, sh_t, q1_t, s1_t, q2, s2, row_map = ctx.saved_tensors
        E = goff.numel() - 1
        x_dtype, w1_dtype, w2_dtype = ctx.dtypes
        dy = dy.contiguous().to(torch.bfloat16)
        M = dy.shape[0]
        ld_t = kernels.qt_ld(qx_t)
        bin_ids = None
        if ctx.has_b1 or ctx.has_b2:  # expert of every row, from the device-side offsets (no host round trip)
            bin_ids = torch.repeat_interleave(torch.arange(E, device=dy.device), goff[1:] - goff[:-1], output_size=M)
        db2 = bias_gather_add_bw(dy, bin_ids, E) if ctx.has_b2 else None
        qdy, sdy, qdy_t, sdy_t = kernels.tile_quant_dual_grouped(dy, goff, E, ld_t=ld_t, blocked=True)
        # through the second linear: dh = dy @ w2^T ([M, F]); dw2[f, h] = sum_m h[m, f] dy[m, h]
        dh = kernels.grouped_gemm_nt(qdy, sdy, q2, s2, goff, out_dtype=torch.bfloat16)
        dw2 = kernels.grouped_gemm_wgrad(qh_t, sh_t, qdy_t, sdy_t, goff, out_dtype=w2_dtype)
        # through the activation: the gradient of fc1 is quantised by the kernel that computes it and is
        # written in bf16 only when a bias gradient needs its row sums
        if ctx.glu:
            res = kernels.swiglu_bwd_tile_quant_dual_grouped(dh, fc1, goff, E, ld_t=ld_t, blocked=True, return_grad=ctx.has_b1)
        else:
            res = kernels.gelu_tile_quant_dual_grouped(fc1, goff, E, dh=dh, ld_t=ld_t, blocked=True, return_activation=ctx.has_b1)
        qg, sg, qg_t, sg_t = res[:4]
        db1 = bias_gather_add_bw(res[4], bin_ids, E) if ctx.has_b1 else None
        # through the first linear: dx = dfc1 @ w1 ([M, H]); dw1[n, h] = sum_m dfc1[m, n] x[m, h]
        dx = kernels.grouped_gemm_nt(qg, sg, q1_t, s1_t, goff, out_dtype=x_dtype)
        if ctx.dispatch_topk:  # back to token order: the sum over a token's copies (index_select's backward)
            dx = kernels.unpermute_combine(dx, row_map, None, ctx.num_tokens, ctx.dispatch_topk)
        if ctx.transpose_w1:
            dw1 = kernels.grouped_gemm_wgrad(qg_t, sg_t, qx_t, sx_t, goff, out_dtype=w1_dtype)
        else:
            dw1 = kernels.grouped_gemm_wgrad(qx_t, sx_t, qg_t, sg_t, goff, out_dtype=w1_dtype)
        dv1 = None
        if ctx.has_v1:  # the gate and the up half of the gradient go back to their own parameters
            dim = 1 if ctx.transpose_w1 else 2
            dw1, dv1 = (t.contiguous() for t in torch.chunk(dw1, 2, dim=dim))
        return dx, dw1, dw2, dv1, db1, db2, None, None, None, None, None, None


def grouped_mlp(hidden_states: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor,
                tokens_per_expert: Optional[torch.Tensor], v1: Optional[torch.Tensor] = None,
                b1: Optional[torch.Tensor] = None, b2: Optional[torch.Tensor] = None, activation: str = "swiglu",
                transpose_w1: bool = True, *, dispatch: Optional[TokenDispatch] = None,
                is_first_microbatch: Optional[bool] = None,
                weight_cache: Optional[WeightCodeCache] = None) -> torch.Tensor:
    """The expert MLP: ``gmm -> (bias) -> activation -> gmm -> (bias)``.

    ``hidden_states [M, H]`` bf16 rows grouped by expert; ``tokens_per_expert`` int64 ``[E]`` (CPU or
    device).  ``activation="swiglu"``: ``w1 [E, 2F, H]`` (merged gate / up), or ``w1`` and ``v1`` ``[E, F, H]``
    each; ``activation="gelu"``: ``w1 [E, F, H]``.  With ``transpose_w1=False`` the first weights are stored
    ``[E, H, *]``.  ``w2 [E, F, H]``; ``b1 [E, N1]`` / ``b2 [E, H]`` optional (not with ``v1``, as in the
    reference).  H and F multiples of 128.  Returns ``[M, H]``.

    ``dispatch``: the permute fused in; ``hidden_states`` is then ``[T, H]`` in token order,
    ``tokens_per_expert`` is not used (the dispatch carries the group offsets) and the result is the ``[M, H]``
    expert output in permuted order, ready for the combine.  ``weight_cache`` / ``is_first_microbatch``: codes of
    the weights kept between microbatches under the grouped linear's rule (``WeightCodeCache``); without a cache
    the weights are quantised in every call."""
    assert hidden_states.dtype == torch.bfloat16, "the fused activation kernels read bf16"
    assert activation in ("swiglu", "gelu"), f"unknown activation {activation}"
    assert v1 is None or activation == "swiglu", "v1 is the up projection of a gated unit"
    assert v1 is None or (b1 is None and b2 is None), "bias not supported yet for not merge_w1_v1"
    assert dispatch is not None or tokens_per_expert is not None, "tokens_per_expert or a dispatch is needed"
    return _Fp8ExpertMlp.apply(hidden_states, w1, w2, v1, b1, b2, tokens_per_expert, transpose_w1, activation, dispatch,
                               is_first_microbatch, weight_cache)


def grouped_mlp_swiglu(hidden_states: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor,
                       tokens_per_expert: Optional[torch.Tensor], transpose_w1: bool = True, **kw) -> torch.Tensor:
    """``gmm -> SwiGLU -> gmm`` with the merged gate / up weight (``grouped_mlp`` with its defaults)."""
    return grouped_mlp(hidden_states, w1, w2, tokens_per_expert, transpose_w1=transpose_w1, **kw)

"""Token permute / unpermute for the MoE expert path on the gfx950 kernels.

``permute`` and ``unpermute`` keep the signatures and results of
atorch/modules/moe/token_dispatcher.py:89-116 and :119-161 and are differentiable like the torch
ops they replace.  ``MoEAllToAllTokenDispatcher`` has the reference's constructor and return
tuples (token_dispatcher.py:255-262, 355-415, 417-470) for the single-GPU branch, without the host
round trip: tokens per expert stay on the device, and ``token_permutation_fp8`` fuses the 1x128
quantisation into the permute.
"""
from typing import Callable, List, Optional, Tuple

import torch

from . import kernels

MAX_EXPERTS = 1024  # expert ids the router preprocess can sort when the caller does not say how many there are


def _rows(t: torch.Tensor) -> torch.Tensor:
    return t.contiguous().view(-1, t.shape[-1])


class _PermuteRows(torch.autograd.Function):
    """out[row_map[t*topk+j]] = tokens[t]; the gradient sums the topk copies of a token
    (what index_select's backward does, token_dispatcher.py:115)."""

    @staticmethod
    def forward(ctx, tokens, row_map, topk, n_out):
        ctx.save_for_backward(row_map)
        ctx.topk, ctx.num_tokens = topk, tokens.shape[0]
        return kernels.permute_rows(tokens, row_map, topk, n_out)

    @staticmethod
    def backward(ctx, dy):
        (row_map,) = ctx.saved_tensors
        d_tokens = kernels.unpermute_combine(dy.contiguous(), row_map, None, ctx.num_tokens, ctx.topk)
        return d_tokens, None, None, None


class _UnpermuteCombine(torch.autograd.Function):
    """out[t] = sum_j probs[t, j] * permuted[row_map[t*topk+j]] (token_dispatcher.py:155-159) with both
    gradients: d_permuted[row] = d_out[t] * probs[t, j], d_probs[t, j] = <d_out[t], permuted[row]>."""

    @staticmethod
    def forward(ctx, permuted, row_map, probs, num_tokens, topk):
        ctx.save_for_backward(permuted, row_map, probs if probs is not None else row_map)
        ctx.has_probs, ctx.topk = probs is not None, topk
        return kernels.unpermute_combine(permuted, row_map, probs, num_tokens, topk)

    @staticmethod
    def backward(ctx, dout):
        permuted, row_map, probs = ctx.saved_tensors
        if not ctx.has_probs:
            probs = None
        dout = dout.contiguous()
        d_perm = d_probs = None
        if ctx.needs_input_grad[0]:
            d_perm = kernels.permute_rows_scaled(dout, row_map, ctx.topk, permuted.shape[0], probs, permuted.dtype)
        if probs is not None and ctx.needs_input_grad[2]:
            d_probs = kernels.unpermute_probs_grad(dout, permuted, row_map, ctx.topk).to(probs.dtype)
        return d_perm, None, d_probs, None, None


def _check_rows_dtype(t: torch.Tensor, what: str):
    if t.dtype not in (torch.bfloat16, torch.float32):
        raise ValueError(f"{what}: bf16 and fp32 rows are supported, got {t.dtype}")


def permute(tokens: torch.Tensor, indices: torch.Tensor, num_out_tokens: Optional[int] = None,
            num_experts: Optional[int] = None):
    """Group the tokens by expert id.  ``indices`` is ``[T]`` or ``[T, topk]``; rows of one expert
    keep the order of the flattened ``(token, slot)`` index (stable sort).  Returns
    ``(permuted_tokens, sorted_indices)`` like the reference.  ``num_experts`` (an upper bound of the
    ids) is optional: without it ids up to 1023 are sorted and the call checks on the host that none
    was larger (one device round trip; pass ``num_experts`` to avoid it)."""
    topk = 1 if indices.dim() == 1 else indices.size(1)
    E = MAX_EXPERTS if num_experts is None else num_experts
    sorted_indices, row_map, goff = kernels.moe_preprocess(indices.contiguous(), E)
    n = sorted_indices.numel()
    if num_experts is None and n > 0 and int(goff[-1]) != n:
        raise ValueError(f"permute: expert ids must be below {MAX_EXPERTS} when num_experts is not given")
    n_out = n
    if num_out_tokens is not None and int(num_out_tokens) < n:
        n_out = int(num_out_tokens)
        sorted_indices = sorted_indices[:n_out]
        row_map = torch.where(row_map < n_out, row_map, torch.full_like(row_map, -1))
    x = _rows(tokens)
    _check_rows_dtype(x, "permute")
    permuted = _PermuteRows.apply(x, row_map, topk, n_out)
    return permuted, sorted_indices


def unpermute(permuted_tokens: torch.Tensor, sorted_indices: torch.Tensor, probs: Optional[torch.Tensor] = None):
    """Inverse of ``permute`` with the optional weighted merge over topk
    (token_dispatcher.py:119-161): one gather-reduce pass instead of zeros + index_copy_ +
    multiply + sum.  The result has the promoted dtype of rows and probs, as the reference's."""
    assert sorted_indices.numel() == permuted_tokens.size(0)
    if probs is not None:
        num_unpermuted_tokens = probs.numel()
        topk = probs.size(1)
    else:
        num_unpermuted_tokens = permuted_tokens.size(0)
        topk = 1
    row_map = kernels.invert_permutation(sorted_indices, num_unpermuted_tokens)
    x = permuted_tokens.contiguous()
    _check_rows_dtype(x, "unpermute")
    return _UnpermuteCombine.apply(x, row_map, probs, num_unpermuted_tokens // topk, topk)


class MoETokenDispatcher:
    """Single-GPU token dispatcher (no expert parallelism).

    ``token_permutation(hidden, max_prob, max_ind)`` returns ``(permuted rows, group_offsets)``
    and ``token_unpermutation(expert_out)`` restores the original order with the probability
    weighted merge, as token_dispatcher.py:355-415 / 417-470 do for ``ep_size == 1``.
    ``token_permutation_fp8`` is the fused form feeding the fp8 grouped linear: it returns the
    1x128 codes and scales of the permuted rows without ever materialising them in bf16.
    """

    def __init__(self, num_local_experts: int, topk: int):
        self.num_experts = num_local_experts
        self.topk = topk
        self.hidden_shape = None
        self.probs = None
        self.row_map = None
        self.sorted_indices = None
        self.group_offsets = None

    def preprocess(self, indices: torch.Tensor) -> torch.Tensor:
        """Counting sort of the routing on the device; returns ``group_offsets`` [E+1] int64
        (device).  ``tokens_per_expert`` is ``group_offsets.diff()``."""
        self.sorted_indices, self.row_map, self.group_offsets = kernels.moe_preprocess(
            indices.contiguous(), self.num_experts
        )
        return self.group_offsets

    def token_permutation(self, hidden_states: torch.Tensor, max_prob: torch.Tensor, max_ind: torch.Tensor):
        self.hidden_shape = hidden_states.shape
        self.probs = max_prob
        assert max_prob.dim() == 2, "Expected 2D tensor for probs"
        assert max_ind.dim() == 2, "Expected 2D tensor for indices"
        x = _rows(hidden_states)
        _check_rows_dtype(x, "token_permutation")
        goff = self.preprocess(max_ind)
        permuted = _PermuteRows.apply(x, self.row_map, self.topk, self.row_map.numel())
        return permuted, goff

    def token_permutation_fp8(self, hidden_states: torch.Tensor, max_prob: torch.Tensor, max_ind: torch.Tensor,
                              eps: float = 0.0, return_transpose: bool = False):
        """The permute fused into the 1x128 quantisation of the permuted rows, which are never written in bf16.
        Codes have no gradient: this form feeds an inference forward, or a caller that handles the backward
        itself (``expert_mlp.grouped_mlp(..., dispatch=self.dispatch())`` is the differentiable route).
        Returns ``(codes [M, H], scales [M, H/128], group_offsets)``; with ``return_transpose`` (what a training
        step's weight-gradient GEMM reads, quantized_grouped_linear.py:90-101 with ``is_grad_enabled``)
        ``(codes, scales, codes_t [H, ld_t], scales_t [ld_t/128, H], group_offsets)`` in the layouts of
        ``kernels.tile_quant_dual_grouped``."""
        self.hidden_shape = hidden_states.shape
        self.probs = max_prob
        x = _rows(hidden_states.detach())
        self.preprocess(max_ind)  # a subclass may return tokens per expert: the prefix is self.group_offsets
        if return_transpose:
            q, s, q_t, s_t = kernels.permute_tile_quant_dual_grouped(
                x, self.sorted_indices, self.topk, self.group_offsets, self.num_experts, eps=eps
            )
            return q, s, q_t, s_t, self.group_offsets
        q, s = kernels.permute_tile_quant(x, self.row_map, self.topk, self.row_map.numel(), eps=eps)
        return q, s, self.group_offsets

    def dispatch(self):
        """The routing of the last ``preprocess`` as the ``TokenDispatch`` that ``expert_mlp.grouped_mlp`` takes to
        fuse the permute into its first quantiser."""
        from .expert_mlp import TokenDispatch

        assert self.row_map is not None, "preprocess() first"
        return TokenDispatch(self.sorted_indices, self.row_map, self.topk, self.group_offsets)

    def token_unpermutation(self, hidden_states: torch.Tensor, bias: torch.Tensor = None):
        assert bias is None, "Bias is not supported in MoETokenDispatcher"
        T = self.row_map.numel() // self.topk
        x = hidden_states.contiguous()
        _check_rows_dtype(x, "token_unpermutation")
        out = _UnpermuteCombine.apply(x, self.row_map, self.probs, T, self.topk)
        return out.view(self.hidden_shape), None


class MoEAllToAllTokenDispatcher(MoETokenDispatcher):
    """The reference's dispatcher class for one GPU: same constructor, same call signatures and
    return tuples (token_dispatcher.py:255-262, 355-361, 417-423).

    ``token_permutation`` returns ``(permuted_tokens, tokens_per_expert, se_intermediate)``;
    ``tokens_per_expert`` is an int64 tensor **on the device** (the reference copies it to the host,
    :341); ``self.group_offsets`` holds its exclusive prefix for the grouped kernels.
    ``token_unpermutation`` returns ``(output, None, se_output)``.  The shared-expert hooks run only
    in the reference's expert-parallel branch (:392-409, :440-457), which one GPU does not have, so
    both extra results are ``None``.  ``use_expert_parallelism=True`` raises.
    """

    def __init__(self, num_local_experts: int, local_expert_indices: List[int], num_moe_experts: int, topk: int,
                 add_bias: bool, use_expert_parallelism: bool) -> None:
        assert num_local_experts > 0, "Expected at least one expert"
        assert len(local_expert_indices) == num_local_experts, "Invalid local expert indices"
        if use_expert_parallelism:
            raise NotImplementedError("MoEAllToAllTokenDispatcher: this build runs on one GPU (no expert parallelism)")
        if num_local_experts != num_moe_experts:
            raise NotImplementedError("MoEAllToAllTokenDispatcher: without expert parallelism every expert is local")
        super().__init__(num_moe_experts, topk)
        self.use_expert_parallelism = use_expert_parallelism
        self.num_local_experts = num_local_experts
        self.local_expert_indices = local_expert_indices
        self.router_topk = topk
        self.add_bias = add_bias
        self.ep_size = 1
        self.num_out_tokens = None
        self.reversed_local_input_permutation_mapping = None

    def preprocess(self, indices: torch.Tensor) -> torch.Tensor:
        """Tokens per local expert, int64 ``[E]`` on the device (token_dispatcher.py:297-353 without its
        ``.cpu()`` copies)."""
        goff = super().preprocess(indices)
        self.num_out_tokens = indices.numel()
        self.reversed_local_input_permutation_mapping = self.sorted_indices
        return goff[1:] - goff[:-1]

    def token_permutation(self, hidden_states: torch.Tensor, max_prob: torch.Tensor, max_ind: torch.Tensor,
                          se_fn1: Optional[Callable] = None):
        self.hidden_shape = hidden_states.shape
        self.probs = max_prob
        assert max_prob.dim() == 2, "Expected 2D tensor for probs"
        assert max_ind.dim() == 2, "Expected 2D tensor for indices"
        x = _rows(hidden_states)
        _check_rows_dtype(x, "token_permutation")
        tokens_per_expert = self.preprocess(max_ind)
        permuted = _PermuteRows.apply(x, self.row_map, self.topk, self.row_map.numel())
        return permuted, tokens_per_expert, None

    def token_unpermutation(self, hidden_states: torch.Tensor, bias: torch.Tensor = None,
                            se_fn2: Optional[Callable] = None, se_fn2_input: Optional[Tuple] = None):
        assert bias is None, "Bias is not supported in MoEAlltoAllTokenDispatcher"
        out, _ = super().token_unpermutation(hidden_states)
        return out, None, None

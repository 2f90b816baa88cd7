"""Token permute / unpermute for the MoE expert path on the gfx950 kernels.

``permute`` and ``unpermute`` keep the signatures and results of
atorch/modules/moe/token_dispatcher.py:89-116 and :119-161.  ``MoETokenDispatcher`` is the
single-GPU branch of ``MoEAllToAllTokenDispatcher`` (token_dispatcher.py:297-470) without the
host round trip: tokens per expert stay on the device as ``group_offsets``, and the fp8 forms
fuse the 1x128 quantisation into the permute.
"""
from typing import Optional, Tuple

import torch

from . import kernels

MAX_EXPERTS = 1024


def permute(tokens: torch.Tensor, indices: torch.Tensor, num_out_tokens: Optional[int] = None,
            num_experts: Optional[int] = None):
    """Group the tokens by expert id.  ``indices`` is ``[T]`` or ``[T, topk]``; rows of one expert
    keep the order of the flattened ``(token, slot)`` index (stable sort).  Returns
    ``(permuted_tokens, sorted_indices)`` like the reference; ``num_experts`` (an upper bound of
    the ids) is optional and only saves scratch memory."""
    topk = 1 if indices.dim() == 1 else indices.size(1)
    E = MAX_EXPERTS if num_experts is None else num_experts
    sorted_indices, row_map, _ = kernels.moe_preprocess(indices.contiguous(), E)
    n = sorted_indices.numel()
    n_out = n
    if num_out_tokens is not None and int(num_out_tokens) < n:
        n_out = int(num_out_tokens)
        sorted_indices = sorted_indices[:n_out]
        row_map = torch.where(row_map < n_out, row_map, torch.full_like(row_map, -1))
    x = tokens.contiguous().view(-1, tokens.shape[-1])
    permuted = kernels.permute_rows(x, row_map, topk, n_out)
    return permuted, sorted_indices


def unpermute(permuted_tokens: torch.Tensor, sorted_indices: torch.Tensor, probs: Optional[torch.Tensor] = None):
    """Inverse of ``permute`` with the optional weighted merge over topk
    (token_dispatcher.py:119-161): one gather-reduce pass instead of zeros + index_copy_ +
    multiply + sum."""
    assert sorted_indices.numel() == permuted_tokens.size(0)
    if probs is not None:
        num_unpermuted_tokens = probs.numel()
        topk = probs.size(1)
    else:
        num_unpermuted_tokens = permuted_tokens.size(0)
        topk = 1
    row_map = kernels.invert_permutation(sorted_indices, num_unpermuted_tokens)
    x = permuted_tokens.contiguous()
    if x.dtype != torch.bfloat16:
        raise ValueError(f"unpermute: bf16 rows are supported, got {x.dtype}")
    return kernels.unpermute_combine(x, row_map, probs, num_unpermuted_tokens // topk, topk)


class MoETokenDispatcher:
    """Single-GPU token dispatcher (no expert parallelism).

    ``token_permutation(hidden, max_prob, max_ind)`` returns ``(permuted bf16 rows, group_offsets)``
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
        x = hidden_states.contiguous().view(-1, self.hidden_shape[-1])
        goff = self.preprocess(max_ind)
        permuted = kernels.permute_rows(x, self.row_map, self.topk, self.row_map.numel())
        return permuted, goff

    def token_permutation_fp8(self, hidden_states: torch.Tensor, max_prob: torch.Tensor, max_ind: torch.Tensor,
                              eps: float = 0.0) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        self.hidden_shape = hidden_states.shape
        self.probs = max_prob
        x = hidden_states.contiguous().view(-1, self.hidden_shape[-1])
        goff = self.preprocess(max_ind)
        q, s = kernels.permute_tile_quant(x, self.row_map, self.topk, self.row_map.numel(), eps=eps)
        return q, s, goff

    def token_unpermutation(self, hidden_states: torch.Tensor, bias: torch.Tensor = None):
        assert bias is None, "Bias is not supported in MoETokenDispatcher"
        T = self.row_map.numel() // self.topk
        out = kernels.unpermute_combine(hidden_states.contiguous(), self.row_map, self.probs, T, self.topk)
        return out.view(self.hidden_shape), None

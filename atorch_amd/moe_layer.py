"""The MoE layer of one GPU on the fp8 grouped kernels: dispatch -> expert MLP -> combine.

Constructor, parameter names (``w1``, ``w2``, ``v1``, ``b1``, ``b2``) and ``forward(hidden_states, expert_weights,
top_experts, se_fn1, se_fn2, se_fn2_additional_input)`` follow ``Grouped_GEMM_MoE``
(atorch/modules/moe/grouped_gemm_moe.py:349-518, 644-682) for the branch a single GPU takes: no expert
parallelism, the "Megatron" composite ``token_permutation -> compute_expert -> token_unpermutation`` with the
AllToAll dispatcher, whose exchange steps are no-ops without a process group.  Nothing on the way waits for the
device: the router preprocess leaves the group offsets in device memory (the reference copies the counts to the
host, :837), the permute is fused into the quantiser of the first GEMM's operand, the activation into the
quantiser of the second one's, and the combine is one gather-reduce pass, so a forward (and a backward) is a fixed
sequence of launches that a HIP graph can capture and replay on other routings of the same shape.

Differences from the reference, none of which changes results on one GPU: ``implementation_type`` "MegaBlocks"
runs the same composite (its sort / gather / scatter ops compute the same permutation and weighted sum);
``use_bias`` is honoured for both implementation types (the reference's Megatron branch switches it off, :396-400);
``use_expert_parallelism=True`` raises.
"""
import logging
from typing import Callable, List, Optional, Tuple, Union

import torch

from .expert_mlp import grouped_mlp
from .quantization import WeightCodeCache
from .token_dispatcher import MoEAllToAllTokenDispatcher

logger = logging.getLogger(__name__)


class Grouped_GEMM_MoE(torch.nn.Module):
    """A mixture-of-experts feed-forward block with grouped fp8 GEMMs (one GPU)."""

    def __init__(
        self,
        hidden_size,
        expert_intermediate_size,
        output_dropout_prob,
        num_experts,
        topk,
        use_swiglu=False,
        use_bias=False,
        initializer_range=0.02,
        use_expert_parallelism=False,
        expert_parallel_group=None,
        merge_w1_v1=True,
        transpose_w1=True,
        is_scale_gradient=False,
        implementation_type="MegaBlocks",
        token_dispatcher_type="AllToAll",
        device=None,
        dtype=None,
    ) -> None:
        super().__init__()
        if use_expert_parallelism or expert_parallel_group is not None:
            raise NotImplementedError("Grouped_GEMM_MoE: this build runs on one GPU (no expert parallelism)")
        if implementation_type not in ("MegaBlocks", "Megatron"):
            raise ValueError(f"'{implementation_type}' is not a valid MOEImplmenterType")
        if token_dispatcher_type not in ("AllToAll", "AllGather", "MindSpeedAllGather", "MindSpeedAllToAll"):
            raise ValueError(f"'{token_dispatcher_type}' is not a valid MOETokenDispatcherType")
        if token_dispatcher_type != "AllToAll":
            logger.warning("Grouped_GEMM_MoE: one GPU has one dispatcher; using the AllToAll dispatcher's local branch")
        self.implementation_type = implementation_type
        self.hidden_size = hidden_size
        self.expert_intermediate_size = expert_intermediate_size
        self.output_dropout_prob = output_dropout_prob
        self.num_experts = num_experts
        self.num_local_experts = num_experts
        self.use_expert_parallelism = False
        self.is_scale_gradient = is_scale_gradient
        self.gradient_scale = None  # 1 / expert-parallel size in the reference: one GPU scales by nothing
        self.topk = topk
        self.use_swiglu = use_swiglu
        self.use_bias = use_bias
        self.merge_w1_v1 = merge_w1_v1
        self.transpose_w1 = transpose_w1
        kw = {"device": device, "dtype": dtype}

        E, F, H = num_experts, expert_intermediate_size, hidden_size
        if use_swiglu and not merge_w1_v1:
            shape = (E, F, H) if transpose_w1 else (E, H, F)
            self.w1 = torch.nn.Parameter(torch.empty(shape, **kw))
            self.w2 = torch.nn.Parameter(torch.empty((E, F, H), **kw))
            self.v1 = torch.nn.Parameter(torch.empty(shape, **kw))
            assert not use_bias, "bias not supported yet for not merge_w1_v1"
        else:
            n1 = F * (2 if use_swiglu else 1)
            self.w1 = torch.nn.Parameter(torch.empty((E, n1, H) if transpose_w1 else (E, H, n1), **kw))
            self.w2 = torch.nn.Parameter(torch.empty((E, F, H), **kw))
        if use_bias:
            self.b1 = torch.nn.Parameter(torch.empty((E, F * (2 if use_swiglu else 1)), **kw))
            self.b2 = torch.nn.Parameter(torch.empty((E, H), **kw))
        self.dropout = torch.nn.Dropout(output_dropout_prob)

        self.w1.data.normal_(mean=0.0, std=initializer_range)
        self.w2.data.normal_(mean=0.0, std=initializer_range)
        if self.has_v1():
            self.v1.data.normal_(mean=0.0, std=initializer_range)
        if use_bias:
            self.b1.data.zero_()
            self.b2.data.zero_()

        self.token_dispatcher = MoEAllToAllTokenDispatcher(
            self.num_local_experts, list(range(self.num_local_experts)), self.num_experts, topk=self.topk,
            add_bias=self.use_bias, use_expert_parallelism=False,
        )  # fmt: skip
        self.weight_code_cache = WeightCodeCache()
        self.hidden_shape = None

    def has_v1(self):
        return hasattr(self, "v1") and self.v1 is not None

    def scale_grad(self, w):
        return w  # gradient_scale is None without expert parallelism (grouped_gemm_moe.py:427-431, 632-636)

    def _mlp(self, hidden_states, tokens_per_expert, dispatch, is_first_microbatch):
        out = grouped_mlp(
            hidden_states, self.scale_grad(self.w1), self.scale_grad(self.w2), tokens_per_expert,
            v1=self.scale_grad(self.v1) if self.has_v1() else None,
            b1=self.b1 if self.use_bias else None, b2=self.b2 if self.use_bias else None,
            activation="swiglu" if self.use_swiglu else "gelu", transpose_w1=self.transpose_w1,
            dispatch=dispatch, is_first_microbatch=is_first_microbatch, weight_cache=self.weight_code_cache,
        )  # fmt: skip
        return self.dropout(out)

    def compute_expert(self, _hidden_states, _tokens_per_expert, bin_ids=None, is_first_microbatch=None):
        """``compute_expert`` of the reference (:816-834) on rows that are already permuted: ``_tokens_per_expert``
        int64 ``[E]``, on the device or the host.  ``bin_ids`` is not needed: rows are grouped by expert."""
        if _hidden_states.nelement() == 0:
            return _hidden_states.new_zeros((0, self.hidden_size))
        return self._mlp(_hidden_states, _tokens_per_expert, None, is_first_microbatch)

    def forward(
        self,
        hidden_states: torch.Tensor,
        expert_weights: torch.Tensor,
        top_experts: torch.Tensor,
        se_fn1: Optional[Callable] = None,
        se_fn2: Optional[Callable] = None,
        se_fn2_additional_input: Optional[Union[torch.Tensor, Tuple, List]] = None,
        is_first_microbatch: Optional[bool] = None,
    ):
        """``is_first_microbatch`` (not in the reference's signature): the expert weights' fp8 codes are kept
        between the microbatches of a step under the grouped linear's rule; None quantises in every call."""
        if torch.is_autocast_enabled():
            expert_weights = expert_weights.to(torch.get_autocast_gpu_dtype())
            hidden_states = hidden_states.to(torch.get_autocast_gpu_dtype())
        return self._forward_megatron(hidden_states, expert_weights, top_experts, se_fn1, se_fn2,
                                      se_fn2_additional_input, is_first_microbatch)  # fmt: skip

    def _forward_megatron(self, hidden_states, expert_weights, top_experts, se_fn1=None, se_fn2=None,
                          se_fn2_additional_input=None, is_first_microbatch=None):
        expert_weights = expert_weights.view(-1, expert_weights.shape[-1])
        top_experts = top_experts.view(-1, top_experts.shape[-1])
        self.hidden_shape = hidden_states.shape
        d = self.token_dispatcher
        x = hidden_states.reshape(-1, self.hidden_shape[-1])
        if x.shape[0] == 0:
            return hidden_states.clone()
        # dispatch: only the routing is computed here; the permute itself happens inside the first quantiser
        d.hidden_shape, d.probs = self.hidden_shape, expert_weights
        d.preprocess(top_experts)

        se_intermediate = se_fn1(x) if se_fn1 is not None else None

        expert_output = self._mlp(x, None, d.dispatch(), is_first_microbatch)

        compute_fn_input = None
        if se_fn2_additional_input is not None:
            if isinstance(se_fn2_additional_input, (tuple, list)):
                compute_fn_input = (se_intermediate,) + tuple(se_fn2_additional_input)
            else:
                compute_fn_input = (se_intermediate, se_fn2_additional_input)
        elif se_fn2 is not None:
            compute_fn_input = (se_intermediate,)

        output, _, _ = d.token_unpermutation(expert_output)
        if se_fn2 is not None:
            se_output = se_fn2(*compute_fn_input)
            if se_output is not None:
                output = output + se_output.view(self.hidden_shape)
        return output

"""Per-expert bias on expert-tagged rows, the interface of atorch/kernels/triton_jit/bias_gather_add.py.

``bias_gather_add(inp, bias, bin_ids)`` adds ``bias[bin_ids[t]]`` to row ``t`` (:50-66, :147-160); its
backward passes the gradient through and sums it per expert in fp32 (:101-127), returning the sum in
the gradient's dtype.  Both directions are one HIP kernel each behind the C ABI.
"""
import torch

from ._lib import check, lib, ptr, stream

_DT = {torch.bfloat16: 0, torch.float32: 1}


def _ids(bin_ids: torch.Tensor):
    assert bin_ids.ndim == 1
    if bin_ids.dtype not in (torch.int64, torch.int32):
        bin_ids = bin_ids.to(torch.int64)
    return bin_ids.contiguous(), int(bin_ids.dtype == torch.int64)


def bias_gather_add_fw(inp: torch.Tensor, bias: torch.Tensor, bin_ids: torch.Tensor) -> torch.Tensor:
    assert inp.ndim == 2
    assert bias.ndim == 2
    assert bin_ids.ndim == 1
    assert inp.shape[1] == bias.shape[1]
    assert inp.shape[0] == bin_ids.shape[0]
    assert inp.dtype == bias.dtype and inp.dtype in _DT, "bf16 or fp32 tensors of one dtype"
    inp, bias = inp.contiguous(), bias.contiguous()
    ids, i64 = _ids(bin_ids)
    out = torch.empty_like(inp)
    T, H = inp.shape
    check(lib().aamd_bias_gather_add(ptr(inp), ptr(bias), ptr(ids), i64, T, H, bias.shape[0], _DT[inp.dtype], ptr(out), stream()))
    return out


def bias_gather_add_bw(grad: torch.Tensor, bin_ids: torch.Tensor, num_experts: int) -> torch.Tensor:
    assert grad.ndim == 2
    assert grad.shape[0] == bin_ids.shape[0]
    assert grad.dtype in _DT, "bf16 or fp32 gradients"
    grad = grad.contiguous()
    ids, i64 = _ids(bin_ids)
    T, H = grad.shape
    bgrad = torch.empty((num_experts, H), device=grad.device, dtype=torch.float32)
    check(lib().aamd_bias_gather_add_bgrad(ptr(grad), ptr(ids), i64, T, H, num_experts, _DT[grad.dtype], ptr(bgrad), stream()))
    return bgrad.to(grad.dtype)


class BiasGatherAddOp(torch.autograd.Function):
    @staticmethod
    def forward(ctx, inp, bias, bin_ids):
        ctx.save_for_backward(bin_ids)
        ctx.num_experts = bias.shape[0]
        return bias_gather_add_fw(inp, bias, bin_ids)

    @staticmethod
    def backward(ctx, grad):
        grad = grad.contiguous()
        (bin_ids,) = ctx.saved_tensors
        bgrad = bias_gather_add_bw(grad, bin_ids, ctx.num_experts)
        return grad, bgrad, None


def bias_gather_add(inp: torch.Tensor, bias: torch.Tensor, bin_ids: torch.Tensor) -> torch.Tensor:
    """``inp [token_num, hidden]`` + ``bias [expert_num, hidden][bin_ids]``; ``bin_ids [token_num]`` in ``[0, expert_num)``."""
    return BiasGatherAddOp.apply(inp, bias, bin_ids)

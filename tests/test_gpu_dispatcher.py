"""Token dispatch on the GPU against the reference's torch ops run on the CPU, gradients included:
permute = argsort(stable) + index_select (token_dispatcher.py:107-115), unpermute = zeros + index_copy_ +
multiply + sum (:146-159); and the reference-shaped dispatcher class (:255-262, 355-361, 417-423)."""
import pytest
import torch

from helpers import heavy_tailed, randn_bf16, topk_routing

pytestmark = pytest.mark.gpu


def _ref_permute(tokens, indices):
    topk = 1 if indices.dim() == 1 else indices.size(1)
    sorted_indices = torch.argsort(indices.view(-1), stable=True)
    return tokens.index_select(0, sorted_indices // topk), sorted_indices


def _ref_unpermute(permuted, sorted_indices, probs):
    if probs is not None:
        n, topk = probs.numel(), probs.size(1)
    else:
        n, topk = permuted.size(0), 1
    buf = torch.zeros([n, permuted.shape[-1]], dtype=permuted.dtype)
    buf = buf.index_copy(0, sorted_indices, permuted)
    buf = buf.reshape(-1, topk, permuted.size(-1))
    if probs is not None:
        buf = buf * probs.unsqueeze(-1)
    return buf.sum(dim=1)


def _ulps(a, b):
    """distance in units of the last place of a's dtype"""
    if a.dtype == torch.bfloat16:
        ia, ib = a.view(torch.int16).int(), b.view(torch.int16).int()
    else:
        ia, ib = a.view(torch.int32).long(), b.view(torch.int32).long()
    ia = torch.where(ia < 0, -(ia & 0x7FFFFFFF if a.dtype != torch.bfloat16 else ia & 0x7FFF), ia)
    ib = torch.where(ib < 0, -(ib & 0x7FFFFFFF if a.dtype != torch.bfloat16 else ib & 0x7FFF), ib)
    return (ia - ib).abs().max().item()


@pytest.mark.parametrize("rows_dtype", [torch.bfloat16, torch.float32], ids=["bf16", "fp32"])
@pytest.mark.parametrize("probs_dtype", [torch.bfloat16, torch.float32, None], ids=["pbf16", "pfp32", "noprobs"])
def test_permute_unpermute_forward_and_backward(dev, rows_dtype, probs_dtype):
    from atorch_amd.token_dispatcher import permute, unpermute

    T, H, E, k = 300, 256, 8, 4 if probs_dtype is not None else 1
    x0 = heavy_tailed((T, H), 1).to(rows_dtype)
    idx, probs0 = topk_routing(T, E, k, seed=2)
    if k == 1:
        idx = idx.view(-1)
    g0 = randn_bf16((T, H), 3).float()

    # reference ops on the CPU under autograd
    xr = x0.clone().requires_grad_(True)
    pr = probs0.to(probs_dtype).clone().requires_grad_(True) if probs_dtype is not None else None
    perm_r, sorted_r = _ref_permute(xr, idx)
    y_r = perm_r * 1.0  # a non-leaf between the two ops, as the expert MLP is
    y_r.retain_grad()
    out_r = _ref_unpermute(y_r, sorted_r, pr)
    out_r.backward(g0.to(out_r.dtype))

    xg = x0.clone().to(dev).requires_grad_(True)
    pg = probs0.to(probs_dtype).clone().to(dev).requires_grad_(True) if probs_dtype is not None else None
    perm_g, sorted_g = permute(xg, idx.to(dev), num_experts=E)
    assert torch.equal(sorted_g.cpu(), sorted_r) and torch.equal(perm_g.detach().cpu(), perm_r.detach())
    y_g = perm_g * 1.0
    y_g.retain_grad()
    out_g = unpermute(y_g, sorted_g, pg)
    assert out_g.dtype == out_r.dtype
    out_g.backward(g0.to(out_g.dtype).to(dev))

    # forward: bf16 products rounded like the reference's; the sum of k terms may differ in its last
    # place from the CPU's summation order (the device order is pinned against torch's GPU sum elsewhere)
    assert _ulps(out_g.detach().cpu(), out_r.detach()) <= 1
    # gradient of the combine w.r.t. the permuted rows: one multiply, one rounding: exact
    assert torch.equal(y_g.grad.cpu(), y_r.grad)
    # gradient of the permute: sum of the k copies' gradients (fp32 sum rounded once here, bf16 adds in
    # the reference): within two units in the last place
    assert _ulps(xg.grad.cpu(), xr.grad) <= (2 if rows_dtype == torch.bfloat16 else 8)
    if pg is not None:
        ref = pr.grad.double()
        tol = 2e-2 if probs_dtype == torch.bfloat16 or rows_dtype == torch.bfloat16 else 1e-5
        scale = ref.abs().max().clamp_min(1e-30)
        assert float((pg.grad.cpu().double() - ref).abs().max() / scale) <= tol


def test_permute_without_num_experts_checks_the_ids(dev):
    from atorch_amd.token_dispatcher import permute

    x = randn_bf16((16, 128), 1).to(dev)
    ids = torch.randint(0, 1024, (16, 2), generator=torch.Generator().manual_seed(1)).to(dev)
    out, srt = permute(x, ids)
    assert torch.equal(srt.cpu(), torch.argsort(ids.cpu().view(-1), stable=True))
    ids[3, 1] = 5000
    with pytest.raises(ValueError, match="below 1024"):
        permute(x, ids)


def test_reference_shaped_dispatcher_class(dev, oracle):
    from atorch_amd.token_dispatcher import MoEAllToAllTokenDispatcher

    T, H, E, k = 257, 384, 6, 2
    with pytest.raises(NotImplementedError):
        MoEAllToAllTokenDispatcher(E, list(range(E)), E, k, False, True)
    d = MoEAllToAllTokenDispatcher(E, list(range(E)), E, k, add_bias=False, use_expert_parallelism=False)
    x = heavy_tailed((T, 1, H), 5)  # [seq, batch, hidden] as the MoE layer passes it
    idx, probs = topk_routing(T, E, k, seed=6)
    probs = probs.bfloat16()
    xg = x.to(dev).requires_grad_(True)
    permuted, tokens_per_expert, se = d.token_permutation(xg, probs.to(dev), idx.to(dev), se_fn1=None)
    xp, so, counts = oracle.permute(x.view(T, H), idx, E)
    assert se is None and tokens_per_expert.is_cuda and tokens_per_expert.dtype == torch.int64
    assert torch.equal(tokens_per_expert.cpu(), counts) and torch.equal(permuted.detach().cpu(), xp)
    assert torch.equal(d.reversed_local_input_permutation_mapping.cpu(), so)
    assert torch.equal(d.group_offsets.cpu()[1:], counts.cumsum(0))
    out, bias, se_out = d.token_unpermutation(permuted, bias=None, se_fn2=None, se_fn2_input=None)
    assert bias is None and se_out is None and out.shape == x.shape
    assert torch.equal(out.detach().cpu().view(T, H), oracle.unpermute(xp, so, probs))
    out.sum().backward()  # a training graph through the dispatcher reaches the hidden states
    assert xg.grad is not None and xg.grad.shape == x.shape
    with pytest.raises(AssertionError):
        d.token_unpermutation(permuted, bias=torch.zeros(1))


@pytest.mark.parametrize("k", [2, 5, 8])
def test_unpermute_fp32_rows_match_torch_ops_on_the_gpu(dev, k):
    """fp32 expert outputs (mm_fprop.out_dtype = float32): the combine equals the reference's torch ops
    run on the same GPU bit for bit, with bf16 and fp32 probs (token_dispatcher.py:146-159)."""
    from atorch_amd import kernels

    T, H, E = 200, 512, 16
    idx, probs = topk_routing(T, E, k, seed=k)
    y = torch.randn(T * k, H, generator=torch.Generator().manual_seed(9)).to(dev)
    so, row_map, _ = kernels.moe_preprocess(idx.to(dev), E)
    for pd in (torch.bfloat16, torch.float32, None):
        p = probs.to(pd).to(dev) if pd is not None else None
        if p is None and k != 2:
            continue
        buf = torch.zeros(T * k, H, dtype=y.dtype, device=dev).index_copy_(0, so, y).reshape(T, k, H)
        ref = (buf * p.unsqueeze(-1) if p is not None else buf).sum(dim=1)
        got = kernels.unpermute_combine(y, row_map, p, T, k)
        assert got.dtype == ref.dtype and torch.equal(got, ref)

"""The MoE expert path captured into one HIP graph and replayed on new tokens and a new routing.

Every entry point of the library only launches kernels (no allocation, copy or host synchronisation) and
takes its group boundaries from device memory, where the reference moves ``tokens_per_expert`` to the host
(grouped_gemm_moe.py:837) and sizes its launches from it.  So the router preprocessing, the permute, the two
grouped GEMMs with the fused SwiGLU quantiser and the weighted combine form one graph whose launch shapes do
not depend on the routing.  Each replay is checked bit for bit against the same calls made eagerly."""
import pytest
import torch

from helpers import randn_bf16, topk_routing

pytestmark = pytest.mark.gpu


def test_expert_path_replays_from_one_graph_on_new_routing():
    from atorch_amd import expert_mlp, kernels

    dev = torch.device("cuda:0")
    T, H, F, E, k = 1024, 256, 384, 8, 2
    w1 = randn_bf16((E, 2 * F, H), 1, std=0.05).to(dev)
    w2 = randn_bf16((E, F, H), 2, std=0.05).to(dev)
    x = torch.zeros((T, H), dtype=torch.bfloat16, device=dev)
    idx = torch.zeros((T, k), dtype=torch.int64, device=dev)
    probs = torch.zeros((T, k), dtype=torch.bfloat16, device=dev)

    def layer():
        _, row_map, goff = kernels.moe_preprocess(idx, E, want_sorted=False)
        xp = kernels.permute_rows(x, row_map, k, T * k)
        with torch.no_grad():
            y = expert_mlp.grouped_mlp_swiglu(xp, w1, w2, goff[1:] - goff[:-1])
        return kernels.unpermute_combine(y, row_map, probs, T, k), goff

    def fill(case):
        x.copy_(randn_bf16((T, H), 10 + case))
        if case == 0:
            ids, p = topk_routing(T, E, k, seed=20)
        elif case == 1:  # skewed: the busiest expert takes most rows, the tail experts few or none
            ids, p = topk_routing(T, E, k, seed=21, zipf_s=2.0)
        elif case == 2:  # two experts share all tokens, six groups are empty
            ids = torch.stack([torch.full((T,), 2), torch.full((T,), 5)], dim=1)
            p = torch.full((T, k), 0.5)
        else:
            ids, p = topk_routing(T, E, k, seed=23)
        idx.copy_(ids.to(torch.int64))
        probs.copy_(p.to(torch.bfloat16))

    fill(0)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # allocator warm-up, as graph capture in torch asks for
        layer()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out, goff = layer()

    sizes = []
    for case in range(4):
        fill(case)
        graph.replay()
        torch.cuda.synchronize()
        got, got_goff = out.clone(), goff.clone()
        want, want_goff = layer()  # eager work and a synchronisation between the replays
        torch.cuda.synchronize()
        assert torch.equal(got_goff, want_goff)
        assert torch.equal(got, want), f"replay {case} differs from the eager result"
        assert torch.isfinite(got.float()).all() and got.float().abs().max() > 0
        sizes.append((got_goff[1:] - got_goff[:-1]).tolist())
    assert sizes[2].count(0) == E - 2 and sizes[0] != sizes[1]  # the replays really saw different group sizes


@pytest.mark.filterwarnings("ignore:The AccumulateGrad node")  # the warm-up ran on a side stream, as capture asks for
def test_training_step_replays_from_one_graph_on_new_routing():
    """Forward and backward of the expert MLP (six grouped GEMMs, among them the two weight-gradient launches whose
    contraction runs over the ragged token blocks, and the quantisers between them) under one graph."""
    from atorch_amd import expert_mlp, kernels

    dev = torch.device("cuda:0")
    T, H, F, E, k = 768, 256, 256, 6, 2
    w1 = randn_bf16((E, 2 * F, H), 3, std=0.05).to(dev).requires_grad_(True)
    w2 = randn_bf16((E, F, H), 4, std=0.05).to(dev).requires_grad_(True)
    x = torch.zeros((T, H), dtype=torch.bfloat16, device=dev)
    dy = torch.zeros((T * k, H), dtype=torch.bfloat16, device=dev)
    idx = torch.zeros((T, k), dtype=torch.int64, device=dev)

    def step():
        _, row_map, goff = kernels.moe_preprocess(idx, E, want_sorted=False)
        xp = kernels.permute_rows(x, row_map, k, T * k).requires_grad_(True)
        y = expert_mlp.grouped_mlp_swiglu(xp, w1, w2, goff[1:] - goff[:-1])
        return (y,) + torch.autograd.grad(y, (xp, w1, w2), dy)

    def fill(case):
        x.copy_(randn_bf16((T, H), 30 + case))
        dy.copy_(randn_bf16((T * k, H), 40 + case, std=0.02))
        if case == 1:  # expert 0 and expert 4 only: the weight gradients of the others are zero
            ids = torch.stack([torch.zeros(T, dtype=torch.int64), torch.full((T,), 4)], dim=1)
        else:
            ids, _ = topk_routing(T, E, k, seed=50 + case, zipf_s=1.0 if case == 2 else None)
        idx.copy_(ids.to(torch.int64))

    fill(0)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = step()

    for case in range(3):
        fill(case)
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in outs]
        want = step()
        torch.cuda.synchronize()
        for name, a, b in zip(("y", "dx", "dw1", "dw2"), got, want):
            assert torch.equal(a, b), f"replay {case}: {name} differs from the eager result"
        if case == 1:
            dw1 = got[2].float()
            assert dw1[0].abs().max() > 0 and dw1[4].abs().max() > 0
            assert all(dw1[e].abs().max() == 0 for e in (1, 2, 3, 5))

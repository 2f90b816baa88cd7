"""The training path with the permute fused into the quantiser, the weight-code cache of the functional forms
and the single-GPU MoE layer composite.

  * aamd_permute_quant_1x128_dual_grouped (token_dispatcher.py:89-116 fused into quantized_grouped_linear.py:90-101
    with return_transpose) equals permute_rows -> tile_quant_dual_grouped bit for bit, and the oracle's
    permute -> tile_quant / tile_quant_t_grouped;
  * grouped_mlp(..., dispatch=...) equals permute -> grouped_mlp -> and the same gradients, bit for bit;
  * gmm / grouped_mlp with a WeightCodeCache give identical results with and without reuse (the reference's own
    invariant for the module, atorch/tests/common_tests/fp8/test_quantized_grouped_linear.py:515-557);
  * Grouped_GEMM_MoE (grouped_gemm_moe.py:644-682) against the composition of the tested parts (bit for bit),
    against a float32 torch MoE (tolerance of two chained fp8 GEMMs), and replayed from a HIP graph.
"""
import pytest
import torch

from helpers import TILE, heavy_tailed, randn_bf16, rel_err, topk_routing

pytestmark = pytest.mark.gpu


def _padded_total(counts):
    return sum((int(c) + TILE - 1) // TILE * TILE for c in counts)


@pytest.mark.parametrize("T,H,E,k,zipf,dtype", [
    (300, 384, 7, 3, 1.5, torch.bfloat16),   # ragged, empty groups, partial tiles, odd top-k
    (1024, 1024, 4, 2, None, torch.bfloat16),  # eight column tiles: the re-dealt workgroup order
    (257, 256, 5, 1, None, torch.float32),   # top-1, fp32 tokens
    (128, 128, 130, 8, None, torch.float16),  # more groups than lanes of a wave, most of them tiny
])  # fmt: skip
def test_permute_quant_dual_grouped_equals_permute_then_quant(oracle, dev, T, H, E, k, zipf, dtype):
    from atorch_amd import kernels

    x = heavy_tailed((T, H), 3, dtype=dtype)
    idx, _ = topk_routing(T, E, k, seed=4, zipf_s=zipf)
    sorted_idx, row_map, goff = kernels.moe_preprocess(idx.to(dev), E)
    M = T * k
    counts = (goff[1:] - goff[:-1]).cpu().tolist()
    pe = _padded_total(counts)
    xd = x.to(dev)
    q, s, q_t, s_t = kernels.permute_tile_quant_dual_grouped(xd, sorted_idx, k, goff, E)
    xp = kernels.permute_rows(xd, row_map, k, M) if dtype != torch.float16 else xd[sorted_idx // k].contiguous()
    q2, s2, q_t2, s_t2 = kernels.tile_quant_dual_grouped(xp, goff, E, ld_t=q_t.shape[1])
    u8 = lambda t: t.view(torch.uint8)  # noqa: E731
    assert torch.equal(u8(q), u8(q2)) and torch.equal(s, s2)
    assert torch.equal(u8(q_t)[:, :pe], u8(q_t2)[:, :pe]) and torch.equal(s_t[: pe // TILE], s_t2[: pe // TILE])
    # and against the oracle's permute followed by its quantisers
    xo, so, co = oracle.permute(x.float() if dtype == torch.float16 else x, idx, E)
    assert torch.equal(sorted_idx.cpu(), so) and co.tolist() == counts
    qo, sco = oracle.tile_quant(xo)
    qto, sto = oracle.tile_quant_t_grouped(xo, counts)
    assert torch.equal(u8(q).cpu(), u8(qo)) and torch.equal(s.cpu(), sco)
    assert torch.equal(u8(q_t)[:, :pe].cpu(), u8(qto)[:, :pe]) and torch.equal(s_t[: pe // TILE].cpu(), sto[: pe // TILE])
    # transposed outputs only
    _, _, q_t3, s_t3 = kernels.permute_tile_quant_dual_grouped(xd, sorted_idx, k, goff, E, rowwise=False)
    assert torch.equal(u8(q_t3)[:, :pe], u8(q_t)[:, :pe]) and torch.equal(s_t3[: pe // TILE], s_t[: pe // TILE])


def test_permute_quant_dual_grouped_rejects_bad_arguments(dev):
    from atorch_amd import kernels

    x = torch.zeros((8, 128), dtype=torch.bfloat16, device=dev)
    si = torch.zeros(16, dtype=torch.int64, device=dev)
    goff = torch.tensor([0, 16], dtype=torch.int64, device=dev)
    with pytest.raises(ValueError, match="topk"):
        kernels.permute_tile_quant_dual_grouped(x, si, 0, goff, 1)
    with pytest.raises(ValueError, match="within"):
        kernels.permute_tile_quant_dual_grouped(x, si, 1, goff, 1)  # 16 permuted rows from 8 tokens, top-1


def _mlp_inputs(dev, T, H, F, E, k, seed, zipf=None):
    x = randn_bf16((T, H), seed)
    w1 = randn_bf16((E, 2 * F, H), seed + 1, std=0.05)
    w2 = randn_bf16((E, F, H), seed + 2, std=0.05)
    idx, probs = topk_routing(T, E, k, seed=seed + 3, zipf_s=zipf)
    dout = randn_bf16((T, H), seed + 4, std=1e-2)
    return x, w1, w2, idx, probs.bfloat16(), dout


def test_grouped_mlp_with_fused_dispatch_equals_permute_then_mlp(dev):
    """Forward and every gradient (hidden states in token order, both weights, the router probabilities) of
    dispatch -> expert MLP -> combine are the same bits whether the permute is a kernel of its own under
    autograd or fused into the first quantiser."""
    from atorch_amd.expert_mlp import grouped_mlp
    from atorch_amd.token_dispatcher import MoETokenDispatcher

    T, H, F, E, k = 333, 256, 384, 6, 3
    x, w1, w2, idx, probs, dout = _mlp_inputs(dev, T, H, F, E, k, 1, zipf=1.2)
    res = []
    for fused in (False, True):
        xg = x.to(dev).requires_grad_(True)
        w1g, w2g = w1.to(dev).requires_grad_(True), w2.to(dev).requires_grad_(True)
        pg = probs.to(dev).requires_grad_(True)
        d = MoETokenDispatcher(E, k)
        if fused:
            d.hidden_shape, d.probs = xg.shape, pg
            d.preprocess(idx.to(dev))
            y = grouped_mlp(xg, w1g, w2g, None, dispatch=d.dispatch())
        else:
            permuted, goff = d.token_permutation(xg, pg, idx.to(dev))
            y = grouped_mlp(permuted, w1g, w2g, goff[1:] - goff[:-1])
        out, _ = d.token_unpermutation(y)
        out.backward(dout.to(dev))
        res.append((out.detach(), xg.grad, w1g.grad, w2g.grad, pg.grad))
    for name, a, b in zip(("out", "dx", "dw1", "dw2", "dprobs"), *res):
        assert a is not None and torch.equal(a, b), f"{name} differs between the fused and the separate permute"
    assert res[0][1].shape == (T, H) and res[0][1].abs().max() > 0
    # inference: every token quantised once and scattered; the same forward
    with torch.no_grad():
        d = MoETokenDispatcher(E, k)
        d.hidden_shape, d.probs = x.shape, probs.to(dev)
        d.preprocess(idx.to(dev))
        y = grouped_mlp(x.to(dev), w1.to(dev), w2.to(dev), None, dispatch=d.dispatch())
        out, _ = d.token_unpermutation(y)
    assert torch.equal(out, res[0][0])


def test_dispatcher_fp8_forms_on_both_dispatcher_classes(oracle, dev):
    """token_permutation_fp8 with and without the transposed codes; the reference-shaped subclass, whose
    preprocess returns tokens per expert, still hands out the [E + 1] group offsets."""
    from atorch_amd.token_dispatcher import MoEAllToAllTokenDispatcher, MoETokenDispatcher

    T, H, E, k = 200, 256, 5, 2
    x = heavy_tailed((T, H), 8)
    idx, probs = topk_routing(T, E, k, seed=9)
    xo, so, counts = oracle.permute(x, idx, E)
    qo, sco = oracle.tile_quant(xo)
    qto, sto = oracle.tile_quant_t_grouped(xo, counts.tolist())
    pe = _padded_total(counts.tolist())
    want_goff = [0] + counts.cumsum(0).tolist()
    for d in (MoETokenDispatcher(E, k), MoEAllToAllTokenDispatcher(E, list(range(E)), E, k, False, False)):
        q, s, goff = d.token_permutation_fp8(x.to(dev), probs.to(dev), idx.to(dev))
        assert goff.numel() == E + 1 and goff.cpu().tolist() == want_goff
        assert torch.equal(q.view(torch.uint8).cpu(), qo.view(torch.uint8)) and torch.equal(s.cpu(), sco)
        q, s, q_t, s_t, goff = d.token_permutation_fp8(x.to(dev), probs.to(dev), idx.to(dev), return_transpose=True)
        assert goff.numel() == E + 1 and goff.cpu().tolist() == want_goff
        assert torch.equal(q.view(torch.uint8).cpu(), qo.view(torch.uint8)) and torch.equal(s.cpu(), sco)
        assert torch.equal(q_t.view(torch.uint8)[:, :pe].cpu(), qto.view(torch.uint8)[:, :pe])
        assert torch.equal(s_t[: pe // TILE].cpu(), sto[: pe // TILE])


@pytest.mark.parametrize("trans_b", [True, False])
def test_gmm_weight_code_cache(dev, trans_b, monkeypatch):
    """Cached codes give the bits of fresh ones; the weight is quantised once per step, again after it changed
    (even when the caller forgets to say so), and on every call with FORCE_QUANTIZE_PER_MICROBATCH."""
    from atorch_amd import kernels
    from atorch_amd.gmm import gmm
    from atorch_amd.quantization import WeightCodeCache

    E, K, N = 3, 256, 384
    splits = torch.tensor([100, 0, 156])
    calls = []
    real = kernels.block_quant_batched
    monkeypatch.setattr(kernels, "block_quant_batched", lambda *a, **kw: (calls.append(1), real(*a, **kw))[1])
    w = randn_bf16((E, N, K) if trans_b else (E, K, N), 2, std=0.02).to(dev).requires_grad_(True)
    cache = WeightCodeCache()

    def run(seed, **kw):
        a = randn_bf16((256, K), seed).to(dev).requires_grad_(True)
        out = gmm(a, w, splits, trans_b=trans_b, **kw)
        out.backward(randn_bf16((256, N), seed + 50, std=1e-2).to(dev))
        g = (out.detach().clone(), a.grad.clone(), w.grad.clone())
        w.grad = None
        return g

    for mb in range(3):
        fresh = run(10 + mb)
        n0 = len(calls)
        cached = run(10 + mb, is_first_microbatch=(mb == 0), weight_cache=cache)
        assert len(calls) - n0 == (1 if mb == 0 else 0)
        for a, b in zip(fresh, cached):
            assert torch.equal(a, b)
    with torch.no_grad():
        w.mul_(1.5)  # an optimizer step; the caller does not announce it
    n0 = len(calls)
    cached = run(20, is_first_microbatch=False, weight_cache=cache)
    assert len(calls) - n0 == 1
    for a, b in zip(run(20), cached):
        assert torch.equal(a, b)
    # a cache filled under no_grad (no transposed codes with trans_b) serves a training call by quantising again
    cache2 = WeightCodeCache()
    with torch.no_grad():
        o1 = gmm(randn_bf16((256, K), 30).to(dev), w, splits, trans_b=trans_b, is_first_microbatch=True, weight_cache=cache2)
        o2 = gmm(randn_bf16((256, K), 30).to(dev), w, splits, trans_b=trans_b, is_first_microbatch=False, weight_cache=cache2)
    assert torch.equal(o1, o2)
    for a, b in zip(run(31), run(31, is_first_microbatch=False, weight_cache=cache2)):
        assert torch.equal(a, b)
    monkeypatch.setenv("FORCE_QUANTIZE_PER_MICROBATCH", "True")
    n0 = len(calls)
    run(32, is_first_microbatch=False, weight_cache=cache)
    assert len(calls) - n0 == 1


def test_grouped_mlp_weight_code_cache(dev, monkeypatch):
    from atorch_amd import kernels
    from atorch_amd.expert_mlp import grouped_mlp
    from atorch_amd.quantization import WeightCodeCache

    T, H, F, E = 300, 256, 256, 4
    splits = torch.tensor([90, 110, 0, 100])
    w1 = randn_bf16((E, F, H), 1, std=0.05).to(dev).requires_grad_(True)
    v1 = randn_bf16((E, F, H), 2, std=0.05).to(dev).requires_grad_(True)
    w2 = randn_bf16((E, F, H), 3, std=0.05).to(dev).requires_grad_(True)
    calls = []
    real = kernels.block_quant_batched
    monkeypatch.setattr(kernels, "block_quant_batched", lambda *a, **kw: (calls.append(1), real(*a, **kw))[1])
    cache = WeightCodeCache()

    def run(seed, **kw):
        x = randn_bf16((T, H), seed).to(dev).requires_grad_(True)
        out = grouped_mlp(x, w1, w2, splits, v1=v1, **kw)
        out.backward(randn_bf16((T, H), seed + 50, std=1e-2).to(dev))
        g = [out.detach().clone(), x.grad.clone()] + [p.grad.clone() for p in (w1, v1, w2)]
        for p in (w1, v1, w2):
            p.grad = None
        return g

    for mb in range(2):
        fresh = run(5 + mb)
        n0 = len(calls)
        cached = run(5 + mb, is_first_microbatch=(mb == 0), weight_cache=cache)
        assert len(calls) - n0 == (3 if mb == 0 else 0)  # w1, v1, w2
        for a, b in zip(fresh, cached):
            assert torch.equal(a, b)
    with torch.no_grad():
        v1.add_(0.01)  # only the up projection changed: both first-layer weights are requantised, w2 is not
    n0 = len(calls)
    cached = run(9, is_first_microbatch=False, weight_cache=cache)
    assert len(calls) - n0 == 2
    for a, b in zip(run(9), cached):
        assert torch.equal(a, b)


def _float_moe(x, w1, w2, idx, probs, use_swiglu):
    """The layer's function in float32 torch ops: per token, the probability-weighted sum of its experts' MLPs."""
    T, H = x.shape
    out = torch.zeros(T, H, dtype=torch.float32)
    xf = x.float()
    for t in range(T):
        for j in range(idx.shape[1]):
            e = int(idx[t, j])
            fc1 = w1[e].float() @ xf[t]
            if use_swiglu:
                a, b = fc1.chunk(2)
                h = torch.nn.functional.silu(a) * b
            else:
                h = torch.nn.functional.gelu(fc1)
            out[t] += probs[t, j].float() * (h @ w2[e].float())
    return out


@pytest.mark.parametrize("use_swiglu", [True, False])
def test_moe_layer_matches_composition_and_float_reference(dev, use_swiglu):
    from atorch_amd.expert_mlp import grouped_mlp
    from atorch_amd.moe_layer import Grouped_GEMM_MoE
    from atorch_amd.token_dispatcher import MoEAllToAllTokenDispatcher

    T, H, F, E, k = 96, 256, 256, 5, 2
    torch.manual_seed(0)
    layer = Grouped_GEMM_MoE(H, F, 0.0, E, k, use_swiglu=use_swiglu, implementation_type="Megatron",
                             device=dev, dtype=torch.bfloat16)  # fmt: skip
    assert layer.w1.shape == (E, F * (2 if use_swiglu else 1), H) and layer.w2.shape == (E, F, H)
    x = randn_bf16((T, 1, H), 3)  # [seq, batch, hidden]
    idx, probs = topk_routing(T, E, k, seed=4)
    probs = probs.bfloat16()
    dout = randn_bf16((T, 1, H), 5, std=1e-2)
    xg = x.to(dev).requires_grad_(True)
    pg = probs.to(dev).requires_grad_(True)
    out = layer(xg, pg, idx.to(dev), is_first_microbatch=True)
    assert out.shape == x.shape and out.dtype == torch.bfloat16
    out.backward(dout.to(dev))
    got = (out.detach().clone(), xg.grad.clone(), layer.w1.grad.clone(), layer.w2.grad.clone(), pg.grad.clone())
    layer.zero_grad()

    # the reference's composite with the tested parts: permute, expert MLP on permuted rows, combine
    d = MoEAllToAllTokenDispatcher(E, list(range(E)), E, k, False, False)
    xg2, pg2 = x.to(dev).requires_grad_(True), probs.to(dev).requires_grad_(True)
    permuted, tokens_per_expert, _ = d.token_permutation(xg2, pg2, idx.to(dev))
    y = grouped_mlp(permuted, layer.w1, layer.w2, tokens_per_expert, activation="swiglu" if use_swiglu else "gelu")
    out2, _, _ = d.token_unpermutation(y)
    out2.backward(dout.to(dev))
    want = (out2.detach(), xg2.grad, layer.w1.grad, layer.w2.grad, pg2.grad)
    for name, a, b in zip(("out", "dx", "dw1", "dw2", "dprobs"), got, want):
        assert torch.equal(a, b), f"{name}: the layer differs from the composition of its parts"
    layer.zero_grad()

    # the unquantised float32 function, a sanity bound only: e4m3 keeps three mantissa bits, so each operand carries
    # about 3.6 % of rms rounding noise and two chained GEMMs of quantised operands land near 6-7 %
    ref = _float_moe(x.view(T, H), layer.w1.detach().cpu(), layer.w2.detach().cpu(), idx, probs, use_swiglu)
    o = got[0].view(T, H).float().cpu()
    rms = ref.pow(2).mean().sqrt()
    assert float((o - ref).pow(2).mean().sqrt() / rms) < 0.1 and rel_err(o, ref) < 0.5
    # second microbatch on cached codes, and the no_grad path: the same forward
    out3 = layer(x.to(dev), probs.to(dev), idx.to(dev), is_first_microbatch=False)
    with torch.no_grad():
        out4 = layer(x.to(dev), probs.to(dev), idx.to(dev))
    assert torch.equal(out3.detach(), got[0]) and torch.equal(out4, got[0])
    # shared-expert hooks: se_fn1 on the token rows, se_fn2 on its result, added to the output
    se = layer(x.to(dev), probs.to(dev), idx.to(dev), se_fn1=lambda h: h * 2, se_fn2=lambda h: h * 0.5)
    assert torch.equal(se.detach(), (got[0] + (x.to(dev) * 2 * 0.5)))
    # compute_expert on permuted rows (the reference's entry for callers that dispatch themselves)
    with torch.no_grad():
        y2 = layer.compute_expert(permuted.detach(), tokens_per_expert)
    assert torch.equal(y2, y.detach())
    with pytest.raises(NotImplementedError):
        Grouped_GEMM_MoE(H, F, 0.0, E, k, use_expert_parallelism=True)


@pytest.mark.parametrize("variant", ["separate_kn", "bias_gelu", "bias_swiglu_megablocks"])
def test_moe_layer_other_parameterisations(dev, variant):
    """Separate gate / up weights stored [E, H, F] (merge_w1_v1=False, transpose_w1=False), and use_bias with both
    activations: the layer equals permute -> grouped_mlp with the same parameters -> combine, bit for bit, gradients of
    every parameter included."""
    from atorch_amd.expert_mlp import grouped_mlp
    from atorch_amd.moe_layer import Grouped_GEMM_MoE
    from atorch_amd.token_dispatcher import MoETokenDispatcher

    T, H, F, E, k = 160, 256, 128, 4, 2
    torch.manual_seed(2)
    kw = {"device": dev, "dtype": torch.bfloat16}
    if variant == "separate_kn":
        layer = Grouped_GEMM_MoE(H, F, 0.0, E, k, use_swiglu=True, merge_w1_v1=False, transpose_w1=False, **kw)
        assert layer.w1.shape == (E, H, F) and layer.v1.shape == (E, H, F) and layer.has_v1()
    elif variant == "bias_gelu":
        layer = Grouped_GEMM_MoE(H, F, 0.0, E, k, use_swiglu=False, use_bias=True, implementation_type="Megatron", **kw)
    else:
        layer = Grouped_GEMM_MoE(H, F, 0.0, E, k, use_swiglu=True, use_bias=True, implementation_type="MegaBlocks", **kw)
    if layer.use_bias:
        with torch.no_grad():
            layer.b1.copy_(randn_bf16(tuple(layer.b1.shape), 11, std=0.5))
            layer.b2.copy_(randn_bf16(tuple(layer.b2.shape), 12, std=0.5))
    params = [p for p in layer.parameters()]
    x = randn_bf16((T, H), 13)
    idx, probs = topk_routing(T, E, k, seed=14, zipf_s=1.0)
    probs = probs.bfloat16()
    dout = randn_bf16((T, H), 15, std=1e-2).to(dev)

    xg = x.to(dev).requires_grad_(True)
    out = layer(xg, probs.to(dev), idx.to(dev))
    out.backward(dout)
    got = [out.detach().clone(), xg.grad.clone()] + [p.grad.clone() for p in params]
    layer.zero_grad()

    d = MoETokenDispatcher(E, k)
    xg2 = x.to(dev).requires_grad_(True)
    permuted, goff = d.token_permutation(xg2, probs.to(dev), idx.to(dev))
    y = grouped_mlp(permuted, layer.w1, layer.w2, goff[1:] - goff[:-1], v1=layer.v1 if layer.has_v1() else None,
                    b1=layer.b1 if layer.use_bias else None, b2=layer.b2 if layer.use_bias else None,
                    activation="swiglu" if layer.use_swiglu else "gelu", transpose_w1=layer.transpose_w1)  # fmt: skip
    out2, _ = d.token_unpermutation(y)
    out2.backward(dout)
    want = [out2.detach(), xg2.grad] + [p.grad for p in params]
    assert len(got) == len(want) and all(g is not None for g in want)
    for i, (a, b) in enumerate(zip(got, want)):
        if layer.use_bias and a.shape in (tuple(layer.b1.shape), tuple(layer.b2.shape)):
            torch.testing.assert_close(a.float(), b.float(), rtol=2e-2, atol=1e-4)  # atomics: order of an fp32 sum
        else:
            assert torch.equal(a, b), f"tensor {i} differs from the composition"
    assert float(out.detach().float().abs().max()) > 0


@pytest.mark.filterwarnings("ignore:The AccumulateGrad node")
def test_moe_layer_training_step_replays_from_one_graph(dev):
    """Forward and backward of the whole layer (router preprocess, fused permute + quantise, six grouped GEMMs, the
    fused activation quantisers, combine and its gradients) captured once and replayed on other routings."""
    from atorch_amd.moe_layer import Grouped_GEMM_MoE

    T, H, F, E, k = 512, 256, 256, 6, 2
    torch.manual_seed(1)
    layer = Grouped_GEMM_MoE(H, F, 0.0, E, k, use_swiglu=True, device=dev, dtype=torch.bfloat16)
    x = torch.zeros((T, H), dtype=torch.bfloat16, device=dev, requires_grad=True)
    probs = torch.zeros((T, k), dtype=torch.bfloat16, device=dev, requires_grad=True)
    idx = torch.zeros((T, k), dtype=torch.int64, device=dev)
    dout = torch.zeros((T, H), dtype=torch.bfloat16, device=dev)

    def step():
        out = layer(x, probs, idx)
        return (out,) + torch.autograd.grad(out, (x, probs, layer.w1, layer.w2), dout)

    def fill(case):
        with torch.no_grad():
            x.copy_(randn_bf16((T, H), 60 + case))
            dout.copy_(randn_bf16((T, H), 70 + case, std=0.02))
            if case == 1:
                ids = torch.stack([torch.full((T,), 1), torch.full((T,), 3)], dim=1)
                p = torch.full((T, k), 0.5)
            else:
                ids, p = topk_routing(T, E, k, seed=80 + case, zipf_s=1.0 if case == 2 else None)
            idx.copy_(ids.to(torch.int64))
            probs.copy_(p.to(torch.bfloat16))

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
        for name, a, b in zip(("out", "dx", "dprobs", "dw1", "dw2"), got, want):
            assert torch.equal(a, b), f"replay {case}: {name} differs from the eager result"
        if case == 1:
            dw1 = got[3].float()
            assert dw1[1].abs().max() > 0 and all(dw1[e].abs().max() == 0 for e in (0, 2, 4, 5))

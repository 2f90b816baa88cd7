"""Module-level parity on the GPU, in the shape of the reference's own test
(atorch/tests/common_tests/fp8/test_quantized_grouped_linear.py:607-737): the grouped module
against a sequential loop of single-group modules sharing its weights (bit-wise), and against
the CPU oracle (GEMM tolerance 1e-2); plus the gmm adapter and the dispatcher round trip."""
import pytest
import torch

from helpers import OracleQuantizeOp, heavy_tailed, ragged_splits, randn_bf16, rel_err, topk_routing

pytestmark = pytest.mark.gpu
TOL = 1e-2


def _run(module, x, m_splits, fuse):
    out = module(x, m_splits)
    out.sum().backward()
    res = [out.detach(), x.grad.detach()]
    for p in module.parameters():
        if getattr(p, "main_grad", None) is not None and fuse:
            assert p.grad is None
            res.append(p.main_grad)
        else:
            res.append(p.grad)
    return res


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("batch_size", [1, 2])
@pytest.mark.parametrize("num_gemms", [3, 6])
@pytest.mark.parametrize("fuse_wgrad_accumulation", [True, False])
def test_grouped_linear_recipes(dev, dtype, batch_size, num_gemms, fuse_wgrad_accumulation, oracle):
    from atorch_amd.grouped_linear import ATorchGroupedLinear

    hidden, out_size, seq = 256, 128, 2048
    torch.manual_seed(0)
    grouped = ATorchGroupedLinear(num_gemms, hidden, out_size, bias=False, params_dtype=dtype, device=dev,
                                  fuse_wgrad_accumulation=fuse_wgrad_accumulation)
    singles = [ATorchGroupedLinear(1, hidden, out_size, bias=False, params_dtype=dtype, device=dev,
                                   fuse_wgrad_accumulation=fuse_wgrad_accumulation) for _ in range(num_gemms)]
    main_grad0 = []
    with torch.no_grad():
        for i in range(num_gemms):
            w = getattr(grouped, f"weight{i}")
            singles[i].weight0.copy_(w)
            if fuse_wgrad_accumulation:
                w.main_grad = torch.rand_like(w, dtype=torch.float32)
                singles[i].weight0.main_grad = w.main_grad.clone()
                main_grad0.append(w.main_grad.cpu().clone())
    splits = ragged_splits(seq, num_gemms, seed=0, multiple=16)
    assert 0 in splits
    m_splits = [m * batch_size for m in splits]
    x0 = randn_bf16((seq, batch_size, hidden), 0, dtype=dtype).to(dev)

    xg = x0.clone().requires_grad_(True)
    res = _run(grouped, xg, m_splits, fuse_wgrad_accumulation)

    xs = x0.clone().requires_grad_(True)
    outs = [singles[i](inp, [inp.shape[0] * batch_size]) for i, inp in enumerate(torch.split(xs, splits))]
    out_seq = torch.cat(outs)
    out_seq.sum().backward()
    ref = [out_seq.detach(), xs.grad.detach()]
    for s in singles:
        p = s.weight0
        ref.append(p.main_grad if fuse_wgrad_accumulation else p.grad)
    # should be a bit-wise match
    for o, r in zip(res, ref):
        torch.testing.assert_close(o, r, rtol=0, atol=0)

    # and against the CPU oracle
    ws = [getattr(grouped, f"weight{i}").detach().cpu() for i in range(num_gemms)]
    orc = oracle.grouped_linear_fwd_bwd(x0.cpu(), ws, m_splits, torch.ones(seq * batch_size, out_size, dtype=dtype))
    assert rel_err(res[0].cpu().view(-1, out_size), orc["out"]) <= TOL
    assert rel_err(res[1].cpu().view(-1, hidden), orc["dgrad"]) <= TOL
    # weight gradients; with fused accumulation the module adds them into main_grad
    # (quantized_grouped_linear.py:225-241), which held main_grad0 before the step
    for i in range(num_gemms):
        got = res[2 + i].cpu()
        if fuse_wgrad_accumulation:
            got = got.double() - main_grad0[i].double()
        assert rel_err(got, orc["wgrad"][i]) <= TOL + (2e-6 if fuse_wgrad_accumulation else 0)


def test_grouped_linear_bias_cache_and_nograd(dev, oracle):
    from atorch_amd.grouped_linear import ATorchGroupedLinear

    E, K, N = 4, 256, 384
    torch.manual_seed(1)
    mod = ATorchGroupedLinear(E, K, N, bias=True, params_dtype=torch.bfloat16, device=dev)
    with torch.no_grad():
        for i in range(E):
            getattr(mod, f"bias{i}").copy_(randn_bf16((N,), 40 + i).to(dev))
    splits = [100, 0, 313, 99]
    x = heavy_tailed((sum(splits), K), 6).to(dev)
    ws = [getattr(mod, f"weight{i}").detach().cpu() for i in range(E)]
    bs = [getattr(mod, f"bias{i}").detach().cpu() for i in range(E)]
    dy = randn_bf16((sum(splits), N), 7, std=1e-2)
    orc = oracle.grouped_linear_fwd_bwd(x.cpu(), ws, splits, dy, biases=bs)
    xg = x.clone().requires_grad_(True)
    o1 = mod(xg, splits, is_first_microbatch=True)
    o1.backward(dy.to(dev))
    assert rel_err(o1.detach().cpu(), orc["out"]) <= TOL
    assert rel_err(xg.grad.cpu(), orc["dgrad"]) <= TOL
    for i in range(E):
        assert rel_err(getattr(mod, f"weight{i}").grad.cpu(), orc["wgrad"][i]) <= TOL
        torch.testing.assert_close(getattr(mod, f"bias{i}").grad.cpu().float(), orc["bgrad"][i], rtol=2e-2, atol=1e-3)
    assert torch.all(mod.weight1.grad == 0)
    # cached weights give identical results (test_quantized_grouped_linear.py:515-557)
    o2 = mod(x, splits, is_first_microbatch=False)
    assert torch.equal(o1.detach(), o2.detach())
    with torch.no_grad():
        o3 = mod(x, splits)
    assert torch.equal(o1.detach(), o3)


def test_plugin_list_interface_unfused_operands(dev, oracle):
    """quantize_op.quantize per expert + grouped_qgemm on lists that do NOT tile one buffer:
    the operator falls back to one HIP launch per group and gives the same results."""
    from atorch_amd.quantization import HipQuantizeOp, MMParams, QParams

    op = HipQuantizeOp()
    xp, wp = QParams(quant_tile_shape=(1, 128)), QParams(quant_tile_shape=(128, 128))
    E, K, N = 3, 256, 128
    splits = [70, 0, 200]
    xs = [randn_bf16((m, K), 50 + i).to(dev) for i, m in enumerate(splits)]
    ws = [randn_bf16((N, K), 60 + i, std=0.02).to(dev) for i in range(E)]
    dys = [randn_bf16((m, N), 70 + i, std=1e-2).to(dev) for i, m in enumerate(splits)]
    qx = [op.quantize(x, xp, return_transpose=True) for x in xs]
    qw = [op.quantize(w, wp, return_transpose=True) for w in ws]
    qd = [op.quantize(d, xp, return_transpose=True) for d in dys]
    outs = [torch.empty((m, N), dtype=torch.bfloat16, device=dev) for m in splits]
    op.grouped_qgemm([r.data for r in qx], [r.data for r in qw], MMParams(), [r.scale for r in qx],
                     [r.scale for r in qw], outs, qparams_x=xp, qparams_w=wp)
    dgr = [torch.empty((m, K), dtype=torch.bfloat16, device=dev) for m in splits]
    op.grouped_qgemm([r.data for r in qd], [r.data_t for r in qw], MMParams(), [r.scale for r in qd],
                     [r.scale_t for r in qw], dgr, qparams_x=xp, qparams_w=wp)
    wgr = [torch.full((N, K), 7.0, dtype=torch.float32, device=dev) for _ in range(E)]
    op.grouped_qgemm([r.data_t for r in qd], [r.data_t for r in qx], MMParams(), [r.scale_t for r in qd],
                     [r.scale_t for r in qx], wgr, accumulate=False, qparams_x=xp, qparams_w=xp)
    x_all, dy_all = torch.cat(xs).cpu(), torch.cat(dys).cpu()
    orc = oracle.grouped_linear_fwd_bwd(x_all, [w.cpu() for w in ws], splits, dy_all)
    assert rel_err(torch.cat(outs).cpu(), orc["out"]) <= TOL
    assert rel_err(torch.cat(dgr).cpu(), orc["dgrad"]) <= TOL
    for e in range(E):
        assert rel_err(wgr[e].cpu(), orc["wgrad"][e]) <= TOL
    assert torch.all(wgr[1] == 0)
    # the transposed results have the reference's shapes
    assert qx[2].data_t.shape == (K, 200) and qx[2].scale_t.shape == (K, 2)
    assert qw[0].data_t.shape == (K, N) and qw[0].scale_t.shape == (K // 128, N // 128)


def test_module_with_oracle_operator_matches_hip_operator(dev):
    """Same module code, two operator plugins: the HIP one on the GPU and the oracle one on the
    CPU agree within the GEMM tolerance."""
    from atorch_amd.grouped_linear import ATorchGroupedLinear
    from atorch_amd.quantization import QLinearParams

    E, K, N = 3, 128, 256
    torch.manual_seed(3)
    hip = ATorchGroupedLinear(E, K, N, bias=False, params_dtype=torch.bfloat16, device=dev)
    cpu = ATorchGroupedLinear(E, K, N, bias=False, params_dtype=torch.bfloat16, device="cpu",
                              qlinear_params=QLinearParams(quantize_op=OracleQuantizeOp()))
    with torch.no_grad():
        for i in range(E):
            getattr(cpu, f"weight{i}").copy_(getattr(hip, f"weight{i}").cpu())
    splits = [33, 150, 73]
    x = randn_bf16((256, K), 9)
    a = x.clone().to(dev).requires_grad_(True)
    b = x.clone().requires_grad_(True)
    oa, ob = hip(a, splits), cpu(b, splits)
    oa.sum().backward()
    ob.sum().backward()
    assert rel_err(oa.detach().cpu(), ob.detach().float()) <= TOL
    assert rel_err(a.grad.cpu(), b.grad.float()) <= TOL
    for i in range(E):
        assert rel_err(getattr(hip, f"weight{i}").grad.cpu(), getattr(cpu, f"weight{i}").grad.float()) <= TOL


@pytest.mark.parametrize("trans_b", [True, False])
def test_gmm_adapter(dev, trans_b, oracle):
    """gmm(a, b, batch_sizes, trans_b) (grouped_gemm_moe.py:841-850, grouped_gemm_gmm.py:10-52) on the fp8
    path, forward and both gradients, against the quantised oracle at the GEMM tolerance; b is
    [E, N, K] with trans_b and [E, K, N] without."""
    from atorch_amd.gmm import gmm

    E, K, N = 4, 256, 384
    splits = [120, 0, 300, 92]
    M = sum(splits)
    a0 = randn_bf16((M, K), 1)
    w_nk = randn_bf16((E, N, K), 2, std=0.02)  # [out features, in features] per expert
    dy = randn_bf16((M, N), 3, std=1e-2)
    a = a0.to(dev).requires_grad_(True)
    w = (w_nk if trans_b else w_nk.transpose(1, 2).contiguous()).to(dev).requires_grad_(True)
    bs = torch.tensor(splits, dtype=torch.int64)
    out = gmm(a, w, bs, trans_b=trans_b)
    out.backward(dy.to(dev))
    orc = oracle.grouped_linear_fwd_bwd(a0, [w_nk[e] for e in range(E)], splits, dy)
    assert out.shape == (M, N) and out.dtype == torch.bfloat16
    assert rel_err(out.detach().cpu(), orc["out"]) <= TOL
    assert rel_err(a.grad.cpu(), orc["dgrad"]) <= TOL
    assert w.grad.shape == w.shape
    for e in range(E):
        dw = w.grad[e].cpu()
        assert rel_err(dw if trans_b else dw.t(), orc["wgrad"][e]) <= TOL
    assert torch.all(w.grad[1] == 0)


def test_dispatcher_round_trip(dev, oracle):
    from atorch_amd.token_dispatcher import MoETokenDispatcher

    T, H, E, k = 500, 512, 16, 4
    x = heavy_tailed((T, H), 12)
    idx, probs = topk_routing(T, E, k, seed=13)
    probs = probs.bfloat16()
    d = MoETokenDispatcher(E, k)
    permuted, goff = d.token_permutation(x.to(dev), probs.to(dev), idx.to(dev))
    xp, so, counts = oracle.permute(x, idx, E)
    assert torch.equal(permuted.cpu(), xp)
    assert torch.equal((goff[1:] - goff[:-1]).cpu(), counts)
    out, _ = d.token_unpermutation(permuted)
    assert torch.equal(out.cpu(), oracle.unpermute(xp, so, probs))
    q, s, goff2 = d.token_permutation_fp8(x.to(dev), probs.to(dev), idx.to(dev))
    qo, sco = oracle.tile_quant(xp)
    assert torch.equal(q.view(torch.uint8).cpu(), qo) and torch.equal(s.cpu(), sco)


# ------------------------------------------------------------------------------------------
# expert MLP with SwiGLU fused into the quantiser (the body of compute_moe)
# ------------------------------------------------------------------------------------------
@pytest.mark.parametrize("transpose_w1", [True, False])
def test_grouped_mlp_swiglu_matches_oracle_composition(oracle, dev, transpose_w1):
    """gmm -> SwiGLU -> gmm (grouped_gemm_moe.py:836-855, :331-334) forward and backward against the
    CPU composition: oracle grouped linear, oracle SwiGLU, torch autograd through SwiGLU, oracle
    grouped linear.  Tolerances are those of two chained bf16-output fp8 GEMMs."""
    from atorch_amd.expert_mlp import grouped_mlp_swiglu

    E, H, F, M = 3, 256, 384, 416
    splits = [200, 0, 216]
    x = randn_bf16((M, H), 1)
    w1 = randn_bf16((E, 2 * F, H), 2, std=0.05)
    w2 = randn_bf16((E, F, H), 3, std=0.05)
    dy = randn_bf16((M, H), 4, std=1e-2)

    xg = x.to(dev).requires_grad_(True)
    w1g = (w1 if transpose_w1 else w1.transpose(1, 2).contiguous()).to(dev).requires_grad_(True)
    w2g = w2.to(dev).requires_grad_(True)
    out = grouped_mlp_swiglu(xg, w1g, w2g, torch.tensor(splits), transpose_w1=transpose_w1)
    out.backward(dy.to(dev))

    r1 = oracle.grouped_linear_fwd_bwd(x, [w1[e] for e in range(E)], splits)
    fc1 = r1["out"].bfloat16().requires_grad_(True)
    h = oracle.torch_swiglu(fc1)
    assert torch.equal(h.detach(), oracle.swiglu(fc1.detach()))
    w2_t = [w2[e].t().contiguous() for e in range(E)]  # [H, F]: out features x in features
    r2 = oracle.grouped_linear_fwd_bwd(h.detach(), w2_t, splits, dy)
    h.backward(r2["dgrad"].bfloat16())
    r1b = oracle.grouped_linear_fwd_bwd(x, [w1[e] for e in range(E)], splits, fc1.grad)

    # The device's first GEMM differs from the oracle's in the last bf16 bit of some outputs; the
    # re-quantisation to fp8 turns such a bit into a whole fp8 step (6 - 12 %) of that element, so
    # the chained result is compared in the rms sense, with a loose bound on single outputs.
    def close(got, ref):
        got, ref = got.double(), ref.double()
        rms = ref.pow(2).mean().sqrt().clamp_min(1e-30)
        return float((got - ref).pow(2).mean().sqrt() / rms) < 1e-2 and rel_err(got, ref) < 0.15

    assert close(out.detach().cpu().float(), r2["out"])
    assert close(xg.grad.cpu().float(), r1b["dgrad"])
    dw1 = w1g.grad.cpu().float()
    if not transpose_w1:
        dw1 = dw1.transpose(1, 2)
    for e in range(E):
        if splits[e] == 0:
            continue
        assert close(dw1[e], r1b["wgrad"][e])
        assert close(w2g.grad[e].cpu().float(), r2["wgrad"][e].t())
    assert torch.all(w2g.grad[1] == 0) and torch.all(w1g.grad[1] == 0)

    # no_grad: the inference path (row-wise quantisation only) gives the same forward
    with torch.no_grad():
        out2 = grouped_mlp_swiglu(x.to(dev), w1g.detach(), w2g.detach(), torch.tensor(splits), transpose_w1=transpose_w1)
    assert torch.equal(out2, out.detach())


def test_baseline_first_configuration_end_to_end(oracle, dev):
    """The CPU-runnable configuration the path is specified on: 4 experts, hidden 512, ffn 1024,
    2048 tokens, bf16 activations ~ N(0, 1), bf16 weights ~ N(0, 0.02), top-1 routing with uniform
    random expert assignment, 1x128 activation and 128x128 weight quantisation to e4m3fn with fp32
    scales amax / 448, grouped GEMM forward with bf16 output.  Device path: router preprocess,
    fused permute + quantise, batched weight quantisation, grouped GEMM.  Checked step by step
    against the oracle: permutation, codes and scales bit-exact, outputs within 1e-2."""
    from atorch_amd import kernels
    from atorch_amd.token_dispatcher import MoETokenDispatcher

    E, H, F, T = 4, 512, 1024, 2048
    x = randn_bf16((T, H), 0)
    w = randn_bf16((E, F, H), 1, std=0.02)
    ids = torch.randint(0, E, (T, 1), generator=torch.Generator().manual_seed(2))
    probs = torch.ones(T, 1, dtype=torch.bfloat16)

    # oracle: stable sort by expert, gather, quantise, per-expert block-scaled GEMM
    sorted_idx, counts = oracle.permute_indices(ids, E)
    splits = counts.tolist()
    assert sum(splits) == T and min(splits) > 0
    xp = x.index_select(0, sorted_idx)
    qx_o, sx_o = oracle.tile_quant(xp)
    qw_o = torch.stack([oracle.block_quant(w[e])[0] for e in range(E)])
    sw_o = torch.stack([oracle.block_quant(w[e])[1] for e in range(E)])
    y_o = oracle.grouped_gemm_nt(qx_o, sx_o, qw_o, sw_o, splits)

    disp = MoETokenDispatcher(E, 1)
    q, s, goff = disp.token_permutation_fp8(x.to(dev), probs.to(dev), ids.to(dev))
    assert goff.cpu().tolist() == [0] + torch.tensor(splits).cumsum(0).tolist()
    assert torch.equal(disp.sorted_indices.cpu(), sorted_idx)
    assert torch.equal(q.view(torch.uint8).cpu(), qx_o.view(torch.uint8)) and torch.equal(s.cpu(), sx_o)
    qw, sw, _, _ = kernels.block_quant_batched(w.to(dev))
    assert torch.equal(qw.view(torch.uint8).cpu(), qw_o.view(torch.uint8)) and torch.equal(sw.cpu(), sw_o)
    y = kernels.grouped_gemm_nt(q, s, qw, sw, goff, out_dtype=torch.bfloat16)
    assert y.dtype == torch.bfloat16 and y.shape == (T, F)
    assert rel_err(y.cpu(), y_o) <= 1e-2
    # and against the plain matmul of the dequantised operands in float64 (the definition of the GEMM)
    off = 0
    for e, m in enumerate(splits):
        full = oracle.torch_dequant_tile(qx_o[off : off + m], sx_o[off : off + m]).double() @ oracle.torch_dequant_block(qw_o[e], sw_o[e]).double().t()
        assert rel_err(y[off : off + m].cpu(), full.float()) <= 1e-2
        off += m
    # back to token order (top-1, probability 1): every token's row returns to its place
    # (the dispatcher's own un-permutation restores the hidden size of its input, as the reference's
    # does, so the ffn-wide rows go through the kernel wrapper)
    out = kernels.unpermute_combine(y, disp.row_map, probs.to(dev), T, 1)
    assert torch.equal(out.cpu()[sorted_idx], y.cpu())


# ------------------------------------------------------------------------------------------
# boundary: device-side offsets, fp16 activations, registration hook
# ------------------------------------------------------------------------------------------
@pytest.mark.parametrize("bias", [False, True])
@pytest.mark.parametrize("fuse", [False, True])
def test_module_with_device_group_offsets_equals_host_splits(dev, bias, fuse):
    """forward(inp, None, group_offsets=...) runs the same kernels as forward(inp, m_splits): identical
    outputs and gradients, bit for bit, with bias, fused wgrad accumulation and under no_grad."""
    from atorch_amd import kernels
    from atorch_amd.grouped_linear import ATorchGroupedLinear

    E, K, N = 5, 256, 384
    splits = [130, 0, 257, 64, 91]
    M = sum(splits)
    torch.manual_seed(4)
    mods = [ATorchGroupedLinear(E, K, N, bias=bias, params_dtype=torch.bfloat16, device=dev,
                                fuse_wgrad_accumulation=fuse) for _ in range(2)]  # fmt: skip
    with torch.no_grad():
        for i in range(E):
            mods[1].get_parameter(f"weight{i}").copy_(mods[0].get_parameter(f"weight{i}"))
            if bias:
                b = randn_bf16((N,), 80 + i).to(dev)
                mods[0].get_parameter(f"bias{i}").copy_(b)
                mods[1].get_parameter(f"bias{i}").copy_(b)
            if fuse:
                mg = torch.rand(N, K, generator=torch.Generator().manual_seed(i)).to(dev)
                mods[0].get_parameter(f"weight{i}").main_grad = mg.clone()
                mods[1].get_parameter(f"weight{i}").main_grad = mg.clone()
    x = heavy_tailed((M, K), 21).to(dev)
    dy = randn_bf16((M, N), 22, std=1e-2).to(dev)
    goff = kernels.group_offsets_from_splits(splits, dev)
    xa, xb = x.clone().requires_grad_(True), x.clone().requires_grad_(True)
    oa = mods[0](xa, splits)
    ob = mods[1](xb, None, group_offsets=goff)
    assert torch.equal(oa, ob)
    oa.backward(dy)
    ob.backward(dy)
    assert torch.equal(xa.grad, xb.grad)
    for i in range(E):
        wa, wb = mods[0].get_parameter(f"weight{i}"), mods[1].get_parameter(f"weight{i}")
        if fuse:
            assert wa.grad is None and wb.grad is None and torch.equal(wa.main_grad, wb.main_grad)
        else:
            assert torch.equal(wa.grad, wb.grad)
        if bias:
            ga, gb = mods[0].get_parameter(f"bias{i}").grad, mods[1].get_parameter(f"bias{i}").grad
            torch.testing.assert_close(ga.float(), gb.float(), rtol=2e-2, atol=1e-4)  # order of an fp32 sum
    with torch.no_grad():
        assert torch.equal(mods[1](x, None, group_offsets=goff, is_first_microbatch=False), oa.detach())


def test_module_moved_to_the_device_runs_the_device_offset_path(dev):
    """A module built on the CPU and moved with .to(): its weights (and main_grads taken one by one from the
    allocator) may be adjacent in memory without sharing a storage.  The device-offset path and the fused
    weight-gradient accumulation then take their fallbacks and give the bits of a module built on the device."""
    from atorch_amd import kernels
    from atorch_amd.grouped_linear import ATorchGroupedLinear

    E, K, N = 3, 256, 128
    splits = [100, 0, 156]
    torch.manual_seed(6)
    ref = ATorchGroupedLinear(E, K, N, bias=False, params_dtype=torch.bfloat16, device=dev, fuse_wgrad_accumulation=True)
    mod = ATorchGroupedLinear(E, K, N, bias=False, params_dtype=torch.bfloat16, device="cpu", fuse_wgrad_accumulation=True)
    with torch.no_grad():
        for i in range(E):
            mod.get_parameter(f"weight{i}").copy_(ref.get_parameter(f"weight{i}").cpu())
    mod = mod.to(dev)
    for m in (ref, mod):
        for i in range(E):
            m.get_parameter(f"weight{i}").main_grad = torch.full((N, K), 0.25, device=dev)
    x = randn_bf16((sum(splits), K), 41).to(dev)
    dy = randn_bf16((sum(splits), N), 42, std=1e-2).to(dev)
    goff = kernels.group_offsets_from_splits(splits, dev)
    outs = []
    for m in (ref, mod):
        xg = x.clone().requires_grad_(True)
        for mb in (True, False):  # the second microbatch accumulates into main_grad
            out = m(xg, None, group_offsets=goff, is_first_microbatch=mb)
            out.backward(dy)
        outs.append((out.detach(), xg.grad, [m.get_parameter(f"weight{i}").main_grad for i in range(E)]))
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])
    for a, b in zip(outs[0][2], outs[1][2]):
        assert torch.equal(a, b)
    assert torch.all(outs[1][2][1] == 0)  # the empty group's gradient: written as zeros by the first microbatch


def test_stacked_weight_codes_follow_the_per_expert_caches(dev):
    """The two call forms of the module share one weight-code cache: after the m_splits form has requantised
    (first microbatch of a new step), a group_offsets call with is_first_microbatch=False uses the new codes."""
    from atorch_amd import kernels
    from atorch_amd.grouped_linear import ATorchGroupedLinear

    E, K, N = 2, 128, 128
    splits = [64, 64]
    torch.manual_seed(7)
    mod = ATorchGroupedLinear(E, K, N, bias=False, params_dtype=torch.bfloat16, device=dev)
    x = randn_bf16((128, K), 43).to(dev)
    goff = kernels.group_offsets_from_splits(splits, dev)
    with torch.no_grad():
        mod(x, None, group_offsets=goff, is_first_microbatch=True)
        for i in range(E):
            mod.get_parameter(f"weight{i}").mul_(2.0)  # the optimizer step
        want = mod(x, splits, is_first_microbatch=True)  # new step, host-split form: refreshes the per-expert caches
        got = mod(x, None, group_offsets=goff, is_first_microbatch=False)
    assert torch.equal(got, want)


def test_module_accepts_fp16_activations(dev, oracle):
    """fp16 inputs and parameters (quantized_grouped_linear.py:533-534): codes and scales come from the fp16
    values exactly; outputs and gradients are fp16 and within the GEMM tolerance of the oracle."""
    from atorch_amd import kernels
    from atorch_amd.grouped_linear import ATorchGroupedLinear

    E, K, N = 3, 256, 128
    splits = [100, 0, 156]
    torch.manual_seed(5)
    mod = ATorchGroupedLinear(E, K, N, bias=False, params_dtype=torch.float16, device=dev)
    x = randn_bf16((sum(splits), K), 31, dtype=torch.float16)
    dy = randn_bf16((sum(splits), N), 32, std=1e-2, dtype=torch.float16)
    q, s = kernels.tile_quant(x.to(dev))
    qo, so = oracle.tile_quant(x.float())
    assert torch.equal(q.view(torch.uint8).cpu(), qo.view(torch.uint8)) and torch.equal(s.cpu(), so)
    xg = x.to(dev).requires_grad_(True)
    out = mod(xg, splits)
    out.backward(dy.to(dev))
    assert out.dtype == torch.float16 and xg.grad.dtype == torch.float16
    ws = [mod.get_parameter(f"weight{i}").detach().float().cpu() for i in range(E)]
    orc = oracle.grouped_linear_fwd_bwd(x.float(), ws, splits, dy.float())
    assert rel_err(out.detach().float().cpu(), orc["out"]) <= TOL
    assert rel_err(xg.grad.float().cpu(), orc["dgrad"]) <= TOL
    for i in range(E):
        g = mod.get_parameter(f"weight{i}").grad
        assert g.dtype == torch.float16 and rel_err(g.float().cpu(), orc["wgrad"][i]) <= TOL


@pytest.mark.parametrize("variant", ["swiglu_separate", "swiglu_separate_kn", "gelu", "gelu_bias", "swiglu_bias"])
def test_grouped_mlp_bodies_match_oracle_composition(oracle, dev, variant):
    """The other bodies of compute_moe (grouped_gemm_moe.py:836-855): separate gate / up weights (:840-843),
    GELU (:449, :849) and the use_bias composition with bias_gather_add (:846-853), forward and backward,
    against the CPU composition: oracle grouped linear (+ bias), the reference's activation op under
    torch autograd, oracle grouped linear (+ bias).  Tolerances as for the merged SwiGLU body."""
    from atorch_amd.expert_mlp import grouped_mlp

    E, H, F, M = 3, 256, 384, 416
    splits = [200, 0, 216]
    glu = variant.startswith("swiglu")
    separate = "separate" in variant
    kn = variant.endswith("_kn")  # first weights stored [E, H, *] (transpose_w1 = False)
    use_bias = variant.endswith("_bias")
    n1 = 2 * F if glu else F
    x = randn_bf16((M, H), 1)
    w1 = randn_bf16((E, n1, H), 2, std=0.05)  # logical [E, N1, H]: gate rows on top of up rows
    w2 = randn_bf16((E, F, H), 3, std=0.05)
    dy = randn_bf16((M, H), 4, std=1e-2)
    b1 = randn_bf16((E, n1), 5, std=0.5) if use_bias else None
    b2 = randn_bf16((E, H), 6, std=0.5) if use_bias else None

    def store(w):  # logical [E, n, H] -> the parameter's storage orientation
        return (w.transpose(1, 2).contiguous() if kn else w.contiguous()).to(dev).requires_grad_(True)

    xg = x.to(dev).requires_grad_(True)
    w2g = w2.to(dev).requires_grad_(True)
    if separate:
        w1g, v1g = store(w1[:, :F]), store(w1[:, F:])
    else:
        w1g, v1g = store(w1), None
    b1g = b1.to(dev).requires_grad_(True) if use_bias else None
    b2g = b2.to(dev).requires_grad_(True) if use_bias else None
    out = grouped_mlp(xg, w1g, w2g, torch.tensor(splits), v1=v1g, b1=b1g, b2=b2g,
                      activation="swiglu" if glu else "gelu", transpose_w1=not kn)  # fmt: skip
    out.backward(dy.to(dev))

    r1 = oracle.grouped_linear_fwd_bwd(x, [w1[e] for e in range(E)], splits, biases=[b1[e] for e in range(E)] if use_bias else None)
    fc1 = r1["out"].bfloat16().requires_grad_(True)
    h = oracle.torch_swiglu(fc1) if glu else torch.nn.functional.gelu(fc1)
    w2_t = [w2[e].t().contiguous() for e in range(E)]
    r2 = oracle.grouped_linear_fwd_bwd(h.detach(), w2_t, splits, dy, biases=[b2[e] for e in range(E)] if use_bias else None)
    h.backward(r2["dgrad"].bfloat16())
    r1b = oracle.grouped_linear_fwd_bwd(x, [w1[e] for e in range(E)], splits, fc1.grad)

    def close(got, ref):
        got, ref = got.double(), ref.double()
        rms = ref.pow(2).mean().sqrt().clamp_min(1e-30)
        return float((got - ref).pow(2).mean().sqrt() / rms) < 1e-2 and rel_err(got, ref) < 0.15

    assert close(out.detach().cpu().float(), r2["out"])
    assert close(xg.grad.cpu().float(), r1b["dgrad"])

    def logical(g):  # gradient in storage orientation -> [E, n, H]
        g = g.cpu().float()
        return g.transpose(1, 2) if kn else g

    dw1 = torch.cat([logical(w1g.grad), logical(v1g.grad)], dim=1) if separate else logical(w1g.grad)
    for e in range(E):
        if splits[e] == 0:
            continue
        assert close(dw1[e], r1b["wgrad"][e])
        assert close(w2g.grad[e].cpu().float(), r2["wgrad"][e].t())
        if use_bias:
            assert close(b2g.grad[e].cpu().float(), r2["bgrad"][e])
            assert close(b1g.grad[e].cpu().float(), r1b["bgrad"][e])
    assert torch.all(w2g.grad[1] == 0) and torch.all(w1g.grad[1] == 0)
    if use_bias:
        assert torch.all(b1g.grad[1] == 0) and torch.all(b2g.grad[1] == 0)
    with torch.no_grad():
        out2 = grouped_mlp(x.to(dev), w1g.detach(), w2g.detach(), torch.tensor(splits), v1=v1g.detach() if separate else None,
                           b1=b1g, b2=b2g, activation="swiglu" if glu else "gelu", transpose_w1=not kn)  # fmt: skip
    assert torch.equal(out2, out.detach())

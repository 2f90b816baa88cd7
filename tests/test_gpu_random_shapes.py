"""Seeded sweeps over random shapes and routings: the grouped GEMMs against the float64 definition
(triton_kernel.py:179-190 for one group; quantized_grouped_linear.py:243-253 for the weight gradient), and the
row-wise + transposed quantisers of ragged groups and the dispatch kernels against the oracle, bit for bit.

The parametrised tests pick their shapes by hand; this one draws them: group counts from 1 to 130, empty
groups, a few rows or tens of thousands (both tile configurations and every scale path of the kernel: batches
of eight contraction blocks with 16-byte and with 4-byte loads, single loads below eight blocks), bias or
none, bf16 or fp32 output, and the weight gradient of the same routing with and without accumulation."""
import random

import pytest
import torch

from helpers import rel_err

pytestmark = pytest.mark.gpu
TILE = 128


def _deq_tile(q, s):
    return q.float() * s.repeat_interleave(TILE, -1)


def _deq_block(q, s):
    return q.float() * s.repeat_interleave(TILE, -2).repeat_interleave(TILE, -1)


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_grouped_gemms_on_random_shapes(seed):
    from atorch_amd import kernels

    dev = torch.device("cuda:0")
    rng = random.Random(seed)
    torch.manual_seed(seed)
    for case in range(8):
        E = rng.choice([1, 2, 3, 5, 8, 17, 64, 130])
        N = TILE * rng.choice([1, 2, 3, 4, 5, 8, 11])
        K = TILE * rng.choice([1, 2, 3, 4, 8, 9, 11, 16, 22])
        M = rng.randint(20000, 70000) if rng.random() < 0.5 else rng.randint(1, 3000)
        cuts = sorted(rng.randint(0, M) for _ in range(E - 1))
        if E > 3 and rng.random() < 0.5:
            cuts[1] = cuts[0]  # an empty group
        bounds = [0] + cuts + [M]
        splits = [bounds[i + 1] - bounds[i] for i in range(E)]
        use_bias = rng.random() < 0.4
        out_dtype = rng.choice([torch.bfloat16, torch.float32])
        what = f"seed {seed} case {case}: M={M} N={N} K={K} E={E} out={out_dtype} bias={use_bias}"
        print(what, flush=True)

        x = torch.randn(M, K, device=dev).bfloat16()
        w = (torch.randn(E, N, K, device=dev) * 0.02).bfloat16()
        bias = torch.randn(E, N, device=dev).bfloat16() if use_bias else None
        qx, sx = kernels.tile_quant(x)
        qw, sw, _, _ = kernels.block_quant_batched(w)
        goff = kernels.group_offsets_from_splits(splits, dev)
        y = kernels.grouped_gemm_nt(qx, sx, qw, sw, goff, out_dtype=out_dtype, bias=bias)
        xd = _deq_tile(qx, sx).double()
        ref = torch.zeros(M, N, dtype=torch.float64, device=dev)
        row = 0
        for e, m in enumerate(splits):
            if m:
                ref[row : row + m] = xd[row : row + m] @ _deq_block(qw[e], sw[e]).double().t()
                if use_bias:
                    ref[row : row + m] += bias[e].double()
            row += m
        err = rel_err(y.cpu(), ref.float().cpu())
        assert err <= (1e-2 if out_dtype == torch.bfloat16 else 5e-4), (what, err)

        if M > 40000 or N * K * E > 32 * 1024 * 1024:
            continue
        dy = (torch.randn(M, N, device=dev) * 0.01).bfloat16()
        blocked = (seed + case) % 2 == 0  # the two layouts of the transposed codes in turn
        _, _, qxt, sxt = kernels.tile_quant_dual_grouped(x, goff, E, rowwise=False, blocked=blocked)
        _, _, qdt, sdt = kernels.tile_quant_dual_grouped(dy, goff, E, ld_t=kernels.qt_ld(qxt), rowwise=False, blocked=blocked)
        base = torch.randn(E, N, K, device=dev)
        acc = base.clone()
        kernels.grouped_gemm_wgrad(qdt, sdt, qxt, sxt, goff, out=acc, accumulate=True)
        dw = kernels.grouped_gemm_wgrad(qdt, sdt, qxt, sxt, goff, out_dtype=torch.float32)
        qxt, qdt = kernels.qt_rows(qxt), kernels.qt_rows(qdt)  # [rows, ld_t] for the definition below
        refw = torch.zeros(E, N, K, dtype=torch.float64, device=dev)
        col = 0  # groups are padded to whole 128-token blocks along the transposed operands' columns
        for e, m in enumerate(splits):
            pad = (m + TILE - 1) // TILE * TILE
            if m:
                a = qdt[:, col : col + pad].float() * sdt[col // TILE : (col + pad) // TILE].t().repeat_interleave(TILE, 1)
                c = qxt[:, col : col + pad].float() * sxt[col // TILE : (col + pad) // TILE].t().repeat_interleave(TILE, 1)
                refw[e] = a.double() @ c.double().t()
            col += pad
        refw = refw.float().cpu()
        assert rel_err(dw.cpu(), refw) <= 5e-4, what
        assert rel_err((acc - base).cpu(), refw) <= 2e-3, what  # the difference of two fp32 numbers near 1
        for e, m in enumerate(splits):
            if m == 0:  # an empty group: zeros, and with accumulation the old values untouched
                assert dw[e].abs().max() == 0 and torch.equal(acc[e], base[e]), what


@pytest.mark.parametrize("seed", [21, 22])
def test_dual_quantisers_on_random_shapes(oracle, seed):
    """Row-wise + transposed quantisation of ragged groups, plain and with the activations fused in, over drawn
    shapes (triton_kernel.py:94-140 per row; the transposed codes follow quantized_grouped_linear.py:75-77 per
    group).  Feature counts of 1024 and more take the workgroup order that deals eight neighbouring column
    tiles to one XCD, with and without a remainder of token tiles outside that order."""
    from atorch_amd import kernels

    dev = torch.device("cuda:0")
    rng = random.Random(seed)
    for case in range(6):
        F = TILE * rng.choice([1, 3, 8, 8, 16, 24])
        E = rng.choice([1, 2, 3, 5, 9, 40])
        M = rng.randint(1, 2500)
        cuts = sorted(rng.randint(0, M) for _ in range(E - 1))
        if E > 3 and rng.random() < 0.5:
            cuts[1] = cuts[0]
        bounds = [0] + cuts + [M]
        splits = [bounds[i + 1] - bounds[i] for i in range(E)]
        what = f"seed {seed} case {case}: M={M} F={F} E={E}"
        print(what, flush=True)
        g = torch.Generator().manual_seed(seed * 100 + case)
        x = (torch.randn(M, F, generator=g) * torch.randn(M, 1, generator=g).exp()).bfloat16()
        goff = kernels.group_offsets_from_splits(splits, dev)
        ptot = oracle.padded_offsets(splits)[-1]

        blocked = (seed + case) % 2 == 0  # the fused kernels write the two layouts of the transposed codes in turn

        def same_as_plain(res, h):
            # the fused kernel's codes and scales are those of the plain kernel on the fused kernel's own values
            q, s, q_t, s_t = res
            q2, s2, q_t2, s_t2 = kernels.tile_quant_dual_grouped(h, goff, E, ld_t=kernels.qt_ld(q_t))
            assert torch.equal(q.view(torch.uint8), q2.view(torch.uint8)) and torch.equal(s, s2), what
            assert torch.equal(kernels.qt_rows(q_t).view(torch.uint8)[:, :ptot], q_t2.view(torch.uint8)[:, :ptot]), what
            assert torch.equal(s_t[: ptot // TILE], s_t2[: ptot // TILE]), what

        q, s, q_t, s_t = kernels.tile_quant_dual_grouped(x.to(dev), goff, E)
        qo, so = oracle.tile_quant(x)
        qto, sto = oracle.tile_quant_t_grouped(x, splits, ld_t=q_t.shape[1])
        assert torch.equal(q.view(torch.uint8).cpu(), qo) and torch.equal(s.cpu(), so), what
        assert torch.equal(q_t.view(torch.uint8).cpu()[:, :ptot], qto[:, :ptot]), what
        assert torch.equal(s_t.cpu()[: ptot // TILE], sto[: ptot // TILE]), what

        fc1 = torch.cat([x, (torch.randn(M, F, generator=g)).bfloat16()], dim=1).contiguous().to(dev)
        dh = (torch.randn(M, F, generator=g) * 0.1).bfloat16().to(dev)
        *res, h = kernels.swiglu_tile_quant_dual_grouped(fc1, goff, E, return_activation=True, blocked=blocked)
        same_as_plain(res, h)
        *res, h = kernels.gelu_tile_quant_dual_grouped(x.to(dev), goff, E, return_activation=True, blocked=blocked)
        same_as_plain(res, h)
        *res, gx = kernels.gelu_tile_quant_dual_grouped(x.to(dev), goff, E, dh=dh, return_activation=True, blocked=blocked)
        same_as_plain(res, gx)
        *res, gfc1 = kernels.swiglu_bwd_tile_quant_dual_grouped(dh, fc1, goff, E, return_grad=True, blocked=blocked)
        same_as_plain(res, gfc1)
        assert torch.equal(gfc1.cpu(), oracle.swiglu_bwd(dh.cpu(), fc1.cpu())) or rel_err(
            gfc1.float().cpu(), oracle.swiglu_bwd(dh.cpu(), fc1.cpu()).float()
        ) < 2.0**-6, what  # one or two bf16 units in the last place on a few inputs (hardware exp2 and reciprocal)


@pytest.mark.parametrize("seed", [31, 32])
def test_dispatch_kernels_on_random_shapes(oracle, seed):
    """Router preprocessing, the fused permute + quantise and the weighted combine over drawn token counts, widths,
    expert counts and top-k (token_dispatcher.py:89-161), bit for bit against the oracle."""
    from atorch_amd import kernels
    from helpers import topk_routing

    dev = torch.device("cuda:0")
    rng = random.Random(seed)
    for case in range(6):
        E = rng.choice([2, 3, 8, 17, 64, 200])
        k = rng.randint(1, min(E, 9))
        T = rng.randint(1, 1500)
        H = TILE * rng.choice([1, 2, 5, 8, 20, 40, 56])
        probs_dtype = rng.choice([torch.bfloat16, torch.float32])
        what = f"seed {seed} case {case}: T={T} H={H} E={E} k={k} probs={probs_dtype}"
        print(what, flush=True)
        g = torch.Generator().manual_seed(seed * 100 + case)
        idx, probs = topk_routing(T, E, k, seed=seed * 100 + case, zipf_s=rng.choice([None, 1.2]))
        probs = probs.to(probs_dtype)
        x = (torch.randn(T, H, generator=g) * torch.randn(T, 1, generator=g).exp()).bfloat16()

        sorted_idx, row_map, goff = kernels.moe_preprocess(idx.to(dev), E)
        so, counts = oracle.permute_indices(idx, E)
        assert torch.equal(sorted_idx.cpu(), so), what
        assert torch.equal((goff[1:] - goff[:-1]).cpu(), counts.to(torch.int64)), what
        q, s = kernels.permute_tile_quant(x.to(dev), row_map, k, T * k)
        xp, _, _ = oracle.permute(x, idx, E)
        qo, sco = oracle.tile_quant(xp)
        assert torch.equal(q.view(torch.uint8).cpu(), qo) and torch.equal(s.cpu(), sco), what
        assert torch.equal(kernels.permute_rows(x.to(dev), row_map, k, T * k).cpu(), xp), what

        y = torch.randn(T * k, H, generator=g).bfloat16()
        out = kernels.unpermute_combine(y.to(dev), row_map, probs.to(dev), T, k)
        ref = oracle.unpermute(y, so, probs)
        assert out.dtype == ref.dtype and torch.equal(out.cpu(), ref), what

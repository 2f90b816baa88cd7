"""Seeded sweep of the grouped GEMMs over random shapes and routings against the float64 definition
(triton_kernel.py:179-190 for one group; quantized_grouped_linear.py:243-253 for the weight gradient).

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
        _, _, qxt, sxt = kernels.tile_quant_dual_grouped(x, goff, E, rowwise=False)
        _, _, qdt, sdt = kernels.tile_quant_dual_grouped(dy, goff, E, ld_t=qxt.shape[1], rowwise=False)
        base = torch.randn(E, N, K, device=dev)
        acc = base.clone()
        kernels.grouped_gemm_wgrad(qdt, sdt, qxt, sxt, goff, out=acc, accumulate=True)
        dw = kernels.grouped_gemm_wgrad(qdt, sdt, qxt, sxt, goff, out_dtype=torch.float32)
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

#!/usr/bin/env python3
"""Writes the golden vectors under tests/golden/ (small .npz files: inputs and expected outputs).

    python tests/golden/make_fixtures.py

The reference keeps no stored vectors for this path: its cases are executable tests that need a
GPU (scaled_linear_test.py:116-133, 244-297, 305-319; test_quantized_grouped_linear.py:607-655).
The vectors here re-create those cases (same values, same shapes where they are small, scaled-down
shapes otherwise) plus seeded random cases, with expected outputs computed by the CPU oracle.
tests/test_golden.py checks them three ways: the oracle must reproduce them, an independent
exact-rational rounder must agree with the stored codes, and the HIP kernels must match them.

bf16 tensors are stored as their uint16 bit patterns, fp8 codes as uint8.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

from helpers import heavy_tailed, ragged_splits, randn_bf16, topk_routing  # noqa: E402

from oracle import oracle as O  # noqa: E402

TILE = 128


def bits(t):
    assert t.dtype == torch.bfloat16
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def save(name, **arrays):
    path = os.path.join(HERE, name + ".npz")
    np.savez_compressed(path, **{k: np.asarray(v) for k, v in arrays.items()})
    print(f"{name}.npz: {os.path.getsize(path)} bytes")


def quant_known_answers():
    """scaled_linear_test.py:305-319 (ones / 1000 / -512 rows), :116-133 (outlier 1e4, zeros)."""
    x = torch.ones(8, 256, dtype=torch.bfloat16)
    x[1] = 1000.0
    x[2] = -512.0
    x[3] = 0.0
    x[4] = randn_bf16((256,), 1)
    x[4, 7] = 1e4  # an outlier flushes its neighbours towards zero
    x[5, :128] = 0.0  # one zero tile beside a non-zero one
    x[6] = randn_bf16((256,), 2) * 1e-30  # tiny values: scale is subnormal-free but small
    x[7] = heavy_tailed((1, 256), 3)[0]
    q, s = O.tile_quant(x)
    xb = x[:, :128].repeat(16, 1).contiguous()  # 128 x 128 block made of the same rows
    qb, sb = O.block_quant(xb)
    save("quant_known_answers", x=bits(x), q=q.numpy(), s=s.numpy(), xb=bits(xb), qb=qb.numpy(), sb=sb.numpy())


def quant_random():
    x = heavy_tailed((64, 256), 11)
    q, s = O.tile_quant(x)
    q_eps, s_eps = O.tile_quant(x, eps=0.5)
    w = randn_bf16((256, 128), 12, std=0.02)
    qw, sw = O.block_quant(w)
    xf = randn_bf16((40, 256), 13, dtype=torch.float32)
    qf, sf = O.tile_quant(xf)
    save("quant_random", x=bits(x), q=q.numpy(), s=s.numpy(), q_eps=q_eps.numpy(), s_eps=s_eps.numpy(),
         w=bits(w), qw=qw.numpy(), sw=sw.numpy(), xf=xf.numpy(), qf=qf.numpy(), sf=sf.numpy())  # fmt: skip


def quant_transposed_grouped():
    """Transposed 1x128 quantisation along the tokens of ragged groups: partial tiles, an empty
    group, a group that is a multiple of 128 (scaled_linear.py:402-414 per group)."""
    splits = [100, 0, 300, 128, 16]
    x = heavy_tailed((sum(splits), 128), 21)
    q, s = O.tile_quant(x)
    q_t, s_t = O.tile_quant_t_grouped(x, splits)
    save("quant_transposed_grouped", x=bits(x), splits=np.array(splits), q=q.numpy(), s=s.numpy(),
         q_t=q_t.numpy(), s_t=s_t.numpy())  # fmt: skip


def grouped_linear():
    """A scaled-down test_quantized_grouped_linear.py:607-655: 3 experts, splits that are multiples
    of 16 with one empty group, forward + dgrad + wgrad from bf16 inputs."""
    E, K, N = 3, 256, 128
    splits = [176, 0, 80]
    M = sum(splits)
    x = randn_bf16((M, K), 31)
    ws = [randn_bf16((N, K), 32 + i, std=0.02) for i in range(E)]
    dy = randn_bf16((M, N), 40, std=1e-2)
    r = O.grouped_linear_fwd_bwd(x, ws, splits, dy)
    # the operands of the three grouped GEMMs, so that a GEMM can be checked on stored fp8 inputs
    qx, sx = O.tile_quant(x)
    qw = torch.stack([O.block_quant(w)[0] for w in ws])
    sw = torch.stack([O.block_quant(w)[1] for w in ws])
    y32 = O.grouped_gemm_nt(qx, sx, qw, sw, splits)
    qdy_t, sdy_t = O.tile_quant_t_grouped(dy, splits)
    qx_t, sx_t = O.tile_quant_t_grouped(x, splits)
    dw32 = O.grouped_gemm_wgrad(qdy_t, sdy_t, qx_t, sx_t, splits)
    assert all(torch.equal(dw32[e], r["wgrad"][e]) for e in range(E))
    save("grouped_linear", x=bits(x), w=np.stack([bits(w) for w in ws]), dy=bits(dy), splits=np.array(splits),
         out=bits(r["out"].bfloat16()), dgrad=bits(r["dgrad"].bfloat16()),
         qx=qx.numpy(), sx=sx.numpy(), qw=qw.numpy(), sw=sw.numpy(), y32=y32.numpy(),
         qdy_t=qdy_t.numpy(), sdy_t=sdy_t.numpy(), qx_t=qx_t.numpy(), sx_t=sx_t.numpy(), dw32=dw32.numpy())  # fmt: skip


def permute_combine():
    """token_dispatcher.py:89-161 on 48 tokens, top-3 into 5 experts."""
    T, E, k, H = 48, 5, 3, 128
    idx, probs = topk_routing(T, E, k, seed=51)
    tokens = randn_bf16((T, H), 52)
    permuted, sorted_idx, counts = O.permute(tokens, idx, E)
    y = randn_bf16((T * k, H), 53)
    out_bf16 = O.unpermute(y, sorted_idx, probs.bfloat16())
    out_f32 = O.unpermute(y, sorted_idx, probs.float())
    out_plain = O.unpermute(y, sorted_idx, None)
    save("permute_combine", tokens=bits(tokens), idx=idx.numpy(), probs=probs.float().numpy(),
         permuted=bits(permuted), sorted_idx=sorted_idx.numpy(), counts=counts.numpy(), y=bits(y),
         out_bf16=bits(out_bf16), out_f32=out_f32.numpy(), out_plain=bits(out_plain))  # fmt: skip


if __name__ == "__main__":
    O.build()
    quant_known_answers()
    quant_random()
    quant_transposed_grouped()
    grouped_linear()
    permute_combine()

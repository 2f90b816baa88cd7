"""The entry point that allocates nothing, aamd_grouped_gemm_fp8_nt_static: the tile prefix lives in a
static device array of the library instead of a caller workspace.  Called through the C ABI with raw
ctypes and compared bit for bit with aamd_grouped_gemm_fp8_nt on the same operands and, within the GEMM
tolerance, with the float64 dequantise-and-matmul definition, twice in a row: first a launch that takes the
256 x 256 tiles (a prefix of 256-row tiles in the scratch), then a smaller one with fewer groups and rows on the
128 x 128 tiles, so stale scratch contents would show."""
import ctypes

import pytest
import torch

from helpers import TILE, ragged_splits, randn_bf16, rel_err

pytestmark = pytest.mark.gpu


def _case(dev, M, N, K, E, seed, bias):
    from atorch_amd import kernels

    x = randn_bf16((M, K), seed).to(dev)
    w = randn_bf16((E, N, K), seed + 1, std=0.02).to(dev)
    qx, sx = kernels.tile_quant(x)
    qw, sw, _, _ = kernels.block_quant_batched(w)
    splits = ragged_splits(M, E, seed=seed, multiple=1)
    goff = kernels.group_offsets_from_splits(splits, dev)
    b = randn_bf16((E, N), seed + 2).to(dev) if bias else None
    return qx, sx, qw, sw, goff, b, splits


def _call(fn, with_ws, ops, M, N, K, E, out, dev):
    from atorch_amd import _lib

    qx, sx, qw, sw, goff, bias, _ = ops
    vp = ctypes.c_void_p
    args = [vp(qx.data_ptr()), K, vp(sx.data_ptr()), vp(qw.data_ptr()), vp(sw.data_ptr()), 0, vp(goff.data_ptr()), E]
    ws = None
    if with_ws:
        ws = torch.empty(E + 1, dtype=torch.int32, device=dev)
        args.append(vp(ws.data_ptr()))
    args += [M, N, K, vp(out.data_ptr()), _lib.BF16, N,
             vp(bias.data_ptr()) if bias is not None else None, _lib.BF16 if bias is not None else _lib.NONE,
             vp(torch.cuda.current_stream().cuda_stream)]  # fmt: skip
    rc = fn(*args)
    assert rc == _lib.OK, _lib.lib().aamd_last_error()
    return ws


def test_static_scratch_entry_point_matches_the_workspace_one(dev):
    from atorch_amd import _lib

    L = _lib.lib()
    # first a large-tile launch with many groups (at least 512 tiles of 256 x 256 and eight contraction blocks
    # select that configuration), then a smaller one with fewer groups and rows
    for (M, N, K, E, seed, bias) in [(40000, 1024, 1024, 130, 1, True), (700, 256, 384, 5, 2, False)]:
        ops = _case(dev, M, N, K, E, seed, bias)
        assert 0 in ops[-1]
        ref = torch.full((M, N), 7.0, dtype=torch.bfloat16, device=dev)
        got = torch.full((M, N), 7.0, dtype=torch.bfloat16, device=dev)
        _call(L.aamd_grouped_gemm_fp8_nt, True, ops, M, N, K, E, ref, dev)
        free_before = torch.cuda.mem_get_info()[0]
        _call(L.aamd_grouped_gemm_fp8_nt_static, False, ops, M, N, K, E, got, dev)
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before, "the call must not allocate device memory"
        assert torch.equal(got, ref)
        assert not torch.all(got == 7.0)
        # the definition, in float64 on the device: dequantised rows times the dequantised weight of their group
        qx, sx, qw, sw, _, b, splits = ops
        xd = (qx.float() * sx.repeat_interleave(TILE, 1)).double()
        want = torch.full((M, N), 7.0, dtype=torch.float64, device=dev)
        off = 0
        for e, m in enumerate(splits):
            if m:
                wd = (qw[e].float() * sw[e].repeat_interleave(TILE, 0).repeat_interleave(TILE, 1)).double()
                want[off : off + m] = xd[off : off + m] @ wd.t() + (b[e].double() if b is not None else 0.0)
            off += m
        assert rel_err(got.float().cpu(), want.float().cpu()) <= 1e-2


def test_static_scratch_entry_point_rejects_too_many_groups(dev):
    from atorch_amd import _lib

    L = _lib.lib()
    one = ctypes.c_void_p(16)
    rc = L.aamd_grouped_gemm_fp8_nt_static(one, 128, one, one, one, 0, one, 5000, 8, 128, 128, one, _lib.BF16, 128,
                                           None, _lib.NONE, None)
    assert rc == _lib.ERR_ARG and b"static scratch" in L.aamd_last_error()

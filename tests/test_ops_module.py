"""``atorch_amd.ops``: the module the reference's dense FP8 wrappers load through the
``FP8_GEMM_MODULE_OPS`` environment variable (atorch/modules/fp8/cuda_kernel.py:7-81)."""
import inspect

import pytest
import torch

from helpers import randn_bf16, rel_err


def test_ops_module_exposes_the_names_the_reference_calls():
    from atorch_amd import ops

    for name in ("quantize_vector_blockwise", "quantize_square_blockwise", "fp8_gemm_blockwise",
                 "cutlass_gemm_fp8_blockwise"):  # fmt: skip
        assert callable(getattr(ops, name))
    assert {m.name for m in ops.Backend} == {"CUTLASS", "CUBLAS"}
    # keyword names used at the reference's call sites (cuda_kernel.py:30-38, 53-61, 69-81)
    q = inspect.signature(ops.quantize_vector_blockwise).parameters
    assert list(q)[:3] == ["x", "dtype", "block_size"]
    assert {"return_transpose", "eps", "pow_2_scale", "backend"} <= set(q)
    g = inspect.signature(ops.fp8_gemm_blockwise).parameters
    assert list(g)[:5] == ["a", "a_s", "b", "b_s", "dtype"]
    assert {"out", "accumulate", "use_split_accumulator", "is_a_1d_scaled", "is_b_1d_scaled"} <= set(g)
    with pytest.raises(NotImplementedError):
        ops.quantize_vector_blockwise(torch.zeros(1, 128), torch.float8_e4m3fn, 128, pow_2_scale=True)
    with pytest.raises(NotImplementedError):
        ops.quantize_square_blockwise(torch.zeros(128, 128), torch.float8_e5m2, 128)


@pytest.mark.gpu
def test_dense_linear_recipe_through_ops_module(oracle, dev):
    """Forward, dgrad and wgrad of a dense linear the way ScaledLinear's tile/block recipe drives the
    wrappers (scaled_linear.py:359-365, 402-446), against the oracle."""
    from atorch_amd import ops

    M, K, N = 384, 256, 512
    x, w, dy = randn_bf16((M, K), 1), randn_bf16((N, K), 2, std=0.02), randn_bf16((M, N), 3, std=1e-2)
    fp8 = torch.float8_e4m3fn
    qx, sx, qx_t, sx_t = ops.quantize_vector_blockwise(x.to(dev), fp8, 128, return_transpose=True)
    qw, sw, qw_t, sw_t = ops.quantize_square_blockwise(w.to(dev), fp8, 128, return_transpose=True)
    qdy, sdy, qdy_t, sdy_t = ops.quantize_vector_blockwise(dy.to(dev), fp8, 128, return_transpose=True)
    oq, os_ = oracle.tile_quant(x)
    assert torch.equal(qx.view(torch.uint8).cpu(), oq) and torch.equal(sx.cpu(), os_)
    oqt, ost = oracle.tile_quant(x.t().contiguous())
    assert torch.equal(qx_t.view(torch.uint8).cpu(), oqt) and torch.equal(sx_t.cpu(), ost)
    owq, ows = oracle.block_quant(w)
    assert torch.equal(qw.view(torch.uint8).cpu(), owq) and torch.equal(sw_t.cpu(), ows.t().contiguous())
    ref = oracle.grouped_linear_fwd_bwd(x, [w], [M], dy)
    y = ops.cutlass_gemm_fp8_blockwise(qx, sx, qw, sw, torch.bfloat16, out=None, accumulate=False,
                                       use_split_accumulator=True, is_a_1d_scaled=True, is_b_1d_scaled=False)  # fmt: skip
    assert rel_err(y.cpu().float(), ref["out"]) < 1e-2
    dx = ops.fp8_gemm_blockwise(qdy, sdy, qw_t, sw_t, torch.bfloat16)
    assert rel_err(dx.cpu().float(), ref["dgrad"]) < 1e-2
    out = torch.empty(N, K, dtype=torch.float32, device=dev)
    dw = ops.fp8_gemm_blockwise(qdy_t, sdy_t, qx_t, sx_t, torch.float32, out=out, is_b_1d_scaled=True)
    assert dw is out and rel_err(dw.cpu(), ref["wgrad"][0]) < 5e-4
    q1, s1, n1, n2 = ops.quantize_vector_blockwise(x.to(dev).view(3, 128, K), fp8, 128)
    assert n1 is None and n2 is None and q1.shape == (3, 128, K) and s1.shape == (3, 128, K // 128)


@pytest.mark.gpu
def test_dense_wgrad_through_ops_module_at_a_size_that_takes_large_tiles(dev):
    """The dense weight gradient dW = dY^T X of the tile/block recipe (scaled_linear.py:431-446) with
    an 8192 x 4096 weight: both operands 1x128-scaled along the tokens, large-tile configuration;
    against the float64 definition evaluated on the device."""
    from atorch_amd import ops

    M, K, N = 2048, 4096, 8192
    fp8 = torch.float8_e4m3fn
    x, dy = randn_bf16((M, K), 5).to(dev), randn_bf16((M, N), 6, std=1e-2).to(dev)
    _, _, qx_t, sx_t = ops.quantize_vector_blockwise(x, fp8, 128, return_transpose=True)
    _, _, qdy_t, sdy_t = ops.quantize_vector_blockwise(dy, fp8, 128, return_transpose=True)
    assert qx_t.shape == (K, M) and sx_t.shape == (K, M // 128)
    dw = ops.fp8_gemm_blockwise(qdy_t, sdy_t, qx_t, sx_t, torch.float32, is_b_1d_scaled=True)

    def deq(q, s):
        return (q.float() * s.repeat_interleave(128, -1)).double()

    ref = deq(qdy_t, sdy_t) @ deq(qx_t, sx_t).t()
    assert dw.shape == (N, K) and rel_err(dw.cpu(), ref.float().cpu()) < 5e-4

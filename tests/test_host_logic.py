"""Host-side logic without a GPU: the grouped linear's autograd function and module run on CPU
tensors through an oracle-backed ``quantize_op`` (the plugin interface), and the view-recognition
helpers of the HIP operator are exercised on CPU tensors (pointer arithmetic only)."""
import os

import pytest
import torch

from helpers import TILE, OracleQuantizeOp, randn_bf16, ragged_splits


def _params(op=None):
    from atorch_amd.quantization import QLinearParams

    return QLinearParams(quantize_op=op or OracleQuantizeOp())


def _module(E, K, N, dtype=torch.bfloat16, **kw):
    from atorch_amd.grouped_linear import ATorchGroupedLinear

    torch.manual_seed(0)
    return ATorchGroupedLinear(E, K, N, params_dtype=dtype, device="cpu", qlinear_params=_params(), **kw)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("batch", [1, 2])
def test_forward_backward_match_oracle(oracle, dtype, batch):
    """Shapes of the reference test (hidden 256 -> 128, splits that are multiples of 16 with one
    empty group, [seq, batch, hidden] input: test_quantized_grouped_linear.py:607-641)."""
    E, K, N, seq = 3, 256, 128, 256
    mod = _module(E, K, N, dtype=dtype, bias=False)
    splits = [m * batch for m in ragged_splits(seq, E, seed=1, multiple=16)]
    assert 0 in splits
    x = randn_bf16((seq, batch, K), 3, dtype=dtype).requires_grad_(True)
    out = mod(x, splits)
    assert out.shape == (seq, batch, N) and out.dtype == dtype
    out.sum().backward()
    ws = [getattr(mod, f"weight{i}").detach() for i in range(E)]
    ref = oracle.grouped_linear_fwd_bwd(x.detach(), ws, splits, torch.ones(seq * batch, N, dtype=dtype))
    assert torch.equal(out.detach().view(-1, N), ref["out"].to(dtype))
    assert torch.equal(x.grad.view(-1, K), ref["dgrad"].to(dtype))
    for i in range(E):
        assert torch.equal(getattr(mod, f"weight{i}").grad, ref["wgrad"][i].to(dtype))
    assert torch.all(getattr(mod, f"weight{splits.index(0)}").grad == 0)


def test_bias_and_return_bias(oracle):
    E, K, N = 2, 128, 128
    splits = [48, 80]
    x = randn_bf16((128, K), 1)
    mod = _module(E, K, N, bias=True)
    with torch.no_grad():
        for i in range(E):
            getattr(mod, f"bias{i}").copy_(randn_bf16((N,), 10 + i))
    ws = [getattr(mod, f"weight{i}").detach() for i in range(E)]
    bs = [getattr(mod, f"bias{i}").detach() for i in range(E)]
    xg = x.clone().requires_grad_(True)
    out = mod(xg, splits)
    ref = oracle.grouped_linear_fwd_bwd(x, ws, splits, torch.ones(128, N, dtype=torch.bfloat16), biases=bs)
    assert torch.equal(out.detach(), ref["out"].bfloat16())
    out.sum().backward()
    for i in range(E):
        assert torch.equal(getattr(mod, f"bias{i}").grad.float(), ref["bgrad"][i].bfloat16().float())
    mod2 = _module(E, K, N, bias=True, return_bias=True)
    out2, biases = mod2(x, splits)
    assert len(biases) == E and out2.shape == (128, N)
    ref2 = oracle.grouped_linear_fwd_bwd(x, [getattr(mod2, f"weight{i}").detach() for i in range(E)], splits)
    assert torch.equal(out2.detach(), ref2["out"].bfloat16())


def test_weight_cache_and_env_flag(monkeypatch):
    """Weights are re-quantised when is_first_microbatch is True / None and served from the cache
    otherwise; FORCE_QUANTIZE_PER_MICROBATCH re-quantises always and leaves the cache alone
    (quantized_grouped_linear.py:103-134).  Results are identical either way."""
    E, K, N = 2, 128, 128
    splits = [64, 64]
    x = randn_bf16((128, K), 2)
    mod = _module(E, K, N, bias=False)
    op = mod.qlinear_params.quantize_op
    n_x = E  # per forward: one quantize per group of x
    o1 = mod(x, splits, is_first_microbatch=True)
    assert op.calls["quantize"] == n_x + E
    cached = [c.data for c in mod.weight_qresult_caches]
    assert all(c is not None for c in cached) and mod.weight_qresult_caches[0].data_t is not None
    o2 = mod(x, splits, is_first_microbatch=False)
    assert op.calls["quantize"] == 2 * n_x + E  # weights came from the cache
    assert torch.equal(o1, o2)
    o3 = mod(x, splits, is_first_microbatch=None)
    assert op.calls["quantize"] == 3 * n_x + 2 * E
    assert torch.equal(o1, o3)
    monkeypatch.setenv("FORCE_QUANTIZE_PER_MICROBATCH", "1")
    before = [c.data for c in mod.weight_qresult_caches]
    o4 = mod(x, splits, is_first_microbatch=False)
    assert op.calls["quantize"] == 4 * n_x + 3 * E
    assert all(a is b for a, b in zip(before, [c.data for c in mod.weight_qresult_caches]))
    assert torch.equal(o1, o4)
    monkeypatch.setenv("FORCE_QUANTIZE_PER_MICROBATCH", "maybe")
    with pytest.raises(ValueError):
        mod(x, splits)


def test_no_grad_path_skips_transposes():
    E, K, N = 2, 128, 128
    mod = _module(E, K, N, bias=False)
    x = randn_bf16((128, K), 4)
    with torch.no_grad():
        out = mod(x, [100, 28], is_first_microbatch=True)
    assert out.requires_grad is False
    assert mod.weight_qresult_caches[0].data_t is None
    # a later grad-enabled call finds the cache without transposes and re-quantises
    out2 = mod(x.clone().requires_grad_(True), [100, 28], is_first_microbatch=False)
    assert mod.weight_qresult_caches[0].data_t is not None
    assert torch.equal(out, out2.detach())


def test_fused_wgrad_accumulation(oracle):
    """accumulate = fuse and not is_first_microbatch (or = fuse when the flag is None); the result
    lands in main_grad and autograd sees no grad (quantized_grouped_linear.py:225-241;
    test_quantized_grouped_linear.py:648-654, 559-599: cumulative sum of the unfused wgrads)."""
    E, K, N = 2, 128, 128
    splits = [80, 48]
    mod = _module(E, K, N, bias=False, fuse_wgrad_accumulation=True)
    ws = [getattr(mod, f"weight{i}") for i in range(E)]
    g = torch.Generator().manual_seed(0)
    init = [torch.rand(N, K, generator=g) for _ in range(E)]
    for w, m in zip(ws, init):
        w.main_grad = m.clone()
    xs = [randn_bf16((128, K), 5 + i) for i in range(3)]
    unfused = []
    for x in xs:
        r = oracle.grouped_linear_fwd_bwd(x, [w.detach() for w in ws], splits, torch.ones(128, N, dtype=torch.bfloat16))
        unfused.append(r["wgrad"])
    # first microbatch overwrites, the following ones accumulate
    for i, x in enumerate(xs):
        mod(x.clone().requires_grad_(True), splits, is_first_microbatch=(i == 0)).sum().backward()
    for e, w in enumerate(ws):
        assert w.grad is None
        want = unfused[0][e] + unfused[1][e] + unfused[2][e]
        torch.testing.assert_close(w.main_grad, want, rtol=1e-6, atol=1e-6)
    # is_first_microbatch None -> always accumulate on top of what main_grad holds
    for w, m in zip(ws, init):
        w.main_grad = m.clone()
    mod(xs[0].clone().requires_grad_(True), splits).sum().backward()
    for e, w in enumerate(ws):
        torch.testing.assert_close(w.main_grad, init[e] + unfused[0][e], rtol=1e-6, atol=1e-6)
    # Megatron-style flag: a placeholder gradient is returned and the flag is raised
    for w in ws:
        w.grad_added_to_main_grad = False
    mod(xs[0].clone().requires_grad_(True), splits).sum().backward()
    assert all(w.grad_added_to_main_grad for w in ws) and all(w.grad is not None for w in ws)


def test_module_argument_errors():
    from atorch_amd.grouped_linear import ATorchGroupedLinear

    mod = _module(2, 128, 128, bias=False)
    x = randn_bf16((128, 128), 1)
    with pytest.raises(AssertionError, match="Number of splits"):
        mod(x, [128])
    with pytest.raises(AssertionError, match="GEMM not possible"):
        mod(randn_bf16((128, 256), 1), [64, 64])
    with pytest.raises(AssertionError, match="not supported"):
        mod(x.to(torch.float64), [64, 64])
    with pytest.raises(ValueError, match="bias when TP > 1"):
        ATorchGroupedLinear(2, 128, 128, tp_size=2, bias=True, device="cpu", qlinear_params=_params())
    with pytest.raises(AssertionError, match="parallel_mode"):
        ATorchGroupedLinear(2, 128, 128, parallel_mode="diag", bias=False, device="cpu", qlinear_params=_params())
    col = ATorchGroupedLinear(2, 128, 256, tp_size=2, parallel_mode="column", bias=False, device="cpu",
                              qlinear_params=_params())
    assert col.weight0.shape == (128, 128)
    row = ATorchGroupedLinear(2, 256, 128, tp_size=2, parallel_mode="row", bias=False, device="cpu",
                              qlinear_params=_params())
    assert row.weight0.shape == (128, 128)
    mod.qlinear_params.quantize = False
    with pytest.raises(AssertionError, match="Quantization must be enabled"):
        mod(x, [64, 64])


def test_weights_share_one_buffer_and_are_recognised():
    from atorch_amd.quantization import _base_of_rows, _base_of_stack

    mod = _module(4, 128, 256, bias=False)
    ws = [getattr(mod, f"weight{i}").detach() for i in range(4)]
    base = _base_of_stack(ws)
    assert base == (ws[0].data_ptr(), 128 * 256)
    assert _base_of_stack([ws[0], ws[2], ws[3], ws[1]]) is None
    buf = torch.zeros(100, 64, dtype=torch.uint8)
    parts = list(torch.split(buf, [30, 0, 50, 20]))
    assert _base_of_rows(parts) == (buf.data_ptr(), 64)
    assert _base_of_rows([parts[2], parts[0], parts[1], parts[3]]) is None
    wide = torch.zeros(100, 128, dtype=torch.uint8)[:, :64]
    assert _base_of_rows(list(torch.split(wide, [30, 0, 50, 20]))) == (wide.data_ptr(), 128)


def test_stack_view_needs_one_storage_not_only_adjacent_addresses():
    """Tensors that sit side by side in memory but own separate storages (what module.to(), .bfloat16() or
    load_state_dict into new parameters leave behind) cannot be viewed as one strided tensor: the helper
    declines instead of raising, and callers fall back to a copy or a per-tensor loop."""
    import numpy as np

    from atorch_amd.grouped_linear import _stack_of
    from atorch_amd.quantization import WeightCodeCache

    mod = _module(3, 128, 128, bias=False)
    ws = [getattr(mod, f"weight{i}").detach() for i in range(3)]
    st = _stack_of(ws)
    assert st is not None and st.shape == (3, 128, 128) and st.data_ptr() == ws[0].data_ptr()
    raw = np.zeros(2 * 64 * 4, dtype=np.uint8)
    a = torch.frombuffer(memoryview(raw)[: 64 * 4], dtype=torch.float32)
    b = torch.frombuffer(memoryview(raw)[64 * 4 :], dtype=torch.float32)
    assert b.data_ptr() == a.data_ptr() + 64 * 4  # adjacent, two storages
    assert _stack_of([a, b]) is None
    buf = torch.zeros(3 * 16)
    assert _stack_of([buf[0:16], buf[16:32], buf[32:48]]) is not None
    moved = _module(3, 128, 128, bias=False).to(torch.float64)  # every parameter gets a storage of its own
    assert _stack_of([getattr(moved, f"weight{i}").detach() for i in range(3)]) is None
    # the functional forms' cache: reuse only while the weight is unchanged
    cache, calls = WeightCodeCache(), []
    w = torch.zeros(4, 4)
    make = lambda t: (calls.append(t), (1, 2, 3 if t else None, 4 if t else None))[1]  # noqa: E731
    assert cache.codes("w", (w,), True, False, make) == (1, 2, None, None)
    assert cache.codes("w", (w,), False, False, make) == (1, 2, None, None) and calls == [False]
    assert cache.codes("w", (w,), False, True, make)[2] == 3 and calls == [False, True]  # transposes were missing
    w.add_(1)
    cache.codes("w", (w,), False, True, make)
    assert calls == [False, True, True]  # written in place since: quantised again without being told
    cache.codes("w", (w,), None, True, make)
    assert len(calls) == 4  # None quantises on every call, like the module


def test_transposed_layout_recognition():
    from atorch_amd.quantization import HipQuantizeOp

    R, splits = 64, [100, 0, 300, 128]
    ld = sum((m + TILE - 1) // TILE * TILE for m in splits)
    q_t = torch.zeros(R, ld, dtype=torch.uint8)
    s_t = torch.zeros(ld // TILE, R)
    qs, ss, p = [], [], 0
    for m in splits:
        nb = (m + TILE - 1) // TILE
        qs.append(q_t[:, p : p + m])
        ss.append(s_t[p // TILE : p // TILE + nb].t())
        p += nb * TILE
    assert HipQuantizeOp._transposed_layout(qs, ss, splits) == (q_t.data_ptr(), ld, s_t.data_ptr())
    qs2 = [q.clone() for q in qs]
    assert HipQuantizeOp._transposed_layout(qs2, ss, splits) is None


def test_hip_library_is_required(monkeypatch):
    """No silent fallback: with the library file missing every op raises."""
    from atorch_amd import _lib

    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", os.path.join(os.path.dirname(_lib.LIB_PATH), "missing.so"))
    with pytest.raises(_lib.HipLibraryMissing):
        _lib.lib()


def test_patch_grouped_linear_hook():
    import types

    from atorch_amd.grouped_linear import ATorchGroupedLinear, _ATorchQuantizedGroupedLinear, patch_grouped_linear

    ns = types.SimpleNamespace(_QuantizedGroupedLinear=object, GroupedLinear=object, ATorchGroupedLinear=object)
    patch_grouped_linear(ns)
    assert ns._QuantizedGroupedLinear is _ATorchQuantizedGroupedLinear
    assert ns.GroupedLinear is ATorchGroupedLinear and ns.ATorchGroupedLinear is ATorchGroupedLinear
    assert not hasattr(ns, "_ATorchQuantizedGroupedLinear")
    patch_grouped_linear(None)


def test_layouts_of_the_transposed_codes_on_the_host():
    """The token-block-major layout [ld_t/128, R, 128] holds byte (r, t) at ((t / 128) R + r) 128 + t % 128;
    ``qt_rows`` turns it into the row layout [R, ld_t] and ``qt_ld`` reads the padded token count of either."""
    from atorch_amd import kernels

    R, ld_t = 5, 384
    rows = torch.arange(R * ld_t, dtype=torch.int64).remainder(251).to(torch.uint8).view(R, ld_t)
    blocked = torch.empty(ld_t // TILE * R * TILE, dtype=torch.uint8)
    for r in range(R):
        for t in range(0, ld_t, 37):
            blocked[((t // TILE) * R + r) * TILE + t % TILE] = rows[r, t]
    blocked = blocked.view(ld_t // TILE, R, TILE)
    back = kernels.qt_rows(blocked)
    assert back.shape == (R, ld_t) and kernels.qt_ld(blocked) == ld_t and kernels.qt_ld(rows) == ld_t
    for r in range(R):
        for t in range(0, ld_t, 37):
            assert back[r, t] == rows[r, t]
    assert kernels.qt_rows(rows) is rows
    assert kernels._alloc_qt(R, ld_t, True, "cpu").shape == (ld_t // TILE, R, TILE)
    assert kernels._alloc_qt(R, ld_t, False, "cpu").shape == (R, ld_t)

"""Parity of the HIP kernels (through the C ABI) against the CPU oracle, at sizes the oracle
finishes in seconds.  Bit-exact for codes, scales and index work; GEMM outputs within
max relative error 1e-2 (bf16 out, fp32 accumulate)."""
import pytest
import torch

from helpers import TILE, heavy_tailed, ragged_splits, randn_bf16, rel_err, topk_routing

pytestmark = pytest.mark.gpu

GEMM_TOL = 1e-2  # bf16 output, the tolerance the path is specified to
# fp32 output: the fp8 MFMA does not round its 128-term dot product exactly (measured about
# 1e-4 of the output rms on MI355X), so the fp32 comparison is looser than fp32 epsilon.
GEMM_TOL_F32 = 5e-4


def _u8q(t):
    return t.view(torch.uint8)


def _u8(t):
    return t.view(torch.uint8).cpu()


# ------------------------------------------------------------------------------------------
# SwiGLU fused into the quantisation of the intermediate activations
# ------------------------------------------------------------------------------------------
def _ulp_diff(a, b):
    return (a.view(torch.int16).int() - b.view(torch.int16).int()).abs()


def test_swiglu_over_all_bf16_values(oracle, dev):
    """h from the fused kernel against the oracle for every finite bf16 value of a: the kernel
    evaluates sigmoid with the hardware exp2 and reciprocal (a few fp32 ulps), the oracle with a
    correctly rounded expf, so bf16(silu) may differ by one ulp on a small fraction of inputs; the
    product with b is rounded again, which can turn that into two ulps of h, never more."""
    from atorch_amd import kernels

    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    a = bits[bits.float().abs() < 2.0**100]  # larger values overflow the product: out of the quantiser's contract
    a = a[: a.numel() // 128 * 128].view(-1, 128)
    g = torch.Generator().manual_seed(4)
    b = (torch.randn(a.shape, generator=g) * 2).bfloat16()
    fc1 = torch.cat([a, b], dim=1).contiguous()
    q, s, h = kernels.swiglu_tile_quant(fc1.to(dev), return_activation=True)
    ho = oracle.swiglu(fc1)
    d = _ulp_diff(h.cpu(), ho)
    # +-0 differ by 0x8000 as integers but are equal values
    d = torch.where(h.cpu().float() == ho.float(), torch.zeros_like(d), d)
    assert int(d.max()) <= 2, int(d.max())
    assert float((d > 0).float().mean()) < 2e-3
    # the codes and scales are exactly the quantisation of the kernel's own activation
    qo, so = oracle.tile_quant(h.cpu())
    assert torch.equal(_u8(q), qo) and torch.equal(s.cpu(), so)


@pytest.mark.parametrize("M,F,E", [(300, 256, 3), (1000, 1408 // 128 * 128, 5)])
def test_swiglu_quant_dual_grouped(oracle, dev, M, F, E):
    """The fused kernel equals SwiGLU followed by the dual (row + transposed) grouped quantisation:
    its outputs are bit-identical to tile_quant_dual_grouped applied to its own activation, which
    is within two bf16 ulps of the oracle's (one for bf16(silu), rounded again in the product)."""
    from atorch_amd import kernels

    splits = ragged_splits(M, E, seed=5)
    goff = kernels.group_offsets_from_splits(splits, dev)
    fc1 = randn_bf16((M, 2 * F), 6, std=2.0)
    q, s, q_t, s_t, h = kernels.swiglu_tile_quant_dual_grouped(fc1.to(dev), goff, E, return_activation=True)
    ho = oracle.swiglu(fc1)
    d = _ulp_diff(h.cpu(), ho)
    d = torch.where(h.cpu().float() == ho.float(), torch.zeros_like(d), d)
    assert int(d.max()) <= 2 and float((d > 0).float().mean()) < 2e-3
    q2, s2, q_t2, s_t2 = kernels.tile_quant_dual_grouped(h, goff, E, ld_t=q_t.shape[1])
    assert torch.equal(_u8(q), _u8(q2)) and torch.equal(s, s2)
    # columns / scale rows past the padded total are not written by either kernel
    ptot = kernels.padded_total(splits)
    assert torch.equal(s_t[: ptot // TILE], s_t2[: ptot // TILE])
    assert torch.equal(_u8(q_t[:, :ptot]), _u8(q_t2[:, :ptot]))
    # transposed only
    _, _, q_t3, s_t3 = kernels.swiglu_tile_quant_dual_grouped(fc1.to(dev), goff, E, ld_t=q_t.shape[1], rowwise=False)
    assert torch.equal(_u8(q_t3[:, :ptot]), _u8(q_t[:, :ptot])) and torch.equal(s_t3[: ptot // TILE], s_t[: ptot // TILE])


def test_swiglu_bwd_over_all_bf16_values(oracle, dev):
    """[da | db] from the fused backward kernel against the oracle (which equals torch's CPU autograd)
    for every bf16 value of a below 2^100 in magnitude: hardware exp and reciprocal against correctly
    rounded ones, so differences of one bf16 ulp (two in db, whose bf16(silu) factor is rounded
    again in the product) on a small fraction of inputs."""
    from atorch_amd import kernels

    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    a = bits[bits.float().abs() < 2.0**100]
    a = a[: a.numel() // 128 * 128].view(-1, 128)
    g = torch.Generator().manual_seed(14)
    b = (torch.randn(a.shape, generator=g) * 2).bfloat16()
    dh = torch.randn(a.shape, generator=g).bfloat16()
    fc1 = torch.cat([a, b], dim=1).contiguous()
    M = fc1.shape[0]
    goff = kernels.group_offsets_from_splits([M], dev)
    q, s, q_t, s_t, gr = kernels.swiglu_bwd_tile_quant_dual_grouped(dh.to(dev), fc1.to(dev), goff, 1, return_grad=True)
    go = oracle.swiglu_bwd(dh, fc1)
    d = _ulp_diff(gr.cpu(), go)
    d = torch.where(gr.cpu().float() == go.float(), torch.zeros_like(d), d)
    assert int(d.max()) <= 2, int(d.max())
    assert float((d > 0).float().mean()) < 2e-3
    qo, so = oracle.tile_quant(gr.cpu())
    assert torch.equal(_u8(q), qo) and torch.equal(s.cpu(), so)


@pytest.mark.parametrize("M,F,E", [(300, 256, 3), (1000, 1408 // 128 * 128, 5)])
def test_swiglu_bwd_quant_dual_grouped(oracle, dev, M, F, E):
    """The fused backward equals autograd's SwiGLU backward followed by the dual grouped quantisation:
    outputs bit-identical to tile_quant_dual_grouped of its own gradient, which is within two bf16
    ulps of the oracle's."""
    from atorch_amd import kernels

    splits = ragged_splits(M, E, seed=15)
    goff = kernels.group_offsets_from_splits(splits, dev)
    fc1 = randn_bf16((M, 2 * F), 16, std=2.0)
    dh = randn_bf16((M, F), 17, std=0.5)
    q, s, q_t, s_t, gr = kernels.swiglu_bwd_tile_quant_dual_grouped(dh.to(dev), fc1.to(dev), goff, E, return_grad=True)
    go = oracle.swiglu_bwd(dh, fc1)
    d = _ulp_diff(gr.cpu(), go)
    d = torch.where(gr.cpu().float() == go.float(), torch.zeros_like(d), d)
    assert int(d.max()) <= 2 and float((d > 0).float().mean()) < 2e-3
    q2, s2, q_t2, s_t2 = kernels.tile_quant_dual_grouped(gr, goff, E, ld_t=q_t.shape[1])
    assert torch.equal(_u8(q), _u8(q2)) and torch.equal(s, s2)
    ptot = kernels.padded_total(splits)
    assert torch.equal(s_t[: ptot // TILE], s_t2[: ptot // TILE])
    assert torch.equal(_u8(q_t[:, :ptot]), _u8(q_t2[:, :ptot]))
    _, _, q_t3, s_t3 = kernels.swiglu_bwd_tile_quant_dual_grouped(dh.to(dev), fc1.to(dev), goff, E, ld_t=q_t.shape[1], rowwise=False)
    assert torch.equal(_u8(q_t3[:, :ptot]), _u8(q_t[:, :ptot])) and torch.equal(s_t3[: ptot // TILE], s_t[: ptot // TILE])


def test_swiglu_forward_and_backward_against_torch_on_the_gpu(dev):
    """The reference's two torch ops and their autograd, run on this GPU, against the fused kernels:
    the same bounds as against the oracle (one bf16 ulp where sigmoid enters once, two where a bf16
    product with it is rounded again), on a small fraction of elements."""
    from atorch_amd import kernels

    g = torch.Generator().manual_seed(41)
    M, F = 640, 512
    fc1 = (torch.randn(M, 2 * F, generator=g) * 2).bfloat16().to(dev)
    dh = torch.randn(M, F, generator=g).bfloat16().to(dev)
    leaf = fc1.clone().requires_grad_(True)
    a, b = torch.chunk(leaf, 2, dim=-1)
    h_ref = torch.nn.functional.silu(a) * b
    h_ref.backward(dh)
    _, _, h = kernels.swiglu_tile_quant(fc1, return_activation=True)
    goff = kernels.group_offsets_from_splits([M], dev)
    _, _, _, _, gr = kernels.swiglu_bwd_tile_quant_dual_grouped(dh, fc1, goff, 1, return_grad=True)
    for got, ref in ((h, h_ref.detach()), (gr, leaf.grad)):
        d = _ulp_diff(got.cpu(), ref.cpu())
        d = torch.where(got.cpu().float() == ref.cpu().float(), torch.zeros_like(d), d)
        assert int(d.max()) <= 2, int(d.max())
        assert float((d > 0).float().mean()) < 2e-3


def test_swiglu_quant_rejects_bad_shapes(dev):
    from atorch_amd import kernels

    with pytest.raises(AssertionError):
        kernels.swiglu_tile_quant(torch.zeros(4, 384, dtype=torch.bfloat16, device=dev))  # F = 192
    with pytest.raises(AssertionError):
        kernels.swiglu_tile_quant(torch.zeros(4, 256, dtype=torch.float32, device=dev))


# ------------------------------------------------------------------------------------------
# a1: 1x128 quant
# ------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("shape", [(1, 128), (7, 256), (2048, 512), (33, 7168)])
def test_tile_quant_matches_oracle(oracle, dev, dtype, shape):
    from atorch_amd import kernels

    x = heavy_tailed(shape, seed=shape[0], dtype=dtype)
    q, s = kernels.tile_quant(x.to(dev))
    qo, so = oracle.tile_quant(x)
    assert torch.equal(s.cpu(), so)
    assert torch.equal(_u8(q), qo)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("rows,cols,pad", [(37, 128, 8), (50, 384, 64), (21, 5120, 128), (3, 4096 + 128, 1 << 20)])
def test_tile_quant_of_strided_rows_and_scatter_through_the_c_abi(oracle, dev, dtype, rows, cols, pad):
    """Rows ldx = cols + pad elements apart (a column slice of a wider tensor), which only the C entry point takes:
    the same codes as the dense copy, for tile counts per row below and above a workgroup's 32 tiles and row counts
    that leave the last workgroup partly filled; and the scatter form (every row to two destinations) on the same
    strided input."""
    import ctypes

    from atorch_amd import _lib

    L = _lib.lib()
    wide = heavy_tailed((rows, cols + pad), seed=rows + cols, dtype=dtype).to(dev) if pad < 4096 else None
    if wide is None:  # a stride of a million elements: only the rows themselves are allocated densely elsewhere
        buf = torch.zeros(rows * (cols + pad), dtype=dtype, device=dev)
        wide = buf.view(rows, cols + pad)
        wide[:, :cols] = heavy_tailed((rows, cols), seed=rows + cols, dtype=dtype).to(dev)
    x = wide[:, :cols]
    qo, so = oracle.tile_quant(x.cpu().contiguous())
    vp = ctypes.c_void_p
    q = torch.zeros((rows, cols), dtype=torch.uint8, device=dev)
    sc = torch.zeros((rows, cols // TILE), dtype=torch.float32, device=dev)
    st = vp(torch.cuda.current_stream().cuda_stream)
    code = _lib.dtype_code(dtype)
    rc = L.aamd_quant_1x128(vp(x.data_ptr()), code, rows, cols, cols + pad, vp(q.data_ptr()), vp(sc.data_ptr()), 0.0, st)
    assert rc == _lib.OK, L.aamd_last_error()
    assert torch.equal(q.cpu(), qo) and torch.equal(sc.cpu(), so)
    # scatter: row r goes to rows r and rows + (rows - 1 - r) of a [2 rows, cols] output
    row_map = torch.stack([torch.arange(rows), 2 * rows - 1 - torch.arange(rows)], 1).to(torch.int32).to(dev).contiguous()
    q2 = torch.zeros((2 * rows, cols), dtype=torch.uint8, device=dev)
    s2 = torch.zeros((2 * rows, cols // TILE), dtype=torch.float32, device=dev)
    rc = L.aamd_permute_quant_1x128(vp(x.data_ptr()), code, rows, cols, cols + pad, vp(row_map.data_ptr()), 2, 2 * rows,
                                    vp(q2.data_ptr()), vp(s2.data_ptr()), 0.0, st)
    assert rc == _lib.OK, L.aamd_last_error()
    assert torch.equal(q2[:rows].cpu(), qo) and torch.equal(q2[rows:].flip(0).cpu(), qo)
    assert torch.equal(s2[:rows].cpu(), so) and torch.equal(s2[rows:].flip(0).cpu(), so)
    # a row stride of 2^24 elements or more is refused
    rc = L.aamd_quant_1x128(vp(x.data_ptr()), code, 1, cols, 1 << 24, vp(q.data_ptr()), vp(sc.data_ptr()), 0.0, st)
    assert rc == _lib.ERR_ARG and b"2^24" in L.aamd_last_error()


def test_swiglu_quant_of_wide_and_strided_rows(oracle, dev):
    """The gated width above a workgroup's 32 tiles (F = 4224: 33 tiles per row) and rows ld > 2F apart, through the
    C entry point: codes and scales equal to the 1x128 quantisation of the kernel's own activation."""
    import ctypes

    from atorch_amd import _lib, kernels

    L = _lib.lib()
    rows, F, ld = 19, 4224, 2 * 4224 + 256
    wide = randn_bf16((rows, ld), 41, std=2.0).to(dev)
    q = torch.zeros((rows, F), dtype=torch.uint8, device=dev)
    sc = torch.zeros((rows, F // TILE), dtype=torch.float32, device=dev)
    h = torch.zeros((rows, F), dtype=torch.bfloat16, device=dev)
    vp = ctypes.c_void_p
    rc = L.aamd_swiglu_quant_1x128(vp(wide.data_ptr()), rows, F, ld, vp(h.data_ptr()), vp(q.data_ptr()), vp(sc.data_ptr()),
                                   vp(torch.cuda.current_stream().cuda_stream))
    assert rc == _lib.OK, L.aamd_last_error()
    q1, s1, h1 = kernels.swiglu_tile_quant(wide[:, : 2 * F].contiguous(), return_activation=True)
    assert torch.equal(h, h1) and torch.equal(q, _u8q(q1)) and torch.equal(sc, s1)
    ho = oracle.swiglu(wide[:, : 2 * F].cpu().contiguous())
    d = _ulp_diff(h.cpu(), ho)
    d = torch.where(h.cpu().float() == ho.float(), torch.zeros_like(d), d)
    assert int(d.max()) <= 2
    qo, so = oracle.tile_quant(h.cpu())
    assert torch.equal(q.cpu(), qo) and torch.equal(sc.cpu(), so)


def test_tile_quant_all_bf16_patterns(oracle, dev):
    """Every bf16 bit pattern as an element, for several tile maxima: pins the division and the
    hardware fp8 conversion (RNE, subnormals) against the integer encoder of the oracle."""
    from atorch_amd import kernels

    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    finite = bits[torch.isfinite(bits.float())]
    rows = []
    for amax in (1.0, 448.0, 3.0e-3, 1.7e4, 2.0**-120, 6.0e37, 1.0e-38):
        v = finite[finite.float().abs() <= amax]
        pad = (-v.numel()) % (TILE - 1)
        v = torch.cat([v, torch.zeros(pad, dtype=torch.bfloat16)])
        v = v.view(-1, TILE - 1)
        col = torch.full((v.shape[0], 1), amax, dtype=torch.bfloat16)
        rows.append(torch.cat([col, v], dim=1))
    x = torch.cat(rows).contiguous()
    q, s = kernels.tile_quant(x.to(dev))
    qo, so = oracle.tile_quant(x)
    assert torch.equal(s.cpu(), so)
    assert torch.equal(_u8(q), qo)


def test_tile_quant_division_is_exact_over_the_whole_bf16_domain(oracle, dev):
    """The kernels divide by a tile's scale with a hoisted reciprocal and an FMA correction instead
    of one IEEE division per element.  Every pair (x, amax) of finite bf16 values with |x| <= amax
    (about 10^9 quotients) must give the code of the IEEE quotient fl(x / fl(amax / 448)); the
    reference is torch's own fp32 division and fp8 cast on the device, itself compared with the
    CPU oracle on a sample of the same tiles."""
    from atorch_amd import kernels

    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    finite = bits[torch.isfinite(bits.float())]
    pad = (-finite.numel()) % (TILE - 1)
    vals = torch.cat([finite, torch.zeros(pad, dtype=torch.bfloat16)]).view(-1, TILE - 1).to(dev)  # [515, 127]
    amaxes = finite[finite.float() > 0].to(dev)  # every positive finite bf16 value, subnormals included
    absvals = vals.float().abs()
    chunk = 64
    bad = 0
    for lo in range(0, amaxes.numel(), chunk):
        a = amaxes[lo : lo + chunk]  # [c]
        keep = absvals.unsqueeze(0) <= a.float().view(-1, 1, 1)
        body = torch.where(keep, vals.unsqueeze(0), torch.zeros((), dtype=torch.bfloat16, device=dev))
        first = a.view(-1, 1, 1).expand(-1, vals.shape[0], 1)
        x = torch.cat([first, body], dim=2).reshape(-1, TILE).contiguous()
        q, s = kernels.tile_quant(x)
        s_ref = (a.float().cpu() / torch.full((a.numel(),), 448.0)).to(dev)  # IEEE division on the host
        s_ref = s_ref.view(-1, 1).expand(-1, vals.shape[0]).reshape(-1, 1)
        assert torch.equal(s, s_ref)
        q_ref = (x.float() / s_ref).to(torch.float8_e4m3fn)
        neq = _u8q(q) != _u8q(q_ref)
        bad += int(neq.sum())
        if lo % (chunk * 64) == 0:  # the device-side reference against the oracle
            rows = torch.arange(0, x.shape[0], 97, device=dev)
            qo, so = oracle.tile_quant(x[rows].cpu())
            assert torch.equal(_u8q(q_ref[rows]).cpu(), qo) and torch.equal(s[rows].cpu(), so)
    assert bad == 0, f"{bad} quotients differ from the IEEE division"


def test_tile_quant_known_answers(dev):
    """zeros -> s = 1, codes 0; ones -> s = fl(1/448), codes 0x7E; rows of 1000 / -512 -> +-448
    (atorch/tests/common_tests/scaled_linear_test.py:131-133, 305-311)."""
    from atorch_amd import kernels

    x = torch.ones(4, 256, dtype=torch.bfloat16)
    x[0] = 0
    x[1] = 1000
    x[2] = -512
    q, s = kernels.tile_quant(x.to(dev))
    q, s = _u8(q), s.cpu()
    assert torch.all(s[0] == 1.0) and torch.all(q[0] == 0)
    assert torch.all(s[1] == torch.tensor(1000.0) / 448.0) and torch.all(q[1] == 0x7E)
    assert torch.all(s[2] == torch.tensor(512.0) / 448.0) and torch.all(q[2] == 0xFE)
    assert torch.all(s[3] == torch.tensor(1.0) / 448.0) and torch.all(q[3] == 0x7E)


def test_tile_quant_eps(oracle, dev):
    from atorch_amd import kernels

    x = randn_bf16((16, 256), 3, std=1e-3)
    q, s = kernels.tile_quant(x.to(dev), eps=0.5)
    qo, so = oracle.tile_quant(x, eps=0.5)
    assert torch.equal(s.cpu(), so) and torch.equal(_u8(q), qo)


def test_tile_quant_rejects_bad_shapes(dev):
    from atorch_amd import kernels

    with pytest.raises(AssertionError):
        kernels.tile_quant(torch.zeros(4, 100, dtype=torch.bfloat16, device=dev))


# ------------------------------------------------------------------------------------------
# a1 + a9: permute fused into the quant; a9 alone; a11 preprocess
# ------------------------------------------------------------------------------------------
@pytest.mark.parametrize("T,E,k", [(64, 4, 1), (1000, 8, 2), (777, 64, 8), (3000, 200, 4)])
def test_moe_preprocess_matches_stable_sort(oracle, dev, T, E, k):
    from atorch_amd import kernels

    idx, _ = topk_routing(T, E, k, seed=T, zipf_s=1.2 if E >= 64 else None)
    sorted_idx, row_map, goff = kernels.moe_preprocess(idx.to(dev), E)
    so, counts = oracle.permute_indices(idx, E)
    assert torch.equal(sorted_idx.cpu(), so)
    assert torch.equal(sorted_idx.cpu(), torch.argsort(idx.reshape(-1), stable=True))
    assert torch.equal(goff.cpu()[1:] - goff.cpu()[:-1], counts)
    inv = torch.empty(T * k, dtype=torch.int32)
    inv[so] = torch.arange(T * k, dtype=torch.int32)
    assert torch.equal(row_map.cpu(), inv)


def test_moe_preprocess_int32_ids_and_empty(dev):
    from atorch_amd import kernels

    idx = torch.tensor([3, 3, 0, 3], dtype=torch.int32)
    sorted_idx, row_map, goff = kernels.moe_preprocess(idx.to(dev), 5)
    assert sorted_idx.cpu().tolist() == [2, 0, 1, 3]
    assert goff.cpu().tolist() == [0, 1, 1, 1, 4, 4]
    s2, r2, g2 = kernels.moe_preprocess(torch.zeros(0, dtype=torch.int64, device=dev), 3)
    assert s2.numel() == 0 and g2.cpu().tolist() == [0, 0, 0, 0]


@pytest.mark.parametrize("T,E,k,H", [(512, 8, 2, 512), (300, 64, 8, 1024)])
def test_permute_quant_commutes(oracle, dev, T, E, k, H):
    """quant is row local, so permute(quant(x)) == quant(permute(x)) on codes and scales."""
    from atorch_amd import kernels

    x = heavy_tailed((T, H), seed=11)
    idx, _ = topk_routing(T, E, k, seed=5)
    sorted_idx, row_map, goff = kernels.moe_preprocess(idx.to(dev), E)
    q, s = kernels.permute_tile_quant(x.to(dev), row_map, k, T * k)
    xp, so, _ = oracle.permute(x, idx, E)
    qo, sco = oracle.tile_quant(xp)
    assert torch.equal(_u8(q), qo) and torch.equal(s.cpu(), sco)
    # the un-quantised permute and the reference-shaped functions
    from atorch_amd.token_dispatcher import permute

    p, si = permute(x.to(dev), idx.to(dev), num_experts=E)
    assert torch.equal(p.cpu(), xp) and torch.equal(si.cpu(), so)
    p2, si2 = permute(x.to(dev), idx.to(dev))
    assert torch.equal(p2.cpu(), xp) and torch.equal(si2.cpu(), so)


# ------------------------------------------------------------------------------------------
# a10: unpermute + combine
# ------------------------------------------------------------------------------------------
@pytest.mark.parametrize("probs_dtype", [torch.bfloat16, torch.float32, None])
@pytest.mark.parametrize("T,E,k,H", [(256, 8, 2, 512), (100, 64, 8, 1024), (37, 8, 2, 7168), (64, 4, 3, 5120)])
def test_unpermute_combine(oracle, dev, probs_dtype, T, E, k, H):
    from atorch_amd.token_dispatcher import unpermute

    if probs_dtype is None:
        k = 1
    idx, probs = topk_routing(T, E, k, seed=9)
    so, _ = oracle.permute_indices(idx, E)
    y = randn_bf16((T * k, H), 21)
    pr = None if probs_dtype is None else probs.to(probs_dtype)
    out = unpermute(y.to(dev), so.to(dev), None if pr is None else pr.to(dev))
    ref = oracle.unpermute(y, so, pr)
    assert out.dtype == ref.dtype
    assert torch.equal(out.cpu(), ref)
    # against the torch restatement of the reference: <= 1 ulp of the output type
    tref = oracle.torch_unpermute(y, so, pr)
    assert tref.dtype == ref.dtype
    torch.testing.assert_close(out.cpu().float(), tref.float(), rtol=2**-7 if ref.dtype == torch.bfloat16 else 1e-6, atol=1e-6)


def test_unpermute_inverts_permute_top1(dev):
    from atorch_amd.token_dispatcher import permute, unpermute

    x = randn_bf16((333, 256), 2).to(dev)
    idx = torch.randint(0, 7, (333,), generator=torch.Generator().manual_seed(0)).to(dev)
    p, si = permute(x, idx, num_experts=7)
    assert torch.equal(unpermute(p, si), x)


# ------------------------------------------------------------------------------------------
# a2 + a4: block quant
# ------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("E,N,K", [(1, 128, 128), (3, 256, 384), (4, 1024, 512)])
def test_block_quant_matches_oracle(oracle, dev, dtype, E, N, K):
    from atorch_amd import kernels

    w = randn_bf16((E, N, K), seed=N + K, std=0.02, dtype=dtype)
    w[0, :128, :128] = 0  # an all-zero block -> scale 1
    q, s, q_t, s_t = kernels.block_quant_batched(w.to(dev), return_transpose=True)
    for e in range(E):
        qo, so = oracle.block_quant(w[e])
        assert torch.equal(s[e].cpu(), so) and torch.equal(_u8(q[e]), qo)
        assert torch.equal(_u8(q_t[e]), qo.t()) and torch.equal(s_t[e].cpu(), so.t())
    assert s[0, 0, 0].item() == 1.0
    q1, s1 = kernels.block_quant(w[0].to(dev))
    assert torch.equal(_u8(q1), _u8(q[0])) and torch.equal(s1.cpu(), s[0].cpu())


# ------------------------------------------------------------------------------------------
# a3: row-wise + transposed quant of ragged groups
# ------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("M,K,E,mult", [(512, 256, 4, 128), (1000, 384, 6, 16), (777, 128, 5, 1), (3000, 128, 700, 1)])
def test_dual_grouped_quant(oracle, dev, dtype, M, K, E, mult):
    from atorch_amd import kernels

    x = heavy_tailed((M, K), seed=M, dtype=dtype)
    splits = ragged_splits(M, E, seed=K, multiple=mult)
    goff = kernels.group_offsets_from_splits(splits, dev)
    q, s, q_t, s_t = kernels.tile_quant_dual_grouped(x.to(dev), goff, E)
    qo, so = oracle.tile_quant(x)
    assert torch.equal(_u8(q), qo) and torch.equal(s.cpu(), so)
    qto, sto = oracle.tile_quant_t_grouped(x, splits, ld_t=q_t.shape[1])
    ptot = oracle.padded_offsets(splits)[-1]
    assert torch.equal(_u8(q_t)[:, :ptot], qto[:, :ptot])
    assert torch.equal(s_t.cpu()[: ptot // TILE], sto[: ptot // TILE])
    # transposed only
    _, _, q_t2, s_t2 = kernels.tile_quant_dual_grouped(x.to(dev), goff, E, rowwise=False)
    assert torch.equal(_u8(q_t2)[:, :ptot], qto[:, :ptot])


def test_tile_quant_return_transpose_equals_quant_of_transpose(oracle, dev):
    """M % 128 == 0: the transposed result is tile_quant(x.t().contiguous())
    (atorch/modules/fp8/scaled_linear.py:404-414)."""
    from atorch_amd import kernels

    x = randn_bf16((256, 384), 4)
    y, s, y_t, s_t = kernels.tile_quant(x.to(dev), return_transpose=True)
    qo, so = oracle.tile_quant(x.t().contiguous())
    assert y_t.shape == (384, 256) and s_t.shape == (384, 2)
    assert torch.equal(_u8(y_t.contiguous()), qo) and torch.equal(s_t.cpu(), so)


# ------------------------------------------------------------------------------------------
# dequant
# ------------------------------------------------------------------------------------------
def test_dequant(oracle, dev):
    from atorch_amd import kernels

    x = randn_bf16((256, 384), 8)
    q, s = kernels.tile_quant(x.to(dev))
    d = kernels.dequant(q, s)
    assert torch.equal(d.cpu(), oracle.dequant(_u8(q), s.cpu()))
    qb, sb = kernels.block_quant(x.to(dev))
    db = kernels.dequant(qb, sb, dtype=torch.bfloat16)
    assert torch.equal(db.cpu(), oracle.dequant(_u8(qb), sb.cpu()).bfloat16())
    # tile error <= block error (scaled_linear_test.py:305-319)
    t = torch.ones(512, 512, dtype=torch.bfloat16)
    t[1] = 1000
    t[2] = -512
    tq, ts = kernels.tile_quant(t.to(dev))
    bq, bs = kernels.block_quant(t.to(dev))
    et = (t.float() - kernels.dequant(tq, ts).cpu()).abs()
    eb = (t.float() - kernels.dequant(bq, bs).cpu()).abs()
    assert torch.all(eb >= et)


# ------------------------------------------------------------------------------------------
# a5/a6/a7: GEMMs
# ------------------------------------------------------------------------------------------
def _quant_inputs(oracle, M, N, K, E, seed):
    x = randn_bf16((M, K), seed)
    w = randn_bf16((E, N, K), seed + 1, std=0.02)
    qx, sx = oracle.tile_quant(x)
    qw = torch.stack([oracle.block_quant(w[e])[0] for e in range(E)])
    sw = torch.stack([oracle.block_quant(w[e])[1] for e in range(E)])
    return x, w, qx, sx, qw, sw


@pytest.mark.parametrize("M,N,K", [(128, 128, 128), (200, 256, 384), (64, 128, 1024), (513, 384, 256)])
def test_fp8_gemm_dense(oracle, dev, M, N, K):
    from atorch_amd import kernels

    _, _, qx, sx, qw, sw = _quant_inputs(oracle, M, N, K, 1, seed=M + N)
    ref = oracle.fp8_gemm(qx, sx, qw[0], sw[0])
    for dt in (torch.bfloat16, torch.float32):
        c = kernels.fp8_gemm(qx.to(dev).view(kernels.FP8), sx.to(dev), qw[0].to(dev).view(kernels.FP8), sw[0].to(dev), dtype=dt)
        assert c.dtype == dt
        assert rel_err(c.cpu(), ref) <= (GEMM_TOL if dt == torch.bfloat16 else GEMM_TOL_F32)
    # textbook check: dequantise and multiply in fp64
    full = (oracle.torch_dequant_tile(qx, sx).double() @ oracle.torch_dequant_block(qw[0], sw[0]).double().t())
    assert rel_err(c.cpu(), full.float()) <= GEMM_TOL_F32


def test_fp8_gemm_tile_scaled_b(oracle, dev):
    from atorch_amd import kernels

    M, N, K = 192, 256, 384
    a, b = randn_bf16((M, K), 1), randn_bf16((N, K), 2)
    qa, sa = oracle.tile_quant(a)
    qb, sb = oracle.tile_quant(b)
    ref = oracle.fp8_gemm(qa, sa, qb, sb)
    c = kernels.fp8_gemm(qa.to(dev).view(kernels.FP8), sa.to(dev), qb.to(dev).view(kernels.FP8), sb.to(dev), dtype=torch.float32)
    assert rel_err(c.cpu(), ref) <= GEMM_TOL_F32


def _deq_tile(q, s):
    return q.float() * s.repeat_interleave(TILE, -1)


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32], ids=["bf16", "fp32"])
def test_fp8_gemm_tile_scaled_b_large_tiles(dev, out_dtype):
    """NT GEMM whose B carries 1x128 scales (the dense weight-gradient form, scaled_linear.py:431-446)
    at a size that takes the large-tile configuration with per-row R scales: partial L tile, odd
    number of 128-row R tiles; against the float64 definition evaluated on the device."""
    from atorch_amd import kernels

    M, N, K = 4100, 8320, 512
    a, b = randn_bf16((M, K), 21).to(dev), randn_bf16((N, K), 22, std=0.02).to(dev)
    qa, sa = kernels.tile_quant(a)
    qb, sb = kernels.tile_quant(b)
    ref = _deq_tile(qa, sa).double() @ _deq_tile(qb, sb).double().t()
    c = kernels.fp8_gemm(qa, sa, qb, sb, dtype=out_dtype)
    tol = GEMM_TOL if out_dtype == torch.bfloat16 else GEMM_TOL_F32
    assert rel_err(c.cpu(), ref.float().cpu()) <= tol
    # the small-tile configuration computes the same sums in the same order
    with kernels.gemm_options(tile=0):
        c_small = kernels.fp8_gemm(qa, sa, qb, sb, dtype=out_dtype)
    assert torch.equal(c, c_small)


@pytest.mark.parametrize("K", [512, 1024, 1536, 2560, 1152, 1408, 2816], ids=lambda k: f"K{k}")
def test_grouped_gemm_nt_scale_batches_of_the_large_tiles(dev, K):
    """The 256x256 configuration takes its scales in batches of eight contraction blocks: exactly one
    batch (K = 1024), a last batch shifted back to end at the last block (1536, 2560), scale rows that are
    not 16-byte aligned and take 4-byte loads, with an odd number of steps (1152, 1408) and an even one
    (2816), and a contraction with fewer than eight blocks (512), which the launcher gives to the 128x128
    configuration.  Ragged groups with an empty one, a partial last R tile (N = 640), bias; against the
    float64 definition on the device and, bit for bit, against the pinned 128x128 configuration, which adds
    the same products in the same order."""
    from atorch_amd import kernels

    E, N = 4, 640
    splits = [700, 0, 1301, 255]
    M = sum(splits)
    x = randn_bf16((M, K), 51).to(dev)
    w = randn_bf16((E, N, K), 52, std=0.02).to(dev)
    bias = randn_bf16((E, N), 53).to(dev)
    qx, sx = kernels.tile_quant(x)
    qw, sw, _, _ = kernels.block_quant_batched(w)
    goff = kernels.group_offsets_from_splits(splits, dev)
    with kernels.gemm_options(tile=1):
        y = kernels.grouped_gemm_nt(qx, sx, qw, sw, goff, out_dtype=torch.float32, bias=bias)
    with kernels.gemm_options(tile=0):
        y_small = kernels.grouped_gemm_nt(qx, sx, qw, sw, goff, out_dtype=torch.float32, bias=bias)
    assert torch.equal(y, y_small)
    xd = _deq_tile(qx, sx).double()
    ref = torch.zeros(M, N, dtype=torch.float64, device=dev)
    off = 0
    for e, m in enumerate(splits):
        if m:
            wd = qw[e].float() * sw[e].repeat_interleave(TILE, -2).repeat_interleave(TILE, -1)
            ref[off : off + m] = xd[off : off + m] @ wd.double().t() + bias[e].double()
        off += m
    assert rel_err(y.cpu(), ref.float().cpu()) <= GEMM_TOL_F32


@pytest.mark.parametrize("tile", [0, 1], ids=["128x128", "256x128"])
def test_grouped_gemm_wgrad_pinned_tile_configurations(dev, tile):
    """The tile configurations of the weight-gradient GEMM (the product library runs the first; the others are
    measurement builds) on ragged
    groups with an empty group and partial token tiles, with and without accumulation, against the
    float64 definition on the device."""
    from atorch_amd import kernels

    E, N, K = 5, 640, 384
    splits = [300, 0, 1111, 128, 77]
    M = sum(splits)
    x = randn_bf16((M, K), 31).to(dev)
    dy = randn_bf16((M, N), 32, std=1e-2).to(dev)
    goff = kernels.group_offsets_from_splits(splits, dev)
    _, _, qxt, sxt = kernels.tile_quant_dual_grouped(x, goff, E, rowwise=False)
    _, _, qdt, sdt = kernels.tile_quant_dual_grouped(dy, goff, E, ld_t=qxt.shape[1], rowwise=False)
    base = torch.randn(E, N, K, generator=torch.Generator().manual_seed(3)).to(dev)
    acc = base.clone()
    with kernels.gemm_options(tile=tile):
        dw = kernels.grouped_gemm_wgrad(qdt, sdt, qxt, sxt, goff, out_dtype=torch.float32)
        dw16 = kernels.grouped_gemm_wgrad(qdt, sdt, qxt, sxt, goff, out_dtype=torch.bfloat16)
        kernels.grouped_gemm_wgrad(qdt, sdt, qxt, sxt, goff, out=acc, accumulate=True)
    refw = torch.zeros(E, N, K, dtype=torch.float64, device=dev)
    pos = 0
    for e, m in enumerate(splits):
        pad = (m + TILE - 1) // TILE * TILE
        if m:
            a = qdt[:, pos : pos + pad].float() * sdt[pos // TILE : (pos + pad) // TILE].t().repeat_interleave(TILE, 1)
            c = qxt[:, pos : pos + pad].float() * sxt[pos // TILE : (pos + pad) // TILE].t().repeat_interleave(TILE, 1)
            refw[e] = a.double() @ c.double().t()
        pos += pad
    refw = refw.float().cpu()
    assert rel_err(dw.cpu(), refw) <= GEMM_TOL_F32
    assert rel_err(dw16.cpu(), refw) <= GEMM_TOL
    assert rel_err((acc - base).cpu(), refw) <= 4 * GEMM_TOL_F32
    assert torch.all(dw[1] == 0) and torch.equal(acc[1], base[1])


def test_grouped_gemm_wgrad_short_operand_buffers_give_nan(dev):
    """ld_t below the padded token total: the groups that do not fit get NaN, never a finite wrong sum."""
    from atorch_amd import kernels

    E, N, K = 2, 128, 128
    splits = [128, 128]
    goff = kernels.group_offsets_from_splits(splits, dev)
    qt = torch.zeros((N, 128), dtype=torch.uint8, device=dev).view(kernels.FP8)  # room for one token block only
    st = torch.ones((1, N), dtype=torch.float32, device=dev)
    dw = kernels.grouped_gemm_wgrad(qt, st, qt, st, goff, out_dtype=torch.float32)
    assert torch.all(dw[0] == 0) and torch.all(torch.isnan(dw[1]))


@pytest.mark.parametrize("M,N,K,E,mult", [(512, 256, 256, 4, 16), (1000, 128, 384, 6, 1), (300, 384, 128, 3, 128)])
def test_grouped_gemm_nt(oracle, dev, M, N, K, E, mult):
    from atorch_amd import kernels

    _, _, qx, sx, qw, sw = _quant_inputs(oracle, M, N, K, E, seed=M)
    splits = ragged_splits(M, E, seed=N, multiple=mult)
    goff = kernels.group_offsets_from_splits(splits, dev)
    ref = oracle.grouped_gemm_nt(qx, sx, qw, sw, splits)
    bias = randn_bf16((E, N), 77)
    args = (qx.to(dev).view(kernels.FP8), sx.to(dev), qw.to(dev).view(kernels.FP8), sw.to(dev), goff)
    c32 = kernels.grouped_gemm_nt(*args, out_dtype=torch.float32)
    assert rel_err(c32.cpu(), ref) <= GEMM_TOL_F32
    c16 = kernels.grouped_gemm_nt(*args, out_dtype=torch.bfloat16)
    assert rel_err(c16.cpu(), ref) <= GEMM_TOL
    cb = kernels.grouped_gemm_nt(*args, out_dtype=torch.float32, bias=bias.to(dev))
    refb = ref + torch.repeat_interleave(bias.float(), torch.tensor(splits), dim=0)
    assert rel_err(cb.cpu(), refb) <= GEMM_TOL_F32
    # grouped == per-expert loop, bit-wise (test_quantized_grouped_linear.py:735-737)
    off = 0
    for e, m in enumerate(splits):
        if m:
            ce = kernels.fp8_gemm(args[0][off : off + m].contiguous(), args[1][off : off + m].contiguous(), args[2][e], args[3][e], dtype=torch.bfloat16)
            assert torch.equal(ce, c16[off : off + m])
        off += m


@pytest.mark.parametrize("M,N,K,E,mult", [(512, 128, 256, 4, 128), (1000, 256, 128, 6, 16), (333, 128, 128, 3, 1), (3000, 128, 128, 700, 1)])
def test_grouped_gemm_wgrad(oracle, dev, M, N, K, E, mult):
    from atorch_amd import kernels

    x = randn_bf16((M, K), 1)
    dy = randn_bf16((M, N), 2, std=1e-2)
    splits = ragged_splits(M, E, seed=M, multiple=mult)
    goff = kernels.group_offsets_from_splits(splits, dev)
    ld_t = kernels.padded_total(splits)
    qxt, sxt = oracle.tile_quant_t_grouped(x, splits, ld_t=ld_t)
    qdt, sdt = oracle.tile_quant_t_grouped(dy, splits, ld_t=ld_t)
    ref = oracle.grouped_gemm_wgrad(qdt, sdt, qxt, sxt, splits)
    args = (qdt.to(dev).view(kernels.FP8), sdt.to(dev), qxt.to(dev).view(kernels.FP8), sxt.to(dev), goff)
    dw = kernels.grouped_gemm_wgrad(*args, out_dtype=torch.float32)
    assert rel_err(dw.cpu(), ref) <= GEMM_TOL_F32
    for e, m in enumerate(splits):
        if m == 0:
            assert torch.all(dw[e] == 0)
    dw16 = kernels.grouped_gemm_wgrad(*args, out_dtype=torch.bfloat16)
    assert rel_err(dw16.cpu(), ref) <= GEMM_TOL
    # accumulate: second call adds; empty groups stay untouched
    base = torch.rand(E, N, K, generator=torch.Generator().manual_seed(5))
    acc = base.clone().to(dev)
    kernels.grouped_gemm_wgrad(*args, out=acc, accumulate=True)
    assert rel_err(acc.cpu() - base, ref) <= GEMM_TOL_F32
    for e, m in enumerate(splits):
        if m == 0:
            assert torch.equal(acc[e].cpu(), base[e])


def test_tile_and_block_quant_match_torch_ops_on_the_gpu(dev):
    """The reference formula (triton_kernel.py:21-46, 94-140: s = max(amax, eps) / 448, 0 -> 1,
    code = e4m3fn(x / s)) written with torch ops and run on this GPU (tensor / tensor is an IEEE
    division, the cast rounds to nearest even), against the kernels: bit for bit."""
    from atorch_amd import kernels

    g = torch.Generator().manual_seed(33)
    x = (torch.randn(257, 1024, generator=g) * torch.exp(torch.randn(257, 1, generator=g) * 3)).bfloat16().to(dev)
    x[5] = 0
    t = x.float().view(257, 8, 128)
    s_ref = t.abs().amax(dim=-1) / torch.full((), 448.0, device=dev)
    s_ref = torch.where(s_ref == 0, torch.ones_like(s_ref), s_ref)
    q_ref = (t / s_ref.unsqueeze(-1)).to(torch.float8_e4m3fn).view(257, 1024)
    q, s = kernels.tile_quant(x)
    assert torch.equal(s, s_ref) and torch.equal(_u8(q), _u8(q_ref))
    w = (torch.randn(384, 512, generator=g) * 0.05).bfloat16().to(dev)
    b = w.float().view(3, 128, 4, 128)
    sb_ref = b.abs().amax(dim=(1, 3)) / torch.full((), 448.0, device=dev)
    sb_ref = torch.where(sb_ref == 0, torch.ones_like(sb_ref), sb_ref)
    qb_ref = (b / sb_ref[:, None, :, None]).to(torch.float8_e4m3fn).view(384, 512)
    qb, sb = kernels.block_quant(w)
    assert torch.equal(sb, sb_ref) and torch.equal(_u8(qb), _u8(qb_ref))


def test_unpermute_matches_torch_ops_on_the_gpu(dev):
    """The reference's own sequence (token_dispatcher.py:119-161: zeros, index_copy_, multiply by the
    probabilities, sum over top-k) run with torch ops on this GPU, against the fused kernel: bit for bit
    with bf16 and with fp32 probabilities.  torch reduces the strided top-k dimension with four
    interleaved accumulators, ((a0 + a1) + a2) + a3; the kernel and the oracle add in that order."""
    from atorch_amd import token_dispatcher

    g = torch.Generator().manual_seed(31)
    for T, H, k, E in [(1024, 512, 8, 16), (512, 1024, 2, 8), (256, 256, 3, 8), (300, 2048, 6, 8), (128, 512, 13, 16)]:
        x = torch.randn(T, H, generator=g).bfloat16().to(dev)
        ids = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).to(dev)
        sorted_idx = torch.argsort(ids.reshape(-1), stable=True)
        y = x.index_select(0, sorted_idx // k)
        for pd in (torch.bfloat16, torch.float32):
            probs = torch.rand(T, k, generator=g).to(pd).to(dev)
            un = torch.zeros(T * k, H, dtype=y.dtype, device=dev)
            un.index_copy_(0, sorted_idx, y)
            ref = (un.reshape(T, k, H) * probs.unsqueeze(-1)).sum(dim=1)
            out = token_dispatcher.unpermute(y, sorted_idx, probs=probs)
            assert out.dtype == ref.dtype
            assert torch.equal(out, ref), (T, H, k, pd)


# ------------------------------------------------------------------------------------------
# f4: per-expert bias on expert-tagged rows
# ------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("ids_dtype", [torch.int64, torch.int32])
@pytest.mark.parametrize("T,H,E", [(1, 8, 1), (300, 136, 5), (4097, 1024, 64), (513, 7168, 8)])
def test_bias_gather_add_matches_oracle(oracle, dev, dtype, ids_dtype, T, H, E):
    from atorch_amd.bias_gather_add import bias_gather_add_bw, bias_gather_add_fw

    g = torch.Generator().manual_seed(T + H)
    ids = torch.randint(0, E, (T,), generator=g).sort().values  # grouped by expert, as the dispatcher leaves them
    inp = torch.randn(T, H, generator=g).to(dtype)
    bias = torch.randn(E, H, generator=g).to(dtype)
    out = bias_gather_add_fw(inp.to(dev), bias.to(dev), ids.to(ids_dtype).to(dev))
    assert torch.equal(out.cpu().view(torch.uint8), oracle.bias_gather_add(inp, bias, ids).view(torch.uint8))
    # sums that are exact in fp32: any order of additions gives the same bits
    small = torch.randint(-8, 9, (T, H), generator=g).to(dtype)
    bg = bias_gather_add_bw(small.to(dev), ids.to(ids_dtype).to(dev), E)
    assert bg.dtype == dtype
    assert torch.equal(bg.cpu().float(), oracle.bias_gather_bgrad(small, ids, E).to(dtype).float())
    # random data and unsorted tags: fp32 sums in another order, compared in fp32 before the final cast
    ids_u = ids[torch.randperm(T, generator=g)]
    bg2 = bias_gather_add_bw(inp.float().to(dev), ids_u.to(ids_dtype).to(dev), E)
    ref = oracle.bias_gather_bgrad(inp.float(), ids_u, E)
    assert float((bg2.cpu() - ref).abs().max()) <= 1e-5 * max(1.0, float(ref.abs().max()))


def test_bias_gather_add_autograd_and_edges(oracle, dev):
    from atorch_amd.bias_gather_add import bias_gather_add, bias_gather_add_bw, bias_gather_add_fw

    g = torch.Generator().manual_seed(8)
    T, H, E = 515, 256, 6
    ids = torch.randint(0, E, (T,), generator=g).sort().values.to(dev)
    inp = torch.randn(T, H, generator=g).bfloat16().to(dev).requires_grad_(True)
    bias = torch.randn(E, H, generator=g).bfloat16().to(dev).requires_grad_(True)
    dy = torch.randint(-4, 5, (T, H), generator=g).bfloat16().to(dev)
    bias_gather_add(inp, bias, ids).backward(dy)
    assert torch.equal(inp.grad, dy)
    assert torch.equal(bias.grad.cpu().float(), oracle.bias_gather_bgrad(dy.cpu(), ids.cpu(), E).bfloat16().float())
    # no rows: empty output, zero gradient
    z = bias_gather_add_fw(torch.empty(0, H, dtype=torch.bfloat16, device=dev), bias.detach(), torch.empty(0, dtype=torch.int64, device=dev))
    assert z.shape == (0, H)
    zb = bias_gather_add_bw(torch.empty(0, H, dtype=torch.bfloat16, device=dev), torch.empty(0, dtype=torch.int64, device=dev), E)
    assert zb.shape == (E, H) and float(zb.abs().max()) == 0.0
    with pytest.raises(ValueError):
        bias_gather_add_fw(torch.zeros(4, 12, dtype=torch.bfloat16, device=dev), torch.zeros(2, 12, dtype=torch.bfloat16, device=dev),
                           torch.zeros(4, dtype=torch.int64, device=dev))  # 24-byte rows



@pytest.mark.parametrize("M,N,K,E", [(4096, 128, 128, 700), (140000, 512, 128, 700)], ids=["tiles128", "tiles256"])
def test_grouped_gemm_more_groups_than_threads(oracle, dev, M, N, K, E):
    """More groups than a workgroup has threads (256 and 512 in the two tile configurations), most
    of them tiny and many empty: the group lookup of a tile then needs more than one pass over the
    offsets.  Reference: dequantise and multiply in float64, expert by expert."""
    from atorch_amd import kernels

    g = torch.Generator().manual_seed(E + M)
    x = randn_bf16((M, K), 3)
    w = randn_bf16((E, N, K), 4, std=0.02)
    cuts = torch.sort(torch.randint(0, M + 1, (E - 1,), generator=g)).values
    cuts[100:300] = cuts[100]  # a run of empty groups
    cuts = torch.sort(cuts).values.tolist()
    b = [0] + cuts + [M]
    splits = [b[i + 1] - b[i] for i in range(E)]
    assert sum(splits) == M and splits.count(0) >= 199
    qx, sx = kernels.tile_quant(x.to(dev))
    qw, sw, _, _ = kernels.block_quant_batched(w.to(dev))
    goff = kernels.group_offsets_from_splits(splits, dev)
    y = kernels.grouped_gemm_nt(qx, sx, qw, sw, goff, out_dtype=torch.float32).cpu()
    xd = oracle.torch_dequant_tile(qx.cpu().view(torch.uint8), sx.cpu()).double()
    ref = torch.zeros(M, N, dtype=torch.float64)
    off = 0
    for e, m in enumerate(splits):
        if m:
            ref[off : off + m] = xd[off : off + m] @ oracle.torch_dequant_block(qw[e].cpu().view(torch.uint8), sw[e].cpu()).double().t()
        off += m
    assert rel_err(y, ref.float()) <= GEMM_TOL_F32


def test_grouped_gemm_random_shapes(dev):
    """Seeded sweep over ragged shapes (both tile configurations, empty groups, partial tiles on both
    sides, bias, both output types; wgrad with and without accumulation on the same routing) against
    the definition of the GEMM evaluated in float64 on the device: dequantise, multiply, add."""
    import random

    from atorch_amd import kernels

    rnd = random.Random(11)

    def deq_tile(q, s):
        return q.float() * s.repeat_interleave(TILE, -1)

    def deq_block(q, s):
        return q.float() * s.repeat_interleave(TILE, -2).repeat_interleave(TILE, -1)

    for case in range(12):
        E = rnd.choice([1, 2, 3, 5, 8, 17, 64, 130])
        N = TILE * rnd.choice([1, 2, 3, 4, 5, 8, 11])
        K = TILE * rnd.choice([1, 2, 3, 4, 8, 9])
        M = rnd.randint(1, 3000) if case % 2 else rnd.randint(20000, 40000)
        cuts = sorted(rnd.randint(0, M) for _ in range(E - 1))
        if E > 3:
            cuts[1] = cuts[0]  # an empty group
        b = [0] + cuts + [M]
        splits = [b[i + 1] - b[i] for i in range(E)]
        x = randn_bf16((M, K), 100 + case).to(dev)
        w = randn_bf16((E, N, K), 200 + case, std=0.02).to(dev)
        qx, sx = kernels.tile_quant(x)
        qw, sw, _, _ = kernels.block_quant_batched(w)
        goff = kernels.group_offsets_from_splits(splits, dev)
        bias = randn_bf16((E, N), 300 + case).to(dev) if case % 3 == 0 else None
        odt = torch.bfloat16 if case % 4 < 2 else torch.float32
        y = kernels.grouped_gemm_nt(qx, sx, qw, sw, goff, out_dtype=odt, bias=bias)
        xd = deq_tile(qx, sx).double()
        ref = torch.zeros(M, N, dtype=torch.float64, device=dev)
        off = 0
        for e, m in enumerate(splits):
            if m:
                ref[off : off + m] = xd[off : off + m] @ deq_block(qw[e], sw[e]).double().t()
                if bias is not None:
                    ref[off : off + m] += bias[e].double()
            off += m
        tol = GEMM_TOL if odt == torch.bfloat16 else GEMM_TOL_F32
        assert rel_err(y.cpu(), ref.float().cpu()) <= tol, (case, M, N, K, E)
        if N * K * E > 32 * 1024 * 1024:
            continue
        dy = randn_bf16((M, N), 400 + case, std=1e-2).to(dev)
        _, _, qxt, sxt = kernels.tile_quant_dual_grouped(x, goff, E, rowwise=False)
        _, _, qdt, sdt = kernels.tile_quant_dual_grouped(dy, goff, E, ld_t=qxt.shape[1], rowwise=False)
        base = torch.randn(E, N, K, generator=torch.Generator().manual_seed(case)).to(dev)
        acc = base.clone()
        kernels.grouped_gemm_wgrad(qdt, sdt, qxt, sxt, goff, out=acc, accumulate=True)
        dw = kernels.grouped_gemm_wgrad(qdt, sdt, qxt, sxt, goff, out_dtype=torch.float32)
        refw = torch.zeros(E, N, K, dtype=torch.float64, device=dev)
        pos = 0
        for e, m in enumerate(splits):
            pad = (m + TILE - 1) // TILE * TILE
            if m:
                a = qdt[:, pos : pos + pad].float() * sdt[pos // TILE : (pos + pad) // TILE].t().repeat_interleave(TILE, 1)
                c = qxt[:, pos : pos + pad].float() * sxt[pos // TILE : (pos + pad) // TILE].t().repeat_interleave(TILE, 1)
                refw[e] = a.double() @ c.double().t()
            pos += pad
        assert rel_err(dw.cpu(), refw.float().cpu()) <= GEMM_TOL_F32, (case, M, N, K, E)
        # the sum with the old values rounds once more in fp32
        assert rel_err((acc - base).cpu(), refw.float().cpu()) <= 4 * GEMM_TOL_F32, (case, M, N, K, E)


# ------------------------------------------------------------------------------------------
# GELU (the expert MLP's default activation) fused into the quantisers
# ------------------------------------------------------------------------------------------
def _gelu_close(got, ref, x):
    """One bf16 unit in the last place of the result (up to 2^-7 of it) plus a few fp32 roundings of 1 + erf(x / sqrt 2) scaled by |x| (that sum
    cancels for x << 0, where device and host erf legitimately differ); and, where nothing cancels
    (x >= -4), at most one unit in the last place on a small fraction of the inputs."""
    got, ref, x = got.cpu(), ref.cpu(), x.cpu()
    err = (got.double() - ref.double()).abs()
    bound = 2.0**-7 * ref.double().abs() + 2.0**-21 * x.double().abs().clamp_min(1.0) + 1e-37
    assert bool((err <= bound).all()), float((err / bound).max())
    mid = x.float() >= -4.0
    d = _ulp_diff(got, ref)
    d = torch.where(got.float() == ref.float(), torch.zeros_like(d), d)[mid]
    assert int(d.max()) <= 1 and float((d > 0).float().mean()) < 5e-3


def test_gelu_forward_and_backward_over_all_bf16_values(oracle, dev):
    """h = gelu(x) and g = dh * gelu'(x) from the fused kernels against the oracle (torch's CPU op and its
    autograd) for every bf16 x of sensible magnitude; codes and scales are exactly the quantisation of
    the kernel's own values."""
    from atorch_amd import kernels

    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    # beyond 2^100 the op's own fp32 product x (1 + erf) overflows; below 2^-100 the CPU op flushes the
    # denormal result x / 2 to zero and the device keeps it: neither occurs among activations
    ax = bits.float().abs()
    x = bits[(ax < 2.0**100) & ((ax > 2.0**-100) | (ax == 0))]
    x = x[: x.numel() // 128 * 128].view(-1, 128).contiguous()
    g = torch.Generator().manual_seed(24)
    dh = torch.randn(x.shape, generator=g).bfloat16()
    M = x.shape[0]
    q, s, h = kernels.gelu_tile_quant(x.to(dev), return_activation=True)
    _gelu_close(h, oracle.gelu(x), x)
    qo, so = oracle.tile_quant(h.cpu())
    assert torch.equal(_u8(q), qo) and torch.equal(s.cpu(), so)
    goff = kernels.group_offsets_from_splits([M], dev)
    qb, sb, qb_t, sb_t, gr = kernels.gelu_tile_quant_dual_grouped(x.to(dev), goff, 1, dh=dh.to(dev), return_activation=True)
    _gelu_close(gr, oracle.gelu_bwd(dh, x), x)
    qo, so = oracle.tile_quant(gr.cpu())
    assert torch.equal(_u8(qb), qo) and torch.equal(sb.cpu(), so)
    # Against the mathematics: x Phi(x) = x erfc(-x / sqrt 2) / 2 and Phi(x) + x pdf(x) evaluated in float64 and
    # rounded once.  Where 1 + erf(x / sqrt 2) keeps its digits the kernels return exactly that value (the CPU op
    # itself misses it on a few inputs).
    xd = x.double()
    phi = 0.5 * torch.special.erfc(-xd / 2.0**0.5)
    want_h = (xd * phi).to(torch.bfloat16)
    assert torch.equal(h.cpu()[x.float() >= -6.0], want_h[x.float() >= -6.0])
    one = torch.ones_like(x)
    gr1 = kernels.gelu_tile_quant_dual_grouped(x.to(dev), goff, 1, dh=one.to(dev), return_activation=True)[4]
    want_g = (phi + xd * torch.exp(-0.5 * xd * xd) / (2.0 * torch.pi) ** 0.5).to(torch.bfloat16)
    assert torch.equal(gr1.cpu()[x.float() >= -4.0], want_g[x.float() >= -4.0])


@pytest.mark.parametrize("backward", [False, True], ids=["fwd", "bwd"])
def test_gelu_quant_dual_grouped(oracle, dev, backward):
    """The fused kernels equal GELU (or its backward) followed by the dual grouped quantisation: outputs
    bit-identical to tile_quant_dual_grouped of their own activation / gradient."""
    from atorch_amd import kernels

    M, F, E = 1000, 384, 5
    splits = ragged_splits(M, E, seed=25)
    goff = kernels.group_offsets_from_splits(splits, dev)
    x = randn_bf16((M, F), 26, std=2.0).to(dev)
    dh = randn_bf16((M, F), 27, std=0.5).to(dev) if backward else None
    q, s, q_t, s_t, h = kernels.gelu_tile_quant_dual_grouped(x, goff, E, dh=dh, return_activation=True)
    ref = oracle.gelu_bwd(dh.cpu(), x.cpu()) if backward else oracle.gelu(x.cpu())
    _gelu_close(h, ref, x)
    q2, s2, q_t2, s_t2 = kernels.tile_quant_dual_grouped(h, goff, E, ld_t=q_t.shape[1])
    ptot = kernels.padded_total(splits)
    assert torch.equal(_u8(q), _u8(q2)) and torch.equal(s, s2)
    assert torch.equal(s_t[: ptot // TILE], s_t2[: ptot // TILE]) and torch.equal(_u8(q_t[:, :ptot]), _u8(q_t2[:, :ptot]))


@pytest.mark.parametrize("M,F,E,mult", [(1000, 384, 6, 1), (512, 256, 4, 128), (3000, 128, 700, 1)])
def test_blocked_layout_of_the_transposed_codes(oracle, dev, M, F, E, mult):
    """Every dual quantiser writes the same transposed codes in the token-block-major layout
    [ld_t/128, rows, 128] as in the row layout [rows, ld_t] (bit for bit, scales included), the oracle's
    transposed quantisation holds for the blocked form directly, and the weight-gradient GEMM gives the same bits
    from operands in either layout."""
    from atorch_amd import kernels

    splits = ragged_splits(M, E, seed=M + F, multiple=mult)
    goff = kernels.group_offsets_from_splits(splits, dev)
    ptot = kernels.padded_total(splits)
    x = heavy_tailed((M, F), seed=3, dtype=torch.bfloat16).to(dev)
    fc1 = randn_bf16((M, 2 * F), 4, std=2.0).to(dev)
    dh = randn_bf16((M, F), 5, std=0.5).to(dev)
    # the same rows as a top-2 dispatch of M / 2 tokens (stable sort of random expert ids)
    T, k = M // 2, 2
    ids = torch.randint(0, E, (T, k), generator=torch.Generator().manual_seed(6)).to(dev)
    sorted_idx, _, pgoff = kernels.moe_preprocess(ids, E)
    xt = x[:T].contiguous()

    calls = {
        "plain": lambda **kw: kernels.tile_quant_dual_grouped(x, goff, E, **kw),
        "permute": lambda **kw: kernels.permute_tile_quant_dual_grouped(xt, sorted_idx, k, pgoff, E, **kw),
        "swiglu": lambda **kw: kernels.swiglu_tile_quant_dual_grouped(fc1, goff, E, **kw),
        "swiglu_bwd": lambda **kw: kernels.swiglu_bwd_tile_quant_dual_grouped(dh, fc1, goff, E, **kw),
        "gelu": lambda **kw: kernels.gelu_tile_quant_dual_grouped(x, goff, E, **kw),
        "gelu_bwd": lambda **kw: kernels.gelu_tile_quant_dual_grouped(x, goff, E, dh=dh, **kw),
    }
    kept = {}
    for name, call in calls.items():
        q, s, q_t, s_t = call()[:4]
        ld_t = q_t.shape[1]
        n = ptot if name != "permute" else int(((pgoff[1:] - pgoff[:-1] + TILE - 1) // TILE * TILE).sum())
        for rowwise in (True, False):
            qb, sb, qb_t, sb_t = call(blocked=True, rowwise=rowwise)[:4]
            assert qb_t.shape == (ld_t // TILE, q_t.shape[0], TILE) and kernels.qt_ld(qb_t) == ld_t
            assert torch.equal(_u8(kernels.qt_rows(qb_t))[:, :n], _u8(q_t)[:, :n]), name
            assert torch.equal(sb_t[: n // TILE], s_t[: n // TILE]), name
            if rowwise:
                assert torch.equal(_u8(qb), _u8(q)) and torch.equal(sb, s), name
        kept[name] = (q_t, s_t, qb_t, sb_t)
    # the definition, on the blocked form itself: block b of column c holds tokens [128 b, 128 b + 128)
    qto, sto = oracle.tile_quant_t_grouped(x.cpu(), splits, ld_t=kept["plain"][0].shape[1])
    blocked = _u8(kept["plain"][2])
    for b in range(ptot // TILE):
        assert torch.equal(blocked[b], qto[:, b * TILE : (b + 1) * TILE])
    # weight gradient of the SwiGLU backward's output against the plain operand, both layouts
    g_t, sg_t, gb_t, sgb_t = kept["swiglu_bwd"]
    x_t, sx_t, xb_t, sxb_t = kept["plain"]
    dw = kernels.grouped_gemm_wgrad(g_t, sg_t, x_t, sx_t, goff, out_dtype=torch.float32)
    dwb = kernels.grouped_gemm_wgrad(gb_t, sgb_t, xb_t, sxb_t, goff, out_dtype=torch.float32)
    assert torch.equal(dw, dwb) and bool(torch.isfinite(dwb).all())
    # heavy-tailed operands (a few codes near 448 among many small ones) show more of the fp8 MFMA's inexact
    # 128-term sums than normal ones do: about 1e-3 measured, against the 1e-2 the path is specified to
    ref = oracle.grouped_gemm_wgrad(_u8(g_t), sg_t.cpu(), _u8(x_t), sx_t.cpu(), splits)
    assert rel_err(dwb.cpu(), ref) <= 4 * GEMM_TOL_F32
    acc = torch.ones_like(dwb)
    kernels.grouped_gemm_wgrad(gb_t, sgb_t, xb_t, sxb_t, goff, out=acc, accumulate=True)
    assert rel_err(acc.cpu() - 1.0, ref) <= 4 * GEMM_TOL_F32
    with pytest.raises(AssertionError, match="same layout"):
        kernels.grouped_gemm_wgrad(gb_t, sgb_t, x_t, sx_t, goff)

"""Pins the CPU oracle: against torch's own fp8 cast, against an exact rational rounder,
against the known answers the reference's tests describe, and against what the mathematics
fixes.  Nothing here re-types an oracle formula: every check is an independent route to the
same answer, chosen so that a dropped term, a wrong index or a transposed operand fails."""
import math

import pytest
import torch

from helpers import TILE, heavy_tailed, ragged_splits, randn_bf16, topk_routing


def _nan_code(u):
    return (u & 0x7F) == 0x7F


# ------------------------------------------------------------------------------------------
# the e4m3fn encoder
# ------------------------------------------------------------------------------------------
def test_encoder_matches_torch_cast_on_all_bf16_patterns(oracle):
    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16)
    x = bits.view(torch.bfloat16).float()
    c = oracle.f32_to_e4m3fn(x)
    t = x.to(torch.float8_e4m3fn).view(torch.uint8)
    assert bool(((c == t) | (_nan_code(c) & _nan_code(t))).all())


def test_encoder_matches_torch_cast_on_random_fp32(oracle):
    g = torch.Generator().manual_seed(0)
    y = torch.randn(1_000_000, generator=g) * torch.exp(torch.randn(1_000_000, generator=g) * 4)
    c = oracle.f32_to_e4m3fn(y)
    t = y.to(torch.float8_e4m3fn).view(torch.uint8)
    assert bool(((c == t) | (_nan_code(c) & _nan_code(t))).all())


def test_encoder_matches_exact_rational_rounder(oracle):
    """Ties, subnormals, the 448/464/465 edge (464 ties to 448, above it NaN)."""
    pts = [0.0, -0.0, 2.0**-10, 1.5 * 2.0**-9, 2.0**-9, 2.0**-10 * 1.0000001, 447.9, 448.0, 449.0, 464.0, 465.0,
           -464.0, 0.0625, 0.0683, 17.0, 18.0, 19.0, 2.0**-6, 2.0**-6 - 2.0**-10, 240.0, 0.3, -0.3, 1e-8]
    g = torch.Generator().manual_seed(1)
    pts += (torch.randn(300, generator=g) * 50).tolist()
    pts += (torch.randn(300, generator=g) * 0.01).tolist()
    # midpoints between neighbouring codes (ties) and their fp32 neighbours
    vals = oracle.e4m3fn_to_f32(torch.arange(0, 0x7F, dtype=torch.uint8)).tolist()
    for a, b in zip(vals[:-1], vals[1:]):
        mid = (a + b) / 2
        pts += [mid, float(torch.nextafter(torch.tensor(mid), torch.tensor(1e9))),
                float(torch.nextafter(torch.tensor(mid), torch.tensor(-1e9)))]
    x = torch.tensor(pts, dtype=torch.float32)
    c = oracle.f32_to_e4m3fn(x).tolist()
    for v, code in zip(x.tolist(), c):
        want = oracle.exact_e4m3fn_code(v)
        assert code == want or (code & 0x7F == 0x7F and want & 0x7F == 0x7F), (v, code, want)


def test_decoder_round_trip(oracle):
    codes = torch.arange(256, dtype=torch.uint8)
    f = oracle.e4m3fn_to_f32(codes)
    t = codes.view(torch.float8_e4m3fn).float()
    ok = torch.isnan(f) == torch.isnan(t)
    assert bool(ok.all()) and torch.equal(f[~torch.isnan(f)], t[~torch.isnan(t)])
    fin = ~torch.isnan(f)
    back = oracle.f32_to_e4m3fn(f[fin])
    # -0 keeps its sign bit, everything finite round-trips
    assert torch.equal(back, codes[fin])


def test_bf16_rounding_matches_torch(oracle):
    g = torch.Generator().manual_seed(2)
    x = torch.randn(200_000, generator=g) * torch.exp(torch.randn(200_000, generator=g) * 3)
    assert torch.equal(oracle.f32_to_bf16(x).view(torch.int16), x.bfloat16().view(torch.int16))


# ------------------------------------------------------------------------------------------
# a1 / a2: tile and block quant
# ------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_tile_and_block_quant_match_torch_restatement(oracle, dtype):
    x = heavy_tailed((384, 512), seed=3, dtype=dtype)
    x[5, :128] = 0
    x[128:256, 128:256] = 0
    q, s = oracle.tile_quant(x)
    q2, s2 = oracle.torch_tile_quant(x)
    assert torch.equal(q, q2) and torch.equal(s, s2)
    q, s = oracle.block_quant(x)
    q2, s2 = oracle.torch_block_quant(x)
    assert torch.equal(q, q2) and torch.equal(s, s2)
    q, s = oracle.tile_quant(x, eps=0.25)
    q2, s2 = oracle.torch_tile_quant(x, eps=0.25)
    assert torch.equal(q, q2) and torch.equal(s, s2)


def test_quant_known_answers(oracle):
    """atorch/tests/common_tests/scaled_linear_test.py:131-133 (zeros), :305-311 (ones, 1000, -512)."""
    x = torch.ones(512, 512, dtype=torch.bfloat16)
    x[0] = 0
    x[1] = 1000
    x[2] = -512
    q, s = oracle.tile_quant(x)
    assert torch.all(s[0] == 1.0) and torch.all(q[0] == 0)
    assert torch.all(q[1] == 0x7E) and torch.all(s[1] == torch.tensor(1000.0) / 448)
    assert torch.all(q[2] == 0xFE) and torch.all(s[2] == torch.tensor(512.0) / 448)
    assert torch.all(q[3:] == 0x7E) and torch.all(s[3:] == torch.tensor(1.0) / 448)
    # any non-zero tile has max |code| = 0x7E
    y = heavy_tailed((64, 256), seed=4)
    qy, _ = oracle.tile_quant(y)
    assert torch.all((qy & 0x7F).view(64, 2, 128).amax(-1) == 0x7E)
    # block quant of the same tensor: first block row holds the 1000 -> one scale for the block
    qb, sb = oracle.block_quant(x)
    assert torch.all(sb[0] == torch.tensor(1000.0) / 448) and torch.all(sb[1:] == torch.tensor(1.0) / 448)
    # tile error <= block error elementwise (scaled_linear_test.py:319)
    et = (x.float() - oracle.dequant(q, s)).abs()
    eb = (x.float() - oracle.dequant(qb, sb)).abs()
    assert torch.all(eb >= et)


def test_quant_error_bound_and_underflow_ordering(oracle):
    """|x - code*s| <= half an fp8 ulp at that magnitude; and the underflow ordering of
    scaled_linear_test.py:116-126 (an outlier hurts block scaling more than tile scaling)."""
    x = torch.rand(512, 512, generator=torch.Generator().manual_seed(5)).bfloat16()
    x[0, 0] = 1e4
    q, s = oracle.tile_quant(x)
    d = oracle.dequant(q, s)
    v = oracle.e4m3fn_to_f32(q).abs()
    ulp = torch.where(v < 2.0**-6, torch.tensor(2.0**-9), torch.exp2(torch.floor(torch.log2(v.clamp_min(2.0**-9))) - 3))
    assert torch.all((x.float() - d).abs() <= 0.5 * ulp * s.repeat_interleave(128, 1) * (1 + 1e-6) + 1e-30)
    qb, sb = oracle.block_quant(x)
    under_tile = ((q & 0x7F) == 0) & (x != 0)
    under_block = ((qb & 0x7F) == 0) & (x != 0)
    assert under_block.sum() >= under_tile.sum()


def test_block_quant_commutes_with_transpose(oracle):
    w = randn_bf16((256, 384), 6, std=0.02)
    q, s = oracle.block_quant(w)
    qt, st = oracle.block_quant(w.t().contiguous())
    assert torch.equal(q.t(), qt) and torch.equal(s.t(), st)


def test_tile_quant_is_row_local(oracle):
    x = heavy_tailed((200, 256), seed=7)
    perm = torch.randperm(200, generator=torch.Generator().manual_seed(0))
    q, s = oracle.tile_quant(x)
    qp, sp = oracle.tile_quant(x[perm])
    assert torch.equal(q[perm], qp) and torch.equal(s[perm], sp)


# ------------------------------------------------------------------------------------------
# a3: transposed quant of ragged groups
# ------------------------------------------------------------------------------------------
def test_transposed_grouped_quant_is_quant_of_padded_transpose(oracle):
    M, K, E = 700, 256, 5
    x = heavy_tailed((M, K), seed=8)
    splits = ragged_splits(M, E, seed=1, multiple=1)
    q_t, s_t = oracle.tile_quant_t_grouped(x, splits)
    off = p = 0
    for m in splits:
        nb = (m + TILE - 1) // TILE
        if m:
            xt = torch.zeros(K, nb * TILE, dtype=x.dtype)
            xt[:, :m] = x[off : off + m].t()
            qo, so = oracle.torch_tile_quant(xt)  # scaled_linear.py:404-414 on the zero padded transpose
            assert torch.equal(q_t[:, p : p + nb * TILE], qo)
            assert torch.equal(s_t[p // TILE : p // TILE + nb].t(), so)
        off += m
        p += nb * TILE
    assert q_t.shape[1] == p


# ------------------------------------------------------------------------------------------
# a5: block-scaled GEMM
# ------------------------------------------------------------------------------------------
def _quantised(oracle, M, N, K, seed):
    a, b = randn_bf16((M, K), seed), randn_bf16((N, K), seed + 1, std=0.02)
    qa, sa = oracle.tile_quant(a)
    qb, sb = oracle.block_quant(b)
    return a, b, qa, sa, qb, sb


def test_gemm_reduces_to_dequantise_and_matmul(oracle):
    M, N, K = 96, 256, 384
    a, b, qa, sa, qb, sb = _quantised(oracle, M, N, K, 10)
    c = oracle.fp8_gemm(qa, sa, qb, sb)
    full = oracle.torch_dequant_tile(qa, sa).double() @ oracle.torch_dequant_block(qb, sb).double().t()
    torch.testing.assert_close(c.double(), full, rtol=1e-5, atol=1e-6)
    # loose sanity against the unquantised product (MSE as in scaled_linear_test.py:92-114)
    exact = a.double() @ b.double().t()
    assert ((c.double() - exact) ** 2).mean() < 0.05 * (exact**2).mean()
    # tile-scaled B (triton_kernel.py:205-208)
    qb2, sb2 = oracle.tile_quant(b)
    c2 = oracle.fp8_gemm(qa, sa, qb2, sb2)
    full2 = oracle.torch_dequant_tile(qa, sa).double() @ oracle.torch_dequant_tile(qb2, sb2).double().t()
    torch.testing.assert_close(c2.double(), full2, rtol=1e-5, atol=1e-6)


def test_gemm_brute_force_tiny(oracle):
    """Pure-python loops in the reference's accumulation order (triton_kernel.py:179-190)."""
    M, N, K = 3, 130, 256
    g = torch.Generator().manual_seed(11)
    qa = torch.randint(0, 0x7F, (M, K), generator=g, dtype=torch.uint8)
    qb = torch.randint(0x80, 0xFF, (N, K), generator=g, dtype=torch.uint8)
    sa = torch.rand(M, K // 128, generator=g) + 0.5
    sb_full = torch.rand(2, K // 128, generator=g) + 0.5  # N=130 -> 2 block rows
    qb_pad = torch.zeros(256, K, dtype=torch.uint8)
    qb_pad[:N] = qb
    c = oracle.fp8_gemm(qa, sa, qb_pad, sb_full)[:, :N]
    va, vb = oracle.e4m3fn_to_f32(qa).double(), oracle.e4m3fn_to_f32(qb).double()
    for m in range(M):
        for n in range(0, N, 43):
            acc = torch.tensor(0.0, dtype=torch.float32)
            for kb in range(K // 128):
                dot = (va[m, kb * 128 : kb * 128 + 128] * vb[n, kb * 128 : kb * 128 + 128]).sum().float()
                acc = acc + dot * sa[m, kb] * sb_full[n // 128, kb]
            assert c[m, n].item() == acc.item()


def test_gemm_linearity_and_accumulate(oracle):
    M, N, K = 40, 128, 256
    _, _, qa, sa, qb, sb = _quantised(oracle, M, N, K, 12)
    c = oracle.fp8_gemm(qa, sa, qb, sb)
    # scaling every A scale by 2 doubles C exactly (power of two)
    assert torch.equal(oracle.fp8_gemm(qa, sa * 2, qb, sb), c * 2)
    out = torch.full((M, N), 1.5)
    oracle.fp8_gemm(qa, sa, qb, sb, out=out, accumulate=True)
    assert torch.equal(out, c + 1.5)


def test_grouped_gemm_equals_per_expert_and_handles_empty_groups(oracle):
    M, N, K, E = 300, 128, 256, 4
    x = randn_bf16((M, K), 13)
    w = randn_bf16((E, N, K), 14, std=0.02)
    splits = [100, 0, 150, 50]
    qx, sx = oracle.tile_quant(x)
    qw = torch.stack([oracle.block_quant(w[e])[0] for e in range(E)])
    sw = torch.stack([oracle.block_quant(w[e])[1] for e in range(E)])
    c = oracle.grouped_gemm_nt(qx, sx, qw, sw, splits)
    d = oracle.torch_grouped_gemm_dequant(qx, sx, qw, sw, splits, out_dtype=torch.float32)
    torch.testing.assert_close(c, d, rtol=1e-5, atol=1e-6)
    # wgrad: dW_g = dY_g^T X_g, both 1x128 along tokens; empty group -> zeros
    dy = randn_bf16((M, N), 15, std=1e-2)
    qdt, sdt = oracle.tile_quant_t_grouped(dy, splits)
    qxt, sxt = oracle.tile_quant_t_grouped(x, splits)
    dw = oracle.grouped_gemm_wgrad(qdt, sdt, qxt, sxt, splits)
    assert torch.all(dw[1] == 0)
    po = oracle.padded_offsets(splits)
    for e in (0, 2, 3):
        a = oracle.e4m3fn_to_f32(qdt[:, po[e] : po[e + 1]]).double() * sdt[po[e] // 128 : po[e + 1] // 128].t().repeat_interleave(128, 1).double()
        b = oracle.e4m3fn_to_f32(qxt[:, po[e] : po[e + 1]]).double() * sxt[po[e] // 128 : po[e + 1] // 128].t().repeat_interleave(128, 1).double()
        ref = a @ b.t()
        torch.testing.assert_close(dw[e].double(), ref, rtol=1e-5, atol=1e-5 * float(ref.abs().max()))
        off = sum(splits[:e])
        exact = dy[off : off + splits[e]].double().t() @ x[off : off + splits[e]].double()
        assert ((dw[e].double() - exact) ** 2).mean() < 0.05 * (exact**2).mean()
    base = torch.ones(E, N, K)
    out = base.clone()
    oracle.grouped_gemm_wgrad(qdt, sdt, qxt, sxt, splits, out=out, accumulate=True)
    assert torch.equal(out[1], base[1])
    torch.testing.assert_close(out, base + dw, rtol=1e-6, atol=1e-7)


# ------------------------------------------------------------------------------------------
# a9 / a10: permute and unpermute
# ------------------------------------------------------------------------------------------
def test_permute_is_stable_sort_by_expert(oracle):
    T, E, k = 61, 5, 2
    idx, _ = topk_routing(T, E, k, seed=16)
    tokens = randn_bf16((T, 32), 17)
    p, so, counts = oracle.permute(tokens, idx, E)
    # brute force: for every expert in order, every flat index in order
    flat = idx.reshape(-1).tolist()
    want = [i for e in range(E) for i in range(T * k) if flat[i] == e]
    assert so.tolist() == want
    assert counts.tolist() == [flat.count(e) for e in range(E)]
    assert torch.equal(p, tokens[torch.tensor(want) // k])
    tp, tso = oracle.torch_permute(tokens, idx)
    assert torch.equal(tso, so) and torch.equal(tp, p)


@pytest.mark.parametrize("pdtype", [torch.bfloat16, torch.float32])
def test_unpermute_brute_force_and_torch_restatement(oracle, pdtype):
    T, E, k, H = 37, 6, 4, 24
    idx, probs = topk_routing(T, E, k, seed=18)
    probs = probs.to(pdtype)
    y = randn_bf16((T * k, H), 19)
    so, _ = oracle.permute_indices(idx, E)
    out = oracle.unpermute(y, so, probs)
    inv = {int(f): j for j, f in enumerate(so.tolist())}
    for t in range(0, T, 5):
        for h in range(0, H, 7):
            acc = torch.tensor(0.0)
            for j in range(k):
                term = y[inv[t * k + j], h] * probs[t, j]  # rounds to the promoted dtype
                acc = acc + term.float()
            assert out[t, h].item() == acc.to(out.dtype).item()
    ref = oracle.torch_unpermute(y, so, probs)
    assert ref.dtype == out.dtype
    tol = 2.0**-7 if out.dtype == torch.bfloat16 else 1e-6
    torch.testing.assert_close(out.float(), ref.float(), rtol=tol, atol=1e-6)


def test_unpermute_inverts_permute(oracle):
    T, E = 50, 4
    idx = torch.randint(0, E, (T,), generator=torch.Generator().manual_seed(20))
    x = randn_bf16((T, 16), 21)
    p, so, _ = oracle.permute(x, idx, E)
    assert torch.equal(oracle.unpermute(p, so), x)
    # top-2 with probs 1/2 each: returns x up to bf16 rounding of the halves (exact: power of two)
    idx2, _ = topk_routing(T, E, 2, seed=22)
    p2, so2, _ = oracle.permute(x, idx2, E)
    half = torch.full((T, 2), 0.5, dtype=torch.bfloat16)
    assert torch.equal(oracle.unpermute(p2, so2, half), x)


# ------------------------------------------------------------------------------------------
# a6 / a7: the grouped linear as a whole
# ------------------------------------------------------------------------------------------
def test_grouped_linear_oracle_against_fp64_autograd(oracle):
    """fwd / dgrad / wgrad of the quantised path track the exact bf16-input results
    (loose: quantisation noise only), which catches transposed operands and swapped roles."""
    M, K, N, E = 320, 256, 128, 3
    x = randn_bf16((M, K), 23)
    ws = [randn_bf16((N, K), 24 + e, std=0.02) for e in range(E)]
    dy = randn_bf16((M, N), 30, std=1e-2)
    splits = [128, 0, 192]
    r = oracle.grouped_linear_fwd_bwd(x, ws, splits, dy)
    xd = x.double().requires_grad_(True)
    wd = [w.double().requires_grad_(True) for w in ws]
    outs, off = [], 0
    for e, m in enumerate(splits):
        outs.append(xd[off : off + m] @ wd[e].t())
        off += m
    out = torch.cat(outs)
    out.backward(dy.double())

    def close(a, b):
        return ((a.double() - b) ** 2).mean() <= 2e-3 * (b**2).mean() + 1e-30

    assert close(r["out"], out.detach())
    assert close(r["dgrad"], xd.grad)
    for e in range(E):
        assert close(r["wgrad"][e], wd[e].grad)
    assert torch.all(r["wgrad"][1] == 0)
    assert math.isclose(float(r["bgrad"][0].sum()), float(dy[:128].float().sum()), rel_tol=1e-5)


def test_swiglu_matches_torch_and_closed_forms(oracle):
    """grouped_gemm_moe.py:331-334: F.silu(a) * b on bf16 tensors.  Over every finite bf16 value of a
    (b = 1 and b random) the oracle equals torch's CPU ops; silu(0) = 0, silu(x) = x for large x and
    -0 for very negative x; and h tracks a * sigmoid(a) * b computed in float64 within bf16 rounding."""
    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    a = bits[torch.isfinite(bits.float())]
    n = a.numel() // 128 * 128
    a = a[:n].view(-1, 128)
    g = torch.Generator().manual_seed(3)
    for b in (torch.ones_like(a), (torch.randn(a.shape, generator=g) * 2).bfloat16()):
        fc1 = torch.cat([a, b], dim=1).contiguous()
        h = oracle.swiglu(fc1)
        t = oracle.torch_swiglu(fc1)
        assert torch.equal(h.view(torch.int16), t.view(torch.int16))
        exact = a.double() * torch.sigmoid(a.double()) * b.double()
        ok = (exact.abs() < 1e37) & (exact.abs() > 1e-30) & (a.double() > -87.0)  # below: exp(-a) overflows in fp32
        rel = ((h.double() - exact).abs() / exact.abs())[ok]
        assert float(rel.max()) < 2.0**-7  # two bf16 roundings
    z = torch.tensor([[0.0, -0.0, 80.0, -120.0] + [0.0] * 124 + [3.0] * 128]).bfloat16()
    h = oracle.swiglu(z)
    assert h[0, 0].item() == 0.0 and h[0, 2].item() == 240.0 and h[0, 3].item() == 0.0


def test_swiglu_bwd_matches_torch_autograd_and_finite_differences(oracle):
    """Gradient of F.silu(a) * b through torch's CPU autograd on bf16 tensors, over every finite bf16
    value of a: the oracle reproduces it bit for bit.  Independently of torch, the analytic gradient
    agrees with a float64 central difference of h = a * sigmoid(a) * b within bf16 rounding, and
    db = dh * silu(a), da(a = 0) = dh * b / 2."""
    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    a = bits[torch.isfinite(bits.float())]
    a = a[: a.numel() // 128 * 128].view(-1, 128)
    g = torch.Generator().manual_seed(13)
    b = (torch.randn(a.shape, generator=g) * 2).bfloat16()
    dh = torch.randn(a.shape, generator=g).bfloat16()
    fc1 = torch.cat([a, b], dim=1).contiguous()
    leaf = fc1.clone().requires_grad_(True)
    x0, x1 = torch.chunk(leaf, 2, dim=-1)
    (torch.nn.functional.silu(x0) * x1).backward(dh)
    mine = oracle.swiglu_bwd(dh, fc1)
    same = (mine.view(torch.int16) == leaf.grad.view(torch.int16)) | (mine.float() == leaf.grad.float())
    assert bool(same.all())
    # float64 finite differences on a moderate range (where bf16 spacing of a is far above the step)
    sel = (a.double().abs() < 20.0) & (a.double().abs() > 1e-3)
    ad, bd, dd = a.double(), b.double(), dh.double()
    f = lambda t: t * torch.sigmoid(t)
    eps = 1e-6
    da_fd = dd * bd * (f(ad + eps) - f(ad - eps)) / (2 * eps)
    db_ex = dd * f(ad)
    da, db = mine[:, :128].double(), mine[:, 128:].double()
    tol = lambda ref: 3 * 2.0**-8 * ref.abs() + 1e-30  # three bf16 roundings
    assert bool(((da - da_fd).abs() <= tol(da_fd) + 1e-6 * (dd * bd).abs())[sel].all())
    assert bool(((db - db_ex).abs() <= tol(db_ex))[sel].all())
    z = torch.zeros(1, 256, dtype=torch.bfloat16)
    z[0, 128:] = 3.0
    d1 = torch.full((1, 128), 2.0, dtype=torch.bfloat16)
    out = oracle.swiglu_bwd(d1, z)
    assert float(out[0, 0]) == 3.0 and float(out[0, 128]) == 0.0  # dh * b / 2 and dh * silu(0)


def test_bias_gather_add_matches_torch(oracle):
    """bias_gather_add.py:24-47, :80-98: forward equals torch's ``inp + bias[bin_ids]`` bit for bit
    (bf16 and fp32); the bias gradient equals ``index_add_`` in float64 within fp32 summation error,
    exactly on data whose sums are exact, and rows of absent experts stay zero."""
    g = torch.Generator().manual_seed(21)
    T, H, E = 257, 136, 7
    ids = torch.randint(0, E - 1, (T,), generator=g)  # expert E-1 gets no rows
    for dt in (torch.bfloat16, torch.float32):
        inp = torch.randn(T, H, generator=g).to(dt)
        bias = torch.randn(E, H, generator=g).to(dt)
        out = oracle.bias_gather_add(inp, bias, ids)
        ref = inp + bias[ids]
        assert torch.equal(out.view(torch.int16 if dt == torch.bfloat16 else torch.int32),
                           ref.view(torch.int16 if dt == torch.bfloat16 else torch.int32))
        bg = oracle.bias_gather_bgrad(inp, ids, E)
        ref64 = torch.zeros(E, H, dtype=torch.float64).index_add_(0, ids, inp.double())
        assert float((bg.double() - ref64).abs().max()) < 1e-4
        assert float(bg[E - 1].abs().max()) == 0.0
        small = torch.randint(-8, 9, (T, H), generator=g).to(dt)  # integer sums are exact in fp32
        exact = torch.zeros(E, H, dtype=torch.float64).index_add_(0, ids, small.double())
        assert torch.equal(oracle.bias_gather_bgrad(small, ids, E).double(), exact)



def test_gelu_oracle_against_the_closed_form_over_all_bf16_values(oracle):
    """oracle.gelu / gelu_bwd (torch's CPU op and its autograd) against x/2 (1 + erf(x/sqrt 2)) and
    dh (cdf + x pdf) evaluated in float64, for every finite bf16 x.  The op works in fp32, where
    1 + erf(x/sqrt 2) cancels for x << 0, so the bound is one bf16 rounding of the result plus an fp32
    rounding of x; where neither cancellation nor denormals play (1e-30 <= |x| <= 4) the results agree
    to one unit in the last place."""
    import math

    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    x = bits[bits.float().abs() < 2.0**100]  # beyond, the op's own fp32 product x (1 + erf) overflows
    x64 = x.double()
    cdf = 0.5 * (1.0 + torch.special.erf(x64 / math.sqrt(2.0)))
    pdf = torch.exp(-0.5 * x64 * x64) / math.sqrt(2.0 * math.pi)
    g = torch.Generator().manual_seed(3)
    dh = torch.randn(x.shape, generator=g).bfloat16()
    mid = (x64.abs() >= 1e-30) & (x64.abs() <= 4.0)

    def ulps(a, b):
        d = (a.view(torch.int16).int() - b.view(torch.int16).int()).abs()
        return torch.where(a.float() == b.float(), torch.zeros_like(d), d)

    for got, ref64 in ((oracle.gelu(x), x64 * cdf), (oracle.gelu_bwd(dh, x), dh.double() * (cdf + x64 * pdf))):
        err = (got.double() - ref64).abs()
        scale = x64.abs() if got is not None else None
        bound = 2.0**-8 * ref64.abs() + 2.0**-22 * torch.maximum(scale, torch.ones_like(scale)) + 1e-37
        assert bool((err <= bound).all()), float((err / bound).max())
        d = ulps(got, ref64.to(torch.bfloat16))[mid]
        assert int(d.max()) <= 1 and float((d > 0).float().mean()) < 5e-3
    # known answers: gelu(0) = 0, gelu(large) = x, gelu(-large) = -0; gelu'(0) = 1/2, gelu'(large) = 1
    assert oracle.gelu(torch.tensor([0.0, 40.0, -40.0]).bfloat16()).float().tolist() == [0.0, 40.0, -0.0]
    one = torch.ones(3).bfloat16()
    assert oracle.gelu_bwd(one, torch.tensor([0.0, 40.0, -40.0]).bfloat16()).float().tolist() == [0.5, 1.0, 0.0]

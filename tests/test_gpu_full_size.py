"""Full-size runs of the benchmark configurations on the GPU, checked through size-independent
properties and through sampled rows against the CPU oracle:

  * quantise / permute at 65536 x 7168, top-8 into 64 experts: sampled rows bit-exact against the
    oracle, permute-then-quantise == quantise-then-permute, unpermute inverts permute;
  * grouped GEMMs at the Mixtral-like, DeepSeek-like (Zipf-ragged, empty groups) and Qwen-like
    shapes: sampled output rows against a float64 dequantise-and-matmul, and a checksum of
    checksums (the column sums of a group's output equal the summed rows of the group times the
    weight), both computed with plain torch float64 on the same device, independent of the HIP kernels.
"""
import pytest
import torch

from helpers import TILE

pytestmark = pytest.mark.gpu
FP8 = torch.float8_e4m3fn
GEMM_TOL = 1e-2  # bf16 outputs, max relative error (rms floor)
SUM_TOL = 2e-3  # checksums of fp32 outputs relative to the checksum's rms


def _randn(shape, dev, std, seed):
    g = torch.Generator(device=dev).manual_seed(seed)
    out = torch.empty(shape, dtype=torch.bfloat16, device=dev)
    step = max(1, (1 << 27) // max(1, out[0].numel()))
    for r in range(0, shape[0], step):
        n = min(step, shape[0] - r)
        out[r : r + n] = (torch.randn((n, *shape[1:]), generator=g, device=dev) * std).to(torch.bfloat16)
    return out


def _student_t(shape, dev, seed):
    g = torch.Generator(device=dev).manual_seed(seed)
    out = torch.empty(shape, dtype=torch.bfloat16, device=dev)
    step = max(1, (1 << 25) // shape[1])
    for r in range(0, shape[0], step):
        n = min(step, shape[0] - r)
        z = torch.randn((n, shape[1]), generator=g, device=dev)
        chi = torch.randn((n, shape[1], 3), generator=g, device=dev).pow(2).sum(-1)
        out[r : r + n] = (z / torch.sqrt(chi / 3)).to(torch.bfloat16)
    return out


def _routing(T, E, k, dev, zipf_s=None, seed=2):
    g = torch.Generator(device=dev).manual_seed(seed)
    if zipf_s is None:
        logits = torch.randn(T, E, generator=g, device=dev)
    else:
        p = torch.arange(1, E + 1, dtype=torch.float32, device=dev).pow(-zipf_s)
        u = torch.rand(T, E, generator=g, device=dev).clamp_min(1e-30)
        logits = p.log() - torch.log(-torch.log(u))
    vals, idx = torch.topk(logits, k, dim=1)
    return idx, torch.softmax(vals, dim=1)


def _rel(c, ref):
    c, ref = c.double(), ref.double()
    floor = ref.pow(2).mean().sqrt().clamp_min(1e-30)
    return float(((c - ref).abs() / torch.maximum(ref.abs(), floor)).max())


def _f64(q):
    """fp8 codes (as fp8 or as their uint8 view) to float64."""
    return (q.view(FP8) if q.dtype == torch.uint8 else q).float().double()


def _deq_rows(q, s):
    """float64 dequantisation of 1x128-scaled rows on the device (plain torch)."""
    return _f64(q) * s.double().repeat_interleave(TILE, dim=1)


def _deq_block(q, s):
    return _f64(q) * s.double().repeat_interleave(TILE, 0).repeat_interleave(TILE, 1)


# ------------------------------------------------------------------------------------------
# quantise / permute at full size
# ------------------------------------------------------------------------------------------
def test_permute_quant_full_size(oracle, dev):
    from atorch_amd import kernels as K

    T, H, E, k = 65536, 7168, 64, 8
    x = _student_t((T, H), dev, seed=0)
    idx, probs = _routing(T, E, k, dev)
    sorted_idx, row_map, goff = K.moe_preprocess(idx, E)
    M = T * k
    # the permutation is the stable sort of the flattened ids
    flat = idx.view(-1)
    ids_sorted = flat[sorted_idx]
    assert bool((ids_sorted[1:] >= ids_sorted[:-1]).all())
    same = ids_sorted[1:] == ids_sorted[:-1]
    assert bool((sorted_idx[1:][same] > sorted_idx[:-1][same]).all())  # stability
    assert torch.equal(torch.bincount(flat, minlength=E), goff[1:] - goff[:-1])
    assert torch.equal(row_map.view(-1)[sorted_idx], torch.arange(M, device=dev, dtype=row_map.dtype))

    q, s = K.permute_tile_quant(x, row_map, k, M)
    # quantise-then-permute: the codes of a token are the same in each of its k copies
    q0, s0 = K.tile_quant(x)
    src = (sorted_idx // k).to(torch.int64)
    q0u = q0.view(torch.uint8)
    for lo in range(0, M, 1 << 16):
        hi = min(M, lo + (1 << 16))
        assert torch.equal(q[lo:hi].view(torch.uint8), q0u[src[lo:hi]])
        assert torch.equal(s[lo:hi], s0[src[lo:hi]])
    # sampled source rows bit-exact against the CPU oracle
    g = torch.Generator().manual_seed(1)
    rows = torch.randint(0, T, (96,), generator=g)
    amax_row = x.float().abs().amax(dim=1).argmax().item()  # include the heaviest outlier
    rows[0] = amax_row
    qo, so = oracle.tile_quant(x[rows.to(dev)].cpu())
    assert torch.equal(q0u[rows.to(dev)].cpu(), qo)
    assert torch.equal(s0[rows.to(dev)].cpu(), so)
    del q, s, q0, s0, q0u

    # unpermute inverts permute: with probs = 1/k the combine returns x up to bf16 rounding of
    # each product and of the sum; with exact weights (k = 8 -> 0.125) every step is exact
    y = K.permute_rows(x, row_map, k, M)
    assert torch.equal(y[: 1 << 14], x[src[: 1 << 14]])
    w = torch.full((T, k), 1.0 / k, dtype=torch.bfloat16, device=dev)
    back = K.unpermute_combine(y, row_map, w, T, k)
    assert torch.equal(back, x)
    # real probabilities: sampled tokens against the oracle
    pb = probs.to(torch.bfloat16)
    out = K.unpermute_combine(y, row_map, pb, T, k)
    toks = torch.randint(0, T, (64,), generator=g)
    for tkn in toks.tolist():
        rows_of = row_map.view(T, k)[tkn].to(torch.int64)
        ref = oracle.unpermute(y[rows_of].cpu(), torch.arange(k), pb[tkn : tkn + 1].cpu())
        assert torch.equal(out[tkn : tkn + 1].cpu(), ref)


def test_dual_grouped_quant_full_size(oracle, dev):
    """Transposed 1x128 quantisation along tokens inside ragged groups at the Qwen-like size
    (131072 rows x 2048, 60 groups): columns of sampled tiles against the oracle, and the row
    output equal to the plain 1x128 kernel."""
    from atorch_amd import kernels as K

    T, E, k, H = 32768, 60, 4, 2048
    idx, _ = _routing(T, E, k, dev)
    _, _, goff = K.moe_preprocess(idx, E, want_sorted=False)
    M = T * k
    x = _student_t((M, H), dev, seed=3)
    q, s, q_t, s_t = K.tile_quant_dual_grouped(x, goff, E)
    q1, s1 = K.tile_quant(x)
    assert torch.equal(q.view(torch.uint8), q1.view(torch.uint8)) and torch.equal(s, s1)
    counts = (goff[1:] - goff[:-1]).cpu().tolist()
    pad = [0]
    for c in counts:
        pad.append(pad[-1] + (c + TILE - 1) // TILE * TILE)
    offs = goff.cpu().tolist()
    for e in (0, 17, E - 1):
        m = counts[e]
        xe = x[offs[e] : offs[e] + m, :256].cpu()  # 256 of the 2048 columns keep the CPU work small
        qt_o, st_o = oracle.tile_quant_t_grouped(xe, [m])
        assert torch.equal(q_t[:256, pad[e] : pad[e + 1]].view(torch.uint8).cpu(), qt_o[:, : pad[e + 1] - pad[e]])
        assert torch.equal(s_t[pad[e] // TILE : pad[e + 1] // TILE, :256].cpu(), st_o[: (pad[e + 1] - pad[e]) // TILE])
        # the padding columns of a partial tile hold zero codes
        assert bool((q_t[:, pad[e] + m : pad[e + 1]].view(torch.uint8) == 0).all())


@pytest.mark.parametrize("T,E,k,H,heavy", [(65536, 64, 8, 7168, True), (32768, 60, 4, 2048, False)],
                         ids=["c5_shape", "c4_shape"])
def test_permute_quant_dual_grouped_full_size(oracle, dev, T, E, k, H, heavy):
    """The training form of the fused permute at the sizes of the quant / permute configuration (65536 x 7168, top-8
    into 64 experts) and of the Qwen-like one: equal to permute_rows followed by the dual grouped quantiser bit for
    bit over the whole outputs, its row-wise part equal to the scatter form (every token quantised once), and sampled
    columns of sampled groups against the oracle.  The fused kernel writes its transposed codes token-block-major,
    the separate ones a row per column: the comparison covers both layouts."""
    from atorch_amd import kernels as K

    x = _student_t((T, H), dev, seed=0) if heavy else _randn((T, H), dev, 1.0, 7)
    idx, _ = _routing(T, E, k, dev)
    sorted_idx, row_map, goff = K.moe_preprocess(idx, E)
    M = T * k
    # the token-block-major layout the training path uses, compared below with the row layout of the separate kernels
    q, s, q_tb, s_t = K.permute_tile_quant_dual_grouped(x, sorted_idx, k, goff, E, blocked=True)
    q_t = K.qt_rows(q_tb)
    del q_tb
    counts = (goff[1:] - goff[:-1]).cpu().tolist()
    pad = [0]
    for c in counts:
        pad.append(pad[-1] + (c + TILE - 1) // TILE * TILE)
    pe = pad[-1]
    # row-wise part: the codes and scales of the scatter form
    q1, s1 = K.permute_tile_quant(x, row_map, k, M)
    assert torch.equal(q.view(torch.uint8), q1.view(torch.uint8)) and torch.equal(s, s1)
    del q1, s1
    # everything: the two separate kernels
    xp = K.permute_rows(x, row_map, k, M)
    q2, s2, q_t2, s_t2 = K.tile_quant_dual_grouped(xp, goff, E, ld_t=q_t.shape[1])
    assert torch.equal(q.view(torch.uint8), q2.view(torch.uint8)) and torch.equal(s, s2)
    assert torch.equal(q_t.view(torch.uint8)[:, :pe], q_t2.view(torch.uint8)[:, :pe])
    assert torch.equal(s_t[: pe // TILE], s_t2[: pe // TILE])
    del q2, s2, q_t2, s_t2
    # sampled groups against the oracle (256 columns keep the CPU work small)
    offs = goff.cpu().tolist()
    for e in (0, E // 3, E - 1):
        m = counts[e]
        xe = xp[offs[e] : offs[e] + m, :256].cpu()
        qt_o, st_o = oracle.tile_quant_t_grouped(xe, [m])
        assert torch.equal(q_t[:256, pad[e] : pad[e + 1]].view(torch.uint8).cpu(), qt_o[:, : pad[e + 1] - pad[e]])
        assert torch.equal(s_t[pad[e] // TILE : pad[e + 1] // TILE, :256].cpu(), st_o[: (pad[e + 1] - pad[e]) // TILE])
        assert bool((q_t[:, pad[e] + m : pad[e + 1]].view(torch.uint8) == 0).all())


# ------------------------------------------------------------------------------------------
# grouped GEMMs at full size
# ------------------------------------------------------------------------------------------
def _check_nt(K_, qa, sa, qb, sb, goff, dev, seed):
    """Forward / dgrad launch: bf16 output rows sampled in every group against float64, and the
    per-group checksum of an fp32 output."""
    M, Kd = qa.shape
    E, N, _ = qb.shape
    y = K_.grouped_gemm_nt(qa, sa, qb, sb, goff)
    offs = goff.cpu().tolist()
    g = torch.Generator().manual_seed(seed)
    worst = 0.0
    for e in range(E):
        m = offs[e + 1] - offs[e]
        if m == 0:
            continue
        if E > 16 and e % 7 and m > 8:  # many experts: sample every 7th plus all tiny groups
            continue
        rows = offs[e] + torch.randint(0, m, (min(m, 6),), generator=g)
        rows = torch.unique(torch.cat([rows, torch.tensor([offs[e], offs[e + 1] - 1])])).to(dev)
        ref = _deq_rows(qa.view(torch.uint8)[rows], sa[rows]) @ _deq_block(qb[e], sb[e]).t()
        worst = max(worst, _rel(y[rows], ref))
    assert worst < GEMM_TOL, worst
    del y
    y32 = K_.grouped_gemm_nt(qa, sa, qb, sb, goff, out_dtype=torch.float32)
    worst = 0.0
    for e in range(E):
        m = offs[e + 1] - offs[e]
        if m == 0 or (E > 16 and e % 5):
            continue
        u = torch.zeros(Kd, dtype=torch.float64, device=dev)
        for lo in range(offs[e], offs[e + 1], 4096):
            hi = min(offs[e + 1], lo + 4096)
            u += _deq_rows(qa[lo:hi], sa[lo:hi]).sum(0)
        want = _deq_block(qb[e], sb[e]) @ u
        got = y32[offs[e] : offs[e + 1]].double().sum(0)
        worst = max(worst, _rel(got, want))
    assert worst < SUM_TOL, worst


def _layer_operands(K_, M, Kd, N, E, goff, dev, seed, backward):
    x = _randn((M, Kd), dev, 1.0, seed)
    w = _randn((E, N, Kd), dev, 0.02, seed + 1)
    ops = {}
    if backward:
        ops["qx"], ops["sx"], ops["qx_t"], ops["sx_t"] = K_.tile_quant_dual_grouped(x, goff, E)
        dy = _randn((M, N), dev, 1e-2, seed + 2)
        ops["qdy"], ops["sdy"], ops["qdy_t"], ops["sdy_t"] = K_.tile_quant_dual_grouped(dy, goff, E)
        ops["qw"], ops["sw"], ops["qw_t"], ops["sw_t"] = K_.block_quant_batched(w, return_transpose=True)
    else:
        ops["qx"], ops["sx"] = K_.tile_quant(x)
        ops["qw"], ops["sw"], _, _ = K_.block_quant_batched(w)
    return ops


def _check_wgrad(K_, ops, goff, E, N, Kd, dev, seed):
    dw = K_.grouped_gemm_wgrad(ops["qdy_t"], ops["sdy_t"], ops["qx_t"], ops["sx_t"], goff)
    counts = (goff[1:] - goff[:-1]).cpu().tolist()
    pad = [0]
    for c in counts:
        pad.append(pad[-1] + (c + TILE - 1) // TILE * TILE)
    g = torch.Generator().manual_seed(seed)
    worst = 0.0
    for e in range(E):
        if E > 16 and e % 9:
            continue
        p0, p1 = pad[e], pad[e + 1]
        if p1 == p0:
            assert bool((dw[e] == 0).all())
            continue
        rows = torch.randint(0, N, (8,), generator=g).to(dev)
        a = _f64(ops["qdy_t"].view(torch.uint8)[rows, p0:p1]) * ops["sdy_t"][p0 // TILE : p1 // TILE][:, rows].t().double().repeat_interleave(TILE, 1)
        b = _f64(ops["qx_t"][:, p0:p1]) * ops["sx_t"][p0 // TILE : p1 // TILE].t().double().repeat_interleave(TILE, 1)
        worst = max(worst, _rel(dw[e][rows], a @ b.t()))
    assert worst < 5e-4, worst  # fp32 output
    # accumulate: a second launch on top doubles the result
    dw2 = dw.clone()
    K_.grouped_gemm_wgrad(ops["qdy_t"], ops["sdy_t"], ops["qx_t"], ops["sx_t"], goff, out=dw2, accumulate=True)
    assert torch.equal(dw2, dw + dw)
    del dw2
    # the token-block-major operand layout [ld_t/128, rows, 128] (what the training path hands over), made here by
    # plain torch from the row layout: the same bits
    blk = lambda t: t.view(torch.uint8).view(t.shape[0], -1, TILE).permute(1, 0, 2).contiguous().view(FP8)  # noqa: E731
    dwb = K_.grouped_gemm_wgrad(blk(ops["qdy_t"]), ops["sdy_t"], blk(ops["qx_t"]), ops["sx_t"], goff)
    assert torch.equal(dwb, dw)


def test_grouped_gemm_mixtral_full_size(dev):
    """8 experts, 16384 tokens top-2 (32768 rows), 4096 -> 28672 and 14336 -> 4096."""
    from atorch_amd import kernels as K_

    E, T, k = 8, 16384, 2
    idx, _ = _routing(T, E, k, dev)
    _, _, goff = K_.moe_preprocess(idx, E, want_sorted=False)
    M = T * k
    for i, (Kd, N) in enumerate([(4096, 28672), (14336, 4096)]):
        ops = _layer_operands(K_, M, Kd, N, E, goff, dev, 10 * i, backward=True)
        _check_nt(K_, ops["qx"], ops["sx"], ops["qw"], ops["sw"], goff, dev, 1)
        _check_nt(K_, ops["qdy"], ops["sdy"], ops["qw_t"], ops["sw_t"], goff, dev, 2)
        _check_wgrad(K_, ops, goff, E, N, Kd, dev, 3)
        del ops
        torch.cuda.empty_cache()


def test_grouped_gemm_deepseek_ragged_full_size(dev):
    """64 experts, 8192 tokens top-8 with Zipf(1.2) popularity: heavily ragged, empty groups."""
    from atorch_amd import kernels as K_

    E, T, k = 64, 8192, 8
    idx, _ = _routing(T, E, k, dev, zipf_s=1.2)
    # the batch must hold at least one empty group: drop the rarest experts' few tokens onto expert 0
    counts = torch.bincount(idx.view(-1), minlength=E)
    if int((counts == 0).sum()) == 0:
        rare = counts.argmin()
        idx = torch.where(idx == rare, torch.zeros_like(idx), idx)
    _, _, goff = K_.moe_preprocess(idx, E, want_sorted=False)
    assert int(((goff[1:] - goff[:-1]) == 0).sum()) >= 1
    M = T * k
    for i, (Kd, N) in enumerate([(7168, 4096), (2048, 7168)]):
        ops = _layer_operands(K_, M, Kd, N, E, goff, dev, 20 + 10 * i, backward=False)
        _check_nt(K_, ops["qx"], ops["sx"], ops["qw"], ops["sw"], goff, dev, 4)
        del ops
        torch.cuda.empty_cache()


def test_grouped_gemm_qwen_full_size(dev):
    """60 experts, 32768 tokens top-4 (131072 rows), 2048 -> 2816 and 1408 -> 2048, fwd + dgrad + wgrad."""
    from atorch_amd import kernels as K_

    E, T, k = 60, 32768, 4
    idx, _ = _routing(T, E, k, dev)
    _, _, goff = K_.moe_preprocess(idx, E, want_sorted=False)
    M = T * k
    for i, (Kd, N) in enumerate([(2048, 2816), (1408, 2048)]):
        ops = _layer_operands(K_, M, Kd, N, E, goff, dev, 40 + 10 * i, backward=True)
        _check_nt(K_, ops["qx"], ops["sx"], ops["qw"], ops["sw"], goff, dev, 5)
        _check_nt(K_, ops["qdy"], ops["sdy"], ops["qw_t"], ops["sw_t"], goff, dev, 6)
        _check_wgrad(K_, ops, goff, E, N, Kd, dev, 7)
        del ops
        torch.cuda.empty_cache()

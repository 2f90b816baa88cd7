"""Golden vectors (tests/golden/*.npz, written by tests/golden/make_fixtures.py).

CPU: the oracle reproduces the stored outputs; independent of the oracle's C code, the stored
codes and scales satisfy the closed form (exact rational rounding, known answers of
scaled_linear_test.py:305-319 and :116-133) and the stored GEMM results equal a float64
dequantise-and-matmul of the stored fp8 operands.
GPU: the HIP kernels, through the C ABI, reproduce the stored outputs (bit-exact for codes, scales,
permutations and the combine; within 1e-2 for the bf16 GEMM outputs, the stated GEMM tolerance).
"""
import os
from fractions import Fraction

import numpy as np
import pytest
import torch

from helpers import TILE, rel_err

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
GEMM_TOL = 1e-2  # max relative error of a bf16 GEMM output
GEMM_TOL_F32 = 5e-4  # fp32 outputs: the fp8 MFMA's 128-term dot is not exactly rounded (about 1e-4 of rms)


def load(name):
    with np.load(os.path.join(GOLDEN, name + ".npz"), allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


def bf16(a):
    return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)


def t(a):
    return torch.from_numpy(a.copy())


# ------------------------------------------------------------------------------------------
# CPU
# ------------------------------------------------------------------------------------------
def test_oracle_reproduces_quant_vectors(oracle):
    g = load("quant_known_answers")
    q, s = oracle.tile_quant(bf16(g["x"]))
    assert np.array_equal(q.numpy(), g["q"]) and np.array_equal(s.numpy(), g["s"])
    qb, sb = oracle.block_quant(bf16(g["xb"]))
    assert np.array_equal(qb.numpy(), g["qb"]) and np.array_equal(sb.numpy(), g["sb"])
    g = load("quant_random")
    q, s = oracle.tile_quant(bf16(g["x"]))
    assert np.array_equal(q.numpy(), g["q"]) and np.array_equal(s.numpy(), g["s"])
    q, s = oracle.tile_quant(bf16(g["x"]), eps=0.5)
    assert np.array_equal(q.numpy(), g["q_eps"]) and np.array_equal(s.numpy(), g["s_eps"])
    q, s = oracle.block_quant(bf16(g["w"]))
    assert np.array_equal(q.numpy(), g["qw"]) and np.array_equal(s.numpy(), g["sw"])
    q, s = oracle.tile_quant(t(g["xf"]))
    assert np.array_equal(q.numpy(), g["qf"]) and np.array_equal(s.numpy(), g["sf"])
    g = load("quant_transposed_grouped")
    q_t, s_t = oracle.tile_quant_t_grouped(bf16(g["x"]), g["splits"].tolist())
    assert np.array_equal(q_t.numpy(), g["q_t"]) and np.array_equal(s_t.numpy(), g["s_t"])


def test_known_answers_in_vectors():
    """scaled_linear_test.py:305-319: rows of ones, 1000 and -512 quantise to +-448 with scale
    value/448; an all-zero tile gets scale 1 and zero codes (triton_kernel.py:107-108)."""
    g = load("quant_known_answers")
    q, s = g["q"], g["s"]
    f32 = np.float32
    assert np.all(q[0] == 0x7E) and np.all(s[0] == f32(1.0) / f32(448.0))
    assert np.all(q[1] == 0x7E) and np.all(s[1] == f32(1000.0) / f32(448.0))
    assert np.all(q[2] == 0xFE) and np.all(s[2] == f32(512.0) / f32(448.0))
    assert np.all(q[3] == 0) and np.all(s[3] == 1.0)
    outlier = f32(bf16(g["x"])[4, 7].float().item())  # 1e4 rounded to bf16
    assert q[4, 7] == 0x7E and s[4, 0] == outlier / f32(448.0)
    assert np.all(q[5, :128] == 0) and s[5, 0] == 1.0 and s[5, 1] != 1.0
    # every non-zero tile holds the code of 448 somewhere
    for r in (4, 6, 7):
        for tile in range(2):
            assert (q[r, tile * TILE : (tile + 1) * TILE] & 0x7F).max() == 0x7E


def _check_codes_exact(oracle, x_f32, q, s, rows):
    """codes == RNE_e4m3fn(fl32(x / s)) with the rounding done in exact rational arithmetic."""
    x = x_f32.astype(np.float32)
    for r in rows:
        for c in range(x.shape[1]):
            sc = s[r, c // TILE]
            quotient = np.float32(x[r, c]) / np.float32(sc)  # IEEE fp32 division
            assert q[r, c] == oracle.exact_e4m3fn_code(float(quotient)), (r, c)


def test_vectors_satisfy_closed_form(oracle):
    g = load("quant_known_answers")
    x = bf16(g["x"]).float().numpy()
    amax = np.abs(x.reshape(8, 2, TILE)).max(-1)
    want_s = np.where(amax == 0, np.float32(1.0), amax.astype(np.float32) / np.float32(448.0))
    assert np.array_equal(g["s"], want_s.astype(np.float32))
    _check_codes_exact(oracle, x, g["q"], g["s"], range(8))
    g = load("quant_random")
    x = bf16(g["x"]).float().numpy()
    amax = np.abs(x.reshape(x.shape[0], -1, TILE)).max(-1)
    assert np.array_equal(g["s"], amax.astype(np.float32) / np.float32(448.0))
    assert np.array_equal(g["s_eps"], np.maximum(amax, np.float32(0.5)).astype(np.float32) / np.float32(448.0))
    _check_codes_exact(oracle, x, g["q"], g["s"], range(0, x.shape[0], 7))
    _check_codes_exact(oracle, x, g["q_eps"], g["s_eps"], range(3, x.shape[0], 11))
    w = bf16(g["w"]).float().numpy()
    bmax = np.abs(w.reshape(2, TILE, 1, TILE)).max(axis=(1, 3))
    assert np.array_equal(g["sw"], bmax.astype(np.float32) / np.float32(448.0))
    srow = np.repeat(g["sw"], TILE, axis=0)
    _check_codes_exact(oracle, w, g["qw"], srow, range(0, 256, 37))


def test_transposed_vectors_are_quant_of_padded_transpose(oracle):
    """a3: per group, the transposed output is the 1x128 quantisation of zero_pad(X_g^T)
    (scaled_linear.py:402-414), checked here with the torch restatement."""
    g = load("quant_transposed_grouped")
    x = bf16(g["x"])
    splits = g["splits"].tolist()
    q_t, s_t = g["q_t"], g["s_t"]
    off = pad = 0
    for m in splits:
        nb = (m + TILE - 1) // TILE
        if m:
            xt = torch.zeros(x.shape[1], nb * TILE, dtype=torch.bfloat16)
            xt[:, :m] = x[off : off + m].t()
            q, s = oracle.torch_tile_quant(xt)
            assert np.array_equal(q.view(torch.uint8).numpy(), q_t[:, pad : pad + nb * TILE])
            assert np.array_equal(s.numpy(), s_t[pad // TILE : pad // TILE + nb].T)
        off += m
        pad += nb * TILE
    assert pad == q_t.shape[1]


def test_gemm_vectors_equal_float64_dequant_matmul(oracle):
    g = load("grouped_linear")
    splits = g["splits"].tolist()
    qx, sx, qw, sw = t(g["qx"]), t(g["sx"]), t(g["qw"]), t(g["sw"])
    a = oracle.e4m3fn_to_f32(qx).double() * sx.double().repeat_interleave(TILE, 1)
    off = 0
    for e, m in enumerate(splits):
        b = oracle.e4m3fn_to_f32(qw[e]).double() * sw[e].double().repeat_interleave(TILE, 0).repeat_interleave(TILE, 1)
        want = a[off : off + m] @ b.t()
        assert rel_err(t(g["y32"])[off : off + m], want) < 1e-5
        off += m
    # wgrad from the transposed operands
    qdy_t, sdy_t, qx_t, sx_t = t(g["qdy_t"]), t(g["sdy_t"]), t(g["qx_t"]), t(g["sx_t"])
    dyt = oracle.e4m3fn_to_f32(qdy_t).double() * sdy_t.double().t().repeat_interleave(TILE, 1)
    xt = oracle.e4m3fn_to_f32(qx_t).double() * sx_t.double().t().repeat_interleave(TILE, 1)
    pad = 0
    for e, m in enumerate(splits):
        w = (m + TILE - 1) // TILE * TILE
        want = dyt[:, pad : pad + w] @ xt[:, pad : pad + w].t()
        if m:
            assert rel_err(t(g["dw32"])[e], want) < 1e-5
        else:
            assert np.all(g["dw32"][e] == 0)
        pad += w
    # and the module-level vectors are the bf16 roundings of the same numbers
    assert np.array_equal(g["out"], t(g["y32"]).bfloat16().view(torch.int16).numpy().view(np.uint16))


def test_oracle_reproduces_grouped_linear_and_permute_vectors(oracle):
    g = load("grouped_linear")
    ws = [bf16(w) for w in g["w"]]
    r = oracle.grouped_linear_fwd_bwd(bf16(g["x"]), ws, g["splits"].tolist(), bf16(g["dy"]))
    assert torch.equal(r["out"].bfloat16(), bf16(g["out"]))
    assert torch.equal(r["dgrad"].bfloat16(), bf16(g["dgrad"]))
    assert all(np.array_equal(r["wgrad"][e].numpy(), g["dw32"][e]) for e in range(len(ws)))
    g = load("permute_combine")
    idx = t(g["idx"])
    E = int(g["counts"].shape[0])
    permuted, sorted_idx, counts = oracle.permute(bf16(g["tokens"]), idx, E)
    assert torch.equal(permuted, bf16(g["permuted"])) and np.array_equal(sorted_idx.numpy(), g["sorted_idx"])
    assert np.array_equal(counts.numpy(), g["counts"])
    # independent of the C code: torch's stable argsort and index_copy / multiply / sum
    assert np.array_equal(torch.argsort(idx.view(-1), stable=True).numpy(), g["sorted_idx"])
    probs = t(g["probs"])
    y = bf16(g["y"])
    assert torch.equal(oracle.torch_unpermute(y, t(g["sorted_idx"]), probs.bfloat16()), bf16(g["out_bf16"]))
    torch.testing.assert_close(oracle.torch_unpermute(y, t(g["sorted_idx"]), probs), t(g["out_f32"]), rtol=1e-6, atol=1e-6)
    assert torch.equal(oracle.torch_unpermute(y, t(g["sorted_idx"])), bf16(g["out_plain"]))


def test_fraction_rounder_is_independent_of_the_c_code(oracle):
    """The rational rounder used above agrees with torch's own cast on a sweep, so the checks on
    the vectors do not lean on the oracle's C conversion."""
    vals = [0.0, 448.0, 449.0, 464.0, -464.0, 2.0**-9, 2.0**-10, 1.5 * 2.0**-9, 0.4375, 17.0, 18.0, 19.0, 1e-8]
    got = [oracle.exact_e4m3fn_code(v) for v in vals]
    want = torch.tensor(vals).to(torch.float8_e4m3fn).view(torch.uint8).tolist()
    assert got == want
    assert Fraction(448) == Fraction(float(torch.tensor([0x7E], dtype=torch.uint8).view(torch.float8_e4m3fn).float()))


# ------------------------------------------------------------------------------------------
# GPU
# ------------------------------------------------------------------------------------------
@pytest.mark.gpu
def test_hip_quant_matches_vectors(dev):
    from atorch_amd import kernels as K

    g = load("quant_known_answers")
    q, s = K.tile_quant(bf16(g["x"]).to(dev))
    assert np.array_equal(q.view(torch.uint8).cpu().numpy(), g["q"]) and np.array_equal(s.cpu().numpy(), g["s"])
    qb, sb = K.block_quant(bf16(g["xb"]).to(dev))
    assert np.array_equal(qb.view(torch.uint8).cpu().numpy(), g["qb"]) and np.array_equal(sb.cpu().numpy(), g["sb"])
    g = load("quant_random")
    q, s = K.tile_quant(bf16(g["x"]).to(dev))
    assert np.array_equal(q.view(torch.uint8).cpu().numpy(), g["q"]) and np.array_equal(s.cpu().numpy(), g["s"])
    q, s = K.tile_quant(bf16(g["x"]).to(dev), eps=0.5)
    assert np.array_equal(q.view(torch.uint8).cpu().numpy(), g["q_eps"]) and np.array_equal(s.cpu().numpy(), g["s_eps"])
    q, s = K.block_quant(bf16(g["w"]).to(dev))
    assert np.array_equal(q.view(torch.uint8).cpu().numpy(), g["qw"]) and np.array_equal(s.cpu().numpy(), g["sw"])
    q, s = K.tile_quant(t(g["xf"]).to(dev))
    assert np.array_equal(q.view(torch.uint8).cpu().numpy(), g["qf"]) and np.array_equal(s.cpu().numpy(), g["sf"])


@pytest.mark.gpu
def test_hip_transposed_grouped_quant_matches_vectors(dev):
    from atorch_amd import kernels as K

    g = load("quant_transposed_grouped")
    splits = g["splits"].tolist()
    goff = K.group_offsets_from_splits(splits, dev)
    q, s, q_t, s_t = K.tile_quant_dual_grouped(bf16(g["x"]).to(dev), goff, len(splits), ld_t=g["q_t"].shape[1])
    assert np.array_equal(q.view(torch.uint8).cpu().numpy(), g["q"]) and np.array_equal(s.cpu().numpy(), g["s"])
    assert np.array_equal(q_t.view(torch.uint8).cpu().numpy(), g["q_t"])
    assert np.array_equal(s_t.cpu().numpy(), g["s_t"])


@pytest.mark.gpu
def test_hip_grouped_gemms_match_vectors(dev):
    from atorch_amd import kernels as K

    g = load("grouped_linear")
    splits = g["splits"].tolist()
    goff = K.group_offsets_from_splits(splits, dev)
    fp8 = torch.float8_e4m3fn
    y = K.grouped_gemm_nt(t(g["qx"]).to(dev).view(fp8), t(g["sx"]).to(dev), t(g["qw"]).to(dev).view(fp8),
                          t(g["sw"]).to(dev), goff, out_dtype=torch.float32)  # fmt: skip
    assert rel_err(y.cpu(), t(g["y32"])) < GEMM_TOL_F32
    yb = K.grouped_gemm_nt(t(g["qx"]).to(dev).view(fp8), t(g["sx"]).to(dev), t(g["qw"]).to(dev).view(fp8),
                           t(g["sw"]).to(dev), goff)  # fmt: skip
    assert rel_err(yb.cpu().float(), bf16(g["out"]).float()) < GEMM_TOL
    dw = K.grouped_gemm_wgrad(t(g["qdy_t"]).to(dev).view(fp8), t(g["sdy_t"]).to(dev), t(g["qx_t"]).to(dev).view(fp8),
                              t(g["sx_t"]).to(dev), goff)  # fmt: skip
    assert rel_err(dw.cpu(), t(g["dw32"])) < GEMM_TOL_F32
    assert torch.all(dw[splits.index(0)] == 0)


@pytest.mark.gpu
def test_hip_module_matches_vectors(dev):
    """The module end to end from the bf16 inputs: quantise, three grouped GEMMs, bf16 outputs."""
    from atorch_amd.grouped_linear import ATorchGroupedLinear

    g = load("grouped_linear")
    E, N, Kdim = g["w"].shape
    mod = ATorchGroupedLinear(E, Kdim, N, bias=False, params_dtype=torch.bfloat16, device=dev)
    with torch.no_grad():
        for e in range(E):
            getattr(mod, f"weight{e}").copy_(bf16(g["w"][e]))
    x = bf16(g["x"]).to(dev).requires_grad_(True)
    out = mod(x, g["splits"].tolist())
    out.backward(bf16(g["dy"]).to(dev))
    assert rel_err(out.detach().cpu().float(), bf16(g["out"]).float()) < GEMM_TOL
    assert rel_err(x.grad.cpu().float(), bf16(g["dgrad"]).float()) < GEMM_TOL
    for e in range(E):
        assert rel_err(getattr(mod, f"weight{e}").grad.cpu().float(), t(g["dw32"][e])) < GEMM_TOL


@pytest.mark.gpu
def test_hip_permute_combine_matches_vectors(dev):
    from atorch_amd import kernels as K
    from atorch_amd.token_dispatcher import permute, unpermute

    g = load("permute_combine")
    idx = t(g["idx"]).to(dev)
    E = int(g["counts"].shape[0])
    sorted_idx, row_map, goff = K.moe_preprocess(idx, E)
    assert np.array_equal(sorted_idx.cpu().numpy(), g["sorted_idx"])
    assert np.array_equal((goff[1:] - goff[:-1]).cpu().numpy(), g["counts"])
    permuted, sorted2 = permute(bf16(g["tokens"]).to(dev), idx)
    assert torch.equal(permuted.cpu(), bf16(g["permuted"])) and np.array_equal(sorted2.cpu().numpy(), g["sorted_idx"])
    y = bf16(g["y"]).to(dev)
    probs = t(g["probs"]).to(dev)
    assert torch.equal(unpermute(y, sorted2, probs.bfloat16()).cpu(), bf16(g["out_bf16"]))
    assert np.array_equal(unpermute(y, sorted2, probs).cpu().numpy(), g["out_f32"])
    assert torch.equal(unpermute(y, sorted2).cpu(), bf16(g["out_plain"]))

"""Shared input generators and comparison helpers for the tests."""
import torch

TILE = 128


def randn_bf16(shape, seed, std=1.0, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * std).to(dtype)


def heavy_tailed(shape, seed, dtype=torch.bfloat16):
    """Student-t (df=3) like values: normal / sqrt(chi2_3 / 3)."""
    g = torch.Generator().manual_seed(seed)
    z = torch.randn(shape, generator=g)
    chi = torch.randn((*shape, 3), generator=g).pow(2).sum(-1)
    return (z / torch.sqrt(chi / 3)).to(dtype)


def ragged_splits(total, num_groups, seed, multiple=1, zero_group=True):
    """Random splits of ``total`` rows into ``num_groups`` groups (multiples of ``multiple``),
    one of them empty when asked (the reference test forces a zero-length split,
    atorch/tests/common_tests/fp8/test_quantized_grouped_linear.py:619-628)."""
    g = torch.Generator().manual_seed(seed)
    m = total // multiple
    n_cut = num_groups - 1 - (1 if zero_group and num_groups > 2 else 0)
    cuts = torch.sort(torch.randint(0, m + 1, (n_cut,), generator=g)).values.tolist()
    if zero_group and num_groups > 2:
        cuts.append(cuts[-1])
    b = [0] + cuts + [m]
    splits = [(b[i + 1] - b[i]) * multiple for i in range(num_groups)]
    splits[-1] += total - sum(splits)
    assert sum(splits) == total and len(splits) == num_groups
    return splits


def topk_routing(T, E, k, seed, zipf_s=None):
    """Distinct top-k experts per token.  zipf_s: popularity p_e ~ (e+1)^-s, else N(0,1) logits."""
    g = torch.Generator().manual_seed(seed)
    if zipf_s is None:
        logits = torch.randn(T, E, generator=g)
    else:
        p = torch.arange(1, E + 1, dtype=torch.float64).pow(-zipf_s)
        # Gumbel top-k == sampling without replacement proportional to p
        u = torch.rand(T, E, generator=g, dtype=torch.float64).clamp_min(1e-300)
        logits = (p.log() - torch.log(-torch.log(u))).float()
    vals, idx = torch.topk(logits, k, dim=1)
    probs = torch.softmax(vals, dim=1)
    return idx, probs


def rel_err(c: torch.Tensor, ref: torch.Tensor) -> float:
    """max |c - ref| / max(|ref|, rms(ref)): relative error with the rms of the reference as
    the floor of the denominator, so that entries near zero do not dominate."""
    c, ref = c.double(), ref.double()
    floor = ref.pow(2).mean().sqrt().clamp_min(1e-30)
    return float(((c - ref).abs() / torch.maximum(ref.abs(), floor)).max()) if ref.numel() else 0.0

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


class OracleQuantizeOp:
    """A ``quantize_op`` (the plugin interface of the grouped linear) that runs the CPU oracle.
    Test infrastructure: it lets the host logic of the autograd function be checked without a
    GPU and serves as the module-level reference on the GPU box.  Per-expert API only."""

    supports_fused_grouped = False

    def __init__(self):
        from oracle import oracle as O

        self.O = O
        self.calls = {"quantize": 0, "grouped_qgemm": 0}

    def quantize(self, t, qparams, return_transpose=False):
        from atorch_amd.quantization import QuantizeResult

        O = self.O
        self.calls["quantize"] += 1
        t = t.detach().cpu()
        if tuple(qparams.quant_tile_shape) == (1, TILE):
            q, s = O.tile_quant(t, qparams.eps)
            if not return_transpose:
                return QuantizeResult(q, s)
            m = t.shape[0]
            q_t, s_t = O.tile_quant_t_grouped(t, [m], qparams.eps)
            nb = (m + TILE - 1) // TILE
            return QuantizeResult(q, s, q_t[:, :m].contiguous(), s_t[:nb].t().contiguous())
        q, s = O.block_quant(t, qparams.eps)
        if not return_transpose:
            return QuantizeResult(q, s)
        return QuantizeResult(q, s, q.t().contiguous(), s.t().contiguous())

    def grouped_qgemm(self, qa_list, qb_list, mm_params, sa_list, sb_list, out_list, bias=None, accumulate=False,
                      qparams_x=None, qparams_w=None):
        O = self.O
        self.calls["grouped_qgemm"] += 1
        wgrad = tuple(qparams_w.quant_tile_shape) == (1, TILE)
        for e, (qa, qb, sa, sb, out) in enumerate(zip(qa_list, qb_list, sa_list, sb_list, out_list)):
            if not wgrad:
                if qa.shape[0] == 0:
                    continue
                c = O.fp8_gemm(qa.contiguous(), sa.contiguous(), qb.contiguous(), sb.contiguous())
                if bias is not None:
                    c = c + bias[e].float()
                out.copy_(c.to(out.dtype))
            else:
                m = qa.shape[1]
                if m == 0:
                    if not accumulate:
                        out.zero_()
                    continue
                ld = (m + TILE - 1) // TILE * TILE
                a = torch.zeros((qa.shape[0], ld), dtype=torch.uint8)
                b = torch.zeros((qb.shape[0], ld), dtype=torch.uint8)
                a[:, :m], b[:, :m] = qa, qb
                c = O.fp8_gemm(a, sa.contiguous(), b, sb.contiguous())  # b tile-scaled: sb [K, nb]
                if accumulate:
                    out.add_(c.to(out.dtype))
                else:
                    out.copy_(c.to(out.dtype))

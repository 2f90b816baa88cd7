"""The ``quantize_op`` plugin object and its configuration types.

The reference's grouped linear is written against an operator object
(``qlinear_params.quantize_op``) with two methods, ``quantize`` and ``grouped_qgemm``
(atorch/modules/fp8/quantized_grouped_linear.py:92-101, 141-151, 214-223, 243-253), and
against the config types ``QLinearParams`` / ``QParams`` / ``MMParams`` / ``ScalingType`` /
``QuantizeResultCache`` whose use is visible at
atorch/tests/common_tests/fp8/test_quantized_grouped_linear.py:164-175 and
quantized_grouped_linear.py:129,467-470.  In the reference those come from an external package
that is not part of its tree; this module supplies them, with ``HipQuantizeOp`` running the
gfx950 kernels.

Layout conventions of ``HipQuantizeOp`` results
  1x128 (``quant_tile_shape == (1, 128)``), input ``[M, K]``:
      data ``[M, K]`` fp8, scale ``[M, K/128]`` fp32;
      data_t ``[K, M]`` - a view (row stride = padded token count) of the transposed codes,
      scale_t ``[K, ceil(M/128)]`` - a transposed view of a ``[ceil(M/128), K]`` buffer.
  128x128, input ``[N, K]``:
      data ``[N, K]``, scale ``[N/128, K/128]``, data_t ``[K, N]``, scale_t ``[K/128, N/128]``.
"""
import enum
import os
from dataclasses import dataclass, field
from typing import Any, List, Optional, Sequence, Tuple

import torch

from . import _lib, kernels
from ._lib import check, dtype_code, lib, stream

TILE = kernels.TILE
FP8 = kernels.FP8


def parse_bool_env(name: str, default: str = "False") -> bool:
    """Same accepted spellings as atorch/common/env.py:6-13."""
    v = os.getenv(name, default)
    if v in ("1", "True", "true"):
        return True
    if v in ("0", "False", "false"):
        return False
    raise ValueError(f"Env {name} should be True or False")


def force_quantize_per_microbatch() -> bool:
    """FORCE_QUANTIZE_PER_MICROBATCH, atorch/common/env.py:33-34 (read on every forward)."""
    return parse_bool_env("FORCE_QUANTIZE_PER_MICROBATCH", "False")


class ScalingType(enum.Enum):
    VECTOR_TILED_X_AND_G_BLOCK_TILED_W = "vector_tiled_x_and_g_block_tiled_w"


@dataclass
class QParams:
    quant_dtype: torch.dtype = FP8
    scaling_type: ScalingType = ScalingType.VECTOR_TILED_X_AND_G_BLOCK_TILED_W
    quant_tile_shape: Tuple[int, int] = (1, TILE)
    eps: float = 0.0
    pow_2_scale: bool = False


@dataclass
class MMParams:
    out_dtype: Optional[torch.dtype] = None
    use_split_accumulator: bool = True


@dataclass
class QuantizeResult:
    data: Optional[torch.Tensor]
    scale: Optional[torch.Tensor]
    data_t: Optional[torch.Tensor] = None
    scale_t: Optional[torch.Tensor] = None


@dataclass
class QuantizeResultCache:
    """Per-weight cache of the fp8 copies between microbatches
    (quantized_grouped_linear.py:121-129, 467-470)."""

    data: Optional[torch.Tensor] = None
    scale: Optional[torch.Tensor] = None
    data_t: Optional[torch.Tensor] = None
    scale_t: Optional[torch.Tensor] = None

    def to_qresult(self) -> QuantizeResult:
        return QuantizeResult(self.data, self.scale, self.data_t, self.scale_t)


class WeightCodeCache:
    """Block-quantised codes of expert weights kept between the microbatches of one optimizer step, for the
    functional forms (``gmm``, ``grouped_mlp``) that have no module to hold ``QuantizeResultCache`` objects.

    The rule is the module's (atorch/modules/fp8/quantized_grouped_linear.py:103-134): quantise when
    ``is_first_microbatch`` is True or None, when the cached entry lacks the transposed codes a training call
    needs, or when FORCE_QUANTIZE_PER_MICROBATCH is set (and then leave the cache alone); otherwise reuse.
    Beyond the reference, an entry is also dropped when the weight it was made from has been written in place
    or replaced since (its version counter, address, shape or dtype changed), so a forgotten
    ``is_first_microbatch=True`` after an optimizer step cannot feed stale codes to the GEMMs."""

    def __init__(self):
        self._slots = {}

    @staticmethod
    def _stamp(tensors):
        return tuple((t.data_ptr(), t._version, tuple(t.shape), t.dtype) for t in tensors if t is not None)

    def codes(self, name: str, tensors, is_first_microbatch: Optional[bool], need_transpose: bool, quantise):
        """``quantise(need_transpose) -> (q, s, q_t | None, s_t | None)`` for the weight tensors ``tensors``."""
        force = force_quantize_per_microbatch()
        slot = self._slots.get(name)
        stamp = self._stamp(tensors)
        update = is_first_microbatch or is_first_microbatch is None
        if force or update or slot is None or slot[0] != stamp or (need_transpose and slot[1][2] is None):
            codes = quantise(need_transpose)
            if not force:
                self._slots[name] = (stamp, codes)
            return codes
        return slot[1]

    def clear(self):
        self._slots.clear()


@dataclass
class QLinearParams:
    x_params: QParams = field(default_factory=lambda: QParams(quant_tile_shape=(1, TILE)))
    w_params: QParams = field(default_factory=lambda: QParams(quant_tile_shape=(TILE, TILE)))
    g_params: QParams = field(default_factory=lambda: QParams(quant_tile_shape=(1, TILE)))
    mm_fprop: MMParams = field(default_factory=MMParams)
    mm_dgrad: MMParams = field(default_factory=MMParams)
    mm_wgrad: MMParams = field(default_factory=MMParams)
    quantize_op: Any = None
    quantize: bool = True
    allgather_fp8: bool = False


def _check_params(qparams: QParams):
    if qparams.quant_dtype != FP8:
        raise ValueError(f"HipQuantizeOp quantises to torch.float8_e4m3fn only, got {qparams.quant_dtype}")
    if qparams.pow_2_scale:
        raise ValueError("pow_2_scale is not supported")
    shape = tuple(qparams.quant_tile_shape)
    if shape not in ((1, TILE), (TILE, TILE)):
        raise ValueError(f"quant_tile_shape must be (1, 128) or (128, 128), got {shape}")
    return shape


# ------------------------------------------------------------------------------------------
# helpers: recognise lists of views that tile one buffer
# ------------------------------------------------------------------------------------------
def _base_of_rows(ts: Sequence[torch.Tensor]):
    """If the 2-D tensors are consecutive row slices of one row-major buffer return
    ``(base_ptr, row_stride_elems)`` else None.  Empty slices carry no address and are skipped."""
    ld = None
    for t in ts:
        if t.dim() != 2 or (t.numel() > 0 and t.stride(1) != 1):
            return None
        if t.shape[0] > 1 and t.numel() > 0:
            if ld is None:
                ld = t.stride(0)
            elif ld != t.stride(0):
                return None
    if ld is None:  # only single-row slices: take them as dense
        ld = ts[0].shape[1]
    base = None
    off = 0
    for t in ts:
        if t.numel() > 0:
            b = t.data_ptr() - off * ld * t.element_size()
            if base is None:
                base = b
            elif b != base:
                return None
        off += t.shape[0]
    if base is None:
        return None
    return base, ld


def _base_of_stack(ts: Sequence[torch.Tensor]):
    """If the tensors are equally shaped, contiguous and equally spaced in memory return
    ``(base_ptr, stride_elems)`` else None."""
    t0 = ts[0]
    if any((not t.is_contiguous()) or t.shape != t0.shape or t.dtype != t0.dtype for t in ts):
        return None
    if t0.numel() == 0:
        return None
    if len(ts) == 1:
        return t0.data_ptr(), t0.numel()
    step = ts[1].data_ptr() - t0.data_ptr()
    if step < t0.numel() * t0.element_size() or step % t0.element_size():
        return None
    for i, t in enumerate(ts):
        if t.data_ptr() != t0.data_ptr() + i * step:
            return None
    return t0.data_ptr(), step // t0.element_size()


class HipQuantizeOp:
    """``quantize_op`` backed by the gfx950 kernels (1x128 activations / gradients,
    128x128 weights, e4m3fn, fp32 ``amax/448`` scales)."""

    supports_fused_grouped = True

    def __init__(self):
        self._offsets_cache = {}

    # -- group offsets on the device ---------------------------------------------------------
    def group_offsets(self, m_splits: Sequence[int], device) -> torch.Tensor:
        key = (tuple(int(m) for m in m_splits), str(device))
        t = self._offsets_cache.get(key)
        if t is None:
            if len(self._offsets_cache) > 64:
                self._offsets_cache.clear()
            t = kernels.group_offsets_from_splits(key[0], device)
            self._offsets_cache[key] = t
        return t

    # -- plugin interface: quantize ---------------------------------------------------------------
    def quantize(self, t: torch.Tensor, qparams: QParams, return_transpose: bool = False) -> QuantizeResult:
        """quantized_grouped_linear.py:92-96, 114, 202."""
        shape = _check_params(qparams)
        assert t.dim() == 2, "quantize expects a 2-D tensor"
        t = t.contiguous()
        if shape == (1, TILE):
            if return_transpose:
                y, s, y_t, s_t = kernels.tile_quant(t, eps=qparams.eps, return_transpose=True)
                return QuantizeResult(y, s, y_t, s_t)
            y, s = kernels.tile_quant(t, eps=qparams.eps)
            return QuantizeResult(y, s)
        if return_transpose:
            y, s, y_t, s_t = kernels.block_quant(t, eps=qparams.eps, return_transpose=True)
            return QuantizeResult(y, s, y_t, s_t)
        y, s = kernels.block_quant(t, eps=qparams.eps)
        return QuantizeResult(y, s)

    # -- fused forms (what the reference's "TODO: Add fused_multi_quantize" asks for) ---------------
    def quantize_grouped(
        self, x: torch.Tensor, m_splits: Sequence[int], qparams: QParams, return_transpose: bool = False
    ) -> Tuple[List[torch.Tensor], List[torch.Tensor], List[torch.Tensor], List[torch.Tensor]]:
        """One launch for all groups of ``x [sum(m_splits), K]``.  Returns the four per-group lists
        (data, scale, data_t, scale_t) as views of the fused buffers; the last two are empty
        without ``return_transpose``."""
        shape = _check_params(qparams)
        assert shape == (1, TILE)
        x = x.contiguous()
        m_splits = [int(m) for m in m_splits]
        if not return_transpose:
            q, s = kernels.tile_quant(x, eps=qparams.eps)
            return list(torch.split(q, m_splits)), list(torch.split(s, m_splits)), [], []
        goff = self.group_offsets(m_splits, x.device)
        ld_t = max(kernels.padded_total(m_splits), TILE)
        q, s, q_t, s_t = kernels.tile_quant_dual_grouped(x, goff, len(m_splits), eps=qparams.eps, ld_t=ld_t)
        data_t, scale_t = [], []
        p = 0
        for m in m_splits:
            nb = (m + TILE - 1) // TILE
            data_t.append(q_t[:, p : p + m])
            scale_t.append(s_t[p // TILE : p // TILE + nb].t())
            p += nb * TILE
        return list(torch.split(q, m_splits)), list(torch.split(s, m_splits)), data_t, scale_t

    def quantize_weights(self, weights: Sequence[torch.Tensor], qparams: QParams, return_transpose: bool = False):
        """Block-quantise E equally shaped weights; one launch when they are equally spaced views
        of one buffer, else one launch per weight.  Returns per-weight lists of views."""
        shape = _check_params(qparams)
        assert shape == (TILE, TILE)
        E = len(weights)
        N, K = weights[0].shape
        ws = [w.detach() for w in weights]
        stacked = _base_of_stack(ws)
        dev = ws[0].device
        q = torch.empty((E, N, K), dtype=FP8, device=dev)
        s = torch.empty((E, N // TILE, K // TILE), dtype=torch.float32, device=dev)
        q_t = torch.empty((E, K, N), dtype=FP8, device=dev) if return_transpose else None
        s_t = torch.empty((E, K // TILE, N // TILE), dtype=torch.float32, device=dev) if return_transpose else None
        dt = dtype_code(ws[0].dtype, True)
        if stacked is not None:
            base, estride = stacked
            check(
                lib().aamd_quant_128x128(
                    base, dt, E, N, K, estride, q.data_ptr(), s.data_ptr(),
                    q_t.data_ptr() if return_transpose else None, s_t.data_ptr() if return_transpose else None,
                    qparams.eps, stream(),
                )
            )  # fmt: skip
        else:
            for e, w in enumerate(ws):
                w = w.contiguous()
                check(
                    lib().aamd_quant_128x128(
                        w.data_ptr(), dt, 1, N, K, N * K, q[e].data_ptr(), s[e].data_ptr(),
                        q_t[e].data_ptr() if return_transpose else None,
                        s_t[e].data_ptr() if return_transpose else None,
                        qparams.eps, stream(),
                    )
                )  # fmt: skip
        unb = lambda t: list(t.unbind(0)) if t is not None else []  # noqa: E731
        return unb(q), unb(s), unb(q_t), unb(s_t)

    # -- plugin interface: grouped_qgemm -------------------------------------------------------------
    def grouped_qgemm(
        self,
        qa_list: Sequence[torch.Tensor],
        qb_list: Sequence[torch.Tensor],
        mm_params: MMParams,
        sa_list: Sequence[torch.Tensor],
        sb_list: Sequence[torch.Tensor],
        out_list: Sequence[torch.Tensor],
        bias: Optional[Sequence[torch.Tensor]] = None,
        accumulate: bool = False,
        qparams_x: Optional[QParams] = None,
        qparams_w: Optional[QParams] = None,
    ) -> None:
        """E block-scaled GEMMs written in place into ``out_list``
        (quantized_grouped_linear.py:141-151 fprop, 214-223 dgrad, 243-253 wgrad)."""
        E = len(qa_list)
        assert len(qb_list) == E and len(sa_list) == E and len(sb_list) == E and len(out_list) == E
        if E == 0:
            return
        if out_list[0].dtype == torch.float16:
            # fp16 activations (quantized_grouped_linear.py:533-534): the kernels write fp32 or bf16, so the
            # GEMM runs into one fp32 buffer laid out like the outputs and is cast once
            rows = [int(o.shape[0]) for o in out_list]
            stacked_out = out_list[0].dim() == 2 and all(o.shape[1:] == out_list[0].shape[1:] for o in out_list)
            assert stacked_out, "fp16 outputs must share their trailing shape"
            buf = torch.empty((sum(rows), *out_list[0].shape[1:]), dtype=torch.float32, device=out_list[0].device)
            tmp = list(torch.split(buf, rows))
            if accumulate:
                for t, o in zip(tmp, out_list):
                    t.copy_(o)
            if bias is not None:
                bias = [b.float() for b in bias]
            self.grouped_qgemm(qa_list, qb_list, mm_params, sa_list, sb_list, tmp, bias=bias, accumulate=accumulate,
                               qparams_x=qparams_x, qparams_w=qparams_w)  # fmt: skip
            for t, o in zip(tmp, out_list):
                o.copy_(t)
            return
        w_shape = tuple(qparams_w.quant_tile_shape) if qparams_w is not None else None
        if w_shape is None:
            # infer: block-scaled B has a [N/128, K/128] scale grid
            n_b = qb_list[0].shape[0]
            w_shape = (TILE, TILE) if sb_list[0].shape[0] * TILE == n_b else (1, TILE)
        if w_shape == (TILE, TILE):
            assert not accumulate, "accumulate is only defined for the wgrad GEMM"
            self._gemm_nt(qa_list, qb_list, sa_list, sb_list, out_list, bias)
        else:
            assert bias is None
            self._gemm_wgrad(qa_list, qb_list, sa_list, sb_list, out_list, accumulate)

    def _gemm_nt(self, qa_list, qb_list, sa_list, sb_list, out_list, bias):
        E = len(qa_list)
        N, K = qb_list[0].shape
        m_splits = [int(a.shape[0]) for a in qa_list]
        M = sum(m_splits)
        if M == 0:
            return
        dev = qb_list[0].device
        out_dt = dtype_code(out_list[0].dtype)
        a, sa, b, sb, c = (
            _base_of_rows(qa_list),
            _base_of_rows(sa_list),
            _base_of_stack(qb_list),
            _base_of_stack(sb_list),
            _base_of_rows(out_list),
        )
        fused = (
            None not in (a, sa, b, sb, c)
            and sa[1] == K // TILE
            and b[1] == N * K
            and sb[1] == (N // TILE) * (K // TILE)
        )
        bias_t = None
        if bias is not None:
            bias_t = torch.stack([bb.detach() for bb in bias]).contiguous()
            assert bias_t.shape == (E, N)
        bias_dt = dtype_code(bias_t.dtype) if bias_t is not None else _lib.NONE
        if fused:
            goff = self.group_offsets(m_splits, dev)
            ws = torch.empty(E + 1, dtype=torch.int32, device=dev)
            check(
                lib().aamd_grouped_gemm_fp8_nt(
                    a[0], a[1], sa[0], b[0], sb[0], 0, goff.data_ptr(), E, ws.data_ptr(), M, N, K,
                    c[0], out_dt, c[1], bias_t.data_ptr() if bias_t is not None else None, bias_dt, stream(),
                )
            )  # fmt: skip
            return
        for e in range(E):
            if m_splits[e] == 0:
                continue
            qa, s_a = qa_list[e], sa_list[e].contiguous()
            qb, s_b, o = qb_list[e].contiguous(), sb_list[e].contiguous(), out_list[e]
            assert qa.stride(1) == 1 and o.stride(1) == 1
            check(
                lib().aamd_grouped_gemm_fp8_nt(
                    qa.data_ptr(), qa.stride(0), s_a.data_ptr(), qb.data_ptr(), s_b.data_ptr(), 0, None, 1, None,
                    m_splits[e], N, K, o.data_ptr(), out_dt, o.stride(0),
                    bias_t[e].data_ptr() if bias_t is not None else None, bias_dt, stream(),
                )
            )  # fmt: skip

    @staticmethod
    def _transposed_layout(q_list, s_list, m_splits):
        """Recognise the per-group views ``quantize_grouped`` hands out: q_list[g] = q_t[:, p_g:p_g+M_g]
        and s_list[g] = s_t[p_g/128 : p_g/128+nb_g].t().  Returns (q_base, ld_t, s_base) or None."""
        R = q_list[0].shape[0]
        ld_t = None
        q_base = s_base = None
        p = 0
        for q, s, m in zip(q_list, s_list, m_splits):
            nb = (m + TILE - 1) // TILE
            if m > 0:
                if q.dim() != 2 or q.shape != (R, m) or q.stride(1) != 1 or s.shape != (R, nb):
                    return None
                this_ld = q.stride(0)
                if R > 1:
                    if ld_t is None:
                        ld_t = this_ld
                    elif ld_t != this_ld:
                        return None
                if s.stride(0) != 1 or (nb > 1 and s.stride(1) != R):
                    return None
                qb = q.data_ptr() - p
                sb = s.data_ptr() - (p // TILE) * R * 4
                if q_base is None:
                    q_base, s_base = qb, sb
                elif qb != q_base or sb != s_base:
                    return None
            p += nb * TILE
        if q_base is None or ld_t is None or ld_t % TILE or ld_t < p:
            return None
        return q_base, ld_t, s_base

    def _gemm_wgrad(self, qdy_t_list, qx_t_list, sdy_t_list, sx_t_list, out_list, accumulate):
        E = len(qdy_t_list)
        N, K = qdy_t_list[0].shape[0], qx_t_list[0].shape[0]
        m_splits = [int(t.shape[1]) for t in qdy_t_list]
        assert [int(t.shape[1]) for t in qx_t_list] == m_splits
        dev = out_list[0].device
        out_dt = dtype_code(out_list[0].dtype)
        if sum(m_splits) == 0:
            if not accumulate:
                for o in out_list:
                    o.zero_()
            return
        la = self._transposed_layout(qdy_t_list, sdy_t_list, m_splits)
        lb = self._transposed_layout(qx_t_list, sx_t_list, m_splits)
        oc = _base_of_stack(list(out_list))
        if la is not None and lb is not None and oc is not None and la[1] == lb[1]:
            goff = self.group_offsets(m_splits, dev)
            ws = torch.empty(E + 1, dtype=torch.int32, device=dev)
            check(
                lib().aamd_grouped_gemm_fp8_wgrad(
                    la[0], la[2], lb[0], lb[2], la[1], _lib.QT_ROWS, goff.data_ptr(), E, ws.data_ptr(), N, K,
                    oc[0], out_dt, oc[1], int(accumulate), stream(),
                )
            )  # fmt: skip
            return
        # generic path: one launch per group on densely re-laid operands
        pairs = torch.tensor([[0, m] for m in m_splits], dtype=torch.int64, device=dev)
        ws = torch.empty(2, dtype=torch.int32, device=dev)
        for e in range(E):
            o = out_list[e]
            assert o.is_contiguous()
            m = m_splits[e]
            if m == 0:
                if not accumulate:
                    o.zero_()
                continue
            ld = (m + TILE - 1) // TILE * TILE
            dyt = self._dense_transposed(qdy_t_list[e], ld)
            xt = self._dense_transposed(qx_t_list[e], ld)
            sdyt = sdy_t_list[e].t().contiguous()
            sxt = sx_t_list[e].t().contiguous()
            check(
                lib().aamd_grouped_gemm_fp8_wgrad(
                    dyt.data_ptr(), sdyt.data_ptr(), xt.data_ptr(), sxt.data_ptr(), ld, _lib.QT_ROWS, pairs[e].data_ptr(), 1,
                    ws.data_ptr(), N, K, o.data_ptr(), out_dt, N * K, int(accumulate), stream(),
                )
            )  # fmt: skip

    @staticmethod
    def _dense_transposed(q: torch.Tensor, ld: int) -> torch.Tensor:
        """[R, m] codes -> zero padded [R, ld] buffer (code 0 is +0.0, so padding adds nothing)."""
        R, m = q.shape
        if q.stride(1) == 1 and q.stride(0) == ld and m == ld:
            return q
        buf = torch.zeros((R, ld), dtype=torch.uint8, device=q.device)
        buf[:, :m] = q.view(torch.uint8) if q.dtype != torch.uint8 else q
        return buf


def default_qlinear_params() -> QLinearParams:
    """The 1x128 / 128x128 all-e4m3fn recipe of
    atorch/tests/common_tests/fp8/test_quantized_grouped_linear.py:164-175 on the HIP kernels."""
    return QLinearParams(quantize_op=HipQuantizeOp())

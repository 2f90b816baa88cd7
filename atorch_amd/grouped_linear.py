"""FP8 grouped linear: the module and autograd function of
atorch/modules/fp8/quantized_grouped_linear.py with the same names, argument order and
error behaviour, running on the gfx950 kernels through ``qlinear_params.quantize_op``.

Differences that do not change results:

* when the operator object offers the fused forms (``supports_fused_grouped``), all groups are
  quantised in one launch and the grouped GEMMs run as one launch each (the reference loops
  over experts, quantized_grouped_linear.py:90-101, 113-119, 200-206);
* the ``weight{i}`` parameters are views of one ``[num_gemms, out, in]`` buffer so that the
  weight quantisation is one launch as well.
"""
import logging
from typing import Any, Callable, List, Optional, Tuple, Union

import torch

from .quantization import (
    QLinearParams,
    QuantizeResultCache,
    default_qlinear_params,
    force_quantize_per_microbatch,
)

logger = logging.getLogger(__name__)


def cast_if_needed(t: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    return t if t.dtype == dtype else t.to(dtype)


def divide(numerator: int, denominator: int) -> int:
    assert numerator % denominator == 0, f"{numerator} is not divisible by {denominator}"
    return numerator // denominator


def init_method_constant(val: float) -> Callable:
    def init_(tensor: torch.Tensor) -> torch.Tensor:
        return torch.nn.init.constant_(tensor, val)

    return init_


def reset_wgrad_if_needed(ctx, weight: torch.Tensor, wgrad: Optional[torch.Tensor]):
    """What is returned as the gradient of a weight (quantized_grouped_linear.py:255).  With
    fused accumulation the result already sits in ``weight.main_grad``: autograd gets None, or a
    placeholder of the weight's shape when the parameter carries the ``grad_added_to_main_grad``
    flag that Megatron-style optimizers look at (the convention the reference test checks:
    ``p.grad is None`` and the result in ``p.main_grad``,
    atorch/tests/common_tests/fp8/test_quantized_grouped_linear.py:648-654)."""
    if not ctx.fuse_wgrad_accumulation:
        return wgrad
    if hasattr(weight, "grad_added_to_main_grad"):
        weight.grad_added_to_main_grad = True
        make = torch.zeros if getattr(weight, "zero_out_wgrad", False) else torch.empty
        return make(weight.main_grad.shape, dtype=weight.dtype, device=weight.device, requires_grad=False)
    return None


def _quantize_groups(op, rows: torch.Tensor, m_splits: List[int], qparams, want_transpose: bool):
    """1x128 codes of the row groups of ``rows`` as four per-group lists (codes, scales and, with
    ``want_transpose``, the codes and scales quantised along the tokens; else two empty lists): one launch where the
    operator offers the fused form, the reference's loop over the groups (quantized_grouped_linear.py:90-101,
    200-206) otherwise."""
    if getattr(op, "supports_fused_grouped", False):
        return op.quantize_grouped(rows, m_splits, qparams, return_transpose=want_transpose)
    results = [op.quantize(part, qparams, return_transpose=want_transpose) for part in torch.split(rows, m_splits)]
    transposed = results if want_transpose else []
    return ([r.data for r in results], [r.scale for r in results],
            [r.data_t for r in transposed], [r.scale_t for r in transposed])  # fmt: skip


def _weight_codes(op, weights, caches, qlinear_params, is_first_microbatch, want_transpose: bool):
    """Block-quantised weights as four per-expert lists, under the caching rule of
    quantized_grouped_linear.py:103-134: quantise on the first microbatch (True or None), when
    FORCE_QUANTIZE_PER_MICROBATCH is set, or when a backward needs transposes the caches do not hold; otherwise
    serve the caches.  Fresh codes are written back to the caches unless the environment flag forces
    quantisation anyway."""
    forced = force_quantize_per_microbatch()
    first = is_first_microbatch or is_first_microbatch is None
    stale = want_transpose and caches[0].data_t is None
    if not (forced or first or stale):
        held = [c.to_qresult() for c in caches]
        transposed = held if want_transpose else []
        return ([r.data for r in held], [r.scale for r in held],
                [r.data_t for r in transposed], [r.scale_t for r in transposed])  # fmt: skip
    if getattr(op, "supports_fused_grouped", False):
        q, s, q_t, s_t = op.quantize_weights(weights, qlinear_params.w_params, return_transpose=want_transpose)
    else:
        fresh = [op.quantize(w, qlinear_params.w_params, return_transpose=want_transpose) for w in weights]
        transposed = fresh if want_transpose else []
        q, s = [r.data for r in fresh], [r.scale for r in fresh]
        q_t, s_t = [r.data_t for r in transposed], [r.scale_t for r in transposed]
    if not forced:
        for i, cache in enumerate(caches):
            cache.data, cache.scale = q[i], s[i]
            cache.data_t = q_t[i] if want_transpose else None
            cache.scale_t = s_t[i] if want_transpose else None
    return q, s, q_t, s_t


def _adds_to_main_grad(fuse_wgrad_accumulation: bool, is_first_microbatch) -> bool:
    """Does this backward add to ``main_grad`` (True) or overwrite it?  quantized_grouped_linear.py:232-235: with
    fused accumulation every microbatch but the one flagged first adds; an unflagged call (None) adds."""
    return bool(fuse_wgrad_accumulation and not (is_first_microbatch is not None and is_first_microbatch))


class _ATorchQuantizedGroupedLinear(torch.autograd.Function):
    """Grouped linear with 1x128 / 128x128 fp8 quantisation.

    fwd   : Y_g  = X_g W_g^T (+ b_g)
    dgrad : dX_g = dY_g W_g
    wgrad : dW_g = dY_g^T X_g

    Argument order and the gradient tuple are those of the reference's function
    (quantized_grouped_linear.py:51-71, 257-270); the work between them goes through the operator object's
    list-of-groups interface, fused where it can be.
    """

    NUM_NON_TENSOR_ARGS = 9  # m_splits .. fuse_wgrad_accumulation: a None each in the gradient tuple

    @staticmethod
    def forward(  # type: ignore
        ctx,
        x: torch.Tensor,
        m_splits: List[int],
        use_bias: bool,
        x_metas,
        weight_qresult_caches,
        qlinear_params,
        activation_dtype: torch.dtype,
        is_grad_enabled: bool,
        is_first_microbatch,
        fuse_wgrad_accumulation: bool,
        *weights_and_biases: torch.Tensor,
    ) -> torch.Tensor:
        op = qlinear_params.quantize_op
        assert op is not None
        num_gemms = len(m_splits)
        weights, biases = weights_and_biases[:num_gemms], list(weights_and_biases[num_gemms:])
        out_features, in_features = weights[0].shape
        assert x.shape[-1] == in_features, "GEMM not possible"
        if use_bias:
            assert len(biases) == num_gemms, "Number of biases should match number of GEMMs."
            biases = [cast_if_needed(b, activation_dtype) for b in biases]
        rows = x.view(-1, in_features)

        qx, sx, qx_t, sx_t = _quantize_groups(op, rows, m_splits, qlinear_params.x_params, is_grad_enabled)
        qw, sw, qw_t, sw_t = _weight_codes(op, weights, weight_qresult_caches, qlinear_params, is_first_microbatch,
                                           is_grad_enabled)  # fmt: skip

        y_dtype = qlinear_params.mm_fprop.out_dtype or x.dtype
        out = torch.empty((sum(m_splits), out_features), dtype=y_dtype, device=x.device)
        op.grouped_qgemm(qx, qw, qlinear_params.mm_fprop, sx, sw, list(torch.split(out, m_splits)),
                         bias=biases if use_bias else None,
                         qparams_x=qlinear_params.x_params, qparams_w=qlinear_params.w_params)  # fmt: skip

        if is_grad_enabled:
            ctx.m_splits, ctx.num_gemms, ctx.use_bias, ctx.x_shape = m_splits, num_gemms, use_bias, x.shape
            ctx.qlinear_params, ctx.quantize_op, ctx.device = qlinear_params, op, x.device
            ctx.is_first_microbatch, ctx.fuse_wgrad_accumulation = is_first_microbatch, fuse_wgrad_accumulation
            # the Python-side attributes (main_grad, grad_added_to_main_grad) are read from
            # these references, not from the re-materialised saved tensors
            ctx.weight_refs = list(weights)
            ctx.save_for_backward(*qx_t, *sx_t, *qw_t, *sw_t, *weights)
        return out.view(-1, *x.shape[1:-1], out_features)

    @staticmethod
    def backward(ctx, *dy_tup: torch.Tensor) -> Tuple[Union[torch.Tensor, None], ...]:
        (dy,) = dy_tup
        n, qp, op, m_splits = ctx.num_gemms, ctx.qlinear_params, ctx.quantize_op, ctx.m_splits
        saved = ctx.saved_tensors
        assert len(saved) == 5 * n
        qx_t, sx_t, qw_t, sw_t = (saved[i * n : (i + 1) * n] for i in range(4))
        weights = ctx.weight_refs
        out_features, in_features = weights[0].shape

        dy_rows = dy.contiguous().view(-1, dy.shape[-1])
        bias_grads = [part.sum(dim=0) if ctx.use_bias else None for part in torch.split(dy_rows, m_splits)]
        qdy, sdy, qdy_t, sdy_t = _quantize_groups(op, dy_rows, m_splits, qp.g_params, True)

        # dX_g = dY_g W_g
        dgrad = torch.empty((sum(m_splits), in_features), dtype=qp.mm_dgrad.out_dtype or dy.dtype, device=ctx.device)
        op.grouped_qgemm(qdy, qw_t, qp.mm_dgrad, sdy, sw_t, list(torch.split(dgrad, m_splits)),
                         qparams_x=qp.g_params, qparams_w=qp.w_params)  # fmt: skip

        # dW_g = dY_g^T X_g, into main_grad or into a fresh buffer
        if ctx.fuse_wgrad_accumulation:
            wgrads = [w.main_grad for w in weights]
        else:
            wgrads = list(torch.empty((n, out_features, in_features), dtype=qp.mm_wgrad.out_dtype or dy.dtype,
                                      device=ctx.device).unbind(0))  # fmt: skip
        op.grouped_qgemm(qdy_t, qx_t, qp.mm_wgrad, sdy_t, sx_t, wgrads,
                         accumulate=_adds_to_main_grad(ctx.fuse_wgrad_accumulation, ctx.is_first_microbatch),
                         qparams_x=qp.g_params, qparams_w=qp.x_params)  # fmt: skip
        wgrads = [reset_wgrad_if_needed(ctx, w, g) for w, g in zip(weights, wgrads)]

        nones = (None,) * _ATorchQuantizedGroupedLinear.NUM_NON_TENSOR_ARGS
        return (dgrad.view(ctx.x_shape), *nones, *wgrads, *bias_grads)


def _stack_of(ts) -> Optional[torch.Tensor]:
    """The equally shaped tensors as one ``[len(ts), ...]`` tensor without a copy when they are dense,
    equally spaced views of one buffer (the module's weights are); else None."""
    from .quantization import _base_of_stack

    ts = list(ts)
    info = _base_of_stack(ts)
    if info is None or info[1] != ts[0].numel():
        return None
    # Adjacent addresses are not enough for a strided view: after module.to() / .bfloat16() /
    # load_state_dict the tensors may sit side by side in memory and still own separate storages.
    t0 = ts[0]
    st0 = t0.untyped_storage()
    if any(t.untyped_storage().data_ptr() != st0.data_ptr() for t in ts):
        return None
    if (t0.storage_offset() + len(ts) * t0.numel()) * t0.element_size() > st0.nbytes():
        return None
    return torch.as_strided(t0, (len(ts), *t0.shape), (t0.numel(), *t0.stride()))


class _GroupedLinearDeviceOffsets(torch.autograd.Function):
    """The same three GEMMs driven by device-side ``group_offsets`` (int64 ``[E + 1]``) instead of the
    host list ``m_splits``: nothing in forward or backward waits for the device, which is what the
    ``tokens_per_expert.cpu()`` upstream of the reference's call costs (grouped_gemm_moe.py:837).
    Needs the fused kernels, i.e. the HIP operator; arithmetic, weight cache and gradient
    conventions are those of ``_ATorchQuantizedGroupedLinear``."""

    @staticmethod
    def forward(ctx, x, group_offsets, module, is_grad_enabled, is_first_microbatch, *weights_and_biases):
        from . import kernels
        from .bias_gather_add import bias_gather_add_bw  # noqa: F401  (used in backward)

        qp = module.qlinear_params
        E = module.num_gemms
        weights, biases = weights_and_biases[:E], weights_and_biases[E:]
        K = weights[0].shape[-1]
        assert x.shape[-1] == K, "GEMM not possible"
        assert group_offsets.dtype == torch.int64 and group_offsets.numel() == E + 1 and group_offsets.is_cuda
        x2d = x.reshape(-1, K).contiguous()
        out_dtype = x.dtype if qp.mm_fprop.out_dtype is None else qp.mm_fprop.out_dtype
        kdt = torch.float32 if out_dtype == torch.float16 else out_dtype

        cached = getattr(module, "_stacked_weight_codes", None)
        # one cache for both call forms: the stacked codes are valid only while the per-expert caches, which the
        # m_splits form refreshes, still hold their slices
        if cached is not None and any(
            c.data is None or c.data.data_ptr() != cached[0][i].data_ptr()
            for i, c in enumerate(module.weight_qresult_caches)
        ):
            cached = None
        update = is_first_microbatch or is_first_microbatch is None or force_quantize_per_microbatch()
        if update or cached is None or (is_grad_enabled and cached[2] is None):
            wstack = _stack_of([w.detach() for w in weights])
            if wstack is None:
                wstack = torch.stack([w.detach() for w in weights])
            cached = kernels.block_quant_batched(wstack, eps=qp.w_params.eps, return_transpose=is_grad_enabled)
            if not force_quantize_per_microbatch():
                module._stacked_weight_codes = cached
                for i, cache in enumerate(module.weight_qresult_caches):
                    cache.data, cache.scale = cached[0][i], cached[1][i]
                    cache.data_t = cached[2][i] if is_grad_enabled else None
                    cache.scale_t = cached[3][i] if is_grad_enabled else None
        qw, sw, qw_t, sw_t = cached

        if is_grad_enabled:
            qx, sx, qx_t, sx_t = kernels.tile_quant_dual_grouped(x2d, group_offsets, E, eps=qp.x_params.eps, blocked=True)
        else:
            qx, sx = kernels.tile_quant(x2d, eps=qp.x_params.eps)
        bias = None
        if module.apply_bias:
            bias = torch.stack([cast_if_needed(b, module.activation_dtype) for b in biases])
            if bias.dtype == torch.float16:
                bias = bias.float()
        out = kernels.grouped_gemm_nt(qx, sx, qw, sw, group_offsets, out_dtype=kdt, bias=bias)
        if is_grad_enabled:
            ctx.module, ctx.x_shape, ctx.is_first_microbatch = module, x.shape, is_first_microbatch
            ctx.weight_refs = list(weights)
            ctx.num_bias_inputs = len(biases)
            ctx.fuse_wgrad_accumulation = module.fuse_wgrad_accumulation
            ctx.save_for_backward(group_offsets, qx_t, sx_t, qw_t, sw_t)
        return out.to(out_dtype).view(*x.shape[:-1], out.shape[-1])

    @staticmethod
    def backward(ctx, dy):
        from . import kernels
        from .bias_gather_add import bias_gather_add_bw

        goff, qx_t, sx_t, qw_t, sw_t = ctx.saved_tensors
        module, weights = ctx.module, ctx.weight_refs
        qp, E = module.qlinear_params, module.num_gemms
        dy2d = dy.reshape(-1, dy.shape[-1]).contiguous()
        M = dy2d.shape[0]
        dgrad_dtype = dy.dtype if qp.mm_dgrad.out_dtype is None else qp.mm_dgrad.out_dtype
        wgrad_dtype = dy.dtype if qp.mm_wgrad.out_dtype is None else qp.mm_wgrad.out_dtype
        f32_if_half = lambda dt: torch.float32 if dt == torch.float16 else dt  # noqa: E731

        bgrads = [None] * ctx.num_bias_inputs
        if module.apply_bias:
            counts = goff[1:] - goff[:-1]
            bin_ids = torch.repeat_interleave(torch.arange(E, device=dy.device), counts, output_size=M)
            g = dy2d if dy2d.dtype != torch.float16 else dy2d.float()
            bgrads = list(bias_gather_add_bw(g, bin_ids, E).to(dy.dtype).unbind(0))
        qdy, sdy, qdy_t, sdy_t = kernels.tile_quant_dual_grouped(
            dy2d, goff, E, eps=qp.g_params.eps, ld_t=kernels.qt_ld(qx_t), blocked=True
        )
        dgrad = kernels.grouped_gemm_nt(qdy, sdy, qw_t, sw_t, goff, out_dtype=f32_if_half(dgrad_dtype)).to(dgrad_dtype)

        accumulate = _adds_to_main_grad(ctx.fuse_wgrad_accumulation, ctx.is_first_microbatch)
        if ctx.fuse_wgrad_accumulation:
            main = _stack_of([w.main_grad for w in weights])
            if main is not None and main.dtype in (torch.float32, torch.bfloat16):
                kernels.grouped_gemm_wgrad(qdy_t, sdy_t, qx_t, sx_t, goff, out=main, accumulate=accumulate)
            else:  # main_grad tensors that do not tile one buffer: one extra pass
                tmp = kernels.grouped_gemm_wgrad(qdy_t, sdy_t, qx_t, sx_t, goff, out_dtype=torch.float32)
                for i, w in enumerate(weights):
                    w.main_grad.add_(tmp[i]) if accumulate else w.main_grad.copy_(tmp[i])
            wgrads = [w.main_grad for w in weights]
        else:
            wbuf = kernels.grouped_gemm_wgrad(qdy_t, sdy_t, qx_t, sx_t, goff, out_dtype=f32_if_half(wgrad_dtype))
            wgrads = list(wbuf.to(wgrad_dtype).unbind(0))
        wgrads = [reset_wgrad_if_needed(ctx, w, g) for w, g in zip(weights, wgrads)]
        return (dgrad.view(ctx.x_shape), None, None, None, None, *wgrads, *bgrads)


def patch_grouped_linear(module) -> None:
    """Registration hook in the shape of ``patch_kitchen_grouped_linear``
    (quantized_grouped_linear.py:572-584): replaces ``module._QuantizedGroupedLinear`` and
    ``module.GroupedLinear`` (and, when the module defines them, the reference's own
    ``_ATorchQuantizedGroupedLinear`` / ``ATorchGroupedLinear`` names) by the classes of this package.
    ``module`` is ``kitchen.grouped_linear``, ``atorch.modules.fp8.quantized_grouped_linear`` or any
    namespace a model builds its grouped linears from."""
    if module is None:
        return
    module._QuantizedGroupedLinear = _ATorchQuantizedGroupedLinear
    module.GroupedLinear = ATorchGroupedLinear
    for name, cls in (("_ATorchQuantizedGroupedLinear", _ATorchQuantizedGroupedLinear),
                      ("ATorchGroupedLinear", ATorchGroupedLinear)):  # fmt: skip
        if hasattr(module, name):
            setattr(module, name, cls)
    logger.info("grouped linear of %s patched to the MI355X kernels", getattr(module, "__name__", module))


class ATorchGroupedLinear(torch.nn.Module):
    """Applies ``y_i = x_i A_i^T + b_i`` to ``num_gemms`` row groups of one input tensor.

    Constructor and ``forward`` follow atorch/modules/fp8/quantized_grouped_linear.py:349-371,
    498-569.  ``tp_size`` / ``parallel_mode`` only change the parameter shapes; no communication
    happens here.  ``qlinear_params`` defaults to the 1x128 / 128x128 e4m3fn recipe on the HIP
    kernels.
    """

    def __init__(
        self,
        num_gemms: int,
        in_features: int,
        out_features: int,
        sequence_parallel: bool = False,
        fuse_wgrad_accumulation: bool = False,
        tp_group: Optional[Any] = None,
        tp_size: int = 1,
        get_rng_state_tracker: Optional[Callable] = None,
        rng_tracker_name: Optional[str] = None,
        init_method: Optional[Callable] = None,
        bias: bool = True,
        return_bias: bool = False,
        params_dtype: Optional[torch.dtype] = None,
        parallel_mode: Optional[str] = None,
        device: Union[torch.device, str] = "cuda",
        ub_overlap_rs: bool = False,
        ub_overlap_ag: bool = False,
        ub_name: Optional[str] = None,
        layer_number: Optional[int] = None,
        qlinear_params: Optional[QLinearParams] = None,
    ) -> None:
        super().__init__()
        self.tp_group = tp_group
        self.tp_size = tp_size if tp_group is None else torch.distributed.get_world_size(tp_group)
        self.tp_group_initialized = tp_group is not None or self.tp_size == 1
        self.sequence_parallel = sequence_parallel
        self.fsdp_group = None

        params_dtype = torch.get_default_dtype() if params_dtype is None else params_dtype
        self.num_gemms = num_gemms
        self.in_features = in_features
        self.out_features = out_features
        self.fuse_wgrad_accumulation = fuse_wgrad_accumulation
        if self.tp_size > 1 and bias:
            raise ValueError(
                "GroupedLinear doesn't support bias when TP > 1. "
                "Because the TP communication is handled outside of this module."
            )
        self.use_bias = bias
        self.return_bias = return_bias
        self.apply_bias = bias and not return_bias
        self.ub_overlap_rs = ub_overlap_rs
        self.ub_overlap_ag = ub_overlap_ag
        self.ub_name = ub_name
        assert not ub_overlap_rs and not ub_overlap_ag, "GroupedLinear doesn't support Userbuffer overlap."
        self.layer_name = ub_name
        self.layer_number = layer_number
        self.get_rng_state_tracker = get_rng_state_tracker
        self.rng_tracker_name = rng_tracker_name

        self.qlinear_params = self.set_qlinear_params(qlinear_params, layer_number, self.layer_name)

        self.parallel_mode = parallel_mode
        assert self.parallel_mode in ("row", "column", None), f"parallel_mode {parallel_mode} not supported"
        if self.parallel_mode == "column":
            self.out_features = divide(self.out_features, self.tp_size)
        elif self.parallel_mode == "row":
            self.in_features = divide(self.in_features, self.tp_size)

        self._init_method = init_method
        # all expert weights live in one buffer; weight{i} are views of it
        wbuf = torch.empty(num_gemms, self.out_features, self.in_features, device=device, dtype=params_dtype)
        for i in range(self.num_gemms):
            self.register_parameter(f"weight{i}", torch.nn.Parameter(wbuf[i]))
            if self.use_bias:
                self.register_parameter(
                    f"bias{i}", torch.nn.Parameter(torch.empty(self.out_features, device=device, dtype=params_dtype))
                )
            else:
                setattr(self, f"bias{i}", torch.Tensor().to(dtype=params_dtype, device=device))
        self.reset_parameters(defer_init=(str(device) == "meta"))

        # quantized weight cache between microbatches
        self.weight_qresult_caches = [QuantizeResultCache() for _ in range(self.num_gemms)]
        self.activation_dtype = params_dtype

    # -- services the reference takes from its base class ------------------------------------------
    @staticmethod
    def set_qlinear_params(qlinear_params, layer_number=None, layer_name=None) -> QLinearParams:
        if qlinear_params is None:
            qlinear_params = default_qlinear_params()
        if qlinear_params.quantize_op is None:
            raise ValueError("qlinear_params.quantize_op must be set")
        return qlinear_params

    def set_tensor_parallel_group(self, tp_group) -> None:
        self.tp_group = tp_group
        self.tp_group_initialized = True

    def set_activation_dtype(self, inp: torch.Tensor) -> None:
        if torch.is_autocast_enabled():
            self.activation_dtype = torch.get_autocast_gpu_dtype()
        else:
            self.activation_dtype = inp.dtype

    def reset_parameters(self, defer_init: bool = False) -> None:
        if defer_init:
            return
        with torch.no_grad():
            for i in range(self.num_gemms):
                w = getattr(self, f"weight{i}")
                ctx = None
                if self.get_rng_state_tracker is not None:
                    tracker = self.get_rng_state_tracker()
                    ctx = tracker.fork(self.rng_tracker_name) if self.rng_tracker_name else tracker.fork()
                if ctx is not None:
                    with ctx:
                        self._init_weight(w)
                else:
                    self._init_weight(w)
                # tensor-parallel attributes, as set_tensor_model_parallel_attributes would
                setattr(w, "tensor_model_parallel", True)
                setattr(w, "partition_dim", 1 if self.parallel_mode == "row" else 0)
                setattr(w, "partition_stride", 1)
                if self.use_bias:
                    b = getattr(self, f"bias{i}")
                    b.zero_()
                    if self.parallel_mode == "row":
                        setattr(b, "sequence_parallel", self.sequence_parallel)
                    elif self.parallel_mode == "column":
                        setattr(b, "tensor_model_parallel", True)
                        setattr(b, "partition_dim", 0)
                        setattr(b, "partition_stride", 1)

    def _init_weight(self, w: torch.Tensor) -> None:
        if self._init_method is not None:
            self._init_method(w)
        else:
            torch.nn.init.normal_(w, mean=0.0, std=0.023)

    @torch._dynamo.disable(recursive=True)
    def forward(
        self,
        inp: torch.Tensor,
        m_splits: Optional[List[int]],
        is_first_microbatch: Optional[bool] = None,
        inp_metas=None,
        group_offsets: Optional[torch.Tensor] = None,
    ):
        """``group_offsets`` (not in the reference): exclusive row prefix per group, int64 ``[num_gemms + 1]``
        on the device, as the dispatcher of this package produces it.  When given, ``m_splits`` may be
        None and no host copy of the routing is needed."""
        self.set_activation_dtype(inp)
        inp = inp.contiguous()
        assert self.tp_group_initialized, "TP group not initialized"
        input_dtypes = (torch.float, torch.float16, torch.bfloat16, torch.float32)
        assert inp.dtype in input_dtypes, f"Input dtype {inp.dtype} not supported"
        assert all(
            isinstance(c, QuantizeResultCache) for c in self.weight_qresult_caches
        ), "weight_qresult_cache must be QuantizeResultCache"
        assert self.qlinear_params.quantize, "Quantization must be enabled for GroupedLinear"

        weight_tensors = [getattr(self, f"weight{i}") for i in range(self.num_gemms)]
        bias_tensors = [getattr(self, f"bias{i}") for i in range(self.num_gemms)]

        if group_offsets is not None:
            if not getattr(self.qlinear_params.quantize_op, "supports_fused_grouped", False):
                raise ValueError("group_offsets needs the fused grouped kernels of the HIP operator")
            fn = _GroupedLinearDeviceOffsets.apply if torch.is_grad_enabled() else _GroupedLinearDeviceOffsets.forward
            head = () if torch.is_grad_enabled() else (None,)
            out = fn(*head, inp, group_offsets, self, torch.is_grad_enabled(), is_first_microbatch,
                     *weight_tensors, *(bias_tensors if self.use_bias else []))  # fmt: skip
            if self.return_bias:
                return out, [cast_if_needed(b, self.activation_dtype) for b in bias_tensors]
            return out
        assert len(m_splits) == self.num_gemms, "Number of splits should match number of GEMMs."

        if torch.is_grad_enabled():
            linear_fn = _ATorchQuantizedGroupedLinear.apply
            args: List[Any] = []
        else:
            linear_fn = _ATorchQuantizedGroupedLinear.forward
            args = [None]
        args += (
            inp,
            m_splits,
            self.apply_bias,
            inp_metas,
            self.weight_qresult_caches,
            self.qlinear_params,
            self.activation_dtype,
            torch.is_grad_enabled(),
            is_first_microbatch,
            self.fuse_wgrad_accumulation,
            *weight_tensors,
            *bias_tensors,
        )
        out = linear_fn(*args)

        if self.return_bias:
            return out, [cast_if_needed(b, self.activation_dtype) for b in bias_tensors]
        return out


GroupedLinear = ATorchGroupedLinear

"""MI355X-native FP8 grouped-linear MoE expert path.

Hand-written gfx950 kernels behind a C ABI (``include/atorch_amd_fp8.h``), with a host side
that mirrors the reference's Python surfaces for this path:

* ``atorch_amd.kernels``          - ``tile_quant`` / ``block_quant`` / ``dequant`` / ``fp8_gemm`` and the
  fused / grouped forms;
* ``atorch_amd.quantization``     - the ``quantize_op`` plugin object and its config types;
* ``atorch_amd.grouped_linear``   - ``ATorchGroupedLinear`` and its autograd function;
* ``atorch_amd.token_dispatcher`` - ``permute`` / ``unpermute`` and the single-GPU dispatcher;
* ``atorch_amd.gmm``              - the ``gmm(a, b, batch_sizes, trans_b)`` adapter;
* ``atorch_amd.expert_mlp``       - ``gmm -> SwiGLU -> gmm`` of an expert MLP, SwiGLU fused into the quantiser;
* ``atorch_amd.bias_gather_add``  - per-expert bias on expert-tagged rows and its bias gradient;
* ``atorch_amd.ops``              - the module the reference's dense FP8 wrappers load by name.
"""
__version__ = "0.1.0"

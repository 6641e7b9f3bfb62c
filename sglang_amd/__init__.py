"""MI355X-native (gfx950) quantized-linear kernels behind SGLang's ``torch.ops.sgl_kernel``
operator boundary.

Importing this package loads ``libsglamd.so`` (hand-written HIP kernels behind a C ABI)
and registers the operators; it raises if the library is not built.  The functions
re-exported here have the signatures of ``sgl_kernel``'s Python shims
(sgl-kernel/python/sgl_kernel/__init__.py:53-98).
"""
from . import ops  # noqa: F401  (registers torch.ops.sgl_kernel.*)
from .gemm import (fp8_blockwise_scaled_mm, fp8_scaled_mm, int8_scaled_mm, sgl_per_token_group_quant_8bit,  # noqa: F401
                   sgl_per_token_group_quant_fp8, sgl_per_token_group_quant_int8, sgl_per_token_quant_fp8)
from .moe import (apply_shuffle_mul_sum, es_fp8_blockwise_scaled_grouped_mm, fp8_blockwise_scaled_grouped_mm, gelu_and_mul,  # noqa: F401
                  gelu_tanh_and_mul, moe_align_block_size, moe_sum_reduce, prepare_moe_input, shuffle_rows, silu_and_mul, topk_sigmoid, topk_softmax)

__version__ = "0.1.0"

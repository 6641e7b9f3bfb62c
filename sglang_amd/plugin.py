"""SGLang general plugin (entry-point group ``sglang.srt.plugins``): routes the quantized-linear and fused-MoE
path of a running SGLang to this library through the hook registry
(python/sglang/srt/plugins/hook_registry.py:59-118 register, :146-165 apply_hooks; plugins are discovered and
called by python/sglang/srt/plugins/__init__.py:35-87,104-130).

``register()`` is the entry point.  It only records hooks; SGLang's ``load_plugins()`` applies them.  Functions
whose whole contract is implemented here are replaced; functions of which only some configurations are
implemented are wrapped (AROUND) and fall through to SGLang's own implementation when this library raises
NotImplementedError before doing any work.  A hook patches the attribute of the defining module, so call sites
that bound the function by ``from ... import`` before the plugins were loaded keep SGLang's version; the targets
below are the ones SGLang looks up at call time."""
from typing import Callable, List, Tuple

_Q = "sglang.srt.layers.quantization."
_M = "sglang.srt.layers.moe."


def _fallthrough(ours: Callable) -> Callable:
    """AROUND hook: try this library, hand unimplemented configurations to the original."""

    def around(original_fn, *args, **kwargs):
        try:
            return ours(*args, **kwargs)
        except NotImplementedError:
            return original_fn(*args, **kwargs)

    around.__qualname__ = f"sglang_amd[{getattr(ours, '__qualname__', repr(ours))}]"
    return around


def hook_table() -> List[Tuple[str, Callable, str]]:
    """(target, hook, "replace" | "around") for every function of the path."""
    from .moe_runner.cutlass_moe import cutlass_fused_experts_fp8
    from .moe_runner.fused_moe import fused_experts_impl
    from .moe_runner.moe_align_block_size import moe_align_block_size
    from .quantization import fp8_kernel, fp8_utils, int8_kernel

    return [
        # activation quantisation (fp8_kernel.py:498-678, int8_kernel.py:59-226)
        (_Q + "fp8_kernel.sglang_per_token_group_quant_fp8", fp8_kernel.sglang_per_token_group_quant_fp8, "replace"),
        (_Q + "fp8_kernel.sglang_per_token_group_quant_8bit", fp8_kernel.sglang_per_token_group_quant_8bit, "replace"),
        (_Q + "fp8_kernel.per_token_group_quant_fp8", fp8_kernel.per_token_group_quant_fp8, "replace"),
        (_Q + "fp8_kernel.sglang_per_token_quant_fp8", fp8_kernel.sglang_per_token_quant_fp8, "replace"),
        (_Q + "int8_kernel.per_token_quant_int8", int8_kernel.per_token_quant_int8, "replace"),
        (_Q + "int8_kernel.per_token_group_quant_int8", int8_kernel.per_token_group_quant_int8, "replace"),
        # block-scaled GEMMs: other block shapes stay with SGLang (fp8_kernel.py:1285-1300, int8_kernel.py:355-425)
        (_Q + "fp8_kernel.w8a8_block_fp8_matmul", _fallthrough(fp8_kernel.w8a8_block_fp8_matmul), "around"),
        (_Q + "int8_kernel.w8a8_block_int8_matmul", _fallthrough(int8_kernel.w8a8_block_int8_matmul), "around"),
        # linear wrappers (fp8_utils.py:350-365, 1458-1560)
        (_Q + "fp8_utils.dispatch_w8a8_block_fp8_linear", lambda: fp8_utils.aiter_w8a8_block_fp8_linear, "replace"),
        (_Q + "fp8_utils.apply_fp8_linear", _fallthrough(fp8_utils.apply_fp8_linear), "around"),
        # fused MoE (triton_utils/fused_moe.py:788-893, moe_align_block_size.py:19-87, cutlass_moe.py:29-341)
        (_M + "moe_runner.triton_utils.fused_moe.fused_experts_impl", _fallthrough(fused_experts_impl),
         "around"),
        (_M + "moe_runner.triton_utils.moe_align_block_size.moe_align_block_size",
         moe_align_block_size, "replace"),
        (_M + "cutlass_moe.cutlass_fused_experts_fp8", _fallthrough(cutlass_fused_experts_fp8), "around"),
    ]


def register() -> int:
    """Registers the hooks of hook_table() with SGLang's HookRegistry and returns how many were registered.
    Raises ImportError when SGLang (or this library's HIP build) is not importable: a plugin that silently did
    nothing would leave the slow path in place unnoticed."""
    from sglang.srt.plugins.hook_registry import HookRegistry, HookType

    kinds = {"replace": HookType.REPLACE, "around": HookType.AROUND}
    table = hook_table()
    for target, hook, kind in table:
        HookRegistry.register(target, hook, kinds[kind])
    return len(table)

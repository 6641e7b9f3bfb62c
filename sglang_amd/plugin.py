"""SGLang general plugin (entry-point group ``sglang.srt.plugins``): routes the quantized-linear and fused-MoE
path of a running SGLang to this library through the hook registry
(python/sglang/srt/plugins/hook_registry.py:59-118 register, :146-165 apply_hooks; plugins are discovered and
called by python/sglang/srt/plugins/__init__.py:35-87,104-141).

``register()`` is the entry point.  It records hooks (SGLang's ``load_plugins()`` applies them right after), puts
this library's fused function into the MoE runner pool and announces its FP8 GEMM backend name.  Functions whose
whole contract is implemented here are replaced; functions of which only some configurations are implemented are
wrapped (AROUND) and fall through to SGLang's own implementation when this library raises NotImplementedError,
which it does before doing any work.

A hook patches ONE attribute of ONE module (hook_registry.py:183-197), and SGLang binds most of these functions
with ``from ... import`` at import time, long before plugins are loaded: patching only the defining module would
leave every such importer on SGLang's own function.  So each hook is registered on the defining module and on
every importing name: the ones listed in IMPORTERS (module-scope ``from`` imports in the reference tree) when
their module is already loaded, plus any other loaded ``sglang.*`` module attribute that is the very same
function object.  Modules imported after the hooks are applied pick the patched function up from the defining
module by themselves."""
import sys
from typing import Callable, Dict, List, Tuple

_Q = "sglang.srt.layers.quantization."
_M = "sglang.srt.layers.moe."
_T = _M + "moe_runner.triton_utils."

FP8_GEMM_BACKEND_NAME = "sglang_amd"

# defining name -> names that bind the same function by `from ... import` at module scope
IMPORTERS: Dict[str, List[str]] = {
    _Q + "fp8_utils.dispatch_w8a8_block_fp8_linear": [
        _Q + "fp8.dispatch_w8a8_block_fp8_linear",
        _Q + "compressed_tensors.schemes.compressed_tensors_w8a8_fp8.dispatch_w8a8_block_fp8_linear",
    ],
    _Q + "fp8_utils.apply_fp8_linear": [
        _Q + "fp8.apply_fp8_linear",
        _Q + "w8a8_fp8.apply_fp8_linear",
        _Q + "fpgemm_fp8.apply_fp8_linear",
        _Q + "modelopt_quant.apply_fp8_linear",
        _Q + "compressed_tensors.schemes.compressed_tensors_w8a8_fp8.apply_fp8_linear",
        _Q + "quark.schemes.quark_w8a8_fp8.apply_fp8_linear",
    ],
    _Q + "fp8_kernel.sglang_per_token_group_quant_fp8": [
        _Q + "fp8_utils.sglang_per_token_group_quant_fp8",
        _T + "fused_moe_triton_kernels.sglang_per_token_group_quant_fp8",
        _M + "token_dispatcher.deepep.sglang_per_token_group_quant_fp8",
        _M + "ep_moe.kernels.per_token_group_quant_fp8",
        "sglang.srt.models.deepseek_v4.sglang_per_token_group_quant_fp8",
    ],
    _Q + "fp8_kernel.per_token_group_quant_fp8": [
        _Q + "fp8.per_token_group_quant_fp8",
        _Q + "fp8_utils.per_token_group_quant_fp8",
        _Q + "w8a8_fp8.per_token_group_quant_fp8",
        _T + "fused_moe_triton_kernels.per_token_group_quant_fp8",
        _M + "moe_runner.flashinfer_trtllm.per_token_group_quant_fp8",
    ],
    _Q + "fp8_kernel.sglang_per_token_quant_fp8": [_Q + "fp8_utils.sglang_per_token_quant_fp8"],
    _Q + "fp8_kernel.static_quant_fp8": [_Q + "fp8_utils.static_quant_fp8"],
    _Q + "fp8_kernel.w8a8_block_fp8_matmul_triton": [_Q + "fp8_utils.w8a8_block_fp8_matmul_triton"],
    _Q + "int8_kernel.per_token_quant_int8": [
        _Q + "w8a8_int8.per_token_quant_int8",
        _Q + "qoq.per_token_quant_int8",
        _Q + "compressed_tensors.schemes.compressed_tensors_w8a8_int8.per_token_quant_int8",
        _T + "fused_moe_triton_kernels.per_token_quant_int8",
    ],
    _Q + "int8_kernel.per_token_group_quant_int8": [
        _Q + "int8_utils.per_token_group_quant_int8",
        _T + "fused_moe_triton_kernels.per_token_group_quant_int8",
    ],
    _Q + "int8_kernel.w8a8_block_int8_matmul": [_Q + "int8_utils.w8a8_block_int8_matmul"],
    _T + "moe_align_block_size.moe_align_block_size": [
        _T + "moe_align_block_size",  # the package re-exports the function under the submodule's name
        _T + "fused_moe.moe_align_block_size",
        _M + "fused_moe_triton.moe_align_block_size",
        "sglang.srt.lora.lora_moe_runner_marlin.moe_align_block_size",
    ],
    _M + "cutlass_moe.cutlass_fused_experts_fp8": [_Q + "fp8.cutlass_fused_experts_fp8"],
}


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
    """(defining target, hook, "replace" | "around") for every function of the path."""
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
        (_Q + "fp8_kernel.static_quant_fp8", fp8_kernel.static_quant_fp8, "replace"),
        (_Q + "int8_kernel.per_token_quant_int8", int8_kernel.per_token_quant_int8, "replace"),
        (_Q + "int8_kernel.per_token_group_quant_int8", int8_kernel.per_token_group_quant_int8, "replace"),
        # block-scaled GEMMs: other block shapes stay with SGLang (fp8_kernel.py:1201-1300, int8_kernel.py:355-425)
        (_Q + "fp8_kernel.w8a8_block_fp8_matmul", _fallthrough(fp8_kernel.w8a8_block_fp8_matmul), "around"),
        (_Q + "fp8_kernel.w8a8_block_fp8_matmul_triton", _fallthrough(fp8_kernel.w8a8_block_fp8_matmul), "around"),
        (_Q + "int8_kernel.w8a8_block_int8_matmul", _fallthrough(int8_kernel.w8a8_block_int8_matmul), "around"),
        # linear wrappers (fp8_utils.py:350-365, 1458-1560); the selector hands out a linear that itself falls
        # back to what SGLang would have selected
        (_Q + "fp8_utils.dispatch_w8a8_block_fp8_linear", _dispatch_around, "around"),
        (_Q + "fp8_utils.apply_fp8_linear", _fallthrough(fp8_utils.apply_fp8_linear), "around"),
        # fused MoE (triton_utils/fused_moe.py:788-893, moe_align_block_size.py:19-87, cutlass_moe.py:29-341)
        (_T + "fused_moe.fused_experts_impl", _fallthrough(fused_experts_impl), "around"),
        (_T + "moe_align_block_size.moe_align_block_size", moe_align_block_size, "replace"),
        (_M + "cutlass_moe.cutlass_fused_experts_fp8", _fallthrough(cutlass_fused_experts_fp8), "around"),
    ]


def _dispatch_around(original_dispatch, *args, **kwargs):
    """dispatch_w8a8_block_fp8_linear returns the linear function the layer will call for its whole life
    (fp8.py:350, fp8_utils.py:350-365).  Ours is returned wrapped so that a call it does not implement (a static
    input scale in an unexpected form, say) still reaches the function SGLang would have picked."""
    from .quantization import fp8_utils

    theirs = original_dispatch(*args, **kwargs)
    ours = fp8_utils.aiter_w8a8_block_fp8_linear

    def w8a8_block_fp8_linear(*a, **k):
        try:
            return ours(*a, **k)
        except NotImplementedError:
            return theirs(*a, **k)

    return w8a8_block_fp8_linear


def _resolve(dotted: str):
    """The object a dotted `module.attr` names, importing nothing that is not loaded yet (None if absent)."""
    mod_name, _, attr = dotted.rpartition(".")
    mod = sys.modules.get(mod_name)
    return getattr(mod, attr, None) if mod is not None else None


def binding_targets(defining: str) -> List[str]:
    """Every name a hook for `defining` has to be registered on: the defining name itself (its module is imported
    if need be), the listed importers whose module is loaded and still binds the original function, and any
    other loaded sglang.* module attribute that is the same object."""
    import importlib

    mod_name, _, attr = defining.rpartition(".")
    try:
        original = getattr(importlib.import_module(mod_name), attr)
    except (ImportError, AttributeError):
        return []
    out = [defining]
    for name in IMPORTERS.get(defining, []):
        if _resolve(name) is original:
            out.append(name)
    for mname, mod in list(sys.modules.items()):
        if mod is None or not mname.startswith("sglang.") or mname == mod_name:
            continue
        for a, v in list(getattr(mod, "__dict__", {}).items()):
            if v is original and f"{mname}.{a}" not in out:
                out.append(f"{mname}.{a}")
    return out


def register_moe_fused_func() -> bool:
    """Puts this library's fused function into the ("none", "triton") slot of the MoE runner pool
    (python/sglang/srt/layers/moe/moe_runner/base.py:118-143; SGLang's own entry is registered at
    moe_runner/triton.py:139-172), keeping the previous entry as the fall-through for configurations that raise
    NotImplementedError here.  register_fused_func refuses a second registration of a slot, so the pool's table
    is updated directly."""
    from sglang.srt.layers.moe.moe_runner.base import FusedOpPool

    from .moe_runner.base import fused_experts_none_to_triton

    try:
        import sglang.srt.layers.moe.moe_runner.triton  # noqa: F401  (registers SGLang's own entry first)
    except ImportError:
        pass
    key = ("none", "triton")
    previous = FusedOpPool._fused_funcs.get(key)
    if getattr(previous, "_sglang_amd", False):
        return False

    def fused(dispatch_output, quant_info, runner_config):
        try:
            return fused_experts_none_to_triton(dispatch_output, quant_info, runner_config)
        except NotImplementedError:
            if previous is None:
                raise
            return previous(dispatch_output, quant_info, runner_config)

    fused._sglang_amd = True
    FusedOpPool._fused_funcs[key] = fused
    return True


def register() -> int:
    """Registers the hooks of hook_table() on every binding of each function with SGLang's HookRegistry, the fused
    MoE function and the backend name; returns how many hooks were registered.  Raises ImportError when SGLang
    (or this library's HIP build) is not importable: a plugin that silently did nothing would leave the slow
    path in place unnoticed."""
    from sglang.srt.plugins.hook_registry import HookRegistry, HookType

    kinds = {"replace": HookType.REPLACE, "around": HookType.AROUND}
    count = 0
    for defining, hook, kind in hook_table():
        for target in binding_targets(defining):
            HookRegistry.register(target, hook, kinds[kind])
            count += 1
    try:
        register_moe_fused_func()
    except ImportError:
        pass  # an SGLang without the runner pool: the fused_experts_impl hook still reroutes the layer
    try:
        from sglang.srt.server_args import add_fp8_gemm_runner_backend_choices

        add_fp8_gemm_runner_backend_choices([FP8_GEMM_BACKEND_NAME])
    except ImportError:
        pass
    return count

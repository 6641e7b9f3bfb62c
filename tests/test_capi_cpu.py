"""CPU-side checks of the boundary: the C-ABI library loads, exports every function that
include/sglamd.h declares (and the ctypes table matches it), the operators are registered under
torch.ops.sgl_kernel with the reference's schemas, and the host-side helpers allocate the
reference's scale layouts.  No kernel is launched."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "sglamd.h")


def _declared():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(sglamd_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from sglang_amd import _lib

    names = _declared()
    assert len(names) >= 12
    raw = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(raw, n), f"{n} is declared in include/sglamd.h but not exported"
    assert set(_lib.SIGNATURES) | {"sglamd_last_error", "sglamd_abi_version"} == set(names)
    assert _lib.lib.sglamd_abi_version() >= 1


def test_argument_counts_match_header():
    from sglang_amd import _lib

    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    for name, args in _lib.SIGNATURES.items():
        m = re.search(name + r"\s*\((.*?)\)\s*;", text, flags=re.S)
        assert m, name
        assert len([a for a in m.group(1).split(",") if a.strip() not in ("", "void")]) == len(args), name


def test_host_side_validation_returns_error_codes_without_a_gpu():
    from sglang_amd import _lib

    rc = _lib.lib.sglamd_per_token_group_quant_8bit(None, 2, None, 3, None, 1, 128, 128, 0, 0, 1e-10, -448.0, 448.0, 0,
                                                    None)
    assert rc == -1 and b"null" in _lib.lib.sglamd_last_error()
    rc = _lib.lib.sglamd_fp8_blockwise_scaled_mm(16, 128, 16, 128, 16, 1, 1, 16, 1, 1, 16, 128, 2, 4, 128, 100, None, 0,
                                                 None)
    assert rc == -1 and b"multiple of 16" in _lib.lib.sglamd_last_error()
    with pytest.raises(_lib.SglAmdError):
        _lib.check(rc)


def test_ops_are_registered_with_reference_schemas():
    """Schema strings of sgl-kernel/csrc/common_extension.cc:76-77,116-142,164-181,483-487, compared after
    parsing (argument names, types, optionality, which arguments are written, return type)."""
    import sglang_amd  # noqa: F401

    reference = [
        "int8_scaled_mm(Tensor mat_a, Tensor mat_b, Tensor scales_a, Tensor scales_b, ScalarType out_dtype, Tensor? "
        "bias) -> Tensor",
        "fp8_scaled_mm(Tensor mat_a, Tensor mat_b, Tensor scales_a, Tensor scales_b, ScalarType out_dtype, Tensor? "
        "bias) -> Tensor",
        "fp8_blockwise_scaled_mm(Tensor mat_a, Tensor mat_b, Tensor scales_a, Tensor scales_b, ScalarType out_dtype) -> "
        "Tensor",
        "sgl_per_token_group_quant_8bit(Tensor input, Tensor! output_q, Tensor! output_s, int group_size,"
        " float eps, float fp8_min, float fp8_max, bool scale_ue8m0) -> ()",
        "sgl_per_token_group_quant_8bit_v2(Tensor input, Tensor! output_q, Tensor! output_s, int group_size,"
        " float eps, float fp8_min, float fp8_max, bool scale_ue8m0, bool fuse_silu_and_mul, Tensor? masked_m) -> ()",
        "sgl_per_token_quant_fp8(Tensor input, Tensor! output_q, Tensor! output_s) -> ()",
        "moe_align_block_size(Tensor topk_ids, int num_experts, int block_size, Tensor! sorted_token_ids, Tensor! "
        "experts_ids, Tensor! num_tokens_post_pad, Tensor! cumsum_buffer, bool "
        "pad_sorted_token_ids) -> ()",
        "silu_and_mul(Tensor! out, Tensor input) -> ()",
        # common_extension.cc:79-83
        "gelu_tanh_and_mul(Tensor! out, Tensor input) -> ()",
        "gelu_and_mul(Tensor! out, Tensor input) -> ()",
        "moe_sum_reduce(Tensor input, Tensor output, float routed_scaling_factor) -> ()",
        # common_extension.cc:170-177
        "topk_softmax(Tensor! topk_weights, Tensor! topk_indices, Tensor gating_output, bool renormalize, float "
        "moe_softcapping, Tensor? correction_bias) -> ()",
        "topk_sigmoid(Tensor! topk_weights, Tensor! topk_indices, Tensor gating_output, bool renormalize, Tensor? "
        "correction_bias) -> ()",
        # common_extension.cc:483-487
        "es_fp8_blockwise_scaled_grouped_mm(Tensor output, Tensor a, Tensor b, Tensor scales_a, Tensor scales_b, Tensor "
        "stride_a, Tensor stride_b, Tensor stride_d, Tensor problem_sizes, Tensor expert_offsets, Tensor workspace) -> "
        "()",
    ]

    def sig(schema):
        args = [(a.name, str(a.type), bool(a.alias_info and a.alias_info.is_write)) for a in schema.arguments]
        return args, [str(r.type) for r in schema.returns]

    for text in reference:
        name = text.split("(", 1)[0]
        want = torch._C.parse_schema("sgl_kernel::" + text)
        got = getattr(torch.ops.sgl_kernel, name).default._schema
        assert sig(got) == sig(want), name


def test_ops_refuse_cpu_tensors():
    import sglang_amd

    x = torch.zeros(2, 128, dtype=torch.bfloat16)
    q = torch.zeros(2, 128, dtype=torch.float8_e4m3fn)
    s = torch.zeros(2, 1)
    with pytest.raises((RuntimeError, NotImplementedError)):
        sglang_amd.sgl_per_token_group_quant_8bit(x, q, s, 128, 1e-10, -448.0, 448.0)


def test_scale_buffer_layouts():
    from sglang_amd.quantization.fp8_kernel import create_per_token_group_quant_fp8_output_scale as mk

    s = mk((6, 7168), "cpu", 128, False, False, False)
    assert s.shape == (6, 56) and s.is_contiguous()
    s = mk((6, 7168), "cpu", 128, True, False, False)
    assert s.shape == (6, 56) and s.stride() == (1, 6)
    s = mk((6, 7168), "cpu", 128, True, True, False)
    assert s.shape == (6, 56) and s.stride() == (1, 8)
    s = mk((6, 7168), "cpu", 128, True, True, True)
    assert s.shape == (6, 14) and s.stride() == (1, 8) and s.dtype == torch.int32
    s = mk((6, 640), "cpu", 128, True, True, True)
    assert s.shape == (6, 2)


def test_moe_default_block_heights():
    from sglang_amd.moe_runner import get_default_config

    assert get_default_config(1, 256, 8)["BLOCK_SIZE_M"] == 16
    assert get_default_config(256, 256, 8)["BLOCK_SIZE_M"] == 16
    assert get_default_config(512, 256, 8)["BLOCK_SIZE_M"] == 64
    assert get_default_config(2048, 256, 8)["BLOCK_SIZE_M"] == 128
    assert get_default_config(4096, 256, 8)["BLOCK_SIZE_M"] == 192


def _fake_sglang(monkeypatch):
    """A stand-in `sglang` package tree with the pieces the plugin talks to: the hook registry's interface
    (python/sglang/srt/plugins/hook_registry.py:59-197: register, apply_hooks patching ONE attribute of ONE object),
    defining modules for a few functions of the path, a module that bound them by `from ... import` before the
    plugin ran (as layers/quantization/fp8.py:55-66 does), the MoE runner pool (moe_runner/base.py:118-143) and the
    backend-choice list (server_args.py:309-310).  Every stand-in function returns a string naming itself."""
    import enum
    import functools
    import sys
    import types

    class HookType(enum.Enum):
        BEFORE = "before"
        AFTER = "after"
        AROUND = "around"
        REPLACE = "replace"

    class HookRegistry:
        hooks = []

        @classmethod
        def register(cls, target, hook, hook_type=HookType.AFTER, *, source=None):
            cls.hooks.append((target, hook, hook_type))

        @classmethod
        def apply_hooks(cls):
            for target, hook, kind in cls.hooks:
                mod_name, _, attr = target.rpartition(".")
                obj = sys.modules[mod_name]
                original = getattr(obj, attr)
                setattr(obj, attr, hook if kind == HookType.REPLACE else functools.partial(hook, original))

    def module(name, **attrs):
        m = types.ModuleType(name)
        m.__dict__.update(attrs)
        monkeypatch.setitem(sys.modules, name, m)
        return m

    def named(name):
        def fn(*a, **k):
            return "sglang:" + name
        fn.__name__ = name
        return fn

    for pkg in ("sglang", "sglang.srt", "sglang.srt.plugins", "sglang.srt.layers", "sglang.srt.layers.quantization",
                "sglang.srt.layers.moe", "sglang.srt.layers.moe.moe_runner",
                "sglang.srt.layers.moe.moe_runner.triton_utils"):
        module(pkg)
    module("sglang.srt.plugins.hook_registry", HookRegistry=HookRegistry, HookType=HookType)
    q = "sglang.srt.layers.quantization."
    kern = module(q + "fp8_kernel", **{n: named(n) for n in (
        "sglang_per_token_group_quant_fp8", "sglang_per_token_group_quant_8bit", "per_token_group_quant_fp8",
        "sglang_per_token_quant_fp8", "w8a8_block_fp8_matmul", "w8a8_block_fp8_matmul_triton")})
    module(q + "int8_kernel", **{n: named(n) for n in (
        "per_token_quant_int8", "per_token_group_quant_int8", "w8a8_block_int8_matmul")})
    their_linear = named("their_block_linear")
    utils = module(q + "fp8_utils", dispatch_w8a8_block_fp8_linear=lambda: their_linear,
                   apply_fp8_linear=named("apply_fp8_linear"),
                   per_token_group_quant_fp8=kern.per_token_group_quant_fp8)
    # bound by name before the plugin runs, like `from ...fp8_utils import ...` in layers/quantization/fp8.py
    fp8 = module(q + "fp8", dispatch_w8a8_block_fp8_linear=utils.dispatch_w8a8_block_fp8_linear,
                 apply_fp8_linear=utils.apply_fp8_linear, per_token_group_quant_fp8=kern.per_token_group_quant_fp8)
    # a module the static table does not know about that binds the same function under another name
    other = module("sglang.srt.models.some_new_model", quant=kern.per_token_group_quant_fp8)
    t = "sglang.srt.layers.moe.moe_runner.triton_utils."
    module(t + "fused_moe", fused_experts_impl=named("fused_experts_impl"))
    module(t + "moe_align_block_size", moe_align_block_size=named("moe_align_block_size"))
    module("sglang.srt.layers.moe.cutlass_moe", cutlass_fused_experts_fp8=named("cutlass_fused_experts_fp8"))

    class FusedOpPool:
        _fused_funcs = {("none", "triton"): named("fused_experts_none_to_triton")}

    module("sglang.srt.layers.moe.moe_runner.base", FusedOpPool=FusedOpPool)
    choices = []
    module("sglang.srt.server_args", add_fp8_gemm_runner_backend_choices=choices.extend)
    return types.SimpleNamespace(HookRegistry=HookRegistry, HookType=HookType, fp8=fp8, utils=utils, kern=kern,
                                 other=other, FusedOpPool=FusedOpPool, choices=choices, their_linear=their_linear)


def test_plugin_reroutes_names_bound_by_from_import_and_falls_through(monkeypatch):
    """register() + apply_hooks() against the stand-in tree: the functions of the path are rerouted where they
    are defined AND where another module had already bound them by `from ... import`; configurations this
    library refuses reach SGLang's own function; the fused MoE function and the backend name are registered."""
    from sglang_amd import plugin
    from sglang_amd.quantization import fp8_kernel as ours_kernel

    env = _fake_sglang(monkeypatch)
    n = plugin.register()
    targets = [t for t, _, _ in env.HookRegistry.hooks]
    assert n == len(targets) and len(set(targets)) == n
    q = "sglang.srt.layers.quantization."
    for must in (q + "fp8_utils.dispatch_w8a8_block_fp8_linear", q + "fp8.dispatch_w8a8_block_fp8_linear",
                 q + "fp8_utils.apply_fp8_linear", q + "fp8.apply_fp8_linear",
                 q + "fp8_kernel.per_token_group_quant_fp8", q + "fp8.per_token_group_quant_fp8",
                 q + "fp8_utils.per_token_group_quant_fp8", "sglang.srt.models.some_new_model.quant",
                 "sglang.srt.layers.moe.moe_runner.triton_utils.fused_moe.fused_experts_impl"):
        assert must in targets, must
    env.HookRegistry.apply_hooks()

    # a REPLACE hook lands on the defining module, the listed importer and the importer found by identity
    for holder, attr in ((env.kern, "per_token_group_quant_fp8"), (env.fp8, "per_token_group_quant_fp8"),
                         (env.utils, "per_token_group_quant_fp8"), (env.other, "quant")):
        assert getattr(holder, attr) is ours_kernel.per_token_group_quant_fp8

    # the block linear the importing module now selects is this library's, with SGLang's as its fall-through:
    # a static activation scale on a bf16 input is refused here before any work and reaches theirs
    for holder in (env.fp8, env.utils):
        linear = holder.dispatch_w8a8_block_fp8_linear()
        assert linear is not env.their_linear
        x = torch.zeros(2, 256, dtype=torch.bfloat16)
        w = torch.zeros(256, 256).to(torch.float8_e4m3fn)
        got = linear(x, w, [128, 128], torch.ones(2, 2), input_scale=torch.ones(1), bias=None)
        assert got == "sglang:their_block_linear"
    # apply_fp8_linear: what is not implemented (a static scale that is not per tensor, group-wise weight scales,
    # a 32-bit activation) falls through instead of raising
    x = torch.zeros(2, 256, dtype=torch.bfloat16)
    w = torch.zeros(256, 256).to(torch.float8_e4m3fn).t()
    assert env.fp8.apply_fp8_linear(x, w, torch.ones(256), input_scale=torch.ones(2)) == "sglang:apply_fp8_linear"
    assert env.fp8.apply_fp8_linear(x, w, torch.ones(2)) == "sglang:apply_fp8_linear"
    assert env.utils.apply_fp8_linear(x.float(), w, torch.ones(256)) == "sglang:apply_fp8_linear"

    # fused MoE: an AROUND hook hands a configuration this library refuses (a weight-only MoE) to the original
    import sys
    fm = sys.modules["sglang.srt.layers.moe.moe_runner.triton_utils.fused_moe"]
    x = torch.zeros(2, 256, dtype=torch.bfloat16)
    w = torch.zeros(2, 256, 256).to(torch.float8_e4m3fn)
    got = fm.fused_experts_impl(x, w, w, torch.ones(2, 1), torch.zeros(2, 1, dtype=torch.int32), use_int8_w8a16=True)
    assert got == "sglang:fused_experts_impl"

    # the runner pool's ("none", "triton") slot is this library's fused function with the previous one behind it
    from sglang_amd.moe_runner import MoeRunnerConfig, StandardDispatchOutput, StandardTopKOutput, TritonMoeQuantInfo

    fused = env.FusedOpPool._fused_funcs[("none", "triton")]
    assert getattr(fused, "_sglang_amd", False)
    topk = StandardTopKOutput(torch.ones(2, 1), torch.zeros(2, 1, dtype=torch.int32), None)
    info = TritonMoeQuantInfo(w13_weight=w, w2_weight=w, use_int4_w4a16=True)  # weight-only: refused
    assert fused(StandardDispatchOutput(x, None, topk), info, MoeRunnerConfig(inplace=False)) == \
        "sglang:fused_experts_none_to_triton"
    assert plugin.register_moe_fused_func() is False  # a second registration leaves the slot alone
    assert env.choices == [plugin.FP8_GEMM_BACKEND_NAME]


def test_runner_records_carry_the_reference_fields():
    """MoeRunnerConfig / TritonMoeQuantInfo / the standard dispatch records have the reference's field names and
    defaults (moe_runner/base.py:45-67, moe_runner/triton.py:52-69, token_dispatcher/standard.py:59-82,
    topk.py:252-262): a running SGLang passes its own instances, which are read by attribute."""
    import dataclasses

    from sglang_amd.moe_runner import (MoeRunnerConfig, StandardCombineInput, StandardDispatchOutput,
                                       StandardTopKOutput, TritonMoeQuantInfo)

    cfg = {f.name: f.default for f in dataclasses.fields(MoeRunnerConfig)}
    assert cfg["activation"] == "silu" and cfg["is_gated"] is True and cfg["inplace"] is True
    assert cfg["no_combine"] is False and cfg["routed_scaling_factor"] is None
    assert list(cfg)[:9] == ["num_experts", "num_local_experts", "hidden_size", "intermediate_size_per_partition",
                             "layer_id", "top_k", "num_fused_shared_experts", "params_dtype", "routing_method_type"]
    assert [f.name for f in dataclasses.fields(TritonMoeQuantInfo)] == [
        "w13_weight", "w2_weight", "b13", "b2", "use_fp8_w8a8", "use_int8_w8a8", "use_int8_w8a16", "use_int4_w4a16",
        "per_channel_quant", "w13_scale", "w2_scale", "w13_zp", "w2_zp", "a13_scale", "a2_scale", "block_shape"]
    assert StandardTopKOutput._fields == ("topk_weights", "topk_ids", "router_logits")
    assert StandardDispatchOutput._fields == ("hidden_states", "hidden_states_scale", "topk_output")
    assert StandardCombineInput._fields == ("hidden_states",)


def test_fused_experts_custom_ops_are_registered():
    """inplace_fused_experts / outplace_fused_experts are opaque operators with the reference's argument lists
    (triton_utils/fused_moe.py:91-215), registered under this library's own namespace."""
    import sglang_amd.moe_runner  # noqa: F401

    inplace = torch.ops.sglang_amd.inplace_fused_experts.default._schema
    outplace = torch.ops.sglang_amd.outplace_fused_experts.default._schema
    names = [a.name for a in inplace.arguments]
    assert names[:7] == ["hidden_states", "w1", "w2", "topk_weights", "topk_ids", "b1", "b2"]
    assert names[-5:] == ["routed_scaling_factor", "gemm1_alpha", "gemm1_limit", "filter_expert", "swiglu_limit"]
    assert inplace.arguments[0].alias_info is not None and inplace.arguments[0].alias_info.is_write
    assert len(inplace.returns) == 0 and len(outplace.returns) == 1
    assert [a.name for a in outplace.arguments][22:24] == ["no_combine", "routed_scaling_factor"]


def test_importing_this_library_first_leaves_sglangs_operator_names_free():
    """SGLang registers inplace_/outplace_fused_experts lazily and skips a name that torch.ops.sglang already has
    (python/sglang/srt/utils/custom_op.py:152-165).  If this library had defined those names first, SGLang's own
    wrappers would end up calling this library's operator, which has no fall-through.  So: with this library
    imported first, a registration with the reference's skip-if-present rule still registers SGLang's function."""
    import sglang_amd.moe_runner  # noqa: F401
    from sglang_amd import plugin

    plugin.hook_table()  # what register() imports before it touches SGLang's modules
    registered = {}

    def reference_style_register(op_name, op_func):
        if not hasattr(torch.ops.sglang, op_name):
            registered[op_name] = op_func
        return registered.get(op_name)

    theirs = lambda *a, **k: "sglang:original"
    for name in ("inplace_fused_experts", "outplace_fused_experts"):
        assert reference_style_register(name, theirs) is theirs, f"torch.ops.sglang.{name} was taken by this library"


def test_streaming_kernel_never_fetches_past_the_end_of_a_ragged_row():
    """The weight-streaming kernel reads 16-byte pieces of 128-byte K blocks; with K % 128 != 0 the pieces past
    the end of the row must not be fetched (their lanes re-read a piece inside the row and are zeroed).  Sweeps the
    library's own offset function over every K % 16 == 0 up to 4 blocks."""
    from sglang_amd import _lib

    off = ctypes.c_int64(0)
    for K in range(16, 4 * 128 + 1, 16):
        nkb = (K + 127) // 128
        covered = set()
        for kb in range(nkb):
            for chunk in range(8):
                dead = _lib.lib.sglamd_streaming_piece_offset(kb, chunk, K, ctypes.byref(off))
                assert 0 <= off.value and off.value + 16 <= K, (K, kb, chunk, off.value)
                assert off.value % 16 == 0
                if not dead:
                    assert off.value == kb * 128 + chunk * 16
                    covered.add(off.value)
                else:
                    assert kb * 128 + chunk * 16 >= K
        assert covered == set(range(0, K, 16)), K


def test_pyproject_declares_the_plugin_entry_point():
    import importlib

    text = open(os.path.join(ROOT, "pyproject.toml")).read()
    m = re.search(r'\[project\.entry-points\."sglang\.srt\.plugins"\]\s*\n\s*\w+\s*=\s*"([\w.]+):(\w+)"', text)
    assert m, "entry point group sglang.srt.plugins is missing"
    assert callable(getattr(importlib.import_module(m.group(1)), m.group(2)))


def test_bench_refuses_more_than_one_gpu_and_parses_its_flags():
    """bench.py measures one GPU: any other --gpus value ends with a message and a non-zero status before
    anything touches a device."""
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2", "--steps", "1", "--warmup", "0"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "single-GPU" in r.stderr and r.stdout.strip() == ""
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--help"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode == 0
    for flag in ("--gpus", "--steps", "--warmup"):
        assert flag in r.stdout

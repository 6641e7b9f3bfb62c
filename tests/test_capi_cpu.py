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
    """Schema strings of sgl-kernel/csrc/common_extension.cc:76-77,116-142,164-168,180-181, compared after
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
        "moe_sum_reduce(Tensor input, Tensor output, float routed_scaling_factor) -> ()",
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


def test_plugin_registers_hooks_with_the_reference_registry_interface(monkeypatch):
    """register() speaks the interface of sglang.srt.plugins.hook_registry (register(target, hook, hook_type),
    HookType.REPLACE / AROUND; python/sglang/srt/plugins/hook_registry.py:59-118).  SGLang is not installed here,
    so a stand-in module with that interface records the calls; wrapped targets must fall through to the
    original when this library does not implement the configuration."""
    import enum
    import sys
    import types

    calls = []

    class HookType(enum.Enum):
        BEFORE = "before"
        AFTER = "after"
        AROUND = "around"
        REPLACE = "replace"

    class HookRegistry:
        @classmethod
        def register(cls, target, hook, hook_type=HookType.AFTER, *, source=None):
            calls.append((target, hook, hook_type))

    mod = types.ModuleType("sglang.srt.plugins.hook_registry")
    mod.HookRegistry, mod.HookType = HookRegistry, HookType
    for name in ("sglang", "sglang.srt", "sglang.srt.plugins"):
        monkeypatch.setitem(sys.modules, name, types.ModuleType(name))
    monkeypatch.setitem(sys.modules, "sglang.srt.plugins.hook_registry", mod)

    from sglang_amd import plugin

    n = plugin.register()
    assert n == len(calls) >= 12
    targets = {t for t, _, _ in calls}
    assert len(targets) == n and all(t.startswith("sglang.srt.layers.") for t in targets)
    for must in ("quantization.fp8_utils.dispatch_w8a8_block_fp8_linear", "quantization.fp8_kernel.per_token_group_quant_fp8",
                 "quantization.fp8_utils.apply_fp8_linear", "moe.moe_runner.triton_utils.fused_moe.fused_experts_impl"):
        assert "sglang.srt.layers." + must in targets
    by_target = {t: (h, k) for t, h, k in calls}
    assert all(callable(h) and k in (HookType.REPLACE, HookType.AROUND) for h, k in by_target.values())
    # the dispatcher replacement hands back a linear with the reference's signature
    linear = by_target["sglang.srt.layers.quantization.fp8_utils.dispatch_w8a8_block_fp8_linear"][0]()
    assert linear.__code__.co_varnames[:6] == ("input", "weight", "block_size", "weight_scale", "input_scale", "bias")
    # an AROUND hook hands a configuration this library refuses (per-tensor fp8 MoE) to the original
    hook, kind = by_target["sglang.srt.layers.moe.moe_runner.triton_utils.fused_moe.fused_experts_impl"]
    assert kind == HookType.AROUND
    x = torch.zeros(2, 256, dtype=torch.bfloat16)
    w = torch.zeros(2, 256, 256).to(torch.float8_e4m3fn)
    got = hook(lambda *a, **k: "original", x, w, w, torch.ones(2, 1), torch.zeros(2, 1, dtype=torch.int32),
               use_fp8_w8a8=True, block_shape=None)
    assert got == "original"


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

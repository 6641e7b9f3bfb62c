"""The plugin on the GPU: after register() + apply_hooks() against a stand-in `sglang` tree, device tensors go
THROUGH the patched names (the closures plugin.py installs, not this library's functions called directly) and the
results are compared with the CPU oracle; a configuration this library refuses must reach the stand-in's
original.  Mirrors how SGLang's layers reach the path: fp8.py:350 (block linear picked once per layer),
fp8_utils.py:1458-1560 (apply_fp8_linear), moe_runner/triton.py:139-172 (fused function of the runner pool)."""
import sys

import numpy as np
import pytest
import torch

from oracle import gemm as og
from oracle import moe as om
from oracle import quant as oq
from tests.test_capi_cpu import _fake_sglang
from tests.util import assert_gemm_close

pytestmark = pytest.mark.gpu


def _fp8(a: np.ndarray, dev):
    return torch.from_numpy(a).to(dev).view(torch.float8_e4m3fn)


@pytest.fixture()
def env(monkeypatch, dev):
    from sglang_amd import plugin

    e = _fake_sglang(monkeypatch)
    assert plugin.register() > 0
    e.HookRegistry.apply_hooks()
    return e


def test_block_linear_through_the_patched_selector(env, dev):
    """fp8.dispatch_w8a8_block_fp8_linear()(x, w, block, w_scale): dynamic activation quant + block GEMM."""
    g = torch.Generator().manual_seed(5)
    x = torch.randn(3, 7, 1024, generator=g).to(torch.bfloat16)
    w = torch.randn(768, 1024, generator=g) * 0.02
    wq, ws = oq.block_quant_weight(w)
    xq, xs, _ = oq.group_quant(x.view(-1, 1024), 128, form="reciprocal")
    ref = og.block_fp8_matmul(xq, wq, xs, ws, return_fp32=True).view(3, 7, 768)
    for holder in (env.fp8, env.utils):
        linear = holder.dispatch_w8a8_block_fp8_linear()
        assert linear is not env.their_linear
        out = linear(x.to(dev), _fp8(wq, dev), [128, 128], torch.from_numpy(ws).to(dev), input_scale=None, bias=None)
        assert out.shape == (3, 7, 768) and out.dtype == torch.bfloat16
        assert_gemm_close(out, ref, "block linear through the plugin")
        bias = torch.randn(768, generator=g).to(torch.bfloat16)
        out_b = linear(x.to(dev), _fp8(wq, dev), [128, 128], torch.from_numpy(ws).to(dev), bias=bias.to(dev))
        assert_gemm_close(out_b, ref + bias.float(), "block linear + bias through the plugin")
        # refused here (a static scale on a 16-bit input, another block shape): SGLang's own linear answers
        assert linear(x.to(dev), _fp8(wq, dev), [128, 128], torch.from_numpy(ws).to(dev),
                      input_scale=torch.ones(1, device=dev)) == "sglang:their_block_linear"
        assert linear(x.to(dev), _fp8(wq, dev), [32, 32], torch.ones(24, 32, device=dev)) == "sglang:their_block_linear"


def test_apply_fp8_linear_through_the_patched_name(env, dev):
    """fp8.apply_fp8_linear with dynamic per-token scales and with a static per-tensor input scale."""
    g = torch.Generator().manual_seed(6)
    x = torch.randn(29, 1024, generator=g).to(torch.bfloat16)
    w = torch.randn(640, 1024, generator=g) * 0.02
    wq, ws = oq.per_channel_quant_weight(w, "fp8")
    wd, wsd = _fp8(wq, dev).t(), torch.from_numpy(ws).to(dev).view(-1, 1)
    xq, xs = oq.per_token_quant_fp8(x)
    ref = og.fp8_scaled_mm(xq, wq, xs, ws, return_fp32=True)
    for holder in (env.fp8, env.utils):
        out = holder.apply_fp8_linear(x.to(dev), wd, wsd)
        assert out.shape == (29, 640) and out.dtype == torch.bfloat16
        assert_gemm_close(out, ref, "apply_fp8_linear (dynamic) through the plugin")
    s_in = 0.0151
    xq3, xs3 = oq.static_quant_fp8(x, s_in)
    ref3 = og.fp8_scaled_mm(xq3, wq, xs3, ws, return_fp32=True)
    out3 = env.fp8.apply_fp8_linear(x.to(dev), wd, wsd, input_scale=torch.tensor([s_in], device=dev))
    assert_gemm_close(out3, ref3, "apply_fp8_linear (static input scale) through the plugin")
    # a static scale per token is not built: the stand-in's original is reached
    assert env.fp8.apply_fp8_linear(x.to(dev), wd, wsd, input_scale=torch.ones(29, device=dev)) == "sglang:apply_fp8_linear"


def test_quant_functions_bound_by_importers_run_on_the_device(env, dev):
    """A REPLACE hook on a name another module bound with `from ... import`: calling it there quantises on the GPU
    with this library's kernel, bit for bit the oracle's bytes."""
    g = torch.Generator().manual_seed(7)
    x = torch.randn(33, 512, generator=g).to(torch.bfloat16)
    for holder, attr in ((env.fp8, "per_token_group_quant_fp8"), (env.other, "quant")):
        q, s = getattr(holder, attr)(x.to(dev), 128)
        rq, rs, _ = oq.group_quant(x, 128, form="divide")
        alt, alt_s, _ = oq.group_quant(x, 128, form="reciprocal")
        got = q.cpu().view(torch.uint8).numpy()
        assert np.array_equal(got, rq) or np.array_equal(got, alt)
        assert np.array_equal(s.cpu().numpy(), rs) or np.array_equal(s.cpu().numpy(), alt_s)


def test_fused_moe_through_the_runner_pool_and_the_patched_impl(env, dev):
    """FusedOpPool's ("none", "triton") function on StandardDispatchOutput / TritonMoeQuantInfo / MoeRunnerConfig,
    and fused_experts_impl through its AROUND hook; an unsupported configuration reaches the original."""
    from sglang_amd.moe_runner import MoeRunnerConfig, StandardDispatchOutput, StandardTopKOutput, TritonMoeQuantInfo

    M, H, I, E, topk = 19, 512, 256, 8, 2
    g = torch.Generator().manual_seed(8)
    x = torch.randn(M, H, generator=g).to(torch.bfloat16)
    w13 = torch.randn(E, 2 * I, H, generator=g) * 0.02
    w2 = torch.randn(E, H, I, generator=g) * 0.02
    q13, s13 = zip(*(oq.block_quant_weight(w13[e]) for e in range(E)))
    q2, s2 = zip(*(oq.block_quant_weight(w2[e]) for e in range(E)))
    q13, s13, q2, s2 = np.stack(q13), np.stack(s13), np.stack(q2), np.stack(s2)
    tw, ti = om.topk_softmax(torch.randn(M, E, generator=g), topk, True)
    ref = om.fused_moe_block_fp8(x, q13, q2, s13, s2, tw, ti, quant_form="reciprocal")

    fused = env.FusedOpPool._fused_funcs[("none", "triton")]
    assert getattr(fused, "_sglang_amd", False)
    topk_out = StandardTopKOutput(tw.to(dev), ti.to(dev), None)
    info = TritonMoeQuantInfo(w13_weight=_fp8(q13, dev), w2_weight=_fp8(q2, dev), use_fp8_w8a8=True,
                              w13_scale=torch.from_numpy(s13).to(dev), w2_scale=torch.from_numpy(s2).to(dev),
                              block_shape=[128, 128])
    combine = fused(StandardDispatchOutput(x.to(dev), None, topk_out), info, MoeRunnerConfig(inplace=False))
    assert combine.hidden_states.shape == (M, H)
    assert_gemm_close(combine.hidden_states, ref.float(), "runner pool")
    # in place, with the routed scaling factor of the runner configuration
    xin = x.to(dev).clone()
    combine = fused(StandardDispatchOutput(xin, None, topk_out), info,
                    MoeRunnerConfig(inplace=True, routed_scaling_factor=2.5))
    assert combine.hidden_states.data_ptr() == xin.data_ptr()
    ref25 = om.fused_moe_block_fp8(x, q13, q2, s13, s2, tw, ti, quant_form="reciprocal", routed_scaling_factor=2.5)
    assert_gemm_close(xin, ref25.float(), "runner pool, in place")
    # a 16-bit (unquantised) MoE is not this library's: the pool's previous entry answers
    plain = TritonMoeQuantInfo(w13_weight=torch.zeros(E, 2 * I, H, device=dev, dtype=torch.bfloat16),
                               w2_weight=torch.zeros(E, H, I, device=dev, dtype=torch.bfloat16))
    assert fused(StandardDispatchOutput(x.to(dev), None, topk_out), plain, MoeRunnerConfig(inplace=False)) == \
        "sglang:fused_experts_none_to_triton"

    fm = sys.modules["sglang.srt.layers.moe.moe_runner.triton_utils.fused_moe"]
    out = fm.fused_experts_impl(x.to(dev), _fp8(q13, dev), _fp8(q2, dev), tw.to(dev), ti.to(dev), use_fp8_w8a8=True,
                                w1_scale=torch.from_numpy(s13).to(dev), w2_scale=torch.from_numpy(s2).to(dev),
                                block_shape=[128, 128])
    assert_gemm_close(out, ref.float(), "fused_experts_impl through its hook")
    assert fm.fused_experts_impl(x.to(dev), plain.w13_weight, plain.w2_weight, tw.to(dev), ti.to(dev)) == \
        "sglang:fused_experts_impl"

"""GPU parity of the configurations beyond block [128, 128]: scale blocks of 64 in either direction (dense block
GEMM and fused MoE; the reference's own fused-MoE test sweeps [[64,64],[64,128],[128,64],[128,128]],
test/manual/quant/test_block_fp8.py:557), per-channel and per-tensor scaled fused MoE with biases, and the sigmoid
router.  Everything is compared with the CPU oracle under the north-star tolerances."""
import numpy as np
import pytest
import torch

from oracle import gemm as og
from oracle import moe as om
from oracle import quant as oq
from tests.util import assert_gemm_close, codes

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def sa(dev):
    import sglang_amd

    return sglang_amd


def _fp8(a: np.ndarray, dev):
    return torch.from_numpy(a).to(dev).view(torch.float8_e4m3fn)


BLOCKS = [[64, 64], [64, 128], [128, 64]]


@pytest.mark.parametrize("block", BLOCKS)
@pytest.mark.parametrize("M,N,K", [(1, 256, 512), (33, 576, 1024), (130, 1000, 1088), (7, 192, 192), (300, 384, 7168)])
def test_block_fp8_matmul_other_block_shapes(sa, dev, block, M, N, K):
    """w8a8_block_fp8_matmul with a general block_size against native_w8a8_block_fp8_matmul's restatement; ragged N
    and K (K % 16 == 0) included."""
    from sglang_amd.quantization.fp8_kernel import w8a8_block_fp8_matmul

    bn, bk = block
    g = torch.Generator().manual_seed(M + N + K + bn * 3 + bk)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = torch.randn(N, K, generator=g) * 0.02
    if K % bk == 0:
        xq, xs, _ = oq.group_quant(x, bk)
    else:
        xq = codes(((torch.rand(M, K, generator=g) - 0.5) * 2 * 448).to(torch.float8_e4m3fn))
        xs = (torch.rand(M, -(-K // bk), generator=g) * 1e-2 + 1e-3).numpy()
    wq, ws = oq.block_quant_weight(w, block=(bn, bk))
    ref = og.block_fp8_matmul(xq, wq, xs, ws, block=(bn, bk), return_fp32=True)
    out = w8a8_block_fp8_matmul(_fp8(xq, dev), _fp8(wq, dev), torch.from_numpy(xs).to(dev),
                                torch.from_numpy(ws).to(dev), block, torch.bfloat16)
    assert out.shape == (M, N) and out.dtype == torch.bfloat16
    assert_gemm_close(out, ref, f"M={M} N={N} K={K} block={block}")


@pytest.mark.parametrize("block", BLOCKS)
def test_block_int8_matmul_other_block_shapes(sa, dev, block):
    from sglang_amd.quantization.int8_kernel import w8a8_block_int8_matmul

    bn, bk = block
    M, N, K = 77, 448, 1152
    g = torch.Generator().manual_seed(bn + 2 * bk)
    a = torch.randint(-127, 128, (M, K), generator=g, dtype=torch.int8)
    b = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8)
    a_s = torch.rand(M, K // bk, generator=g) * 1e-2 + 1e-3
    b_s = torch.rand(-(-N // bn), K // bk, generator=g) * 1e-2 + 1e-3
    ref = og.block_int8_matmul(a.numpy(), b.numpy(), a_s.numpy(), b_s.numpy(), block=(bn, bk), return_fp32=True)
    out = w8a8_block_int8_matmul(a.to(dev), b.to(dev), a_s.to(dev), b_s.to(dev), block, torch.float16)
    assert out.dtype == torch.float16
    assert_gemm_close(out, ref, f"int8 block={block}")


def test_block_linear_with_64_wide_blocks(sa, dev):
    """The linear wrappers route other block shapes to the row-major-scale path."""
    from sglang_amd.quantization.fp8_utils import (
        cutlass_w8a8_block_fp8_linear_with_fallback,
        triton_w8a8_block_fp8_linear,
    )

    g = torch.Generator().manual_seed(17)
    x = torch.randn(2, 5, 512, generator=g).to(torch.bfloat16)
    w = torch.randn(320, 512, generator=g) * 0.02
    wq, ws = oq.block_quant_weight(w, block=(64, 64))
    xq, xs, _ = oq.group_quant(x.view(-1, 512), 64, form="reciprocal")
    ref = og.block_fp8_matmul(xq, wq, xs, ws, block=(64, 64), return_fp32=True).view(2, 5, 320)
    for fn in (cutlass_w8a8_block_fp8_linear_with_fallback, triton_w8a8_block_fp8_linear):
        out = fn(x.to(dev), _fp8(wq, dev), [64, 64], torch.from_numpy(ws).to(dev))
        assert_gemm_close(out, ref, fn.__name__)


def _moe_weights(E, I, H, g, dst, block=None, gated=True):
    w13 = torch.randn(E, (2 if gated else 1) * I, H, generator=g) * 0.02
    w2 = torch.randn(E, H, I, generator=g) * 0.02
    if block is not None:
        q13, s13 = zip(*(oq.block_quant_weight(w13[e], block=block, dst=dst) for e in range(E)))
        q2, s2 = zip(*(oq.block_quant_weight(w2[e], block=block, dst=dst) for e in range(E)))
    else:
        q13, s13 = zip(*(oq.per_channel_quant_weight(w13[e], dst) for e in range(E)))
        q2, s2 = zip(*(oq.per_channel_quant_weight(w2[e], dst) for e in range(E)))
    return np.stack(q13), np.stack(s13), np.stack(q2), np.stack(s2)


def _dev_w(q, dev, int8):
    return torch.from_numpy(q).to(dev) if int8 else _fp8(q, dev)


@pytest.mark.parametrize("block", BLOCKS)
@pytest.mark.parametrize("int8", [False, True])
@pytest.mark.parametrize("M,H,I,E,topk", [(1, 512, 256, 8, 2), (33, 512, 256, 8, 2), (222, 768, 256, 24, 6)])
def test_fused_moe_other_block_shapes(sa, dev, block, int8, M, H, I, E, topk):
    """test_w8a8_block_fp8_fused_moe's sweep of block shapes (test/manual/quant/test_block_fp8.py:549-620) and its
    int8 twin (test/registered/quant/test_block_int8.py:134-207)."""
    from tests.util import moe_layer as fused_moe

    g = torch.Generator().manual_seed(M + H + E + block[0] + 2 * block[1] + int(int8))
    x = torch.randn(M, H, generator=g).to(torch.bfloat16)
    dst = "int8" if int8 else "fp8"
    q13, s13, q2, s2 = _moe_weights(E, I, H, g, dst, block=tuple(block))
    tw, ti = om.topk_softmax(torch.randn(M, E, generator=g), topk, True)
    ref = om.fused_moe_block_fp8(x, q13, q2, s13, s2, tw, ti, block=tuple(block), quant_form="reciprocal", int8=int8)
    kw = dict(use_int8_w8a8=True) if int8 else dict(use_fp8_w8a8=True)
    out = fused_moe(x.to(dev), _dev_w(q13, dev, int8), _dev_w(q2, dev, int8), (tw.to(dev), ti.to(dev), None),
                    w1_scale=torch.from_numpy(s13).to(dev), w2_scale=torch.from_numpy(s2).to(dev),
                    block_shape=block, **kw)
    assert out.shape == (M, H) and out.dtype == torch.bfloat16
    assert_gemm_close(out, ref.float(), f"M={M} E={E} topk={topk} block={block} int8={int8}")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("name", ["gelu_and_mul", "gelu_tanh_and_mul", "silu_and_mul"])
def test_act_and_mul(sa, dev, name, dtype):
    """The three gated activations (sgl-kernel/tests/test_activation.py: dims 128..16384 with 11008 among them,
    against torch's own functions at rtol = atol = 1e-3), and against the oracle: erf / tanh / exp differ by an ulp
    between libraries, so a few elements may land on the neighbouring 16-bit value."""
    g = torch.Generator().manual_seed(3)
    torch_act = {"gelu_and_mul": lambda t: torch.nn.functional.gelu(t, approximate="none"),
                 "gelu_tanh_and_mul": lambda t: torch.nn.functional.gelu(t, approximate="tanh"),
                 "silu_and_mul": torch.nn.functional.silu}[name]
    for rows, d in ((1, 128), (7, 11008), (33, 4096), (512, 256), (4, 16384)):
        x = (torch.randn(rows, 2 * d, generator=g) * 2).to(dtype)
        out = getattr(sa, name)(x.to(dev)).cpu()
        assert out.shape == (rows, d) and out.dtype == dtype
        ref = getattr(om, name)(x)
        # Allowed distance: the activation is rounded to 16 bits before the multiply, so where the libraries' fp32
        # values straddle a rounding boundary the factor moves by one step and the product by up to |u| times that
        # (two steps of the product) before its own rounding adds one; plus what an ulp of erf / tanh / exp near
        # -1 does to 1 + f(x) in the negative tail, where the reference's formula cancels (absolute error of the
        # fp32 activation <= ~2e-7 |x|, times |u|): there the result depends on the math library, not the kernel.
        step = 3 * ref.float().abs() * 2.0 ** (-10 if dtype == torch.float16 else -7) + 6e-8
        diff = (out.float() - ref.float()).abs()
        slack = 4e-7 * (x[..., :d].float() * x[..., d:].float()).abs()
        assert bool((diff <= step + slack).all()), (name, rows, d, float((diff - step - slack).max()))
        assert float((diff > 0).float().mean()) < 2e-2, (name, rows, d)
        if dtype == torch.float16:
            torch.testing.assert_close(out, x[..., d:] * torch_act(x[..., :d]), rtol=1e-3, atol=1e-3)
    out = torch.empty(5, 64, dtype=dtype, device=dev)
    assert getattr(sa, name)(torch.zeros(5, 128, dtype=dtype, device=dev), out) is out and not out.any()
    with pytest.raises(ValueError):
        getattr(sa, name)(torch.zeros(2, 12, dtype=dtype, device=dev))


@pytest.mark.parametrize("activation,is_gated", [("gelu", True), ("silu", False), ("gelu", False), ("relu2", False)])
@pytest.mark.parametrize("form", ["block_fp8", "block_int8", "channel_fp8", "channel_int8"])
def test_fused_moe_other_activations(sa, dev, form, activation, is_gated):
    """The activations fused_experts_impl accepts besides gated SiLU
    (python/sglang/srt/layers/moe/moe_runner/triton_utils/fused_moe.py:530-647): gated GELU through gelu_and_mul,
    and the layers that are not gated (w13 is [E, I, H]) with SiLU, GELU or squared ReLU on the whole row."""
    from tests.util import moe_layer as fused_moe

    M, H, I, E, topk = 70, 512, 256, 8, 2
    int8 = form.endswith("int8")
    block = (128, 128) if form.startswith("block") else None
    g = torch.Generator().manual_seed(len(form) + 3 * len(activation) + int(is_gated))
    x = torch.randn(M, H, generator=g).to(torch.bfloat16)
    q13, s13, q2, s2 = _moe_weights(E, I, H, g, "int8" if int8 else "fp8", block=block, gated=is_gated)
    tw, ti = om.topk_softmax(torch.randn(M, E, generator=g), topk, True)
    if block is not None:
        ref = om.fused_moe_block_fp8(x, q13, q2, s13, s2, tw, ti, quant_form="reciprocal", int8=int8,
                                     activation=activation, is_gated=is_gated)
        kw = dict(block_shape=list(block))
    else:
        ref = om.fused_moe_row_scaled(x, q13, q2, s13, s2, tw, ti, int8=int8, activation=activation, is_gated=is_gated)
        kw = dict(per_channel_quant=True)
    kw.update(dict(use_int8_w8a8=True) if int8 else dict(use_fp8_w8a8=True))
    out = fused_moe(x.to(dev), _dev_w(q13, dev, int8), _dev_w(q2, dev, int8), (tw.to(dev), ti.to(dev), None),
                    w1_scale=torch.from_numpy(s13).to(dev), w2_scale=torch.from_numpy(s2).to(dev),
                    activation=activation, is_gated=is_gated, **kw)
    assert out.shape == (M, H)
    assert_gemm_close(out, ref.float(), f"{form} {activation} gated={is_gated}")
    with pytest.raises(ValueError):
        fused_moe(x.to(dev), _dev_w(q13, dev, int8), _dev_w(q2, dev, int8), (tw.to(dev), ti.to(dev), None),
                  w1_scale=torch.from_numpy(s13).to(dev), w2_scale=torch.from_numpy(s2).to(dev),
                  activation="relu2", is_gated=True, **kw)


@pytest.mark.parametrize("act_kw", [dict(gemm1_limit=1.5), dict(gemm1_alpha=1.702, gemm1_limit=1.5),
                                    dict(swiglu_limit=10)])
@pytest.mark.parametrize("int8", [False, True])
def test_fused_moe_clamped_swiglu(sa, dev, int8, act_kw):
    """The clamped gated-SiLU variants between the two GEMMs (fused_moe.py:315-331,530-580) through
    fused_experts_impl, block-scaled FP8 and INT8; the weights are large enough for the limits of 1.5 to cut
    (swiglu_limit is fixed at 10 by the reference, so that case checks the unclamped range)."""
    from sglang_amd.moe_runner import fused_experts_impl

    M, H, I, E, topk = 50, 512, 256, 8, 2
    g = torch.Generator().manual_seed(31 + int(int8) + len(act_kw))
    x = torch.randn(M, H, generator=g).to(torch.bfloat16)
    w13 = torch.randn(E, 2 * I, H, generator=g) * 0.06
    w2 = torch.randn(E, H, I, generator=g) * 0.02
    dst = "int8" if int8 else "fp8"
    q13, s13 = zip(*(oq.block_quant_weight(w13[e], dst=dst) for e in range(E)))
    q2, s2 = zip(*(oq.block_quant_weight(w2[e], dst=dst) for e in range(E)))
    q13, s13, q2, s2 = np.stack(q13), np.stack(s13), np.stack(q2), np.stack(s2)
    tw, ti = om.topk_softmax(torch.randn(M, E, generator=g), topk, True)
    ref = om.fused_moe_block_fp8(x, q13, q2, s13, s2, tw, ti, quant_form="reciprocal", int8=int8, **act_kw)
    plain = om.fused_moe_block_fp8(x, q13, q2, s13, s2, tw, ti, quant_form="reciprocal", int8=int8)
    if "gemm1_limit" in act_kw:
        assert (ref.float() - plain.float()).abs().max() > 0.05 * plain.float().abs().max(), "the limit must cut"
    kw = dict(use_int8_w8a8=True) if int8 else dict(use_fp8_w8a8=True)
    out = fused_experts_impl(x.to(dev), _dev_w(q13, dev, int8), _dev_w(q2, dev, int8), tw.to(dev), ti.to(dev),
                             w1_scale=torch.from_numpy(s13).to(dev), w2_scale=torch.from_numpy(s2).to(dev),
                             block_shape=[128, 128], **kw, **act_kw)
    assert_gemm_close(out, ref.float(), f"clamped swiglu {act_kw} int8={int8}")


@pytest.mark.parametrize("int8", [False, True])
@pytest.mark.parametrize("bias", [False, True])
@pytest.mark.parametrize("M,H,I,E,topk", [(1, 512, 256, 8, 2), (40, 512, 384, 8, 2), (200, 1024, 256, 16, 4)])
def test_fused_moe_per_channel(sa, dev, int8, bias, M, H, I, E, topk):
    """per_channel_quant: per-token activation scales, per-channel weight scales
    (fused_moe_triton_kernels.py:504-513,586-589; model test/registered/quant/test_int8_kernel.py:39-79)."""
    from tests.util import moe_layer as fused_moe

    g = torch.Generator().manual_seed(M + H + E + 5 * int(int8) + 11 * int(bias))
    x = torch.randn(M, H, generator=g).to(torch.bfloat16)
    dst = "int8" if int8 else "fp8"
    q13, s13, q2, s2 = _moe_weights(E, I, H, g, dst)
    b1 = (torch.randn(E, 2 * I, generator=g) * 0.1).to(torch.bfloat16) if bias else None
    b2 = (torch.randn(E, H, generator=g) * 0.1).to(torch.bfloat16) if bias else None
    tw, ti = om.topk_softmax(torch.randn(M, E, generator=g), topk, True)
    ref = om.fused_moe_row_scaled(x, q13, q2, s13, s2, tw, ti, int8=int8, b1=b1, b2=b2)
    kw = dict(use_int8_w8a8=True) if int8 else dict(use_fp8_w8a8=True)
    out = fused_moe(x.to(dev), _dev_w(q13, dev, int8), _dev_w(q2, dev, int8), (tw.to(dev), ti.to(dev), None),
                    b1=None if b1 is None else b1.to(dev), b2=None if b2 is None else b2.to(dev),
                    w1_scale=torch.from_numpy(s13).to(dev), w2_scale=torch.from_numpy(s2).to(dev),
                    per_channel_quant=True, **kw)
    assert out.shape == (M, H)
    assert_gemm_close(out, ref.float(), f"per-channel M={M} E={E} int8={int8} bias={bias}")


def test_fused_moe_per_tensor_static_scales_and_router_weight_on_input(sa, dev):
    """FP8 with one static activation scale per GEMM and one weight scale per expert
    (fused_moe_triton_kernels.py:514-516,737-746); apply_router_weight_on_input with top-1 routing multiplies the
    first GEMM's result instead of the second's."""
    from tests.util import moe_layer as fused_moe

    M, H, I, E = 37, 512, 256, 8
    g = torch.Generator().manual_seed(99)
    x = torch.randn(M, H, generator=g).to(torch.bfloat16)
    w13 = torch.randn(E, 2 * I, H, generator=g) * 0.02
    w2 = torch.randn(E, H, I, generator=g) * 0.02
    s13 = (w13.abs().amax(dim=(1, 2)) / 448.0).numpy().astype(np.float32)
    s2 = (w2.abs().amax(dim=(1, 2)) / 448.0).numpy().astype(np.float32)
    q13 = np.stack([oq.static_quant_fp8(w13[e], float(s13[e]))[0] for e in range(E)])
    q2 = np.stack([oq.static_quant_fp8(w2[e], float(s2[e]))[0] for e in range(E)])
    a1, a2 = 0.011, 0.0007
    for topk, on_input in ((2, False), (1, True)):
        tw, ti = om.topk_softmax(torch.randn(M, E, generator=g), topk, False)
        ref = om.fused_moe_row_scaled(x, q13, q2, s13, s2, tw, ti, a1_scale=a1, a2_scale=a2,
                                      apply_router_weight_on_input=on_input)
        from sglang_amd.moe_runner import MoeRunnerConfig, fused_moe as layer

        cfg = MoeRunnerConfig(inplace=False, apply_router_weight_on_input=on_input)
        out = layer(x.to(dev), _fp8(q13, dev), _fp8(q2, dev), (tw.to(dev), ti.to(dev), None), cfg, use_fp8_w8a8=True,
                    w1_scale=torch.from_numpy(s13).to(dev), w2_scale=torch.from_numpy(s2).to(dev),
                    a1_scale=torch.tensor(a1, device=dev), a2_scale=torch.tensor(a2, device=dev))
        assert_gemm_close(out, ref.float(), f"per-tensor static topk={topk} on_input={on_input}")
    # a static activation scale wins over per-token quantisation also when the weights are scaled per channel
    # (scaled_fp8_quant(A, A_scale, use_per_token_if_dynamic=per_channel_quant), fused_moe_triton_kernels.py:748-751)
    q13c, s13c, q2c, s2c = _moe_weights(E, I, H, g, "fp8")
    tw, ti = om.topk_softmax(torch.randn(M, E, generator=g), 2, True)
    ref = om.fused_moe_row_scaled(x, q13c, q2c, s13c, s2c, tw, ti, a1_scale=a1, a2_scale=a2)
    out = fused_moe(x.to(dev), _fp8(q13c, dev), _fp8(q2c, dev), (tw.to(dev), ti.to(dev), None), use_fp8_w8a8=True,
                    per_channel_quant=True, w1_scale=torch.from_numpy(s13c).to(dev),
                    w2_scale=torch.from_numpy(s2c).to(dev), a1_scale=torch.tensor(a1, device=dev),
                    a2_scale=torch.tensor(a2, device=dev))
    assert_gemm_close(out, ref.float(), "static activation scales with per-channel weights")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_scaled_fp8_quant(sa, dev, dtype):
    """scaled_fp8_quant like the reference's own tests drive it (test/manual/quant/test_custom_ops.py:20-140):
    dynamic per tensor, static, dynamic per token, and row padding; bytes and scales bit-exact against the oracle."""
    from sglang_amd.quantization.fp8_kernel import scaled_fp8_quant

    g = torch.Generator().manual_seed(3)
    for shape in ((11, 16), (257, 1024), (4096, 512)):
        x = (torch.randn(*shape, generator=g) * 13).to(dtype)
        y, scale = scaled_fp8_quant(x.to(dev), None)
        rq, rs = oq.dynamic_per_tensor_quant_fp8(x)
        assert scale.shape == (1,) and np.array_equal(scale.cpu().numpy(), rs)
        assert np.array_equal(codes(y), rq)
        y2, s2 = scaled_fp8_quant(x.to(dev), scale)              # static with the same scale: the same bytes
        assert np.array_equal(codes(y2), rq) and s2 is scale
        y3, s3 = scaled_fp8_quant(x.to(dev), None, use_per_token_if_dynamic=True)
        rq3, rs3 = oq.per_token_quant_fp8(x)
        assert s3.shape == (shape[0], 1) and np.array_equal(s3.cpu().numpy().reshape(-1), rs3)
        assert np.array_equal(codes(y3), rq3)
        y4, s4 = scaled_fp8_quant(x.to(dev), None, num_token_padding=shape[0] + 5)
        assert y4.shape == (shape[0] + 5, shape[1]) and np.array_equal(codes(y4[:shape[0]]), rq)
    z, zs = scaled_fp8_quant(torch.zeros(8, 64, device=dev, dtype=dtype), None)
    assert float(zs) > 0 and not codes(z).any()


def test_fused_moe_dynamic_per_tensor_scales(sa, dev):
    """FP8 'tensor-wise' MoE without static scales: each GEMM's input is quantised with max|A| / 448
    (fused_moe_triton_kernels.py:737-746 with A_scale None and per_channel_quant False)."""
    from tests.util import moe_layer as fused_moe

    M, H, I, E, topk = 29, 512, 256, 8, 2
    g = torch.Generator().manual_seed(101)
    x = torch.randn(M, H, generator=g).to(torch.bfloat16)
    w13 = torch.randn(E, 2 * I, H, generator=g) * 0.02
    w2 = torch.randn(E, H, I, generator=g) * 0.02
    s13 = (w13.abs().amax(dim=(1, 2)) / 448.0).numpy().astype(np.float32)
    s2 = (w2.abs().amax(dim=(1, 2)) / 448.0).numpy().astype(np.float32)
    q13 = np.stack([oq.static_quant_fp8(w13[e], float(s13[e]))[0] for e in range(E)])
    q2 = np.stack([oq.static_quant_fp8(w2[e], float(s2[e]))[0] for e in range(E)])
    tw, ti = om.topk_softmax(torch.randn(M, E, generator=g), topk, True)
    ref = om.fused_moe_row_scaled(x, q13, q2, s13, s2, tw, ti, per_tensor_dynamic=True)
    out = fused_moe(x.to(dev), _fp8(q13, dev), _fp8(q2, dev), (tw.to(dev), ti.to(dev), None), use_fp8_w8a8=True,
                    w1_scale=torch.from_numpy(s13).to(dev), w2_scale=torch.from_numpy(s2).to(dev))
    assert_gemm_close(out, ref.float(), "dynamic per-tensor MoE")


@pytest.mark.parametrize("num_tokens", [1, 16, 512, 2048])
@pytest.mark.parametrize("num_experts", [4, 8, 64, 128, 256, 384])
@pytest.mark.parametrize("topk", [1, 2, 4, 8])
def test_topk_sigmoid(sa, dev, num_tokens, num_experts, topk):
    """The sweep of sgl-kernel/tests/test_moe_topk_sigmoid.py:23-58 (plus a non-power-of-two expert count and
    top-8): ids equal to the oracle's, weights to fp32 rounding; with bias and renormalisation as well."""
    if topk > num_experts:
        pytest.skip("topk > experts")
    g = torch.Generator().manual_seed(num_tokens * 1000 + num_experts + topk)
    for dtype in (torch.float32, torch.bfloat16, torch.float16):
        logits = torch.randn(num_tokens, num_experts, generator=g).to(dtype)
        for bias, renorm in ((None, False), (torch.randn(num_experts, generator=g) * 0.1, True)):
            w = torch.empty(num_tokens, topk, device=dev, dtype=torch.float32)
            ids = torch.empty(num_tokens, topk, device=dev, dtype=torch.int32)
            sa.topk_sigmoid(w, ids, logits.to(dev), renorm, None if bias is None else bias.to(dev))
            rw, rids = om.topk_sigmoid(logits, topk, renorm, bias)
            same = ids.cpu() == rids
            # an expf that differs by an ulp between libraries can swap two near-tied experts: such rows must
            # still carry the same weights to rounding
            assert same.float().mean() > 0.999, f"ids differ in {(~same).sum()} places"
            torch.testing.assert_close(w.cpu(), rw, rtol=1e-5, atol=1e-6)


def test_topk_sigmoid_argument_checks(sa, dev):
    w = torch.empty(4, 2, device=dev)
    ids = torch.empty(4, 2, device=dev, dtype=torch.int32)
    with pytest.raises(RuntimeError, match="correction_bias must be float32"):
        sa.topk_sigmoid(w, ids, torch.zeros(4, 8, device=dev), False, torch.zeros(8, device=dev, dtype=torch.bfloat16))
    with pytest.raises(RuntimeError, match="topk must be less than or equal to num_experts"):
        sa.topk_sigmoid(torch.empty(4, 9, device=dev), torch.empty(4, 9, device=dev, dtype=torch.int32),
                        torch.zeros(4, 8, device=dev), False, None)

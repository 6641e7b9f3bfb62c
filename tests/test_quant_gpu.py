"""GPU parity of the quantisation operators against the CPU oracle: bytes and scales
bit-exact, called through torch.ops.sgl_kernel (which goes through the C ABI)."""
import numpy as np
import pytest
import torch

from oracle import quant as oq
from oracle.fp8 import e4m3fn_decode
from tests.util import codes, outlier_input

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def sa(dev):
    import sglang_amd

    return sglang_amd


def _special_rows(hidden, dtype):
    """Rows that exercise edges: all zero, one tiny value, huge values, exact ties, negatives only."""
    rows = torch.zeros(8, hidden, dtype=torch.float32)
    rows[1, 3] = 1e-12
    rows[2] = 3.0e38 if dtype == torch.bfloat16 else 60000.0
    rows[2, ::2] *= -1
    rows[3] = torch.linspace(-1, 1, hidden)
    rows[4, :] = -0.5
    rows[5] = torch.arange(hidden) % 17 - 8  # small integers: exact ties after scaling
    rows[6, 0] = 448.0
    rows[6, 1:] = torch.arange(hidden - 1) % 449
    rows[7] = torch.randn(hidden, generator=torch.Generator().manual_seed(7)) * 1e-6
    return rows.to(dtype)


@pytest.mark.parametrize("form", ["divide", "reciprocal"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows,hidden,group", [(1, 7168, 128), (16, 7168, 128), (33, 512, 128), (256, 7168, 128),
                                                (7, 1536, 64), (5, 256, 32), (3, 128, 16), (127, 2048, 128)])
def test_group_quant_row_major_fp8(sa, dev, form, dtype, rows, hidden, group):
    x = torch.cat([outlier_input(rows, hidden, dtype, 50.0), _special_rows(hidden, dtype)])
    xd = x.to(dev)
    q = torch.empty_like(xd, dtype=torch.float8_e4m3fn)
    s = torch.empty(x.shape[0], hidden // group, device=dev, dtype=torch.float32)
    sa.sgl_per_token_group_quant_8bit(xd, q, s, group, 1e-10, -448.0, 448.0, False, enable_v2=(form == "reciprocal"))
    rq, rs, _ = oq.group_quant(x, group, form=form)
    assert np.array_equal(s.cpu().numpy().view(np.uint32), rs.view(np.uint32)), "scales differ"
    assert np.array_equal(codes(q), rq), "fp8 bytes differ"


@pytest.mark.parametrize("form", ["divide", "reciprocal"])
@pytest.mark.parametrize("rows,hidden", [(1, 7168), (6, 7168), (16, 7168), (37, 640), (256, 7168), (9, 1536)])
def test_group_quant_column_major_layouts(sa, dev, form, rows, hidden):
    from sglang_amd.quantization.fp8_kernel import create_per_token_group_quant_fp8_output_scale as mk

    x = outlier_input(rows, hidden, torch.bfloat16, 50.0)
    xd = x.to(dev)
    g = hidden // 128
    v2 = form == "reciprocal"
    rq, rs, _ = oq.group_quant(x, 128, form=form)
    for aligned in (False, True):
        q = torch.empty_like(xd, dtype=torch.float8_e4m3fn)
        s = mk(xd.shape, dev, 128, True, aligned, False)
        assert s.shape == (rows, g) and s.stride(0) == 1
        sa.sgl_per_token_group_quant_8bit(xd, q, s, 128, 1e-10, -448.0, 448.0, False, enable_v2=v2)
        assert np.array_equal(s.cpu().numpy().view(np.uint32), rs.view(np.uint32))
        assert np.array_equal(codes(q), rq)
    # UE8M0 packed
    rq8, rs8, re8 = oq.group_quant(x, 128, form=form, scale_ue8m0=True)
    q = torch.empty_like(xd, dtype=torch.float8_e4m3fn)
    s = mk(xd.shape, dev, 128, True, True, True)
    s.fill_(-1)  # tail bytes must be overwritten with zeros by the kernel
    sa.sgl_per_token_group_quant_8bit(xd, q, s, 128, 1e-10, -448.0, 448.0, True, enable_v2=v2)
    assert np.array_equal(s.cpu().numpy(), oq.pack_ue8m0(re8))
    assert np.array_equal(codes(q), rq8)


@pytest.mark.parametrize("form", ["divide", "reciprocal"])
def test_group_quant_int8(sa, dev, form):
    x = outlier_input(19, 1024, torch.bfloat16, 50.0)
    xd = x.to(dev)
    q = torch.empty_like(xd, dtype=torch.int8)
    s = torch.empty(19, 8, device=dev, dtype=torch.float32)
    sa.sgl_per_token_group_quant_8bit(xd, q, s, 128, 1e-10, -128.0, 127.0, False, enable_v2=(form == "reciprocal"))
    rq, rs, _ = oq.group_quant(x, 128, form=form, dst="int8")
    assert np.array_equal(s.cpu().numpy().view(np.uint32), rs.view(np.uint32))
    assert np.array_equal(codes(q), rq)


def test_group_quant_divide_generic_group_and_fp32(sa, dev):
    x = outlier_input(11, 1152, torch.float32, 50.0)
    xd = x.to(dev)
    for group in (128, 384, 1152, 48):
        q = torch.empty_like(xd, dtype=torch.float8_e4m3fn)
        s = torch.empty(11, 1152 // group, device=dev, dtype=torch.float32)
        sa.sgl_per_token_group_quant_8bit(xd, q, s, group, 1e-10, -448.0, 448.0, False, enable_v2=False)
        rq, rs, _ = oq.group_quant(x, group, form="divide")
        assert np.array_equal(s.cpu().numpy().view(np.uint32), rs.view(np.uint32)), group
        assert np.array_equal(codes(q), rq), group


def test_group_quant_exhaustive_bf16_values(sa, dev):
    """Every finite bf16 bit pattern goes through the divide and the reciprocal form in groups
    whose maximum is pinned, so the fp32 divide, the clamp and the e4m3 rounding are all hit."""
    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16)
    v = bits.view(torch.bfloat16)
    v = v[torch.isfinite(v.float())]
    n = v.numel() // 127 * 127
    body = v[:n].view(-1, 127)
    for amax in (448.0, 1.0, 3.3895e38, 1e-3, 77.0):
        lead = torch.full((body.shape[0], 1), amax, dtype=torch.bfloat16)
        x = torch.cat([lead, body], dim=1).contiguous()
        x = torch.where(x.float().abs() <= lead.float(), x, torch.zeros_like(x))
        x[:, 0] = lead[:, 0]
        xd = x.to(dev)
        for form in ("divide", "reciprocal"):
            q = torch.empty_like(xd, dtype=torch.float8_e4m3fn)
            s = torch.empty(x.shape[0], 1, device=dev, dtype=torch.float32)
            sa.sgl_per_token_group_quant_8bit(xd, q, s, 128, 1e-10, -448.0, 448.0, False,
                                              enable_v2=(form == "reciprocal"))
            rq, rs, _ = oq.group_quant(x, 128, form=form)
            assert np.array_equal(s.cpu().numpy().view(np.uint32), rs.view(np.uint32)), (amax, form)
            assert np.array_equal(codes(q), rq), (amax, form)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("rows,hidden,scale", [(1, 8192, 0.0371), (64, 8192, 0.5), (128, 1080, 0.0123), (3, 1096, 0.3), (3, 28672, 2.0),
                                                (4096, 7168, 0.0089)])
def test_static_quant_fp8(sa, dev, dtype, rows, hidden, scale):
    """Static per-tensor quantisation (fp8_kernel.py:724-777): bytes bit-exact, the scale repeated once per row."""
    from sglang_amd.quantization.fp8_kernel import static_quant_fp8

    x = outlier_input(rows, hidden, dtype, 50.0)
    s = torch.tensor([scale], dtype=torch.float32, device=dev)
    q, rep = static_quant_fp8(x.to(dev), s, repeat_scale=True)
    rq, rs = oq.static_quant_fp8(x, scale)
    assert q.shape == x.shape and q.dtype == torch.float8_e4m3fn and rep.shape == (rows, 1)
    assert np.array_equal(codes(q), rq)
    assert np.array_equal(rep.cpu().numpy().reshape(-1).view(np.uint32), rs.view(np.uint32))
    q2, same = static_quant_fp8(x.to(dev), s)
    assert same is s and torch.equal(q2.view(torch.uint8), q.view(torch.uint8))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("rows,hidden", [(1, 8192), (64, 8192), (128, 1076), (256, 1368), (3, 28672), (512, 512)])
def test_per_token_quant_fp8(sa, dev, dtype, rows, hidden):
    x = outlier_input(rows, hidden, dtype, 50.0)
    x[0] = 0  # all-zero row: scale 0, zero bytes
    from sglang_amd.quantization.fp8_kernel import sglang_per_token_quant_fp8

    q, s = sglang_per_token_quant_fp8(x.to(dev))
    rq, rs = oq.per_token_quant_fp8(x)
    assert s.shape == (rows, 1)
    assert np.array_equal(s.cpu().numpy().reshape(-1).view(np.uint32), rs.view(np.uint32))
    assert np.array_equal(codes(q), rq)


@pytest.mark.parametrize("rows,hidden", [(1, 8192), (64, 8192), (33, 1000), (5, 28672), (7, 77)])
def test_per_token_quant_int8(sa, dev, rows, hidden):
    from sglang_amd.quantization.int8_kernel import per_token_quant_int8

    x = outlier_input(rows, hidden, torch.bfloat16, 50.0)
    q, s = per_token_quant_int8(x.to(dev))
    rq, rs = oq.per_token_quant_int8(x)
    assert np.array_equal(s.cpu().numpy().reshape(-1).view(np.uint32), rs.view(np.uint32))
    assert np.array_equal(codes(q), rq)


def test_quant_error_paths(sa, dev):
    x = torch.randn(4, 256, device=dev, dtype=torch.bfloat16)
    q = torch.empty_like(x, dtype=torch.float8_e4m3fn)
    s = torch.empty(4, 2, device=dev, dtype=torch.float32)
    with pytest.raises(RuntimeError):
        torch.ops.sgl_kernel.sgl_per_token_group_quant_8bit_v2(x, q, s, 128, 1e-6, -448.0, 448.0, False, False, None)
    with pytest.raises(RuntimeError):
        torch.ops.sgl_kernel.sgl_per_token_group_quant_8bit_v2(x, q, s, 48, 1e-10, -448.0, 448.0, False, False, None)
    with pytest.raises(RuntimeError):
        torch.ops.sgl_kernel.sgl_per_token_group_quant_8bit(x.t(), q, s, 128, 1e-10, -448.0, 448.0, False)
    with pytest.raises(RuntimeError):
        torch.ops.sgl_kernel.sgl_per_token_group_quant_8bit_v2(x, q, s, 128, 1e-10, -224.0, 224.0, False, False, None)
    with pytest.raises(RuntimeError):
        torch.ops.sgl_kernel.sgl_per_token_quant_fp8(torch.randn(2, 6, device=dev), q[:2, :6].contiguous(), s[:2, :1].contiguous())


# ---- fused RMSNorm + group quant -------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,N1,N2", [(32, 128, 7168), (128, 7168, 7168), (5, 1536, 512), (3, 200, 0), (1, 16384, 8)])
@pytest.mark.parametrize("with_res,w_dtype", [(True, torch.float32), (False, None)])
def test_fused_rms_fp8_group_quant(sa, dev, dtype, M, N1, N2, with_res, w_dtype):
    """Shapes of test/registered/quant/test_fused_rms_fp8_group_quant.py:72-75 and more (strided views, a last
    group that is not full, weights in the activation dtype).  Floating-point tolerances, because the sum of
    squares is reduced in a different order than the oracle's: unquantised outputs within one ulp of the storage
    dtype, scales to 1e-5 relative, dequantised values within one fp8 step of the oracle's y (and equal to the
    oracle's codes almost everywhere)."""
    from sglang_amd.quantization.fused_fp8_quant import fused_rms_fp8_group_quant

    g = torch.Generator().manual_seed(M + N1 + N2)
    w_dtype = w_dtype or dtype
    wide = torch.randn(M, N1 + N2 + 64, generator=g).to(dtype) / 10
    x1 = wide[:, :N1]                  # row-strided views, as the q / k_nope slices of a fused projection are
    x2 = wide[:, N1 + 64:] if N2 else None
    res = (torch.randn(M, N1, generator=g) / 10).to(dtype) if with_res else None
    w1 = (torch.rand(N1, generator=g) + 0.5).to(w_dtype)
    w2 = (torch.rand(N2, generator=g) + 0.5).to(w_dtype) if N2 else None
    ref = oq.fused_rms_group_quant(x1, w1, 1e-6, res1=res, x2=x2, w2=w2, eps2=1e-5)

    d = lambda t: t.to(dev) if t is not None else None
    wide_d = wide.to(dev)
    (q, s), y1, y2, res_out = fused_rms_fp8_group_quant(
        wide_d[:, :N1], d(w1), 1e-6, wide_d[:, N1 + 64:] if N2 else None, d(w2), 1e-5 if N2 else None,
        group_size=128, dtype_quant=torch.float8_e4m3fn, res1=d(res), output_unquantized_inp1=True)
    assert q.shape == (M, N1) and q.dtype == torch.float8_e4m3fn and s.shape == (M, -(-N1 // 128))
    ulp = 2.0 ** (-7 if dtype == torch.bfloat16 else -10)

    def close_in_dtype(got, want_f32):
        want = torch.from_numpy(want_f32)
        err = (got.cpu().float() - want).abs()
        assert bool((err <= want.abs() * ulp + 1e-6).all())

    close_in_dtype(y1, ref["y1"])
    if N2:
        close_in_dtype(y2, ref["y2"])
    else:
        assert y2 is None
    if with_res:
        assert torch.equal(res_out.cpu(), torch.from_numpy(ref["res"]).to(dtype))
    else:
        assert res_out is None
    assert np.allclose(s.cpu().numpy(), ref["s"], rtol=1e-5)
    step = np.repeat(ref["s"], 128, axis=1)[:, :N1] * 32.0  # widest e4m3 spacing (256..448) times the scale
    deq = e4m3fn_decode(codes(q)) * np.repeat(s.cpu().numpy(), 128, axis=1)[:, :N1]
    assert bool((np.abs(deq - ref["y1"]) <= step * 0.5 * 1.001 + 1e-7).all())
    assert (codes(q) != ref["q"]).mean() < 2e-3
    # without the optional outputs
    (q2, s2), y1n, _, _ = fused_rms_fp8_group_quant(wide_d[:, :N1], d(w1), 1e-6, res1=d(res))
    assert y1n is None and torch.equal(q2.view(torch.uint8), q.view(torch.uint8)) and torch.equal(s2, s)


def test_fused_rms_quant_feeds_the_block_linear(sa, dev):
    """The (fp8, scale) pair goes straight into the block-FP8 linear as a pre-quantised input
    (python/sglang/srt/layers/quantization/fp8.py:794-802): the result is the GEMM of the oracle's
    quantised activations, in bfloat16."""
    from sglang_amd.quantization.fp8_utils import aiter_w8a8_block_fp8_linear
    from sglang_amd.quantization.fused_fp8_quant import fused_rms_fp8_group_quant
    from oracle import gemm as og
    from tests.util import assert_gemm_close

    g = torch.Generator().manual_seed(77)
    M, K, N = 48, 1536, 768
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    wn = (torch.rand(K, generator=g) + 0.5).to(torch.bfloat16)
    wq, ws = oq.block_quant_weight(torch.randn(N, K, generator=g) * 0.02)
    ref_q = oq.fused_rms_group_quant(x, wn, 1e-6)
    ref = og.block_fp8_matmul(ref_q["q"], wq, ref_q["s"], ws, return_fp32=True)
    xq = fused_rms_fp8_group_quant(x.to(dev), wn.to(dev), 1e-6)[0]
    out = aiter_w8a8_block_fp8_linear(xq[0], torch.from_numpy(wq).to(dev).view(torch.float8_e4m3fn), [128, 128],
                                      torch.from_numpy(ws).to(dev), input_scale=xq[1])
    assert out.dtype == torch.bfloat16 and out.shape == (M, N)
    assert_gemm_close(out, ref, "rms-quant -> block linear")
    with pytest.raises(NotImplementedError):
        fused_rms_fp8_group_quant(x.to(dev), wn.to(dev), 1e-6, group_size=64)
    with pytest.raises(RuntimeError, match="multiple of 8"):
        fused_rms_fp8_group_quant(x.to(dev)[:, :100], wn.to(dev)[:100].contiguous(), 1e-6)

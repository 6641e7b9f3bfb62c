"""GPU parity of the quantisation operators against the CPU oracle: bytes and scales
bit-exact, called through torch.ops.sgl_kernel (which goes through the C ABI)."""
import numpy as np
import pytest
import torch

from oracle import quant as oq
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

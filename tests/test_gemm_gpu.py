"""GPU parity of the scaled GEMMs against the CPU oracle (fp32-accumulated torch-native path).
Tolerance (north star): rel-L2 <= 1e-2 and max-abs <= 2e-2 * max|ref|; int8 accumulators are exact,
so that path is additionally checked against assert_close defaults as the reference's test does."""
import numpy as np
import pytest
import torch

from oracle import gemm as og
from oracle import quant as oq
from tests.util import assert_gemm_close, codes, outlier_input

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def sa(dev):
    import sglang_amd

    return sglang_amd


def _fp8(a: np.ndarray, dev):
    return torch.from_numpy(a).to(dev).view(torch.float8_e4m3fn)


def _block_case(M, N, K, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = torch.randn(N, K, generator=g) * 0.02
    xq, xs, _ = oq.group_quant(x, 128)
    wq, ws = oq.block_quant_weight(w)
    return xq, xs, wq, ws


@pytest.mark.parametrize("M", [1, 3, 16, 17, 33, 64, 127, 128, 300])
@pytest.mark.parametrize("N,K", [(256, 512), (1536, 7168), (512, 1536), (384, 2048)])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float16])
def test_fp8_blockwise_scaled_mm(sa, dev, M, N, K, out_dtype):
    if out_dtype == torch.float16 and (M not in (1, 33, 128)):
        pytest.skip("fp16 output covered on a subset")
    xq, xs, wq, ws = _block_case(M, N, K, M * 7 + N + K)
    ref = og.block_fp8_matmul(xq, wq, xs, ws, return_fp32=True)
    a = _fp8(xq, dev)
    b = _fp8(wq, dev)                      # [N, K]
    # M-major activation scales and K-major weight scales, as the operator requires
    sa_t = torch.from_numpy(xs).to(dev).t().contiguous().t()
    sb_t = torch.from_numpy(ws).to(dev).t()  # [kb, nb] view with stride(0) == 1
    out = sa.fp8_blockwise_scaled_mm(a, b.t(), sa_t, sb_t, out_dtype)
    assert out.shape == (M, N) and out.dtype == out_dtype
    assert_gemm_close(out, ref, f"M={M} N={N} K={K}")


@pytest.mark.parametrize("M,N,K", [(1, 256, 512), (32, 256, 512), (5, 200, 384), (77, 576, 7168), (130, 1000, 1040)])
def test_w8a8_block_fp8_matmul_row_major_scales(sa, dev, M, N, K):
    """Triton-style entry: row-major scales, N and K need not be multiples of 128 (K % 16 == 0)."""
    from sglang_amd.quantization.fp8_kernel import w8a8_block_fp8_matmul

    g = torch.Generator().manual_seed(M + N + K)
    kb, nb = -(-K // 128), -(-N // 128)
    xq = codes(((torch.rand(M, K, generator=g) - 0.5) * 2 * 448).to(torch.float8_e4m3fn))
    wq = codes(((torch.rand(N, K, generator=g) - 0.5) * 2 * 448).to(torch.float8_e4m3fn))
    xs = (torch.rand(M, kb, generator=g) * 1e-2).numpy()
    ws = (torch.rand(nb, kb, generator=g) * 1e-2).numpy()
    ref = og.block_fp8_matmul(xq, wq, xs, ws, return_fp32=True)
    out = w8a8_block_fp8_matmul(_fp8(xq, dev), _fp8(wq, dev), torch.from_numpy(xs).to(dev),
                                torch.from_numpy(ws).to(dev), [128, 128], torch.bfloat16)
    assert_gemm_close(out, ref, f"M={M} N={N} K={K}")


def _pack_ue8m0(exps: torch.Tensor) -> torch.Tensor:
    """[rows, groups] exponent bytes -> int32 words of four bytes each, groups padded to a multiple of four."""
    rows, groups = exps.shape
    padded = torch.zeros(rows, -(-groups // 4) * 4, dtype=torch.uint8)
    padded[:, :groups] = exps
    return padded.view(torch.int32).contiguous()


@pytest.mark.parametrize("M,N,K,kernel", [(768, 33280, 1024, 7), (520, 33024, 512, 7), (2304, 10240, 768, 7),
                                          (1024, 33280, 16640, 7), (64, 36864, 512, 2), (40, 512, 7168, 2),
                                          (128, 33024, 512, 3), (128, 7168, 18432, 3), (1000, 14336, 512, 4),
                                          (1024, 36864, 512, 7)])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float16])
def test_block_gemm_with_packed_power_of_two_scales(sa, dev, M, N, K, kernel, out_dtype):
    """Packed UE8M0 scales on both operands: the persistent kernel (code 7; the last shape is cut in two along N)
    hands their exponent bytes to the MFMA instead of multiplying every partial product; launches that take the
    one-tile-per-workgroup kernels (codes 2-4, with and without split K) use the expanded scales as floats.  Exponents differ per row and K block (activations, 2^-14..2^-5) and per
    128x128 block (weights), so a scale applied to the wrong row, block or operand shows; the oracle gets the
    powers of two as fp32.  The result must also agree with the same launch through the fp32-scale entry, which
    runs the multiply-add form of the kernel."""
    from sglang_amd._lib import lib
    from sglang_amd.ops import ue8m0_unpack_, w8a8_block_fp8_matmul_
    from sglang_amd.quantization.fp8_kernel import w8a8_block_fp8_matmul

    if out_dtype == torch.float16 and (M, K) not in ((768, 1024), (40, 7168)):
        pytest.skip("fp16 output covered on one shape")
    g = torch.Generator().manual_seed(M + N + K)
    kb, nb = K // 128, -(-N // 128)
    c = torch.randint(0, 256, (N, K), generator=g, dtype=torch.uint8)
    wq = torch.where((c & 0x7F) == 0x7F, c & 0x80, c)
    c = torch.randint(0, 256, (M, K), generator=g, dtype=torch.uint8)
    xq = torch.where((c & 0x7F) == 0x7F, c & 0x80, c)
    xe = torch.randint(113, 123, (M, kb), generator=g, dtype=torch.uint8)   # 2^-14 .. 2^-5
    we = torch.randint(108, 118, (nb, kb), generator=g, dtype=torch.uint8)  # 2^-19 .. 2^-10
    xs = torch.exp2(xe.float() - 127)
    ws = torch.exp2(we.float() - 127)
    xs_packed = _pack_ue8m0(xe).to(dev)
    ws_packed = _pack_ue8m0(we.repeat_interleave(128, dim=0)[:N]).to(dev)  # the same words on every row of a block
    assert torch.equal(ue8m0_unpack_(xs_packed, M, kb).cpu(), xs)
    a, b = xq.to(dev).view(torch.float8_e4m3fn), wq.to(dev).view(torch.float8_e4m3fn)
    print(f"pow2-scale block-fp8 M={M} N={N} K={K}", flush=True)
    out = w8a8_block_fp8_matmul(a, b, xs_packed, ws_packed, [128, 128], out_dtype)
    assert lib.sglamd_last_gemm_kernel() == kernel, "not the kernel this case is about: choose another shape"
    plain = torch.empty_like(out)
    w8a8_block_fp8_matmul_(a, b, xs.to(dev), ws.to(dev), plain)
    assert lib.sglamd_last_gemm_kernel() == (5 if kernel == 7 else kernel)
    assert_gemm_close(out, plain.float().cpu(), f"M={M} N={N} K={K}: MFMA-scaled against multiply-add form")
    blocks = torch.unique(torch.cat([torch.tensor([0, 1, nb - 2, nb - 1]), torch.randint(0, nb, (6,), generator=g)]))
    for blk in blocks.tolist():
        rows = slice(blk * 128, min((blk + 1) * 128, N))
        ref = og.block_fp8_matmul(xq.numpy(), wq[rows].numpy(), xs.numpy(), ws[blk:blk + 1].numpy(), return_fp32=True)
        assert_gemm_close(out[:, rows], ref, f"M={M} N={N} K={K} weight-row block {blk}")


@pytest.mark.parametrize("K", [16640, 32768])
def test_persistent_block_gemm_with_more_than_128_k_blocks(sa, dev, K):
    """The persistent kernel keeps a tile's weight-block scales in two LDS tables of 128 K blocks each: 130 blocks
    just reach into the second table, 256 fill both.  Scales differ from block to block, so a scale taken from the
    wrong table entry shows.  The oracle is evaluated on sampled weight-row blocks (first, last, and some from
    every part of the matrix), all rows."""
    from sglang_amd._lib import lib
    from sglang_amd.quantization.fp8_kernel import w8a8_block_fp8_matmul

    M, N = 520, 33280
    g = torch.Generator().manual_seed(K)
    kb, nb = K // 128, N // 128
    c = torch.randint(0, 256, (N, K), generator=g, dtype=torch.uint8)
    wq = torch.where((c & 0x7F) == 0x7F, c & 0x80, c)  # the two NaN codes -> +-0
    c = torch.randint(0, 256, (M, K), generator=g, dtype=torch.uint8)
    xq = torch.where((c & 0x7F) == 0x7F, c & 0x80, c)
    xs = torch.rand(M, kb, generator=g) * 1e-2 + 1e-3
    ws = torch.rand(nb, kb, generator=g) * 1e-2 + 1e-3
    print(f"persistent block-fp8 M={M} N={N} K={K}", flush=True)
    out = w8a8_block_fp8_matmul(xq.to(dev).view(torch.float8_e4m3fn), wq.to(dev).view(torch.float8_e4m3fn),
                                xs.to(dev), ws.to(dev), [128, 128], torch.bfloat16)
    assert lib.sglamd_last_gemm_kernel() == 5, "not the persistent kernel: choose another shape"
    blocks = torch.unique(torch.cat([torch.tensor([0, 1, nb - 2, nb - 1]),
                                     torch.randint(0, nb, (8,), generator=g)]))
    for b in blocks.tolist():
        rows = slice(b * 128, (b + 1) * 128)
        ref = og.block_fp8_matmul(xq.numpy(), wq[rows].numpy(), xs.numpy(), ws[b:b + 1].numpy(), return_fp32=True)
        assert_gemm_close(out[:, rows], ref, f"K={K} weight-row block {b}")


@pytest.mark.parametrize("M,N,K,kernel", [(768, 33280, 1024, 5), (520, 33024, 512, 5), (2304, 10240, 768, 5),
                                          (768, 23176, 512, 5), (1024, 33024, 512, 5), (768, 23040, 1024, 4),
                                          (2304, 7424, 768, 4)])
@pytest.mark.parametrize("int8", [False, True])
def test_block_gemm_more_tiles_than_cus(sa, dev, M, N, K, kernel, int8):
    """More 256x256 tiles than the chip has CUs: the workgroups walk several tiles each, with the operand
    stream, the weight-scale tables and the output staging crossing tile boundaries (ragged last row tile,
    rows and scales that differ from tile to tile so that a tile fed with its neighbour's data fails).
    The last three shapes leave a short last round of tiles and are cut in two along N (516 = 512 + 4 tiles with the
    persistent kernel on the first part; 270 = 255 + 15 and 261 = 252 + 9 tiles with one tile per workgroup)."""
    g = torch.Generator().manual_seed(M + N + K)
    kb, nb = K // 128, -(-N // 128)  # the last case ends inside a column tile and inside a scale block
    xs = (torch.rand(M, kb, generator=g) * 1e-2 + 1e-3).numpy()
    ws = (torch.rand(nb, kb, generator=g) * 1e-2 + 1e-3).numpy()
    if int8:
        from sglang_amd.quantization.int8_kernel import w8a8_block_int8_matmul

        aq = torch.randint(-128, 128, (M, K), generator=g, dtype=torch.int32).numpy().astype(np.int8)
        bq = torch.randint(-128, 128, (N, K), generator=g, dtype=torch.int32).numpy().astype(np.int8)
        ref = og.block_int8_matmul(aq, bq, xs, ws, return_fp32=True)
        out = w8a8_block_int8_matmul(torch.from_numpy(aq).to(dev), torch.from_numpy(bq).to(dev),
                                     torch.from_numpy(xs).to(dev), torch.from_numpy(ws).to(dev), [128, 128],
                                     torch.bfloat16)
    else:
        from sglang_amd.quantization.fp8_kernel import w8a8_block_fp8_matmul

        xq = codes(((torch.rand(M, K, generator=g) - 0.5) * 2 * 448).to(torch.float8_e4m3fn))
        wq = codes(((torch.rand(N, K, generator=g) - 0.5) * 2 * 448).to(torch.float8_e4m3fn))
        ref = og.block_fp8_matmul(xq, wq, xs, ws, return_fp32=True)
        out = w8a8_block_fp8_matmul(_fp8(xq, dev), _fp8(wq, dev), torch.from_numpy(xs).to(dev),
                                    torch.from_numpy(ws).to(dev), [128, 128], torch.bfloat16)
    # the shapes are chosen so that the launch heuristics pick the kernel this test is about
    from sglang_amd._lib import lib

    assert lib.sglamd_last_gemm_kernel() == kernel, "not the 256x256 kernel this case is about: choose other shapes"
    assert_gemm_close(out, ref, f"M={M} N={N} K={K}")
    # per 256x256 tile as well: one wrong tile among hundreds barely moves the global norm
    for m0 in range(0, M, 256):
        blk = slice(m0, min(m0 + 256, M))
        o, r = out[blk].float().cpu(), ref[blk]
        pad = (-N) % 256
        o, r = torch.nn.functional.pad(o, (0, pad)), torch.nn.functional.pad(r, (0, pad))
        err = (o - r).view(o.shape[0], -1, 256).norm(dim=(0, 2)) / r.view(o.shape[0], -1, 256).norm(dim=(0, 2))
        assert float(err.max()) <= 1e-2, f"tile row {m0}: worst column tile {int(err.argmax())} rel-L2 {float(err.max()):.3e}"


def test_block_gemm_unit_scales_and_one_hot(sa, dev):
    """All scales 1 -> plain matmul of the fp8 values (exactly representable small integers here, so
    the result is exact); one-hot activation rows read back scaled weight rows."""
    M, N, K = 16, 256, 512
    g = torch.Generator().manual_seed(5)
    xi = torch.randint(-8, 9, (M, K), generator=g).float()
    wi = torch.randint(-8, 9, (N, K), generator=g).float()
    a = xi.to(torch.float8_e4m3fn).to(dev)
    b = wi.to(torch.float8_e4m3fn).to(dev)
    ones_a = torch.ones(K // 128, M, device=dev).t()
    ones_b = torch.ones(N // 128, K // 128, device=dev).t()
    out = sa.fp8_blockwise_scaled_mm(a, b.t(), ones_a, ones_b, torch.bfloat16)
    exact = (xi @ wi.t()).to(torch.bfloat16)
    assert torch.equal(out.cpu(), exact)
    # one-hot rows: row m selects k = 37*m; scale column picks the weight block scale
    oh = torch.zeros(M, K)
    for m in range(M):
        oh[m, (37 * m) % K] = 1.0
    sb = (torch.arange(1, (N // 128) * (K // 128) + 1).float().view(N // 128, K // 128) / 8).to(dev)
    out = sa.fp8_blockwise_scaled_mm(oh.to(torch.float8_e4m3fn).to(dev), b.t(), ones_a, sb.t(), torch.bfloat16)
    exp = torch.zeros(M, N)
    for m in range(M):
        k = (37 * m) % K
        exp[m] = wi[:, k] * sb.cpu()[:, k // 128].repeat_interleave(128)
    assert torch.equal(out.cpu(), exp.to(torch.bfloat16))


def _int8(a: np.ndarray, dev):
    return torch.from_numpy(a).to(dev)


@pytest.mark.parametrize("M", [1, 3, 16, 17, 33, 64, 127, 128, 300, 700])
@pytest.mark.parametrize("N,K", [(256, 512), (1536, 7168), (512, 1536), (384, 2048), (200, 400)])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float16])
def test_w8a8_block_int8_matmul(sa, dev, M, N, K, out_dtype):
    """Block-scaled INT8 (test/registered/quant/test_block_int8.py:45-98 is the native model): int8 operands in
    the full range, random block scales; covers the decode kernel, both large tiles, split-K and -- with the
    ragged 200x400 shape -- the generic kernel."""
    from sglang_amd.quantization.int8_kernel import w8a8_block_int8_matmul

    if out_dtype == torch.float16 and (M not in (1, 33, 128)):
        pytest.skip("fp16 output covered on a subset")
    g = torch.Generator().manual_seed(M * 7 + N + K)
    kb, nb = -(-K // 128), -(-N // 128)
    aq = torch.randint(-128, 128, (M, K), generator=g, dtype=torch.int32).numpy().astype(np.int8)
    bq = torch.randint(-128, 128, (N, K), generator=g, dtype=torch.int32).numpy().astype(np.int8)
    xs = (torch.rand(M, kb, generator=g) * 1e-2 + 1e-4).numpy()
    ws = (torch.rand(nb, kb, generator=g) * 1e-2 + 1e-4).numpy()
    ref = og.block_int8_matmul(aq, bq, xs, ws, return_fp32=True)
    out = w8a8_block_int8_matmul(_int8(aq, dev), _int8(bq, dev), torch.from_numpy(xs).to(dev),
                                 torch.from_numpy(ws).to(dev), [128, 128], out_dtype)
    assert out.shape == (M, N) and out.dtype == out_dtype
    assert_gemm_close(out, ref, f"M={M} N={N} K={K}")
    # per-block products are exact integers, so only fp32 summation order and the final cast differ
    torch.testing.assert_close(out.cpu().float(), ref.to(out_dtype).float(), rtol=2e-2, atol=2e-3 * float(ref.abs().max()))


def test_block_int8_unit_scales_exact_and_quantised_linear(sa, dev):
    """Unit scales: every output is an exact integer below 2^24, so fp32 accumulation must reproduce the int64
    matmul bit for bit before the cast (checked on values an fp16 holds exactly).  Then the full chain
    per_token_group_quant_int8 -> matmul against the oracle on the oracle's quantised bytes."""
    from sglang_amd.quantization.int8_kernel import per_token_group_quant_int8, w8a8_block_int8_matmul

    g = torch.Generator().manual_seed(21)
    for M in (4, 48, 256):
        N, K = 384, 1024
        aq = torch.randint(-2, 3, (M, K), generator=g, dtype=torch.int32).to(torch.int8)
        bq = torch.randint(-2, 3, (N, K), generator=g, dtype=torch.int32).to(torch.int8)
        exact = (aq.long() @ bq.long().t())
        assert int(exact.abs().max()) < 2048  # fp16 represents these integers exactly
        out = w8a8_block_int8_matmul(aq.to(dev), bq.to(dev), torch.ones(M, K // 128, device=dev),
                                     torch.ones(N // 128, K // 128, device=dev), [128, 128], torch.float16)
        assert torch.equal(out.cpu().long(), exact)
    x = torch.randn(3, 7, 1024, generator=g).to(torch.bfloat16)
    w = torch.randn(384, 1024, generator=g) * 0.02
    wblk = w.view(3, 128, 8, 128)
    wsc = (wblk.abs().amax(dim=(1, 3)) / 127).float()
    wq = torch.round(wblk / wsc[:, None, :, None]).clamp(-128, 127).to(torch.int8).view(384, 1024)
    xq_ref, xs_ref, _ = oq.group_quant(x.view(-1, 1024), 128, form="reciprocal", dst="int8")  # the default form at group 128
    xq, xs = per_token_group_quant_int8(x.to(dev), 128)
    assert np.array_equal(codes(xq).reshape(-1, 1024), xq_ref) and np.array_equal(xs.cpu().numpy().reshape(-1, 8), xs_ref)
    ref = og.block_int8_matmul(xq_ref, wq.numpy(), xs_ref, wsc.numpy(), return_fp32=True).view(3, 7, 384)
    out = w8a8_block_int8_matmul(xq, wq.to(dev), xs, wsc.to(dev), [128, 128], torch.bfloat16)
    assert out.shape == (3, 7, 384)
    assert_gemm_close(out, ref, "int8 quantised linear")
    with pytest.raises(NotImplementedError):
        w8a8_block_int8_matmul(xq, wq.to(dev), xs, wsc.to(dev), [32, 128], torch.bfloat16)


@pytest.mark.parametrize("M", [1, 16, 64, 100, 512])
@pytest.mark.parametrize("N,K", [(256, 512), (1024, 8192), (2048, 1024), (16, 512)])
@pytest.mark.parametrize("with_bias", [False, True])
def test_fp8_scaled_mm(sa, dev, M, N, K, with_bias):
    g = torch.Generator().manual_seed(M + N + K)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = torch.randn(N, K, generator=g) * 0.02
    xq, xs = oq.per_token_quant_fp8(x)
    wq, ws = oq.per_channel_quant_weight(w, "fp8")
    bias = (torch.randn(N, generator=g)).to(torch.bfloat16) if with_bias else None
    ref = og.fp8_scaled_mm(xq, wq, xs, ws, bias=bias, return_fp32=True)
    out = sa.fp8_scaled_mm(_fp8(xq, dev), _fp8(wq, dev).t(), torch.from_numpy(xs).to(dev).view(M, 1),
                           torch.from_numpy(ws).to(dev).view(N, 1), torch.bfloat16,
                           bias.to(dev) if with_bias else None)
    assert_gemm_close(out, ref, f"M={M} N={N} K={K}")


@pytest.mark.parametrize("M", [1, 16, 64, 100, 512])
@pytest.mark.parametrize("N,K", [(256, 512), (1024, 8192), (2048, 1024), (16, 512)])
@pytest.mark.parametrize("with_bias", [False, True])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float16])
def test_int8_scaled_mm(sa, dev, M, N, K, with_bias, out_dtype):
    g = torch.Generator().manual_seed(M + N + K)
    aq = torch.randint(-128, 128, (M, K), generator=g, dtype=torch.int32).to(torch.int8)
    bq = torch.randint(-128, 128, (N, K), generator=g, dtype=torch.int32).to(torch.int8)
    sa_ = torch.rand(M, generator=g) * 1e-2
    sb_ = torch.rand(N, generator=g) * 1e-2
    bias = (torch.randn(N, generator=g) * 10).to(out_dtype) if with_bias else None
    ref = og.int8_scaled_mm(aq.numpy(), bq.numpy(), sa_.numpy(), sb_.numpy(), out_dtype=out_dtype, bias=bias)
    out = sa.int8_scaled_mm(aq.to(dev), bq.to(dev).t(), sa_.to(dev).view(M, 1), sb_.to(dev).view(N, 1), out_dtype,
                            bias.to(dev) if with_bias else None)
    torch.testing.assert_close(out.cpu(), ref)  # exact int32 accumulation -> default tolerances
    assert_gemm_close(out, ref.float())


def test_linear_wrappers(sa, dev):
    from sglang_amd.quantization.fp8_utils import (
        apply_fp8_linear,
        cutlass_w8a8_block_fp8_linear_with_fallback,
        triton_w8a8_block_fp8_linear,
    )

    g = torch.Generator().manual_seed(11)
    x = torch.randn(2, 9, 1024, generator=g).to(torch.bfloat16)
    w = torch.randn(768, 1024, generator=g) * 0.02
    wq, ws = oq.block_quant_weight(w)
    xq, xs, _ = oq.group_quant(x.view(-1, 1024), 128, form="reciprocal")
    ref = og.block_fp8_matmul(xq, wq, xs, ws, return_fp32=True).view(2, 9, 768)
    wd, wsd = _fp8(wq, dev), torch.from_numpy(ws).to(dev)
    for fn in (cutlass_w8a8_block_fp8_linear_with_fallback, triton_w8a8_block_fp8_linear):
        out = fn(x.to(dev), wd, [128, 128], wsd)
        assert out.shape == (2, 9, 768) and out.dtype == torch.bfloat16
        assert_gemm_close(out, ref, fn.__name__)
    # per-token / per-channel
    wq2, ws2 = oq.per_channel_quant_weight(w, "fp8")
    xq2, xs2 = oq.per_token_quant_fp8(x.view(-1, 1024))
    ref2 = og.fp8_scaled_mm(xq2, wq2, xs2, ws2, return_fp32=True).view(2, 9, 768)
    out2 = apply_fp8_linear(x.to(dev), _fp8(wq2, dev).t(), torch.from_numpy(ws2).to(dev).view(-1, 1))
    assert_gemm_close(out2, ref2, "apply_fp8_linear")
    # static per-tensor activation scale (fp8_utils.py:1518-1524), per-channel and per-tensor weight scales
    s_in = 0.0137
    xq3, xs3 = oq.static_quant_fp8(x.view(-1, 1024), s_in)
    ref3 = og.fp8_scaled_mm(xq3, wq2, xs3, ws2, return_fp32=True).view(2, 9, 768)
    out3 = apply_fp8_linear(x.to(dev), _fp8(wq2, dev).t(), torch.from_numpy(ws2).to(dev).view(-1, 1),
                            input_scale=torch.tensor([s_in], device=dev))
    assert_gemm_close(out3, ref3, "apply_fp8_linear, static input scale")
    w_t = float(np.abs(w.numpy()).max() / 448.0)
    wq4 = oq.static_quant_fp8(w, w_t)[0]
    ref4 = og.fp8_scaled_mm(xq3, wq4, xs3, np.full((768,), w_t, dtype=np.float32), return_fp32=True).view(2, 9, 768)
    out4 = apply_fp8_linear(x.to(dev), _fp8(wq4, dev).t(), torch.tensor(w_t, device=dev),
                            input_scale=torch.tensor(s_in, device=dev))
    assert_gemm_close(out4, ref4, "apply_fp8_linear, static input scale, per-tensor weight scale")
    # dynamic per-tensor activation scale with a per-tensor weight scale (fp8_utils.py:1534-1540), and the same
    # through compressed_tensor_quant with per-channel weights (:1480-1516); input_scale_ub is accepted and unused
    amax = float(x.float().abs().max())
    xq6, xs6 = oq.static_quant_fp8(x.view(-1, 1024), amax / 448.0)
    ref6 = og.fp8_scaled_mm(xq6, wq4, xs6, np.full((768,), w_t, dtype=np.float32), return_fp32=True).view(2, 9, 768)
    out6 = apply_fp8_linear(x.to(dev), _fp8(wq4, dev).t(), torch.tensor(w_t, device=dev),
                            input_scale_ub=torch.ones(1, device=dev))
    assert_gemm_close(out6, ref6, "apply_fp8_linear, dynamic per-tensor scale")
    ref7 = og.fp8_scaled_mm(xq6, wq2, xs6, ws2, return_fp32=True).view(2, 9, 768)
    out7 = apply_fp8_linear(x.to(dev), _fp8(wq2, dev).t(), torch.from_numpy(ws2).to(dev).view(-1, 1),
                            compressed_tensor_quant=True, pad_output=True)
    assert_gemm_close(out7, ref7, "apply_fp8_linear, compressed-tensors dynamic per-tensor scale")
    with pytest.raises(NotImplementedError):
        apply_fp8_linear(x.to(dev), _fp8(wq2, dev).t(), torch.from_numpy(ws2).to(dev), input_scale=torch.ones(18, device=dev))
    # UE8M0 checkpoints (fp8_utils.py:645-696): weight scales rounded up to powers of two and handed over as packed
    # exponent words, one row of words per weight row; the activations are quantised to the same format
    from sglang_amd.quantization.fp8_utils import deepgemm_w8a8_block_fp8_linear_with_fallback

    amax = np.abs(w.numpy().reshape(6, 128, 8, 128)).max(axis=(1, 3))
    we = np.ceil(np.log2(np.maximum(amax, 1e-4) / 448.0)).astype(np.int32) + 127     # biased exponents [6, 8]
    ws5 = np.exp2(we.astype(np.float32) - 127)
    w5 = np.clip(w.numpy().reshape(6, 128, 8, 128) / ws5[:, None, :, None], -448, 448).reshape(768, 1024)
    wq5 = oq.e4m3fn_encode(w5.astype(np.float32))
    xq5, xs5, _ = oq.group_quant(x.view(-1, 1024), 128, form="reciprocal", scale_ue8m0=True)
    ref5 = og.block_fp8_matmul(xq5, wq5, xs5, ws5, return_fp32=True).view(2, 9, 768)
    packed = torch.from_numpy(oq.pack_ue8m0(np.repeat(we.astype(np.uint8), 128, axis=0))).to(dev)
    for fn in (deepgemm_w8a8_block_fp8_linear_with_fallback, cutlass_w8a8_block_fp8_linear_with_fallback):
        out5 = fn(x.to(dev), _fp8(wq5, dev), [128, 128], packed)
        assert out5.shape == (2, 9, 768) and out5.dtype == torch.bfloat16
        assert_gemm_close(out5, ref5, fn.__name__ + ", UE8M0 scales")


def test_gemm_error_paths(sa, dev):
    a = torch.zeros(4, 256, device=dev).to(torch.float8_e4m3fn)
    b = torch.zeros(128, 256, device=dev).to(torch.float8_e4m3fn)
    s_a = torch.ones(2, 4, device=dev).t()
    s_b = torch.ones(1, 2, device=dev).t()
    sa.fp8_blockwise_scaled_mm(a, b.t(), s_a, s_b, torch.bfloat16)
    with pytest.raises(RuntimeError, match="column major"):
        sa.fp8_blockwise_scaled_mm(a, b.t().contiguous(), s_a, s_b, torch.bfloat16)
    with pytest.raises(RuntimeError, match="Float8_e4m3fn"):
        sa.fp8_blockwise_scaled_mm(a.view(torch.int8), b.t(), s_a, s_b, torch.bfloat16)
    with pytest.raises(RuntimeError, match="out_dtype"):
        sa.fp8_blockwise_scaled_mm(a, b.t(), s_a, s_b, torch.float32)
    with pytest.raises(RuntimeError, match="M major"):
        sa.fp8_blockwise_scaled_mm(a, b.t(), torch.ones(4, 2, device=dev), s_b, torch.bfloat16)
    with pytest.raises(RuntimeError, match="scales_b"):
        sa.fp8_blockwise_scaled_mm(a, b.t(), s_a, torch.ones(2, 2, device=dev).t(), torch.bfloat16)
    with pytest.raises(RuntimeError, match="bias"):
        sa.fp8_scaled_mm(a, b.t(), torch.ones(4, device=dev), torch.ones(128, device=dev), torch.bfloat16,
                         torch.ones(128, device=dev))
    with pytest.raises(RuntimeError, match="Int8"):
        sa.int8_scaled_mm(a, b.t(), torch.ones(4, device=dev), torch.ones(128, device=dev), torch.bfloat16, None)


def test_golden_config1_on_gpu(sa, dev):
    """The committed golden vectors (tests/golden/config1.npz): quantised bytes and scales bit-exact in both
    arithmetic forms and both scale layouts, GEMM within tolerance of the golden bf16 output."""
    import os

    from sglang_amd.quantization.fp8_kernel import sglang_per_token_group_quant_fp8

    z = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "config1.npz"))
    a = torch.from_numpy(z["a_bf16_bits"]).view(torch.bfloat16).to(dev)
    for v2, key in ((False, "divide"), (True, "reciprocal")):
        for col in (False, True):
            q, s = sglang_per_token_group_quant_fp8(a, 128, column_major_scales=col, enable_v2=v2)
            assert np.array_equal(codes(q), z[f"aq_{key}"])
            assert np.array_equal(s.cpu().numpy(), z[f"as_{key}"])
    q, s = sglang_per_token_group_quant_fp8(a, 128, column_major_scales=True, enable_v2=False)
    wq = _fp8(z["wq"], dev)
    c = sa.fp8_blockwise_scaled_mm(q, wq.t(), s, torch.from_numpy(z["ws"]).to(dev).t(), torch.bfloat16)
    gold = torch.from_numpy(z["c_bf16_bits"]).view(torch.bfloat16)
    assert_gemm_close(c, gold.float(), "golden config 1")
    assert (c.cpu() != gold).float().mean() < 0.05  # same bf16 value almost everywhere


@pytest.mark.parametrize("mode", ["block_fp8", "block_int8", "row_fp8", "row_int8"])
def test_streaming_kernel_with_two_row_tiles_and_three_or_four_column_tiles(sa, dev, mode):
    """17..32 rows stream the weights in workgroup tiles of 32 x 16*FN; which FN a launch gets depends on how its
    column tiles divide over the chip.  Both wide forms (FN = 3 and 4) have to appear among these weights, each
    checked against the oracle at 17, 24 and 32 rows (rows 17..31 of the second row tile are padding there)."""
    from sglang_amd._lib import lib

    seen = {}
    for N in (36864, 57344, 10240, 24576, 43008, 28672, 14336, 49152):
        K = 512
        for M in (24, 17, 32):
            g = torch.Generator().manual_seed(N + M)
            if mode.endswith("int8"):
                a = torch.randint(-128, 128, (M, K), generator=g, dtype=torch.int32).to(torch.int8)
                b = torch.randint(-128, 128, (N, K), generator=g, dtype=torch.int32).to(torch.int8)
                ad, bd = a.to(dev), b.to(dev)
            else:
                c = torch.randint(0, 256, (M, K), generator=g, dtype=torch.uint8)
                a = torch.where((c & 0x7F) == 0x7F, c & 0x80, c)
                c = torch.randint(0, 256, (N, K), generator=g, dtype=torch.uint8)
                b = torch.where((c & 0x7F) == 0x7F, c & 0x80, c)
                ad, bd = a.to(dev).view(torch.float8_e4m3fn), b.to(dev).view(torch.float8_e4m3fn)
            print(f"{mode} M={M} N={N} K={K}", flush=True)
            if mode.startswith("block"):
                xs = torch.rand(M, K // 128, generator=g) * 1e-2 + 1e-3
                ws = torch.rand(N // 128, K // 128, generator=g) * 1e-2 + 1e-3
                if mode == "block_fp8":
                    from sglang_amd.quantization.fp8_kernel import w8a8_block_fp8_matmul as mm
                    ref = og.block_fp8_matmul(a.numpy(), b.numpy(), xs.numpy(), ws.numpy(), return_fp32=True)
                else:
                    from sglang_amd.quantization.int8_kernel import w8a8_block_int8_matmul as mm
                    ref = og.block_int8_matmul(a.numpy(), b.numpy(), xs.numpy(), ws.numpy(), return_fp32=True)
                out = mm(ad, bd, xs.to(dev), ws.to(dev), [128, 128], torch.bfloat16)
            else:
                s_a = torch.rand(M, generator=g) * 1e-2 + 1e-3
                s_b = torch.rand(N, generator=g) * 1e-2 + 1e-3
                if mode == "row_fp8":
                    ref = og.fp8_scaled_mm(a.numpy(), b.numpy(), s_a.numpy(), s_b.numpy(), return_fp32=True)
                    out = sa.fp8_scaled_mm(ad, bd.t(), s_a.to(dev).view(M, 1), s_b.to(dev).view(N, 1), torch.bfloat16)
                else:
                    ref = og.int8_scaled_mm(a.numpy(), b.numpy(), s_a.numpy(), s_b.numpy(), return_fp32=True)
                    out = sa.int8_scaled_mm(ad, bd.t(), s_a.to(dev).view(M, 1), s_b.to(dev).view(N, 1), torch.bfloat16)
            assert lib.sglamd_last_gemm_kernel() == 1, "17..32 rows take the streaming kernel"
            shape = lib.sglamd_last_streaming_shape()
            fm, fn = shape >> 16, (shape >> 8) & 0xFF
            assert fm == 2
            if M == 24 and fn in seen:
                break  # this column-tile count is covered
            seen.setdefault(fn, []).append((M, N))
            assert_gemm_close(out, ref, f"{mode} M={M} N={N} FN={fn}")
    assert 3 in seen and 4 in seen, f"the wide forms did not both appear: {seen}"


# kernel codes of include/sglamd.h
_STREAMING, _TILE64, _TILE128, _TILE256, _PERSISTENT256, _GENERIC, _WIDE = 1, 2, 3, 4, 5, 6, 8


@pytest.mark.parametrize("M,N,K,kernel", [
    (9, 512, 1024, _STREAMING),
    (40, 512, 1024, _STREAMING),       # up to 64 rows and a small weight: the streaming kernel's 64-row form
    (24, 768, 2048, _STREAMING),       # ... and its 32-row form
    (40, 8192, 1024, _TILE64),         # one row of 64-row tiles, K not split (8 K blocks)
    (40, 512, 7168, _TILE64),          # the same with K split over the workgroups
    (24, 24576, 512, _STREAMING),      # up to 32 rows: the streaming kernel whatever the weight
    (48, 24576, 512, _TILE64),         # 33..64 rows go to the tile kernel once about a hundred workgroups come together
    (40, 36864, 5120, _WIDE),          # 33..64 rows, many weight rows, long K: 256 workgroups of 144 weight rows (nine column tiles)
    (64, 24576, 5248, _WIDE),          # ... of 96 weight rows (six column tiles)
    (50, 32768, 5632, _WIDE),          # ... of 128 weight rows (eight column tiles)
    (33, 30016, 5184, _WIDE),          # ... trimmed rows per workgroup, ragged last workgroup, ragged last K block
    (128, 33024, 512, _TILE128),       # 129 column tiles: 64-row tiles would need a second round
    (128, 7168, 18432, _TILE128),      # few column tiles, long K: 128-row tiles with K split 9 ways
    (1000, 14336, 512, _TILE256),      # 224 tiles of 256 rows in one round, last row tile ragged
    (100, 520, 400, _GENERIC),         # K not a multiple of 128
])
@pytest.mark.parametrize("mode", ["block_fp8", "block_int8", "row_fp8", "row_int8"])
def test_every_dense_kernel_in_every_mode(sa, dev, M, N, K, kernel, mode):
    """The kernel behind a GEMM call is chosen from the shape; each case here names the kernel it is meant for and
    fails if the launch heuristics send it elsewhere, so that no kernel loses its parity test to a retuning."""
    from sglang_amd._lib import lib
    from sglang_amd.quantization.fp8_kernel import w8a8_block_fp8_matmul
    from sglang_amd.quantization.int8_kernel import w8a8_block_int8_matmul

    g = torch.Generator().manual_seed(M * 7 + N + K)
    kb, nb = -(-K // 128), -(-N // 128)
    if mode.endswith("fp8"):
        c = torch.randint(0, 256, (M + N, K), generator=g, dtype=torch.int32).to(torch.uint8)
        c = torch.where((c & 0x7F) == 0x7F, c & 0x80, c)
        aq, bq = c[:M].numpy(), c[M:].numpy()
        a_d, b_d = _fp8(aq, dev), _fp8(bq, dev)
    else:
        c = torch.randint(-128, 128, (M + N, K), generator=g, dtype=torch.int32).to(torch.int8)
        aq, bq = c[:M].numpy(), c[M:].numpy()
        a_d, b_d = torch.from_numpy(aq).to(dev), torch.from_numpy(bq).to(dev)
    if mode.startswith("block"):
        xs = (torch.rand(M, kb, generator=g) * 1e-2 + 1e-3).numpy()
        ws = (torch.rand(nb, kb, generator=g) * 1e-2 + 1e-3).numpy()
        mm, ref_mm = ((w8a8_block_fp8_matmul, og.block_fp8_matmul) if mode == "block_fp8"
                      else (w8a8_block_int8_matmul, og.block_int8_matmul))
        ref = ref_mm(aq, bq, xs, ws, return_fp32=True)
        out = mm(a_d, b_d, torch.from_numpy(xs).to(dev), torch.from_numpy(ws).to(dev), [128, 128], torch.bfloat16)
    else:
        xs = (torch.rand(M, generator=g) * 1e-2 + 1e-3).numpy()
        ws = (torch.rand(N, generator=g) * 1e-2 + 1e-3).numpy()
        if mode == "row_fp8":
            ref = og.fp8_scaled_mm(aq, bq, xs, ws, return_fp32=True)
            out = sa.fp8_scaled_mm(a_d, b_d.t(), torch.from_numpy(xs).to(dev).view(M, 1),
                                   torch.from_numpy(ws).to(dev).view(N, 1), torch.bfloat16, None)
        else:
            ref = og.int8_scaled_mm(aq, bq, xs, ws, out_dtype=torch.bfloat16).float()
            out = sa.int8_scaled_mm(a_d, b_d.t(), torch.from_numpy(xs).to(dev).view(M, 1),
                                    torch.from_numpy(ws).to(dev).view(N, 1), torch.bfloat16, None)
    assert lib.sglamd_last_gemm_kernel() == kernel, f"ran kernel {lib.sglamd_last_gemm_kernel()}, meant for {kernel}"
    assert_gemm_close(out, ref, f"{mode} M={M} N={N} K={K}")
    o, r = out.float().cpu(), torch.as_tensor(ref).float()
    per_row = (o - r).norm(dim=1) / r.norm(dim=1).clamp_min(1e-30)
    assert float(per_row.max()) <= 1e-2, f"row {int(per_row.argmax())}: rel-L2 {float(per_row.max()):.3e}"

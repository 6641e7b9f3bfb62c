"""Parity at the full sizes the benchmark is quoted on.  The CPU oracle cannot redo 2 TFLOP in a test, so each
case checks (a) the oracle on a sample of rows (every output row depends on its own activation row only, so the
rows of a sample are computed by the oracle exactly as inside the full problem), (b) that two runs agree bit for
bit (a race between a tile's output and the next tile's work shows up here first) and (c) that permuting the
activation rows permutes the output rows bit for bit (a row's arithmetic does not depend on the tile or the
position inside a tile it lands in).  Tolerances as in the small-size tests: bytes and scales bit-exact,
GEMM outputs rel-L2 <= 1e-2 and max-abs <= 2e-2 * max|ref| against the fp32 oracle."""
import numpy as np
import pytest
import torch

from oracle import gemm as og
from oracle import quant as oq
from tests.util import assert_gemm_close, codes, outlier_input

pytestmark = pytest.mark.gpu

PERSISTENT256 = 5  # SGLAMD_KERNEL_PERSISTENT256 of include/sglamd.h


def _rand_fp8_codes(shape, gen):
    """Uniform e4m3fn codes without the two NaN encodings, on the host."""
    c = torch.randint(0, 256, shape, generator=gen, dtype=torch.int32).to(torch.uint8)
    return torch.where((c & 0x7F) == 0x7F, c & 0x80, c)  # NaN codes -> +-0


def _sample_rows(M, count, gen):
    # rows from every 256-row tile, at positions that fall into every 32-row step of both wave rows
    base = torch.arange(0, M, 256).repeat_interleave(max(1, count // max(1, M // 256)))
    off = torch.randint(0, 256, base.shape, generator=gen)
    return torch.unique((base + off).clamp_max(M - 1))


@pytest.mark.parametrize("int8", [False, True])
def test_gate_up_m4096_block_gemm(dev, int8):
    """DeepSeek-V3 gate_up at M=4096 (N=36864, K=7168): the benchmark's headline launch."""
    import sglang_amd  # noqa: F401
    from sglang_amd._lib import lib
    from sglang_amd.quantization.fp8_kernel import w8a8_block_fp8_matmul
    from sglang_amd.quantization.int8_kernel import w8a8_block_int8_matmul

    M, N, K = 4096, 36864, 7168
    g = torch.Generator().manual_seed(4096 + int8)
    xs = torch.rand(M, K // 128, generator=g) * 1e-2 + 1e-3
    ws = torch.rand(N // 128, K // 128, generator=g) * 1e-2 + 1e-3
    if int8:
        xq = torch.randint(-128, 128, (M, K), generator=g, dtype=torch.int32).to(torch.int8)
        wq = torch.randint(-128, 128, (N, K), generator=g, dtype=torch.int32).to(torch.int8)
        to_dev = lambda t: t.to(dev)  # noqa: E731
        mm, ref_mm = w8a8_block_int8_matmul, og.block_int8_matmul
    else:
        xq, wq = _rand_fp8_codes((M, K), g), _rand_fp8_codes((N, K), g)
        to_dev = lambda t: t.to(dev).view(torch.float8_e4m3fn)  # noqa: E731
        mm, ref_mm = w8a8_block_fp8_matmul, og.block_fp8_matmul
    wq_d, ws_d, xs_d = to_dev(wq), ws.to(dev), xs.to(dev)

    out = mm(to_dev(xq), wq_d, xs_d, ws_d, [128, 128], torch.bfloat16)
    assert lib.sglamd_last_gemm_kernel() == PERSISTENT256
    again = mm(to_dev(xq), wq_d, xs_d, ws_d, [128, 128], torch.bfloat16)
    assert torch.equal(out, again), "two runs of the same launch differ"

    perm = torch.randperm(M, generator=g)
    out_p = mm(to_dev(xq[perm]), wq_d, xs_d[perm.to(dev)].contiguous(), ws_d, [128, 128], torch.bfloat16)
    assert torch.equal(out_p, out[perm.to(dev)]), "output rows depend on where their activation rows sit"

    rows = _sample_rows(M, 48, g)
    ref = ref_mm(xq[rows].numpy(), wq.numpy(), xs[rows].numpy(), ws.numpy(), return_fp32=True)
    assert_gemm_close(out[rows.to(dev)], ref, f"rows sampled from M={M} N={N} K={K}")
    # every sampled row on its own: a row with a few wrong 16-byte pieces hides in the norm over all of them
    o, r = out[rows.to(dev)].float().cpu(), torch.as_tensor(ref)
    per_row = (o - r).norm(dim=1) / r.norm(dim=1)
    assert float(per_row.max()) <= 1e-2, f"row {int(rows[int(per_row.argmax())])}: rel-L2 {float(per_row.max()):.3e}"


def test_group_quant_m16384(dev):
    """Group quant of 16384 x 7168 bf16 (the largest quant configuration): sampled rows bit-exact against the
    oracle, and the whole output invariant under a row permutation."""
    from sglang_amd.quantization.fp8_kernel import sglang_per_token_group_quant_fp8

    M, K = 16384, 7168
    x = outlier_input(M, K, torch.bfloat16, scale=50.0)
    g = torch.Generator().manual_seed(7)
    for column_major in (False, True):
        q, s = sglang_per_token_group_quant_fp8(x.to(dev), 128, column_major_scales=column_major)
        rows = torch.unique(torch.randint(0, M, (96,), generator=g))
        rq, rs, _ = oq.group_quant(x[rows], 128, form="reciprocal")
        assert np.array_equal(codes(q[rows.to(dev)]), rq)
        assert np.array_equal(s[rows.to(dev)].cpu().numpy(), rs)
        perm = torch.randperm(M, generator=g)
        qp, sp = sglang_per_token_group_quant_fp8(x[perm].to(dev), 128, column_major_scales=column_major)
        assert torch.equal(qp.view(torch.uint8), q.view(torch.uint8)[perm.to(dev)])
        assert torch.equal(sp, s[perm.to(dev)])

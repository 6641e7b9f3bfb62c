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


def test_dsv3_moe_layer_m4096(dev):
    """The DeepSeek-V3 MoE layer (256 experts, top-8, hidden 7168, intermediate 2048) at M=4096: the same tokens in
    chunks of 512 take other sorted-block heights and tile shapes and must give the same rows; a sample of tokens
    is checked against the oracle on the experts those tokens use."""
    from oracle import moe as om
    from tests.util import moe_layer as fused_moe

    M, H, I, E, topk = 4096, 7168, 2048, 256, 8
    g = torch.Generator().manual_seed(256)
    gd = torch.Generator(device=dev).manual_seed(256)

    def rand_codes(shape):  # e4m3fn codes without NaN, generated on the device (11 GB in all)
        c = torch.randint(0, 256, shape, generator=gd, dtype=torch.int32, device=dev).to(torch.uint8)
        return torch.where((c & 0x7F) == 0x7F, c & 0x80, c).view(torch.float8_e4m3fn)

    w13 = torch.empty(E, 2 * I, H, dtype=torch.float8_e4m3fn, device=dev)
    w2 = torch.empty(E, H, I, dtype=torch.float8_e4m3fn, device=dev)
    for e in range(0, E, 16):
        w13[e:e + 16] = rand_codes((16, 2 * I, H))
        w2[e:e + 16] = rand_codes((16, H, I))
    w13s = torch.rand(E, 2 * I // 128, H // 128, generator=gd, device=dev) * 2e-4 + 1e-5
    w2s = torch.rand(E, H // 128, I // 128, generator=gd, device=dev) * 2e-4 + 1e-5
    x = torch.randn(M, H, generator=g).to(torch.bfloat16)
    tw, ti = torch.topk(torch.softmax(torch.randn(M, E, generator=g), dim=-1), topk, dim=-1)
    tw = (tw / tw.sum(-1, keepdim=True)).contiguous()
    ti = ti.to(torch.int32).contiguous()

    def layer(rows):
        return fused_moe(x[rows].to(dev), w13, w2, (tw[rows].to(dev), ti[rows].to(dev), None), use_fp8_w8a8=True,
                         w1_scale=w13s, w2_scale=w2s, block_shape=[128, 128])

    whole = layer(slice(0, M))
    assert torch.equal(whole, layer(slice(0, M))), "two runs of the same layer differ"
    for c in range(0, M, 512):
        assert_gemm_close(whole[c:c + 512], layer(slice(c, c + 512)).float(), f"tokens {c}..{c + 512}")

    sample = torch.randperm(M, generator=g)[:6]
    used = torch.unique(ti[sample])
    remap = torch.full((E,), -1, dtype=torch.int32)
    remap[used.long()] = torch.arange(len(used), dtype=torch.int32)
    sel = used.long().to(dev)
    ref = om.fused_moe_block_fp8(x[sample], codes(w13[sel]), codes(w2[sel]), w13s[sel].cpu().numpy(),
                                 w2s[sel].cpu().numpy(), tw[sample], remap[ti[sample].long()],
                                 quant_form="reciprocal")
    assert_gemm_close(whole[sample.to(dev)], ref.float(), "sampled tokens of the M=4096 layer")

"""GPU parity of the expert-major ("grouped") MoE interface against the CPU oracle: index arrays and moved
rows bit-exact, the weighted sum bit-exact (fp32 fused multiply-adds in a fixed order), GEMM and whole-layer
outputs within the GEMM tolerance (rel-L2 <= 1e-2, max-abs <= 2e-2 * max|ref|)."""
import numpy as np
import pytest
import torch

from oracle import moe as om
from oracle import quant as oq
from oracle.fp8 import e4m3fn_encode
from tests.util import assert_gemm_close, codes

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def sa(dev):
    import sglang_amd

    return sglang_amd


def _ids(tokens, topk, E, seed, drop=None):
    g = torch.Generator().manual_seed(seed)
    ids = torch.stack([torch.randperm(E, generator=g)[:topk] for _ in range(tokens)]).to(torch.int32)
    if drop is not None:
        ids[ids == drop] = -1
    return ids


@pytest.mark.parametrize("tokens,topk,E", [(1, 8, 256), (33, 2, 8), (222, 6, 24), (4096, 8, 256), (1000, 1, 3),
                                           (5000, 4, 2047)])
@pytest.mark.parametrize("with_blockscale", [False, True])
def test_prepare_moe_input(sa, dev, tokens, topk, E, with_blockscale):
    ids = _ids(tokens, topk, E, tokens + E, drop=1 if tokens == 222 else None)
    n, k = 2048, 7168
    offs, bs, ps1, ps2, a_map, c_map = om.prepare_moe_input(ids.numpy(), E, n, k)
    i32 = lambda *shape: torch.full(shape, -1, dtype=torch.int32, device=dev)
    d_offs, d_bs, d_ps1, d_ps2 = i32(E + 1), i32(E + 1), i32(E, 3), i32(E, 3)
    d_a, d_c = i32(tokens * topk), i32(tokens * topk)
    sa.prepare_moe_input(ids.to(dev), d_offs, d_ps1, d_ps2, d_a, d_c, E, n, k, d_bs if with_blockscale else None)
    assert np.array_equal(d_offs.cpu().numpy(), offs)
    assert np.array_equal(d_ps1.cpu().numpy(), ps1) and np.array_equal(d_ps2.cpu().numpy(), ps2)
    valid = int(offs[-1])
    assert np.array_equal(d_a.cpu().numpy()[:valid], a_map[:valid])
    assert np.array_equal(d_c.cpu().numpy(), c_map)  # entries of dropped ids keep their initial -1
    if with_blockscale:
        assert np.array_equal(d_bs.cpu().numpy(), bs)
    else:
        assert bool((d_bs == -1).all())
    with pytest.raises(RuntimeError, match="int32"):
        sa.prepare_moe_input(ids.to(dev).long(), d_offs, d_ps1, d_ps2, d_a, d_c, E, n, k)


@pytest.mark.parametrize("dtype,cols", [(torch.bfloat16, 7168), (torch.float16, 200), (torch.float32, 56),
                                        (torch.float8_e4m3fn, 7168), (torch.uint8, 33), (torch.float32, 3)])
def test_shuffle_rows(sa, dev, dtype, cols):
    g = torch.Generator().manual_seed(cols)
    src_rows, dst_rows = 37, 150
    raw = torch.randint(0, 256, (src_rows, cols * torch.empty((), dtype=dtype).element_size()), generator=g,
                        dtype=torch.uint8)
    x = raw.view(dtype) if dtype != torch.uint8 else raw
    mp = torch.randint(0, src_rows, (dst_rows,), generator=g, dtype=torch.int32)
    out = sa.shuffle_rows(x.to(dev), mp.to(dev), (dst_rows, cols))
    assert out.dtype == dtype and out.shape == (dst_rows, cols)
    want = om.shuffle_rows(raw.numpy(), mp.numpy())
    assert np.array_equal(out.cpu().view(torch.uint8).numpy().reshape(dst_rows, -1), want)
    with pytest.raises(RuntimeError, match="same data type"):
        torch.ops.sgl_kernel.shuffle_rows(x.to(dev), mp.to(dev), torch.empty(dst_rows, cols, device=dev,
                                                                             dtype=torch.int16))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("m,topk,cols", [(1, 8, 7168), (50, 2, 512), (19, 6, 100), (300, 1, 4096)])
def test_apply_shuffle_mul_sum(sa, dev, dtype, m, topk, cols):
    g = torch.Generator().manual_seed(m + cols)
    c2 = torch.randn(m * topk, cols, generator=g).to(dtype)
    perm = torch.randperm(m * topk, generator=g).to(torch.int32)
    w = torch.rand(m, topk, generator=g).to(dtype)
    out = torch.empty(m, cols, device=dev, dtype=dtype)
    sa.apply_shuffle_mul_sum(c2.to(dev), out, perm.to(dev), w.to(dev))
    assert torch.equal(out.cpu(), om.apply_shuffle_mul_sum(c2, perm.numpy(), w, m))
    sa.apply_shuffle_mul_sum(c2.to(dev), out, perm.to(dev), None)
    assert torch.equal(out.cpu(), om.apply_shuffle_mul_sum(c2, perm.numpy(), None, m))
    with pytest.raises(RuntimeError, match="Factors must match output dtype"):
        sa.apply_shuffle_mul_sum(c2.to(dev), out, perm.to(dev), w.float().to(dev))


def _grouped_case(E, N, K, counts, seed, dev):
    g = torch.Generator().manual_seed(seed)
    offs = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    rows = int(offs[-1])
    a = torch.randn(rows, K, generator=g).to(torch.bfloat16)
    aq, a_s, _ = oq.group_quant(a, 128)
    wq, ws = [], []
    for e in range(E):
        q, s = oq.block_quant_weight(torch.randn(N, K, generator=g) * 0.02)
        wq.append(q)
        ws.append(s)
    bq, b_s = np.stack(wq), np.stack(ws)
    ps = np.array([[c, N, K] for c in counts], dtype=np.int32)
    return offs, ps, aq, a_s, bq, b_s


def _call_grouped(sa, dev, out_dtype, offs, ps, aq, a_s, bq, b_s, workspace_bytes=1 << 22):
    E, N, K = bq.shape
    rows = aq.shape[0]
    f8 = lambda x: torch.from_numpy(x).to(dev).view(torch.float8_e4m3fn)
    out = torch.full((rows, N), 7.0, device=dev, dtype=out_dtype)
    i64 = lambda: torch.empty(E, device=dev, dtype=torch.int64)
    lay = lambda: torch.zeros(E, 5, device=dev, dtype=torch.int32)
    strides = torch.full((E,), K, device=dev, dtype=torch.int64)
    c_strides = torch.full((E,), N, device=dev, dtype=torch.int64)
    sa.fp8_blockwise_scaled_grouped_mm(
        out, i64(), i64(), i64(), i64(), i64(), f8(aq), f8(bq).transpose(1, 2), torch.from_numpy(a_s).to(dev),
        torch.from_numpy(b_s).to(dev).transpose(1, 2), strides, strides, c_strides, lay(), lay(),
        torch.from_numpy(ps).to(dev), torch.from_numpy(offs[:-1].copy()).to(dev),
        torch.empty(workspace_bytes, device=dev, dtype=torch.uint8))
    return out


@pytest.mark.parametrize("E,N,K,lo,hi", [(8, 256, 512, 1, 20), (16, 512, 1024, 1, 256), (4, 1024, 384, 100, 400),
                                         (64, 256, 256, 0, 3), (3, 4096, 7168, 1, 9)])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float16])
def test_fp8_blockwise_scaled_grouped_mm(sa, dev, E, N, K, lo, hi, out_dtype):
    """Shapes after sgl-kernel/tests/test_fp8_blockwise_moe.py:109-213 (random rows per expert, n and k multiples
    of 128); the row ranges walk through every sorted-block height, empty experts included."""
    rng = np.random.default_rng(E + N)
    counts = rng.integers(lo, hi + 1, size=E).tolist()
    if lo == 0:
        counts[0] = 0
        counts[-1] = 0
    offs, ps, aq, a_s, bq, b_s = _grouped_case(E, N, K, counts, E * 3 + N, dev)
    ref = om.fp8_blockwise_scaled_grouped_mm(aq, a_s, bq, b_s, ps, offs[:-1], out_dtype=torch.float32)
    # a workspace too small for the schedule makes the op take its own
    out = _call_grouped(sa, dev, out_dtype, offs, ps, aq, a_s, bq, b_s, workspace_bytes=(1 << 22) if E != 8 else 16)
    assert_gemm_close(out, ref, f"E={E} N={N} K={K} rows={offs[-1]}")


def test_grouped_mm_rows_outside_every_span_are_left_alone(sa, dev):
    E, N, K = 4, 256, 256
    counts = [5, 0, 7, 3]
    offs, ps, aq, a_s, bq, b_s = _grouped_case(E, N, K, counts, 9, dev)
    ps2 = ps.copy()
    ps2[2, 0] = 4  # expert 2 is told to do fewer rows than its span holds
    out = _call_grouped(sa, dev, torch.bfloat16, offs, ps2, aq, a_s, bq, b_s)
    ref = om.fp8_blockwise_scaled_grouped_mm(aq, a_s, bq, b_s, ps2, offs[:-1], out_dtype=torch.float32)
    untouched = slice(int(offs[2]) + 4, int(offs[3]))
    assert bool((out[untouched] == 7.0).all())
    keep = np.ones(out.shape[0], dtype=bool)
    keep[untouched] = False
    assert_gemm_close(out[torch.from_numpy(keep).to(dev)], ref[torch.from_numpy(keep)], "partial span")
    with pytest.raises(RuntimeError, match="kFloat8_e4m3fn"):
        sa.fp8_blockwise_scaled_grouped_mm(out, *[torch.empty(E, device=dev, dtype=torch.int64)] * 5,
                                           torch.zeros(15, K, device=dev), torch.zeros(E, K, N, device=dev),
                                           torch.zeros(15, 2, device=dev), torch.zeros(E, 2, 2, device=dev),
                                           *[torch.zeros(E, device=dev, dtype=torch.int64)] * 3,
                                           *[torch.zeros(E, 5, device=dev, dtype=torch.int32)] * 2,
                                           torch.from_numpy(ps).to(dev), torch.from_numpy(offs[:-1].copy()).to(dev),
                                           torch.empty(16, device=dev, dtype=torch.uint8))


@pytest.mark.parametrize("M,H,I,E,topk", [(1, 512, 256, 8, 2), (33, 512, 256, 8, 2), (222, 768, 256, 24, 6),
                                           (600, 512, 256, 4, 2), (4, 7168, 2048, 8, 8)])
def test_cutlass_fused_experts_fp8(sa, dev, M, H, I, E, topk):
    from sglang_amd.moe_runner.cutlass_moe import cutlass_fused_experts_fp8

    g = torch.Generator().manual_seed(M + H + E)
    x = torch.randn(M, H, generator=g).to(torch.bfloat16)
    w13q, w13s, w2q, w2s = [], [], [], []
    for e in range(E):
        q, s = oq.block_quant_weight(torch.randn(2 * I, H, generator=g) * 0.02); w13q.append(q); w13s.append(s)
        q, s = oq.block_quant_weight(torch.randn(H, I, generator=g) * 0.02); w2q.append(q); w2s.append(s)
    w13q, w13s, w2q, w2s = np.stack(w13q), np.stack(w13s), np.stack(w2q), np.stack(w2s)
    tw, ti = om.topk_softmax(torch.randn(M, E, generator=g), topk, True)
    ref = om.cutlass_fused_experts_fp8(x, w13q, w2q, w13s, w2s, tw, ti)
    f8 = lambda a: torch.from_numpy(a).to(dev).view(torch.float8_e4m3fn)
    i64 = lambda v: torch.full((E,), v, device=dev, dtype=torch.int64)
    ptr = lambda: torch.empty(E, device=dev, dtype=torch.int64)
    out = cutlass_fused_experts_fp8(
        x.to(dev), f8(w13q).transpose(1, 2), f8(w2q).transpose(1, 2), torch.from_numpy(w13s).to(dev).transpose(1, 2),
        torch.from_numpy(w2s).to(dev).transpose(1, 2), tw.to(dev), ti.to(dev), i64(H), i64(2 * I), i64(I), i64(H),
        torch.empty(1 << 22, device=dev, dtype=torch.uint8), ptr(), ptr(), ptr(), ptr(), ptr(),
        torch.empty(E + 1, device=dev, dtype=torch.int32), torch.empty(E, 3, device=dev, dtype=torch.int32),
        torch.empty(E, 3, device=dev, dtype=torch.int32))
    assert out.shape == (M, H) and out.dtype == torch.bfloat16
    assert_gemm_close(out, ref.float(), f"grouped layer M={M} E={E} topk={topk}")
    # the sorted-block formulation computes the same layer
    assert_gemm_close(out, om.fused_moe_block_fp8(x, w13q, w2q, w13s, w2s, tw, ti, quant_form="reciprocal").float(),
                      "grouped vs sorted-block layer")
    # enable_es: the expert-specialisation operator in place of the plain one for either GEMM -- the same bits
    out_es = cutlass_fused_experts_fp8(
        x.to(dev), f8(w13q).transpose(1, 2), f8(w2q).transpose(1, 2), torch.from_numpy(w13s).to(dev).transpose(1, 2),
        torch.from_numpy(w2s).to(dev).transpose(1, 2), tw.to(dev), ti.to(dev), i64(H), i64(2 * I), i64(I), i64(H),
        torch.empty(1 << 22, device=dev, dtype=torch.uint8), ptr(), ptr(), ptr(), ptr(), ptr(),
        torch.empty(E + 1, device=dev, dtype=torch.int32), torch.empty(E, 3, device=dev, dtype=torch.int32),
        torch.empty(E, 3, device=dev, dtype=torch.int32), enable_es=(True, True))
    assert torch.equal(out_es, out)
    with pytest.raises(NotImplementedError):
        cutlass_fused_experts_fp8(x.to(dev), f8(w13q).transpose(1, 2), f8(w2q).transpose(1, 2), None, None, tw.to(dev),
                                  ti.to(dev), *[None] * 13, use_mxfp8=True)

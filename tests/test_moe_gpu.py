"""GPU parity of moe_align_block_size (bit-exact), silu_and_mul / moe_sum_reduce and the
block-FP8 fused MoE (tolerance) against the CPU oracle."""
import numpy as np
import pytest
import torch

from oracle import moe as om
from oracle import quant as oq
from tests.util import assert_gemm_close

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def sa(dev):
    import sglang_amd

    return sglang_amd


def _check_align(topk_ids: torch.Tensor, E: int, bs: int, dev, pad=True):
    from sglang_amd.moe import moe_align_block_size as op

    numel = topk_ids.numel()
    max_padded = om.max_num_tokens_padded(numel, E, bs)
    sorted_ids = torch.full((max_padded,), -7, dtype=torch.int32, device=dev)
    expert_ids = torch.full(((max_padded + bs - 1) // bs,), -7, dtype=torch.int32, device=dev)
    post = torch.empty(1, dtype=torch.int32, device=dev)
    cumsum = torch.empty(E + 2, dtype=torch.int32, device=dev)
    op(topk_ids.to(dev), E + 1, bs, sorted_ids, expert_ids, post, cumsum, pad)
    r_sorted, r_expert, r_post, r_cum = om.moe_align_block_size(topk_ids.numpy(), E + 1, bs, max_padded, pad)
    assert int(post.item()) == r_post
    nblk = r_post // bs
    assert np.array_equal(expert_ids.cpu().numpy()[:nblk], r_expert[:nblk])
    got = sorted_ids.cpu().numpy()
    if pad:
        assert np.array_equal(got, r_sorted)  # ascending order inside spans: fully deterministic
    else:
        valid = r_sorted != -1
        assert np.array_equal(got[valid], r_sorted[valid])
    assert np.array_equal(cumsum.cpu().numpy()[: E + 1], r_cum[: E + 1])


@pytest.mark.parametrize("bs", [16, 32, 64, 128, 256])
@pytest.mark.parametrize("tokens,topk,E", [(1, 8, 256), (32, 8, 256), (512, 8, 256), (4096, 8, 256), (7, 1, 64),
                                            (129, 2, 8), (1000, 6, 160), (33, 64, 64), (300, 4, 257), (64, 8, 264)])
def test_moe_align_block_size(sa, dev, bs, tokens, topk, E):
    g = torch.Generator().manual_seed(tokens * 131 + topk * 7 + E + bs)
    ids = torch.stack([torch.randperm(E, generator=g)[:topk] for _ in range(tokens)]).to(torch.int32)
    _check_align(ids, E, bs, dev)


def test_moe_align_edge_cases(sa, dev):
    g = torch.Generator().manual_seed(3)
    # filtered ids (-1), int64 ids, one hot expert, no padding fill
    ids = torch.randint(-1, 16, (257, 4), generator=g, dtype=torch.int64)
    _check_align(ids, 16, 64, dev)
    _check_align(ids.to(torch.int32), 16, 64, dev, pad=False)
    _check_align(torch.full((100, 2), 5, dtype=torch.int32), 8, 32, dev)
    _check_align(torch.full((3, 1), -1, dtype=torch.int32), 8, 16, dev)
    # many buckets (more than one scan round)
    ids = torch.randint(0, 1500, (700, 3), generator=g, dtype=torch.int32)
    _check_align(ids, 1500, 16, dev)


@pytest.mark.parametrize("tokens,experts,topk", [(1, 8, 2), (16, 64, 4), (33, 128, 6), (128, 256, 8), (257, 512, 8),
                                                   (5, 384, 5), (9, 160, 3), (3, 1000, 9)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_topk_softmax(sa, dev, tokens, experts, topk, dtype):
    """Shapes after sgl-kernel/tests/test_moe_topk_softmax.py:18-150 (powers of two up to 256, 512 and odd expert
    counts); ids exact, weights to fp32 rounding of a differently ordered sum."""
    g = torch.Generator().manual_seed(tokens * 1000 + experts)
    logits = torch.randn(tokens, experts, generator=g).to(dtype)
    for renorm in (False, True):
        w = torch.empty(tokens, topk, dtype=torch.float32, device=dev)
        ids = torch.empty(tokens, topk, dtype=torch.int32, device=dev)
        sa.topk_softmax(w, ids, logits.to(dev), renorm)
        rw, rids = om.topk_softmax(logits, topk, renorm)
        assert torch.equal(ids.cpu(), rids)
        torch.testing.assert_close(w.cpu(), rw, rtol=2e-5, atol=1e-9)


def test_topk_softmax_softcap_bias_ties_and_errors(sa, dev):
    g = torch.Generator().manual_seed(12)
    logits = torch.randn(40, 256, generator=g) * 3
    bias = torch.randn(256, generator=g)
    for cap, b in ((30.0, None), (0.0, bias), (2.0, bias)):
        w = torch.empty(40, 8, dtype=torch.float32, device=dev)
        ids = torch.empty(40, 8, dtype=torch.int32, device=dev)
        sa.topk_softmax(w, ids, logits.to(dev), True, cap, None if b is None else b.to(dev))
        rw, rids = om.topk_softmax(logits, 8, True, cap, b)
        assert torch.equal(ids.cpu(), rids)
        torch.testing.assert_close(w.cpu(), rw, rtol=5e-5, atol=1e-9)
    # equal logits: the lower expert index wins (moe_topk_softmax_kernels.cu:540-548)
    tied = torch.zeros(3, 128)
    tied[:, 70] = 1.0
    w = torch.empty(3, 4, dtype=torch.float32, device=dev)
    ids = torch.empty(3, 4, dtype=torch.int32, device=dev)
    sa.topk_softmax(w, ids, tied.to(dev), False)
    assert ids.cpu().tolist() == [[70, 0, 1, 2]] * 3
    with pytest.raises(RuntimeError, match="topk must be less than or equal to num_experts"):
        sa.topk_softmax(torch.empty(2, 9, device=dev), torch.empty(2, 9, dtype=torch.int32, device=dev),
                        torch.zeros(2, 8, device=dev), False)
    with pytest.raises(RuntimeError, match="correction_bias must be float32"):
        sa.topk_softmax(w, ids, tied.to(dev), False, 0.0, torch.zeros(128, dtype=torch.bfloat16, device=dev))
    with pytest.raises(RuntimeError, match="gating_output must be float32, float16, or bfloat16"):
        sa.topk_softmax(w, ids, tied.to(dev).double(), False)


def test_silu_and_mul_and_sum_reduce(sa, dev):
    g = torch.Generator().manual_seed(1)
    for dt in (torch.bfloat16, torch.float16):
        x = (torch.randn(37, 2 * 2048, generator=g) * 3).to(dt)
        out = sa.silu_and_mul(x.to(dev))
        ref = om.silu_and_mul(x)
        diff = (out.cpu().float() - ref.float()).abs()
        # expf differs by an ulp between libraries -> allow one storage-ulp on a few elements
        assert (diff > 0).float().mean() < 2e-2
        torch.testing.assert_close(out.cpu(), ref, rtol=1.6e-2, atol=1e-6)
        y = (torch.randn(19, 8, 7168, generator=g)).to(dt)
        o = torch.empty(19, 7168, dtype=dt, device=dev)
        sa.moe_sum_reduce(y.to(dev), o, 2.5)
        ref = (y.float().sum(dim=1) * 2.5).to(dt)
        torch.testing.assert_close(o.cpu(), ref, rtol=1e-2, atol=1e-2)
        assert (o.cpu() != ref).float().mean() < 1e-2


def _moe_case(M, H, I, E, topk, seed, dst="fp8"):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, H, generator=g).to(torch.bfloat16)
    logits = torch.randn(M, E, generator=g)
    w13 = torch.randn(E, 2 * I, H, generator=g) * 0.02
    w2 = torch.randn(E, H, I, generator=g) * 0.02
    w13q, w13s, w2q, w2s = [], [], [], []
    for e in range(E):
        q, s = oq.block_quant_weight(w13[e], dst=dst); w13q.append(q); w13s.append(s)
        q, s = oq.block_quant_weight(w2[e], dst=dst); w2q.append(q); w2s.append(s)
    tw, ti = om.topk_softmax(logits, topk, True)
    return x, np.stack(w13q), np.stack(w13s), np.stack(w2q), np.stack(w2s), tw, ti


@pytest.mark.parametrize("M,H,I,E,topk", [(1, 512, 256, 8, 2), (33, 512, 256, 8, 2), (64, 1024, 384, 16, 4),
                                           (222, 768, 256, 24, 6), (4, 7168, 2048, 8, 8)])
@pytest.mark.parametrize("block_m", [None, 16, 32, 64, 128, 192])
def test_fused_moe_block_fp8(sa, dev, M, H, I, E, topk, block_m):
    from tests.util import moe_layer as fused_moe

    if block_m in (16, 128, 192) and H == 7168:
        pytest.skip("large case runs with the default and 64")
    x, w13q, w13s, w2q, w2s, tw, ti = _moe_case(M, H, I, E, topk, M + H + E)
    ref = om.fused_moe_block_fp8(x, w13q, w2q, w13s, w2s, tw, ti, quant_form="reciprocal")
    f8 = lambda a: torch.from_numpy(a).to(dev).view(torch.float8_e4m3fn)
    cfg = None if block_m is None else {"BLOCK_SIZE_M": block_m}
    out = fused_moe(x.to(dev), f8(w13q), f8(w2q), (tw.to(dev), ti.to(dev), None), use_fp8_w8a8=True,
                    w1_scale=torch.from_numpy(w13s).to(dev), w2_scale=torch.from_numpy(w2s).to(dev),
                    block_shape=[128, 128], config=cfg)
    assert out.shape == (M, H) and out.dtype == torch.bfloat16
    assert_gemm_close(out, ref.float(), f"M={M} E={E} topk={topk} bm={block_m}")


@pytest.mark.parametrize("M,H,I,E,topk", [(1, 256, 128, 8, 2), (33, 512, 256, 8, 2), (64, 1024, 384, 24, 6),
                                           (222, 4096, 512, 8, 2), (520, 512, 256, 4, 1)])
@pytest.mark.parametrize("block_m", [None, 16, 32, 64, 128, 192])
def test_fused_moe_block_int8(sa, dev, M, H, I, E, topk, block_m):
    """Block-INT8 twin of the layer (shapes after test/registered/quant/test_block_int8.py:136-143): int8 weights
    with [128,128] scale blocks, activations group-quantised to int8 on both GEMM inputs; every sorted-block
    height, the default among them."""
    from tests.util import moe_layer as fused_moe

    if block_m in (16, 32, 192) and H == 4096:
        pytest.skip("large case runs with the default, 64 and 128")
    x, w13q, w13s, w2q, w2s, tw, ti = _moe_case(M, H, I, E, topk, M + H + E, dst="int8")
    ref = om.fused_moe_block_fp8(x, w13q, w2q, w13s, w2s, tw, ti, quant_form="reciprocal", int8=True)
    i8 = lambda a: torch.from_numpy(a).to(dev)
    cfg = None if block_m is None else {"BLOCK_SIZE_M": block_m}
    out = fused_moe(x.to(dev), i8(w13q), i8(w2q), (tw.to(dev), ti.to(dev), None), use_int8_w8a8=True,
                    w1_scale=torch.from_numpy(w13s).to(dev), w2_scale=torch.from_numpy(w2s).to(dev),
                    block_shape=[128, 128], config=cfg)
    assert out.shape == (M, H) and out.dtype == torch.bfloat16
    assert_gemm_close(out, ref.float(), f"int8 M={M} E={E} topk={topk} bm={block_m}")
    if block_m is None and M == 33:
        # no_combine returns the unweighted per-expert outputs; fp8 weights with the int8 flag are refused
        parts = fused_moe(x.to(dev), i8(w13q), i8(w2q), (tw.to(dev), ti.to(dev), None), use_int8_w8a8=True,
                          w1_scale=torch.from_numpy(w13s).to(dev), w2_scale=torch.from_numpy(w2s).to(dev),
                          block_shape=[128, 128], no_combine=True)
        assert_gemm_close((parts.float() * tw.to(dev).unsqueeze(-1)).sum(dim=1), out.float(), "int8 no_combine")
        with pytest.raises(AssertionError):
            fused_moe(x.to(dev), i8(w13q).view(torch.float8_e4m3fn), i8(w2q).view(torch.float8_e4m3fn),
                      (tw.to(dev), ti.to(dev), None), use_int8_w8a8=True, w1_scale=torch.from_numpy(w13s).to(dev),
                      w2_scale=torch.from_numpy(w2s).to(dev), block_shape=[128, 128])


def test_fused_moe_many_rows_per_expert_takes_the_192_slot_blocks(sa, dev):
    """Above 96 rows per expert the layer sorts into 192-slot blocks (one block per expert at ~128 rows); uneven
    routing makes some experts spill into a second block and leaves others nearly empty."""
    from tests.util import moe_layer as fused_moe

    M, H, I, E, topk = 520, 512, 256, 4, 1
    x, w13q, w13s, w2q, w2s, tw, ti = _moe_case(M, H, I, E, topk, 77)
    ti = ti.clone()
    ti[:300] = 2  # expert 2 gets > 192 rows, the others share the rest
    ref = om.fused_moe_block_fp8(x, w13q, w2q, w13s, w2s, tw, ti, quant_form="reciprocal")
    f8 = lambda a: torch.from_numpy(a).to(dev).view(torch.float8_e4m3fn)
    out = fused_moe(x.to(dev), f8(w13q), f8(w2q), (tw.to(dev), ti.to(dev), None), use_fp8_w8a8=True,
                    w1_scale=torch.from_numpy(w13s).to(dev), w2_scale=torch.from_numpy(w2s).to(dev),
                    block_shape=[128, 128])
    assert_gemm_close(out, ref.float(), "192-slot blocks")


@pytest.mark.parametrize("int8", [False, True])
@pytest.mark.parametrize("M,H,I,E,topk,hot", [(2048, 1024, 512, 32, 4, None), (1200, 1280, 640, 24, 6, 5),
                                               (2400, 768, 1152, 16, 2, None), (1500, 1280, 640, 24, 6, None)])
def test_fused_moe_more_192_slot_tiles_than_cus(sa, dev, int8, M, H, I, E, topk, hot, block_m=192):
    """Enough (sorted block, column tile) pairs that both GEMMs of the layer run the persistent walk: one workgroup
    per CU takes several tiles in turn, with a tile's first blocks requested under the epilogue of the tile before.
    Every expert gets well over 96 rows (192-slot blocks); `hot` sends a third of the tokens' first choice to one
    expert so that block counts differ between experts (256, 300 and 375 rows per expert on average: one full block
    and a part, or two).  In the FP8 layer the first GEMM's epilogue also applies the activation and its
    quantisation."""
    from tests.util import moe_layer as fused_moe

    dst = "int8" if int8 else "fp8"
    x, w13q, w13s, w2q, w2s, tw, ti = _moe_case(M, H, I, E, topk, M + E, dst=dst)
    ti = ti.clone()
    if hot is not None:
        ti[: M // 3, 0] = hot
        ti[: M // 3, 1:][ti[: M // 3, 1:] == hot] = (hot + 1) % E  # keep a token's experts distinct
    print(f"MoE with more tiles than CUs: M={M} H={H} I={I} E={E} topk={topk} int8={int8}", flush=True)
    ref = om.fused_moe_block_fp8(x, w13q, w2q, w13s, w2s, tw, ti, quant_form="reciprocal", int8=int8)
    conv = (lambda a: torch.from_numpy(a).to(dev)) if int8 else (lambda a: torch.from_numpy(a).to(dev).view(torch.float8_e4m3fn))
    kw = {"use_int8_w8a8": True} if int8 else {"use_fp8_w8a8": True}
    out = fused_moe(x.to(dev), conv(w13q), conv(w2q), (tw.to(dev), ti.to(dev), None), w1_scale=torch.from_numpy(w13s).to(dev),
                    w2_scale=torch.from_numpy(w2s).to(dev), block_shape=[128, 128], config={"BLOCK_SIZE_M": block_m}, **kw)
    assert_gemm_close(out, ref.float(), f"persistent MoE walk M={M} E={E} block_m={block_m}")


_LAYER_IN_A_CHILD = """
import sys, torch
sys.path.insert(0, {root!r})
from tests.test_moe_gpu import _moe_case
from tests.util import moe_layer
dev = torch.device("cuda:0")
x, w13q, w13s, w2q, w2s, tw, ti = _moe_case({M}, {H}, {I}, {E}, {topk}, {seed})
f8 = lambda a: torch.from_numpy(a).to(dev).view(torch.float8_e4m3fn)
out = moe_layer(x.to(dev).to({dtype}), f8(w13q), f8(w2q), (tw.to(dev), ti.to(dev), None), use_fp8_w8a8=True,
                w1_scale=torch.from_numpy(w13s).to(dev), w2_scale=torch.from_numpy(w2s).to(dev),
                block_shape=[128, 128], config={{"BLOCK_SIZE_M": {block_m}}})
torch.save(out.cpu(), {path!r})
"""


@pytest.mark.parametrize("M,H,I,E,topk,block_m,dtype", [(2048, 1024, 512, 32, 4, 192, torch.bfloat16),
                                                        (1200, 1280, 640, 24, 6, 192, torch.float16),
                                                        (1500, 768, 384, 32, 5, 128, torch.bfloat16),
                                                        (1100, 512, 1024, 16, 8, 128, torch.float16)])
def test_fused_activation_epilogue_gives_the_bits_of_the_separate_launches(sa, dev, tmp_path, M, H, I, E, topk, block_m,
                                                                           dtype):
    """Where the persistent walk runs the first GEMM of the one-call layer, its epilogue applies SiLU * up and the
    group quantisation itself.  The layer's output must be the bits of the sequence with the activation as a launch
    of its own, which a child process computes with SGLAMD_MOE_ACTQ=0 (the knob is read once per process)."""
    import os
    import subprocess
    import sys

    from tests.util import moe_layer

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    path = str(tmp_path / "separate.pt")
    code = _LAYER_IN_A_CHILD.format(root=root, M=M, H=H, I=I, E=E, topk=topk, seed=M + E, path=path, block_m=block_m,
                                    dtype=str(dtype))
    env = dict(os.environ, SGLAMD_MOE_ACTQ="0")
    r = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=280)
    assert r.returncode == 0, r.stderr[-2000:]
    separate = torch.load(path, weights_only=True)
    x, w13q, w13s, w2q, w2s, tw, ti = _moe_case(M, H, I, E, topk, M + E)
    f8 = lambda a: torch.from_numpy(a).to(dev).view(torch.float8_e4m3fn)
    out = moe_layer(x.to(dev).to(dtype), f8(w13q), f8(w2q), (tw.to(dev), ti.to(dev), None), use_fp8_w8a8=True,
                    w1_scale=torch.from_numpy(w13s).to(dev), w2_scale=torch.from_numpy(w2s).to(dev),
                    block_shape=[128, 128], config={"BLOCK_SIZE_M": block_m})
    assert out.dtype == dtype and separate.dtype == dtype
    assert torch.equal(out.cpu().view(torch.int16), separate.view(torch.int16))
    ref = om.fused_moe_block_fp8(x.to(dtype), w13q, w2q, w13s, w2s, tw, ti, quant_form="reciprocal")
    assert_gemm_close(out, ref.float(), f"fused activation epilogue M={M} block_m={block_m} {dtype}")


@pytest.mark.parametrize("block_m", [128, 64])
def test_fused_moe_more_shorter_tiles_than_cus(sa, dev, block_m):
    """The same with 128- and 64-slot blocks on a grid larger than the chip (two and one 32-row tile per wave)."""
    test_fused_moe_more_192_slot_tiles_than_cus(sa, dev, False, 2048, 1024, 512, 32, 4, None, block_m=block_m)
    test_fused_moe_more_192_slot_tiles_than_cus(sa, dev, True, 1200, 1280, 640, 24, 6, 5, block_m=block_m)
    test_fused_moe_more_192_slot_tiles_than_cus(sa, dev, False, 1500, 1280, 640, 24, 6, None, block_m=block_m)


def test_fused_moe_filtered_experts_and_scaling(sa, dev):
    """ids == -1 (expert lives on another rank) contribute zeros; routed_scaling_factor scales the sum."""
    from tests.util import moe_layer as fused_moe

    M, H, I, E, topk = 40, 512, 256, 8, 4
    x, w13q, w13s, w2q, w2s, tw, ti = _moe_case(M, H, I, E, topk, 99)
    ti = ti.clone()
    ti[ti >= 6] = -1
    ref = om.fused_moe_block_fp8(x, w13q, w2q, w13s, w2s, tw, ti, routed_scaling_factor=2.5, quant_form="reciprocal")
    f8 = lambda a: torch.from_numpy(a).to(dev).view(torch.float8_e4m3fn)
    out = fused_moe(x.to(dev), f8(w13q), f8(w2q), (tw.to(dev), ti.to(dev), None), use_fp8_w8a8=True,
                    w1_scale=torch.from_numpy(w13s).to(dev), w2_scale=torch.from_numpy(w2s).to(dev),
                    block_shape=[128, 128], routed_scaling_factor=2.5)
    assert_gemm_close(out, ref.float(), "filtered")


def test_fused_moe_unsupported_flags_raise(sa, dev):
    from tests.util import moe_layer as fused_moe

    x = torch.zeros(2, 256, device=dev, dtype=torch.bfloat16)
    w = torch.zeros(2, 256, 256, device=dev).to(torch.float8_e4m3fn)
    tk = (torch.ones(2, 1, device=dev), torch.zeros(2, 1, device=dev, dtype=torch.int32), None)
    with pytest.raises(AssertionError):                      # the reference's own assertion
        fused_moe(x, w.view(torch.int8), w.view(torch.int8), tk, use_int8_w8a8=True,
                  w1_scale=torch.ones(2, 256, device=dev), w2_scale=torch.ones(2, 256, device=dev))
    with pytest.raises(NotImplementedError):
        fused_moe(x, w, w, tk, use_fp8_w8a8=True, block_shape=[32, 32])
    with pytest.raises(NotImplementedError):
        fused_moe(x, w, w, tk)                              # unquantised experts
    with pytest.raises(NotImplementedError):
        fused_moe(x, w, w, tk, use_int8_w8a16=True)


def test_fused_silu_mul_group_quant(sa, dev):
    """fuse_silu_and_mul variant of the v2 quant op against oracle silu_and_mul -> group_quant(reciprocal).
    expf differs by an ulp between libraries, so a tiny fraction of one-code differences is allowed
    (criterion of sgl-kernel/python/sgl_kernel/test_utils.py:96-125)."""
    from sglang_amd.quantization.fp8_kernel import sglang_per_token_group_quant_fp8

    g = torch.Generator().manual_seed(8)
    x = (torch.randn(77, 2 * 2048, generator=g) * 2).to(torch.bfloat16)
    q, s = sglang_per_token_group_quant_fp8(x.to(dev), 128, fuse_silu_and_mul=True)
    assert q.shape == (77, 2048) and s.shape == (77, 16)
    act = om.silu_and_mul(x)
    rq, rs, _ = oq.group_quant(act, 128, form="reciprocal")
    got = q.cpu().view(torch.uint8).numpy()
    diff = np.abs((got & 0x7F).astype(int) - (rq & 0x7F).astype(int))
    assert diff.max() <= 1 and (diff > 0).mean() < 5e-3
    assert np.all(((got ^ rq) & 0x80 == 0) | ((got & 0x7F) <= 1) | ((rq & 0x7F) <= 1))
    np.testing.assert_allclose(s.cpu().numpy(), rs, rtol=1e-2)


@pytest.mark.parametrize("mode", ["balanced", "imbalanced", "extreme"])
def test_fused_silu_mul_group_quant_masked_layout(sa, dev, mode):
    """masked_m (DeepEP low-latency layout) of the v2 quant op, shapes and splits after
    sgl-kernel/tests/test_per_token_group_quant_8bit.py:63-102 and sgl_kernel/test_utils.py:20-60: only the first
    masked_m[e] tokens of expert e are written (the rest keeps its sentinel), scales are packed UE8M0 words in the
    per-expert column-major layout."""
    from sglang_amd.quantization.fp8_kernel import sglang_per_token_group_quant_fp8

    E, T, hidden, total = 6, 40, 512, 57
    g = torch.Generator().manual_seed(31)
    x = (torch.randn(E, T, 2 * hidden, generator=g) * 2).to(torch.bfloat16)
    if mode == "balanced":
        mm = [total // E + (1 if i < total % E else 0) for i in range(E)]
    elif mode == "imbalanced":
        mm = [0, 33, 1, 17, 40, 5]
    else:
        mm = [T] + [0] * (E - 1)
    masked_m = torch.tensor(mm, dtype=torch.int32)
    q, s = sglang_per_token_group_quant_fp8(x.to(dev), 128, column_major_scales=True, scale_tma_aligned=True,
                                            scale_ue8m0=True, fuse_silu_and_mul=True, masked_m=masked_m.to(dev))
    assert q.shape == (E, T, hidden) and s.shape == (E, T, 1) and s.dtype == torch.int32
    rq, reb, valid = oq.silu_mul_group_quant_masked(x, masked_m.numpy(), 128)
    got = q.cpu().view(torch.uint8).numpy()
    words = s.cpu().numpy().astype(np.uint32)
    got_eb = np.stack([(words[..., k // 4] >> (8 * (k % 4))) & 0xFF for k in range(hidden // 128)], axis=-1)
    v = valid
    # expf differs by an ulp between libraries: allow the reference test's tiny fraction of one-code differences
    diff = np.abs((got[v] & 0x7F).astype(int) - (rq[v] & 0x7F).astype(int))
    assert diff.max() <= 1 and (diff > 0).mean() < 5e-3
    assert np.mean(got_eb[v] != reb[v]) < 5e-3 and np.abs(got_eb[v].astype(int) - reb[v].astype(int)).max() <= 1

    # untouched region: run again on sentinel-filled outputs through the operator itself
    q2 = torch.full((E, T, hidden), 0x55, dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn)
    s2 = torch.full((E, 1, 40), 0x11111111, dtype=torch.int32, device=dev).transpose(-1, -2)
    torch.ops.sgl_kernel.sgl_per_token_group_quant_8bit_v2.default(x.to(dev), q2, s2, 128, 1e-10, -448.0, 448.0, True,
                                                                   True, masked_m.to(dev))
    q2h = q2.cpu().view(torch.uint8).numpy()
    s2h = s2.cpu().numpy()
    assert np.all(q2h[~v] == 0x55) and np.all(s2h[~v] == 0x11111111)
    assert np.array_equal(q2h[v], got[v])
    # 512/128 = 4 groups fill the word exactly
    assert np.array_equal(s2h[v].astype(np.uint32), words[v])


def test_fused_moe_no_combine_uses_the_op_by_op_path(sa, dev):
    from tests.util import moe_layer as fused_moe

    M, H, I, E, topk = 19, 512, 256, 8, 2
    x, w13q, w13s, w2q, w2s, tw, ti = _moe_case(M, H, I, E, topk, 5)
    f8 = lambda a: torch.from_numpy(a).to(dev).view(torch.float8_e4m3fn)
    kw = dict(use_fp8_w8a8=True, w1_scale=torch.from_numpy(w13s).to(dev), w2_scale=torch.from_numpy(w2s).to(dev),
              block_shape=[128, 128])
    full = fused_moe(x.to(dev), f8(w13q), f8(w2q), (tw.to(dev), ti.to(dev), None), **kw)
    parts = fused_moe(x.to(dev), f8(w13q), f8(w2q), (tw.to(dev), ti.to(dev), None), no_combine=True, **kw)
    assert parts.shape == (M, topk, H)
    # no_combine returns the unweighted per-expert outputs; weighting and summing them reproduces the layer
    recon = (parts.float() * tw.to(dev).unsqueeze(-1)).sum(dim=1)
    assert_gemm_close(recon, full.float(), "no_combine")
    # in-place variant writes the result into the input tensor
    xin = x.to(dev).clone()
    res = fused_moe(xin, f8(w13q), f8(w2q), (tw.to(dev), ti.to(dev), None), inplace=True, **kw)
    assert res.data_ptr() == xin.data_ptr() and torch.equal(res, full)


@pytest.mark.parametrize("M", [24, 1, 3])
def test_fused_moe_replayed_from_a_hip_graph_matches_eager(sa, dev, M):
    """The whole layer is capturable (no allocation outside torch's graph pool, no memset nodes, no host reads):
    every replay, with fresh inputs written into the captured tensors and eager work in between, equals the
    eager result bit for bit.  One and three tokens run the shorter launch sequences, whose routing is sorted
    inside the GEMMs from the ids the replay finds in the captured tensor."""
    from tests.util import moe_layer as fused_moe

    H, I, E, topk = 512, 256, 8, 2
    x, w13q, w13s, w2q, w2s, tw, ti = _moe_case(M, H, I, E, topk, 123)
    f8 = lambda a: torch.from_numpy(a).to(dev).view(torch.float8_e4m3fn)
    w13, w2 = f8(w13q), f8(w2q)
    kw = dict(use_fp8_w8a8=True, w1_scale=torch.from_numpy(w13s).to(dev), w2_scale=torch.from_numpy(w2s).to(dev),
              block_shape=[128, 128])
    xs, tws, tis = x.to(dev).clone(), tw.to(dev).clone(), ti.to(dev).clone()
    fused_moe(xs, w13, w2, (tws, tis, None), **kw)  # warm-up outside the capture
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            out_static = fused_moe(xs, w13, w2, (tws, tis, None), **kw)
    torch.cuda.synchronize()
    g = torch.Generator().manual_seed(7)
    for rep in range(4):
        xn = torch.randn(M, H, generator=g).to(torch.bfloat16).to(dev)
        twn, tin = om.topk_softmax(torch.randn(M, E, generator=g), topk, True)
        xs.copy_(xn)
        tws.copy_(twn.to(dev))
        tis.copy_(tin.to(dev))
        graph.replay()
        torch.cuda.synchronize()
        eager = fused_moe(xn, w13, w2, (twn.to(dev), tin.to(dev), None), **kw)  # eager work between replays
        torch.cuda.synchronize()
        assert torch.equal(out_static, eager), f"replay {rep}"


def _layer_by_its_kernel_sequence(x, w13, w13s, w2, w2s, tw, ti, dev):
    """The launches the fused layer entry point issues, one by one through the C ABI with caller-owned
    intermediates: align (16-slot blocks), group quant, grouped GEMM, silu*mul + group quant, grouped GEMM with the
    routing weights, top-k sum."""
    import ctypes

    from sglang_amd import ops
    from sglang_amd._lib import BF16, F16, FORM_RECIPROCAL, FP8_E4M3, SCALE_ROW_MAJOR, check, lib

    dt, tag = x.dtype, (BF16 if x.dtype == torch.bfloat16 else F16)

    M, H = x.shape
    E, N2, _ = w13.shape
    I, topk, T, bm = N2 // 2, ti.shape[1], ti.numel(), 16
    max_padded = om.max_num_tokens_padded(T, E, bm)
    sorted_ids = torch.empty(max_padded, dtype=torch.int32, device=dev)
    expert_ids = torch.empty((max_padded + bm - 1) // bm, dtype=torch.int32, device=dev)
    post = torch.empty(1, dtype=torch.int32, device=dev)
    cumsum = torch.empty(E + 2, dtype=torch.int32, device=dev)
    ops.moe_align_block_size(ti, E + 1, bm, sorted_ids, expert_ids, post, cumsum, True)
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    f = ctypes.c_float
    xq = torch.empty(M, H, dtype=torch.float8_e4m3fn, device=dev)
    xs = torch.empty(M, H // 128, dtype=torch.float32, device=dev)
    check(lib.sglamd_per_token_group_quant_8bit(x.data_ptr(), tag, xq.data_ptr(), FP8_E4M3, xs.data_ptr(), M, H, 128,
                                                SCALE_ROW_MAJOR, 0, f(1e-10), f(-448.0), f(448.0), FORM_RECIPROCAL, st))
    c1 = torch.empty(T, 2 * I, dtype=dt, device=dev)
    ops.fused_moe_block_fp8_gemm_(xq, xs, w13, w13s, c1, None, sorted_ids, expert_ids, post, False, topk, bm)
    aq = torch.empty(T, I, dtype=torch.float8_e4m3fn, device=dev)
    a_s = torch.empty(T, I // 128, dtype=torch.float32, device=dev)
    check(lib.sglamd_silu_mul_group_quant_8bit(c1.data_ptr(), tag, aq.data_ptr(), FP8_E4M3, a_s.data_ptr(), T, I, 128,
                                               SCALE_ROW_MAJOR, 0, f(1e-10), f(-448.0), f(448.0), FORM_RECIPROCAL, st))
    c3 = torch.empty(M, topk, H, dtype=dt, device=dev)
    ops.fused_moe_block_fp8_gemm_(aq, a_s, w2, w2s, c3, tw, sorted_ids, expert_ids, post, True, 1, bm)
    out = torch.empty(M, H, dtype=dt, device=dev)
    ops.moe_sum_reduce(c3, out, 1.0)
    return out


@pytest.mark.parametrize("M,H,I,E,topk,same", [(1, 1024, 512, 16, 4, False), (2, 1024, 512, 16, 4, False),
                                                (3, 512, 256, 8, 2, True), (4, 1024, 512, 16, 4, True),
                                                (4, 7168, 2048, 32, 8, False), (1, 7168, 2048, 32, 8, False),
                                                (1, 7168, 2048, 32, 8, "i64"), (1, 1024, 512, 16, 4, "elsewhere"),
                                                (2, 1024, 512, 16, 4, "elsewhere"), (1, 1024, 512, 16, 4, "f16"),
                                                (3, 1024, 512, 16, 4, "f16"), (5, 1024, 512, 16, 4, False),
                                                (1, 1024, 512, 16, 8, "repeated"), (1, 1024, 512, 16, 8, "one expert"),
                                                (1, 1024, 512, 16, 8, "repeated elsewhere"),
                                                (1, 512, 256, 4, 8, "one expert")])
def test_fused_moe_layer_equals_its_kernel_sequence_bit_for_bit(sa, dev, M, H, I, E, topk, same):
    """Up to four tokens the layer runs with fewer launches: the first GEMM writes silu(gate)*up itself, the second
    one quantises those rows itself, and for a single token both sort the routed pairs and the first one quantises
    the hidden state.  The result has to be the same bits as the full launch sequence (`same`: every token routed
    to the same experts, so a sorted block holds M rows; "i64": int64 ids; "elsewhere": two ids are -1, experts of
    another rank, whose rows count as zeros; "f16": half instead of bfloat16 activations; M = 5 is the first size
    that keeps every separate kernel; "repeated": the token names one expert five times, "one expert": eight
    times, "repeated elsewhere": five ids are -1 -- more pairs than the four rows of a block of the in-kernel
    sort; with 4 experts and top-k 8 the single token takes the launch in front again)."""
    from sglang_amd.ops import fused_moe_block_fp8_

    x, w13q, w13s, w2q, w2s, tw, ti = _moe_case(M, H, I, E, min(topk, E), 11 * M + H)
    if topk > E:  # more pairs than experts: only possible with repeated ids
        ti = ti[:, :1].repeat(1, topk).contiguous()
        tw = (torch.rand(M, topk, generator=torch.Generator().manual_seed(5)) / topk).to(tw.dtype)
    if same is True:
        ti = ti[:1].repeat(M, 1).contiguous()
    if same == "elsewhere":
        ti = ti.clone()
        ti[0, 1] = -1
        ti[-1, topk - 1] = -1
    if same == "repeated":
        ti = ti.clone()
        ti[0, [0, 2, 3, 5, 7]] = int(ti[0, 4])
    if same == "one expert":
        ti = torch.full_like(ti, int(ti[0, 0]))
    if same == "repeated elsewhere":
        ti = ti.clone()
        ti[0, [1, 2, 4, 6, 7]] = -1
    f8 = lambda a: torch.from_numpy(a).to(dev).view(torch.float8_e4m3fn)
    x, tw = x.to(dev), tw.to(dev).float().contiguous()
    if same == "f16":
        x = x.to(torch.float16)
    ti = ti.to(dev).to(torch.int64 if same == "i64" else torch.int32).contiguous()
    w13, w2 = f8(w13q), f8(w2q)
    w13s, w2s = torch.from_numpy(w13s).to(dev), torch.from_numpy(w2s).to(dev)
    want = _layer_by_its_kernel_sequence(x, w13, w13s, w2, w2s, tw, ti, dev)
    got = torch.empty_like(x)
    fused_moe_block_fp8_(x, w13, w2, w13s, w2s, tw, ti, got, 1.0, block_m=16)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    if same == "f16":
        return  # the oracle models bfloat16 intermediates
    ref = om.fused_moe_block_fp8(x.cpu(), w13q, w2q, w13s.cpu().numpy(), w2s.cpu().numpy(), tw.cpu(), ti.cpu(),
                                 quant_form="reciprocal")
    assert_gemm_close(got, ref.float(), f"M={M} fused activation quant")

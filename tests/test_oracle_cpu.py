"""CPU tests that pin the oracle: closed forms against library routines, invariants, special
cases that reduce to textbook results, brute force on tiny inputs, and the frozen golden vectors."""
import math
import os
from fractions import Fraction

import numpy as np
import pytest
import torch

from oracle import gemm as og
from oracle import moe as om
from oracle import quant as oq
from oracle.fp8 import e4m3fn_decode, e4m3fn_encode
from tests.util import outlier_input

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "config1.npz")


# ---- e4m3fn ----------------------------------------------------------------------------------
def test_e4m3_encode_matches_torch_cast_on_all_bf16_and_boundaries():
    bits = np.arange(65536, dtype=np.uint32) << 16
    v = bits.view(np.float32)
    v = v[np.isfinite(v) & (np.abs(v) <= 448)]
    t = torch.from_numpy(v).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(t, e4m3fn_encode(v))
    codes = np.arange(0, 0x7E, dtype=np.uint8)
    lo, hi = e4m3fn_decode(codes).astype(np.float64), e4m3fn_decode(codes + 1).astype(np.float64)
    mid = ((lo + hi) / 2).astype(np.float32)
    for d in (mid, np.nextafter(mid, np.float32(0)), np.nextafter(mid, np.float32(1e9)), -mid):
        t = torch.from_numpy(d).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
        assert np.array_equal(t, e4m3fn_encode(d))
    # ties go to the even code
    assert np.array_equal(e4m3fn_encode(mid), np.where(codes % 2 == 0, codes, codes + 1))


def test_e4m3_decode_encode_round_trip_and_known_values():
    codes = np.array([c for c in range(256) if (c & 0x7F) != 0x7F], dtype=np.uint8)
    assert np.array_equal(e4m3fn_encode(e4m3fn_decode(codes)) & 0x7F, codes & 0x7F)
    known = {0.3: 0.3125, 0.0019: 0.001953125, 448.0: 448.0, -448.0: -448.0, 2.0 ** -10: 0.0, 3 * 2.0 ** -10: 2.0 ** -8}
    for x, y in known.items():
        assert e4m3fn_decode(e4m3fn_encode(np.float32(x))) == np.float32(y)
    assert e4m3fn_encode(np.float32(np.nan)) & 0x7F == 0x7F


# ---- group quant -----------------------------------------------------------------------------
def _native_per_token_group_quant_fp8(x, group_size, eps=1e-10):
    """Line-by-line torch evaluation of test/manual/quant/test_block_fp8.py:55-64 (torch ops and torch's
    fp8 cast, not the oracle's numpy path)."""
    x_ = x.reshape(x.numel() // group_size, group_size)
    amax = x_.abs().max(dim=-1, keepdim=True)[0].clamp(min=eps).to(torch.float32)
    x_s = amax / 448.0
    x_q = (x_ / x_s).clamp(min=-448.0, max=448.0).to(torch.float8_e4m3fn)
    return x_q.reshape(x.shape), x_s.reshape(x.shape[:-1] + (x.shape[-1] // group_size,))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_group_quant_divide_equals_torch_native(dtype):
    x = outlier_input(64, 1024, dtype, 50.0)
    q, s, _ = oq.group_quant(x, 128)
    tq, ts = _native_per_token_group_quant_fp8(x, 128)
    assert np.array_equal(q, tq.view(torch.uint8).numpy())
    assert np.array_equal(s.view(np.uint32), ts.numpy().view(np.uint32))


def test_group_quant_invariants():
    x = outlier_input(128, 2048, torch.bfloat16, 50.0)
    x[5] = 0  # all-zero row
    q, s, _ = oq.group_quant(x, 128)
    x32 = x.float().numpy().reshape(128, 16, 128)
    deq = e4m3fn_decode(q).reshape(128, 16, 128) * s[..., None]
    # the arg-max element quantises to exactly +-448; the scale is a pure function of the amax
    am = np.abs(x32).argmax(-1)
    qa = np.take_along_axis(e4m3fn_decode(q).reshape(128, 16, 128), am[..., None], -1)[..., 0]
    nz = np.abs(x32).max(-1) > 0
    assert np.all(np.abs(qa[nz]) == 448.0)
    assert np.array_equal(s, (np.maximum(np.abs(x32).max(-1), np.float32(1e-10)) / np.float32(448)).astype(np.float32))
    # relative error <= 2^-4 in the normal range, absolute <= s * 2^-10 below it
    y = np.abs(x32 / s[..., None])
    err = np.abs(deq - x32)
    normal = y >= 2.0 ** -6
    assert np.all(err[normal] <= np.abs(x32[normal]) * (2.0 ** -4) * (1 + 1e-6))
    assert np.all(err[~normal] <= (s[..., None] * np.ones_like(x32))[~normal] * 2.0 ** -10 * (1 + 1e-6))
    # all-zero groups: scale 1e-10/448, zero bytes
    assert np.all(q[5] == 0) and np.all(s[5] == np.float32(1e-10) / np.float32(448))


def test_group_quant_recovers_exactly_representable_inputs():
    """Construction of test/registered/quant/test_fp8_kernel.py:34-57: x = q * s with q on the fp8 grid and
    the group maximum at 448 -> the quantiser must return q and s."""
    g = torch.Generator().manual_seed(0)
    rows, groups = 32, 8
    codes = torch.randint(0, 0x7F, (rows, groups, 128), generator=g, dtype=torch.int32).to(torch.uint8)
    sign = torch.randint(0, 2, codes.shape, generator=g, dtype=torch.int32).to(torch.uint8) << 7
    codes = (codes | sign).numpy()
    codes[..., 0] = 0x7E  # 448
    scale = (2.0 ** torch.randint(-8, 4, (rows, groups), generator=g)).numpy().astype(np.float32)
    x = torch.from_numpy(e4m3fn_decode(codes) * scale[..., None]).reshape(rows, -1)  # exact in fp32
    for form in ("divide", "reciprocal"):
        q, s, _ = oq.group_quant(x, 128, form=form)
        assert np.array_equal(s, scale)
        assert np.array_equal(q.reshape(codes.shape), codes), form  # signed zero keeps its sign bit


def test_group_quant_reciprocal_form_stays_within_one_code_and_one_ulp():
    x = outlier_input(256, 2048, torch.bfloat16, 50.0)
    q1, s1, _ = oq.group_quant(x, 128, form="divide")
    q2, s2, _ = oq.group_quant(x, 128, form="reciprocal")
    assert np.abs(s1.view(np.int32) - s2.view(np.int32)).max() <= 1
    d = np.abs((q1 & 0x7F).astype(int) - (q2 & 0x7F).astype(int))
    assert d.max() <= 1 and (d > 0).mean() < 5e-3
    assert np.array_equal(q1 & 0x80, q2 & 0x80) or np.all(((q1 ^ q2) & 0x80 == 0) | ((q1 & 0x7F) == 0) | ((q2 & 0x7F) == 0))


def test_ue8m0_brute_force_over_exponents_and_mantissa_edges():
    """scale = 2^ceil(log2(amax/448)), byte = biased exponent; checked with exact rational arithmetic."""
    vals = []
    for e in range(-60, 100):
        for man in (0, 1, 0x400000, 0x7FFFFF):
            bits = ((e + 127) << 23) | man
            vals.append(np.array([bits], dtype=np.uint32).view(np.float32)[0])
    amax = np.array(vals, dtype=np.float32)
    x = torch.zeros(len(vals), 128)
    x[:, 0] = torch.from_numpy(amax)
    for form in ("divide", "reciprocal"):
        q, s, e8 = oq.group_quant(x, 128, form=form, scale_ue8m0=True)
        for i, a in enumerate(amax):
            a = max(np.float32(a), np.float32(1e-10))  # the group maximum is floored at eps first
            y = (np.float32(a) / np.float32(448)) if form == "divide" else np.float32(np.float32(a) * (np.float32(1) / np.float32(448)))
            y = max(Fraction(float(y)), Fraction(float(np.float32(1e-10)))) if form == "divide" else Fraction(float(y))
            k = math.ceil(math.log2(y)) if y != 2 ** round(math.log2(y)) else round(math.log2(y))
            # exact: smallest k with 2^k >= y
            while Fraction(2) ** k < y:
                k += 1
            while Fraction(2) ** (k - 1) >= y:
                k -= 1
            assert s[i, 0] == np.float32(2.0 ** k), (form, a)
            assert int(e8[i, 0]) == k + 127
            # quantised maximum never exceeds 448 and uses at least half the range
            assert abs(float(e4m3fn_decode(q[i, 0]))) <= 448


def test_ue8m0_packing_layout():
    e = np.arange(3 * 6, dtype=np.uint8).reshape(3, 6) + 100
    p = oq.pack_ue8m0(e)
    assert p.shape == (3, 2) and p.dtype == np.int32
    assert p[1, 0] == int.from_bytes(bytes(e[1, :4]), "little")
    assert p[2, 1] == int.from_bytes(bytes(list(e[2, 4:6]) + [0, 0]), "little")


def test_int8_group_quant_truncates_toward_zero():
    x = torch.tensor([[127.0, -63.9, 63.9, 0.4, -0.9] + [0.0] * 123])
    q, s, _ = oq.group_quant(x, 128, dst="int8")
    assert s[0, 0] == np.float32(1.0)
    assert list(q[0, :5]) == [127, -63, 63, 0, 0]


def test_static_quant_equals_torch_evaluation_of_the_reference_expression():
    """The reference writes the same step as plain torch for the compiler path (fp8_utils.py:1497-1501):
    (input * scale.reciprocal()).clamp(min, max).to(fp8).  Evaluated on the CPU it pins the oracle: every finite
    bf16 value, several scales (a power of two, one that makes products land between codes, a tiny and a huge one)."""
    bits = torch.arange(0, 65536, dtype=torch.int32).to(torch.int16)
    x = bits.view(torch.bfloat16)
    x = x[torch.isfinite(x.float())].reshape(1, -1)
    x = torch.cat([x, outlier_input(1, x.shape[1], torch.bfloat16, 50.0)])
    for scale in (0.5, 0.0371, 1e-6, 3000.0, 1.0):
        s = torch.tensor([scale], dtype=torch.float32)
        want = (x * s.reciprocal()).clamp(min=-448.0, max=448.0).to(torch.float8_e4m3fn)
        q, rows = oq.static_quant_fp8(x, scale)
        assert np.array_equal(q, want.view(torch.uint8).numpy()), scale
        assert rows.shape == (2,) and np.all(rows == np.float32(scale))


def test_per_token_quant_closed_forms():
    x = outlier_input(16, 1024, torch.bfloat16, 50.0)
    x[3] = 0
    q, s = oq.per_token_quant_fp8(x)
    assert s[3] == 0 and np.all(q[3] == 0)
    x32 = x.float().numpy()
    assert np.array_equal(s, (np.abs(x32).max(-1) / np.float32(448)).astype(np.float32))
    am = np.abs(x32).argmax(-1)
    nz = s > 0
    assert np.all(np.abs(e4m3fn_decode(q)[np.arange(16), am])[nz] >= 416)  # x*(1/s) may land one code below 448
    qi, si = oq.per_token_quant_int8(x)
    assert np.all(np.abs(qi[np.arange(16), am][nz]) == 127)
    assert np.abs(qi.astype(np.float32) * si[:, None] - x32).max() <= si.max() * 0.5 * (1 + 1e-3)
    # round half away from zero
    y = torch.tensor([[127.0, 0.5, -0.5, 1.5, -2.5, 2.4999]])
    qy, _ = oq.per_token_quant_int8(y)
    assert list(qy[0]) == [127, 1, -1, 2, -3, 2]


# ---- GEMMs -------------------------------------------------------------------------------------
def test_block_gemm_special_cases():
    g = torch.Generator().manual_seed(2)
    M, N, K = 8, 256, 384
    xi = torch.randint(-8, 9, (M, K), generator=g).float()
    wi = torch.randint(-8, 9, (N, K), generator=g).float()
    xq, wq = e4m3fn_encode(xi.numpy()), e4m3fn_encode(wi.numpy())
    ones_a, ones_b = np.ones((M, 3), np.float32), np.ones((2, 3), np.float32)
    c = og.block_fp8_matmul(xq, wq, ones_a, ones_b, return_fp32=True)
    assert torch.equal(c, xi @ wi.t())  # unit scales: plain matmul of the fp8 values
    # one-hot rows read back weight rows times the block scale; a transposed or mis-indexed scale fails here
    oh = np.zeros((M, K), np.float32)
    ks = [(37 * m) % K for m in range(M)]
    for m, k in enumerate(ks):
        oh[m, k] = 1
    sb = (np.arange(1, 7, dtype=np.float32).reshape(2, 3)) / 8
    sa = (np.arange(1, M * 3 + 1, dtype=np.float32).reshape(M, 3)) / 4
    c = og.block_fp8_matmul(e4m3fn_encode(oh), wq, sa, sb, return_fp32=True)
    for m, k in enumerate(ks):
        exp = wi[:, k].numpy() * np.repeat(sb[:, k // 128], 128) * sa[m, k // 128]
        assert np.allclose(c[m].numpy(), exp, rtol=1e-6)


def test_block_gemm_equals_dequantise_then_matmul_float64():
    """Second formulation (baseline_scaled_mm, sgl-kernel/tests/test_fp8_blockwise_gemm.py:20-60): scale both
    operands elementwise, one float64 matmul."""
    g = torch.Generator().manual_seed(3)
    M, N, K = 17, 384, 640
    xq = e4m3fn_encode(((torch.rand(M, K, generator=g) - 0.5) * 2 * 448).numpy())
    wq = e4m3fn_encode(((torch.rand(N, K, generator=g) - 0.5) * 2 * 448).numpy())
    sa = (torch.rand(M, 5, generator=g) * 1e-2).numpy()
    sb = (torch.rand(3, 5, generator=g) * 1e-2).numpy()
    a = e4m3fn_decode(xq).astype(np.float64) * np.repeat(sa, 128, axis=1)
    b = e4m3fn_decode(wq).astype(np.float64) * np.repeat(np.repeat(sb, 128, axis=0), 128, axis=1)
    ref = a @ b.T
    c = og.block_fp8_matmul(xq, wq, sa, sb, return_fp32=True).numpy()
    assert np.abs(c - ref).max() <= 1e-5 * np.abs(ref).max()


def test_block_int8_gemm_exact_integer_and_scaled():
    """Unit scales: exact int64 matmul of the int8 operands (extreme values included).  Random scales:
    dequantise both operands elementwise in float64, one matmul -- a second formulation of
    native_w8a8_block_int8_matmul (test/registered/quant/test_block_int8.py:45-98).  K and N deliberately not
    multiples of 128 so the ragged last tiles are exercised."""
    g = torch.Generator().manual_seed(12)
    M, N, K = 11, 200, 400
    aq = torch.randint(-128, 128, (M, K), generator=g, dtype=torch.int32).numpy().astype(np.int8)
    bq = torch.randint(-128, 128, (N, K), generator=g, dtype=torch.int32).numpy().astype(np.int8)
    aq[0, :] = -128
    bq[0, :] = -128
    kb, nb = 4, 2
    c = og.block_int8_matmul(aq, bq, np.ones((M, kb), np.float32), np.ones((nb, kb), np.float32), return_fp32=True)
    exact = aq.astype(np.int64) @ bq.astype(np.int64).T
    assert np.array_equal(c.numpy().astype(np.int64), exact)  # |sum| <= 400 * 2^14 < 2^24: fp32 holds it exactly
    sa = (torch.rand(M, kb, generator=g) * 1e-2).numpy()
    sb = (torch.rand(nb, kb, generator=g) * 1e-2).numpy()
    a = aq.astype(np.float64) * np.repeat(sa, 128, axis=1)[:, :K]
    b = bq.astype(np.float64) * np.repeat(np.repeat(sb, 128, axis=0), 128, axis=1)[:N, :K]
    ref = a @ b.T
    c = og.block_int8_matmul(aq, bq, sa, sb, return_fp32=True).numpy()
    assert np.abs(c - ref).max() <= 1e-5 * np.abs(ref).max()
    # one-hot rows read back scaled weight rows: a transposed or mis-indexed scale fails here
    oh = np.zeros((M, K), np.int8)
    ks = [(37 * m) % K for m in range(M)]
    for m, k in enumerate(ks):
        oh[m, k] = 1
    c = og.block_int8_matmul(oh, bq, sa, sb, return_fp32=True).numpy()
    for m, k in enumerate(ks):
        exp = bq[:, k].astype(np.float32) * np.repeat(sb[:, k // 128], 128)[:N] * sa[m, k // 128]
        assert np.allclose(c[m], exp, rtol=1e-6)


def test_rowwise_gemms():
    g = torch.Generator().manual_seed(4)
    M, N, K = 9, 40, 96
    aq = torch.randint(-128, 128, (M, K), generator=g, dtype=torch.int32).numpy().astype(np.int8)
    bq = torch.randint(-128, 128, (N, K), generator=g, dtype=torch.int32).numpy().astype(np.int8)
    sa, sb = np.ones(M, np.float32), np.ones(N, np.float32)
    exact = np.array([[sum(int(aq[m, k]) * int(bq[n, k]) for k in range(K)) for n in range(N)] for m in range(M)])
    c = og.int8_scaled_mm(aq, bq, sa, sb, return_fp32=True)
    assert np.array_equal(c.numpy(), exact.astype(np.float32))
    bias = torch.arange(N, dtype=torch.float32).to(torch.bfloat16)
    sa2 = np.linspace(0.5, 2, M).astype(np.float32)
    sb2 = np.linspace(0.1, 1, N).astype(np.float32)
    c2 = og.int8_scaled_mm(aq, bq, sa2, sb2, bias=bias, return_fp32=True)
    assert np.allclose(c2.numpy(), exact * sa2[:, None] * sb2[None, :] + bias.float().numpy()[None], rtol=1e-6)
    # above 2^27 multiply-adds the oracle accumulates in float64 instead of int64: the same exact integers
    # (extreme values on a long K, where a fp32 accumulator would already round)
    Mb, Nb, Kb = 5, 13, 2 ** 21 + 64
    ab = torch.randint(-128, 128, (Mb, Kb), generator=g, dtype=torch.int32).numpy().astype(np.int8)
    bb = torch.randint(-128, 128, (Nb, Kb), generator=g, dtype=torch.int32).numpy().astype(np.int8)
    ab[0], bb[0] = -128, -128  # |acc| = K * 2^14 = 2^35 + 2^20: not representable in fp32's 24 bits
    big = og.int8_scaled_mm(ab, bb, np.ones(Mb, np.float32), np.ones(Nb, np.float32), return_fp32=True)
    want = torch.from_numpy(ab.astype(np.int64)) @ torch.from_numpy(bb.astype(np.int64)).t()
    assert Mb * Nb * Kb > (1 << 27) and int(want[0, 0]) == Kb * 16384
    assert torch.equal(big, want.to(torch.float32))
    # fp8: unit scales -> exact small-integer matmul, bias added before the cast
    xi = torch.randint(-8, 9, (M, K), generator=g).float()
    wi = torch.randint(-8, 9, (N, K), generator=g).float()
    c3 = og.fp8_scaled_mm(e4m3fn_encode(xi.numpy()), e4m3fn_encode(wi.numpy()), sa, sb, bias=bias, return_fp32=True)
    assert torch.equal(c3, xi @ wi.t() + bias.float()[None])


# ---- MoE ---------------------------------------------------------------------------------------
def _brute_align(ids, nb, bs):
    flat = [int(v) + 1 for v in np.asarray(ids).reshape(-1)]
    spans = []
    for b in range(nb):
        members = [i for i, v in enumerate(flat) if v == b]
        pad = (-len(members)) % bs
        spans.append((b - 1, members + [len(flat)] * pad))
    sorted_ids = [t for _, sp in spans for t in sp]
    expert_ids = [e for e, sp in spans for _ in range(len(sp) // bs)]
    return sorted_ids, expert_ids


@pytest.mark.parametrize("bs", [1, 4, 16])
def test_moe_align_brute_force_and_invariants(bs):
    g = torch.Generator().manual_seed(bs)
    for tokens, topk, E in [(1, 2, 4), (5, 3, 6), (40, 4, 9), (64, 8, 256)]:
        ids = torch.randint(-1, E, (tokens, topk), generator=g).numpy()
        mp = om.max_num_tokens_padded(ids.size, E, bs)
        s, e, post, _ = om.moe_align_block_size(ids, E + 1, bs, mp)
        bs_sorted, bs_expert = _brute_align(ids, E + 1, bs)
        assert post == len(bs_sorted) and post <= mp
        assert list(s[:post]) == bs_sorted and np.all(s[post:] == ids.size)
        assert list(e[: post // bs]) == bs_expert
        # invariants the reference's own test checks (sgl-kernel/tests/test_moe_align.py:233-255)
        assert sorted(int(v) for v in s[:post] if v < ids.size) == list(range(ids.size))
        assert np.all(np.diff(e[: post // bs]) >= 0)


def test_moe_align_docstring_example():
    ids = np.array([[2, 3, 4], [1, 2, 4], [1, 3, 4], [1, 2, 3]])
    s, e, post, _ = om.moe_align_block_size(ids, 6, 4, om.max_num_tokens_padded(12, 5, 4))
    # moe_align_block_size.py:47-52 of the reference wrapper
    assert list(s[:post]) == [3, 6, 9, 12, 0, 4, 10, 12, 1, 7, 11, 12, 2, 5, 8, 12]
    assert post == 16 and list(e[:4]) == [1, 2, 3, 4]


def _tiny_moe(M, H, I, E, seed, dst="fp8"):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, H, generator=g).to(torch.bfloat16)
    w13 = [oq.block_quant_weight(torch.randn(2 * I, H, generator=g) * 0.05, dst=dst) for _ in range(E)]
    w2 = [oq.block_quant_weight(torch.randn(H, I, generator=g) * 0.05, dst=dst) for _ in range(E)]
    return (x, np.stack([q for q, _ in w13]), np.stack([q for q, _ in w2]), np.stack([s for _, s in w13]),
            np.stack([s for _, s in w2]))


@pytest.mark.parametrize("int8", [False, True])
def test_fused_moe_top1_equals_dense_mlp_and_permutation_equivariance(int8):
    M, H, I, E = 6, 256, 128, 3
    dst = "int8" if int8 else "fp8"
    mm = og.block_int8_matmul if int8 else og.block_fp8_matmul
    x, w13q, w2q, w13s, w2s = _tiny_moe(M, H, I, E, 0, dst)
    ids = torch.tensor([[1]] * M, dtype=torch.int32)
    w = torch.ones(M, 1)
    out = om.fused_moe_block_fp8(x, w13q, w2q, w13s, w2s, w, ids, int8=int8)
    xq, xs, _ = oq.group_quant(x, 128, dst=dst)
    h = mm(xq, w13q[1], xs, w13s[1], out_dtype=torch.bfloat16)
    a = torch.nn.functional.silu(h[:, :I]) * h[:, I:]
    aq, as_, _ = oq.group_quant(a, 128, dst=dst)
    dense = mm(aq, w2q[1], as_, w2s[1], out_dtype=torch.bfloat16)
    assert torch.equal(out, dense)
    # the quantised layer tracks the unquantised one: dequantised weights, fp32 activations throughout
    w13f = torch.from_numpy((e4m3fn_decode(w13q[1]) if not int8 else w13q[1].astype(np.float32))
                            * np.repeat(np.repeat(w13s[1], 128, 0), 128, 1))
    w2f = torch.from_numpy((e4m3fn_decode(w2q[1]) if not int8 else w2q[1].astype(np.float32))
                           * np.repeat(np.repeat(w2s[1], 128, 0), 128, 1))
    hf = x.float() @ w13f.t()
    full = (torch.nn.functional.silu(hf[:, :I]) * hf[:, I:]) @ w2f.t()
    assert float((out.float() - full).norm() / full.norm()) < 0.06  # int8 activations truncate toward zero: ~4 %
    # permuting tokens permutes outputs
    logits = torch.randn(M, E, generator=torch.Generator().manual_seed(1))
    tw, ti = om.topk_softmax(logits, 2)
    perm = torch.randperm(M, generator=torch.Generator().manual_seed(2))
    o1 = om.fused_moe_block_fp8(x, w13q, w2q, w13s, w2s, tw, ti, int8=int8)
    o2 = om.fused_moe_block_fp8(x[perm], w13q, w2q, w13s, w2s, tw[perm], ti[perm], int8=int8)
    assert torch.equal(o1[perm], o2)
    assert torch.allclose(tw.sum(-1), torch.ones(M))


def _native_w8a8_block_fp8_matmul(A, B, As, Bs, block_size, output_dtype):
    """Line-by-line torch evaluation of native_w8a8_block_fp8_matmul, test/manual/quant/test_block_fp8.py:291-343
    (torch ops on torch tensors, not the oracle's numpy path)."""
    A = A.to(torch.float32)
    B = B.to(torch.float32)
    assert A.shape[-1] == B.shape[-1]
    assert B.ndim == 2 and B.is_contiguous() and Bs.ndim == 2
    block_n, block_k = block_size
    assert (A.shape[-1] + block_k - 1) // block_k == As.shape[-1]
    assert A.shape[:-1] == As.shape[:-1]
    M = A.numel() // A.shape[-1]
    N, K = B.shape
    origin_C_shape = A.shape[:-1] + (N,)
    A = A.reshape(M, A.shape[-1])
    As = As.reshape(M, As.shape[-1])
    n_tiles = (N + block_n - 1) // block_n
    k_tiles = (K + block_k - 1) // block_k
    C = torch.zeros((M, N), dtype=torch.float32)
    A_tiles = [A[:, i * block_k:min((i + 1) * block_k, K)] for i in range(k_tiles)]
    B_tiles = [[B[j * block_n:min((j + 1) * block_n, N), i * block_k:min((i + 1) * block_k, K)]
                for i in range(k_tiles)] for j in range(n_tiles)]
    C_tiles = [C[:, j * block_n:min((j + 1) * block_n, N)] for j in range(n_tiles)]
    As_tiles = [As[:, i:i + 1] for i in range(k_tiles)]
    for i in range(k_tiles):
        for j in range(n_tiles):
            a, b, c = A_tiles[i], B_tiles[j][i], C_tiles[j]
            s = As_tiles[i] * Bs[j][i]
            c[:, :] += torch.matmul(a, b.t()) * s
    return C.reshape(origin_C_shape).to(output_dtype)


def _torch_w8a8_block_fp8_moe(a, w1, w2, w1_s, w2_s, score, topk, block_shape):
    """Line-by-line torch evaluation of torch_w8a8_block_fp8_moe, test/manual/quant/test_block_fp8.py:518-547
    (SiluAndMul.forward_native = F.silu(x[..., :d]) * x[..., d:])."""
    B, D = a.shape
    a = a.view(B, -1, D).repeat(1, topk, 1).reshape(-1, D)
    out = torch.zeros(B * topk, w2.shape[1], dtype=a.dtype)
    score = torch.softmax(score, dim=-1, dtype=torch.float32)
    topk_weight, topk_ids = torch.topk(score, topk)
    topk_weight = topk_weight.view(-1)
    topk_ids = topk_ids.view(-1)
    _, block_k = block_shape[0], block_shape[1]
    a_q, a_s = _native_per_token_group_quant_fp8(a, block_k)
    a_q = a_q.to(torch.float32)
    for i in range(w1.shape[0]):
        mask = topk_ids == i
        if mask.sum():
            inter_out = _native_w8a8_block_fp8_matmul(a_q[mask], w1[i], a_s[mask], w1_s[i], block_shape, a.dtype)
            d = inter_out.shape[-1] // 2
            act_out = torch.nn.functional.silu(inter_out[..., :d]) * inter_out[..., d:]
            act_out_q, act_out_s = _native_per_token_group_quant_fp8(act_out, block_k)
            out[mask] = _native_w8a8_block_fp8_matmul(act_out_q, w2[i], act_out_s, w2_s[i], block_shape, a.dtype)
    return (out.view(B, -1, w2.shape[1]) * topk_weight.view(B, -1, 1).to(out.dtype)).sum(dim=1), topk_weight, topk_ids


@pytest.mark.parametrize("M,H,I,E,topk", [(33, 256, 128, 8, 2), (7, 512, 256, 8, 6), (64, 384, 128, 24, 6)])
def test_fused_moe_topk_gt1_against_the_reference_tests_torch_model(M, H, I, E, topk):
    """Direct pin of om.fused_moe_block_fp8 for top-k > 1: the reference test's own torch model evaluated line by
    line on torch tensors (recipe of test_block_fp8.py:567-611: a = randn / 10, routing by softmax + topk without
    renormalisation).  The model rounds each expert's output to bf16 and then multiplies by a bf16 routing weight
    and sums in bf16; the oracle follows the fused kernels (weight on the fp32 accumulator, fp32 sum), so the two
    differ by a few bf16 roundings per output: rel-L2 a few 1e-3, and the reference test's own criterion
    (mean |diff| / mean |ref| < 0.02, :623) holds with a wide margin.  A dropped routing weight, a wrong expert or
    a missing SiLU changes the result by tens of percent."""
    g = torch.Generator().manual_seed(M + H + E + topk)
    a = (torch.randn(M, H, generator=g) / 10).to(torch.bfloat16)
    w1 = [oq.block_quant_weight(torch.randn(2 * I, H, generator=g) * 0.05) for _ in range(E)]
    w2 = [oq.block_quant_weight(torch.randn(H, I, generator=g) * 0.05) for _ in range(E)]
    w1q, w1s = np.stack([q for q, _ in w1]), np.stack([s for _, s in w1])
    w2q, w2s = np.stack([q for q, _ in w2]), np.stack([s for _, s in w2])
    score = torch.randn(M, E, generator=g)
    f8 = lambda c: torch.from_numpy(c).view(torch.float8_e4m3fn)  # noqa: E731
    ref, tw, ti = _torch_w8a8_block_fp8_moe(a, f8(w1q), f8(w2q), torch.from_numpy(w1s), torch.from_numpy(w2s), score,
                                            topk, [128, 128])
    out = om.fused_moe_block_fp8(a, w1q, w2q, w1s, w2s, tw.view(M, topk), ti.view(M, topk).to(torch.int32),
                                 quant_form="divide")
    o, r = out.float(), ref.float()
    assert float((o - r).abs().mean() / r.abs().mean()) < 0.02
    assert float((o - r).norm() / r.norm()) < 8e-3
    # the routing weight matters at this size: leaving it out is far outside the bound
    flat = om.fused_moe_block_fp8(a, w1q, w2q, w1s, w2s, torch.ones(M, topk), ti.view(M, topk).to(torch.int32))
    assert float((flat.float() - r).norm() / r.norm()) > 0.3


@pytest.mark.parametrize("block", [[64, 64], [64, 128], [128, 64]])
def test_fused_moe_other_block_shapes_against_the_reference_tests_torch_model(block):
    """The same pin for the scale-block shapes the reference's test sweeps besides [128, 128]
    (test_block_fp8.py:557): the torch model evaluated line by line with that block_shape."""
    M, H, I, E, topk = 24, 256, 128, 8, 2
    g = torch.Generator().manual_seed(block[0] * 7 + block[1])
    a = (torch.randn(M, H, generator=g) / 10).to(torch.bfloat16)
    w1 = [oq.block_quant_weight(torch.randn(2 * I, H, generator=g) * 0.05, block=tuple(block)) for _ in range(E)]
    w2 = [oq.block_quant_weight(torch.randn(H, I, generator=g) * 0.05, block=tuple(block)) for _ in range(E)]
    w1q, w1s = np.stack([q for q, _ in w1]), np.stack([s for _, s in w1])
    w2q, w2s = np.stack([q for q, _ in w2]), np.stack([s for _, s in w2])
    score = torch.randn(M, E, generator=g)
    f8 = lambda c: torch.from_numpy(c).view(torch.float8_e4m3fn)  # noqa: E731
    ref, tw, ti = _torch_w8a8_block_fp8_moe(a, f8(w1q), f8(w2q), torch.from_numpy(w1s), torch.from_numpy(w2s), score,
                                            topk, block)
    out = om.fused_moe_block_fp8(a, w1q, w2q, w1s, w2s, tw.view(M, topk), ti.view(M, topk).to(torch.int32),
                                 block=tuple(block), quant_form="divide")
    o, r = out.float(), ref.float()
    assert float((o - r).abs().mean() / r.abs().mean()) < 0.02
    assert float((o - r).norm() / r.norm()) < 8e-3
    # the block shape matters: evaluating with [128, 128] scales indexing is not even shape-compatible, and a
    # transposed block (bn, bk swapped) on a non-square shape is far off
    if block[0] != block[1]:
        with pytest.raises(AssertionError):
            om.fused_moe_block_fp8(a, w1q, w2q, w1s, w2s, tw.view(M, topk), ti.view(M, topk).to(torch.int32),
                                   block=(block[1], block[0]))


def _native_w8a8_per_token_matmul(A, B, As, Bs, output_dtype):
    """Line-by-line torch evaluation of native_w8a8_per_token_matmul, test/registered/quant/test_int8_kernel.py:17-36."""
    A = A.to(torch.float32)
    B = B.to(torch.float32)
    assert A.shape[-1] == B.shape[-1]
    M = A.numel() // A.shape[-1]
    B = B.t()
    N, K = B.shape
    A = A.reshape(M, N)
    C = torch.matmul(A, B)
    C = As * C * Bs.view(1, -1)
    return C.to(output_dtype)


@pytest.mark.parametrize("int8", [True, False])
def test_row_scaled_moe_against_the_reference_tests_torch_model(int8):
    """om.fused_moe_row_scaled against torch_w8a8_per_column_moe (test_int8_kernel.py:39-79) evaluated line by line
    (per-token quantisation by the reference's formula, round() for int8; the FP8 twin quantises with
    max|x| / 448 per token as sgl_per_token_quant_fp8 does).  As for the block form the model applies the routing
    weight to bf16 outputs and sums in bf16, the oracle on the fp32 result with an fp32 sum."""
    M, H, I, E, topk = 33, 256, 128, 8, 2
    g = torch.Generator().manual_seed(5 + int(int8))
    a = (torch.randn(M, H, generator=g) / 10).to(torch.bfloat16)
    dst = "int8" if int8 else "fp8"
    w1 = [oq.per_channel_quant_weight(torch.randn(2 * I, H, generator=g) * 0.05, dst) for _ in range(E)]
    w2 = [oq.per_channel_quant_weight(torch.randn(H, I, generator=g) * 0.05, dst) for _ in range(E)]
    w1q, w1s = np.stack([q for q, _ in w1]), np.stack([s for _, s in w1])
    w2q, w2s = np.stack([q for q, _ in w2]), np.stack([s for _, s in w2])
    score = torch.softmax(torch.randn(M, E, generator=g), dim=-1, dtype=torch.float32)
    tw, ti = torch.topk(score, topk)

    def quant(t):
        t32 = t.to(torch.float32)
        if int8:
            amax = t32.abs().amax(dim=-1, keepdim=True).clamp_min(1e-10)
            scale = amax / 127.0
            y = t32 * (127.0 / amax)
            return torch.where(y >= 0, torch.floor(y + 0.5), -torch.floor(-y + 0.5)).to(torch.int8).to(torch.float32), scale
        amax = t32.abs().amax(dim=-1, keepdim=True)
        scale = amax / 448.0
        inv = torch.where(scale == 0, torch.zeros_like(scale), 1.0 / scale)
        return (t32 * inv).clamp(-448, 448).to(torch.float8_e4m3fn).to(torch.float32), scale

    def dq(c):
        return torch.from_numpy(c.astype(np.float32)) if int8 else torch.from_numpy(c).view(torch.float8_e4m3fn).to(torch.float32)

    a_rep = a.view(M, -1, H).repeat(1, topk, 1).reshape(-1, H)
    a_q, a_s = quant(a_rep)
    out = torch.zeros(M * topk, H, dtype=a.dtype)
    flat_ids = ti.reshape(-1)
    for i in range(E):
        mask = flat_ids == i
        if mask.sum():
            inter = _native_w8a8_per_token_matmul(a_q[mask], dq(w1q[i]), a_s[mask], torch.from_numpy(w1s[i]), a.dtype)
            d = inter.shape[-1] // 2
            act = torch.nn.functional.silu(inter[..., :d]) * inter[..., d:]
            act_q, act_s = quant(act)
            out[mask] = _native_w8a8_per_token_matmul(act_q, dq(w2q[i]), act_s, torch.from_numpy(w2s[i]), a.dtype)
    ref = (out.view(M, -1, H) * tw.view(M, -1, 1).to(out.dtype)).sum(dim=1)
    got = om.fused_moe_row_scaled(a, w1q, w2q, w1s, w2s, tw, ti.to(torch.int32), int8=int8)
    o, r = got.float(), ref.float()
    assert float((o - r).abs().mean() / r.abs().mean()) < 0.02
    assert float((o - r).norm() / r.norm()) < 8e-3
    flat = om.fused_moe_row_scaled(a, w1q, w2q, w1s, w2s, torch.ones(M, topk), ti.to(torch.int32), int8=int8)
    assert float((flat.float() - r).norm() / r.norm()) > 0.3


def test_row_scaled_moe_special_cases():
    """Top-1 with weight 1 is a dense two-layer MLP per expert; biases enter after the scales; per-tensor static
    scales equal per-channel scales that happen to be constant; the routing weight on the input of a top-1 layer
    scales the first GEMM's result."""
    M, H, I, E = 9, 128, 64, 3
    g = torch.Generator().manual_seed(77)
    x = torch.randn(M, H, generator=g).to(torch.bfloat16)
    w13 = torch.randn(E, 2 * I, H, generator=g) * 0.05
    w2 = torch.randn(E, H, I, generator=g) * 0.05
    q13, s13 = zip(*(oq.per_channel_quant_weight(w13[e], "fp8") for e in range(E)))
    q2, s2 = zip(*(oq.per_channel_quant_weight(w2[e], "fp8") for e in range(E)))
    q13, s13, q2, s2 = np.stack(q13), np.stack(s13), np.stack(q2), np.stack(s2)
    ids = torch.randint(0, E, (M, 1), generator=g).to(torch.int32)
    ones = torch.ones(M, 1)
    out = om.fused_moe_row_scaled(x, q13, q2, s13, s2, ones, ids)
    for t in range(M):
        e = int(ids[t, 0])
        xq, xs = oq.per_token_quant_fp8(x[t:t + 1])
        h = og.fp8_scaled_mm(xq, q13[e], xs, s13[e], out_dtype=torch.bfloat16)
        act = om.silu_and_mul(h)
        aq, a_s = oq.per_token_quant_fp8(act)
        y = og.fp8_scaled_mm(aq, q2[e], a_s, s2[e], out_dtype=torch.bfloat16)
        assert torch.equal(out[t], y[0])
    # bias: zero weights leave exactly silu(b1_gate) * b1_up pushed through w2 = 0 plus b2
    b1 = (torch.randn(E, 2 * I, generator=g)).to(torch.bfloat16)
    b2 = (torch.randn(E, H, generator=g)).to(torch.bfloat16)
    zero13, zero2 = np.zeros_like(q13), np.zeros_like(q2)
    outb = om.fused_moe_row_scaled(x, zero13, zero2, s13, s2, ones, ids, b1=b1, b2=b2)
    assert torch.equal(outb, b2[ids[:, 0].long()])
    # per-tensor static scales == constant per-channel scales with the same static activation quantisation
    c13, c2 = np.full(E, 3e-4, dtype=np.float32), np.full(E, 2e-4, dtype=np.float32)
    a = om.fused_moe_row_scaled(x, q13, q2, c13, c2, ones, ids, a1_scale=0.02, a2_scale=0.001)
    b = om.fused_moe_row_scaled(x, q13, q2, np.repeat(c13[:, None], 2 * I, 1), np.repeat(c2[:, None], H, 1), ones, ids,
                                a1_scale=0.02, a2_scale=0.001)
    assert torch.equal(a, b)
    # routing weight on the input: with weight w the gate and up halves both scale by w before the activation
    w = torch.full((M, 1), 0.5)
    on_in = om.fused_moe_row_scaled(x, q13, q2, s13, s2, w, ids, apply_router_weight_on_input=True)
    on_out = om.fused_moe_row_scaled(x, q13, q2, s13, s2, w, ids)
    assert not torch.equal(on_in, on_out)
    assert float((on_in.float() - on_out.float()).norm()) > 0


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_dynamic_per_tensor_quant_against_the_reference_tests_statement(dtype):
    """test_scaled_fp8_quant_per_tensor's reference (test/manual/quant/test_custom_ops.py:20-44) evaluated in torch:
    scale = max|x| / 448, q = (x.float() * scale.reciprocal()).clamp(-448, 448).to(float8_e4m3fn); its own 11 x 11
    input recipe and a larger one with outliers."""
    g = torch.Generator().manual_seed(7)
    for shape, mul in (((11, 11), 13.0), ((64, 384), 1.0), ((3, 16), 1e-3)):
        x = (torch.randn(*shape, generator=g) * mul).to(dtype)
        q, s = oq.dynamic_per_tensor_quant_fp8(x)
        scale = (x.float().abs().max() / 448.0).reshape(1)
        assert np.array_equal(s, scale.numpy())
        ref = (x.to(torch.float32) * scale.reciprocal()).clamp(min=-448.0, max=448.0).to(torch.float8_e4m3fn)
        assert np.array_equal(q, ref.view(torch.uint8).numpy())
    q, s = oq.dynamic_per_tensor_quant_fp8(torch.zeros(4, 16, dtype=dtype))
    assert float(s[0]) > 0 and not q.any()


def test_topk_sigmoid_brute_force_and_reference_model():
    """float64 python loops on tiny rows; torch.topk(torch.sigmoid(x)) (the model of
    sgl-kernel/tests/test_moe_topk_sigmoid.py:47-58) where there are no ties; ties pick the lower index; the bias
    steers the choice but not the weight; renormalised weights sum to one."""
    import math

    g = torch.Generator().manual_seed(123)
    for E, k in [(4, 1), (8, 2), (16, 4), (37, 5)]:
        x = torch.randn(6, E, generator=g)
        bias = torch.randn(E, generator=g) * 0.2
        for b in (None, bias):
            for renorm in (False, True):
                w, ids = om.topk_sigmoid(x, k, renorm, b)
                for r in range(x.shape[0]):
                    s = [1.0 / (1.0 + math.exp(-float(v))) for v in x[r]]
                    c = [s[e] + (float(b[e]) if b is not None else 0.0) for e in range(E)]
                    order = sorted(range(E), key=lambda e: (-c[e], e))[:k]
                    assert ids[r].tolist() == order
                    ws = [s[e] for e in order]
                    if renorm:
                        tot = sum(ws)
                        ws = [v / tot for v in ws]
                    assert np.allclose(w[r].numpy(), ws, rtol=1e-5, atol=1e-6)
        w, ids = om.topk_sigmoid(x, k)
        rw, rids = torch.topk(torch.sigmoid(x), k, dim=-1)
        assert torch.equal(ids.long(), rids) and torch.allclose(w, rw, rtol=1e-6, atol=1e-7)
    tied = torch.zeros(2, 8)
    assert om.topk_sigmoid(tied, 3)[1].tolist() == [[0, 1, 2], [0, 1, 2]]
    w, _ = om.topk_sigmoid(torch.randn(5, 16, generator=g), 4, True, torch.randn(16, generator=g))
    assert torch.allclose(w.sum(-1), torch.ones(5), atol=1e-6)


# ---- expert-major ("grouped") MoE interface --------------------------------------------------------
def test_prepare_moe_input_brute_force():
    g = torch.Generator().manual_seed(31)
    for tokens, topk, E in [(1, 2, 4), (7, 3, 5), (40, 4, 9), (300, 1, 3)]:
        ids = torch.stack([torch.randperm(E, generator=g)[:topk] for _ in range(tokens)]).numpy().astype(np.int32)
        if tokens == 40:
            ids[ids == 2] = -1  # an expert that lives elsewhere
        offs, bs, ps1, ps2, a_map, c_map = om.prepare_moe_input(ids, E, 24, 40)
        flat = ids.reshape(-1)
        valid = int((flat >= 0).sum())
        assert offs[0] == 0 and offs[-1] == valid and bs[0] == 0
        for e in range(E):
            members = [i for i in range(flat.size) if flat[i] == e]
            assert list(ps1[e]) == [len(members), 48, 40] and list(ps2[e]) == [len(members), 40, 24]
            assert offs[e + 1] - offs[e] == len(members)
            assert bs[e + 1] - bs[e] == -(-len(members) // 128) * 128
            # the span holds exactly this expert's tokens, in ascending flat index, and c_map inverts it
            assert list(a_map[offs[e]:offs[e + 1]]) == [i // topk for i in members]
            assert [int(c_map[i]) for i in members] == list(range(offs[e], offs[e + 1]))
        assert all(c_map[i] == -1 for i in range(flat.size) if flat[i] < 0)


def test_grouped_mm_and_shuffle_mul_sum_against_float64():
    g = torch.Generator().manual_seed(32)
    E, N, K, topk, m = 3, 256, 384, 2, 5
    counts = [4, 0, 6]
    offs = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    rows = int(offs[-1])
    aq = e4m3fn_encode(((torch.rand(rows, K, generator=g) - 0.5) * 2 * 448).numpy())
    bq = e4m3fn_encode(((torch.rand(E, N, K, generator=g) - 0.5) * 2 * 448).numpy().reshape(E * N, K)).reshape(E, N, K)
    a_s = (torch.rand(rows, K // 128, generator=g) * 1e-2).numpy()
    b_s = (torch.rand(E, N // 128, K // 128, generator=g) * 1e-2).numpy()
    ps = np.array([[c, N, K] for c in counts], dtype=np.int32)
    out = om.fp8_blockwise_scaled_grouped_mm(aq, a_s, bq, b_s, ps, offs[:-1], out_dtype=torch.float32).numpy()
    for e in range(E):
        lo, hi = offs[e], offs[e + 1]
        a = e4m3fn_decode(aq[lo:hi]).astype(np.float64) * np.repeat(a_s[lo:hi], 128, axis=1)
        b = e4m3fn_decode(bq[e]).astype(np.float64) * np.repeat(np.repeat(b_s[e], 128, axis=0), 128, axis=1)
        ref = a @ b.T
        if hi > lo:
            assert np.abs(out[lo:hi] - ref).max() <= 1e-5 * np.abs(ref).max()
    # weighted un-permuting sum: the torch expression of the reference's doc comment, in float64
    c2 = torch.randn(m * topk, 64, generator=g).to(torch.bfloat16)
    c_map = torch.randperm(m * topk, generator=g).numpy().astype(np.int32)
    w = torch.rand(m, topk, generator=g).to(torch.bfloat16)
    got = om.apply_shuffle_mul_sum(c2, c_map, w, m)
    want = (c2[torch.from_numpy(c_map.astype(np.int64))].view(m, topk, 64).double() * w.view(m, topk, 1).double()).sum(dim=1)
    assert float((got.double() - want).abs().max()) <= 2 ** -8 * float(want.abs().max())
    ones = om.apply_shuffle_mul_sum(c2, c_map, None, m)
    assert torch.equal(ones, c2[torch.from_numpy(c_map.astype(np.int64))].view(m, topk, 64).float().sum(dim=1).to(torch.bfloat16))


def test_grouped_layer_matches_the_sorted_block_layer():
    """Both MoE formulations compute the same layer; they differ only in where the routing weight is applied
    (fp32 accumulator there, cast activation-dtype rows here).  With top-1 and weight 1 they are identical."""
    M, H, I, E = 6, 256, 128, 3
    x, w13q, w2q, w13s, w2s = _tiny_moe(M, H, I, E, 3)
    ids = torch.tensor([[2], [0], [2], [1], [0], [2]], dtype=torch.int32)
    one = torch.ones(M, 1)
    a = om.cutlass_fused_experts_fp8(x, w13q, w2q, w13s, w2s, one, ids)
    b = om.fused_moe_block_fp8(x, w13q, w2q, w13s, w2s, one, ids, quant_form="reciprocal")
    assert torch.equal(a, b)
    tw, ti = om.topk_softmax(torch.randn(M, E, generator=torch.Generator().manual_seed(4)), 2, True)
    a = om.cutlass_fused_experts_fp8(x, w13q, w2q, w13s, w2s, tw, ti)
    b = om.fused_moe_block_fp8(x, w13q, w2q, w13s, w2s, tw, ti, quant_form="reciprocal")
    assert float((a.float() - b.float()).norm() / b.float().norm()) < 1e-2


# ---- golden vectors ----------------------------------------------------------------------------
def test_golden_config1_is_reproduced_by_the_oracle():
    z = np.load(GOLDEN)
    a = torch.from_numpy(z["a_bf16_bits"]).view(torch.bfloat16)
    torch.manual_seed(0)
    assert torch.equal(a, torch.randn(32, 512).to(torch.bfloat16))  # the recipe itself
    w = torch.from_numpy(z["w_f32"])
    aq, a_s, _ = oq.group_quant(a, 128)
    assert np.array_equal(aq, z["aq_divide"]) and np.array_equal(a_s, z["as_divide"])
    aq2, a_s2, _ = oq.group_quant(a, 128, form="reciprocal")
    assert np.array_equal(aq2, z["aq_reciprocal"]) and np.array_equal(a_s2, z["as_reciprocal"])
    wq, ws = oq.block_quant_weight(w)
    assert np.array_equal(wq, z["wq"]) and np.array_equal(ws, z["ws"])
    c = og.block_fp8_matmul(aq, wq, a_s, ws, out_dtype=torch.bfloat16)
    assert np.array_equal(c.view(torch.int16).numpy(), z["c_bf16_bits"])
    assert a_s.shape == (32, 4) and ws.shape == (2, 4) and c.shape == (32, 256)


def test_masked_silu_mul_group_quant_is_the_unmasked_op_on_each_experts_prefix():
    """The masked-layout restatement adds nothing but the token mask: on every expert it must equal
    silu_and_mul -> group_quant(reciprocal, UE8M0) applied to that expert's first masked_m[e] tokens, and be
    empty elsewhere (per_token_group_quant_8bit_v2.cu:237-246 visits exactly those tokens)."""
    from oracle import moe as om

    g = torch.Generator().manual_seed(5)
    E, T, hidden = 4, 9, 384
    x = (torch.randn(E, T, 2 * hidden, generator=g) * 3).to(torch.bfloat16)
    masked_m = np.array([0, 9, 4, 1], dtype=np.int32)
    q, eb, valid = oq.silu_mul_group_quant_masked(x, masked_m, 128)
    assert valid.sum() == masked_m.sum()
    for e in range(E):
        m = masked_m[e]
        assert valid[e, :m].all() and not valid[e, m:].any()
        assert not q[e, m:].any() and not eb[e, m:].any()
        if m:
            rq, _, reb = oq.group_quant(om.silu_and_mul(x[e, :m]), 128, form="reciprocal", scale_ue8m0=True)
            assert np.array_equal(q[e, :m], rq) and np.array_equal(eb[e, :m], reb)


def test_topk_softmax_oracle_against_brute_force_and_ties():
    """topk_softmax restatement: brute force on tiny rows (python loops over a float64 softmax), the renormalised
    weights sum to one, soft-capping and bias act on the logits before the softmax
    (moe_topk_softmax_kernels.cu:108-115), equal probabilities pick the lower expert index (:540-548)."""
    import math

    g = torch.Generator().manual_seed(3)
    logits = torch.randn(7, 12, generator=g)
    bias = torch.randn(12, generator=g)
    for cap, b in ((0.0, None), (2.5, None), (0.0, bias), (1.5, bias)):
        w, ids = om.topk_softmax(logits, 4, renormalize=False, moe_softcapping=cap, correction_bias=b)
        wr, _ = om.topk_softmax(logits, 4, renormalize=True, moe_softcapping=cap, correction_bias=b)
        for r in range(7):
            x = [float(v) for v in logits[r]]
            if cap:
                x = [math.tanh(v / cap) * cap for v in x]
            if b is not None:
                x = [v + float(bv) for v, bv in zip(x, b)]
            m = max(x)
            e = [math.exp(v - m) for v in x]
            p = [v / sum(e) for v in e]
            order = sorted(range(12), key=lambda i: (-p[i], i))[:4]
            assert [int(i) for i in ids[r]] == order
            np.testing.assert_allclose(w[r].numpy(), [p[i] for i in order], rtol=2e-6)
            np.testing.assert_allclose(wr[r].numpy(), np.array([p[i] for i in order]) / sum(p[i] for i in order), rtol=2e-6)
    tied = torch.tensor([[1.0, 3.0, 3.0, 0.5, 3.0, 1.0]])
    _, ids = om.topk_softmax(tied, 4, renormalize=False)
    assert ids.tolist() == [[1, 2, 4, 0]]


# ---- fused RMSNorm + group quant -------------------------------------------------------------------
def test_fused_rms_group_quant_against_the_reference_tests_torch_model():
    """The torch model of test/registered/quant/test_fused_rms_fp8_group_quant.py:23-52,84-95, evaluated line by
    line on fp32 inputs (where its arithmetic and the oracle's coincide up to summation order), plus closed
    forms: a constant row normalises to +-w, and the residual enters before the norm."""
    g = torch.Generator().manual_seed(41)
    M, N1, N2 = 5, 200, 384  # N1 is not a multiple of 128: the last group is zero-padded
    x1 = torch.randn(M, N1, generator=g) / 10
    res = torch.randn(M, N1, generator=g) / 10
    x2 = torch.randn(M, N2, generator=g) / 10
    w1 = torch.rand(N1, generator=g) + 0.5
    w2 = torch.rand(N2, generator=g) + 0.5

    def rmsnorm(x, weight, eps):
        row_norm = (x * x).sum(dim=-1)
        norm = torch.rsqrt(row_norm / x.shape[1] + eps)
        return x * norm[:, None] * weight[None, :]

    s = x1 + res
    y1 = rmsnorm(s, w1, 1e-6)
    y2 = rmsnorm(x2, w2, 1e-5)
    pad = torch.nn.functional.pad(y1, (0, 256 - N1))
    v = pad.view(M, 2, 128)
    x_max = v.abs().amax(dim=-1, keepdim=True).clamp_min(1e-10)
    x_scale = x_max / 448.0
    deq_model = (torch.clamp(v * (1.0 / x_scale), -448, 448).to(torch.float8_e4m3fn).float() * x_scale).view(M, 256)[:, :N1]

    r = oq.fused_rms_group_quant(x1, w1, 1e-6, res1=res, x2=x2, w2=w2, eps2=1e-5)
    assert np.allclose(r["y1"], y1.numpy(), rtol=2e-6, atol=1e-7)
    assert np.allclose(r["y2"], y2.numpy(), rtol=2e-6, atol=1e-7)
    assert np.array_equal(r["res"], s.numpy())
    assert np.allclose(r["s"], x_scale.view(M, 2).numpy(), rtol=2e-6)
    deq = e4m3fn_decode(r["q"]) * np.repeat(r["s"], 128, axis=1)[:, :N1]
    # a last-bit difference of y can move a value across an fp8 rounding boundary: rare, and one code apart
    assert (np.abs(deq - deq_model.numpy()) > 1e-6).mean() < 2e-3
    assert np.abs(deq - y1.numpy()).max() <= np.abs(y1.numpy()).max() * 2 ** -4
    # closed forms
    c = oq.fused_rms_group_quant(torch.full((2, 128), -3.0), torch.arange(128, dtype=torch.float32), 0.0)
    assert np.allclose(c["y1"], -np.arange(128, dtype=np.float32)[None].repeat(2, 0), rtol=1e-6)
    assert np.allclose(c["s"], 127.0 / 448.0, rtol=1e-6) and c["q"][0, 127] == 0xFE  # arg-max lands on -448
    z = oq.fused_rms_group_quant(torch.zeros(1, 128), torch.ones(128), 1e-6)
    assert np.all(z["q"] == 0) and np.allclose(z["s"], 1e-10 / 448.0)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_gated_activations_against_torch_and_closed_forms(dtype):
    """act_and_mul's three activations: against torch's own functions the way the reference's test states them
    (sgl-kernel/tests/test_activation.py: x[..., d:] * F.silu / F.gelu(approximate="none" | "tanh")(x[..., :d]),
    rtol = atol = 1e-3 in fp16), and against what the mathematics fixes: gelu(x) - gelu(-x) = x for the erf and the
    tanh form alike (a wrong sign or a dropped 0.5 breaks it), gelu(0) = 0, gelu(x) -> x and gelu(-x) -> 0 for large
    x, silu(x) - silu(-x) = x, and the value at 1: 0.8413447 (erf), 0.8411920 (tanh), 0.7310586 (silu)."""
    import torch.nn.functional as F

    g = torch.Generator().manual_seed(4)
    d = 1024
    x = (torch.randn(64, 2 * d, generator=g) * 2).to(dtype)
    models = {"silu": F.silu, "gelu": lambda t: F.gelu(t, approximate="none"),
              "gelu_tanh": lambda t: F.gelu(t, approximate="tanh")}
    tol = 1e-3 if dtype == torch.float16 else 1.6e-2
    for name, fn in models.items():
        got = om.act_and_mul(x, name)
        assert got.dtype == dtype and got.shape == (64, d)
        torch.testing.assert_close(got, x[..., d:] * fn(x[..., :d].float()).to(dtype), rtol=tol, atol=1e-3)
        t = torch.linspace(-6, 6, 241)
        torch.testing.assert_close(om._act_f32(t, name) - om._act_f32(-t, name), t, rtol=0, atol=2e-6)
        assert float(om._act_f32(torch.zeros(1), name)) == 0.0
        torch.testing.assert_close(om._act_f32(torch.tensor([12.0, -12.0]), name), torch.tensor([12.0, 0.0]),
                                   rtol=0, atol=1e-4)
    one = torch.ones(1)
    assert abs(float(om._act_f32(one, "gelu")) - 0.8413447) < 1e-6
    assert abs(float(om._act_f32(one, "gelu_tanh")) - 0.8411920) < 1e-6
    assert abs(float(om._act_f32(one, "silu")) - 0.7310586) < 1e-6
    assert om.gelu_and_mul(x).equal(om.act_and_mul(x, "gelu")) and om.silu_and_mul(x).equal(om.act_and_mul(x, "silu"))
    assert om.gelu_tanh_and_mul(x).equal(om.act_and_mul(x, "gelu_tanh"))


def test_moe_activation_forms_and_their_use_in_the_layer():
    """moe_activation follows fused_experts_impl's chain (fused_moe.py:530-647): gated -> act_and_mul on the two
    halves; not gated -> F.silu / F.gelu / relu(x)^2 on the whole row, anything else refused.  In the layer oracle a
    one-expert top-1 case with weight 1 must equal the dense chain GEMM -> activation -> quant -> GEMM."""
    import torch.nn.functional as F

    g = torch.Generator().manual_seed(9)
    h = (torch.randn(5, 256, generator=g) * 2).to(torch.bfloat16)
    assert om.moe_activation(h, "silu", True).equal(om.silu_and_mul(h))
    assert om.moe_activation(h, "gelu", True).equal(om.gelu_and_mul(h))
    assert om.moe_activation(h, "silu", False).equal(F.silu(h)) and om.moe_activation(h, "gelu", False).equal(F.gelu(h))
    assert om.moe_activation(h, "relu2", False).equal(torch.square(F.relu(h)))
    assert om.moe_activation(h, "relu2", False)[h < 0].abs().sum() == 0
    with pytest.raises(ValueError):
        om.moe_activation(h, "tanh", False)
    with pytest.raises(ValueError):
        om.moe_activation(h, "relu2", True)
    M, H, I = 6, 256, 128
    x = torch.randn(M, H, generator=g).to(torch.bfloat16)
    for act, gated in (("gelu", True), ("relu2", False), ("silu", False)):
        w13 = torch.randn((2 if gated else 1) * I, H, generator=g) * 0.05
        w2 = torch.randn(H, I, generator=g) * 0.05
        q13, s13 = oq.block_quant_weight(w13)
        q2, s2 = oq.block_quant_weight(w2)
        tw, ti = torch.ones(M, 1), torch.zeros(M, 1, dtype=torch.int32)
        got = om.fused_moe_block_fp8(x, q13[None], q2[None], s13[None], s2[None], tw, ti, activation=act, is_gated=gated)
        xq, xs, _ = oq.group_quant(x, 128)
        a = om.moe_activation(og.block_fp8_matmul(xq, q13, xs, s13, (128, 128), out_dtype=x.dtype), act, gated)
        aq, a_s, _ = oq.group_quant(a, 128)
        want = og.block_fp8_matmul(aq, q2, a_s, s2, (128, 128), out_dtype=x.dtype)
        assert got.equal(want), (act, gated)


def test_clamped_swiglu_forms_reduce_to_silu_and_clamp_where_they_must():
    """The three clamped gated-SiLU variants of fused_experts_impl (fused_moe.py:315-331,530-580).  With an
    infinite limit each must reduce to a library routine: gemm1_limit alone to F.silu(gate) * up; gemm1_alpha = 1
    to F.silu(gate) * (up + 1) on the interleaved halves; swiglu_limit to silu_and_mul.  With a finite limit, on
    values chosen by hand: the gate is cut from above only, the up projection on both sides, and the limit-only form
    clamps silu(gate), not the gate.  These pins fix term order, signs and which half is which; the compiled
    functions' evaluation in fp32 with one rounding is the oracle's reading of torch.compile's pointwise code
    generation and has no fixture in the reference."""
    import torch.nn.functional as F

    g = torch.Generator().manual_seed(12)
    h = (torch.randn(9, 64, generator=g) * 3).to(torch.bfloat16)
    inf = float("inf")
    d = 32
    got = om.moe_activation(h, gemm1_limit=inf)
    assert got.equal((F.silu(h[..., :d].float()) * h[..., d:].float()).to(torch.bfloat16))
    got = om.moe_activation(h, gemm1_alpha=1.0, gemm1_limit=inf)
    assert got.equal((F.silu(h[..., ::2].float()) * (h[..., 1::2].float() + 1)).to(torch.bfloat16))
    assert om.moe_activation(h, swiglu_limit=inf).equal(om.silu_and_mul(h))
    # hand-made rows: [gate | up] = [20, -20 | 30, -30] with limit 10
    row = torch.tensor([[20.0, -20.0, 30.0, -30.0]], dtype=torch.bfloat16)
    silu20, silum20 = float(F.silu(torch.tensor(20.0))), float(F.silu(torch.tensor(-20.0)))
    got = om.moe_activation(row, gemm1_limit=10.0).float()
    torch.testing.assert_close(got, torch.tensor([[10.0 * 10.0, silum20 * -10.0]]), rtol=8e-3, atol=0)
    got = om.moe_activation(row, swiglu_limit=10.0).float()  # gate cut to 10 first, then silu
    silu10 = float(F.silu(torch.tensor(10.0)).to(torch.bfloat16))
    torch.testing.assert_close(got, torch.tensor([[silu10 * 10.0, float(torch.tensor(silum20).to(torch.bfloat16)) * -10.0]]),
                               rtol=8e-3, atol=1e-12)
    # interleaved: (gate, up) = (20, 30), (-20, -30), alpha 1.702, limit 7: gate -> 7 / -20, up -> 7 / -7
    row = torch.tensor([[20.0, 30.0, -20.0, -30.0]], dtype=torch.bfloat16)
    got = om.moe_activation(row, gemm1_alpha=1.702, gemm1_limit=7.0).float()
    want = torch.tensor([[7.0 * float(torch.sigmoid(torch.tensor(7.0 * 1.702))) * 8.0,
                          -20.0 * float(torch.sigmoid(torch.tensor(-20.0 * 1.702))) * -6.0]])
    torch.testing.assert_close(got, want, rtol=8e-3, atol=1e-12)
    with pytest.raises(AssertionError):
        om.moe_activation(h, "gelu", True, gemm1_limit=7.0)

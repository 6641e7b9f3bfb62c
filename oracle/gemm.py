"""Scaled GEMMs of the path, restated from the reference's torch-native oracles (CPU).

Quantised operands come in as numpy arrays (uint8 e4m3fn codes or int8); results are
torch tensors of the requested output dtype.
"""
import numpy as np
import torch

from .fp8 import e4m3fn_decode


def _t(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(a))


def block_fp8_matmul(aq: np.ndarray, bq: np.ndarray, a_s: np.ndarray, b_s: np.ndarray,
                     block=(128, 128), out_dtype=torch.bfloat16, return_fp32=False):
    """C = sum_kb (A[:,kb] @ B[nb,kb].T) * (As[:,kb] * Bs[nb,kb]), fp32 accumulation, then cast.
    Follows native_w8a8_block_fp8_matmul, test/manual/quant/test_block_fp8.py:291-343
    (tile loop :335-341); same math as baseline_scaled_mm,
    sgl-kernel/tests/test_fp8_blockwise_gemm.py:20-60.
    aq [M,K] codes, bq [N,K] codes, a_s [M, ceil(K/bk)], b_s [ceil(N/bn), ceil(K/bk)]."""
    bn, bk = block
    a = _t(e4m3fn_decode(aq))
    b = _t(e4m3fn_decode(bq))
    a_s = _t(a_s.astype(np.float32))
    b_s = _t(b_s.astype(np.float32))
    m, k = a.shape
    n = b.shape[0]
    n_tiles, k_tiles = -(-n // bn), -(-k // bk)
    assert a_s.shape == (m, k_tiles) and b_s.shape == (n_tiles, k_tiles)
    c = torch.zeros(m, n, dtype=torch.float32)
    for i in range(k_tiles):
        a_i = a[:, i * bk:(i + 1) * bk]
        for j in range(n_tiles):
            b_ji = b[j * bn:(j + 1) * bn, i * bk:(i + 1) * bk]
            c[:, j * bn:(j + 1) * bn] += torch.matmul(a_i, b_ji.t()) * (a_s[:, i:i + 1] * b_s[j, i])
    return c if return_fp32 else c.to(out_dtype)


def block_int8_matmul(aq: np.ndarray, bq: np.ndarray, a_s: np.ndarray, b_s: np.ndarray,
                      block=(128, 128), out_dtype=torch.bfloat16, return_fp32=False):
    """Block-scaled INT8 matmul: the same tile loop as block_fp8_matmul over int8 operands converted to fp32
    (native_w8a8_block_int8_matmul, test/registered/quant/test_block_int8.py:45-98, tile loop :90-95).
    A 128-deep int8 dot product stays below 2^21, so the fp32 tile product is the exact integer."""
    bn, bk = block
    a = _t(aq.astype(np.float32))
    b = _t(bq.astype(np.float32))
    a_s = _t(a_s.astype(np.float32))
    b_s = _t(b_s.astype(np.float32))
    m, k = a.shape
    n = b.shape[0]
    n_tiles, k_tiles = -(-n // bn), -(-k // bk)
    assert a_s.shape == (m, k_tiles) and b_s.shape == (n_tiles, k_tiles)
    c = torch.zeros(m, n, dtype=torch.float32)
    for i in range(k_tiles):
        a_i = a[:, i * bk:(i + 1) * bk]
        for j in range(n_tiles):
            b_ji = b[j * bn:(j + 1) * bn, i * bk:(i + 1) * bk]
            c[:, j * bn:(j + 1) * bn] += torch.matmul(a_i, b_ji.t()) * (a_s[:, i:i + 1] * b_s[j, i])
    return c if return_fp32 else c.to(out_dtype)


def fp8_scaled_mm(aq: np.ndarray, bq_nk: np.ndarray, sa: np.ndarray, sb: np.ndarray,
                  out_dtype=torch.bfloat16, bias: torch.Tensor = None, return_fp32=False):
    """C = cast(acc * sa[m] * sb[n] (+ bias[n])): torch_scaled_mm,
    sgl-kernel/tests/test_fp8_gemm.py:8-16, with the bias folded in before the cast as the
    kernel's epilogue does (sgl-kernel/csrc/gemm/fp8_gemm_kernel.cu:100-137).
    bq_nk is the weight as [N,K] (the operator sees its [K,N] column-major view)."""
    a = _t(e4m3fn_decode(aq))
    b = _t(e4m3fn_decode(bq_nk))
    o = torch.matmul(a, b.t())
    o = o * _t(sa.astype(np.float32)).view(-1, 1) * _t(sb.astype(np.float32)).view(1, -1)
    if bias is not None:
        o = o + bias.to(torch.float32).view(1, -1)
    return o if return_fp32 else o.to(out_dtype)


def int8_scaled_mm(aq: np.ndarray, bq_nk: np.ndarray, sa: np.ndarray, sb: np.ndarray,
                   out_dtype=torch.bfloat16, bias: torch.Tensor = None, return_fp32=False):
    """C = cast(float(acc_i32) * (sb[n] * sa[m]) + float(bias[n])): exact int32 accumulation,
    fp32 epilogue (sgl-kernel/tests/test_int8_gemm.py:13-21;
    sgl-kernel/csrc/cutlass_extensions/epilogue/epilogue_per_row_per_col_scale.h:232-253,273-305)."""
    if aq.shape[0] * bq_nk.shape[0] * aq.shape[1] <= (1 << 27):
        acc = torch.matmul(_t(aq.astype(np.int64)), _t(bq_nk.astype(np.int64)).t())  # exact
    else:
        # int64 matmul has no BLAS path; float64 is exact too while |acc| <= K * 128 * 128 < 2^53 (K < 2^39),
        # and checked equal to the int64 result in tests/test_oracle_cpu.py
        acc = torch.matmul(_t(aq.astype(np.float64)), _t(bq_nk.astype(np.float64)).t())
    o = acc.to(torch.float32) * (_t(sb.astype(np.float32)).view(1, -1) * _t(sa.astype(np.float32)).view(-1, 1))
    if bias is not None:
        o = o + bias.to(torch.float32).view(1, -1)
    return o if return_fp32 else o.to(out_dtype)

"""OCP e4m3fn encode/decode in closed form (no torch cast involved).

e4m3fn: 1 sign, 4 exponent (bias 7), 3 mantissa bits; no infinities; 0x7f/0xff are NaN;
largest finite 448 (0x7e); subnormal step 2**-9.  Encoding rounds to nearest, ties to
even, which is what `static_cast<__nv_fp8_e4m3>(float)` / `__nv_cvt_float2_to_fp8x2`
(sgl-kernel/csrc/gemm/per_token_group_quant_8bit.cu:110,
per_token_group_quant_8bit_v2.cu:383-388) and torch's `.to(torch.float8_e4m3fn)`
(test/manual/quant/test_block_fp8.py:62) do for in-range inputs.  Callers clamp to
[-448, 448] first, as the reference does; anything larger is saturated here.
"""
import numpy as np

E4M3_MAX = 448.0


def e4m3fn_encode(v) -> np.ndarray:
    """float array -> uint8 codes (RNE, saturating, NaN -> 0x7f|sign)."""
    v = np.asarray(v, dtype=np.float32)
    sign = (np.signbit(v).astype(np.uint8)) << 7
    a = np.abs(v.astype(np.float64))
    nan = np.isnan(a)
    a = np.where(nan, 0.0, a)
    a = np.minimum(a, 464.0)  # anything >= 464 saturates below anyway
    # subnormal range: multiples of 2**-9 below 2**-6
    sub = a < 2.0 ** -6
    m_sub = np.rint(a * 512.0)  # 0..8 ; 8 is the smallest normal (code 0x08)
    mant, ex = np.frexp(np.where(a == 0, 1.0, a))  # a = mant * 2**ex, mant in [0.5, 1)
    e = ex - 1
    frac = mant * 2.0 - 1.0  # [0, 1)
    m = np.rint(frac * 8.0)
    carry = m == 8
    e = np.where(carry, e + 1, e)
    m = np.where(carry, 0, m)
    code_norm = ((e + 7).astype(np.int64) << 3) | m.astype(np.int64)
    code = np.where(sub, m_sub.astype(np.int64), code_norm)
    code = np.minimum(code, 0x7E)  # saturate to 448
    code = np.where(nan, 0x7F, code)
    return (code.astype(np.uint8) | sign).astype(np.uint8)


def _decode_table() -> np.ndarray:
    t = np.zeros(256, dtype=np.float32)
    for c in range(256):
        s = -1.0 if c & 0x80 else 1.0
        e = (c >> 3) & 0xF
        m = c & 7
        if e == 0xF and m == 7:
            t[c] = np.nan
        elif e == 0:
            t[c] = s * m * 2.0 ** -9
        else:
            t[c] = s * (1.0 + m / 8.0) * 2.0 ** (e - 7)
    return t


E4M3_TABLE = _decode_table()


def e4m3fn_decode(codes) -> np.ndarray:
    """uint8 codes -> float32 values."""
    return E4M3_TABLE[np.asarray(codes, dtype=np.uint8)]

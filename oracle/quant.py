"""Activation quantisation, restated from the reference (CPU, torch + numpy).

Inputs are torch tensors (bf16/fp16/fp32); outputs are numpy arrays: `q` uint8 e4m3fn
codes or int8 values, scales float32 (or uint8 UE8M0 exponent bytes).  Layout helpers at
the bottom turn the logical `[rows, groups]` scale array into the buffers the operators
write.
"""
import numpy as np
import torch

from .fp8 import e4m3fn_encode

_F32 = np.float32


def _to_f32(x: torch.Tensor) -> np.ndarray:
    return x.detach().to(torch.float32).cpu().numpy()


def _log2_ceil_bits(y: np.ndarray) -> np.ndarray:
    """ceil(log2(y)) of positive normal float32 values from their bits
    (per_token_group_quant_8bit_v2.cu:61-66; exact form of per_token_group_quant_8bit.cu:88)."""
    b = y.astype(_F32).view(np.uint32)
    e = ((b >> 23) & 0xFF).astype(np.int32)
    return e - 127 + ((b & 0x7FFFFF) != 0)


def _pow2(e: np.ndarray) -> np.ndarray:
    return ((e.astype(np.int32) + 127).astype(np.uint32) << 23).view(_F32)


def group_quant(x: torch.Tensor, group_size: int, *, form: str = "divide", dst: str = "fp8",
                scale_ue8m0: bool = False, eps: float = 1e-10):
    """Per-token-group quantisation.

    form="divide": s = amax/max8, q = cvt(clamp(x / s))
        sgl-kernel/csrc/gemm/per_token_group_quant_8bit.cu:45,80-86,110 and
        test/manual/quant/test_block_fp8.py:55-64.
    form="reciprocal": s = amax*(1/max8), q = cvt(clamp(x * (max8/amax)))
        sgl-kernel/csrc/gemm/per_token_group_quant_8bit_v2.cu:69-80,344-389.
    scale_ue8m0: the scale is rounded up to a power of two
        (per_token_group_quant_8bit.cu:87-97; v2.cu:72-75,83-90) and the biased exponent
        byte is returned as well.
    dst="fp8": e4m3fn codes, clamp +-448; dst="int8": clamp [-128,127] then C++ float->int8
        conversion, i.e. truncation toward zero (per_token_group_quant_8bit.cu:110-111).

    Returns (q[rows, hidden] uint8|int8, s[rows, groups] float32, e[rows, groups] uint8|None).
    """
    hidden = x.shape[-1]
    assert hidden % group_size == 0
    x32 = _to_f32(x).reshape(-1, hidden // group_size, group_size)
    max8, min8 = (_F32(448.0), _F32(-448.0)) if dst == "fp8" else (_F32(127.0), _F32(-128.0))
    amax = np.maximum(np.abs(x32).max(axis=-1), _F32(eps)).astype(_F32)
    if form == "divide":
        s = (amax / max8).astype(_F32)
        if scale_ue8m0:
            s = _pow2(_log2_ceil_bits(np.maximum(s, _F32(1e-10))))
        y = (x32 / s[..., None]).astype(_F32)
    elif form == "reciprocal":
        inv_max = _F32(1.0) / max8
        if scale_ue8m0:
            e = _log2_ceil_bits((amax * inv_max).astype(_F32))
            s = _pow2(e)
            mul = _pow2(-e)
        else:
            s = (amax * inv_max).astype(_F32)
            mul = (max8 / amax).astype(_F32)
        y = (x32 * mul[..., None]).astype(_F32)
    else:
        raise ValueError(form)
    y = np.minimum(np.maximum(y, min8), max8)
    rows = x32.shape[0]
    if dst == "fp8":
        q = e4m3fn_encode(y).reshape(rows, hidden)
    else:
        q = np.trunc(y).astype(np.int8).reshape(rows, hidden)
    ebyte = ((s.view(np.uint32) >> 23) & 0xFF).astype(np.uint8) if scale_ue8m0 else None
    return q, s, ebyte


def silu_mul_group_quant_masked(x: torch.Tensor, masked_m: np.ndarray, group_size: int = 128):
    """Masked ("DeepEP low-latency") layout of the fused SiLU*mul + UE8M0 group quant:
    x[E, T, 2*hidden]; of expert e only tokens t < masked_m[e] are produced
    (sgl-kernel/csrc/gemm/per_token_group_quant_8bit_v2.cu:203-247 walks exactly those tokens, :349-354 forms
    T(silu(gate)) * up in the storage dtype, :69-90 the power-of-two scale).  Returns q[E, T, hidden] uint8,
    ebyte[E, T, groups] uint8 and valid[E, T] bool; entries outside `valid` are zero here and unspecified in the
    operator (it never touches them)."""
    E, T, h2 = x.shape
    hidden = h2 // 2
    groups = hidden // group_size
    q = np.zeros((E, T, hidden), dtype=np.uint8)
    eb = np.zeros((E, T, groups), dtype=np.uint8)
    valid = np.zeros((E, T), dtype=bool)
    for e in range(E):
        m = int(masked_m[e])
        if m <= 0:
            continue
        xe = x[e, :m]
        gate32 = xe[:, :hidden].float()
        act = (gate32 * torch.sigmoid(gate32)).to(x.dtype) * xe[:, hidden:]
        qe, _, ee = group_quant(act, group_size, form="reciprocal", scale_ue8m0=True)
        q[e, :m] = qe
        eb[e, :m] = ee
        valid[e, :m] = True
    return q, eb, valid


def per_token_quant_fp8(x: torch.Tensor):
    """sgl-kernel/csrc/gemm/per_token_quant_fp8.cu:71-80,102-105: scale = max|x|/448 (no
    eps), scale_inv = 0 if scale == 0 else 1/scale, q = e4m3(clamp(x * scale_inv))."""
    x32 = _to_f32(x).reshape(-1, x.shape[-1])
    amax = np.abs(x32).max(axis=-1).astype(_F32)
    scale = (amax / _F32(448.0)).astype(_F32)
    with np.errstate(divide="ignore"):
        inv = np.where(scale == 0, _F32(0), _F32(1.0) / scale).astype(_F32)
    y = (x32 * inv[:, None]).astype(_F32)
    y = np.maximum(np.minimum(y, _F32(448.0)), _F32(-448.0))
    return e4m3fn_encode(y), scale


def static_quant_fp8(x: torch.Tensor, scale: float):
    """python/sglang/srt/layers/quantization/fp8_kernel.py:714-717 (_static_quant_fp8): with a given per-tensor
    scale, q = e4m3(clamp(float32(x) * (float32(1) / scale), -448, 448)); the scale is handed back once per row."""
    x32 = _to_f32(x).reshape(-1, x.shape[-1])
    inv = _F32(1.0) / _F32(scale)
    with np.errstate(over="ignore"):  # a product beyond float32 is +-inf and clamps like any large value
        y = (x32 * inv).astype(_F32)
    y = np.maximum(np.minimum(y, _F32(448.0)), _F32(-448.0))
    return e4m3fn_encode(y), np.full((x32.shape[0],), _F32(scale), dtype=_F32)


def dynamic_per_tensor_quant_fp8(x: torch.Tensor):
    """Dynamic per-tensor FP8 quantisation, the scale-less branch of scaled_fp8_quant
    (python/sglang/srt/layers/quantization/fp8_kernel.py:1719-1726): scale = max(max|x|, 1e-12) / 448 (the floor is
    the native model's, :1675-1680), q = e4m3(clamp(float32(x) * (1 / scale))) -- the arithmetic the reference's own
    test states as the one its kernels align to (test/manual/quant/test_custom_ops.py:22-30,38-44).
    Returns (codes, scale as a float32 scalar array)."""
    x32 = _to_f32(x)
    scale = _F32(max(float(np.abs(x32).max()) if x32.size else 0.0, 1e-12)) / _F32(448.0)
    q, _ = static_quant_fp8(x, float(scale))
    return q, np.asarray([scale], dtype=_F32)


def per_token_quant_int8(x: torch.Tensor):
    """python/sglang/srt/layers/quantization/int8_kernel.py:46-50: amax = max(max|x|, 1e-10),
    scale = amax/127, q = int8(round_half_away(x * (127/amax)))."""
    x32 = _to_f32(x).reshape(-1, x.shape[-1])
    amax = np.maximum(np.abs(x32).max(axis=-1), _F32(1e-10)).astype(_F32)
    scale = (amax / _F32(127.0)).astype(_F32)
    y = (x32 * (_F32(127.0) / amax).astype(_F32)[:, None]).astype(_F32)
    q = (np.sign(y) * np.floor(np.abs(y) + _F32(0.5))).astype(np.int8)  # libdevice round(): half away from zero
    return q, scale


def block_quant_weight(w: torch.Tensor, block=(128, 128), dst: str = "fp8"):
    """Weight preparation used by the BASELINE configs: 128x128 blocks, s = max(amax, 1e-4)/448,
    q = e4m3(clamp(w / s)) (recipe of sgl-kernel/tests/test_fp8_blockwise_moe.py:44-60); dst="int8"
    rounds to the nearest integer in [-127, 127] with s = amax/127 instead (test input preparation only).
    Returns (q[N,K] uint8|int8, s[ceil(N/bn), ceil(K/bk)] float32)."""
    w32 = _to_f32(w)
    n, k = w32.shape
    bn, bk = block
    nb, kb = -(-n // bn), -(-k // bk)
    pad = np.zeros((nb * bn, kb * bk), dtype=_F32)
    pad[:n, :k] = w32
    v = pad.reshape(nb, bn, kb, bk)
    amax = np.maximum(np.abs(v).max(axis=(1, 3)), _F32(1e-4)).astype(_F32)
    max8 = _F32(448.0) if dst == "fp8" else _F32(127.0)
    s = (amax / max8).astype(_F32)
    y = (v / s[:, None, :, None]).astype(_F32)
    y = np.minimum(np.maximum(y, -max8), max8)
    q = e4m3fn_encode(y) if dst == "fp8" else np.rint(y).astype(np.int8)
    q = q.reshape(nb * bn, kb * bk)[:n, :k]
    return np.ascontiguousarray(q), s


def per_channel_quant_weight(w: torch.Tensor, dst: str = "fp8"):
    """Per-output-channel weight quantisation for the rowwise GEMMs: s_n = amax_n / max8."""
    w32 = _to_f32(w)
    max8 = _F32(448.0) if dst == "fp8" else _F32(127.0)
    amax = np.maximum(np.abs(w32).max(axis=1), _F32(1e-10)).astype(_F32)
    s = (amax / max8).astype(_F32)
    y = (w32 / s[:, None]).astype(_F32)
    y = np.minimum(np.maximum(y, -max8), max8)
    q = e4m3fn_encode(y) if dst == "fp8" else np.rint(y).astype(np.int8)
    return q, s


# ---- scale buffer layouts (python/sglang/srt/layers/quantization/fp8_kernel.py:454-495) ----

def pack_ue8m0(ebytes: np.ndarray) -> np.ndarray:
    """[rows, groups] exponent bytes -> logical int32 [rows, ceil(groups/4)]; byte g%4 of
    word g//4, unused tail bytes zero (per_token_group_quant_8bit_v2.cu:318-342)."""
    rows, groups = ebytes.shape
    words = -(-groups // 4)
    padded = np.zeros((rows, words * 4), dtype=np.uint8)
    padded[:, :groups] = ebytes
    return np.ascontiguousarray(padded).view("<i4").reshape(rows, words)


def fused_rms_group_quant(x1: torch.Tensor, w1: torch.Tensor, eps1: float, res1: torch.Tensor = None,
                          x2: torch.Tensor = None, w2: torch.Tensor = None, eps2: float = None, group_size: int = 128):
    """The native model of the fused RMSNorm + group quant (test/registered/quant/test_fused_rms_fp8_group_quant.py:
    _rmsnorm :23-27, _per_token_fp8_group_quant :30-52, _run_ref :84-95), evaluated in fp32 on the fp32 sum
    x1 + res1 as the fused kernel does (the test's torch model squares in the storage dtype and is compared at
    atol = rtol = 0.1).  The fused op itself lives in AITER (aiter.ops.triton.fused_fp8_quant, not part of the
    reference tree and not installed).
      s = x1 + res1;  y = s * rsqrt(sum(s^2)/N + eps) * w;  per group: amax = max(max|y|, 1e-10),
      scale = amax/448, q = e4m3(clamp(y * (1/scale))), the last group zero-padded.
    Returns dict(q uint8 [M,N1], s f32 [M,G], y1 f32 [M,N1] (unrounded), y2 f32 or None, res f32 or None)."""
    def rms(v, w, eps):
        n = _F32(v.shape[1])
        ss = (v * v).sum(axis=1, dtype=_F32)
        r = (_F32(1.0) / np.sqrt((ss / n + _F32(eps)).astype(_F32))).astype(_F32)
        return ((v * r[:, None]).astype(_F32) * _to_f32(w)[None, :]).astype(_F32)

    s = _to_f32(x1)
    if res1 is not None:
        s = (s + _to_f32(res1)).astype(_F32)
    y1 = rms(s, w1, eps1)
    m, n1 = y1.shape
    g = -(-n1 // group_size)
    pad = np.zeros((m, g * group_size), dtype=_F32)
    pad[:, :n1] = y1
    v = pad.reshape(m, g, group_size)
    amax = np.maximum(np.abs(v).max(axis=2), _F32(1e-10)).astype(_F32)
    scale = (amax / _F32(448.0)).astype(_F32)
    inv = (_F32(1.0) / scale).astype(_F32)
    yq = np.minimum(np.maximum((v * inv[:, :, None]).astype(_F32), _F32(-448.0)), _F32(448.0))
    q = e4m3fn_encode(yq).reshape(m, g * group_size)[:, :n1]
    y2 = rms(_to_f32(x2), w2, eps2) if x2 is not None else None
    return {"q": np.ascontiguousarray(q), "s": scale, "y1": y1, "y2": y2, "res": s if res1 is not None else None}

"""Fused RMSNorm + per-token-group FP8 quantisation with the call signature of
aiter.ops.triton.fused_fp8_quant.fused_rms_fp8_group_quant, as the reference uses it on gfx95
(python/sglang/srt/layers/communicator.py:552-624,
python/sglang/srt/models/deepseek_common/attention_forward_methods/forward_mla.py:175-203): the (fp8, scale)
pair it returns is what the block-FP8 linears accept as a pre-quantised input
(python/sglang/srt/layers/quantization/fp8.py:794-802)."""
from typing import Optional, Tuple

import torch

from .. import _lib
from .._lib import check, lib
from ..ops import _DT, _require, _stream


def fused_rms_fp8_group_quant(
    inp1: torch.Tensor,
    inp1_weight: torch.Tensor,
    inp1_epsilon: float,
    inp2: Optional[torch.Tensor] = None,
    inp2_weight: Optional[torch.Tensor] = None,
    inp2_epsilon: Optional[float] = None,
    group_size: int = 128,
    dtype_quant: torch.dtype = torch.float8_e4m3fn,
    res1: Optional[torch.Tensor] = None,
    output_unquantized_inp1: bool = False,
) -> Tuple[Tuple[torch.Tensor, torch.Tensor], Optional[torch.Tensor], Optional[torch.Tensor], Optional[torch.Tensor]]:
    """((y1_q [M, N1] fp8, y1_s [M, ceil(N1/128)] fp32), y1 or None, y2 or None, inp1 + res1 or None).
    inp1 [M, N1] and inp2 [M, N2] half/bfloat16, rows contiguous (a row stride is fine); res1 like inp1;
    weights fp32 or the activation dtype.  Everything is computed in fp32 from one read of each row; y1 is
    quantised before it is rounded to the activation dtype."""
    _require(inp1.dim() == 2 and inp1.is_cuda, "inp1 must be a 2D device tensor")
    _require(inp1.dtype in (torch.float16, torch.bfloat16), "inp1 must be Half or BFloat16")
    if dtype_quant != torch.float8_e4m3fn:
        raise NotImplementedError("only torch.float8_e4m3fn is implemented as dtype_quant")
    if group_size != 128:
        raise NotImplementedError("only group_size 128 is implemented")
    M, N1 = inp1.shape
    dev, dt = inp1.device, inp1.dtype
    _require(inp1.stride(1) == 1, "inp1 rows must be contiguous")
    _require(inp1_weight.numel() == N1 and inp1_weight.is_contiguous(), "inp1_weight must be contiguous [N1]")
    _require(inp1_weight.dtype in (torch.float32, torch.float16, torch.bfloat16), "weights must be Float, Half or BFloat16")
    res_out = None
    if res1 is not None:
        _require(res1.shape == inp1.shape and res1.dtype == dt and res1.is_contiguous(), "res1 must match inp1")
        res_out = torch.empty((M, N1), device=dev, dtype=dt)
    y2 = None
    N2 = 0
    if inp2 is not None:
        _require(inp2.dim() == 2 and inp2.size(0) == M and inp2.dtype == dt and inp2.stride(1) == 1,
                 "inp2 must be [M, N2] in inp1's dtype with contiguous rows")
        _require(inp2_weight is not None and inp2_epsilon is not None, "inp2 needs its weight and epsilon")
        N2 = inp2.size(1)
        _require(inp2_weight.numel() == N2 and inp2_weight.is_contiguous() and inp2_weight.dtype == inp1_weight.dtype,
                 "inp2_weight must be contiguous [N2] in inp1_weight's dtype")
        y2 = torch.empty((M, N2), device=dev, dtype=dt)
    y1_q = torch.empty((M, N1), device=dev, dtype=torch.float8_e4m3fn)
    y1_s = torch.empty((M, (N1 + 127) // 128), device=dev, dtype=torch.float32)
    y1 = torch.empty((M, N1), device=dev, dtype=dt) if output_unquantized_inp1 else None
    ptr = lambda t: t.data_ptr() if t is not None else None
    with torch.cuda.device(dev):
        check(lib.sglamd_fused_rms_fp8_group_quant(
            inp1.data_ptr(), inp1.stride(0), inp1_weight.data_ptr(), float(inp1_epsilon), ptr(res1), M, N1,
            y1_q.data_ptr(), y1_s.data_ptr(), ptr(y1), ptr(res_out), ptr(inp2), inp2.stride(0) if inp2 is not None else 0,
            ptr(inp2_weight), float(inp2_epsilon) if inp2 is not None else 0.0, N2, ptr(y2), _DT[dt],
            _DT[inp1_weight.dtype], 128, _stream(inp1)))
    return (y1_q, y1_s), y1, y2, res_out

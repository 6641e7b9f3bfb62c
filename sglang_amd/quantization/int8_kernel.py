"""INT8 activation quantisation callers
(python/sglang/srt/layers/quantization/int8_kernel.py:59-89)."""
import torch

from ..ops import per_token_quant_int8_


def per_token_quant_int8(x: torch.Tensor, scale_dtype=torch.float32, cal_sum: bool = False):
    """Returns (x_q int8 like x, scales [..., 1]); cal_sum additionally returns the row sums."""
    assert x.is_contiguous()
    assert scale_dtype == torch.float32, "only fp32 scales are produced"
    x_q = torch.empty_like(x, dtype=torch.int8)
    scales = torch.empty(x.shape[:-1] + (1,), device=x.device, dtype=torch.float32)
    per_token_quant_int8_(x, x_q, scales)
    if cal_sum:
        return x_q, scales, x.to(torch.float32).sum(dim=-1).to(x.dtype)
    return x_q, scales

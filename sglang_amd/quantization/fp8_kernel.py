"""Activation-quantisation callers and the block-FP8 matmul entry, with the reference's
names, arguments and scale-buffer layouts
(python/sglang/srt/layers/quantization/fp8_kernel.py:454-678,1135-1300)."""
from typing import List, Optional, Tuple

import torch

from ..gemm import (
    sgl_per_token_group_quant_8bit,
    sgl_per_token_quant_fp8,
)

fp8_dtype = torch.float8_e4m3fn
fp8_max = 448.0
fp8_min = -448.0


def ceil_align(x: int, y: int) -> int:
    return -(-x // y) * y


def _column_major(storage: torch.Tensor, rows: int) -> torch.Tensor:
    """View a [..., groups, padded_rows] buffer as [..., rows, groups] with unit stride along rows."""
    return storage.mT[..., :rows, :]


def create_per_token_group_quant_fp8_output_scale(
    x_shape, device, group_size, column_major_scales: bool, scale_tma_aligned: bool, scale_ue8m0: bool
):
    """Allocate the scale buffer in one of the four layouts of fp8_kernel.py:454-495:
      * UE8M0: four exponent bytes per int32, [..., rows, ceil(groups/4)] over column-major storage whose
        row count is padded to a multiple of 4 (groups are always 128 wide in this layout);
      * column-major fp32 with the row count padded to a multiple of 4;
      * column-major fp32 unpadded (the group index becomes the slowest dimension of the storage);
      * row-major fp32."""
    lead, rows, cols = tuple(x_shape[:-2]), x_shape[-2], x_shape[-1]
    f32 = dict(device=device, dtype=torch.float32)
    if scale_ue8m0:
        assert column_major_scales and scale_tma_aligned
        words = ceil_align(cols // 128, 4) // 4
        storage = torch.empty(lead + (words, ceil_align(rows, 4)), device=device, dtype=torch.int32)
        return _column_major(storage, rows)
    groups = cols // group_size
    if not column_major_scales:
        return torch.empty(lead + (rows, groups), **f32)
    if scale_tma_aligned:
        return torch.empty(lead + (groups, ceil_align(rows, 4)), **f32).transpose(-1, -2)[:rows, :]
    return torch.empty((groups,) + lead + (rows,), **f32).permute(-1, -2)


def _launch_group_quant(x, x_q, x_s, group_size, eps, lo, hi, ue8m0, silu_mul, masked_m, enable_v2):
    # the operator rejects empty launches; an empty batch has nothing to write
    if x.shape[0] > 0:
        sgl_per_token_group_quant_8bit(x, x_q, x_s, group_size, eps, lo, hi, ue8m0, silu_mul, masked_m,
                                       enable_v2=enable_v2)
    return x_q, x_s


def sglang_per_token_group_quant_fp8(
    x: torch.Tensor,
    group_size: int,
    eps: float = 1e-10,
    column_major_scales: bool = False,
    scale_tma_aligned: bool = False,
    scale_ue8m0: bool = False,
    fuse_silu_and_mul: bool = False,
    masked_m: Optional[torch.Tensor] = None,
    enable_v2: Optional[bool] = None,
):
    """fp8_kernel.py:498-565.  With `fuse_silu_and_mul` the input holds [gate | up] halves and the output has
    half its width.  `enable_v2=None` picks the second arithmetic for the group sizes it supports."""
    assert x.shape[-1] % group_size == 0, "the last dimension of `x` cannot be divisible by `group_size`"
    assert x.is_contiguous(), "`x` is not contiguous"
    width = x.shape[-1] // 2 if fuse_silu_and_mul else x.shape[-1]
    q_shape = x.shape[:-1] + (width,)
    x_q = x.new_empty(q_shape, dtype=fp8_dtype)
    x_s = create_per_token_group_quant_fp8_output_scale(q_shape, x.device, group_size, column_major_scales,
                                                        scale_tma_aligned, scale_ue8m0)
    v2 = group_size in (16, 32, 64, 128) if enable_v2 is None else enable_v2
    return _launch_group_quant(x, x_q, x_s, group_size, eps, fp8_min, fp8_max, scale_ue8m0, fuse_silu_and_mul,
                               masked_m, v2)


def sglang_per_token_group_quant_fp8_ue8m0(x: torch.Tensor, group_size: int, eps: float = 1e-10):
    """fp8_kernel.py:568-610: packed power-of-two scales; unlike the general entry the words per row follow
    `group_size` rather than a fixed 128."""
    assert x.shape[-1] % group_size == 0, f"hidden ({x.shape[-1]}) must be divisible by group_size ({group_size})"
    assert x.is_contiguous(), "x must be contiguous"
    rows = x.shape[-2]
    words = ceil_align(x.shape[-1] // group_size, 4) // 4
    x_q = x.new_empty(x.shape, dtype=fp8_dtype)
    x_s = _column_major(x.new_empty(x.shape[:-2] + (words, ceil_align(rows, 4)), dtype=torch.int32), rows)
    return _launch_group_quant(x, x_q, x_s, group_size, eps, fp8_min, fp8_max, True, False, None, True)


def sglang_per_token_group_quant_int8(x: torch.Tensor, group_size: int, eps: float = 1e-10,
                                      dtype: torch.dtype = torch.int8, enable_v2: Optional[bool] = None):
    """int8 sibling (python/sglang/srt/layers/quantization/int8_kernel.py:184-225): row-major fp32 scales."""
    assert x.shape[-1] % group_size == 0
    assert x.is_contiguous()
    x_q = torch.empty_like(x, dtype=dtype)
    x_s = torch.empty(x.shape[:-1] + (x.shape[-1] // group_size,), device=x.device, dtype=torch.float32)
    if x.numel() > 0:
        sgl_per_token_group_quant_8bit(x, x_q, x_s, group_size, eps, -128.0, 127.0, False, enable_v2=enable_v2)
    return x_q, x_s


def sglang_per_token_group_quant_8bit(
    x: torch.Tensor,
    group_size: int,
    dst_dtype: torch.dtype,
    eps: float = 1e-10,
    column_major_scales: bool = False,
    scale_tma_aligned: bool = False,
    scale_ue8m0: bool = False,
    fuse_silu_and_mul: bool = False,
    masked_m: Optional[torch.Tensor] = None,
    enable_v2: Optional[bool] = None,
):
    """fp8_kernel.py:614-653: int8 takes none of the layout or fusion options."""
    if dst_dtype != torch.int8:
        return sglang_per_token_group_quant_fp8(x, group_size, eps, column_major_scales, scale_tma_aligned,
                                                scale_ue8m0, fuse_silu_and_mul, masked_m, enable_v2)
    assert not (column_major_scales or scale_tma_aligned or fuse_silu_and_mul), \
        "int8 group quantisation writes plain row-major scales"
    assert masked_m is None
    return sglang_per_token_group_quant_int8(x, group_size, eps, dst_dtype, enable_v2)


def sglang_per_token_quant_fp8(x: torch.Tensor, dtype: torch.dtype = fp8_dtype):
    """fp8_kernel.py:656-672: one scale per row, shape [rows, 1]."""
    assert x.is_contiguous(), "`x` is not contiguous"
    x_q = x.new_empty(x.shape, dtype=dtype)
    x_s = x.new_empty((x.shape[0], 1), dtype=torch.float32)
    sgl_per_token_quant_fp8(x, x_q, x_s)
    return x_q, x_s


def static_quant_fp8(x: torch.Tensor, x_s: torch.Tensor, repeat_scale: bool = False):
    """fp8_kernel.py:724-777: quantise with a given per-tensor scale, q = e4m3(clamp(x * (1 / x_s))); with
    `repeat_scale` the scale comes back broadcast to one per row, [rows, 1], as the row-scaled GEMM takes it."""
    from ..ops import static_quant_fp8_

    assert x.is_contiguous(), "`x` is not contiguous"
    assert x_s.numel() == 1, "only supports per-tensor scale"
    x_q = torch.empty_like(x, dtype=fp8_dtype)
    rows = x.numel() // x.shape[-1]
    x_s_repeat = torch.empty((rows, 1), device=x.device, dtype=torch.float32) if repeat_scale else None
    scale = x_s.reshape(1) if x_s.dtype == torch.float32 else x_s.reshape(1).to(torch.float32)
    static_quant_fp8_(x.view(rows, x.shape[-1]), x_q.view(rows, x.shape[-1]), scale, x_s_repeat)
    return x_q, (x_s_repeat if repeat_scale else x_s)


def scaled_fp8_quant(input: torch.Tensor, scale: Optional[torch.Tensor] = None,
                     num_token_padding: Optional[int] = None, use_per_token_if_dynamic: bool = False):
    """fp8_kernel.py:1693-1777: FP8 quantisation of a 2D tensor with a given per-tensor scale (static), or with a
    scale computed here: one per token ([rows, 1]) or one for the tensor ([1], max|x| / 448).  The output has
    max(num_token_padding, rows) rows; rows past the input are left unwritten, as in the reference."""
    from ..ops import static_quant_fp8_, tensor_absmax_scale_

    assert input.ndim == 2, f"Expected 2D input tensor, got {input.ndim}D"
    rows, hidden = input.shape
    out_rows = max(num_token_padding, rows) if num_token_padding else rows
    output = torch.empty((out_rows, hidden), device=input.device, dtype=fp8_dtype)
    x = input if input.is_contiguous() else input.contiguous()
    if scale is None and use_per_token_if_dynamic:
        scale = torch.empty((out_rows, 1), device=input.device, dtype=torch.float32)
        if rows:
            sgl_per_token_quant_fp8(x, output[:rows], scale[:rows])
        return output, scale
    if scale is None:
        scale = torch.zeros(1, device=input.device, dtype=torch.float32)
        tensor_absmax_scale_(x, scale)
    else:
        assert scale.numel() == 1, f"Expected scalar scale, got numel={scale.numel()}"
    if rows:
        s32 = scale.reshape(1) if scale.dtype == torch.float32 else scale.reshape(1).to(torch.float32)
        static_quant_fp8_(x, output[:rows], s32, None)
    return output, scale


# on this backend the operator is always the sgl_kernel one (fp8_kernel.py:675-678)
per_token_group_quant_fp8 = sglang_per_token_group_quant_fp8


def _cdiv(a: int, b: int) -> int:
    return (a + b - 1) // b


def prepare_block_fp8_matmul_inputs(A, B, As, Bs, block_size: List[int], output_dtype: torch.dtype = torch.float16):
    """Shape checks and output allocation of fp8_kernel.py:1135-1180: fp32 scales, or int32 words of four packed
    UE8M0 exponents (activations [..., ceil(kb/4)], weights one row of words per weight row)."""
    assert len(block_size) == 2
    block_n, block_k = block_size
    K = A.shape[-1]
    assert A.shape[-1] == B.shape[-1]
    assert A.shape[:-1] == As.shape[:-1]
    assert A.is_contiguous()
    if As.dtype == torch.float32:
        assert _cdiv(K, block_k) == As.shape[-1]
    elif As.dtype == torch.int32:
        assert _cdiv(_cdiv(K, block_k), 4) == As.shape[-1], f"{A.shape=} {As.shape=} {block_size=}"
    else:
        raise NotImplementedError
    M = A.numel() // K
    assert B.ndim == 2
    assert B.is_contiguous()
    assert Bs.ndim == 2
    N = B.shape[0]
    if Bs.dtype == torch.float32:
        assert _cdiv(N, block_n) == Bs.shape[0]
        assert _cdiv(K, block_k) == Bs.shape[1]
    elif Bs.dtype == torch.int32:
        assert N == Bs.shape[0], f"{B.shape=} {Bs.shape=} {block_size=}"
        assert _cdiv(_cdiv(K, block_k), 4) == Bs.shape[1], f"{B.shape=} {Bs.shape=} {block_size=}"
    else:
        raise NotImplementedError
    C = A.new_empty(A.shape[:-1] + (N,), dtype=output_dtype)
    return M, N, K, C


def w8a8_block_fp8_matmul(A, B, As, Bs, block_size: List[int], output_dtype: torch.dtype = torch.float16):
    """Block-wise W8A8 matmul with row-major scales (fp8_kernel.py:1201-1300): A [..., K] e4m3fn,
    B [N, K] e4m3fn, As [..., ceil(K/block_k)], Bs [ceil(N/block_n), ceil(K/block_k)] -> [..., N]; block_size
    [128, 128] runs the specialised kernels, 64 in either direction the generic one.  Packed UE8M0 scales
    (what the quantiser writes with scale_ue8m0=True; for the weights the same words on every row of a block)
    are expanded to the fp32 powers of two they stand for by one small launch each; when both operands came with
    such scales the GEMM is told so (the large-tile kernel then applies them inside the MFMA)."""
    from ..ops import ue8m0_unpack_, w8a8_block_fp8_matmul_

    M, N, K, C = prepare_block_fp8_matmul_inputs(A, B, As, Bs, block_size, output_dtype)
    assert output_dtype in (torch.float16, torch.bfloat16)
    if list(block_size) != [128, 128]:
        # other scale-block shapes (the reference's kernel is generic in them): the generic kernel, float scales
        from ..ops import block_scaled_mm_any_

        if not all(b in (64, 128) for b in block_size) or As.dtype != torch.float32 or Bs.dtype != torch.float32:
            raise NotImplementedError("scale blocks of 64 or 128 in each direction with float scales are implemented")
        As2 = As.reshape(M, As.shape[-1])
        block_scaled_mm_any_(A.view(M, K), B, As2 if As2.is_contiguous() else As2.contiguous(), Bs, C.view(M, N),
                             block_size[0], block_size[1])
        return C
    kb = _cdiv(K, 128)
    pow2 = As.dtype == torch.int32 and Bs.dtype == torch.int32
    if As.dtype == torch.int32:
        As = ue8m0_unpack_(As.reshape(M, As.shape[-1]) if As.dim() != 2 else As, M, kb, row_step=1)
    elif not As.is_contiguous():
        As = As.contiguous()
    if Bs.dtype == torch.int32:
        Bs = ue8m0_unpack_(Bs, _cdiv(N, 128), kb, row_step=128)
    w8a8_block_fp8_matmul_(A.view(M, K), B, As.view(M, -1), Bs, C.view(M, N), pow2_scales=pow2)
    return C


w8a8_block_fp8_matmul_triton = w8a8_block_fp8_matmul  # same contract; there is no Triton here
w8a8_block_fp8_matmul_deepgemm = w8a8_block_fp8_matmul  # fp8_kernel.py:1149-1174: the packed-UE8M0 caller

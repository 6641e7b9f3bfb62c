"""Registers the quantized-linear operators under ``torch.ops.sgl_kernel`` with the
reference's schema strings (sgl-kernel/csrc/common_extension.cc:76-77,116-142,164-168,
180-181) and implements each for device tensors by unpacking the tensors into raw
pointers / sizes / element strides / the current HIP stream and calling the C-ABI library.

The checks in each implementation raise RuntimeError with the reference's message text
before anything is launched, mirroring its TORCH_CHECKs.  Nothing here allocates except
the value-returning GEMMs, which allocate their output like the reference does.

This module must be the only provider of the ``sgl_kernel`` namespace in the process: a
second library defining the same schemas is a hard error in the dispatcher.
"""
from typing import Optional

import torch

from . import _lib
from ._lib import check, lib

_DT = {
    torch.float32: _lib.F32,
    torch.float16: _lib.F16,
    torch.bfloat16: _lib.BF16,
    torch.float8_e4m3fn: _lib.FP8_E4M3,
    torch.int8: _lib.I8,
    torch.int32: _lib.I32,
    torch.int64: _lib.I64,
}

_library = torch.library.Library("sgl_kernel", "FRAGMENT")
_registered = []


def _stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _require(cond: bool, msg: str) -> None:
    if not cond:
        raise RuntimeError(msg)


def _check_input(t: torch.Tensor, name: str) -> None:
    # CHECK_INPUT of the reference: device tensor + contiguous
    _require(t.is_cuda, f"{name} must be a CUDA tensor")
    _require(t.is_contiguous(), f"{name} must be contiguous")


def _op(schema: str):
    """Defines `schema` in sgl_kernel and registers the decorated function for device tensors."""
    name = schema.split("(", 1)[0]

    def deco(fn):
        _library.define(schema)
        _library.impl(name, fn, "CUDA")
        _registered.append(name)
        return fn

    return deco


# --------------------------------------------------------------------------------------
# group quant (v1: divide form; v2: reciprocal form)
# --------------------------------------------------------------------------------------
def _group_quant(input, output_q, output_s, group_size, eps, min8, max8, scale_ue8m0, form, col_major,
                 fuse_silu_and_mul=False):
    hidden = input.size(-1)
    rows = input.numel() // hidden
    if fuse_silu_and_mul:
        # input rows are [gate | up]; the quantised row has half the width (v2.cu:412-424)
        _require(hidden % 2 == 0 and output_q.size(-1) == hidden // 2, "output_q must have half of input's last dim")
        hidden //= 2
        _require(hidden % group_size == 0, "hidden size must be a multiple of group_size")
    fn = lib.sglamd_silu_mul_group_quant_8bit if fuse_silu_and_mul else lib.sglamd_per_token_group_quant_8bit
    if col_major:
        layout = _lib.SCALE_COL_MAJOR_UE8M0 if scale_ue8m0 else _lib.SCALE_COL_MAJOR
        scale_stride = output_s.stride(-1)
    else:
        _require(not scale_ue8m0, "scale_ue8m0 requires column-major scales")
        _require(output_s.is_contiguous(), "row-major output_s must be contiguous")
        layout, scale_stride = _lib.SCALE_ROW_MAJOR, 0
    _require(input.dtype in (torch.float32, torch.float16, torch.bfloat16), "input must be Float, Half or BFloat16")
    _require(output_q.dtype in (torch.float8_e4m3fn, torch.int8), "output_q must be Float8_e4m3fn or Char")
    if scale_ue8m0:
        _require(output_s.dtype == torch.int32, "UE8M0 output_s must be Int (four exponents per element)")
    else:
        _require(output_s.dtype == torch.float32, "output_s must be Float32")
    with torch.cuda.device(input.device):
        check(fn(
            input.data_ptr(), _DT[input.dtype], output_q.data_ptr(), _DT[output_q.dtype], output_s.data_ptr(),
            rows, hidden, int(group_size), layout, int(scale_stride), float(eps), float(min8), float(max8), form,
            _stream(input)))


@_op("sgl_per_token_group_quant_8bit(Tensor input, Tensor! output_q, Tensor! output_s, int group_size,"
     " float eps, float fp8_min, float fp8_max, bool scale_ue8m0) -> ()")
def sgl_per_token_group_quant_8bit(input, output_q, output_s, group_size, eps, fp8_min, fp8_max, scale_ue8m0):
    """per_token_group_quant_8bit.cu:116-217: contiguous inputs, numel % group == 0, 2-D scales,
    column-major when output_s.stride(0) < output_s.stride(1)."""
    _check_input(input, "input")
    _check_input(output_q, "output_q")
    _require(input.numel() % group_size == 0, "input.numel() % group_size must be 0")
    _require(output_s.dim() == 2, "output_s.dim() must be 2")
    _require(input.size(-1) % group_size == 0, "hidden size must be a multiple of group_size")
    col_major = output_s.stride(0) < output_s.stride(1)
    _group_quant(input, output_q, output_s, group_size, eps, fp8_min, fp8_max, scale_ue8m0, _lib.FORM_DIVIDE,
                 col_major)


@_op("sgl_per_token_group_quant_8bit_v2(Tensor input, Tensor! output_q, Tensor! output_s, int group_size,"
     " float eps, float fp8_min, float fp8_max, bool scale_ue8m0, bool fuse_silu_and_mul, Tensor? masked_m) -> ()")
def sgl_per_token_group_quant_8bit_v2(input, output_q, output_s, group_size, eps, fp8_min, fp8_max, scale_ue8m0,
                                      fuse_silu_and_mul, masked_m):
    """per_token_group_quant_8bit_v2.cu:411-542 (checks :425-447,482-527)."""
    _check_input(input, "input")
    _check_input(output_q, "output_q")
    _require(input.numel() > 0, "input.numel() must be > 0")
    _require(abs(1e-10 - eps) < 1e-13, "eps must be 1e-10")
    _require(input.numel() % group_size == 0, "input.numel() % group_size must be 0")
    masked_layout = masked_m is not None
    _require(output_s.dim() == (3 if masked_layout else 2), f"output_s.dim() must be {3 if masked_layout else 2}")
    _require(group_size in (16, 32, 64, 128), "Unsupported group_size")
    _require(input.dtype in (torch.float16, torch.bfloat16), "input must be Half or BFloat16")
    if output_q.dtype == torch.int8:
        _require(fp8_min == -128 and fp8_max == 127, "min_8bit/max_8bit must be -128/127 for int8")
    else:
        _require(output_q.dtype == torch.float8_e4m3fn, "output_q must be Float8_e4m3fn or Char")
        _require(fp8_min == -448 and fp8_max == 448, "min_8bit/max_8bit must be -448/448 for float8_e4m3fn")
    if masked_layout and scale_ue8m0 and fuse_silu_and_mul and output_s.stride(-2) < output_s.stride(-1):
        # the one combination that walks the masked layout (v2.cu:489-494): [experts, tokens, 2*hidden] input,
        # only the first masked_m[e] tokens of each expert are processed
        _require(input.dim() == 3 and output_q.dim() == 3, "masked layout takes [experts, tokens, hidden] tensors")
        _require(masked_m.dtype == torch.int32 and masked_m.is_cuda and masked_m.is_contiguous(),
                 "masked_m must be a contiguous CUDA Int tensor")
        experts, tokens, hidden2 = input.shape
        _require(masked_m.numel() == experts, "masked_m must hold one count per local expert")
        _require(hidden2 % 2 == 0 and output_q.size(-1) == hidden2 // 2 and output_q.size(-2) == tokens,
                 "output_q must have half of input's last dim")
        _require((hidden2 // 2) % group_size == 0, "hidden size must be a multiple of group_size")
        _require(output_s.dtype == torch.int32 and output_s.stride(-2) == 1,
                 "UE8M0 output_s must be Int (four exponents per element), token-contiguous")
        with torch.cuda.device(input.device):
            check(lib.sglamd_silu_mul_group_quant_8bit_masked(
                input.data_ptr(), _DT[input.dtype], output_q.data_ptr(), _DT[output_q.dtype], output_s.data_ptr(),
                experts, tokens, hidden2 // 2, int(group_size), int(output_s.stride(0)), int(output_s.stride(-1)),
                masked_m.data_ptr(), float(eps), float(fp8_min), float(fp8_max), _stream(input)))
        return
    # every other combination ignores masked_m and walks all tokens (NaiveScheduler, v2.cu:495-510)
    col_major = output_s.stride(-2) < output_s.stride(-1)
    _group_quant(input, output_q, output_s, group_size, eps, fp8_min, fp8_max, scale_ue8m0, _lib.FORM_RECIPROCAL,
                 col_major, fuse_silu_and_mul=bool(fuse_silu_and_mul))


@_op("sgl_per_token_quant_fp8(Tensor input, Tensor! output_q, Tensor! output_s) -> ()")
def sgl_per_token_quant_fp8(input, output_q, output_s):
    """per_token_quant_fp8.cu:242-314."""
    _check_input(input, "input")
    _check_input(output_q, "output_q")
    _check_input(output_s, "output_s")
    _require(input.dim() == 2, "input must be 2D")
    rows, hidden = input.shape
    _require(hidden % 4 == 0, f"Hidden dimension must be divisible by 4, but got {hidden}")
    _require(output_q.dtype == torch.float8_e4m3fn and output_s.dtype == torch.float32,
             "output_q must be Float8_e4m3fn and output_s Float32")
    _require(output_s.numel() == rows, "output_s must hold one scale per token")
    if rows == 0:
        return
    with torch.cuda.device(input.device):
        check(lib.sglamd_per_token_quant_fp8(input.data_ptr(), _DT[input.dtype], output_q.data_ptr(),
                                             output_s.data_ptr(), rows, hidden, _stream(input)))


def static_quant_fp8_(input: torch.Tensor, output_q: torch.Tensor, scale: torch.Tensor, scale_rows=None) -> None:
    """Launcher of the static per-tensor quantiser (the Triton _static_quant_fp8, fp8_kernel.py:681-721): input
    [rows, hidden] contiguous, scale one float32 on the device, scale_rows an optional float32 [rows] that receives
    the scale once per row."""
    _check_input(input, "input")
    _check_input(output_q, "output_q")
    _require(input.dim() == 2 and output_q.shape == input.shape, "input and output_q must be 2D of the same shape")
    _require(output_q.dtype == torch.float8_e4m3fn, "output_q must be Float8_e4m3fn")
    _require(scale.is_cuda and scale.dtype == torch.float32 and scale.numel() == 1, "scale must be one Float32 on the device")
    rows, hidden = input.shape
    if scale_rows is not None:
        _require(scale_rows.is_cuda and scale_rows.dtype == torch.float32 and scale_rows.is_contiguous()
                 and scale_rows.numel() == rows, "scale_rows must be a contiguous Float32 tensor of one scale per row")
    _require(hidden % 8 == 0, f"the row length must be a multiple of 8, but got {hidden}")
    if rows == 0:
        return
    with torch.cuda.device(input.device):
        check(lib.sglamd_static_quant_fp8(input.data_ptr(), _DT[input.dtype], output_q.data_ptr(), scale.data_ptr(),
                                          scale_rows.data_ptr() if scale_rows is not None else None, rows, hidden,
                                          _stream(input)))


def tensor_absmax_scale_(input: torch.Tensor, scale: torch.Tensor, eps: float = 1e-12, fp8_max: float = 448.0) -> None:
    """scale[0] = max(max|input|, eps) / fp8_max: the scale of dynamic per-tensor quantisation
    (fp8_kernel.py:1675-1685,1719-1726)."""
    _require(input.is_cuda and input.is_contiguous() and input.dtype in (torch.float32, torch.float16, torch.bfloat16),
             "input must be a contiguous float32, float16 or bfloat16 CUDA tensor")
    _require(scale.is_cuda and scale.dtype == torch.float32 and scale.numel() >= 1, "scale must be a Float32 CUDA tensor")
    if input.numel() == 0:
        scale.fill_(eps / fp8_max)
        return
    ws = torch.empty(1024, device=input.device, dtype=torch.float32)
    with torch.cuda.device(input.device):
        check(lib.sglamd_tensor_absmax_scale(input.data_ptr(), _DT[input.dtype], input.numel(), float(eps), float(fp8_max),
                                             scale.data_ptr(), ws.data_ptr(), _stream(input)))


def per_token_quant_int8_(input: torch.Tensor, output_q: torch.Tensor, output_s: torch.Tensor) -> None:
    """In-place launcher for the per-token INT8 quantiser (int8_kernel.py:28-89 is a Triton
    kernel in the reference, so there is no sgl_kernel schema to mirror)."""
    _check_input(input, "input")
    _check_input(output_q, "output_q")
    _check_input(output_s, "output_s")
    hidden = input.size(-1)
    rows = input.numel() // hidden
    if rows == 0:
        return
    with torch.cuda.device(input.device):
        check(lib.sglamd_per_token_quant_int8(input.data_ptr(), _DT[input.dtype], output_q.data_ptr(),
                                              output_s.data_ptr(), rows, hidden, _stream(input)))


# --------------------------------------------------------------------------------------
# GEMMs
# --------------------------------------------------------------------------------------
_workspaces = {}


def _gemm_workspace(M: int, N: int, K: int, device):
    """fp32 split-K scratch when the library can use one for this shape.  One grow-only buffer per device and
    stream: calls on one stream are ordered, so they can share it, and the mid-sized shapes that split K do not pay
    an allocator round trip per call.  Under stream capture the buffer comes from the capturing graph's pool
    instead (a buffer cached outside could be freed while the graph still names it)."""
    need = int(lib.sglamd_gemm_workspace_bytes(M, N, K))
    if need <= 0:
        return None, 0, 0
    if torch.cuda.is_current_stream_capturing():
        ws = torch.empty(need, dtype=torch.uint8, device=device)
        return ws, ws.data_ptr(), need
    key = (device.index if device.index is not None else torch.cuda.current_device(),
           torch.cuda.current_stream(device).cuda_stream)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < need:
        ws = torch.empty(max(need, 1 << 20), dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws, ws.data_ptr(), need


def _is_contiguous_vector(t: torch.Tensor) -> bool:
    return t.is_contiguous() and (t.dim() == 1 or (t.dim() == 2 and min(t.shape) == 1))


def _check_mm_operands(mat_a, mat_b, dtype, dtype_name, out_dtype):
    _require(mat_a.is_cuda, "mat_a must be a CUDA tensor")
    _require(mat_b.is_cuda, "mat_b must be a CUDA tensor")
    _require(mat_a.dim() == 2, "mat_a must be a 2D tensor")
    _require(mat_b.dim() == 2, "mat_b must be a 2D tensor")
    _require(mat_a.stride(1) == 1, "mat_a must be a row major tensor")
    _require(mat_b.stride(0) == 1, "mat_b must be a column major tensor")
    _require(mat_a.size(1) == mat_b.size(0), "mat_a and mat_b shapes cannot be multiplied")
    _require((mat_a.size(1) * mat_a.element_size()) % 16 == 0,
             "mat_a must be multiple of 16 bytes for memory alignment")
    _require((mat_b.size(0) * mat_b.element_size()) % 16 == 0,
             "mat_b must be multiple of 16 bytes for memory alignment")
    _require(mat_a.dtype == dtype, f"mat_a must be {dtype_name}")
    _require(mat_b.dtype == dtype, f"mat_b must be {dtype_name}")
    _require(out_dtype in (torch.float16, torch.bfloat16), "out_dtype must be Half or BFloat16")


def _ld(t: torch.Tensor, dim: int) -> int:
    """Leading stride for a matrix whose other dimension is contiguous (a 1-row matrix may
    report any stride there; use the row length then)."""
    other = 1 - dim
    return t.stride(dim) if t.size(dim) > 1 else max(t.stride(dim), t.size(other))


@_op("fp8_blockwise_scaled_mm(Tensor mat_a, Tensor mat_b, Tensor scales_a, Tensor scales_b, ScalarType out_dtype) -> "
     "Tensor")
def fp8_blockwise_scaled_mm(mat_a, mat_b, scales_a, scales_b, out_dtype):
    """fp8_blockwise_gemm_kernel.cu:425-522 (checks :431-463)."""
    _check_mm_operands(mat_a, mat_b, torch.float8_e4m3fn, "Float8_e4m3fn", out_dtype)
    M, K = mat_a.shape
    N = mat_b.size(1)
    _require(scales_a.dim() == 2 and scales_b.dim() == 2, "scales must be 2D tensors")
    _require(M == scales_a.size(0), "size of scales_a is not matched")
    _require(K // 128 == scales_a.size(1), "size of scales_a is not matched")
    _require(scales_a.stride(0) == 1 or _is_contiguous_vector(scales_a), "scales_a must be M major")
    _require(K // 128 == scales_b.size(0), "size of scales_b is not matched")
    _require(N // 128 == scales_b.size(1), "size of scales_b is not matched")
    _require(scales_b.stride(0) == 1 or _is_contiguous_vector(scales_b), "scales_b must be K major")
    _require(scales_a.dtype == torch.float32, "scales_a must be Float32")
    _require(scales_b.dtype == torch.float32, "scales_b must be Float32")
    _require(K % 128 == 0 and N % 128 == 0, "K and N must be multiples of the 128x128 scale block")
    out = torch.empty((M, N), device=mat_a.device, dtype=out_dtype)
    _require((N * out.element_size()) % 16 == 0, "out must be multiple of 16 bytes for memory alignment")
    if M == 0:
        return out
    with torch.cuda.device(mat_a.device):
        ws, ws_ptr, ws_bytes = _gemm_workspace(M, N, K, mat_a.device)
        check(lib.sglamd_fp8_blockwise_scaled_mm(
            mat_a.data_ptr(), _ld(mat_a, 0), mat_b.data_ptr(), _ld(mat_b, 1),
            scales_a.data_ptr(), scales_a.stride(0), scales_a.stride(1),
            scales_b.data_ptr(), scales_b.stride(1), scales_b.stride(0),
            out.data_ptr(), N, _DT[out_dtype], M, N, K, ws_ptr, ws_bytes, _stream(mat_a)))
    return out


def w8a8_block_fp8_matmul_(A, B, As, Bs, C, pow2_scales: bool = False) -> None:
    """Row-major-scale entry used by w8a8_block_fp8_matmul (fp8_kernel.py:1135-1281): A [M,K], B [N,K]
    both contiguous, As [M, ceil(K/128)], Bs [ceil(N/128), ceil(K/128)], C [M,N] preallocated.  pow2_scales: the
    caller vouches that every scale is a power of two (expanded UE8M0 scales), which lets the large-tile kernel apply
    them inside the MFMA."""
    M, K = A.shape
    N = B.shape[0]
    if M == 0:
        return
    with torch.cuda.device(A.device):
        ws, ws_ptr, ws_bytes = _gemm_workspace(M, N, K, A.device)
        entry = lib.sglamd_fp8_blockwise_scaled_mm_pow2 if pow2_scales else lib.sglamd_fp8_blockwise_scaled_mm
        check(entry(
            A.data_ptr(), _ld(A, 0), B.data_ptr(), _ld(B, 0),
            As.data_ptr(), As.stride(0), As.stride(1),
            Bs.data_ptr(), Bs.stride(0), Bs.stride(1),
            C.data_ptr(), C.stride(0), _DT[C.dtype], M, N, K, ws_ptr, ws_bytes, _stream(A)))


def ue8m0_unpack_(packed: torch.Tensor, rows: int, groups: int, row_step: int = 1) -> torch.Tensor:
    """fp32 [rows, groups] scales out of int32 words of four UE8M0 exponent bytes each: row r reads row
    r * row_step of `packed` ([packed_rows, ceil(groups/4)], any strides).  The expansion (byte << 23 as a float)
    is the reference's own (fp8_utils.py:1348-1383)."""
    _require(packed.is_cuda and packed.dtype == torch.int32 and packed.dim() == 2, "packed scales must be a 2D CUDA Int tensor")
    _require(packed.size(1) * 4 >= groups and (rows == 0 or packed.size(0) > (rows - 1) * row_step),
             "packed scales do not cover the requested rows and groups")
    out = torch.empty((rows, groups), device=packed.device, dtype=torch.float32)
    with torch.cuda.device(packed.device):
        check(lib.sglamd_ue8m0_unpack(packed.data_ptr(), packed.stride(0), packed.stride(1), int(row_step),
                                      out.data_ptr(), rows, groups, _stream(packed)))
    return out


def w8a8_block_int8_matmul_(A, B, As, Bs, C) -> None:
    """Block-scaled INT8 twin of w8a8_block_fp8_matmul_ (int8_kernel.py:355-425): A [M,K] int8, B [N,K] int8
    both contiguous, As [M, ceil(K/128)], Bs [ceil(N/128), ceil(K/128)] fp32, C [M,N] preallocated."""
    M, K = A.shape
    N = B.shape[0]
    if M == 0:
        return
    with torch.cuda.device(A.device):
        ws, ws_ptr, ws_bytes = _gemm_workspace(M, N, K, A.device)
        check(lib.sglamd_int8_blockwise_scaled_mm(
            A.data_ptr(), _ld(A, 0), B.data_ptr(), _ld(B, 0),
            As.data_ptr(), As.stride(0), As.stride(1),
            Bs.data_ptr(), Bs.stride(0), Bs.stride(1),
            C.data_ptr(), C.stride(0), _DT[C.dtype], M, N, K, ws_ptr, ws_bytes, _stream(A)))


def block_scaled_mm_any_(A, B, As, Bs, C, block_n: int, block_k: int) -> None:
    """The block-scaled GEMM with a general scale-block shape (fp8_kernel.py:780-869, int8_kernel.py:228-441):
    A [M, K], B [N, K] e4m3fn or int8, As [M, ceil(K/block_k)], Bs [ceil(N/block_n), ceil(K/block_k)] fp32,
    C [M, N] preallocated; block_n, block_k in {64, 128}."""
    M, K = A.shape
    N = B.shape[0]
    if M == 0:
        return
    _require(A.dtype in (torch.float8_e4m3fn, torch.int8) and B.dtype == A.dtype,
             "A and B must both be Float8_e4m3fn or both Int8")
    with torch.cuda.device(A.device):
        check(lib.sglamd_block_scaled_mm_any(
            A.data_ptr(), _ld(A, 0), B.data_ptr(), _ld(B, 0),
            As.data_ptr(), As.stride(0), As.stride(1),
            Bs.data_ptr(), Bs.stride(0), Bs.stride(1),
            C.data_ptr(), C.stride(0), _DT[C.dtype], _DT[A.dtype], M, N, K, int(block_n), int(block_k), _stream(A)))


def _rowwise_mm(fn, mat_a, mat_b, scales_a, scales_b, out_dtype, bias):
    M, K = mat_a.shape
    N = mat_b.size(1)
    _require(scales_a.numel() == M, "size of scales_a is not matched")
    _require(scales_b.numel() == N, "size of scales_b is not matched")
    _require(scales_a.is_contiguous(), "scales_a must be contiguous")
    _require(scales_b.is_contiguous(), "scales_b msut be contiguous")
    _require(scales_a.dtype == torch.float32, "scales_a must be Float32")
    _require(scales_b.dtype == torch.float32, "scales_b must be Float32")
    if bias is not None:
        _require(bias.numel() == N, "size of bias is not matched")
        _require(bias.is_contiguous(), "bias must be contiguous")
        _require(bias.dtype == out_dtype, "bias dtype must match output dtype")
    out = torch.empty((M, N), device=mat_a.device, dtype=out_dtype)
    if M == 0:
        return out
    with torch.cuda.device(mat_a.device):
        ws, ws_ptr, ws_bytes = _gemm_workspace(M, N, K, mat_a.device)
        check(fn(mat_a.data_ptr(), _ld(mat_a, 0), mat_b.data_ptr(), _ld(mat_b, 1), scales_a.data_ptr(),
                 scales_b.data_ptr(), bias.data_ptr() if bias is not None else None, out.data_ptr(), N,
                 _DT[out_dtype], M, N, K, ws_ptr, ws_bytes, _stream(mat_a)))
    return out


@_op("fp8_scaled_mm(Tensor mat_a, Tensor mat_b, Tensor scales_a, Tensor scales_b, ScalarType out_dtype, Tensor? "
     "bias) -> Tensor")
def fp8_scaled_mm(mat_a, mat_b, scales_a, scales_b, out_dtype, bias=None):
    """fp8_gemm_kernel.cu:1095-1173 (checks :1102-1132)."""
    _check_mm_operands(mat_a, mat_b, torch.float8_e4m3fn, "Float8_e4m3fn", out_dtype)
    _require((mat_b.size(1) * 2) % 16 == 0, "out must be multiple of 16 bytes for memory alignment")
    return _rowwise_mm(lib.sglamd_fp8_scaled_mm, mat_a, mat_b, scales_a, scales_b, out_dtype, bias)


@_op("int8_scaled_mm(Tensor mat_a, Tensor mat_b, Tensor scales_a, Tensor scales_b, ScalarType out_dtype, Tensor? "
     "bias) -> Tensor")
def int8_scaled_mm(mat_a, mat_b, scales_a, scales_b, out_dtype, bias=None):
    """int8_gemm_kernel.cu:663-747 (checks :670-695)."""
    _require(mat_a.is_cuda, "mat_a must be a CUDA tensor")
    _require(mat_b.is_cuda, "mat_b must be a CUDA tensor")
    _require(mat_a.dim() == 2, "mat_a must be a 2D tensor")
    _require(mat_b.dim() == 2, "mat_b must be a 2D tensor")
    _require(mat_a.stride(1) == 1, "mat_a must be a row major tensor")
    _require(mat_b.stride(0) == 1, "mat_b must be a column major tensor")
    _require(mat_a.size(1) == mat_b.size(0), "mat_a and mat_b shapes cannot be multiplied")
    _require(mat_a.size(1) % 16 == 0, "mat_a.size(1) must be multiple of 16 for memory alignment")
    _require(mat_b.size(0) % 16 == 0, "mat_b.size(0) must be multiple of 16 for memory alignment")
    _require(mat_b.size(1) % 8 == 0, "mat_b.size(1) must be multiple of 8 for memory alignment")
    _require(mat_a.dtype == torch.int8, "mat_a must be Int8")
    _require(mat_b.dtype == torch.int8, "mat_b must be Int8")
    _require(out_dtype in (torch.float16, torch.bfloat16), "out_dtype must be Half or BFloat16")
    return _rowwise_mm(lib.sglamd_int8_scaled_mm, mat_a, mat_b, scales_a, scales_b, out_dtype, bias)


# --------------------------------------------------------------------------------------
# MoE
# --------------------------------------------------------------------------------------
@_op("topk_softmax(Tensor! topk_weights, Tensor! topk_indices, Tensor gating_output, bool renormalize, float "
     "moe_softcapping, Tensor? correction_bias) -> ()")
def topk_softmax(topk_weights, topk_indices, gating_output, renormalize, moe_softcapping, correction_bias):
    """moe_topk_softmax_kernels.cu:718-810 (checks :726-775)."""
    _require(gating_output.dtype in (torch.float32, torch.float16, torch.bfloat16),
             "gating_output must be float32, float16, or bfloat16")
    _require(gating_output.dim() == 2, "gating_output must be 2D tensor [num_tokens, num_experts]")
    _require(topk_weights.dim() == 2, "topk_weights must be 2D tensor [num_tokens, topk]")
    _require(topk_indices.dim() == 2, "topk_indices must be 2D tensor [num_tokens, topk]")
    _require(gating_output.size(0) == topk_weights.size(0),
             "First dimension of topk_weights must match num_tokens in gating_output")
    _require(gating_output.size(0) == topk_indices.size(0),
             "First dimension of topk_indices must match num_tokens in gating_output")
    _require(topk_weights.size(-1) == topk_indices.size(-1),
             "Second dimension of topk_indices must match topk in topk_weights")
    _require(topk_weights.size(-1) <= gating_output.size(-1), "topk must be less than or equal to num_experts")
    _require(topk_weights.dtype == torch.float32 and topk_indices.dtype == torch.int32,
             "topk_weights must be Float and topk_indices Int")
    for t, n in ((topk_weights, "topk_weights"), (topk_indices, "topk_indices"), (gating_output, "gating_output")):
        _check_input(t, n)
    bias_ptr = 0
    if correction_bias is not None:
        _require(correction_bias.dim() == 1, "correction_bias must be 1D tensor [num_experts]")
        _require(correction_bias.size(0) == gating_output.size(-1), "correction_bias size must match num_experts")
        _require(correction_bias.dtype == torch.float32,
                 f"correction_bias must be float32, got {correction_bias.dtype}")
        _check_input(correction_bias, "correction_bias")
        bias_ptr = correction_bias.data_ptr()
    num_tokens, num_experts = gating_output.shape
    if num_tokens == 0:
        return
    with torch.cuda.device(gating_output.device):
        check(lib.sglamd_topk_softmax(
            topk_weights.data_ptr(), topk_indices.data_ptr(), gating_output.data_ptr(), _DT[gating_output.dtype],
            num_tokens, num_experts, topk_weights.size(-1), 1 if renormalize else 0, float(moe_softcapping), bias_ptr,
            _stream(gating_output)))


@_op("topk_sigmoid(Tensor! topk_weights, Tensor! topk_indices, Tensor gating_output, bool renormalize, Tensor? "
     "correction_bias) -> ()")
def topk_sigmoid(topk_weights, topk_indices, gating_output, renormalize, correction_bias):
    """moe_topk_sigmoid_kernels.cu:496-600 (checks :503-548)."""
    _require(gating_output.dtype in (torch.float32, torch.float16, torch.bfloat16),
             "gating_output must be float32, float16, or bfloat16")
    _require(gating_output.dim() == 2, "gating_output must be 2D tensor [num_tokens, num_experts]")
    _require(topk_weights.dim() == 2, "topk_weights must be 2D tensor [num_tokens, topk]")
    _require(topk_indices.dim() == 2, "topk_indices must be 2D tensor [num_tokens, topk]")
    _require(gating_output.size(0) == topk_weights.size(0),
             "First dimension of topk_weights must match num_tokens in gating_output")
    _require(gating_output.size(0) == topk_indices.size(0),
             "First dimension of topk_indices must match num_tokens in gating_output")
    _require(topk_weights.size(-1) == topk_indices.size(-1),
             "Second dimension of topk_indices must match topk in topk_weights")
    _require(topk_weights.size(-1) <= gating_output.size(-1), "topk must be less than or equal to num_experts")
    _require(topk_weights.dtype == torch.float32 and topk_indices.dtype == torch.int32,
             "topk_weights must be Float and topk_indices Int")
    for t, n in ((topk_weights, "topk_weights"), (topk_indices, "topk_indices"), (gating_output, "gating_output")):
        _check_input(t, n)
    bias_ptr = 0
    if correction_bias is not None:
        _require(correction_bias.dim() == 1, "correction_bias must be 1D tensor [num_experts]")
        _require(correction_bias.size(0) == gating_output.size(-1), "correction_bias size must match num_experts")
        _require(correction_bias.dtype == torch.float32,
                 f"correction_bias must be float32, got {correction_bias.dtype}")
        _check_input(correction_bias, "correction_bias")
        bias_ptr = correction_bias.data_ptr()
    num_tokens, num_experts = gating_output.shape
    if num_tokens == 0:
        return
    with torch.cuda.device(gating_output.device):
        check(lib.sglamd_topk_sigmoid(
            topk_weights.data_ptr(), topk_indices.data_ptr(), gating_output.data_ptr(), _DT[gating_output.dtype],
            num_tokens, num_experts, topk_weights.size(-1), 1 if renormalize else 0, bias_ptr,
            _stream(gating_output)))


@_op("moe_align_block_size(Tensor topk_ids, int num_experts, int block_size, Tensor! sorted_token_ids, Tensor! "
     "experts_ids, Tensor! num_tokens_post_pad, Tensor! cumsum_buffer, bool "
     "pad_sorted_token_ids) -> ()")
def moe_align_block_size(topk_ids, num_experts, block_size, sorted_token_ids, experts_ids, num_tokens_post_pad,
                         cumsum_buffer, pad_sorted_token_ids):
    """moe_align_kernel.cu:317-383.  Sizes of the outputs are the caller's responsibility there;
    here the ones that would make the kernel write out of bounds are checked."""
    _require(topk_ids.is_cuda and topk_ids.is_contiguous(), "topk_ids must be a contiguous CUDA tensor")
    _require(topk_ids.dtype in (torch.int32, torch.int64), "topk_ids must be an integral tensor (int32/int64)")
    for t, n in ((sorted_token_ids, "sorted_token_ids"), (experts_ids, "experts_ids"),
                 (num_tokens_post_pad, "num_tokens_post_pad"), (cumsum_buffer, "cumsum_buffer")):
        _require(t.is_cuda and t.is_contiguous() and t.dtype == torch.int32, f"{n} must be a contiguous int32 CUDA tensor")
    numel = topk_ids.numel()
    max_padded = sorted_token_ids.size(0)
    worst = numel + min(numel, num_experts) * (block_size - 1)
    _require(max_padded >= min(worst, numel * block_size), "sorted_token_ids is too small for the padded spans")
    _require(experts_ids.numel() * block_size >= max_padded - block_size + 1, "experts_ids is too small")
    _require(cumsum_buffer.numel() >= num_experts + 1, "cumsum_buffer must hold num_experts + 1 entries")
    with torch.cuda.device(topk_ids.device):
        check(lib.sglamd_moe_align_block_size(
            topk_ids.data_ptr(), _DT[topk_ids.dtype], numel, int(num_experts), int(block_size),
            sorted_token_ids.data_ptr(), max_padded, experts_ids.data_ptr(), num_tokens_post_pad.data_ptr(),
            cumsum_buffer.data_ptr(), 1 if pad_sorted_token_ids else 0, _stream(topk_ids)))


def _act_and_mul(name, fn, out, input):
    _check_input(input, "input")
    _check_input(out, "out")
    _require(input.dtype in (torch.float16, torch.bfloat16) and out.dtype == input.dtype,
             f"{name} takes Half or BFloat16 tensors of one dtype")
    d = input.size(-1) // 2
    rows = input.numel() // input.size(-1) if input.numel() else 0
    _require(out.numel() == rows * d, "out has the wrong number of elements")
    with torch.cuda.device(input.device):
        check(fn(input.data_ptr(), out.data_ptr(), _DT[input.dtype], rows, d, _stream(input)))


@_op("silu_and_mul(Tensor! out, Tensor input) -> ()")
def silu_and_mul(out, input):
    """elementwise/activation.cu:82-101."""
    _act_and_mul("silu_and_mul", lib.sglamd_silu_and_mul, out, input)


@_op("gelu_tanh_and_mul(Tensor! out, Tensor input) -> ()")
def gelu_tanh_and_mul(out, input):
    """elementwise/activation.cu:107-127 (schema common_extension.cc:79-80)."""
    _act_and_mul("gelu_tanh_and_mul", lib.sglamd_gelu_tanh_and_mul, out, input)


@_op("gelu_and_mul(Tensor! out, Tensor input) -> ()")
def gelu_and_mul(out, input):
    """elementwise/activation.cu:129-149 (schema common_extension.cc:82-83)."""
    _act_and_mul("gelu_and_mul", lib.sglamd_gelu_and_mul, out, input)


@_op("moe_sum_reduce(Tensor input, Tensor output, float routed_scaling_factor) -> ()")
def moe_sum_reduce(input, output, routed_scaling_factor):
    """common_extension.cc:180-181 (input [tokens, topk, hidden] -> output [tokens, hidden])."""
    _check_input(input, "input")
    _check_input(output, "output")
    _require(input.dim() == 3 and output.dim() == 2, "input must be 3D and output 2D")
    tokens, topk, d = input.shape
    _require(output.shape[0] == tokens and output.shape[1] == d, "output shape does not match input")
    _require(input.dtype in (torch.float16, torch.bfloat16) and output.dtype == input.dtype,
             "moe_sum_reduce takes Half or BFloat16 tensors of one dtype")
    with torch.cuda.device(input.device):
        check(lib.sglamd_moe_sum_reduce(input.data_ptr(), output.data_ptr(), _DT[input.dtype], tokens, topk, d,
                                        float(routed_scaling_factor), _stream(input)))


# --------------------------------------------------------------------------------------
# expert-major ("grouped") MoE interface
# --------------------------------------------------------------------------------------
@_op("prepare_moe_input(Tensor topk_ids, Tensor expert_offsets, Tensor? blockscale_offsets, Tensor problem_sizes1,"
     " Tensor problem_sizes2, Tensor input_permutation, Tensor output_permutation, int num_experts, int n, int k) -> "
     "()")
def prepare_moe_input(topk_ids, expert_offsets, blockscale_offsets, problem_sizes1, problem_sizes2, input_permutation,
                      output_permutation, num_experts, n, k):
    """sgl-kernel/csrc/moe/prepare_moe_input.cu:130-156 (dtype check :141)."""
    _require(topk_ids.dtype == torch.int32, "topk_ids must be int32")
    _check_input(topk_ids, "topk_ids")
    numel = topk_ids.numel()
    topk = topk_ids.size(1) if topk_ids.dim() == 2 else 1
    for t, name, need in ((expert_offsets, "expert_offsets", num_experts + 1),
                          (problem_sizes1, "problem_sizes1", num_experts * 3),
                          (problem_sizes2, "problem_sizes2", num_experts * 3),
                          (input_permutation, "input_permutation", numel),
                          (output_permutation, "output_permutation", numel)):
        _check_input(t, name)
        _require(t.dtype == torch.int32 and t.numel() >= need, f"{name} must be int32 with at least {need} elements")
    if blockscale_offsets is not None:
        _check_input(blockscale_offsets, "blockscale_offsets")
        _require(blockscale_offsets.dtype == torch.int32 and blockscale_offsets.numel() >= num_experts + 1,
                 "blockscale_offsets must be int32 with num_experts + 1 elements")
    with torch.cuda.device(topk_ids.device):
        check(lib.sglamd_prepare_moe_input(
            topk_ids.data_ptr(), numel, topk, int(num_experts), int(n), int(k), expert_offsets.data_ptr(),
            blockscale_offsets.data_ptr() if blockscale_offsets is not None else None, problem_sizes1.data_ptr(),
            problem_sizes2.data_ptr(), input_permutation.data_ptr(), output_permutation.data_ptr(),
            _stream(topk_ids)))


@_op("shuffle_rows(Tensor input, Tensor dst2src_map, Tensor output) -> ()")
def shuffle_rows(input, dst2src_map, output):
    """prepare_moe_input.cu:213-246 (same-dtype check :215-217; float32, half, bfloat16, fp8 and uint8 rows)."""
    _require(input.dtype == output.dtype, "Input and output tensors must have the same data type")
    _require(input.dtype in (torch.float16, torch.bfloat16, torch.float32, torch.float8_e4m3fn, torch.uint8),
             "[moe replicate input] data type dispatch fail!")
    _check_input(input, "input")
    _check_input(output, "output")
    _check_input(dst2src_map, "dst2src_map")
    _require(dst2src_map.dtype == torch.int32 and dst2src_map.numel() >= output.size(0),
             "dst2src_map must be int32 with one entry per output row")
    _require(input.dim() == 2 and output.dim() == 2 and input.size(1) == output.size(1),
             "input and output must be 2D with the same number of columns")
    with torch.cuda.device(input.device):
        check(lib.sglamd_shuffle_rows(input.data_ptr(), dst2src_map.data_ptr(), output.data_ptr(), output.size(0),
                                      input.size(1) * input.element_size(), _stream(input)))


@_op("apply_shuffle_mul_sum(Tensor input, Tensor output, Tensor permutation, Tensor? factors) -> ()")
def apply_shuffle_mul_sum(input, output, permutation, factors):
    """prepare_moe_input.cu:300-376 (checks :306-327)."""
    _require(input.dim() == 2, "input_tensor must be 2D [m * topk, row_stride]")
    _require(output.dim() == 2, "output_tensor must be 2D [m, row_stride]")
    _require(permutation.dim() == 1, "permutation must be 1D [m * topk]")
    m, row_stride = output.shape
    topk = permutation.size(0) // m if m else 1
    _require(permutation.size(0) == m * topk, "permutation size must match m * topk")
    _require(permutation.dtype == torch.int32, "permutation must be int32")
    _require(output.dtype in (torch.float16, torch.bfloat16) and input.dtype == output.dtype,
             "input and output must both be Half or BFloat16")
    _require(input.size(1) == row_stride and input.size(0) >= m * topk, "input shape does not match output")
    _check_input(input, "input")
    _check_input(output, "output")
    _check_input(permutation, "permutation")
    if factors is not None:
        _require(factors.dtype == output.dtype, "Factors must match output dtype")
        _require(factors.numel() == m * topk, "Factors must have shape [m * topk]")
        _check_input(factors, "factors")
    if m == 0:
        return
    with torch.cuda.device(input.device):
        check(lib.sglamd_apply_shuffle_mul_sum(
            input.data_ptr(), output.data_ptr(), permutation.data_ptr(),
            factors.data_ptr() if factors is not None else None, _DT[output.dtype], m, topk, row_stride,
            _stream(input)))


@_op("fp8_blockwise_scaled_grouped_mm(Tensor output, Tensor a_ptrs, Tensor b_ptrs, Tensor out_ptrs, Tensor "
     "a_scales_ptrs, Tensor b_scales_ptrs, Tensor a, Tensor b, Tensor scales_a, Tensor scales_b, Tensor "
     "stride_a, Tensor stride_b, Tensor stride_c, Tensor layout_sfa, Tensor layout_sfb, Tensor problem_sizes, Tensor "
     "expert_offsets, Tensor workspace) -> ()")
def fp8_blockwise_scaled_grouped_mm(output, a_ptrs, b_ptrs, out_ptrs, a_scales_ptrs, b_scales_ptrs, a, b, scales_a,
                                    scales_b, stride_a, stride_b, stride_c, layout_sfa, layout_sfb, problem_sizes,
                                    expert_offsets, workspace):
    """sgl-kernel/csrc/moe/fp8_blockwise_moe_kernel.cu:650-810 (checks :669-707).  The pointer, stride and layout
    containers are scratch of the reference's CUTLASS launch; they are checked like the reference checks them and
    otherwise unused.  `b` is the [E, K, N] column-major view of contiguous [E, N, K] weights, `scales_b` the
    [E, K/128, N/128] view of contiguous [E, N/128, K/128] scales.  The sorted-block schedule is built in
    `workspace` when it is large enough, else in a buffer from torch's caching allocator."""
    _require(problem_sizes.dim() == 2, "problem_sizes must be 2D tensor")
    _require(problem_sizes.size(1) == 3, "problem_sizes must have shape (num_experts, 3)")
    _require(problem_sizes.size(0) == expert_offsets.size(0),
             "Number of experts in problem_sizes must match expert_offsets")
    _require(problem_sizes.dtype == torch.int32, "problem_sizes must be int32")
    _require(a.dtype == torch.float8_e4m3fn, "a must be kFloat8_e4m3fn")
    _require(b.dtype == torch.float8_e4m3fn, "b must be kFloat8_e4m3fn")
    _require(output.dtype in (torch.bfloat16, torch.float16), "output must be bfloat16 or half")
    _require(scales_a.dtype == torch.float32, "scales_a must be float32")
    _require(scales_b.dtype == torch.float32, "scales_b must be float32")
    _require(stride_a.dtype == torch.int64, "stride_a must be int64")
    _require(stride_b.dtype == torch.int64, "stride_b must be int64")
    _require(stride_c.dtype == torch.int64, "stride_c must be int64")
    _require(layout_sfa.dtype == torch.int32, "layout_sfa must be int32")
    _require(layout_sfb.dtype == torch.int32, "layout_sfb must be int32")
    _require(expert_offsets.dtype == torch.int32, "expert_offsets must be int32")
    _require(output.dim() == 2, "output must be 2D tensor")
    _require(a.dim() == 2, "a must be 2D tensor")
    _require(b.dim() == 3, "b must be 3D tensor")
    _require(scales_a.dim() == 2, "scales_a must be 2D tensor")
    _require(scales_b.dim() == 3, "scales_b must be 3D tensor")
    _require(stride_a.dim() == 1 and stride_b.dim() == 1 and stride_c.dim() == 1, "strides must be 1D tensors")
    _require(expert_offsets.dim() == 1, "expert_offsets must be 1D tensor")
    _require(workspace.dim() == 1, "workspace must be 1D tensor")
    E, K, N = b.shape
    rows = a.size(0)
    _require(a.size(1) == K and a.is_contiguous(), "a must be contiguous [rows, K]")
    _require(b.stride(1) == 1 and b.stride(2) == K and (E == 1 or b.stride(0) == N * K),
             "b must be the [E, K, N] view of contiguous [E, N, K] weights")
    _require(tuple(scales_a.shape) == (rows, K // 128) and scales_a.is_contiguous(),
             "scales_a must be contiguous [rows, K / 128]")
    _require(tuple(scales_b.shape) == (E, K // 128, N // 128) and scales_b.stride(1) == 1
             and scales_b.stride(2) == K // 128, "scales_b must be the [E, K/128, N/128] view of [E, N/128, K/128]")
    _require(tuple(output.shape) == (rows, N) and output.is_contiguous(), "output must be contiguous [rows, N]")
    _require(problem_sizes.size(0) == E, "problem_sizes must have one row per expert")
    _check_input(problem_sizes, "problem_sizes")
    _require(expert_offsets.stride(0) == 1, "expert_offsets must be contiguous")
    if rows == 0:
        return
    with torch.cuda.device(a.device):
        need = int(lib.sglamd_grouped_mm_workspace_bytes(rows, E))
        ws = workspace
        if (not ws.is_cuda or ws.numel() * ws.element_size() < need or ws.data_ptr() % 16 or not ws.is_contiguous()):
            ws = torch.empty(need, dtype=torch.uint8, device=a.device)
        check(lib.sglamd_fp8_blockwise_scaled_grouped_mm(
            output.data_ptr(), _DT[output.dtype], a.data_ptr(), b.data_ptr(), scales_a.data_ptr(),
            scales_b.data_ptr(), problem_sizes.data_ptr(), expert_offsets.data_ptr(), E, rows, N, K, ws.data_ptr(),
            ws.numel() * ws.element_size(), _stream(a)))


@_op("es_fp8_blockwise_scaled_grouped_mm(Tensor output, Tensor a, Tensor b, Tensor scales_a, Tensor scales_b, Tensor "
     "stride_a, Tensor stride_b, Tensor stride_d, Tensor problem_sizes, Tensor expert_offsets, Tensor workspace) -> "
     "()")
def es_fp8_blockwise_scaled_grouped_mm(output, a, b, scales_a, scales_b, stride_a, stride_b, stride_d, problem_sizes,
                                       expert_offsets, workspace):
    """The "expert specialisation" launch of the same grouped GEMM (schema sgl-kernel/csrc/common_extension.cc:483-487;
    called in place of fp8_blockwise_scaled_grouped_mm at python/sglang/srt/layers/moe/cutlass_moe.py:224-237,290-303
    with the same operands and without the pointer / layout scratch).  Same arithmetic, one implementation here."""
    E = b.shape[0]
    scratch_i64 = torch.empty(0, dtype=torch.int64, device=a.device)
    scratch_i32 = torch.empty((E, 5), dtype=torch.int32, device=a.device)
    fp8_blockwise_scaled_grouped_mm(output, scratch_i64, scratch_i64, scratch_i64, scratch_i64, scratch_i64, a, b,
                                    scales_a, scales_b, stride_a, stride_b, stride_d, scratch_i32, scratch_i32,
                                    problem_sizes, expert_offsets, workspace)


def fused_moe_block_fp8_gemm_(A, A_scale, B, B_scale, C, topk_weights, sorted_token_ids, expert_ids,
                              num_tokens_post_padded, mul_routed_weight: bool, top_k: int, block_m: int) -> None:
    """Launcher of the sorted-block grouped GEMM (the fp8_w8a8 or int8_w8a8 / block [128,128] configuration
    of invoke_fused_moe_kernel, fused_moe_triton_kernels.py:702-930).  A e4m3fn or int8 [rows, K] quantised
    activations with scales A_scale [rows, ceil(K/128)]; B of the same type [E, N, K]; B_scale [E, ceil(N/128),
    ceil(K/128)]; C [num_valid, N] where num_valid = topk_ids.numel()."""
    E, N, K = B.shape
    num_valid = C.numel() // N
    int8 = A.dtype == torch.int8
    _require(A.dtype in (torch.float8_e4m3fn, torch.int8) and B.dtype == A.dtype,
             "A and B must both be Float8_e4m3fn or both Int8")
    _require(A.stride(-1) == 1 and B.stride(-1) == 1 and C.is_contiguous(), "A, B rows and C must be contiguous")
    _require(A_scale.dtype == torch.float32 and B_scale.dtype == torch.float32, "scales must be Float32")
    _require(A_scale.shape[-1] == (K + 127) // 128 and B_scale.shape[-1] == (K + 127) // 128
             and B_scale.shape[-2] == (N + 127) // 128, "scale shapes do not match the 128x128 blocks")
    max_blocks = (sorted_token_ids.numel() + block_m - 1) // block_m
    _require(expert_ids.numel() >= max_blocks, "expert_ids is too small")
    with torch.cuda.device(A.device):
        fn = lib.sglamd_fused_moe_block_int8_gemm if int8 else lib.sglamd_fused_moe_block_fp8_gemm
        check(fn(
            A.data_ptr(), A.stride(0), A_scale.data_ptr(), A_scale.stride(0), A_scale.stride(1),
            B.data_ptr(), B.stride(0), B.stride(1), B_scale.data_ptr(), B_scale.stride(0), B_scale.stride(1),
            B_scale.stride(2), C.data_ptr(), N, _DT[C.dtype], sorted_token_ids.data_ptr(), expert_ids.data_ptr(),
            num_tokens_post_padded.data_ptr(), topk_weights.data_ptr() if topk_weights is not None else None,
            num_valid, int(top_k), 1 if mul_routed_weight else 0, int(block_m), max_blocks, N, K, _stream(A)))


def fused_moe_gemm_any_(A, A_scale, B, B_scale, C, topk_weights, sorted_token_ids, expert_ids, num_tokens_post_padded,
                        mul_routed_weight: bool, top_k: int, block_m: int, block_shape=None, bias=None) -> None:
    """The sorted-block grouped GEMM in the configurations of invoke_fused_moe_kernel
    (fused_moe_triton_kernels.py:702-930) beyond block [128, 128]: `block_shape` [block_n, block_k] with 64 or 128
    each (A_scale [rows, ceil(K/block_k)], B_scale [E, ceil(N/block_n), ceil(K/block_k)]), or None for row scaling:
    A_scale one value per activation row (or a single value: per tensor), B_scale [E, N] per channel (or [E]: per
    expert).  bias: optional [E, N] in C's dtype."""
    E, N, K = B.shape
    num_valid = C.numel() // N
    _require(A.dtype in (torch.float8_e4m3fn, torch.int8) and B.dtype == A.dtype,
             "A and B must both be Float8_e4m3fn or both Int8")
    _require(A.stride(-1) == 1 and B.stride(-1) == 1 and C.is_contiguous(), "A, B rows and C must be contiguous")
    _require(A_scale.dtype == torch.float32 and B_scale.dtype == torch.float32, "scales must be Float32")
    if block_shape is not None:
        bn, bk = int(block_shape[0]), int(block_shape[1])
        _require(A_scale.shape[-1] == -(-K // bk) and B_scale.shape[-1] == -(-K // bk)
                 and B_scale.shape[-2] == -(-N // bn), "scale shapes do not match the scale blocks")
        a_strides = (A_scale.stride(0), A_scale.stride(1))
        b_strides = (B_scale.stride(0), B_scale.stride(1), B_scale.stride(2))
    else:
        bn = bk = 0
        rows = A.shape[0]
        _require(A_scale.numel() in (1, rows), "the activation scale must be per tensor or per row")
        _require(B_scale.numel() in (E, E * N), "the weight scale must be per expert or per channel")
        a_strides = (0 if A_scale.numel() == 1 else 1, 0)
        b_strides = (1, 0, 0) if B_scale.numel() == E else (N, 1, 0)
        A_scale, B_scale = A_scale.contiguous(), B_scale.contiguous()
    if bias is not None:
        _require(bias.dtype == C.dtype and bias.shape == (E, N) and bias.is_contiguous(),
                 "bias must be a contiguous [E, N] tensor of the output dtype")
    max_blocks = (sorted_token_ids.numel() + block_m - 1) // block_m
    _require(expert_ids.numel() >= max_blocks, "expert_ids is too small")
    with torch.cuda.device(A.device):
        check(lib.sglamd_fused_moe_gemm_any(
            A.data_ptr(), A.stride(0), A_scale.data_ptr(), a_strides[0], a_strides[1],
            B.data_ptr(), B.stride(0), B.stride(1), B_scale.data_ptr(), b_strides[0], b_strides[1], b_strides[2],
            bias.data_ptr() if bias is not None else None, N, C.data_ptr(), N, _DT[C.dtype], _DT[A.dtype], bn, bk,
            sorted_token_ids.data_ptr(), expert_ids.data_ptr(), num_tokens_post_padded.data_ptr(),
            topk_weights.data_ptr() if topk_weights is not None else None,
            num_valid, int(top_k), 1 if mul_routed_weight else 0, int(block_m), max_blocks, N, K, _stream(A)))


def fused_moe_block_fp8_workspace_bytes(M: int, H: int, I: int, E: int, topk: int, block_m: int = 0) -> int:
    return int(lib.sglamd_fused_moe_block_fp8_workspace(M, H, I, E, topk, block_m))


def fused_moe_block_fp8_(hidden_states, w1, w2, w1_scale, w2_scale, topk_weights, topk_ids, out,
                         routed_scaling_factor: float, block_m: int = 0, workspace: Optional[torch.Tensor] = None):
    """One-call launcher of the whole block-FP8 MoE layer (the kernel sequence of
    fused_moe.py:401-785 issued from C on the current stream).  `workspace` is a uint8 device tensor
    of at least fused_moe_block_fp8_workspace_bytes(...) bytes; one is taken from torch's caching
    allocator when omitted."""
    M, H = hidden_states.shape
    E, N2, _ = w1.shape
    I = N2 // 2
    topk = topk_ids.shape[1]
    _require(w1.dtype == torch.float8_e4m3fn and w2.dtype == torch.float8_e4m3fn, "expert weights must be Float8_e4m3fn")
    _require(w1.is_contiguous() and w2.is_contiguous() and w1_scale.is_contiguous() and w2_scale.is_contiguous(),
             "expert weights and scales must be contiguous")
    _require(tuple(w2.shape) == (E, H, I), "w2 must be [E, hidden, intermediate]")
    _require(tuple(w1_scale.shape) == (E, N2 // 128, H // 128) and tuple(w2_scale.shape) == (E, H // 128, I // 128),
             "scale shapes do not match the 128x128 blocks")
    _require(w1_scale.dtype == torch.float32 and w2_scale.dtype == torch.float32, "scales must be Float32")
    _require(topk_weights.dtype == torch.float32 and topk_weights.is_contiguous(), "topk_weights must be contiguous Float32")
    _require(topk_ids.dtype in (torch.int32, torch.int64) and topk_ids.is_contiguous(), "topk_ids must be contiguous int32/int64")
    _require(hidden_states.is_contiguous() and out.is_contiguous(), "hidden_states and out must be contiguous")
    need = fused_moe_block_fp8_workspace_bytes(M, H, I, E, topk, block_m)
    if workspace is None:
        workspace = torch.empty(need, dtype=torch.uint8, device=hidden_states.device)
    _require(workspace.numel() * workspace.element_size() >= need, "workspace is too small")
    with torch.cuda.device(hidden_states.device):
        check(lib.sglamd_fused_moe_block_fp8(
            hidden_states.data_ptr(), _DT[hidden_states.dtype], M, H, I, E, topk, w1.data_ptr(), w1_scale.data_ptr(),
            w2.data_ptr(), w2_scale.data_ptr(), topk_weights.data_ptr(), topk_ids.data_ptr(), _DT[topk_ids.dtype],
            out.data_ptr(), float(routed_scaling_factor), int(block_m), workspace.data_ptr(),
            workspace.numel() * workspace.element_size(), _stream(hidden_states)))

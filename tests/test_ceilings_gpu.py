"""The benchmark's bare-loop entry points: they have to run and, where they produce data, produce the right data."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def test_hbm_copy_and_read_and_mfma_loops(dev):
    from sglang_amd._lib import check, lib

    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    n = (1 << 22) + 4096 + 16  # not a multiple of the grid stride
    src = torch.empty(n, device=dev, dtype=torch.uint8).random_(0, 256)
    dst = torch.zeros(n, device=dev, dtype=torch.uint8)
    sink = torch.zeros(1, device=dev, dtype=torch.int32)
    p = lambda t: ctypes.c_void_p(t.data_ptr())  # noqa: E731
    check(lib.sglamd_ceiling_hbm(p(dst), p(src), ctypes.c_int64(n), p(sink), stream))
    assert torch.equal(dst, src)
    check(lib.sglamd_ceiling_hbm(None, p(src), ctypes.c_int64(n), p(sink), stream))
    assert lib.sglamd_ceiling_hbm(None, p(src), ctypes.c_int64(n - 8), p(sink), stream) != 0  # not a multiple of 16

    check(lib.sglamd_ceiling_hbm_lds(p(src), ctypes.c_int64(n), stream))   # runs to completion, reads only
    torch.cuda.synchronize()
    assert lib.sglamd_ceiling_hbm_lds(p(src), ctypes.c_int64(512), stream) != 0  # less than one piece

    # the L2-resident read, both load paths: runs to completion; too small a buffer or no passes are refused
    big = torch.empty(torch.cuda.get_device_properties(dev).multi_processor_count * 65536, device=dev, dtype=torch.uint8).random_(0, 256)
    for lds in (1, 0):
        check(lib.sglamd_ceiling_l2_read(p(big), ctypes.c_int64(big.numel()), 3, lds, p(sink), stream))
    torch.cuda.synchronize()
    assert lib.sglamd_ceiling_l2_read(p(big), ctypes.c_int64(big.numel() - 1), 3, 1, p(sink), stream) != 0
    assert lib.sglamd_ceiling_l2_read(p(big), ctypes.c_int64(big.numel()), 0, 1, p(sink), stream) != 0

    out = torch.full((256 * 512,), float("nan"), device=dev)
    for int8 in (0, 1):
        for rnd in (0, 1):
            check(lib.sglamd_ceiling_mfma(int8, rnd, 3, p(out), stream))
            torch.cuda.synchronize()
            assert bool(torch.isfinite(out).all())
    # constant operands: every product is 1.0 * 1.0 (e4m3 0x38), 64 per MFMA and element, 16 elements x 8 tiles
    check(lib.sglamd_ceiling_mfma(0, 0, 3, p(out), stream))
    assert float(out[0]) == 3 * 64 * 16 * 8


def test_l2_resident_gemm_ceiling_computes_tile_zero_everywhere(dev):
    """The ceiling form of the persistent kernel: every 256x256 tile of the output must hold the product of the
    two 256-row panels (checked against the oracle), which shows that the loop it times is the real one."""
    import numpy as np

    from oracle import gemm as og
    from sglang_amd._lib import check, lib
    from tests.util import assert_gemm_close

    M, N, K = 1280, 256 * 60, 1024   # 300 tiles on 256 CUs
    g = torch.Generator().manual_seed(3)
    a = ((torch.rand(256, K, generator=g) - 0.5) * 16).to(torch.float8_e4m3fn)
    b = ((torch.rand(256, K, generator=g) - 0.5) * 16).to(torch.float8_e4m3fn)
    sa = torch.rand(K // 128, 256, generator=g) + 0.5
    sb = torch.rand(2, K // 128, generator=g) + 0.5
    out = torch.zeros(M, N, device=dev, dtype=torch.bfloat16)
    p = lambda t: ctypes.c_void_p(t.data_ptr())  # noqa: E731
    da, db, dsa, dsb = a.to(dev), b.to(dev), sa.to(dev), sb.to(dev)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    check(lib.sglamd_ceiling_gemm_l2_resident(p(da), p(db), p(dsa), p(dsb), p(out), ctypes.c_int64(M), ctypes.c_int64(N),
                                              ctypes.c_int64(K), stream))
    torch.cuda.synchronize()
    ref = og.block_fp8_matmul(a.view(torch.uint8).numpy(), b.view(torch.uint8).numpy(), sa.t().contiguous().numpy(),
                              sb.numpy(), return_fp32=True)
    tiles = out.cpu().view(M // 256, 256, N // 256, 256).permute(0, 2, 1, 3)
    assert_gemm_close(tiles[0, 0], ref, "tile (0, 0)")
    assert bool((tiles == tiles[0, 0]).all()), "a tile differs from tile (0, 0)"
    assert lib.sglamd_ceiling_gemm_l2_resident(p(da), p(db), p(dsa), p(dsb), p(out), ctypes.c_int64(256),
                                               ctypes.c_int64(256), ctypes.c_int64(K), stream) != 0  # one tile only

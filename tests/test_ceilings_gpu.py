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

    out = torch.full((256 * 512,), float("nan"), device=dev)
    for int8 in (0, 1):
        for rnd in (0, 1):
            check(lib.sglamd_ceiling_mfma(int8, rnd, 3, p(out), stream))
            torch.cuda.synchronize()
            assert bool(torch.isfinite(out).all())
    # constant operands: every product is 1.0 * 1.0 (e4m3 0x38), 64 per MFMA and element, 16 elements x 8 tiles
    check(lib.sglamd_ceiling_mfma(0, 0, 3, p(out), stream))
    assert float(out[0]) == 3 * 64 * 16 * 8

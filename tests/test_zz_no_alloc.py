"""The fused MoE layer through the entry point that allocates nothing (sglamd_fused_moe_block_fp8_static: the
intermediates live in a device array that is part of the library) against the workspace entry point it is a
variant of (sglamd_fused_moe_block_fp8), both called through the C ABI with ctypes.  Outputs must be bit-equal:
the two run the same kernels on the same data, only the scratch address differs.  Two calls in a row, the second
on a smaller input, so that whatever the first call left in the shared array is there when the second one runs;
then a size beyond the array is refused before anything is launched."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

BF16, I32 = 2, 5  # SGLAMD_BF16, SGLAMD_I32 of include/sglamd.h


def _case(M, H, I, E, topk, dev, seed):
    g = torch.Generator(device=dev).manual_seed(seed)
    codes = lambda *shape: torch.randint(0, 0x7F, shape, generator=g, device=dev, dtype=torch.int32).to(torch.uint8)  # noqa: E731
    x = torch.randn(M, H, generator=g, device=dev).to(torch.bfloat16)
    w13, w2 = codes(E, 2 * I, H), codes(E, H, I)
    w13s = torch.rand(E, 2 * I // 128, H // 128, generator=g, device=dev) * 2e-4 + 1e-5
    w2s = torch.rand(E, H // 128, I // 128, generator=g, device=dev) * 2e-4 + 1e-5
    tw, ti = torch.topk(torch.softmax(torch.randn(M, E, generator=g, device=dev), dim=-1), topk, dim=-1)
    tw = (tw / tw.sum(-1, keepdim=True)).contiguous()
    return x, w13, w2, w13s, w2s, tw, ti.to(torch.int32).contiguous()


def _run(lib, static, M, H, I, E, topk, dev, seed):
    x, w13, w2, w13s, w2s, tw, ti = _case(M, H, I, E, topk, dev, seed)
    out = torch.full((M, H), float("nan"), device=dev, dtype=torch.bfloat16)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    head = (x.data_ptr(), BF16, M, H, I, E, topk, w13.data_ptr(), w13s.data_ptr(), w2.data_ptr(), w2s.data_ptr(),
            tw.data_ptr(), ti.data_ptr(), I32, out.data_ptr(), 1.0, 0)
    if static:
        rc = lib.sglamd_fused_moe_block_fp8_static(*head, stream)
    else:
        need = lib.sglamd_fused_moe_block_fp8_workspace(M, H, I, E, topk, 0)
        ws = torch.empty(need, device=dev, dtype=torch.uint8)
        rc = lib.sglamd_fused_moe_block_fp8(*head, ws.data_ptr(), need, stream)
    assert rc == 0, lib.sglamd_last_error().decode()
    torch.cuda.synchronize()
    return out


def test_static_scratch_entry_point_equals_the_workspace_entry_point(dev):
    from sglang_amd._lib import lib

    limit = lib.sglamd_fused_moe_block_fp8_static_max_bytes()
    assert limit == 16 << 20
    # first a batch that uses most of the array, then a smaller one with other dimensions
    for M, H, I, E, topk, seed in ((48, 7168, 2048, 16, 8, 1), (5, 1024, 512, 8, 2, 2), (2, 1024, 512, 8, 2, 3),
                                   (1, 1024, 512, 16, 4, 4)):  # the last two: the few-token launch sequences
        assert lib.sglamd_fused_moe_block_fp8_workspace(M, H, I, E, topk, 0) <= limit
        print(f"static-scratch MoE M={M} H={H} I={I} E={E} topk={topk}", flush=True)
        got = _run(lib, True, M, H, I, E, topk, dev, seed)
        want = _run(lib, False, M, H, I, E, topk, dev, seed)
        assert not torch.isnan(got.float()).any()
        assert torch.equal(got, want), f"M={M}: static-scratch output differs from the workspace entry point's"
    # beyond the array: refused with a message, nothing launched, the output untouched
    M, H, I, E, topk = 512, 7168, 2048, 16, 8
    assert lib.sglamd_fused_moe_block_fp8_workspace(M, H, I, E, topk, 0) > limit
    x, w13, w2, w13s, w2s, tw, ti = _case(8, H, I, E, topk, dev, 3)
    out = torch.zeros(8, H, device=dev, dtype=torch.bfloat16)
    rc = lib.sglamd_fused_moe_block_fp8_static(x.data_ptr(), BF16, M, H, I, E, topk, w13.data_ptr(), w13s.data_ptr(),
                                               w2.data_ptr(), w2s.data_ptr(), tw.data_ptr(), ti.data_ptr(), I32,
                                               out.data_ptr(), 1.0, 0,
                                               ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == -1 and b"bytes of scratch" in lib.sglamd_last_error()
    torch.cuda.synchronize()
    assert not out.any()


def test_static_entry_point_replayed_from_a_hip_graph(dev):
    """The entry point's use under HIP graph capture: one eager call per device first (it looks the array's address
    up then), after which the call is captured and replayed; every replay, with eager work and synchronisations
    of the program in between, must give the eager result bit for bit."""
    from sglang_amd._lib import lib

    M, H, I, E, topk = 3, 1024, 512, 8, 2
    x, w13, w2, w13s, w2s, tw, ti = _case(M, H, I, E, topk, dev, 11)
    eager = torch.full((M, H), float("nan"), device=dev, dtype=torch.bfloat16)
    out = torch.full((M, H), float("nan"), device=dev, dtype=torch.bfloat16)

    def call(dst, stream):
        rc = lib.sglamd_fused_moe_block_fp8_static(x.data_ptr(), BF16, M, H, I, E, topk, w13.data_ptr(),
                                                   w13s.data_ptr(), w2.data_ptr(), w2s.data_ptr(), tw.data_ptr(),
                                                   ti.data_ptr(), I32, dst.data_ptr(), 1.0, 0,
                                                   ctypes.c_void_p(stream.cuda_stream))
        assert rc == 0, lib.sglamd_last_error().decode()

    call(eager, torch.cuda.current_stream())  # warm-up: resolves the array's address outside any capture
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            call(out, side)
    torch.cuda.synchronize()
    for i in range(4):
        out.fill_(float("nan"))
        x2 = torch.randn(64, 64, device=dev) @ torch.randn(64, 64, device=dev)  # the program's own eager work
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay {i} differs from the eager call"
        del x2

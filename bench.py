#!/usr/bin/env python3
"""Headline benchmark of the quantized-linear hot path on one MI355X.

A "step" is one block-FP8 GEMM (fp8_blockwise_scaled_mm) at the DeepSeek-V3 dense gate_up shape
N=36864, K=7168 with M=4096 tokens: e4m3fn activations quantised per 1x128 group, e4m3fn weights with
128x128 block scales, bf16 output; operands are resident in HBM before the timed region.  The kernel
is launched through the C ABI on torch's current stream and timed with HIP events on that stream.

The LAST stdout line is one small JSON object (under 4 KB).  `value` is TFLOP/s of the timed GEMM; `roofline`
prices the same kernel against the dense FP8 MFMA peak; `cpu_baseline` is the CPU oracle (torch-native
restatement) timed on the host; `targets` holds a dozen named figures of the other workloads of the path
(decode GEMM GB/s, mid-M GEMMs, fused MoE GB/s, activation quant GB/s) measured in the same run.  The full
per-workload table goes to the file named by `--detail` and, one workload per line, to
stderr; it is never part of the last line.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP8_TFLOPS = 5000.0  # MI355X dense FP8 MFMA
PEAK_HBM_GBS = 8000.0     # MI355X HBM3E

# Bytes per launch of the headline kernel that cross the L2 boundary, from rocprofv3 --pmc FETCH_SIZE /
# WRITE_SIZE scaled by what the same counters read for a plain copy (see profiles/).
MEASURED_TRAFFIC_BYTES = 1.925e9  # profiles/gemm8_big_persist_kernel_dsv3_gate_up_M4096.md: FETCH x2.0 + WRITE x1.0


# The chip raises its clocks over the first tens of milliseconds of sustained load: the headline launch takes
# 1.39 ms as the first ten launches after an idle gap (0.2 s is enough), 0.97 ms as launches 11-20 and 0.88 ms from
# about the 60th on.  Every measurement therefore keeps its own operation running for SETTLE_MS of device time
# before its warm-up steps, so that what is timed is the sustained rate a serving process sees, not the ramp.
SETTLE_MS = 100.0


def _settle(run, ms=None):
    """Runs `run()` (one or more launches) back to back until `ms` of device time have passed."""
    import torch

    ms = SETTLE_MS if ms is None else ms
    if ms <= 0:
        return
    done, a, b = 0.0, torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    per = 4
    while done < ms:
        a.record()
        for _ in range(per):
            run()
        b.record()
        b.synchronize()
        took = a.elapsed_time(b)
        done += took
        per = max(1, min(256, int(per * 10.0 / max(took, 0.05))))  # about 10 ms between host syncs


def _time_events(fn, steps, warmup):
    import torch

    _settle(fn)
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for _ in range(steps):
        fn()
    end.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) / steps
    return start.elapsed_time(end) / steps * 1e-3, wall  # seconds per step (device, host wall)


def _time_graph(fn, steps, warmup, replays=5):
    """Captures `steps` calls of fn into one HIP graph and replays it: removes the host launch path from the
    measurement (decode-sized kernels are shorter than a Python call).  Returns seconds per step."""
    import torch

    for _ in range(max(1, warmup)):
        fn()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        fn()
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            for _ in range(steps):
                fn()
    torch.cuda.synchronize()
    graph.replay()
    _settle(graph.replay)
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(replays):
        graph.replay()
    end.record()
    torch.cuda.synchronize()
    sec = start.elapsed_time(end) * 1e-3 / (replays * steps)
    return sec, None  # no host-side time: a replay's launches never pass through the host


def _us(sec):
    return None if sec is None else sec * 1e6


def _rand_fp8(shape, dev, scale=1.0, seed=0):
    import torch

    g = torch.Generator(device=dev).manual_seed(seed)
    out = torch.empty(shape, device=dev, dtype=torch.float8_e4m3fn)
    rows = shape[0]
    step = max(1, (1 << 28) // max(1, shape[-1] * (shape[1] if len(shape) == 3 else 1)))
    for r in range(0, rows, step):
        blk = torch.randn((min(step, rows - r),) + tuple(shape[1:]), device=dev, generator=g) * scale
        out[r:r + step] = blk.clamp_(-448, 448).to(torch.float8_e4m3fn)
    return out


def bench_dense(dev, M, N, K, steps, warmup, copies=1, graph=False, pow2=False):
    """Block-FP8 GEMM, operands prepared like BASELINE config 3: A ~N(0,1) group-quantised, W ~N(0,0.02)
    block-quantised (here drawn directly on the fp8 grid with matching scale magnitudes).  pow2: the same with
    UE8M0 scales (activations quantised with scale_ue8m0, weight scales rounded up to powers of two), expanded to
    fp32 once and handed to the entry point for power-of-two scales."""
    import torch

    import sglang_amd
    from sglang_amd.quantization.fp8_kernel import sglang_per_token_group_quant_fp8

    x = torch.randn(M, K, device=dev, dtype=torch.bfloat16)
    ws_list, w_list = [], []
    for c in range(copies):
        w_list.append(_rand_fp8((N, K), dev, 100.0, seed=c + 1))
        ws = torch.rand(N // 128, K // 128, device=dev) * 0.02 / 448 * 4
        ws_list.append(torch.exp2(torch.ceil(torch.log2(ws.clamp_min(1e-10)))).contiguous() if pow2 else ws.contiguous())
    state = {"i": 0}
    if pow2:
        from sglang_amd.ops import ue8m0_unpack_, w8a8_block_fp8_matmul_

        xq, xs_packed = sglang_per_token_group_quant_fp8(x, 128, column_major_scales=True, scale_tma_aligned=True,
                                                         scale_ue8m0=True)
        xs = ue8m0_unpack_(xs_packed, M, K // 128)
        outs = [torch.empty(M, N, device=dev, dtype=torch.bfloat16) for _ in range(2)]

        def step():
            i = state["i"] % copies
            state["i"] += 1
            w8a8_block_fp8_matmul_(xq, w_list[i], xs, ws_list[i], outs[state["i"] & 1], pow2_scales=True)
    else:
        xq, xs = sglang_per_token_group_quant_fp8(x, 128, column_major_scales=True)

        def step():
            i = state["i"] % copies
            state["i"] += 1
            return sglang_amd.fp8_blockwise_scaled_mm(xq, w_list[i].t(), xs, ws_list[i].t(), torch.bfloat16)

    sec, wall = (_time_graph if graph else _time_events)(step, steps, warmup)
    flops = 2.0 * M * N * K
    byts = M * K + N * K + 2 * M * N + 4 * M * (K // 128) + 4 * (N // 128) * (K // 128)
    rec = {"M": M, "N": N, "K": K, "us": sec * 1e6, "wall_us": _us(wall), "tflops": flops / sec / 1e12,
           "gbs": byts / sec / 1e9, "flops": flops, "bytes": byts}
    if graph:
        # what a caller without a graph gets: the same launches issued one by one from Python
        e_sec, e_wall = _time_events(step, steps, 2)
        rec["eager_us"], rec["eager_wall_us"] = e_sec * 1e6, e_wall * 1e6
    return rec


def bench_rowwise(dev, M, N, K, steps, warmup, int8=False, copies=1, graph=False, bias=False):
    """Per-token / per-channel scaled GEMM (fp8_scaled_mm or int8_scaled_mm), operands like BASELINE config 5;
    `copies` weight sets are rotated so that a decode-sized launch streams its weights from HBM."""
    import torch

    import sglang_amd

    ws = []
    for c in range(copies):
        if int8:
            ws.append(torch.randint(-127, 128, (N, K), device=dev, dtype=torch.int8))
        else:
            ws.append(_rand_fp8((N, K), dev, 100.0, seed=22 + c))
    a = torch.randint(-127, 128, (M, K), device=dev, dtype=torch.int8) if int8 else _rand_fp8((M, K), dev, 100.0, seed=21)
    sa = torch.rand(M, 1, device=dev) * 1e-2
    sb = torch.rand(N, 1, device=dev) * 1e-4
    b = torch.randn(N, device=dev).to(torch.bfloat16) if bias else None
    fn = sglang_amd.int8_scaled_mm if int8 else sglang_amd.fp8_scaled_mm
    state = {"i": 0}

    def step():
        i = state["i"] % copies
        state["i"] += 1
        return fn(a, ws[i].t(), sa, sb, torch.bfloat16, b)

    sec, wall = (_time_graph if graph else _time_events)(step, steps, warmup)
    flops = 2.0 * M * N * K
    byts = M * K + N * K + 2 * M * N + 4 * M + 4 * N + (2 * N if bias else 0)
    return {"M": M, "N": N, "K": K, "us": sec * 1e6, "wall_us": _us(wall), "tflops": flops / sec / 1e12,
            "gbs": byts / sec / 1e9, "flops": flops, "bytes": byts}


def bench_block_int8(dev, M, N, K, steps, warmup, copies=1, graph=False):
    """Block-scaled INT8 GEMM (w8a8_block_int8_matmul): full-range int8 operands, [128,128] scale blocks."""
    import torch

    from sglang_amd.quantization.int8_kernel import w8a8_block_int8_matmul

    a = torch.randint(-127, 128, (M, K), device=dev, dtype=torch.int8)
    ws = [torch.randint(-127, 128, (N, K), device=dev, dtype=torch.int8) for _ in range(copies)]
    sa = torch.rand(M, K // 128, device=dev) * 1e-2
    sb = torch.rand(N // 128, K // 128, device=dev) * 1e-4
    state = {"i": 0}

    def step():
        i = state["i"] % copies
        state["i"] += 1
        return w8a8_block_int8_matmul(a, ws[i], sa, sb, [128, 128], torch.bfloat16)

    sec, wall = (_time_graph if graph else _time_events)(step, steps, warmup)
    flops = 2.0 * M * N * K
    byts = M * K + N * K + 2 * M * N + 4 * M * (K // 128) + 4 * (N // 128) * (K // 128)
    return {"M": M, "N": N, "K": K, "us": sec * 1e6, "wall_us": _us(wall), "tflops": flops / sec / 1e12,
            "gbs": byts / sec / 1e9, "flops": flops, "bytes": byts}


def bench_quant(dev, M, K, steps, warmup, layout="row"):
    """Group quant bf16 -> e4m3fn, scales in one of the reference's layouts: "row" (fp32 row-major), "col"
    (fp32 column-major, rows padded to 4) or "ue8m0" (packed power-of-two exponents, column-major)."""
    import torch

    from sglang_amd.quantization.fp8_kernel import create_per_token_group_quant_fp8_output_scale as mk
    import sglang_amd

    copies = max(1, min(8, (1 << 30) // (M * K * 3)))
    xs = [torch.randn(M, K, device=dev, dtype=torch.bfloat16) for _ in range(copies)]
    q = [torch.empty(M, K, device=dev, dtype=torch.float8_e4m3fn) for _ in range(copies)]
    col, ue = layout != "row", layout == "ue8m0"
    s = [mk((M, K), dev, 128, col, col, ue) for _ in range(copies)]
    state = {"i": 0}

    def step():
        i = state["i"] % copies
        state["i"] += 1
        sglang_amd.sgl_per_token_group_quant_8bit(xs[i], q[i], s[i], 128, 1e-10, -448.0, 448.0, ue, enable_v2=True)

    sec, wall = _time_graph(step, steps, warmup)
    byts = 3 * M * K + (M * (K // 128) if ue else 4 * M * (K // 128))
    return {"M": M, "K": K, "layout": layout, "us": sec * 1e6, "wall_us": _us(wall), "gbs": byts / sec / 1e9,
            "bytes": byts}


def bench_static_quant(dev, M, K, steps, warmup):
    """Static per-tensor FP8 quantisation of a bf16 matrix (the activation step of apply_fp8_linear with a static
    input_scale); 2 bytes read + 1 written per element, + 4 per row for the repeated scale."""
    import torch

    from sglang_amd import ops

    copies = max(1, min(8, (1 << 30) // (M * K * 3)))
    xs = [torch.randn(M, K, device=dev, dtype=torch.bfloat16) for _ in range(copies)]
    q = [torch.empty(M, K, device=dev, dtype=torch.float8_e4m3fn) for _ in range(copies)]
    rows = [torch.empty(M, 1, device=dev, dtype=torch.float32) for _ in range(copies)]
    s = torch.tensor([0.01], device=dev)
    state = {"i": 0}

    def step():
        i = state["i"] % copies
        state["i"] += 1
        ops.static_quant_fp8_(xs[i], q[i], s, rows[i])

    sec, wall = _time_graph(step, steps, warmup)
    byts = M * K * 3 + 4 * M
    return {"M": M, "K": K, "us": sec * 1e6, "gbs": byts / sec / 1e9, "bytes": byts}


def bench_rms_quant(dev, M, K, steps, warmup):
    """Fused residual add + RMSNorm + group quant: reads x and the residual, writes the new residual, the fp8
    row and its scales."""
    import torch

    from sglang_amd.quantization.fused_fp8_quant import fused_rms_fp8_group_quant

    x = torch.randn(M, K, device=dev, dtype=torch.bfloat16)
    res = torch.randn(M, K, device=dev, dtype=torch.bfloat16)
    w = torch.rand(K, device=dev, dtype=torch.bfloat16) + 0.5

    def step():
        return fused_rms_fp8_group_quant(x, w, 1e-6, res1=res)

    sec, wall = _time_events(step, steps, warmup)
    byts = M * K * (2 + 2 + 2 + 1) + 4 * M * (K // 128) + 2 * K
    return {"M": M, "K": K, "us": sec * 1e6, "wall_us": _us(wall), "gbs": byts / sec / 1e9, "bytes": byts}


_MOE_WEIGHTS = {}


def bench_moe(dev, M, steps, warmup, E=256, H=7168, I=2048, topk=8):
    """The DeepSeek-V3 MoE layer.  Several routings are rotated between launches so that the experts a launch
    streams were not touched by the launches just before it: at M = 1 a routing uses 8 experts (352 MB), which
    would otherwise sit in the 256 MB last-level cache from one replay to the next; the rotation covers
    more than 1 GB of distinct expert weights (disjoint expert sets at small M)."""
    import torch

    from sglang_amd.moe_runner import MoeRunnerConfig, fused_moe

    out_of_place = MoeRunnerConfig(inplace=False)
    if "w" not in _MOE_WEIGHTS:
        _MOE_WEIGHTS["w"] = (_rand_fp8((E, 2 * I, H), dev, 100.0, seed=11), _rand_fp8((E, H, I), dev, 100.0, seed=12),
                             torch.rand(E, 2 * I // 128, H // 128, device=dev) * 2e-4,
                             torch.rand(E, H // 128, I // 128, device=dev) * 2e-4)
    w13, w2, w13s, w2s = _MOE_WEIGHTS["w"]
    x = torch.randn(M, H, device=dev, dtype=torch.bfloat16)
    sets = 8 if M * topk * 8 <= E else 4
    routings, n_active = [], []
    for r in range(sets):
        logits = torch.randn(M, E, device=dev)
        if M * topk * sets <= E:
            # disjoint expert ranges: set r routes inside experts [r*E/sets, (r+1)*E/sets)
            mask = torch.full((E,), float("-inf"), device=dev)
            mask[r * (E // sets):(r + 1) * (E // sets)] = 0
            logits = logits + mask
        p = torch.softmax(logits, dim=-1)
        tw, ti = torch.topk(p, topk, dim=-1)
        routings.append(((tw / tw.sum(-1, keepdim=True)).contiguous(), ti.to(torch.int32).contiguous()))
        n_active.append(int(torch.unique(ti).numel()))
    state = {"i": 0}

    def step():
        tw, ti = routings[state["i"] % sets]
        state["i"] += 1
        return fused_moe(x, w13, w2, (tw, ti, None), out_of_place, use_fp8_w8a8=True, w1_scale=w13s, w2_scale=w2s,
                         block_shape=[128, 128])

    steps = max(steps, sets)
    sec, wall = _time_graph(step, steps - steps % sets, warmup)
    act = sum(n_active) / sets
    byts = act * (44040192 + 10752) + 4 * M * H + 64 * M
    flops = 2.0 * M * topk * (2 * I * H + H * I)
    return {"M": M, "n_active": act, "routings_rotated": sets, "us": sec * 1e6, "wall_us": _us(wall),
            "gbs": byts / sec / 1e9, "tflops": flops / sec / 1e12, "bytes": byts}


def bench_moe_grouped(dev, M, steps, warmup, E=256, H=7168, I=2048, topk=8):
    """The same DSV3 MoE layer through the expert-major interface (prepare_moe_input, shuffle_rows,
    fp8_blockwise_scaled_grouped_mm x2, apply_shuffle_mul_sum): 10 launches, replayed from a HIP graph."""
    import torch

    from sglang_amd.moe_runner.cutlass_moe import cutlass_fused_experts_fp8

    if "w" not in _MOE_WEIGHTS:
        _MOE_WEIGHTS["w"] = (_rand_fp8((E, 2 * I, H), dev, 100.0, seed=11), _rand_fp8((E, H, I), dev, 100.0, seed=12),
                             torch.rand(E, 2 * I // 128, H // 128, device=dev) * 2e-4,
                             torch.rand(E, H // 128, I // 128, device=dev) * 2e-4)
    w13, w2, w13s, w2s = _MOE_WEIGHTS["w"]
    x = torch.randn(M, H, device=dev, dtype=torch.bfloat16)
    p = torch.softmax(torch.randn(M, E, device=dev), dim=-1)
    tw, ti = torch.topk(p, topk, dim=-1)
    tw = (tw / tw.sum(-1, keepdim=True)).contiguous()
    ti = ti.to(torch.int32).contiguous()
    n_active = int(torch.unique(ti).numel())
    i64 = lambda v: torch.full((E,), v, device=dev, dtype=torch.int64)
    ptrs = [torch.empty(E, device=dev, dtype=torch.int64) for _ in range(5)]
    ws = torch.empty(1 << 24, device=dev, dtype=torch.uint8)
    offs = torch.empty(E + 1, device=dev, dtype=torch.int32)
    ps1 = torch.empty(E, 3, device=dev, dtype=torch.int32)
    ps2 = torch.empty(E, 3, device=dev, dtype=torch.int32)
    s1, s2, s3, s4 = i64(H), i64(2 * I), i64(I), i64(H)

    def step():
        return cutlass_fused_experts_fp8(x, w13.transpose(1, 2), w2.transpose(1, 2), w13s.transpose(1, 2),
                                         w2s.transpose(1, 2), tw, ti, s1, s2, s3, s4, ws, *ptrs, offs, ps1, ps2)

    sec, wall = _time_graph(step, steps, warmup)
    byts = n_active * (44040192 + 10752) + 4 * M * H + 64 * M
    flops = 2.0 * M * topk * (2 * I * H + H * I)
    return {"M": M, "n_active": n_active, "us": sec * 1e6, "wall_us": _us(wall), "gbs": byts / sec / 1e9,
            "tflops": flops / sec / 1e12, "bytes": byts}


def cpu_baseline(N, K, rows):
    """The CPU oracle (torch-native block-FP8 matmul restated in oracle/) on `rows` tokens of the same
    weight shape, host cores only.  Baseline only -- never the product path."""
    import numpy as np
    import torch

    from oracle import gemm as og

    rng = np.random.default_rng(0)
    aq = rng.integers(0, 0x7E, size=(rows, K), dtype=np.uint8)
    wq = rng.integers(0, 0x7E, size=(N, K), dtype=np.uint8)
    a_s = rng.random((rows, K // 128), dtype=np.float32)
    w_s = rng.random((N // 128, K // 128), dtype=np.float32)
    t0 = time.perf_counter()
    og.block_fp8_matmul(aq, wq, a_s, w_s, out_dtype=torch.bfloat16)
    dt = time.perf_counter() - t0
    return {"value": 2.0 * rows * N * K / dt / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(),
            "kind": "port", "seconds": dt,
            "sample": f"oracle block_fp8_matmul (dequantise + fp32 torch.matmul per 128x128 block), M={rows} rows of "
                      f"the N={N}, K={K} workload, one pass"}


def bench_ceilings(dev):
    """Bare loops of the library (ceilings.hip): the matrix pipe with register operands, and HBM through plain
    16-byte loads over 1 GiB (four times the last-level cache)."""
    import ctypes

    import torch

    from sglang_amd._lib import check, lib

    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    out = torch.empty(256 * 512, device=dev, dtype=torch.float32)
    res = {}
    iters = 10000
    for name, int8, rnd in (("mfma_fp8_constant_operands", 0, 0), ("mfma_fp8_random_operands", 0, 1),
                            ("mfma_int8_constant_operands", 1, 0), ("mfma_int8_random_operands", 1, 1)):
        def step():
            check(lib.sglamd_ceiling_mfma(int8, rnd, iters, ctypes.c_void_p(out.data_ptr()), stream))

        sec, _ = _time_events(step, 5, 2)
        res[name] = {"tops": 256 * 8 * iters * 8 * 131072.0 / sec / 1e12, "us": sec * 1e6}
    # the headline kernel's own loop with every load served by L2 (all tiles read the panels of tile (0, 0)),
    # random finite e4m3 bytes, at the headline shape: what the loop's MFMA + fold + LDS + DMA + barrier + store
    # stream reaches on this box when global memory is out of the picture
    hm, hn, hk = 4096, 36864, 7168
    pa = torch.randint(0, 0x78, (256, hk), device=dev, dtype=torch.uint8) | (torch.randint(0, 2, (256, hk), device=dev, dtype=torch.uint8) << 7)
    pb = torch.randint(0, 0x78, (256, hk), device=dev, dtype=torch.uint8) | (torch.randint(0, 2, (256, hk), device=dev, dtype=torch.uint8) << 7)
    psa = torch.rand(hk // 128, 256, device=dev) * 1e-2 + 1e-3
    psb = torch.rand(2, hk // 128, device=dev) * 1e-4 + 1e-5
    pc = torch.empty(hm, hn, device=dev, dtype=torch.bfloat16)

    def shaped():
        check(lib.sglamd_ceiling_gemm_l2_resident(ctypes.c_void_p(pa.data_ptr()), ctypes.c_void_p(pb.data_ptr()),
                                                  ctypes.c_void_p(psa.data_ptr()), ctypes.c_void_p(psb.data_ptr()),
                                                  ctypes.c_void_p(pc.data_ptr()), ctypes.c_int64(hm), ctypes.c_int64(hn),
                                                  ctypes.c_int64(hk), stream))

    sec, _ = _time_events(shaped, 10, 3)
    res["kernel_shaped_fp8_random_operands"] = {"tops": 2.0 * hm * hn * hk / sec / 1e12, "us": sec * 1e6,
                                                "M": hm, "N": hn, "K": hk}
    del pa, pb, pc
    nbytes = 1 << 30
    src = torch.empty(nbytes, device=dev, dtype=torch.uint8).random_(0, 256)
    dst = torch.empty(nbytes, device=dev, dtype=torch.uint8)
    sink = torch.zeros(1, device=dev, dtype=torch.int32)
    for name, d in (("hbm_read", None), ("hbm_copy", dst)):
        def step():
            check(lib.sglamd_ceiling_hbm(ctypes.c_void_p(d.data_ptr()) if d is not None else None,
                                         ctypes.c_void_p(src.data_ptr()), ctypes.c_int64(nbytes),
                                         ctypes.c_void_p(sink.data_ptr()), stream))

        sec, _ = _time_events(step, 10, 3)
        # a copy moves every byte twice (read + write)
        res[name] = {"gbs": nbytes * (2 if d is not None else 1) / sec / 1e9, "us": sec * 1e6}
    del dst
    # L2 -> CU: every CU re-reads its own 64 KB (L2 resident after the first pass) through direct-to-LDS loads
    # and through register loads: what a CU can take in when neither HBM nor the fabric is in the way
    passes = 400
    for name, lds in (("l2_read_lds", 1), ("l2_read_registers", 0)):
        def step():
            check(lib.sglamd_ceiling_l2_read(ctypes.c_void_p(src.data_ptr()), ctypes.c_int64(nbytes), passes, lds,
                                             ctypes.c_void_p(sink.data_ptr()), stream))

        sec, _ = _time_events(step, 5, 2)
        cus = torch.cuda.get_device_properties(dev).multi_processor_count
        res[name] = {"gbs": passes * cus * 65536 / sec / 1e9, "us": sec * 1e6}
    # The decode launches' own ceiling: a bare read of as many bytes as their weights, cold (the copies of the
    # buffer are read in turn, like the benchmark's weight copies), replayed from a HIP graph like they are.
    for label, mbytes, copies in (("q_b", 24576 * 1536, 8), ("o_proj", 7168 * 16384, 3), ("down", 7168 * 18432, 3),
                                  ("gate_up", 36864 * 7168, 3)):
        state = {"i": 0}

        def step():
            i = state["i"] % copies
            state["i"] += 1
            check(lib.sglamd_ceiling_hbm(None, ctypes.c_void_p(src.data_ptr() + i * mbytes), ctypes.c_int64(mbytes),
                                         ctypes.c_void_p(sink.data_ptr()), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))

        # a ceiling is a best case: the fastest of three measurements of each read pattern
        sec = min(_time_graph(step, 12, 3)[0] for _ in range(3))

        def step_lds():
            i = state["i"] % copies
            state["i"] += 1
            check(lib.sglamd_ceiling_hbm_lds(ctypes.c_void_p(src.data_ptr() + i * mbytes), ctypes.c_int64(mbytes),
                                             ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))

        sec_lds = min(_time_graph(step_lds, 12, 3)[0] for _ in range(3))
        # the ceiling is the faster of the two read patterns (register loads / direct-to-LDS loads)
        best = min(sec, sec_lds)
        res[f"hbm_read_graph_{label}_bytes"] = {"bytes": mbytes, "us": best * 1e6, "gbs": mbytes / best / 1e9,
                                               "register_loads_us": sec * 1e6, "lds_loads_us": sec_lds * 1e6}
    del src
    return res


def main():
    global SETTLE_MS
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--settle-ms", type=float, default=SETTLE_MS, help="device time every measurement keeps its "
                    "operation running before its warm-up steps, so that the chip's clocks have settled (0 = none)")
    ap.add_argument("--no-extra", action="store_true", help="only the headline GEMM and the CPU baseline")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--shape", default="", help="M,N,K of one more dense block-FP8 GEMM to time (cold weights from a HIP "
                    "graph up to 256 rows); with --only noheadline it is the only workload: the form used for profiles")
    ap.add_argument("--detail", default=os.path.join(ROOT, "gpurun_out", "bench_extra.json"),
                    help="file for the full per-workload table ('' = do not write)")
    ap.add_argument("--only", default="", help="comma-separated subset of the extra workloads to run "
                    "(ceilings, quant, decode, prefill, mid, rowwise, llama, int8block, moe1, moe32, moe512, moe4096, moegrouped); implies --no-cpu; the headline GEMM "
                    "always runs unless 'noheadline' is listed")
    args = ap.parse_args()
    SETTLE_MS = args.settle_ms
    if args.gpus != 1:
        print("bench.py: this path is a single-GPU kernel path; only --gpus 1 is measured "
              "(sharding is by slicing N or K above the kernels)", file=sys.stderr)
        sys.exit(2)

    import torch

    import sglang_amd  # noqa: F401  (raises if the HIP library is missing)

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    M, N, K = 4096, 36864, 7168
    only = set(x for x in args.only.split(",") if x)
    want = (lambda name: name in only) if only else (lambda name: not args.no_extra)
    if "noheadline" in only:
        head = {"tflops": 0.0, "us": 0.0, "flops": 0.0, "bytes": 0}
    else:
        head = bench_dense(dev, M, N, K, args.steps, args.warmup)
    extra = {}
    k = max(5, args.steps)
    if args.shape:
        sm, sn, sk = (int(v) for v in args.shape.split(","))
        small = sm <= 256
        extra[f"gemm_M{sm}_N{sn}_K{sk}"] = bench_dense(dev, sm, sn, sk, k, 3, copies=3 if small else 1, graph=small)
    if want("quant"):
        # BASELINE configs[1]: every M, row-major; the column-major and packed-UE8M0 layouts at the ends
        for m in (16384, 4096, 256, 16, 1):
            extra[f"quant_group128_bf16_M{m}_K7168"] = bench_quant(dev, m, 7168, k, 3)
        for m in (16384, 4096, 16):
            extra[f"quant_group128_bf16_M{m}_K7168_colmajor"] = bench_quant(dev, m, 7168, k, 3, layout="col")
            extra[f"quant_group128_bf16_M{m}_K7168_ue8m0"] = bench_quant(dev, m, 7168, k, 3, layout="ue8m0")
        extra["rms_add_quant_bf16_M16384_K7168"] = bench_rms_quant(dev, 16384, 7168, k, 3)
        for m in (16384, 4096, 16):
            extra[f"static_quant_bf16_M{m}_K8192"] = bench_static_quant(dev, m, 8192, k, 3)
    if want("decode"):
        extra["gemm_decode_gate_up_M16"] = bench_dense(dev, 16, N, K, k, 3, copies=3, graph=True)
        extra["gemm_decode_down_M16"] = bench_dense(dev, 16, 7168, 18432, k, 3, copies=3, graph=True)
        extra["gemm_decode_q_b_M16"] = bench_dense(dev, 16, 24576, 1536, k, 3, copies=8, graph=True)
        extra["gemm_decode_o_proj_M16"] = bench_dense(dev, 16, 7168, 16384, k, 3, copies=3, graph=True)
        extra["gemm_decode_gate_up_M1"] = bench_dense(dev, 1, N, K, k, 3, copies=3, graph=True)
        extra["gemm_decode_down_M1"] = bench_dense(dev, 1, 7168, 18432, k, 3, copies=3, graph=True)
        extra["gemm_decode_q_b_M1"] = bench_dense(dev, 1, 24576, 1536, k, 3, copies=8, graph=True)
        extra["gemm_decode_o_proj_M1"] = bench_dense(dev, 1, 7168, 16384, k, 3, copies=3, graph=True)
    if want("prefill"):
        extra["gemm_prefill_down_M4096"] = bench_dense(dev, 4096, 7168, 18432, k, 3)
        extra["gemm_prefill_q_b_M4096"] = bench_dense(dev, 4096, 24576, 1536, k, 3)
        extra["gemm_prefill_o_proj_M4096"] = bench_dense(dev, 4096, 7168, 16384, k, 3)
        extra["gemm_prefill_gate_up_M8192"] = bench_dense(dev, 8192, N, K, max(3, k // 2), 2)
        # the headline shape and the long-K one with UE8M0 (power-of-two) scales: applied inside the MFMA
        extra["gemm_prefill_gate_up_M4096_ue8m0_scales"] = bench_dense(dev, 4096, N, K, k, 3, pow2=True)
        extra["gemm_prefill_down_M4096_ue8m0_scales"] = bench_dense(dev, 4096, 7168, 18432, k, 3, pow2=True)
    if want("mid"):
        for m in (32, 64, 128, 1024):
            extra[f"gemm_gate_up_M{m}"] = bench_dense(dev, m, N, K, k, 3, copies=3, graph=True)
            extra[f"gemm_down_M{m}"] = bench_dense(dev, m, 7168, 18432, k, 3, copies=3, graph=True)
            extra[f"gemm_q_b_M{m}"] = bench_dense(dev, m, 24576, 1536, k, 3, copies=8, graph=True)
            extra[f"gemm_o_proj_M{m}"] = bench_dense(dev, m, 7168, 16384, k, 3, copies=3, graph=True)
    if want("rowwise"):
        extra["fp8_scaled_mm_gate_up_M4096"] = bench_rowwise(dev, 4096, N, K, k, 3)
        extra["int8_scaled_mm_gate_up_M4096"] = bench_rowwise(dev, 4096, N, K, k, 3, int8=True)
    if want("llama"):
        # BASELINE configs[4]: Llama-3-70B unsharded layers (sgl-kernel/benchmark/bench_fp8_gemm.py:45-49),
        # fp8_scaled_mm and int8_scaled_mm (the latter with its bf16 bias); decode-sized M from a graph, cold weights
        for name, (n, kk) in (("qkv", (10240, 8192)), ("o", (8192, 8192)), ("gate_up", (57344, 8192)),
                              ("down", (8192, 28672))):
            cp = max(2, min(8, -(-(600 << 20) // (n * kk))))
            for m in (1, 64, 512, 4096):
                small = m <= 64
                kw = dict(copies=cp if small else 1, graph=small)
                extra[f"llama70b_fp8_scaled_mm_{name}_M{m}"] = bench_rowwise(dev, m, n, kk, k if small else max(3, k // 2), 2, **kw)
                extra[f"llama70b_int8_scaled_mm_bias_{name}_M{m}"] = bench_rowwise(dev, m, n, kk, k if small else max(3, k // 2), 2,
                                                                               int8=True, bias=True, **kw)
            torch.cuda.empty_cache()
    if want("int8block"):
        extra["block_int8_gate_up_M4096"] = bench_block_int8(dev, 4096, N, K, k, 3)
        extra["block_int8_gate_up_M16"] = bench_block_int8(dev, 16, N, K, k, 3, copies=3, graph=True)
    if want("ceilings"):
        extra["measured_ceilings"] = bench_ceilings(dev)
    torch.cuda.empty_cache()
    if want("moe1"):
        extra["moe_dsv3_M1"] = bench_moe(dev, 1, k, 3)
    if want("moe32"):
        extra["moe_dsv3_M32"] = bench_moe(dev, 32, k, 3)
    if want("moe512"):
        extra["moe_dsv3_M512"] = bench_moe(dev, 512, max(3, k // 2), 2)
    if want("moegrouped"):
        extra["moe_grouped_dsv3_M32"] = bench_moe_grouped(dev, 32, k, 3)
        extra["moe_grouped_dsv3_M512"] = bench_moe_grouped(dev, 512, max(3, k // 2), 2)
        extra["moe_grouped_dsv3_M4096"] = bench_moe_grouped(dev, 4096, max(3, k // 2), 2)
    if want("moe4096"):
        extra["moe_dsv3_M4096"] = bench_moe(dev, 4096, max(3, k // 2), 2)
    torch.cuda.empty_cache()
    cpu = None if (args.no_cpu or only) else cpu_baseline(N, K, M)  # the whole workload, one pass (~10 s)

    line = build_line(head, extra, cpu, args.steps, args.warmup)
    detail = dict(line, extra=extra)
    for name, v in extra.items():
        print(json.dumps({name: v}), file=sys.stderr)
    if args.detail:
        try:
            os.makedirs(os.path.dirname(os.path.abspath(args.detail)), exist_ok=True)
            with open(args.detail, "w") as f:
                json.dump(detail, f, indent=1)
        except OSError as e:  # a read-only tree must not cost the headline line
            print(f"bench.py: could not write {args.detail}: {e}", file=sys.stderr)
    sys.stderr.flush()
    print(json.dumps(line), flush=True)


# Workloads whose figure is repeated on the last line, as (key on the line, workload name, field).
TARGETS = (
    ("decode_gate_up_M16_gbs", "gemm_decode_gate_up_M16", "gbs"),
    ("decode_down_M16_gbs", "gemm_decode_down_M16", "gbs"),
    ("decode_o_proj_M16_gbs", "gemm_decode_o_proj_M16", "gbs"),
    ("decode_q_b_M16_gbs", "gemm_decode_q_b_M16", "gbs"),
    ("decode_down_M16_eager_us", "gemm_decode_down_M16", "eager_us"),
    ("gate_up_M64_gbs", "gemm_gate_up_M64", "gbs"),
    ("down_M64_gbs", "gemm_down_M64", "gbs"),
    ("o_proj_M64_gbs", "gemm_o_proj_M64", "gbs"),
    ("gate_up_M128_gbs", "gemm_gate_up_M128", "gbs"),
    ("down_M128_gbs", "gemm_down_M128", "gbs"),
    ("o_proj_M128_gbs", "gemm_o_proj_M128", "gbs"),
    ("gate_up_M1024_tflops", "gemm_gate_up_M1024", "tflops"),
    ("down_M1024_tflops", "gemm_down_M1024", "tflops"),
    ("o_proj_M1024_tflops", "gemm_o_proj_M1024", "tflops"),
    ("q_b_M1024_tflops", "gemm_q_b_M1024", "tflops"),
    ("gate_up_M4096_ue8m0_tflops", "gemm_prefill_gate_up_M4096_ue8m0_scales", "tflops"),
    ("down_M4096_tflops", "gemm_prefill_down_M4096", "tflops"),
    ("moe_M1_gbs", "moe_dsv3_M1", "gbs"),
    ("moe_M32_gbs", "moe_dsv3_M32", "gbs"),
    ("moe_M512_gbs", "moe_dsv3_M512", "gbs"),
    ("moe_M4096_ms", "moe_dsv3_M4096", "ms"),
    ("quant_M16384_gbs", "quant_group128_bf16_M16384_K7168", "gbs"),
    ("quant_M4096_gbs", "quant_group128_bf16_M4096_K7168", "gbs"),
    ("llama_fp8_down_M4096_tflops", "llama70b_fp8_scaled_mm_down_M4096", "tflops"),
    ("llama_int8_down_M4096_tops", "llama70b_int8_scaled_mm_bias_down_M4096", "tflops"),
)


def build_line(head, extra, cpu, steps, warmup):
    """The last stdout line: the contract's fields plus `targets`, never the per-workload table.  Also adds the
    two peak fractions (and the decode GEMMs' bare-read comparison) to the entries of `extra` in place."""
    for v in extra.values():
        if isinstance(v, dict) and "us" in v:
            if "gbs" in v:
                v["frac_hbm_peak"] = v["gbs"] / PEAK_HBM_GBS
            if "tflops" in v:
                v["frac_mfma_peak"] = v["tflops"] / PEAK_FP8_TFLOPS
    r3 = lambda x: None if x is None else float(f"{x:.4g}")
    line = {
        "metric": "block-FP8 GEMM TFLOP/s (% FP8 MFMA peak) at DSV3 shapes; quant+MoE GB/s",
        "value": r3(head["tflops"]),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "settle_ms": SETTLE_MS,  # device time the operation runs before the warm-up steps (clock ramp, see _settle)
        "ms_per_step": r3(head["us"] / 1e3),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp8_e4m3fn (fp32 accumulate, bf16 out)",
        "data": "synthetic: A ~N(0,1) group-quantised by the library; W on the e4m3 grid, block scales U[0,1.8e-4]",
        "config": {"workload": "dsv3_dense_gate_up block-FP8 GEMM M=4096 N=36864 K=7168 (BASELINE configs[2])",
                   "op": "fp8_blockwise_scaled_mm", "block": [128, 128], "out_dtype": "bf16"},
        "roofline": {"bound": "mfma", "achieved": r3(head["tflops"]), "peak": PEAK_FP8_TFLOPS, "unit": "TFLOP/s",
                     "frac": r3(head["tflops"] / PEAK_FP8_TFLOPS), "traffic": MEASURED_TRAFFIC_BYTES,
                     "kernel_us": r3(head["us"]), "algorithmic_flops": head["flops"],
                     "algorithmic_bytes": head["bytes"]},
        "cpu_baseline": cpu,
    }
    ceil = extra.get("measured_ceilings")
    if ceil and head["tflops"] > 0:
        # beside the published peak: ceilings measured in this run (bare MFMA loop on random operand bits, and
        # the loop with the shipped kernel's LDS traffic, DMA and barriers but no global-memory misses)
        top = ceil["mfma_fp8_random_operands"]["tops"]
        line["roofline"]["measured_ceiling"] = r3(top)
        line["roofline"]["frac_of_measured_ceiling"] = r3(head["tflops"] / top)
        shaped = ceil.get("kernel_shaped_fp8_random_operands")
        if shaped:
            line["roofline"]["kernel_shaped_ceiling"] = r3(shaped["tops"])
            line["roofline"]["frac_of_kernel_shaped_ceiling"] = r3(head["tflops"] / shaped["tops"])
    if ceil:
        # decode GEMMs beside a bare read of their weight bytes, timed the same way in this run
        for name, v in extra.items():
            for label in ("q_b", "o_proj", "down", "gate_up"):
                c = ceil.get(f"hbm_read_graph_{label}_bytes")
                if c and name.startswith(f"gemm_decode_{label}_M"):
                    v["bare_read_of_the_weights_us"] = c["us"]
                    v["frac_of_measured_ceiling"] = c["us"] / v["us"]
    targets = {}
    for key, name, field in TARGETS:
        v = extra.get(name)
        if not v:
            continue
        targets[key] = r3(v["us"] / 1e3) if field == "ms" else r3(v.get(field))
    if ceil:
        targets["ceiling_hbm_read_gbs"] = r3(ceil["hbm_read"]["gbs"])
        targets["ceiling_mfma_fp8_constant_tflops"] = r3(ceil["mfma_fp8_constant_operands"]["tops"])
    line["targets"] = targets
    return line


if __name__ == "__main__":
    main()

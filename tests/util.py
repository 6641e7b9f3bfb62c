"""Shared helpers for the parity tests: seeded inputs in the reference tests' recipes and
the tolerances of the north-star contract."""
import numpy as np
import torch


def outlier_input(rows: int, hidden: int, dtype=torch.bfloat16, scale: float = 10.0, seed=None) -> torch.Tensor:
    """randn with ~0.1% of entries multiplied by `scale`, seeded by rows*10000+hidden
    (recipe of sgl-kernel/python/sgl_kernel/test_utils.py:4-62)."""
    g = torch.Generator().manual_seed(rows * 10000 + hidden if seed is None else seed)
    x = torch.randn(rows, hidden, generator=g, dtype=torch.float32)
    mask = torch.rand(rows, hidden, generator=g) < 0.001
    x = torch.where(mask, x * scale, x)
    return x.to(dtype)


def codes(t: torch.Tensor) -> np.ndarray:
    """fp8 / int8 tensor -> numpy bytes on the host."""
    if t.dtype == torch.float8_e4m3fn:
        return t.detach().cpu().view(torch.uint8).numpy()
    return t.detach().cpu().numpy()


def rel_l2(out: torch.Tensor, ref: torch.Tensor) -> float:
    o, r = out.detach().double().cpu(), ref.detach().double().cpu()
    return float((o - r).norm() / r.norm().clamp_min(1e-30))


def max_abs_ratio(out: torch.Tensor, ref: torch.Tensor) -> float:
    o, r = out.detach().double().cpu(), ref.detach().double().cpu()
    return float((o - r).abs().max() / r.abs().max().clamp_min(1e-30))


# north-star tolerances for GEMM / MoE outputs
REL_L2_TOL = 1e-2
MAX_ABS_TOL = 2e-2


def assert_gemm_close(out: torch.Tensor, ref: torch.Tensor, what: str = "") -> None:
    rl, ma = rel_l2(out, ref), max_abs_ratio(out, ref)
    assert rl <= REL_L2_TOL, f"{what}: rel-L2 {rl:.3e} > {REL_L2_TOL}"
    assert ma <= MAX_ABS_TOL, f"{what}: max-abs/max|ref| {ma:.3e} > {MAX_ABS_TOL}"


def moe_layer(hidden_states, w1, w2, topk_output, *, inplace=False, no_combine=False, routed_scaling_factor=None,
              config=None, activation="silu", is_gated=True, **quant_kw):
    """The fused MoE layer through the reference's entry point: fused_moe with a MoeRunnerConfig carrying the
    runner flags (the reference's default configuration works in place; tests want a fresh output unless they
    say otherwise).  `config` forces the sorted-block height, which only fused_experts_impl takes."""
    from sglang_amd.moe_runner import MoeRunnerConfig, fused_experts_impl, fused_moe

    if config is not None:
        return fused_experts_impl(hidden_states, w1, w2, topk_output[0], topk_output[1], inplace=inplace,
                                  no_combine=no_combine, routed_scaling_factor=routed_scaling_factor, config=config,
                                  activation=activation, is_gated=is_gated, **quant_kw)
    cfg = MoeRunnerConfig(inplace=inplace, no_combine=no_combine, routed_scaling_factor=routed_scaling_factor,
                          activation=activation, is_gated=is_gated)
    return fused_moe(hidden_states, w1, w2, topk_output, cfg, **quant_kw)

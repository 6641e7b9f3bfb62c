"""bench.py's last stdout line must stay small enough for a reader that keeps only a tail of stdout: the
per-workload table belongs in the detail file, never on that line."""
import importlib.util
import json
import os

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench():
    spec = importlib.util.spec_from_file_location("bench_under_test", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def _stub_extra(bench):
    """An entry for every workload name a full run produces (several times more than the line may carry)."""
    rec = lambda i: {"M": 4096, "N": 36864, "K": 7168, "us": 100.123456789 + i, "wall_us": None,
                     "tflops": 2345.678901234 + i, "gbs": 5432.10987654321 + i, "flops": 2.1e12, "bytes": 5.9e8,
                     "eager_us": 17.5, "eager_wall_us": 18.5}
    extra = {name: rec(i) for i, (_, name, _) in enumerate(bench.TARGETS)}
    for i in range(120):
        extra[f"some_other_workload_with_a_long_name_{i}"] = rec(i)
    ceil = {k: {"tops": 4000.123456 + i, "us": 1.0} for i, k in enumerate(
        ("mfma_fp8_constant_operands", "mfma_fp8_random_operands", "mfma_int8_constant_operands",
         "mfma_int8_random_operands", "kernel_shaped_fp8_random_operands"))}
    ceil["hbm_read"] = {"gbs": 6789.123456, "us": 1.0}
    for label in ("q_b", "o_proj", "down", "gate_up"):
        ceil[f"hbm_read_graph_{label}_bytes"] = {"bytes": 1, "us": 20.0, "gbs": 5000.0}
    extra["measured_ceilings"] = ceil
    return extra


def test_last_line_is_small_and_carries_the_contract():
    bench = _bench()
    head = {"tflops": 2234.56789, "us": 968.7654321, "flops": 2.164663517184e12, "bytes": 596573184}
    cpu = {"value": 0.6466228165618186, "unit": "TFLOP/s", "cores": 16, "kind": "port", "seconds": 3.35,
           "sample": "oracle block_fp8_matmul (dequantise + fp32 torch.matmul per 128x128 block), M=4096 rows of "
                     "the N=36864, K=7168 workload, one pass"}
    extra = _stub_extra(bench)
    text = json.dumps(bench.build_line(head, extra, cpu, 20, 5))
    assert len(text) < 4096, len(text)
    line = json.loads(text)
    assert "extra" not in line
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline", "targets"):
        assert key in line, key
    assert line["steps"] == 20 and line["warmup"] == 5 and line["n_gpus"] == 1
    assert abs(line["roofline"]["frac"] - 2234.56789 / 5000.0) < 1e-3
    assert line["roofline"]["bound"] == "mfma" and line["roofline"]["peak"] == 5000.0
    assert abs(line["ms_per_step"] - 0.9687654) < 1e-3
    assert line["cpu_baseline"]["kind"] == "port" and line["cpu_baseline"]["cores"] == 16
    assert "workload" in line["config"] and "model" not in line["config"]
    assert len(line["targets"]) >= 12
    # the builder annotates the table entries in place for the detail file
    assert "frac_hbm_peak" in extra["gemm_decode_down_M16"]
    assert abs(extra["gemm_decode_down_M16"]["frac_of_measured_ceiling"] - 20.0 / extra["gemm_decode_down_M16"]["us"]) < 1e-9


def test_line_without_extras_still_parses():
    bench = _bench()
    head = {"tflops": 2000.0, "us": 1000.0, "flops": 2.1e12, "bytes": 5.9e8}
    line = json.loads(json.dumps(bench.build_line(head, {}, None, 3, 1)))
    assert line["roofline"]["frac"] == 0.4 and line["targets"] == {} and line["cpu_baseline"] is None

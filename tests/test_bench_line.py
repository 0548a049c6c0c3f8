"""The one JSON line bench.py prints must stay short enough for a reader that keeps only the tail of stdout, and
must carry the roofline and CPU-baseline objects whatever else is dropped."""
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

import bench  # noqa: E402
from therock_amd import inputs as mi  # noqa: E402


def _stub_result(cfg, ms):
    kern = {"moe_sorting_count": 0.00696, "moe_sorting_scan": 0.01419, "moe_sorting_scatter": 0.00965,
            "moe_gemm0_gate_up_silu": ms * 0.56, "moe_gemm1_down": ms * 0.38, "moe_combine": ms * 0.05}
    T, K = cfg.tokens, cfg.topk
    return {"workload": cfg.name, "dtype": cfg.dtype, "fused_quant": 0, "tokens": T, "hidden": cfg.hidden,
            "inter": cfg.inter, "experts": cfg.experts, "topk": K, "block_m": cfg.unit, "tile_rows": 320,
            "ms_per_step": ms, "tflops": cfg.flops / ms / 1e9, "tokens_per_s": T / ms * 1e3, "algorithmic_GB": 11.46,
            "hbm_GBps": 11.46e3 / ms, "frac_mfma_peak": cfg.flops / ms / 1e9 / bench.PEAK_MFMA[cfg.dtype],
            "frac_hbm_peak": 11.46e3 / ms / bench.PEAK_HBM, "gemm_only_ms": ms * 0.99, "post_pad": T * K + 4000,
            "active_experts": cfg.experts, "kernel_avg_ms": kern, "gemm0_tflops": 2000.123456, "gemm1_tflops": 1500.123456}


def _line(n_workloads):
    cfg = mi.CONFIGS[bench.HEADLINE]
    res = _stub_result(cfg, 3.2987654321)
    roof, roof1 = bench.roofline_of(cfg, res), bench.roofline_of(cfg, res, 1)
    cpu = {"value": 0.004612345, "unit": "TFLOP/s", "cores": 1, "kind": "reference", "seconds": 13.912345,
           "sample": "the rows routed to experts [1, 2, 3] of cfg3 " + "x" * 400}
    names = list(mi.CONFIGS) + [f"extra_workload_with_a_long_name_{i}" for i in range(n_workloads)]
    others = {n: _stub_result(mi.CONFIGS.get(n, cfg), 0.4 + 0.01 * i) for i, n in enumerate(names)}
    others["one_that_failed"] = {"error": "RuntimeError('" + "boom " * 100 + "')"}
    router = {"kernel": "topk_softmax_kernel", "avg_launch_ms": 0.0109876, "bytes": 1, "GBps": 840.0}
    nb = {k: {"ms": 0.123456, "what": "w" * 80} for k in ("rowwise_quant", "moe_smoothquant", "permute_weights",
                                                          "flatmm_gate_up", "flatmm_down")}
    return bench.build_line(cfg, 20, 3, res, roof, roof1, cpu, router, nb, others)


def test_line_is_short_and_complete():
    line = _line(9)
    text = json.dumps(line, separators=(",", ":"))
    assert len(text) < bench.MAX_LINE_BYTES, len(text)
    back = json.loads(text)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in back, key
    assert back["vs_baseline"] is None and back["n_gpus"] == 1 and "model" not in back["config"]
    for roof in (back["roofline"], back["roofline_gemm1"]):
        assert set(("bound", "achieved", "peak", "unit", "frac", "traffic")) <= set(roof)
        assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3
    assert set(("value", "unit", "cores", "kind", "sample")) <= set(back["cpu_baseline"])
    assert back["workloads"]["cfg4_decode_int8_t64"]["unit"] == "GB/s"
    assert "workloads" in back and "error" in back["workloads"]["one_that_failed"]


def test_line_sheds_optional_parts_before_it_outgrows_the_limit():
    line = _line(200)
    text = json.dumps(line, separators=(",", ":"))
    assert len(text) < bench.MAX_LINE_BYTES
    assert "workloads" not in line and line["roofline"] and line["cpu_baseline"]


def test_power_reading_is_parsed_and_reported():
    text = """GPU: 0
    POWER:
        SOCKET_POWER: 1395 W
        GFX_VOLTAGE: N/A
    CLOCK:
        GFX_0:
            CLK: 1921 MHz
            MIN_CLK: 500 MHz
        GFX_1:
            CLK: 1874 MHz
"""
    assert bench.parse_smi(text) == (1395.0, 1921.0)
    assert bench.parse_smi("ERROR:root:Unable to get devices") is None
    assert bench.parse_smi("        SOCKET_POWER: 640 W\n") == (640.0, None)
    cfg = mi.CONFIGS[bench.HEADLINE]
    res = _stub_result(cfg, 3.3)
    line = bench.build_line(cfg, 20, 3, res, bench.roofline_of(cfg, res), bench.roofline_of(cfg, res, 1), None, None, None, {},
                            {"random_operands": 3912.4, "zero_operands": 4948.1, "unit": "TFLOP/s"},
                            {"socket_power_w": 1389.7, "power_cap_w": 1400.0, "gfx_clock_mhz": 1905.3})
    assert line["power"] == {"socket_power_w": 1390.0, "power_cap_w": 1400.0, "gfx_clock_mhz": 1905.0}
    assert abs(line["mfma_sustained"]["frac_of_sustained"] - res["tflops"] / 3912.4) < 1e-3
    assert len(json.dumps(line, separators=(",", ":"))) < bench.MAX_LINE_BYTES

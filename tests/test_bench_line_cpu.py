"""The last stdout line of bench.py has to stay short enough for a harness that keeps only a tail of
the output: built here from stub figures of the real tables' shape."""
import json
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import bench  # noqa: E402


def _stub_tables():
    layers = ("qkv", "o", "gate_up", "down")
    extra = {
        "read_floor": {**{n: {"us": 3.5, "GBps": 3700.0} for n in layers}, "step_of_four_reads_us": 22.4,
                       "step_measured_over_floor": 1.21, "dominant_kernel_over_its_read": 1.16},
        "gemv_M1": {f"{n}_b{b}_{z}": {"us": 11.11, "weight_GBps": 5000.1, "pct_hbm_peak": 62.5}
                    for n in layers for b in (8, 6, 4, 3, 2) for z in ("zp", "sym")},
        "prefill_llama3_70b": {f"{n}_b{b}_M2048_zp": {"ms": 0.28, "TFLOPs": 1200.1, "pct_mfma_peak": 48.0 + b,
                                                      "kernel": "prefill b4 g128 zp1 cfg8"}
                               for n in layers for b in (2, 3, 4, 6, 8)},
        "medium_batch_llama3_70b_b4": {f"{n}_M{m}": {"us": 95.0, "dense_us": 84.1, "speedup": 0.88 + m / 1e4}
                                       for n in layers for m in (128, 256, 512, 1024)},
        "mixnmatch_decoder_end_to_end": {"tokens_per_s_graph": 517.2},
        # bulk that must NOT reach the line
        "speedup_over_dense_fp16": {f"{s}_M{m}": {f"b{b}": 1.0 for b in (2, 3, 4, 6, 8)}
                                    for s in (2048, 4096, 8192, 16384) for m in (1, 2, 4, 8, 16, 32, 64)},
    }
    headline = {"value": 3993.9, "steps": 200, "warmup": 20, "ms_per_step": 0.0273, "wall_s_timed_region": 0.13}
    roofline = {"kernel": "gemv b4 g128 zp1 T4 R1 W8 pad0", "bound": "hbm", "achieved": 5258.2, "peak": 8000.0,
                "unit": "GB/s", "frac": 0.6573, "traffic": 62563275, "kernel_source_hash": "e1bf11cff8329e68",
                "us_per_launch": 11.88, "algorithmic_bytes": 62455808}
    cpu = {"value": 0.999, "unit": "GB/s", "cores": 16, "kind": "port", "sample": "one full step " * 8,
           "config4_prefill_o_layer": {"x": list(range(200))}}
    return headline, roofline, cpu, extra


def test_final_line_is_short_and_complete():
    headline, roofline, cpu, extra = _stub_tables()
    line = bench.final_line(headline, roofline, cpu, extra, "gpurun_out/bench_extra.json")
    assert "\n" not in line and len(line) < bench.LINE_LIMIT
    out = json.loads(line)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better",
                "scaling", "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in out
    assert out["config"]["workload"].startswith("configs[1]")
    assert set(out["roofline"]) >= {"bound", "achieved", "peak", "unit", "frac", "traffic"}
    assert out["roofline"]["frac"] == 0.6573
    assert set(out["cpu_baseline"]) == {"value", "unit", "cores", "kind", "sample"}
    assert out["summary"]["prefill_b4_M2048_qkv_pct_mfma_peak"] == 52.0
    assert out["summary"]["prefill_b6_b8_min_pct_mfma_peak"] == 54.0
    assert out["summary"]["medium_batch_min_speedup_over_dense_fp16"] == 0.8928
    assert "2048_M1" not in line


def test_final_line_without_tables_and_with_oversized_scalars():
    headline, roofline, _cpu, _extra = _stub_tables()
    out = json.loads(bench.final_line(headline, roofline, None, {}, None))
    assert out["cpu_baseline"] is None and out["summary"] == {} and out["tables"] is None
    roofline = dict(roofline, kernel="k" * 3000)
    huge = {"read_floor": {"step_measured_over_floor": "x" * 3000}}
    line = bench.final_line(headline, roofline, None, huge, None)
    assert len(line) < bench.LINE_LIMIT and json.loads(line)["summary"] == {}

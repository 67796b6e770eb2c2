"""The benchmark's stdout contract: every line it prints is one compact JSON object short enough for a recorder
that keeps only the tail of stdout, and the last line carries the headline keys."""
import json

import bench


def fake_result(workload, long_sample=False):
    roofline = {"bound": "hbm", "kernel": "moe_route_gate_up_shared", "achieved": 5110.6, "peak": 8000.0, "unit": "GB/s",
                "frac": 0.6388, "traffic": 34027038, "traffic_source": "profiles/hbm_traffic.json",
                "alg_bytes_per_launch": 439410688, "avg_launch_us": 85.98, "floor_launch_us": 72.909, "achievable_frac": 0.7534,
                "frac_of_data_movement_floor": 0.7777}
    sample = ("scalar auto-vectorised C restatement of the reference's CPU path, not its AVX2/AVX-512/VNNI tiers; "
              "192 passes of layer 0 (routed experts, 256 token rows), 1259.11 ms each, int8-activation production numerics, "
              "scaled to 48 layers")
    if long_sample:
        sample += " and more words" * 400
    return {
        "metric": "MoE decode tok/s", "value": 123456.78, "unit": "tok/s", "n_gpus": 1, "steps": 200, "warmup": 20,
        "ms_per_step": 1.0912, "ms_per_step_min": 1.0901, "ms_per_step_max": 1.1003, "spread": "x" * 200,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "i8dot-23bit-act/f32-acc",
        "data": "synthetic",
        "config": {"workload": workload, "layers": 48, "hidden": 2048, "experts": 128, "top_k": 8, "intermediate": 768,
                   "gate_up": "Q4K", "down": "Q6K", "shared_intermediate": 1536, "batch": 2048, "parallelism": "single-gpu",
                   "resident_weight_bytes": 125983129600},
        "layer": {"us_per_layer": 178.253, "alg_bytes_per_layer": 763265024, "achieved_GBps": 4281.9,
                  "frac_of_hbm_peak": 0.5352, "distinct_experts_layer0": 61},
        "roofline": roofline, "floor": {"note": "y" * 500}, "kernels": {f"k{i}": {"avg_us": 1.0} for i in range(40)},
        "cpu_baseline": {"value": 3.383, "unit": "tok/s", "cores": 16, "kind": "port", "sample": sample, "ms_per_layer": 59.112},
        "device": "AMD Instinct MI355X", "compute_units": 256, "setup_s": 12.3, "detail": "gpurun_out/bench_configs.json",
    }


def test_headline_line_is_compact_and_complete():
    line = bench.compact(fake_result("c2-qwen3-30b-a3b-q4k-q6k-48L"), headline=True)
    assert "\n" not in line and len(line.encode()) < 2000
    d = json.loads(line)
    for k in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
              "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert k in d, k
    assert d["config"]["workload"].startswith("c2-") and "model" not in d["config"]
    for k in ("bound", "achieved", "peak", "unit", "frac", "traffic"):
        assert k in d["roofline"], k
    for k in ("value", "unit", "cores", "kind", "sample"):
        assert k in d["cpu_baseline"], k
    assert "kernels" not in d and "floor" not in d


def test_other_configs_and_oversized_prose_stay_under_the_limit():
    line = bench.compact(fake_result("c5-large-moe-256e-shared-q4k-q6k-40L"), headline=False)
    assert len(line.encode()) < 2000 and json.loads(line)["cpu_baseline"]["cores"] == 16
    line = bench.compact(fake_result("c2-qwen3-30b-a3b-q4k-q6k-48L", long_sample=True), headline=True)
    assert len(line.encode()) < 2000
    assert json.loads(line)["roofline"]["frac"] == 0.6388

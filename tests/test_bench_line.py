"""The benchmark's one stdout line must stay short enough for a harness that keeps a bounded tail of stdout, and must
carry the keys the measurement contract names.  Built here from the per-workload records of a real run
(tests/golden/bench_records_sample.json: 29 workloads, 21 KB as one line), no GPU involved."""
import importlib.util
import json
import os

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench():
    spec = importlib.util.spec_from_file_location("bench_under_test", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def _records():
    with open(os.path.join(ROOT, "tests", "golden", "bench_records_sample.json")) as f:
        return json.load(f)


def test_result_line_is_short_and_complete():
    bench, rec = _bench(), _records()
    text = bench.result_line(rec["workloads"], 5, rec["cpu_baseline"])
    assert "\n" not in text
    assert len(text) < 4096
    line = json.loads(text)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "gemm", "cpu_baseline"):
        assert key in line, key
    assert line["metric"] == "Q4_0 GEMV GB/s (% HBM peak); int8 prefill GEMM TOPS (% MFMA peak)"
    assert line["n_gpus"] == 1 and line["vs_baseline"] is None and "workload" in line["config"]
    assert "model" not in line["config"] and "workloads" not in line
    roof = line["roofline"]
    for key in ("bound", "achieved", "peak", "unit", "frac", "traffic"):
        assert key in roof, key
    assert roof["bound"] == "hbm" and roof["peak"] == 8000.0
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3
    # achieved = algorithmic bytes per launch / average launch duration
    assert abs(roof["achieved"] - roof["algorithmic_bytes_per_launch"] / roof["kernel_avg_us"] / 1e3) < 2.0
    g = line["gemm"]["roofline"]
    assert g["bound"] == "mfma" and g["peak"] == 5000.0 and abs(g["frac"] - g["achieved"] / g["peak"]) < 1e-3
    cpu = line["cpu_baseline"]
    for key in ("value", "unit", "cores", "kind", "sample"):
        assert key in cpu, key
    # one timing method is named for the headline; the other stays a field
    assert line["config"]["timed_region"] == "one captured graph of the K steps"
    assert "call_by_call_us" in line["config"]
    assert line["value"] == bench._r(rec["workloads"]["q4_0_gemv_9728x2560"]["GBps"])


def test_result_line_stays_bounded_with_many_workloads():
    bench, rec = _bench(), _records()
    work = dict(rec["workloads"])
    for i in range(200):   # far more workloads than the line can summarise: the summary is cut, the line stays whole
        work[f"extra_workload_with_a_long_descriptive_name_{i}"] = dict(work["q8_0_gemv_2560x9728_m1"])
    text = bench.result_line(work, 5, rec["cpu_baseline"])
    assert len(text) < 4096
    line = json.loads(text)
    assert "roofline" in line and "cpu_baseline" in line and "gemm" in line


def test_result_line_without_floors_or_cpu():
    bench, rec = _bench(), _records()
    work = {k: v for k, v in rec["workloads"].items() if k != "machine_floors"}
    line = json.loads(bench.result_line(work, 5, None))
    assert "cpu_baseline" not in line and "read_only_floor_us" not in line["roofline"]

"""The stdout line of bench.py is read by a harness that keeps only a few KB: whatever a run measured, the line that
carries the metric, the roofline and the CPU baseline stays under 4 KB and parses."""
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

import bench  # noqa: E402  (imports nothing of the package at module level)


def _point(i):
    return {"offered_rps": 12345.678901 * i, "achieved_rps": 12001.123456 * i, "p50_us": 88.123456, "p99_us": 6665.123456,
            "small_cnn_p50_us": 83.7, "small_cnn_p99_us": 211.123456, "small_cnn_count": 9216, "inception_v3_p50_us": 4443.1,
            "inception_v3_p99_us": 7945.123456, "inception_v3_count": 1024, "meets_slo": bool(i % 2), "attempt": 0}


def _full_result():
    arms = ["full3", "full3_hip_launch", "fifo2_direct_dispatch", "fifo2_hip_launch", "fifo_direct_dispatch", "fifo_multi_stream", "direct_multi_stream"]
    searches = {a: {"saturation_rps": 45170.123456, "rate_at_slo_rps": 44820.123456, "points": [_point(i) for i in range(1, 15)]} for a in arms}
    rf = {"bound": "mfma", "achieved": 25.398179995648714, "peak": 157.3, "unit": "TFLOP/s", "frac": 0.16146331847201978, "traffic": 9430000.0,
          "kernel": "x" * 300, "flops_per_launch_avg": 243028429.617, "us_per_launch_avg": 9.5687340, "algorithmic_bytes_per_launch_avg": 4220463.23,
          "served": {"forward_passes_per_s": 5257.04, "conv_tflops": 60.04, "frac": 0.3817, "how": "y" * 400},
          "under_load": {"forward_passes_per_s": 4686.6, "conv_tflops": 53.5, "frac": 0.34, "how": "y" * 400},
          "full_device": {"achieved": 71.5, "frac": 0.455, "unit": "TFLOP/s", "how": "z" * 400}, "peak_measured": 154.2, "empty_kernel_us": 3.96}
    return {
        "metric": bench.METRIC, "value": 45027.31234, "unit": "requests/s", "n_gpus": 1, "steps": 20, "warmup": 2, "ms_per_step": 45.4812345,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "w" * 600, "slo_us": {"small_cnn": 256.12, "inception_v3": 8687.52}, "slo_factor": 10.0,
                   "alone_latency": {"small_cnn": {"p50_us": 25.6}, "inception_v3": {"p50_us": 868.7}}, "requests_per_step": 2048,
                   "timed_requests": 40960, "timed_seconds": 0.9096, "pools": {"small_cnn": 96, "inception_v3": 16}},
        "offered_rps": 44820.1, "latency_us": {k: v for k, v in _point(1).items() if k.endswith("_us")}, "slo_met": True,
        "verified_requests": 40960, "mismatches": 0,
        "timed_run_attempts": [_point(1)] * 8, "rate_search": searches,
        "arms_at_equal_offered_load": {"offered_rps": 35000.0, "arms": {a: _point(2) for a in arms}},
        "roofline": rf, "roofline_resnet18": dict(rf),
        "cpu_baseline": {"value": 19.13, "unit": "requests/s", "cores": 16, "kind": "port", "sample": "s" * 500},
        "cpu_baseline_torch": {"value": 380.4, "unit": "requests/s", "cores": 16, "kind": "port", "sample": "s" * 500},
        "side_workloads": dict({"k%d" % i: {"points": [_point(j) for j in range(6)]} for i in range(8)},
                               policy_reference_two_model_workload={"arms": {a: [dict(_point(j), resnet18_p99_us=1234.56789, inception_v3_p99_us=23456.789)
                                                                                 for j in range(1, 4)] for a in arms[:4]}}),
        "per_op_us": {op: {"launches": 3, "us": 12.3, "gflop": 1.0, "mbytes": 2.0, "tflops": 3.0, "gbytes_per_s": 4.0} for op in ("conv", "pool", "dense", "gap")},
        "notify_us": {"ring_drain_64_blocks_us_per_kernel": 11.87, "launch_plus_flag_store_us": 6.25, "launch_plus_stream_sync_us": 9.5,
                      "echo_round_trip_us": {"p50": 2.98, "p99": 3.29, "what": "q" * 200}, "gpu_to_host_us": {"upper_bound_p50": 2.98, "upper_bound_p99": 3.29, "what": "q" * 200, "clock_translated": {"p50": -1.6, "p99": -1.4, "plausible": False}}},
    }


def test_headline_is_short_and_carries_the_contract():
    out = _full_result()
    assert len(json.dumps(out)) > 20000  # the detail really is too long for the harness
    text = bench.headline(out)
    assert "\n" not in text and len(text.encode()) < 4096, len(text.encode())
    line = json.loads(text)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling", "vs_baseline", "dtype", "data", "config",
                "roofline", "cpu_baseline"):
        assert key in line, key
    assert set(("bound", "achieved", "peak", "unit", "frac", "traffic")) <= set(line["roofline"])
    assert set(("value", "unit", "cores", "kind", "sample")) <= set(line["cpu_baseline"])
    assert "workload" in line["config"] and "model" not in line["config"]
    assert abs(line["value"] - out["value"]) <= 1e-5 * out["value"]
    assert abs(line["roofline"]["frac"] - line["roofline"]["achieved"] / line["roofline"]["peak"]) < 1e-4


def test_headline_survives_an_unmet_slo_and_missing_parts():
    out = _full_result()
    out.update({"value": None, "slo_met": False, "cpu_baseline": None, "cpu_baseline_torch": None, "rate_search": {}, "notify_us": {}})
    line = json.loads(bench.headline(out))
    assert line["value"] is None and line["cpu_baseline"] is None

"""Workload tooling on the device: a pre-generated log-normal trace replayed through the client library, the
deficit-threshold knob of full3 moving per-type latency the way the fairness sweep relies on, and the direct
no-server multi-stream arm (reference tests/utils/workload_pregen.cpp:72-112, sosp23_artifact/gen_data_fig13.sh:37-60,
tests/simple/tvm_direct_multistream.cpp:143-301)."""
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

_n = [0]


def server_name(tag):
    _n[0] += 1
    return "wl%d_%s_%d" % (os.getpid(), tag, _n[0])


def test_pregenerated_lognormal_trace_replays_with_its_own_type_counts(cuda, tmp_path):
    """Two models, log-normal gaps (sigma 1.5): the replay serves exactly the trace's requests, type by type, and the
    run lasts about as long as the trace says."""
    from paella_amd import serve
    os.environ["LLIS_MODEL_SEED"] = "1"
    n = 600
    path = serve.workload_pregen(tmp_path / "w", [0.7, 0.3], iat_us=400.0, num_jobs=n, seed=5, dist="ln", ln_sigma=1.5)
    assert os.path.basename(path) == "w_iat400_lns1.5_n600_seed5.txt"
    trace = [l.split() for l in open(path)]
    assert len(trace) == n
    want = [sum(1 for t in trace if t[0] == str(k)) for k in (0, 1)]
    assert sum(want) == n and min(want) > 100
    span_us = float(trace[-1][1])
    jobs = [(serve.job_path("tvm_mnist"), 0.7, 16), (serve.job_path("tvm_resnet18"), 0.3, 16)]
    print("case trace replay", want, span_us, flush=True)
    with serve.Server(server_name("trace"), "full3", num_streams=32, extra_kernels=16) as srv:
        r = serve.client_run(srv.name, jobs, 400.0, 32, n, warmup_jobs=0, seed=99, dist="ln", ln_sigma=1.5, trace_path=path)
    assert [r["per_type"][k]["count"] for k in (0, 1)] == want       # the trace decides, not seed 99
    assert r["all"]["count"] == n
    assert 0.9 * span_us <= r["elapsed_us"] <= span_us + 50_000       # open loop: the clock follows the trace


def test_deficit_threshold_moves_latency_between_the_types(cuda):
    """ResNet-18 : Inception-v3 = 0.952 : 0.048 at saturation (the fairness sweep's mix).  Shortest-remaining-work-first
    alone (threshold 1e6) starves the long model; a threshold of 1 lets its deficit counter win turns, so its mean
    latency drops and the short model pays for it."""
    from paella_amd import serve
    os.environ["LLIS_MODEL_SEED"] = "1"
    jobs = [(serve.job_path("tvm_resnet18"), 0.952, 60), (serve.job_path("tvm_inception_v3"), 0.048, 6)]
    mean = {}
    for unfair in (1.0, 1e6):
        print("case fairness threshold", unfair, flush=True)
        with serve.Server(server_name("fair"), "full3", num_streams=96, extra_kernels=16, unfair=unfair) as srv:
            r = serve.client_run(srv.name, jobs, 0.0, 66, 2500, warmup_jobs=300, seed=1)
        assert r["per_type"][1]["count"] > 60
        mean[unfair] = [r["per_type"][k]["mean"] for k in (0, 1)]
    assert mean[1.0][1] < 0.85 * mean[1e6][1], mean      # the long model gains
    assert mean[1.0][0] > 0.98 * mean[1e6][0], mean      # and not at no cost to the short one


def test_direct_multistream_arm_serves_the_mix(cuda):
    from paella_amd import serve
    tenants = [("mnist", 0.9, 24), ("inception_v3", 0.1, 8)]
    print("case direct multistream", flush=True)
    r = serve.direct_multistream(tenants, iat_us=200.0, num_streams=32, num_jobs=1500, warmup_jobs=100, seed=3)
    counts = [r["per_type"][k]["count"] for k in (0, 1)]
    assert sum(counts) == 1500 and counts[1] > 80
    assert 0.25e6 <= r["elapsed_us"] <= 0.6e6                         # 1500 arrivals at 5000 per second
    # a request's latency is at least its own kernels' time
    assert r["per_type"][1]["p50"] > 300 and r["per_type"][0]["p50"] > 5
    sat = serve.direct_multistream(tenants, iat_us=0.0, num_streams=32, num_jobs=1500, seed=3)
    assert sat["throughput_rps"] > r["throughput_rps"]

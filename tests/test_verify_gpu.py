"""Every output checked while the device is under load.  The load generator's verify mode (include/paella_serve.h) learns, per
job type and seeded input, what the idle server answers and compares every completion of the loaded run with it byte for byte;
here those idle answers are held against the CPU oracle, so request number 17 000 of a saturated run is pinned to the oracle through
two links: bit-identical to the idle answer, idle answer within the fp32 tolerance of the oracle.  Launch packing, grouped
launches with per-problem notifier counts, the staging helper thread, zero-copy I/O and instance recycling only meet on the
loaded server."""
import os

import numpy as np
import pytest

from oracle import models as om

pytestmark = pytest.mark.gpu

ATOL, RTOL = 1e-4, 1e-3
_counter = [0]


def server_name(tag):
    _counter[0] += 1
    return "gv%d_%s_%d" % (os.getpid(), tag, _counter[0])


# (zoo model, adapter, proportion, pooled instances), mean inter-arrival time (0 = saturation), requests
MIXES = {
    "two_tenants": ([("mnist", "tvm_mnist", 0.9, 48), ("inception_v3", "tvm_inception_v3", 0.1, 16)], 6000),
    "mobilenet_resnet50": ([("mobilenetv2", "tvm_mobilenet", 0.5, 16), ("resnet50", "tvm_resnet50", 0.5, 16)], 2000),
    "eight_models": ([(m, "tvm_" + m, 0.125, 6) for m in ("densenet121", "googlenet", "squeezenet1_1", "resnet34", "ultraface320",
                                                          "arcfaceresnet100")] + [("mobilenetv2", "tvm_mobilenet", 0.125, 6), ("mnist", "tvm_mnist", 0.125, 6)],
                     2000),
}
VARIANTS = 4


def run_verified(serve, models, srv, types, iat_us, n, seed, warmup=200):
    out_bytes = [models.io_bytes(m)[1] for m, _, _, _ in types]
    r = serve.client_run(srv.name, [(serve.job_path(job), prop, pool) for _, job, prop, pool in types], iat_us, sum(t[3] for t in types), n,
                         warmup_jobs=warmup, seed=seed, verify=VARIANTS, expected_bytes=VARIANTS * sum(out_bytes))
    pools = sum(t[3] for t in types)
    assert r["all"]["count"] == n
    assert r["verified_requests"] == pools - VARIANTS * len(types) + pools + warmup + n, r["verified_requests"]
    return r, out_bytes


def expectations_match_the_oracle(models, types, r, out_bytes, seed, which=(0, VARIANTS - 1)):
    at = 0
    for t, ((model, _, _, _), nbytes) in enumerate(zip(types, out_bytes)):
        desc = models.describe(model)
        in_floats = models.io_bytes(model)[0] // 4
        for v in range(VARIANTS):
            got = r["expected"][at:at + nbytes].view(np.float32)
            at += nbytes
            if v not in which:
                continue
            from paella_amd import serve
            x = serve.verify_input(seed, t, v, in_floats)
            ref = om.run(desc, x, seed=1).reshape(-1)
            err = np.abs(got.astype(np.float64) - ref.astype(np.float64))
            assert np.all(err <= ATOL + RTOL * np.abs(ref)), (model, v, err.max())
    assert at == len(r["expected"])


@pytest.mark.parametrize("mix", sorted(MIXES))
def test_every_completion_at_saturation_is_its_own_models_answer(cuda, mix):
    """full3 on direct dispatch at saturation (every pooled instance in flight), packing, groups, staging helper and zero-copy
    I/O on: not one of the completions differs from what the idle server answered for the same input, and those idle answers
    match the oracle."""
    from paella_amd import models, serve
    os.environ["LLIS_MODEL_SEED"] = "1"
    types, n = MIXES[mix]
    print("case", mix, flush=True)
    with serve.Server(server_name(mix), "full3", num_streams=128, extra_kernels=32) as srv:
        r, out_bytes = run_verified(serve, models, srv, types, 0.0, n, seed=3)
    assert r["mismatches"] == 0
    expectations_match_the_oracle(models, types, r, out_bytes, seed=3)


@pytest.mark.parametrize("sched_name,dispatch", [("fifo2", "direct"), ("fifo", "hip"), ("fifo", "direct"), ("full3", "hip")])
def test_every_completion_is_checked_under_the_other_schedulers_and_launch_paths(cuda, sched_name, dispatch):
    """The two-tenant mix under open-loop Poisson arrivals near its knee through fifo2 (packed direct dispatch), fifo (whole
    requests on HIP streams, and whole requests on ordered direct-dispatch queues with the upload as a kernel) and full3 on HIP
    launches."""
    from paella_amd import models, serve
    os.environ["LLIS_MODEL_SEED"] = "1"
    os.environ["PAELLA_DISPATCH"] = dispatch
    types = [("mnist", "tvm_mnist", 0.9, 32), ("inception_v3", "tvm_inception_v3", 0.1, 8)]
    rate = {"fifo2": 30000.0, "fifo": 6000.0, "full3": 12000.0}[sched_name]
    print("case", sched_name, dispatch, flush=True)
    try:
        with serve.Server(server_name(sched_name), sched_name, num_streams=64, extra_kernels=32) as srv:
            r, out_bytes = run_verified(serve, models, srv, types, 1e6 / rate, 3000, seed=5)
    finally:
        os.environ.pop("PAELLA_DISPATCH", None)
    assert r["mismatches"] == 0
    expectations_match_the_oracle(models, types, r, out_bytes, seed=5, which=(1,))


def test_two_job_types_of_one_client_have_request_pools_of_their_own(cuda):
    """Two registrations from one loop used to name their shared-memory pools after the same stack address (the reference's
    naming, src/client/job_ref.cpp:24), so both types' request slots aliased: ResNet-18 twice, with different inputs per type,
    must each get their own answers."""
    from paella_amd import models, serve
    os.environ["LLIS_MODEL_SEED"] = "1"
    types = [("resnet18", "tvm_resnet18", 0.5, 8), ("resnet18", "tvm_resnet18", 0.5, 8)]
    with serve.Server(server_name("pools"), "full3", num_streams=32, extra_kernels=16) as srv:
        r, out_bytes = run_verified(serve, models, srv, types, 0.0, 800, seed=9, warmup=50)
    assert r["mismatches"] == 0
    e = r["expected"].view(np.float32).reshape(2, VARIANTS, -1)
    assert not np.array_equal(e[0, 0], e[1, 0])  # different inputs per type, so different answers
    expectations_match_the_oracle(models, types, r, out_bytes, seed=9, which=(0,))

"""End to end on the GPU, through the real path: client library -> shared-memory rings -> server thread ->
scheduler -> instrumented HIP kernels -> notification ring -> completion.  Everything runs inside this
process (threads), because a process that has touched the GPU must not spawn the server binaries."""
import ctypes
import os

import numpy as np
import pytest

from oracle import models as om
from oracle import sched

pytestmark = pytest.mark.gpu

ATOL, RTOL = 1e-4, 1e-3
_counter = [0]


def server_name(tag):
    _counter[0] += 1
    return "gt%d_%s_%d" % (os.getpid(), tag, _counter[0])


def device_budget():
    from paella_amd import _abi
    caps = _abi.DeviceCaps()
    _abi.check(_abi.hip().llis_hip_get_device_caps(ctypes.byref(caps)))
    n = caps.num_cus
    # register lanes and wave slots in the hardware's units: 4 SIMDs x 512 registers x 64 lanes, 4 x 8 waves of 64
    return (n * 4 * 512 * 64, n * caps.lds_bytes_per_cu, n * 4 * 8 * 64, n * 32)


def close(got, ref):
    err = np.abs(got.astype(np.float64) - ref.astype(np.float64))
    assert np.all(err <= ATOL + RTOL * np.abs(ref)), err.max()


@pytest.mark.parametrize("sched_name", ["fifo", "fifo2", "full3"])
@pytest.mark.parametrize("model,job", [("mnist", "tvm_mnist"), ("resnet18", "tvm_resnet18")])
def test_request_output_through_the_server_matches_oracle(cuda, sched_name, model, job):
    from paella_amd import models, serve
    os.environ["LLIS_MODEL_SEED"] = "1"
    desc = models.describe(model)
    x = om.make_input(desc, 21, "uniform" if model == "mnist" else "normal")
    ref = om.run(desc, x, seed=1)
    print("case", sched_name, model, flush=True)
    with serve.Server(server_name(sched_name), sched_name, num_streams=8) as srv:
        out, lat = serve.client_single(srv.name, serve.job_path(job), x, ref.size, n=5)
    close(out, ref)


@pytest.mark.parametrize("dispatch", ["hip", "direct"])
def test_resident_input_mode_and_both_dispatch_paths_match_oracle(cuda, dispatch):
    """Measurement mode (input uploaded once per instance, no host-to-device stage) and the HIP-launch fallback of
    the model adapters must give the same answers as the default path."""
    from paella_amd import models, serve
    os.environ["LLIS_MODEL_SEED"] = "1"
    desc = models.describe("resnet18")
    x = om.make_input(desc, 5, "normal")
    ref = om.run(desc, x, seed=1)
    old = {k: os.environ.get(k) for k in ("PAELLA_INPUT_RESIDENT", "PAELLA_DISPATCH")}
    os.environ["PAELLA_INPUT_RESIDENT"] = "1"
    os.environ["PAELLA_DISPATCH"] = dispatch
    try:
        with serve.Server(server_name("res" + dispatch), "full3", num_streams=8) as srv:
            out, lat = serve.client_single(srv.name, serve.job_path("tvm_resnet18"), x, ref.size, n=4)
    finally:
        for k, v in old.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v
    close(out, ref)


@pytest.mark.parametrize("sched_name,helper", [("full3", "0"), ("full3", "1"), ("fifo2", "1"), ("fifo", "1")])
def test_input_staging_on_and_off_the_serving_thread(cuda, sched_name, helper):
    """The host-side copy of a request's input into the pinned staging buffer: on the serving thread (PAELLA_STAGE_THREAD=0,
    and always under fifo, which issues every stage at once) or as a copy stage of its own that the operator library's helper
    thread finishes and reports.  Requests in a burst (the helper is awake) and one at a time (it sleeps in between and the
    adapter copies by itself) must both give the oracle's result for their own input."""
    import time
    from paella_amd import models, serve
    os.environ["LLIS_MODEL_SEED"] = "1"
    desc = models.describe("resnet18")
    xs = [om.make_input(desc, 40 + i, "normal") for i in range(2)]
    refs = [om.run(desc, x, seed=1) for x in xs]
    old = os.environ.get("PAELLA_STAGE_THREAD")
    os.environ["PAELLA_STAGE_THREAD"] = helper
    try:
        with serve.Server(server_name("stage" + helper), sched_name, num_streams=8) as srv:
            burst, _ = serve.client_single(srv.name, serve.job_path("tvm_resnet18"), xs[0], refs[0].size, n=6)
            time.sleep(0.01)  # the helper has gone to sleep
            lone, _ = serve.client_single(srv.name, serve.job_path("tvm_resnet18"), xs[1], refs[1].size, n=1)
            load = serve.client_run(srv.name, [(serve.job_path("tvm_resnet18"), 1.0, 8)], 0.0, 8, 64)
    finally:
        if old is None:
            os.environ.pop("PAELLA_STAGE_THREAD", None)
        else:
            os.environ["PAELLA_STAGE_THREAD"] = old
    close(burst, refs[0])
    close(lone, refs[1])
    assert load["all"]["count"] == 64


@pytest.mark.parametrize("mem_marker", [True, False])
def test_both_copy_completion_paths_on_the_gpu(cuda, mem_marker):
    from paella_amd import serve
    x = np.arange(32000, dtype=np.float32)
    with serve.Server(server_name("mem"), "full3", num_streams=4, mem_marker=mem_marker) as srv:
        out, lat = serve.client_single(srv.name, serve.job_path("vec_add_coroutine"), x, 32000, n=4)
    np.testing.assert_array_equal(out, 10 * x)


def test_vec_add_at_the_reference_batch_size_sends_13_plus_13_messages_per_kernel(cuda):
    """--noti_batch 16 (the reference's constant, reference include/llis/job/finished_block_notifier.h:118): each of
    vec_add's ten 200-workgroup kernels reports 12 x 16 + 8 started and 12 x 16 + 8 finished workgroups in 13 + 13
    messages (reference finished_block_notifier.h:27-43, jobs/vec_add_coroutine/vec_add_coroutine.cu:115-141)."""
    from paella_amd import serve
    x = np.arange(32000, dtype=np.float32)
    with serve.Server(server_name("b16"), "full3", num_streams=4, event_log=True, noti_batch=16) as srv:
        out, lat = serve.client_single(srv.name, serve.job_path("vec_add_coroutine"), x, 32000, n=2)
    np.testing.assert_array_equal(out, 10 * x)
    ev = sched.parse_log(srv.event_log())
    for kind in (1, 0):
        nums = [e[3] for e in ev if e[0] == "B" and e[2] == kind]
        assert len(nums) == 2 * 10 * 13
        assert sorted(nums) == sorted(2 * 10 * ([16] * 12 + [8]))
    with serve.Server(server_name("b64"), "full3", num_streams=4, event_log=True) as srv:
        serve.client_single(srv.name, serve.job_path("vec_add_coroutine"), x, 32000, n=1)
    nums = [e[3] for e in sched.parse_log(srv.event_log()) if e[0] == "B" and e[2] == 0]
    assert sorted(nums) == sorted(10 * ([64] * 3 + [8]))


@pytest.mark.parametrize("starts", ["0", "1"])
def test_over_budget_kernels_report_starts_only_on_request(cuda, starts):
    """ResNet-18 under full3 with several requests in flight: kernels admitted beyond the occupancy budget report their
    workgroup starts only with PAELLA_UNFIT_STARTS=1 (the credit then returns at full residency, otherwise at the kernel's
    end: reference src/server/scheduler_full3.cpp:123-144 and :196-204); the answers are the same either way."""
    from paella_amd import models, serve
    os.environ["LLIS_MODEL_SEED"] = "1"
    desc = models.describe("resnet18")
    x = om.make_input(desc, 3, "normal")
    ref = om.run(desc, x, seed=1)
    old = os.environ.get("PAELLA_UNFIT_STARTS")
    os.environ["PAELLA_UNFIT_STARTS"] = starts
    try:
        with serve.Server(server_name("starts" + starts), "full3", num_streams=64, extra_kernels=16, event_log=True) as srv:
            jobs = [(serve.job_path("tvm_resnet18"), 1.0, 12)]
            r = serve.client_run(srv.name, jobs, 0.0, 12, 300, warmup_jobs=50)
            out, _ = serve.client_single(srv.name, serve.job_path("tvm_resnet18"), x, ref.size, n=2)
    finally:
        if old is None:
            os.environ.pop("PAELLA_UNFIT_STARTS", None)
        else:
            os.environ["PAELLA_UNFIT_STARTS"] = old
    close(out, ref)
    assert r["all"]["count"] == 300
    ev = sched.parse_log(srv.event_log())
    unfit_dispatches = sum(1 for e in ev if e[0] == "D" and e[6] == 1)
    start_messages = sum(1 for e in ev if e[0] == "B" and e[2] == 1)
    assert unfit_dispatches > 0, "twelve requests in flight must over-subscribe the budget"
    assert (start_messages > 0) == (starts == "1")


def test_plain_job_with_raw_hooks(cuda):
    from paella_amd import serve
    with serve.Server(server_name("hello"), "full3", num_streams=4, event_log=True) as srv:
        serve.client_single(srv.name, serve.job_path("helloworld"), np.zeros(5, np.uint8), 0, n=3)
    ev = sched.parse_log(srv.event_log())
    # stage i launches i workgroups, each sending its own start and end message
    starts = sum(e[3] for e in ev if e[0] == "B" and e[2] == 1)
    ends = sum(e[3] for e in ev if e[0] == "B" and e[2] == 0)
    assert starts == ends == 3 * (1 + 2 + 3 + 4 + 5)


DUMMY_STAGES = {"dummy_short": 10, "dummy_long": 50, "dummy_10": 10, "dummy_11": 11, "dummy_20": 20, "dummy_21": 21}


@pytest.mark.parametrize("job,sched_name", [("dummy_short", "fifo"), ("dummy_short", "fifo2"), ("dummy_short", "full3"),
                                            ("dummy_long", "fifo"), ("dummy_long", "fifo2"), ("dummy_long", "full3"),
                                            ("dummy_11", "full3"), ("dummy_20", "full3"), ("dummy_10", "fifo2"), ("dummy_21", "fifo")])
def test_dummy_job_event_log_is_bit_exact_closed_form(cuda, job, sched_name):
    """One dummy job alone, three requests back to back: per stage exactly one dispatch, one start message and
    one end message with num=5; stream, notifier and job id come from LIFO pools; the wake-up is sent when the
    last stage is dispatched (fifo: when the work up to the pre-notify stage has finished).  Stage counts follow
    reference jobs/dummy_long/dummy_long.cu:29-78 (50) and jobs/dummy_{10,11,20,21}/dummy.cu; the 50-stage form is the
    one that would show a job id, stream or notifier that does not return to its pool."""
    from paella_amd import serve
    streams, stages = 6, DUMMY_STAGES[job]
    with serve.Server(server_name("dummy"), sched_name, num_streams=streams, event_log=True) as srv:
        serve.client_single(srv.name, serve.job_path(job), np.zeros(5, np.uint8), 0, n=3)
    ev = [e for e in sched.parse_log(srv.event_log()) if e[0] != "L"]
    top = streams - 1
    expect = []
    base = ev[0][3]  # arrival counter of this process when the server started
    for req in range(3):
        expect.append(("J", 0, 0, base + req, 0))
        if sched_name == "fifo":
            expect += [("D", 0, s, top, top, 0, 0) for s in range(stages)]
            for s in range(stages):
                expect += [("B", 0, 1, 5), ("B", 0, 0, 5)]
            expect += [("S", 0), ("E", 0)]
        else:
            for s in range(stages):
                expect.append(("D", 0, s, top, top, 0, 0))
                if s == stages - 1:
                    expect.append(("S", 0))
                expect += [("B", 0, 1, 5), ("B", 0, 0, 5)]
            expect.append(("E", 0))
    assert ev == expect


@pytest.mark.parametrize("sched_name", ["fifo", "fifo2", "full3"])
def test_concurrent_dummy_jobs_replay_exactly(cuda, sched_name):
    """Several dummy jobs of two types in flight: the order in which the GPU posts messages is not determined,
    but given the observed inputs every decision of the server must equal the oracle's."""
    from paella_amd import serve
    streams = 8
    with serve.Server(server_name("mix"), sched_name, num_streams=streams, event_log=True) as srv:
        r = serve.client_run(srv.name, [(serve.job_path("dummy_10"), 0.6, 3), (serve.job_path("dummy_21"), 0.4, 2)], 3000.0, 5, 24, seed=3)
    assert r["all"]["count"] == 24
    events = sched.parse_log(srv.event_log())
    types = [sched.dummy_stages(10), sched.dummy_stages(21)]
    expected, actual = sched.replay(sched_name, types, streams, events, budget=device_budget())
    assert expected == actual
    assert sum(1 for e in actual if e[0] == "E") == 24 + 5  # plus one warm-up run per pooled instance


def test_per_workgroup_timing_reaches_the_profiler(cuda, tmp_path):
    """--measure_block_time: every workgroup of every kernel reports its entry and exit clock (24 bits, 10 ns units)
    through the second ring; with block-exec-time recording on, the saved file has one line per workgroup."""
    from paella_amd import serve
    prof = str(tmp_path / "bt")
    n = 6
    with serve.Server(server_name("bt"), "full3", num_streams=8, measure_block_time=True) as srv:
        serve.client_run(srv.name, [(serve.job_path("dummy_short"), 0.5, 2), (serve.job_path("tvm_mnist"), 0.5, 2)], 0.0, 2, n, profile_prefix=prof)
    pairs = [tuple(int(v) for v in l.split()) for l in open(prof + "_block_exec_times.txt")]
    assert pairs and all(0 <= s < (1 << 24) and 0 <= e < (1 << 24) for s, e in pairs)
    dur = [((e - s) & 0xFFFFFF) * 10e-3 for s, e in pairs]  # microseconds
    assert min(dur) >= 0 and max(dur) < 1e5
    # dummy_short: 10 stages of 5 workgroups, about 15 ms of spinning in all -> its workgroups take > 100 us each,
    # the small CNN's take a few microseconds: both kinds must be present
    assert sum(d > 100 for d in dur) >= 5 and sum(d < 50 for d in dur) >= 5
    kinfo = [l.split() for l in open(prof + "_kernel_info.txt")]
    assert len(pairs) == sum(int(k[2]) for k in kinfo)  # one sample pair per workgroup of every recorded kernel
    # ... and the recording covers whole jobs: the server applies the switches when nothing is in flight, so neither the last
    # kernel of a warm-up run (its client is woken at dispatch) leaks in nor the last kernels of the measured requests drop out:
    # three dummy_short requests of ten kernels and three small-CNN requests (one stage each) in this seed's draw
    assert sorted(int(k[2]) for k in kinfo) == [3] * 3 + [5] * 30


def test_mixed_model_load_then_outputs_still_correct(cuda):
    """Small CNN : ResNet-18 = 9 : 1 Poisson load under full3, then a checked request of each model on the same
    server (the instances and their buffers were recycled by the load)."""
    from paella_amd import models, serve
    os.environ["LLIS_MODEL_SEED"] = "1"
    with serve.Server(server_name("mixed"), "full3", num_streams=32) as srv:
        r = serve.client_run(srv.name, [(serve.job_path("tvm_mnist"), 0.9, 16), (serve.job_path("tvm_resnet18"), 0.1, 8)], 200.0, 24, 1500,
                             warmup_jobs=100, seed=1)
        assert r["all"]["count"] == 1500 and r["per_type"][0]["count"] > r["per_type"][1]["count"] > 50
        for model, job in [("mnist", "tvm_mnist"), ("resnet18", "tvm_resnet18")]:
            desc = models.describe(model)
            x = om.make_input(desc, 33, "uniform" if model == "mnist" else "normal")
            out, _ = serve.client_single(srv.name, serve.job_path(job), x, models.io_bytes(model)[1] // 4, n=2)
            close(out, om.run(desc, x, seed=1))


@pytest.mark.parametrize("model,job", [("mnist", "tvm_mnist"), ("resnet18", "tvm_resnet18")])
def test_reference_stage_sequence_still_serves_when_the_shortcuts_are_switched_off(cuda, model, job):
    """PAELLA_ZERO_COPY_BYTES=0 and PAELLA_GROUP_THREADS=0: every request goes host-to-device copy -> one stage per kernel
    -> device-to-host copy (pre-notify), the reference's stage sequence; same results."""
    from paella_amd import models, serve
    os.environ["LLIS_MODEL_SEED"] = "1"
    os.environ["PAELLA_ZERO_COPY_BYTES"] = "0"
    os.environ["PAELLA_GROUP_THREADS"] = "0"
    try:
        desc = models.describe(model)
        x = om.make_input(desc, 23, "uniform" if model == "mnist" else "normal")
        with serve.Server(server_name("copies"), "full3", num_streams=8) as srv:
            out, _ = serve.client_single(srv.name, serve.job_path(job), x, models.io_bytes(model)[1] // 4, n=3)
        close(out, om.run(desc, x, seed=1))
    finally:
        del os.environ["PAELLA_ZERO_COPY_BYTES"]
        del os.environ["PAELLA_GROUP_THREADS"]


MIXES = {
    # small CNN : Inception-v3 = 9 : 1
    "two_tenants": ([("mnist", "tvm_mnist", 0.9), ("inception_v3", "tvm_inception_v3", 0.1)], 400.0, 600),
    # MobileNetV2 + ResNet-50 at equal rates
    "mobilenet_resnet50": ([("mobilenetv2", "tvm_mobilenet", 0.5), ("resnet50", "tvm_resnet50", 0.5)], 600.0, 400),
    # eight models, uniform
    "eight_models": ([(m, "tvm_" + m, 0.125) for m in ("densenet121", "googlenet", "squeezenet1_1", "resnet34", "ultraface320",
                                                       "arcfaceresnet100")] + [("mobilenetv2", "tvm_mobilenet", 0.125), ("mnist", "tvm_mnist", 0.125)],
                     1500.0, 400),
}


@pytest.mark.parametrize("mix", sorted(MIXES))
def test_benchmark_mixes_serve_and_every_model_still_answers_correctly(cuda, mix):
    """The multi-model configurations of the benchmark under open-loop Poisson arrivals and full3: every request
    completes, every model gets its share, and afterwards one checked request per model on the same server."""
    from paella_amd import models, serve
    os.environ["LLIS_MODEL_SEED"] = "1"
    types, iat_us, n = MIXES[mix]
    with serve.Server(server_name(mix), "full3", num_streams=64, extra_kernels=16) as srv:
        r = serve.client_run(srv.name, [(serve.job_path(job), prop, 4) for _, job, prop in types], iat_us, 16, n, warmup_jobs=4 * len(types), seed=1)
        assert r["all"]["count"] == n
        counts = [r["per_type"][i]["count"] for i in range(len(types))]
        assert sum(counts) == n and min(counts) > 0.4 * n * min(p for _, _, p in types), counts
        for model, job, _ in types:
            desc = models.describe(model)
            x = om.make_input(desc, 41, "uniform" if model == "mnist" else "normal")
            print("case", mix, model, flush=True)
            out, _ = serve.client_single(srv.name, serve.job_path(job), x, models.io_bytes(model)[1] // 4, n=1)
            close(out, om.run(desc, x, seed=1))


def test_stream_order_independence_of_results(cuda):
    """Stages of one request issued on different streams, each only after the previous stage's end message was
    read from the ring, give the same bits as the single-stream forward: the end hook's ordering is sufficient."""
    from paella_amd import _abi, models
    lib, hip = _abi.ops(), _abi.hip()
    name = "resnet18"
    desc = models.describe(name)
    x = om.make_input(desc, 5)
    ex = models.Exec(name, seed=1)
    ring = ctypes.c_void_p()
    _abi.check(lib.paella_ring_create(65536, 4, ctypes.byref(ring)))
    streams = []
    for _ in range(4):
        s = ctypes.c_void_p()
        _abi.check(hip.llis_hip_stream_create(ctypes.byref(s)))
        streams.append(s)
    try:
        ex.set_input(x)
        ex.forward()
        ref = ex.get_output()
        b = lib.paella_ring_batch_size()
        for rep in range(20):
            ex.set_input(x)
            for i in range(ex.num_stages):
                grid = ex.stage_dims(i).grid
                ex.launch_stage(i, streams[(i + rep) % 4], job_id=i, notifier=ctypes.c_void_p(lib.paella_ring_notifier(ring, (i + rep) % 4)))
                want = 2 * ((grid + b - 1) // b)
                assert lib.paella_ring_drain(ring, None, want, 20.0) == want
            # the last end message has been read: the output must be complete without any stream synchronisation
            np.testing.assert_array_equal(ex.get_output(), ref)
    finally:
        for s in streams:
            hip.llis_hip_stream_synchronize(s)
            hip.llis_hip_stream_destroy(s)
        lib.paella_ring_destroy(ring)
        ex.close()


def device_topology():
    from paella_amd import _abi
    caps = _abi.DeviceCaps()
    _abi.check(_abi.hip().llis_hip_get_device_caps(ctypes.byref(caps)))
    return (caps.num_cus, 8 if caps.num_cus % 8 == 0 else 1, caps.vgprs_per_cu, caps.lds_bytes_per_cu, caps.max_threads_per_cu, caps.max_blocks_per_cu)


def test_per_cu_placement_on_the_device_replays_and_fills_the_mis_alloc_record(cuda, tmp_path):
    """--placement per_cu under full3 with a raw-hook job (dummy_raw: kernels of 64, 300 and 24 workgroups whose every
    message names the compute unit it ran on) next to an aggregated-hook job (dummy_10): the event log -- with the compute
    units the hardware reported -- replays through the oracle's per-compute-unit model decision for decision, one R record
    per raw-hook kernel, and the profiler's kernel_block_mis_alloc file holds the same figures for the measured phase."""
    from paella_amd import serve
    streams, n = 8, 12
    prof = str(tmp_path / "pc")
    with serve.Server(server_name("percu"), "full3", num_streams=streams, event_log=True, placement="per_cu") as srv:
        r = serve.client_run(srv.name, [(serve.job_path("dummy_raw"), 0.6, 3), (serve.job_path("dummy_10"), 0.4, 2)], 2000.0, 4, n, seed=5,
                             profile_prefix=prof)
    assert r["all"]["count"] == n
    events = sched.parse_log(srv.event_log())
    topo = device_topology()
    expected, actual = sched.replay("full3", [sched.DUMMY_RAW, sched.dummy_stages(10)], streams, events, per_cu=topo)
    assert expected == actual, next((i, a, b) for i, (a, b) in enumerate(zip(expected + [None], actual + [None])) if a != b)
    recon = [e for e in events if e[0] == "R"]
    raw_jobs = sum(1 for e in events if e[0] == "J" and e[2] == 0)
    assert len(recon) == 3 * raw_jobs and raw_jobs >= 3 + 2            # warm-up runs of the three pooled instances and some of the n
    cus = [e[4] for e in events if e[0] == "B" and len(e) > 4]
    assert len(cus) == 2 * (64 + 300 + 24) * raw_jobs and max(cus) < topo[0]
    rows = [tuple(int(v) for v in l.split()) for l in open(prof + "_kernel_block_mis_alloc.txt")]
    assert rows, "kernel_block_mis_alloc must not be empty under per_cu placement with a raw-hook job"
    assert all(total in (64, 300, 24) and wrong <= total and wrong_cus <= min(wrong, topo[0]) for total, wrong, wrong_cus in rows)
    # the file covers the measured phase: its rows are the tail of the log's R records
    assert [(w, c) for _, w, c in rows] == [(e[2], e[3]) for e in recon][-len(rows):]
    # how good the prediction is on this part: the XCD is right by construction, the compute unit inside it often is not
    by_grid = {}
    for total, wrong, _ in rows:
        by_grid.setdefault(total, []).append(wrong / total)
    print("mispredicted share of workgroups by grid size:", {k: round(sum(v) / len(v), 3) for k, v in sorted(by_grid.items())})


def test_per_cu_placement_serves_models_with_correct_outputs(cuda):
    """The aggregated-hook path under per_cu placement (charged and released where predicted): ResNet-18 and the small CNN
    under load with every output checked."""
    from paella_amd import serve
    os.environ["LLIS_MODEL_SEED"] = "1"
    with serve.Server(server_name("percu_models"), "full3", num_streams=32, extra_kernels=8, placement="per_cu") as srv:
        r = serve.client_run(srv.name, [(serve.job_path("tvm_mnist"), 0.8, 16), (serve.job_path("tvm_resnet18"), 0.2, 8)], 0.0, 24, 1500,
                             warmup_jobs=100, seed=1, verify=2)
    assert r["all"]["count"] == 1500 and r["mismatches"] == 0 and r["verified_requests"] >= 1500

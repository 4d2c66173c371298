"""The shipped binaries (llis_server, llis_app_client, llis_app_single_latency) and the in-process serve ABI,
end to end over the real shared-memory rings and sockets, with the scripted device standing in for the GPU."""
import ctypes
import json
import os
import subprocess
import time

import pytest

from _fake import BIN, FAKE_LIB, ensure_built, fake_env, fake_job


@pytest.fixture(scope="module", autouse=True)
def built():
    ensure_built()


def start_server(name, sched, streams=64, **env):
    p = subprocess.Popen([os.path.join(BIN, "llis_server"), "--name", name, "--sched", sched, "--num_streams", str(streams)],
                         env=fake_env(**env), stderr=subprocess.PIPE, text=True)
    for _ in range(200):
        if os.path.exists("/dev/shm/llis:channel:c2s:" + name):
            return p
        time.sleep(0.01)
    p.kill()
    raise AssertionError("server did not come up: " + p.stderr.read())


@pytest.mark.parametrize("sched", ["fifo", "fifo2", "full3"])
def test_load_generator_against_server_process(tmp_path, sched):
    name = "pt%d%s" % (os.getpid(), sched)
    srv = start_server(name, sched, FAKE_HIP_OP_US="20")
    prefix = str(tmp_path / "run")
    out = subprocess.run([os.path.join(BIN, "llis_app_client"), "--server_name", name, "--iat", "300", "--dist", "exp", "--concurrency", "48",
                          "--num_jobs", "600", "--start_record_num", "100", "--seed", "1", "--prefix", prefix, "--no_pin",
                          fake_job("fake_short"), "0.7", "30", fake_job("fake_mem3"), "0.3", "30"],
                         env=fake_env(), capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stderr
    stats = json.loads(out.stdout.strip().splitlines()[-1])
    assert stats["num_jobs"] == 600 and stats["throughput_rps"] > 100
    assert sum(stats["per_type_count"]) == 500  # 100 unrecorded
    assert srv.wait(timeout=30) == 0           # EXIT_CMD ends the server cleanly
    # stats row: x,num_jobs,elapsed then 7 numbers overall and per type (reference app/client.cpp:479-495)
    row = open(prefix + ".txt").read().strip().split(",")
    assert row[0] == "300" and row[1] == "600" and len(row) == 3 + 7 * 3
    assert len(open(prefix + "_raw.txt").read().split()) == 500
    assert not [f for f in os.listdir("/dev/shm") if name in f and "channel" in f]


def test_profiler_files_have_the_reference_line_formats(tmp_path):
    """--profile: the client switches every recording on around the measured phase and asks the server to save.
    Line formats follow reference src/server/profiler.cpp:76-131."""
    name = "ptprof%d" % os.getpid()
    srv = start_server(name, "full3", FAKE_HIP_OP_US="20")
    prof = str(tmp_path / "prof")
    out = subprocess.run([os.path.join(BIN, "llis_app_client"), "--server_name", name, "--iat", "200", "--dist", "exp", "--concurrency", "16",
                          "--num_jobs", "60", "--seed", "1", "--prefix", str(tmp_path / "run"), "--no_pin", "--profile", prof,
                          fake_job("fake_short"), "0.5", "8", fake_job("fake_mem3"), "0.5", "8"],
                         env=fake_env(), capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stderr
    assert srv.wait(timeout=30) == 0
    for suffix in ("kernel_info", "block_exec_times", "kernel_block_mis_alloc", "run_next_times", "job_events", "resource_events"):
        assert os.path.exists("%s_%s.txt" % (prof, suffix)), suffix
    kernel_info = [l.split() for l in open(prof + "_kernel_info.txt")]
    assert kernel_info and all(len(l) == 8 and int(l[0]) <= int(l[1]) for l in kernel_info)
    run_next = [l.split() for l in open(prof + "_run_next_times.txt")]
    assert run_next and all(len(l) == 4 and abs(float(l[1]) - float(l[0]) - float(l[2])) < 1e-2 for l in run_next)
    jobs = [l.split() for l in open(prof + "_job_events.txt")]
    assert len(jobs) == 60
    kernels_finished = 0
    for l in jobs:  # pairs "event time"; a job starts with JOB_SUBMITTED (0) and ends with JOB_FINISHED (6), times non-decreasing
        ev, t = [int(x) for x in l[0::2]], [float(x) for x in l[1::2]]
        assert ev[0] == 0 and ev[-1] == 6 and t == sorted(t)
        kernels_finished += ev.count(5)
    # the switches are applied when nothing is in flight, so the recordings cover the same whole jobs: one kernel-info line per
    # KERNEL_FINISHED event (a job that wakes its client when its last stage is dispatched is still recorded to its end)
    assert kernels_finished == len(kernel_info)
    res = [l.split() for l in open(prof + "_resource_events.txt")]
    assert res and all(len(l) == 8 and l[2] in ("0", "1", "2") for l in res)
    acquired = sum(int(l[4]) for l in res if l[2] == "0")
    released = sum(int(l[4]) for l in res if l[2] == "1")
    assert acquired == released > 0   # every workgroup that was admitted has been given back
    assert open(prof + "_block_exec_times.txt").read() == ""


def test_arrival_process_is_reproducible_for_a_seed():
    """Same seed, same job mix => same sequence of job types (draw order: type first, then inter-arrival)."""
    counts = []
    for rep in range(2):
        name = "ptseed%d_%d" % (os.getpid(), rep)
        srv = start_server(name, "fifo2")
        out = subprocess.run([os.path.join(BIN, "llis_app_client"), "--server_name", name, "--iat", "100", "--dist", "ln", "--ln_sigma", "1.5",
                              "--concurrency", "32", "--num_jobs", "400", "--seed", "7", "--prefix", "/tmp/ptseed", "--no_pin",
                              fake_job("fake_short"), "0.25", "16", fake_job("fake_mem3"), "0.75", "16"],
                             env=fake_env(), capture_output=True, text=True, timeout=120)
        assert out.returncode == 0, out.stderr
        counts.append(json.loads(out.stdout.strip().splitlines()[-1])["per_type_count"])
        srv.wait(timeout=30)
    assert counts[0] == counts[1] and abs(counts[0][0] - 100) < 40


def test_pregenerated_trace_matches_the_live_arrival_process(tmp_path):
    """llis_app_workload_pregen makes the same draws in the same order as the live generator (type first, then the
    gap), writes the reference's file set, and a replay of its trace serves the same request mix."""
    pre = subprocess.run([os.path.join(BIN, "llis_app_workload_pregen"), "--iat", "150", "--ln_sigma", "1.5", "--num_jobs", "300", "--seed", "7",
                          "--pregen_prefix", str(tmp_path / "w"), "0.25", "0.75"], capture_output=True, text=True, timeout=60)
    assert pre.returncode == 0, pre.stderr
    trace_path = pre.stdout.strip()
    assert os.path.basename(trace_path) == "w_iat150_lns1.5_n300_seed7.txt"
    trace = [l.split() for l in open(trace_path)]
    assert len(trace) == 300 and trace[0][1] == "0.000000"
    times = [float(l[1]) for l in trace]
    assert times == sorted(times) and 0.5 * 150 < times[-1] / 299 < 2.0 * 150
    for t in (0, 1):
        own = [l.split() for l in open(trace_path.replace(".txt", "_job%d.txt" % t))]
        assert [l[1] for l in own] == [l[1] for l in trace if l[0] == str(t)] and all(l[0] == "0" for l in own)
    counts = []
    for mode in ("live", "trace"):
        name = "pttr%d_%s" % (os.getpid(), mode)
        srv = start_server(name, "fifo2")
        extra = ["--trace", trace_path] if mode == "trace" else []
        out = subprocess.run([os.path.join(BIN, "llis_app_client"), "--server_name", name, "--iat", "150", "--dist", "ln", "--ln_sigma", "1.5",
                              "--concurrency", "32", "--num_jobs", "300", "--seed", "7", "--prefix", str(tmp_path / mode), "--no_pin"] + extra +
                             [fake_job("fake_short"), "0.25", "16", fake_job("fake_mem3"), "0.75", "16"],
                             env=fake_env(), capture_output=True, text=True, timeout=120)
        assert out.returncode == 0, out.stderr
        assert srv.wait(timeout=30) == 0
        counts.append(json.loads(out.stdout.strip().splitlines()[-1])["per_type_count"])
    assert counts[0] == counts[1] == [sum(l[0] == "0" for l in trace), sum(l[0] == "1" for l in trace)]


def test_unknown_scheduler_is_an_error_not_a_crash():
    out = subprocess.run([os.path.join(BIN, "llis_server"), "--name", "x", "--sched", "nope"], env=fake_env(), capture_output=True, text=True, timeout=30)
    assert out.returncode == 4 and "unknown scheduler" in out.stderr and "full3" in out.stderr


def test_single_latency_client(tmp_path):
    name = "ptsl%d" % os.getpid()
    srv = start_server(name, "full3", 4)
    out = subprocess.run([os.path.join(BIN, "llis_app_single_latency"), name, fake_job("fake_mem3"), "50", "--quiet"], env=fake_env(),
                         capture_output=True, text=True, timeout=60)
    assert out.returncode == 0, out.stderr
    assert json.loads(out.stdout.strip().splitlines()[-1])["num_jobs"] == 50
    assert srv.wait(timeout=30) == 0


@pytest.mark.parametrize("sched_name", ["fifo2", "full3"])
def test_a_copy_stage_completed_from_another_thread(sched_name):
    """fake_self with FAKE_SELF_THREAD=1: the first copy stage is finished by a thread of the job's own, 300 us later, through
    Context::post_mem_completion; the server binaries serve fifty such requests."""
    name = "ptself%d%s" % (os.getpid(), sched_name)
    srv = start_server(name, sched_name, 4, FAKE_SELF_THREAD="1")
    out = subprocess.run([os.path.join(BIN, "llis_app_single_latency"), name, fake_job("fake_self"), "50", "--quiet"], env=fake_env(),
                         capture_output=True, text=True, timeout=60)
    assert out.returncode == 0, out.stderr
    stats = json.loads(out.stdout.strip().splitlines()[-1])
    assert stats["num_jobs"] == 50 and stats["min_us"] >= 300  # every request waited for its thread
    assert srv.wait(timeout=30) == 0


def test_in_process_serve_abi_on_the_scripted_device():
    """paella_server_start / paella_client_run / paella_client_single in a child interpreter that loads the
    scripted device first (same soname as the HIP layer)."""
    code = r'''
import ctypes, os, sys, json
sys.path.insert(0, %r)
os.environ["FAKE_HIP_AUTORUN"] = "1"
ctypes.CDLL(%r, mode=ctypes.RTLD_GLOBAL)
from paella_amd import serve, _abi
_abi._cache["llis_hip"] = True
import numpy as np
with serve.Server("inproc%%d" %% os.getpid(), "full3", num_streams=8, event_log=True) as s:
    r = serve.client_run(s.name, [(%r, 1.0, 6)], 0.0, 6, 200, warmup_jobs=30)
    x = np.full(100, 5, np.uint8)
    out, lat = serve.client_single(s.name, %r, x, 25, n=3)
log = s.event_log()
print(json.dumps({"rps": r["throughput_rps"], "count": r["all"]["count"], "out": out.view(np.uint8)[:4].tolist(), "log_lines": len(log.splitlines())}))
''' % (os.path.dirname(os.path.dirname(os.path.abspath(__file__))), os.path.join(FAKE_LIB, "libllis_hip.so"), fake_job("fake_short"), fake_job("fake_mem3"))
    out = subprocess.run(["python3", "-c", code], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stderr
    res = json.loads(out.stdout.strip().splitlines()[-1])
    assert res["count"] == 200 and res["out"] == [6, 6, 6, 6] and res["log_lines"] > 1000


def test_server_outlives_a_client_killed_mid_run(tmp_path):
    """A client that dies with requests in flight leaves wake-ups nobody will ever read: the server writes them off
    after the peer has refused them for two seconds, and a second client is served as if nothing had happened."""
    name = "ptdead%d" % os.getpid()
    srv = start_server(name, "full3", FAKE_HIP_OP_US="20")
    victim = None
    try:
        args = ["--server_name", name, "--iat", "100", "--dist", "exp", "--concurrency", "32", "--seed", "1", "--no_pin"]
        jobs = [fake_job("fake_short"), "0.7", "16", fake_job("fake_mem3"), "0.3", "16"]
        victim = subprocess.Popen([os.path.join(BIN, "llis_app_client")] + args + ["--num_jobs", "2000000", "--prefix", str(tmp_path / "a")] + jobs,
                                  env=fake_env(LLIS_CLIENT_KEEP_SERVER="1"), stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
        time.sleep(0.5)
        assert victim.poll() is None, "the first client should still be submitting"
        victim.kill()
        victim.wait()
        time.sleep(2.5)  # longer than the server's patience with a peer that refuses every wake-up
        assert srv.poll() is None, srv.stderr.read()
        out = subprocess.run([os.path.join(BIN, "llis_app_client")] + args + ["--num_jobs", "400", "--prefix", str(tmp_path / "b")] + jobs,
                             env=fake_env(), capture_output=True, text=True, timeout=120)
        assert out.returncode == 0, out.stderr
        stats = json.loads(out.stdout.strip().splitlines()[-1])
        assert stats["num_jobs"] == 400 and sum(stats["per_type_count"]) == 400
        assert srv.wait(timeout=30) == 0
    finally:
        for p in (victim, srv):
            if p is not None and p.poll() is None:
                p.kill()
                p.wait()
        for f in os.listdir("/dev/shm"):
            if name in f:
                os.unlink(os.path.join("/dev/shm", f))


def test_verify_mode_checks_every_completion(tmp_path):
    """llis_app_client --verify: seeded inputs per job type, expectations learnt one request at a time during the warm-up,
    every completion of the loaded run compared byte for byte: all equal for jobs that answer input + 1."""
    name = "ptver%d" % os.getpid()
    srv = start_server(name, "full3", FAKE_HIP_OP_US="20")
    out = subprocess.run([os.path.join(BIN, "llis_app_client"), "--server_name", name, "--iat", "200", "--dist", "exp", "--concurrency", "24",
                          "--num_jobs", "500", "--warmup", "60", "--seed", "4", "--prefix", str(tmp_path / "v"), "--no_pin", "--verify", "3",
                          fake_job("fake_mem3"), "0.6", "12", fake_job("fake_self"), "0.4", "12"],
                         env=fake_env(), capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stderr
    stats = json.loads(out.stdout.strip().splitlines()[-1])
    # 24 warm-up runs one at a time, of which 2 x 3 taught the expectations, 24 more all at once, 60 extra warm-up requests, 500 measured
    assert stats["verified_requests"] == 24 - 6 + 24 + 60 + 500 and stats["mismatches"] == 0
    assert srv.wait(timeout=30) == 0


def test_verify_mode_counts_wrong_answers(tmp_path):
    """A job whose every 50th run answers with one wrong byte: verify mode counts exactly those, names the byte and the
    client exits with code 3."""
    name = "ptflaky%d" % os.getpid()
    srv = start_server(name, "fifo2", FAKE_HIP_OP_US="20", FAKE_FLAKY_EVERY="50")
    out = subprocess.run([os.path.join(BIN, "llis_app_client"), "--server_name", name, "--iat", "0", "--dist", "exp", "--concurrency", "8",
                          "--num_jobs", "400", "--seed", "2", "--prefix", str(tmp_path / "f"), "--no_pin", "--verify", "2",
                          fake_job("fake_flaky"), "1.0", "8"],
                         env=fake_env(), capture_output=True, text=True, timeout=120)
    stats = json.loads(out.stdout.strip().splitlines()[-1])
    assert stats["verified_requests"] == 8 - 2 + 8 + 400
    assert stats["mismatches"] == (8 + 8 + 400) // 50 and out.returncode == 3
    assert "first differing byte 7" in out.stderr
    assert srv.wait(timeout=30) == 0


def test_verify_input_restated_in_numpy_is_the_generator_bit_for_bit():
    code = r"""
import ctypes, os, sys
sys.path.insert(0, %r)
ctypes.CDLL(%r, mode=ctypes.RTLD_GLOBAL)
from paella_amd import serve, _abi
_abi._cache["llis_hip"] = True
import numpy as np
for seed, t, v, n in [(1, 0, 0, 1000), (7, 3, 2, 268203), (123456, 15, 7, 5)]:
    want = np.zeros(n, np.float32)
    assert serve.lib().paella_verify_input(seed, t, v, want.ctypes.data, n) == 0
    got = serve.verify_input(seed, t, v, n)
    assert got.dtype == np.float32 and np.array_equal(got.view(np.uint32), want.view(np.uint32)), (seed, t, v)
    assert -1.0 <= got.min() and got.max() < 1.0 and (n < 100 or abs(got.mean()) < 0.1)
a, b = serve.verify_input(1, 0, 0, 64), serve.verify_input(1, 0, 1, 64)
assert not np.array_equal(a, b)
print("ok")
""" % (os.path.dirname(os.path.dirname(os.path.abspath(__file__))), os.path.join(FAKE_LIB, "libllis_hip.so"))
    out = subprocess.run(["python3", "-c", code], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0 and out.stdout.strip().endswith("ok"), out.stderr


@pytest.mark.parametrize("timed", [False, True])
def test_launch_job_with_and_without_its_send_time(tmp_path, timed):
    """Both encodings of LAUNCH_JOB through the shipped binaries: 28 bytes, or 36 with the client's send time behind the message
    type (the reference's PRINT_LAUNCH_JOB_IPC_LATENCY build, src/client/job_instance_ref.cpp:35-38); with the switch on both
    sides the server prints the request ring's mean latency in the reference's words (src/server/server.cpp:121-141)."""
    name = "ptipc%d%d" % (os.getpid(), timed)
    extra = ["--print_ipc_latency"] if timed else []
    p = subprocess.Popen([os.path.join(BIN, "llis_server"), "--name", name, "--sched", "full3", "--num_streams", "16"] + extra,
                         env=fake_env(FAKE_HIP_OP_US="5", LLIS_IPC_LATENCY_SKIP="100"), stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    for _ in range(200):
        if os.path.exists("/dev/shm/llis:channel:c2s:" + name):
            break
        time.sleep(0.01)
    out = subprocess.run([os.path.join(BIN, "llis_app_client"), "--server_name", name, "--iat", "100", "--dist", "exp", "--concurrency", "8",
                          "--num_jobs", "2500", "--seed", "1", "--prefix", str(tmp_path / "i"), "--no_pin", "--verify", "2"] + extra +
                         [fake_job("fake_mem3"), "1.0", "8"], env=fake_env(), capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stderr
    stats = json.loads(out.stdout.strip().splitlines()[-1])
    assert stats["num_jobs"] == 2500 and stats["mismatches"] == 0  # every request decoded: pool slot, offset and handle arrived intact
    sout, serr = p.communicate(timeout=30)
    assert p.returncode == 0, serr
    lines = [l for l in sout.splitlines() if l.startswith("Avg launch job IPC latency: ")]
    if not timed:
        assert not lines
        return
    # 8 + 8 warm-up runs + 2500 requests, the first 100 left out: the running mean at 1000 and 2000, the final figure on exit
    assert len(lines) == 3 and lines[-1].endswith("over 2416 requests"), lines
    for l in lines:
        us = float(l.split()[5])
        assert 0.0 < us < 5000.0, l


def test_a_client_without_the_send_time_is_not_understood_by_a_server_that_expects_it():
    """The two encodings cannot be told apart on the ring (as with two reference builds): the record sizes differ by the
    eight bytes of the time stamp, which is all this asserts about a mismatch."""
    import ctypes as c

    class Plain(c.Structure):
        _pack_ = 1
        _fields_ = [("type", c.c_uint32), ("job_ref", c.c_uint32), ("pool", c.c_int32), ("offset", c.c_size_t), ("handle", c.c_void_p)]

    class Timed(c.Structure):
        _pack_ = 1
        _fields_ = [("type", c.c_uint32), ("sent", c.c_uint64), ("job_ref", c.c_uint32), ("pool", c.c_int32), ("offset", c.c_size_t), ("handle", c.c_void_p)]

    assert c.sizeof(Plain) == 28 and c.sizeof(Timed) == 36 and Timed.sent.offset == 4 and Timed.job_ref.offset == 12

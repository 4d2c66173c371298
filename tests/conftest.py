import json
import os
import subprocess
import sys
import time

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# Filled at session start (before this interpreter has touched the GPU) when GPU tests are selected on a box with a
# device: the result of one llis_server + llis_app_client run as two fresh processes.  tests/test_two_process_gpu.py
# checks it.
TWO_PROCESS = {}


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def _two_process_run():
    """The shipped binaries as two processes on the device, started from a launcher that holds no GPU state (a process
    that has initialised the GPU must not start them): the two-tenant mix, open-loop Poisson arrivals."""
    bin_dir, lib_dir = os.path.join(ROOT, "paella_amd", "bin"), os.path.join(ROOT, "paella_amd", "lib")
    out_dir = os.path.join(ROOT, "gpurun_out")
    os.makedirs(out_dir, exist_ok=True)
    name = "twoproc%d" % os.getpid()
    env = dict(os.environ, LLIS_MODEL_SEED="1")
    res = {"server_name": name}
    with open(os.path.join(out_dir, "two_process_server.err"), "w") as err:
        srv = subprocess.Popen([os.path.join(bin_dir, "llis_server"), "--name", name, "--sched", "full3", "--num_streams", "64", "--extra_kernels", "16"],
                               env=env, stdout=subprocess.DEVNULL, stderr=err)
        try:
            deadline = time.time() + 90
            while not os.path.exists("/dev/shm/llis:channel:c2s:" + name):
                if srv.poll() is not None or time.time() > deadline:
                    res["error"] = "server did not come up (exit code %s)" % srv.poll()
                    return res
                time.sleep(0.05)
            prefix = os.path.join(out_dir, "two_process")
            for suffix in (".txt", "_raw.txt", "_timeline.txt"):  # the client appends, as the reference's does: one session, one row
                if os.path.exists(prefix + suffix):
                    os.remove(prefix + suffix)
            cmd = [os.path.join(bin_dir, "llis_app_client"), "--server_name", name, "--iat", "100", "--dist", "exp", "--concurrency", "56",
                   "--num_jobs", "6000", "--start_record_num", "500", "--seed", "1", "--prefix", prefix,
                   os.path.join(lib_dir, "libjob_tvm_mnist.so"), "0.9", "48", os.path.join(lib_dir, "libjob_tvm_inception_v3.so"), "0.1", "8"]
            res["client_cmd"] = " ".join(os.path.relpath(c, ROOT) if c.startswith(ROOT) else c for c in cmd)
            out = subprocess.run(cmd, env=env, capture_output=True, text=True, timeout=180)
            res["client_rc"], res["client_stderr"] = out.returncode, out.stderr[-2000:]
            if out.returncode == 0:
                res["stats"] = json.loads(out.stdout.strip().splitlines()[-1])
                res["csv_row"] = open(prefix + ".txt").read().strip()
            try:
                res["server_rc"] = srv.wait(timeout=60)  # the client's EXIT_CMD ends it
            except subprocess.TimeoutExpired:
                res["server_rc"] = "still running after the client left"
        except Exception as ex:  # reported by the test, not raised during collection
            res["error"] = repr(ex)
        finally:
            if srv.poll() is None:
                srv.kill()
                srv.wait()
    with open(os.path.join(out_dir, "two_process.json"), "w") as f:
        json.dump(res, f, indent=1)
    return res


def pytest_sessionstart(session):
    expr = session.config.getoption("markexpr", "") or ""
    if "gpu" in expr and "not gpu" not in expr and os.path.exists("/dev/kfd") and not session.config.getoption("collectonly", False):
        TWO_PROCESS.update(_two_process_run())


@pytest.fixture(scope="session")
def cuda():
    import torch

    if not torch.cuda.is_available():
        pytest.fail("this test is marked gpu and needs a GPU; there is no CPU fallback")
    torch.cuda.set_device(0)
    return torch.device("cuda:0")

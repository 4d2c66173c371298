"""Helpers for the CPU tests that drive the real server code on the scripted test device."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
FAKE_DIR = os.path.join(ROOT, "tests", "fake_device")
FAKE_LIB = os.path.join(FAKE_DIR, "lib")
BIN = os.path.join(ROOT, "paella_amd", "bin")
LIB = os.path.join(ROOT, "paella_amd", "lib")


def ensure_built():
    if not os.path.exists(os.path.join(LIB, "libllis_server.so")):
        subprocess.check_call(["make", "-s", "-j8", "-C", os.path.join(ROOT, "paella_amd", "csrc")])
    subprocess.check_call(["make", "-s", "-C", FAKE_DIR])


def fake_job(name):
    return os.path.join(FAKE_LIB, "libjob_%s.so" % name)


def run_harness(script, timeout=60):
    """Runs tests/fake_device/lib/sched_harness on a scenario; returns (replies, event log text)."""
    ensure_built()
    # The script steps the device itself; whatever else set in this interpreter's environment (the in-process
    # serving tests ask the scripted device for a background thread) must not reach the harness.
    env = {k: v for k, v in os.environ.items() if not k.startswith("FAKE_HIP_")}
    out = subprocess.run([os.path.join(FAKE_LIB, "sched_harness")], input=script, capture_output=True, text=True, timeout=timeout, env=env)
    assert out.returncode == 0, "sched_harness exit %d\n--- stderr\n%s\n--- stdout\n%s" % (out.returncode, out.stderr, out.stdout)
    head, _, log = out.stdout.partition("--- event log\n")
    return head.splitlines(), log


def fake_env(**extra):
    env = dict(os.environ)
    env["LD_LIBRARY_PATH"] = FAKE_LIB + ":" + env.get("LD_LIBRARY_PATH", "")
    env["FAKE_HIP_AUTORUN"] = "1"
    env.update(extra)
    return env

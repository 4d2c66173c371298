"""Per-compute-unit placement model (llis::server::GpuResources) on the CPU: closed forms of the XCD rule, conservation,
the case the pooled budget cannot see, and a randomised lock-step run against the Python restatement."""
import os
import random
import subprocess

import pytest

from oracle import sched

HERE = os.path.dirname(os.path.abspath(__file__))
BIN = os.path.join(HERE, "fake_device", "lib", "gpu_resources_check")


@pytest.fixture(scope="module")
def binary():
    subprocess.run(["make", "-s", "-C", os.path.join(HERE, "fake_device")], check=True, capture_output=True)
    return BIN


def run(binary, script):
    out = subprocess.run([binary], input="\n".join(script) + "\n", capture_output=True, text=True, timeout=60)
    assert out.returncode == 0, out.stderr
    return out.stdout.strip().splitlines()


def pred_of(line):
    assert line.startswith("pred")
    return {int(a): int(b) for a, b in (t.split(":") for t in line.split()[1:])}


def test_workgroups_go_round_the_xcds_and_spread_inside_them(binary):
    # 256 CUs in 8 XCDs; 19 workgroups: XCDs 0..2 get 3, the others 2; the next dispatch starts on XCD 3
    out = run(binary, ["new 256 8 131072 163840 2048 32", "job 1 19 256 0 32", "run 1", "job 2 8 256 0 32", "run 2"])
    p1, p2 = pred_of(out[0]), pred_of(out[1])
    per_xcd = [sum(n for cu, n in p1.items() if cu // 32 == x) for x in range(8)]
    assert per_xcd == [3, 3, 3, 2, 2, 2, 2, 2] and max(p1.values()) == 1          # never two on one CU while others are empty
    assert sorted(cu // 32 for cu in p2) == list(range(8)) and not set(p1) & set(p2)  # fresh CUs, one per XCD


def test_exact_prediction_costs_nothing_and_everything_is_returned(binary):
    script = ["new 64 8 65536 65536 2048 16", "job 1 40 512 4096 24", "run 1", "dump"]
    out = run(binary, script)
    pred = pred_of(out[0])
    starts = [cu for cu, n in pred.items() for _ in range(n)]
    script = script[:3] + ["start 1 %d" % cu for cu in starts] + ["reconcile 1"] + ["finish 1 %d" % cu for cu in starts] + ["dump"]
    out = run(binary, script)
    assert out[1] == "wrong 0 0"
    fields = out[2].split()
    assert fields[1] == "full=0" and fields[3] == "total_threads=%d" % (64 * 2048) and set(fields[5:]) == {"2048/16"}


def test_a_kernel_can_fit_the_pooled_budget_and_still_not_fit_its_xcd(binary):
    # 2 XCDs of one CU with 4 slots.  Job 1 is predicted 2 + 2 but all four workgroups report CU 0.
    out = run(binary, ["new 2 2 1000000 1000000 1024 4", "job 1 4 64 0 8", "run 1"] + ["start 1 0"] * 4 + ["reconcile 1", "dump", "job 2 4 64 0 8", "fits 2",
                       "job 3 2 64 0 8", "fits 3", "job 4 1 64 0 8", "fits 4"])
    assert pred_of(out[0]) == {0: 2, 1: 2} and out[1] == "wrong 2 1"
    assert out[2].split()[5:] == ["768/0", "1024/4"]      # CU 0 is full, CU 1 untouched: 4 slots free in total
    # 4 more workgroups fit the pooled count (4 free slots) but XCD 0 would get two of them; so would 2.
    # One workgroup lands on the XCD the next dispatch starts on -- XCD 0 again (4 dispatched so far) -- which is full.
    assert out[3:] == ["fits 0", "fits 0", "fits 0"]


@pytest.mark.parametrize("seed", range(6))
def test_lock_step_with_the_python_restatement(binary, seed):
    rng = random.Random(seed)
    cus, xcds = rng.choice([(16, 4), (32, 8), (256, 8), (12, 1)])
    caps = (rng.choice([65536, 131072]), rng.choice([65536, 163840]), 2048, rng.choice([8, 32]))
    model = sched.GpuResources(cus, xcds, *caps)
    script, expect = ["new %d %d %d %d %d %d" % ((cus, xcds) + caps)], []
    live = {}   # job -> (stage, predicted, started list, to_finish list)
    for step in range(300):
        action = rng.random()
        if action < 0.35 or not live:
            j = step
            st = sched.Stage(False, rng.randint(1, 3 * cus), rng.choice([64, 256, 512, 1024]), rng.choice([0, 4096, 65536]), rng.choice([16, 64, 128]))
            script += ["job %d %d %d %d %d" % (j, st.blocks, st.threads, st.smem, st.regs), "fits %d" % j]
            expect.append("fits %d" % int(model.fits(st)))
            script.append("run %d" % j)
            pred = model.choose(st)
            expect.append("pred" + "".join(" %d:%d" % (c, pred[c]) for c in sorted(pred)))
            live[j] = [st, pred, [], st.blocks]
        else:
            j = rng.choice(sorted(live))
            st, pred, started, pending = live[j]
            if pending > 0:
                # most workgroups land where predicted, some elsewhere in the same XCD, a few anywhere
                for _ in range(min(pending, rng.randint(1, 40))):
                    guess = [c for c, n in pred.items() if n > 0]
                    r = rng.random()
                    cu = rng.choice(guess) if guess and r < 0.7 else rng.randrange(cus)
                    script.append("start %d %d" % (j, cu))
                    model.observe_start(st, pred, cu)
                    started.append(cu)
                    live[j][3] -= 1
                if live[j][3] == 0:
                    script.append("reconcile %d" % j)
                    expect.append("wrong %d %d" % model.reconcile(st, pred))
            else:
                for _ in range(min(len(started), rng.randint(1, 60))):
                    cu = started.pop()
                    script.append("finish %d %d" % (j, cu))
                    model.cus[cu].release(st, 1)
                if not started:
                    del live[j]
        if step % 25 == 24:
            script.append("dump")
            expect.append("state full=%d all_full=%d total_threads=%d :%s" % (
                model.num_full(), int(model.num_full() >= cus), sum(r.free[2] for r in model.cus),
                "".join(" %d/%d" % (r.free[2], r.free[3]) for r in model.cus)))
    assert run(binary, script) == expect

"""The real Server + schedulers + rings (C++), driven message by message on the scripted device, against the
scheduler oracle: every decision (job ids, dispatch order, stream and notifier handed out, wake-ups,
completions) must be reproduced bit for bit from the inputs recorded in the same log."""
import pytest

from _fake import fake_job, run_harness
from oracle import sched

TYPES = ["fake_mem3", "fake_short", "fake_long", "fake_big"]


def scenario(policy, streams, body, extra="", types=TYPES):
    script = "sched %s streams %d %s\nclient\n" % (policy, streams, extra)
    for t in types:
        script += "job %s\n" % fake_job(t)
    return script + body


def check(policy, streams, body, extra="", types=TYPES, **kw):
    replies, log = run_harness(scenario(policy, streams, body, extra, types))
    events = sched.parse_log(log)
    assert any(e[0] == "E" for e in events)
    expected, actual = sched.replay(policy, [sched.FAKE_TYPES[t] for t in types], streams, events, **kw)
    assert expected == actual, next((i, a, b) for i, (a, b) in enumerate(zip(expected + [None], actual + [None])) if a != b)
    return replies, events


MIXED = "launch 1 0\nlaunch 0 0\nlaunch 1 1\nstep 2\nlaunch 2 0\nlaunch 0 1\nstep 5\nlaunch 1 2\ndrain\n"


@pytest.mark.parametrize("policy", ["fifo", "fifo2", "full3"])
@pytest.mark.parametrize("streams", [1, 2, 8])
def test_policy_matches_oracle_on_a_mixed_scenario(policy, streams):
    replies, events = check(policy, streams, MIXED)
    done = [r for r in replies if r.startswith("done")]
    assert len(done) == 6
    summary = [r for r in replies if r.startswith("wakeups")][0].split()
    assert summary[1] == "6" and summary[3] == "6" and summary[5] == "0"  # every request woke the client once
    hooks = [r for r in replies if r.startswith("hooks")][0].split()
    assert int(hooks[1]) == int(hooks[3]) > 0  # a job library's hook runs once per turn of the serving loop, however often it registered


@pytest.mark.parametrize("mem", ["marker", "hostfunc"])
def test_both_copy_completion_paths(mem):
    check("full3", 2, "launch 0 0\nlaunch 0 1\ndrain\n", extra="mem " + mem)
    check("fifo", 2, "launch 0 0\nlaunch 0 1\ndrain\n", extra="mem " + mem)


def test_request_bytes_travel_through_the_pool_slots():
    """fake_mem3 returns input + 1: checks the (chunk, offset) addressing of the shared-memory pool."""
    replies, _ = run_harness(scenario("full3", 4, "put 0 0 7\nput 0 3 41\nlaunch 0 0\nlaunch 0 3\ndrain\nget 0 0\nget 0 3\n"))
    outs = [r for r in replies if r.startswith("out")]
    assert outs == ["out 8 8 8 8 8 8 8 8", "out 42 42 42 42 42 42 42 42"]
    assert sorted(r for r in replies if r.startswith("done")) == ["done 1000", "done 1003"]


@pytest.mark.parametrize("policy", ["fifo2", "full3"])
def test_a_copy_stage_that_reports_its_own_completion(policy):
    """fake_self: its first copy stage posts its completion itself (Job::set_completes_itself, Context::post_mem_completion):
    the scheduler launches no marker behind it -- the device sees only the two real copies and the kernel -- and goes on to the
    next stage when the message arrives; the bytes staged in that stage come back as input + 1."""
    replies, log = run_harness(scenario(policy, 2, "put 4 0 9\nput 4 1 30\nlaunch 4 0\nlaunch 4 1\ndrain\nget 4 0\nget 4 1\n", types=TYPES + ["fake_self"]))
    assert [r for r in replies if r.startswith("out")] == ["out 10 10 10 10 10 10 10 10", "out 31 31 31 31 31 31 31 31"]
    assert sorted(r for r in replies if r.startswith("done")) == ["done 5000", "done 5001"]
    events = sched.parse_log(log)
    for job in (0, 1):
        mine = [e for e in events if e[0] in ("D", "M") and e[1] == job]
        # dispatch of the self-reporting stage, its completion, the host-to-device copy, its completion, the kernel, the last copy
        assert [e[0] for e in mine[:5]] == ["D", "M", "D", "M", "D"] and [e[5] for e in mine if e[0] == "D"] == [1, 1, 0, 1]


def test_oversubscription_credit_path():
    """fake_big (3000 x 256 x 64 regs) never fits a small budget: it is admitted as an 'unfit' kernel while
    credits last, the credit returns when its start messages are complete (or at its end), and the
    head-of-queue job blocks everything behind it once credits are gone."""
    budget = (2_000_000, 1 << 20, 100_000, 400)
    body = "launch 3 0\nlaunch 3 1\nlaunch 1 0\nlaunch 3 2\nstart 7\nstart 6\nfinish 7\ndrain\n"
    replies, events = check("full3", 8, body, extra="extra 1 budget %d %d %d %d" % budget, budget=budget, extra_kernels=1)
    dispatches = [e for e in events if e[0] == "D"]
    assert dispatches[0][6] == 1, "first big kernel must go out as unfit"
    # with one credit the second big job cannot start until the first is fully resident
    first_start_done = next(i for i, e in enumerate(events) if e[0] == "B" and e[2] == 1)
    assert all(e[1] == 0 for e in events[:first_start_done] if e[0] == "D")


def test_fairness_threshold_changes_the_order():
    body = "".join("launch 1 %d\n" % i for i in range(4)) + "launch 2 0\n" + "drain\n"
    _, fair = check("full3", 1, body, extra="unfair 1", unfair=1.0)
    _, unfair = check("full3", 1, body, extra="unfair 1000000", unfair=1e6)
    order = lambda evs: [e[1:3] for e in evs if e[0] == "D"]
    assert order(fair) != order(unfair)


def test_job_ids_are_reused_most_recent_first():
    _, events = check("fifo2", 4, "launch 1 0\nlaunch 1 1\nlaunch 1 2\ndrain\nlaunch 1 0\nlaunch 1 1\ndrain\n")
    js = [e for e in events if e[0] == "J"]
    assert [j[1] for j in js[:3]] == [0, 1, 2]
    ends = [e[1] for e in events if e[0] == "E"][:3]
    assert [j[1] for j in js[3:]] == [ends[-1], ends[-2]]  # LIFO free list
    assert [j[3] for j in js] == list(range(5))            # unique ids count arrivals


def test_dummy_shape_closed_form_through_the_real_server():
    """One fake_short alone under full3: per stage exactly D, B start 5, B end 5; wake-up at the last dispatch."""
    _, events = check("full3", 3, "launch 1 0\ndrain\n")
    core = [e for e in events if e[0] != "L"]
    expect = [("J", 0, 1, 0, 0)]
    for s in range(10):
        expect.append(("D", 0, s, 2, 2, 0, 0))
        if s == 9:
            expect.append(("S", 0))
        expect += [("B", 0, 1, 5), ("B", 0, 0, 5)]
    expect.append(("E", 0))
    assert core == expect


def test_reference_notification_batch_reaches_the_scheduler_in_sixteens():
    """`batch 16`: the scripted device posts what notifiers created with the reference's batch size post, and the
    scheduler's bookkeeping (pending / running workgroups) follows message by message: fake_big's 3000 workgroups
    arrive as 187 x 16 + 8, twice."""
    budget = (1 << 40, 1 << 40, 1 << 40, 1 << 40)
    replies, events = check("full3", 2, "launch 3 0\ndrain\n", extra="batch 16 budget %d %d %d %d" % budget, budget=budget)
    for kind in (1, 0):
        nums = [e[3] for e in events if e[0] == "B" and e[2] == kind]
        per_stage = [16] * 187 + [8]
        assert len(nums) % 188 == 0 and nums == per_stage * (len(nums) // 188)
    assert [r for r in replies if r.startswith("done")] == ["done 4000"]


# ---- per-compute-unit placement (--placement per_cu)

PER_CU = (256, 8, 131072, 163840, 2048, 32)   # the scripted device's topology: compute units, XCDs, and per compute unit registers, LDS, threads, workgroups
RAW_TYPES = ["fake_mem3", "fake_raw", "fake_big"]
RAW_MIX = "launch 1 0\nlaunch 0 0\nstep 3\nlaunch 1 1\nlaunch 2 0\nstep 4\nlaunch 0 1\nlaunch 1 2\ndrain\n"


@pytest.mark.parametrize("streams", [2, 8])
def test_per_cu_placement_matches_oracle_and_reports_mispredictions(streams):
    """full3 admitting against the per-compute-unit model: jobs with aggregated hooks are charged and released where the
    model predicted them, jobs with un-aggregated hooks (fake_raw: every message names a compute unit, and the scripted
    device scatters workgroups inside an XCD in its own way) are reconciled -- one R record per raw-hook kernel with the
    number of workgroups predicted elsewhere.  Every decision, every R record and the compute units in the log replay
    through the oracle's GpuResources."""
    replies, events = check("full3", streams, RAW_MIX, extra="extra 2 percu %d %d %d %d %d %d" % PER_CU, types=RAW_TYPES, per_cu=PER_CU, extra_kernels=2)
    assert len([r for r in replies if r.startswith("done")]) == 6
    recon = [e for e in events if e[0] == "R"]
    assert len(recon) == 3 * 3                                # three raw-hook kernels in each of three fake_raw requests
    assert any(e[2] > 0 for e in recon) and all(e[2] <= 500 and e[3] <= 256 for e in recon)
    raw_msgs = [e for e in events if e[0] == "B" and len(e) > 4]
    assert len(raw_msgs) == 3 * 2 * (40 + 300 + 500)          # a start and an end message per workgroup, each with its compute unit
    assert any(e[0] == "D" and e[6] == 1 for e in events)     # fake_big (3000 workgroups of 4 waves) never fits: credit path taken


def test_per_cu_model_admits_by_the_share_of_each_xcd():
    """One workgroup per compute unit: an XCD of 32 compute units takes 32.  fake_raw's 40 workgroups (5 per XCD) fit, its
    300 (38 per XCD) do not and go out on credit; with two per compute unit (64 per XCD) they fit, and so do the 500 (63)."""
    tight = (256, 8, 1 << 30, 1 << 30, 1 << 30, 1)
    _, events = check("full3", 4, "launch 1 0\ndrain\n", extra="extra 1 percu %d %d %d %d %d %d" % tight, types=RAW_TYPES, per_cu=tight, extra_kernels=1)
    assert [e[6] for e in events if e[0] == "D"] == [0, 1, 0, 1]
    roomy = (256, 8, 1 << 30, 1 << 30, 1 << 30, 2)
    _, events = check("full3", 4, "launch 1 0\ndrain\n", extra="extra 1 percu %d %d %d %d %d %d" % roomy, types=RAW_TYPES, per_cu=roomy, extra_kernels=1)
    assert [e[6] for e in events if e[0] == "D"] == [0, 0, 0, 0]


def test_raw_hook_jobs_under_the_pooled_budget_log_no_compute_units():
    _, events = check("full3", 4, "launch 1 0\nlaunch 0 0\ndrain\n", types=RAW_TYPES)
    assert all(len(e) == 4 for e in events if e[0] == "B") and not any(e[0] == "R" for e in events)

"""Pins the scheduler oracle (oracle/sched.py) with hand-derived logs, closed forms and brute force, so that
replaying a product log through it means something."""
import itertools
import random

from oracle import sched
from oracle.sched import Stage


def kernel(blocks, pre=False, threads=256, regs=32, smem=0):
    return Stage(False, blocks, threads, smem, regs, pre)


def test_dummy_job_closed_form_full3():
    """dummy_short alone: 10 stages, each dispatched on the same (LIFO) stream and notifier, one start and one
    end message of num=5 per stage, client woken at the dispatch of the last stage, then the completion."""
    s = sched.Full3([sched.dummy_stages(10)], num_streams=4)
    s.new_job(0)
    expect = [("J", 0, 0, 0, 0)]
    for stage in range(10):
        expect.append(("D", 0, stage, 3, 3, 0, 0))
        if stage == 9:
            expect.append(("S", 0))
        s.block(0, True, 5)
        s.block(0, False, 5, lambda: 100.0)
    expect.append(("E", 0))
    assert s.out == expect
    # the id returns to the pool and is reused first
    s.new_job(0)
    assert s.out[-1] == ("D", 0, 0, 3, 3, 0, 0) and s.out[-2] == ("J", 0, 0, 1, 0)


def test_fifo_hand_derived_two_jobs_one_stream():
    """Job-by-job on one stream: A (mem, kernel 3 blocks, mem+pre-notify) is issued whole; B waits for the
    stream.  A's wake-up fires when everything up to and including its pre-notify stage finished = its end."""
    a = [Stage(True), kernel(3), Stage(True, pre_notify=True)]
    b = [kernel(2, pre=True)]
    s = sched.Fifo([a, b], num_streams=1)
    s.new_job(0)
    s.new_job(1)
    assert s.out == [("J", 0, 0, 0, 1), ("D", 0, 0, 0, 0, 1, 0), ("D", 0, 1, 0, 0, 0, 0), ("D", 0, 2, 0, 0, 1, 0), ("J", 1, 1, 1, 0)]
    s.mem(0)
    s.block(0, True, 3)
    s.block(0, False, 3)
    assert s.out[5:] == []
    s.mem(0)
    assert s.out[5:] == [("S", 0), ("E", 0), ("D", 1, 0, 0, 0, 0, 0)]
    s.block(1, False, 2)
    assert s.out[8:] == [("S", 1), ("E", 1)]


def test_fifo2_arrival_order_and_lifo_pools():
    """Kernel-by-kernel FIFO: with two streams, two 2-stage jobs alternate; a finished stage's stream goes back
    on top of the pool and is handed to whichever job arrived first among those waiting."""
    t = [kernel(1), kernel(1, pre=True)]
    s = sched.Fifo2([t], num_streams=2)
    s.new_job(0)
    s.new_job(0)
    s.new_job(0)  # no stream left: queued
    assert [e for e in s.out if e[0] == "D"] == [("D", 0, 0, 1, 1, 0, 0), ("D", 1, 0, 0, 0, 0, 0)]
    s.block(1, False, 1)  # job 1's stage ends first; job 2 (unique 2) waits, job 1 (unique 1) re-queues: 1 goes first
    assert s.out[-2:] == [("D", 1, 1, 0, 0, 0, 0), ("S", 1)]
    s.block(0, False, 1)
    assert s.out[-2:] == [("D", 0, 1, 1, 1, 0, 0), ("S", 0)]
    s.block(0, False, 1)
    assert s.out[-2:] == [("E", 0), ("D", 2, 0, 1, 1, 0, 0)]


def test_sm_resources_closed_form():
    """One workgroup of 8 threads, 10 registers, 20 bytes of LDS is charged a whole wave of 64 lanes, 16 registers per
    lane and one 1280-byte LDS granule; the pooling itself is reference src/server/sm_resources.cpp:36-66."""
    r = sched.SmResources(10000, 5000, 256, 4)
    st = kernel(2, threads=8, regs=10, smem=20)
    assert r.fits(st)
    r.acquire(st, 2)
    assert r.free == [10000 - 2 * 64 * 16, 5000 - 2 * 1280, 256 - 2 * 64, 2]
    assert not r.fits(kernel(3, threads=8, regs=10))      # workgroup slots
    assert r.fits(kernel(1, threads=8, regs=10, smem=1280))
    assert not r.fits(kernel(1, threads=8, regs=10, smem=1281))  # two granules, 2440 bytes left
    assert not r.fits(kernel(2, threads=65, regs=10))     # two waves each: 256 lanes, 128 left
    r.release(st, 1)
    assert r.free == [10000 - 64 * 16, 5000 - 1280, 256 - 64, 3]


def test_stage_length_estimator_recurrence():
    t = sched.TypeStats()
    for v in (8.0, 4.0, 10.0):
        t.update_length(0, v)
    assert t.lengths == [((8.0 + 4.0) / 2 + 10.0) / 2]
    t.update_length(1, 3.0)
    t.set_resource(0, 1.0)
    t.set_resource(1, 1.0)
    t.set_resource(1, 5.0)  # resources never change once set
    assert t.remaining_rl(0) == 8.0 + 3.0 and t.remaining_rl(1) == 3.0 and t.remaining_rl(2) == 0.0


def test_srpt_prefers_the_job_with_less_remaining_work():
    """Two types with learned stage lengths; with one stream the queued job with less remaining work goes first."""
    short = [kernel(1), kernel(1, pre=True)]
    long_ = [kernel(1)] * 5 + [kernel(1, pre=True)]
    s = sched.Full3([short, long_], num_streams=1)
    # teach the estimator: run one job of each type alone
    for type_id, n in ((0, 2), (1, 6)):
        s.new_job(type_id)
        for _ in range(n):
            s.block(0, True, 1)
            s.block(0, False, 1, lambda: 10.0)
    s.out.clear()
    s.new_job(1)   # long: takes the stream
    s.new_job(1)   # another long queued, remaining 60
    s.new_job(0)   # short queued, remaining 20 -> higher priority (-20 > -60)
    s.block(0, True, 1)
    s.block(0, False, 1, lambda: 10.0)
    # candidates now: job 0 (long, 50 left), job 1 (long, 60), job 2 (short, 20)
    d = [e for e in s.out if e[0] == "D"]
    assert d[0][1] == 0 and d[1][1] == 2


class NaiveQueue:
    """Independent model of the fairness rule, written from the policy's description: every pop credits each
    active type 1/n and charges the served type 1; a type joins (or re-joins after running dry) at the baseline."""

    def __init__(self, threshold):
        self.credit = 0.0          # total credit handed out per type so far
        self.th0 = threshold
        self.items = []            # (priority, order, type)
        self.join = {}             # type -> (credit at join, charges since, order)
        self.order = 0

    def push(self, pri, typ):
        if typ not in self.join:
            self.join[typ] = [self.credit, 0, self.order]
            self.order += 1
        self.items.append((pri, self.order, typ))
        self.order += 1

    def pop(self):
        # deficit of a type = credits since it joined - charges; fairness when the largest reaches the threshold
        def deficit(t):
            return (self.credit - self.join[t][0]) - self.join[t][1]
        best_t = min(self.join, key=lambda t: (-deficit(t), self.join[t][2]))
        pool = [i for i in self.items if i[2] == best_t] if deficit(best_t) >= self.th0 else self.items
        item = min(pool, key=lambda i: (-i[0], i[1]))
        self.items.remove(item)
        self.credit += 1.0 / len(self.join)
        t = item[2]
        if any(i[2] == t for i in self.items):
            self.join[t][1] += 1
            self.join[t][2] = self.order
            self.order += 1
        else:
            del self.join[t]
        return item


def test_jobqueue_against_naive_model_on_small_cases():
    """Random short push/pop programs with 2 types, so that every fair share (1 or 1/2), priority and threshold
    is exact in binary and the two formulations cannot differ by rounding."""
    rng = random.Random(5)
    for trial in range(2000):
        th = rng.choice([0.5, 1.0, 2.0, 1e6])
        q, naive = sched.JobQueue(th), NaiveQueue(th)
        live = 0
        for step in range(14):
            if live == 0 or (live < 6 and rng.random() < 0.6):
                pri, typ = -float(rng.randrange(0, 4)), rng.randrange(0, 2)
                job = sched.Job(typ, [])
                job.priority = pri
                job.tag = (pri, typ)
                q.push(job)
                naive.push(pri, typ)
                live += 1
            else:
                got = q.pop()
                want = naive.pop()
                assert got.tag == (want[0], want[2]), (trial, step, th)
                live -= 1


def test_jobqueue_fairness_triggers_and_is_fifo_among_equals():
    q = sched.JobQueue(1.0)
    jobs = []
    for i, (pri, typ) in enumerate([(-1.0, 0), (-1.0, 0), (-1.0, 0), (-5.0, 1)]):
        j = sched.Job(typ, [])
        j.priority = pri
        j.tag = i
        q.push(j)
        jobs.append(j)
    # first pops follow priority with FIFO ties; type 1's deficit grows by 1/2 per pop: 0 -> .5 -> 1.0 >= threshold(1 - .5 - .5 = 0)...
    order = [q.pop().tag for _ in range(4)]
    assert order[0] == 0
    assert 3 in order[:3], "the starved type must be served before type 0 is exhausted"


def test_occupancy_closed_form_in_gfx950_units():
    """Hand-derived: 4 SIMDs, 512 registers per lane and at most 8 waves per SIMD, registers in steps of 8, LDS in steps of
    1280 bytes out of 160 KiB, at most 32 workgroups per compute unit."""
    cases = [
        ((512, 64, 32768), 4),    # 8 waves x 64 regs: 8 waves/SIMD -> 32 waves / 8; LDS 163840 // 33280 = 4
        ((512, 64, 40960), 4),    # LDS exactly 32 granules: 163840 // 40960 = 4
        ((512, 64, 40961), 3),    # one byte more takes another granule: 163840 // 42240 = 3
        ((256, 128, 0), 4),       # 4 waves/SIMD -> 16 waves / 4
        ((256, 129, 0), 3),       # 129 -> 136 regs: 3 waves/SIMD -> 12 / 4
        ((256, 32, 0), 8),        # register-unbound: 32 waves / 4
        ((10, 16, 0), 32),        # a 10-thread workgroup still takes a whole wave; capped by the 32 workgroup slots
        ((1024, 128, 0), 1),      # 16 waves of 128 regs fill the unit
        ((1024, 129, 0), 0),      # and do not fit with one register more
        ((64, 72, 0), 28),        # 512 // 72 = 7 waves/SIMD
        ((128, 512, 0), 2),       # one wave per SIMD
    ]
    for (threads, regs, lds), want in cases:
        assert sched.blocks_per_cu(threads, regs, lds) == want, (threads, regs, lds)
    # the pooled budget charges the same units: a 10-thread workgroup with 20 registers and 100 bytes of LDS
    assert sched.wg_charge(sched.Stage(False, 3, 10, 100, 20)) == (64 * 24, 1280, 64)
    r = sched.SmResources(64 * 24 * 3, 1280 * 3, 64 * 3, 3)
    assert r.fits(sched.Stage(False, 3, 10, 100, 20)) and not r.fits(sched.Stage(False, 3, 10, 100, 25))


def test_per_cu_placement_hand_derived_reconciliation():
    """Two XCDs of two compute units, one workgroup of 64 threads each.  A raw-hook kernel of 4 workgroups: the model sends
    workgroup 0 to XCD 0 (compute unit 0: ties go to the search pointer), 1 to XCD 1 (unit 2), 2 to XCD 0 (unit 1, the pointer
    has moved on), 3 to XCD 1 (unit 3).  The device reports 0, 2, 0, 3: the second report of unit 0 was not predicted, the
    prediction for unit 1 never came true -> one mispredicted workgroup on one compute unit; unit 0 then holds two, unit 1
    none.  A second kernel of 3 workgroups starts on XCD 0 again (4 mod 2) and no longer fits: XCD 0 has one free slot for
    a share of two."""
    topo = (4, 2, 1 << 20, 1 << 20, 64, 4)
    st4 = sched.Stage(False, 4, 64, 0, 16, raw=True)
    g = sched.GpuResources(*topo)
    assert g.fits(st4)
    pred = g.choose(st4)
    assert pred == {0: 1, 2: 1, 1: 1, 3: 1}
    for cu in (0, 2, 0, 3):
        g.observe_start(st4, pred, cu)
    assert g.reconcile(st4, pred) == (1, 1)
    assert [r.free[2] for r in g.cus] == [64 - 128, 64, 0, 0]
    st3 = sched.Stage(False, 3, 64, 0, 16, raw=True)
    assert g.next_xcd == 0 and not g.fits(st3)
    # the whole path through the policy: the same kernel as a one-stage job, messages as above
    f = sched.Full3([[sched.Stage(False, 4, 64, 0, 16, True, raw=True)]], 2, per_cu=topo)
    f.new_job(0)
    for cu in (0, 2, 0, 3):
        f.block(0, True, 1, cu=cu)
    for i, cu in enumerate((0, 2, 0, 3)):
        f.block(0, False, 1, length=lambda: 5.0, cu=cu)
    assert f.out == [("J", 0, 0, 0, 0), ("D", 0, 0, 1, 1, 0, 0), ("S", 0), ("R", 0, 1, 1), ("E", 0)]
    assert all(r.free == [1 << 20, 1 << 20, 64, 4] for r in f.per_cu.cus)   # everything given back

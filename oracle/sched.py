"""Scheduler oracle (TEST INFRASTRUCTURE ONLY): a plain-Python restatement of the three dispatch policies,
used to replay a server's event log and check every decision bit for bit.

Restates (reference paths):
  JobQueue        include/llis/server/scheduler_full3.h:26-208   priority queue + deficit-counter fairness
  full3           src/server/scheduler_full3.cpp:123-459          SRPT priority, occupancy admission, unfit credit
  fifo            src/server/scheduler_fifo.cpp:83-255            job-by-job, block counting, pre-notify
  fifo2           src/server/scheduler_fifo2.cpp:90-257           kernel-by-kernel in arrival order
  SmResources     src/server/sm_resources.cpp:36-66, sm_resources.h:29-31
  stage estimator src/server/registered_job.cpp:112-182           len <- (len + new) / 2, remaining = sum len*res
  Job counters    include/llis/job/job.h:138-191,278-292
Pools of streams, notifiers and job ids are LIFO (scheduler_full3.cpp:206-207,280-287,391-396).

Deliberate deviations shared with the product: a stage whose length is not yet
in the job's snapshot counts as zero remaining work (the reference indexes past the end of the snapshot);
a job without stages is released without touching the id pool.

Log grammar (one event per line), inputs J/B/M/L and decisions D/S/E:
  J id type unique first_is_mem | B id is_start num | M id | L id stage hexfloat
  D id stage stream notifier is_mem unfit | S id | E id
With per-compute-unit placement (Full3(per_cu=...), this build's own: the reference's full3 has only the pooled budget; the
reconciliation restates reference src/server/scheduler_full.cpp:98-121) a B line of a raw-hook stage carries a fourth
value, the compute unit, and the decisions gain  R id mispredicted_workgroups compute_units.
Pinning: hand-derived logs and closed forms in tests/test_sched_oracle.py; the JobQueue is written as a
brute-force search over plain lists, so it doubles as the naive model for the product's tree-based queue.
"""
from dataclasses import dataclass, field
from typing import List, Optional


@dataclass
class Stage:
    is_mem: bool
    blocks: int = 0
    threads: int = 0
    smem: int = 0
    regs: int = 0
    pre_notify: bool = False
    raw: bool = False   # kernel with un-aggregated hooks: one message per workgroup, naming its compute unit


def dummy_stages(n):
    """n kernels of 5 x 256, 32 registers, pre-notify on the last (reference jobs/dummy_long/dummy_long.cu:43-62)."""
    return [Stage(False, 5, 256, 0, 32, i == n - 1) for i in range(n)]


FAKE_TYPES = {
    "fake_short": dummy_stages(10),
    "fake_long": dummy_stages(50),
    "fake_mem3": [Stage(True), Stage(False, 40, 128, 1024, 64), Stage(False, 200, 64, 0, 32), Stage(False, 17, 256, 8192, 128),
                  Stage(True, pre_notify=True)],
    "fake_big": [Stage(False, 3000, 256, 0, 64, i == 2) for i in range(3)],
    "fake_raw": [Stage(False, 40, 256, 0, 32, raw=True), Stage(False, 300, 64, 2048, 64, raw=True), Stage(False, 17, 256, 8192, 128),
                 Stage(False, 500, 256, 0, 32, True, raw=True)],
}
# dummy_raw of the real device (csrc/jobs/dummy_raw.hip)
DUMMY_RAW = [Stage(False, 64, 256, 0, 32, raw=True), Stage(False, 300, 256, 0, 32, raw=True), Stage(False, 24, 256, 0, 32, True, raw=True)]


@dataclass
class Job:
    type_id: int
    stages: List[Stage]
    id: int = -1
    unique: int = -1
    cur_stage: int = -1
    running: bool = False
    unfit: bool = False
    started: bool = False
    pending_blocks: int = 0
    running_blocks: int = 0
    priority: float = 0.0
    cur_rl: float = 0.0
    lengths: List[float] = field(default_factory=list)
    resources: List[float] = field(default_factory=list)
    stream: int = -1
    notifier: int = -1
    cur: Optional[Stage] = None
    predicted: dict = field(default_factory=dict)   # per-compute-unit placement: {cu: workgroups predicted there}

    @property
    def next(self):
        return self.stages[self.cur_stage + 1]

    def has_next(self):
        return self.cur_stage + 1 < len(self.stages)

    def dec_cur_rl(self):
        n = self.cur_stage + 1
        if n < len(self.lengths) and n < len(self.resources):
            self.cur_rl -= self.lengths[n] * self.resources[n]


class TypeStats:
    def __init__(self):
        self.lengths = []
        self.resources = []

    def update_length(self, stage, length):
        if stage < len(self.lengths):
            self.lengths[stage] = (self.lengths[stage] + length) / 2
        else:
            self.lengths.append(length)

    def set_resource(self, stage, res):
        if len(self.resources) <= stage:
            self.resources.append(res)

    def remaining_rl(self, frm):
        total = 0.0
        for i in range(frm, min(len(self.lengths), len(self.resources))):
            total += self.lengths[i] * self.resources[i]
        return total


class JobQueue:
    """Brute-force restatement: plain lists, linear scans."""

    def __init__(self, threshold):
        self.threshold = float(threshold)
        self.new_type_deficit = 0.0
        self.seq = 0
        self.jobs = []       # (priority, seq, job)
        self.types = {}      # type_id -> [deficit, seq] while the type has queued jobs

    def __len__(self):
        return len(self.jobs)

    def push(self, job):
        t = job.type_id
        if t not in self.types:
            self.types[t] = [self.new_type_deficit, self.seq]
            self.seq += 1
        self.jobs.append((job.priority, self.seq, job))
        self.seq += 1

    def _select(self):
        starved = min(self.types.items(), key=lambda kv: (-kv[1][0], kv[1][1]))
        if starved[1][0] >= self.threshold:
            cands = [e for e in self.jobs if e[2].type_id == starved[0]]
        else:
            cands = self.jobs
        return min(cands, key=lambda e: (-e[0], e[1]))

    def top(self):
        return self._select()[2]

    def pop(self):
        entry = self._select()
        self.jobs.remove(entry)
        t = entry[2].type_id
        share = 1.0 / len(self.types)
        self.new_type_deficit -= share
        self.threshold -= share
        if any(e[2].type_id == t for e in self.jobs):
            self.types[t] = [self.types[t][0] - 1.0, self.seq]
            self.seq += 1
        else:
            del self.types[t]
        return entry[2]


WAVE_LANES, VGPR_GRANULE, LDS_GRANULE = 64, 8, 1280  # gfx950 allocation units (include/llis/server/sm_resources.h)
SIMDS_PER_CU, VGPRS_PER_SIMD_LANE, MAX_WAVES_PER_SIMD = 4, 512, 8


def _up(v, g):
    return -(-v // g) * g


def wg_charge(st):
    """(register lanes, LDS bytes, wave-slot threads) one workgroup of the stage takes: whole waves, registers in
    granules of 8 per lane, LDS in granules of 1280 bytes.  The pooling is reference src/server/sm_resources.cpp:36-66;
    the reference charges the declared regs x threads, threads and bytes (the CUDA allocation model)."""
    thr = _up(st.threads, WAVE_LANES)
    return thr * _up(st.regs, VGPR_GRANULE), _up(st.smem, LDS_GRANULE), thr


def blocks_per_cu(threads, regs, smem, lds_per_cu=160 * 1024, max_blocks=32):
    """Workgroups of one shape a gfx950 compute unit holds: the closed form the runtime's occupancy query follows."""
    if threads == 0:
        return 0
    waves_per_wg = _up(threads, WAVE_LANES) // WAVE_LANES
    per_simd = MAX_WAVES_PER_SIMD if regs == 0 else min(MAX_WAVES_PER_SIMD, VGPRS_PER_SIMD_LANE // _up(regs, VGPR_GRANULE))
    n = SIMDS_PER_CU * per_simd // waves_per_wg
    if smem > 0:
        n = min(n, lds_per_cu // _up(smem, LDS_GRANULE))
    return max(min(n, max_blocks), 0)


class SmResources:
    def __init__(self, regs, smem, threads, blocks):
        self.free = [regs, smem, threads, blocks]

    @staticmethod
    def _need(st, n):
        r, s, t = wg_charge(st)
        return [r * n, s * n, t * n, n]

    def fits(self, st):
        return all(f >= need for f, need in zip(self.free, self._need(st, st.blocks)))

    def acquire(self, st, n):
        self.free = [f - x for f, x in zip(self.free, self._need(st, n))]

    def release(self, st, n):
        self.free = [f + x for f, x in zip(self.free, self._need(st, n))]


class GpuResources:
    """Per-compute-unit budget with the XCD-aware placement prediction (restates include/llis/server/gpu_resources.h;
    accounting as reference src/server/gpu_resources.cpp:38-64, reconciliation as reference
    src/server/scheduler_full.cpp:98-121).  A stage is a Stage (regs, smem, threads, blocks).  The placement rule is
    this build's own (the reference's table is for another vendor's part): workgroup i of a dispatch goes to XCD
    (first + i) mod xcds, inside it to the compute unit with the most free threads, searching from a pointer that
    moves past the last choice."""

    def __init__(self, cus, xcds, regs, smem, threads, blocks):
        self.cus = [SmResources(regs, smem, threads, blocks) for _ in range(cus)]
        self.xcds, self.per = xcds, cus // xcds
        self.next_cu = [0] * xcds
        self.next_xcd = 0

    @staticmethod
    def _full(r):
        return any(f <= 0 for f in r.free)

    @staticmethod
    def _room(r, st):
        if GpuResources._full(r):
            return 0
        n = r.free[3]
        regs, smem, thr = wg_charge(st)
        if st.threads > 0:
            if regs > 0:
                n = min(n, r.free[0] // regs)
            n = min(n, r.free[2] // thr)
        if st.smem > 0:
            n = min(n, r.free[1] // smem)
        return max(n, 0)

    def num_full(self):
        return sum(self._full(r) for r in self.cus)

    def fits(self, st):
        for x in range(self.xcds):
            lane = (x - self.next_xcd) % self.xcds
            share = (st.blocks - lane + self.xcds - 1) // self.xcds if st.blocks > lane else 0
            if sum(self._room(r, st) for r in self.cus[x * self.per:(x + 1) * self.per]) < share:
                return False
        return True

    def choose(self, st):
        """Returns {cu: workgroups predicted there}; acquires them."""
        predicted = {}
        for i in range(st.blocks):
            x = (self.next_xcd + i) % self.xcds
            best, best_room = None, None
            for k in range(self.per):
                c = x * self.per + (self.next_cu[x] + k) % self.per
                room = -1 if self._full(self.cus[c]) else self.cus[c].free[2]
                if best is None or room > best_room:
                    best, best_room = c, room
            self.next_cu[x] = (best % self.per + 1) % self.per
            self.cus[best].acquire(st, 1)
            predicted[best] = predicted.get(best, 0) + 1
        self.next_xcd = (self.next_xcd + st.blocks) % self.xcds
        return predicted

    def observe_start(self, st, predicted, cu):
        if predicted.get(cu, 0) > 0:
            predicted[cu] -= 1
        else:
            self.cus[cu].acquire(st, 1)

    def reconcile(self, st, predicted):
        wrong = sum(predicted.values())
        wrong_cus = sum(1 for n in predicted.values() if n > 0)
        for cu, n in predicted.items():
            if n > 0:
                self.cus[cu].release(st, n)
        predicted.clear()
        return wrong, wrong_cus


# Budget the scripted test device reports: 256 CUs x {131072 regs, 160 KiB LDS, 2048 threads, 32 workgroups}.
FAKE_BUDGET = (256 * 131072, 256 * 163840, 256 * 2048, 256 * 32)


class Base:
    def __init__(self, types, num_streams):
        self.types = types                       # list of stage lists, indexed by type id
        self.stats = [TypeStats() for _ in types]
        self.streams = list(range(num_streams))  # LIFO
        self.notifiers = list(range(num_streams))
        self.free_ids = []
        self.jobs = {}
        self.next_unique = 0
        self.out = []

    def adopt(self, type_id):
        job = Job(type_id, self.types[type_id])
        job.id = self.free_ids.pop() if self.free_ids else len(self.jobs_ever)
        job.unique = self.next_unique
        self.next_unique += 1
        return job

    @property
    def jobs_ever(self):
        return self._ever

    def _register(self, job):
        if job.id == len(self._ever):
            self._ever.append(job)
        else:
            self._ever[job.id] = job

    def emit(self, *ev):
        self.out.append(tuple(ev))

    def set_running(self, job, stream):
        job.running = True
        job.stream = stream
        job.cur = job.next
        job.running_blocks = job.pending_blocks = job.cur.blocks
        job.cur_stage += 1


class Full3(Base):
    def __init__(self, types, num_streams, extra_kernels=2, unfair=1e6, budget=FAKE_BUDGET, per_cu=None):
        super().__init__(types, num_streams)
        self._ever = []
        self.queue = JobQueue(unfair)
        self.res = SmResources(*budget)
        self.per_cu = GpuResources(*per_cu) if per_cu else None   # (cus, xcds, regs, smem, threads, blocks per compute unit)
        self.extra = extra_kernels
        self.outstanding = 0

    def _take_priority(self, job):
        p = -job.cur_rl
        job.dec_cur_rl()
        return p

    def new_job(self, type_id):
        job = self.adopt(type_id)
        self._register(job)
        self.emit("J", job.id, type_id, job.unique, int(job.next.is_mem))
        st = self.stats[type_id]
        st.set_resource(0, 1.0)
        job.cur_rl = st.remaining_rl(0)
        job.lengths = list(st.lengths)
        job.resources = list(st.resources)
        job.priority = self._take_priority(job)
        self.queue.push(job)
        self.schedule()

    def _release_predicted(self, job, num):
        for cu in sorted(job.predicted):
            n = min(job.predicted[cu], num)
            if n:
                self.per_cu.cus[cu].release(job.cur, n)
                job.predicted[cu] -= n
                num -= n

    def block(self, job_id, is_start, num, length=None, cu=None):
        job = self._ever[job_id]
        names_cu = self.per_cu is not None and job.cur.raw
        if is_start:
            if names_cu:
                self.per_cu.observe_start(job.cur, job.predicted, cu)
            job.pending_blocks -= num
            if job.pending_blocks == 0 and names_cu:
                self.emit("R", job.id, *self.per_cu.reconcile(job.cur, job.predicted))
            if job.pending_blocks == 0 and job.unfit:
                job.unfit = False
                self.outstanding -= 1
                self.schedule()
            return
        job.running_blocks -= num
        over = job.running_blocks == 0
        if over:
            job.running = False
            self._requeue_or_finish(job, length())
            if job.unfit:
                job.unfit = False
                self.outstanding -= 1
            self.streams.append(job.stream)
            self.notifiers.append(job.notifier)
        if self.per_cu is None:
            self.res.release(job.cur, num)
        elif names_cu:
            self.per_cu.cus[cu].release(job.cur, 1)
        else:
            self._release_predicted(job, num)
        if over and not job.has_next():
            self.free_ids.append(job.id)
        self.schedule()

    def mem(self, job_id, length):
        job = self._ever[job_id]
        job.running = False
        self._requeue_or_finish(job, length())
        self.streams.append(job.stream)
        if not job.has_next():
            self.free_ids.append(job.id)
        self.schedule()

    def _requeue_or_finish(self, job, length):
        st = self.stats[job.type_id]
        st.update_length(job.cur_stage, length)
        if job.has_next():
            st.set_resource(job.cur_stage + 1, 1.0)
            job.priority = self._take_priority(job)
            self.queue.push(job)
        else:
            self.emit("E", job.id)

    def schedule(self):
        while self.streams and len(self.queue):
            job = self.queue.top()
            st = job.next
            unfit = False
            if not st.is_mem and not (self.per_cu.fits(st) if self.per_cu else self.res.fits(st)):
                if self.outstanding >= self.extra:
                    break
                self.outstanding += 1
                job.unfit = unfit = True
            popped = self.queue.pop()
            assert popped is job
            job.started = True
            self.set_running(job, self.streams.pop())
            notifier = -1
            if not st.is_mem:
                notifier = job.notifier = self.notifiers.pop()
                if self.per_cu:
                    job.predicted = self.per_cu.choose(job.cur)
                else:
                    self.res.acquire(job.cur, job.cur.blocks)
            self.emit("D", job.id, job.cur_stage, job.stream, notifier, int(st.is_mem), int(unfit))
            if st.pre_notify:
                self.emit("S", job.id)


class Fifo(Base):
    def __init__(self, types, num_streams, **_):
        super().__init__(types, num_streams)
        self._ever = []
        self.queue = []
        self.progress = {}

    def new_job(self, type_id):
        job = self.adopt(type_id)
        self._register(job)
        self.progress[job.id] = [0, 0, False]  # remaining, pre_notify_blocks, sent
        self.emit("J", job.id, type_id, job.unique, int(job.next.is_mem))
        self.queue.append(job)
        self.schedule()

    def _account(self, job, num):
        pr = self.progress[job.id]
        pr[0] -= num
        pr[1] -= num
        if pr[1] <= 0 and not pr[2]:
            self.emit("S", job.id)
            pr[2] = True
        if pr[0] == 0:
            self.emit("E", job.id)
            self.streams.append(job.stream)
            self.notifiers.append(job.notifier)
            self.free_ids.append(job.id)
        self.schedule()

    def block(self, job_id, is_start, num, length=None):
        if not is_start:
            self._account(self._ever[job_id], num)

    def mem(self, job_id, length=None):
        self._account(self._ever[job_id], 1)

    def schedule(self):
        while self.streams and self.queue:
            job = self.queue.pop(0)
            job.stream = self.streams.pop()
            job.notifier = self.notifiers.pop()
            pr = self.progress[job.id]
            saw = False
            for i, st in enumerate(job.stages):
                units = 1 if st.is_mem else st.blocks
                pr[0] += units
                if not saw:
                    pr[1] += units
                    saw = st.pre_notify
                self.emit("D", job.id, i, job.stream, job.notifier, int(st.is_mem), 0)
            job.cur_stage = len(job.stages) - 1


class Fifo2(Base):
    def __init__(self, types, num_streams, **_):
        super().__init__(types, num_streams)
        self._ever = []
        self.queue = []

    def new_job(self, type_id):
        job = self.adopt(type_id)
        self._register(job)
        self.emit("J", job.id, type_id, job.unique, int(job.next.is_mem))
        self.queue.append(job)
        self.schedule()

    def _stage_done(self, job, was_kernel):
        more = job.has_next()
        if more:
            self.queue.append(job)
        else:
            self.emit("E", job.id)
        self.streams.append(job.stream)
        if was_kernel:
            self.notifiers.append(job.notifier)
        if not more:
            self.free_ids.append(job.id)

    def block(self, job_id, is_start, num, length=None):
        if is_start:
            return
        job = self._ever[job_id]
        job.running_blocks -= num
        if job.running_blocks == 0:
            job.running = False
            self._stage_done(job, True)
        self.schedule()

    def mem(self, job_id, length=None):
        job = self._ever[job_id]
        job.running = False
        self._stage_done(job, False)
        self.schedule()

    def schedule(self):
        while self.streams and self.queue:
            job = min(self.queue, key=lambda j: j.unique)
            self.queue.remove(job)
            st = job.next
            self.set_running(job, self.streams.pop())
            notifier = -1
            if not st.is_mem:
                notifier = job.notifier = self.notifiers.pop()
            self.emit("D", job.id, job.cur_stage, job.stream, notifier, int(st.is_mem), 0)
            if st.pre_notify:
                self.emit("S", job.id)


POLICIES = {"full3": Full3, "fifo": Fifo, "fifo2": Fifo2}


def parse_log(text):
    events = []
    for line in text.splitlines():
        f = line.split()
        if not f or f[0] not in "JBMLDSER":
            continue
        if f[0] == "L":
            events.append(("L", int(f[1]), int(f[2]), float.fromhex(f[3])))
        else:
            events.append((f[0],) + tuple(int(v) for v in f[1:]))
    return events


def replay(policy, types, num_streams, events, **kw):
    """Feeds the log's inputs (J/B/M with the L lengths) to the oracle and returns (expected, actual) decision
    lists including the ids chosen for J, for comparison with ==."""
    sched = POLICIES[policy](types, num_streams, **kw)
    # unique ids count arrivals per PROCESS (a function-local static in Job::set_id), so a server that is not the
    # first in its process starts from a non-zero base: take it from the first admission in the log
    first = next((e for e in events if e[0] == "J"), None)
    if first is not None:
        sched.next_unique = first[3]
    pos = {"i": 0}

    def next_length(job_id, stage):
        # the measured length of the stage that just ended is the next L line of the log
        j = pos["i"] + 1
        while events[j][0] != "L":
            j += 1
        assert events[j][1] == job_id, (events[j], job_id)
        return events[j][3]

    for i, ev in enumerate(events):
        pos["i"] = i
        if ev[0] == "J":
            sched.new_job(ev[2])
        elif ev[0] == "B":
            job = sched.jobs_ever[ev[1]]
            if len(ev) > 4:
                sched.block(ev[1], ev[2] == 1, ev[3], lambda: next_length(ev[1], job.cur_stage), cu=ev[4])
            else:
                sched.block(ev[1], ev[2] == 1, ev[3], lambda: next_length(ev[1], job.cur_stage))
        elif ev[0] == "M":
            job = sched.jobs_ever[ev[1]]
            if policy == "full3":
                sched.mem(ev[1], lambda: next_length(ev[1], job.cur_stage))
            else:
                sched.mem(ev[1])
    actual = [e for e in events if e[0] in "JDSER"]
    return sched.out, actual

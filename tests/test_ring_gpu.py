"""The GPU->host notification ring and the workgroup hooks on a real device.

Closed forms being checked (they follow from the notifier's counter arithmetic): a grid of n workgroups
produces exactly ceil(n/B) start and ceil(n/B) end messages for its job id (B = the library's batch size), whose
`num` fields are B except for one remainder message n mod B, summing to n; the un-aggregated hooks produce n + n messages of
num 1.  Message bit layout: byte0 is_start, byte1 cu id, byte2 num, byte3 ready, bytes4-7 job id.
"""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def decode(bits):
    bits = np.asarray(bits, dtype=np.uint64)
    return {
        "is_start": (bits & np.uint64(0xFF)).astype(int),
        "smid": ((bits >> np.uint64(8)) & np.uint64(0xFF)).astype(int),
        "num": ((bits >> np.uint64(16)) & np.uint64(0xFF)).astype(int),
        "status": ((bits >> np.uint64(24)) & np.uint64(0xFF)).astype(int),
        "job_id": (bits >> np.uint64(32)).astype(np.int64),
    }


@pytest.fixture()
def ring(cuda):
    from paella_amd import _abi
    lib = _abi.ops()
    handle = ctypes.c_void_p()
    _abi.check(lib.paella_ring_create(4096, 4, ctypes.byref(handle)), "paella_ring_create")
    yield lib, handle
    lib.paella_ring_destroy(handle)


REFERENCE_BATCH = 16  # reference include/llis/job/finished_block_notifier.h:118


@pytest.fixture()
def ring16(cuda):
    """Notifiers created with the reference's batch size."""
    from paella_amd import _abi
    lib = _abi.ops()
    handle = ctypes.c_void_p()
    _abi.check(lib.paella_ring_create_batched(4096, 4, REFERENCE_BATCH, ctypes.byref(handle)), "paella_ring_create_batched")
    yield lib, handle
    lib.paella_ring_destroy(handle)


def batch():
    from paella_amd import _abi
    return _abi.ops().paella_ring_batch_size()


def expected_nums(n, b=None):
    b = b or batch()
    return sorted([b] * (n // b) + ([n % b] if n % b else []))


@pytest.mark.parametrize("grid", [(1, 1, 1), (5, 1, 1), (16, 1, 1), (17, 1, 1), (200, 1, 1), (7, 5, 3), (1000, 1, 1)])
def test_aggregated_notifier_message_count_and_layout(ring, grid):
    lib, h = ring
    n = grid[0] * grid[1] * grid[2]
    want = 2 * ((n + batch() - 1) // batch())
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for rep in range(3):  # the counters must self-reset between kernels
        job_id = 1000 + rep
        from paella_amd import _abi
        _abi.check(lib.paella_ring_probe_launch(h, rep % 4, grid[0], grid[1], grid[2], 128, job_id, 0, stream))
        out = np.zeros(want, np.uint64)
        got = lib.paella_ring_drain(h, out.ctypes.data, want, 20.0)
        assert got == want
        torch.cuda.synchronize()
        assert lib.paella_ring_can_read(h) == 0  # nothing extra
        m = decode(out)
        assert np.all(m["job_id"] == job_id) and np.all(m["status"] == 0)
        starts, ends = m["num"][m["is_start"] == 1], m["num"][m["is_start"] == 0]
        assert sorted(starts.tolist()) == expected_nums(n)
        assert sorted(ends.tolist()) == expected_nums(n)
        # every end batch is preceded by at least as many started workgroups
        started = finished = 0
        for s, k in zip(m["is_start"], m["num"]):
            if s:
                started += k
            else:
                finished += k
            assert finished <= started + batch() - 1


@pytest.mark.parametrize("n", [1, 5, 16, 17, 200, 1000])
def test_reference_batch_size_gives_the_reference_message_sequence(ring16, n):
    """At batch 16 a grid of n workgroups sends ceil(n/16) start and ceil(n/16) end messages, `num` = 16 except one
    remainder n mod 16 (reference include/llis/job/finished_block_notifier.h:27-43): 2 + 2 for 17, 13 + 13 for 200
    (12 x 16 + 8), 63 + 63 for 1000 (62 x 16 + 8)."""
    lib, h = ring16
    from paella_amd import _abi
    per_kind = -(-n // REFERENCE_BATCH)
    assert per_kind == {1: 1, 5: 1, 16: 1, 17: 2, 200: 13, 1000: 63}[n]
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for rep in range(2):  # the counters reset themselves
        _abi.check(lib.paella_ring_probe_launch(h, rep, n, 1, 1, 64, 500 + rep, 0, stream))
        out = np.zeros(2 * per_kind, np.uint64)
        assert lib.paella_ring_drain(h, out.ctypes.data, 2 * per_kind, 20.0) == 2 * per_kind
        torch.cuda.synchronize()
        assert lib.paella_ring_can_read(h) == 0
        m = decode(out)
        assert np.all(m["job_id"] == 500 + rep)
        for kind in (1, 0):
            nums = sorted(m["num"][m["is_start"] == kind].tolist())
            assert nums == expected_nums(n, REFERENCE_BATCH) and sum(nums) == n


def test_batch_size_must_be_a_power_of_two_up_to_128(cuda):
    from paella_amd import _abi
    lib = _abi.ops()
    for bad in (0, 3, 48, 256):
        handle = ctypes.c_void_p()
        assert lib.paella_ring_create_batched(4096, 1, bad, ctypes.byref(handle)) == -1 and not handle.value


def test_raw_hooks_one_message_pair_per_workgroup(ring):
    lib, h = ring
    from paella_amd import _abi
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    n = 37
    _abi.check(lib.paella_ring_probe_launch(h, 0, n, 1, 1, 64, 77, 1, stream))
    out = np.zeros(2 * n, np.uint64)
    assert lib.paella_ring_drain(h, out.ctypes.data, 2 * n, 20.0) == 2 * n
    m = decode(out)
    assert np.all(m["job_id"] == 77) and np.all(m["num"] == 1)
    assert (m["is_start"] == 1).sum() == n and (m["is_start"] == 0).sum() == n


def test_ring_wraps_without_losing_messages(ring):
    """4096-slot ring, > 3 laps of traffic, drained between kernels."""
    lib, h = ring
    from paella_amd import _abi
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    total = 0
    for i in range(14):
        n = 500
        _abi.check(lib.paella_ring_probe_launch(h, 0, n, 1, 1, 64, i, 1, stream))
        out = np.zeros(2 * n, np.uint64)
        assert lib.paella_ring_drain(h, out.ctypes.data, 2 * n, 20.0) == 2 * n
        assert np.all(decode(out)["job_id"] == i)
        total += 2 * n
    assert total > 3 * 4096


def test_ops_kernels_carry_the_hooks(ring, cuda):
    """A conv launched with a notifier reports exactly its planned grid."""
    lib, h = ring
    from paella_amd import ops
    rng = np.random.default_rng(5)
    wt = rng.standard_normal((64, 32, 3, 3)).astype(np.float32) * 0.05
    conv = ops.Conv2d(wt, None, pad=1, in_hw=(28, 28))
    x = torch.tensor(rng.standard_normal((1, 32, 28, 28)).astype(np.float32), device=cuda)
    y0 = conv(x)
    y1 = conv(x, job_id=9, notifier=ctypes.c_void_p(lib.paella_ring_notifier(h, 1)))
    n = conv.plan.dims.grid
    want = 2 * ((n + batch() - 1) // batch())
    out = np.zeros(want, np.uint64)
    assert lib.paella_ring_drain(h, out.ctypes.data, want, 20.0) == want
    m = decode(out)
    assert np.all(m["job_id"] == 9) and m["num"][m["is_start"] == 0].sum() == n
    torch.cuda.synchronize()
    assert torch.equal(y0, y1)


def test_notify_latency_probes_report_sane_numbers(ring):
    lib, h = ring
    us = ctypes.c_double()
    from paella_amd import _abi
    _abi.check(lib.paella_ring_bench_drain(h, 64, 6400, 20, 200, ctypes.byref(us)))
    assert 1.0 < us.value < 5000.0
    flag, sync = ctypes.c_double(), ctypes.c_double()
    _abi.check(lib.paella_ring_bench_pingpong(50, 500, ctypes.byref(flag), ctypes.byref(sync), None))
    assert 0.5 < flag.value < 2000.0 and 0.5 < sync.value < 5000.0
    floor = ctypes.c_double()
    _abi.check(_abi.probes().paella_empty_kernel_probe(50, ctypes.byref(floor)))
    assert 0.2 < floor.value < 200.0
    print("ring drain 64 blocks: %.2f us/iter; flag ping-pong %.2f us; stream sync %.2f us; empty kernel %.2f us" %
          (us.value, flag.value, sync.value, floor.value))


def test_resident_echo_measures_the_notification_without_a_launch(ring):
    """A resident lane answers host pings through the ring: every ping is answered in order, the round trip is a
    few microseconds, and where the runtime can translate the device clock the one-way figure lies inside it."""
    lib, h = ring
    n = 2000
    rtt = np.zeros(n, np.float64)
    one_way = np.zeros(n, np.float64)
    from paella_amd import _abi
    _abi.check(lib.paella_ring_bench_echo(h, 200, n, rtt.ctypes.data, one_way.ctypes.data))
    assert np.all(rtt > 0) and 0.3 < np.median(rtt) < 200.0
    assert lib.paella_ring_can_read(h) == 0
    have = one_way > -1e29
    print("echo round trip p50 %.2f us p99 %.2f us; device->host p50 %.2f us p99 %.2f us (%d of %d samples translated)" %
          (np.median(rtt), np.sort(rtt)[int(n * 0.99)], np.median(one_way[have]) if have.any() else float("nan"),
           np.sort(one_way[have])[int(have.sum() * 0.99)] if have.any() else float("nan"), have.sum(), n))
    if have.any():
        # the translation interpolates between clock samples taken by the runtime and has been seen off by several
        # microseconds either way: only its order of magnitude is checked
        assert abs(np.median(one_way[have])) < 100.0

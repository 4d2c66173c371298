"""Host IPC: byte ring, fixed-slot ring, datagram socket, names, and the byte layout of the wire.

The ordered-integer checks are the reference's own functional tests for this layer
(tests/ipc/shm_channel/shmc_read.cpp, shmc_write.cpp, shmc_read_write_same_proc.cpp: 10 000 ints through a
64-byte ring, which forces wrap-around and back-pressure thousands of times)."""
import mmap
import os
import struct
import subprocess

import pytest

from _fake import FAKE_LIB, ensure_built

CHECK = os.path.join(FAKE_LIB, "ipc_check")


@pytest.fixture(scope="module", autouse=True)
def built():
    ensure_built()


@pytest.mark.parametrize("check", ["threads", "messages", "multiwriter", "pring", "socket", "pollhooks", "deadclient"])
def test_ipc_self_checks(check):
    out = subprocess.run([CHECK, check], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0 and out.stdout.startswith("OK"), out.stdout + out.stderr


def test_ordered_ints_between_two_processes():
    name = "pytest%d" % os.getpid()
    reader = subprocess.Popen([CHECK, "reader", name], stdout=subprocess.PIPE, text=True)
    assert reader.stdout.readline().strip() == "READY"
    writer = subprocess.run([CHECK, "writer", name], capture_output=True, text=True, timeout=120)
    rest, _ = reader.communicate(timeout=120)
    assert writer.stdout.strip() == "OK writer" and rest.strip() == "OK reader"
    assert not os.path.exists("/dev/shm/llis:channel:" + name)  # the creator unlinks the name


def test_byte_ring_layout_and_message_encoding():
    """Header [size_t capacity][size_t read][size_t write][1-byte lock] then the ring at offset 25; enums are
    u32, strings are size_t length + bytes, host endian."""
    name = "layout%d" % os.getpid()
    p = subprocess.Popen([CHECK, "hold", name], stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    try:
        line = p.stdout.readline().split()
        assert line[0] == "READY" and line[1] == "c2s:x"
        path = "/dev/shm/llis:channel:" + name
        assert os.path.getsize(path) == 25 + 64
        with open(path, "r+b") as f:
            m = mmap.mmap(f.fileno(), 0)
            cap, rd, wr = struct.unpack_from("<QQQ", m, 0)
            assert (cap, rd) == (64, 0)
            payload = struct.pack("<II", 1, 0xAABBCCDD) + struct.pack("<Q", 2) + b"hi"  # REGISTER_JOB == 1
            assert wr == len(payload) == 18
            assert m[24] == 0  # writer lock free
            assert m[25:25 + wr] == payload
            m.close()
    finally:
        p.stdin.write("\n")
        p.stdin.flush()
        p.wait(timeout=30)
    assert not os.path.exists("/dev/shm/llis:channel:" + name)


def test_instrument_info_bit_layout():
    """byte0 is_start, byte1 cu id, byte2 num, byte3 ready (1 on construction), bytes4-7 job id: checked on
    the messages the scripted device posts through the real ring."""
    from _fake import fake_job, run_harness
    _, log = run_harness("sched fifo2 streams 1\nclient\njob %s\nlaunch 0 0\ndrain\n" % fake_job("fake_mem3"))
    blocks = [l.split() for l in log.splitlines() if l.startswith("B ")]
    # kernels of 40, 200 and 17 workgroups with the library's batch size
    from oracle import sched
    assert len(blocks) > 0 and all(b[1] == "0" for b in blocks)
    nums = [int(b[3]) for b in blocks if b[2] == "0"]
    assert sum(nums) == 40 + 200 + 17

"""The C-ABI libraries load without a GPU and export every function their headers declare; the pure-host
parts of the operator ABI (planning, weight packing, output-extent arithmetic) do what the headers say."""
import ctypes
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

HEADERS = {"paella_hip.h": "llis_hip", "paella_ops.h": "paella_ops", "paella_ring.h": "paella_ops", "paella_models.h": "paella_ops",
           "paella_serve.h": "paella_serve", "paella_probes.h": "paella_probes"}


def declared(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b((?:llis_hip|paella)_[a-z0-9_]+)\s*\(", text)))


@pytest.mark.parametrize("header", sorted(HEADERS))
def test_every_declared_symbol_is_exported(header):
    from paella_amd import _abi
    _abi.hip()
    lib = ctypes.CDLL(os.path.join(_abi.LIB_DIR, "lib%s.so" % HEADERS[header]), mode=ctypes.RTLD_GLOBAL)
    names = declared(header)
    assert len(names) >= 4
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing


def test_python_tables_cover_the_headers():
    from paella_amd import _abi, _abi_models, serve
    tables = {"paella_hip.h": _abi.HIP_SYMBOLS, "paella_ops.h": _abi.OPS_SYMBOLS, "paella_ring.h": _abi.RING_SYMBOLS,
              "paella_models.h": _abi_models.MODEL_SYMBOLS, "paella_serve.h": serve.SERVE_SYMBOLS,
              "paella_probes.h": _abi.PROBE_SYMBOLS}
    for header, table in tables.items():
        assert sorted(table) == declared(header), header


def plan(desc_args, has_res=0, hint=0):
    from paella_amd import _abi
    lib = _abi.ops()
    d = _abi.ConvDesc(*desc_args)
    p = _abi.ConvPlan()
    rc = lib.paella_conv2d_plan(ctypes.byref(d), has_res, hint, ctypes.byref(p))
    return rc, p


def test_conv_plan_arithmetic_and_rejections():
    rc, p = plan((64, 56, 56, 64, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 0, 0))
    assert rc == 0 and (p.P, p.Q) == (56, 56) and p.flops == 2.0 * 64 * 64 * 9 * 56 * 56
    assert p.bytes == 4.0 * (64 * 56 * 56 + 64 * 64 * 9 + 64 + 64 * 56 * 56)
    tiles = -(-64 // (32 * p.mi)) * -(-(56 * 56) // (32 * p.ni))
    assert p.dims.grid == tiles and p.dims.block == 64 * p.kw and p.k_pad == 576 and p.m_pad % (32 * p.mi) == 0
    assert plan((64, 56, 56, 64, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 0, 0), has_res=1)[1].bytes == p.bytes + 4.0 * 64 * 56 * 56
    rc, p = plan((32, 112, 112, 32, 3, 3, 2, 2, 1, 1, 1, 1, 32, 2, 0, 0))      # depthwise
    assert rc == 0 and p.kind == 1 and (p.P, p.Q) == (56, 56) and p.blob_bytes == 32 * 9 * 4
    assert plan((8, 8, 8, 8, 3, 3, 1, 1, 1, 1, 1, 1, 4, 0, 0, 0))[0] == -2      # grouped but not depthwise
    assert plan((8, 8, 8, 8, 3, 3, 0, 1, 1, 1, 1, 1, 1, 0, 0, 0))[0] == -1      # stride 0
    assert plan((8, 2, 2, 8, 5, 5, 1, 1, 0, 0, 1, 1, 1, 0, 0, 0))[0] == -1      # empty output
    assert plan((8, 8, 8, 8, 3, 3, 1, 1, 1, 1, 1, 1, 1, 9, 0, 0))[0] == -1      # unknown activation
    assert plan((8, 8, 8, 8, 3, 3, 1, 1, 1, 1, 1, 1, 1, 0, 0, 0), hint=(3 << 8) | (1 << 4))[0] == -1  # no such tile


def test_transformed_launch_accounts_for_its_table_in_lds():
    """The scheduler's figure for a conv that transforms its input on the way: the plan's dynamic LDS (the partial tiles of the
    cross-wave sum) plus the table of scales and shifts, 64 bytes of zeros and 8 bytes per input channel; without a device the
    kernel's static LDS and register count are left as planned."""
    from paella_amd import _abi
    lib = _abi.ops()
    for c in (8, 64, 512, 1024):
        rc, p = plan((c, 14, 14, 128, 1, 1, 1, 1, 0, 0, 1, 1, 1, 0, 0, 0))
        assert rc == 0 and lib.paella_conv2d_plan_takes_input_transform(ctypes.byref(p)) == 1
        plain, pre = _abi.LaunchDims(), _abi.LaunchDims()
        assert lib.paella_conv2d_dims(ctypes.byref(p), ctypes.byref(plain)) == 0
        assert lib.paella_conv2d_transformed_dims(ctypes.byref(p), ctypes.byref(pre)) == 0
        assert (pre.grid, pre.block) == (plain.grid, plain.block)
        assert pre.lds_bytes - p.dims.lds_bytes in range(64 + 8 * c, 64 + 8 * c + 256)   # + the kernel's few static bytes on a device
    rc, p = plan((3, 32, 32, 16, 3, 3, 1, 1, 1, 1, 1, 1, 1, 0, 0, 0))           # channel-major reduction order: no such form
    assert rc == 0 and lib.paella_conv2d_transformed_dims(ctypes.byref(p), ctypes.byref(_abi.LaunchDims())) == -2


def test_weight_packing_layout():
    """Blob = weights as [k/4][m_pad][4] with k = (c, r, s) flattened, zero padded."""
    from paella_amd import _abi
    lib = _abi.ops()
    c, h, w, k, r, s = 5, 9, 7, 6, 3, 2
    rc, p = plan((c, h, w, k, r, s, 1, 1, 1, 0, 2, 1, 1, 0, 0, 0))
    assert rc == 0 and p.k_order == 0
    wt = np.arange(k * c * r * s, dtype=np.float32).reshape(k, c, r, s)
    blob = np.zeros(p.blob_bytes, np.uint8)
    assert lib.paella_conv2d_pack(ctypes.byref(p), wt.ctypes.data, blob.ctypes.data) == 0
    kdim = c * r * s
    assert p.blob_bytes == p.k_pad * p.m_pad * 4
    packed = blob.view(np.float32).reshape(p.k_pad // 4, p.m_pad, 4)
    flat = wt.reshape(k, kdim)
    for m in range(k):
        for kk in range(kdim):
            assert packed[kk // 4, m, kk % 4] == flat[m, kk]
    assert packed[:, k:, :].sum() == 0 and packed.reshape(-1).sum() == flat.sum()


def test_weight_packing_layout_tap_major():
    """C % 8 == 0: the blob's reduction index runs (r, s, c), so a chunk of 8 shares one filter tap."""
    from paella_amd import _abi
    lib = _abi.ops()
    c, h, w, k, r, s = 16, 9, 7, 6, 3, 2
    rc, p = plan((c, h, w, k, r, s, 1, 1, 1, 0, 1, 1, 1, 0, 0, 0))
    assert rc == 0 and p.k_order == 1 and p.k_pad == c * r * s
    wt = np.random.default_rng(1).standard_normal((k, c, r, s)).astype(np.float32)
    blob = np.zeros(p.blob_bytes, np.uint8)
    assert lib.paella_conv2d_pack(ctypes.byref(p), wt.ctypes.data, blob.ctypes.data) == 0
    packed = blob.view(np.float32).reshape(p.k_pad // 4, p.m_pad, 4)
    for m in range(k):
        for cc in range(c):
            for rr in range(r):
                for ss in range(s):
                    kp = (rr * s + ss) * c + cc
                    assert packed[kp // 4, m, kp % 4] == wt[m, cc, rr, ss]


@pytest.mark.parametrize("pad_w,first", [(0, 0), (1, 1)])
def test_weight_packing_layout_with_paired_filter_columns(pad_w, first):
    """Stride 2 across a 3-wide filter: per filter row the unpaired column's C values (chunks of eight channels), then the pair's 2 C
    values as chunks of (first column | second column) x four channels; the pair's first column is the padding."""
    from paella_amd import _abi
    lib = _abi.ops()
    c, h, w, k, r, s = 16, 9, 12, 6, 3, 3
    rc, p = plan((c, h, w, k, r, s, 1, 2, 1, pad_w, 1, 1, 1, 0, 0, 0))
    assert rc == 0 and p.k_order == 1 and p.pair_taps == 1 + first and p.k_pad == c * r * s
    wt = np.random.default_rng(2).standard_normal((k, c, r, s)).astype(np.float32)
    blob = np.zeros(p.blob_bytes, np.uint8)
    assert lib.paella_conv2d_pack(ctypes.byref(p), wt.ctypes.data, blob.ctypes.data) == 0
    packed = blob.view(np.float32).reshape(p.k_pad // 4, p.m_pad, 4)
    unpaired = 2 - 2 * first
    seen = set()
    for m in range(k):
        for cc in range(c):
            for rr in range(r):
                for ss in range(s):
                    if ss == unpaired:
                        kp = rr * 3 * c + cc
                    else:
                        kp = rr * 3 * c + c + (cc // 4) * 8 + (ss - first) * 4 + cc % 4
                    seen.add(kp)
                    assert packed[kp // 4, m, kp % 4] == wt[m, cc, rr, ss]
    assert seen == set(range(c * r * s))   # a permutation of the reduction
    # not paired: odd width with padding (the last pair would leave the image), stride 1, a 5-wide filter
    assert plan((c, h, 13, k, r, s, 1, 2, 1, 1, 1, 1, 1, 0, 0, 0))[1].pair_taps == 0
    assert plan((c, h, w, k, r, s, 1, 1, 1, 1, 1, 1, 1, 0, 0, 0))[1].pair_taps == 0
    assert plan((c, h, w, k, r, 5, 1, 2, 1, 2, 1, 1, 1, 0, 0, 0))[1].pair_taps == 0


def test_pool_out_matches_oracle():
    from oracle import ops as orc
    from paella_amd import _abi
    lib = _abi.ops()
    for n in range(3, 40):
        for k, s, p in [(2, 2, 0), (3, 2, 1), (3, 2, 0), (3, 1, 1), (3, 3, 0)]:
            for ceil in (0, 1):
                assert lib.paella_pool_out(n, k, s, p, ceil) == orc.pool_out(n, k, s, p, bool(ceil))


def test_product_has_no_cpu_compute_path():
    """Nothing under paella_amd/ or include/ may reference the oracle."""
    offenders = []
    for base in ("paella_amd", "include"):
        for dirpath, _, files in os.walk(os.path.join(ROOT, base)):
            if "/build" in dirpath or dirpath.endswith("/lib") or dirpath.endswith("/bin"):
                continue
            for f in files:
                if f.endswith((".py", ".h", ".cpp", ".hip")):
                    if re.search(r"\boracle\b", open(os.path.join(dirpath, f), errors="ignore").read()):
                        offenders.append(os.path.join(dirpath, f))
    assert not offenders, offenders


REFERENCE = "/root/reference"


@pytest.mark.skipif(not os.path.isdir(REFERENCE), reason="the reference tree is not on this machine")
@pytest.mark.parametrize("source", ["app/client.cpp", "tests/client/client.cpp", "tests/client/client_concurrent_runs.cpp",
                                    "tests/client/client_single_latency.cpp", "tests/client/client_concurrent_run_latencies.cpp",
                                    "tests/client/client_concurrent_run_latencies_set_load.cpp"])
def test_reference_client_programs_compile_against_these_headers(source):
    """The client API is a drop-in boundary: the reference's own load generator and client test programs must compile
    unchanged against include/llis/client/*.h (syntax and types only; nothing of the reference is built or run)."""
    import subprocess
    path = os.path.join(REFERENCE, source)
    if not os.path.exists(path):
        pytest.skip(source + " is not in this copy of the reference")
    out = subprocess.run(["g++", "-std=c++17", "-fsyntax-only", "-I" + os.path.join(ROOT, "include"), path], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stderr[-3000:]


def test_host_copy_helper_copies_in_order_and_declines_while_asleep():
    """paella_host_copy_submit: copies land before done() runs, in submission order; after half a millisecond without work the
    helper sleeps and the next call is declined (PAELLA_EBUSY, nothing copied, the caller copies by itself) but wakes it."""
    import threading
    import time
    from paella_amd import _abi
    lib = _abi.ops()
    done_t = ctypes.CFUNCTYPE(None, ctypes.c_void_p)
    order, lock = [], threading.Lock()

    @done_t
    def done(arg):
        with lock:
            order.append(arg)

    def submit_until_taken(dst, src, tag):
        for _ in range(2000):  # a declined call wakes the helper; it is up within microseconds
            rc = lib.paella_host_copy_submit(dst.ctypes.data, src.ctypes.data, src.nbytes, done, tag)
            if rc == 0:
                return
            assert rc == -5
            time.sleep(0.0001)
        raise AssertionError("the helper never woke up")

    rng = np.random.default_rng(5)
    srcs = [rng.integers(0, 255, 300000 + 7 * i, dtype=np.uint8) for i in range(6)]
    dsts = [np.zeros_like(s) for s in srcs]
    submit_until_taken(dsts[0], srcs[0], 1)
    for i in range(1, 6):  # right behind: the helper is awake
        assert lib.paella_host_copy_submit(dsts[i].ctypes.data, srcs[i].ctypes.data, srcs[i].nbytes, done, i + 1) == 0
    deadline = time.time() + 10
    while len(order) < 6 and time.time() < deadline:
        time.sleep(0.001)
    assert order == [1, 2, 3, 4, 5, 6]
    assert all(np.array_equal(d, s) for d, s in zip(dsts, srcs))
    time.sleep(0.05)  # a hundred times the helper's spin: asleep now
    late = np.zeros_like(srcs[0])
    assert lib.paella_host_copy_submit(late.ctypes.data, srcs[0].ctypes.data, srcs[0].nbytes, done, 7) == -5
    time.sleep(0.01)
    assert not late.any() and order == [1, 2, 3, 4, 5, 6]  # declined means untouched
    assert lib.paella_host_copy_submit(None, srcs[0].ctypes.data, 1, done, 0) == -1

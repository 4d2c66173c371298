"""The allocation-free conv entry point (paella_conv2d_launch_static: split-reduction workspace in a fixed array of the
device image) against paella_conv2d_launch with a caller-supplied workspace: same kernels, so bit-identical outputs.
Two calls in a row on one stream, the second with a smaller input, so the second finds what the first left in the
array; then the first shape again."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

PAELLA_ETOOBIG = -4
STATIC_BYTES = 4 << 20


def make(c, hw, k, r, seed, **kw):
    from paella_amd import ops
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((k, c, r, r)) * (2.0 / (c * r * r)) ** 0.5).astype(np.float32)
    b = rng.standard_normal(k).astype(np.float32)
    conv = ops.Conv2d(w, b, pad=r // 2, in_hw=(hw, hw), act=ops.ACT_RELU, **kw)
    x = torch.tensor(rng.standard_normal((1, c, hw, hw)).astype(np.float32), device="cuda:0")
    return conv, x


def launch_static(conv, x):
    from paella_amd import _abi
    p = conv.plan
    y = torch.full((1, p.d.K, p.P, p.Q), float("nan"), device=x.device, dtype=torch.float32)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = conv.lib.paella_conv2d_launch_static(ctypes.byref(p), ctypes.c_void_p(x.data_ptr()), ctypes.c_void_p(conv.blob.data_ptr()),
                                              ctypes.c_void_p(conv.bias.data_ptr()), None, None, ctypes.c_void_p(y.data_ptr()),
                                              stream, 0, None)
    return rc, y


def test_static_workspace_conv_matches_the_workspace_entry_point_twice_in_a_row(cuda):
    big, xb = make(256, 14, 256, 3, seed=11)      # 56 tiles, reduction split over several workgroups
    small, xs = make(512, 7, 128, 3, seed=12)     # smaller input, 8 tiles, deeper split
    assert big.plan.splits > 1 and small.plan.splits > 1
    assert 0 < small.plan.workspace_bytes < big.plan.workspace_bytes <= STATIC_BYTES
    assert xs.numel() < xb.numel()
    print("case static conv: big grid %d splits %d, small grid %d splits %d" % (big.plan.dims.grid, big.plan.splits, small.plan.dims.grid, small.plan.splits), flush=True)
    want_big, want_small = big(xb), small(xs)
    torch.cuda.synchronize()
    for conv, x, want in ((big, xb, want_big), (small, xs, want_small), (big, xb, want_big)):
        rc, got = launch_static(conv, x)
        assert rc == 0
        torch.cuda.synchronize()
        assert torch.equal(got, want)  # same kernels, same summation order: bit for bit


def test_static_workspace_rejects_what_does_not_fit_and_unsplit_plans_need_none(cuda):
    plain, x = make(64, 56, 64, 3, seed=13)       # 196 tiles: no split, no workspace
    assert plain.plan.workspace_bytes == 0
    rc, got = launch_static(plain, x)
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.equal(got, plain(x))
    # force a split of 16 over a large-tile layer: partial tiles beyond the array
    huge, xh = make(64, 112, 256, 3, seed=14, tile_hint=(4 << 12) | (2 << 8) | (2 << 4) | 2)
    assert huge.plan.workspace_bytes > STATIC_BYTES
    rc, got = launch_static(huge, xh)
    assert rc == PAELLA_ETOOBIG
    torch.cuda.synchronize()
    assert bool(torch.isnan(got).all())           # nothing was launched


def test_static_workspace_survives_counters_left_dirty(cuda):
    """An interrupted call may leave arrival counters at any value: the array is dirtied through its device address (every
    word a call could use as a counter or a partial sum set to a pattern) and the next call still gives the same bits."""
    from paella_amd import _abi
    conv, x = make(512, 7, 128, 3, seed=15)
    assert conv.plan.splits > 1
    want = conv(x)
    torch.cuda.synchronize()
    assert conv.lib.paella_conv2d_static_init() == 0
    ws = ctypes.c_void_p()
    assert conv.lib.paella_conv2d_static_workspace(ctypes.byref(ws)) == 0 and ws.value
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for pattern in (0xFFFFFFFF, 0x00000001, 0x7FC00000):
        _abi.check(_abi.hip().llis_hip_fill_u32_async(ws, pattern, STATIC_BYTES // 4, stream))
        rc, got = launch_static(conv, x)
        assert rc == 0
        torch.cuda.synchronize()
        assert torch.equal(got, want), hex(pattern)


def test_static_entry_point_checks_its_arguments_before_it_launches_anything(cuda):
    """A refused call must not have sent the counter fill either: the array keeps the pattern written before the call."""
    from paella_amd import _abi
    conv, x = make(512, 7, 128, 3, seed=16)
    ws = ctypes.c_void_p()
    assert conv.lib.paella_conv2d_static_workspace(ctypes.byref(ws)) == 0
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    _abi.check(_abi.hip().llis_hip_fill_u32_async(ws, 0xA5A5A5A5, 1024, stream))
    p = conv.plan
    y = torch.zeros((1, p.d.K, p.P, p.Q), device="cuda:0")
    rc = conv.lib.paella_conv2d_launch_static(ctypes.byref(p), None, ctypes.c_void_p(conv.blob.data_ptr()), ctypes.c_void_p(conv.bias.data_ptr()),
                                              None, None, ctypes.c_void_p(y.data_ptr()), stream, 0, None)
    assert rc == -1  # PAELLA_EINVAL: no input
    head = torch.empty(1024, dtype=torch.int32, device="cuda:0")
    _abi.check(_abi.hip().llis_hip_memcpy_async(ctypes.c_void_p(head.data_ptr()), ws, 4096, 3, stream))  # device to device
    torch.cuda.synchronize()
    assert bool((head == torch.tensor(0xA5A5A5A5 - (1 << 32), dtype=torch.int32, device="cuda:0")).all())
    rc, got = launch_static(conv, x)   # and the entry point still works afterwards
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.equal(got, conv(x))

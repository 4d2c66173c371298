"""Functional front-end over the operator C-ABI for tests and benches.

Tensors are torch CUDA tensors (torch is only the allocator and stream provider here); weights are packed
on the host with paella_conv2d_pack and uploaded.  Everything runs on the calling thread's current torch
stream unless a stream handle is given.
"""
import ctypes

import numpy as np
import torch

from . import _abi
from ._abi import ConvDesc, ConvOperands, ConvPlan, LaunchDims, PoolDesc, check

ACT_NONE, ACT_RELU, ACT_RELU6, ACT_PRELU, ACT_CLIP = range(5)


def _ptr(t):
    if t is None:
        return None
    assert t.is_cuda and t.dtype == torch.float32 and t.is_contiguous()
    return ctypes.c_void_p(t.data_ptr())


def _stream(stream):
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream if stream is None else stream)


def _pair(v):
    return (v, v) if isinstance(v, int) else tuple(v)


class Conv2d:
    """One planned conv layer: packed weights resident on the device."""

    def __init__(self, w, bias=None, stride=1, pad=0, dil=1, groups=1, act=ACT_NONE, lo=0.0, hi=0.0,
                 in_hw=None, has_residual=False, slope=None, tile_hint=0, device="cuda:0"):
        lib = _abi.ops()
        w = np.ascontiguousarray(w, dtype=np.float32)
        k, cg, r, s = w.shape
        sh, sw = _pair(stride)
        ph, pw = _pair(pad)
        dh, dw = _pair(dil)
        h, wd = in_hw
        self.desc = ConvDesc(cg * groups, h, wd, k, r, s, sh, sw, ph, pw, dh, dw, groups, act, lo, hi)
        self.plan = ConvPlan()
        check(lib.paella_conv2d_plan(ctypes.byref(self.desc), int(has_residual), tile_hint, ctypes.byref(self.plan)),
              "paella_conv2d_plan")
        blob = np.zeros(self.plan.blob_bytes, dtype=np.uint8)
        check(lib.paella_conv2d_pack(ctypes.byref(self.plan), w.ctypes.data, blob.ctypes.data), "paella_conv2d_pack")
        self.blob = torch.from_numpy(blob).to(device)
        self.bias = None if bias is None else torch.tensor(np.asarray(bias, np.float32), device=device)
        self.slope = None if slope is None else torch.tensor(np.asarray(slope, np.float32), device=device)
        self.workspace = torch.zeros(max(self.plan.workspace_bytes, 4) // 4, dtype=torch.int32, device=device) if self.plan.workspace_bytes else None
        self.lib = lib

    def takes_input_transform(self):
        return bool(self.lib.paella_conv2d_plan_takes_input_transform(ctypes.byref(self.plan)))

    def __call__(self, x, residual=None, out=None, stream=None, job_id=0, notifier=None, in_scale=None, in_shift=None, in_act=ACT_NONE):
        """in_scale / in_shift (per input channel, device tensors): the conv reads in_act(x * in_scale + in_shift), padded
        with zeros after that transform."""
        p = self.plan
        assert x.shape == (1, p.d.C, p.d.H, p.d.W), (tuple(x.shape), p.d.C, p.d.H, p.d.W)
        y = out if out is not None else torch.empty((1, p.d.K, p.P, p.Q), device=x.device, dtype=torch.float32)
        if in_scale is not None:
            assert in_scale.numel() == p.d.C and in_shift.numel() == p.d.C
            check(self.lib.paella_conv2d_launch_transformed(ctypes.byref(p), _ptr(x), _ptr(in_scale), _ptr(in_shift), in_act,
                                                            ctypes.c_void_p(self.blob.data_ptr()), _ptr(self.bias), _ptr(residual),
                                                            _ptr(self.slope), _ptr(y),
                                                            ctypes.c_void_p(self.workspace.data_ptr()) if self.workspace is not None else None,
                                                            _stream(stream), job_id, notifier), "paella_conv2d_launch_transformed")
            return y
        check(self.lib.paella_conv2d_launch(ctypes.byref(p), _ptr(x), ctypes.c_void_p(self.blob.data_ptr()),
                                            _ptr(self.bias), _ptr(residual), _ptr(self.slope), _ptr(y),
                                            ctypes.c_void_p(self.workspace.data_ptr()) if self.workspace is not None else None,
                                            _stream(stream), job_id, notifier), "paella_conv2d_launch")
        return y


    def operands(self, x, residual=None, out=None):
        p = self.plan
        assert x.shape == (1, p.d.C, p.d.H, p.d.W), (tuple(x.shape), p.d.C, p.d.H, p.d.W)
        y = out if out is not None else torch.empty((1, p.d.K, p.P, p.Q), device=x.device, dtype=torch.float32)
        data = lambda t: None if t is None else _ptr(t).value
        ops = ConvOperands(ctypes.pointer(p), data(x), self.blob.data_ptr(), data(self.bias), data(residual), data(self.slope), data(y),
                           None if self.workspace is None else self.workspace.data_ptr())
        return ops, y


def conv2d_pair(first, x1, second, x2, residual1=None, residual2=None, stream=None, job_id=0, notifier=None):
    """Two independent Conv2d layers as one launch (paella_conv2d_launch_pair); returns both outputs."""
    a, y1 = first.operands(x1, residual1)
    b, y2 = second.operands(x2, residual2)
    check(first.lib.paella_conv2d_launch_pair(ctypes.byref(a), ctypes.byref(b), _stream(stream), job_id, notifier), "paella_conv2d_launch_pair")
    return y1, y2


def conv2d_group(convs, xs, residuals=None, stream=None, job_id=0, notifier=None):
    """Up to four independent Conv2d layers as one launch (paella_conv2d_launch_group); returns their outputs."""
    residuals = residuals or [None] * len(convs)
    members = (ConvOperands * len(convs))()
    outs = []
    for k, (c, x, r) in enumerate(zip(convs, xs, residuals)):
        members[k], y = c.operands(x, r)
        outs.append(y)
    check(convs[0].lib.paella_conv2d_launch_group(members, len(convs), _stream(stream), job_id, notifier), "paella_conv2d_launch_group")
    return outs


def conv2d_group_pool(convs, xs, pool_x, k, stride, pad=0, ceil_mode=False, is_avg=False, count_include_pad=True, residuals=None,
                      stream=None, job_id=0, notifier=None):
    """Up to three independent Conv2d layers and one pooling operator as one launch (paella_conv2d_launch_group_pool);
    returns the convs' outputs and the pool's."""
    residuals = residuals or [None] * len(convs)
    members = (ConvOperands * len(convs))()
    outs = []
    for i, (c, x, r) in enumerate(zip(convs, xs, residuals)):
        members[i], y = c.operands(x, r)
        outs.append(y)
    lib = convs[0].lib
    _, c, h, w = pool_x.shape
    r, s = _pair(k)
    sh, sw = _pair(stride)
    ph, pw = _pair(pad)
    d = PoolDesc(c, h, w, r, s, sh, sw, ph, pw, int(ceil_mode), int(is_avg), int(count_include_pad))
    p = lib.paella_pool_out(h, r, sh, ph, int(ceil_mode))
    q = lib.paella_pool_out(w, s, sw, pw, int(ceil_mode))
    pool_y = torch.empty((1, c, p, q), device=pool_x.device, dtype=torch.float32)
    check(lib.paella_conv2d_launch_group_pool(members, len(convs), ctypes.byref(d), _ptr(pool_x), _ptr(pool_y), _stream(stream), job_id,
                                              notifier), "paella_conv2d_launch_group_pool")
    return outs, pool_y


def pair_dims(first, second):
    d = LaunchDims()
    rc = first.lib.paella_conv2d_pair_dims(ctypes.byref(first.plan), ctypes.byref(second.plan), ctypes.byref(d))
    return rc, d


def dense(x, w, bias=None, act=ACT_NONE, stream=None, job_id=0, notifier=None):
    lib = _abi.ops()
    o, i = w.shape
    y = torch.empty((1, o), device=x.device, dtype=torch.float32)
    check(lib.paella_dense_launch(_ptr(x), _ptr(w), _ptr(bias), _ptr(y), i, o, act, _stream(stream), job_id, notifier),
          "paella_dense_launch")
    return y


def pool2d(x, k, stride, pad=0, ceil_mode=False, is_avg=False, count_include_pad=True, stream=None, job_id=0,
           notifier=None):
    lib = _abi.ops()
    _, c, h, w = x.shape
    r, s = _pair(k)
    sh, sw = _pair(stride)
    ph, pw = _pair(pad)
    d = PoolDesc(c, h, w, r, s, sh, sw, ph, pw, int(ceil_mode), int(is_avg), int(count_include_pad))
    p = lib.paella_pool_out(h, r, sh, ph, int(ceil_mode))
    q = lib.paella_pool_out(w, s, sw, pw, int(ceil_mode))
    y = torch.empty((1, c, p, q), device=x.device, dtype=torch.float32)
    check(lib.paella_pool2d_launch(ctypes.byref(d), _ptr(x), _ptr(y), _stream(stream), job_id, notifier),
          "paella_pool2d_launch")
    return y


def global_avgpool(x, stream=None, job_id=0, notifier=None):
    lib = _abi.ops()
    _, c, h, w = x.shape
    y = torch.empty((1, c, 1, 1), device=x.device, dtype=torch.float32)
    check(lib.paella_global_avgpool_launch(_ptr(x), _ptr(y), c, h * w, _stream(stream), job_id, notifier),
          "paella_global_avgpool_launch")
    return y


def eltwise(a, b=None, scale=None, shift=None, slope=None, act=ACT_NONE, lo=0.0, hi=0.0, stream=None, job_id=0,
            notifier=None):
    lib = _abi.ops()
    c = a.shape[1]
    y = torch.empty_like(a)
    check(lib.paella_eltwise_launch(_ptr(a), _ptr(b), _ptr(scale), _ptr(shift), _ptr(slope), _ptr(y), c,
                                    a.numel() // c, act, lo, hi, _stream(stream), job_id, notifier),
          "paella_eltwise_launch")
    return y


def copy(x, stream=None, job_id=0, notifier=None):
    lib = _abi.ops()
    y = torch.empty_like(x)
    check(lib.paella_copy_launch(_ptr(x), _ptr(y), x.numel(), _stream(stream), job_id, notifier), "paella_copy_launch")
    return y


def softmax(x, stream=None, job_id=0, notifier=None):
    lib = _abi.ops()
    cols = x.shape[-1]
    y = torch.empty_like(x)
    check(lib.paella_softmax_launch(_ptr(x), _ptr(y), x.numel() // cols, cols, _stream(stream), job_id, notifier),
          "paella_softmax_launch")
    return y


def lrn(x, size, alpha, beta, k, stream=None, job_id=0, notifier=None):
    lib = _abi.ops()
    c = x.shape[1]
    y = torch.empty_like(x)
    check(lib.paella_lrn_launch(_ptr(x), _ptr(y), c, x.numel() // c, size, alpha, beta, k, _stream(stream), job_id,
                                notifier), "paella_lrn_launch")
    return y


class DirectQueue:
    """A user-mode hardware queue of the operator library; pass `.handle` as `stream=` to any launch."""

    def __init__(self, ordered=False):
        self.lib = _abi.ops()
        h = ctypes.c_void_p()
        check(self.lib.paella_direct_queue_create(ctypes.byref(h)), "paella_direct_queue_create")
        self.handle = h.value
        if ordered:
            check(self.lib.paella_direct_queue_set_ordered(h, 1), "paella_direct_queue_set_ordered")

    def wait(self):
        check(self.lib.paella_direct_queue_wait(ctypes.c_void_p(self.handle)), "paella_direct_queue_wait")

    def close(self):
        if self.handle:
            check(self.lib.paella_direct_queue_destroy(ctypes.c_void_p(self.handle)), "paella_direct_queue_destroy")
            self.handle = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

"""numpy front-end of oracle/ops.c (TEST INFRASTRUCTURE ONLY; see the header of ops.c for what it restates).

Every function takes and returns contiguous float32 numpy arrays in NCHW.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle_ops.so")

ACT_NONE, ACT_RELU, ACT_RELU6, ACT_PRELU, ACT_CLIP = range(5)


def build():
    subprocess.check_call(["make", "-s", "-C", _HERE])


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    return ctypes.CDLL(_LIB_PATH)


_lib = _load()
_f32p = ctypes.POINTER(ctypes.c_float)
_i = ctypes.c_int
_f = ctypes.c_float


def _p(a):
    if a is None:
        return ctypes.cast(None, _f32p)
    assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(_f32p)


def _c(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.float32)


_lib.orc_conv_out.restype = _i
_lib.orc_pool_out.restype = _i
for _name in ("orc_conv2d", "orc_conv2d_fast"):
    getattr(_lib, _name).argtypes = [_f32p] * 5 + [_i] * 14 + [_i, _f32p, _f, _f]
_lib.orc_dense.argtypes = [_f32p] * 4 + [_i] * 4
_lib.orc_maxpool2d.argtypes = [_f32p] * 2 + [_i] * 11
_lib.orc_avgpool2d.argtypes = [_f32p] * 2 + [_i] * 12
_lib.orc_global_avgpool.argtypes = [_f32p] * 2 + [_i] * 3
_lib.orc_add.argtypes = [_f32p] * 3 + [_i] * 3 + [_f32p, _f, _f]
_lib.orc_scale_shift.argtypes = [_f32p] * 4 + [_i] * 3 + [_f32p, _f, _f]
_lib.orc_softmax.argtypes = [_f32p] * 2 + [_i] * 2
_lib.orc_lrn.argtypes = [_f32p] * 2 + [_i] * 3 + [_f] * 3
_lib.orc_fill_normal.argtypes = [_f32p, ctypes.c_size_t, ctypes.c_uint64, ctypes.c_uint64, ctypes.c_double]
_lib.orc_fill_uniform.argtypes = [_f32p, ctypes.c_size_t, ctypes.c_uint64, ctypes.c_uint64, ctypes.c_double,
                                  ctypes.c_double]


def _pair(v):
    return (v, v) if isinstance(v, int) else tuple(v)


def conv_out(n, k, stride, pad, dil=1):
    return _lib.orc_conv_out(n, k, stride, pad, dil)


def pool_out(n, k, stride, pad, ceil_mode=False):
    return _lib.orc_pool_out(n, k, stride, pad, int(ceil_mode))


def conv2d(x, w, bias=None, stride=1, pad=0, dil=1, groups=1, act=ACT_NONE, residual=None, slope=None,
           lo=0.0, hi=0.0, fast=False):
    x, w, bias, residual, slope = _c(x), _c(w), _c(bias), _c(residual), _c(slope)
    n, c, h, wd = x.shape
    k, cg, r, s = w.shape
    assert cg * groups == c and k % groups == 0
    sh, sw = _pair(stride)
    ph, pw = _pair(pad)
    dh, dw = _pair(dil)
    p, q = conv_out(h, r, sh, ph, dh), conv_out(wd, s, sw, pw, dw)
    y = np.empty((n, k, p, q), np.float32)
    if residual is not None:
        assert residual.shape == y.shape
    fn = _lib.orc_conv2d_fast if fast else _lib.orc_conv2d
    fn(_p(x), _p(w), _p(bias), _p(residual), _p(y), n, c, h, wd, k, r, s, sh, sw, ph, pw, dh, dw, groups,
       act, _p(slope), lo, hi)
    return y


def dense(x, w, bias=None, act=ACT_NONE):
    x, w, bias = _c(x), _c(w), _c(bias)
    n, i = x.shape
    o = w.shape[0]
    assert w.shape[1] == i
    y = np.empty((n, o), np.float32)
    _lib.orc_dense(_p(x), _p(w), _p(bias), _p(y), n, i, o, act)
    return y


def maxpool2d(x, k, stride, pad=0, ceil_mode=False):
    x = _c(x)
    n, c, h, w = x.shape
    r, s = _pair(k)
    sh, sw = _pair(stride)
    ph, pw = _pair(pad)
    y = np.empty((n, c, pool_out(h, r, sh, ph, ceil_mode), pool_out(w, s, sw, pw, ceil_mode)), np.float32)
    _lib.orc_maxpool2d(_p(x), _p(y), n, c, h, w, r, s, sh, sw, ph, pw, int(ceil_mode))
    return y


def avgpool2d(x, k, stride, pad=0, ceil_mode=False, count_include_pad=True):
    x = _c(x)
    n, c, h, w = x.shape
    r, s = _pair(k)
    sh, sw = _pair(stride)
    ph, pw = _pair(pad)
    y = np.empty((n, c, pool_out(h, r, sh, ph, ceil_mode), pool_out(w, s, sw, pw, ceil_mode)), np.float32)
    _lib.orc_avgpool2d(_p(x), _p(y), n, c, h, w, r, s, sh, sw, ph, pw, int(ceil_mode), int(count_include_pad))
    return y


def global_avgpool(x):
    x = _c(x)
    n, c, h, w = x.shape
    y = np.empty((n, c, 1, 1), np.float32)
    _lib.orc_global_avgpool(_p(x), _p(y), n, c, h * w)
    return y


def add(a, b, act=ACT_NONE, slope=None, lo=0.0, hi=0.0):
    a, b, slope = _c(a), _c(b), _c(slope)
    assert a.shape == b.shape and a.shape[0] == 1
    y = np.empty_like(a)
    c = a.shape[1]
    _lib.orc_add(_p(a), _p(b), _p(y), c, a.size // c, act, _p(slope), lo, hi)
    return y


def scale_shift(x, scale=None, shift=None, act=ACT_NONE, slope=None, lo=0.0, hi=0.0):
    x, scale, shift, slope = _c(x), _c(scale), _c(shift), _c(slope)
    assert x.shape[0] == 1
    y = np.empty_like(x)
    c = x.shape[1]
    _lib.orc_scale_shift(_p(x), _p(scale), _p(shift), _p(y), c, x.size // c, act, _p(slope), lo, hi)
    return y


def softmax(x):
    x = _c(x)
    y = np.empty_like(x)
    cols = x.shape[-1]
    _lib.orc_softmax(_p(x), _p(y), x.size // cols, cols)
    return y


def lrn(x, size, alpha, beta, k):
    x = _c(x)
    assert x.shape[0] == 1
    y = np.empty_like(x)
    c = x.shape[1]
    _lib.orc_lrn(_p(x), _p(y), c, x.size // c, size, alpha, beta, k)
    return y


def fill_normal(shape, seed, stream, std):
    out = np.empty(shape, np.float32)
    _lib.orc_fill_normal(_p(out), out.size, seed, stream, std)
    return out


def fill_uniform(shape, seed, stream, lo, hi):
    out = np.empty(shape, np.float32)
    _lib.orc_fill_uniform(_p(out), out.size, seed, stream, lo, hi)
    return out


def num_threads():
    _lib.orc_num_threads.restype = ctypes.c_int
    return _lib.orc_num_threads()

"""Pins oracle/ops.c against torch.nn.functional on the CPU and against closed forms.

The reference keeps no numeric vectors for its operators (they come from an un-vendored TVM fork), so the
oracle is pinned against an independent third-party implementation plus identities that a dropped term,
a transposed operand or a wrong index would break.
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import ops

RNG = np.random.default_rng(1234)


def rnd(*shape):
    return RNG.standard_normal(shape).astype(np.float32)


CONV_CASES = [
    # C, H, W, K, R, S, stride, pad, dil, groups
    (1, 28, 28, 8, 5, 5, 1, 2, 1, 1),
    (8, 14, 14, 16, 5, 5, 1, 2, 1, 1),
    (3, 33, 31, 16, 7, 7, 2, 3, 1, 1),
    (16, 17, 17, 24, 1, 7, 1, (0, 3), 1, 1),
    (16, 17, 17, 24, 7, 1, 1, (3, 0), 1, 1),
    (12, 9, 11, 12, 3, 3, 2, 1, 1, 12),
    (8, 10, 10, 6, 3, 3, 1, 2, 2, 2),
    (32, 7, 7, 64, 1, 1, 2, 0, 1, 1),
]


@pytest.mark.parametrize("case", CONV_CASES)
@pytest.mark.parametrize("fast", [False, True])
def test_conv2d_matches_torch(case, fast):
    c, h, w, k, r, s, stride, pad, dil, groups = case
    x, wt, b = rnd(1, c, h, w), rnd(k, c // groups, r, s), rnd(k)
    got = ops.conv2d(x, wt, b, stride=stride, pad=pad, dil=dil, groups=groups, fast=fast)
    ref = F.conv2d(torch.tensor(x).double(), torch.tensor(wt).double(), torch.tensor(b).double(), stride=stride,
                   padding=pad, dilation=dil, groups=groups).float().numpy()
    assert got.shape == ref.shape
    np.testing.assert_allclose(got, ref, rtol=1e-5 if not fast else 1e-4, atol=1e-5 if not fast else 1e-4)


def test_conv2d_epilogue_order_and_activations():
    x, wt, b, res = rnd(1, 4, 6, 6), rnd(5, 4, 3, 3), rnd(5), rnd(1, 5, 6, 6)
    lin = F.conv2d(torch.tensor(x), torch.tensor(wt), torch.tensor(b), padding=1) + torch.tensor(res)
    slope = np.abs(rnd(5))
    cases = {
        ops.ACT_NONE: lin,
        ops.ACT_RELU: F.relu(lin),
        ops.ACT_RELU6: F.relu6(lin),
        ops.ACT_PRELU: F.prelu(lin, torch.tensor(slope)),
        ops.ACT_CLIP: torch.clamp(lin, -0.5, 0.75),
    }
    for act, ref in cases.items():
        got = ops.conv2d(x, wt, b, pad=1, act=act, residual=res, slope=slope, lo=-0.5, hi=0.75)
        np.testing.assert_allclose(got, ref.numpy(), rtol=1e-5, atol=1e-5)


def test_conv2d_closed_forms():
    x = rnd(1, 3, 8, 8)
    # identity kernel passes the input through
    w = np.zeros((3, 3, 3, 3), np.float32)
    for c in range(3):
        w[c, c, 1, 1] = 1
    np.testing.assert_array_equal(ops.conv2d(x, w, pad=1), x)
    # zero weights leave the bias
    b = rnd(3)
    y = ops.conv2d(x, np.zeros_like(w), b, pad=1)
    np.testing.assert_array_equal(y, np.broadcast_to(b[None, :, None, None], y.shape))
    # linear in the weights
    w1, w2 = rnd(4, 3, 3, 3), rnd(4, 3, 3, 3)
    np.testing.assert_allclose(ops.conv2d(x, w1 + w2, pad=1), ops.conv2d(x, w1, pad=1) + ops.conv2d(x, w2, pad=1),
                               rtol=1e-5, atol=1e-5)
    # a 1x1 conv is a matrix product over channels
    w11 = rnd(5, 3, 1, 1)
    np.testing.assert_allclose(ops.conv2d(x, w11)[0].reshape(5, -1), w11.reshape(5, 3).astype(np.float64) @ x[0].reshape(3, -1),
                               rtol=1e-5, atol=1e-5)
    # a shifted delta kernel shifts the image (catches transposed r/s or wrong sign of the offset)
    wd = np.zeros((1, 1, 3, 3), np.float32)
    wd[0, 0, 0, 2] = 1  # tap at row -1, col +1
    img = rnd(1, 1, 6, 7)
    y = ops.conv2d(img, wd, pad=1)
    np.testing.assert_array_equal(y[0, 0, 1:, :-1], img[0, 0, :-1, 1:])
    assert np.all(y[0, 0, 0, :] == 0) and np.all(y[0, 0, :, -1] == 0)


def test_output_extent_formula():
    for n, k, s, p, d in [(224, 7, 2, 3, 1), (299, 3, 2, 0, 1), (56, 3, 1, 1, 1), (17, 7, 1, 3, 1), (10, 3, 1, 2, 2)]:
        assert ops.conv_out(n, k, s, p, d) == F.conv2d(torch.zeros(1, 1, n, n), torch.zeros(1, 1, k, k), stride=s, padding=p,
                                                       dilation=d).shape[-1]
    for n, k, s, p, ceil in [(112, 3, 2, 1, False), (147, 3, 2, 0, False), (111, 3, 2, 0, True), (13, 3, 2, 0, True),
                             (28, 3, 3, 0, False), (7, 2, 2, 0, True), (6, 3, 2, 1, True)]:
        assert ops.pool_out(n, k, s, p, ceil) == F.max_pool2d(torch.zeros(1, 1, n, n), k, s, p, ceil_mode=ceil).shape[-1]


@pytest.mark.parametrize("k,s,p,ceil", [(2, 2, 0, False), (3, 3, 0, False), (3, 2, 1, False), (3, 2, 0, True), (3, 1, 1, False)])
def test_maxpool_matches_torch(k, s, p, ceil):
    x = rnd(1, 5, 13, 15)
    np.testing.assert_array_equal(ops.maxpool2d(x, k, s, p, ceil), F.max_pool2d(torch.tensor(x), k, s, p, ceil_mode=ceil).numpy())


@pytest.mark.parametrize("k,s,p,ceil,cip", [(2, 2, 0, False, True), (3, 1, 1, False, True), (3, 1, 1, False, False),
                                            (3, 2, 1, True, True), (3, 2, 0, True, False), (7, 1, 0, False, True)])
def test_avgpool_matches_torch(k, s, p, ceil, cip):
    x = rnd(1, 5, 13, 15)
    ref = F.avg_pool2d(torch.tensor(x), k, s, p, ceil_mode=ceil, count_include_pad=cip).numpy()
    np.testing.assert_allclose(ops.avgpool2d(x, k, s, p, ceil, cip), ref, rtol=1e-6, atol=1e-6)


def test_global_avgpool_dense_softmax_lrn_eltwise():
    x = rnd(1, 6, 7, 7)
    np.testing.assert_allclose(ops.global_avgpool(x), x.mean(axis=(2, 3), keepdims=True), rtol=1e-6, atol=1e-6)
    v, w, b = rnd(1, 37), rnd(11, 37), rnd(11)
    np.testing.assert_allclose(ops.dense(v, w, b), v.astype(np.float64) @ w.T.astype(np.float64) + b, rtol=1e-5, atol=1e-5)
    z = rnd(3, 50) * 4
    np.testing.assert_allclose(ops.softmax(z), F.softmax(torch.tensor(z), dim=-1).numpy(), rtol=1e-5, atol=1e-7)
    np.testing.assert_allclose(ops.softmax(z).sum(-1), 1.0, rtol=1e-6)
    for size in (3, 5):  # odd windows: ONNX and torch agree on the window placement
        np.testing.assert_allclose(ops.lrn(x, size, 1e-4 * 50, 0.75, 1.0),
                                   F.local_response_norm(torch.tensor(x), size, 1e-4 * 50, 0.75, 1.0).numpy(), rtol=1e-5, atol=1e-6)
    # even window: ONNX places it at [c - floor((n-1)/2), c + ceil((n-1)/2)]
    xd = x[0].astype(np.float64)
    ref = np.empty_like(xd)
    for c in range(6):
        lo_c, hi_c = max(0, c - 1), min(5, c + 2)
        ref[c] = xd[c] / (2.0 + 0.3 / 4 * (xd[lo_c:hi_c + 1] ** 2).sum(0)) ** 0.6
    np.testing.assert_allclose(ops.lrn(x, 4, 0.3, 0.6, 2.0)[0], ref, rtol=1e-5, atol=1e-6)
    a, b2, sc, sf = rnd(1, 6, 7, 7), rnd(1, 6, 7, 7), rnd(6), rnd(6)
    np.testing.assert_allclose(ops.add(a, b2, ops.ACT_RELU), np.maximum(a + b2, 0), rtol=1e-6, atol=1e-6)
    ref = np.maximum(a * sc[None, :, None, None] + sf[None, :, None, None], 0)
    np.testing.assert_allclose(ops.scale_shift(a, sc, sf, ops.ACT_RELU), ref, rtol=1e-6, atol=1e-6)


def test_seeded_generator_is_a_pure_function_and_standard_normal():
    a = ops.fill_normal((4096,), 7, 3, 1.0)
    b = ops.fill_normal((4096,), 7, 3, 1.0)
    np.testing.assert_array_equal(a, b)
    assert not np.array_equal(a, ops.fill_normal((4096,), 7, 4, 1.0))
    assert not np.array_equal(a, ops.fill_normal((4096,), 8, 3, 1.0))
    # prefix property: element i does not depend on the tensor length
    np.testing.assert_array_equal(a[:100], ops.fill_normal((100,), 7, 3, 1.0))
    big = ops.fill_normal((200000,), 1, 0, 2.0)
    assert abs(big.mean()) < 0.02 and abs(big.std() - 2.0) < 0.02
    u = ops.fill_uniform((200000,), 1, 0, 0.0, 1.0)
    assert 0.0 <= u.min() and u.max() < 1.0 and abs(u.mean() - 0.5) < 0.005
    # independent restatement of the documented recipe in numpy (uint64 wrap-around arithmetic)
    def splitmix(z):
        z = (z + np.uint64(0x9E3779B97F4A7C15))
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))
    with np.errstate(over="ignore"):
        idx = np.arange(64, dtype=np.uint64)
        key = np.uint64(7) * np.uint64(0x9E3779B97F4A7C15) + np.uint64(3) * np.uint64(0xD1B54A32D192ED03)
        u1 = ((splitmix(key + np.uint64(2) * idx) >> np.uint64(11)).astype(np.float64) + 0.5) / 9007199254740992.0
        u2 = ((splitmix(key + np.uint64(2) * idx + np.uint64(1)) >> np.uint64(11)).astype(np.float64) + 0.5) / 9007199254740992.0
    z = np.sqrt(-2.0 * np.log(u1)) * np.cos(2 * np.pi * u2)
    np.testing.assert_allclose(a[:64], z.astype(np.float32), rtol=2e-7, atol=1e-7)

"""Direct dispatch (AQL packets on the library's own hardware queues) must run the very same kernels as the
HIP launch path: every result here is compared bit for bit with the stream path, which the other GPU tests
hold against the CPU oracle."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

RNG = np.random.default_rng(7)


def rnd(*shape, scale=1.0):
    return (RNG.standard_normal(shape) * scale).astype(np.float32)


def test_copy_through_direct_queue(cuda):
    from paella_amd import ops
    x = torch.tensor(rnd(1, 3, 37, 41), device=cuda)
    with ops.DirectQueue() as q:
        y = torch.zeros_like(x)
        torch.cuda.synchronize()
        from paella_amd import _abi
        import ctypes
        _abi.check(_abi.ops().paella_copy_launch(ctypes.c_void_p(x.data_ptr()), ctypes.c_void_p(y.data_ptr()), x.numel(),
                                                 ctypes.c_void_p(q.handle), 0, None), "copy")
        q.wait()
        assert torch.equal(x, y)


CONV_CASES = [
    # C, H, W, K, R, S, stride, pad, tile_hint
    (64, 56, 56, 64, 3, 3, 1, 1, 0),
    (512, 7, 7, 512, 3, 3, 1, 1, 0),                       # grid-level split of the reduction
    (256, 14, 14, 256, 3, 3, 1, 1, (2 << 12) | (1 << 8) | (1 << 4) | 2),
    (3, 224, 224, 64, 7, 7, 2, 3, 0),
    (5, 9, 11, 7, 3, 3, 1, 1, 0),
    (96, 20, 20, 96, 3, 3, 1, 1, (1 << 8) | (1 << 4) | 0),  # one wave per workgroup
]


@pytest.mark.parametrize("case", CONV_CASES)
def test_conv_direct_equals_stream(cuda, case):
    from paella_amd import ops
    c, h, w, k, r, s, stride, pad, hint = case
    conv = ops.Conv2d(rnd(k, c, r, s, scale=(2.0 / (c * r * s)) ** 0.5), rnd(k, scale=0.1), stride=stride, pad=pad, act=ops.ACT_RELU,
                      in_hw=(h, w), has_residual=True, tile_hint=hint)
    x = torch.tensor(rnd(1, c, h, w), device=cuda)
    res = torch.tensor(rnd(1, k, conv.plan.P, conv.plan.Q), device=cuda)
    ref = conv(x, residual=res)
    torch.cuda.synchronize()
    with ops.DirectQueue() as q:
        for _ in range(3):  # the split-k counters must be left at zero by every launch
            got = torch.zeros_like(ref)
            torch.cuda.synchronize()
            conv(x, residual=res, out=got, stream=q.handle)
            q.wait()
            assert torch.equal(got, ref)


def test_misc_ops_direct_equal_stream(cuda):
    from paella_amd import ops
    x = torch.tensor(rnd(1, 24, 29, 31), device=cuda)
    b = torch.tensor(rnd(1, 24, 29, 31), device=cuda)
    w = torch.tensor(rnd(100, 24 * 29 * 31, scale=0.01), device=cuda)
    bias = torch.tensor(rnd(100), device=cuda)
    flat = x.reshape(1, -1).contiguous()
    dw = ops.Conv2d(rnd(24, 1, 3, 3), rnd(24), stride=1, pad=1, groups=24, act=ops.ACT_RELU6, in_hw=(29, 31))
    calls = {
        "dense": lambda st: ops.dense(flat, w, bias, act=ops.ACT_RELU, stream=st),
        "maxpool": lambda st: ops.pool2d(x, 3, 2, 1, stream=st),
        "avgpool": lambda st: ops.pool2d(x, 3, 2, 1, is_avg=True, count_include_pad=False, stream=st),
        "gap": lambda st: ops.global_avgpool(x, stream=st),
        "add_relu": lambda st: ops.eltwise(x, b, act=ops.ACT_RELU, stream=st),
        "softmax": lambda st: ops.softmax(flat[:, :1000].contiguous(), stream=st),
        "lrn": lambda st: ops.lrn(x, 5, 1e-4, 0.75, 1.0, stream=st),
        "depthwise": lambda st: dw(x, stream=st),
    }
    with ops.DirectQueue() as q:
        for name, fn in calls.items():
            ref = fn(None)
            torch.cuda.synchronize()
            got = fn(q.handle)
            q.wait()
            assert torch.equal(got, ref), name


@pytest.mark.parametrize("model", ["mnist", "resnet18", "mobilenetv2"])
def test_model_forward_on_ordered_direct_queue(cuda, model):
    from oracle import models as om
    from paella_amd import models, ops
    desc = models.describe(model)
    x = om.make_input(desc, 3)
    ex = models.Exec(model, seed=1)
    try:
        ex.set_input(x)
        ex.forward(None)
        torch.cuda.synchronize()
        ref = ex.get_output().copy()
        with ops.DirectQueue(ordered=True) as q:
            for _ in range(2):
                ex.set_input(x)
                ex.forward(q.handle)
                q.wait()
                assert np.array_equal(ex.get_output(), ref)
    finally:
        ex.close()


def test_queue_concurrency_probe_runs_and_reports_a_time(cuda):
    """The probe behind bench.py --queue-probe: rejects shapes it is not for, returns a positive time otherwise, and four
    queues are not slower than one."""
    from paella_amd import _abi
    from paella_amd._abi import ConvDesc
    lib = _abi.ops()
    d = ConvDesc(64, 14, 14, 64, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 0.0, 0.0)
    us = ctypes.c_double()
    assert _abi.probes().paella_queue_concurrency_probe(ctypes.byref(d), 8, 3, 2, 1, 5, ctypes.byref(us)) == -1  # 8 instances, 3 per launch
    _abi.check(_abi.probes().paella_queue_concurrency_probe(ctypes.byref(d), 8, 1, 1, 1, 20, ctypes.byref(us)), "probe, one queue")
    one = us.value
    _abi.check(_abi.probes().paella_queue_concurrency_probe(ctypes.byref(d), 8, 1, 4, 1, 20, ctypes.byref(us)), "probe, four queues")
    four = us.value
    _abi.check(_abi.probes().paella_queue_concurrency_probe(ctypes.byref(d), 8, 4, 4, 1, 20, ctypes.byref(us)), "probe, four per launch")
    assert 0.1 < four <= one * 1.1 and 0.05 < us.value < one * 1.1, (one, four, us.value)


def test_vector_alu_work_adds_to_matrix_instruction_time(cuda):
    """paella_mfma_valu_overlap_probe: on this device a SIMD's vector-ALU instructions do not hide behind its matrix
    instructions -- the loop with both takes the matrix loop's time plus the vector loop's time (which is why the conv
    kernel keeps its per-chunk address arithmetic on the scalar unit)."""
    from paella_amd import _abi
    lib = _abi.ops()

    def probe(n):
        both, alone, tf = ctypes.c_double(), ctypes.c_double(), ctypes.c_double()
        _abi.check(_abi.probes().paella_mfma_valu_overlap_probe(n, ctypes.byref(both), ctypes.byref(alone), ctypes.byref(tf)), "paella_mfma_valu_overlap_probe")
        return both.value, alone.value, tf.value

    base, _, peak = probe(0)
    assert 120.0 < peak < 165.0  # the matrix loop alone runs near the fp32 peak
    for n in (32, 128):
        both, alone, tf = probe(n)
        assert alone > 0 and 0.9 * (base + alone) < both < 1.1 * (base + alone), (n, base, alone, both)
        assert tf < peak
    assert _abi.probes().paella_mfma_valu_overlap_probe(7, None, None, None) == -1

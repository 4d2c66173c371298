"""Launch packing (paella_pack_*): convs of several jobs held back and sent as one grid must give the bits they give alone,
and every job's notifier must see exactly its own workgroups."""
import ctypes

import numpy as np
import pytest
import torch

from test_ring_gpu import decode

pytestmark = pytest.mark.gpu

NO_START = 0x80000000  # PAELLA_JOB_ID_NO_START


def layers(cuda, rng):
    """Ten layers on the 32 x 32 tile with eight waves in tap-major order, with and without a split reduction."""
    from paella_amd import ops
    shapes = [  # C, K, H, R, stride, pad
        (64, 64, 56, 3, 1, 1), (128, 128, 28, 3, 1, 1), (256, 256, 14, 3, 1, 1), (512, 512, 7, 3, 1, 1), (768, 192, 17, 1, 1, 0),
        (1280, 320, 8, 1, 1, 0), (288, 64, 35, 1, 1, 0), (256, 512, 14, 1, 2, 0), (64, 96, 19, 3, 1, 1), (160, 40, 9, 3, 2, 1),
    ]
    out = []
    for c, k, h, r, st, pd in shapes:
        w = rng.standard_normal((k, c, r, r)).astype(np.float32) * (1.0 / np.sqrt(c * r * r))
        b = rng.standard_normal(k).astype(np.float32)
        conv = ops.Conv2d(w, b, stride=st, pad=pd, act=ops.ACT_RELU, in_hw=(h, h))
        assert (conv.plan.mi, conv.plan.ni, conv.plan.kw, conv.plan.k_order) == (1, 1, 8, 1)
        x = torch.tensor(rng.standard_normal((1, c, h, h)).astype(np.float32), device=cuda)
        out.append((conv, x))
    return out


@pytest.fixture()
def ring(cuda):
    from paella_amd import _abi
    lib = _abi.ops()
    handle = ctypes.c_void_p()
    _abi.check(lib.paella_ring_create(8192, 16, ctypes.byref(handle)), "paella_ring_create")
    yield lib, handle
    lib.paella_pack_enable(0)
    lib.paella_ring_destroy(handle)


def held(lib):
    return lib.paella_pack_stats(None, None)


def stats(lib):
    a, b = ctypes.c_uint64(), ctypes.c_uint64()
    lib.paella_pack_stats(ctypes.byref(a), ctypes.byref(b))
    return a.value, b.value


def test_packed_convs_are_bit_identical_and_report_to_their_own_jobs(ring, cuda):
    lib, h = ring
    from paella_amd import ops
    rng = np.random.default_rng(11)
    ls = layers(cuda, rng)
    alone = [conv(x) for conv, x in ls]
    torch.cuda.synchronize()
    batch = lib.paella_ring_batch_size()
    with ops.DirectQueue() as q:  # unordered: what the serving path launches on
        assert lib.paella_pack_enable(1) == 0
        try:
            before = stats(lib)
            outs, want_msgs, grids = [], 0, {}
            # jobs 1..8 one conv each; job 9 two convs in one call (a request's independent pair)
            for j in range(8):
                conv, x = ls[j]
                y = torch.zeros_like(alone[j])
                conv(x, out=y, stream=q.handle, job_id=j + 1, notifier=ctypes.c_void_p(lib.paella_ring_notifier(h, j)))
                outs.append(y)
                grids[j + 1] = conv.plan.dims.grid
            pair = ops.conv2d_group([ls[8][0], ls[9][0]], [ls[8][1], ls[9][1]], stream=q.handle, job_id=9 | NO_START,
                                    notifier=ctypes.c_void_p(lib.paella_ring_notifier(h, 8)))
            outs += pair
            grids[9] = ls[8][0].plan.dims.grid + ls[9][0].plan.dims.grid
            # job 10: two pointwise convs and a 3x3 average pool over one input in one call (the head of an inception module)
            c288, x288 = ls[6]
            w2 = rng.standard_normal((48, 288, 1, 1)).astype(np.float32) / 17.0
            second = ops.Conv2d(w2, None, act=ops.ACT_RELU, in_hw=(35, 35))
            ref_pool_convs, ref_pool = ops.conv2d_group_pool([c288, second], [x288, x288], x288, 3, 1, pad=1, is_avg=True, count_include_pad=False)
            torch.cuda.synchronize()
            got_pool_convs, got_pool = ops.conv2d_group_pool([c288, second], [x288, x288], x288, 3, 1, pad=1, is_avg=True, count_include_pad=False,
                                                             stream=q.handle, job_id=10 | NO_START, notifier=ctypes.c_void_p(lib.paella_ring_notifier(h, 9)))
            pool_wgs = (288 * 35 * 35 + 511) // 512
            grids[10] = c288.plan.dims.grid + second.plan.dims.grid + pool_wgs
            assert held(lib) == 10
            sent = lib.paella_pack_flush()
            assert sent == 2 and held(lib) == 0  # eight problems in the first launch; the pair, two convs and a pool in the second
            after = stats(lib)
            assert (after[0] - before[0], after[1] - before[1]) == (2, 13)
            per = lambda n: (n + batch - 1) // batch
            want_msgs = sum(2 * per(grids[j]) for j in range(1, 9)) + per(grids[9]) + per(grids[10])
            buf = np.zeros(want_msgs, np.uint64)
            assert lib.paella_ring_drain(h, buf.ctypes.data, want_msgs, 20.0) == want_msgs
            m = decode(buf)
            for j in range(1, 11):
                ends = (m["job_id"] == j) & (m["is_start"] == 0)
                starts = (m["job_id"] == j) & (m["is_start"] == 1)
                assert m["num"][ends].sum() == grids[j], j
                assert m["num"][starts].sum() == (grids[j] if j < 9 else 0), j
                assert ends.sum() == per(grids[j])
            extra = np.zeros(1, np.uint64)
            assert lib.paella_ring_drain(h, extra.ctypes.data, 1, 0.05) == 0  # nothing else was sent
        finally:
            lib.paella_pack_enable(0)
    torch.cuda.synchronize()
    for a, b in zip(alone, outs):
        assert torch.equal(a, b)
    for a, b in zip(ref_pool_convs + [ref_pool], got_pool_convs + [got_pool]):
        assert torch.equal(a, b)


def test_poll_sends_at_once_on_idle_queues_and_ordered_queues_are_not_held(ring, cuda):
    lib, h = ring
    from paella_amd import ops
    rng = np.random.default_rng(12)
    ls = layers(cuda, rng)[:3]
    alone = [conv(x) for conv, x in ls]
    torch.cuda.synchronize()
    with ops.DirectQueue() as q, ops.DirectQueue(ordered=True) as qo:
        assert lib.paella_pack_enable(1) == 0
        try:
            y_ordered = ls[0][0](ls[0][1], stream=qo.handle)  # ordered queue: launched at once
            assert held(lib) == 0
            qo.wait()
            assert torch.equal(y_ordered, alone[0])
            ys = [torch.zeros_like(a) for a in alone]
            for k, (conv, x) in enumerate(ls):
                conv(x, out=ys[k], stream=q.handle, job_id=(k + 1) | NO_START, notifier=ctypes.c_void_p(lib.paella_ring_notifier(h, k)))
            assert held(lib) == 3
            assert lib.paella_pack_poll() == 1 and held(lib) == 0  # no queue has anything waiting: one launch of three problems
            batch = lib.paella_ring_batch_size()
            want = sum((c.plan.dims.grid + batch - 1) // batch for c, _ in ls)
            buf = np.zeros(want, np.uint64)
            assert lib.paella_ring_drain(h, buf.ctypes.data, want, 20.0) == want
            # a HIP stream is never held
            y_stream = ls[1][0](ls[1][1])
            assert held(lib) == 0
        finally:
            lib.paella_pack_enable(0)
    torch.cuda.synchronize()
    for a, b in zip(alone, ys):
        assert torch.equal(a, b)
    assert torch.equal(y_stream, alone[1])


def small_net(cuda, rng):
    """The small CNN's operators (conv 5x5, max pool, conv 5x5, max pool, dense) as library calls on one stream or queue."""
    from paella_amd import ops
    w1 = rng.standard_normal((8, 1, 5, 5)).astype(np.float32) * 0.2
    w2 = rng.standard_normal((16, 8, 5, 5)).astype(np.float32) * 0.07
    c1 = ops.Conv2d(w1, rng.standard_normal(8).astype(np.float32), pad=2, act=ops.ACT_RELU, in_hw=(28, 28))
    c2 = ops.Conv2d(w2, rng.standard_normal(16).astype(np.float32), pad=2, act=ops.ACT_RELU, in_hw=(14, 14))
    wd = torch.tensor(rng.standard_normal((10, 256)).astype(np.float32) * 0.06, device=cuda)
    bd = torch.tensor(rng.standard_normal(10).astype(np.float32), device=cuda)

    keep = []  # held launches read and write the intermediate tensors long after this function has returned

    def run(x, stream=None, job_id=0, notifier=None, gap=False):
        y1 = c1(x, stream=stream)
        y2 = ops.pool2d(y1, 2, 2, stream=stream)
        y3 = c2(y2, stream=stream)
        y4 = ops.pool2d(y3, 3, 3, stream=stream)
        keep.extend([y1, y2, y3, y4])
        if gap:  # an operator the recorder does not take
            g = ops.global_avgpool(y4, stream=stream)
        out = ops.dense(y4.reshape(1, 256), wd, bd, stream=stream, job_id=job_id, notifier=notifier)
        return (out, g) if gap else out
    return run


def test_recorded_sequences_of_several_requests_go_out_together(ring, cuda):
    lib, h = ring
    from paella_amd import ops
    rng = np.random.default_rng(13)
    net = small_net(cuda, rng)
    xs = [torch.tensor(rng.standard_normal((1, 1, 28, 28)).astype(np.float32), device=cuda) for _ in range(11)]
    alone = [net(x) for x in xs]
    torch.cuda.synchronize()
    key = ctypes.c_void_p(0x1234)
    with ops.DirectQueue(ordered=True) as q:
        assert lib.paella_pack_sequence_begin(key, ctypes.c_void_p(q.handle)) == -2  # packing is off on this thread
        assert lib.paella_pack_enable(1) == 0
        try:
            before = stats(lib)
            outs = []
            for j, x in enumerate(xs):
                assert lib.paella_pack_sequence_begin(key, ctypes.c_void_p(q.handle)) == 0
                outs.append(net(x, stream=q.handle, job_id=(j + 1) | NO_START, notifier=ctypes.c_void_p(lib.paella_ring_notifier(h, j))))
                assert lib.paella_pack_sequence_end() == 0
            assert held(lib) == 11
            assert lib.paella_pack_poll() == 10 and held(lib) == 0  # idle queues: eight requests in five launches, three in five more
            after = stats(lib)
            assert (after[0] - before[0], after[1] - before[1]) == (10, 55)
            buf = np.zeros(11, np.uint64)
            assert lib.paella_ring_drain(h, buf.ctypes.data, 11, 20.0) == 11  # one end message per request: its dense layer's three workgroups, as launched alone
            m = decode(buf)
            assert sorted(m["job_id"]) == list(range(1, 12)) and np.all(m["num"] == 3) and np.all(m["is_start"] == 0)
            # a sequence with an operator the recorder does not take: sent at once, in order, nothing held
            assert lib.paella_pack_sequence_begin(key, ctypes.c_void_p(q.handle)) == 0
            out_gap, g = net(xs[0], stream=q.handle, gap=True)
            assert lib.paella_pack_sequence_end() == 0 and held(lib) == 0
            q.wait()
            assert torch.equal(out_gap, alone[0])
        finally:
            lib.paella_pack_enable(0)
    torch.cuda.synchronize()
    for a, b in zip(alone, outs):
        assert torch.equal(a, b)


def test_convs_with_a_fused_input_transform_are_packed_among_themselves(ring, cuda):
    lib, h = ring
    from paella_amd import ops
    rng = np.random.default_rng(14)
    cases = []
    for c, k, hw, r, pad in [(256, 128, 14, 1, 0), (128, 32, 14, 3, 1), (512, 128, 7, 1, 0), (128, 32, 28, 3, 1), (64, 128, 56, 1, 0)]:
        w = rng.standard_normal((k, c, r, r)).astype(np.float32) / np.sqrt(c * r * r)
        conv = ops.Conv2d(w, None, pad=pad, in_hw=(hw, hw))
        assert conv.takes_input_transform()
        x = torch.tensor(rng.standard_normal((1, c, hw, hw)).astype(np.float32), device=cuda)
        sc = torch.tensor(rng.uniform(0.5, 1.5, c).astype(np.float32), device=cuda)
        sh = torch.tensor(rng.standard_normal(c).astype(np.float32) * 0.1, device=cuda)
        cases.append((conv, x, sc, sh))
    alone = [conv(x, in_scale=sc, in_shift=sh, in_act=ops.ACT_RELU) for conv, x, sc, sh in cases]
    torch.cuda.synchronize()
    batch = lib.paella_ring_batch_size()
    with ops.DirectQueue() as q:
        assert lib.paella_pack_enable(1) == 0
        try:
            before = stats(lib)
            outs = []
            for j, (conv, x, sc, sh) in enumerate(cases):
                y = torch.zeros_like(alone[j])
                conv(x, out=y, stream=q.handle, job_id=(j + 1) | NO_START, notifier=ctypes.c_void_p(lib.paella_ring_notifier(h, j)),
                     in_scale=sc, in_shift=sh, in_act=ops.ACT_RELU)
                outs.append(y)
            assert held(lib) == 5
            assert lib.paella_pack_flush() == 1 and held(lib) == 0
            after = stats(lib)
            assert (after[0] - before[0], after[1] - before[1]) == (1, 5)
            want = sum((c[0].plan.dims.grid + batch - 1) // batch for c in cases)
            buf = np.zeros(want, np.uint64)
            assert lib.paella_ring_drain(h, buf.ctypes.data, want, 20.0) == want
            m = decode(buf)
            for j, c in enumerate(cases):
                assert m["num"][m["job_id"] == j + 1].sum() == c[0].plan.dims.grid
        finally:
            lib.paella_pack_enable(0)
    torch.cuda.synchronize()
    for a, b in zip(alone, outs):
        assert torch.equal(a, b)


def test_depthwise_convs_are_packed_among_themselves(ring, cuda):
    """Depthwise convs of several jobs in one launch (dwconv_group_kernel): bit-identical to launches of their own -- the small
    layers with one output per thread and the large ones with four -- and every notifier counts its own workgroups; a depthwise
    conv alone in the list goes out through the plain kernel."""
    lib, h = ring
    from paella_amd import ops
    rng = np.random.default_rng(17)
    cases = []
    for c, hw, stride, act in [(32, 112, 1, ops.ACT_RELU6), (96, 112, 2, ops.ACT_RELU6), (144, 56, 1, ops.ACT_RELU6), (192, 28, 2, ops.ACT_NONE),
                               (384, 14, 1, ops.ACT_RELU6), (960, 7, 1, ops.ACT_RELU), (24, 19, 1, ops.ACT_RELU)]:
        w = rng.standard_normal((c, 1, 3, 3)).astype(np.float32) / 3.0
        b = rng.standard_normal(c).astype(np.float32)
        conv = ops.Conv2d(w, b, stride=stride, pad=1, groups=c, act=act, in_hw=(hw, hw))
        assert conv.plan.kind == 1
        x = torch.tensor(rng.standard_normal((1, c, hw, hw)).astype(np.float32), device=cuda)
        cases.append((conv, x))
    assert any(c.plan.dims.grid * 256 < c.plan.d.K * c.plan.P * c.plan.Q for c, _ in cases)      # four outputs per thread
    assert any(c.plan.dims.grid * 256 >= c.plan.d.K * c.plan.P * c.plan.Q for c, _ in cases)     # one output per thread
    alone = [conv(x) for conv, x in cases]
    torch.cuda.synchronize()
    batch = lib.paella_ring_batch_size()
    with ops.DirectQueue() as q:
        assert lib.paella_pack_enable(1) == 0
        try:
            before = stats(lib)
            outs = []
            for j, (conv, x) in enumerate(cases):
                y = torch.zeros_like(alone[j])
                conv(x, out=y, stream=q.handle, job_id=(j + 1) | NO_START, notifier=ctypes.c_void_p(lib.paella_ring_notifier(h, j)))
                outs.append(y)
            assert held(lib) == len(cases)
            assert lib.paella_pack_flush() == 1 and held(lib) == 0
            after = stats(lib)
            assert (after[0] - before[0], after[1] - before[1]) == (1, len(cases))
            want = sum((c[0].plan.dims.grid + batch - 1) // batch for c in cases)
            buf = np.zeros(want, np.uint64)
            assert lib.paella_ring_drain(h, buf.ctypes.data, want, 20.0) == want
            m = decode(buf)
            for j, c in enumerate(cases):
                assert m["num"][m["job_id"] == j + 1].sum() == c[0].plan.dims.grid
            # one alone: the plain kernel, same bits
            y = torch.zeros_like(alone[0])
            cases[0][0](cases[0][1], out=y, stream=q.handle, job_id=9 | NO_START, notifier=ctypes.c_void_p(lib.paella_ring_notifier(h, 9)))
            assert held(lib) == 1 and lib.paella_pack_flush() == 1
            want = (cases[0][0].plan.dims.grid + batch - 1) // batch
            buf = np.zeros(want, np.uint64)
            assert lib.paella_ring_drain(h, buf.ctypes.data, want, 20.0) == want
            assert torch.equal(y, alone[0])
        finally:
            lib.paella_pack_enable(0)
    torch.cuda.synchronize()
    for a, b in zip(alone, outs):
        assert torch.equal(a, b)


@pytest.mark.parametrize("seed", [21, 22, 23])
def test_random_mixes_of_calls_pack_to_the_bits_of_separate_launches(ring, cuda, seed):
    """Seeded mixes of single convs (both reduction orders, 2 to 8 waves), pairs and conv + pool calls, each under its own job id:
    whatever way the packer cuts them into launches, outputs equal those of separate launches bit for bit and every notifier
    counts exactly its own workgroups."""
    lib, h = ring
    from paella_amd import ops
    rng = np.random.default_rng(seed)

    def conv_of(c, k, hw, r, stride=1):
        w = rng.standard_normal((k, c, r, r)).astype(np.float32) / np.sqrt(c * r * r)
        b = rng.standard_normal(k).astype(np.float32) if rng.random() < 0.7 else None
        conv = ops.Conv2d(w, b, stride=stride, pad=r // 2, act=ops.ACT_RELU if rng.random() < 0.5 else ops.ACT_NONE, in_hw=(hw, hw))
        assert (conv.plan.mi, conv.plan.ni) == (1, 1)
        x = torch.tensor(rng.standard_normal((1, c, hw, hw)).astype(np.float32), device=cuda)
        return conv, x

    calls = []  # (kind, [(conv, x), ...])
    for _ in range(14):
        kind = rng.choice(["single", "single", "single", "pair", "pool"])
        hw = int(rng.choice([7, 9, 14, 17, 28, 35]))
        if kind == "single":
            c = int(rng.choice([3, 5, 8, 16, 24, 64, 160, 512]))
            calls.append(("single", [conv_of(c, int(rng.choice([8, 24, 40, 96, 200])), hw, int(rng.choice([1, 3])), int(rng.choice([1, 2])))]))
        else:
            c = int(rng.choice([16, 64, 192]))  # tap-major, eight waves: what the executor groups
            members = [conv_of(c, int(rng.choice([32, 48, 96])), hw, 1) for _ in range(2)]
            if members[0][0].plan.kw != members[1][0].plan.kw:
                continue
            members[1] = (members[1][0], members[0][1])  # both read one input, as the branches of a module do
            calls.append((kind, members))
    alone = []
    for kind, members in calls:
        ys = [conv(x) for conv, x in members]
        if kind == "pool":
            ys.append(ops.pool2d(members[0][1], 3, 1, pad=1, is_avg=True, count_include_pad=False))
        alone.append(ys)
    torch.cuda.synchronize()
    batch = lib.paella_ring_batch_size()
    per = lambda n: (n + batch - 1) // batch
    with ops.DirectQueue() as q:
        assert lib.paella_pack_enable(1) == 0
        try:
            got, grids = [], []
            for j, (kind, members) in enumerate(calls):
                nf = ctypes.c_void_p(lib.paella_ring_notifier(h, j))
                jid = (j + 1) | NO_START
                if kind == "single":
                    conv, x = members[0]
                    got.append([conv(x, stream=q.handle, job_id=jid, notifier=nf)])
                    grids.append(conv.plan.dims.grid)
                elif kind == "pair":
                    got.append(ops.conv2d_group([m[0] for m in members], [m[1] for m in members], stream=q.handle, job_id=jid, notifier=nf))
                    grids.append(sum(m[0].plan.dims.grid for m in members))
                else:
                    x = members[0][1]
                    ys, py = ops.conv2d_group_pool([m[0] for m in members], [x, x], x, 3, 1, pad=1, is_avg=True, count_include_pad=False,
                                                   stream=q.handle, job_id=jid, notifier=nf)
                    got.append(ys + [py])
                    block = 64 * members[0][0].plan.kw
                    grids.append(sum(m[0].plan.dims.grid for m in members) + (x.shape[1] * x.shape[2] * x.shape[3] + block - 1) // block)
            assert held(lib) == len(calls)
            assert lib.paella_pack_flush() >= 1 and held(lib) == 0
            want = sum(per(g) for g in grids)
            buf = np.zeros(want, np.uint64)
            assert lib.paella_ring_drain(h, buf.ctypes.data, want, 20.0) == want
            m = decode(buf)
            for j, g in enumerate(grids):
                mine = m["job_id"] == j + 1
                assert m["num"][mine].sum() == g and mine.sum() == per(g) and np.all(m["is_start"][mine] == 0), (j, calls[j][0])
        finally:
            lib.paella_pack_enable(0)
    torch.cuda.synchronize()
    for ys, zs in zip(alone, got):
        for a, b in zip(ys, zs):
            assert torch.equal(a, b)

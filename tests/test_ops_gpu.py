"""Parity of the hand-written gfx950 operator kernels (through the C-ABI) against the CPU oracle.

Tolerance for fp32 outputs: |got - ref| <= 1e-4 + 1e-3 * |ref|  (max-abs 1e-4 / rel 1e-3).
Pure data-movement ops (max pool, copy) are bit-exact.
"""
import numpy as np
import pytest
import torch

from oracle import ops as orc

pytestmark = pytest.mark.gpu

ATOL, RTOL = 1e-4, 1e-3
RNG = np.random.default_rng(99)


def rnd(*shape, scale=1.0):
    return (RNG.standard_normal(shape) * scale).astype(np.float32)


def close(got, ref):
    got = got.detach().cpu().numpy() if hasattr(got, "detach") else got
    assert got.shape == ref.shape, (got.shape, ref.shape)
    err = np.abs(got.astype(np.float64) - ref.astype(np.float64))
    bound = ATOL + RTOL * np.abs(ref)
    assert np.all(err <= bound), "max err %g (bound there %g), %d bad of %d" % (err.max(), bound.flat[err.argmax()], (err > bound).sum(), err.size)


# C, H, W, K, R, S, stride, pad, dil  -- the layer shapes of the benchmark models plus ragged edge cases
CONV_SHAPES = [
    (1, 28, 28, 8, 5, 5, 1, 2, 1),          # small CNN conv1
    (8, 14, 14, 16, 5, 5, 1, 2, 1),         # small CNN conv2
    (3, 224, 224, 64, 7, 7, 2, 3, 1),       # ResNet stem
    (64, 56, 56, 64, 3, 3, 1, 1, 1),        # ResNet layer1
    (64, 56, 56, 128, 3, 3, 2, 1, 1),       # stage entry, stride 2
    (64, 56, 56, 128, 1, 1, 2, 0, 1),       # 1x1 stride-2 downsample
    (256, 14, 14, 256, 3, 3, 1, 1, 1),
    (512, 7, 7, 512, 3, 3, 1, 1, 1),        # 49 pixels: ragged pixel tile
    (3, 299, 299, 32, 3, 3, 2, 0, 1),       # Inception stem
    (128, 17, 17, 192, 1, 7, 1, (0, 3), 1),  # factorised 1x7
    (160, 17, 17, 160, 7, 1, 1, (3, 0), 1),  # factorised 7x1
    (48, 35, 35, 64, 5, 5, 1, 2, 1),
    (384, 8, 8, 384, 1, 3, 1, (0, 1), 1),
    (384, 8, 8, 384, 3, 1, 1, (1, 0), 1),
    (960, 7, 7, 320, 1, 1, 1, 0, 1),        # MobileNetV2 pointwise
    (24, 56, 56, 144, 1, 1, 1, 0, 1),
    (5, 9, 11, 7, 3, 3, 1, 1, 1),           # nothing is a multiple of anything
    (16, 12, 12, 40, 3, 3, 1, 2, 2),        # dilation
    (2048, 1, 1, 1000, 1, 1, 1, 0, 1),      # a dense layer expressed as 1x1 conv
    (288, 35, 35, 384, 3, 3, 2, 0, 1),      # Inception reduction: stride 2 without padding (filter columns 0 and 1 paired)
    (192, 17, 17, 320, 3, 3, 2, 0, 1),
    (256, 14, 14, 512, 3, 3, 2, 1, 1),      # residual stage entry: stride 2 with padding (columns 1 and 2 paired)
    (16, 9, 12, 40, 3, 3, 2, 1, 1),         # even width, ragged everything else
    (16, 9, 13, 40, 3, 3, 2, 1, 1),         # odd width with padding: the last pair would leave the image, so not paired
    (24, 11, 10, 33, 1, 3, (1, 2), (0, 1), 1),  # one filter row, stride 2 across only
    (8, 20, 20, 32, 3, 3, (1, 2), (1, 0), 1),   # stride 2 across, 1 down
]


def test_paired_filter_columns_are_planned_where_both_columns_stay_inside(cuda):
    """Stride 2 across a 3-wide filter with C a multiple of 8: paired when 2 Q <= W, first column = the padding."""
    from paella_amd import ops
    def planned(c, h, w, k, r, s, stride, pad):
        return ops.Conv2d(rnd(k, c, r, s), None, stride=stride, pad=pad, in_hw=(h, w)).plan.pair_taps
    assert planned(288, 35, 35, 384, 3, 3, 2, 0) == 1
    assert planned(256, 14, 14, 512, 3, 3, 2, 1) == 2
    assert planned(16, 9, 13, 40, 3, 3, 2, 1) == 0      # Q = 7, W = 13
    assert planned(16, 9, 12, 40, 3, 3, 1, 1) == 0      # stride 1
    assert planned(12, 9, 12, 40, 3, 3, 2, 1) == 0      # C no multiple of 8: the other reduction order
    assert planned(16, 9, 12, 40, 3, 5, 2, (1, 2)) == 0  # 5-wide filter


@pytest.mark.parametrize("shape", CONV_SHAPES)
def test_conv2d_mfma_parity(cuda, shape):
    from paella_amd import ops
    c, h, w, k, r, s, stride, pad, dil = shape
    x = rnd(1, c, h, w)
    wt = rnd(k, c, r, s, scale=(2.0 / (c * r * s)) ** 0.5)
    b = rnd(k, scale=0.1)
    ref = orc.conv2d(x, wt, b, stride=stride, pad=pad, dil=dil, act=orc.ACT_RELU)
    conv = ops.Conv2d(wt, b, stride=stride, pad=pad, dil=dil, act=ops.ACT_RELU, in_hw=(h, w))
    got = conv(torch.tensor(x, device=cuda))
    torch.cuda.synchronize()
    close(got, ref)


@pytest.mark.parametrize("mi,ni,kwlog", [(1, 1, 0), (1, 1, 1), (1, 1, 2), (1, 1, 3), (1, 2, 0), (1, 2, 2), (1, 2, 3),
                                         (2, 1, 1), (2, 1, 2), (2, 2, 0), (2, 2, 1), (2, 2, 2), (2, 2, 3), (2, 1, 3)])
def test_conv2d_every_tile_variant(cuda, mi, ni, kwlog):
    from paella_amd import ops
    c, h, w, k = 40, 19, 23, 72
    x, wt, b = rnd(1, c, h, w), rnd(k, c, 3, 3, scale=0.05), rnd(k, scale=0.1)
    res = rnd(1, k, h, w)
    slope = np.abs(rnd(k, scale=0.3))
    ref = orc.conv2d(x, wt, b, pad=1, act=orc.ACT_PRELU, residual=res, slope=slope)
    conv = ops.Conv2d(wt, b, pad=1, act=ops.ACT_PRELU, slope=slope, in_hw=(h, w), has_residual=True,
                      tile_hint=(mi << 8) | (ni << 4) | kwlog)
    assert (conv.plan.mi, conv.plan.ni, conv.plan.kw) == (mi, ni, 1 << kwlog)
    got = conv(torch.tensor(x, device=cuda), residual=torch.tensor(res, device=cuda))
    torch.cuda.synchronize()
    close(got, ref)


# C, H, W, K, R, S, stride, pad, input activation, waves (log2; -1: the library's choice), residual
TRANSFORMED = [
    (64, 56, 56, 128, 1, 1, 1, 0, orc.ACT_RELU, -1, False),    # DenseNet bottleneck: norm + ReLU in front of a 1x1
    (352, 14, 14, 128, 1, 1, 1, 0, orc.ACT_RELU, -1, False),
    (64, 28, 28, 64, 3, 3, 1, 1, orc.ACT_NONE, -1, False),     # ArcFace unit: norm in front of a zero-padded 3x3
    (128, 14, 14, 128, 3, 3, 2, 1, orc.ACT_NONE, -1, True),
    (512, 7, 7, 512, 3, 3, 1, 1, orc.ACT_NONE, -1, False),     # split reduction
    (40, 19, 23, 72, 3, 3, 1, 2, orc.ACT_RELU, 0, True),       # padding wider than the filter's reach; every wave count
    (40, 19, 23, 72, 3, 3, 1, 2, orc.ACT_RELU, 1, True),
    (40, 19, 23, 72, 3, 3, 1, 2, orc.ACT_NONE, 2, False),
    (40, 19, 23, 72, 5, 3, 2, (2, 1), orc.ACT_RELU, 3, True),
    (1024, 7, 7, 128, 1, 1, 1, 0, orc.ACT_RELU, -1, False),    # the widest table of scales and shifts in the zoo
    (8, 9, 11, 40, 3, 3, 1, 1, orc.ACT_NONE, 3, False),        # one chunk per tap: the tap changes with every chunk
    (64, 16, 16, 96, 3, 3, 2, 1, orc.ACT_RELU, -1, True),      # paired filter columns under the transform, with a bound
    (24, 12, 20, 48, 3, 3, 2, 0, orc.ACT_NONE, 1, False),      # paired, no padding, two waves
]


@pytest.mark.parametrize("case", TRANSFORMED)
def test_conv2d_on_transformed_input(cuda, case):
    """conv(act(x * scale + shift)) in one launch against the oracle's scale-shift followed by its conv.  The shifts are
    large and of both signs, so a padding tap that wrongly carried act(shift) instead of 0 would show at every border."""
    from paella_amd import ops
    c, h, w, k, r, s, stride, pad, in_act, kwlog, with_res = case
    x = rnd(1, c, h, w)
    wt, b = rnd(k, c, r, s, scale=(2.0 / (c * r * s)) ** 0.5), rnd(k, scale=0.1)
    scale, shift = rnd(c) + 1.5, rnd(c, scale=2.0)
    mid = orc.scale_shift(x, scale, shift, act=in_act)
    conv = ops.Conv2d(wt, b, stride=stride, pad=pad, act=ops.ACT_RELU, in_hw=(h, w), has_residual=with_res,
                      tile_hint=0 if kwlog < 0 else (1 << 8) | (1 << 4) | kwlog)
    assert conv.takes_input_transform()
    res = rnd(1, k, conv.plan.P, conv.plan.Q) if with_res else None
    ref = orc.conv2d(mid, wt, b, stride=stride, pad=pad, act=orc.ACT_RELU, residual=res)
    dev = lambda a: None if a is None else torch.tensor(a, device=cuda)
    got = conv(dev(x), residual=dev(res), in_scale=dev(scale), in_shift=dev(shift), in_act=in_act)
    torch.cuda.synchronize()
    close(got, ref)
    # and the two-launch form gives the same within the tolerance (the fused form rounds x * scale + shift once, as a
    # fused multiply-add)
    two = conv(ops.eltwise(dev(x), scale=dev(scale), shift=dev(shift), act=in_act), residual=dev(res))
    torch.cuda.synchronize()
    close(two, ref)


@pytest.mark.parametrize("n_convs,avg,kwlogs", [(3, False, (3, 3, 3)), (3, True, (2, 2, 2)), (1, False, (3,)), (2, True, (1, 1)), (1, True, (0,))])
def test_convs_and_a_pool_in_one_launch_change_no_bit(cuda, n_convs, avg, kwlogs):
    """An inception module's first launch: 1x1 convs and the 3x3 stride-1 pool, all reading the module's input, against the
    same operators launched one by one (and against the oracle)."""
    from paella_amd import ops
    c, h, w = 192, 35, 35
    x = rnd(1, c, h, w)
    ks = [64, 48, 96][:n_convs]
    convs, refs = [], []
    for k, kwlog in zip(ks, kwlogs):
        wt, b = rnd(k, c, 1, 1, scale=(2.0 / c) ** 0.5), rnd(k, scale=0.1)
        convs.append(ops.Conv2d(wt, b, act=ops.ACT_RELU, in_hw=(h, w), tile_hint=(1 << 8) | (1 << 4) | kwlog))
        refs.append(orc.conv2d(x, wt, b, act=orc.ACT_RELU))
    xd = torch.tensor(x, device=cuda)
    alone = [conv(xd) for conv in convs]
    pool_alone = ops.pool2d(xd, 3, 1, pad=1, is_avg=avg, count_include_pad=False)
    outs, pool_y = ops.conv2d_group_pool(convs, [xd] * n_convs, xd, 3, 1, pad=1, is_avg=avg, count_include_pad=False)
    torch.cuda.synchronize()
    for got, one, ref in zip(outs, alone, refs):
        assert torch.equal(got, one)
        close(got, ref)
    assert torch.equal(pool_y, pool_alone)
    pool_ref = orc.avgpool2d(x, 3, 1, pad=1, count_include_pad=False) if avg else orc.maxpool2d(x, 3, 1, pad=1)
    close(pool_y, pool_ref)


def test_convs_and_a_pool_in_one_launch_refuses_other_plans(cuda):
    from paella_amd import ops
    xd = torch.zeros((1, 5, 9, 11), device=cuda)
    table_order = ops.Conv2d(rnd(7, 5, 1, 1), None, in_hw=(9, 11))     # C is no multiple of 8
    with pytest.raises(RuntimeError):
        ops.conv2d_group_pool([table_order], [xd], xd, 3, 1, pad=1)
    x8 = torch.zeros((1, 8, 9, 11), device=cuda)
    a = ops.Conv2d(rnd(8, 8, 1, 1), None, in_hw=(9, 11), tile_hint=(1 << 8) | (1 << 4) | 1)
    b = ops.Conv2d(rnd(8, 8, 1, 1), None, in_hw=(9, 11), tile_hint=(1 << 8) | (1 << 4) | 2)   # another wave count
    with pytest.raises(RuntimeError):
        ops.conv2d_group_pool([a, b], [x8, x8], x8, 3, 1, pad=1)
    with pytest.raises(RuntimeError):
        ops.conv2d_group_pool([a, a, a, a], [x8] * 4, x8, 3, 1, pad=1)   # at most three convs beside a pool


def test_conv2d_input_transform_is_refused_where_not_built(cuda):
    from paella_amd import ops
    x = torch.zeros((1, 5, 9, 11), device=cuda)
    conv = ops.Conv2d(rnd(7, 5, 3, 3), None, pad=1, in_hw=(9, 11))      # C is no multiple of 8: offset-table order
    assert not conv.takes_input_transform()
    ones = torch.ones(5, device=cuda)
    with pytest.raises(RuntimeError):
        conv(x, in_scale=ones, in_shift=ones)
    big = ops.Conv2d(rnd(72, 40, 3, 3), None, pad=1, in_hw=(19, 23), tile_hint=(2 << 8) | (1 << 4) | 2)   # 64 x 32 tile
    assert not big.takes_input_transform()
    conv8 = ops.Conv2d(rnd(8, 8, 3, 3), None, pad=1, in_hw=(9, 11))
    ones8 = torch.ones(8, device=cuda)
    with pytest.raises(RuntimeError):
        conv8(torch.zeros((1, 8, 9, 11), device=cuda), in_scale=ones8, in_shift=ones8, in_act=ops.ACT_RELU6)


@pytest.mark.parametrize("act", [orc.ACT_NONE, orc.ACT_RELU6, orc.ACT_CLIP])
def test_conv2d_epilogues_and_channel_slice_output(cuda, act):
    """Output written into channels [8, 8+24) of a 40-channel concat buffer; the rest must stay untouched."""
    from paella_amd import ops
    c, h, w, k = 16, 10, 10, 24
    x, wt = rnd(1, c, h, w, scale=3.0), rnd(k, c, 3, 3, scale=0.3)
    ref = orc.conv2d(x, wt, None, pad=1, act=act, lo=-1.0, hi=2.0)
    conv = ops.Conv2d(wt, None, pad=1, act=act, lo=-1.0, hi=2.0, in_hw=(h, w))
    buf = torch.full((1, 40, h, w), 7.0, device=cuda)
    conv(torch.tensor(x, device=cuda), out=buf[:, 8:32])
    torch.cuda.synchronize()
    out = buf.cpu().numpy()
    close(out[:, 8:32], ref)
    assert np.all(out[:, :8] == 7.0) and np.all(out[:, 32:] == 7.0)


def test_conv2d_is_deterministic(cuda):
    from paella_amd import ops
    x, wt = rnd(1, 64, 28, 28), rnd(96, 64, 3, 3, scale=0.05)
    conv = ops.Conv2d(wt, None, pad=1, in_hw=(28, 28))
    xd = torch.tensor(x, device=cuda)
    a = conv(xd).cpu()
    for _ in range(3):
        assert torch.equal(conv(xd).cpu(), a)


# (first conv, second conv): C, H, W, K, R, stride, pad, tile_hint -- both on the 32 x 32 tile with the same wave count
PAIRS = [
    ((64, 56, 56, 128, 3, 2, 1, 0x1113), (64, 56, 56, 128, 1, 2, 0, 0x113)),     # residual block entry and its projection: split 3x3 + tiny 1x1
    ((256, 14, 14, 512, 3, 2, 1, 0x3113), (256, 14, 14, 512, 1, 2, 0, 0x1113)),  # both split over the reduction
    ((192, 35, 35, 64, 1, 1, 0, 0x112), (192, 35, 35, 48, 1, 1, 0, 0x112)),      # two branches of an inception module
    ((5, 9, 11, 7, 3, 1, 1, 0x111), (3, 13, 7, 40, 3, 1, 1, 0x111)),             # reduction order (c, r, s), different inputs
    ((24, 20, 20, 33, 3, 1, 1, 0x110), (16, 9, 9, 70, 1, 1, 0, 0x110)),          # one wave per workgroup
]


@pytest.mark.parametrize("pair", PAIRS)
def test_two_convs_in_one_launch_equal_two_launches_bit_for_bit(cuda, pair):
    from paella_amd import ops
    convs, xs, res, refs = [], [], [], []
    for idx, (c, h, w, k, r, stride, pad, hint) in enumerate(pair):
        x = rnd(1, c, h, w)
        wt = rnd(k, c, r, r, scale=(2.0 / (c * r * r)) ** 0.5)
        b = rnd(k, scale=0.1)
        conv = ops.Conv2d(wt, b, stride=stride, pad=pad, act=ops.ACT_RELU if idx == 0 else ops.ACT_NONE, in_hw=(h, w),
                          has_residual=idx == 1, tile_hint=hint)
        assert (conv.plan.mi, conv.plan.ni, conv.plan.kw, conv.plan.splits > 1) == (1, 1, 1 << (hint & 15), (hint >> 12) > 0)
        convs.append(conv)
        xs.append(torch.tensor(x, device=cuda))
        r_np = rnd(1, k, conv.plan.P, conv.plan.Q) if idx == 1 else None
        res.append(None if r_np is None else torch.tensor(r_np, device=cuda))
        refs.append(orc.conv2d(x, wt, b, stride=stride, pad=pad, act=orc.ACT_RELU if idx == 0 else orc.ACT_NONE, residual=r_np))
    rc, dims = ops.pair_dims(convs[0], convs[1])
    assert rc == 0 and dims.grid == convs[0].plan.dims.grid + convs[1].plan.dims.grid and dims.block == convs[0].plan.dims.block
    alone = [convs[0](xs[0]).clone(), convs[1](xs[1], residual=res[1]).clone()]
    for _ in range(2):  # the second call finds the split counters as the first left them
        y1, y2 = ops.conv2d_pair(convs[0], xs[0], convs[1], xs[1], residual2=res[1])
        torch.cuda.synchronize()
        assert torch.equal(y1, alone[0]) and torch.equal(y2, alone[1])
    close(y1, refs[0])
    close(y2, refs[1])


@pytest.mark.parametrize("count", [3, 4])
def test_group_of_convs_in_one_launch_equals_separate_launches_bit_for_bit(cuda, count):
    """Branches of an inception module: 1x1, 1x1 ahead of a 5x5, 1x1 ahead of a 3x3, 1x1 behind a pool, one of them split
    over the reduction; every member on its own workspace."""
    from paella_amd import ops
    shapes = [(192, 35, 35, 64, 1, 0, 0x113), (192, 35, 35, 48, 1, 0, 0x1113), (96, 35, 35, 96, 3, 1, 0x113), (192, 35, 35, 32, 1, 0, 0x113)][:count]
    convs, xs, alone, refs = [], [], [], []
    for c, h, w, k, r, pad, hint in shapes:
        x, wt, b = rnd(1, c, h, w), rnd(k, c, r, r, scale=(2.0 / (c * r * r)) ** 0.5), rnd(k, scale=0.1)
        conv = ops.Conv2d(wt, b, pad=pad, act=ops.ACT_RELU, in_hw=(h, w), tile_hint=hint)
        convs.append(conv)
        xs.append(torch.tensor(x, device=cuda))
        alone.append(conv(xs[-1]).clone())
        refs.append(orc.conv2d(x, wt, b, pad=pad, act=orc.ACT_RELU))
    for _ in range(2):
        outs = ops.conv2d_group(convs, xs)
        torch.cuda.synchronize()
        for got, want, ref in zip(outs, alone, refs):
            assert torch.equal(got, want)
            close(got, ref)


def test_pair_launch_refuses_plans_that_do_not_match(cuda):
    from paella_amd import ops
    a = ops.Conv2d(rnd(64, 64, 3, 3), None, pad=1, in_hw=(28, 28), tile_hint=0x113)
    b = ops.Conv2d(rnd(64, 64, 1, 1), None, in_hw=(28, 28), tile_hint=0x112)      # other wave count
    c = ops.Conv2d(rnd(64, 64, 3, 3), None, pad=1, in_hw=(28, 28), tile_hint=0x123)  # larger tile
    d = ops.Conv2d(rnd(64, 3, 3, 3), None, pad=1, in_hw=(28, 28), tile_hint=0x113)   # other reduction order
    for other in (b, c, d):
        assert ops.pair_dims(a, other)[0] == -2
    x = torch.zeros(1, 64, 28, 28, device=cuda)
    with pytest.raises(RuntimeError, match="unsupported"):
        ops.conv2d_pair(a, x, b, x)


@pytest.mark.parametrize("shape", [(64, 56, 56, 64, 3, 1, 1), (8, 9, 9, 40, 1, 1, 0), (2048, 1, 1, 1000, 1, 1, 0), (5, 9, 11, 7, 3, 1, 1),
                                   (256, 14, 14, 256, 3, 2, 1), (16, 33, 1, 24, 3, 1, 1)])
def test_conv2d_index_arithmetic_shortcut_changes_no_bit(cuda, shape):
    """The kernel divides by multiply-high with constants from the host; plan.fast_div = 0 makes it divide.
    Divisors of 1 (one output column, 1x1 filters, 8 input channels, a single tile) are the special case of the shortcut."""
    from paella_amd import ops
    c, h, w, k, r, stride, pad = shape
    x, wt, b = rnd(1, c, h, w), rnd(k, c, r, r, scale=(2.0 / (c * r * r)) ** 0.5), rnd(k, scale=0.1)
    conv = ops.Conv2d(wt, b, stride=stride, pad=pad, act=ops.ACT_RELU, in_hw=(h, w))
    xd = torch.tensor(x, device=cuda)
    fast = conv(xd).clone()
    assert conv.plan.fast_div == 1
    conv.plan.fast_div = 0
    slow = conv(xd).clone()
    torch.cuda.synchronize()
    assert torch.equal(fast, slow)
    close(fast, orc.conv2d(x, wt, b, stride=stride, pad=pad, act=orc.ACT_RELU))


def test_conv2d_rejects_what_it_does_not_implement(cuda):
    from paella_amd import ops
    with pytest.raises(RuntimeError, match="unsupported"):
        ops.Conv2d(rnd(8, 2, 3, 3), None, groups=4, in_hw=(8, 8))
    with pytest.raises(RuntimeError, match="invalid"):
        ops.Conv2d(rnd(8, 8, 3, 3), None, stride=0, in_hw=(8, 8))


# every depthwise layer shape of MobileNetV2 and of the face detector's backbone, plus ragged cases: odd widths, two channels, a
# filter larger than the image, dilation, no padding, a very wide image
DEPTHWISE = [(32, 112, 112, 3, 1, 1, 1), (96, 112, 112, 3, 2, 1, 1), (144, 56, 56, 3, 1, 1, 1), (144, 56, 56, 3, 2, 1, 1), (192, 28, 28, 3, 1, 1, 1),
             (192, 28, 28, 3, 2, 1, 1), (384, 14, 14, 3, 1, 1, 1), (576, 14, 14, 3, 2, 1, 1), (960, 7, 7, 3, 1, 1, 1), (16, 120, 160, 3, 2, 1, 1),
             (64, 30, 40, 3, 1, 1, 1), (7, 13, 9, 3, 2, 1, 1), (16, 20, 20, 5, 1, 2, 1), (2, 5, 3, 3, 1, 1, 1), (3, 2, 2, 3, 1, 1, 1), (5, 17, 31, 3, 1, 2, 2),
             (9, 11, 11, 3, 1, 0, 1), (2, 1, 1, 3, 1, 1, 1), (33, 9, 600, 3, 1, 1, 1)]


@pytest.mark.parametrize("c,h,w,r,stride,pad,dil", DEPTHWISE)
def test_depthwise_conv_parity(cuda, c, h, w, r, stride, pad, dil):
    from paella_amd import ops
    x, wt, b = rnd(1, c, h, w), rnd(c, 1, r, r, scale=0.3), rnd(c, scale=0.1)
    ref = orc.conv2d(x, wt, b, stride=stride, pad=pad, dil=dil, groups=c, act=orc.ACT_RELU6)
    conv = ops.Conv2d(wt, b, stride=stride, pad=pad, dil=dil, groups=c, act=ops.ACT_RELU6, in_hw=(h, w))
    assert conv.plan.kind == 1
    close(conv(torch.tensor(x, device=cuda)), ref)


@pytest.mark.parametrize("i,o", [(256, 10), (512, 1000), (2048, 1000), (1280, 1000), (25088, 512), (37, 11), (25088, 511), (8192, 3), (8196, 5), (9001, 4),
                                 (16388, 1)])
def test_dense_parity(cuda, i, o):
    from paella_amd import ops
    x, w, b = rnd(1, i), rnd(o, i, scale=i ** -0.5), rnd(o)
    ref = orc.dense(x, w, b)
    got = ops.dense(torch.tensor(x, device=cuda), torch.tensor(w, device=cuda), torch.tensor(b, device=cuda))
    close(got, ref)


POOLS = [
    # c, h, w, k, stride, pad, ceil, avg, count_include_pad
    (8, 28, 28, 2, 2, 0, False, False, True),
    (16, 14, 14, 3, 3, 0, False, False, True),
    (64, 112, 112, 3, 2, 1, False, False, True),
    (64, 111, 111, 3, 2, 0, True, False, True),
    (192, 28, 28, 3, 1, 1, False, False, True),
    (64, 147, 147, 3, 2, 0, False, False, True),
    (128, 56, 56, 2, 2, 0, False, True, True),
    (288, 35, 35, 3, 1, 1, False, True, False),
    (288, 35, 35, 3, 1, 1, False, True, True),
    (5, 13, 15, 3, 2, 1, True, True, True),
    (5, 13, 15, 3, 2, 0, True, True, False),
]


@pytest.mark.parametrize("case", POOLS)
def test_pool_parity(cuda, case):
    from paella_amd import ops
    c, h, w, k, stride, pad, ceil, avg, cip = case
    x = rnd(1, c, h, w)
    got = ops.pool2d(torch.tensor(x, device=cuda), k, stride, pad, ceil, avg, cip).cpu().numpy()
    if avg:
        close(got, orc.avgpool2d(x, k, stride, pad, ceil, cip))
    else:
        np.testing.assert_array_equal(got, orc.maxpool2d(x, k, stride, pad, ceil))


def test_global_avgpool_eltwise_copy_softmax_lrn_parity(cuda):
    from paella_amd import ops
    for c, hw in [(512, 7), (2048, 8), (1000, 13), (3, 5)]:
        x = rnd(1, c, hw, hw)
        close(ops.global_avgpool(torch.tensor(x, device=cuda)), orc.global_avgpool(x))
    for shape in [(1, 64, 56, 56), (1, 7, 5, 3)]:
        a, b = rnd(*shape), rnd(*shape)
        c = shape[1]
        sc, sf, sl = rnd(c), rnd(c), np.abs(rnd(c))
        ad, bd = torch.tensor(a, device=cuda), torch.tensor(b, device=cuda)
        close(ops.eltwise(ad, bd, act=ops.ACT_RELU), orc.add(a, b, orc.ACT_RELU))
        close(ops.eltwise(ad, scale=torch.tensor(sc, device=cuda), shift=torch.tensor(sf, device=cuda), act=ops.ACT_RELU),
              orc.scale_shift(a, sc, sf, orc.ACT_RELU))
        close(ops.eltwise(ad, slope=torch.tensor(sl, device=cuda), act=ops.ACT_PRELU), orc.scale_shift(a, None, None, orc.ACT_PRELU, sl))
        close(ops.eltwise(ad, act=ops.ACT_CLIP, lo=-0.3, hi=0.6), orc.scale_shift(a, None, None, orc.ACT_CLIP, None, -0.3, 0.6))
        assert torch.equal(ops.copy(ad), ad)
    z = rnd(1, 1000, scale=4.0)
    close(ops.softmax(torch.tensor(z, device=cuda)), orc.softmax(z))
    z2 = rnd(4420, 2, scale=3.0)
    close(ops.softmax(torch.tensor(z2, device=cuda)), orc.softmax(z2))
    for rows, cols in [(1, 1), (257, 8), (300, 9), (5, 3)]:   # either side of the short-row kernel's limit, ragged row counts
        z3 = rnd(rows, cols, scale=3.0)
        close(ops.softmax(torch.tensor(z3, device=cuda)), orc.softmax(z3))
    x = rnd(1, 64, 28, 28, scale=3.0)
    close(ops.lrn(torch.tensor(x, device=cuda), 5, 1e-4, 0.75, 1.0), orc.lrn(x, 5, 1e-4, 0.75, 1.0))
    close(ops.lrn(torch.tensor(x, device=cuda), 4, 0.3, 0.6, 2.0), orc.lrn(x, 4, 0.3, 0.6, 2.0))


def test_conv_linearity_at_full_size(cuda):
    """Size-independent property at a full-size layer: conv(x, w1 + w2) == conv(x, w1) + conv(x, w2)."""
    from paella_amd import ops
    x = torch.tensor(rnd(1, 64, 112, 112), device=cuda)
    w1, w2 = rnd(64, 64, 3, 3, scale=0.05), rnd(64, 64, 3, 3, scale=0.05)
    ya = ops.Conv2d(w1 + w2, None, pad=1, in_hw=(112, 112))(x)
    yb = ops.Conv2d(w1, None, pad=1, in_hw=(112, 112))(x) + ops.Conv2d(w2, None, pad=1, in_hw=(112, 112))(x)
    close(ya, yb.cpu().numpy())


def test_random_conv_shapes_match_the_oracle(cuda):
    """200 seeded shapes over channel counts on both reduction orders, strides, paddings past the filter's reach, dilations,
    bias / residual / activation present or not: whatever plan they get (split reductions, paired filter columns)."""
    from paella_amd import ops
    rng = np.random.default_rng(7)
    paired = split = done = 0
    while done < 200:
        c = int(rng.choice([3, 5, 8, 16, 24, 40, 64, 96, 128, 256]))
        k = int(rng.integers(1, 130))
        r, s = int(rng.choice([1, 3, 5])), int(rng.choice([1, 3, 3, 3, 5, 7]))
        sh, sw = int(rng.choice([1, 2])), int(rng.choice([1, 2, 2]))
        ph, pw = int(rng.integers(0, r // 2 + 2)), int(rng.integers(0, s // 2 + 2))
        dh, dw = int(rng.choice([1, 1, 2])), int(rng.choice([1, 1, 1, 2]))
        h, w = int(rng.integers(1, 40)), int(rng.integers(1, 40))
        if h + 2 * ph - (r - 1) * dh - 1 < 0 or w + 2 * pw - (s - 1) * dw - 1 < 0:
            continue
        done += 1
        act = int(rng.choice([orc.ACT_NONE, orc.ACT_RELU, orc.ACT_RELU6]))
        x = rng.standard_normal((1, c, h, w)).astype(np.float32)
        wt = (rng.standard_normal((k, c, r, s)) * (2.0 / (c * r * s)) ** 0.5).astype(np.float32)
        b = None if rng.random() < 0.3 else (rng.standard_normal(k) * 0.1).astype(np.float32)
        ref = orc.conv2d(x, wt, b, stride=(sh, sw), pad=(ph, pw), dil=(dh, dw))
        res = rng.standard_normal(ref.shape).astype(np.float32) if rng.random() < 0.3 else None
        if res is not None:
            ref = ref + res
        ref = np.maximum(ref, 0) if act != orc.ACT_NONE else ref
        ref = np.minimum(ref, 6) if act == orc.ACT_RELU6 else ref
        conv = ops.Conv2d(wt, b, stride=(sh, sw), pad=(ph, pw), dil=(dh, dw), act=act, in_hw=(h, w), has_residual=res is not None)
        paired += conv.plan.pair_taps != 0
        split += conv.plan.splits > 1
        got = conv(torch.tensor(x, device=cuda), residual=None if res is None else torch.tensor(res, device=cuda))
        torch.cuda.synchronize()
        close(got, ref.astype(np.float32))
    assert paired >= 10 and split >= 50   # the sweep reaches both


def test_random_transformed_input_conv_shapes_match_the_oracle(cuda):
    """120 seeded shapes of conv(act(x * scale + shift)) in one launch: channel counts from one chunk per tap to a table of 512
    entries, every wave count, strides with and without paired filter columns, paddings past the filter's reach, shifts of both
    signs (a padding tap that carried act(shift) instead of 0 would show at every border)."""
    from paella_amd import ops
    rng = np.random.default_rng(11)
    paired = bounded = done = 0
    while done < 120:
        c = int(rng.choice([8, 16, 24, 40, 64, 128, 256, 512]))
        k = int(rng.integers(1, 130))
        r, s = int(rng.choice([1, 3, 3])), int(rng.choice([1, 3, 3, 5]))
        sh, sw = int(rng.choice([1, 2])), int(rng.choice([1, 2, 2]))
        ph, pw = int(rng.integers(0, r // 2 + 2)), int(rng.integers(0, s // 2 + 2))
        h, w = int(rng.integers(1, 30)), int(rng.integers(1, 30))
        if h + 2 * ph - r < 0 or w + 2 * pw - s < 0:
            continue
        kwlog = int(rng.integers(-1, 4))
        in_act = int(rng.choice([orc.ACT_NONE, orc.ACT_RELU]))
        x = rng.standard_normal((1, c, h, w)).astype(np.float32)
        wt = (rng.standard_normal((k, c, r, s)) * (2.0 / (c * r * s)) ** 0.5).astype(np.float32)
        b = (rng.standard_normal(k) * 0.1).astype(np.float32)
        scale, shift = (rng.standard_normal(c) + 1.5).astype(np.float32), (rng.standard_normal(c) * 2.0).astype(np.float32)
        conv = ops.Conv2d(wt, b, stride=(sh, sw), pad=(ph, pw), act=ops.ACT_RELU, in_hw=(h, w),
                          tile_hint=0 if kwlog < 0 else (1 << 8) | (1 << 4) | kwlog)
        if not conv.takes_input_transform():
            continue
        done += 1
        paired += conv.plan.pair_taps != 0
        bounded += in_act == orc.ACT_RELU
        ref = orc.conv2d(orc.scale_shift(x, scale, shift, act=in_act), wt, b, stride=(sh, sw), pad=(ph, pw), act=orc.ACT_RELU)
        dev = lambda a: torch.tensor(a, device=cuda)
        got = conv(dev(x), in_scale=dev(scale), in_shift=dev(shift), in_act=in_act)
        torch.cuda.synchronize()
        close(got, ref)
    assert paired >= 5 and 30 <= bounded <= 90   # the sweep reaches paired columns and both copies of the loop


def test_random_depthwise_and_pooling_shapes_match_the_oracle(cuda):
    """150 seeded shapes each; maximum pooling bit for bit."""
    from paella_amd import ops
    rng = np.random.default_rng(5)
    done = 0
    while done < 150:
        c, h, w = int(rng.integers(1, 200)), int(rng.integers(3, 60)), int(rng.integers(3, 60))
        r, st, pad, dil = int(rng.choice([3, 3, 3, 5])), int(rng.choice([1, 2])), int(rng.integers(0, 3)), int(rng.choice([1, 1, 2]))
        if h + 2 * pad - (r - 1) * dil - 1 < 0 or w + 2 * pad - (r - 1) * dil - 1 < 0:
            continue
        done += 1
        x = rng.standard_normal((1, c, h, w)).astype(np.float32)
        wt = (rng.standard_normal((c, 1, r, r)) * 0.3).astype(np.float32)
        b = None if rng.random() < 0.3 else (rng.standard_normal(c) * 0.1).astype(np.float32)
        act = int(rng.choice([orc.ACT_NONE, orc.ACT_RELU, orc.ACT_RELU6]))
        ref = orc.conv2d(x, wt, b, stride=st, pad=pad, dil=dil, groups=c, act=act)
        got = ops.Conv2d(wt, b, stride=st, pad=pad, dil=dil, groups=c, act=act, in_hw=(h, w))(torch.tensor(x, device=cuda))
        torch.cuda.synchronize()
        close(got, ref)
    done = 0
    while done < 150:
        c, h, w = int(rng.integers(1, 300)), int(rng.integers(2, 50)), int(rng.integers(2, 50))
        k, st = int(rng.choice([2, 3, 3])), int(rng.choice([1, 2, 2]))
        pad, ceil = int(rng.integers(0, k // 2 + 1)), bool(rng.random() < 0.4)
        is_avg, cip = bool(rng.random() < 0.5), bool(rng.random() < 0.5)
        if h + 2 * pad < k or w + 2 * pad < k:
            continue
        done += 1
        x = rng.standard_normal((1, c, h, w)).astype(np.float32)
        ref = orc.avgpool2d(x, k, st, pad=pad, ceil_mode=ceil, count_include_pad=cip) if is_avg else orc.maxpool2d(x, k, st, pad=pad, ceil_mode=ceil)
        got = ops.pool2d(torch.tensor(x, device=cuda), k, st, pad=pad, ceil_mode=ceil, is_avg=is_avg, count_include_pad=cip)
        torch.cuda.synchronize()
        got = got.cpu().numpy()
        assert got.shape == ref.shape
        if is_avg:
            assert np.all(np.abs(got - ref) <= 1e-5 + 1e-5 * np.abs(ref))
        else:
            assert np.array_equal(got, ref)


"""Model zoo on the CPU: topology totals against published counts, the seeded generator of the product against
the oracle's, and an independent torch restatement of every model of the zoo against the oracle."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import models as om
from paella_amd import models

# multiply-accumulates and parameters per forward pass (batch-norm folded: conv weights + one bias per channel)
EXACT = {
    "mnist": (786_560, 5_994),
    "resnet18": (1_814_073_344, 11_684_712),
    "resnet34": (3_663_761_408, 21_789_160),
    "resnet50": (4_089_184_256, 25_530_472),
    "mobilenetv2": (300_774_272, 3_487_816),
}
ANCHORS = {"inception_v3": (5.7e9, 23.8e6), "densenet121": (2.85e9, 7.98e6), "googlenet": (1.55e9, 7.0e6), "squeezenet1_1": (0.35e9, 1.24e6),
           "arcfaceresnet100": (12.1e9, 65.1e6)}
IO = {"mnist": (28 * 28 * 4, 10 * 4), "resnet18": (224 * 224 * 3 * 4, 4000), "inception_v3": (299 * 299 * 3 * 4, 4000),
      "ultraface320": (240 * 320 * 3 * 4, 4420 * 2 * 4), "arcfaceresnet100": (112 * 112 * 3 * 4, 512 * 4)}


def test_zoo_lists_the_eleven_models():
    assert sorted(models.names()) == sorted(["mnist", "resnet18", "resnet34", "resnet50", "mobilenetv2", "inception_v3", "squeezenet1_1",
                                             "googlenet", "densenet121", "ultraface320", "arcfaceresnet100"])


@pytest.mark.parametrize("name", sorted(EXACT))
def test_exact_mac_and_parameter_counts(name):
    t = models.totals(name)
    assert (t["macs"], t["params"]) == EXACT[name]


@pytest.mark.parametrize("name", sorted(ANCHORS))
def test_literature_anchors(name):
    t = models.totals(name)
    macs, params = ANCHORS[name]
    assert abs(t["macs"] / macs - 1) < 0.03 and abs(t["params"] / params - 1) < 0.03


@pytest.mark.parametrize("name", sorted(IO))
def test_io_sizes_match_the_adapters(name):
    assert models.io_bytes(name) == IO[name]


def test_seeded_generator_matches_the_oracle_bit_for_bit():
    for name, seed in [("mnist", 1), ("resnet18", 3), ("densenet121", 9)]:
        desc = om.Desc(models.describe(name))
        for idx, w in enumerate(desc.d["weights"][:12]):
            n = int(np.prod(w["shape"]))
            np.testing.assert_array_equal(models.weight_values(name, seed, idx, n), desc.weight(idx, seed).reshape(-1))


def _w(desc, seed):
    return [torch.tensor(desc.weight(i, seed)) for i in range(len(desc.d["weights"]))]


def test_small_cnn_oracle_equals_independent_torch_graph():
    desc = om.Desc(models.describe("mnist"))
    w = _w(desc, 2)
    x = om.make_input(desc.d, 4, "uniform")
    t = torch.tensor(x)
    t = F.max_pool2d(F.relu(F.conv2d(t, w[0], w[1], padding=2)), 2, 2)
    t = F.max_pool2d(F.relu(F.conv2d(t, w[2], w[3], padding=2)), 3, 3)
    ref = F.linear(t.flatten(1), w[4], w[5]).numpy().reshape(-1)
    assert torch.count_nonzero(w[1]) == 0  # zero biases
    np.testing.assert_allclose(om.run(desc, x, seed=2), ref, rtol=1e-4, atol=1e-5)
    assert 0.0 <= x.min() and x.max() < 1.0


def test_resnet18_oracle_equals_independent_torch_graph():
    desc = om.Desc(models.describe("resnet18"))
    w = iter(_w(desc, 2))
    x = om.make_input(desc.d, 4)
    t = torch.tensor(x).double()
    nxt = lambda: next(w).double()
    t = F.max_pool2d(F.relu(F.conv2d(t, nxt(), nxt(), stride=2, padding=3)), 3, 2, 1)
    for stage, planes in enumerate([64, 128, 256, 512]):
        for block in range(2):
            stride = 2 if (stage > 0 and block == 0) else 1
            identity = t
            if stride != 1 or t.shape[1] != planes:
                identity = F.conv2d(t, nxt(), nxt(), stride=stride)
            y = F.relu(F.conv2d(t, nxt(), nxt(), stride=stride, padding=1))
            t = F.relu(F.conv2d(y, nxt(), nxt(), padding=1) + identity)
    t = F.adaptive_avg_pool2d(t, 1).flatten(1)
    ref = F.linear(t, nxt(), nxt()).float().numpy().reshape(-1)
    assert next(w, None) is None
    got = om.run(desc, x, seed=2)
    np.testing.assert_allclose(got, ref, rtol=1e-4, atol=1e-4)
    assert np.abs(ref).max() > 0.1 and np.abs(ref).max() < 1e3


def _resnet_reference(name, bottleneck, layers, seed=2):
    """Textbook ResNet (v1.5 bottleneck: the stride sits on the 3x3) written directly in torch; weights are taken
    in the zoo's creation order: shortcut projection first, then the block's convs."""
    desc = om.Desc(models.describe(name))
    w = iter(_w(desc, seed))
    nxt = lambda: next(w).double()
    x = om.make_input(desc.d, 4)
    t = torch.tensor(x).double()
    t = F.max_pool2d(F.relu(F.conv2d(t, nxt(), nxt(), stride=2, padding=3)), 3, 2, 1)
    for stage, planes in enumerate([64, 128, 256, 512]):
        for block in range(layers[stage]):
            stride = 2 if (stage > 0 and block == 0) else 1
            out_ch = planes * (4 if bottleneck else 1)
            identity = t
            if stride != 1 or t.shape[1] != out_ch:
                identity = F.conv2d(t, nxt(), nxt(), stride=stride)
            if bottleneck:
                y = F.relu(F.conv2d(t, nxt(), nxt()))
                y = F.relu(F.conv2d(y, nxt(), nxt(), stride=stride, padding=1))
                t = F.relu(F.conv2d(y, nxt(), nxt()) + identity)
            else:
                y = F.relu(F.conv2d(t, nxt(), nxt(), stride=stride, padding=1))
                t = F.relu(F.conv2d(y, nxt(), nxt(), padding=1) + identity)
    ref = F.linear(F.adaptive_avg_pool2d(t, 1).flatten(1), nxt(), nxt()).float().numpy().reshape(-1)
    assert next(w, None) is None
    return desc, x, ref


@pytest.mark.parametrize("name,bottleneck,layers", [("resnet34", False, [3, 4, 6, 3]), ("resnet50", True, [3, 4, 6, 3])])
def test_deeper_resnets_equal_independent_torch_graphs(name, bottleneck, layers):
    desc, x, ref = _resnet_reference(name, bottleneck, layers)
    np.testing.assert_allclose(om.run(desc, x, seed=2), ref, rtol=1e-4, atol=1e-4)
    assert 0.05 < np.abs(ref).max() < 1e3


def test_squeezenet_equals_independent_torch_graph():
    desc = om.Desc(models.describe("squeezenet1_1"))
    w = iter(_w(desc, 2))
    nxt = lambda: next(w).double()
    x = om.make_input(desc.d, 4)
    t = torch.tensor(x).double()

    def fire(t):
        s = F.relu(F.conv2d(t, nxt(), nxt()))
        return torch.cat([F.relu(F.conv2d(s, nxt(), nxt())), F.relu(F.conv2d(s, nxt(), nxt(), padding=1))], 1)

    t = F.max_pool2d(F.relu(F.conv2d(t, nxt(), nxt(), stride=2)), 3, 2, ceil_mode=True)
    t = fire(fire(t))
    t = F.max_pool2d(t, 3, 2, ceil_mode=True)
    t = fire(fire(t))
    t = F.max_pool2d(t, 3, 2, ceil_mode=True)
    t = fire(fire(fire(fire(t))))
    assert t.shape == (1, 512, 13, 13)
    ref = F.adaptive_avg_pool2d(F.relu(F.conv2d(t, nxt(), nxt())), 1).float().numpy().reshape(-1)
    assert next(w, None) is None
    np.testing.assert_allclose(om.run(desc, x, seed=2), ref, rtol=1e-4, atol=1e-4)


def test_mobilenetv2_equals_independent_torch_graph():
    desc = om.Desc(models.describe("mobilenetv2"))
    w = iter(_w(desc, 2))
    nxt = lambda: next(w).double()
    x = om.make_input(desc.d, 4)
    t = torch.tensor(x).double()
    relu6 = lambda v: torch.clamp(v, 0.0, 6.0)
    t = relu6(F.conv2d(t, nxt(), nxt(), stride=2, padding=1))
    for expand, out_ch, repeats, first_stride in [(1, 16, 1, 1), (6, 24, 2, 2), (6, 32, 3, 2), (6, 64, 4, 2), (6, 96, 3, 1), (6, 160, 3, 2), (6, 320, 1, 1)]:
        for i in range(repeats):
            stride = first_stride if i == 0 else 1
            y = t
            if expand != 1:
                y = relu6(F.conv2d(y, nxt(), nxt()))
            y = relu6(F.conv2d(y, nxt(), nxt(), stride=stride, padding=1, groups=y.shape[1]))
            y = F.conv2d(y, nxt(), nxt())
            t = t + y if (stride == 1 and t.shape[1] == out_ch) else y
    t = relu6(F.conv2d(t, nxt(), nxt()))
    assert t.shape == (1, 1280, 7, 7)
    ref = F.linear(F.adaptive_avg_pool2d(t, 1).flatten(1), nxt(), nxt()).float().numpy().reshape(-1)
    assert next(w, None) is None
    np.testing.assert_allclose(om.run(desc, x, seed=2), ref, rtol=1e-4, atol=1e-4)


class _Torch:
    """Weight cursor + the handful of layer shorthands the independent graphs below share."""

    def __init__(self, name, seed=2):
        self.desc = om.Desc(models.describe(name))
        self._w = iter(_w(self.desc, seed))
        self.x = om.make_input(self.desc.d, 4)
        self.t = torch.tensor(self.x).double()

    def nxt(self):
        return next(self._w).double()

    def conv(self, t, stride=1, padding=0, act=F.relu, groups=1):
        y = F.conv2d(t, self.nxt(), self.nxt(), stride=stride, padding=padding, groups=groups)
        return act(y) if act else y

    def norm(self, t, act=F.relu):
        y = t * self.nxt().view(1, -1, 1, 1) + self.nxt().view(1, -1, 1, 1)
        return act(y) if act else y

    def dense(self, t):
        return F.linear(t.flatten(1), self.nxt(), self.nxt())

    def check(self, ref, rtol=1e-4, atol=1e-4):
        assert next(self._w, None) is None
        ref = ref.float().numpy().reshape(-1)
        np.testing.assert_allclose(om.run(self.desc, self.x, seed=2), ref, rtol=rtol, atol=atol)
        assert np.isfinite(ref).all() and np.abs(ref).max() > 1e-4


def test_googlenet_equals_independent_torch_graph():
    g = _Torch("googlenet")
    lrn = lambda t: F.local_response_norm(t, 5, alpha=1e-4, beta=0.75, k=1.0)
    pool = lambda t: F.max_pool2d(t, 3, 2, ceil_mode=True)

    def inception(t):
        b1 = g.conv(t)
        b3 = g.conv(g.conv(t), padding=1)
        b5 = g.conv(g.conv(t), padding=2)
        bp = g.conv(F.max_pool2d(t, 3, 1, 1))
        return torch.cat([b1, b3, b5, bp], 1)

    t = lrn(pool(g.conv(g.t, stride=2, padding=3)))
    t = pool(lrn(g.conv(g.conv(t), padding=1)))
    t = pool(inception(inception(t)))
    assert t.shape == (1, 480, 14, 14)
    for _ in range(5):
        t = inception(t)
    t = inception(inception(pool(t)))
    assert t.shape == (1, 1024, 7, 7)
    g.check(F.softmax(g.dense(F.adaptive_avg_pool2d(t, 1)), 1), atol=1e-6)


def test_densenet121_equals_independent_torch_graph():
    g = _Torch("densenet121")
    t = F.max_pool2d(g.conv(g.t, stride=2, padding=3), 3, 2, 1)
    for stage, layers in enumerate([6, 12, 24, 16]):
        for _ in range(layers):
            y = g.conv(g.norm(t))
            t = torch.cat([t, g.conv(y, padding=1, act=None)], 1)
        if stage < 3:
            t = F.avg_pool2d(g.conv(g.norm(t), act=None), 2, 2)
    assert t.shape == (1, 1024, 7, 7)
    g.check(g.dense(F.adaptive_avg_pool2d(g.norm(t), 1)))


def test_inception_v3_equals_independent_torch_graph():
    g = _Torch("inception_v3")
    avg = lambda t: F.avg_pool2d(t, 3, 1, 1)

    def block_a(t):
        b1 = g.conv(t)
        b5 = g.conv(g.conv(t), padding=2)
        b3 = g.conv(g.conv(g.conv(t), padding=1), padding=1)
        return torch.cat([b1, b5, b3, g.conv(avg(t))], 1)

    def block_b(t):
        b3 = g.conv(t, stride=2)
        bd = g.conv(g.conv(g.conv(t), padding=1), stride=2)
        return torch.cat([b3, bd, F.max_pool2d(t, 3, 2)], 1)

    def block_c(t):
        b1 = g.conv(t)
        b7 = g.conv(g.conv(g.conv(t), padding=(0, 3)), padding=(3, 0))
        bd = g.conv(t)
        for pad in [(3, 0), (0, 3), (3, 0), (0, 3)]:
            bd = g.conv(bd, padding=pad)
        return torch.cat([b1, b7, bd, g.conv(avg(t))], 1)

    def block_d(t):
        b3 = g.conv(g.conv(t), stride=2)
        b7 = g.conv(g.conv(g.conv(g.conv(t), padding=(0, 3)), padding=(3, 0)), stride=2)
        return torch.cat([b3, b7, F.max_pool2d(t, 3, 2)], 1)

    def block_e(t):
        b1 = g.conv(t)
        y = g.conv(t)
        b3 = [g.conv(y, padding=(0, 1)), g.conv(y, padding=(1, 0))]
        y = g.conv(g.conv(t), padding=1)
        bd = [g.conv(y, padding=(0, 1)), g.conv(y, padding=(1, 0))]
        return torch.cat([b1] + b3 + bd + [g.conv(avg(t))], 1)

    t = g.conv(g.conv(g.conv(g.t, stride=2)), padding=1)
    t = F.max_pool2d(t, 3, 2)
    t = F.max_pool2d(g.conv(g.conv(t)), 3, 2)
    assert t.shape == (1, 192, 35, 35)
    t = block_b(block_a(block_a(block_a(t))))
    assert t.shape == (1, 768, 17, 17)
    t = block_d(block_c(block_c(block_c(block_c(t)))))
    t = block_e(block_e(t))
    assert t.shape == (1, 2048, 8, 8)
    g.check(g.dense(F.adaptive_avg_pool2d(t, 1)))


def test_face_embedding_resnet100_equals_independent_torch_graph():
    g = _Torch("arcfaceresnet100")

    def conv_prelu(t, **kw):
        w, b, slope = g.nxt(), g.nxt(), g.nxt()
        return F.prelu(F.conv2d(t, w, b, **kw), slope)

    t = conv_prelu(g.t, padding=1)
    for units in [3, 13, 30, 3]:
        for i in range(units):
            stride = 2 if i == 0 else 1
            shortcut = g.conv(t, stride=stride, act=None) if i == 0 else t
            y = conv_prelu(g.norm(t, act=None), padding=1)
            t = g.conv(y, stride=stride, padding=1, act=None) + shortcut
    assert t.shape == (1, 512, 7, 7)
    g.check(g.dense(g.norm(t, act=None)))


def test_face_detector_scores_equal_independent_torch_graph():
    g = _Torch("ultraface320")

    def separable(t, stride=1, act=F.relu):
        return g.conv(g.conv(t, stride=stride, padding=1, groups=t.shape[1]), act=act)

    t = g.conv(g.t, stride=2, padding=1)
    feats = []
    for strides in [[1, 2, 1, 2, 1, 1, 1], [2, 1, 1], [2, 1]]:
        for s in strides:
            t = separable(t, s)
        feats.append(t)
    t = g.conv(g.conv(g.conv(t), stride=2, padding=1, groups=64))
    feats.append(t)
    assert [tuple(f.shape[1:]) for f in feats] == [(64, 30, 40), (128, 15, 20), (256, 8, 10), (256, 4, 5)]
    # each head's [anchors*2][H][W] logits are laid flat one after the other; prior r is the pair (2r, 2r+1)
    logits = torch.cat([separable(f, act=None).reshape(-1) for f in feats])
    assert logits.numel() == 4420 * 2
    g.check(F.softmax(logits.view(4420, 2), 1), atol=1e-6)


def test_io_shapes_match_the_reference_dim_sidecars(tmp_path):
    """The reference ships one .dim file per compiled model (input dims, -1, output dims).  The zoo's models must
    have the same I/O shapes -- except Inception-v3, which the reference compiled at 224x224 and which is served
    at 299x299 here on purpose (the benchmark configuration) -- and paella_model_write_dim must reproduce the format."""
    import json
    import os
    from paella_amd import _abi, models
    golden = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "tvm_models_dim.json")))["files"]
    ours = {"densenet-9": "densenet121", "googlenet-9": "googlenet", "inception_v3": "inception_v3", "mnist-8": "mnist",
            "mobilenetv2-7": "mobilenetv2", "resnet18-v2-7": "resnet18", "resnet34-v2-7": "resnet34", "resnet50-v2-7": "resnet50",
            "squeezenet1.1-7": "squeezenet1_1"}
    assert len(golden) == 9
    for fname, dims in golden.items():
        model = ours[fname.replace("-cuda-pack.so.dim", "")]
        in_bytes, out_bytes = models.io_bytes(model)
        want_in = list(dims["input"])
        if model == "inception_v3":
            assert want_in == [1, 3, 224, 224]
            want_in = [1, 3, 299, 299]
        assert in_bytes == 4 * int(np.prod(want_in)), model
        assert out_bytes == 4 * int(np.prod(dims["output"])), model
        path = str(tmp_path / (model + ".dim"))
        assert _abi.ops().paella_model_write_dim(model.encode(), path.encode()) == 0
        vals = [int(v) for v in open(path).read().split()]
        cut = vals.index(-1)
        assert vals[:cut] == want_in
        assert int(np.prod(vals[cut + 1:])) == int(np.prod(dims["output"])) and vals[cut + 1:cut + 3] == dims["output"][:2]


ZOO = ["mnist", "resnet18", "resnet34", "resnet50", "mobilenetv2", "inception_v3", "squeezenet1_1", "googlenet", "densenet121",
       "ultraface320", "arcfaceresnet100"]


@pytest.mark.parametrize("name", ZOO)
def test_launch_plan_keeps_every_dependence_of_the_graph(name):
    """The executor launches independent convs together and re-issues nodes to bring partners side by side.  Whatever
    the order, every operator appears exactly once, a launch holds at most four of them and only convs when it holds
    several, and an operator stays behind every earlier one it shares memory with when one of the two writes it."""
    import os
    from paella_amd import models
    desc = models.describe(name)
    nodes = desc["nodes"]
    before = os.environ.get("PAELLA_CONV_PAIRS")
    try:
        os.environ["PAELLA_CONV_PAIRS"] = "0"
        assert models.launch_plan(name) == [[i] for i in range(len(nodes))]
        os.environ["PAELLA_CONV_PAIRS"] = "1"
        plan = models.launch_plan(name)
    finally:
        if before is None:
            del os.environ["PAELLA_CONV_PAIRS"]
        else:
            os.environ["PAELLA_CONV_PAIRS"] = before
    assert sorted(i for launch in plan for i in launch) == list(range(len(nodes)))
    assert all(1 <= len(launch) <= 4 for launch in plan)
    # a scale-shift operator may lead the conv that applies it to its own input; apart from that, shared launches hold convs only
    absorbed = {launch[0]: launch[1] for launch in plan if len(launch) == 2 and nodes[launch[0]]["op"] == "eltwise"}
    for e, c in absorbed.items():
        assert nodes[c]["op"] == "conv" and nodes[c]["groups"] == 1 and nodes[c]["x"] == nodes[e]["y"] and nodes[e]["x2"]["buf"] < 0
        assert nodes[e]["act"] in (0, 1), nodes[e]
    # ... and one pooling operator may ride at the end of a launch of at most three convs
    riding = [launch for launch in plan if len(launch) > 1 and nodes[launch[-1]]["op"] == "pool"]
    assert all(len(launch) <= 4 for launch in riding)
    assert all(nodes[i]["op"] == "conv" and nodes[i]["groups"] == 1 for launch in plan if len(launch) > 1 and launch[0] not in absorbed
               for i in (launch[:-1] if launch in riding else launch))
    stage_of = {i: k for k, launch in enumerate(plan) for i in launch}
    # An absorbed operator's output is never written: its readers read its input instead, at their own position.
    readers = {e: [j for j in range(e + 1, len(nodes)) if nodes[j]["x"] == nodes[e]["y"]] for e in absorbed}

    def span(v):
        return None if v["buf"] < 0 else (v["buf"], v["off"], v["off"] + v["C"] * v["H"] * v["W"])

    def hit(a, b):
        return a is not None and b is not None and a[0] == b[0] and a[1] < b[2] and b[1] < a[2]

    spans = [(span(n["x"]), span(n["x2"]), span(n["y"])) for n in nodes]
    for e, c in absorbed.items():
        # the absorbed operator itself touches nothing; every conv that read its output reads its input
        first = [j for j in range(e + 1, len(nodes)) if hit(spans[j][2], spans[e][2])]
        live = [j for j in readers[e] if not first or j <= first[0]]
        assert live and live[0] == c
        for j in range(e + 1, (first[0] + 1) if first else len(nodes)):   # nobody else reads the output that is never written
            assert j in live or not (hit(spans[j][0], spans[e][2]) or hit(spans[j][1], spans[e][2])), (name, e, j)
        for j in live:
            spans[j] = (spans[e][0], spans[j][1], spans[j][2])
        spans[e] = (None, None, None)
    for j, (xj, x2j, yj) in enumerate(spans):
        for i in range(j):
            xi, x2i, yi = spans[i]
            if hit(yi, xj) or hit(yi, x2j) or hit(yi, yj) or hit(yj, xi) or hit(yj, x2i):
                assert stage_of[i] < stage_of[j], (name, i, j)
    if name in ("densenet121", "arcfaceresnet100"):
        assert len(absorbed) >= 49 and sum(n["op"] == "eltwise" for n in nodes) - len(absorbed) == 1
    if name == "resnet18":
        assert [launch for launch in plan if len(launch) > 1] == [[7, 6], [12, 11], [17, 16]]  # first 3x3 of the block, then its projection
    if name in ("inception_v3", "googlenet"):
        assert max(len(launch) for launch in plan) >= 3 and len(plan) < 0.5 * len(nodes)
        assert len(riding) >= 9   # the 3x3 pool of every inception module goes out with the module's first convs

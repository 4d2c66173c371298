"""Model zoo on the CPU: topology totals against published counts, the seeded generator of the product against
the oracle's, and an independent torch restatement of the small CNN and ResNet-18 against the oracle."""
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

"""ONNX import on the CPU.  Two independent producers of files: torch's own ONNX exporter (genuine files of small
networks in the styles of the served families) and a hand encoder for what that exporter does not emit.  The imported
graph -- stages, fused activations and residuals, folded norms, re-based concatenations, the file's own weights -- is
executed by the CPU oracle and must reproduce torch's forward pass of the original network."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import _onnx_writer as ow
import _torch_nets as nets
from oracle import models as om
from paella_amd import models

ATOL, RTOL = 2e-4, 1e-3


def imported(path):
    name = "onnx:" + str(path)
    d = models.describe(name)
    desc = om.Desc(d, external=lambda idx: models.weight_values(name, 0, idx, int(np.prod(d["weights"][idx]["shape"]))))
    return d, desc


def run_imported(path, x):
    d, desc = imported(path)
    return d, om.run(desc, x)


def close(got, ref):
    ref = np.asarray(ref, np.float64).reshape(-1)
    err = np.abs(got.astype(np.float64) - ref)
    assert got.shape == ref.shape and np.all(err <= ATOL + RTOL * np.abs(ref)), float(err.max())


@pytest.mark.parametrize("net", sorted(nets.NETS))
def test_torch_exported_networks_import_and_match_torch(tmp_path, net):
    make, shape = nets.NETS[net]
    module = nets.randomize(make(), seed=11)
    x = torch.randn(shape, generator=torch.Generator().manual_seed(5))
    path = tmp_path / (net + ".onnx")
    if not ow.export_torch(module, x, str(path)):
        pytest.skip("torch's TorchScript ONNX exporter is not usable here")
    with torch.no_grad():
        ref = module(x).numpy()
    d, got = run_imported(path, x.numpy())
    close(got, ref)
    ops = [n["op"] for n in d["nodes"]]
    assert all(w["fill"] == "external" for w in d["weights"])
    convs = sum(isinstance(m, torch.nn.Conv2d) for m in module.modules())
    assert ops.count("conv") == convs and ops.count("dense") == sum(isinstance(m, torch.nn.Linear) for m in module.modules())
    # what must have been fused away: every norm behind a conv, every relu, every residual add, every concat
    # resnet_v2_style: the norm on the input, the pre-activation norm+relu of each unit (its input is also the shortcut,
    # or the sum feeds two readers), and the last norm stay stages of their own; the norm between a unit's convs folds
    standalone = {"resnet_v2_style": 5, "resnet_style": 0, "squeeze_style": 0, "mobile_style": 0, "dense_style": 5, "inception_style": 0, "face_style": 2}[net]
    assert ops.count("eltwise") == standalone, ops


def test_resnet_blocks_fuse_the_way_the_zoo_writes_them(tmp_path):
    """Exported with torchvision's layout (main path, then the projection shortcut, then Add, Relu), a block becomes
    conv+relu, conv, conv(projection)+residual+relu -- three stages, no elementwise stage."""
    module = nets.randomize(nets.ResNet((1, 1), 8, 10), seed=3)
    x = torch.randn(1, 3, 32, 32, generator=torch.Generator().manual_seed(1))
    path = tmp_path / "r.onnx"
    if not ow.export_torch(module, x, str(path)):
        pytest.skip("torch's TorchScript ONNX exporter is not usable here")
    d, _ = imported(path)
    n = d["nodes"]
    assert [k["op"] for k in n] == ["conv", "pool", "conv", "conv", "conv", "conv", "conv", "gap", "dense"]
    assert [k["act"] for k in n if k["op"] == "conv"] == [1, 1, 1, 1, 0, 1]
    assert [k["x2"]["buf"] >= 0 for k in n if k["op"] == "conv"] == [False, False, True, False, False, True]
    # the identity block adds the block input; the projection conv (last of its block) adds the main path's output
    assert n[3]["x2"] == n[2]["x"] and n[6]["x2"] == n[5]["y"] and n[6]["R"] == 1


def test_folded_batchnorm_values(tmp_path):
    module = nets.randomize(torch.nn.Sequential(torch.nn.Conv2d(3, 5, 3, bias=True), torch.nn.BatchNorm2d(5, eps=1e-3)), seed=9)
    x = torch.randn(1, 3, 6, 6)
    path = tmp_path / "bn.onnx"
    if not ow.export_torch(module, x, str(path)):
        pytest.skip("torch's TorchScript ONNX exporter is not usable here")
    d, desc = imported(path)
    conv, bn = module[0], module[1]
    s = (bn.weight / torch.sqrt(bn.running_var + bn.eps)).detach().double()
    np.testing.assert_allclose(desc.weight(0, 0), (conv.weight.detach().double() * s.view(-1, 1, 1, 1)).numpy(), rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(desc.weight(1, 0), ((conv.bias.detach().double() - bn.running_mean.double()) * s + bn.bias.detach().double()).numpy(), rtol=1e-6, atol=1e-7)
    assert len(d["nodes"]) == 1


def test_shape_arithmetic_in_front_of_a_reshape_is_folded(tmp_path):
    """x.view(x.size(0), -1) exports as Shape -> Gather -> Unsqueeze -> Concat -> Reshape: all static at batch 1."""
    class Net(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.conv, self.fc = torch.nn.Conv2d(3, 4, 3), torch.nn.Linear(4 * 5 * 5, 6)

        def forward(self, x):
            x = F.relu(self.conv(x))
            return self.fc(x.view(x.size(0), -1))
    module = nets.randomize(Net(), seed=2)
    x = torch.randn(1, 3, 7, 7, generator=torch.Generator().manual_seed(8))
    path = tmp_path / "view.onnx"
    if not ow.export_torch(module, x, str(path), dynamic_batch=True):
        pytest.skip("torch's TorchScript ONNX exporter is not usable here")
    raw = open(path, "rb").read()
    assert b"Shape" in raw and b"Gather" in raw
    d, got = run_imported(path, x.numpy())
    with torch.no_grad():
        close(got, module(x).numpy())
    assert [n["op"] for n in d["nodes"]] == ["conv", "dense"]


# ---------------------------------------------------------------- hand-encoded files

def hand(tmp_path, build, in_shape, out_shape, **kw):
    b = ow.Builder(np.random.default_rng(4))
    out = build(b)
    path = tmp_path / "hand.onnx"
    b.save(str(path), [("x", in_shape)], [(out, out_shape)], **kw)
    ow.check(str(path))
    return b, path


def test_old_style_file_matmul_add_clip_attributes_constant_node_and_float_data(tmp_path):
    """The layout of the small-CNN zoo file: Conv, Add of a [K,1,1] constant, Relu, MaxPool with auto_pad, Reshape from a
    constant, MatMul, Add; plus Clip with min/max attributes (opset 6), LRN, a Constant node, non-raw float_data,
    unpacked dims, and the initializers also listed as graph inputs (IR version 3 files)."""
    def build(b):
        w = b.const(b.randn(4, 1, 5, 5, scale=0.3), raw=False, packed=False)
        bias = b.const(b.randn(4, 1, 1, scale=0.1))
        t = b.op("Conv", ["x", w], kernel_shape=[5, 5], auto_pad="SAME_UPPER", strides=[1, 1])
        t = b.op("Relu", [b.op("Add", [t, bias])])
        t = b.op("MaxPool", [t], kernel_shape=[2, 2], strides=[2, 2], auto_pad="VALID")
        t = b.op("LRN", [t], size=3, alpha=2e-3, beta=0.6, bias=1.5)
        t = b.op("Clip", [t], min=-0.25, max=0.5)
        b.nodes.append(ow.node("Constant", [], ["shape"], value=ow.tensor("", np.array([1, 4 * 6 * 6], np.int64))))
        t = b.op("Reshape", [t, "shape"])
        t = b.op("MatMul", [t, b.const(b.randn(144, 10, scale=0.1))])
        return b.op("Add", [t, b.const(b.randn(1, 10, scale=0.1))])
    b, path = hand(tmp_path, build, [1, 1, 12, 12], [1, 10], opset=6)
    x = np.random.default_rng(1).random((1, 1, 12, 12), dtype=np.float32)
    d, got = run_imported(path, x)
    a = {k: torch.tensor(v) for k, v in b.arrays.items()}
    w = list(b.arrays)
    t = F.conv2d(torch.tensor(x), a[w[0]], padding=2) + a[w[1]]
    t = F.max_pool2d(F.relu(t), 2, 2)
    t = torch.clamp(F.local_response_norm(t, 3, alpha=2e-3, beta=0.6, k=1.5), -0.25, 0.5)
    ref = t.reshape(1, -1) @ a[w[2]] + a[w[3]]
    close(got, ref.numpy())
    assert [n["op"] for n in d["nodes"]] == ["conv", "pool", "lrn", "eltwise", "dense"] and d["nodes"][0]["act"] == 1 and d["nodes"][3]["act"] == 4


def test_gemm_variants_half_and_double_tensors_input_normalisation(tmp_path):
    """The conv's weight and bias are stored as float16 and float64 on purpose (to exercise the tensor decoder): the
    file passes the checker's structural pass, its type inference remarks on the mix."""
    def build(b):
        t = b.op("Sub", ["x", b.const(np.array(0.5, np.float32))])
        t = b.op("Mul", [t, b.const(np.array([[[2.0]], [[0.5]], [[-1.0]]], np.float32))])
        t = b.op("Conv", [t, b.const(b.randn(6, 3, 3, 3, scale=0.2).astype(np.float16)), b.const(b.randn(6, scale=0.1).astype(np.float64))],
                 kernel_shape=[3, 3], pads=[1, 1, 1, 1])
        t = b.op("GlobalMaxPool", [t])
        t = b.op("Flatten", [t], axis=1)
        t = b.op("Gemm", [t, b.const(b.randn(6, 8, scale=0.3)), b.const(b.randn(8, scale=0.1))], alpha=0.5, beta=2.0)
        t = b.op("LeakyRelu", [t], alpha=0.2)
        t = b.op("Gemm", [t, b.const(b.randn(4, 8, scale=0.3))], transB=1)
        return b.op("Softmax", [t], axis=1)
    b, path = hand(tmp_path, build, ["N", 3, 9, 9], ["N", 4], opset=11, initializers_as_inputs=False)
    x = np.random.default_rng(2).standard_normal((1, 3, 9, 9)).astype(np.float32)
    d, got = run_imported(path, x)
    a = [torch.tensor(np.asarray(v, np.float32)) for v in b.arrays.values()]
    t = (torch.tensor(x) - a[0]) * a[1]
    t = F.conv2d(t, a[2], a[3], padding=1).amax((2, 3))
    t = F.leaky_relu(0.5 * t @ a[4] + 2.0 * a[5], 0.2)
    ref = F.softmax(t @ a[6].T, 1)
    close(got, ref.numpy())
    # Sub and Mul on the graph input are stages of their own, and so is a leaky relu behind a dense stage (the dense
    # kernel has no slope input); everything else fuses or is a view
    assert [n["op"] for n in d["nodes"]] == ["eltwise", "eltwise", "conv", "pool", "dense", "eltwise", "dense", "softmax"]


def test_concat_of_shared_and_input_tensors_copies_only_what_it_must(tmp_path):
    """A tensor that feeds two concatenations can live in only one of them, and the graph input cannot move: those
    operands are copied by a stage; the others are re-based for free."""
    def build(b):
        u = b.op("Relu", [b.op("Conv", ["x", b.const(b.randn(4, 3, 1, 1))], kernel_shape=[1, 1])])
        v = b.op("Relu", [b.op("Conv", ["x", b.const(b.randn(2, 3, 1, 1))], kernel_shape=[1, 1])])
        c1 = b.op("Concat", [u, v], axis=1)
        c2 = b.op("Concat", ["x", u, c1], axis=1)
        return b.op("AveragePool", [c2], kernel_shape=[3, 3], strides=[2, 2], pads=[1, 1, 1, 1], count_include_pad=1)
    b, path = hand(tmp_path, build, [1, 3, 7, 7], [1, 13, 4, 4])
    x = np.random.default_rng(3).standard_normal((1, 3, 7, 7)).astype(np.float32)
    d, got = run_imported(path, x)
    a = [torch.tensor(v) for v in b.arrays.values()]
    xt = torch.tensor(x)
    u, v = F.relu(F.conv2d(xt, a[0])), F.relu(F.conv2d(xt, a[1]))
    ref = F.avg_pool2d(torch.cat([xt, u, torch.cat([u, v], 1)], 1), 3, 2, 1, count_include_pad=True)
    close(got, ref.numpy())
    ops = [n["op"] for n in d["nodes"]]
    assert ops.count("conv") == 2 and ops.count("eltwise") == 2   # copies of x and of u (u already lives inside c1)


@pytest.mark.parametrize("avg", [False, True])
def test_end_padding_of_ceil_mode_converters_becomes_ceil_mode(tmp_path, avg):
    """pads = [0, 0, 1, 1] on a stride-2 pool (how Caffe-derived zoo files spell ceil mode) equals torch's ceil_mode."""
    def build(b):
        t = b.op("Relu", [b.op("Conv", ["x", b.const(b.randn(4, 3, 3, 3))], kernel_shape=[3, 3])])
        return b.op("AveragePool" if avg else "MaxPool", [t], kernel_shape=[3, 3], strides=[2, 2], pads=[0, 0, 1, 1])
    b, path = hand(tmp_path, build, [1, 3, 14, 14], [1, 4, 6, 6])
    x = np.random.default_rng(6).standard_normal((1, 3, 14, 14)).astype(np.float32)
    d, got = run_imported(path, x)
    t = F.relu(F.conv2d(torch.tensor(x), torch.tensor(list(b.arrays.values())[0])))
    ref = F.avg_pool2d(t, 3, 2, ceil_mode=True, count_include_pad=False) if avg else F.max_pool2d(t, 3, 2, ceil_mode=True)
    assert ref.shape == (1, 4, 6, 6) and d["nodes"][1]["ceil"] == 1
    close(got, ref.numpy())


@pytest.mark.parametrize("case", ["unknown_op", "asymmetric_pads", "batch_two", "two_inputs", "inner_axis_concat", "missing_weight"])
def test_unsupported_files_are_refused_not_approximated(tmp_path, case, capfd):
    def build(b):
        w = b.const(b.randn(4, 3, 3, 3))
        if case == "unknown_op":
            return b.op("Sigmoid", [b.op("Conv", ["x", w], kernel_shape=[3, 3])])
        if case == "asymmetric_pads":
            return b.op("Conv", ["x", w], kernel_shape=[3, 3], pads=[0, 0, 1, 1])
        if case == "inner_axis_concat":
            t = b.op("Conv", ["x", w], kernel_shape=[3, 3])
            return b.op("Concat", [t, t], axis=2)
        if case == "missing_weight":
            return b.op("Conv", ["x", "nowhere"], kernel_shape=[3, 3])
        return b.op("Conv", ["x", w], kernel_shape=[3, 3])
    b = ow.Builder(np.random.default_rng(0))
    out = build(b)
    path = tmp_path / "bad.onnx"
    inputs = [("x", [2 if case == "batch_two" else 1, 3, 8, 8])] + ([("x2", [1, 3, 8, 8])] if case == "two_inputs" else [])
    b.save(str(path), inputs, [(out, [1, 4, 6, 6])])
    with pytest.raises(RuntimeError):
        models.describe("onnx:" + str(path))
    msg = capfd.readouterr().err
    expect = {"unknown_op": "Sigmoid", "asymmetric_pads": "asymmetric", "batch_two": "batch 1", "two_inputs": "more than one graph input",
              "inner_axis_concat": "outermost", "missing_weight": "nowhere"}[case]
    assert expect in msg, msg


def test_garbage_and_missing_files_are_errors(tmp_path, capfd):
    bad = tmp_path / "junk.onnx"
    bad.write_bytes(b"\xff" * 64)
    for name in ("onnx:" + str(bad), "onnx:" + str(tmp_path / "absent.onnx")):
        with pytest.raises(RuntimeError):
            models.describe(name)
    assert "onnx import" in capfd.readouterr().err
    # a tensor whose dims promise far more data than the file holds must be refused before anything is allocated for it
    b = ow.Builder(np.random.default_rng(0))
    lie = ow._len(1, ow._varint(1 << 30) + ow._varint(1 << 30)) + ow._int(2, 11) + ow._len(9, b"\0" * 8) + ow._str(8, "w")
    b.inits.append(lie)
    b.nodes.append(ow.node("Conv", ["x", "w"], ["y"], kernel_shape=[3, 3]))
    b.save(str(tmp_path / "lie.onnx"), [("x", [1, 3, 8, 8])], [("y", [1, 4, 6, 6])])
    with pytest.raises(RuntimeError):
        models.describe("onnx:" + str(tmp_path / "lie.onnx"))
    assert "holds" in capfd.readouterr().err


def _bn(b, t, c):
    return b.op("BatchNormalization", [t, b.const(b.randn(c) * 0.2 + 1.0), b.const(b.randn(c)), b.const(b.randn(c) * 0.1),
                                       b.const(np.abs(b.randn(c)) + 0.5)], epsilon=1e-5)


def test_norm_in_front_of_convs_is_launched_only_where_a_reader_cannot_apply_it(tmp_path):
    """The executor drops a batch-norm (+ ReLU) stage when every reader of its output is a conv that can apply it to its own
    input (smallest tile, input channels a multiple of 8); the launch plan lists the stage with its first reader."""
    from paella_amd import models

    def plan_of(build, c, out_c, tag):
        b = ow.Builder(np.random.default_rng(4))
        out = build(b)
        path = tmp_path / (tag + ".onnx")
        b.save(str(path), [("x", ["N", c, 9, 9])], [(out, ["N", out_c, 9, 9])], opset=11, initializers_as_inputs=False)
        ow.check(str(path))
        name = "onnx:" + str(path)
        return [n["op"] for n in models.describe(name)["nodes"]], models.launch_plan(name)

    conv = lambda b, t, c, k: b.op("Conv", [t, b.const(b.randn(k, c, 3, 3, scale=0.2)), b.const(b.randn(k, scale=0.1))], kernel_shape=[3, 3], pads=[1, 1, 1, 1])
    # one reader that can
    ops, plan = plan_of(lambda b: conv(b, b.op("Relu", [_bn(b, "x", 8)]), 8, 16), 8, 16, "one")
    assert ops == ["eltwise", "conv"] and plan == [[0, 1]]
    # two readers that can: listed with the first, the second stands alone and applies it too (or shares a launch with nothing)
    def two(b):
        t = _bn(b, "x", 8)
        return b.op("Concat", [conv(b, t, 8, 8), conv(b, t, 8, 8)], axis=1)
    ops, plan = plan_of(two, 8, 16, "two")
    assert ops == ["eltwise", "conv", "conv"] and sorted(map(tuple, plan)) == [(0, 1), (2,)]
    # the normalised tensor is also the residual of the conv: it has to exist
    def residual(b):
        t = _bn(b, "x", 8)
        return b.op("Add", [conv(b, t, 8, 8), t])
    ops, plan = plan_of(residual, 8, 8, "res")
    assert ops == ["eltwise", "conv"] and plan == [[0], [1]]
    # six input channels: the conv reads through the offset table, which has no transform
    ops, plan = plan_of(lambda b: conv(b, _bn(b, "x", 6), 6, 16), 6, 16, "six")
    assert ops == ["eltwise", "conv"] and plan == [[0], [1]]

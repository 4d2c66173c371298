"""ONNX import on the GPU: files written by torch's own ONNX exporter, imported, executed by the HIP operators through
the C-ABI executor and through a job adapter under the server, against torch's forward pass of the original network.
Tolerance |got - ref| <= 1e-4 + 1e-3 |ref| (fp32)."""
import os

import numpy as np
import pytest
import torch

import _onnx_writer as ow
import _torch_nets as nets

pytestmark = pytest.mark.gpu

ATOL, RTOL = 1e-4, 1e-3


def close(got, ref, what):
    ref = np.asarray(ref, np.float64).reshape(-1)
    err = np.abs(got.astype(np.float64) - ref)
    assert got.shape == ref.shape and np.isfinite(got).all()
    assert np.all(err <= ATOL + RTOL * np.abs(ref)), "%s: max err %g" % (what, err.max())
    assert np.abs(ref).max() > 1e-3


def export(tmp_path, name, module, x):
    path = tmp_path / (name + ".onnx")
    if not ow.export_torch(module, x, str(path)):
        pytest.skip("torch's TorchScript ONNX exporter is not usable here")
    with torch.no_grad():
        return str(path), module(x).numpy()


def run_on_gpu(path, x):
    from paella_amd import models
    ex = models.Exec("onnx:" + path)
    try:
        ex.set_input(x)
        ex.forward()
        return ex.get_output()
    finally:
        ex.close()


@pytest.mark.parametrize("net", sorted(nets.NETS))
def test_imported_networks_match_torch(cuda, tmp_path, net):
    make, shape = nets.NETS[net]
    module = nets.randomize(make(), seed=21)
    x = torch.randn(shape, generator=torch.Generator().manual_seed(6))
    path, ref = export(tmp_path, net, module, x)
    print("case", net, flush=True)
    close(run_on_gpu(path, x.numpy()), ref, net)


def test_resnet18_at_full_size_from_its_onnx_file(cuda, tmp_path):
    """torchvision's ResNet-18 layout with batch norms, 224 x 224, 1000 classes: 20 convs after folding, no elementwise stage."""
    from paella_amd import models
    module = nets.randomize(nets.ResNet((2, 2, 2, 2), 64, 1000), seed=4)
    x = torch.randn(1, 3, 224, 224, generator=torch.Generator().manual_seed(2))
    path, ref = export(tmp_path, "resnet18_torchvision_layout", module, x)
    d = models.describe("onnx:" + path)
    ops = [n["op"] for n in d["nodes"]]
    assert ops.count("conv") == 20 and ops.count("eltwise") == 0 and len(ops) == 23
    assert models.totals("onnx:" + path)["macs"] == 1_814_073_344
    close(run_on_gpu(path, x.numpy()), ref, "resnet18")


def test_adapter_serves_the_onnx_file_found_in_the_models_directory(cuda, tmp_path):
    """$LLIS_MODELS_DIR/resnet18-v2-7.onnx replaces the built-in ResNet-18 behind the tvm_resnet18 adapter: request
    sizes, graph and weights come from the file."""
    from paella_amd import serve
    module = nets.randomize(nets.ResNet((1, 1), 16, 12), seed=8)
    x = torch.randn(1, 3, 64, 64, generator=torch.Generator().manual_seed(3))
    path, ref = export(tmp_path, "resnet18-v2-7", module, x)
    before = os.environ.get("LLIS_MODELS_DIR")
    os.environ["LLIS_MODELS_DIR"] = str(tmp_path)
    try:
        with serve.Server("gt%d_onnx" % os.getpid(), "full3", num_streams=8) as srv:
            out, _ = serve.client_single(srv.name, serve.job_path("tvm_resnet18"), x.numpy(), 12, n=3)
    finally:
        if before is None:
            del os.environ["LLIS_MODELS_DIR"]
        else:
            os.environ["LLIS_MODELS_DIR"] = before
    close(out, ref, "served")


def test_output_that_a_later_stage_reads_back_cannot_be_bound_to_host_memory(cuda, tmp_path):
    """The graph's output tensor also feeds a pooling stage: the executor must keep it in device memory."""
    import ctypes
    from paella_amd import _abi, models
    b = ow.Builder(np.random.default_rng(1))
    y1 = b.op("Relu", [b.op("Conv", ["x", b.const(b.randn(4, 3, 3, 3))], kernel_shape=[3, 3])])
    b.op("GlobalAveragePool", [y1])
    path = str(tmp_path / "readback.onnx")
    b.save(path, [("x", [1, 3, 8, 8])], [(y1, [1, 4, 6, 6])])
    ex = models.Exec("onnx:" + path)
    host = ctypes.c_void_p()
    _abi.check(_abi.hip().llis_hip_host_alloc_pinned(ctypes.byref(host), 4096))
    try:
        assert ex.lib.paella_exec_bind_output(ex.handle, host) == -2
        assert ex.lib.paella_exec_bind_input(ex.handle, host) == 0
    finally:
        ex.close()
        _abi.hip().llis_hip_host_free(host)


@pytest.mark.parametrize("shared", ["two_readers", "also_residual"])
def test_norm_shared_by_convs_matches_torch(cuda, tmp_path, shared):
    """A batch-norm on the input read by two convs (both apply it themselves, the norm is not launched), and one that is
    also the residual of its conv (it has to exist, so it is launched): hand-written files against torch."""
    import torch.nn.functional as F
    from paella_amd import models
    b = ow.Builder(np.random.default_rng(8))
    c = 8
    bn = [b.randn(c) * 0.2 + 1.0, b.randn(c), b.randn(c) * 0.1, np.abs(b.randn(c)) + 0.5]
    t = b.op("BatchNormalization", ["x"] + [b.const(a) for a in bn], epsilon=1e-5)
    w1, b1, w2, b2 = b.randn(8, c, 3, 3, scale=0.2), b.randn(8, scale=0.1), b.randn(8, c, 3, 3, scale=0.2), b.randn(8, scale=0.1)
    conv = lambda t, w, bias: b.op("Conv", [t, b.const(w), b.const(bias)], kernel_shape=[3, 3], pads=[1, 1, 1, 1])
    if shared == "two_readers":
        out, out_c = b.op("Concat", [conv(t, w1, b1), conv(t, w2, b2)], axis=1), 16
    else:
        out, out_c = b.op("Add", [conv(t, w1, b1), t]), 8
    path = tmp_path / (shared + ".onnx")
    b.save(str(path), [("x", ["N", c, 11, 13])], [(out, ["N", out_c, 11, 13])], opset=11, initializers_as_inputs=False)
    ow.check(str(path))
    x = torch.randn(1, c, 11, 13, generator=torch.Generator().manual_seed(3))
    tt = lambda a: torch.tensor(np.asarray(a, np.float32))
    n = F.batch_norm(x, tt(bn[2]), tt(bn[3]), tt(bn[0]), tt(bn[1]), False, 0.0, 1e-5)
    if shared == "two_readers":
        ref = torch.cat([F.conv2d(n, tt(w1), tt(b1), padding=1), F.conv2d(n, tt(w2), tt(b2), padding=1)], 1)
    else:
        ref = F.conv2d(n, tt(w1), tt(b1), padding=1) + n
    plan = models.launch_plan("onnx:" + str(path))
    assert (sorted(map(tuple, plan)) == [(0, 1), (2,)]) if shared == "two_readers" else (plan == [[0], [1]])
    close(run_on_gpu(str(path), x.numpy()), ref.numpy(), shared)

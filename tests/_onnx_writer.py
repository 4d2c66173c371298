"""Minimal ONNX file writer for the import tests: protobuf wire format by hand (field numbers from the public
onnx.proto), because the onnx package is not available.  Only what the tests need: float / int64 tensors, nodes with
int / float / ints / string / tensor attributes, one graph with inputs, outputs and initializers."""
import struct

import numpy as np


def _varint(v):
    v &= (1 << 64) - 1
    out = bytearray()
    while True:
        b = v & 0x7F
        v >>= 7
        if v:
            out.append(b | 0x80)
        else:
            out.append(b)
            return bytes(out)


def _key(field, wire):
    return _varint(field << 3 | wire)


def _len(field, payload):
    return _key(field, 2) + _varint(len(payload)) + payload


def _int(field, v):
    return _key(field, 0) + _varint(v)


def _str(field, s):
    return _len(field, s.encode())


def tensor(name, array, raw=True, packed=True):
    """TensorProto: dims=1, data_type=2, float_data=4, int64_data=7, name=8, raw_data=9."""
    a = np.asarray(array)
    out = b""
    if packed:
        out += _len(1, b"".join(_varint(d) for d in a.shape)) if a.ndim else b""
    else:
        out += b"".join(_int(1, d) for d in a.shape)
    if a.dtype == np.float32:
        out += _int(2, 1)
        out += _len(9, a.tobytes()) if raw else _len(4, a.astype("<f4").tobytes())
    elif a.dtype == np.int64:
        out += _int(2, 7)
        out += _len(9, a.tobytes()) if raw else _len(7, b"".join(_varint(int(v)) for v in a.reshape(-1)))
    elif a.dtype == np.float16:
        out += _int(2, 10) + _len(9, a.tobytes())
    elif a.dtype == np.float64:
        out += _int(2, 11) + _len(9, a.tobytes())
    else:
        raise TypeError(a.dtype)
    return out + _str(8, name)


def _attr(name, value):
    """AttributeProto: name=1, f=2, i=3, s=4, t=5, floats=7, ints=8, type=20."""
    out = _str(1, name)
    if isinstance(value, float):
        return out + _key(2, 5) + struct.pack("<f", value) + _int(20, 1)
    if isinstance(value, (int, np.integer)):
        return out + _int(3, int(value)) + _int(20, 2)
    if isinstance(value, str):
        return out + _str(4, value) + _int(20, 3)
    if isinstance(value, bytes):   # an already encoded TensorProto
        return out + _len(5, value) + _int(20, 4)
    if isinstance(value, (list, tuple)) and all(isinstance(v, (int, np.integer)) for v in value):
        return out + b"".join(_int(8, int(v)) for v in value) + _int(20, 7)
    if isinstance(value, (list, tuple)):
        return out + b"".join(_key(7, 5) + struct.pack("<f", float(v)) for v in value) + _int(20, 6)
    raise TypeError(type(value))


def node(op, inputs, outputs, name="", **attrs):
    """NodeProto: input=1, output=2, name=3, op_type=4, attribute=5."""
    out = b"".join(_str(1, s) for s in inputs) + b"".join(_str(2, s) for s in outputs)
    if name:
        out += _str(3, name)
    out += _str(4, op)
    for k, v in attrs.items():
        out += _len(5, _attr(k, v))
    return out


def value_info(name, shape):
    """ValueInfoProto{name=1, type=2{tensor_type=1{elem_type=1, shape=2{dim=1{dim_value=1 | dim_param=2}}}}}."""
    dims = b""
    for d in shape:
        dims += _len(1, _str(2, d) if isinstance(d, str) else _int(1, d))
    return _str(1, name) + _len(2, _len(1, _int(1, 1) + _len(2, dims)))


def model(nodes, inputs, outputs, initializers, opset=11, initializers_as_inputs=False):
    """ModelProto{ir_version=1, opset_import=8{version=2}, graph=7{node=1, name=2, initializer=5, input=11, output=12}}.
    inputs / outputs: [(name, shape)], initializers: [encoded TensorProto]."""
    g = b"".join(_len(1, n) for n in nodes) + _str(2, "g")
    g += b"".join(_len(5, t) for t in initializers)
    g += b"".join(_len(11, value_info(n, s)) for n, s in inputs)
    if initializers_as_inputs:
        g += b"".join(_len(11, value_info(n, s)) for n, s in initializers_as_inputs)
    g += b"".join(_len(12, value_info(n, s)) for n, s in outputs)
    return _int(1, 7) + _str(2, "paella-tests") + _len(8, _str(1, "") + _int(2, opset)) + _len(7, g)


class Builder:
    """Collects nodes and initializers; names tensors t0, t1, ..."""

    def __init__(self, rng):
        self.rng = rng
        self.nodes, self.inits, self.arrays = [], [], {}
        self._n = 0

    def name(self, prefix="t"):
        self._n += 1
        return "%s%d" % (prefix, self._n)

    def const(self, array, raw=True, packed=True, name=None):
        name = name or self.name("w")
        self.arrays[name] = np.asarray(array)
        self.inits.append(tensor(name, self.arrays[name], raw=raw, packed=packed))
        return name

    def randn(self, *shape, scale=1.0):
        return (self.rng.standard_normal(shape) * scale).astype(np.float32)

    def op(self, op, inputs, n_out=1, **attrs):
        outs = [self.name() for _ in range(n_out)]
        self.nodes.append(node(op, inputs, outs, name=self.name(op.lower()), **attrs))
        return outs[0] if n_out == 1 else outs

    def save(self, path, inputs, outputs, **kw):
        with open(path, "wb") as f:
            f.write(model(self.nodes, inputs, outputs, self.inits, **kw))


def export_torch(module, x, path, opset=11, dynamic_batch=False):
    """ONNX file written by torch's own TorchScript exporter (its C++ protobuf serializer): an independent producer
    of genuine ONNX files.  The exporter's last step wants the onnx package only to splice in onnxscript functions,
    which these models do not have; that step is bypassed.  Returns False when the exporter is unusable here."""
    import warnings

    import torch
    try:
        from torch.onnx._internal.torchscript_exporter import onnx_proto_utils
    except ImportError:
        return False
    keep = onnx_proto_utils._add_onnxscript_fn
    onnx_proto_utils._add_onnxscript_fn = lambda model_bytes, custom_opsets: model_bytes
    try:
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")
            extra = dict(input_names=["input"], dynamic_axes={"input": {0: "batch"}}) if dynamic_batch else {}
            torch.onnx.export(module.eval(), (x,), path, dynamo=False, opset_version=opset, do_constant_folding=False,
                              training=torch.onnx.TrainingMode.EVAL, **extra)
    finally:
        onnx_proto_utils._add_onnxscript_fn = keep
    return True


def check(path):
    """Runs the ONNX checker built into torch over a file (raises on a malformed model)."""
    import warnings

    import torch
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")   # shape-inference remarks; structural errors raise
        torch._C._check_onnx_proto(open(path, "rb").read())

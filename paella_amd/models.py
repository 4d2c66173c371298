"""Python front-end of the model zoo / executor C-ABI (include/paella_models.h) for tests and benches."""
import ctypes
import json

import numpy as np

from . import _abi
from ._abi import LaunchDims, check


def names():
    return _abi.ops().paella_model_names().decode().split(",")


def describe(name):
    lib = _abi.ops()
    need = ctypes.c_size_t()
    check(lib.paella_model_describe(name.encode(), None, 0, ctypes.byref(need)), "paella_model_describe")
    buf = ctypes.create_string_buffer(need.value)
    check(lib.paella_model_describe(name.encode(), buf, need.value, None), "paella_model_describe")
    return json.loads(buf.value.decode())


def totals(name):
    lib = _abi.ops()
    m, p, f, b = (ctypes.c_double() for _ in range(4))
    s = ctypes.c_int()
    check(lib.paella_model_totals(name.encode(), m, p, f, b, s), "paella_model_totals")
    return {"macs": m.value, "params": p.value, "flops": f.value, "bytes": b.value, "stages": s.value}


def launch_plan(name):
    """The launches of a model as lists of node indices (host arithmetic only, no device needed)."""
    lib = _abi.ops()
    need = lib.paella_model_launch_plan(name.encode(), None, 0)
    if need < 0:
        raise RuntimeError("paella_model_launch_plan failed: %d" % need)
    buf = (ctypes.c_int * need)()
    lib.paella_model_launch_plan(name.encode(), buf, need)
    out, i = [], 0
    while i < need:
        out.append(list(buf[i + 1:i + 1 + buf[i]]))
        i += 1 + buf[i]
    return out


def io_bytes(name):
    lib = _abi.ops()
    i, o = ctypes.c_size_t(), ctypes.c_size_t()
    check(lib.paella_model_io_bytes(name.encode(), ctypes.byref(i), ctypes.byref(o)), "paella_model_io_bytes")
    return i.value, o.value


def weight_values(name, seed, tensor, count):
    out = np.empty(count, np.float32)
    check(_abi.ops().paella_model_weight_values(name.encode(), seed, tensor, out.ctypes.data, count), "paella_model_weight_values")
    return out


class Exec:
    """One request's worth of activations of a model resident on the GPU."""

    def __init__(self, name, seed=1):
        self.lib = _abi.ops()
        self.name = name
        self.model = ctypes.c_void_p()
        check(self.lib.paella_model_get(name.encode(), seed, ctypes.byref(self.model)), "paella_model_get")
        self.handle = ctypes.c_void_p()
        check(self.lib.paella_exec_create(self.model, ctypes.byref(self.handle)), "paella_exec_create")
        self.in_bytes, self.out_bytes = io_bytes(name)
        self.num_stages = self.lib.paella_model_num_stages(self.model)

    def close(self):
        if self.handle:
            self.lib.paella_exec_destroy(self.handle)
            self.handle = None

    def stage_dims(self, i):
        d = LaunchDims()
        check(self.lib.paella_model_stage_dims(self.model, i, ctypes.byref(d)), "paella_model_stage_dims")
        return d

    def stage_nodes(self, i):
        """Indices of the graph nodes that stage i launches (one operator, or several convs sharing a launch)."""
        nodes = (ctypes.c_int * 8)()
        count = self.lib.paella_model_stage_nodes(self.model, i, nodes, 8)
        if count < 1:
            raise RuntimeError("paella_model_stage_nodes failed: %d" % count)
        return list(nodes)[:count]

    def stage_work(self, i):
        op, f, b = ctypes.c_char_p(), ctypes.c_double(), ctypes.c_double()
        check(self.lib.paella_model_stage_work(self.model, i, ctypes.byref(op), f, b), "paella_model_stage_work")
        return op.value.decode(), f.value, b.value

    def set_input(self, x):
        x = np.ascontiguousarray(x, np.float32)
        assert x.nbytes == self.in_bytes
        check(_abi.hip().llis_hip_memcpy(self.lib.paella_exec_input(self.handle), x.ctypes.data, x.nbytes, 1), "H2D")

    def get_output(self):
        out = np.empty(self.out_bytes // 4, np.float32)
        check(_abi.hip().llis_hip_memcpy(out.ctypes.data, self.lib.paella_exec_output(self.handle), out.nbytes, 2), "D2H")
        return out

    def bind_io(self, in_ptr=None, out_ptr=None):
        """Device-visible host memory (addresses) in place of the request's input / output device buffers; None restores."""
        check(self.lib.paella_exec_bind_input(self.handle, ctypes.c_void_p(in_ptr)), "paella_exec_bind_input")
        check(self.lib.paella_exec_bind_output(self.handle, ctypes.c_void_p(out_ptr)), "paella_exec_bind_output")

    def forward(self, stream=None):
        check(self.lib.paella_exec_forward(self.handle, stream), "paella_exec_forward")

    def launch_stage(self, i, stream=None, job_id=0, notifier=None):
        check(self.lib.paella_exec_launch_stage(self.handle, i, stream, job_id, notifier), "paella_exec_launch_stage")

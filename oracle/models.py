"""Whole-model CPU oracle (TEST INFRASTRUCTURE ONLY).

Executes a model description -- the JSON that paella_model_describe() emits: buffers, seeded weight tensors
and operator nodes in stage order -- with the operators of oracle/ops.c and weights from the oracle's own
seeded generator.  The description is data (which layer feeds which, with what shape); every number is
computed here, independently of the GPU path.

What it restates: the forward pass the reference obtains from `run_()` of a TVM-compiled model
(reference jobs/tvm_mnist/tvm_mnist.cpp:41).  Pinning: the reference has no numeric outputs for any model,
so (a) the operators are pinned in tests/test_oracle_ops.py, (b) the topologies are pinned through their
published multiply-accumulate and parameter counts and through an independent torch.nn.functional
restatement of each of the eleven models in tests/test_models_cpu.py.
"""
import numpy as np

from . import ops


class Desc:
    def __init__(self, d, external=None):
        """external(idx) -> array supplies the values of weight tensors marked "external" (imported models carry
        their own weights instead of seeded ones); tests pass what they read back from the importer."""
        self.d = d
        self.name = d["name"]
        self.external = external

    def weight(self, idx, seed):
        w = self.d["weights"][idx]
        shape = tuple(w["shape"])
        if w["fill"] == "external":
            return np.asarray(self.external(idx), np.float32).reshape(shape)
        if w["fill"] == "normal":
            return ops.fill_normal(shape, seed, idx, w["a"])
        if w["fill"] == "uniform":
            return ops.fill_uniform(shape, seed, idx, w["a"], w["b"])
        return np.full(shape, w["a"], np.float32)


def _get(bufs, v):
    if v["buf"] < 0:
        return None
    n = v["C"] * v["H"] * v["W"]
    return bufs[v["buf"]][v["off"]:v["off"] + n].reshape(1, v["C"], v["H"], v["W"])


def _put(bufs, v, val):
    n = v["C"] * v["H"] * v["W"]
    assert val.size == n, (val.shape, v)
    bufs[v["buf"]][v["off"]:v["off"] + n] = val.reshape(-1)


def run(desc, x, seed=1, fast=False, keep=None):
    """Forward pass.  `keep`, if a dict, receives the output of every node (index -> array copy)."""
    d = desc.d if isinstance(desc, Desc) else desc
    desc = desc if isinstance(desc, Desc) else Desc(d)
    bufs = [np.zeros(b["C"] * b["H"] * b["W"], np.float32) for b in d["buffers"]]
    _put(bufs, d["input"], np.asarray(x, np.float32))
    wcache = {}

    def W(i):
        if i < 0:
            return None
        if i not in wcache:
            wcache[i] = desc.weight(i, seed)
        return wcache[i]

    for k, n in enumerate(d["nodes"]):
        xin, x2 = _get(bufs, n["x"]), _get(bufs, n["x2"])
        op = n["op"]
        if op == "conv":
            y = ops.conv2d(xin, W(n["w"]), W(n["bias"]), stride=tuple(n["stride"]), pad=tuple(n["pad"]), dil=tuple(n["dil"]),
                           groups=n["groups"], act=n["act"], residual=x2, slope=W(n["slope"]), lo=n["lo"], hi=n["hi"], fast=fast)
        elif op == "dense":
            y = ops.dense(xin.reshape(1, -1), W(n["w"]), W(n["bias"]), act=n["act"])
        elif op == "pool":
            assert n["k"][0] == n["k"][1] or True
            if n["avg"]:
                y = ops.avgpool2d(xin, tuple(n["k"]), tuple(n["stride"]), tuple(n["pad"]), bool(n["ceil"]), bool(n["count_include_pad"]))
            else:
                y = ops.maxpool2d(xin, tuple(n["k"]), tuple(n["stride"]), tuple(n["pad"]), bool(n["ceil"]))
        elif op == "gap":
            y = ops.global_avgpool(xin)
        elif op == "eltwise":
            if x2 is not None:
                assert n["scale"] < 0 and n["shift"] < 0
                y = ops.add(xin, x2, n["act"], W(n["slope"]), n["lo"], n["hi"])
            else:
                y = ops.scale_shift(xin, W(n["scale"]), W(n["shift"]), n["act"], W(n["slope"]), n["lo"], n["hi"])
        elif op == "softmax":
            y = ops.softmax(xin.reshape(n["rows"], n["cols"]))
        elif op == "lrn":
            y = ops.lrn(xin, n["size"], n["alpha"], n["beta"], n["k"])
        else:
            raise ValueError(op)
        _put(bufs, n["y"], y)
        if keep is not None:
            keep[k] = y.copy()
    o = d["output"]
    return _get(bufs, o).reshape(-1).copy()


def make_input(desc, seed, kind="normal"):
    """Synthetic request input: N(0,1) (or U[0,1) for the small CNN), stream 1_000_000 of the seeded generator."""
    d = desc.d if isinstance(desc, Desc) else desc
    v = d["input"]
    shape = (1, v["C"], v["H"], v["W"])
    if kind == "uniform":
        return ops.fill_uniform(shape, seed, 1000000, 0.0, 1.0)
    return ops.fill_normal(shape, seed, 1000000, 1.0)

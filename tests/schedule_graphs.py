"""Lowered-graph descriptions for the schedule estimator tests, and the FX graph
built from one.

A description is plain data (what the golden file stores):
    {"nodes": [{"kind": ..., "args": [node indices], "shape": [...], "dur": float,
                "group": "0", "name": ...}, ...], "outputs": [node indices]}
kinds: placeholder, relu, add, view (aliases its input), all_gather, all_reduce,
reduce_scatter (asynchronous collectives on group ``group``), alltoall (the
blocking _dtensor collective), wait (wait_tensor of args[0]).
``random_description(seed)`` draws one; ``build_graph(desc)`` makes the
fx.GraphModule with fake CUDA tensors as ``meta['val']`` (no GPU is touched) and
the runtime estimator (a lookup of ``dur`` by node name).
"""
import random

import torch
import torch.distributed._functional_collectives  # noqa: F401  (registers _c10d_functional)
import torch.fx as fx
from torch._subclasses.fake_tensor import FakeTensorMode

GROUP_SIZE = 4


def random_description(seed: int, n_ops: int = 40):
    rng = random.Random(seed)
    nodes, pending = [], []  # pending: collectives not waited for yet
    shapes = {}

    def add(kind, args=(), shape=None, dur=0.0, group=None, name=None):
        i = len(nodes)
        nodes.append({"kind": kind, "args": list(args), "shape": list(shape), "dur": float(dur),
                      "group": group, "name": name or f"{kind}_{i}"})
        shapes[i] = tuple(shape)
        return i

    def draw_dur():
        r = rng.random()
        if r < 0.15:
            return 0.0
        if r < 0.6:
            return round(rng.uniform(0.1, 30.0), 3)
        return rng.uniform(20.0, 900.0)

    base = (GROUP_SIZE * rng.choice([4, 8, 16]), rng.choice([32, 64, 96]))
    tensors = []
    for k in range(rng.randint(2, 5)):
        name = f"primals_{k + 1}" if rng.random() < 0.6 else f"tangents_{k + 1}"
        tensors.append(add("placeholder", shape=base, name=name))
    for _ in range(n_ops):
        r = rng.random()
        same = lambda s: [t for t in tensors if shapes[t] == s]  # noqa: E731
        a = rng.choice(tensors)
        if r < 0.30:
            tensors.append(add("relu", [a], shapes[a], draw_dur()))
        elif r < 0.45:
            b = rng.choice(same(shapes[a]))
            tensors.append(add("add", [a, b], shapes[a], draw_dur()))
        elif r < 0.52:
            s = shapes[a]
            tensors.append(add("view", [a], (s[0] * s[1],) if len(s) == 2 else s, 0.0))
        elif r < 0.75:
            kind = rng.choice(["all_gather", "all_reduce", "reduce_scatter"])
            s = shapes[a]
            if kind == "reduce_scatter" and s[0] % GROUP_SIZE:
                kind = "all_reduce"
            out = {"all_gather": (s[0] * GROUP_SIZE,) + s[1:], "all_reduce": s,
                   "reduce_scatter": (s[0] // GROUP_SIZE,) + s[1:]}[kind]
            pending.append(add(kind, [a], out, draw_dur(), group=str(rng.randint(0, 2))))
        elif r < 0.80:
            tensors.append(add("alltoall", [a], shapes[a], draw_dur(), group=str(rng.randint(0, 2))))
        else:
            q = rng.random()
            if pending and q < 0.75:
                c = pending.pop(rng.randrange(len(pending)))
                if rng.random() < 0.15:  # through a wrapper node that is not a collective
                    c_arg = add("view", [c], shapes[c], 0.0)
                    shapes[c_arg] = shapes[c]
                else:
                    c_arg = c
                w = add("wait", [c_arg], shapes[c], 0.0)
                tensors.append(w)
                if rng.random() < 0.15:  # a second wait on the same collective, or a chained one
                    tensors.append(add("wait", [rng.choice([c_arg, w])], shapes[c], 0.0))
            elif q < 0.9:
                tensors.append(add("wait", [rng.choice([t for t in tensors if nodes[t]["kind"] == "placeholder"])],
                                   base, 0.0))
    outputs = rng.sample(tensors, k=min(len(tensors), rng.randint(1, 3)))
    return {"nodes": nodes, "outputs": outputs}


def build_graph(desc, device="cuda"):
    """(gm, runtime_estimator) of a description."""
    g = fx.Graph()
    fm = FakeTensorMode()
    made = []
    ops = torch.ops
    with fm:
        for nd in desc["nodes"]:
            kind, args = nd["kind"], [made[i] for i in nd["args"]]
            vals = [a.meta["val"] for a in args]
            shape = tuple(nd["shape"])
            if kind == "placeholder":
                n = g.placeholder(nd["name"])
                val = torch.empty(shape, dtype=torch.bfloat16, device=device)
            elif kind == "relu":
                n = g.call_function(ops.aten.relu.default, (args[0],))
                val = ops.aten.relu.default(vals[0])
            elif kind == "add":
                n = g.call_function(ops.aten.add.Tensor, (args[0], args[1]))
                val = ops.aten.add.Tensor(vals[0], vals[1])
            elif kind == "view":
                n = g.call_function(ops.aten.view.default, (args[0], list(shape)))
                val = ops.aten.view.default(vals[0], list(shape))
            elif kind == "all_gather":
                n = g.call_function(ops._c10d_functional.all_gather_into_tensor.default,
                                    (args[0], GROUP_SIZE, nd["group"]))
                val = ops._c10d_functional.all_gather_into_tensor.default(vals[0], GROUP_SIZE, nd["group"])
            elif kind == "all_reduce":
                n = g.call_function(ops._c10d_functional.all_reduce.default, (args[0], "sum", nd["group"]))
                val = ops._c10d_functional.all_reduce.default(vals[0], "sum", nd["group"])
            elif kind == "reduce_scatter":
                n = g.call_function(ops._c10d_functional.reduce_scatter_tensor.default,
                                    (args[0], "sum", GROUP_SIZE, nd["group"]))
                val = ops._c10d_functional.reduce_scatter_tensor.default(vals[0], "sum", GROUP_SIZE, nd["group"])
            elif kind == "alltoall":
                n = g.call_function(ops._dtensor.shard_dim_alltoall.default, (args[0], 0, 1, nd["group"]))
                val = torch.empty_like(vals[0])  # its fake kernel wants a registered process group
            elif kind == "wait":
                n = g.call_function(ops._c10d_functional.wait_tensor.default, (args[0],))
                val = ops._c10d_functional.wait_tensor.default(vals[0])
            else:
                raise ValueError(kind)
            assert tuple(val.shape) == shape, (kind, tuple(val.shape), shape)
            if kind != "placeholder":
                n.name = nd["name"]
            n.meta["val"] = val
            made.append(n)
        g.output(tuple(made[i] for i in desc["outputs"]))
    gm = fx.GraphModule(torch.nn.Module(), g)
    durs = {nd["name"]: nd["dur"] for nd in desc["nodes"]}
    return gm, (lambda node: durs.get(node.name, 0.0))

"""Shape-level generators for the benchmark graphs.

The reference obtains its joint forward+backward graph from Dynamo/AOTAutograd
and its per-node strategies from DTensor's sharding propagator
(autoparallel/api.py:157-228, autoparallel/shardings/placement_options.py:279-359);
neither is part of the cost engine.  This module produces inputs of the same
shape without either: a small tape-based tracer records aten-granularity ops
on symbolic (shape, stride, dtype) tensors, differentiates them, and
enumerates per-op strategies as the product over mesh dims of single-dim
options, the way DTensor's ``expand_to_full_mesh_op_strategy`` does, followed
by the reference's validity filter and de-duplication
(autoparallel/shardings/propagation_rules.py:127-158,
autoparallel/shardings/placement_options.py:151-170).  Linear layers appear as
two-operand einsums, as after the reference's view-mm-view rewrite
(autoparallel/graph_passes/graph_utils.py:415-439), with the single-dim
options of autoparallel/shardings/propagation_rules.py:573-590 (no Partial
inputs).

Strategy sets are *input data* for the cost engine; what is checked against
the reference is the cost of every entry given these inputs.
"""
from __future__ import annotations

import dataclasses
import itertools
import math
from typing import Callable, Dict, List, Optional, Sequence, Tuple

import numpy as np

from . import opprog
from .packed import (
    DT_BF16,
    DT_F32,
    DT_OTHER,
    OP_PROGRAM,
    OP_ZERO,
    PARTIAL_SUM,
    PARTIAL_AVG,
    PLC_KIND_MASK,
    PLC_PARTIAL,
    PLC_R,
    GraphBuilder,
    NodeDesc,
    PackedGraph,
    is_shard,
    shard,
)

R = PLC_R
P = PARTIAL_SUM
MASK_PARTIAL = PLC_PARTIAL | 8  # embedding's MaskPartial: equal only to itself

_ITEMSIZE = {DT_BF16: 2, DT_F32: 4, DT_OTHER: 8}


def contiguous_stride(shape: Sequence[int]) -> Tuple[int, ...]:
    st = []
    acc = 1
    for s in reversed(shape):
        st.append(acc)
        acc *= max(int(s), 1)
    return tuple(reversed(st))


@dataclasses.dataclass
class T:
    """Symbolic tensor: which node (and tuple element) produces it."""

    node: int
    out_index: Optional[int]
    shape: Tuple[int, ...]
    stride: Tuple[int, ...]
    dtype: int
    requires_grad: bool = False

    @property
    def rank(self) -> int:
        return len(self.shape)

    @property
    def itemsize(self) -> int:
        return _ITEMSIZE[self.dtype]


# one single-mesh-dim option: (placements of the outputs, placements of the args)
Option = Tuple[Tuple[Optional[int], ...], Tuple[Optional[int], ...]]


def _valid(shape: Sequence[int], plc: Sequence[int], mesh_shape: Sequence[int]) -> bool:
    # per-spec rule of remove_invalid_configs (propagation_rules.py:143-154)
    shape = list(shape)
    for n, p in zip(mesh_shape, plc):
        if is_shard(p):
            d = p & 0x3F
            if shape[d] >= n:
                shape[d] = (shape[d] + n - 1) // n
            else:
                return False
    return True


class Tracer:
    def __init__(self, mesh_shape: Sequence[int], devices_per_host: int = 8):
        self.mesh_shape = tuple(int(x) for x in mesh_shape)
        self.ndim = len(self.mesh_shape)
        self.b = GraphBuilder(self.mesh_shape, devices_per_host)
        self._tape: List[Tuple[List[T], List[T], Callable]] = []
        self._strategy_cache: Dict[tuple, tuple] = {}
        self.param_nodes: List[int] = []
        self.grad_nodes: Dict[int, int] = {}  # param node -> grad node
        self.node_users: Dict[int, List[int]] = {}
        self.node_inputs: Dict[int, List[int]] = {}
        self.outputs: List[T] = []

    # -- strategy expansion --------------------------------------------------
    def _expand(
        self,
        sig: tuple,
        options: List[Option],
        out_metas: List[Optional[T]],
        in_metas: List[Optional[T]],
    ):
        """Product over mesh dims of single-dim options -> validity filter ->
        dedup.  Returns (in_plcs[o][a], out_plcs[o][k])."""
        key = (sig, tuple(options), tuple((t.shape if t else None) for t in out_metas),
               tuple((t.shape if t else None) for t in in_metas))
        hit = self._strategy_cache.get(key)
        if hit is not None:
            return hit
        seen = set()
        ins_all, outs_all = [], []
        for combo in itertools.product(options, repeat=self.ndim):
            outs = tuple(
                None if combo[0][0][k] is None else tuple(c[0][k] for c in combo)
                for k in range(len(out_metas))
            )
            ins = tuple(
                None if combo[0][1][a] is None else tuple(c[1][a] for c in combo)
                for a in range(len(in_metas))
            )
            ok = True
            for plc, t in list(zip(outs, out_metas)) + list(zip(ins, in_metas)):
                if plc is None or t is None:
                    continue
                if not _valid(t.shape, plc, self.mesh_shape):
                    ok = False
                    break
            if not ok:
                continue
            k2 = (ins, outs)
            if k2 in seen:
                continue
            seen.add(k2)
            ins_all.append(ins)
            outs_all.append(outs)
        assert ins_all, f"no valid strategy for {sig}"
        res = (ins_all, outs_all)
        self._strategy_cache[key] = res
        return res

    # -- node emission -------------------------------------------------------
    def _emit(
        self,
        name: str,
        args: List[T],
        outs_meta: List[Tuple[Tuple[int, ...], Tuple[int, ...], int]],
        options: List[Option],
        program: Optional[List[int]],
        tuple_output: bool = False,
        sig_extra: tuple = (),
    ) -> List[T]:
        v = len(self.b.nodes)
        out_ts = [
            T(v, (k if tuple_output else None), tuple(s), tuple(st), dt)
            for k, (s, st, dt) in enumerate(outs_meta)
        ]
        ins_all, outs_all = self._expand((name.split(".")[0],) + sig_extra, options, out_ts, args)
        in_meta_ids = [self.b.meta(a.shape, a.stride, a.itemsize, a.dtype) for a in args]
        out_meta_ids = [self.b.meta(t.shape, t.stride, t.itemsize, t.dtype) for t in out_ts]
        in_specs, out_specs = [], []
        for ins, outs in zip(ins_all, outs_all):
            in_specs.append([
                -1 if plc is None else self.b.spec(m, plc) for plc, m in zip(ins, in_meta_ids)
            ])
            out_specs.append([
                -1 if plc is None else self.b.spec(m, plc) for plc, m in zip(outs, out_meta_ids)
            ])
        inputs, getitem = [], None
        for a in args:
            inputs.append(a.node)
        nd = NodeDesc(
            name=f"{name}_{v}",
            in_specs=in_specs,
            out_specs=out_specs,
            inputs=inputs,
            op=OP_PROGRAM if program is not None else OP_ZERO,
            program=program,
            tuple_output=tuple_output,
        )
        self.b.add_node(nd)
        self.node_inputs[v] = list(inputs)
        for u in inputs:
            self.node_users.setdefault(u, []).append(v)
        return out_ts

    def _emit_fixed(self, name: str, args: List[T], outs_meta, in_plcs, out_plcs, tuple_output: bool) -> List[T]:
        """A node with exactly one strategy and no compute estimate."""
        v = len(self.b.nodes)
        out_ts = [T(v, (k if tuple_output else None), tuple(s), tuple(st), dt) for k, (s, st, dt) in enumerate(outs_meta)]
        for plc, t_ in list(zip(in_plcs, args)) + list(zip(out_plcs, out_ts)):
            assert _valid(t_.shape, plc, self.mesh_shape), (name, t_.shape, plc)
        ins = [self.b.spec(self.b.meta(a.shape, a.stride, a.itemsize, a.dtype), tuple(p)) for a, p in zip(args, in_plcs)]
        outs = [self.b.spec(self.b.meta(t_.shape, t_.stride, t_.itemsize, t_.dtype), tuple(p))
                for t_, p in zip(out_ts, out_plcs)]
        inputs = [a.node for a in args]
        self.b.add_node(NodeDesc(name=f"{name}_{v}", in_specs=[ins], out_specs=[outs], inputs=inputs, op=OP_ZERO,
                                 tuple_output=tuple_output))
        self.node_inputs[v] = list(inputs)
        for u in inputs:
            self.node_users.setdefault(u, []).append(v)
        return out_ts

    def local_map(self, name: str, args: List[T], in_plcs, out_meta, out_plc, grad_plcs) -> T:
        """An opaque region with declared placements, as the reference sees a
        ``local_map`` call: one strategy (the declared input/output placements,
        autoparallel/shardings/placement_options.py:455-490) and no compute
        estimate (the target is a higher-order op, not an OpOverload:
        autoparallel/cost_models/compute_estimation.py:368-380); only the
        redistribution of its inputs into ``in_plcs`` is priced.  The backward
        is another such node taking the output gradient and the saved inputs,
        producing one gradient per input with placement ``grad_plcs[i]``."""
        out = self._emit_fixed(name, args, [out_meta], in_plcs, [out_plc], tuple_output=False)[0]

        def vjp(g):
            metas = [(a.shape, a.stride, a.dtype) for a in args]
            gs = self._emit_fixed(name + "_backward", [g[0]] + list(args), metas, [out_plc] + list(in_plcs),
                                  list(grad_plcs), tuple_output=True)
            return [self.getitem(x) for x in gs]

        self._record(list(args), [out], vjp)
        return out

    def placeholder(self, name: str, shape, dtype: int, param: bool = False, requires_grad=False) -> T:
        """Parameters and inputs: every {Replicate, Shard(d)} combination that
        survives the validity filter (propagation_rules.py:184-201)."""
        shape = tuple(int(s) for s in shape)
        stride = contiguous_stride(shape)
        v = len(self.b.nodes)
        t = T(v, None, shape, stride, dtype, requires_grad=requires_grad or param)
        m = self.b.meta(shape, stride, t.itemsize, dtype)
        opts = [R] + [shard(i) for i in range(len(shape))]
        specs = []
        for plc in itertools.product(opts, repeat=self.ndim):
            if _valid(shape, plc, self.mesh_shape):
                specs.append(self.b.spec(m, plc))
        self.b.add_node(
            NodeDesc(
                name=name,
                in_specs=[[s] for s in specs],
                out_specs=[[s] for s in specs],
                inputs=[],
                default_rows=[[[0.0]] for _ in specs],
            )
        )
        self.node_inputs[v] = []
        if param:
            self.param_nodes.append(v)
        return t

    def getitem(self, src: T) -> T:
        """operator.getitem on a tuple-producing node: follows the producer's
        strategies one to one (propagation_rules.py:209+)."""
        assert src.out_index is not None
        prod = self.b.nodes[src.node]
        v = len(self.b.nodes)
        k = src.out_index
        specs = [o[k] for o in prod.out_specs]
        # strategies with equal (input, output) collapse (keep_unique_configs)
        uniq = list(dict.fromkeys(specs))
        self.b.add_node(
            NodeDesc(
                name=f"getitem_{v}",
                in_specs=[[s] for s in uniq],
                out_specs=[[s] for s in uniq],
                inputs=[src.node],
                getitem_index=k,
            )
        )
        self.node_inputs[v] = [src.node]
        self.node_users.setdefault(src.node, []).append(v)
        return T(v, None, src.shape, src.stride, src.dtype)

    # -- autograd tape -------------------------------------------------------
    def _record(self, ins: List[T], outs: List[T], vjp: Callable):
        if any(t.requires_grad for t in ins):
            for o in outs:
                o.requires_grad = True
            self._tape.append((ins, outs, vjp))

    def backward(self, roots: List[Tuple[T, T]]):
        """Differentiate: ``roots`` pairs each output with its tangent."""
        grads: Dict[Tuple[int, Optional[int]], T] = {}
        if getattr(self, "_bwd_start", None) is None:
            self._bwd_start = len(self.b.nodes)  # nodes from here on belong to the backward pass

        def key(t: T):
            return (t.node, t.out_index)

        def acc(t: T, g: Optional[T]):
            if g is None or not t.requires_grad:
                return
            k = key(t)
            if k in grads:
                grads[k] = self.add(grads[k], g)
            else:
                grads[k] = g

        for out, tangent in roots:
            acc(out, tangent)
        for ins, outs, vjp in reversed(self._tape):
            gouts = [grads.get(key(o)) for o in outs]
            if all(g is None for g in gouts):
                continue
            gins = vjp(gouts)
            for t, g in zip(ins, gins):
                acc(t, g)
        self._tape = []
        return grads

    # ======================= primitive ops ==================================
    @staticmethod
    def _bshape(shapes: List[Tuple[int, ...]]) -> Tuple[int, ...]:
        r = max(len(s) for s in shapes)
        out = [1] * r
        for s in shapes:
            for i, x in enumerate(s):
                j = r - len(s) + i
                if x != 1:
                    out[j] = x
        return tuple(out)

    def pointwise(self, name: str, args: List[T], partial: str = "none", out_dtype: Optional[int] = None,
                  vjp: Optional[Callable] = None) -> T:
        shape = self._bshape([a.shape for a in args])
        r = len(shape)
        dt = args[0].dtype if out_dtype is None else out_dtype
        opts: List[Option] = [((R,), tuple(R for _ in args))]
        for d in range(r):
            if shape[d] == 1:
                continue
            ins = []
            for a in args:
                da = d - (r - a.rank)
                ins.append(shard(da) if da >= 0 and a.shape[da] != 1 else R)
            opts.append(((shard(d),), tuple(ins)))
        if partial == "add":
            opts.append(((P,), tuple(P for _ in args)))
        elif partial == "mul":
            for i in range(len(args)):
                opts.append(((P,), tuple(P if j == i else R for j in range(len(args)))))
        elif partial == "unary":
            opts.append(((P,), (P,) + tuple(R for _ in args[1:])))
        out = self._emit(name, args, [(shape, contiguous_stride(shape), dt)], opts,
                         opprog.pointwise(r, _ITEMSIZE[dt]), sig_extra=(partial, dt))[0]
        if vjp is not None:
            self._record(args, [out], vjp)
        return out

    def _unbroadcast(self, g: T, like: T) -> T:
        if g.shape == like.shape:
            return g
        lead = g.rank - like.rank
        dims = list(range(lead)) + [lead + i for i, s in enumerate(like.shape) if s == 1 and g.shape[lead + i] != 1]
        out = self.sum(g, dims, keepdim=False) if lead and len(dims) == lead else self.sum(g, dims, keepdim=True)
        if out.shape != like.shape:
            out = self.view(out, like.shape)
        return out

    def add(self, a: T, b: T) -> T:
        return self.pointwise("add", [a, b], "add",
                              vjp=lambda g: [self._unbroadcast(g[0], a), self._unbroadcast(g[0], b)])

    def mul(self, a: T, b: T) -> T:
        return self.pointwise(
            "mul", [a, b], "mul",
            vjp=lambda g: [
                self._unbroadcast(self.mul(g[0], b), a) if a.requires_grad else None,
                self._unbroadcast(self.mul(g[0], a), b) if b.requires_grad else None,
            ])

    def scale(self, a: T, name: str = "mul_scalar") -> T:
        """a * python scalar (also add-scalar-free linear unary ops)."""
        return self.pointwise(name, [a], "unary", vjp=lambda g: [self.scale(g[0], name)])

    def neg(self, a: T) -> T:
        return self.pointwise("neg", [a], "unary", vjp=lambda g: [self.neg(g[0])])

    def unary(self, name: str, a: T, bwd_name: Optional[str] = None) -> T:
        """Non-linear unary op; backward is one fused binary op (grad, saved)."""
        bn = bwd_name or (name + "_backward")
        return self.pointwise(name, [a], "none",
                              vjp=lambda g: [self.pointwise(bn, [g[0], a], "none")])

    def add_scalar(self, a: T) -> T:
        return self.pointwise("add_scalar", [a], "none", vjp=lambda g: [g[0]])

    def to_dtype(self, a: T, dtype: int) -> T:
        if a.dtype == dtype:
            return a
        src = a.dtype
        return self.pointwise("_to_copy", [a], "unary", out_dtype=dtype,
                              vjp=lambda g: [self.to_dtype(g[0], src)])

    def alias(self, a: T) -> T:
        """View-like identity (alias/detach): zero compute cost."""
        opts: List[Option] = [((R,), (R,))] + [((shard(d),), (shard(d),)) for d in range(a.rank)] + [((P,), (P,))]
        return self._emit("alias", [a], [(a.shape, a.stride, a.dtype)], opts, None)[0]

    # ---- einsum (linear layers) -------------------------------------------
    def einsum_fwd(self, x: T, w: T) -> T:
        """"{batch}k,kn->{batch}n"."""
        assert w.rank == 2 and x.shape[-1] == w.shape[0]
        r = x.rank
        opts: List[Option] = [((R,), (R, R))]
        for d in range(r - 1):
            opts.append(((shard(d),), (shard(d), R)))
        opts.append(((shard(r - 1),), (R, shard(1))))  # n
        opts.append(((P,), (shard(r - 1), shard(0))))  # k -> Partial
        shape = x.shape[:-1] + (w.shape[1],)
        out = self._emit("einsum_fwd", [x, w], [(shape, contiguous_stride(shape), x.dtype)], opts,
                         opprog.einsum_fwd(r, x.itemsize))[0]

        def vjp(g):
            gx = self.einsum_fwd(g[0], self.permute(w, [1, 0])) if x.requires_grad else None
            gw = self.einsum_bwd(g[0], x) if w.requires_grad else None  # [k, n]
            return [gx, gw]

        self._record([x, w], [out], vjp)
        return out

    def einsum_bwd(self, a: T, b: T) -> T:
        """"{batch}n,{batch}k->kn" (weight gradient)."""
        assert a.shape[:-1] == b.shape[:-1]
        r = a.rank
        opts: List[Option] = [((R,), (R, R))]
        for d in range(r - 1):
            opts.append(((P,), (shard(d), shard(d))))
        opts.append(((shard(1),), (shard(r - 1), R)))  # n
        opts.append(((shard(0),), (R, shard(r - 1))))  # k
        shape = (b.shape[-1], a.shape[-1])
        return self._emit("einsum_bwd", [a, b], [(shape, contiguous_stride(shape), a.dtype)], opts,
                          opprog.einsum_bwd(r, a.itemsize))[0]

    # ---- views --------------------------------------------------------------
    def permute(self, x: T, perm: Sequence[int]) -> T:
        perm = [p % x.rank for p in perm]
        shape = tuple(x.shape[p] for p in perm)
        stride = tuple(x.stride[p] for p in perm)
        opts: List[Option] = [((R,), (R,)), ((P,), (P,))]
        for j, p in enumerate(perm):
            opts.append(((shard(j),), (shard(p),)))
        out = self._emit("permute", [x], [(shape, stride, x.dtype)], opts, None, sig_extra=(tuple(perm),))[0]
        inv = [perm.index(i) for i in range(x.rank)]
        self._record([x], [out], lambda g: [self.permute(g[0], inv)])
        return out

    def transpose(self, x: T, d0: int, d1: int) -> T:
        perm = list(range(x.rank))
        perm[d0], perm[d1] = perm[d1], perm[d0]
        return self.permute(x, perm)

    def view(self, x: T, shape: Sequence[int]) -> T:
        """Reshape.  Sharding follows DTensor's dim-map rule: in a flatten
        group only the leading input dim may stay sharded; in a split group
        the shard moves to the leading output dim."""
        shape = tuple(int(s) for s in shape)
        assert math.prod(shape) == math.prod(x.shape), (x.shape, shape)
        opts: List[Option] = [((R,), (R,)), ((P,), (P,))]
        i = j = 0
        while i < x.rank and j < len(shape):
            i0, j0 = i, j
            pi, pj = x.shape[i], shape[j]
            i += 1
            j += 1
            while pi != pj:
                if pi < pj:
                    pi *= x.shape[i]
                    i += 1
                else:
                    pj *= shape[j]
                    j += 1
            # leading non-1 dims of the group map to each other
            ii = next((t for t in range(i0, i) if x.shape[t] != 1), None)
            jj = next((t for t in range(j0, j) if shape[t] != 1), None)
            if ii is not None and jj is not None:
                opts.append(((shard(jj),), (shard(ii),)))
        out = self._emit("view", [x], [(shape, contiguous_stride(shape), x.dtype)], opts, None,
                         sig_extra=(shape,))[0]
        src_shape = x.shape
        self._record([x], [out], lambda g: [self.view(g[0], src_shape)])
        return out

    def slice(self, x: T, dim: int, start: int, end: int) -> T:
        dim %= x.rank
        shape = tuple((end - start) if i == dim else s for i, s in enumerate(x.shape))
        opts: List[Option] = [((R,), (R,)), ((P,), (P,))]
        for d in range(x.rank):
            if d != dim:
                opts.append(((shard(d),), (shard(d),)))
        out = self._emit("slice", [x], [(shape, x.stride, x.dtype)], opts, None, sig_extra=(dim, start, end))[0]
        self._record([x], [out], lambda g: [self.slice_backward(g[0], x.shape, dim)])
        return out

    def slice_backward(self, g: T, shape: Tuple[int, ...], dim: int) -> T:
        opts: List[Option] = [((R,), (R,)), ((P,), (P,))]
        for d in range(g.rank):
            if d != dim:
                opts.append(((shard(d),), (shard(d),)))
        prog = opprog.program([], [(g.itemsize, [opprog.const(shape[i]) if i == dim else opprog.argdim(0, i)
                                                 for i in range(len(shape))])])
        return self._emit("slice_backward", [g], [(shape, contiguous_stride(shape), g.dtype)], opts, prog,
                          sig_extra=(dim, shape[dim]))[0]

    def cat(self, xs: List[T], dim: int) -> T:
        dim %= xs[0].rank
        shape = tuple(sum(x.shape[dim] for x in xs) if i == dim else s for i, s in enumerate(xs[0].shape))
        n = len(xs)
        opts: List[Option] = [((R,), (R,) * n), ((P,), (P,) * n)]
        for d in range(xs[0].rank):
            if d != dim:
                opts.append(((shard(d),), (shard(d),) * n))
        # output numel = sum of input numels: written as one output per input
        prog = opprog.program([], [(x.itemsize, [opprog.argdim(k, i) for i in range(x.rank)])
                                   for k, x in enumerate(xs)])
        out = self._emit("cat", xs, [(shape, contiguous_stride(shape), xs[0].dtype)], opts, prog,
                         sig_extra=(dim, n))[0]

        def vjp(g):
            res, off = [], 0
            for x in xs:
                res.append(self.slice(g[0], dim, off, off + x.shape[dim]))
                off += x.shape[dim]
            return res

        self._record(xs, [out], vjp)
        return out

    def expand(self, x: T, dim: int, n: int) -> T:
        """expand a size-1 dim to n (view, stride 0)."""
        assert x.shape[dim] == 1
        shape = tuple(n if i == dim else s for i, s in enumerate(x.shape))
        stride = tuple(0 if i == dim else s for i, s in enumerate(x.stride))
        opts: List[Option] = [((R,), (R,)), ((P,), (P,))]
        for d in range(x.rank):
            if d != dim and x.shape[d] != 1:
                opts.append(((shard(d),), (shard(d),)))
        out = self._emit("expand", [x], [(shape, stride, x.dtype)], opts, None, sig_extra=(dim, n))[0]
        self._record([x], [out], lambda g: [self.sum(g[0], [dim], keepdim=True)])
        return out

    def clone(self, x: T) -> T:
        shape = x.shape
        opts: List[Option] = [((R,), (R,)), ((P,), (P,))] + [((shard(d),), (shard(d),)) for d in range(x.rank)]
        out = self._emit("clone", [x], [(shape, contiguous_stride(shape), x.dtype)], opts,
                         opprog.same_as_arg(0, x.rank, x.itemsize))[0]
        self._record([x], [out], lambda g: [g[0]])
        return out

    # ---- reductions -----------------------------------------------------------
    def sum(self, x: T, dims: Sequence[int], keepdim: bool, mean: bool = False) -> T:
        dims = sorted({d % x.rank for d in dims})
        shape = tuple(
            (1 if i in dims else s) for i, s in enumerate(x.shape) if keepdim or i not in dims
        )
        pcode = PARTIAL_AVG if mean else P
        opts: List[Option] = [((R,), (R,)), ((pcode,), (pcode,))]
        j = 0
        for d in range(x.rank):
            if d in dims:
                opts.append(((pcode,), (shard(d),)))
                if keepdim:
                    j += 1
            else:
                opts.append(((shard(j),), (shard(d),)))
                j += 1
        out = self._emit("mean" if mean else "sum", [x], [(shape, contiguous_stride(shape), x.dtype)], opts,
                         opprog.reduction(x.rank, dims, keepdim, x.itemsize),
                         sig_extra=(tuple(dims), keepdim))[0]
        src = x.shape

        def vjp(g):
            gg = g[0]
            if not keepdim:
                gg = self.view(gg, tuple(1 if i in dims else s for i, s in enumerate(src)))
            for d in dims:
                gg = self.expand(gg, d, src[d])
            if mean:
                gg = self.scale(gg, "div_scalar")
            return [gg]

        self._record([x], [out], vjp)
        return out

    def softmax_like(self, name: str, args: List[T], dim: int, n_out: int = 1) -> T:
        x = args[0]
        dim %= x.rank
        opts: List[Option] = [((R,), (R,) * len(args))]
        for d in range(x.rank):
            if d != dim:
                opts.append(((shard(d),), (shard(d),) * len(args)))
        return self._emit(name, args, [(x.shape, contiguous_stride(x.shape), x.dtype)], opts,
                          opprog.same_as_arg(0, x.rank, x.itemsize), sig_extra=(dim,))[0]

    def softmax(self, x: T, dim: int = -1) -> T:
        out = self.softmax_like("softmax", [x], dim)

        def vjp(g):
            return [self.softmax_like("softmax_backward", [g[0], out], dim)]

        self._record([x], [out], vjp)
        return out

    # ---- attention ------------------------------------------------------------
    def sdpa(self, q: T, k: T, v: T) -> T:
        """aten._scaled_dot_product_flash_attention: tuple output (out, lse)."""
        b, h, sq, d = q.shape
        opts: List[Option] = [
            ((R, R), (R, R, R)),
            ((shard(0), shard(0)), (shard(0),) * 3),
            ((shard(1), shard(1)), (shard(1),) * 3),
        ]
        out_shape = (b, h, sq, v.shape[3])
        lse_shape = (b, h, sq)
        outs = self._emit(
            "sdpa_flash", [q, k, v],
            [(out_shape, contiguous_stride(out_shape), q.dtype), (lse_shape, contiguous_stride(lse_shape), DT_F32)],
            opts, opprog.sdpa_flash_fwd(q.itemsize), tuple_output=True)
        o = self.getitem(outs[0])
        lse = self.getitem(outs[1])

        def vjp(g):
            bopts: List[Option] = [
                ((R, R, R), (R,) * 6),
                ((shard(0),) * 3, (shard(0),) * 6),
                ((shard(1),) * 3, (shard(1),) * 6),
            ]
            gs = self._emit(
                "sdpa_flash_backward", [g[0], q, k, v, o, lse],
                [(q.shape, contiguous_stride(q.shape), q.dtype), (k.shape, contiguous_stride(k.shape), k.dtype),
                 (v.shape, contiguous_stride(v.shape), v.dtype)],
                bopts, opprog.sdpa_flash_bwd(q.itemsize), tuple_output=True)
            return [self.getitem(t) for t in gs]

        self._record([q, k, v], [o], vjp)
        return o

    # ---- embedding ------------------------------------------------------------
    def embedding(self, w: T, idx: T) -> T:
        r = idx.rank
        shape = idx.shape + (w.shape[1],)
        opts: List[Option] = [((R,), (R, R))]
        for d in range(r):
            opts.append(((shard(d),), (R, shard(d))))
        opts.append(((shard(r),), (shard(1), R)))
        opts.append(((MASK_PARTIAL,), (shard(0), R)))
        out = self._emit("embedding", [w, idx], [(shape, contiguous_stride(shape), w.dtype)], opts,
                         opprog.embedding(r, w.itemsize))[0]

        def vjp(g):
            bopts: List[Option] = [((R,), (R, R))]
            for d in range(r):
                bopts.append(((P,), (shard(d), shard(d))))
            bopts.append(((shard(1),), (shard(r), R)))
            gw = self._emit("embedding_dense_backward", [g[0], idx],
                            [(w.shape, contiguous_stride(w.shape), w.dtype)], bopts,
                            opprog.embedding_dense_backward(w.shape[0], w.itemsize, g[0].rank))[0]
            return [gw, None]

        self._record([w, idx], [out], vjp)
        return out

    # ---- finishing ---------------------------------------------------------
    def finish(self, param_grads: Dict[int, T], outputs: List[T]) -> PackedGraph:
        """Mark prefetchable edges and pack.

        Param-derived: every input is a parameter or param-derived
        (autoparallel/graph_passes/graph_utils.py:447-459).  Terminal-derived:
        every user is a parameter-gradient node or terminal-derived (:462-484);
        the graph's output node counts as the only user of a gradient node."""
        n = len(self.b.nodes)
        param_derived = set(self.param_nodes)
        for v in range(n):
            ins = self.node_inputs.get(v, [])
            if ins and all(u in param_derived for u in ins):
                param_derived.add(v)
        terminal = set(t.node for t in param_grads.values())
        out_nodes = set(t.node for t in outputs) | terminal
        for v in reversed(range(n)):
            users = self.node_users.get(v, [])
            if v in out_nodes and v not in terminal:
                continue  # also used by the output node
            if users and all(u in terminal for u in users):
                terminal.add(v)
        for v in range(n):
            for a, u in enumerate(self.node_inputs.get(v, [])):
                if u in param_derived or v in terminal:
                    self.b.prefetchable_edges.add((v, a))
        self.param_derived = param_derived
        self.terminal_derived = terminal
        g = self.b.pack()
        g.roles = self._roles(param_grads, outputs)
        g.node_kind = np.asarray([0 if self.node_inputs.get(v) or self.b.nodes[v].op != 0 else 1 for v in range(n)],
                                 np.uint8)
        start = getattr(self, "_bwd_start", None)
        g.node_phase = (np.arange(n) >= (n if start is None else start)).astype(np.int32)
        return g

    def _roles(self, param_grads: Dict[int, T], outputs: List[T]):
        """Forward/backward pairs and dtype-cast chains, as the reference derives
        them from the AOT graph (autoparallel/optimize_sharding.py:1463-1606)."""
        from .sharding_problem import GraphRoles

        names = [n.name for n in self.b.nodes]
        is_cast = lambda v: names[v].startswith("_to_copy")
        roles = GraphRoles()
        roles.param_grad = [(p, (param_grads[p].node if p in param_grads else -1)) for p in self.param_nodes]
        roles.output_tangent = [(o.node, t.node) for o, t in getattr(self, "_tangents", [])]
        metas = self.b._meta_rows
        itemsize_of = lambda v: metas[self.b.nodes[v].out_specs[0][0] >> 12][2]
        for p in self.param_nodes:
            # forward: param -> single-user unary chain -> cast that lowers precision
            chain, n = [], p
            while not is_cast(n):
                users = list(dict.fromkeys(self.node_users.get(n, [])))
                if len(users) != 1 or len(set(self.node_inputs[users[0]])) != 1:
                    break
                n = users[0]
                chain.append(n)
            if is_cast(n) and n != p and itemsize_of(n) < itemsize_of(p):
                roles.fwd_pre_cast.update(chain)
            # backward: grad <- unary chain <- cast
            if p in param_grads:
                g_ = param_grads[p].node
                chain, n = [g_], g_
                while len(set(self.node_inputs.get(n, []))) == 1:
                    parent = self.node_inputs[n][0]
                    if len(set(self.node_inputs.get(parent, []))) != 1:
                        break
                    chain.append(parent)
                    n = parent
                for i, v in enumerate(chain):
                    if is_cast(v):
                        roles.bwd_pre_cast.update(chain[i:])
                        break
        return roles


# ===========================================================================
# Model graphs
# ===========================================================================
def _rmsnorm(t: Tracer, x: T, w: T) -> T:
    xf = t.to_dtype(x, DT_F32)
    sq = t.unary("pow", xf)
    ms = t.sum(sq, [-1], keepdim=True, mean=True)
    ms = t.add_scalar(ms)
    rs = t.unary("rsqrt", ms)
    y = t.mul(xf, rs)
    y = t.to_dtype(y, x.dtype)
    return t.mul(y, w)


def _linear(t: Tracer, x: T, w: T) -> T:
    # nn.Linear weight is [out, in]; the einsum consumes its transposed view
    return t.einsum_fwd(x, t.permute(w, [1, 0]))


def _rope(t: Tracer, x: T, cos: T, sin: T) -> T:
    # rotate-half formulation in fp32, cast back
    xf = t.to_dtype(x, DT_F32)
    d = x.shape[-1]
    x1 = t.slice(xf, -1, 0, d // 2)
    x2 = t.slice(xf, -1, d // 2, d)
    rot = t.cat([t.neg(x2), x1], -1)
    out = t.add(t.mul(xf, cos), t.mul(rot, sin))
    return t.to_dtype(out, x.dtype)


def _repeat_kv(t: Tracer, x: T, n_rep: int) -> T:
    if n_rep == 1:
        return x
    b, s, h, d = x.shape
    x = t.view(x, (b, s, h, 1, d))
    x = t.expand(x, 3, n_rep)
    x = t.clone(x)
    return t.view(x, (b, s, h * n_rep, d))


def llama_graph(
    mesh_shape: Sequence[int],
    n_layers: int,
    dim: int,
    n_heads: int,
    n_kv_heads: int,
    ffn_dim: int,
    vocab: int,
    seq: int,
    batch: int,
    devices_per_host: int = 8,
    dtype: int = DT_BF16,
) -> PackedGraph:
    """Llama-3-style decoder (RMSNorm, RoPE, GQA, SwiGLU), forward + backward,
    logits as the output with a tangent input, as an AOT joint graph has."""
    t = Tracer(mesh_shape, devices_per_host)
    hd = dim // n_heads
    params: Dict[str, T] = {}

    def P_(name, shape):
        params[name] = t.placeholder(name, shape, dtype, param=True)
        return params[name]

    tok_emb = P_("tok_embeddings.weight", (vocab, dim))
    layers = []
    for i in range(n_layers):
        layers.append(
            dict(
                attn_norm=P_(f"layers.{i}.attention_norm.weight", (dim,)),
                wq=P_(f"layers.{i}.attention.wq.weight", (n_heads * hd, dim)),
                wk=P_(f"layers.{i}.attention.wk.weight", (n_kv_heads * hd, dim)),
                wv=P_(f"layers.{i}.attention.wv.weight", (n_kv_heads * hd, dim)),
                wo=P_(f"layers.{i}.attention.wo.weight", (dim, n_heads * hd)),
                ffn_norm=P_(f"layers.{i}.ffn_norm.weight", (dim,)),
                w1=P_(f"layers.{i}.feed_forward.w1.weight", (ffn_dim, dim)),
                w2=P_(f"layers.{i}.feed_forward.w2.weight", (dim, ffn_dim)),
                w3=P_(f"layers.{i}.feed_forward.w3.weight", (ffn_dim, dim)),
            )
        )
    norm_w = P_("norm.weight", (dim,))
    out_w = P_("output.weight", (vocab, dim))
    cos = t.placeholder("rope_cos", (1, seq, 1, hd), DT_F32)
    sin = t.placeholder("rope_sin", (1, seq, 1, hd), DT_F32)
    tokens = t.placeholder("tokens", (batch, seq), DT_OTHER)
    tangent = t.placeholder("tangents_1", (batch, seq, vocab), dtype)

    h = t.embedding(tok_emb, tokens)
    for L in layers:
        x = _rmsnorm(t, h, L["attn_norm"])
        q = t.view(_linear(t, x, L["wq"]), (batch, seq, n_heads, hd))
        k = t.view(_linear(t, x, L["wk"]), (batch, seq, n_kv_heads, hd))
        v = t.view(_linear(t, x, L["wv"]), (batch, seq, n_kv_heads, hd))
        q = _rope(t, q, cos, sin)
        k = _rope(t, k, cos, sin)
        k = _repeat_kv(t, k, n_heads // n_kv_heads)
        v = _repeat_kv(t, v, n_heads // n_kv_heads)
        q, k, v = (t.transpose(z, 1, 2) for z in (q, k, v))
        o = t.sdpa(q, k, v)
        o = t.clone(t.transpose(o, 1, 2))
        o = t.view(o, (batch, seq, n_heads * hd))
        h = t.add(h, _linear(t, o, L["wo"]))
        x = _rmsnorm(t, h, L["ffn_norm"])
        g = t.unary("silu", _linear(t, x, L["w1"]))
        u = _linear(t, x, L["w3"])
        h = t.add(h, _linear(t, t.mul(g, u), L["w2"]))
    h = _rmsnorm(t, h, norm_w)
    logits = _linear(t, h, out_w)
    grads = t.backward([(logits, tangent)])
    t._tangents = [(logits, tangent)]
    param_grads = {}
    for name, p in params.items():
        g = grads.get((p.node, None))
        if g is not None:
            param_grads[p.node] = t.alias(g)
    return t.finish(param_grads, [logits])


def moe_dispatch_bytes(n_layers: int, n_experts: int, top_k: int, tokens: int, dim: int, itemsize: int,
                       dp: int, ep: int, seed: int = 0) -> np.ndarray:
    """Bytes one expert-parallel group moves in the dispatch all-to-all of each
    MoE layer when the tokens per expert follow a Zipf(1.1) law (a benchmark
    extension: the reference prices a local_map region at zero and only charges
    the redistribution of its inputs).  Per layer: expert popularity is
    rank^-1.1 over a random permutation of the experts
    (numpy.random.default_rng(seed)); the tokens * top_k / dp routed slots of
    one data-parallel group are split in that proportion; the collective is as
    slow as its most loaded rank, so the volume is ep * (slots of the most
    loaded rank's experts) * dim * itemsize."""
    rng = np.random.default_rng(seed)
    w = np.arange(1, n_experts + 1, dtype=np.float64) ** -1.1
    w /= w.sum()
    slots = tokens * top_k // dp
    out = np.zeros(n_layers, np.int64)
    per_rank = n_experts // ep
    for i in range(n_layers):
        load = np.floor(w[rng.permutation(n_experts)] * slots).astype(np.int64)
        rank_load = load.reshape(ep, per_rank).sum(axis=1)
        out[i] = int(ep * rank_load.max() * dim * itemsize)
    return out


def moe_graph(
    mesh_shape: Sequence[int] = (8, 8),
    n_layers: int = 16,
    dim: int = 2048,
    n_heads: int = 16,
    n_experts: int = 64,
    top_k: int = 6,
    expert_ffn: int = 1408,
    vocab: int = 129280,
    seq: int = 4096,
    batch: int = 32,
    devices_per_host: int = 8,
    dtype: int = DT_BF16,
) -> PackedGraph:
    """DeepSeek-V3-style MoE decoder, forward + backward, on a (dp, ep) mesh:
    attention and a dense shared expert are planned by the optimizer; the
    routed-expert dispatch is a ``local_map`` region with the declared
    placements of the reference's MoE recipe (docs/local_map_and_moe.md:246-268):
    tokens and gate scores (Shard(0), Shard(0)), expert weights
    (Replicate, Shard(0)), output (Shard(0), Shard(0))."""
    t = Tracer(mesh_shape, devices_per_host)
    assert t.ndim == 2, "the MoE recipe is written for a (dp, ep) mesh"
    hd = dim // n_heads
    params: Dict[str, T] = {}

    def P_(name, shape):
        params[name] = t.placeholder(name, shape, dtype, param=True)
        return params[name]

    S0, PS = shard(0), PARTIAL_SUM
    tok_emb = P_("tok_embeddings.weight", (vocab, dim))
    layers = []
    for i in range(n_layers):
        layers.append(dict(
            attn_norm=P_(f"layers.{i}.attention_norm.weight", (dim,)),
            wq=P_(f"layers.{i}.attention.wq.weight", (dim, dim)),
            wk=P_(f"layers.{i}.attention.wk.weight", (dim, dim)),
            wv=P_(f"layers.{i}.attention.wv.weight", (dim, dim)),
            wo=P_(f"layers.{i}.attention.wo.weight", (dim, dim)),
            ffn_norm=P_(f"layers.{i}.ffn_norm.weight", (dim,)),
            gate=P_(f"layers.{i}.moe.gate.weight", (n_experts, dim)),
            ew1=P_(f"layers.{i}.moe.expert_w1", (n_experts, dim, expert_ffn)),
            ew2=P_(f"layers.{i}.moe.expert_w2", (n_experts, expert_ffn, dim)),
            sw1=P_(f"layers.{i}.moe.shared.w1.weight", (expert_ffn, dim)),
            sw2=P_(f"layers.{i}.moe.shared.w2.weight", (dim, expert_ffn)),
            sw3=P_(f"layers.{i}.moe.shared.w3.weight", (expert_ffn, dim)),
        ))
    norm_w = P_("norm.weight", (dim,))
    out_w = P_("output.weight", (vocab, dim))
    cos = t.placeholder("rope_cos", (1, seq, 1, hd), DT_F32)
    sin = t.placeholder("rope_sin", (1, seq, 1, hd), DT_F32)
    tokens = t.placeholder("tokens", (batch, seq), DT_OTHER)
    tangent = t.placeholder("tangents_1", (batch, seq, vocab), dtype)

    h = t.embedding(tok_emb, tokens)
    for L in layers:
        x = _rmsnorm(t, h, L["attn_norm"])
        q, k, v = (t.view(_linear(t, x, L[w]), (batch, seq, n_heads, hd)) for w in ("wq", "wk", "wv"))
        q = _rope(t, q, cos, sin)
        k = _rope(t, k, cos, sin)
        q, k, v = (t.transpose(z, 1, 2) for z in (q, k, v))
        o = t.clone(t.transpose(t.sdpa(q, k, v), 1, 2))
        h = t.add(h, _linear(t, t.view(o, (batch, seq, dim)), L["wo"]))
        x = _rmsnorm(t, h, L["ffn_norm"])
        scores = t.softmax(_linear(t, x, L["gate"]))
        x_flat = t.view(x, (batch * seq, dim))
        g_flat = t.view(scores, (batch * seq, n_experts))
        routed = t.local_map(
            "local_map_moe", [x_flat, g_flat, L["ew1"], L["ew2"]],
            in_plcs=[(S0, S0), (S0, S0), (R, S0), (R, S0)],
            out_meta=(x_flat.shape, x_flat.stride, x_flat.dtype), out_plc=(S0, S0),
            grad_plcs=[(S0, S0), (S0, S0), (PS, S0), (PS, S0)])
        shared = _linear(t, t.mul(t.unary("silu", _linear(t, x, L["sw1"])), _linear(t, x, L["sw3"])), L["sw2"])
        h = t.add(t.add(h, t.view(routed, (batch, seq, dim))), shared)
    h = _rmsnorm(t, h, norm_w)
    logits = _linear(t, h, out_w)
    grads = t.backward([(logits, tangent)])
    t._tangents = [(logits, tangent)]
    param_grads = {}
    for name, p in params.items():
        g = grads.get((p.node, None))
        if g is not None:
            param_grads[p.node] = t.alias(g)
    return t.finish(param_grads, [logits])


def config_moe(n_layers: int = 16) -> PackedGraph:
    return moe_graph((8, 8), n_layers)


def _layernorm(t: Tracer, x: T, w: T, b: T) -> T:
    xf = t.to_dtype(x, DT_F32)
    mu = t.sum(xf, [-1], keepdim=True, mean=True)
    xc = t.add(xf, t.neg(mu))
    var = t.sum(t.unary("pow", xc), [-1], keepdim=True, mean=True)
    rs = t.unary("rsqrt", t.add_scalar(var))
    y = t.to_dtype(t.mul(xc, rs), x.dtype)
    return t.add(t.mul(y, w), b)


def gpt2_graph(
    mesh_shape: Sequence[int],
    n_layers: int = 12,
    dim: int = 768,
    n_heads: int = 12,
    ffn_dim: int = 3072,
    vocab: int = 50257,
    seq: int = 1024,
    batch: int = 8,
    devices_per_host: int = 8,
) -> PackedGraph:
    """GPT-2-style decoder: fp32 master parameters cast to bf16 for compute
    (so gradients come back in fp32), LayerNorm, GELU MLP, learned positions,
    tied output embedding."""
    t = Tracer(mesh_shape, devices_per_host)
    hd = dim // n_heads
    params: Dict[str, T] = {}

    def P_(name, shape):
        params[name] = t.placeholder(name, shape, DT_F32, param=True)
        return t.to_dtype(params[name], DT_BF16)

    wte = P_("wte.weight", (vocab, dim))
    wpe = P_("wpe.weight", (seq, dim))
    tokens = t.placeholder("tokens", (batch, seq), DT_OTHER)
    pos = t.placeholder("positions", (1, seq), DT_OTHER)
    tangent = t.placeholder("tangents_1", (batch, seq, vocab), DT_BF16)
    h = t.add(t.embedding(wte, tokens), t.embedding(wpe, pos))
    for i in range(n_layers):
        ln1w, ln1b = P_(f"h.{i}.ln_1.weight", (dim,)), P_(f"h.{i}.ln_1.bias", (dim,))
        wqkv, bqkv = P_(f"h.{i}.attn.c_attn.weight", (3 * dim, dim)), P_(f"h.{i}.attn.c_attn.bias", (3 * dim,))
        wo, bo = P_(f"h.{i}.attn.c_proj.weight", (dim, dim)), P_(f"h.{i}.attn.c_proj.bias", (dim,))
        ln2w, ln2b = P_(f"h.{i}.ln_2.weight", (dim,)), P_(f"h.{i}.ln_2.bias", (dim,))
        wfc, bfc = P_(f"h.{i}.mlp.c_fc.weight", (ffn_dim, dim)), P_(f"h.{i}.mlp.c_fc.bias", (ffn_dim,))
        wpr, bpr = P_(f"h.{i}.mlp.c_proj.weight", (dim, ffn_dim)), P_(f"h.{i}.mlp.c_proj.bias", (dim,))
        x = _layernorm(t, h, ln1w, ln1b)
        qkv = t.add(_linear(t, x, wqkv), bqkv)
        q, k, v = (t.slice(qkv, -1, j * dim, (j + 1) * dim) for j in range(3))
        q, k, v = (t.transpose(t.view(z, (batch, seq, n_heads, hd)), 1, 2) for z in (q, k, v))
        o = t.sdpa(q, k, v)
        o = t.view(t.clone(t.transpose(o, 1, 2)), (batch, seq, dim))
        h = t.add(h, t.add(_linear(t, o, wo), bo))
        x = _layernorm(t, h, ln2w, ln2b)
        m = t.unary("gelu", t.add(_linear(t, x, wfc), bfc))
        h = t.add(h, t.add(_linear(t, m, wpr), bpr))
    lnfw, lnfb = P_("ln_f.weight", (dim,)), P_("ln_f.bias", (dim,))
    h = _layernorm(t, h, lnfw, lnfb)
    logits = _linear(t, h, wte)
    grads = t.backward([(logits, tangent)])
    t._tangents = [(logits, tangent)]
    param_grads = {}
    for name, p in params.items():
        g = grads.get((p.node, None))
        if g is not None:
            param_grads[p.node] = t.alias(g)
    return t.finish(param_grads, [logits])


# ---- named benchmark configurations ----------------------------------------
def config_gpt2_small() -> PackedGraph:
    return gpt2_graph((8,))


def config_llama3_8b(n_layers: int = 32) -> PackedGraph:
    return llama_graph((8, 8), n_layers, 4096, 32, 8, 14336, 128256, 8192, 64)


def config_llama3_70b(n_layers: int = 80) -> PackedGraph:
    return llama_graph((4, 8, 8), n_layers, 8192, 64, 8, 28672, 128256, 8192, 256)


def _cap_numel(shape: Tuple[int, ...], limit: int = 2**48) -> Tuple[int, ...]:
    """Four dims drawn up to 65536 each can describe a tensor of 2**64 elements,
    which no device holds and int64 byte counts cannot express: the largest dim
    is halved until the tensor has at most ``limit`` elements (no random draw is
    consumed, so everything else about the graph is as before)."""
    shape = list(shape)
    while math.prod(shape) > limit:
        k = shape.index(max(shape))
        shape[k] = max(shape[k] // 2, 1)
    return tuple(shape)


def stress_graph(
    n_nodes: int,
    mesh_shape: Sequence[int] = (4, 8, 8),
    seed: int = 0,
    s_min: int = 4,
    s_max: int = 512,
    mean_out_degree: float = 1.8,
    devices_per_host: int = 8,
) -> PackedGraph:
    """Seeded random planner stress graph: a DAG whose nodes have tensor ranks
    1-4, dims log-uniform in [64, 65536], dtype in {bf16, fp32}, op class in
    {matmul, elementwise, reduction, view}, and ``U[s_min, s_max]`` random
    strategies each.  No two nodes share a tensor meta, so nothing repeats:
    the entry kernel evaluates every entry directly."""
    rng = np.random.default_rng(seed)
    nd = len(mesh_shape)
    b = GraphBuilder(mesh_shape, devices_per_host)
    b.share_compute_slots = False
    ranks, metas, dts = [], [], []
    n_in_total = 0
    for v in range(n_nodes):
        r = int(rng.integers(1, 5))
        shape = _cap_numel(tuple(int(2 ** rng.uniform(6, 16)) for _ in range(r)))
        dt = DT_BF16 if rng.random() < 0.5 else DT_F32
        ranks.append(r)
        dts.append(dt)
        metas.append(b.meta(shape, contiguous_stride(shape), _ITEMSIZE[dt], dt))
        S = int(rng.integers(s_min, s_max + 1))

        def tuples(rank, n):
            codes = np.asarray([R] + [shard(d) for d in range(rank)] + [P])
            return [tuple(int(c) for c in row) for row in codes[rng.integers(0, len(codes), size=(n, nd))]]

        out_specs = [[b.spec(metas[v], t)] for t in tuples(r, S)]
        op = ("matmul", "elementwise", "reduction", "view")[int(rng.integers(0, 4))]
        want_in = 0 if v == 0 else {"matmul": 2, "elementwise": int(rng.integers(1, 3)), "reduction": 1, "view": 1}[op]
        # keep the mean out-degree near the target
        if v > 0 and n_in_total / v > mean_out_degree:
            want_in = min(want_in, 1)
        inputs = [int(rng.integers(0, v)) for _ in range(want_in)]
        n_in_total += len(inputs)
        if not inputs:
            b.add_node(NodeDesc(f"in_{v}", in_specs=[[w[0]] for w in out_specs], out_specs=out_specs, inputs=[],
                                default_rows=[[[0.0]] for _ in out_specs]))
            continue
        cols = [[b.spec(metas[u], t) for t in tuples(ranks[u], S)] for u in inputs]
        in_specs = [[c[o] for c in cols] for o in range(S)]
        isz = _ITEMSIZE[dt]
        if op == "view":
            desc = NodeDesc(f"view_{v}", in_specs=in_specs, out_specs=out_specs, inputs=inputs)
        elif op == "matmul":
            from .packed import OP_EXPLICIT

            desc = NodeDesc(f"matmul_{v}", in_specs=in_specs, out_specs=out_specs, inputs=inputs, op=OP_EXPLICIT,
                            flops=[int(x) for x in rng.integers(1, 2**44, size=S)],
                            nbytes=[int(x) for x in rng.integers(1, 2**34, size=S)])
        elif op == "reduction":
            ru = ranks[inputs[0]]
            desc = NodeDesc(f"reduction_{v}", in_specs=in_specs, out_specs=out_specs, inputs=inputs, op=OP_PROGRAM,
                            program=opprog.reduction(ru, [ru - 1], True, isz))
        else:
            ru = max(ranks[u] for u in inputs)
            desc = NodeDesc(f"elementwise_{v}", in_specs=in_specs, out_specs=out_specs, inputs=inputs, op=OP_PROGRAM,
                            program=opprog.pointwise(ru, isz))
        b.add_node(desc)
    return b.pack()


# ---------------------------------------------------------------------------
# The stress DAG in windows: every node is drawn from its own counter-based
# generator, so any range of nodes can be produced without the rest.
# ---------------------------------------------------------------------------
def _stress_header(seed: int, v: int, nd: int, s_min: int, s_max: int):
    """(rank, shape, dtype, out placement tuples) of node v, from (seed, v) alone."""
    rng = np.random.default_rng([seed, v, 0])
    r = int(rng.integers(1, 5))
    shape = _cap_numel(tuple(int(2 ** rng.uniform(6, 16)) for _ in range(r)))
    dt = DT_BF16 if rng.random() < 0.5 else DT_F32
    S = int(rng.integers(s_min, s_max + 1))
    codes = np.asarray([R] + [shard(d) for d in range(r)] + [P])
    out = codes[rng.integers(0, len(codes), size=(S, nd))]  # int array [S, nd]
    return r, shape, dt, out


def _stress_body(seed: int, v: int, nd: int, header):
    """(op class, producers, placement codes int[S, nd] of the input spec per producer and
    strategy, the node's generator for what else it draws) of node v, from (seed, v) and the
    headers of its producers alone."""
    rng = np.random.default_rng([seed, v, 1])
    op = ("matmul", "elementwise", "reduction", "view")[int(rng.integers(0, 4))]
    if v == 0:
        want_in = 0
    elif op == "matmul":
        want_in = 3 if rng.random() < 0.7 else 2  # with or without a bias
    elif op == "elementwise":
        want_in = int(rng.integers(1, 5))
    else:
        want_in = 1
    inputs = [int(rng.integers(0, v)) for _ in range(want_in)]
    S = len(header(v)[3])
    in_codes = []
    for u in inputs:
        ru = header(u)[0]
        codes = np.asarray([R] + [shard(d) for d in range(ru)] + [P])
        in_codes.append(codes[rng.integers(0, len(codes), size=(S, nd))])
    return op, inputs, in_codes, rng


def stress_dag_partial_masks(n_total: int, lo: int, hi: int, mesh_shape: Sequence[int] = (4, 8, 8), seed: int = 0,
                             s_min: int = 4, s_max: int = 512):
    """{v: feasible_plan.NodeMasks} for the nodes [lo, hi) of the stress DAG, without
    building their window: which mesh dims hold a Partial in the output spec of every
    strategy and in its input spec per producer (what feasible_plan.window_masks reads
    off the packed window)."""
    from .feasible_plan import NodeMasks

    assert 0 <= lo < hi <= n_total
    nd = len(mesh_shape)
    headers = {}

    def header(v):
        if v not in headers:
            headers[v] = _stress_header(seed, v, nd, s_min, s_max)
        return headers[v]

    weights = 1 << np.arange(nd)

    def mask(codes):
        return (((codes & PLC_KIND_MASK) == PLC_PARTIAL) * weights).sum(axis=1).astype(np.uint8)

    out = {}
    for v in range(lo, hi):
        _, inputs, in_codes, _ = _stress_body(seed, v, nd, header)
        out[v] = NodeMasks(out=mask(header(v)[3]), producers=list(inputs), wants=[mask(c) for c in in_codes]).finish()
    return out


def stress_dag_window(
    n_total: int,
    lo: int,
    hi: int,
    mesh_shape: Sequence[int] = (4, 8, 8),
    seed: int = 0,
    s_min: int = 4,
    s_max: int = 512,
    devices_per_host: int = 8,
):
    """Nodes [lo, hi) of the seeded n_total-node stress DAG (ranks 1-4, dims
    log-uniform in [64, 65536], bf16 / fp32, op class uniform over {matmul,
    elementwise, reduction, view}, U[s_min, s_max] strategies per node, mean
    in-degree 1.8 with producers uniform over the earlier nodes), as a packed
    graph of its own.  Producers below ``lo`` come first as stand-in input nodes
    with the producer's real output specs, so every edge of the window has its
    producer run; ``window(0, n_total)`` is the whole DAG.
    Returns (graph, node_gid int32[N] index of every local node in the whole
    DAG, n_standin)."""
    assert 0 <= lo < hi <= n_total
    nd = len(mesh_shape)
    headers = {}

    def header(v):
        if v not in headers:
            headers[v] = _stress_header(seed, v, nd, s_min, s_max)
        return headers[v]

    bodies = []
    external = set()
    for v in range(lo, hi):
        op, inputs, in_codes, rng = _stress_body(seed, v, nd, header)
        external.update(u for u in inputs if u < lo)
        bodies.append((v, op, inputs, in_codes, rng))
    standins = sorted(external)
    local = {u: i for i, u in enumerate(standins)}
    local.update({v: len(standins) + (v - lo) for v in range(lo, hi)})

    b = GraphBuilder(mesh_shape, devices_per_host)
    b.share_compute_slots = False
    metas = {}

    def specs_of(v, tuples):
        if v not in metas:
            r, shape, dt, _ = header(v)
            metas[v] = b.meta(shape, contiguous_stride(shape), _ITEMSIZE[dt], dt)
        return b.specs(metas[v], tuples)

    def add_input(v):
        out = [[w] for w in specs_of(v, header(v)[3])]
        b.add_node(NodeDesc(f"in_{v}", in_specs=out, out_specs=out, inputs=[],
                            default_rows=[[[0.0]] for _ in out]))

    for u in standins:
        add_input(u)
    for v, op, inputs, in_codes, rng in bodies:
        r, shape, dt, out_tuples = header(v)
        if not inputs:
            add_input(v)
            continue
        S = len(out_tuples)
        out_specs = [[w] for w in specs_of(v, out_tuples)]
        cols = [specs_of(u, codes) for u, codes in zip(inputs, in_codes)]
        in_specs = [list(row) for row in zip(*cols)]
        loc = [local[u] for u in inputs]
        isz = _ITEMSIZE[dt]
        if op == "view":
            desc = NodeDesc(f"view_{v}", in_specs=in_specs, out_specs=out_specs, inputs=loc)
        elif op == "matmul":
            from .packed import OP_EXPLICIT

            desc = NodeDesc(f"matmul_{v}", in_specs=in_specs, out_specs=out_specs, inputs=loc, op=OP_EXPLICIT,
                            flops=[int(x) for x in rng.integers(1, 2**44, size=S)],
                            nbytes=[int(x) for x in rng.integers(1, 2**34, size=S)])
        elif op == "reduction":
            ru = header(inputs[0])[0]
            desc = NodeDesc(f"reduction_{v}", in_specs=in_specs, out_specs=out_specs, inputs=loc, op=OP_PROGRAM,
                            program=opprog.reduction(ru, [ru - 1], True, isz))
        else:
            ru = max(header(u)[0] for u in inputs)
            desc = NodeDesc(f"elementwise_{v}", in_specs=in_specs, out_specs=out_specs, inputs=loc, op=OP_PROGRAM,
                            program=opprog.pointwise(ru, isz))
        b.add_node(desc)
    gid = np.asarray(standins + list(range(lo, hi)), np.int32)
    return b.pack(), gid, len(standins)

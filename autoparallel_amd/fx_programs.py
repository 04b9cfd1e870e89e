"""From an FX node to what the node kernel consumes: spec words of its tensor
arguments per strategy and either a compute program (closed form) or explicit
(flops, bytes) per strategy.

The reference gets flops and bytes by running the op on sharded FakeTensors
under ``FlopCounterMode`` for every distinct (op, input specs) key
(autoparallel/cost_models/compute_estimation.py:334-365, 383-388, 469-473).
Ops with a closed form here are priced on the device from a program; any other
op takes the reference's route (meta tensors + FlopCounterMode, torch code) on
the host to obtain the two integers, and is counted in ``fallback_ops`` so a
caller can see which ops lack a closed form.  The roofline arithmetic itself
always runs on the device.
"""
from __future__ import annotations

import collections
import ctypes as C
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch
from torch.utils._pytree import tree_flatten

from . import _lib, opprog
from .dtensor_bridge import placement_codes, tensor_meta_key
from .packed import OP_EXPLICIT, OP_PROGRAM, OP_ZERO, GraphBuilder, NodeDesc, spec_word

aten = torch.ops.aten
fallback_ops: "collections.Counter[str]" = collections.Counter()


def non_tensor_args_key(node) -> tuple:
    def h(x):
        if isinstance(x, (list, tuple)):
            return tuple(h(a) for a in x)
        if isinstance(x, torch.Tensor):
            return (tuple(x.shape), tuple(x.stride()), x.dtype)
        return x

    return tuple(h(a) for a in tree_flatten(node.args)[0] if not isinstance(a, torch.fx.Node))


def _tensor_arg_vals(node) -> List[torch.Tensor]:
    vals = []
    for a in tree_flatten(node.args)[0]:
        if isinstance(a, torch.fx.Node) and isinstance(a.meta.get("val"), torch.Tensor):
            vals.append(a.meta["val"])
    return vals


def _out_tensors(node) -> List[torch.Tensor]:
    return [x for x in tree_flatten(node.meta.get("val"))[0] if isinstance(x, torch.Tensor)]


def _closed_form(node) -> Optional[List[int]]:
    """Compute program of the node's op, or None if there is no closed form."""
    t = node.target
    ins = _tensor_arg_vals(node)
    outs = _out_tensors(node)
    if not outs or not ins:
        return None
    o0 = outs[0]
    osz = o0.element_size()
    if t in (aten.mm.default,):
        return opprog.mm(osz)
    if t in (aten.addmm.default,) and len(ins) == 3:
        return opprog.addmm(osz)
    if t in (aten.bmm.default,):
        return opprog.bmm(osz)
    if t is aten.einsum.default and len(ins) == 2:
        a, b = ins
        if b.dim() == 2 and a.dim() >= 3:
            return opprog.einsum_fwd(a.dim(), osz)
        if a.dim() == b.dim() and a.dim() >= 3:
            return opprog.einsum_bwd(a.dim(), osz)
        return None
    if t is aten._scaled_dot_product_flash_attention.default and len(ins) == 3:
        return opprog.sdpa_flash_fwd(ins[0].element_size())
    if t is aten._scaled_dot_product_flash_attention_backward.default and len(ins) >= 6:
        return opprog.sdpa_flash_bwd(ins[1].element_size())
    if t in (aten.sum.dim_IntList, aten.mean.dim) and len(ins) == 1:
        dims = node.args[1] if len(node.args) > 1 else None
        keep = bool(node.args[2]) if len(node.args) > 2 else bool(node.kwargs.get("keepdim", False))
        if dims is None or len(dims) == 0:
            dims = list(range(ins[0].dim()))
        if ins[0].dim() == 0:
            return None
        return opprog.reduction(ins[0].dim(), list(dims), keep, osz)
    if t in (aten._softmax.default, aten._log_softmax.default, aten.clone.default, aten._to_copy.default) and len(ins) == 1:
        return opprog.same_as_arg(0, ins[0].dim(), osz)
    if t in (aten._softmax_backward_data.default, aten._log_softmax_backward_data.default) and len(ins) == 2:
        return opprog.same_as_arg(0, ins[0].dim(), osz)
    if t is aten.embedding.default and len(ins) == 2:
        return opprog.embedding(ins[1].dim(), osz)
    if t is aten.embedding_dense_backward.default and len(ins) == 2 and ins[0].dim() >= 1:
        return opprog.embedding_dense_backward(int(node.args[2]), osz, ins[0].dim())
    if t is aten.cat.default and len(outs) == 1 and all(i.dim() == o0.dim() and i.dtype == o0.dtype for i in ins):
        return opprog.cat(len(ins), osz)
    if t is aten.slice_backward.default and len(ins) == 1 and all(isinstance(x, int) for x in node.args[1]):
        return opprog.constant_shape(node.args[1], osz)
    if t is aten.nll_loss_forward.default and len(outs) == 2 and ins[0].dim() == 2 and isinstance(node.args[3], int):
        # (self [N, C], target [N], weight or None, reduction, ignore_index) -> (loss, total_weight)
        return opprog.nll_loss_forward(node.args[3] == 0, osz, outs[1].element_size())
    if t is aten.nll_loss_backward.default and len(outs) == 1 and len(ins) >= 4:
        # (grad_output, self, target, weight or None, reduction, ignore_index, total_weight) -> grad of self
        return opprog.same_as_arg(1, ins[1].dim(), osz)
    if torch.Tag.pointwise in t.tags and len(outs) == 1:
        # elementwise with broadcasting; the output shape is the broadcast of
        # the tensor arguments only if no argument is shape-expanding by itself
        if tuple(torch.broadcast_shapes(*[tuple(i.shape) for i in ins])) == tuple(o0.shape):
            return opprog.pointwise(o0.dim(), osz)
    return None


def local_shapes(specs: Sequence) -> List[Tuple[List[int], List[int]]]:
    """_get_sharded_shape_stride for a batch of DTensorSpecs, on the device."""
    from .engine import make_model
    from .cost_models.collective_runtime_estimation import _device_name

    if not specs:
        return []
    lib = _lib.load()
    n = len(specs)
    rank = np.zeros(n, np.int32)
    shape = np.ones((n, 8), np.int64)
    stride = np.zeros((n, 8), np.int64)
    plc = np.zeros((n, 4), np.uint8)
    for i, s in enumerate(specs):
        sh, st, _, _ = tensor_meta_key(s.tensor_meta)
        rank[i] = len(sh)
        shape[i, : len(sh)] = sh
        stride[i, : len(st)] = st
        codes = placement_codes(s.placements)
        plc[i, : len(codes)] = codes
    d = lambda a: torch.from_numpy(a).cuda()
    t_rank, t_shape, t_stride, t_plc = d(rank), d(shape), d(stride), d(plc)
    o_shape, o_stride = torch.empty_like(t_shape), torch.empty_like(t_stride)
    m = make_model(tuple(specs[0].mesh.shape), 1, _device_name())
    _lib.check(lib.apc_local_shapes(C.byref(m), n, t_rank.data_ptr(), t_shape.data_ptr(), t_stride.data_ptr(),
                                    t_plc.data_ptr(), o_shape.data_ptr(), o_stride.data_ptr(), None),
               "apc_local_shapes")
    osh, ost = o_shape.cpu().numpy(), o_stride.cpu().numpy()
    return [([int(x) for x in osh[i, : rank[i]]], [int(x) for x in ost[i, : rank[i]]]) for i in range(n)]


def _flops_bytes_via_torch(node, strategies, shapes_fn=None) -> Tuple[List[int], List[int]]:
    """The reference's own route for ops without a closed form: run the op on
    meta tensors of the sharded sizes under FlopCounterMode (torch code).
    ``shapes_fn``: what turns a list of DTensorSpecs into their local (shape,
    stride) pairs; the device's batch form of _get_sharded_shape_stride unless a
    caller brings its own."""
    from torch.utils.flop_counter import FlopCounterMode

    from torch._subclasses.fake_tensor import FakeTensorMode

    flat_specs = [s for st in strategies for s in st.input_specs if s is not None]
    shapes = (shapes_fn or local_shapes)(flat_specs)
    flat_args, treespec = tree_flatten(node.args)
    kwargs = {k: (v.meta["val"] if isinstance(v, torch.fx.Node) else v) for k, v in node.kwargs.items()}
    # Meta tensors carry all the counters need (sizes and dtypes).  An operator that
    # names a device in its arguments (_to_copy) cannot run on them: it runs on fake
    # tensors of the traced tensors' own device instead, as the reference runs
    # every operator (compute_estimation.py:334-365).
    def run(make, mode):
        flops_all, bytes_all = [], []
        it = iter(shapes)
        with mode:
            for st in strategies:
                new_flat, counter = [], 0
                for a in flat_args:
                    if isinstance(a, torch.fx.Node):
                        a = a.meta["val"]
                        if isinstance(a, torch.Tensor):
                            spec = st.input_specs[counter]
                            counter += 1
                            sizes, strides = next(it) if spec is not None else (a.shape, a.stride())
                            a = make(sizes, strides, a)
                    new_flat.append(a)
                args = treespec.unflatten(new_flat)
                with FlopCounterMode(display=False) as fc:
                    out = node.target(*args, **kwargs)
                nbytes = sum(x.numel() * x.element_size() for x in tree_flatten(args)[0] if isinstance(x, torch.Tensor))
                nbytes += sum(x.numel() * x.element_size() for x in tree_flatten(out)[0] if isinstance(x, torch.Tensor))
                flops_all.append(int(fc.get_total_flops()))
                bytes_all.append(int(nbytes))
        return flops_all, bytes_all

    import contextlib

    shapes = list(shapes)
    try:
        return run(lambda sizes, strides, a: torch.empty_strided(sizes, strides, dtype=a.dtype, device="meta"),
                   contextlib.nullcontext())
    except NotImplementedError:
        return run(lambda sizes, strides, a: torch.empty_strided(sizes, strides, dtype=a.dtype, device=a.device),
                   FakeTensorMode(allow_non_fake_inputs=True))


def describe_node(node, strategies, b: GraphBuilder, name: Optional[str] = None,
                  memo: Optional[dict] = None) -> NodeDesc:
    """NodeDesc (without producers) of an FX node with the given OpSpecs.
    ``memo``: a dict kept by the caller over the nodes of one graph (whose specs
    stay alive meanwhile): spec words by spec object, explicit flop/byte counts
    by (operator, spec words, other arguments), so that the repeated layers of a
    model are converted once."""
    words = memo.setdefault("words", {}) if memo is not None else {}
    # tensor metas and placement tuples by value: the specs of a graph are many objects
    # over few distinct metas and tuples, and a dictionary hit costs a tenth of the conversion
    meta_ids = memo.setdefault("meta_ids", {}) if memo is not None else {}
    tuple_ids = memo.setdefault("tuple_ids", {}) if memo is not None else {}

    # ... and by object first: the specs of one answer mostly share their tensor-meta and
    # placement objects (kept alive by the specs, which outlive the memo), and hashing a
    # tensor meta walks its shape and stride tuples
    by_id = memo.setdefault("by_id", {}) if memo is not None else {}

    def word(s) -> int:
        if s is None:
            return -1
        w = words.get(id(s))
        if w is None:
            tm, plc = s.tensor_meta, s.placements
            if tm is None:
                return -1
            m = by_id.get(id(tm))
            t = by_id.get(id(plc))
            if m is None or t is None:
                try:
                    m = meta_ids.get(tm)
                    if m is None:
                        m = meta_ids[tm] = b.meta(*tensor_meta_key(tm))
                    t = tuple_ids.get(plc)
                    if t is None:
                        t = tuple_ids[plc] = b.tuple_id(placement_codes(plc))
                except TypeError:  # a size without a hash
                    m, t = b.meta(*tensor_meta_key(tm)), b.tuple_id(placement_codes(plc))
                by_id[id(tm)] = m
                by_id[id(plc)] = t
            w = spec_word(m, t)
            words[id(s)] = w
        return w

    in_specs, out_specs = [], []
    for st in strategies:
        in_specs.append([word(s) for s in (st.input_specs or [])])
        outs = st.output_specs
        out_specs.append([word(s) for s in (outs if isinstance(outs, (tuple, list)) else [outs])])
    tuple_output = isinstance(strategies[0].output_specs, (tuple, list))
    desc = NodeDesc(name or str(node.name), in_specs=in_specs, out_specs=out_specs, inputs=[],
                    tuple_output=tuple_output)
    # aten._unsafe_view is a reshape that the dispatcher does not tag as a view;
    # run with its global size list on a sharded input it cannot execute at all
    # (the reference rewrites the view-mm-view pattern that produces it away,
    # autoparallel/graph_passes/graph_utils.py:415-439), so it is priced as the
    # view it is.
    zero = (node.op != "call_function" or not isinstance(node.target, torch._ops.OpOverload)
            or node.target.is_view or node.target is aten._unsafe_view.default)
    if zero:
        desc.op = OP_ZERO
        return desc
    prog = _closed_form(node)
    n_tensor_specs = len(in_specs[0])
    if prog is not None and len(_tensor_arg_vals(node)) == n_tensor_specs and all(w >= 0 for r in in_specs for w in r):
        desc.op = OP_PROGRAM
        desc.program = prog
        return desc
    fallback_ops[str(node.target)] += 1
    desc.op = OP_EXPLICIT
    key = None
    if memo is not None:
        try:
            others = tuple(repr(a) if not isinstance(a, torch.fx.Node) else
                           ("T", tuple(a.meta["val"].shape), a.meta["val"].dtype) if isinstance(a.meta.get("val"), torch.Tensor)
                           else ("N",) for a in tree_flatten((node.args, node.kwargs))[0])
            key = (node.target, tuple(map(tuple, in_specs)), others)
            hit = memo.setdefault("explicit", {}).get(key)
            if hit is not None:
                desc.flops, desc.nbytes = list(hit[0]), list(hit[1])
                return desc
        except Exception:
            key = None
    desc.flops, desc.nbytes = _flops_bytes_via_torch(node, strategies)
    if key is not None:
        memo["explicit"][key] = (list(desc.flops), list(desc.nbytes))
    return desc

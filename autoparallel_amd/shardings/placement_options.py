"""Per-node strategy enumeration on the host.

The strategies of an operator come from torch's DTensor sharding propagator
(third-party code, as in the reference:
autoparallel/shardings/dtensor_sharding_helpers.py:327-361); this module wraps
it with the reference's post-processing — tensor-meta fill
(autoparallel/shardings/placement_options.py:60-127), validity filter
(autoparallel/shardings/propagation_rules.py:127-158), de-duplication
(placement_options.py:151-170) — and the few rules DTensor lacks or refuses
(getitem, strict views, alias, two-operand einsum, operators without tensor
inputs: propagation_rules.py:412-554; local_map regions and flex_attention: placement_options.py:380-650; all-Replicate fallback:
dtensor_sharding_helpers.py:364-383).  Its output is input data for the cost
engine.  Input/parameter options are enumerated on the device
(apc_enumerate_input_options).
"""
from __future__ import annotations

import contextlib
import ctypes as C
import itertools
import logging
import operator
import threading
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch
from torch.distributed.tensor import DTensor
from torch.distributed.tensor._dtensor_spec import DTensorSpec, TensorMeta
from torch.distributed.tensor._op_schema import OpSchema, OpSpec, OpStrategy, TupleStrategy
from torch.distributed.tensor.placement_types import Partial, Replicate, Shard
from torch.utils._pytree import tree_flatten

from .. import _lib

aten = torch.ops.aten
logger = logging.getLogger(__name__)

fallback_nodes: List[str] = []  # nodes that got the implicit all-Replicate strategy
fallback_reasons: Dict[str, str] = {}  # node name -> why its operator strategy was not used
refused_candidates: List[str] = []  # one line per query in which a strategy rule refused some of the candidates

# An operator without a registered strategy function gets the all-Replicate
# stand-in, with a warning, as the reference's driver arranges
# (autoparallel/shardings/placement_options.py:331 inside with_implicit_strategies,
# dtensor_sharding_helpers.py:327-361).  Anything else that goes wrong for a
# node (a rule or strategy function that raises, strategies whose input specs do
# not match the node's tensor inputs, no strategy left after the validity
# filter) is an error, as it is there, unless a caller opts into the stand-in
# for those as well.
_stand_in_on_error = False


@contextlib.contextmanager
def replicate_stand_in_on_error():
    """Inside: a node whose strategies cannot be produced gets the
    all-Replicate stand-in (logged as a warning, reason kept in
    ``fallback_reasons``) instead of raising."""
    global _stand_in_on_error
    old, _stand_in_on_error = _stand_in_on_error, True
    try:
        yield
    finally:
        _stand_in_on_error = old


def _tensor_meta(t: torch.Tensor) -> TensorMeta:
    return TensorMeta(t.shape, t.stride(), t.dtype)


# ---------------------------------------------------------------------------
# inputs / parameters
# ---------------------------------------------------------------------------
def enumerate_input_placements(mesh_shape: Sequence[int], shapes: Sequence[Sequence[int]]) -> List[List[tuple]]:
    """Valid {Replicate, Shard(d)} tuples of each shape, itertools.product
    order, from the device kernel."""
    from ..cost_models.collective_runtime_estimation import _device_name
    from ..engine import make_model

    lib = _lib.load()
    n = len(shapes)
    nd = len(mesh_shape)
    rank = np.asarray([len(s) for s in shapes], np.int32)
    shp = np.ones((n, 8), np.int64)
    for i, s in enumerate(shapes):
        shp[i, : len(s)] = [int(x) for x in s]
    off = np.zeros(n + 1, np.int64)
    np.cumsum((rank.astype(np.int64) + 1) ** nd, out=off[1:])
    d = lambda a: torch.from_numpy(a).cuda()
    t_rank, t_shape, t_off = d(rank), d(shp), d(off)
    valid = torch.zeros(int(off[-1]), dtype=torch.uint8, device="cuda")
    plc = torch.zeros(int(off[-1]) * 4, dtype=torch.uint8, device="cuda")
    model = make_model(tuple(mesh_shape), 1, _device_name())
    _lib.check(lib.apc_enumerate_input_options(C.byref(model), n, t_rank.data_ptr(), t_shape.data_ptr(),
                                               t_off.data_ptr(), valid.data_ptr(), plc.data_ptr(), None),
               "apc_enumerate_input_options")
    valid, plc = valid.cpu().numpy(), plc.cpu().numpy().reshape(-1, 4)
    out = []
    for i in range(n):
        rows = []
        for j in range(off[i], off[i + 1]):
            if valid[j]:
                rows.append(tuple(Replicate() if c == 0 else Shard(int(c) & 0x3F) for c in plc[j, :nd]))
        out.append(rows)
    return out


# input / parameter options by (mesh, tensor meta): the specs (which nothing writes to: they
# are complete) and the id of the answer, as for operator queries.  The parameters of a model
# have a handful of distinct shapes; a spec object costs ten microseconds to make and an
# enumeration a kernel launch.
_input_options_cache: Dict[tuple, tuple] = {}
_query_serial = itertools.count()  # never restarts: an id names one answer for the life of the process


def _create_all_options(mesh, shape, tensor_meta=None, tensor=None) -> OpStrategy:
    if tensor is not None:
        tensor_meta = _tensor_meta(tensor)
    if tensor_meta is None:
        t = torch.empty(tuple(shape), device="meta")
        tensor_meta = _tensor_meta(t)
    try:
        key = (mesh, tuple(shape), tensor_meta)
        hit = _input_options_cache.get(key)
    except TypeError:  # a symbolic size
        key = hit = None
    if hit is None:
        rows = enumerate_input_placements(tuple(mesh.shape), [tuple(shape)])[0]
        hit = ([DTensorSpec(mesh, plc, tensor_meta=tensor_meta) for plc in rows], next(_query_serial))
        if key is not None:
            _input_options_cache[key] = hit
    specs, qid = hit
    out = OpStrategy([OpSpec(spec, input_specs=[spec], redistribute_cost=[[0.0]]) for spec in specs])
    out._apc_query_id = qid  # equal ids: equal strategies (what a packer may memoise on)
    return out


# ---------------------------------------------------------------------------
# post-processing of operator strategies
# ---------------------------------------------------------------------------
def _spec_ok(spec: DTensorSpec, mesh_shape) -> bool:
    shape = list(spec.tensor_meta.shape)
    for n, p in zip(mesh_shape, spec.placements):
        if p.is_shard():
            if shape[p.dim] >= n:
                shape[p.dim] = (shape[p.dim] + n - 1) // n
            else:
                return False
    return True


def remove_invalid_configs(out_strat: OpStrategy, mesh) -> OpStrategy:
    kept = []
    mesh_shape = tuple(mesh.shape)  # DeviceMesh.shape rebuilds its layout on every access
    for st in out_strat.strategies:
        outs = st.output_specs
        outs = [outs] if isinstance(outs, DTensorSpec) else list(outs or [])
        specs = list(st.input_specs or []) + outs
        if all(s is None or _spec_ok(s, mesh_shape) for s in specs):
            kept.append(st)
    return OpStrategy(kept)


def keep_unique_configs(op_strat: OpStrategy) -> OpStrategy:
    seen, kept = set(), []
    for st in op_strat.strategies:
        ins = tuple(st.input_specs) if st.input_specs is not None else None
        outs = tuple(st.output_specs) if isinstance(st.output_specs, list) else st.output_specs
        try:
            key = (ins, outs)
            if key in seen:
                continue
            seen.add(key)
        except TypeError:
            pass
        kept.append(st)
    return OpStrategy(kept)


class _SpecWords:
    """Spec words (tensor-meta id << 12 | placement-tuple id, as in the packed
    problem) of the DTensorSpecs of one mesh, interned by value, with the two
    tables on the device; kept between queries."""

    def __init__(self, mesh_shape):
        from ..packed import GraphBuilder

        self.b = GraphBuilder(tuple(mesh_shape))
        self.meta_ids: Dict[object, int] = {}
        self.tuple_ids: Dict[object, int] = {}
        self.uploaded = (-1, -1)
        self.d_rank = self.d_shape = self.d_plc = None

    def word(self, spec) -> int:
        from ..dtensor_bridge import placement_codes, tensor_meta_key
        from ..packed import SPEC_NONE, spec_word

        if spec is None:
            return SPEC_NONE
        tm, plc = spec.tensor_meta, spec.placements
        m = self.meta_ids.get(tm)
        if m is None:
            m = self.meta_ids[tm] = self.b.meta(*tensor_meta_key(tm))
        t = self.tuple_ids.get(plc)
        if t is None:
            t = self.tuple_ids[plc] = self.b.tuple_id(placement_codes(plc))
        return spec_word(m, t)

    def tables(self):
        b = self.b
        n = (len(b._meta_rows), len(b._tuple_rows))
        if n != self.uploaded:
            rank = np.asarray([len(r[0]) for r in b._meta_rows], np.int32)
            shape = np.ones((n[0], 8), np.int64)
            for i, r in enumerate(b._meta_rows):
                shape[i, : len(r[0])] = r[0]
            plc = np.zeros((n[1], 4), np.uint8)
            for i, r in enumerate(b._tuple_rows):
                plc[i, : len(r)] = r
            self.d_rank, self.d_shape, self.d_plc = (torch.from_numpy(a).cuda() for a in (rank, shape, plc))
            self.uploaded = n
        return n, self.d_rank, self.d_shape, self.d_plc


_spec_words: Dict[tuple, _SpecWords] = {}
# sets of at least this many strategies are filtered on the device (below, the launch and
# the two copies cost more than the loop over a few dozen OpSpecs)
DEVICE_FILTER_FROM = 32


def strategy_rows(strategies, table: _SpecWords) -> Optional[np.ndarray]:
    """uint32[n, width]: per strategy the words of its input specs, then of its
    output specs.  None when the set has no such form (strategies of different
    widths, a spec without its tensor meta)."""
    rows = []
    for st in strategies:
        outs = st.output_specs
        outs = [outs] if isinstance(outs, DTensorSpec) else list(outs or [])
        specs = (list(st.input_specs) if st.input_specs is not None else []) + outs
        if any(sp is not None and sp.tensor_meta is None for sp in specs):
            return None
        rows.append([table.word(sp) for sp in specs])
    if not rows or any(len(r) != len(rows[0]) for r in rows) or not rows[0]:
        return None
    return np.asarray(rows, np.int64).astype(np.uint32)


def filter_masks_on_device(mesh_shape, sets: Sequence[np.ndarray], table: _SpecWords):
    """(valid, keep) uint8 per row of every set (apc_filter_strategies), the sets'
    rows one after the other."""
    from ..cost_models.collective_runtime_estimation import _device_name
    from ..engine import make_model

    lib = _lib.load()
    n_rows = np.asarray([r.shape[0] for r in sets], np.int64)
    width = np.asarray([r.shape[1] for r in sets], np.int32)
    set_row = np.zeros(len(sets) + 1, np.int64)
    np.cumsum(n_rows, out=set_row[1:])
    set_word = np.zeros(len(sets), np.int64)
    np.cumsum((n_rows * width)[:-1], out=set_word[1:])
    words = np.concatenate([r.reshape(-1) for r in sets]).view(np.int32)
    (n_meta, n_tuple), d_rank, d_shape, d_plc = table.tables()
    d = lambda a: torch.from_numpy(a).cuda()
    t_row, t_width, t_word, t_words = d(set_row), d(width), d(set_word), d(words)
    masks = torch.empty((2, int(set_row[-1])), dtype=torch.uint8, device="cuda")
    model = make_model(tuple(mesh_shape), 1, _device_name())
    _lib.check(lib.apc_filter_strategies(
        C.byref(model), n_meta, d_rank.data_ptr(), d_shape.data_ptr(), n_tuple, d_plc.data_ptr(), len(sets),
        t_row.data_ptr(), t_width.data_ptr(), t_word.data_ptr(), t_words.data_ptr(), int(n_rows.max()),
        masks[0].data_ptr(), masks[1].data_ptr(), None), "apc_filter_strategies")
    out = masks.cpu().numpy()
    return out[0], out[1]


def filter_strategies(out_strat: OpStrategy, mesh) -> OpStrategy:
    """remove_invalid_configs then keep_unique_configs.  Sets of DEVICE_FILTER_FROM
    strategies or more go through the device in packed form; smaller ones, and sets
    without that form, through the two loops."""
    sts = out_strat.strategies
    if DEVICE_FILTER_FROM <= len(sts) <= 4096:
        mesh_shape = tuple(mesh.shape)
        table = _spec_words.get((mesh, mesh_shape))
        if table is None:
            table = _spec_words[(mesh, mesh_shape)] = _SpecWords(mesh_shape)
        try:
            rows = strategy_rows(sts, table)
        except (TypeError, AssertionError):  # an unhashable size, a tensor of more dims than the tables hold
            rows = None
        if rows is not None:
            _, keep = filter_masks_on_device(mesh_shape, [rows], table)
            return OpStrategy([st for st, k in zip(sts, keep.tolist()) if k])
    return keep_unique_configs(remove_invalid_configs(out_strat, mesh))


def propagate_tensor_meta(node, arg_vals: List[torch.Tensor], out_strat: OpStrategy, mesh=None) -> None:
    out_val = node.meta.get("val")
    for st in out_strat.strategies:
        outs = st.output_specs
        if isinstance(outs, DTensorSpec):
            if isinstance(out_val, torch.Tensor):
                outs.tensor_meta = _tensor_meta(out_val)
            elif isinstance(out_val, (tuple, list)):
                # one spec given for an operator with several outputs (the norms:
                # "out, mean and rstd have the same placements"): one per tensor output
                st.output_specs = tuple(
                    DTensorSpec(outs.mesh, outs.placements, tensor_meta=_tensor_meta(v))
                    if isinstance(v, torch.Tensor) else None for v in out_val)
        elif outs is not None:
            vals = list(out_val) if isinstance(out_val, (tuple, list)) else [out_val]
            # an output DTensor leaves without a spec is Replicate; a spec for an
            # output that does not exist is dropped
            # (autoparallel/shardings/placement_options.py:72-101)
            if mesh is None:
                mesh = st.mesh
            fixed = []
            for s, v in zip(outs, vals):
                if isinstance(v, torch.Tensor):
                    if s is None:
                        s = DTensorSpec(mesh, (Replicate(),) * mesh.ndim)
                    if s.tensor_meta is None or s.tensor_meta != _tensor_meta(v):
                        s.tensor_meta = _tensor_meta(v)
                else:
                    s = None
                fixed.append(s)
            st.output_specs = tuple(fixed) + tuple(outs[len(fixed):])
        if st.input_specs is not None:
            for s, v in zip(st.input_specs, arg_vals):
                if s is not None and s.tensor_meta is None:
                    s.tensor_meta = _tensor_meta(v)


def _unshare_specs(out_strat: OpStrategy, producers: List[OpStrategy]) -> None:
    """Some strategy functions hand back a producer's own spec object as the
    input spec, or one object as both input and output spec (DTensor's select
    when the selected dim is not sharded; the reference copies it there,
    autoparallel/shardings/propagation_rules.py:318-355).  The tensor-meta fill
    writes into specs, so every spec of the new strategies gets an object of its
    own first."""
    import dataclasses

    taken = set()
    for p in producers:
        for st in p.strategies:
            outs = st.output_specs
            for sp in (outs if isinstance(outs, (tuple, list)) else (outs,)):
                if sp is not None:
                    taken.add(id(sp))

    def own(sp):
        if sp is None:
            return None
        if id(sp) in taken:
            sp = dataclasses.replace(sp)
        taken.add(id(sp))
        return sp

    for st in out_strat.strategies:
        if st.input_specs is not None:
            ins = [own(sp) for sp in st.input_specs]
            if any(a is not b for a, b in zip(ins, st.input_specs)):
                st.input_specs = tuple(ins) if isinstance(st.input_specs, tuple) else ins
        outs = st.output_specs
        if isinstance(outs, DTensorSpec):
            st.output_specs = own(outs)
        elif outs is not None:
            new = tuple(own(sp) for sp in outs)
            if any(a is not b for a, b in zip(new, outs)):
                st.output_specs = new


def fill_redistribute_cost(out_strat: OpStrategy, producers: List[OpStrategy]) -> None:
    """Rows of the right shape (one per tensor argument, one column per
    producer strategy); the values are overwritten by the cost engine."""
    for st in out_strat.strategies:
        st.redistribute_cost = [[0.0] * len(p.strategies) for p in producers] or [[0.0]]


# ---------------------------------------------------------------------------
# rules
# ---------------------------------------------------------------------------
def _follow_input(mesh, src: OpStrategy, out_val) -> OpStrategy:
    """One strategy per distinct producer output placement: output == input."""
    tm = _tensor_meta(out_val)
    seen, sts = set(), []
    for s in src.strategies:
        spec = s.output_specs
        if not isinstance(spec, DTensorSpec) or spec.placements in seen:
            continue
        seen.add(spec.placements)
        sts.append(OpSpec(DTensorSpec(mesh, spec.placements, tensor_meta=tm),
                          input_specs=[DTensorSpec(mesh, spec.placements, tensor_meta=spec.tensor_meta)]))
    return OpStrategy(sts)


def _getitem_rule(mesh, node, src: OpStrategy) -> OpStrategy:
    idx = node.args[1]
    seen, sts = set(), []
    for s in src.strategies:
        spec = s.output_specs[idx]
        if spec is None or spec.placements in seen:
            continue
        seen.add(spec.placements)
        sts.append(OpSpec(DTensorSpec(mesh, spec.placements, tensor_meta=spec.tensor_meta),
                          input_specs=[DTensorSpec(mesh, spec.placements, tensor_meta=spec.tensor_meta)]))
    return OpStrategy(sts)


def _einsum_rule(mesh, node, a: OpStrategy, b: OpStrategy) -> OpStrategy:
    """Two-operand einsum: product over mesh dims of the single-dim options
    without Partial inputs (the reference's rule,
    autoparallel/shardings/propagation_rules.py:573-590)."""
    from torch.distributed.tensor._ops._einsum_strategy import gen_einsum_strategies

    eq = node.args[0]
    full = gen_einsum_strategies(eq, mesh)
    sts = []
    for st in full.strategies:
        if any(p.is_partial() for s in st.input_specs for p in s.placements):
            continue
        sts.append(OpSpec(st.output_specs, input_specs=list(st.input_specs)))
    return OpStrategy(sts)


def _replicate_fallback(mesh, node, arg_vals) -> OpStrategy:
    rep = (Replicate(),) * mesh.ndim
    out_val = node.meta.get("val")
    if isinstance(out_val, torch.Tensor):
        out = DTensorSpec(mesh, rep, tensor_meta=_tensor_meta(out_val))
    else:
        out = tuple(DTensorSpec(mesh, rep, tensor_meta=_tensor_meta(v)) if isinstance(v, torch.Tensor) else None
                    for v in out_val)
    ins = [DTensorSpec(mesh, rep, tensor_meta=_tensor_meta(v) if isinstance(v, torch.Tensor) else None)
           for v in arg_vals]
    fallback_nodes.append(str(node.name))
    return OpStrategy([OpSpec(out, input_specs=ins)])


_SHAPE_FACTORY_OPS = {aten.zeros.default, aten.ones.default, aten.full.default, aten.empty.memory_format,
                      aten.rand.default, aten.randn.default}


def _inputless_rule(mesh, node) -> OpStrategy:
    """Operators without tensor inputs.  The per-argument loops of the
    coefficient build want one argument, so every strategy carries its output
    spec as a stand-in input spec with a row of zero costs (no producer: the
    zeros stay).  Factories that take a size (zeros, ones, full, empty, rand,
    randn) get every {Shard(d), Replicate} combination over the mesh, Replicate
    last on each mesh dim, and a row as long as that product before filtering
    (autoparallel/shardings/propagation_rules.py:486-554); anything whose values
    depend on the position (iota, :412-421; arange and other generators are
    treated the same way here) and scalar_tensor (:453-484) are Replicate only."""
    tm = _tensor_meta(node.meta["val"])
    if node.target in _SHAPE_FACTORY_OPS:
        from torch.distributed.tensor._ops.utils import is_tensor_shardable

        shape = tuple(tm.shape)
        per_dim = [Shard(i) for i in range(len(shape))] + [Replicate()]
        combs = list(itertools.product(per_dim, repeat=mesh.ndim))
        sts = []
        for plc in combs:
            spec = DTensorSpec(mesh, tuple(plc), tensor_meta=tm)
            if not is_tensor_shardable(shape, spec):
                continue
            sts.append(OpSpec(spec, input_specs=[spec], redistribute_cost=[[0.0] * len(combs)]))
        return OpStrategy(sts)
    spec = DTensorSpec(mesh, (Replicate(),) * mesh.ndim, tensor_meta=tm)
    return OpStrategy([OpSpec(spec, input_specs=[spec], redistribute_cost=[[0.0]])])


def _view_rule(mesh, node, src: OpStrategy) -> OpStrategy:
    """view as the reference prices it
    (autoparallel/shardings/propagation_rules.py:239-287): one strategy per
    producer strategy, the input demoted to what the view can keep
    (strict_view=False) instead of the refusal of DTensor's own rule; a producer
    strategy the propagation rejects is skipped."""
    from torch.distributed.tensor._ops._view_ops import dim_maps, propagate_shape_and_sharding

    # the target sizes from the result: in a graph traced with symbolic sizes the
    # argument holds nodes (a product of sizes), and a -1 is resolved there already
    rules = dim_maps[torch.Tensor.view](src, tuple(int(d) for d in node.meta["val"].shape))
    out_tm = _tensor_meta(node.meta["val"])
    sts = []
    for s in src.strategies:
        spec = s.output_specs
        try:
            in_plc, out_plc = propagate_shape_and_sharding(spec.placements, tuple(src.shape), rules,
                                                           tuple(mesh.shape), strict_view=False)
        except (AssertionError, RuntimeError):
            continue
        sts.append(OpSpec(DTensorSpec(mesh, tuple(out_plc), tensor_meta=out_tm),
                          input_specs=(DTensorSpec(mesh, tuple(in_plc), tensor_meta=spec.tensor_meta),)))
    return OpStrategy(sts)


def _one_strategy_at_a_time(fn, op, args, kwargs, producers: List[OpStrategy]) -> Optional[OpStrategy]:
    """Some of DTensor's strategy functions (the norms, nll_loss_backward, ...)
    index every tensor argument's strategies with the position in the first
    one's, which holds in eager DTensor (one placement per argument) and fails
    on arguments with different numbers of candidates.  Those are asked once
    per strategy of the argument with the most candidates, every other argument
    standing in with one placement, as at run time: on each mesh dim the lead's
    Shard where it means the same thing for the argument (same rank, same extent
    of that tensor dim), else Replicate.  What the function then asks of an
    argument is priced against the argument's real candidates by the cost engine."""
    if not producers:
        return None
    lead = max(producers, key=lambda p: len(p.strategies))

    def pick(p: OpStrategy, lead_sp: DTensorSpec) -> OpStrategy:
        if p is lead:
            return OpStrategy([lead_st])
        sp = p.strategies[0].output_specs
        if not isinstance(sp, DTensorSpec):
            return OpStrategy([p.strategies[0]])
        a, b = sp.tensor_meta, lead_sp.tensor_meta
        same_rank = a is not None and b is not None and len(a.shape) == len(b.shape)
        plc = tuple(x if same_rank and x.is_shard() and a.shape[x.dim] == b.shape[x.dim] else Replicate()
                    for x in lead_sp.placements)
        spec = DTensorSpec(sp.mesh, plc, tensor_meta=a)
        return OpStrategy([OpSpec(spec, input_specs=(spec,), redistribute_cost=[[0.0]])])

    def narrow(a, plc):
        if isinstance(a, OpStrategy):
            return pick(a, plc)
        if isinstance(a, TupleStrategy):
            return TupleStrategy(tuple(narrow(c, plc) for c in a.children))
        return a

    sts = []
    refused, n_refused = None, 0
    for lead_st in lead.strategies:
        if not isinstance(lead_st.output_specs, DTensorSpec):
            return None
        plc = lead_st.output_specs
        try:
            res = fn(OpSchema(op, tuple(narrow(a, plc) for a in args), kwargs))
        except (ValueError, RuntimeError) as exc:
            # the rule has no answer for this candidate (a mean over shards of unequal size, ...):
            # the operator offers nothing that follows it, and reaching what it does offer
            # from that candidate is priced like any other redistribution
            if refused is None:
                refused = exc
            n_refused += 1
            continue
        if not isinstance(res, OpStrategy):
            return None
        sts.extend(res.strategies)
    if not sts and refused is not None:
        raise refused
    if n_refused:
        # said out loud: a rule that refuses candidates narrows what the node offers, and a
        # rule that does so by mistake would otherwise change plans without a trace
        note = (f"{n_refused} of {len(lead.strategies)} candidates refused by the rule of `{op}`; first: "
                f"{type(refused).__name__}: {refused}")
        logger.warning("%s", note)
        refused_candidates.append(note)
    return OpStrategy(sts)


_reduction_rule_leaks: Optional[bool] = None


def _reduction_rule_carries_state(mesh) -> bool:
    """Whether the installed torch's rule for sum / mean / max ... decides once per call,
    instead of per candidate, if a pending reduction has to be cleared first: one candidate
    that is Partial with another reduce op then makes every later candidate lose its
    shards on the reduced dims (and all of them collapse to the same Replicate answer).
    The reference's tests state the per-candidate behaviour
    (tests/test_reduction_strategies.py:63-117); probed once, on two candidates."""
    global _reduction_rule_leaks
    if _reduction_rule_leaks is None:
        from torch.distributed.tensor._ops._math_ops import common_reduction_strategy

        nd = mesh.ndim
        tm = _tensor_meta(torch.empty((4 * mesh.size(), 4 * mesh.size()), device="meta"))
        cands = [(Partial("avg"),) + (Replicate(),) * (nd - 1), (Shard(0),) + (Replicate(),) * (nd - 1)]
        src = OpStrategy([OpSpec(DTensorSpec(mesh, c, tensor_meta=tm), input_specs=(), redistribute_cost=[]) for c in cands])
        with _without_torch_cost_rows():
            out = common_reduction_strategy(src, reduce_dims=[0], reduction_op="sum")
        _reduction_rule_leaks = not out.strategies[1].output_specs.placements[0].is_partial()
    return _reduction_rule_leaks


def _local_map_rule(mesh, node, schema_args, kw) -> OpStrategy:
    """The single strategy of a ``local_map`` region: the placements its author
    declared (autoparallel/shardings/placement_options.py:380-490).  Arguments
    before the declared ones (the backward region's saved activations) are
    Replicate, as are outputs after the declared ones; an argument or output
    without a placement, or that is not a tensor, has no spec; a tensor with an
    unbacked symbolic size has none either."""
    in_plc, out_plc = kw["in_placements"], kw["out_placements"]
    assert in_plc is not None and out_plc is not None
    assert kw.get("in_grad_placements") is None, "Not yet implemented"
    assert kw.get("device_mesh") in (mesh, None), "Not yet implemented"
    assert "call_local_map" in str(node.target)
    rep = (Replicate(),) * mesh.ndim

    def meta_of(t):
        if any(isinstance(x, torch.SymInt) for x in t.shape) or any(isinstance(x, torch.SymInt) for x in t.stride()):
            return None
        return _tensor_meta(t)

    def spec_of(val, plc):
        if plc is None or not isinstance(val, torch.Tensor):
            return None
        tm = meta_of(val)
        if tm is None:
            return None
        plc = (plc,) if isinstance(plc, (Replicate, Shard, Partial)) else tuple(plc)
        return DTensorSpec(mesh, plc, tensor_meta=tm)

    vals = [a.meta.get("val") if isinstance(a, torch.fx.Node) else a for a in node.args]
    n_act = len(vals) - len(in_plc)
    assert n_act >= 0
    in_specs = [spec_of(v, rep) for v in vals[:n_act]] + [spec_of(v, p) for v, p in zip(vals[n_act:], in_plc)]
    out_val = node.meta["val"]
    outs = list(out_val) if isinstance(out_val, (list, tuple)) else [out_val]
    out_specs = [spec_of(v, p) for v, p in zip(outs, out_plc)] + [spec_of(v, rep) for v in outs[len(out_plc):]]
    kept, rows = [], []
    for arg, spec in zip(schema_args, in_specs):
        if isinstance(arg, OpStrategy):  # other arguments have no sharding and no edge
            kept.append(spec)
            rows.append([0.0] * len(arg.strategies))
    return OpStrategy([OpSpec(tuple(out_specs), input_specs=tuple(kept), redistribute_cost=rows)])


def _product_rule(mesh, rows, n_out: int) -> OpStrategy:
    """Every combination over the mesh dims of single-dim rows
    ``[output placements..., input placements...]``; tensor metas and the
    validity filter come afterwards."""
    sts = []
    for comb in itertools.product(rows, repeat=mesh.ndim):
        specs = [DTensorSpec(mesh, tuple(plc)) for plc in zip(*comb)]
        outs = specs[0] if n_out == 1 else tuple(specs[:n_out])
        sts.append(OpSpec(outs, input_specs=list(specs[n_out:])))
    return OpStrategy(sts)


def _from_propagation_rule(rule, op, mesh, schema_args, producers: List[OpStrategy]) -> Optional[OpStrategy]:
    """Strategies of a gather (``index.Tensor``, ``index_select``) for which the installed torch
    has a run-time propagation rule but no strategy function: the rule is asked once per candidate
    of the indexed tensor, the index tensors Replicate; where it answers with a suggestion (the
    candidate is sharded on an indexed dim) the suggested inputs are taken and it is asked again."""
    if not producers:
        return None

    def replicated(a: OpStrategy) -> DTensorSpec:
        sp = a.strategies[0].output_specs
        return DTensorSpec(mesh, (Replicate(),) * mesh.ndim, tensor_meta=sp.tensor_meta)

    def specs_in(args):
        out = []
        for a in args:
            if isinstance(a, DTensorSpec):
                out.append(a)
            elif isinstance(a, (list, tuple)):
                out.extend(x for x in a if isinstance(x, DTensorSpec))
        return out

    sts, seen = [], set()
    for cand in producers[0].strategies:
        if not isinstance(cand.output_specs, DTensorSpec):
            return None
        first = True
        args = []
        for a in schema_args:
            if isinstance(a, OpStrategy):
                args.append(cand.output_specs if first else replicated(a))
                first = False
            elif isinstance(a, (list, tuple)) and any(isinstance(y, OpStrategy) for y in a):
                args.append([replicated(y) if isinstance(y, OpStrategy) else y for y in a])
            else:
                args.append(a)
        answer = rule(OpSchema(op, tuple(args), {}))
        if answer.output_spec is None and answer.redistribute_schema is not None:
            args = list(answer.redistribute_schema.args_schema)
            answer = rule(answer.redistribute_schema)
        if not isinstance(answer.output_spec, DTensorSpec):
            continue
        ins = specs_in(args)
        key = (answer.output_spec.placements, tuple(x.placements for x in ins))
        if len(ins) == len(producers) and key not in seen:
            seen.add(key)
            sts.append(OpSpec(DTensorSpec(mesh, answer.output_spec.placements),
                              input_specs=tuple(DTensorSpec(mesh, x.placements, tensor_meta=x.tensor_meta) for x in ins)))
    return OpStrategy(sts) if sts else None


def _conv_rule(mesh, node, producers: List[OpStrategy]) -> OpStrategy:
    """Convolution where the installed torch registers no strategy for it (it has a
    run-time propagation rule only): per mesh dim either everything Replicate, or the
    batch sharded with weight and bias Replicate, which is exact because the operator
    is linear in the batch: the output (and the input gradient) is sharded on the batch,
    the weight and bias gradients are pending sums.  Sharding channels or spatial dims
    would need halo exchanges or other collectives inside the operator and is not offered."""
    R, S0, P = Replicate(), Shard(0), Partial()
    if node.target is aten.convolution.default:
        n_in = len(producers)  # input, weight, and bias when there is one
        rows = [[R] + [R] * n_in, [S0] + [S0, R] + [R] * (n_in - 2)]
        return _product_rule(mesh, rows, 1)
    assert len(producers) == 3  # grad_output, input, weight -> grad_input, grad_weight, grad_bias
    rows = [[R, R, R] + [R, R, R], [S0, P, P] + [S0, S0, R]]
    return _product_rule(mesh, rows, 3)


def _stack_rule(mesh, node, producers: List[OpStrategy]) -> OpStrategy:
    """stack: inputs all Replicate or all sharded on the same dim, the output on
    that dim shifted past the new one (autoparallel/shardings/propagation_rules.py:621-656;
    DTensor's own rule only follows the first input's first candidate)."""
    ndim = len(producers[0].shape)
    dim = node.args[1] if len(node.args) > 1 else node.kwargs.get("dim", 0)
    dim = dim + ndim + 1 if dim < 0 else dim
    rows = [[Replicate()] * (1 + len(producers))]
    rows += [[Shard(i if i < dim else i + 1)] + [Shard(i)] * len(producers) for i in range(ndim)]
    return _product_rule(mesh, rows, 1)


def _uniform_rule(mesh, node, src: OpStrategy) -> OpStrategy:
    """uniform_: the output keeps any sharding of the input
    (autoparallel/shardings/propagation_rules.py:663-680)."""
    rows = [[Replicate(), Replicate()]] + [[Shard(d), Shard(d)] for d in range(len(src.shape))]
    return _product_rule(mesh, rows, 1)


def _split_with_sizes_rule(mesh, node, src: OpStrategy) -> OpStrategy:
    """split_with_sizes: the pieces keep the input's placements; candidates sharded
    on the split dim or Partial are not offered
    (autoparallel/shardings/propagation_rules.py:375-409)."""
    dim = node.args[2] if len(node.args) > 2 else node.kwargs.get("dim", 0)
    dim = dim + len(src.shape) if dim < 0 else dim
    n_out = len(node.meta["val"])
    seen, sts = set(), []
    for st in src.strategies:
        plc = st.output_specs.placements
        if plc in seen or any(p.is_shard(dim) or p.is_partial() for p in plc):
            continue
        seen.add(plc)
        sts.append(OpSpec(tuple(DTensorSpec(mesh, plc) for _ in range(n_out)),
                          input_specs=(DTensorSpec(mesh, plc, tensor_meta=st.output_specs.tensor_meta),)))
    return OpStrategy(sts)


def _view_dtype_rule(mesh, node, src: OpStrategy) -> OpStrategy:
    """view(dtype): the bytes of the last dim are regrouped, so candidates sharded
    on it are not offered; the others carry over
    (autoparallel/shardings/propagation_rules.py:289-315)."""
    last = len(src.shape) - 1
    seen, sts = set(), []
    for st in src.strategies:
        plc = st.output_specs.placements
        if plc in seen or any(p.is_shard(last) for p in plc):
            continue
        seen.add(plc)
        sts.append(OpSpec(DTensorSpec(mesh, plc),
                          input_specs=(DTensorSpec(mesh, plc, tensor_meta=st.output_specs.tensor_meta),)))
    return OpStrategy(sts)


def _alias_rule(mesh, node, src: OpStrategy) -> OpStrategy:
    """alias: every valid placement of the tensor, output as input
    (autoparallel/shardings/propagation_rules.py:358-372)."""
    tm = _tensor_meta(node.meta["val"])
    sts = []
    for st in _create_all_options(mesh, tm.shape, tensor_meta=tm).strategies:
        plc = st.output_specs.placements
        sts.append(OpSpec(DTensorSpec(mesh, plc, tensor_meta=tm), input_specs=(DTensorSpec(mesh, plc, tensor_meta=tm),)))
    return OpStrategy(sts)


def _is_flex_attention(node) -> bool:
    t = node.target
    return isinstance(t, torch._ops.HigherOrderOperator) and t.name() in ("flex_attention", "flex_attention_backward")


def _flex_attention_rule(mesh, node) -> OpStrategy:
    """flex_attention and its backward: attention is independent per (batch,
    head), so every combination of {Replicate, Shard(0), Shard(1)} over the mesh
    dims is a strategy.  A tensor takes a Shard only where it can (more than one
    element on that dim, the query's extent a multiple of it, itself a multiple
    of the mesh dim: grouped key/value heads, broadcast dims); the buffers the
    score and mask functions index, and tensors of rank below two, are Replicate
    (autoparallel/shardings/placement_options.py:493-650)."""
    import inspect

    from torch._higher_order_ops.flex_attention import (
        flex_attention_backward_fake_tensor_mode,
        flex_attention_fake_impl,
    )

    impl = flex_attention_fake_impl if node.target.name() == "flex_attention" else flex_attention_backward_fake_tensor_mode
    params = list(inspect.signature(impl).parameters)
    buffers = set()
    for name in ("score_mod_other_buffers", "mask_mod_other_buffers"):
        if name in params and params.index(name) < len(node.args):
            arg = node.args[params.index(name)]
            if isinstance(arg, (tuple, list)):
                buffers.update(x for x in tree_flatten(arg)[0] if isinstance(x, torch.fx.Node))
    tensors = [(a, a.meta["val"]) for a in tree_flatten(node.args)[0]
               if isinstance(a, torch.fx.Node) and isinstance(a.meta.get("val"), torch.Tensor)]
    q = node.args[0].meta["val"]
    ref = {0: q.shape[0], 1: q.shape[1]}
    rep = (Replicate(),) * mesh.ndim

    def fit(t, plc):
        out = []
        for size, p in zip(mesh.shape, plc):
            if p.is_shard() and p.dim in ref:
                n = t.shape[p.dim]
                p = p if n > 1 and ref[p.dim] % n == 0 and n % size == 0 else Replicate()
            out.append(p)
        return tuple(out)

    outs = node.meta["val"]
    assert isinstance(outs, (tuple, list))
    sts = []
    for plc in itertools.product((Replicate(), Shard(0), Shard(1)), repeat=mesh.ndim):
        ins = [DTensorSpec(mesh, rep if (a in buffers or t.ndim < 2) else fit(t, plc), tensor_meta=_tensor_meta(t))
               for a, t in tensors]
        out_specs = tuple(DTensorSpec(mesh, fit(o, plc), tensor_meta=_tensor_meta(o)) if isinstance(o, torch.Tensor) else None
                          for o in outs)
        sts.append(OpSpec(out_specs, input_specs=tuple(ins)))
    return OpStrategy(sts)


def _without_partial(a):
    """The argument with its Partial candidates left out (itself if it has none, or nothing else)."""
    if isinstance(a, TupleStrategy):
        kids = tuple(_without_partial(c) for c in a.children)
        return a if all(x is y for x, y in zip(kids, a.children)) else TupleStrategy(kids)
    if not isinstance(a, OpStrategy):
        return a
    keep = [st for st in a.strategies if isinstance(st.output_specs, DTensorSpec)
            and not any(p.is_partial() for p in st.output_specs.placements)]
    return a if not keep or len(keep) == len(a.strategies) else OpStrategy(keep)


_NONSTRICT_VIEWS = {aten.view.default, aten._unsafe_view.default}
# strategy functions of the installed torch that pair the arguments' strategies by index
# Elementwise operators that the installed torch may leave without a strategy (it tags some of
# them pointwise, not all): they take DTensor's pointwise rule instead of the stand-in.
_ELEMENTWISE_BY_NAME = {getattr(getattr(aten, name), overload) for name, overload in (
    ("floor_divide", "default"), ("floor_divide", "Scalar"), ("hardswish", "default"), ("hardswish_backward", "default"),
    ("leaky_relu", "default"), ("leaky_relu_backward", "default"), ("hardsigmoid", "default"),
    ("hardsigmoid_backward", "default"), ("elu_backward", "default"), ("softplus_backward", "default"),
    ("mish_backward", "default"), ("div", "Scalar_mode")) if hasattr(getattr(aten, name, None), overload)}


def _is_elementwise(op) -> bool:
    return op in _ELEMENTWISE_BY_NAME or torch.Tag.pointwise in getattr(op, "tags", ())


# reshapes that the installed torch may leave without a strategy: planned like a view to the result's shape
_RESHAPES_BY_RESULT = {getattr(aten.squeeze, "dims")} if hasattr(aten.squeeze, "dims") else set()
# (var, mean) in one operator: the strategies of var, the one spec standing for both results
_SAME_AS = {aten.var_mean.correction: aten.var.correction} if hasattr(aten.var_mean, "correction") else {}
_GATHERS = {aten.index.Tensor, aten.index_select.default}
_CONVOLUTIONS = {aten.convolution.default, aten.convolution_backward.default}
_INDEX_PUTS = {getattr(getattr(aten, name), "default") for name in ("index_put", "index_put_", "_index_put_impl_")
               if hasattr(aten, name)}
_INDEX_PAIRED = {getattr(getattr(aten, name), "default") for name in (
    "native_layer_norm", "native_layer_norm_backward", "_fused_rms_norm", "_fused_rms_norm_backward",
    "nll_loss_forward", "nll_loss_backward", "nll_loss2d_forward", "nll_loss2d_backward") if hasattr(aten, name)}
_FOLLOW = {aten.detach.default} | ({torch.ops.prims.convert_element_type.default}
                                  if hasattr(torch.ops.prims, "convert_element_type") else set())


# content of an OpStrategy's output specs -> a small token.  A strategy object is
# summarised once (its specs do not change after it has been returned) and copies
# made from the query cache inherit the token, so a query key holds one token per
# tensor argument instead of a tuple over all of the argument's strategies.
_fp_intern: Dict[tuple, tuple] = {}
_fp_serial = itertools.count()  # never restarts: a token given out once is not given to other content


def _fingerprint(x):
    """Hashable summary of one argument of a strategy query."""
    if isinstance(x, OpStrategy):
        fp = getattr(x, "_apc_fp", None)
        if fp is None:
            content = ("S",) + tuple(_fingerprint(st.output_specs) for st in x.strategies)
            fp = _fp_intern.get(content)
            if fp is None:
                fp = _fp_intern[content] = ("S#", next(_fp_serial))
            x._apc_fp = fp
        return fp
    if isinstance(x, DTensorSpec):
        return (x.placements, x.tensor_meta)
    if isinstance(x, torch.Tensor):
        return ("T", tuple(x.shape), tuple(x.stride()), x.dtype)
    if isinstance(x, (list, tuple)):
        return tuple(_fingerprint(y) for y in x)
    if isinstance(x, dict):
        return tuple((k, _fingerprint(v)) for k, v in x.items())
    return x


def _copy_strategy(src: OpStrategy) -> OpStrategy:
    """New OpSpec wrappers and a new list of cost rows each (a node's rows are
    replaced when its costs are written back); the specs are shared, and so are
    the rows themselves until then: they hold zeros, and copying 1.7 M of them
    for a Llama-3-8B graph took longer than everything else a cache hit does."""
    out = OpStrategy([OpSpec(st.output_specs, input_specs=st.input_specs,
                             redistribute_cost=list(st.redistribute_cost)) for st in src.strategies])
    fp = getattr(src, "_apc_fp", None)
    if fp is not None:
        out._apc_fp = fp
    return out


# strategies by query, as the reference keeps them
# (autoparallel/shardings/placement_options.py:183-217, 279-302): the layers of a
# model repeat the same queries, and one answer from the propagator costs
# milliseconds.  Values: (strategies, why the all-Replicate stand-in was used or None, id of the answer).
_strategy_cache: Dict[tuple, tuple] = {}
strategy_cache_stats = {"hits": 0, "misses": 0}


def reset_placement_options_cache() -> None:
    _strategy_cache.clear()
    _input_options_cache.clear()
    _spec_words.clear()
    _fp_intern.clear()
    strategy_cache_stats.update(hits=0, misses=0)


def get_placement_options_for_node(mesh, node, producers: List[OpStrategy], arg_vals: List[torch.Tensor],
                                   schema_args) -> OpStrategy:
    """Strategies of one call_function node.  ``producers``: OpStrategy of
    each tensor input node in flattened-args order; ``schema_args``: node.args
    with nodes replaced by their OpStrategy (or value for non-tensors)."""
    if node.meta.get("local_map_kwargs"):
        assert not node.kwargs
        return _local_map_rule(mesh, node, schema_args, node.meta["local_map_kwargs"])
    if _is_flex_attention(node):
        out = _flex_attention_rule(mesh, node)
        fill_redistribute_cost(out, producers)
        return out
    try:
        key = (mesh, node.target, _fingerprint(schema_args),
               _fingerprint({k: v for k, v in node.kwargs.items() if not isinstance(v, torch.fx.Node)}),
               _fingerprint(node.meta.get("val")), _fingerprint(arg_vals))
        hit = _strategy_cache.get(key)
    except TypeError:  # something unhashable (a SymInt, ...) in the query
        key = hit = None
    if hit is not None:
        strategy_cache_stats["hits"] += 1
        if hit[1] is not None:
            fallback_nodes.append(str(node.name))
            fallback_reasons[str(node.name)] = hit[1]
        out = _copy_strategy(hit[0])
        out._apc_query_id = hit[2]  # equal ids: equal strategies (what a packer may memoise on)
        return out
    strategy_cache_stats["misses"] += 1
    n_fallback = len(fallback_nodes)
    out = _placement_options_uncached(mesh, node, producers, arg_vals, schema_args)
    if key is not None:
        why = fallback_reasons.get(str(node.name), "") if len(fallback_nodes) > n_fallback else None
        _fingerprint(out)  # summarised here, once: the cached copy and every later copy inherit it
        qid = next(_query_serial)
        _strategy_cache[key] = (_copy_strategy(out), why, qid)
        out._apc_query_id = qid
    return out


def _zero_cost_rows(src_strategy, dst_spec):
    return [0.0] * len(src_strategy.strategies)


_cost_row_users: List = []  # modules of torch's strategy functions that hold generate_redistribute_costs
_cost_row_users_at = -1     # len(sys.modules) when the list was made
_cost_row_lock = threading.RLock()  # the patch below is a change to module globals: one thread at a time


@contextlib.contextmanager
def _without_torch_cost_rows():
    """torch's strategy functions price every (strategy, producer strategy) pair
    with torch's own redistribute_cost while they build their answer; the rows
    are replaced below (fill_redistribute_cost) and priced by the cost engine,
    so for the duration of a query they are made of zeros instead: half of the
    time the propagator takes on a transformer graph."""
    import sys

    global _cost_row_users, _cost_row_users_at
    # Process-wide while it lasts: other threads that enumerate strategies wait here, and a
    # thread that runs DTensor operators meanwhile would see rows of zeros in the strategies it
    # is handed (their specs are unaffected: no strategy function of the installed torch selects
    # by those rows, which tests/test_placement_options_host.py checks on the operators in use).
    with _cost_row_lock:
        if _cost_row_users_at != len(sys.modules):  # strategy modules are imported lazily
            _cost_row_users = [mod for name, mod in list(sys.modules.items())
                               if name.startswith("torch.distributed.tensor._ops") and mod is not None
                               and "generate_redistribute_costs" in getattr(mod, "__dict__", {})]
            _cost_row_users_at = len(sys.modules)
        saved = [(mod, mod.__dict__["generate_redistribute_costs"]) for mod in _cost_row_users]
        for mod, _ in saved:
            mod.generate_redistribute_costs = _zero_cost_rows
        try:
            yield
        finally:
            for mod, fn in saved:
                mod.generate_redistribute_costs = fn


def _placement_options_uncached(mesh, node, producers, arg_vals, schema_args) -> OpStrategy:
    with _without_torch_cost_rows():
        return _placement_options_uncached_inner(mesh, node, producers, arg_vals, schema_args)


def _placement_options_uncached_inner(mesh, node, producers, arg_vals, schema_args) -> OpStrategy:
    prop = DTensor._op_dispatcher.sharding_propagator
    op = node.target
    if not producers and isinstance(node.meta.get("val"), torch.Tensor):
        return keep_unique_configs(remove_invalid_configs(_inputless_rule(mesh, node), mesh))
    out = None
    try:
        if op is operator.getitem:
            out = _getitem_rule(mesh, node, producers[0])
        elif op in _FOLLOW and len(producers) == 1:
            out = _follow_input(mesh, producers[0], node.meta["val"])
        elif op is aten.einsum.default and len(producers) == 2:
            out = _einsum_rule(mesh, node, *producers)
        elif (op in _NONSTRICT_VIEWS or (op in _RESHAPES_BY_RESULT and op not in prop.op_strategy_funcs)) and len(producers) == 1:
            out = _view_rule(mesh, node, producers[0])
        elif op is aten.alias.default and len(producers) == 1:
            out = _alias_rule(mesh, node, producers[0])
        elif op is aten.stack.default and producers:
            out = _stack_rule(mesh, node, producers)
        elif op is aten.uniform.default and len(producers) == 1:
            out = _uniform_rule(mesh, node, producers[0])
        elif op is aten.split_with_sizes.default and len(producers) == 1:
            out = _split_with_sizes_rule(mesh, node, producers[0])
        elif op is aten.view.dtype and len(producers) == 1:
            out = _view_dtype_rule(mesh, node, producers[0])
        elif op in _CONVOLUTIONS and op not in prop.op_strategy_funcs and len(producers) >= 2:
            out = _conv_rule(mesh, node, producers)
        elif op in _GATHERS and op not in prop.op_strategy_funcs and op in prop.op_to_rules:
            out = _from_propagation_rule(prop.op_to_rules[op], op, mesh, schema_args, producers)
        else:
            fn = prop.op_strategy_funcs.get(op)
            if fn is None and op in _SAME_AS:
                fn = prop.op_strategy_funcs.get(_SAME_AS[op])
            if fn is None and producers and _is_elementwise(op):
                from torch.distributed.tensor._ops._pointwise_ops import pointwise_strategy as fn
            if fn is not None and op in _INDEX_PUTS and len(schema_args) > 1 and any(i is None for i in schema_args[1]):
                # `out[:, idx] = ...`: a None among the indices for a dim that is left alone.  The rule
                # of the installed torch takes tensors only (it asserts on the None), so for this
                # form it is as if none were registered: the node gets the all-Replicate stand-in.
                fn = None
            if fn is not None:
                def wrap(x):
                    # a list argument with tensors in it, e.g. index_put's indices with None for
                    # the dims it leaves alone (autoparallel/shardings/placement_options.py:306-316)
                    if isinstance(x, (list, tuple)) and any(isinstance(y, OpStrategy) for y in x):
                        return TupleStrategy(tuple(x))
                    return x
                args = tuple(wrap(a) for a in schema_args)
                if op is aten.select.int and isinstance(args[0], OpStrategy):
                    # DTensor's rule does not take a negative dim or index
                    # (autoparallel/shardings/propagation_rules.py:318-343)
                    d, i = args[1], args[2]
                    d = d + len(args[0].shape) if isinstance(d, int) and d < 0 else d
                    i = i + args[0].shape[d] if isinstance(i, int) and i < 0 else i
                    args = (args[0], d, i) + args[3:]
                kwargs = {k: v for k, v in node.kwargs.items() if not isinstance(v, torch.fx.Node)}
                if op in _INDEX_PAIRED and len(producers) > 1:
                    res = _one_strategy_at_a_time(fn, op, args, kwargs, producers)
                elif (getattr(fn, "__name__", "") == "linear_reduction_strategy" and len(producers) == 1
                      and len(producers[0].strategies) > 1 and _reduction_rule_carries_state(mesh)):
                    # each candidate of the input on its own, as the rule is meant to treat them
                    res = _one_strategy_at_a_time(fn, op, args, kwargs, producers)
                else:
                    try:
                        res = fn(OpSchema(op, args, kwargs))
                    except (IndexError, ValueError):
                        # pairs candidates by index, or refuses one of them outright: candidate by
                        # candidate, the refused ones dropped (raises again if none is accepted)
                        res = _one_strategy_at_a_time(fn, op, args, kwargs, producers)
                    except RuntimeError:
                        # some functions (the random ones) refuse an argument that may
                        # arrive Partial: ask again without those candidates; what it
                        # costs to bring a Partial producer there is priced per entry
                        narrowed = tuple(_without_partial(a) for a in args)
                        if all(x is y for x, y in zip(narrowed, args)):
                            raise
                        res = fn(OpSchema(op, narrowed, kwargs))
                if isinstance(res, OpStrategy):
                    out = res
                    if len(producers) == 1:
                        # a strategy without input specs follows its output
                        # (autoparallel/shardings/placement_options.py:104-116)
                        for st in out.strategies:
                            if st.input_specs is None and isinstance(st.output_specs, DTensorSpec):
                                st.input_specs = (st.output_specs,)
        why = "no strategy registered" if out is None else ""
    except Exception as exc:
        if not _stand_in_on_error:
            logger.error("strategies of node %s (%s) failed: %s: %s", node.name, op, type(exc).__name__, exc)
            raise
        out, why = None, f"{type(exc).__name__}: {exc}"
    unregistered = out is None and why == "no strategy registered"
    ok = out is not None and len(out.strategies) > 0 and all(
        st.input_specs is not None and len(st.input_specs) == len(producers) for st in out.strategies)
    if not ok:
        if out is not None:
            why = "no strategies" if not out.strategies else (
                f"{len(producers)} tensor inputs, input specs of "
                f"{sorted({-1 if st.input_specs is None else len(st.input_specs) for st in out.strategies})}")
        if not unregistered and not _stand_in_on_error:
            raise ValueError(f"node {node.name} ({op}): {why}")
        logger.warning("node %s: all-Replicate stand-in for `%s` (%s)", node.name, op, why)
        fallback_reasons[str(node.name)] = why
        out = _replicate_fallback(mesh, node, arg_vals)
    _unshare_specs(out, producers)
    propagate_tensor_meta(node, arg_vals, out, mesh)
    fill_redistribute_cost(out, producers)
    out = filter_strategies(out, mesh)
    if not out.strategies:
        why = "no strategy is valid for the shapes"
        if not _stand_in_on_error:
            raise ValueError(f"node {node.name} ({op}): {why}")
        logger.warning("node %s: all-Replicate stand-in for `%s` (%s)", node.name, op, why)
        fallback_reasons[str(node.name)] = why
        out = _replicate_fallback(mesh, node, arg_vals)
        fill_redistribute_cost(out, producers)
    return out

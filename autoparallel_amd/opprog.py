"""Compute programs: closed forms for what the reference obtains by running an
op on sharded FakeTensors under ``FlopCounterMode``
(autoparallel/cost_models/compute_estimation.py:383-388, 469-473).

A program is a flat int64 sequence

    [n_terms, n_outs,
     (coeff, nfac, (arg, dim) * nfac) * n_terms,      # flops = sum of monomials
     (itemsize, rank, (kind, a, b) * rank) * n_outs]   # output tensors

evaluated on the *local* shapes of the node's tensor args (global shape after
``_get_sharded_shape_stride``, compute_estimation.py:300-318).  Flop formulas
follow torch/utils/flop_counter.py:58-86 (mm/addmm/bmm), :267-292 and :478-512
(SDPA forward = 2 bmm, backward = 5 bmm) and the reference's einsum formula
(compute_estimation.py:16-44).
"""
from __future__ import annotations

from typing import List, Sequence, Tuple

from .packed import DIM_ARG, DIM_ARGNUMEL, DIM_BCAST, DIM_CONST

Dim = Tuple[int, int, int]


def const(v: int) -> Dim:
    return (DIM_CONST, int(v), 0)


def argdim(arg: int, dim: int) -> Dim:
    return (DIM_ARG, int(arg), int(dim))


def bcast(pos_from_right: int) -> Dim:
    return (DIM_BCAST, int(pos_from_right), 0)


def argnumel(arg: int) -> Dim:
    """All local sizes of an argument as one factor: an output shaped like the
    argument is ``[argnumel(arg)]``, one program word triple whatever its rank."""
    return (DIM_ARGNUMEL, int(arg), 0)


def program(terms: Sequence[Tuple[int, Sequence[Tuple[int, int]]]], outs: Sequence[Tuple[int, Sequence[Dim]]]) -> List[int]:
    # Terms over the same multiset of factors are one term with the sum of their
    # coefficients (the five matmuls of an attention backward are two distinct
    # products): the same integer, and a shorter walk for the lane that
    # interprets the program, whose length sets the length of the launch.
    merged: dict = {}
    for coeff, facs in terms:
        key = tuple(sorted((int(a), int(d)) for a, d in facs))
        merged[key] = merged.get(key, 0) + int(coeff)
    terms = [(c, list(k)) for k, c in merged.items()]
    p: List[int] = [len(terms), len(outs)]
    for coeff, facs in terms:
        p += [int(coeff), len(facs)]
        for a, d in facs:
            p += [int(a), int(d)]
    for itemsize, dims in outs:
        p += [int(itemsize), len(dims)]
        for k, a, b in dims:
            p += [int(k), int(a), int(b)]
    return p


def pointwise(out_rank: int, out_itemsize: int) -> List[int]:
    """Elementwise op with broadcasting: zero flops, one output whose shape is
    the broadcast of the local input shapes."""
    return program([], [(out_itemsize, [bcast(out_rank - 1 - i) for i in range(out_rank)])])


def same_as_arg(arg: int, rank: int, out_itemsize: int, n_out: int = 1) -> List[int]:
    """Zero-flop op whose outputs have the (local) shape of one argument
    (softmax, dtype conversion, clone, ...)."""
    return program([], [(out_itemsize, [argnumel(arg)])] * n_out)


def mm(out_itemsize: int, a: int = 0, b: int = 1) -> List[int]:
    return program(
        [(2, [(a, 0), (a, 1), (b, 1)])],
        [(out_itemsize, [argdim(a, 0), argdim(b, 1)])],
    )


def addmm(out_itemsize: int) -> List[int]:
    # addmm(bias, a, b): the bias is read but adds no flops (flop_counter.py:66-69)
    return mm(out_itemsize, 1, 2)


def bmm(out_itemsize: int) -> List[int]:
    return program(
        [(2, [(0, 0), (0, 1), (0, 2), (1, 2)])],
        [(out_itemsize, [argdim(0, 0), argdim(0, 1), argdim(1, 2)])],
    )


def einsum_fwd(a_rank: int, out_itemsize: int) -> List[int]:
    """"{batch}k,kn->{batch}n" (compute_estimation.py:21-30)."""
    facs = [(0, i) for i in range(a_rank - 1)] + [(1, 1), (0, a_rank - 1)]
    out = [argdim(0, i) for i in range(a_rank - 1)] + [argdim(1, 1)]
    return program([(2, facs)], [(out_itemsize, out)])


def einsum_bwd(a_rank: int, out_itemsize: int) -> List[int]:
    """"{batch}n,{batch}k->kn" (compute_estimation.py:31-42)."""
    facs = [(0, i) for i in range(a_rank - 1)] + [(0, a_rank - 1), (1, a_rank - 1)]
    out = [argdim(1, a_rank - 1), argdim(0, a_rank - 1)]
    return program([(2, facs)], [(out_itemsize, out)])


def reduction(rank: int, dims: Sequence[int], keepdim: bool, out_itemsize: int) -> List[int]:
    dims = {d % rank for d in dims}
    out: List[Dim] = []
    for i in range(rank):
        if i in dims:
            if keepdim:
                out.append(const(1))
        else:
            out.append(argdim(0, i))
    return program([], [(out_itemsize, out)])


def embedding(idx_rank: int, out_itemsize: int) -> List[int]:
    out = [argdim(1, i) for i in range(idx_rank)] + [argdim(0, 1)]
    return program([], [(out_itemsize, out)])


def embedding_dense_backward(num_weights: int, out_itemsize: int, grad_rank: int) -> List[int]:
    # (grad_output, indices, num_weights, ...) -> [num_weights, D]
    return program([], [(out_itemsize, [const(num_weights), argdim(0, grad_rank - 1)])])


def cat(n_inputs: int, out_itemsize: int) -> List[int]:
    """aten.cat of tensors that agree outside the concatenated dim: the output
    has as many elements as the inputs together."""
    return program([], [(out_itemsize, [argnumel(i)]) for i in range(n_inputs)])


def constant_shape(shape: Sequence[int], out_itemsize: int) -> List[int]:
    """Zero-flop op whose output shape is given among its arguments, not taken from
    the local tensor sizes (aten.slice_backward's ``input_sizes``: the operator is
    run with the global list whatever the sharding of its tensor)."""
    return program([], [(out_itemsize, [const(int(s)) for s in shape])])


def nll_loss_forward(unreduced: bool, out_itemsize: int, weight_itemsize: int) -> List[int]:
    """(loss, total_weight) of aten.nll_loss_forward on a [N, C] input: the loss
    per row without a reduction, else a scalar; total_weight is a scalar."""
    return program([], [(out_itemsize, [argdim(0, 0)] if unreduced else []), (weight_itemsize, [])])


# ROCm builds of torch return the philox seed and offset of the flash kernels
# as two scalar int64 tensors (16 bytes in total).
_PHILOX_BYTES_ROCM = 16


def sdpa_flash_fwd(itemsize: int) -> List[int]:
    """aten._scaled_dot_product_flash_attention(q, k, v): outputs attention
    [b,h,sq,dv], logsumexp [b,h,sq] fp32, philox seed/offset, and an empty
    debug mask; flops = q@k^T + p@v (flop_counter.py:267-292)."""
    q, k, v = 0, 1, 2
    terms = [
        (2, [(q, 0), (q, 1), (q, 2), (q, 3), (k, 2)]),
        (2, [(q, 0), (q, 1), (q, 2), (k, 2), (v, 3)]),
    ]
    outs = [
        (itemsize, [argdim(q, 0), argdim(q, 1), argdim(q, 2), argdim(v, 3)]),
        (4, [argdim(q, 0), argdim(q, 1), argdim(q, 2)]),
        (1, [const(_PHILOX_BYTES_ROCM)]),
    ]
    return program(terms, outs)


def sdpa_flash_bwd(itemsize: int) -> List[int]:
    """aten._scaled_dot_product_flash_attention_backward(grad, q, k, v, out,
    lse, ...): five matmuls (flop_counter.py:478-512), outputs dq, dk, dv."""
    g, q, k, v = 0, 1, 2, 3
    terms = [
        # recompute scores: q @ k^T
        (2, [(q, 0), (q, 1), (q, 2), (q, 3), (k, 2)]),
        # grad_out @ v^T -> grad_scores
        (2, [(q, 0), (q, 1), (q, 2), (v, 3), (k, 2)]),
        # scores^T @ grad_out -> dv
        (2, [(q, 0), (q, 1), (k, 2), (q, 2), (v, 3)]),
        # grad_scores @ k -> dq
        (2, [(q, 0), (q, 1), (q, 2), (k, 2), (q, 3)]),
        # grad_scores^T @ q -> dk
        (2, [(q, 0), (q, 1), (k, 2), (q, 2), (q, 3)]),
    ]
    outs = [(itemsize, [argnumel(q)]), (itemsize, [argnumel(k)]), (itemsize, [argnumel(v)])]
    return program(terms, outs)

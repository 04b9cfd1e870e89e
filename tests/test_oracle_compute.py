"""Compute programs + the oracle's roofline against the reference's
estimate_strategy_runtime_cost on hand-built fx nodes (golden vectors), and the
flop formulas against torch's FlopCounterMode on meta tensors."""
import json

import numpy as np
import pytest
import torch

from autoparallel_amd import opprog
from oracle import cost_oracle as O

_DT = {"torch.float64": (0, 8), "torch.float32": (1, 4), "torch.float16": (2, 2),
       "torch.bfloat16": (3, 2), "torch.int8": (4, 1), "torch.int64": (5, 8)}


def _program_for(name, shapes, dtypes):
    isz = _DT[dtypes[0]][1]
    r0 = len(shapes[0])
    return {
        "mm": lambda: opprog.mm(isz),
        "mm_f32": lambda: opprog.mm(isz),
        "bmm": lambda: opprog.bmm(isz),
        "addmm": lambda: opprog.addmm(isz),
        "add": lambda: opprog.pointwise(r0, isz),
        "mul_bcast": lambda: opprog.pointwise(r0, isz),
        "small_add": lambda: opprog.pointwise(r0, isz),
        "silu": lambda: opprog.pointwise(r0, isz),
        "sum_dim": lambda: opprog.reduction(r0, [2], True, isz),
        "mean_dim": lambda: opprog.reduction(r0, [-1], True, isz),
        "einsum_fwd": lambda: opprog.einsum_fwd(r0, isz),
        "einsum_bwd": lambda: opprog.einsum_bwd(r0, isz),
        "softmax": lambda: opprog.same_as_arg(0, r0, isz),
        "embedding": lambda: opprog.embedding(len(shapes[1]), isz),
        "sdpa_flash": lambda: opprog.sdpa_flash_fwd(isz),
    }[name]()


def test_runtime_vectors(golden):
    d = json.loads(bytes(golden["rt_json"]).decode())
    dev = O.DeviceLimit()
    mesh = d["mesh"]
    n = 0
    for name, shapes, dtypes, plcs, flops, nbytes, chex in zip(
        d["names"], d["shapes"], d["dtypes"], d["placements"], d["flops"], d["bytes"], d["cost_hex"]
    ):
        want = float.fromhex(chex)
        if name == "view":
            assert want == 0.0  # is_view -> zero cost (compute_estimation.py:377-378)
            continue
        prog = _program_for(name, shapes, dtypes)
        local = []
        for shape, plc in zip(shapes, plcs):
            stride = list(torch.empty(shape, device="meta").stride())
            ls, _ = O.sharded_shape_stride(shape, stride, plc, mesh)
            local.append(ls)
        f, b = O.run_program(prog, local, [_DT[t][1] for t in dtypes])
        assert (f, b) == (flops, nbytes), (name, plcs, f, b, flops, nbytes)
        got = O.roofline_cost(f, b, _DT[dtypes[0]][0], dev)
        assert float(got) == want, (name, got, want)
        n += 1
    assert n >= 40


@pytest.mark.parametrize("b,h,sq,sk,dq,dv", [(2, 4, 16, 16, 8, 8), (1, 2, 32, 8, 16, 4)])
def test_sdpa_flops_vs_flop_counter(b, h, sq, sk, dq, dv):
    from torch.utils.flop_counter import FlopCounterMode

    q = torch.empty(b, h, sq, dq, device="meta", dtype=torch.bfloat16)
    k = torch.empty(b, h, sk, dq, device="meta", dtype=torch.bfloat16)
    v = torch.empty(b, h, sk, dv, device="meta", dtype=torch.bfloat16)
    if dq != dv:
        pytest.skip("flash meta kernel needs dq == dv")
    with FlopCounterMode(display=False) as fc:
        o = torch.ops.aten._scaled_dot_product_flash_attention.default(q, k, v, 0.0, False)
    f, _ = O.run_program(opprog.sdpa_flash_fwd(2), [list(q.shape), list(k.shape), list(v.shape)], [2, 2, 2])
    assert f == fc.get_total_flops()
    g = torch.empty_like(o[0])
    with FlopCounterMode(display=False) as fc:
        torch.ops.aten._scaled_dot_product_flash_attention_backward.default(
            g, q, k, v, o[0], o[1], None, None, sq, sk, 0.0, False, o[6], o[7])
    f, nb = O.run_program(
        opprog.sdpa_flash_bwd(2),
        [list(g.shape), list(q.shape), list(k.shape), list(v.shape), list(o[0].shape), list(o[1].shape)],
        [2, 2, 2, 2, 2, 4])
    assert f == fc.get_total_flops()


def test_sdpa_bwd_terms_distinct_dims():
    # torch's closed form with all dims different (flop_counter.py:478-512)
    b, h, sq, sk, dq, dv = 3, 5, 7, 11, 13, 17
    want = 2 * b * h * (sq * dq * sk + sq * dv * sk + sk * sq * dv + sq * sk * dq + dq * sq * sk)
    f, nb = O.run_program(
        opprog.sdpa_flash_bwd(2),
        [[b, h, sq, dv], [b, h, sq, dq], [b, h, sk, dq], [b, h, sk, dv]],
        [2, 2, 2, 2])
    assert f == want
    # bytes: the four inputs read, dq / dk / dv (shaped like q / k / v) written
    nq, nk, nv = b * h * sq * dq, b * h * sk * dq, b * h * sk * dv
    assert nb == 2 * (b * h * sq * dv + nq + nk + nv) + 2 * (nq + nk + nv)


def test_output_shaped_like_an_argument():
    """``argnumel`` stands for all of an argument's local sizes: the same bytes as
    the output written dim by dim."""
    shapes = [[3, 5, 7], [11, 13]]
    whole = O.run_program(opprog.same_as_arg(1, 2, 4, n_out=2), shapes, [2, 4])
    by_dim = O.run_program(opprog.program([], [(4, [opprog.argdim(1, 0), opprog.argdim(1, 1)])] * 2), shapes, [2, 4])
    assert whole == by_dim == (0, 3 * 5 * 7 * 2 + 11 * 13 * 4 + 2 * 11 * 13 * 4)
    # equal terms are merged when a program is built: the same flops
    merged = opprog.program([(2, [(0, 0), (1, 1)]), (3, [(1, 1), (0, 0)])], [])
    assert merged[:2] == [1, 0] and O.run_program(merged, shapes, [2, 4])[0] == 5 * 3 * 13


def test_mm_family_vs_flop_counter():
    from torch.utils.flop_counter import FlopCounterMode

    a = torch.empty(6, 10, device="meta")
    b = torch.empty(10, 14, device="meta")
    with FlopCounterMode(display=False) as fc:
        torch.mm(a, b)
    assert O.run_program(opprog.mm(4), [[6, 10], [10, 14]], [4, 4]) == (fc.get_total_flops(), (60 + 140 + 84) * 4)
    a3 = torch.empty(3, 6, 10, device="meta")
    b3 = torch.empty(3, 10, 14, device="meta")
    with FlopCounterMode(display=False) as fc:
        torch.bmm(a3, b3)
    assert O.run_program(opprog.bmm(4), [[3, 6, 10], [3, 10, 14]], [4, 4])[0] == fc.get_total_flops()
    bias = torch.empty(14, device="meta")
    with FlopCounterMode(display=False) as fc:
        torch.addmm(bias, a, b)
    assert O.run_program(opprog.addmm(4), [[14], [6, 10], [10, 14]], [4, 4, 4])[0] == fc.get_total_flops()

"""Linear layers rewritten as einsums before planning: the scenarios of the
reference's tests/test_graph_utils.py:49-300 (which shapes match, which must
not, and that the rewritten graph computes the same numbers)."""
import pytest
import torch
from torch.fx.experimental.proxy_tensor import make_fx

from autoparallel_amd.graph_utils import _replace_view_mm_view_with_einsum, replace_view_mm_view_with_einsum

aten = torch.ops.aten


def _count(gm, target):
    return len(gm.graph.find_nodes(op="call_function", target=target))


def _forward(batch, K, N, out_batch=None, unsafe=False):
    flat = 1
    for d in batch:
        flat *= d
    out_batch = batch if out_batch is None else out_batch
    unflatten = aten._unsafe_view.default if unsafe else aten.view.default

    def f(x, w):
        return unflatten(aten.mm.default(aten.view.default(x, [flat, K]), w), [*out_batch, N])

    return f, (torch.randn(*batch, K), torch.randn(K, N))


def _weight_grad(batch, K, N, perm_in=(1, 0), perm_out=(1, 0), with_t=False):
    flat = 1
    for d in batch:
        flat *= d

    def f(g, x):
        if with_t:  # the transposes as torch 2.10 traces them
            return aten.t.default(aten.mm.default(aten.t.default(aten.view.default(g, [flat, N])),
                                                  aten.view.default(x, [flat, K])))
        gt = aten.permute.default(aten.view.default(g, [flat, N]), list(perm_in))
        return aten.permute.default(aten.mm.default(gt, aten.view.default(x, [flat, K])), list(perm_out))

    return f, (torch.randn(*batch, N), torch.randn(*batch, K))


@pytest.mark.parametrize("case, equation", [
    (_forward((2, 8), 16, 32), "abk,kn->abn"),
    (_forward((2, 4, 3), 16, 32), "abck,kn->abcn"),
    (_forward((2, 8), 16, 32, unsafe=True), "abk,kn->abn"),
    (_weight_grad((2, 8), 16, 32), "abn,abk->kn"),
    (_weight_grad((2, 4, 3), 16, 32), "abcn,abck->kn"),
    (_weight_grad((2, 8), 16, 32, with_t=True), "abn,abk->kn"),
])
def test_matches_and_computes_the_same(case, equation):
    f, args = case
    want = f(*args)
    gm = make_fx(f, tracing_mode="fake")(*args)
    assert _replace_view_mm_view_with_einsum(gm) == 1
    assert _count(gm, aten.einsum.default) == 1 and _count(gm, aten.mm.default) == 0
    assert _count(gm, aten.view.default) == 0 and _count(gm, aten._unsafe_view.default) == 0
    assert _count(gm, aten.permute.default) == 0 and _count(gm, aten.t.default) == 0
    (ein,) = gm.graph.find_nodes(op="call_function", target=aten.einsum.default)
    assert ein.args[0] == equation and tuple(ein.meta["val"].shape) == tuple(want.shape)
    torch.testing.assert_close(gm(*args), want)


def _plain_mm():
    return (lambda a, b: aten.mm.default(a, b)), (torch.randn(4, 8), torch.randn(8, 16))


def _two_users():
    def f(x, w):
        y = aten.mm.default(aten.view.default(x, [16, 16]), w)
        return aten.view.default(y, [2, 8, 32]), aten.relu.default(y)

    return f, (torch.randn(2, 8, 16), torch.randn(16, 32))


@pytest.mark.parametrize("case", [
    _plain_mm(),
    _forward((6,), 16, 32, out_batch=(2, 3)),      # the input has no leading dims to flatten
    _forward((2, 3), 4, 8, out_batch=(3, 2)),      # unflattened into other leading dims
    _forward((16,), 16, 32, out_batch=(16,)),      # 2-D in, 2-D out
    _weight_grad((2, 8), 16, 16, perm_in=(0, 1)),  # not a transpose
    _weight_grad((2, 8), 16, 32, perm_out=(0, 1)),
    _two_users(),
], ids=["plain_mm", "flat_input", "reordered_batch", "two_dims", "identity_permute_in", "identity_permute_out",
        "mm_with_two_users"])
def test_leaves_everything_else_alone(case):
    f, args = case
    want = f(*args)
    gm = make_fx(f, tracing_mode="fake")(*args)
    n_mm = _count(gm, aten.mm.default)
    assert replace_view_mm_view_with_einsum(gm) == 0
    assert _count(gm, aten.einsum.default) == 0 and _count(gm, aten.mm.default) == n_mm == 1
    got = gm(*args)
    for a, b in zip(got if isinstance(got, tuple) else (got,), want if isinstance(want, tuple) else (want,)):
        torch.testing.assert_close(a, b)


def test_autograd_tags_of_the_matmul_are_kept():
    """seq_nr pairs a forward einsum with its backward; recompute / ac_graph_id
    are the activation-checkpointing policy: they come from the mm, the rest of
    the meta from the node that is replaced (autoparallel/graph_passes/graph_utils.py:426-434)."""
    f, args = _forward((2, 8), 16, 32)
    gm = make_fx(f, tracing_mode="fake")(*args)
    (mm,) = gm.graph.find_nodes(op="call_function", target=aten.mm.default)
    mm.meta.update(seq_nr=41, recompute="MUST_SAVE", ac_graph_id=3)
    (user,) = mm.users
    user.meta.update(seq_nr=7, custom={"tag": "out"})
    replace_view_mm_view_with_einsum(gm)
    (ein,) = gm.graph.find_nodes(op="call_function", target=aten.einsum.default)
    assert ein.meta["seq_nr"] == 41 and ein.meta["recompute"] == "MUST_SAVE" and ein.meta["ac_graph_id"] == 3
    assert ein.meta["custom"] == {"tag": "out"}

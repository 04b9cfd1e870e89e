"""Validity filter and de-duplication of operator strategies in packed form
(apc_filter_strategies) against the host's remove_invalid_configs /
keep_unique_configs: the known answers of the reference's own tests
(tests/test_placement_options_utils.py:28-148 there), random sets, and every
node of a traced model planned both ways."""
import contextlib

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@contextlib.contextmanager
def _fake_group(world):
    import torch.distributed as dist
    from torch.testing._internal.distributed.fake_pg import FakeStore

    if dist.is_initialized():
        dist.destroy_process_group()
    dist.init_process_group("fake", store=FakeStore(), rank=0, world_size=world)
    try:
        yield
    finally:
        dist.destroy_process_group()


def _tm(shape, dtype=torch.float32):
    from torch.distributed.tensor._dtensor_spec import TensorMeta

    t = torch.empty(shape, dtype=dtype, device="meta")
    return TensorMeta(t.shape, t.stride(), t.dtype)


def _device_kept(strat, mesh):
    from autoparallel_amd.shardings import placement_options as PO

    table = PO._SpecWords(tuple(mesh.shape))
    rows = PO.strategy_rows(strat.strategies, table)
    assert rows is not None
    valid, keep = PO.filter_masks_on_device(tuple(mesh.shape), [rows], table)
    return valid.tolist(), keep.tolist()


def test_known_answers_of_the_reference_tests():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from torch.distributed.device_mesh import init_device_mesh
    from torch.distributed.tensor._dtensor_spec import DTensorSpec
    from torch.distributed.tensor._op_schema import OpSpec, OpStrategy
    from torch.distributed.tensor.placement_types import Replicate, Shard

    from autoparallel_amd.shardings.placement_options import keep_unique_configs, remove_invalid_configs

    def one(mesh, shape, plc):
        spec = DTensorSpec(mesh, plc, tensor_meta=_tm(shape))
        return OpSpec(spec, input_specs=[spec], redistribute_cost=[[0.0]])

    with _fake_group(256):
        m1 = init_device_mesh("cpu", (256,))
        m2 = init_device_mesh("cpu", (32, 8))
        cases = [  # (mesh, strategies, rows that stay valid)
            (m1, [one(m1, (256, 64), (Shard(0),))], [1]),                    # divisible
            (m1, [one(m1, (100, 64), (Shard(0),))], [0]),                    # a shard would be empty
            (m1, [one(m1, (7, 3), (Replicate(),))], [1]),                    # Replicate always stays
            (m2, [one(m2, (256, 10), (Shard(0), Shard(1)))], [1]),           # 10 over 8: uneven, not empty
            (m1, [one(m1, (256, 64), (Shard(0),)), one(m1, (100, 64), (Shard(0),))], [1, 0]),
            (m2, [one(m2, (257, 64), (Shard(0), Replicate()))], [1]),        # just above the mesh size
            (m2, [one(m2, (40, 64), (Shard(0), Shard(0)))], [0]),            # 40 -> 2 after the first dim, then below 8
        ]
        for mesh, sts, want in cases:
            strat = OpStrategy(sts)
            valid, keep = _device_kept(strat, mesh)
            assert valid == want and keep == want, (mesh.shape, valid, want)
            assert len(remove_invalid_configs(strat, mesh).strategies) == sum(want)
        # an output spec of None is skipped
        spec = DTensorSpec(m1, (Replicate(),), tensor_meta=_tm((256,)))
        strat = OpStrategy([OpSpec(None, input_specs=[spec], redistribute_cost=[[0.0]])])
        rows_valid, rows_keep = _device_kept(strat, m1)
        assert rows_valid == [1] and rows_keep == [1]
        # keep_unique_configs: the same strategy twice is kept once; different ones both
        a = one(m1, (4, 8), (Replicate(),))
        assert _device_kept(OpStrategy([a, a]), m1)[1] == [1, 0]
        assert len(keep_unique_configs(OpStrategy([a, a])).strategies) == 1
        b, c = one(m1, (256, 64), (Replicate(),)), one(m1, (256, 64), (Shard(0),))
        assert _device_kept(OpStrategy([b, c]), m1)[1] == [1, 1]


@pytest.mark.parametrize("mesh_shape", [(8,), (4, 8), (2, 4, 4), (2, 2, 2, 2)])
def test_random_sets_equal_the_two_loops(mesh_shape):
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from torch.distributed.device_mesh import init_device_mesh
    from torch.distributed.tensor._dtensor_spec import DTensorSpec
    from torch.distributed.tensor._op_schema import OpSpec, OpStrategy
    from torch.distributed.tensor.placement_types import Partial, Replicate, Shard

    from autoparallel_amd.shardings import placement_options as PO

    rng = np.random.default_rng(sum(mesh_shape))
    with _fake_group(int(np.prod(mesh_shape))):
        mesh = init_device_mesh("cpu", mesh_shape)
        table = PO._SpecWords(mesh_shape)
        sets, strats = [], []
        for _ in range(24):
            n_in, n_out = int(rng.integers(1, 4)), int(rng.integers(1, 3))
            metas = [_tm(tuple(int(x) for x in rng.choice([1, 3, 4, 7, 8, 16, 33, 64], int(rng.integers(1, 4)))))
                     for _ in range(n_in + n_out)]

            def spec(k):
                if rng.random() < 0.08:
                    return None
                rank = len(metas[k].shape)
                plc = tuple(Replicate() if (r := rng.random()) < 0.4 else Partial() if r < 0.5
                            else Shard(int(rng.integers(0, rank))) for _ in mesh_shape)
                return DTensorSpec(mesh, plc, tensor_meta=metas[k])

            sts = []
            for _ in range(int(rng.integers(1, 160))):
                if sts and rng.random() < 0.3:  # a repeat of an earlier strategy, as new objects
                    src = sts[int(rng.integers(0, len(sts)))]
                    ins = [None if s is None else DTensorSpec(mesh, s.placements, tensor_meta=s.tensor_meta)
                           for s in src.input_specs]
                    sts.append(OpSpec(src.output_specs, input_specs=ins))
                    continue
                outs = tuple(spec(n_in + k) for k in range(n_out))
                sts.append(OpSpec(outs[0] if n_out == 1 and outs[0] is not None else outs,
                                  input_specs=[spec(k) for k in range(n_in)]))
            strat = OpStrategy(sts)
            rows = PO.strategy_rows(sts, table)
            assert rows is not None and rows.shape[0] == len(sts)
            sets.append(rows)
            strats.append(strat)
        valid, keep = PO.filter_masks_on_device(mesh_shape, sets, table)  # all sets in one launch
        at = 0
        for strat in strats:
            n = len(strat.strategies)
            want_valid = PO.remove_invalid_configs(strat, mesh).strategies
            want_keep = PO.keep_unique_configs(PO.remove_invalid_configs(strat, mesh)).strategies
            got_valid = [st for st, k in zip(strat.strategies, valid[at:at + n]) if k]
            got_keep = [st for st, k in zip(strat.strategies, keep[at:at + n]) if k]
            assert len(got_valid) == len(want_valid) and all(a is b for a, b in zip(got_valid, want_valid))
            assert len(got_keep) == len(want_keep) and all(a is b for a, b in zip(got_keep, want_keep))
            at += n
        assert 0 < int(keep.sum()) < int(valid.sum()) < valid.shape[0]


def test_a_traced_model_planned_with_either_filter():
    """Every node of a traced decoder layer gets the same strategies, in the same
    order, whether its candidates are filtered on the device or by the two loops."""
    transformers = pytest.importorskip("transformers")
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from torch._functorch.aot_autograd import aot_export_joint_with_descriptors
    from torch._subclasses.fake_tensor import FakeTensorMode
    from torch.distributed.device_mesh import init_device_mesh

    from autoparallel_amd.optimize_sharding import enumerate_strategies
    from autoparallel_amd.shardings import placement_options as PO

    cfg = transformers.LlamaConfig(
        vocab_size=4096, hidden_size=512, intermediate_size=1024, num_hidden_layers=1, num_attention_heads=8,
        num_key_value_heads=8, max_position_embeddings=512, attention_dropout=0.0, use_cache=False,
        attn_implementation="sdpa")

    class Loss(torch.nn.Module):
        def __init__(self, lm):
            super().__init__()
            self.lm = lm

        def forward(self, ids):
            m = self.lm.model
            x = m.embed_tokens(ids)
            pos = torch.arange(ids.shape[1], device=ids.device)[None]
            pe = m.rotary_emb(x, pos)
            for layer in m.layers:
                out = layer(x, attention_mask=None, position_ids=pos, position_embeddings=pe)
                x = out[0] if isinstance(out, tuple) else out
            logits = self.lm.lm_head(m.norm(x))
            return torch.nn.functional.cross_entropy(logits[:, :-1].reshape(-1, logits.shape[-1]).float(),
                                                     ids[:, 1:].reshape(-1))

    with FakeTensorMode():
        with torch.device("cuda"):
            m = Loss(transformers.LlamaForCausalLM(cfg))
        ids = torch.randint(0, cfg.vocab_size, (16, 256), device="cuda")
        with contextlib.ExitStack() as stack:
            gm = aot_export_joint_with_descriptors(stack, m, (ids,)).graph_module
    with _fake_group(64):
        mesh = init_device_mesh("cpu", (8, 8))
        seen = {}
        saved = PO.DEVICE_FILTER_FROM
        try:
            for label, threshold in (("device", 1), ("host", 1 << 30)):
                PO.DEVICE_FILTER_FROM = threshold
                PO.reset_placement_options_cache()
                strats = enumerate_strategies(gm.graph, mesh)
                seen[label] = {n.name: [(str(s.input_specs), str(s.output_specs)) for s in st.strategies]
                               for n, st in strats.items() if n.op == "call_function"}
        finally:
            PO.DEVICE_FILTER_FROM = saved
        assert seen["device"] == seen["host"] and len(seen["host"]) > 100

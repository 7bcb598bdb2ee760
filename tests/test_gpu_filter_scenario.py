"""The reference's own step-filter scenario (tests/hashtable/ht_filter_hook_test.py:163-751): the
same features, tables, ids per step and expected table contents, driven through EmbeddingEngine +
SparseAdamWTF + HashTableFilterHook + Saver / Loader of this package. Three tables: a coalesced one
(ht2 + ht1, keys evicted one step after their last lookup), ht3 (three steps) and ht4 (fifty)."""
import numpy as np
import pytest
import torch

from recis_amd.hooks import HashTableFilterHook
from recis_amd.nn import EmbeddingEngine, EmbeddingOption
from recis_amd.nn.functional import fused_ops
from recis_amd.nn.hashtable_hook import FilterHook
from recis_amd.nn.initializers import ConstantInitializer
from recis_amd.nn.modules.hashtable import HashtableRegister, split_sparse_dense_state_dict
from recis_amd.nn.modules.hashtable_hook_impl import HashtableHookFactory
from recis_amd.optim import SparseAdamWTF
from recis_amd.ragged.tensor import RaggedTensor
from recis_amd.serialize import Loader, Saver

pytestmark = pytest.mark.gpu


def _rt(values, offsets):
    return RaggedTensor(torch.tensor(values, dtype=torch.int64, device="cuda"),
                        torch.tensor(offsets, dtype=torch.int64, device="cuda"))


def _same_set(a, b):
    a, b = torch.as_tensor(a).cuda().long(), torch.as_tensor(b).cuda().long()
    return a.shape == b.shape and torch.equal(torch.sort(a)[0], torch.sort(b)[0])


def _rows_split(tensor, live_rows, value):
    """Rows outside live_rows hold `value` everywhere; live rows hold it nowhere."""
    mask = torch.zeros(tensor.size(0), dtype=torch.bool, device=tensor.device)
    mask[live_rows.to(tensor.device)] = True
    return bool(torch.all(tensor[~mask] == value)) and not bool(torch.any(tensor[mask] == value))


def _option(name, dim, combiner, init, filter_step, trainable=True):
    return EmbeddingOption(embedding_dim=dim, shared_name=name, combiner=combiner,
                           initializer=ConstantInitializer(init_val=init), device=torch.device("cuda"),
                           filter_hook=FilterHook("GlobalStepFilter", {"filter_step": filter_step}),
                           trainable=trainable)


def test_reference_filter_hook_scenario(tmp_path):
    HashtableRegister().clear()
    HashtableHookFactory().clear_filters()
    same = {"fea_1": _rt([12, 13, 14, 15, 16], [0, 1, 2, 3, 4, 5]),
            "fea_2": _rt([27, 28, 29, 30, 31, 32, 33], [0, 1, 2, 3, 4, 7]),
            "fea_3": _rt([12, 99], [0, 1, 2, 2, 2, 2]),
            "fea_4": _rt([100, 101, 102], [0, 1, 2, 3])}
    steps = {0: same, 1: same, 2: same,
             3: {"fea_1": _rt([12, 13, 16], [0, 1, 2, 3]), "fea_2": _rt([777777, 28], [0, 1, 2, 2])},
             4: {"fea_3": _rt([12, 13, 16, 999], [0, 1, 2, 3, 4])},
             5: {"fea_1": _rt([999], [0, 1]), "fea_2": _rt([12], [0, 1])},
             6: {"fea_2": _rt([1111], [0, 1])}, 7: {"fea_2": _rt([1111], [0, 1])}}
    # the order of the reference's option dict: ht4, ht3, then ht2 before ht1 in the coalesced table
    engine = EmbeddingEngine({
        "fea_5": _option("ht4", 2, "sum", 8.0, 50),
        "fea_4": _option("ht3", 8, "sum", 3.0, 3),
        "fea_2": _option("ht2", 8, "mean", 3.0, 1),
        "fea_1": _option("ht1", 8, "sum", 3.0, 1),
        "fea_3": _option("ht1", 8, "mean", 3.0, 1, trainable=False),
    })
    engine.train()
    sparse_state, dense_state = split_sparse_dense_state_dict(engine.state_dict())
    opt = SparseAdamWTF(sparse_state)
    hook = HashTableFilterHook(1)
    tables = engine.hashtables()
    ht_a = next(t for n, t in tables.items() if n.startswith("CoalescedHashtable_"))
    ht_b, ht_c = tables["ht3"], tables["ht4"]
    tag = {"fea_1": ht_a.children_info().child_index("ht1"), "fea_3": ht_a.children_info().child_index("ht1"),
           "fea_2": ht_a.children_info().child_index("ht2")}
    assert tag["fea_2"] == 0 and tag["fea_1"] == 1

    def slot(ht, name):
        return ht.slot_group().slot_by_name(name)

    def encoded(pairs):
        return fused_ops.fused_ids_encode_gpu([v for v, _ in pairs], [tag[f] for _, f in pairs])

    def train(step, loss_of):
        out = engine(steps[step])
        loss_of(out).backward()
        opt.step()
        opt.zero_grad()
        return out

    for step in range(3):
        batch = steps[step]
        train(step, lambda out: out["fea_1"].sum() + out["fea_2"].sum())
        hook.after_step(-1, step)
        ids, rows = ht_a.ids_map()
        assert _same_set(ht_a.ids(), encoded([(batch["fea_1"].values(), "fea_1"), (batch["fea_2"].values(), "fea_2"),
                                              (torch.tensor([99], device="cuda"), "fea_3")]))
        assert _same_set(ht_b.ids(), [100, 101, 102])
        assert bool((slot(ht_a, "step_filter").value()[:13].view(-1) == step).all())
        assert bool((slot(ht_b, "step_filter").value()[:3].view(-1) == step).all())
        assert int(rows.max()) == 12

    batch = steps[3]
    train(3, lambda out: out["fea_1"].sum() + out["fea_2"].sum())
    hook.after_step(-1, 3)
    ids, rows = ht_a.ids_map()
    assert int(rows.max()) <= 13
    assert _same_set(ht_a.ids(), encoded([(batch["fea_1"].values(), "fea_1"), (batch["fea_2"].values(), "fea_2")]))
    assert _same_set(ht_b.ids(), [100, 101, 102])
    assert _same_set(slot(ht_a, "step_filter").value()[:14].view(-1), [3] * 5 + [2] * 9)
    assert bool((slot(ht_b, "step_filter").value()[:3].view(-1) == 2).all())

    batch = steps[4]
    engine(batch)                        # fea_3 is not trainable: lookup only
    hook.after_step(-1, 4)
    ids, rows = ht_a.ids_map()
    assert int(rows.max()) <= 12         # 999 took a freed row, 777777's row 13 is free again
    assert _same_set(ht_a.ids(), encoded([(batch["fea_3"].values(), "fea_3")]))
    assert _same_set(ht_b.ids(), [100, 101, 102])
    assert _same_set(slot(ht_a, "step_filter").value()[:14].view(-1), [4] * 4 + [3] * 2 + [2] * 8)
    assert bool((slot(ht_b, "step_filter").value()[:3].view(-1) == 2).all())

    batch = steps[5]
    train(5, lambda out: out["fea_1"].sum() + out["fea_2"].sum())
    ids, rows = ht_a.ids_map()
    hook.after_step(-1, 5)
    assert int(rows.max()) <= 13
    assert _same_set(ht_a.ids(), encoded([(batch["fea_1"].values(), "fea_1"), (batch["fea_2"].values(), "fea_2")]))
    assert ht_b.ids().numel() == 0       # last seen at step 2: three steps ago
    assert bool((slot(ht_b, "step_filter").value()[:3].view(-1) == 2).all())

    def check_rows():
        _, rows_a = ht_a.ids_map()
        _, rows_b = ht_b.ids_map()
        for ht, rows, n in ((ht_a, rows_a, 14), (ht_b, rows_b, 3)):
            # evicted rows are back at the initial value with cleared optimizer state; live rows moved
            assert _rows_split(slot(ht, "embedding").value()[:n], rows, 3)
            assert _rows_split(slot(ht, "sparse_adamw_tf_exp_avg").value()[:n], rows, 0)
            assert _rows_split(slot(ht, "sparse_adamw_tf_exp_avg_sq").value()[:n], rows, 0)

    check_rows()
    Saver(shard_index=0, shard_num=1, parallel=1, hashtables=sparse_state, tensors=dense_state,
          path=str(tmp_path)).save()
    saved_steps = {}
    for name, hooks in HashtableHookFactory().get_filters().items():
        for ht, ft in hooks.items():
            saved_steps[ht] = ft._global_step.clone()
            ft._global_step.fill_(0)
    for ht in (ht_a, ht_b):
        slot(ht, "step_filter").values()[0].fill_(0)
        slot(ht, "embedding").values()[0].fill_(3)
        slot(ht, "sparse_adamw_tf_exp_avg").values()[0].fill_(0)
        slot(ht, "sparse_adamw_tf_exp_avg_sq").values()[0].fill_(0)
    Loader(str(tmp_path), hashtables=sparse_state, tensors=dense_state, parallel=1).load()
    for name, hooks in HashtableHookFactory().get_filters().items():
        for ht, ft in hooks.items():
            assert torch.equal(ft._global_step, saved_steps[ht])
    ids_a, _ = ht_a.ids_map()
    assert _same_set(ids_a, [12, 4503599627371495])      # 12 under ht2 (tag 0), 999 under ht1 (tag 1)
    check_rows()

    for step in (6, 7):
        train(step, lambda out: out["fea_2"].sum())
        ids, _ = ht_a.ids_map()
        assert _same_set(ids, [12, 1111, 4503599627371495] if step == 6 else [1111])
        hook.after_step(-1, step)

    # fifty-step filter on ht4, sweeps every ten steps: 61 steps of 5000 x 20 random ids
    hook.reset_filter_interval(10)
    rng = np.random.default_rng(0)
    last_seen = {}
    batches = {}
    for step in range(8, 68):
        vals = rng.integers(0, 99999999, 5000 * 20)
        batches[step] = vals
        for v in vals.tolist():
            last_seen[v] = step
    # the sweep of step 67 (7 + 6 * 10) is the first one that finds keys fifty steps old: last seen <= 17
    stale = [k for k, s in last_seen.items() if s <= 17]
    fresh = [k for k, s in last_seen.items() if s > 17]
    batches[68] = np.arange(100000000, 100000000 + len(stale) + 1)
    before = after = 0
    for step in range(8, 69):
        vals = torch.from_numpy(batches[step]).cuda()
        width = 20 if step < 68 else 1
        out = engine({"fea_5": RaggedTensor(vals, torch.arange(0, vals.numel() + 1, width, dtype=torch.int32,
                                                                device="cuda"))})
        out["fea_5"].sum().backward()
        opt.step()
        opt.zero_grad()
        hook.after_step(-1, step)
        ids, rows = ht_c.ids_map()
        before, after = after, ids.numel()
        if step == 67:
            assert not bool(torch.isin(ids, torch.tensor(stale, device="cuda")).any())
            assert _same_set(ids, fresh)
            assert _rows_split(slot(ht_c, "sparse_adamw_tf_exp_avg").value()[: int(rows.max()) + 1], rows, 0)
        elif step == 68:
            assert int(rows.max()) == ids.numel() - 1      # the freed rows were handed out again first
            assert ids.numel() == before + vals.numel()

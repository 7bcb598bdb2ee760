"""End-to-end parity of the GPU table + pooling + optimizer with the restated
reference CPU path (oracle.cpu_path) on benchmark config 1, and behaviour tests of
the host-side modules that read like the reference's own module tests.

Bars: key -> row assignment bit-exact when new keys are presented in the reference's
order (``dedup="sorted"``), and a bijection-equivalent assignment with the hash dedup;
fp32 rows / optimizer state / pooled outputs within rtol 1e-5, atol 1e-6.
"""
import numpy as np
import pytest
import torch

import oracle
import workloads
from oracle import cpu_path
from recis_amd import _lib, ops
from recis_amd.hooks import HashTableFilterHook
from recis_amd.nn import DynamicEmbedding, EmbeddingEngine, EmbeddingOption, HashTable
from recis_amd.nn.functional.embedding_ops import ragged_embedding_segment_reduce
from recis_amd.nn.hashtable_hook import AdmitHook, FilterHook
from recis_amd.nn.initializers import ConstantInitializer, NormalInitializer, TensorInitializer
from recis_amd.nn.modules.hashtable import HashtableRegister, filter_out_sparse_param
from recis_amd.nn.modules.hashtable_hook_impl import HashtableHookFactory
from recis_amd.optim import SparseAdagrad, SparseAdam, SparseAdamW, SparseAdamWTF
from recis_amd.ragged.tensor import RaggedTensor

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _fresh_registries():
    HashtableRegister().clear()
    HashtableHookFactory().clear_filters()
    yield


def SeededBlockInitializer(seed, std=0.01, blocks=512, bs=1024, dim=16):
    """Hands out the same per-block rows as the CPU side (workloads.seeded_block), so that both
    tables start from identical storage whatever the chunking: the first ``blocks`` blocks as one
    tensor, handed out in order by the tensor-backed generator."""
    rows = np.concatenate([workloads.seeded_block(seed, b, bs, dim, std) for b in range(blocks)])
    return TensorInitializer(torch.from_numpy(rows))


def _close(a, b, msg=""):
    np.testing.assert_allclose(a, b, rtol=1e-5, atol=1e-6, err_msg=msg)


@pytest.mark.parametrize("steps", [100])
def test_config1_hundred_steps_bit_exact_rows(steps):
    """benchmark config 1: Zipf(1.05) ids over 1e6 keys, batch 4096, lengths 1..20, dim 16 fp32,
    rows N(0, 0.01), sum pooling, backward, sparse Adagrad (lr 0.01, eps 1e-8), 100 steps, seed 0."""
    bs, dim = 1024, 16
    cpu = cpu_path.CpuTable(dim, bs, lambda b: workloads.seeded_block(0, b, bs, dim), "adagrad", 0.01, 1e-8)
    table = HashTable([dim], block_size=bs, device="cuda", initializer=SeededBlockInitializer(0),
                      name="c1", dedup="sorted")
    table.train()
    opt = SparseAdagrad(filter_out_sparse_param(table), lr=0.01, eps=1e-8)
    for step in range(steps):
        ids, off, grad = workloads.config1_step(step)
        pooled_c, uniq_c, index_c = cpu_path.train_step(cpu, ids, off, None, grad)
        ids_t, off_t = torch.from_numpy(ids).cuda(), torch.from_numpy(off).cuda()
        rows = table(ids_t)                                                    # [N, dim], request order
        pooled = ragged_embedding_segment_reduce(rows, None, None, off_t, "sum")
        pooled.backward(torch.from_numpy(grad).cuda())
        opt.step()
        opt.zero_grad()
        if step % 10 == 0 or step == steps - 1:
            _close(pooled.detach().cpu().numpy(), pooled_c, "pooled output, step %d" % step)
            got_index = table._hashtable_impl.lookup_index_readonly(torch.from_numpy(uniq_c).cuda())
            np.testing.assert_array_equal(got_index.cpu().numpy(), index_c)     # bit-exact row assignment
    ids_g, idx_g = table.ids_map()
    ids_c, idx_c = cpu.idmap.snapshot()
    assert dict(zip(ids_g.cpu().tolist(), idx_g.cpu().tolist())) == dict(zip(ids_c.tolist(), idx_c.tolist()))
    sg = table.slot_group()
    assert sg.block_num() == len(cpu.emb)
    _close(sg.slot_by_name("embedding").value().cpu().numpy(), np.concatenate(cpu.emb), "embedding rows")
    _close(sg.slot_by_name("sparse_adagrad_accum").value().cpu().numpy(), np.concatenate(cpu.s0), "adagrad state")


def test_config1_hundred_steps_hash_dedup_by_key():
    """Benchmark config 1 again (batch 4096, 100 steps from seed 0, sum pooling, sparse Adagrad) with the
    default dedup, the hash plan: lookup, expansion, the gradient handed over unsummed and the fused
    gather-reduce + Adagrad. The plan orders new keys its own way, so every key that occurs in the 100 steps
    is given its N(0, 0.01) row by key on both sides first (insert); everything is then compared by key with
    the contract's flat tolerance: pooled outputs at every step, rows and Adagrad state at the end."""
    bs, dim, steps = 1024, 16, 100
    batches = [workloads.config1_step(step) for step in range(steps)]
    keys = np.unique(np.concatenate([b[0] for b in batches]))
    rows0 = (0.01 * np.random.default_rng(1).standard_normal((len(keys), dim))).astype(np.float32)
    cpu = cpu_path.CpuTable(dim, bs, lambda b: np.zeros((bs, dim), np.float32), "adagrad", 0.01, 1e-8)
    index_c, _ = cpu.lookup(keys)
    oracle.block_insert(index_c, rows0, cpu.emb, bs)
    table = HashTable([dim], block_size=bs, device="cuda", name="c1h")      # dedup="hash" is the default
    table.insert(torch.from_numpy(keys).cuda(), torch.from_numpy(rows0).cuda())
    table.train()
    opt = SparseAdagrad(filter_out_sparse_param(table), lr=0.01, eps=1e-8)
    for step, (ids, off, grad) in enumerate(batches):
        pooled_c, _, _ = cpu_path.train_step(cpu, ids, off, None, grad)
        rows = table(torch.from_numpy(ids).cuda())                              # [N, dim], request order
        pooled = ragged_embedding_segment_reduce(rows, None, None, torch.from_numpy(off).cuda(), "sum")
        pooled.backward(torch.from_numpy(grad).cuda())
        assert table._hashtable_impl.pending_grads() == [1, 0]                 # handed over unsummed
        opt.step()
        opt.zero_grad()
        _close(pooled.detach().cpu().numpy(), pooled_c, "pooled output, step %d" % step)
    impl = table._hashtable_impl
    rows_g = impl.lookup_index_readonly(torch.from_numpy(keys).cuda())
    assert int(rows_g.min()) >= 0 and torch.unique(rows_g).numel() == len(keys) == impl.id_map_stats()[0]
    rows_c = cpu.idmap.lookup_readonly(keys)
    for slot, blocks in (("embedding", cpu.emb), ("sparse_adagrad_accum", cpu.s0)):
        got = impl.get_slot(slot).index_select(rows_g).cpu().numpy()
        _close(got, oracle.block_gather(rows_c, blocks, bs), slot)
    assert _lib.poll_device_errors() == 0


def test_config1_engine_path_matches_up_to_row_order():
    """Same workload through EmbeddingEngine (hash dedup, fused group pipeline): the row a key
    gets may differ, everything addressed by key must not."""
    bs, dim, steps = 1024, 16, 30
    cpu = cpu_path.CpuTable(dim, bs, lambda b: np.zeros((bs, dim), np.float32), "adam", 1e-3, 1e-8,
                            decay=1.0, beta_dtype=np.float64)
    eng = EmbeddingEngine({"f": EmbeddingOption(embedding_dim=dim, block_size=bs, shared_name="c1e",
                                                combiner="sum", use_weight=False)})
    eng.train()
    opt = SparseAdam({n: t._hashtable_impl for n, t in eng.hashtables().items()}, lr=1e-3)
    for step in range(steps):
        ids, off, grad = workloads.config1_step(step, batch=512)
        pooled_c, uniq_c, _ = cpu_path.train_step(cpu, ids, off, None, grad)
        rt = RaggedTensor(torch.from_numpy(ids).cuda(), torch.from_numpy(off.astype(np.int32)).cuda())
        out = eng({"f": rt})["f"]
        out.backward(torch.from_numpy(grad).cuda())
        opt.step()
        opt.zero_grad()
        _close(out.detach().cpu().numpy(), pooled_c, "pooled, step %d" % step)
    table = eng.hashtables()["c1e"]
    ids_c, _ = cpu.idmap.snapshot()
    ids_c = np.sort(ids_c)
    assert np.array_equal(np.sort(table.ids().cpu().numpy()), ids_c)
    impl = table._hashtable_impl
    rows_g = impl.lookup_index_readonly(torch.from_numpy(ids_c).cuda())
    assert len(set(rows_g.cpu().tolist())) == len(ids_c)                       # bijection key <-> row
    for slot, blocks in (("embedding", cpu.emb), ("sparse_adam_exp_avg", cpu.s0), ("sparse_adam_exp_avg_sq", cpu.s1)):
        got = impl.get_slot(slot).index_select(rows_g).cpu().numpy()
        exp = oracle.block_gather(cpu.idmap.lookup_readonly(ids_c), blocks, bs)
        # the head Zipf keys receive several hundred gradient rows per step, summed in fp32 in a
        # different order on each side: atol scales with that sum (1e-6 per unit, magnitude ~10)
        np.testing.assert_allclose(got, exp, rtol=1e-5, atol=1e-5, err_msg=slot)


# ------------------------------------------------- module behaviour (reference-style tests)
def test_lookup_insert_ids_eval():
    # tests/hashtable/ht_lookup_test.py:16-112
    ht = HashTable([8], block_size=16, device="cuda", name="ht_lookup",
                   initializer=ConstantInitializer(0.0))
    ids = torch.arange(100, device="cuda")
    emb = ht(ids)
    assert emb.shape == (100, 8) and float(emb.abs().sum()) == 0
    vals = torch.randn(100, 8, device="cuda")
    ht.insert(ids, vals)
    torch.testing.assert_close(ht(ids), vals)
    torch.testing.assert_close(ht(torch.tensor([5, 5, 7], device="cuda")), vals[[5, 5, 7]])
    assert torch.equal(torch.sort(ht.ids())[0], ids)
    ht.eval()
    out = ht(torch.arange(90, 110, device="cuda"))
    torch.testing.assert_close(out[:10], vals[90:])
    assert float(out[10:].abs().sum()) == 0
    assert ht.ids().numel() == 100                     # eval() admits nothing
    ht.train()
    out = ht(torch.arange(100, 105, device="cuda"), AdmitHook("ReadOnly"))
    assert float(out.abs().sum()) == 0 and ht.ids().numel() == 100
    ht(torch.arange(100, 105, device="cuda"))
    assert ht.ids().numel() == 105
    # missing keys take rows from the initializer
    ht2 = HashTable([4], block_size=8, device="cuda", name="ht_init", initializer=ConstantInitializer(2.5))
    assert torch.all(ht2(torch.tensor([3, 9], device="cuda")) == 2.5)
    with pytest.raises(ValueError):
        HashTable([4], device="cuda", name="ht_init")  # duplicate table name


def test_slot_metadata_and_block_growth():
    # tests/hashtable/ht_slot_test.py; block_num = (id_num + bs) / bs (hashtable.cc:255-261)
    ht = HashTable([4], block_size=10, device="cuda", name="ht_slot", initializer=ConstantInitializer(1.0))
    ht(torch.arange(25, device="cuda"))
    sg = ht.slot_group()
    slot = sg.slot_by_name("embedding")
    assert slot.name() == "embedding" and slot.block_size() == 10 and slot.flat_size() == 4
    assert len(slot.values()) == 3 and slot.value().shape == (30, 4)
    assert float(slot.value().sum()) == 30 * 4
    ht(torch.arange(25, 30, device="cuda"))
    assert len(ht.slot_group().slot_by_name("embedding").values()) == 4   # 30 ids -> (30+10)/10
    # values() alias live storage
    ht.slot_group().slot_by_name("embedding").values()[0][0].fill_(9.0)
    assert float(ht.embeddings()[0].sum()) == 36.0


def test_grad_accumulation_kat():
    # tests/hashtable/ht_grad_ga_test.py:9-33
    ht = HashTable([4], device="cuda", name="ht_ga")
    ht.accept_grad(torch.tensor([1, 2, 3], device="cuda"), torch.ones(3, 4, device="cuda"))
    ht.accept_grad(torch.tensor([1, 1, 1], device="cuda"), torch.ones(3, 4, device="cuda") * 2)
    ht.accept_grad(torch.tensor([2, 2, 2], device="cuda"), torch.ones(3, 4, device="cuda") * 3)
    ga = ht.grad(3).coalesce()
    assert ga.indices().cpu().tolist() == [[0, 1, 2]]
    exp = torch.tensor([[7.0] * 4, [10.0] * 4, [1.0] * 4]) / 3.0
    torch.testing.assert_close(ga.values().cpu(), exp)
    # the merged pairs the optimizers consume: per-row sums / accumulation steps
    index, g = ht._hashtable_impl.grad_pairs(3)
    got = dict(zip(index.cpu().tolist(), g.cpu()[:, 0].tolist()))
    assert got == pytest.approx({1: 7 / 3, 2: 10 / 3, 3: 1 / 3})


@pytest.mark.parametrize("cls,ref_wd", [(SparseAdamW, "adamw"), (SparseAdamWTF, "tf"), (SparseAdam, "none")])
def test_sparse_adam_family_tracks_torch_adamw(cls, ref_wd):
    # tests/optim/sparse_adamw_test.py:84-175: zero-init rows, every row updated each step
    U, D, steps, lr, wd = 512, 16, 20, 1e-2, 1e-2
    ht = HashTable([D], block_size=128, device="cuda", name="adam_" + ref_wd, dedup="sorted")
    ht.train()
    opt = cls(filter_out_sparse_param(ht), lr=lr, weight_decay=wd)
    torch_wd = {"adamw": wd, "tf": wd / lr, "none": 0.0}[ref_wd]
    p = torch.nn.Parameter(torch.zeros(U, D, device="cuda"))
    topt = torch.optim.AdamW([p], lr=lr, weight_decay=torch_wd)
    ids = torch.arange(U, device="cuda")
    g = torch.Generator(device="cuda").manual_seed(3)
    for _ in range(steps):
        target = torch.randn(U, D, device="cuda", generator=g)
        loss = ((ht(ids) - target) ** 2).sum()
        loss.backward()
        opt.step()
        opt.zero_grad()
        topt.zero_grad()
        ((p - target) ** 2).sum().backward()
        topt.step()
    torch.testing.assert_close(ht(ids).detach(), p.detach(), rtol=1e-5, atol=1e-4)
    # row placement (sparse_adamw_test.py:177-208): first new key takes the largest fresh row
    rows = ht._hashtable_impl.lookup_index_readonly(ids)
    assert torch.equal(rows, torch.arange(U - 1, -1, -1, device="cuda"))
    names = [s.name() for s in ht.slot_group().slots()]
    prefix = {"adamw": "sparse_adamw_", "tf": "sparse_adamw_tf_", "none": "sparse_adam_"}[ref_wd]
    assert names == ["embedding", prefix + "exp_avg", prefix + "exp_avg_sq"]
    assert set(opt.state_dict()) == {prefix + "step", prefix + "beta1", prefix + "beta2"}


def test_grad_reduce_by_id_and_worker():
    for mode in ("worker", "id"):
        ht = HashTable([2], device="cuda", name="gr_" + mode, grad_reduce_by=mode)
        ht.train()
        ids = torch.tensor([4, 4, 4, 9], device="cuda")
        out = ht(ids)
        out.backward(torch.tensor([[1.0, 1], [2, 2], [6, 6], [5, 5]], device="cuda"))
        index, g = ht._hashtable_impl.grad_pairs(1)
        rows = ht._hashtable_impl.lookup_index_readonly(torch.tensor([4, 9], device="cuda"))
        got = {int(i): g[k, 0].item() for k, i in enumerate(index.cpu())}
        exp4 = 9.0 if mode == "worker" else 3.0
        assert got[int(rows[0])] == pytest.approx(exp4) and got[int(rows[1])] == pytest.approx(5.0)


def test_global_step_filter_eviction_matches_cpu_path():
    """Last-seen-step stamping + eviction (hashtable_hook_impl.py:487-551, filter_hook.py:82-117)
    against the same policy on the CPU path; freed rows are recycled by later inserts."""
    dim, bs, filter_step, interval = 4, 64, 3, 4
    cpu = cpu_path.CpuTable(dim, bs, lambda b: np.zeros((bs, dim), np.float32), "adagrad", 0.1, 1e-8,
                            step_filter=True)
    ht = HashTable([dim], block_size=bs, device="cuda", name="evict", dedup="sorted",
                   filter_hook=FilterHook("GlobalStepFilter", {"filter_step": filter_step}))
    ht.train()
    opt = SparseAdagrad(filter_out_sparse_param(ht), lr=0.1)
    hook = HashTableFilterHook(filter_interval=interval)
    rng = np.random.default_rng(5)
    last = 0
    for step in range(1, 25):
        ids = rng.integers(step * 20, step * 20 + 150, size=200)
        off = np.arange(0, 201, 4)
        grad = rng.standard_normal((50, dim)).astype(np.float32)
        cpu_path.train_step(cpu, ids, off, None, grad)          # advances cpu.global_step
        rows = ht(torch.from_numpy(ids).cuda())
        pooled = ragged_embedding_segment_reduce(rows, None, None, torch.from_numpy(off).cuda(), "sum")
        pooled.backward(torch.from_numpy(grad).cuda())
        opt.step()
        opt.zero_grad()
        hook.after_step(None, step)
        if last == 0:
            last = step
        if step - last >= interval:
            ev_ids, ev_rows = cpu.evict_older_than(filter_step)
            # the reference re-initialises every slot but the stamp at the freed rows
            if len(ev_rows):
                oracle.block_insert(ev_rows, np.zeros((1, dim), np.float32), cpu.emb, bs)
                oracle.block_insert(ev_rows, np.zeros((1, dim), np.float32), cpu.s0, bs)
            last = step
        assert np.array_equal(np.sort(ht.ids().cpu().numpy()), np.sort(cpu.idmap.snapshot()[0]))
    live = np.sort(cpu.idmap.snapshot()[0])
    rows_g = ht._hashtable_impl.lookup_index_readonly(torch.from_numpy(live).cuda()).cpu().numpy()
    assert len(set(rows_g.tolist())) == len(live)
    got = ht._hashtable_impl.get_slot("embedding").index_select(torch.from_numpy(rows_g).cuda()).cpu().numpy()
    _close(got, cpu.rows_of(live)[1])
    stamps = ht._hashtable_impl.get_slot("step_filter").index_select(torch.from_numpy(rows_g).cuda())
    exp_stamps = oracle.block_gather(cpu.idmap.lookup_readonly(live), cpu.stamp, bs)
    np.testing.assert_array_equal(stamps.cpu().numpy(), exp_stamps)
    assert ht._hashtable_impl.id_map_stats()[1] < 24 * 150    # rows were reused, not only appended


def test_engine_coalesces_and_pools():
    """Two features sharing one configuration land in one physical table (12-bit tags keep equal
    raw ids apart); a third with another dim gets its own; outputs match a direct computation."""
    opts = {
        "user": EmbeddingOption(embedding_dim=8, shared_name="user", combiner="sum", block_size=64,
                                initializer=NormalInitializer(0, 0.1)),
        "item": EmbeddingOption(embedding_dim=8, shared_name="item", combiner="sum", block_size=64,
                                initializer=NormalInitializer(0, 0.1)),
        "cate": EmbeddingOption(embedding_dim=4, shared_name="cate", combiner="mean", block_size=64,
                                initializer=NormalInitializer(0, 0.1), use_weight=False),
    }
    eng = EmbeddingEngine(opts)
    assert len(eng.hashtables()) == 2
    eng.train()
    user = RaggedTensor(torch.tensor([1, 2, 3, 1], device="cuda"), torch.tensor([0, 3, 4], device="cuda"),
                        weight=torch.tensor([1.0, 2.0, 3.0, 4.0], device="cuda"))
    item = torch.tensor([[1, 2], [3, 3]], device="cuda")
    cate = RaggedTensor(torch.tensor([7, 8, 9], device="cuda"), torch.tensor([0, 0, 3], device="cuda"))
    out = eng({"user": user, "item": item, "cate": cate})
    assert out["user"].shape == (2, 8) and out["item"].shape == (2, 8) and out["cate"].shape == (2, 4)
    big = [t for n, t in eng.hashtables().items() if t.coalesce][0]
    info = big.children_info()
    assert info.children() == ["user", "item"]

    def row(child, raw):
        key = torch.tensor([info.encode_id(raw, info.child_index(child))], device="cuda")
        idx = big._hashtable_impl.lookup_index_readonly(key)
        assert int(idx) >= 0
        return big._hashtable_impl.get_slot("embedding").index_select(idx)[0]

    torch.testing.assert_close(out["user"][0], row("user", 1) + 2 * row("user", 2) + 3 * row("user", 3))
    torch.testing.assert_close(out["user"][1], 4 * row("user", 1))
    torch.testing.assert_close(out["item"][1], 2 * row("item", 3))
    assert not torch.equal(row("user", 1), row("item", 1))
    assert float(out["cate"][0].abs().sum()) == 0
    # gradients flow to the table
    (out["user"].sum() + out["item"].sum() + out["cate"].sum()).backward()
    assert all(t._hashtable_impl.has_grad() for t in eng.hashtables().values())


def test_dynamic_embedding_tile_and_max():
    opt = EmbeddingOption(embedding_dim=4, shared_name="tile_t", combiner="tile",
                          combiner_kwargs={"tile_len": 3}, block_size=32, use_weight=False,
                          initializer=NormalInitializer(0, 1.0))
    emb = DynamicEmbedding(opt)
    emb.train()
    rt = RaggedTensor(torch.tensor([5, 6, 7, 8, 9, 5], device="cuda"), torch.tensor([0, 4, 4, 6], device="cuda"))
    out = emb(rt)
    assert out.shape == (3, 12)
    rows = emb.hashtable(torch.tensor([5, 6, 7, 9], device="cuda")).detach()
    torch.testing.assert_close(out[0].detach(), torch.cat([rows[0], rows[1], rows[2]]))   # truncated at 3
    assert float(out[1].abs().sum()) == 0
    torch.testing.assert_close(out[2].detach(), torch.cat([rows[3], rows[0], torch.zeros(4, device="cuda")]))
    out.sum().backward()
    index, g = emb.hashtable._hashtable_impl.grad_pairs(1)
    r5 = int(emb.hashtable._hashtable_impl.lookup_index_readonly(torch.tensor([5], device="cuda")))
    assert g[index.cpu().tolist().index(r5)].tolist() == [2.0] * 4              # id 5 kept twice
    opt2 = EmbeddingOption(embedding_dim=4, shared_name="max_t", combiner="max", block_size=32,
                           use_weight=False, initializer=NormalInitializer(0, 1.0))
    emb2 = DynamicEmbedding(opt2)
    emb2.train()
    out2 = emb2(rt)
    rows2 = emb2.hashtable(torch.tensor([5, 6, 7, 8, 9], device="cuda")).detach()
    torch.testing.assert_close(out2[0].detach(), rows2[:4].max(0)[0])
    torch.testing.assert_close(out2[2].detach(), rows2[[4, 0]].max(0)[0])


def test_dynamic_embedding_staged_calls_match_forward():
    """exchange_ids -> lookup_exchange_emb -> emb_reduce (embedding.py:498-624), driven by hand as
    the reference's engine does, gives what forward() gives, values and accumulated gradients."""
    rng = np.random.default_rng(5)
    lens = rng.integers(0, 12, 200)
    off = torch.from_numpy(np.concatenate([[0], np.cumsum(lens)])).cuda()
    ids = torch.from_numpy(rng.integers(0, 150, int(off[-1]))).cuda()
    w = torch.from_numpy(rng.random(int(off[-1])).astype(np.float32)).cuda()
    for combiner in ("sum", "mean"):
        embs = []
        for name in ("fused", "staged"):
            opt = EmbeddingOption(embedding_dim=8, shared_name="%s_%s" % (name, combiner), combiner=combiner,
                                  block_size=64, initializer=ConstantInitializer(0.5))
            e = DynamicEmbedding(opt)
            e.train()
            embs.append(e)
        fused, staged = embs
        out_f = fused(RaggedTensor(ids, off, w))
        ex = staged.exchange_ids(ids, off)
        assert ex.parts == ex.parts_reverse == [int(torch.unique(ids).numel())]
        assert torch.equal(ex.ids[ex.reverse_index.long()], ids)
        looked = staged.lookup_exchange_emb(ex, None)
        assert looked.emb_shape == [ex.parts[0], 8] and staged.wait_exchange_emb(looked).shape == (ex.parts[0], 8)
        out_s = staged.emb_reduce(looked, w, combiner, {})
        torch.testing.assert_close(out_s, out_f, rtol=1e-5, atol=1e-6)
        g = torch.from_numpy(rng.standard_normal(tuple(out_f.shape)).astype(np.float32)).cuda()
        out_f.backward(g)
        out_s.backward(g)
        grads = []
        for e in (fused, staged):
            impl = e.hashtable._hashtable_impl
            index, rows = impl.grad_pairs(1)
            key_of_row = dict(zip(*[t.cpu().tolist() for t in impl.ids_map()][::-1]))
            order = np.argsort([key_of_row[r] for r in index.cpu().tolist()])
            grads.append(rows.cpu().numpy()[order])
        np.testing.assert_allclose(grads[1], grads[0], rtol=1e-5, atol=1e-5)


def test_three_tables_state_dict_keys():
    """tests/hashtable/ht_state_dict_test.py:27-49: three tables of 3 * 2^20 + 200 rows each, two
    training steps, then the keys a checkpoint of the model would hold, in the reference's order."""
    class Model(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self._emb_one = HashTable([16], name="16")
            self._emb_two = HashTable([32], name="32")
            self._emb_three = HashTable([64], name="64")

        def forward(self, ids):
            return torch.concat([self._emb_one(ids), self._emb_two(ids), self._emb_three(ids)], dim=1).sum()

    model = Model()
    sparse_state = filter_out_sparse_param(model)
    optim = SparseAdamWTF(sparse_state)
    ids_num = (1 << 20) * 3 + 200
    ids = torch.arange(ids_num, device="cuda")
    for _ in range(2):
        model(ids).backward()
        optim.step()
        optim.zero_grad()
    save_dict = dict(sparse_state)
    assert list(save_dict.keys()) == ["16", "32", "64"]
    save_dict.update(optim.state_dict())
    assert list(save_dict.keys()) == ["16", "32", "64", "sparse_adamw_tf_beta2", "sparse_adamw_tf_beta1",
                                      "sparse_adamw_tf_step"]
    for t, dim in ((model._emb_one, 16), (model._emb_two, 32), (model._emb_three, 64)):
        assert t.ids().numel() == ids_num
        rows = t.embeddings()[:ids_num]
        assert rows.shape == (ids_num, dim)
        # every row took two identical steps from the zero initial value: all rows are equal and moved
        assert bool((rows == rows[0]).all()) and float(rows[0].abs().min()) > 0
    # block_apply_adamw_op.cc:121 calls step.add(1) and drops the result: the stored step stays 0
    assert int(optim.state_dict()["sparse_adamw_tf_step"]) == 0


def test_engine_sequence_pooled_and_tiled_from_one_plan():
    """A sequence feature used twice, mean-pooled and kept row by row (two lengths), plus a second
    sequence: the engine tags / merges / deduplicates the shared inputs once, and every output and
    the accumulated row gradients equal what separate DynamicEmbedding-style calls give."""
    rng = np.random.default_rng(11)
    B = 64

    def seq(max_len):
        lens = rng.integers(0, max_len, B)
        off = torch.from_numpy(np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)).cuda()
        return RaggedTensor(torch.from_numpy(rng.integers(0, 40, int(off[-1]))).cuda(), off)

    a, b = seq(30), seq(12)

    def option(combiner, **kw):
        return EmbeddingOption(embedding_dim=8, shared_name="seq_tab", combiner=combiner, use_weight=False,
                               block_size=64, initializer=NormalInitializer(0, 1.0), **kw)

    engine = EmbeddingEngine({
        "a_mean": option("mean"), "b_mean": option("mean"),
        "a_rows": option("tile", combiner_kwargs={"tile_len": 5}),
        "b_rows": option("tile", combiner_kwargs={"tile_len": 9}),
    })
    engine.train()
    out = engine({"a_mean": a, "b_mean": b, "a_rows": a, "b_rows": b})
    table = next(iter(engine.hashtables().values()))
    assert out["a_mean"].shape == (B, 8) and out["a_rows"].shape == (B, 5 * 8) and out["b_rows"].shape == (B, 9 * 8)

    def rows_of(rt):
        return table(rt.values()).detach()

    for name, rt, t in (("a", a, 5), ("b", b, 9)):
        rows, off = rows_of(rt), rt.offsets()[-1].cpu().numpy()
        mean = torch.stack([rows[off[i]:off[i + 1]].mean(0) if off[i + 1] > off[i] else torch.zeros(8, device="cuda")
                            for i in range(B)])
        torch.testing.assert_close(out[name + "_mean"].detach(), mean, rtol=1e-5, atol=1e-6)
        tiled = torch.zeros(B, t, 8, device="cuda")
        for i in range(B):
            k = min(t, off[i + 1] - off[i])
            tiled[i, :k] = rows[off[i]:off[i] + k]
        assert torch.equal(out[name + "_rows"].detach(), tiled.view(B, t * 8))
    # gradients: every kept row of a_rows passes 1, every pooled occurrence 1 / len
    (out["a_mean"].sum() + out["a_rows"].sum()).backward()
    impl = table._hashtable_impl
    index, g = impl.grad_pairs(1)
    got = torch.zeros(impl.ids_num() + 1, 8, device="cuda").index_add_(0, index, g)
    off = a.offsets()[-1].cpu().numpy()
    exp = torch.zeros_like(got)
    row_of = impl.lookup_index_readonly(a.values())
    for i in range(B):
        n = off[i + 1] - off[i]
        for k in range(n):
            exp[row_of[off[i] + k]] += 1.0 / n + (1.0 if k < 5 else 0.0)
    torch.testing.assert_close(got, exp, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("n_feat,skip", [(3, None), (3, 1), (9, None)])
def test_padded_gather_with_one_output_per_feature(n_feat, skip):
    """RaggedTileParts against the single-output list form of the tile combiner: same rows, same
    gradient of the unique rows, with all gradients present (one gather-reduce launch over separate
    arrays), with one output unused, and with more features than one launch takes (a pass each)."""
    from recis_amd import ops
    from recis_amd.nn.functional.embedding_ops import RaggedTileParts

    rng = np.random.default_rng(n_feat)
    U, D = 50, 16
    bs = [int(rng.integers(3, 9)) for _ in range(n_feat)]
    tile_len = [int(rng.integers(1, 7)) for _ in range(n_feat)]
    lens = rng.integers(0, 9, sum(bs))
    off = torch.from_numpy(np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)).cuda()
    ids = torch.from_numpy(rng.integers(0, 1000, int(off[-1]))).cuda()
    plan = ops.ids_unique_plan(ids)
    emb = torch.randn(plan.U, D, device="cuda")
    e1 = emb.clone().requires_grad_()
    parts = RaggedTileParts.apply(e1, plan.inverse, off, plan, bs, tile_len)
    e2 = emb.clone().requires_grad_()
    whole = ragged_embedding_segment_reduce(e2, None, plan.inverse, off, "tile", {"bs": bs, "tile_len": tile_len},
                                            plan=plan)
    rows = [b * t for b, t in zip(bs, tile_len)]
    for part, ref, b, t in zip(parts, torch.split(whole, rows), bs, tile_len):
        assert part.shape == (b, t * D) and torch.equal(part.detach().reshape(-1, D), ref.detach())
    ups = [torch.randn(p.shape, device="cuda") for p in parts]
    used = [k for k in range(n_feat) if k != skip]
    torch.autograd.backward([parts[k] for k in used], [ups[k] for k in used])
    g_whole = torch.cat([(ups[k] if k != skip else torch.zeros_like(ups[k])).reshape(-1, D) for k in range(n_feat)])
    whole.backward(g_whole)
    torch.testing.assert_close(e1.grad, e2.grad, rtol=1e-5, atol=1e-5)


def test_feature_engine_ops_and_fusion():
    """Restated from tests/feature_engine/op_test.py:17-36,95-131 and feature_engine_test.py: Mod,
    Bucketize, IDMultiHash, Hash known answers, through the fused engine path."""
    from recis_amd.features import Bucketize, Feature, FeatureEngine, Hash, IDMultiHash, Mod, SelectField

    vals = torch.randn(10) * 5
    feats = [
        Feature("a").add_op(SelectField("a")).add_op(Mod(1000)),
        Feature("b").add_op(SelectField("b")).add_op(Mod(7)),
        Feature("c").add_op(SelectField("c")).add_op(Bucketize([1.0, 2, 3, 4, 5])),
        Feature("d").add_op(SelectField("c")).add_op(Bucketize([0.0])),
        Feature("a_dup").add_op(SelectField("a")).add_op(Mod(1000)),
        Feature("h").add_op(SelectField("h")).add_op(Hash("farm")).add_op(Mod(1 << 62)),
        Feature("m").add_op(SelectField("h")).add_op(Hash("murmur")),
        Feature("mh").add_op(SelectField("a")).add_op(IDMultiHash([1000] * 4)),
        # Bucketize -> Mod of one feature: the engine runs the pair as one launch
        Feature("cm").add_op(SelectField("c")).add_op(Bucketize([1.0, 2, 3, 4, 5])).add_op(Mod(4)),
        Feature("cm2").add_op(SelectField("c")).add_op(Bucketize([-1.0, 0.0, 1.0])).add_op(Mod(2)).add_op(Mod(5)),
    ]
    engine = FeatureEngine(feats)
    data = {
        "a": RaggedTensor(torch.tensor([1001, 1002, 1003]).cuda(), torch.tensor([0, 1, 2, 3]).cuda()),
        "b": torch.tensor([-1, 15], device="cuda"),
        "c": RaggedTensor(vals.cuda(), torch.arange(0, 11).cuda()),
        "h": RaggedTensor(torch.tensor([0, 1, 2, 1, 2, 3], dtype=torch.int8).cuda(),
                          [torch.tensor([0, 1, 2]).cuda(), torch.tensor([0, 3, 6]).cuda()]),
    }
    out = engine(data)
    assert out["a"].values().tolist() == [1, 2, 3] and out["a_dup"].values().tolist() == [1, 2, 3]
    assert out["b"].tolist() == [(2 ** 64 - 1) % 7, 1]
    assert torch.equal(out["c"].values().cpu(), torch.bucketize(vals, torch.tensor([1.0, 2, 3, 4, 5]), right=True))
    assert torch.equal(out["d"].values().cpu(), (vals >= 0).long())
    assert torch.equal(out["cm"].values().cpu(), torch.bucketize(vals, torch.tensor([1.0, 2, 3, 4, 5]), right=True) % 4)
    assert torch.equal(out["cm2"].values().cpu(), torch.bucketize(vals, torch.tensor([-1.0, 0.0, 1.0]), right=True) % 2 % 5)
    farm = [-7736835464683084646, -5546720800891377920]
    assert out["h"].values().tolist() == [(f + 2 ** 64) % (1 << 62) for f in farm]
    assert out["m"].values().tolist() == [-4003751876240412087, -1042754718167355375]
    assert out["m"].offsets()[-1].tolist() == [0, 1, 2]
    exp = [[1, 2, 3], [3, 6, 9], [5, 10, 15], [7, 14, 21]]
    for j in range(4):
        assert out["multi_hash_%d" % j].values().tolist() == exp[j]


def test_a_waiting_plan_between_forward_and_backward_does_not_steal_the_unique_count(rng):
    """DynamicEmbedding's forward leaves its unique count on the way to the stream's staging word
    and reads it in backward. Another plan on the same stream in between (here one that waits for
    its own count, with a very different number of distinct ids, as HashTable._unique in eval mode
    or exchange_ids make) reuses that word: backward must still see the count of ITS plan. Checked
    by the gradient per key against the oracle's scatter."""
    from recis_amd.nn.modules.hashtable import HashtableRegister

    HashtableRegister().clear()
    opt = EmbeddingOption(embedding_dim=8, shared_name="interleave", combiner="sum", block_size=256,
                          use_weight=False, initializer=NormalInitializer(0, 0.1))
    emb = DynamicEmbedding(opt)
    emb.train()
    S = 2000
    lens = rng.integers(0, 6, size=S)
    off = np.concatenate([[0], np.cumsum(lens)])
    ids = rng.integers(0, 900, size=int(off[-1]))
    rt = RaggedTensor(torch.from_numpy(ids).cuda(), torch.from_numpy(off.astype(np.int32)).cuda())
    out = emb(rt)
    other = ops.ids_unique_plan(torch.arange(17, device="cuda"), wait=True)     # U = 17 on the same stream
    assert other.U == 17
    third = ops.ids_unique_plan(torch.arange(50000, device="cuda"), wait=False)  # and one that does not wait
    up = rng.standard_normal((S, 8)).astype(np.float32)
    out.backward(torch.from_numpy(up).cuda())
    assert third.U == 50000
    impl = emb.hashtable._hashtable_impl
    index, g = impl.grad_pairs(1)
    uniq, inv = np.unique(ids, return_inverse=True)
    assert index.numel() == len(uniq)
    exp = oracle.segment_reduce_backward(up, None, inv, off, len(uniq), "sum")
    rows = impl.lookup_index_readonly(torch.from_numpy(uniq).cuda())
    order = torch.argsort(index)
    assert torch.equal(index[order], torch.sort(rows).values)
    by_row = dict(zip(rows.tolist(), range(len(uniq))))
    perm = [by_row[r] for r in index[order].tolist()]
    np.testing.assert_allclose(g[order].cpu().numpy(), exp[perm], rtol=1e-5, atol=1e-5)
    assert _lib.poll_device_errors() == 0


@pytest.mark.parametrize("opt_cls", [SparseAdam, SparseAdagrad])
def test_gradient_summed_in_the_optimizer_step_equals_summed_first(opt_cls):
    """The module layer hands the table its gradient unsummed (accept_planned_grad) and the optimizer step
    sums it and updates the rows in one launch. Two engines on the same data, one stepping that way, the other
    made to sum first (grad_pairs() before step(), what any reader of the gradient triggers): rows and state
    agree after every step to the last bit or two (each engine makes its own batch plan, and the order inside an
    id's occurrence list, hence the order of its sum, is not fixed from plan to plan; on one plan the two ways
    are equal bit for bit: test_fused_gather_reduce_update_equals_the_two_calls). A second gradient in the same
    step is summed and merged as before."""
    def make(tag):
        HashtableRegister().clear()
        init = NormalInitializer(0.0, 0.1, generator=torch.Generator(device="cuda").manual_seed(7))
        eng = EmbeddingEngine({
            "a": EmbeddingOption(embedding_dim=16, shared_name="t" + tag, combiner="sum", use_weight=False, initializer=init),
            "b": EmbeddingOption(embedding_dim=16, shared_name="t" + tag, combiner="mean", use_weight=False, initializer=init),
        }).cuda()
        eng.train()
        return eng, opt_cls(filter_out_sparse_param(eng), lr=1e-2)
    (e1, o1), (e2, o2) = make("1"), make("2")
    rng = np.random.default_rng(11)
    for step in range(4):
        dense = torch.from_numpy(rng.integers(0, 300, size=(512, 1))).cuda()           # one id per sample
        lens = rng.integers(0, 9, size=512)
        off = torch.from_numpy(np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)).cuda()
        vals = torch.from_numpy(rng.integers(0, 300, size=int(lens.sum()))).cuda()
        up = torch.randn(512, 16, device="cuda", generator=torch.Generator(device="cuda").manual_seed(step))
        for eng, opt, sum_first in ((e1, o1, False), (e2, o2, True)):
            feats = {"a": dense} if step % 2 == 0 else {"a": dense, "b": RaggedTensor(vals, off)}
            out = eng(feats)
            torch.autograd.backward([out[k] for k in out], [up for _ in out])
            impls = [t._hashtable_impl for t in eng.hashtables().values()]
            if step % 2 == 0:
                assert all(i.pending_grads() == [1, 0] for i in impls)           # waiting unsummed
            if sum_first:
                for i in impls:
                    i.grad_pairs(1)
                    assert i.pending_grads()[0] == 0
            opt.step()
            opt.zero_grad()
        for t1, t2 in zip(e1.hashtables().values(), e2.hashtables().values()):
            for s1, s2 in zip(t1.slot_group().slots(), t2.slot_group().slots()):
                torch.testing.assert_close(s1.value(), s2.value(), rtol=1e-5, atol=1e-7, msg=lambda m: "%s step %d slot %s" % (m, step, s1.name()))
    assert _lib.poll_device_errors() == 0


@pytest.mark.parametrize("opt_cls,dtype", [(SparseAdagrad, torch.float32), (SparseAdam, torch.float32),
                                           (SparseAdagrad, torch.bfloat16)])
def test_two_gradients_of_one_lookup_summed_in_the_optimizer_step(opt_cls, dtype):
    """Sequence features used twice, mean-pooled and kept row by row: both backward passes hand their gradient
    to the table unsummed (the padded one as one array per feature), and the optimizer step sums both and
    updates the rows in one launch (apply_planned2). A second engine on the same data is made to sum first
    (grad_pairs() before step()): rows and state agree after every step up to the order of the fp32 sums (each
    engine makes its own plan; on one plan the two ways are pinned against each other bit for bit in
    test_two_input_fused_update_equals_gather_reduce_then_update)."""
    def make(tag):
        HashtableRegister().clear()
        init = NormalInitializer(0.0, 0.1, generator=torch.Generator(device="cuda").manual_seed(3))
        opt = lambda combiner, **kw: EmbeddingOption(embedding_dim=32, shared_name="s" + tag, combiner=combiner, dtype=dtype,
                                                     use_weight=False, initializer=init, **kw)
        eng = EmbeddingEngine({"a_mean": opt("mean"), "b_mean": opt("mean"),
                               "a_rows": opt("tile", combiner_kwargs={"tile_len": 6}),
                               "b_rows": opt("tile", combiner_kwargs={"tile_len": 11})}).cuda()
        eng.train()
        return eng, opt_cls(filter_out_sparse_param(eng), lr=1e-2)
    (e1, o1), (e2, o2) = make("1"), make("2")
    rng = np.random.default_rng(5)
    B = 256

    def seq(max_len):
        lens = rng.integers(0, max_len, B)
        off = torch.from_numpy(np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)).cuda()
        return RaggedTensor(torch.from_numpy(rng.integers(0, 500, int(off[-1]))).cuda(), off)

    for step in range(3):
        a, b = seq(20), seq(9)
        gen = torch.Generator(device="cuda").manual_seed(step)
        ups = {"a_mean": torch.randn(B, 32, device="cuda", generator=gen), "b_mean": torch.randn(B, 32, device="cuda", generator=gen),
               "a_rows": torch.randn(B, 6 * 32, device="cuda", generator=gen).to(dtype),
               "b_rows": torch.randn(B, 11 * 32, device="cuda", generator=gen).to(dtype)}
        for eng, opt, sum_first in ((e1, o1, False), (e2, o2, True)):
            out = eng({"a_mean": a, "b_mean": b, "a_rows": a, "b_rows": b})
            torch.autograd.backward([out[k] for k in ups], [ups[k].to(out[k].dtype) for k in ups])
            impl = next(iter(eng.hashtables().values()))._hashtable_impl
            assert impl.pending_grads() == [2, 0]                       # both waiting unsummed
            if sum_first:
                impl.grad_pairs(1)
                assert impl.pending_grads()[0] == 0
            opt.step()
            opt.zero_grad()
        t1, t2 = next(iter(e1.hashtables().values())), next(iter(e2.hashtables().values()))
        for s1, s2 in zip(t1.slot_group().slots(), t2.slot_group().slots()):
            tol = dict(rtol=1e-5, atol=1e-6) if dtype == torch.float32 else dict(rtol=2 ** -7, atol=1e-6)
            torch.testing.assert_close(s1.value().float(), s2.value().float(), msg=lambda m: "%s step %d slot %s" % (m, step, s1.name()), **tol)
    assert _lib.poll_device_errors() == 0

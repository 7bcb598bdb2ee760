"""Checkpoint save / load of GPU tables (Saver, Loader, CheckpointReader), restating the
reference's save/load test (tests/serialize/save_load_test.py:141-236): what is saved is read
back by the safetensors library, loaded into fresh tables, and saved again unchanged."""
import json
import os

import pytest
import torch
from safetensors import safe_open

from recis_amd import _lib
from recis_amd.nn import EmbeddingEngine, EmbeddingOption, HashTable
from recis_amd.nn.initializers import ConstantInitializer, NormalInitializer
from recis_amd.nn.modules.hashtable import HashtableRegister, filter_out_sparse_param, gen_slice
from recis_amd.optim import SparseAdamW
from recis_amd.ragged.tensor import RaggedTensor
from recis_amd.serialize import CheckpointReader, Loader, Saver

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _fresh_table_names():
    HashtableRegister().clear()
    yield
    HashtableRegister().clear()


def _read_all(path):
    index = json.load(open(os.path.join(path, "index")))
    out = {}
    for fname in index["file_index"]:
        with safe_open(os.path.join(path, fname), "pt") as f:
            for k in f.keys():
                out[k] = f.get_tensor(k)
    return out


def _rows_by_id(ids, rows):
    order = torch.argsort(ids)
    return ids[order], rows[order]


def _trained_table(name, n, dim=8, slice_=None, seed=0):
    g = torch.Generator(device="cuda").manual_seed(seed)
    ht = HashTable([dim], block_size=1024, device="cuda", name=name, slice=slice_ or gen_slice(0, 1),
                   initializer=NormalInitializer(0, 0.1))
    ht.train()
    opt = SparseAdamW(filter_out_sparse_param(ht), lr=1e-2)
    ids = torch.randperm(10 * n, device="cuda", generator=g)[:n]
    for _ in range(2):
        (ht(ids) * torch.randn(n, dim, device="cuda", generator=g)).sum().backward()
        opt.step()
        opt.zero_grad()
    return ht, opt, ids


@pytest.mark.parametrize("packed", ["0", "1"])
@pytest.mark.parametrize("parallel", [1, 8])
def test_save_then_read_load_and_save_again(tmp_path, parallel, packed, monkeypatch):
    """``packed``: the saved table keeps its optimizer state next to the embedding rows
    (RECIS_PACKED_STATE=1) or in arrays of its own; the table that loads it does the opposite."""
    monkeypatch.setenv("RECIS_PACKED_STATE", packed)
    monkeypatch.setenv("RECIS_BLOCK_WRITE_SIZE", "3000")   # several pieces per slot
    monkeypatch.setenv("RECIS_BLOCK_READ_SIZE", "1700")
    n, dim = 10000, 8
    ht, opt, ids = _trained_table("ckpt_a%d" % parallel, n, dim)
    impl = ht._hashtable_impl
    emb = impl.get_slot("embedding").index_select(impl.lookup_index_readonly(ids))
    dense = {"tower.weight": torch.randn(5, 3, device="cuda"), "step": torch.tensor(3)}
    path = str(tmp_path / "a")
    Saver(0, 1, parallel, path, hashtables={"t": ht}, tensors=dense).save()

    # (1) the safetensors library reads the files: keys and rows as they are in the table
    data = _read_all(path)
    name = "ckpt_a%d" % parallel
    got_ids, got_emb = _rows_by_id(data[name + ".id/part_0_1"], data[name + ".embedding/part_0_1"])
    exp_ids, exp_emb = _rows_by_id(ids.cpu(), emb.cpu())
    assert torch.equal(got_ids, exp_ids) and torch.equal(got_emb, exp_emb)
    assert torch.equal(data["tower.weight^ "], dense["tower.weight"].cpu())
    slot_names = [s.name() for s in impl.slot_group().slots()]
    assert sorted(k for k in data if "/part_" in k) == sorted(
        "%s.%s/part_0_1" % (name, s) for s in ["id"] + slot_names)

    # (2) a fresh table with the same slots loads it; every slot agrees key by key
    HashtableRegister().clear()   # as in a new process that restores the checkpoint
    monkeypatch.setenv("RECIS_PACKED_STATE", "1" if packed == "0" else "0")
    ht2 = HashTable([dim], block_size=1024, device="cuda", name=name + "_copy", children=[name])
    SparseAdamW(filter_out_sparse_param(ht2), lr=1e-2)
    dense2 = {"tower.weight": torch.zeros(5, 3, device="cuda"), "step": torch.tensor(0)}
    Loader(path, hashtables={"t": ht2}, tensors=dense2, parallel=parallel).load()
    impl2 = ht2._hashtable_impl
    assert impl.emb_blocks()[0][0].is_contiguous() == (packed == "0")
    assert impl2.emb_blocks()[0][0].is_contiguous() == (packed == "1")
    assert impl2.ids_num() == n
    rows2 = impl2.lookup_index_readonly(ids)
    rows1 = impl.lookup_index_readonly(ids)
    assert int(rows2.min()) >= 0
    for s in slot_names:
        assert torch.equal(impl2.get_slot(s).index_select(rows2), impl.get_slot(s).index_select(rows1)), s
    assert torch.equal(dense2["tower.weight"], dense["tower.weight"]) and int(dense2["step"]) == 3

    # (3) saving the loaded table gives the same tensors (save_load_test.py:205-236)
    path2 = str(tmp_path / "b")
    Saver(0, 1, parallel, path2, hashtables={"t": ht2}, tensors=dense2).save()
    again = _read_all(path2)
    assert set(again) == set(data)
    o1 = torch.argsort(data[name + ".id/part_0_1"])
    o2 = torch.argsort(again[name + ".id/part_0_1"])
    for k in data:
        if "/part_" in k:
            assert torch.equal(data[k][o1], again[k][o2]), k
        else:
            assert torch.equal(data[k], again[k]), k

    # (4) the reader API
    r = CheckpointReader(path)
    assert name + "@embedding" in r.tensor_names() and r.tensor_shape(name + "@embedding") == [n, dim]
    assert r.tensor_dtype(name + "@id") == torch.int64
    assert torch.equal(r.read_tensor(name + "@id"), data[name + ".id/part_0_1"])
    assert _lib.poll_device_errors() == 0


def test_coalesced_engine_round_trip(tmp_path):
    def make():
        opts = {f: EmbeddingOption(embedding_dim=8, shared_name=f, combiner="sum", block_size=256,
                                   initializer=NormalInitializer(0, 0.1), use_weight=False)
                for f in ("user", "item", "shop")}
        eng = EmbeddingEngine(opts)
        eng.train()
        return eng

    def batch(seed):
        g = torch.Generator(device="cuda").manual_seed(seed)
        return {f: RaggedTensor(torch.randint(0, 500, (3000,), device="cuda", generator=g),
                                torch.arange(0, 3001, 3, device="cuda")) for f in ("user", "item", "shop")}

    eng = make()
    out = eng(batch(1))
    tables = {n: t for n, t in eng.hashtables().items()}
    assert len(tables) == 1
    path = str(tmp_path)
    Saver(0, 1, 4, path, hashtables=tables).save()
    names = set(CheckpointReader(path).tensor_names())
    assert {"user@id", "user@embedding", "item@id", "item@embedding", "shop@id", "shop@embedding"} <= names
    saved_ids = CheckpointReader(path).read_tensor("item@id")
    assert int(saved_ids.max()) < 500            # stored without the 12-bit tag

    HashtableRegister().clear()
    eng2 = make()
    Loader(path, hashtables=dict(eng2.hashtables()), parallel=4).load()
    eng2.eval()                                   # read-only lookups: nothing new is admitted
    out2 = eng2(batch(1))
    for f in out:
        assert torch.equal(out[f].detach(), out2[f].detach()), f
    assert _lib.poll_device_errors() == 0


def test_slices_filter_on_load(tmp_path):
    n, dim = 6000, 4
    ht, _, ids = _trained_table("ckpt_s", n, dim)
    impl = ht._hashtable_impl
    path = str(tmp_path)
    Saver(0, 1, 2, path, hashtables={"t": ht}).save()
    halves = []
    for shard in (0, 1):
        HashtableRegister().clear()
        h = HashTable([dim], block_size=1024, device="cuda", name="ckpt_s_half%d" % shard, slice=gen_slice(shard, 2),
                      children=["ckpt_s"])
        SparseAdamW(filter_out_sparse_param(h), lr=1e-2)
        Loader(path, hashtables={"t": h}).load()
        halves.append(h._hashtable_impl)
    s0 = halves[0].slice_info()
    mine = ((ids % 65536) >= s0[0]) & ((ids % 65536) < s0[1])
    assert halves[0].ids_num() + halves[1].ids_num() >= n  # every key lands in exactly one half
    assert sorted(halves[0].ids().cpu().tolist()) == sorted(ids[mine].cpu().tolist())
    assert sorted(halves[1].ids().cpu().tolist()) == sorted(ids[~mine].cpu().tolist())
    for h, m in ((halves[0], mine), (halves[1], ~mine)):
        rows = h.lookup_index_readonly(ids[m])
        src = impl.lookup_index_readonly(ids[m])
        assert torch.equal(h.get_slot("embedding").index_select(rows), impl.get_slot("embedding").index_select(src))
    # a half-range checkpoint pair loads into one full-range table
    path2 = str(tmp_path / "two")
    for shard in (1, 0):
        Saver(shard, 2, 2, path2, hashtables={"t": _Wrap(halves[shard])}).save()
    HashtableRegister().clear()
    full = HashTable([dim], block_size=1024, device="cuda", name="ckpt_s_full", children=["ckpt_s"])
    SparseAdamW(filter_out_sparse_param(full), lr=1e-2)
    Loader(path2, hashtables={"t": full}).load()
    rows = full._hashtable_impl.lookup_index_readonly(ids)
    assert int(rows.min()) >= 0 and full._hashtable_impl.ids_num() == n
    assert torch.equal(full._hashtable_impl.get_slot("embedding").index_select(rows),
                       impl.get_slot("embedding").index_select(impl.lookup_index_readonly(ids)))
    assert _lib.poll_device_errors() == 0


class _Wrap:
    def __init__(self, impl):
        self._hashtable_impl = impl


def test_resume_training_matches_uninterrupted(tmp_path):
    """Train, save tables and optimizer scalars, restore into fresh objects, train on: rows and
    Adam state equal those of the run that was never interrupted, bit for bit (distinct ids per
    step, so the gradient of a row has one term)."""
    n, dim = 3000, 8

    def make(name):
        HashtableRegister().clear()
        ht = HashTable([dim], block_size=512, device="cuda", name=name, children=["resume"],
                       initializer=ConstantInitializer(0.05))   # new keys start alike in both runs
        ht.train()
        return ht, SparseAdamW(filter_out_sparse_param(ht), lr=1e-2, weight_decay=0.01)

    def steps(ht, opt, first, count):
        for s in range(first, first + count):
            g = torch.Generator(device="cuda").manual_seed(100 + s)
            ids = torch.randperm(2 * n, device="cuda", generator=g)[:n]
            (ht(ids) * torch.randn(n, dim, device="cuda", generator=g)).sum().backward()
            opt.step()
            opt.zero_grad()

    torch.manual_seed(0)
    ht, opt = make("resume_a")
    steps(ht, opt, 0, 3)
    path = str(tmp_path)
    Saver(0, 1, 4, path, hashtables={"t": ht}, tensors=opt.state_dict()).save()
    steps(ht, opt, 3, 2)

    ht2, opt2 = make("resume_b")
    # the optimizer's scalars (step, running beta powers) are restored in place, as in the reference:
    # state_dict() hands out the live tensors and the loader copies into them
    Loader(path, hashtables={"t": ht2}, tensors=opt2.state_dict()).load()
    steps(ht2, opt2, 3, 2)

    a, b = ht._hashtable_impl, ht2._hashtable_impl
    ids = a.ids()
    assert sorted(ids.tolist()) == sorted(b.ids().tolist())
    ra, rb = a.lookup_index_readonly(ids), b.lookup_index_readonly(ids)
    for slot in [s.name() for s in a.slot_group().slots()]:
        assert torch.equal(a.get_slot(slot).index_select(ra), b.get_slot(slot).index_select(rb)), slot
    for k, v in opt.state_dict().items():
        assert torch.equal(v, opt2.state_dict()[k]), k

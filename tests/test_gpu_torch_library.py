"""``torch.ops.recis.*`` and ``torch.classes.recis.*`` (recis_amd/lib/recis.so) on the GPU, called with
the argument lists of the reference's own tests (tests/ops/*_test.py, tests/hashtable/*_test.py,
tests/optim/sparse_adamw_test.py) and checked against the CPU oracle. Integer / index / byte results
bit for bit; pooling within rtol 1e-5 / atol 1e-6 on short unit-weight segments (the reference test's
own 1e-6 bar on its own example); the Adam row update (the op) bit for bit."""
import json
import os

import numpy as np
import pytest
import torch

import oracle
from conftest import ragged_offsets
from oracle import cpu_path
from recis_amd import _lib, torch_library

torch_library.load()
R = torch.ops.recis
C = torch.classes.recis

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.to(dtype)
    return t.cuda()


# ------------------------------------------------------------------------------- pooling
def test_segment_reduce_reference_example():
    # tests/ops/emb_segment_reduce_test.py:59-90, through an autograd function as there
    class Reduce(torch.autograd.Function):
        @staticmethod
        def forward(ctx, emb, weight, rev, offsets, mode):
            ctx.mode, ctx.unique_size = mode, emb.size(0)
            ctx.save_for_backward(weight, rev, offsets)
            return R.segment_reduce_forward(emb, weight, rev, offsets, mode)

        @staticmethod
        def backward(ctx, grad):
            weight, rev, offsets = ctx.saved_tensors
            return R.segment_reduce_backward(grad.clone(), weight, rev, offsets, ctx.unique_size, ctx.mode), \
                None, None, None, None

    torch.manual_seed(0)
    emb = torch.randn(6, 64).cuda()
    rev = torch.tensor([0, 1, 2, 0, 1, 2]).cuda()
    offsets = torch.tensor([0, 3, 6]).cuda()
    weight = torch.randn(6).cuda()
    for mode in ("mean", "sum", "tile"):
        w1, w2 = torch.nn.Parameter(emb.clone()), torch.nn.Parameter(emb.clone())
        ret = Reduce.apply(w2, weight, rev, offsets, mode)
        ref = w1[rev] * weight.view(-1, 1)
        if mode == "sum":
            ref = ref.view(-1, 3, 64).sum(dim=1)
        elif mode == "mean":
            ref = ref.view(-1, 3, 64).mean(dim=1)
        torch.testing.assert_close(ret, ref, rtol=1e-6, atol=1e-6)
        ret.sum().backward()
        ref.sum().backward()
        torch.testing.assert_close(w2.grad, w1.grad, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("mode", ["sum", "mean", "tile"])
@pytest.mark.parametrize("weighted", [False, True])
def test_segment_reduce_vs_oracle(rng, mode, weighted):
    U, D, S = 3000, 48, 2000
    off = ragged_offsets(rng, S, 0, 20, empty_frac=0.1)
    B = int(off[-1])
    emb = rng.standard_normal((U, D)).astype(np.float32)
    rev = rng.integers(0, U, size=B)
    w = rng.random(B).astype(np.float32) if weighted else None
    got = R.segment_reduce_forward(_dev(emb), _dev(w) if weighted else None, _dev(rev), _dev(off), mode)
    np.testing.assert_allclose(got.cpu().numpy(), oracle.segment_reduce_forward(emb, w, rev, off, mode),
                               rtol=1e-5, atol=1e-5 if weighted else 1e-6)
    g = rng.standard_normal((B if mode == "tile" else S, D)).astype(np.float32)
    got = R.segment_reduce_backward(_dev(g), _dev(w) if weighted else None, _dev(rev.astype(np.int32)),
                                    _dev(off.astype(np.int32)), U, mode)
    np.testing.assert_allclose(got.cpu().numpy(), oracle.segment_reduce_backward(g, w, rev, off, U, mode),
                               rtol=1e-5, atol=1e-5)
    with pytest.raises(RuntimeError, match="Invalid mode"):
        R.segment_reduce_forward(_dev(emb), None, _dev(rev), _dev(off), "prod")


def test_merge_offsets_gen_indices_segment_ops(rng):
    # tests/ops/emb_segment_reduce_test.py:50-55,94-98
    r = R.merge_offsets([torch.tensor([0, 2, 5]).cuda(), torch.tensor([0, 3, 6]).cuda()], torch.tensor([5, 8]))
    assert r.tolist() == [0, 2, 5, 8, 11]
    assert R.gen_segment_indices_by_offset(torch.tensor([0, 2, 5]).cuda()).tolist() == [0, 0, 1, 1, 1]
    offs = [ragged_offsets(rng, n, 0, 5) for n in (4096, 10, 300)]
    mv = [int(o[-1]) for o in offs]
    r = R.merge_offsets([_dev(o.astype(np.int32)) for o in offs], torch.tensor(mv))
    np.testing.assert_array_equal(r.cpu().numpy(), oracle.merge_offsets(offs, mv))
    # sparse-mode pooling (tests/nn/segment_ops_test.py): weights, then their normalisation
    n, rows, D, S = 5000, 700, 8, 300
    data = rng.standard_normal((rows, D)).astype(np.float32)
    idx = rng.integers(0, rows, size=n)
    seg = np.sort(rng.integers(0, S, size=n))
    w = rng.random(n).astype(np.float32)
    got = R.segment_sum(_dev(data), _dev(w), _dev(idx), _dev(seg), S)
    np.testing.assert_allclose(got.cpu().numpy(), oracle.segment_sum(data, w, idx, seg, S), rtol=1e-5, atol=1e-5)
    got = R.segment_mean(_dev(data), _dev(w), _dev(seg), S)
    np.testing.assert_allclose(got.cpu().numpy(), oracle.segment_mean_weight(w, seg, S), rtol=1e-6, atol=1e-7)


# ------------------------------------------------------------------------------- row blocks
def test_block_ops_reference_constructions():
    # tests/ops/block_ops_test.py:7-70
    bs, dim, nb, n = 10240, 8, 10, 50000
    blocks = [torch.empty((bs, dim), device="cuda").uniform_() for _ in range(nb)]
    flat = torch.cat(blocks)
    index = torch.arange(n, device="cuda")
    assert torch.equal(R.block_gather(index, blocks, bs, -1, False), flat[:n])
    assert torch.equal(R.gather(index, flat), flat[index])
    emb = torch.empty((n, dim), device="cuda").uniform_() * 1000
    R.block_insert(index, emb, blocks, bs)
    assert torch.equal(torch.cat(blocks)[:n], emb)
    # one row broadcast, masked insert, readonly gather of the default key, the stamp filter
    R.block_insert(torch.tensor([5, 7], device="cuda"), torch.full((1, dim), 2.0, device="cuda"), blocks, bs)
    assert float(blocks[0][5].sum()) == 2.0 * dim and float(blocks[0][7].sum()) == 2.0 * dim
    mask = torch.tensor([True, False, True], device="cuda")
    rows = torch.tensor([1, 2, bs + 3], device="cuda")
    before = blocks[0][2].clone()
    R.block_insert_with_mask(rows, torch.ones(3, dim, device="cuda"), mask, blocks, bs)
    assert float(blocks[0][1].sum()) == dim and torch.equal(blocks[0][2], before) and float(blocks[1][3].sum()) == dim
    got = R.block_gather(torch.tensor([-1, 1], device="cuda"), blocks, bs, -1, True)
    assert float(got[0].abs().sum()) == 0 and float(got[1].sum()) == dim
    stamps = [torch.arange(k * 8, (k + 1) * 8, device="cuda").view(8, 1) for k in range(3)]
    got = R.block_filter(torch.tensor([0, 9, 10, 23], device="cuda"), stamps, 8, 10)
    assert got.tolist() == [True, True, False, False] and got.dtype == torch.bool


@pytest.mark.parametrize("beta_dtype", [torch.float32, torch.float64])
def test_block_apply_adamw_bit_exact(rng, beta_dtype):
    # argument list of tests/ops/block_ops_test.py:112-152; the oracle follows block_apply_adamw_op.cc:32-85
    bs, dim, nb, n = 1024, 8, 4, 3000
    mk = lambda: [rng.random((bs, dim)).astype(np.float32) for _ in range(nb)]
    emb, m, v = mk(), mk(), mk()
    d_emb, d_m, d_v = [_dev(b) for b in emb], [_dev(b) for b in m], [_dev(b) for b in v]
    index = rng.permutation(bs * nb)[:n]
    grad = rng.standard_normal((n, dim)).astype(np.float32)
    npdt = np.float32 if beta_dtype == torch.float32 else np.float64
    b1, b2 = np.array([0.99], npdt), np.array([0.9], npdt)
    d_b1, d_b2 = _dev(b1), _dev(b2)
    step = torch.tensor([10], device="cuda")
    for _ in range(3):
        R.block_apply_adamw(_dev(index), _dev(grad), d_emb, d_b1, d_b2, step, d_m, d_v, 0.001, 0.99, 0.9, 0.9, 1e-5, bs)
        oracle.block_apply_adamw(index, grad, emb, b1, b2, m, v, 0.001, 0.99, 0.9, 0.9, 1e-5, bs)
    for got, want in zip(d_emb + d_m + d_v + [d_b1, d_b2], emb + m + v + [b1, b2]):
        np.testing.assert_array_equal(got.cpu().numpy(), want)
    assert step.item() == 10   # left untouched, as in the reference


# ------------------------------------------------------------------------------- allocator ops
def test_allocator_ops_reference_kats():
    # tests/ops/hashtable_ops_test.py:16-86
    free_block = [torch.arange(100000, dtype=torch.int64, device="cuda")]
    ret = R.generate_ids(10000, free_block, 0, 101, free_block[0].numel())
    assert torch.equal(ret, torch.arange(101, 10101, device="cuda").flip([0]))
    ret = R.generate_ids(10000, free_block, 2000, 101, free_block[0].numel())
    assert torch.equal(ret, torch.cat([torch.arange(101, 8101, device="cuda").flip([0]), free_block[0][:2000]]))
    free_ids = torch.arange(101, 10101, device="cuda")
    R.free_ids(free_ids, free_block, 2000, free_block[0].numel())
    ans = torch.arange(100000, dtype=torch.int64, device="cuda")
    ans[2000:12000] = free_ids
    assert torch.equal(free_block[0], ans)
    g = torch.Generator(device="cuda").manual_seed(1)
    keys = torch.randint(0, 1 << 40, (10000,), device="cuda", generator=g)
    mask = torch.rand(10000, device="cuda", generator=g) < 0.2
    cum = torch.cumsum(mask, 0)            # inclusive, as the reference test passes it
    out_size = int(mask.sum())
    out_keys, out_index = R.mask_key_index(keys, mask, cum, out_size)
    assert torch.equal(out_keys, keys[mask]) and torch.equal(out_index, torch.nonzero(mask).view(-1))
    out = torch.zeros(10000, dtype=torch.int64, device="cuda")
    new_rows = torch.arange(out_size, device="cuda") + 7
    ret = R.scatter_ids_with_mask(out, new_rows, out_index)
    want = torch.zeros_like(out)
    want[mask] = new_rows
    assert torch.equal(ret, want) and ret.data_ptr() == out.data_ptr()


# ------------------------------------------------------------------------------- tagging / dedup
def test_ids_encode_and_partition(rng):
    ids = [rng.integers(-2**62, 2**62, size=n, dtype=np.int64) for n in (1000, 7, 50000)]
    tids = [0, 3, 4094]
    got = R.ids_encode([_dev(i) for i in ids], torch.tensor(tids))
    np.testing.assert_array_equal(got.cpu().numpy(), oracle.ids_encode(ids, tids))
    for n, world in ((10, 1), (1000, 128), (100000, 256), (5000, 3)):
        x = rng.integers(-n * 50, n * 50, size=n)
        u, c, inv = R.ids_partition(_dev(x), world)
        eu, ec, einv = oracle.ids_partition(x, world)
        np.testing.assert_array_equal(u.cpu().numpy(), eu)
        np.testing.assert_array_equal(c.cpu().numpy(), ec)
        np.testing.assert_array_equal(inv.cpu().numpy(), einv)
        assert inv.dtype == torch.int32 and c.dtype == torch.int64


# ------------------------------------------------------------------------------- feature ops
def test_feature_ops_kats_and_oracle(rng):
    # tests/ops/fused_hash_test.py:20-21,37-38
    a = torch.tensor([0, 1, 2, 1, 2, 3], dtype=torch.int8).cuda()
    b = torch.tensor([0, 5, 5, 5, 6, 7], dtype=torch.int8).cuda()
    off = [torch.tensor([0, 3, 6], dtype=torch.int32).cuda()] * 2
    farm, mur = R.fused_hash([a, b], off, "farm"), R.fused_hash([a, b], off, "murmur")
    assert farm[0].tolist() == [-7736835464683084646, -5546720800891377920]
    assert farm[1].tolist() == [-4442022684725028445, -909183002746659612]
    assert mur[0].tolist() == [-4003751876240412087, -1042754718167355375]
    assert mur[1].tolist() == [-5541886947548579749, 4434088491466393040]
    with open(os.path.join(GOLDEN, "hash_vectors.json")) as f:
        vec = json.load(f)["vectors"]
    data = np.frombuffer(b"".join(bytes.fromhex(v["hex"]) for v in vec), dtype=np.uint8)
    offs = np.concatenate([[0], np.cumsum([len(v["hex"]) // 2 for v in vec])])
    assert R.fused_hash([_dev(data.view(np.int8))], [_dev(offs)], "farm")[0].tolist() == [v["farm"] for v in vec]
    assert R.fused_hash([_dev(data.view(np.int8))], [_dev(offs)], "murmur")[0].tolist() == [v["murmur"] for v in vec]
    with pytest.raises(RuntimeError, match="Unsupported hash type"):
        R.fused_hash([a], off[:1], "sha1")
    # tests/feature_engine/op_test.py:17-24 and random inputs
    assert R.uint64_mod(torch.tensor([1001, 1002, 1003], device="cuda"), 1000).tolist() == [1, 2, 3]
    xs = [rng.integers(-2**63, 2**63 - 1, size=n, dtype=np.int64) for n in (1000, 1, 65536)]
    mods = [1000000, 7, 2**40 + 3]
    for g, x, m in zip(R.fused_uint64_mod([_dev(x) for x in xs], torch.tensor(mods)), xs, mods):
        np.testing.assert_array_equal(g.cpu().numpy(), oracle.uint64_mod(x, m))
    bs = [np.sort(rng.standard_normal(n)).astype(np.float32) for n in (64, 5)]
    vs = [(rng.standard_normal(n) * 2).astype(np.float32) for n in (65536, 10)]
    vs[1][:5] = [np.nan, np.inf, -np.inf, bs[1][0], bs[1][-1]]
    got = R.fused_bucketized([_dev(v) for v in vs], [_dev(b) for b in bs])
    for g, v, b in zip(got, vs, bs):
        np.testing.assert_array_equal(g.cpu().numpy(), oracle.bucketize(v, b))
    assert got[0].untyped_storage().data_ptr() == got[1].untyped_storage().data_ptr()
    v = torch.randn(100, device="cuda") * 3
    bd = torch.tensor([1.0, 2, 3, 4, 5], device="cuda")
    assert torch.equal(R.bucketize_op(v, bd), torch.bucketize(v, bd, right=True))
    # tests/feature_engine/op_test.py:95-110
    x2 = torch.tensor([1001, 1002, 1003], device="cuda")
    muls, primes, buckets = torch.tensor([1, 3, 5, 7]), torch.tensor([28979, 46997, 66973, 82997]), torch.tensor([1000] * 4)
    got = R.fused_multi_hash([x2], [muls], [primes], [buckets])
    assert [g.tolist() for g in got] == [[1, 2, 3], [3, 6, 9], [5, 10, 15], [7, 14, 21]]
    x1 = rng.integers(-2**63, 2**63 - 1, size=5000, dtype=np.int64)
    for g, e in zip(R.fused_multi_hash([_dev(x1)], [muls], [primes], [buckets]),
                    oracle.multi_hash(x1, muls.tolist(), primes.tolist(), buckets.tolist())):
        np.testing.assert_array_equal(g.cpu().numpy(), e)


# ------------------------------------------------------------------------------- padded gather
def test_ragged_tile_forward_and_back(rng):
    # the numpy model of tests/nn/test_ragged_tile.py:72-120 is the oracle's
    batch, seq, D, rows = [40, 25, 33], [5, 3, 8], 16, 500
    offs = [ragged_offsets(rng, b, 0, 10) for b in batch]
    value = rng.integers(0, rows, size=sum(int(o[-1]) for o in offs))
    merged = oracle.merge_offsets(offs, [int(o[-1]) for o in offs])
    table = rng.standard_normal((rows, D)).astype(np.float32)
    out, batch_seq = R.ragged_tile(batch, seq, _dev(value), _dev(merged), _dev(table))
    np.testing.assert_array_equal(out.cpu().numpy(), oracle.ragged_tile(batch, seq, value, merged, table))
    dy = rng.standard_normal(tuple(out.shape)).astype(np.float32)
    got = R.ragged_tile_back(batch_seq, [rows, len(batch), max(batch), min(seq)], _dev(value), _dev(merged), _dev(dy))
    np.testing.assert_allclose(got.cpu().numpy(), oracle.ragged_tile_back(batch, seq, value, merged, dy, rows),
                               rtol=1e-5, atol=1e-5)


# ------------------------------------------------------------------------------- sequence ops
def test_sequence_ops_vs_oracle(rng):
    # fused_ragged_cutoff 2-D / 3-D (tests/ops/fused_ragged_cutoff_{2D,3D}_test.py argument lists)
    vals, offs, keep, drop, pad = [], [], [3, 7, 1], [True, False, True], [False, True, False]
    for t in range(3):
        o = ragged_offsets(rng, 50 + t, 0, 12)
        offs.append(o.astype(np.int32))
        vals.append(rng.integers(0, 1000, size=int(o[-1])))
    out = R.fused_ragged_cutoff([_dev(v) for v in vals], [_dev(o) for o in offs], torch.tensor(keep),
                                torch.tensor(drop), torch.tensor(pad))
    for t in range(3):
        ev, eo, ed, ep = oracle.ragged_cutoff_2d(vals[t], offs[t], keep[t], drop[t])
        np.testing.assert_array_equal(out[0][t].cpu().numpy(), ev)
        np.testing.assert_array_equal(out[1][t].cpu().numpy(), eo)
        np.testing.assert_array_equal(out[2][t].cpu().numpy(), ed)
        np.testing.assert_array_equal(out[3][t].cpu().numpy(), ep)
    outer = ragged_offsets(rng, 20, 0, 6)
    inner = ragged_offsets(rng, int(outer[-1]), 0, 5)
    v3 = rng.integers(0, 1000, size=int(inner[-1]))
    o3 = R.fused_ragged_cutoff_3D([_dev(v3)], [_dev(outer)], [_dev(inner)], torch.tensor([4]), torch.tensor([True]),
                                  torch.tensor([False]))
    ev, eouter, einner = oracle.ragged_cutoff_3d(v3, outer, inner, 4, True, False)[:3]
    np.testing.assert_array_equal(o3[0][0].cpu().numpy(), ev)
    np.testing.assert_array_equal(o3[1][0].cpu().numpy(), eouter)
    np.testing.assert_array_equal(o3[2][0].cpu().numpy(), einner)
    # ragged_to_dense / dense_to_ragged (tests/ops/ragged_to_dense_test.py, dense_to_ragged_test.py)
    o = ragged_offsets(rng, 64, 0, 9)
    v = rng.integers(1, 100, size=int(o[-1]))
    dense = R.ragged_to_dense(_dev(v), [_dev(o)], -1)
    np.testing.assert_array_equal(dense.cpu().numpy(), oracle.ragged_to_dense(v, [o], -1))
    gv, go = R.dense_to_ragged(dense, True, torch.tensor([-1]))
    ev, eo = oracle.dense_to_ragged(dense.cpu().numpy(), -1)
    np.testing.assert_array_equal(gv.cpu().numpy(), ev)
    np.testing.assert_array_equal(go.cpu().numpy(), eo)


def test_feature_cross_and_topk_index(rng):
    # tests/feature_engine/op_test.py:39-63 fixes the hash; rows compared as the oracle orders them
    xo, yo = ragged_offsets(rng, 100, 0, 6), ragged_offsets(rng, 100, 0, 4)
    xv, yv = rng.integers(0, 20, size=int(xo[-1])), rng.integers(0, 20, size=int(yo[-1]))
    xw, yw = rng.random(len(xv)).astype(np.float32), rng.random(len(yv)).astype(np.float32)
    val, off, w = R.feature_cross_ragged(_dev(xv), _dev(xo), _dev(xw), _dev(yv), _dev(yo), _dev(yw))
    ev, eo, ew = oracle.feature_cross_ragged(xv, xo, xw, yv, yo, yw)
    np.testing.assert_array_equal(val.cpu().numpy(), ev)
    np.testing.assert_array_equal(off.cpu().numpy(), eo)
    np.testing.assert_array_equal(w.cpu().numpy(), ew)
    # tests/ops/ragged_topk_index_cutoff_test.py:9-22 argument order
    offset = ragged_offsets(rng, 30, 0, 10)
    drop_num = rng.integers(0, 3, size=30)
    topk = rng.integers(0, 8, size=(40, 5))
    indicator = rng.integers(0, 30, size=40)
    gi, go = R.calc_ragged_index(_dev(drop_num), _dev(np.zeros(30, np.int64)), torch.tensor([True]),
                                 torch.tensor([False]), _dev(offset), _dev(topk), _dev(indicator))
    ei, eo = oracle.calc_ragged_index(drop_num, offset, topk, indicator)
    np.testing.assert_array_equal(gi.cpu().numpy(), ei)
    np.testing.assert_array_equal(go.cpu().numpy(), eo)


# ------------------------------------------------------------------------------- custom classes
def _make_table(block_size, dim, gen=None, children=("t",), coalesce=False, dtype=torch.float32):
    if gen is None:
        gen = C.Generator.make_constant_generator([block_size, dim], dtype, 0.0)
    return R.make_hashtable(block_size, [dim], dtype, torch.device("cuda"), coalesce, list(children), gen,
                            0, 65536, 65536)


def test_hashtable_lookup_insert_readonly():
    # the flow of tests/hashtable/ht_lookup_test.py:16-112 on the class the module wraps
    ht = _make_table(1024, 128)
    assert ht.hashtable_tag == -1
    ids = torch.arange(2048, device="cuda")
    index, emb = ht.embedding_lookup(ids, False)
    assert emb.shape == (2048, 128) and float(emb.abs().sum()) == 0
    assert torch.equal(index, torch.arange(2047, -1, -1, device="cuda"))   # sparse_adamw_test.py:177-208
    ids2 = torch.arange(2048, 4096, device="cuda")
    vals = torch.tile(ids2.reshape(-1, 1), [1, 128]).float()
    ht.insert(ids2, vals)
    assert torch.equal(ht.embedding_lookup(ids2, False)[1], vals)
    index, emb = ht.embedding_lookup(torch.arange(4000, 4200, device="cuda"), True)   # read-only: nothing admitted
    assert torch.equal(emb[:96], vals[4000 - 2048:]) and float(emb[96:].abs().sum()) == 0
    assert bool((index[96:] == -1).all())
    assert torch.equal(torch.sort(ht.ids())[0], torch.arange(4096, device="cuda"))
    keys, rows = ht.ids_map()
    assert torch.equal(torch.sort(rows)[0], torch.arange(4096, device="cuda"))
    with pytest.raises(RuntimeError, match="dismatch"):
        ht.insert(ids2[:3], vals[:2])
    ht.clear()
    assert ht.ids().numel() == 0
    assert _lib.poll_device_errors() == 0


def test_hashtable_slots_children_and_delete():
    # tests/hashtable/ht_slot_test.py; block_num = (id_num + bs) / bs (hashtable.cc:255-261)
    gen = C.Generator.make_constant_generator([10, 4], torch.float32, 1.0)
    ht = _make_table(10, 4, gen, children=("a", "b"), coalesce=True)
    ci = ht.children_info()
    assert ci.is_coalesce() and ci.children() == ["a", "b"] and ci.child_index("b") == 1 and ci.has_child("a")
    assert ci.index_bits_num() == 12 and ci.id_bits_num() == 52 and ci.max_children_num() == 4095
    assert ci.encode_id(5, 3) == (3 << 52) | 5 and ci.id_mask() == (1 << 52) - 1 and ci.child_at(0) == "a"
    ht.embedding_lookup(torch.arange(25, device="cuda"), False)
    slot = ht.slot_group().slot_by_name("embedding")
    assert slot.name() == "embedding" and slot.block_size() == 10 and slot.flat_size() == 4
    assert len(slot.values()) == 3 and slot.value().shape == (30, 4) and float(slot.value().sum()) == 120
    slot.values()[0][0].fill_(9.0)                       # values() alias live storage
    assert float(ht.get_slot("embedding").value()[0].sum()) == 36.0
    # a step-filter slot, stamped through update_slot, filtered and deleted as the filter hook does
    # (recis/nn/modules/hashtable_hook_impl.py:487-551)
    ht.append_step_filter_slot("step_filter", 0)
    ids = torch.arange(25, device="cuda")
    index, _ = ht.embedding_lookup(ids, False)
    ht.update_slot("step_filter", index[:10], torch.full((10,), 7, dtype=torch.int64, device="cuda"))
    stamp = ht.get_slot("step_filter")
    keys, rows = ht.ids_map()
    old = R.block_filter(rows, stamp.values(), stamp.block_size(), 5)
    assert int(old.sum()) == 15
    ht.delete(keys[old], rows[old], "step_filter")
    assert torch.equal(torch.sort(ht.ids())[0], ids[:10])
    assert float(ht.embedding_lookup(ids[10:12], True)[1].abs().sum()) == 0   # gone
    new_index, emb = ht.embedding_lookup(torch.arange(100, 115, device="cuda"), False)
    assert set(new_index.tolist()) == set(rows[old].tolist())                 # freed rows are reused
    assert bool((emb == 1.0).all())                                           # and were re-initialised


def test_hashtable_grad_kat():
    # tests/hashtable/ht_grad_ga_test.py:9-33
    ht = _make_table(8, 4)
    ht.accept_grad(torch.tensor([1, 2, 3], device="cuda"), torch.ones(3, 4, device="cuda"))
    ht.accept_grad(torch.tensor([1, 1, 1], device="cuda"), torch.ones(3, 4, device="cuda") * 2)
    ht.accept_grad(torch.tensor([2, 2, 2], device="cuda"), torch.ones(3, 4, device="cuda") * 3)
    ga = ht.grad(3).coalesce()
    assert ga.indices().cpu().tolist() == [[0, 1, 2]]
    torch.testing.assert_close(ga.values().cpu(), torch.tensor([[7.0] * 4, [10.0] * 4, [1.0] * 4]) / 3.0)
    ht.clear_grad()
    ht.accept_grad(torch.tensor([4, 2], device="cuda"), torch.ones(2, 4, device="cuda"))
    g = ht.grad(1)
    assert g.is_sparse and g.shape == (5, 4) and g._indices().tolist() == [[4, 2]]
    with pytest.raises(RuntimeError):
        ht.accept_grad(torch.tensor([1], dtype=torch.int32, device="cuda"), torch.ones(1, 4, device="cuda"))


@pytest.mark.parametrize("cls,prefix,decay,beta_dtype", [
    ("SparseAdam", "sparse_adam_", lambda lr, wd: 1.0, np.float64),
    ("SparseAdamW", "sparse_adamw_", lambda lr, wd: 1.0 - lr * wd, np.float32),
    ("SparseAdamWTF", "sparse_adamw_tf_", lambda lr, wd: 1.0 - wd, np.float32)])
def test_sparse_optimizers_against_cpu_path(rng, cls, prefix, decay, beta_dtype):
    """The training loop of recis/nn/modules/hashtable.py:262-293 + recis/optim/sparse_optim.py on the
    registered classes: unique ids -> embedding_lookup -> pooling ops -> accept_grad -> step, against
    the CPU restatement of the same loop: row indices, the key -> row map and the running beta powers bit
    for bit, rows and both moments to rounding (the backward sums duplicates with fp32 atomics, in another
    order than the CPU loop)."""
    dim, bs, lr, wd = 16, 64, 1e-2, 1e-2
    cpu = cpu_path.CpuTable(dim, bs, lambda b: np.zeros((bs, dim), np.float32), "adam", lr, 1e-8, 0.9, 0.999,
                            decay(lr, wd), beta_dtype)
    ht = _make_table(bs, dim)
    opt = getattr(C, cls).make({"t": ht}, lr, 0.9, 0.999, 1e-8, wd, False)
    for step in range(6):
        ids = rng.integers(0, 150 + 30 * step, size=400)
        off = np.arange(0, 401, 4)
        grad = rng.standard_normal((100, dim)).astype(np.float32)
        pooled_c, uniq_c, index_c = cpu_path.train_step(cpu, ids, off, None, grad)
        uniq, inverse = torch.unique(_dev(ids), return_inverse=True)
        index, rows = ht.embedding_lookup(uniq, False)
        np.testing.assert_array_equal(index.cpu().numpy(), index_c)
        pooled = R.segment_reduce_forward(rows, None, inverse, _dev(off), "sum")
        np.testing.assert_allclose(pooled.cpu().numpy(), pooled_c, rtol=1e-5, atol=1e-6)
        g_unique = R.segment_reduce_backward(_dev(grad), None, inverse, _dev(off), uniq.numel(), "sum")
        ht.accept_grad(index, g_unique)
        opt.step()
        opt.zero_grad()
    sg = ht.slot_group()
    assert [s.name() for s in sg.slots()] == ["embedding", prefix + "exp_avg", prefix + "exp_avg_sq"]
    n_blocks = len(cpu.emb)
    for name, want in (("embedding", cpu.emb), (prefix + "exp_avg", cpu.s0), (prefix + "exp_avg_sq", cpu.s1)):
        blocks = sg.slot_by_name(name).values()
        assert len(blocks) == n_blocks
        for got, w in zip(blocks, want):
            np.testing.assert_allclose(got.cpu().numpy(), w, rtol=2e-5, atol=1e-6)
    keys, rows = ht.ids_map()
    ck, cr = cpu.idmap.snapshot()
    assert dict(zip(keys.tolist(), rows.tolist())) == dict(zip(ck.tolist(), cr.tolist()))
    tables_out, steps = opt.state_dict()
    assert set(steps) == {prefix + "step", prefix + "beta1", prefix + "beta2"} and len(tables_out) == 0
    np.testing.assert_array_equal(steps[prefix + "beta1"].cpu().numpy().reshape(-1), cpu.b1t)
    np.testing.assert_array_equal(steps[prefix + "beta2"].cpu().numpy().reshape(-1), cpu.b2t)
    opt.set_lr(0.5)
    opt.set_grad_accum_steps(2)
    opt.load_state_dict({}, {})
    assert _lib.poll_device_errors() == 0


def test_initialiser_rows_on_device():
    """Rows of a new table come from the Generator, drawn on the table's device when storage is made."""
    gen = C.Generator.make_uniform_generator([32, 8], torch.float32, -0.5, 0.5, None)
    ht = _make_table(32, 8, gen)
    _, emb = ht.embedding_lookup(torch.arange(100, device="cuda"), False)
    assert emb.is_cuda and float(emb.min()) >= -0.5 and float(emb.max()) <= 0.5 and float(emb.std()) > 0.2


def test_config4_shaped_step_through_the_library_boundary():
    """A config-4-shaped step (26 id columns + 13 bucketized float columns on one coalesced table, dim 16,
    sum pooling of one id per sample, SparseAdam) three ways against the CPU restatement of the reference's
    step: (a) the reference's own call sequence operator by operator (fused_bucketized -> fused_uint64_mod ->
    ids_encode -> ids_partition -> embedding_lookup -> segment_reduce_forward -> segment_reduce_backward ->
    accept_grad -> step), (b) the fused calls behind the same classes (dense_lookup_expand ->
    accept_split_grad -> step: one plan, gradient summed where the rows are updated). Each side orders new
    keys its own way (the CPU path by np.unique, ids_partition by shard, the plan by hash bucket), so rows start
    from one constant and are compared by key; pooled outputs sample by sample; fp32 within rtol 1e-5 /
    atol 1e-6."""
    import workloads

    batch, dim, bs, lr = 2048, 16, 1024, 1e-3
    n_feat = 39
    # every row starts at the same value: the three sides hand new keys their rows in different orders
    cpu = cpu_path.CpuTable(dim, bs, lambda b: np.full((bs, dim), 0.05, np.float32), "adam", lr, 1e-8)

    def table():
        gen = C.Generator.make_constant_generator([bs, dim], torch.float32, 0.05)
        ht = _make_table(bs, dim, gen, ["f%d" % i for i in range(n_feat)], True)
        return ht, C.SparseAdam.make({"ctr": ht}, lr, 0.9, 0.999, 1e-8, 0.0, False)

    (ht_a, opt_a), (ht_b, opt_b) = table(), table()
    tags = list(range(n_feat))
    offsets = torch.arange(batch * n_feat + 1, dtype=torch.int32, device="cuda")
    rng = np.random.default_rng(44)
    for step in range(4):
        c = workloads.config4(batch=batch, data_seed=step)
        grad = rng.standard_normal((batch * n_feat, dim)).astype(np.float32)
        extra_c = [oracle.uint64_mod(oracle.bucketize(d.cpu().numpy(), c["boundaries"][0].cpu().numpy()), c["mod"])
                   for d in c["dense"]]
        ids_c = oracle.ids_encode([t.cpu().numpy() for t in c["sparse"]] + extra_c, tags)
        pooled_c, uniq_c, index_c = cpu_path.train_step(cpu, ids_c, np.arange(ids_c.size + 1), None, grad)
        # (a) the reference's sequence
        extra = R.fused_uint64_mod(R.fused_bucketized(c["dense"], c["boundaries"]),
                                   torch.full((len(c["dense"]),), c["mod"], dtype=torch.int64))
        ids = R.ids_encode(c["sparse"] + extra, torch.tensor(tags))
        np.testing.assert_array_equal(ids.cpu().numpy(), ids_c)
        uniq, counts, inverse = R.ids_partition(ids, 1)
        assert counts.tolist() == [uniq.numel()] and torch.equal(uniq[inverse.long()], ids)
        index, emb = ht_a.embedding_lookup(uniq, False)
        pooled = R.segment_reduce_forward(emb, None, inverse, offsets, "sum")
        np.testing.assert_allclose(pooled.cpu().numpy(), pooled_c, rtol=1e-5, atol=1e-6)
        g_unique = R.segment_reduce_backward(_dev(grad), None, inverse, offsets, uniq.numel(), "sum")
        exp_g = oracle.segment_reduce_backward(grad, None, inverse.cpu().numpy().astype(np.int64),
                                               np.arange(ids_c.size + 1), uniq.numel(), "sum")
        np.testing.assert_allclose(g_unique.cpu().numpy(), exp_g, rtol=1e-5, atol=1e-5)
        ht_a.accept_grad(index, g_unique)
        assert ht_a.pending_grads() == [0, 1]
        opt_a.step()
        opt_a.zero_grad()
        # (b) the fused calls: one plan, nothing waits for the unique count, the gradient stays unsummed
        cols = c["sparse"] + R.fused_bucketized_mod(c["dense"], c["boundaries"], [c["mod"]] * len(c["dense"]))
        plan, index_b, out = ht_b.dense_lookup_expand(cols, tags, None, None)
        np.testing.assert_allclose(out.cpu().numpy(), pooled_c, rtol=1e-5, atol=1e-6)
        g = _dev(grad)
        ht_b.accept_split_grad(index_b, plan, list(g.split(batch)), [batch] * n_feat, None, None, plan.serial, False, True)
        assert ht_b.pending_grads() == [1, 0]
        opt_b.step()
        opt_b.zero_grad()
        assert ht_b.pending_grads() == [0, 0]
    keys_c, rows_c = cpu.idmap.snapshot()
    order = np.argsort(keys_c)
    keys_c, rows_c = keys_c[order], rows_c[order]
    want = [np.concatenate(blocks)[rows_c] for blocks in (cpu.emb, cpu.s0, cpu.s1)]
    for ht in (ht_a, ht_b):
        keys, rows = ht.ids_map()
        keys, at = torch.sort(keys)
        np.testing.assert_array_equal(keys.cpu().numpy(), keys_c)
        rows = rows[at]
        assert torch.unique(rows).numel() == rows.numel() and ht.ids_num() == cpu.idmap.id_num()
        for name, exp in zip(("embedding", "sparse_adam_exp_avg", "sparse_adam_exp_avg_sq"), want):
            got = ht.get_slot(name).index_select(rows).cpu().numpy()
            np.testing.assert_allclose(got, exp, rtol=1e-5, atol=1e-6, err_msg=name)
    assert _lib.poll_device_errors() == 0


def test_slot_handle_taken_before_an_insert_sees_the_new_blocks():
    """Slot.values() aliases the live storage: a handle (the optimizer's state slots, a saver's) that was taken
    before later lookups added blocks lists those blocks too (block_num = (id_num + block_size) / block_size,
    csrc/embedding/hashtable.cc:255-261)."""
    ht = _make_table(16, 4)
    emb = ht.slot_group().slot_by_name("embedding")        # taken while the table is empty
    assert len(emb.values()) == 0
    ht.embedding_lookup(torch.arange(10, device="cuda"), False)
    assert len(emb.values()) == 1 and emb.value().shape == (16, 4)
    ht.embedding_lookup(torch.arange(100, 150, device="cuda"), False)   # 60 ids: (60 + 16) / 16 = 4 blocks
    blocks = emb.values()
    assert len(blocks) == 4 and all(b.shape == (16, 4) for b in blocks)
    blocks[3].fill_(2.5)                                                 # a view, not a copy
    assert float(ht.get_slot("embedding").value()[48:].min()) == 2.5
    assert _lib.poll_device_errors() == 0

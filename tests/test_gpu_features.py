"""Parity of the HIP tagging / dedup / feature ops / padded gather (through the
C ABI) with the CPU oracle and the golden vectors: everything here is integer or
byte work and is compared bit for bit (ragged_tile copies rows: exact too; its
backward sums in fp32: rtol 1e-5)."""
import json
import os

import numpy as np
import pytest
import torch

import oracle
from conftest import ragged_offsets
from recis_amd import _lib, ops

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.to(dtype)
    return t.cuda()


def test_hash_kats_and_golden():
    a = torch.tensor([0, 1, 2, 1, 2, 3], dtype=torch.int8).cuda()
    b = torch.tensor([0, 5, 5, 5, 6, 7], dtype=torch.int8).cuda()
    off = [torch.tensor([0, 3, 6], dtype=torch.int32).cuda()] * 2
    farm = ops.fused_hash([a, b], off, "farm")
    mur = ops.fused_hash([a, b], off, "murmur")
    assert farm[0].tolist() == [-7736835464683084646, -5546720800891377920]
    assert farm[1].tolist() == [-4442022684725028445, -909183002746659612]
    assert mur[0].tolist() == [-4003751876240412087, -1042754718167355375]
    assert mur[1].tolist() == [-5541886947548579749, 4434088491466393040]
    with open(os.path.join(GOLDEN, "hash_vectors.json")) as f:
        vec = json.load(f)["vectors"]
    data = np.frombuffer(b"".join(bytes.fromhex(v["hex"]) for v in vec), dtype=np.uint8)
    offs = np.concatenate([[0], np.cumsum([len(v["hex"]) // 2 for v in vec])])
    got = ops.fused_hash([_dev(data.view(np.int8))], [_dev(offs)], "farm")[0]
    assert got.tolist() == [v["farm"] for v in vec]
    got = ops.fused_hash([_dev(data.view(np.int8))], [_dev(offs)], "murmur")[0]
    assert got.tolist() == [v["murmur"] for v in vec]
    with pytest.raises(RuntimeError):
        ops.fused_hash([a], off[:1], "sha1")


def test_hash_random_strings_vs_oracle(rng):
    vals, offs = [], []
    for t in range(5):
        lens = rng.integers(0, 200, size=int(rng.integers(1, 3000)))
        vals.append(rng.integers(-128, 128, size=int(lens.sum()), dtype=np.int8))
        offs.append(np.concatenate([[0], np.cumsum(lens)]).astype(np.int32))
    for kind in ("farm", "murmur"):
        got = ops.fused_hash([_dev(v) for v in vals], [_dev(o) for o in offs], kind)
        for g, v, o in zip(got, vals, offs):
            np.testing.assert_array_equal(g.cpu().numpy(), oracle.hash_strings(v, o, kind))


def test_uint64_mod(rng):
    xs = [rng.integers(-2**63, 2**63 - 1, size=n, dtype=np.int64) for n in (1000, 1, 65536)]
    mods = [1000000, 7, 2**40 + 3]
    got = ops.fused_uint64_mod([_dev(x) for x in xs], mods)
    for g, x, m in zip(got, xs, mods):
        np.testing.assert_array_equal(g.cpu().numpy(), oracle.uint64_mod(x, m))
    assert ops.uint64_mod(torch.tensor([1001, 1002, 1003], device="cuda"), 1000).tolist() == [1, 2, 3]


def test_bucketize(rng):
    bs = [np.sort(rng.standard_normal(n)).astype(np.float32) for n in (64, 5, 9000)]
    vs = [(rng.standard_normal(n) * 2).astype(np.float32) for n in (65536, 10, 3000)]
    vs[0][:64] = bs[0]
    vs[1][:5] = [np.nan, np.inf, -np.inf, bs[1][0], bs[1][-1]]
    got = ops.fused_bucketized([_dev(v) for v in vs], [_dev(b) for b in bs])
    for g, v, b in zip(got, vs, bs):
        np.testing.assert_array_equal(g.cpu().numpy(), oracle.bucketize(v, b))
    # the fused outputs are views of one buffer (fused_bucketized.cc:47-52)
    assert got[0].untyped_storage().data_ptr() == got[1].untyped_storage().data_ptr()
    v = torch.randn(100, device="cuda") * 3
    b = torch.tensor([1.0, 2, 3, 4, 5], device="cuda")
    assert torch.equal(ops.bucketize_op(v, b), torch.bucketize(v, b, right=True))
    # bucketize followed by mod in one pass: the oracle's two functions one after the other
    mods = [7, 100, 1]
    both = ops.fused_bucketized([_dev(v) for v in vs], [_dev(b) for b in bs], mods=mods)
    for g, v, b, m in zip(both, vs, bs, mods):
        np.testing.assert_array_equal(g.cpu().numpy(), oracle.uint64_mod(oracle.bucketize(v, b), m))
    with pytest.raises(_lib.RecisHipError):
        ops.fused_bucketized([_dev(vs[0])], [_dev(bs[0])], mods=[0])


def test_multi_hash(rng):
    x1 = rng.integers(-2**63, 2**63 - 1, size=5000, dtype=np.int64)
    x2 = np.array([1001, 1002, 1003], np.int64)
    muls, primes, buckets = [1, 3, 5, 7], [28979, 46997, 66973, 82997], [1000] * 4
    got = ops.fused_multi_hash([_dev(x1), _dev(x2)], [muls, muls], [primes, primes], [buckets, buckets])
    exp = oracle.multi_hash(x1, muls, primes, buckets) + oracle.multi_hash(x2, muls, primes, buckets)
    assert len(got) == 8
    for g, e in zip(got, exp):
        np.testing.assert_array_equal(g.cpu().numpy(), e)
    assert [g.tolist() for g in got[4:]] == [[1, 2, 3], [3, 6, 9], [5, 10, 15], [7, 14, 21]]


def test_ids_encode_and_merge_offsets(rng):
    ids = [rng.integers(-2**62, 2**62, size=n, dtype=np.int64) for n in (1000, 10000, 7, 100000)]
    tids = [0, 1, 2, 4094]
    got = ops.ids_encode([_dev(i) for i in ids], torch.tensor(tids))
    np.testing.assert_array_equal(got.cpu().numpy(), oracle.ids_encode(ids, tids))
    # tests/ops/emb_segment_reduce_test.py:50-55
    r = ops.merge_offsets([torch.tensor([0, 2, 5]).cuda(), torch.tensor([0, 3, 6]).cuda()], torch.tensor([5, 8]))
    assert r.tolist() == [0, 2, 5, 8, 11]
    offs = [ragged_offsets(rng, n, 0, 5) for n in (65536, 10, 300)]
    mv = [int(o[-1]) for o in offs]
    for dt in (np.int32, np.int64):
        r = ops.merge_offsets([_dev(o.astype(dt)) for o in offs], mv)
        np.testing.assert_array_equal(r.cpu().numpy(), oracle.merge_offsets(offs, mv))
    # more tensors than one launch carries
    many = [np.array([0, 1, 3]) for _ in range(130)]
    r = ops.merge_offsets([_dev(o) for o in many], [3] * 130)
    np.testing.assert_array_equal(r.cpu().numpy(), oracle.merge_offsets(many, [3] * 130))


@pytest.mark.parametrize("n,hi", [(0, 10), (1, 10), (1000, 50), (200000, 3000), (1000000, 10**7)])
def test_unique_first_occurrence_order(rng, n, hi):
    ids = rng.integers(-hi, hi, size=n)
    if n > 5:
        ids[3] = -1  # the empty-marker value is a legal id here
    uniq, inv, count = ops.ids_unique(_dev(ids))
    c = int(count.item())
    u = uniq[:c].cpu().numpy()
    # first-occurrence order == np.unique's first indices, sorted
    _, first = np.unique(ids, return_index=True)
    np.testing.assert_array_equal(u, ids[np.sort(first)])
    np.testing.assert_array_equal(u[inv.cpu().numpy()], ids)
    uniq64, inv64, _ = ops.ids_unique(_dev(ids), inverse_dtype=torch.int64)
    assert torch.equal(inv64, inv.long())


@pytest.mark.parametrize("n,world", [(10, 1), (1000, 128), (100000, 256), (5000, 3)])
def test_ids_partition_matches_oracle(rng, n, world):
    ids = rng.integers(-n * 50, n * 50, size=n)
    u, c, inv = ops.ids_partition(_dev(ids), world)
    eu, ec, einv = oracle.ids_partition(ids, world)
    np.testing.assert_array_equal(u.cpu().numpy(), eu)
    np.testing.assert_array_equal(c.cpu().numpy(), ec)
    np.testing.assert_array_equal(inv.cpu().numpy(), einv)
    assert inv.dtype == torch.int32


@pytest.mark.parametrize("n", [0, 1, 255, 70000, 3000000])
def test_partition_order_is_the_unsigned_sort_of_the_rotated_ids(rng, n):
    # ids_partition_kernel.cu:36-43: ascending by rotr64(id, 16) compared as unsigned
    ids = rng.integers(-(1 << 62), 1 << 62, size=n)
    if n > 100:  # the extremes of the key, and neighbours that differ in the rotated-out bits only
        ids = np.concatenate([ids, [-(1 << 63), (1 << 63) - 1, -1, 0, 65535, 65536], ids[:50] ^ 1, ids[:50] ^ (1 << 15)])
    ids = np.unique(ids)
    rng.shuffle(ids)
    s, order, rank = ops.partition_order(_dev(ids))
    key = (ids.view(np.uint64) >> np.uint64(16)) | (ids.view(np.uint64) << np.uint64(48))
    eorder = np.argsort(key, kind="stable")
    np.testing.assert_array_equal(order.cpu().numpy(), eorder)
    np.testing.assert_array_equal(s.cpu().numpy(), ids[eorder])
    erank = np.empty(ids.size, np.int32)
    erank[eorder] = np.arange(ids.size, dtype=np.int32)
    np.testing.assert_array_equal(rank.cpu().numpy(), erank)
    assert order.dtype == torch.int32 and rank.dtype == torch.int32


def _check_partition_order(ids):
    s, order, rank = ops.partition_order(_dev(ids))
    key = (ids.view(np.uint64) >> np.uint64(16)) | (ids.view(np.uint64) << np.uint64(48))
    eorder = np.argsort(key, kind="stable")
    np.testing.assert_array_equal(order.cpu().numpy(), eorder)
    np.testing.assert_array_equal(s.cpu().numpy(), ids[eorder])
    erank = np.empty(ids.size, np.int32)
    erank[eorder] = np.arange(ids.size, dtype=np.int32)
    np.testing.assert_array_equal(rank.cpu().numpy(), erank)


@pytest.mark.parametrize("case", ["one_slot", "two_slots", "few_top_bits", "sequential", "duplicates", "odd_bins",
                                  "half_empty", "nine_million"])
def test_partition_order_whatever_the_spread_of_the_shard_slots(rng, case):
    # the bins of the fast way are cut by the top bits of the shard slot: inputs that fill them unevenly (down to
    # every id in one slot) must come out the same, by the library sort
    if case == "one_slot":
        ids = np.unique(rng.integers(0, 1 << 40, size=200000)) * 65536 + 77
    elif case == "two_slots":
        ids = np.unique(rng.integers(0, 1 << 40, size=150000)) * 65536 + rng.integers(0, 2, size=1)[0] * 65535
        ids = np.unique(np.concatenate([ids, ids[:70000] ^ 65535]))
    elif case == "few_top_bits":  # slots 0..63 only: the low bits of the slot do not choose the bin
        ids = np.unique(rng.integers(0, 1 << 30, size=300000) * 65536 + rng.integers(0, 64, size=300000))
    elif case == "sequential":
        ids = np.arange(1_000_003, dtype=np.int64) - 500_000
    elif case == "duplicates":  # outside the contract (ids without duplicates), still the stable order
        ids = rng.integers(0, 50000, size=400000)
    elif case == "half_empty":  # every second bin empty, the others fit
        ids = np.unique(rng.integers(0, 1 << 30, size=300000) * 65536 + (rng.integers(0, 32768, size=300000) & ~16))
    elif case == "odd_bins":
        ids = np.unique(rng.integers(-(1 << 62), 1 << 62, size=32769 + 4096))[:32769 + 2048]
    else:  # past the most ids the bins take
        ids = np.unique(rng.integers(-(1 << 62), 1 << 62, size=9_000_000))
    ids = ids.astype(np.int64)
    rng.shuffle(ids)
    _check_partition_order(ids)


def test_partition_order_refuses_bad_arguments():
    import ctypes

    lib = _lib.lib()
    u = _dev(np.arange(8, dtype=np.int64))
    out = torch.empty(8, dtype=torch.int64, device="cuda")
    o32 = torch.empty(8, dtype=torch.int32, device="cuda")
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    n = ctypes.c_int64
    st = _lib.stream_ptr(u.device)
    assert lib.recis_partition_order(p(u), n(8), None, p(o32), p(o32), st) != 0       # a NULL output
    assert lib.recis_partition_order(p(u), n(-1), p(out), p(o32), p(o32), st) != 0    # a negative count
    assert lib.recis_partition_order(p(u), n(1 << 31), p(out), p(o32), p(o32), st) != 0  # positions are 32-bit
    assert lib.recis_partition_order(None, n(0), None, None, None, st) == 0            # nothing to do
    with pytest.raises(TypeError):
        ops.partition_order(o32)


def test_sparse_mode_ops(rng):
    # tests/nn/segment_ops_test.py:62-113
    data = torch.tensor([[1.0, 1.0], [2.0, 2.0], [3.0, 3.0]]).cuda()
    weight = torch.tensor([2.0, 3.0, 0.5, 1.0]).cuda()
    indices = torch.tensor([2, 0, 1, 0]).cuda()
    seg = torch.tensor([0, 1, 1, 2]).cuda()
    wn = ops.segment_mean(data, weight, seg, 4)
    out = ops.segment_sum(data, wn, indices, seg, 4)
    exp = torch.tensor([[3.0, 3.0], [4.0 / 3.5, 4.0 / 3.5], [1.0, 1.0], [0.0, 0]])
    torch.testing.assert_close(out.cpu(), exp, atol=1e-7, rtol=0)
    n, rows, S, D = 3000, 256, 512, 128
    d = rng.random((rows, D)).astype(np.float32)
    w = rng.random(n).astype(np.float32)
    idx = rng.integers(0, rows, size=n)
    sg = rng.integers(0, S, size=n)
    got = ops.segment_sum(_dev(d), _dev(w), _dev(idx), _dev(sg), S).cpu().numpy()
    np.testing.assert_allclose(got, oracle.segment_sum(d, w, idx, sg, S), rtol=1e-5, atol=1e-5)
    got = ops.segment_mean(_dev(d), _dev(w), _dev(sg), S).cpu().numpy()
    np.testing.assert_allclose(got, oracle.segment_mean_weight(w, sg, S), rtol=1e-5, atol=1e-6)
    got = ops.segment_mean(_dev(d), None, _dev(sg), S).cpu().numpy()
    np.testing.assert_allclose(got, oracle.segment_mean_weight(None, sg, S), rtol=1e-5, atol=1e-6)
    # tests/ops/emb_segment_reduce_test.py:94-98
    assert ops.gen_segment_indices_by_offset(torch.tensor([0, 2, 5]).cuda()).tolist() == [0, 0, 1, 1, 1]
    off = ragged_offsets(rng, 5000, 0, 7, empty_frac=0.3)
    for dt in (np.int32, np.int64):
        got = ops.gen_segment_indices_by_offset(_dev(off.astype(dt)))
        np.testing.assert_array_equal(got.cpu().numpy(), oracle.gen_segment_indices(off))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_ragged_tile_forward_backward(rng, dtype):
    batch, seq = [50, 31, 7], [12, 3, 40]
    U, D = 300, 128
    lens = np.concatenate([rng.integers(0, 20, size=b) for b in batch])
    off = np.concatenate([[0], np.cumsum(lens)])
    value = rng.integers(0, U, size=int(off[-1]))
    table = rng.standard_normal((U, D)).astype(np.float32)
    table_t = _dev(table, dtype)
    out, batch_seq = ops.ragged_tile(batch, seq, _dev(value), _dev(off.astype(np.int32)), table_t)
    exp = oracle.ragged_tile(batch, seq, value, off, table_t.float().cpu().numpy())
    np.testing.assert_array_equal(out.float().cpu().numpy(), exp)
    dy = rng.standard_normal(exp.shape).astype(np.float32)
    dy_t = _dev(dy, dtype)
    back = ops.ragged_tile_back(batch_seq, [U, len(batch), max(batch), min(seq)], _dev(value),
                                _dev(off.astype(np.int32)), dy_t)
    exp_b = oracle.ragged_tile_back(batch, seq, value, off, dy_t.float().cpu().numpy(), U)
    tol = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=1e-2, atol=5e-2)
    np.testing.assert_allclose(back.float().cpu().numpy(), exp_b, **tol)
    assert _lib.poll_device_errors() == 0


def _check_plan(ids):
    """Invariants of a batch plan: the unique ids are exactly the set of ids, the inverse maps
    back, the lists partition the occurrences by unique id; the result is a function of the
    input only (two calls agree bit for bit on everything but the order inside a list)."""
    n = len(ids)
    p = ops.ids_unique_plan(_dev(ids))
    uniq = p.unique.cpu().numpy()
    np.testing.assert_array_equal(np.sort(uniq), np.unique(ids))
    inv = p.inverse.cpu().numpy()
    assert p.U == len(uniq) and (n == 0 or (inv.min() >= 0 and inv.max() < p.U))
    np.testing.assert_array_equal(uniq[inv] if n else inv, ids)
    rs, occ, pos = p.row_start.cpu().numpy(), p.occ.cpu().numpy(), p.pos.cpu().numpy()
    assert rs[0] == 0 and rs[p.U] == n and np.all(np.diff(rs[: p.U + 1]) >= 1 if p.U else True)
    np.testing.assert_array_equal(np.sort(occ), np.arange(n))
    np.testing.assert_array_equal(occ[pos], np.arange(n))
    row_of_entry = np.repeat(np.arange(p.U), np.diff(rs[: p.U + 1]))
    np.testing.assert_array_equal(inv[occ], row_of_entry)
    counts = p.counts.cpu().numpy()
    lens = np.diff(rs[: p.U + 1])
    assert counts[0] == p.U and counts[1] == int(np.sum(np.ceil(lens[lens > ops._HOT_LEN] / ops._HOT_CHUNK)))
    hot = p.hot_items.cpu().numpy()[: 2 * counts[1]].reshape(-1, 2)
    exp_hot = sorted((int(u), c) for u in np.nonzero(lens > ops._HOT_LEN)[0] for c in range(-(-int(lens[u]) // ops._HOT_CHUNK)))
    assert sorted(map(tuple, hot.tolist())) == exp_hot
    q = ops.ids_unique_plan(_dev(ids))
    np.testing.assert_array_equal(q.unique.cpu().numpy(), uniq)
    np.testing.assert_array_equal(q.inverse.cpu().numpy(), inv)
    np.testing.assert_array_equal(q.row_start.cpu().numpy()[: p.U + 1], rs[: p.U + 1])
    # a plan made without inverse / pos derives them from its lists on first use: the same arrays
    lean = ops.ids_unique_plan(_dev(ids), need_inverse=False, need_pos=False)
    np.testing.assert_array_equal(lean.unique.cpu().numpy(), uniq)
    np.testing.assert_array_equal(lean.inverse.cpu().numpy(), inv)
    lean_occ = lean.occ.cpu().numpy()
    np.testing.assert_array_equal(lean_occ[lean.pos.cpu().numpy()], np.arange(n))
    assert _lib.poll_device_errors() == 0
    return p


@pytest.mark.parametrize("n,hi", [(0, 10), (1, 10), (1000, 50), (1025, 10**6), (300000, 40), (200000, 3000),
                                  (1000000, 10**7), (3000000, 10**12), (8000000, 10**12),
                                  (2047, 10**6), (2049, 10**6), (4097, 20), (256 * 10240 - 1, 300),
                                  (256 * 10240, 10**12), (256 * 10240 + 1, 10**12)])
def test_unique_plan_lists(rng, n, hi):
    """Random ids from hot (tens of thousands of repeats of each id) to nearly all distinct (the
    largest case has more distinct ids per hash bucket than one LDS table takes: several rounds),
    the id that equals the library's empty marker included. The last cases sit on the edges of the
    partition's geometry: the smallest tile, and one tile of the largest size per compute unit."""
    ids = rng.integers(-hi, hi, size=n)
    if n > 5:
        ids[3] = -1
    _check_plan(ids)


def test_unique_plan_skewed_buckets(rng):
    """Shapes that stress the hash partition: one id everywhere; a few ids present in every tile
    next to a distinct tail (buckets worked in several rounds); ids that differ in the low bits
    only; a sorted run."""
    n = 600000
    _check_plan(np.full(n, 7, dtype=np.int64))
    hot = rng.integers(0, 300, size=n)
    tail = np.arange(n, dtype=np.int64) * 2**32 + 5
    _check_plan(np.where(rng.random(n) < 0.5, hot, tail))
    _check_plan(np.arange(n, dtype=np.int64))
    _check_plan(np.sort(rng.integers(0, 5000, size=n)))
    _check_plan(np.arange(n, dtype=np.int64)[::-1] << 40)


def test_unique_plan_heavy_ids(rng):
    """Batches whose head ids make up a large share of all occurrences (Zipf(1.1) and Zipf(1.2) ranks
    as in the table and sequence workloads; the empty-marker value and another id planted at 14 %
    and 2 %): such ids get columns of their own in the partition and come out as the first unique
    ids. Also through the fused find-or-insert: the rows are those a plain lookup gives."""
    n = 2_000_000
    for alpha in (1.1, 1.2):
        ranks = np.minimum(rng.zipf(alpha, size=n), 10_000_000).astype(np.int64)
        ids = ranks * 2654435761 % (1 << 40)
        p = _check_plan(ids)
        counts = np.diff(p.row_start[: p.U + 1].cpu().numpy())
        assert counts[0] == counts.max() and counts[0] > n // 20   # the head id leads the unique ids
    planted = ids.copy()
    planted[::7] = -1
    planted[1::50] = 77
    _check_plan(planted)
    m = ops.IdMap()
    for _ in range(2):   # all keys new, then all keys known
        p = ops.ids_unique_plan(_dev(ids), idmap=m)
        assert torch.equal(p.index_buf[: p.U], m.lookup_readonly(p.unique))
    assert m.size() == p.U == np.unique(ids).size
    assert sorted(p.index_buf[: p.U].tolist()) == list(range(p.U))   # rows 0 .. U-1, each once
    assert _lib.poll_device_errors() == 0


@pytest.mark.parametrize("mode", ["sum", "mean", "tile"])
@pytest.mark.parametrize("D,dtype", [(16, torch.float32), (128, torch.bfloat16), (40, torch.float32)])
def test_planned_backward_matches_oracle(rng, mode, D, dtype):
    """Gradient scatter over heavily duplicated ids (Zipf-like head + a cold tail) through the plan:
    same numbers as the oracle's sequential scatter, hot rows (many occurrences) included."""
    S = 3000
    off = ragged_offsets(rng, S, 0, 40, empty_frac=0.1)
    N = int(off[-1])
    ids = np.where(rng.random(N) < 0.5, rng.integers(0, 6, size=N), rng.integers(100, 50000, size=N))
    w = rng.random(N).astype(np.float32)
    p = ops.ids_unique_plan(_dev(ids))
    inv = p.inverse.cpu().numpy().astype(np.int64)
    g = rng.standard_normal((N if mode == "tile" else S, D)).astype(np.float32)
    g_t = _dev(g, dtype)
    g_q = g_t.float().cpu().numpy()
    for use_w in (True, False):
        got = ops.segment_reduce_backward_plan(g_t, _dev(w) if use_w else None, _dev(off), p, mode).cpu().numpy()
        exp = oracle.segment_reduce_backward(g_q, w if use_w else None, inv, off, p.U, mode)
        # hot rows sum up to ~N/12 terms of size ~1: atol scales with that (1e-6 per unit)
        np.testing.assert_allclose(got, exp, rtol=1e-5, atol=1e-6 * max(1.0, N / 12.0))
    acc = torch.ones((p.U, D), device="cuda")
    ops.segment_reduce_backward_plan(g_t, None, _dev(off), p, mode, out=acc, accumulate=True)
    exp = 1.0 + oracle.segment_reduce_backward(g_q, None, inv, off, p.U, mode)
    np.testing.assert_allclose(acc.cpu().numpy(), exp, rtol=1e-5, atol=1e-6 * max(1.0, N / 12.0))
    assert _lib.poll_device_errors() == 0


def test_planned_tile_backward_partial_cover(rng):
    """TILE backward through the plan when the offsets cover only part of the occurrences: the rest
    contributes nothing (checked on the device, no host read of the offsets)."""
    N, D = 5000, 8
    ids = rng.integers(0, 300, size=N)
    p = ops.ids_unique_plan(_dev(ids))
    inv = p.inverse.cpu().numpy().astype(np.int64)
    g = rng.standard_normal((N, D)).astype(np.float32)
    off = np.array([700, 900, 900, 4100], dtype=np.int32)
    got = ops.segment_reduce_backward_plan(_dev(g), None, _dev(off), p, "tile").cpu().numpy()
    exp = np.zeros((p.U, D), np.float64)
    np.add.at(exp, inv[700:4100], g[700:4100])
    np.testing.assert_allclose(got, exp, rtol=1e-5, atol=1e-4)
    np.testing.assert_allclose(got, oracle.segment_reduce_backward(g, None, inv, off, p.U, "tile"), rtol=1e-5, atol=1e-4)
    assert _lib.poll_device_errors() == 0


def test_planned_tile_backward_matches_oracle(rng):
    batch, seq = [50, 31, 7], [12, 3, 40]
    D = 32
    lens = np.concatenate([rng.integers(0, 20, size=b) for b in batch])
    off = np.concatenate([[0], np.cumsum(lens)])
    ids = rng.integers(0, 40, size=int(off[-1]))
    p = ops.ids_unique_plan(_dev(ids))
    inv = p.inverse.cpu().numpy().astype(np.int64)
    rows = sum(b * s for b, s in zip(batch, seq))
    dy = rng.standard_normal((rows, D)).astype(np.float32)
    src = p.src_for_tile(batch, seq, _dev(off.astype(np.int32)))
    got = ops.csr_gather_reduce(_dev(dy), p, src).cpu().numpy()
    exp = oracle.ragged_tile_back(batch, seq, inv, off, dy, p.U)
    np.testing.assert_allclose(got, exp, rtol=1e-5, atol=1e-4)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("D", [16, 128])
def test_gather_reduce_over_separate_arrays_equals_the_concatenation(rng, dtype, D):
    """recis_csr_gather_reduce_parts: the rows in up to 8 arrays, numbered end to end, against the
    plain gather-reduce over their concatenation: same kernel arithmetic, so bit for bit."""
    n = 60000
    ids = np.concatenate([rng.integers(0, 40, n // 2), rng.integers(0, 20000, n - n // 2)])  # hot and cold rows
    plan = ops.ids_unique_plan(_dev(ids))
    counts = [7000, 1, 0, 25000, 12999, 15000]
    assert sum(counts) == n
    parts = [torch.randn((c, D), device="cuda").to(dtype) for c in counts]
    src = torch.from_numpy(rng.permutation(n).astype(np.int32)).cuda()
    src[::17] = -1                                            # skipped entries
    whole = ops.csr_gather_reduce(torch.cat(parts), plan, src)
    split = ops.csr_gather_reduce_parts(parts, plan, src)
    assert torch.equal(split, whole)
    again = ops.csr_gather_reduce_parts(parts, plan, src, out=split.clone(), accumulate=True)
    torch.testing.assert_close(again, 2 * whole, rtol=1e-6, atol=1e-6)
    assert _lib.poll_device_errors() == 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("D", [16, 40, 128])
def test_gather_reduce_to_mapped_rows_equals_gather_reduce_then_permutation(rng, dtype, D):
    """recis_csr_gather_reduce_mapped: the sum of unique id u stored at out[out_rows[u]]; the same sums as the
    plain call (hot and cold rows), so bit for bit its result permuted."""
    n = 50000
    ids = np.concatenate([rng.integers(0, 30, n // 2), rng.integers(0, 15000, n - n // 2)])  # hot and cold rows
    plan = ops.ids_unique_plan(_dev(ids))
    rows = torch.randn((n, D), device="cuda").to(dtype)
    src = torch.from_numpy(rng.permutation(n).astype(np.int32)).cuda()
    src[::13] = -1
    coef = torch.rand(n, device="cuda")
    perm = torch.from_numpy(rng.permutation(plan.U).astype(np.int32)).cuda()
    plain = ops.csr_gather_reduce(rows, plan, src, coef)
    mapped = ops.csr_gather_reduce(rows, plan, src, coef, out_rows=perm)
    assert torch.equal(mapped[perm.long()], plain)
    again = ops.csr_gather_reduce(rows, plan, src, coef, out=mapped.clone(), accumulate=True, out_rows=perm)
    torch.testing.assert_close(again[perm.long()], 2 * plain, rtol=1e-6, atol=1e-6)
    with pytest.raises(TypeError):
        ops.csr_gather_reduce(rows, plan, src, coef, out_rows=perm.long())
    assert _lib.poll_device_errors() == 0


@pytest.mark.parametrize("kind", ["adamw", "adagrad"])
@pytest.mark.parametrize("D,row_dtype,grad_dtype", [(16, torch.float32, torch.float32), (128, torch.bfloat16, torch.bfloat16),
                                                    (40, torch.float32, torch.float32), (32, torch.bfloat16, torch.float32)])
def test_fused_gather_reduce_update_equals_the_two_calls(rng, kind, D, row_dtype, grad_dtype):
    """recis_csr_gather_reduce_adamw / _adagrad against recis_csr_gather_reduce into an fp32 buffer followed
    by recis_block_apply_adamw / _adagrad (which is bit-exact against the oracle, test_gpu_table.py): the
    same rows, moments and beta powers bit for bit. Ids with tens of thousands of occurrences (hot work
    items), rows the table does not hold (negative row index), pooled segments with weights."""
    n, S, bs, nb = 120000, 30000, 4096, 5
    ids = np.where(rng.random(n) < 0.3, rng.integers(0, 6, size=n), rng.integers(0, 15000, size=n))
    plan = ops.ids_unique_plan(_dev(ids))
    U = plan.U
    off = ragged_offsets(rng, S, 0, 8)
    off[-1] = n
    off = np.minimum.accumulate(off[::-1])[::-1]
    weight = _dev(rng.random(n).astype(np.float32))
    src, coef = plan.src_coef_for_pool(_dev(off), weight, mean=True)
    grad_rows = _dev(rng.standard_normal((S, D)).astype(np.float32)).to(grad_dtype)
    row_index = torch.from_numpy(rng.permutation(bs * nb)[:U]).cuda()
    row_index[::17] = -1
    mk = lambda: [_dev(rng.random((bs, D)).astype(np.float32)).to(row_dtype) for _ in range(nb)]
    emb, s0, s1 = mk(), mk(), mk()
    emb2, s02, s12 = [b.clone() for b in emb], [b.clone() for b in s0], [b.clone() for b in s1]
    b1, b2 = torch.tensor([0.9], device="cuda", dtype=torch.float64), torch.tensor([0.999], device="cuda", dtype=torch.float64)
    b1f, b2f = b1.clone(), b2.clone()
    keep = row_index >= 0
    for _ in range(2):
        g = ops.csr_gather_reduce(grad_rows, plan, src, coef)
        if kind == "adamw":
            ops.block_apply_adamw(row_index[keep], g[keep], emb, b1, b2, None, s0, s1, 1e-2, 0.9, 0.999, 0.99, 1e-8, bs)
            ops.csr_gather_reduce_adamw(grad_rows, plan, src, coef, row_index, emb2, b1f, b2f, s02, s12, 1e-2, 0.9, 0.999,
                                        0.99, 1e-8, bs)
        else:
            ops.block_apply_adagrad(row_index[keep], g[keep], emb, s0, 1e-2, 1e-8, bs)
            ops.csr_gather_reduce_adagrad(grad_rows, plan, src, coef, row_index, emb2, s02, 1e-2, 1e-8, bs)
    for a, b in zip(emb + s0 + (s1 if kind == "adamw" else []), emb2 + s02 + (s12 if kind == "adamw" else [])):
        assert torch.equal(a, b)
    assert torch.equal(b1, b1f) and torch.equal(b2, b2f)
    assert _lib.poll_device_errors() == 0


def _two_gradient_case(rng, D, tile_dtype, n_hot=3):
    """A lookup whose rows feed a mean-pooled output and a padded gather: ids (a few of them with
    thousands of occurrences), the plan, and both gradients with their src / coef arrays."""
    batch, seq = [300, 211, 64], [12, 5, 40]
    lens = np.concatenate([rng.integers(0, 30, size=b) for b in batch])
    off = np.concatenate([[0], np.cumsum(lens)])
    n = int(off[-1])
    ids = np.where(rng.random(n) < 0.4, rng.integers(0, n_hot, size=n), rng.integers(0, 3000, size=n))
    plan = ops.ids_unique_plan(_dev(ids))
    off_dev = _dev(off.astype(np.int32))
    S = len(off) - 1
    g_pool = rng.standard_normal((S, D)).astype(np.float32)
    rows = sum(b * s for b, s in zip(batch, seq))
    g_tile = _dev(rng.standard_normal((rows, D)).astype(np.float32)).to(tile_dtype)
    src_p, coef_p = plan.src_coef_for_pool(off_dev, None, True)
    src_t = plan.src_for_tile(batch, seq, off_dev)
    return plan, batch, seq, off, (_dev(g_pool), src_p, coef_p), (g_tile, src_t, None)


@pytest.mark.parametrize("D,tile_dtype,pool_dtype", [(16, torch.float32, torch.float32), (128, torch.bfloat16, torch.float32),
                                                     (40, torch.float16, torch.float32), (64, torch.float32, torch.float32),
                                                     (128, torch.bfloat16, torch.bfloat16), (32, torch.float32, torch.float16)])
def test_two_input_gather_reduce_matches_oracle(rng, D, tile_dtype, pool_dtype):
    """recis_csr_gather_reduce2 against the oracle's two backward passes added up (the backward of
    mean pooling and of the padded gather into the same unique rows), and against the two
    single-input calls it replaces."""
    plan, batch, seq, off, first, second = _two_gradient_case(rng, D, tile_dtype)
    first = (first[0].to(pool_dtype),) + first[1:]
    inv = plan.inverse.cpu().numpy().astype(np.int64)
    got = ops.csr_gather_reduce2(plan, first, second)
    g_tile32 = second[0].float().cpu().numpy()
    exp = (oracle.segment_reduce_backward(first[0].float().cpu().numpy(), None, inv, off, plan.U, "mean").astype(np.float64)
           + oracle.ragged_tile_back(batch, seq, inv, off, g_tile32, plan.U))
    # fp32 sums of up to thousands of terms in another order: atol scales with the summed magnitude
    mag = np.zeros(plan.U)
    np.add.at(mag, inv, 1.0)
    tol = 1e-6 * np.maximum(1.0, mag)[:, None] * 8
    assert np.all(np.abs(got.cpu().numpy() - exp) <= 1e-5 * np.abs(exp) + tol)
    two = ops.csr_gather_reduce(first[0], plan, first[1], first[2])
    two = ops.csr_gather_reduce(second[0], plan, second[1], None, out=two, accumulate=True)
    assert np.all(np.abs(got.cpu().numpy() - two.cpu().numpy()) <= 1e-5 * np.abs(exp) + tol)
    again = ops.csr_gather_reduce2(plan, first, second, out=got.clone(), accumulate=True)
    torch.testing.assert_close(again, 2 * got, rtol=1e-6, atol=1e-6)
    assert _lib.poll_device_errors() == 0


@pytest.mark.parametrize("kind", ["adamw", "adagrad"])
@pytest.mark.parametrize("D,row_dtype,tile_dtype,pool_dtype", [
    (16, torch.float32, torch.float32, torch.float32), (128, torch.bfloat16, torch.bfloat16, torch.float32),
    (128, torch.bfloat16, torch.float32, torch.float32), (24, torch.float16, torch.float16, torch.float32),
    (128, torch.bfloat16, torch.bfloat16, torch.bfloat16), (32, torch.float16, torch.float32, torch.float16)])
def test_two_input_fused_update_equals_gather_reduce_then_update(rng, kind, D, row_dtype, tile_dtype, pool_dtype):
    """recis_csr_gather_reduce2_adamw / _adagrad against recis_csr_gather_reduce2 into an fp32 buffer
    followed by the row update (bit-exact against the oracle in test_gpu_table.py): the same rows
    and state bit for bit, negative row indices skipped, two steps."""
    plan, batch, seq, off, first, second = _two_gradient_case(rng, D, tile_dtype)
    first = (first[0].to(pool_dtype),) + first[1:]
    U, bs, nb = plan.U, 1024, 4
    row_index = torch.from_numpy(rng.permutation(bs * nb)[:U]).cuda()
    row_index[::13] = -1
    mk = lambda: [_dev(rng.random((bs, D)).astype(np.float32)).to(row_dtype) for _ in range(nb)]
    emb, s0, s1 = mk(), mk(), mk()
    emb2, s02, s12 = [b.clone() for b in emb], [b.clone() for b in s0], [b.clone() for b in s1]
    b1, b2 = torch.tensor(0.9, device="cuda"), torch.tensor(0.999, device="cuda")
    b1f, b2f = b1.clone(), b2.clone()
    keep = row_index >= 0
    for _ in range(2):
        g = ops.csr_gather_reduce2(plan, first, second)
        if kind == "adamw":
            ops.block_apply_adamw(row_index[keep], g[keep], emb, b1, b2, None, s0, s1, 1e-2, 0.9, 0.999, 0.99, 1e-8, bs)
            ops.csr_gather_reduce2_adamw(plan, first, second, row_index, emb2, b1f, b2f, s02, s12, 1e-2, 0.9, 0.999,
                                         0.99, 1e-8, bs)
        else:
            ops.block_apply_adagrad(row_index[keep], g[keep], emb, s0, 1e-2, 1e-8, bs)
            ops.csr_gather_reduce2_adagrad(plan, first, second, row_index, emb2, s02, 1e-2, 1e-8, bs)
    for a, b in zip(emb + s0 + (s1 if kind == "adamw" else []), emb2 + s02 + (s12 if kind == "adamw" else [])):
        assert torch.equal(a, b)
    assert torch.equal(b1, b1f) and torch.equal(b2, b2f)
    assert _lib.poll_device_errors() == 0


def test_two_input_gather_reduce_refuses_what_it_does_not_support(rng):
    plan, batch, seq, off, first, second = _two_gradient_case(rng, 16, torch.float32)
    with pytest.raises(RuntimeError):                                # two half-precision inputs of different types
        ops.csr_gather_reduce2(plan, (first[0].to(torch.bfloat16), first[1], first[2]),
                               (second[0].to(torch.float16), second[1], None))
    with pytest.raises(ValueError):
        ops.csr_gather_reduce2(plan, first, (second[0][:, :8].contiguous(), second[1], None))


def test_two_input_gather_reduce_second_input_in_parts(rng):
    """The second input as separate arrays (one per feature of the padded gather) equals the same
    rows concatenated, bit for bit; with the fused Adagrad update too."""
    plan, batch, seq, off, first, second = _two_gradient_case(rng, 64, torch.bfloat16)
    n_rows = [b * s for b, s in zip(batch, seq)]
    parts = [p.clone() for p in torch.split(second[0], n_rows)]
    whole = ops.csr_gather_reduce2(plan, first, second)
    split = ops.csr_gather_reduce2(plan, first, (parts, second[1], None))
    assert torch.equal(whole, split)
    U, bs, nb = plan.U, 1024, 4
    row_index = torch.from_numpy(rng.permutation(bs * nb)[:U]).cuda()
    mk = lambda: [_dev(rng.random((bs, 64)).astype(np.float32)).to(torch.bfloat16) for _ in range(nb)]
    emb, acc = mk(), mk()
    emb2, acc2 = [b.clone() for b in emb], [b.clone() for b in acc]
    ops.csr_gather_reduce2_adagrad(plan, first, second, row_index, emb, acc, 1e-2, 1e-8, bs)
    ops.csr_gather_reduce2_adagrad(plan, first, (parts, second[1], None), row_index, emb2, acc2, 1e-2, 1e-8, bs)
    for x, y in zip(emb + acc, emb2 + acc2):
        assert torch.equal(x, y)
    swapped = ops.csr_gather_reduce2(plan, (parts, second[1], None), first)     # the parts are made the second input
    assert torch.equal(swapped, whole)
    with pytest.raises(TypeError):
        ops.csr_gather_reduce2(plan, ([first[0]], first[1], first[2]), (parts, second[1], None))   # not both in parts
    assert _lib.poll_device_errors() == 0


@pytest.mark.parametrize("sizes,with_tags", [([70000, 0, 1, 123457, 8192, 300], True), ([5000] * 40, True),
                                             ([1], True), ([100000, 250000], False), ([3] * 64, False)])
def test_unique_plan_from_separate_arrays_equals_the_plan_of_the_encoded_batch(rng, sizes, with_tags):
    """recis_unique_plan_jobs (the batch as separate arrays, tagged on the way in) against
    recis_ids_encode + recis_unique_plan: the same unique ids in the same order, the same lists
    (as sets per id: the order inside a list is unspecified), inverse and counts; with an id map,
    the same rows. Empty arrays, arrays that end inside a tile, a heavy id, more arrays than a tile
    has threads to spare."""
    parts = [rng.integers(0, 5000, size=s) if k % 3 else rng.integers(0, 3, size=s) for k, s in enumerate(sizes)]
    dev_parts = [_dev(p.astype(np.int64)) for p in parts]
    tags = [(7 * k + 1) % 4096 for k in range(len(sizes))] if with_tags else None
    batch = ops.ids_encode(dev_parts, tags) if with_tags else torch.cat(dev_parts)
    ref = ops.ids_unique_plan(batch)
    got = ops.ids_unique_plan(dev_parts, tags=tags)
    assert got.U == ref.U and got.n == ref.n
    U = ref.U
    assert torch.equal(got.unique[:U], ref.unique[:U])
    assert torch.equal(got.inverse, ref.inverse)
    assert torch.equal(got.row_start[: U + 1], ref.row_start[: U + 1])
    rs = ref.row_start[: U + 1].cpu().numpy()
    a, b = got.occ.cpu().numpy(), ref.occ.cpu().numpy()
    owner = np.repeat(np.arange(U), np.diff(rs))
    assert np.array_equal(a[np.lexsort((a, owner))], b[np.lexsort((b, owner))])   # the same occurrences per id
    assert torch.equal(got.counts, ref.counts)
    # with an id map: rows of known keys are found, new keys get the rows the encoded batch would have got
    from recis_amd.ops import IdMap
    m1, m2 = IdMap(reserve=1 << 16), IdMap(reserve=1 << 16)
    p1 = ops.ids_unique_plan(batch, idmap=m1)
    p2 = ops.ids_unique_plan(dev_parts, tags=tags, idmap=m2)
    assert torch.equal(p1.index_buf[:U], p2.index_buf[:U])
    assert m1.stats()[:2] == m2.stats()[:2]
    assert _lib.poll_device_errors() == 0

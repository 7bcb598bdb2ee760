"""Parity of the HIP id map, row-block ops and optimizer row updates (through the
C ABI) with the CPU oracle. Integer / index results are compared bit for bit; the
Adam row update is compared bit for bit too, since the kernel does the same
double-precision arithmetic as the reference's CPU functor; Adagrad within
rtol 1e-6."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from recis_amd import _lib, ops

pytestmark = pytest.mark.gpu


def _dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.to(dtype)
    return t.cuda()


# --------------------------------------------------------------------- id map
def test_row_placement_kat_gpu():
    m = ops.IdMap()
    rows = m.lookup(torch.arange(2048, device="cuda"))
    np.testing.assert_array_equal(rows.cpu().numpy(), 2047 - np.arange(2048))
    assert m.stats()[:3] == (2048, 2048, 0)


def test_idmap_matches_oracle_sequence(rng):
    """Same seeded sequence of lookups / read-only lookups / deletes on both sides."""
    g, c = ops.IdMap(), oracle.IdMap()
    live = {}
    for step in range(30):
        n = int(rng.integers(0, 5000))
        ids = np.unique(rng.integers(-1000, 20000, size=n))
        ids = ids[(ids != -1) & (ids != -2)]  # reserved by the GPU map, as in the reference
        got = g.lookup(_dev(ids)).cpu().numpy()
        exp = c.lookup(ids)
        np.testing.assert_array_equal(got, exp)
        live.update(zip(ids.tolist(), exp.tolist()))
        probe = rng.integers(-1500, 25000, size=3000)
        np.testing.assert_array_equal(g.lookup_readonly(_dev(probe)).cpu().numpy(), c.lookup_readonly(probe))
        if step % 4 == 3:
            keys = np.array(sorted(live))
            victims = keys[rng.random(len(keys)) < 0.25]
            rows = np.array([live[k] for k in victims.tolist()], np.int64)
            g.erase(_dev(victims), _dev(rows))
            c.delete(victims, rows)
            for k in victims.tolist():
                del live[k]
        lv, idn, fr, _ = g.stats()
        assert (lv, idn, fr) == (c.size(), c.id_num(), c.free_size())
    ids_g, idx_g = g.snapshot()
    assert dict(zip(ids_g.cpu().tolist(), idx_g.cpu().tolist())) == live
    assert _lib.poll_device_errors() == 0


def test_idmap_grows_past_initial_capacity(rng):
    g, c = ops.IdMap(), oracle.IdMap()
    cap0 = g.stats()[3]
    total = 0
    while total <= cap0 // 2 + 100000:
        ids = np.arange(total, total + 300000, dtype=np.int64) * 2654435761 % (1 << 40)
        np.testing.assert_array_equal(g.lookup(_dev(ids)).cpu().numpy(), c.lookup(ids))
        total += 300000
    assert g.stats()[3] > cap0
    probe = np.arange(0, total, 997, dtype=np.int64) * 2654435761 % (1 << 40)
    np.testing.assert_array_equal(g.lookup_readonly(_dev(probe)).cpu().numpy(), c.lookup_readonly(probe))


def test_idmap_duplicate_key_in_one_call_gets_one_row():
    g = ops.IdMap()
    ids = torch.tensor([7, 7, 9, 7, 9, 11], device="cuda")
    rows = g.lookup(ids).cpu().numpy()
    assert rows[0] == rows[1] == rows[3] and rows[2] == rows[4]
    assert len({rows[0], rows[2], rows[5]}) == 3
    assert g.stats()[0] == 3
    again = g.lookup(ids).cpu().numpy()
    np.testing.assert_array_equal(rows, again)


def test_idmap_tombstone_reuse_and_clear(rng):
    g, c = ops.IdMap(), oracle.IdMap()
    for rnd in range(6):
        ids = np.arange(rnd * 1000, rnd * 1000 + 50000, dtype=np.int64)
        r = g.lookup(_dev(ids)).cpu().numpy()
        np.testing.assert_array_equal(r, c.lookup(ids))
        g.erase(_dev(ids[::2]), _dev(r[::2]))
        c.delete(ids[::2], r[::2])
    assert g.stats()[:3] == (c.size(), c.id_num(), c.free_size())
    g.clear()
    assert g.stats()[:3] == (0, 0, 0)
    np.testing.assert_array_equal(g.lookup(torch.arange(5, device="cuda")).cpu().numpy(), [4, 3, 2, 1, 0])


def test_reserved_keys_are_reported():
    g = ops.IdMap()
    _lib.poll_device_errors()
    rows = g.lookup(torch.tensor([5, -1, 6], device="cuda")).cpu().numpy()
    assert rows[1] == -1 and _lib.poll_device_errors() & _lib.DEVERR_INDEX_RANGE
    assert g.stats()[0] == 2


def test_allocator_ops_kats():
    # tests/ops/hashtable_ops_test.py:16-54
    fb = [torch.arange(100000, dtype=torch.int64, device="cuda")]
    r = ops.generate_ids(10000, fb, 0, 101, 100000)
    assert torch.equal(r, torch.arange(101, 10101, device="cuda").flip(0))
    r = ops.generate_ids(10000, fb, 2000, 101, 100000)
    assert torch.equal(r, torch.cat([torch.arange(101, 8101, device="cuda").flip(0), fb[0][:2000]]))
    free = torch.arange(101, 10101, device="cuda")
    ops.free_ids(free, fb, 2000, 100000)
    ans = torch.arange(100000, device="cuda")
    ans[2000:12000] = free
    assert torch.equal(fb[0], ans)
    # blocks of 10240 like the reference allocator
    blocks = [torch.zeros(10240, dtype=torch.int64, device="cuda") for _ in range(3)]
    ops.free_ids(torch.arange(25000, device="cuda"), blocks, 100, 10240)
    flat = torch.cat(blocks)
    assert torch.equal(flat[100:25100], torch.arange(25000, device="cuda"))
    r = ops.generate_ids(20000, blocks, 25100, 7, 10240)
    assert torch.equal(r, flat[5100:25100])


def test_mask_key_index_and_scatter(rng):
    n = 10000
    mask = torch.from_numpy(rng.random(n) < 0.2).cuda()
    ids = torch.arange(101, 101 + n, device="cuda")
    index = ids.flip(0).clone()
    cs = torch.cumsum(mask, 0)
    gen = int(cs[-1])
    new_ids, range_index = ops.mask_key_index(ids, mask, cs, gen)
    assert torch.equal(new_ids, ids[mask])
    assert torch.equal(range_index, torch.arange(n, device="cuda")[mask])
    new_index = torch.arange(5000, 5000 + gen, device="cuda")
    exp = index.clone()
    exp[range_index] = new_index
    assert torch.equal(ops.scatter_ids_with_mask(index, new_index, range_index), exp)


# ------------------------------------------------------------------ row blocks
@pytest.mark.parametrize("dtype,D", [(torch.float32, 16), (torch.float32, 5), (torch.bfloat16, 128),
                                     (torch.int64, 1), (torch.int8, 3), (torch.float16, 24)])
def test_block_gather_insert(rng, dtype, D):
    bs, nb = 37, 5
    if dtype.is_floating_point:
        blocks = [torch.randn(bs, D, device="cuda").to(dtype) for _ in range(nb)]
    else:
        blocks = [torch.randint(-100, 100, (bs, D), device="cuda").to(dtype) for _ in range(nb)]
    flat = torch.cat(blocks)
    ids = torch.from_numpy(rng.integers(0, bs * nb, size=500)).cuda()
    assert torch.equal(ops.block_gather(ids, blocks, bs, -1, False), flat[ids])
    assert torch.equal(ops.gather(ids, flat), flat[ids])
    assert torch.equal(ops.gather(ids.int(), flat), flat[ids])
    ro = ids.clone()
    ro[::3] = -1
    exp = flat[ro.clamp(min=0)]
    exp[ro == -1] = 0
    assert torch.equal(ops.block_gather(ro, blocks, bs, -1, True), exp)
    assert torch.equal(ops.block_gather_by_range(ids, blocks, bs, 100, 300), flat[ids[100:300]])
    uids = torch.from_numpy(rng.permutation(bs * nb)[:60]).cuda()
    emb = flat[torch.from_numpy(rng.integers(0, bs * nb, size=60)).cuda()].clone()
    ops.block_insert(uids, emb, blocks, bs)
    flat[uids] = emb
    assert torch.equal(torch.cat(blocks), flat)
    ops.block_insert(uids, emb[:1], blocks, bs)
    flat[uids] = emb[0]
    assert torch.equal(torch.cat(blocks), flat)
    mask = torch.from_numpy(rng.random(60) < 0.5).cuda()
    emb2 = flat[torch.from_numpy(rng.integers(0, bs * nb, size=60)).cuda()].clone()
    ops.block_insert_with_mask(uids, emb2, mask, blocks, bs)
    flat[uids[mask]] = emb2[mask]
    assert torch.equal(torch.cat(blocks), flat)


def test_block_gather_single_big_block_and_errors(rng):
    big = [torch.randn(5000, 32, device="cuda")]
    ids = torch.from_numpy(rng.integers(0, 5000, size=777)).cuda()
    assert torch.equal(ops.block_gather(ids, big, 5000), big[0][ids])
    _lib.poll_device_errors()
    bad = torch.tensor([1, 5000, 2], device="cuda")
    out = ops.block_gather(bad, big, 5000)
    assert _lib.poll_device_errors() & _lib.DEVERR_INDEX_RANGE
    assert torch.equal(out[0], big[0][1]) and float(out[1].abs().sum()) == 0


@pytest.mark.parametrize("dt", [torch.int64, torch.int32])
def test_block_filter(rng, dt):
    bs, nb = 100, 4
    blocks = [torch.randint(0, 200, (bs, 1), device="cuda").to(dt) for _ in range(nb)]
    flat = torch.cat(blocks)[:, 0]
    ids = torch.from_numpy(rng.integers(0, bs * nb, size=333)).cuda()
    assert torch.equal(ops.block_filter(ids, blocks, bs, 77), flat[ids] < 77)


def test_counted_lookup_and_host_bounds(rng):
    """Lookup of "the first n_dev[0] ids of a buffer" (size known to the device only) gives the
    rows of a plain lookup of that prefix and leaves the rest of the output alone; the map's
    host-side bounds never undercut the true allocator mark and settle to it."""
    g, c = ops.IdMap(), oracle.IdMap()
    for rnd in range(5):
        buf = rng.integers(0, 4000, size=3000)
        buf = buf[np.sort(np.unique(buf, return_index=True)[1])]  # unique ids, as a plan hands them over
        n_true = int(rng.integers(0, len(buf) + 1))
        n_dev = torch.tensor([n_true, 123], device="cuda")
        out = g.lookup_counted(_dev(buf), n_dev)
        assert g.id_num_bound() >= c.id_num()          # before anything is known: counts the whole buffer
        got = out.cpu().numpy()
        exp = c.lookup(buf[:n_true])
        np.testing.assert_array_equal(got[:n_true], exp)
        g.settle_count(n_true)
        bound = g.id_num_bound()
        torch.cuda.synchronize()
        assert c.id_num() <= g.id_num_bound() <= bound
        assert g.id_num_bound() == c.id_num() == g.id_num()
        assert g.stats()[:3] == (c.size(), c.id_num(), c.free_size())
        # erase a few, so that recycled rows take part in the next round
        drop = buf[:n_true][::3]
        rows = c.lookup_readonly(drop)
        g.erase(_dev(drop), _dev(rows))
        c.delete(drop, rows)
    # a count beyond the buffer is clamped to the buffer
    buf = np.arange(10**6, 10**6 + 50, dtype=np.int64)
    out = g.lookup_counted(_dev(buf), torch.tensor([10**9], device="cuda"))
    np.testing.assert_array_equal(out.cpu().numpy(), c.lookup(buf))
    assert _lib.poll_device_errors() == 0


@pytest.mark.parametrize("dt", [torch.int64, torch.int32])
def test_evict_older_equals_snapshot_filter_erase(rng, dt):
    """The one-pass eviction sweep against the reference's sequence (snapshot, block_filter,
    masked_select, erase) on a twin map and against the oracle map: same evicted set, same
    live set, same allocator counters; freed rows are handed out again."""
    bs, nb = 1000, 8
    keys = rng.integers(-10**15, 10**15, size=6000)
    keys = np.unique(keys)
    a, b, c = ops.IdMap(), ops.IdMap(), oracle.IdMap()
    rows = a.lookup(_dev(keys)).cpu().numpy()
    np.testing.assert_array_equal(b.lookup(_dev(keys)).cpu().numpy(), rows)
    np.testing.assert_array_equal(c.lookup(keys), rows)
    stamps = rng.integers(0, 100, size=bs * nb)
    blocks = [torch.from_numpy(stamps[i * bs:(i + 1) * bs].reshape(bs, 1)).cuda().to(dt) for i in range(nb)]
    thr = 40
    ev_ids, ev_rows = a.evict_older(blocks, bs, thr)
    ids_b, idx_b = b.snapshot()
    mask = ops.block_filter(idx_b, blocks, bs, thr)
    del_ids, del_rows = torch.masked_select(ids_b, mask), torch.masked_select(idx_b, mask)
    b.erase(del_ids, del_rows)
    exp_mask = stamps[rows] < thr
    order = np.argsort(ev_ids.cpu().numpy())
    np.testing.assert_array_equal(ev_ids.cpu().numpy()[order], np.sort(keys[exp_mask]))
    np.testing.assert_array_equal(ev_rows.cpu().numpy()[order], rows[exp_mask][np.argsort(keys[exp_mask])])
    c.delete(keys[exp_mask], rows[exp_mask])
    assert a.stats()[:3] == b.stats()[:3] == (c.size(), c.id_num(), c.free_size())
    for m in (a, b):
        got = m.lookup_readonly(_dev(keys)).cpu().numpy()
        np.testing.assert_array_equal(got, np.where(exp_mask, -1, rows))
    # new keys take the freed rows (the free list holds exactly the evicted rows)
    fresh = np.arange(10**16, 10**16 + int(exp_mask.sum()), dtype=np.int64)
    assert sorted(a.lookup(_dev(fresh)).cpu().numpy().tolist()) == sorted(rows[exp_mask].tolist())
    # nothing to evict: no change; a buffer smaller than the evictable set evicts just that many
    assert a.evict_older(blocks, bs, -5)[0].numel() == 0
    n_more = int((stamps[b.snapshot()[1].cpu().numpy()] < 90).sum())
    part_ids, _ = b.evict_older(blocks, bs, 90, max_out=7)
    assert part_ids.numel() == min(7, n_more) and b.stats()[0] == c.size() - part_ids.numel()
    assert _lib.poll_device_errors() == 0


# ------------------------------------------------------------------ optimizers
def _np_blocks(w, bs):
    nb = (w.shape[0] + bs - 1) // bs
    pad = np.zeros((nb * bs - w.shape[0], w.shape[1]), w.dtype)
    w = np.concatenate([w, pad])
    return [np.ascontiguousarray(w[i * bs:(i + 1) * bs]) for i in range(nb)]


@pytest.mark.parametrize("beta_dtype", [np.float32, np.float64])
@pytest.mark.parametrize("D,bs", [(16, 64), (32, 10240), (7, 5)])
def test_adamw_bit_exact_vs_oracle(rng, beta_dtype, D, bs):
    U, steps = 300, 12
    lr, b1, b2, eps, decay = 1e-3, 0.9, 0.999, 1e-8, 1 - 1e-3 * 1e-2
    rows0 = (0.01 * rng.standard_normal((U, D))).astype(np.float32)
    c_emb, c_m, c_v = _np_blocks(rows0, bs), _np_blocks(np.zeros_like(rows0), bs), _np_blocks(np.zeros_like(rows0), bs)
    g_emb = [_dev(b) for b in c_emb]
    g_m = [_dev(b) for b in c_m]
    g_v = [_dev(b) for b in c_v]
    cb1, cb2 = np.ones(1, beta_dtype), np.ones(1, beta_dtype)
    gb1, gb2 = _dev(cb1), _dev(cb2)
    step_t = torch.zeros(1, dtype=torch.int64, device="cuda")
    for _ in range(steps):
        idx = np.sort(rng.permutation(U)[:rng.integers(1, U)])
        g = rng.standard_normal((len(idx), D)).astype(np.float32)
        oracle.block_apply_adamw(idx, g, c_emb, cb1, cb2, c_m, c_v, lr, b1, b2, decay, eps, bs)
        ops.block_apply_adamw(_dev(idx), _dev(g), g_emb, gb1, gb2, step_t, g_m, g_v, lr, b1, b2, decay, eps, bs)
    for gl, cl in ((g_emb, c_emb), (g_m, c_m), (g_v, c_v)):
        np.testing.assert_array_equal(torch.cat(gl).cpu().numpy(), np.concatenate(cl))
    np.testing.assert_array_equal(gb1.cpu().numpy(), cb1)
    np.testing.assert_array_equal(gb2.cpu().numpy(), cb2)
    assert int(step_t) == 0  # never advances, as in the reference


def test_adamw_empty_index_still_advances_betas():
    emb = [torch.zeros(4, 8, device="cuda")]
    m, v = [torch.zeros(4, 8, device="cuda")], [torch.zeros(4, 8, device="cuda")]
    b1t = torch.ones(1, device="cuda")
    b2t = torch.ones(1, device="cuda")
    ops.block_apply_adamw(torch.zeros(0, dtype=torch.int64, device="cuda"), torch.zeros(0, 8, device="cuda"),
                          emb, b1t, b2t, torch.zeros(1, dtype=torch.int64, device="cuda"), m, v,
                          1e-3, 0.9, 0.999, 1.0, 1e-8, 4)
    assert abs(float(b1t) - 0.9) < 1e-7 and abs(float(b2t) - 0.999) < 1e-7


@pytest.mark.parametrize("D,bs", [(16, 128), (128, 33)])
def test_adagrad_vs_oracle(rng, D, bs):
    U, steps, lr, eps = 200, 15, 0.01, 1e-8
    rows0 = (0.01 * rng.standard_normal((U, D))).astype(np.float32)
    c_emb, c_acc = _np_blocks(rows0, bs), _np_blocks(np.zeros_like(rows0), bs)
    g_emb, g_acc = [_dev(b) for b in c_emb], [_dev(b) for b in c_acc]
    for _ in range(steps):
        idx = np.sort(rng.permutation(U)[:rng.integers(1, U)])
        g = rng.standard_normal((len(idx), D)).astype(np.float32)
        oracle.block_apply_adagrad(idx, g, c_emb, c_acc, lr, eps, bs)
        ops.block_apply_adagrad(_dev(idx), _dev(g), g_emb, g_acc, lr, eps, bs)
    np.testing.assert_allclose(torch.cat(g_emb).cpu().numpy(), np.concatenate(c_emb), rtol=1e-6, atol=1e-8)
    np.testing.assert_allclose(torch.cat(g_acc).cpu().numpy(), np.concatenate(c_acc), rtol=1e-6, atol=1e-8)


@pytest.mark.parametrize("row_dtype,grad_dtype", [(torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16),
                                                  (torch.bfloat16, torch.float32)])
@pytest.mark.parametrize("D,bs", [(128, 64), (16, 1024), (7, 5)])
def test_adagrad_rows_bit_exact_vs_the_update_with_its_roundings_spelled_out(rng, D, bs, row_dtype, grad_dtype):
    """oracle.block_apply_adagrad_exact (every operation rounded once in float32, the rows rounded to their
    storage type when assigned) against the stand-alone row kernel and the fused gather-reduce ending,
    float32 and bfloat16 rows (what config 5 trains on), bit for bit."""
    U, steps, lr, eps = 300, 8, 0.05, 1e-8
    bf = row_dtype == torch.bfloat16
    rows0 = (0.5 * rng.standard_normal((U, D))).astype(np.float32)
    if bf:
        rows0 = oracle.round_bf16(rows0)
    c_emb, c_acc = _np_blocks(rows0, bs), _np_blocks(np.zeros_like(rows0), bs)
    g_emb, g_acc = [_dev(b, row_dtype) for b in c_emb], [_dev(b, row_dtype) for b in c_acc]
    f_emb, f_acc = [b.clone() for b in g_emb], [b.clone() for b in g_acc]
    for _ in range(steps):
        idx = np.sort(rng.permutation(U)[:rng.integers(1, U)])
        g = rng.standard_normal((len(idx), D)).astype(np.float32)
        if grad_dtype == torch.bfloat16:
            g = oracle.round_bf16(g)
        oracle.block_apply_adagrad_exact(idx, g, c_emb, c_acc, lr, eps, bs, bf16=bf)
        ops.block_apply_adagrad(_dev(idx), _dev(g, grad_dtype), g_emb, g_acc, lr, eps, bs)
        plan = ops.ids_unique_plan(_dev(np.arange(len(idx), dtype=np.int64) * 7919))
        order = plan.unique.cpu().numpy() // 7919          # unique id u is occurrence order[u]
        ops.csr_gather_reduce_adagrad(_dev(g, grad_dtype), plan, plan.occ, None, _dev(idx[order]), f_emb, f_acc, lr, eps, bs)
    for gl, fl, cl in ((g_emb, f_emb, c_emb), (g_acc, f_acc, c_acc)):
        np.testing.assert_array_equal(torch.cat(gl).float().cpu().numpy(), np.concatenate(cl))
        np.testing.assert_array_equal(torch.cat(fl).float().cpu().numpy(), np.concatenate(cl))
    assert _lib.poll_device_errors() == 0


def test_bf16_rows_fp32_grads_track_fp32_path(rng):
    """bf16 row storage: compared with the fp32 oracle within rtol 1e-2 (there is no
    bf16 CPU path in the reference)."""
    U, D, bs, lr, eps = 128, 64, 128, 0.05, 1e-8
    rows0 = rng.standard_normal((U, D)).astype(np.float32)
    c_emb, c_acc = _np_blocks(rows0, bs), _np_blocks(np.zeros_like(rows0), bs)
    g_emb = [_dev(b, torch.bfloat16) for b in c_emb]
    g_acc = [_dev(b, torch.bfloat16) for b in c_acc]
    idx = np.arange(U)
    for _ in range(3):
        g = rng.standard_normal((U, D)).astype(np.float32)
        oracle.block_apply_adagrad(idx, g, c_emb, c_acc, lr, eps, bs)
        ops.block_apply_adagrad(_dev(idx), _dev(g), g_emb, g_acc, lr, eps, bs)
    np.testing.assert_allclose(torch.cat(g_emb).float().cpu().numpy(), np.concatenate(c_emb), rtol=2e-2, atol=2e-2)


def test_plan_with_lookup_matches_the_oracle_map_and_the_separate_lookup(rng):
    """recis_unique_plan_lookup (dedup and find-or-insert in one pass) over a script of batches with
    duplicates, new and known keys, erasures in between (free-list reuse, tombstones) and a batch
    that outgrows the initial slot table: the rows equal, bit for bit, what the oracle's map assigns
    when it is given the plan's unique ids in the plan's order, and what a second GPU map assigns
    through the plan followed by the stand-alone lookup; allocator state and snapshot agree."""
    fused, split, cpu = ops.IdMap(), ops.IdMap(), oracle.IdMap()
    live = {}
    sizes = [0, 1, 700, 30000, 5000, 200000, 64, 1_500_000, 90000]
    for step, n in enumerate(sizes):
        hot = rng.integers(0, 50, size=n)
        cold = rng.integers(-(1 << 62), 1 << 62, size=n)
        seen = np.array(sorted(live))[: n // 3] if live else np.zeros(0, np.int64)
        ids = np.where(rng.random(n) < 0.3, hot, cold)
        if len(seen):
            ids[: len(seen)] = seen                      # keys the maps already hold
        ids_t = _dev(ids)
        p = ops.ids_unique_plan(ids_t, idmap=fused, wait=(step % 2 == 0))
        q = ops.ids_unique_plan(ids_t)
        U = p.U
        assert U == q.U == len(np.unique(ids))
        uniq = p.unique.cpu().numpy()
        np.testing.assert_array_equal(uniq, q.unique.cpu().numpy())
        np.testing.assert_array_equal(p.inverse.cpu().numpy(), q.inverse.cpu().numpy())
        got = p.index_buf[:U].cpu().numpy()
        np.testing.assert_array_equal(got, split.lookup(q.unique).cpu().numpy())
        np.testing.assert_array_equal(got, cpu.lookup(uniq))
        live.update(zip(uniq.tolist(), got.tolist()))
        assert fused.stats()[:3] == split.stats()[:3] == (cpu.size(), cpu.id_num(), cpu.free_size())
        if step in (3, 5):
            keys = np.array(sorted(live))
            victims = keys[rng.random(len(keys)) < 0.4]
            rows = np.array([live[k] for k in victims.tolist()], np.int64)
            for m in (fused, split):
                m.erase(_dev(victims), _dev(rows))
            cpu.delete(victims, rows)
            for k in victims.tolist():
                del live[k]
    ids_g, idx_g = fused.snapshot()
    assert dict(zip(ids_g.cpu().tolist(), idx_g.cpu().tolist())) == live
    assert _lib.poll_device_errors() == 0


def test_plan_with_lookup_flags_the_reserved_keys():
    m = ops.IdMap()
    ids = torch.tensor([5, -1, 7, -2, 5, -1], device="cuda")
    p = ops.ids_unique_plan(ids, idmap=m, wait=False)
    assert int(p.counts[0]) == 4
    rows = dict(zip(p.unique_buf[:4].tolist(), p.index_buf[:4].tolist()))
    assert rows[-1] == -1 and rows[-2] == -1 and sorted((rows[5], rows[7])) == [0, 1]
    # the soft error travels to the host with the staged count: reading the count raises it
    with pytest.raises(RuntimeError, match="index outside"):
        p.U
    assert _lib.poll_device_errors() == 0          # raised once, cleared
    assert m.stats()[:2] == (2, 2)


def test_look_back_gives_up_instead_of_hanging():
    """A workgroup of the plan that waits for the look-back word of an earlier bucket polls a bounded
    number of times. With the bound forced to one poll (from the host) some waits give up: the
    kernel still ends, the error bit says so, and the next plan with the default bound is right."""
    lib = _lib.lib()
    ids = torch.randint(0, 1 << 40, (400000,), device="cuda")
    default = ctypes.c_int64(0)
    _lib.check(lib.recis_plan_get_spin_limit(ctypes.byref(default)))
    assert default.value == 1 << 22          # RECIS_PLAN_SPIN_LIMIT_DEFAULT
    try:
        _lib.check(lib.recis_plan_set_spin_limit(ctypes.c_int64(1)))
        for _ in range(3):
            ops.ids_unique_plan(ids, wait=False)   # the count is not read: a reader would raise the error bit
        torch.cuda.synchronize()
    finally:
        _lib.check(lib.recis_plan_set_spin_limit(default))
    bits = _lib.poll_device_errors()
    assert bits in (0, _lib.DEVERR_PLAN_OVERFLOW)
    p = ops.ids_unique_plan(ids)
    assert torch.equal(torch.sort(p.unique).values, torch.unique(ids))
    assert _lib.poll_device_errors() == 0


@pytest.mark.parametrize("row_bytes", [64, 256])
def test_random_row_probe_reads_nothing_away_and_writes_whole_rows(rng, row_bytes):
    """recis_hip_probe_random_rows (measurement support): the read mode leaves table and sink alone,
    the write mode overwrites exactly the rows it was given, whole; arguments it cannot serve are refused."""
    lib, i64, ptr = _lib.lib(), _lib.i64, _lib.ptr
    rows, n = 5000, 3000
    table = torch.full((rows, row_bytes // 4), 7, dtype=torch.int32, device="cuda")
    sink = torch.zeros(4096, dtype=torch.int32, device="cuda")
    idx = torch.from_numpy(rng.permutation(rows)[:n].astype(np.int32)).cuda()
    stream = _lib.stream_ptr(table.device)
    for in_flight in (1, 2, 4):
        _lib.check(lib.recis_hip_probe_random_rows(ptr(table), i64(rows), i64(row_bytes), ptr(idx), i64(n), in_flight, 0,
                                                   ptr(sink), stream))
    assert int((table != 7).sum()) == 0 and int(sink.abs().sum()) == 0
    _lib.check(lib.recis_hip_probe_random_rows(ptr(table), i64(rows), i64(row_bytes), ptr(idx), i64(n), 2, 1, ptr(sink), stream))
    touched = torch.zeros(rows, dtype=torch.bool, device="cuda")
    touched[idx.long()] = True
    changed = (table != 7).any(dim=1)
    assert torch.equal(changed, touched)
    assert bool((table[touched][:, 1::4] == 1).all()) and bool((table[touched][:, 3::4] == 3).all())
    assert bool((table[~touched] == 7).all())
    assert lib.recis_hip_probe_random_rows(ptr(table), i64(rows), i64(48), ptr(idx), i64(n), 1, 0, ptr(sink), stream) == 1
    assert lib.recis_hip_probe_random_rows(ptr(table), i64(rows), i64(row_bytes), ptr(idx), i64(n), 3, 0, ptr(sink), stream) == 1
    assert _lib.poll_device_errors() == 0


@pytest.mark.parametrize("D,bs", [(16, 64), (24, 33)])
def test_adamw_half_rows_bit_exact_vs_oracle(rng, D, bs):
    """float16 rows and gradients: the roundings of the reference's CPU functor with TEmb = at::Half
    (oracle.block_apply_adamw_f16, itself pinned against the compiled reference): every assignment
    rounds double -> float -> half and the step is rounded to half before it is added. The stand-alone
    row kernel and the fused gather-reduce ending, which share the arithmetic."""
    U, steps = 300, 8
    lr, b1, b2, eps, decay = 1e-2, 0.9, 0.999, 1e-8, 0.99
    rows0 = (0.5 * rng.standard_normal((U, D))).astype(np.float16)
    c_emb, c_m, c_v = _np_blocks(rows0, bs), _np_blocks(np.zeros_like(rows0), bs), _np_blocks(np.zeros_like(rows0), bs)
    g_emb, g_m, g_v = [_dev(b) for b in c_emb], [_dev(b) for b in c_m], [_dev(b) for b in c_v]
    f_emb, f_m, f_v = [b.clone() for b in g_emb], [b.clone() for b in g_m], [b.clone() for b in g_v]
    cb1, cb2 = np.ones(1, np.float32), np.ones(1, np.float32)
    gb1, gb2, fb1, fb2 = _dev(cb1), _dev(cb2), _dev(cb1), _dev(cb2)
    for _ in range(steps):
        idx = np.sort(rng.permutation(U)[:rng.integers(1, U)])
        g = rng.standard_normal((len(idx), D)).astype(np.float16)
        oracle.block_apply_adamw_f16(idx, g, c_emb, cb1, cb2, c_m, c_v, lr, b1, b2, decay, eps, bs)
        ops.block_apply_adamw(_dev(idx), _dev(g), g_emb, gb1, gb2, None, g_m, g_v, lr, b1, b2, decay, eps, bs)
        # the same step through the fused ending: one occurrence per row, so the sum is the gradient itself
        plan = ops.ids_unique_plan(_dev(np.arange(len(idx), dtype=np.int64) * 7919))
        order = plan.unique.cpu().numpy() // 7919          # unique id u is occurrence order[u]
        ops.csr_gather_reduce_adamw(_dev(g), plan, plan.occ, None, _dev(idx[order]), f_emb, fb1, fb2, f_m, f_v, lr, b1, b2,
                                    decay, eps, bs)
    for gl, fl, cl in ((g_emb, f_emb, c_emb), (g_m, f_m, c_m), (g_v, f_v, c_v)):
        np.testing.assert_array_equal(torch.cat(gl).cpu().numpy(), np.concatenate(cl))
        np.testing.assert_array_equal(torch.cat(fl).cpu().numpy(), np.concatenate(cl))
    np.testing.assert_array_equal(gb1.cpu().numpy(), cb1)
    assert _lib.poll_device_errors() == 0


@pytest.mark.parametrize("grad_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("D,bs", [(128, 64), (16, 1024), (7, 5)])
def test_adamw_bfloat16_rows_bit_exact_vs_oracle(rng, D, bs, grad_dtype):
    """bfloat16 rows (what config 5 trains on), gradients in bfloat16 or float32: bit for bit
    oracle.block_apply_adamw_bf16, the Half restatement the compiled reference pins with bfloat16's
    rounding in its place (the reference itself dispatches no bfloat16). The stand-alone row kernel and
    the fused gather-reduce ending."""
    U, steps = 300, 8
    lr, b1, b2, eps, decay = 1e-2, 0.9, 0.999, 1e-8, 0.99
    rows0 = oracle.round_bf16(0.5 * rng.standard_normal((U, D)))
    c_emb, c_m, c_v = _np_blocks(rows0, bs), _np_blocks(np.zeros_like(rows0), bs), _np_blocks(np.zeros_like(rows0), bs)
    g_emb, g_m, g_v = ([_dev(b, torch.bfloat16) for b in c] for c in (c_emb, c_m, c_v))
    f_emb, f_m, f_v = [b.clone() for b in g_emb], [b.clone() for b in g_m], [b.clone() for b in g_v]
    cb1, cb2 = np.ones(1, np.float32), np.ones(1, np.float32)
    gb1, gb2, fb1, fb2 = _dev(cb1), _dev(cb2), _dev(cb1), _dev(cb2)
    for _ in range(steps):
        idx = np.sort(rng.permutation(U)[:rng.integers(1, U)])
        g = rng.standard_normal((len(idx), D)).astype(np.float32)
        if grad_dtype == torch.bfloat16:
            g = oracle.round_bf16(g)
        oracle.block_apply_adamw_bf16(idx, g, c_emb, cb1, cb2, c_m, c_v, lr, b1, b2, decay, eps, bs)
        ops.block_apply_adamw(_dev(idx), _dev(g, grad_dtype), g_emb, gb1, gb2, None, g_m, g_v, lr, b1, b2, decay, eps, bs)
        plan = ops.ids_unique_plan(_dev(np.arange(len(idx), dtype=np.int64) * 7919))
        order = plan.unique.cpu().numpy() // 7919          # unique id u is occurrence order[u]
        ops.csr_gather_reduce_adamw(_dev(g, grad_dtype), plan, plan.occ, None, _dev(idx[order]), f_emb, fb1, fb2, f_m, f_v,
                                    lr, b1, b2, decay, eps, bs)
    for gl, fl, cl in ((g_emb, f_emb, c_emb), (g_m, f_m, c_m), (g_v, f_v, c_v)):
        np.testing.assert_array_equal(torch.cat(gl).float().cpu().numpy(), np.concatenate(cl))
        np.testing.assert_array_equal(torch.cat(fl).float().cpu().numpy(), np.concatenate(cl))
    np.testing.assert_array_equal(gb1.cpu().numpy(), cb1)
    assert _lib.poll_device_errors() == 0


@pytest.mark.parametrize("beta_dtype", [np.float32, np.float64])
def test_adamw_double_rows_bit_exact_vs_oracle(rng, beta_dtype):
    """float64 rows and gradients (the reference's functor is dispatched for them): bit for bit the
    oracle's restatement, which the compiled reference pins; other gradient types are refused."""
    U, D, bs, steps = 200, 5, 64, 6
    lr, b1, b2, eps, decay = 1e-2, 0.9, 0.999, 1e-8, 0.99
    rows0 = rng.standard_normal((U, D))
    c_emb, c_m, c_v = _np_blocks(rows0, bs), _np_blocks(np.zeros_like(rows0), bs), _np_blocks(np.zeros_like(rows0), bs)
    g_emb, g_m, g_v = [_dev(b) for b in c_emb], [_dev(b) for b in c_m], [_dev(b) for b in c_v]
    cb1, cb2 = np.ones(1, beta_dtype), np.ones(1, beta_dtype)
    gb1, gb2 = _dev(cb1), _dev(cb2)
    for _ in range(steps):
        idx = np.sort(rng.permutation(U)[:rng.integers(1, U)])
        g = rng.standard_normal((len(idx), D))
        oracle.block_apply_adamw_f64(idx, g, c_emb, cb1, cb2, c_m, c_v, lr, b1, b2, decay, eps, bs)
        ops.block_apply_adamw(_dev(idx), _dev(g), g_emb, gb1, gb2, None, g_m, g_v, lr, b1, b2, decay, eps, bs)
    for gl, cl in ((g_emb, c_emb), (g_m, c_m), (g_v, c_v)):
        np.testing.assert_array_equal(torch.cat(gl).cpu().numpy(), np.concatenate(cl))
    np.testing.assert_array_equal(gb1.cpu().numpy(), cb1)
    with pytest.raises((TypeError, _lib.RecisHipError)):
        ops.block_apply_adamw(_dev(idx), _dev(g.astype(np.float32)), g_emb, gb1, gb2, None, g_m, g_v, lr, b1, b2, decay, eps, bs)
    assert _lib.poll_device_errors() == 0

"""Pins the id-map / allocator / row-block / optimizer part of the CPU oracle.

Sources of truth: the reference's known-answer vectors (generate_ids, free_ids,
row placement after insert(arange(2048))), closed forms the reference tests use
(masked_select, slicing), torch.optim (AdamW, Adagrad) as library routines, and
a brute-force Python model of the allocator + dict on small inputs.
"""
import numpy as np
import torch

import oracle


# ------------------------------------------------------------------ allocator
def test_generate_ids_kats():
    # tests/ops/hashtable_ops_test.py:16-38
    fb = np.arange(100000, dtype=np.int64)
    r = oracle.generate_ids(10000, fb, 0, 101)
    np.testing.assert_array_equal(r, np.arange(101, 10101)[::-1])
    r = oracle.generate_ids(10000, fb, 2000, 101)
    np.testing.assert_array_equal(r, np.concatenate([np.arange(101, 8101)[::-1], fb[:2000]]))


def test_mask_key_index_vs_masked_select(rng):
    # tests/ops/hashtable_ops_test.py:68-86
    n = 10000
    mask = rng.random(n) < 0.2
    ids = np.arange(101, 101 + n)
    index = ids[::-1].copy()
    cumsum = np.cumsum(mask)
    gen = int(cumsum[-1])
    new_ids, range_index = oracle.mask_key_index(ids, mask, cumsum, gen)
    np.testing.assert_array_equal(new_ids, ids[mask])
    np.testing.assert_array_equal(range_index, np.arange(n)[mask])
    new_index = np.arange(5000, 5000 + gen)
    out = oracle.scatter_ids_with_mask(index, new_index, range_index)
    exp = index.copy()
    exp[np.arange(n)[mask]] = new_index
    np.testing.assert_array_equal(out, exp)


class ModelAllocator:
    """Brute-force model: a Python list as free list, ids handed out one at a time."""

    def __init__(self):
        self.cur = 0
        self.free = []

    def gen(self, n):
        # the last min(n, len(free)) freed ids, in free order, fill the tail;
        # fresh ids descend from cur + n_fresh - 1
        take = min(n, len(self.free))
        n_fresh = n - take
        fresh = [self.cur + n_fresh - 1 - i for i in range(n_fresh)]
        tail = self.free[len(self.free) - take:]
        self.free = self.free[:len(self.free) - take]
        self.cur += n_fresh
        return fresh + tail


def test_row_placement_kat():
    # tests/optim/sparse_adamw_test.py:177-208: after insert(arange(2048)) ids 0..511
    # sit in rows 1536..2047 (first new key takes the largest fresh index)
    m = oracle.IdMap()
    rows = m.lookup(np.arange(2048))
    np.testing.assert_array_equal(rows, 2047 - np.arange(2048))
    assert sorted(rows[:512]) == list(range(1536, 2048))
    assert m.id_num() == 2048 and m.size() == 2048


def test_idmap_vs_dict_model_with_delete_and_reuse(rng):
    m = oracle.IdMap()
    model, alloc = {}, ModelAllocator()
    for step in range(40):
        ids = np.unique(rng.integers(-50, 400, size=rng.integers(0, 120)))
        got = m.lookup(ids)
        missing = [k for k in ids.tolist() if k not in model]
        for k, r in zip(missing, alloc.gen(len(missing))):
            model[k] = r
        np.testing.assert_array_equal(got, [model[k] for k in ids.tolist()])
        # read-only lookups never admit
        probe = rng.integers(-60, 500, size=50)
        ro = m.lookup_readonly(probe)
        np.testing.assert_array_equal(ro, [model.get(k, -1) for k in probe.tolist()])
        if step % 3 == 2 and model:
            keys = np.array(sorted(model))
            victims = keys[rng.random(len(keys)) < 0.3]
            rows = np.array([model[k] for k in victims.tolist()], np.int64)
            m.delete(victims, rows)
            for k in victims.tolist():
                del model[k]
            alloc.free.extend(rows.tolist())
        assert m.size() == len(model)
        assert m.id_num() == alloc.cur
        assert m.free_size() == len(alloc.free)
        sid, sidx = m.snapshot()
        assert dict(zip(sid.tolist(), sidx.tolist())) == model
    # bijection key <-> row over live keys
    assert len(set(model.values())) == len(model)


def test_idmap_free_list_crosses_block_boundary():
    # the reference chunks its free list in blocks of 10240; reuse must be seamless
    m = oracle.IdMap()
    n = 25000
    rows = m.lookup(np.arange(n))
    m.delete(np.arange(n), rows)
    again = m.lookup(np.arange(n, 2 * n))
    np.testing.assert_array_equal(again, rows)  # free_index = i -> free_list[i]
    assert m.id_num() == n
    part = m.lookup(np.arange(2 * n, 2 * n + 10))
    np.testing.assert_array_equal(part, n + 9 - np.arange(10))


def test_idmap_duplicate_in_one_call_keeps_first_insert():
    # cpu_id_map.cc:80-86: insert() does not overwrite, later indices of the batch leak
    m = oracle.IdMap()
    rows = m.lookup(np.array([7, 7, 9]))
    assert rows[0] == rows[1] == 2 and rows[2] == 0
    assert m.id_num() == 3 and m.size() == 2


# ------------------------------------------------------------------ row blocks
def _blocks(rng, nb, bs, D, dtype=np.float32):
    return [np.ascontiguousarray(rng.standard_normal((bs, D)).astype(dtype)) for _ in range(nb)]


def test_block_gather_insert_vs_slicing(rng):
    # tests/ops/block_ops_test.py:21-70
    bs, D = 7, 5
    blocks = _blocks(rng, 4, bs, D)
    flat = np.concatenate(blocks)
    ids = rng.integers(0, 4 * bs, size=33)
    np.testing.assert_array_equal(oracle.block_gather(ids, blocks, bs), flat[ids])
    np.testing.assert_array_equal(oracle.gather(ids, flat), flat[ids])
    ro = ids.copy()
    ro[::4] = -1
    got = oracle.block_gather(ro, blocks, bs, default_key=-1, readonly=True)
    exp = flat[np.maximum(ro, 0)]
    exp[ro == -1] = 0
    np.testing.assert_array_equal(got, exp)
    uids = rng.permutation(4 * bs)[:10]
    emb = rng.standard_normal((10, D)).astype(np.float32)
    oracle.block_insert(uids, emb, blocks, bs)
    flat[uids] = emb
    np.testing.assert_array_equal(np.concatenate(blocks), flat)
    oracle.block_insert(uids, emb[:1], blocks, bs)  # broadcast of one row
    flat[uids] = emb[0]
    np.testing.assert_array_equal(np.concatenate(blocks), flat)
    mask = rng.random(10) < 0.5
    emb2 = rng.standard_normal((10, D)).astype(np.float32)
    oracle.block_insert(uids, emb2, blocks, bs, mask=mask)
    flat[uids[mask]] = emb2[mask]
    np.testing.assert_array_equal(np.concatenate(blocks), flat)


def test_block_filter_predicate(rng):
    bs = 6
    for dt in (np.int64, np.int32):
        blocks = [rng.integers(0, 100, size=(bs, 1)).astype(dt) for _ in range(3)]
        flat = np.concatenate(blocks)[:, 0]
        ids = rng.integers(0, 3 * bs, size=20)
        np.testing.assert_array_equal(oracle.block_filter(ids, blocks, bs, 50), flat[ids] < 50)


# ------------------------------------------------------------------ optimizers
def _run_oracle_adam(rows0, grads, index_seq, lr, b1, b2, eps, decay, beta_dtype, bs):
    U, D = rows0.shape
    nb = (U + bs - 1) // bs
    pad = nb * bs - U
    w = np.concatenate([rows0, np.zeros((pad, D), np.float32)])
    emb = [np.ascontiguousarray(w[i * bs:(i + 1) * bs]) for i in range(nb)]
    m = [np.zeros((bs, D), np.float32) for _ in range(nb)]
    v = [np.zeros((bs, D), np.float32) for _ in range(nb)]
    b1t, b2t = np.ones(1, beta_dtype), np.ones(1, beta_dtype)
    for g, idx in zip(grads, index_seq):
        oracle.block_apply_adamw(idx, g, emb, b1t, b2t, m, v, lr, b1, b2, decay, eps, bs)
    return np.concatenate(emb)[:U], np.concatenate(m)[:U], np.concatenate(v)[:U], b1t, b2t


def test_adamw_tracks_torch_adamw(rng):
    # the construction of tests/optim/sparse_adamw_test.py:84-175: same rows updated
    # every step, dense torch.optim.AdamW as the yardstick, rtol 1e-5 / atol 1e-4
    U, D, steps = 50, 8, 30
    lr, b1, b2, eps, wd = 1e-2, 0.9, 0.999, 1e-8, 1e-2
    rows0 = rng.standard_normal((U, D)).astype(np.float32)
    grads = [rng.standard_normal((U, D)).astype(np.float32) for _ in range(steps)]
    idx = [np.arange(U) for _ in range(steps)]
    w, m, v, b1t, b2t = _run_oracle_adam(rows0, grads, idx, lr, b1, b2, eps, 1 - lr * wd, np.float32, 16)
    p = torch.nn.Parameter(torch.tensor(rows0))
    opt = torch.optim.AdamW([p], lr=lr, betas=(b1, b2), eps=eps, weight_decay=wd)
    for g in grads:
        p.grad = torch.tensor(g)
        opt.step()
    np.testing.assert_allclose(w, p.detach().numpy(), rtol=1e-5, atol=1e-4)
    st = opt.state[p]
    np.testing.assert_allclose(m, st["exp_avg"].numpy(), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(v, st["exp_avg_sq"].numpy(), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(b1t[0], b1 ** steps, rtol=1e-5)
    np.testing.assert_allclose(b2t[0], b2 ** steps, rtol=1e-5)


def test_adam_one_step_closed_form():
    # one element, from zero state: m = (1-b1) g, v = (1-b2) g^2,
    # alpha = -lr / (1-b1) * sqrt(1-b2)  =>  w' = w*decay - lr * g / (|g| + eps / sqrt(1-b2))
    g, w0, lr, b1, b2, eps, decay = 0.5, 2.0, 0.1, 0.9, 0.99, 1e-8, 0.97
    for bdt in (np.float32, np.float64):
        emb, m, v = [np.full((1, 1), w0, np.float32)], [np.zeros((1, 1), np.float32)], [np.zeros((1, 1), np.float32)]
        b1t, b2t = np.ones(1, bdt), np.ones(1, bdt)
        oracle.block_apply_adamw([0], np.full((1, 1), g, np.float32), emb, b1t, b2t, m, v, lr, b1, b2, decay, eps, 1)
        exp = w0 * decay - lr * g / (abs(g) + eps / np.sqrt(1 - b2))
        np.testing.assert_allclose(emb[0][0, 0], exp, rtol=1e-6)
        np.testing.assert_allclose(m[0][0, 0], (1 - b1) * g, rtol=1e-6)
        np.testing.assert_allclose(v[0][0, 0], (1 - b2) * g * g, rtol=1e-6)


def test_adam_untouched_rows_stay(rng):
    rows0 = rng.standard_normal((20, 4)).astype(np.float32)
    g = rng.standard_normal((5, 4)).astype(np.float32)
    idx = np.array([3, 19, 0, 7, 12])
    w, m, v, _, _ = _run_oracle_adam(rows0, [g], [idx], 1e-3, 0.9, 0.999, 1e-8, 1.0, np.float64, 6)
    untouched = np.setdiff1d(np.arange(20), idx)
    np.testing.assert_array_equal(w[untouched], rows0[untouched])
    assert np.all(m[untouched] == 0) and np.all(v[untouched] == 0)
    assert np.all(w[idx] != rows0[idx])


def test_adagrad_vs_torch_adagrad(rng):
    U, D, steps, lr, eps, bs = 40, 6, 25, 0.01, 1e-8, 16
    rows0 = (0.01 * rng.standard_normal((U, D))).astype(np.float32)
    nb = (U + bs - 1) // bs
    w = np.concatenate([rows0, np.zeros((nb * bs - U, D), np.float32)])
    emb = [np.ascontiguousarray(w[i * bs:(i + 1) * bs]) for i in range(nb)]
    acc = [np.zeros((bs, D), np.float32) for _ in range(nb)]
    p = torch.nn.Parameter(torch.tensor(rows0))
    opt = torch.optim.Adagrad([p], lr=lr, eps=eps, lr_decay=0, initial_accumulator_value=0)
    for _ in range(steps):
        idx = np.sort(rng.permutation(U)[:rng.integers(1, U)])
        g = rng.standard_normal((len(idx), D)).astype(np.float32)
        oracle.block_apply_adagrad(idx, g, emb, acc, lr, eps, bs)
        dense = np.zeros((U, D), np.float32)
        dense[idx] = g
        # dense Adagrad leaves rows with zero gradient untouched (0 / (sqrt(s) + eps) = 0)
        p.grad = torch.tensor(dense)
        opt.step()
    np.testing.assert_allclose(np.concatenate(emb)[:U], p.detach().numpy(), rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(np.concatenate(acc)[:U], opt.state[p]["sum"].numpy(), rtol=1e-6, atol=1e-7)


def test_adagrad_exact_restatement_vs_torch_adagrad_and_the_c_oracle(rng):
    """block_apply_adagrad_exact (the update with its roundings spelled out, what the kernels are held to
    bit for bit): float32 rows against torch.optim.Adagrad and against the C restatement; bfloat16
    rows hold bfloat16 values and stay within a bfloat16 step per update of the float32 rows."""
    U, D, steps, lr, eps, bs = 40, 6, 25, 0.01, 1e-8, 16
    rows0 = (0.01 * rng.standard_normal((U, D))).astype(np.float32)
    blocks = lambda w: [np.ascontiguousarray(np.concatenate([w, np.zeros((48 - U, D), np.float32)])[i * bs:(i + 1) * bs])
                        for i in range(3)]
    emb, acc = blocks(rows0), blocks(np.zeros_like(rows0))
    emb_c, acc_c = blocks(rows0), blocks(np.zeros_like(rows0))
    emb_b, acc_b = blocks(oracle.round_bf16(rows0)), blocks(np.zeros_like(rows0))
    p = torch.nn.Parameter(torch.tensor(rows0))
    opt = torch.optim.Adagrad([p], lr=lr, eps=eps, lr_decay=0, initial_accumulator_value=0)
    for _ in range(steps):
        idx = np.sort(rng.permutation(U)[:rng.integers(1, U)])
        g = rng.standard_normal((len(idx), D)).astype(np.float32)
        oracle.block_apply_adagrad_exact(idx, g, emb, acc, lr, eps, bs)
        oracle.block_apply_adagrad(idx, g, emb_c, acc_c, lr, eps, bs)
        oracle.block_apply_adagrad_exact(idx, g, emb_b, acc_b, lr, eps, bs, bf16=True)
        dense = np.zeros((U, D), np.float32)
        dense[idx] = g
        p.grad = torch.tensor(dense)
        opt.step()
    np.testing.assert_allclose(np.concatenate(emb)[:U], p.detach().numpy(), rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(np.concatenate(acc)[:U], opt.state[p]["sum"].numpy(), rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(np.concatenate(emb), np.concatenate(emb_c), rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(np.concatenate(acc), np.concatenate(acc_c), rtol=1e-6, atol=1e-7)
    for arr in (np.concatenate(emb_b), np.concatenate(acc_b)):
        np.testing.assert_array_equal(arr, oracle.round_bf16(arr))        # bfloat16 values
    # bfloat16 storage: 8 bits of mantissa, 25 updates
    np.testing.assert_allclose(np.concatenate(emb_b), np.concatenate(emb), rtol=0, atol=25 * 2.0 ** -8 * 0.05)
    np.testing.assert_allclose(np.concatenate(acc_b), np.concatenate(acc), rtol=25 * 2.0 ** -8, atol=1e-6)

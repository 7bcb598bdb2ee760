"""The CPU oracle against the reference's own CPU operators, compiled from the reference tree
(``oracle/ref_build.sh`` -> ``oracle/_ref/ref_ops``). Skipped where that binary was not built.
Integer results and the float32 optimizer arithmetic must agree bit for bit."""
import numpy as np
import pytest

import oracle
from oracle import ref_ops

pytestmark = pytest.mark.skipif(not ref_ops.available(), reason="oracle/_ref/ref_ops not built")


def _i64(*v):
    return np.asarray(v, dtype=np.int64)


# ------------------------------------------------------------------ id map + allocator
def _idmap_script(rng, steps, key_range, max_len):
    """Batches as the reference's callers form them: inserts carry distinct ids (the hashtable
    deduplicates first), deletes name ids that are present; read-only lookups are free-form."""
    codes, lens, ids = [], [], []
    live = set()
    for _ in range(steps):
        c = int(rng.choice([0, 0, 0, 1, 2]))
        n = int(rng.integers(0, max_len + 1))
        if c == 0:
            batch = np.unique(rng.integers(0, key_range, n).astype(np.int64))
            rng.shuffle(batch)
            live.update(batch.tolist())
        elif c == 1:
            batch = rng.integers(0, key_range, n).astype(np.int64)
        else:
            pool = np.asarray(sorted(live), dtype=np.int64)
            batch = rng.choice(pool, size=min(n, len(pool)), replace=False) if len(pool) else pool
            live.difference_update(batch.tolist())
        codes.append(c), lens.append(len(batch)), ids.append(batch)
    return codes, lens, ids


@pytest.mark.parametrize("seed,key_range,max_len", [(0, 50, 20), (1, 5000, 700), (2, 1 << 40, 300)])
def test_idmap_sequences_match_cpu_id_map(seed, key_range, max_len):
    # csrc/embedding/cpu_id_map.cc:73-190 with one thread: rows are handed out in input order
    rng = np.random.default_rng(seed)
    codes, lens, ids = _idmap_script(rng, 40, key_range, max_len)
    got_ref, snap_ids, snap_idx, id_num = ref_ops.run(
        "idmap", [_i64(*codes), _i64(*lens), np.concatenate(ids) if ids else _i64()])
    m = oracle.IdMap()
    outs = []
    for c, batch in zip(codes, ids):
        if c == 0:
            outs.append(m.lookup(batch))
        elif c == 1:
            outs.append(m.lookup_readonly(batch))
        else:
            idx = m.lookup_readonly(batch)
            m.delete(batch, idx)
            outs.append(idx)
    np.testing.assert_array_equal(np.concatenate(outs), got_ref)
    o_ids, o_idx = m.snapshot()
    order_o, order_r = np.argsort(o_ids), np.argsort(snap_ids)
    np.testing.assert_array_equal(o_ids[order_o], snap_ids[order_r])
    np.testing.assert_array_equal(o_idx[order_o], snap_idx[order_r])
    assert m.id_num() == int(id_num[0])


def test_allocator_gen_free_matches_id_allocator():
    # csrc/embedding/id_allocator.cc:17-60
    rng = np.random.default_rng(3)
    codes, lens, frees = [], [], []
    cur, free_list, live = 0, [], []
    exp = []
    for _ in range(30):
        if live and rng.random() < 0.4:
            k = int(rng.integers(1, len(live) + 1))
            pick = rng.choice(len(live), size=k, replace=False)
            ids = np.asarray([live[i] for i in pick], dtype=np.int64)
            live = [v for i, v in enumerate(live) if i not in set(pick.tolist())]
            codes.append(1), lens.append(k), frees.append(ids)
            free_list.extend(ids.tolist())
        else:
            n = int(rng.integers(1, 400))
            codes.append(0), lens.append(n)
            fl = np.asarray(free_list + [0], dtype=np.int64)
            out = oracle.generate_ids(n, fl, len(free_list), cur)
            take = min(n, len(free_list))
            cur += n - take
            free_list = free_list[:len(free_list) - take]
            exp.append(out)
            live.extend(out.tolist())
    got, sizes = ref_ops.run("alloc", [_i64(*codes), _i64(*lens), np.concatenate(frees) if frees else _i64(),
                                       _i64(0, 128)])
    np.testing.assert_array_equal(np.concatenate(exp), got)
    assert int(sizes[0]) == cur and int(sizes[1]) == len(live)


def test_mask_key_index_and_scatter():
    # csrc/ops/hashtable_ops.cc:150-214
    rng = np.random.default_rng(4)
    n = 5000
    keys = rng.integers(-(1 << 62), 1 << 62, n)
    mask = rng.random(n) < 0.3
    cumsum = np.cumsum(mask).astype(np.int64)
    out_size = int(cumsum[-1])
    rk, ri = ref_ops.run("mask_key_index", [keys, mask, cumsum, _i64(out_size)])
    ok, oi = oracle.mask_key_index(keys, mask, cumsum, out_size)
    np.testing.assert_array_equal(ok, rk)
    np.testing.assert_array_equal(oi, ri)
    base = rng.integers(0, 1 << 40, n)
    new = rng.integers(0, 1 << 40, out_size)
    (rs,) = ref_ops.run("scatter_ids_with_mask", [base.copy(), new, ri])
    np.testing.assert_array_equal(oracle.scatter_ids_with_mask(base, new, oi), rs)


# ------------------------------------------------------------------ row blocks
@pytest.mark.parametrize("dtype", [np.float32, np.int64])
def test_block_gather_insert_filter(dtype):
    # csrc/ops/block_ops.cc:270-397
    rng = np.random.default_rng(5)
    bs, nb, D = 64, 5, 6
    R = bs * nb
    if dtype == np.float32:
        table = rng.standard_normal((R, D)).astype(np.float32)
    else:
        table = rng.integers(-1000, 1000, (R, D)).astype(np.int64)
    blocks = lambda t: [t[i * bs:(i + 1) * bs] for i in range(nb)]
    ids = rng.integers(0, R, 300).astype(np.int64)
    (ref,) = ref_ops.run("block_gather", [ids, table, _i64(bs, -1, 0)])
    np.testing.assert_array_equal(oracle.block_gather(ids, blocks(table), bs, -1, False), ref)
    (ref,) = ref_ops.run("gather", [ids, table])
    np.testing.assert_array_equal(oracle.gather(ids, table), ref)
    ids[::7] = -1  # the default key gives rows of zeros, in read-only mode only (:61-99)
    (ref,) = ref_ops.run("block_gather", [ids, table, _i64(bs, -1, 1)])
    np.testing.assert_array_equal(oracle.block_gather(ids, blocks(table), bs, -1, True), ref)

    uniq = rng.permutation(R)[:200].astype(np.int64)
    rows = (rng.standard_normal((200, D)) * 10).astype(dtype)
    (ref,) = ref_ops.run("block_insert", [uniq, rows, table.copy(), _i64(bs)])
    mine = table.copy()
    oracle.block_insert(uniq, rows, blocks(mine), bs)
    np.testing.assert_array_equal(mine, ref)
    mask = rng.random(200) < 0.5
    (ref,) = ref_ops.run("block_insert_with_mask", [uniq, rows, mask, table.copy(), _i64(bs)])
    mine = table.copy()
    oracle.block_insert(uniq, rows, blocks(mine), bs, mask=mask)
    np.testing.assert_array_equal(mine, ref)


def test_block_filter():
    rng = np.random.default_rng(6)
    bs, nb = 32, 4
    slot = rng.integers(0, 100, (bs * nb, 1)).astype(np.int64)
    ids = rng.integers(0, bs * nb, 500).astype(np.int64)
    for thr in (0, 37, 100):
        (ref,) = ref_ops.run("block_filter", [ids, slot, _i64(bs, thr)])
        mine = oracle.block_filter(ids, [slot[i * bs:(i + 1) * bs] for i in range(nb)], bs, thr)
        np.testing.assert_array_equal(mine, ref.astype(bool))


# ------------------------------------------------------------------ optimizer
@pytest.mark.parametrize("beta_dtype", [np.float32, np.float64])
def test_block_apply_adamw_bit_exact(beta_dtype):
    # csrc/ops/block_apply_adamw_op.cc:12-130, several steps so the running beta powers matter
    rng = np.random.default_rng(7)
    bs, nb, D, T, n = 32, 3, 12, 5, 40
    R = bs * nb
    emb = rng.standard_normal((R, D)).astype(np.float32)
    m = np.zeros((R, D), np.float32)
    v = np.zeros((R, D), np.float32)
    index = np.stack([rng.permutation(R)[:n] for _ in range(T)]).astype(np.int64)
    grad = rng.standard_normal((T, n, D)).astype(np.float32)
    lr, b1, b2, wd, eps = 0.013, 0.9, 0.999, 0.01, 1e-8
    b1t, b2t = np.ones(1, beta_dtype), np.ones(1, beta_dtype)
    r_emb, r_m, r_v, r_b1t, r_b2t = ref_ops.run(
        "adamw", [index, grad, emb.copy(), m.copy(), v.copy(), b1t.copy(), b2t.copy(),
                  np.asarray([lr, b1, b2, wd, eps, bs], np.float64)])
    blocks = lambda t: [t[i * bs:(i + 1) * bs] for i in range(nb)]
    for t in range(T):
        oracle.block_apply_adamw(index[t], grad[t], blocks(emb), b1t, b2t, blocks(m), blocks(v), lr, b1, b2, wd,
                                 eps, bs)
    np.testing.assert_array_equal(b1t, r_b1t)
    np.testing.assert_array_equal(b2t, r_b2t)
    np.testing.assert_array_equal(m, r_m)
    np.testing.assert_array_equal(v, r_v)
    np.testing.assert_array_equal(emb, r_emb)


@pytest.mark.parametrize("beta_dtype", [np.float32, np.float64])
def test_block_apply_adamw_half_rows_bit_exact(beta_dtype):
    # the same functor with TEmb = at::Half (rows AND gradients float16): where the roundings fall,
    # and that `emb_elem += <double>` rounds the step to Half before it is added
    rng = np.random.default_rng(17)
    bs, nb, D, T, n = 32, 3, 12, 6, 50
    R = bs * nb
    emb = (0.5 * rng.standard_normal((R, D))).astype(np.float16)
    m = np.zeros((R, D), np.float16)
    v = np.zeros((R, D), np.float16)
    index = np.stack([rng.permutation(R)[:n] for _ in range(T)]).astype(np.int64)
    grad = rng.standard_normal((T, n, D)).astype(np.float16)
    lr, b1, b2, wd, eps = 0.013, 0.9, 0.999, 0.99, 1e-8
    b1t, b2t = np.ones(1, beta_dtype), np.ones(1, beta_dtype)
    r_emb, r_m, r_v, r_b1t, r_b2t = ref_ops.run(
        "adamw", [index, grad, emb.copy(), m.copy(), v.copy(), b1t.copy(), b2t.copy(),
                  np.asarray([lr, b1, b2, wd, eps, bs], np.float64)])
    assert r_emb.dtype == np.float16
    blocks = lambda t: [t[i * bs:(i + 1) * bs] for i in range(nb)]
    for t in range(T):
        oracle.block_apply_adamw_f16(index[t], grad[t], blocks(emb), b1t, b2t, blocks(m), blocks(v), lr, b1, b2, wd,
                                     eps, bs)
    np.testing.assert_array_equal(b1t, r_b1t)
    np.testing.assert_array_equal(m, r_m)
    np.testing.assert_array_equal(v, r_v)
    np.testing.assert_array_equal(emb, r_emb)


@pytest.mark.parametrize("beta_dtype", [np.float32, np.float64])
def test_block_apply_adamw_double_rows_bit_exact(beta_dtype):
    # the functor with TEmb = double: no rounding but sqrtf's float argument
    rng = np.random.default_rng(27)
    bs, nb, D, T, n = 32, 3, 5, 5, 50
    R = bs * nb
    emb = rng.standard_normal((R, D))
    m, v = np.zeros((R, D)), np.zeros((R, D))
    index = np.stack([rng.permutation(R)[:n] for _ in range(T)]).astype(np.int64)
    grad = rng.standard_normal((T, n, D))
    lr, b1, b2, wd, eps = 0.013, 0.9, 0.999, 0.99, 1e-8
    b1t, b2t = np.ones(1, beta_dtype), np.ones(1, beta_dtype)
    r_emb, r_m, r_v, r_b1t, r_b2t = ref_ops.run(
        "adamw", [index, grad, emb.copy(), m.copy(), v.copy(), b1t.copy(), b2t.copy(),
                  np.asarray([lr, b1, b2, wd, eps, bs], np.float64)])
    assert r_emb.dtype == np.float64
    blocks = lambda t: [t[i * bs:(i + 1) * bs] for i in range(nb)]
    for t in range(T):
        oracle.block_apply_adamw_f64(index[t], grad[t], blocks(emb), b1t, b2t, blocks(m), blocks(v), lr, b1, b2, wd,
                                     eps, bs)
    np.testing.assert_array_equal(m, r_m)
    np.testing.assert_array_equal(v, r_v)
    np.testing.assert_array_equal(emb, r_emb)


# ------------------------------------------------------------------ dedup / tagging / feature ops
def test_ids_partition_matches_cpu_op():
    # csrc/ops/ids_partition.cc:6-37. Non-negative ids: for a negative id the CPU op takes the shard
    # from |id % 65536| while the device kernel (ids_partition_kernel.cu:45-55, what the oracle
    # restates) takes it from id & 0xFFFF, so the two reference paths themselves disagree there.
    rng = np.random.default_rng(8)
    for n, parts in ((1, 1), (1000, 1), (5000, 2), (5000, 8), (777, 3), (65536 * 2, 7)):
        ids = rng.integers(0, 1 << 40, n)
        ids[rng.integers(0, n, n // 3)] = ids[0]
        ru, rc, rinv = ref_ops.run("ids_partition", [ids, _i64(parts)])
        u, c, inv = oracle.ids_partition(ids, parts)
        np.testing.assert_array_equal(np.sort(u), np.sort(ru))
        np.testing.assert_array_equal(c, rc)
        # each shard holds the same set of ids; the order inside a shard is the reference sort's
        np.testing.assert_array_equal(u[inv], ids)
        np.testing.assert_array_equal(ru[rinv], ids)
        b = np.concatenate([[0], np.cumsum(rc)])
        for p in range(parts):
            np.testing.assert_array_equal(np.sort(u[b[p]:b[p + 1]]), np.sort(ru[b[p]:b[p + 1]]))


def test_ids_encode_matches_cpu_op():
    # csrc/ops/ids_encode.cc:5-20
    rng = np.random.default_rng(9)
    lists = [rng.integers(-(1 << 62), 1 << 62, n) for n in (100, 1, 333)]
    tids = _i64(0, 5, 2047)
    (ref,) = ref_ops.run("ids_encode", [tids] + lists)
    np.testing.assert_array_equal(oracle.ids_encode(lists, tids), ref)


def test_feature_ops_match_cpu_ops():
    # csrc/ops/fused_uint64_mod.cc:5-40, fused_bucketized.cc:5-62, multi_hash.cc:4-58
    rng = np.random.default_rng(10)
    xs = [rng.integers(-(1 << 63), (1 << 63) - 1, n) for n in (257, 1000)]
    mods = _i64(1000003, 7)
    ref = ref_ops.run("fused_uint64_mod", [mods] + xs)
    for x, md, r in zip(xs, mods, ref):
        np.testing.assert_array_equal(oracle.uint64_mod(x, md), r)

    vals = [rng.standard_normal(500).astype(np.float32), np.asarray([0.0, 1.0, 2.0, -1.0, np.nan, np.inf], np.float32)]
    bounds = [np.sort(rng.standard_normal(17)).astype(np.float32), np.asarray([0.0, 1.0, 1.0, 2.0], np.float32)]
    ref = ref_ops.run("fused_bucketized", vals + bounds)
    for x, b, r in zip(vals, bounds, ref):
        np.testing.assert_array_equal(oracle.bucketize(x, b), r)

    xs = [rng.integers(-(1 << 31), 1 << 31, 400), rng.integers(0, 1 << 20, 90)]
    muls = [_i64(31, 131, 1313), _i64(7)]
    primes = [_i64(1000003, 998244353, 10007), _i64(97)]
    bks = [_i64(1000, 5000, 77), _i64(10)]
    ref = ref_ops.run("fused_multi_hash", xs + muls + primes + bks)
    k = 0
    for x, mu, pr, bk in zip(xs, muls, primes, bks):
        for o in oracle.multi_hash(x, mu, pr, bk):
            np.testing.assert_array_equal(o, ref[k])
            k += 1


# ------------------------------------------------------------------ table + sparse optimizers, end to end
@pytest.mark.parametrize("kind,beta_dtype,decay_of", [
    (0, np.float64, lambda lr, wd: 1.0),            # SparseAdam ignores weight_decay (adam.cc:70-73)
    (1, np.float32, lambda lr, wd: 1.0 - lr * wd),  # SparseAdamW (adamw.cc:64)
    (2, np.float32, lambda lr, wd: 1.0 - wd),       # SparseAdamWTF (adamw_tf.cc:64)
])
def test_table_training_script_matches_hashtable_and_optimizers(kind, beta_dtype, decay_of):
    # csrc/embedding/hashtable.cc:46-278 + adam*.cc::step on a CPU table: lookups that grow the table
    # across block boundaries, accumulated gradients, deletes that recycle rows, read-only lookups
    from oracle import cpu_path

    rng = np.random.default_rng(20 + kind)
    bs, D, init = 64, 8, 0.25
    lr, b1, b2, eps, wd = 0.02, 0.9, 0.999, 1e-8, 0.05
    codes, lens, ids, grads = [], [], [], []
    live = []
    for step in range(12):
        batch = np.unique(rng.integers(0, 600, int(rng.integers(1, 200)))).astype(np.int64)
        rng.shuffle(batch)
        live = sorted(set(live) | set(batch.tolist()))
        codes += [0, 1]
        lens += [len(batch), 0]
        ids.append(batch)
        grads.append(rng.standard_normal((len(batch), D)).astype(np.float32))
        if step % 3 == 1:
            ro = rng.integers(0, 700, 50).astype(np.int64)
            codes.append(3), lens.append(len(ro)), ids.append(ro)
        if step % 4 == 2:
            gone = rng.choice(np.asarray(live, np.int64), size=len(live) // 3, replace=False)
            live = sorted(set(live) - set(gone.tolist()))
            codes.append(2), lens.append(len(gone)), ids.append(gone)
    r_idx, r_emb, r_ids, r_rows, r_w, r_m, r_v = ref_ops.run("table_train", [
        np.asarray([bs, D, kind, lr, b1, b2, eps, wd, init, 1], np.float64), _i64(*codes), _i64(*lens),
        np.concatenate(ids), np.concatenate(grads)])

    t = cpu_path.CpuTable(D, bs, lambda b: np.full((bs, D), init, np.float32), "adam", lr, eps, b1, b2,
                          decay_of(lr, wd), beta_dtype)
    idx_out, emb_out = [], []
    it_ids, it_grads = iter(ids), iter(grads)
    pending = None
    for c in codes:
        if c == 0:
            batch = next(it_ids)
            index, rows = t.lookup(batch)
            idx_out.append(index), emb_out.append(rows)
            pending = (index, next(it_grads))
        elif c == 1:
            t.apply(*pending)
        elif c == 3:
            batch = next(it_ids)
            index = t.idmap.lookup_readonly(batch)
            t._grow()
            idx_out.append(index), emb_out.append(oracle.block_gather(index, t.emb, bs, -1, True))
        else:
            batch = next(it_ids)
            index = t.idmap.lookup_readonly(batch)
            t.idmap.delete(batch, index)
            # every slot of a freed row goes back to its initial value (slot_group.cc:153-160)
            oracle.block_insert(index, np.full((len(batch), D), init, np.float32), t.emb, bs)
            oracle.block_insert(index, np.zeros((len(batch), D), np.float32), t.s0, bs)
            oracle.block_insert(index, np.zeros((len(batch), D), np.float32), t.s1, bs)
    np.testing.assert_array_equal(np.concatenate(idx_out), r_idx)
    np.testing.assert_array_equal(np.concatenate(emb_out), r_emb)
    o_ids, o_rows = t.idmap.snapshot()
    np.testing.assert_array_equal(o_rows[np.argsort(o_ids)], r_rows[np.argsort(r_ids)])
    np.testing.assert_array_equal(np.sort(o_ids), np.sort(r_ids))
    np.testing.assert_array_equal(np.concatenate(t.emb), r_w)
    np.testing.assert_array_equal(np.concatenate(t.s0), r_m)
    np.testing.assert_array_equal(np.concatenate(t.s1), r_v)


def test_dense_to_ragged_matches_cpu_op():
    # csrc/ops/dense_to_ragged.cc:6-53
    rng = np.random.default_rng(30)
    for dtype in (np.float32, np.int32, np.int64, np.float64):
        data = rng.integers(0, 3, (200, 17)).astype(dtype)
        data[5] = 0
        for invalid in (0, 2):
            rv, ro = ref_ops.run("dense_to_ragged", [data, np.asarray([invalid], dtype)])
            v, o = oracle.dense_to_ragged(data, invalid)
            np.testing.assert_array_equal(v, rv)
            np.testing.assert_array_equal(o, ro)
            assert ro.dtype == np.int32


def test_round_bf16_is_torchs_conversion():
    """oracle.round_bf16 (what block_apply_adamw_bf16 adds to the Half restatement the compiled reference
    pins) against torch's float32 -> bfloat16 on the CPU: random magnitudes, exact ties between two
    neighbours (both parities), subnormals, the largest floats, infinities, NaN."""
    import torch

    rng = np.random.default_rng(11)
    with np.errstate(over="ignore", invalid="ignore"):
        x = (rng.standard_normal(200000) * 10.0 ** rng.integers(-44, 39, 200000)).astype(np.float32)
    ties = ((rng.integers(0, 1 << 16, 100000).astype(np.uint32) << 16) | np.uint32(0x8000)).view(np.float32)
    edge = np.array([0.0, -0.0, np.inf, -np.inf, 1e-45, -1e-45, 3.4e38, -3.4e38, 3.3895e38, 1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -9,
                     1.00390625, 65504.0], np.float32)
    x = np.concatenate([x, ties, edge])
    x = x[~np.isnan(x)]
    got = oracle.round_bf16(x)
    exp = torch.from_numpy(x).to(torch.bfloat16).float().numpy()
    np.testing.assert_array_equal(got.view(np.uint32), exp.view(np.uint32))
    assert np.isnan(oracle.round_bf16(np.array([np.nan, 1.0], np.float32))[0])
    assert got.dtype == np.float32

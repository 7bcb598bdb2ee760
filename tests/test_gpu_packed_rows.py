"""Rows a pitch apart: every entry point that takes a block list gives, on slots that share one
allocation (row r = emb | state 0 | state 1 back to back), bit for bit what it gives on one array
per slot, and a table whose optimizer packs its state (RECIS_PACKED_STATE=1) keeps answering
values() / lookups as before and trains to the same rows. The one-array-per-slot results are the ones the other test files hold
against the oracle."""
import numpy as np
import pytest
import torch

from recis_amd import _lib, ops
from recis_amd.nn import initializers as I

pytestmark = pytest.mark.gpu


def _dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _packed(*slots):
    """The block lists `slots` (same geometry) as strided views of one allocation per block; also
    the allocations, so that a test can see nothing beside the rows was written."""
    nb, (rows, D) = len(slots[0]), slots[0][0].shape
    stores = [torch.full((rows, len(slots) * D), 7, dtype=slots[0][0].dtype, device="cuda") for _ in range(nb)]
    views = []
    for g, blocks in enumerate(slots):
        vs = []
        for b, store in zip(blocks, stores):
            v = store[:, g * D:(g + 1) * D]
            v.copy_(b)
            vs.append(v)
        views.append(vs)
    return views, stores


def _same(packed_views, plain):
    for vs, bs in zip(packed_views, plain):
        for v, b in zip(vs, bs):
            assert torch.equal(v, b)


@pytest.mark.parametrize("dtype,D", [(torch.float32, 16), (torch.float32, 5), (torch.bfloat16, 128), (torch.float16, 24)])
def test_block_gather_and_insert_on_packed_rows(rng, dtype, D):
    bs, nb = 37, 5
    a = [torch.randn(bs, D, device="cuda").to(dtype) for _ in range(nb)]
    b = [torch.randn(bs, D, device="cuda").to(dtype) for _ in range(nb)]
    (pa, pb), stores = _packed(a, b)
    ids = torch.from_numpy(rng.integers(0, bs * nb, size=500)).cuda()
    for plain, packed in ((a, pa), (b, pb)):
        assert torch.equal(ops.block_gather(ids, packed, bs, -1, False), ops.block_gather(ids, plain, bs, -1, False))
        ro = ids.clone()
        ro[::3] = -1
        assert torch.equal(ops.block_gather(ro, packed, bs, -1, True), ops.block_gather(ro, plain, bs, -1, True))
    uids = torch.from_numpy(rng.permutation(bs * nb)[:60]).cuda()
    emb = torch.randn(60, D, device="cuda").to(dtype)
    mask = torch.from_numpy(rng.random(60) < 0.5).cuda()
    for plain, packed in ((a, pa), (b, pb)):
        ops.block_insert(uids, emb, plain, bs)
        ops.block_insert(uids, emb, packed, bs)
        _same((pa, pb), (a, b))
        ops.block_insert(uids[:7], emb[:1], plain, bs)
        ops.block_insert(uids[:7], emb[:1], packed, bs)
        ops.block_insert_with_mask(uids, -emb, mask, plain, bs)
        ops.block_insert_with_mask(uids, -emb, mask, packed, bs)
        _same((pa, pb), (a, b))
    assert _lib.poll_device_errors() == 0


@pytest.mark.parametrize("D,row_dtype,grad_dtype", [(16, torch.float32, torch.float32), (7, torch.float32, torch.float32),
                                                    (128, torch.bfloat16, torch.bfloat16), (32, torch.float16, torch.float32)])
def test_row_updates_on_packed_rows(rng, D, row_dtype, grad_dtype):
    bs, nb, U = 64, 4, 200
    mk = lambda: [torch.rand(bs, D, device="cuda").to(row_dtype) for _ in range(nb)]
    emb, m, v = mk(), mk(), mk()
    (pe, pm, pv), _ = _packed(emb, m, v)
    b1, b2 = torch.ones(1, device="cuda"), torch.ones(1, device="cuda")
    b1p, b2p = b1.clone(), b2.clone()
    for _ in range(3):
        idx = torch.from_numpy(np.sort(rng.permutation(bs * nb)[:U])).cuda()
        g = torch.randn(U, D, device="cuda").to(grad_dtype)
        ops.block_apply_adamw(idx, g, emb, b1, b2, None, m, v, 1e-2, 0.9, 0.999, 0.99, 1e-8, bs)
        ops.block_apply_adamw(idx, g, pe, b1p, b2p, None, pm, pv, 1e-2, 0.9, 0.999, 0.99, 1e-8, bs)
    _same((pe, pm, pv), (emb, m, v))
    assert torch.equal(b1, b1p) and torch.equal(b2, b2p)
    acc = mk()   # (non-negative, as an Adagrad accumulator is)
    (qe, qa), stores = _packed(emb, acc)
    for _ in range(2):
        idx = torch.from_numpy(np.sort(rng.permutation(bs * nb)[:U])).cuda()
        g = torch.randn(U, D, device="cuda").to(grad_dtype)
        ops.block_apply_adagrad(idx, g, emb, acc, 1e-2, 1e-8, bs)
        ops.block_apply_adagrad(idx, g, qe, qa, 1e-2, 1e-8, bs)
    _same((qe, qa), (emb, acc))
    # slots of one call at different pitches are refused
    with pytest.raises(ValueError, match="pitch"):
        ops.block_apply_adagrad(idx, g, qe, m, 1e-2, 1e-8, bs)
    assert _lib.poll_device_errors() == 0


@pytest.mark.parametrize("kind", ["adamw", "adagrad"])
@pytest.mark.parametrize("D,row_dtype", [(16, torch.float32), (128, torch.bfloat16), (40, torch.float32)])
def test_fused_gather_reduce_updates_on_packed_rows(rng, kind, D, row_dtype):
    """One-input and two-input gather-reduce + row update: hot work items, rows the table does not
    hold, two steps; the allocations hold nothing but what the plain slots hold."""
    n, bs, nb = 90000, 4096, 5
    ids = np.where(rng.random(n) < 0.3, rng.integers(0, 6, size=n), rng.integers(0, 15000, size=n))
    plan = ops.ids_unique_plan(_dev(ids))
    U = plan.U
    src = torch.arange(n, dtype=torch.int32, device="cuda")
    src2 = torch.from_numpy(rng.permutation(n).astype(np.int32)).cuda()
    src2[::5] = -1
    grads = torch.randn(n, D, device="cuda").to(row_dtype)
    coef = torch.rand(n, device="cuda")
    row_index = torch.from_numpy(rng.permutation(bs * nb)[:U]).cuda()
    row_index[::17] = -1
    mk = lambda: [torch.rand(bs, D, device="cuda").to(row_dtype) for _ in range(nb)]
    emb, s0, s1 = mk(), mk(), mk()
    b1, b2 = torch.tensor([0.9], device="cuda", dtype=torch.float64), torch.tensor([0.999], device="cuda", dtype=torch.float64)
    b1p, b2p = b1.clone(), b2.clone()
    if kind == "adamw":
        (pe, p0, p1), stores = _packed(emb, s0, s1)
    else:
        (pe, p0), stores = _packed(emb, s0)
    first, second = (grads, src, coef), (grads, src2, None)
    for _ in range(2):
        if kind == "adamw":
            ops.csr_gather_reduce_adamw(grads, plan, src, coef, row_index, emb, b1, b2, s0, s1, 1e-2, 0.9, 0.999, 0.99, 1e-8, bs)
            ops.csr_gather_reduce_adamw(grads, plan, src, coef, row_index, pe, b1p, b2p, p0, p1, 1e-2, 0.9, 0.999, 0.99, 1e-8, bs)
            ops.csr_gather_reduce2_adamw(plan, first, second, row_index, emb, b1, b2, s0, s1, 1e-2, 0.9, 0.999, 0.99, 1e-8, bs)
            ops.csr_gather_reduce2_adamw(plan, first, second, row_index, pe, b1p, b2p, p0, p1, 1e-2, 0.9, 0.999, 0.99, 1e-8, bs)
        else:
            ops.csr_gather_reduce_adagrad(grads, plan, src, coef, row_index, emb, s0, 1e-2, 1e-8, bs)
            ops.csr_gather_reduce_adagrad(grads, plan, src, coef, row_index, pe, p0, 1e-2, 1e-8, bs)
            ops.csr_gather_reduce2_adagrad(plan, first, second, row_index, emb, s0, 1e-2, 1e-8, bs)
            ops.csr_gather_reduce2_adagrad(plan, first, second, row_index, pe, p0, 1e-2, 1e-8, bs)
    if kind == "adamw":
        _same((pe, p0, p1), (emb, s0, s1))
        assert torch.equal(b1, b1p) and torch.equal(b2, b2p)
        for store, e, a, b in zip(stores, emb, s0, s1):
            assert torch.equal(store, torch.cat([e, a, b], 1))
    else:
        _same((pe, p0), (emb, s0))
        for store, e, a in zip(stores, emb, s0):
            assert torch.equal(store, torch.cat([e, a], 1))
    assert _lib.poll_device_errors() == 0


@pytest.mark.parametrize("D,dtype", [(16, torch.float32), (128, torch.bfloat16), (6, torch.float32)])
def test_expand_and_pooling_read_packed_rows(rng, D, dtype):
    n, bs, nb = 50000, 2048, 4
    ids = np.where(rng.random(n) < 0.3, rng.integers(0, 4, size=n), rng.integers(0, 7000, size=n))
    plan = ops.ids_unique_plan(_dev(ids))
    U = plan.U
    emb = [torch.randn(bs, D, device="cuda").to(dtype) for _ in range(nb)]
    other = [torch.randn(bs, D, device="cuda").to(dtype) for _ in range(nb)]
    (pe, _), _ = _packed(emb, other)
    row_index = torch.from_numpy(rng.permutation(bs * nb)[:U]).cuda()
    row_index[::13] = -1
    weight = torch.rand(n, device="cuda")
    stamps = [torch.zeros(bs, 1, dtype=torch.int64, device="cuda") for _ in range(nb)]
    stamps_p = [s.clone() for s in stamps]
    step = torch.tensor([41], dtype=torch.int64, device="cuda")
    a = ops.plan_expand_rows(plan, n, blocks=emb, block_size=bs, row_index=row_index, weight=weight, stamp=(stamps, step))
    b = ops.plan_expand_rows(plan, n, blocks=pe, block_size=bs, row_index=row_index, weight=weight, stamp=(stamps_p, step))
    assert torch.equal(a, b)
    for s, sp in zip(stamps, stamps_p):
        assert torch.equal(s, sp)
    S = 9000
    off = np.sort(rng.integers(0, n + 1, size=S - 1))
    off = _dev(np.concatenate([[0], off, [n]]).astype(np.int64))
    for mode in ("sum", "mean", "tile"):
        x = ops.segment_reduce_forward_blocks(emb, bs, row_index, weight, plan.inverse, off, mode)
        y = ops.segment_reduce_forward_blocks(pe, bs, row_index, weight, plan.inverse, off, mode)
        assert torch.equal(x, y)
    assert _lib.poll_device_errors() == 0


def test_a_pitch_that_does_not_fit_is_refused():
    lib, i64 = _lib.lib(), _lib.i64
    blocks = [torch.zeros(8, 16, device="cuda")]
    tab = ops.block_ptr_table(blocks)
    ids = torch.zeros(4, dtype=torch.int64, device="cuda")
    out = torch.zeros(4, 16, device="cuda")
    # rows moved as bytes: any pitch that holds a row will do (the vector width follows it)
    rc = lib.recis_block_gather(_lib.ptr(ids), _lib.ptr(tab), i64(1), i64(8), i64(32), i64(-1), 0, _lib.ptr(out),
                                i64(4), i64(64), _lib.stream_ptr(out.device))
    assert rc == 1   # RECIS_ERR_ARG: narrower than a row
    # typed rows: a multiple of the element size and of the vector the row width allows
    import ctypes
    g = torch.zeros(4, 16, device="cuda")
    for pitch in (32, 66, 64 + 4):
        rc = lib.recis_block_apply_adagrad(_lib.ptr(ids), _lib.ptr(g), _lib.dtype_code(g.dtype), _lib.ptr(tab), _lib.ptr(tab),
                                           i64(1), i64(8), i64(pitch), _lib.dtype_code(g.dtype), ctypes.c_double(0.1),
                                           ctypes.c_double(1e-8), i64(4), i64(16), _lib.stream_ptr(out.device))
        assert rc == 1, pitch
    assert b"pitch" in lib.recis_hip_last_error()


# ------------------------------------------------------------------------------ the table
def test_optimizer_state_shares_the_embedding_rows_allocation(rng, monkeypatch):
    from recis_amd.nn.modules.hashtable import HashTable
    from recis_amd.optim import SparseAdam
    D = 16
    monkeypatch.setenv("RECIS_PACKED_STATE", "1")
    table = HashTable([D], block_size=128, dtype=torch.float32, device=torch.device("cuda"), name="packed_t",
                      initializer=I.TruncNormalInitializer(std=0.02))
    ids = _dev(rng.integers(0, 10**12, size=700))
    before = table(ids).detach().clone()          # rows exist before the optimizer attaches its state
    impl = table._hashtable_impl
    sg = impl.slot_group()
    chunk0, _ = sg.emb_slot().kernel_blocks()
    assert chunk0[0].is_contiguous()
    opt = SparseAdam({"packed_t": table._hashtable_impl}, lr=1e-2)
    names = [s for s in ("sparse_adam_exp_avg", "sparse_adam_exp_avg_sq") if sg.has_slot(s)]
    assert len(names) == 2
    chunks, chunk_rows = sg.emb_slot().kernel_blocks()
    m_chunks, _ = sg.slot_by_name(names[0]).kernel_blocks()
    v_chunks, _ = sg.slot_by_name(names[1]).kernel_blocks()
    assert chunks[0].stride(0) == 3 * D and m_chunks[0].stride(0) == 3 * D
    assert m_chunks[0].data_ptr() == chunks[0].data_ptr() + 4 * D and v_chunks[0].data_ptr() == chunks[0].data_ptr() + 8 * D
    assert torch.equal(table(ids).detach(), before)  # the rows moved with their values
    assert all(float(c.abs().max()) == 0 for c in m_chunks + v_chunks)
    # growth keeps the layout; values() still hands out [block_size, D] blocks that alias the table
    more = _dev(rng.integers(0, 10**12, size=5000))
    out = table(more)
    out.sum().backward()
    opt.step()
    chunks, _ = sg.emb_slot().kernel_blocks()
    assert len(chunks) >= 1 and all(c.stride(0) == 3 * D for c in chunks)
    vals = sg.emb_slot().values()
    assert all(tuple(v.shape) == (128, D) for v in vals)
    vals[0][3].fill_(9.0)
    assert float(sg.emb_slot().index_select(torch.tensor([3], device="cuda"))[0, 0]) == 9.0
    assert torch.equal(sg.emb_slot().value()[:128], vals[0])
    assert float(torch.cat([m.reshape(-1, D) for m in sg.slot_by_name(names[0]).values()]).abs().max()) > 0
    # one allocation per slot unless asked
    monkeypatch.delenv("RECIS_PACKED_STATE")
    plain = HashTable([D], block_size=128, dtype=torch.float32, device=torch.device("cuda"), name="plain_t")
    plain(ids)
    SparseAdam({"plain_t": plain._hashtable_impl}, lr=1e-2)
    c, _ = plain._hashtable_impl.slot_group().emb_slot().kernel_blocks()
    assert c[0].is_contiguous()


@pytest.mark.parametrize("opt_name", ["SparseAdam", "SparseAdamW", "SparseAdagrad"])
def test_training_on_packed_rows_equals_one_allocation_per_slot(rng, monkeypatch, opt_name):
    """The same seeded steps on a table with packed state and on one with an allocation per slot:
    rows and state bit for bit (the arithmetic does not depend on where the rows lie)."""
    import recis_amd.optim as optim
    from recis_amd.nn.modules.hashtable import HashTable
    D = 16
    batches = [_dev(np.where(rng.random(4000) < 0.3, rng.integers(0, 5, 4000), rng.integers(0, 3000, 4000))) for _ in range(4)]
    # multiples of 1/64: the sums over an id's occurrences are exact in whatever order the plan lists them
    grads = [torch.randint(-8, 9, (4000, D), device="cuda").float() / 64 for _ in batches]
    results = []
    for knob in ("1", "0"):
        monkeypatch.setenv("RECIS_PACKED_STATE", knob)
        table = HashTable([D], block_size=256, dtype=torch.float32, device=torch.device("cuda"), name=opt_name + knob,
                          initializer=I.ConstantInitializer(0.05))
        opt = getattr(optim, opt_name)({opt_name + knob: table._hashtable_impl}, lr=1e-2)
        for ids, g in zip(batches, grads):
            table(ids).backward(g)
            opt.step()
        sg = table._hashtable_impl.slot_group()
        chunks, _ = sg.emb_slot().kernel_blocks()
        assert chunks[0].is_contiguous() == (knob == "0")
        keys, index = table._hashtable_impl.ids_map()
        order = torch.argsort(keys)
        rows = {"embedding": sg.emb_slot().index_select(index[order])}
        for s in sg.slots():
            if s.name().startswith("sparse_"):
                rows[s.name()] = s.index_select(index[order])
        results.append((keys[order], rows))
    assert torch.equal(results[0][0], results[1][0])
    assert results[0][1].keys() == results[1][1].keys() and len(results[0][1]) >= 2
    for name in results[0][1]:
        assert torch.equal(results[0][1][name], results[1][1][name]), name
    assert _lib.poll_device_errors() == 0

"""The benchmark workloads at their full sizes, checked through properties that do not need a
CPU pass over the whole input: the dedup plan is a bijection onto the distinct ids, pooled rows
are the table's rows, the per-row gradients sum to the incoming gradients and agree with a direct
index_add, the optimizer step on a sample of rows equals the CPU oracle bit for bit, new keys get
rows nobody holds. They run the stages of ``bench.py``'s workload classes, so they also check that
the timed step computes what it is meant to."""
import numpy as np
import pytest
import torch

import oracle
import workloads
from recis_amd import _lib, ops

pytestmark = pytest.mark.gpu


def _rows_of(table, index):
    chunks, chunk_rows = table.emb_blocks()
    return ops.block_gather(index, chunks, chunk_rows, -1, True)


def _slot_rows(table, name, index):
    return table.get_slot(name).index_select(index)


def test_config4_step_properties():
    import bench

    wl = bench.Config4()
    for _ in range(2):          # second step: all keys known, rows and Adam state not trivial
        wl.step()
    cols = wl.feature_ops()                       # the 39 id columns; the plan tags them as it reads them
    ids = ops.ids_encode(cols, wl.tags)           # what the plan sees
    N, D = wl.N, wl.D
    assert ids.numel() == N == 39 * 65536
    # feature ops against their definitions on a full column
    d0 = wl.c["dense"][0]
    exp_bucket = torch.bucketize(d0, wl.c["boundaries"][0], right=True) % wl.c["mod"]
    tag = 26
    assert torch.equal(ids[26 * 65536: 27 * 65536], exp_bucket | (tag << 52))
    assert torch.equal(ids[: 65536], wl.c["sparse"][0] & ((1 << 52) - 1))

    plan, _ = wl.dedup(cols)         # tagging + dedup + find-or-insert in one pass; inverse derived from the lists
    inv = plan.inverse
    uniq = plan.unique
    U = plan.U
    assert torch.equal(uniq[inv.long()], ids)                      # inverse maps every id to itself
    assert torch.unique(uniq).numel() == U == torch.unique(ids).numel()
    rs = plan.row_start[: U + 1].long()
    assert int(rs[0]) == 0 and int(rs[-1]) == N and bool((rs[1:] > rs[:-1]).all())
    occ = plan.occ.long()
    assert torch.equal(torch.sort(occ).values, torch.arange(N, device="cuda"))   # every occurrence listed once
    owner = torch.repeat_interleave(torch.arange(U, device="cuda"), rs[1:] - rs[:-1])
    assert torch.equal(inv.long()[occ], owner)                     # and under its own id

    index = wl.lookup(plan)[:U]
    assert torch.equal(index, wl.table.lookup_index_readonly(uniq[:U]))
    assert torch.unique(index).numel() == U and int(index.min()) >= 0

    pooled = wl.pool_fwd(index, inv)
    assert torch.equal(pooled, _rows_of(wl.table, index)[inv.long()])   # one id per segment: its row

    g = wl.pool_bwd(inv)
    ref = torch.zeros(U, D, device="cuda", dtype=torch.float64).index_add_(0, inv.long(), wl.grad_out.double())
    scale = torch.zeros(U, device="cuda", dtype=torch.float64).index_add_(
        0, inv.long(), wl.grad_out.double().abs().sum(1)).clamp_(min=1.0)
    assert float(((g.double() - ref).abs().sum(1) / scale).max()) < 1e-5
    torch.testing.assert_close(g.double().sum(0), wl.grad_out.double().sum(0), rtol=1e-6, atol=1e-3)

    # the fused backward + Adam step on a sample of rows against the CPU oracle's Adam on the gradient rows checked
    # above, bit for bit
    pick = torch.randperm(U, device="cuda")[:4096]
    rows = index[pick]
    names = [s.name() for s in wl.table.slot_group().slots()]
    before = [_slot_rows(wl.table, n, rows).cpu().numpy() for n in names[:3]]
    state = wl.opt.state_dict()[1]
    b1t = [v for k, v in state.items() if k.endswith("beta1")][0].cpu().numpy().copy().reshape(1)
    b2t = [v for k, v in state.items() if k.endswith("beta2")][0].cpu().numpy().copy().reshape(1)
    wl.bwd_update(index)     # what the timed step runs: gradient sum and Adam in one launch (g is not used by it)
    after = [_slot_rows(wl.table, n, rows).cpu().numpy() for n in names[:3]]
    w, m, v = [b.copy() for b in before]
    oracle.block_apply_adamw(np.arange(4096), g[pick].cpu().numpy(), [w], b1t, b2t, [m], [v], 1e-3, 0.9, 0.999, 1.0,
                             1e-8, 4096)
    for got, exp in zip(after, (w, m, v)):
        np.testing.assert_array_equal(got, exp)
    assert _lib.poll_device_errors() == 0


@pytest.mark.parametrize("resident", [20_000_000, 200_000_000])
def test_config3_lookups_at_scale(resident):
    """Config 3 with the full per-step lookup size, at a tenth of its resident set and at the full
    2e8 rows (77 GB of rows and optimizer state, a 2^29-slot id map, 29 GB per slot in one
    allocation, row addresses past 2^32 bytes): known keys keep their rows, never-seen keys get
    rows nobody holds, the expansion gives every lookup its key's row, eviction removes exactly the
    keys not seen."""
    import bench

    wl = bench.Config3(resident=resident, ids_per_step=2_000_000, n_batches=3)
    t = wl.table
    lv0, idn0, _, _ = t.id_map_stats()
    assert lv0 == resident
    ids = wl.batches[0]
    known = t.lookup_index_readonly(ids)
    n_new = int(torch.unique(ids[known < 0]).numel())
    assert 0.05 * ids.numel() < n_new <= 0.1 * ids.numel() + 1
    # step 0 stage by stage (what wl.step() runs), with a look at the table between the stages
    untouched_keys = workloads.splitmix64_torch(torch.arange(resident - 4096, resident, device="cuda"))
    untouched_keys = untouched_keys[~torch.isin(untouched_keys, ids)]
    wl.step_no += 1
    plan = wl.plan_of(ids)
    out = wl.expand(plan)
    U = plan.U
    index = plan.index_buf[:U]
    # the gradient of every unique key, summed over its lookups on the plan the update will use, against a
    # float64 index_add_ over the plan's inverse
    g = ops.csr_gather_reduce(wl.grad_out, plan, plan.occ, cover=wl.span)
    inv = plan.inverse.long()
    assert torch.equal(plan.unique[inv], ids)
    ref = torch.zeros(U, wl.D, device="cuda", dtype=torch.float64).index_add_(0, inv, wl.grad_out.double())
    scale = torch.zeros(U, device="cuda", dtype=torch.float64).index_add_(
        0, inv, wl.grad_out.double().abs().sum(1)).clamp_(min=1.0)
    assert float(((g.double() - ref).abs().sum(1) / scale).max()) < 1e-5
    del ref, scale, inv
    # the fused gather-reduce + Adam on 4096 sampled keys (rows anywhere in the 29 GB slots) against the CPU
    # oracle's Adam on those gradient rows, bit for bit
    pick = torch.randperm(U, device="cuda")[:4096]
    rows = index[pick]
    names = ["embedding", "sparse_adam_exp_avg", "sparse_adam_exp_avg_sq"]
    before = [_slot_rows(t, n, rows).cpu().numpy() for n in names]
    state = wl.opt.state_dict()[1]
    b1t = state["sparse_adam_beta1"].cpu().numpy().copy().reshape(1)
    b2t = state["sparse_adam_beta2"].cpu().numpy().copy().reshape(1)
    wl.update(plan)
    wl.step_t += 1
    wl.settle(plan)
    after = [_slot_rows(t, n, rows).cpu().numpy() for n in names]
    w, m, v = [b.copy() for b in before]
    oracle.block_apply_adamw(np.arange(4096), g[pick].cpu().numpy(), [w], b1t, b2t, [m], [v], 1e-3, 0.9, 0.999, 1.0,
                             1e-8, 4096)
    for name, got, exp in zip(names, after, (w, m, v)):
        np.testing.assert_array_equal(got, exp, err_msg=name)
    # the stamps the expansion wrote: the step (0) at every looked-up row, the initial -1 elsewhere
    assert bool((_slot_rows(t, "step_filter", index) == 0).all())
    assert bool((_slot_rows(t, "step_filter", t.lookup_index_readonly(untouched_keys)) == -1).all())
    del g
    lv1, idn1, _, _ = t.id_map_stats()
    assert lv1 == lv0 + n_new and idn1 == idn0 + n_new
    now = t.lookup_index_readonly(ids)
    assert int(now.min()) >= 0
    assert torch.equal(now[known >= 0], known[known >= 0])     # known keys keep their rows
    fresh = torch.unique(now[known < 0])
    assert fresh.numel() == n_new and int(fresh.min()) >= idn0  # new keys: rows above the old mark
    # one output row per lookup = that key's row as it was read in the step (Adam moved it since):
    # rows of equal keys are equal, rows of a sample agree with the table up to one Adam step
    order = torch.argsort(ids, stable=True)
    same = ids[order][1:] == ids[order][:-1]
    assert torch.equal(out[order][1:][same], out[order][:-1][same])
    drift = (out - _rows_of(t, now)).abs().max()
    assert 0 < float(drift) < 0.02                             # lr 1e-3, a few steps at most
    # eviction by last-seen step: everything not touched in step 0 is older than the threshold
    wl.step_t.fill_(5)
    wl.step()                                                  # batch 1 stamped with step 5
    seen = torch.unique(wl.batches[1])
    live_before = t.id_map_stats()[0]
    gone_ids, gone_rows = t.evict_older("step_filter", 5)
    lv2 = t.id_map_stats()[0]
    assert lv2 == seen.numel() and gone_ids.numel() == live_before - lv2 == gone_rows.numel()
    assert int(t.lookup_index_readonly(seen).min()) >= 0
    assert int(t.lookup_index_readonly(gone_ids[:100000]).max()) == -1
    assert _lib.poll_device_errors() == 0
    del wl, t
    torch.cuda.empty_cache()


def test_config5_step_properties():
    import bench

    wl = bench.Config5()
    wl.step()
    o = ops
    ids = o.ids_encode([f["values"] for f in wl.fields], list(range(len(wl.fields))))
    plan = o.ids_unique_plan(ids)
    inv, U = plan.inverse.long(), plan.U
    assert torch.equal(plan.unique[inv], ids)
    index = wl.table.lookup_index_readonly(plan.unique[:U])
    assert int(index.min()) >= 0
    rows = _rows_of(wl.table, index)                            # bf16 [U, 128]
    off = wl.offsets.long()
    assert int(off[-1]) == wl.N and off.numel() == wl.S + 1
    pooled = o.segment_reduce_forward(rows, None, plan.inverse, wl.offsets, "mean", out_dtype=torch.float32)
    lens = (off[1:] - off[:-1])
    seg = torch.repeat_interleave(torch.arange(wl.S, device="cuda"), lens)
    ref = torch.zeros(wl.S, wl.D, device="cuda", dtype=torch.float64).index_add_(0, seg, rows[inv].double())
    ref /= lens.clamp(min=1).view(-1, 1)
    torch.testing.assert_close(pooled.double(), ref, rtol=1e-5, atol=1e-6)
    # the padded gather: position t of sample b of field f holds the row of its t-th id, zeros past its length
    padded, _ = o.ragged_tile(wl.batch, wl.seq, plan.inverse, wl.offsets, rows)
    assert padded.shape == (wl.pad_rows, wl.D) and padded.dtype == torch.bfloat16
    base_row, base_seg = 0, 0
    for b, L in zip(wl.batch, wl.seq):
        view = padded[base_row: base_row + b * L].view(b, L, wl.D)
        o_f = off[base_seg: base_seg + b + 1]
        l_f = (o_f[1:] - o_f[:-1]).clamp(max=L)
        pos = torch.arange(L, device="cuda").view(1, L)
        mask = pos < l_f.view(-1, 1)
        assert float(view[~mask].abs().sum()) == 0
        src = (o_f[:-1].view(-1, 1) + pos)[mask]
        assert torch.equal(view[mask], rows[inv[src]])
        base_row += b * L
        base_seg += b
    # backward of both outputs: checksum against the incoming gradients
    g = o.segment_reduce_backward_plan(wl.g_pool, None, wl.offsets, plan, "mean")
    exp = (wl.g_pool.double() * (lens > 0).view(-1, 1)).sum(0)
    torch.testing.assert_close(g.double().sum(0), exp, rtol=1e-5, atol=1e-2)
    # what the timed step runs: both gradients summed and the Adagrad update in one launch. On a sample of
    # rows: the oracle's Adagrad (fp32 arithmetic on the bf16 rows widened) with the gradient that the
    # two-input gather-reduce writes, which in turn is the sum of the two single-input passes.
    src_t = plan.src_for_tile(wl.batch, wl.seq, wl.offsets)
    g2 = o.csr_gather_reduce2(plan, (wl.g_pool,) + plan.src_coef_for_pool(wl.offsets, None, True), (wl.g_tile, src_t, None))
    both = o.csr_gather_reduce(wl.g_tile, plan, src_t, out=g.clone(), accumulate=True)
    scale = both.abs().amax(1, keepdim=True).clamp_(min=1.0)
    assert float(((g2 - both).abs() / scale).max()) < 1e-4      # hot rows sum thousands of bf16 terms in another order
    pick = torch.randperm(U, device="cuda")[:4096]
    rows_at = index[pick]
    names = [s.name() for s in wl.table.slot_group().slots()]
    before = [_slot_rows(wl.table, n, rows_at).float().cpu().numpy() for n in names[:2]]
    wl.bwd_update(plan, index)
    after = [_slot_rows(wl.table, n, rows_at).float().cpu().numpy() for n in names[:2]]
    # the accumulator first (the oracle's update of it, stored as bf16), then the oracle's row update
    # reading the STORED accumulator, as a bf16 table does
    bf16 = lambda a: torch.from_numpy(a).to(torch.bfloat16).float().numpy()
    gp = g2[pick].cpu().numpy()
    w, acc = [b.copy() for b in before]
    oracle.block_apply_adagrad(np.arange(4096), gp, [w], [acc], 0.01, 1e-8, 4096)
    acc_stored = bf16(acc)
    np.testing.assert_allclose(after[1], acc_stored, rtol=2 ** -7, atol=1e-12)
    w2, acc2 = before[0].copy(), (acc_stored - gp * gp).astype(np.float32)   # so that acc2 + g*g is the stored value
    oracle.block_apply_adagrad(np.arange(4096), gp, [w2], [acc2], 0.01, 1e-8, 4096)
    step = np.abs(w2 - before[0])
    assert np.all(np.abs(after[0] - w2) <= 2 ** -7 * np.maximum(np.abs(w2), step) + 1e-9)
    assert _lib.poll_device_errors() == 0


@pytest.mark.parametrize("n,key_range", [(40_000_000, 30_000_000), (70_000_000, 1000)])
def test_batch_plan_at_tens_of_millions_of_ids(n, key_range):
    """More tiles than one round of workgroups holds and buckets at their cap: the plan is still a
    bijection onto the distinct ids with every occurrence listed once under its id."""
    g = torch.Generator(device="cuda").manual_seed(0)
    ids = torch.randint(0, key_range, (n,), device="cuda", generator=g)
    plan = ops.ids_unique_plan(ids)
    U = plan.U
    assert torch.equal(torch.sort(plan.unique).values, torch.unique(ids))
    assert bool((plan.unique[plan.inverse.long()] == ids).all())
    rs = plan.row_start[: U + 1].long()
    assert int(rs[0]) == 0 and int(rs[-1]) == n and bool((rs[1:] > rs[:-1]).all())
    owner = torch.repeat_interleave(torch.arange(U, device="cuda"), rs[1:] - rs[:-1])
    assert bool((plan.inverse.long()[plan.occ.long()] == owner).all())
    assert _lib.poll_device_errors() == 0


def test_pooling_past_two_to_the_31_rows():
    """Row counts that no 32-bit index holds (2^31 + 4096 bf16 rows, 17 GB) take the 64-bit
    kernels: sums of 0/1 rows are exact, so the pooled rows are known in closed form."""
    B, D, S = (1 << 31) + 4096, 4, 1 << 20
    emb = torch.ones((B, D), dtype=torch.bfloat16, device="cuda")
    emb[::3] = 0
    off = torch.linspace(0, B, S + 1, device="cuda", dtype=torch.float64).long()
    off[-1] = B
    out = ops.segment_reduce_forward(emb, None, None, off, "sum", out_dtype=torch.float32)

    def ones_before(x):        # rows whose index is not a multiple of 3, below x
        return x - (x + 2) // 3

    exp = (ones_before(off[1:]) - ones_before(off[:-1])).float()
    assert torch.equal(out, exp[:, None].expand(S, D))
    del emb, out
    g = torch.ones((S, D), device="cuda")
    back = ops.segment_reduce_backward(g, None, None, off, B, "sum", out_dtype=torch.bfloat16)
    assert bool((back == 1).all())
    assert _lib.poll_device_errors() == 0

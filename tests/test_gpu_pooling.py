"""Parity of the HIP pooling kernels (through the C ABI) with the CPU oracle.

fp32 tolerance. The contract is rtol 1e-5 / atol 1e-6. It is asserted FLAT, as stated, where the
data keep an fp32 sum inside it whatever the order of the additions: unit weights and rows of the
magnitude the benchmark configurations initialise (config 1: N(0, 0.01), 1..20 ids per sample;
config 4: one id per sample, the row is copied) - test_*_within_the_flat_contract_tolerance and
the copy / plain-store tests below. Sums of up to 200 weighted N(0, 1) terms cannot meet a flat
1e-6 in ANY fp32 order (one rounding of a partial sum near 8 is 4.8e-7), so the tests built on
such data scale the absolute part with the summed magnitude:
|gpu - exact| <= 1e-5 * |exact| + 1e-6 * max(1, sum_i |w_i * x_i|), `exact` being the oracle's
double-precision sum; their names say so (``*_scaled_tolerance_*``) or they state the bound
where they use it. bf16 storage: rtol 1e-2.
"""
import numpy as np
import pytest
import torch

import oracle
from conftest import ragged_offsets
from recis_amd import _lib, ops

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-5, 1e-6


def _dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.to(dtype)
    return t.cuda()


def _assert_pool_close(got, emb, w, rev, off, mode, rtol=RTOL, atol=ATOL):
    exact, mag = oracle.segment_reduce_forward_f64(emb, w, rev, off, mode == "mean")
    err = np.abs(got.astype(np.float64) - exact)
    bound = rtol * np.abs(exact) + atol * np.maximum(1.0, mag)
    bad = err > bound
    assert not bad.any(), "max excess %g at %s" % ((err - bound).max(), np.argwhere(bad)[:3])


def _case(rng, S, U, D, lo, hi, empty_frac=0.1, dup=True):
    off = ragged_offsets(rng, S, lo, hi, empty_frac)
    B = int(off[-1])
    rev = rng.integers(0, U, size=B) if dup else rng.permutation(max(U, B))[:B]
    emb = rng.standard_normal((U, D)).astype(np.float32)
    w = rng.standard_normal(B).astype(np.float32)
    return off, B, rev, emb, w


@pytest.mark.parametrize("mode", ["sum", "mean"])
@pytest.mark.parametrize("std,hi,D", [(0.01, 20, 16), (1.0, 1, 16), (0.02, 20, 64)])
def test_forward_and_backward_within_the_flat_contract_tolerance(rng, mode, std, hi, D):
    """rtol 1e-5 / atol 1e-6 with no scaling: unit weights, 1..hi ids per sample, rows N(0, std).
    (0.01, 20, 16) is benchmark config 1's shape, (1.0, 1, 16) config 4's (one id per sample)."""
    S, U = 4096, 6000
    off = ragged_offsets(rng, S, 1, hi)
    B = int(off[-1])
    rev = rng.integers(0, U, size=B)
    emb = (std * rng.standard_normal((U, D))).astype(np.float32)
    got = ops.segment_reduce_forward(_dev(emb), None, _dev(rev), _dev(off), mode).cpu().numpy()
    exact, _ = oracle.segment_reduce_forward_f64(emb, None, rev, off, mode == "mean")
    np.testing.assert_allclose(got, exact, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(got, oracle.segment_reduce_forward(emb, None, rev, off, mode), rtol=1e-5, atol=1e-6)
    g = (std * rng.standard_normal((S, D))).astype(np.float32)
    plan = ops.ids_unique_plan(_dev(rev))
    inv = plan.inverse.cpu().numpy().astype(np.int64)
    back = ops.segment_reduce_backward_plan(_dev(g), None, _dev(off), plan, mode).cpu().numpy()
    np.testing.assert_allclose(back, oracle.segment_reduce_backward(g, None, inv, off, plan.U, mode),
                               rtol=1e-5, atol=1e-6)
    atomics = ops.segment_reduce_backward(_dev(g), None, _dev(rev), _dev(off), U, mode).cpu().numpy()
    np.testing.assert_allclose(atomics, oracle.segment_reduce_backward(g, None, rev, off, U, mode),
                               rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("D", [1, 3, 4, 6, 16, 32, 48, 64, 128, 260, 512])
@pytest.mark.parametrize("mode", ["sum", "mean"])
def test_forward_fp32_dims_scaled_tolerance_weighted_unit_normal_rows(rng, D, mode):
    off, B, rev, emb, w = _case(rng, 301, 97, D, 0, 40)
    for use_w in (True, False):
        got = ops.segment_reduce_forward(_dev(emb), _dev(w) if use_w else None, _dev(rev),
                                         _dev(off), mode).cpu().numpy()
        _assert_pool_close(got, emb, w if use_w else None, rev, off, mode)


@pytest.mark.parametrize("lo,hi", [(1, 1), (0, 3), (1, 20), (150, 200)])
@pytest.mark.parametrize("off_dtype", [np.int32, np.int64])
@pytest.mark.parametrize("rev_dtype", [np.int32, np.int64])
def test_forward_lengths_and_index_types_scaled_tolerance_up_to_200_terms(rng, lo, hi, off_dtype, rev_dtype):
    off, B, rev, emb, w = _case(rng, 513, 200, 64, lo, hi, empty_frac=0.0)
    got = ops.segment_reduce_forward(_dev(emb), _dev(w), _dev(rev.astype(rev_dtype)),
                                     _dev(off.astype(off_dtype)), "sum").cpu().numpy()
    _assert_pool_close(got, emb, w, rev, off, "sum")


def test_forward_identity_rev(rng):
    off = ragged_offsets(rng, 1000, 1, 60)
    B = int(off[-1])
    emb = rng.standard_normal((B, 64)).astype(np.float32)
    got = ops.segment_reduce_forward(_dev(emb), None, None, _dev(off.astype(np.int32)),
                                     "mean").cpu().numpy()
    _assert_pool_close(got, emb, None, np.arange(B), off, "mean")


def test_forward_empty_inputs():
    emb = torch.zeros((0, 16), device="cuda")
    out = ops.segment_reduce_forward(emb, None, torch.zeros(0, dtype=torch.int64, device="cuda"),
                                     torch.zeros(1, dtype=torch.int64, device="cuda"), "sum")
    assert out.shape == (0, 16)
    emb = torch.randn((5, 16), device="cuda")
    off = torch.zeros(8, dtype=torch.int64, device="cuda")  # 7 empty segments
    out = ops.segment_reduce_forward(emb, None, torch.zeros(0, dtype=torch.int64, device="cuda"),
                                     off, "mean")
    assert out.shape == (7, 16) and float(out.abs().sum()) == 0.0


@pytest.mark.parametrize("mode", ["sum", "mean", "tile"])
@pytest.mark.parametrize("D", [4, 16, 64, 100])
def test_tile_and_backward_fp32(rng, mode, D):
    off, B, rev, emb, w = _case(rng, 211, 150, D, 0, 30)
    B2 = B + 5
    rev = np.concatenate([rev, rng.integers(0, 150, size=5)])  # occurrences after the last offset
    w = np.concatenate([w, np.ones(5, np.float32)])
    if mode == "tile":
        got = ops.segment_reduce_forward(_dev(emb), _dev(w), _dev(rev), _dev(off), mode).cpu().numpy()
        exp = oracle.segment_reduce_forward(emb, w, rev, off, mode)
        np.testing.assert_allclose(got, exp, rtol=RTOL, atol=ATOL)
    rows = B2 if mode == "tile" else 211
    g = rng.standard_normal((rows, D)).astype(np.float32)
    got = ops.segment_reduce_backward(_dev(g), _dev(w), _dev(rev), _dev(off), 150, mode).cpu().numpy()
    exp = oracle.segment_reduce_backward(g, w, rev, off, 150, mode)
    # each gradient row sums up to ~B/U * 30 terms of magnitude ~|g||w|
    np.testing.assert_allclose(got, exp, rtol=1e-5, atol=2e-5)


@pytest.mark.parametrize("mode", ["sum", "mean", "tile"])
def test_backward_unique_rev_plain_stores(rng, mode):
    S, D = 333, 64
    off = ragged_offsets(rng, S, 0, 25)
    off[1:] += 4  # leading occurrences no segment covers
    B = int(off[-1]) + 7
    for U in (B, B + 50):
        rev = rng.permutation(U)[:B]
        w = rng.standard_normal(B).astype(np.float32)
        g = rng.standard_normal((B if mode == "tile" else S, D)).astype(np.float32)
        pre = torch.full((U, D), 7.0, device="cuda")  # stale memory must not leak through
        del pre
        got = ops.segment_reduce_backward(_dev(g), _dev(w), _dev(rev), _dev(off), U, mode,
                                          rev_unique=True).cpu().numpy()
        exp = oracle.segment_reduce_backward(g, w, rev, off, U, mode)
        np.testing.assert_allclose(got, exp, rtol=1e-6, atol=1e-6)
    # identity rev (rows materialised per occurrence)
    g = rng.standard_normal((B if mode == "tile" else S, D)).astype(np.float32)
    got = ops.segment_reduce_backward(_dev(g), _dev(w), None, _dev(off), B, mode).cpu().numpy()
    exp = oracle.segment_reduce_backward(g, w, np.arange(B), off, B, mode)
    np.testing.assert_allclose(got, exp, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("D", [2, 16, 64, 72])
def test_max_forward_backward(rng, D):
    S, U = 257, 120
    off = ragged_offsets(rng, S, 0, 33, empty_frac=0.15)
    B = int(off[-1])
    rev = rng.integers(0, U, size=B)
    emb = np.round(rng.standard_normal((U, D)) * 3).astype(np.float32)  # ties on purpose
    out, arg = ops.segment_reduce_forward(_dev(emb), None, _dev(rev), _dev(off), "max",
                                          return_argmax=True)
    eo, ea = oracle.segment_max_forward(emb, rev, off)
    np.testing.assert_array_equal(out.cpu().numpy(), eo)
    np.testing.assert_array_equal(arg.cpu().numpy(), ea)
    g = rng.standard_normal((S, D)).astype(np.float32)
    got = ops.segment_reduce_backward(_dev(g), None, _dev(rev), _dev(off), U, "max", argmax=arg)
    exp = oracle.segment_max_backward(g, ea, rev, U)
    np.testing.assert_allclose(got.cpu().numpy(), exp, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("kind", ["none", "int32", "int64"])
@pytest.mark.parametrize("D", [2, 16, 64, 72])
def test_max_backward_onto_distinct_rows(rng, D, kind):
    """Max backward when every occurrence has a row of its own (identity, or a permutation promised
    with rev_unique): the kernel that writes each row of a segment whole (gradient where the row
    won, zero elsewhere), in its three index forms, with occurrences before the first and after the
    last offset. Values are only copied, so the comparison is exact."""
    S = 257
    off = ragged_offsets(rng, S, 0, 33, empty_frac=0.15)
    off += 3
    B = int(off[-1]) + 4
    rev = np.arange(B) if kind == "none" else rng.permutation(B)
    emb = np.round(rng.standard_normal((B, D)) * 3).astype(np.float32)   # ties on purpose
    rev_t = None if kind == "none" else _dev(rev.astype(np.int32 if kind == "int32" else np.int64))
    out, arg = ops.segment_reduce_forward(_dev(emb), None, rev_t, _dev(off), "max", return_argmax=True)
    eo, ea = oracle.segment_max_forward(emb, rev, off)
    np.testing.assert_array_equal(out.cpu().numpy(), eo)
    np.testing.assert_array_equal(arg.cpu().numpy(), ea)
    g = rng.standard_normal((S, D)).astype(np.float32)
    stale = torch.full((B, D), 7.0, device="cuda")   # memory the output may land in must not leak through
    del stale
    got = ops.segment_reduce_backward(_dev(g), None, rev_t, _dev(off), B, "max", argmax=arg, rev_unique=True)
    exp = oracle.segment_max_backward(g, ea, rev, B)
    np.testing.assert_array_equal(got.cpu().numpy(), exp)
    assert _lib.poll_device_errors() == 0


@pytest.mark.parametrize("with_rev", [True, False])
def test_max_special_values(rng, with_rev):
    """NaN beats every number and the first NaN is kept, -inf alone still yields its occurrence,
    -0 and +0 tie (first occurrence), +inf wins; segments long enough for several rounds per lane."""
    S, D = 300, 16
    off = ragged_offsets(rng, S, 0, 150, empty_frac=0.1)
    B = int(off[-1])
    U = B if not with_rev else 500
    emb = np.round(rng.standard_normal((U, D)) * 2).astype(np.float32)
    special = np.array([np.nan, np.inf, -np.inf, -0.0, 0.0], np.float32)
    mask = rng.random((U, D)) < 0.15
    emb[mask] = special[rng.integers(0, special.size, int(mask.sum()))]
    emb[: U // 4] = -np.inf                                   # whole rows of -inf
    rev = rng.integers(0, U, size=B) if with_rev else None
    out, arg = ops.segment_reduce_forward(_dev(emb), None, None if rev is None else _dev(rev), _dev(off), "max",
                                          return_argmax=True)
    eo, ea = oracle.segment_max_forward(emb, np.arange(B) if rev is None else rev, off)
    np.testing.assert_array_equal(arg.cpu().numpy(), ea)
    np.testing.assert_array_equal(out.cpu().numpy(), eo)
    assert _lib.poll_device_errors() == 0


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("D", [8, 128, 136])
def test_half_storage_fp32_accumulate(rng, dtype, D):
    off, B, rev, emb, w = _case(rng, 199, 300, D, 0, 50)
    emb_t = torch.from_numpy(emb).to(dtype)
    emb_q = emb_t.float().numpy()  # what the rows really hold
    for out_dtype in (torch.float32, dtype):
        got = ops.segment_reduce_forward(emb_t.cuda(), _dev(w), _dev(rev), _dev(off), "mean",
                                         out_dtype=out_dtype)
        assert got.dtype == out_dtype
        if out_dtype == torch.float32:  # fp32 accumulation: as tight as the fp32 path
            _assert_pool_close(got.cpu().numpy(), emb_q, w, rev, off, "mean")
        else:
            _assert_pool_close(got.float().cpu().numpy(), emb_q, w, rev, off, "mean",
                               rtol=1e-2, atol=1e-2)
    g = rng.standard_normal((199, D)).astype(np.float32)
    g_t = torch.from_numpy(g).to(dtype)
    got = ops.segment_reduce_backward(g_t.cuda(), _dev(w), _dev(rev), _dev(off), 300, "sum",
                                      out_dtype=torch.float32).cpu().numpy()
    exp = oracle.segment_reduce_backward(g_t.float().numpy(), w, rev, off, 300, "sum")
    np.testing.assert_allclose(got, exp, rtol=1e-5, atol=2e-5)


@pytest.mark.parametrize("mode", ["sum", "mean", "tile"])
@pytest.mark.parametrize("D,dtype,lo,hi", [(16, torch.float32, 0, 3), (64, torch.float32, 5, 60),
                                           (128, torch.bfloat16, 10, 90), (40, torch.float32, 0, 12)])
def test_forward_out_of_table_blocks(rng, mode, D, dtype, lo, hi):
    """Pooling straight out of the table blocks (row u = row row_index[u] of the block list, absent
    keys read as zeros) against the oracle on the gathered rows, and bit-identical to
    block_gather + segment_reduce_forward on the device (same kernels, same summation order);
    one-row segments, multi-row segments, several blocks, weights, int32 / int64 indices."""
    bs, nb, U, S = 700, 5, 1500, 900
    blocks_np = [rng.standard_normal((bs, D)).astype(np.float32) for _ in range(nb)]
    blocks = [_dev(b, dtype) for b in blocks_np]
    table = torch.cat(blocks).float().cpu().numpy()
    row_index = rng.permutation(bs * nb)[:U].astype(np.int64)
    row_index[rng.integers(0, U, size=40)] = -1
    rows = np.where(row_index[:, None] >= 0, table[np.maximum(row_index, 0)], 0).astype(np.float32)
    off = ragged_offsets(rng, S, lo, hi, 0.1)
    B = int(off[-1])
    rev = rng.integers(0, U, size=B)
    w = rng.random(B).astype(np.float32)
    for use_w, rev_dt in ((False, np.int32), (True, np.int64), (False, np.int64)):
        wt = _dev(w, dtype) if use_w else None
        got = ops.segment_reduce_forward_blocks(blocks, bs, _dev(row_index), wt, _dev(rev.astype(rev_dt)),
                                                _dev(off.astype(np.int32)), mode, out_dtype=torch.float32)
        dense = ops.block_gather(_dev(row_index), blocks, bs, -1, True)
        ref = ops.segment_reduce_forward(dense, wt, _dev(rev.astype(rev_dt)), _dev(off.astype(np.int32)), mode,
                                         out_dtype=torch.float32)
        assert torch.equal(got, ref)
        wq = wt.float().cpu().numpy() if use_w else None
        if mode == "tile":
            exp = rows[rev] * (wq[:, None] if use_w else 1.0)
            np.testing.assert_allclose(got.cpu().numpy(), exp, rtol=1e-6, atol=1e-6)
        else:
            _assert_pool_close(got.cpu().numpy(), rows, wq, rev, off, mode)
    with pytest.raises(ValueError):
        ops.segment_reduce_forward_blocks(blocks, bs, _dev(row_index), None, _dev(rev), _dev(off), "max")


def test_out_of_range_index_is_reported_not_faulting(rng):
    from recis_amd import _lib

    _lib.poll_device_errors()
    emb = torch.randn((10, 16), device="cuda")
    rev = torch.tensor([0, 3, 99, 2], device="cuda")  # 99 >= U
    off = torch.tensor([0, 2, 4], device="cuda")
    out = ops.segment_reduce_forward(emb, None, rev, off, "sum")
    assert _lib.poll_device_errors() & _lib.DEVERR_INDEX_RANGE
    torch.testing.assert_close(out[0], emb[0] + emb[3])
    torch.testing.assert_close(out[1], emb[2])
    assert _lib.poll_device_errors() == 0


def test_argument_errors():
    emb = torch.randn((10, 16), device="cuda")
    off = torch.tensor([0, 2], device="cuda")
    rev = torch.tensor([0, 1], device="cuda")
    with pytest.raises(ValueError):
        ops.segment_reduce_forward(emb, None, rev, off, "median")
    with pytest.raises(TypeError):
        ops.segment_reduce_forward(emb.double(), None, rev, off, "sum")
    with pytest.raises(TypeError):
        ops.segment_reduce_forward(emb, None, rev.float(), off, "sum")
    with pytest.raises(RuntimeError):  # CPU tensors are refused, there is no CPU path
        ops.segment_reduce_forward(emb.cpu(), None, rev.cpu(), off.cpu(), "sum")


@pytest.mark.parametrize("mode", ["sum", "mean"])
def test_config2_shape_properties(mode):
    """benchmark config 2 at full size: linearity and a sum-of-sums checksum.

    32 x 16384 segments, Poisson(30) lengths clipped to [1, 200], D = 64 fp32,
    rows materialised per occurrence, int32 offsets."""
    import workloads

    c = workloads.config2(device="cuda")
    emb, off, S = c["values"], c["offsets"], c["num_segments"]
    out = ops.segment_reduce_forward(emb, None, None, off, mode)
    assert out.shape == (S, 64)
    # linearity: pool(2a + b) == 2 pool(a) + pool(b)
    b = torch.roll(emb, 1, 0)
    lin = ops.segment_reduce_forward(2 * emb + b, None, None, off, mode)
    ref = 2 * out + ops.segment_reduce_forward(b, None, None, off, mode)
    torch.testing.assert_close(lin, ref, rtol=1e-4, atol=1e-4)
    if mode == "sum":  # checksum of checksums, in double
        total = out.double().sum(0)
        torch.testing.assert_close(total, emb.double().sum(0), rtol=1e-6, atol=1e-3)
    # a slice of it against the oracle
    k = 4096
    nb = int(off[k])
    got = out[:k].cpu().numpy()
    _assert_pool_close(got, emb[:nb].cpu().numpy(), None, np.arange(nb), off[:k + 1].cpu().numpy(), mode)
    # backward is the transpose: <pool(x), g> == <x, pool^T(g)>
    g = torch.randn_like(out)
    gx = ops.segment_reduce_backward(g, None, None, off, emb.shape[0], mode)
    lhs = (out.double() * g.double()).sum()
    rhs = (emb.double() * gx.double()).sum()
    torch.testing.assert_close(lhs, rhs, rtol=1e-6, atol=1e-2)


def test_config2_max_combiner_at_full_size():
    """benchmark config 2, max combiner, at full size (15.7 M rows of 64 floats, 524 288 segments):
    forward against torch.segment_reduce on the device and, for a slice, against the oracle
    (values and argmax, exact); every argmax names a row of its own segment that holds the
    maximum; backward through the kernel the benchmark times (rows written whole): the gradient
    of a segment's column lands on exactly one of its rows, so summing the backward per segment
    returns the incoming gradient bit for bit, and a slice equals the oracle's backward."""
    import workloads

    c = workloads.config2(device="cuda")
    emb, off, S, N = c["values"], c["offsets"], c["num_segments"], c["num_ids"]
    rev = torch.arange(N, device="cuda")
    out, arg = ops.segment_reduce_forward(emb, None, rev, off, "max", return_argmax=True)
    ref = torch.segment_reduce(emb, "max", offsets=off.long(), axis=0)
    assert torch.equal(out, ref)
    lo, hi = off[:-1].long().view(-1, 1), off[1:].long().view(-1, 1)
    a = arg.long()
    assert bool(((a >= lo) & (a < hi)).all())
    assert torch.equal(torch.gather(emb, 0, a), out)
    del ref, a
    k = 4096
    nb = int(off[k])
    eo, ea = oracle.segment_max_forward(emb[:nb].cpu().numpy(), np.arange(nb), off[: k + 1].cpu().numpy())
    np.testing.assert_array_equal(out[:k].cpu().numpy(), eo)
    np.testing.assert_array_equal(arg[:k].cpu().numpy(), ea)
    g = c["grad"]
    gx = ops.segment_reduce_backward(g, None, rev, off, N, "max", argmax=arg, rev_unique=True)
    assert torch.equal(ops.segment_reduce_forward(gx, None, None, off, "sum"), g)
    exp = oracle.segment_max_backward(g[:k].cpu().numpy(), ea, np.arange(nb), nb)
    np.testing.assert_array_equal(gx[:nb].cpu().numpy(), exp)
    plain = ops.segment_reduce_backward(g, None, None, off, N, "max", argmax=arg)   # identity form of the same kernel
    assert torch.equal(plain, gx)
    assert _lib.poll_device_errors() == 0


# ------------------------------------------------------------------ expand (one id per segment)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("D", [1, 3, 16, 32, 128, 300])
def test_expand_rows_equals_pooling_of_unit_segments(dtype, D):
    """Reading each unique row once and writing it to its occurrences gives, bit for bit, what the
    pooling kernels give for segments of one id (sum and mean), with and without weights, out of a
    dense [U, D] array and straight out of table blocks, with hot ids that go through the plan's
    work items."""
    from recis_amd import _lib, ops

    g = torch.Generator(device="cuda").manual_seed(D)
    n = 50000
    ids = torch.randint(0, 4000, (n,), device="cuda", generator=g)
    ids[::3] = 7            # a hot id: ~16 700 occurrences
    ids[1::50] = 9          # a medium one: the wave-cooperative path
    plan = ops.ids_unique_plan(ids)
    U = plan.U
    rows = torch.randn(U, D, device="cuda", generator=g).to(dtype)
    offsets = torch.arange(n + 1, device="cuda", dtype=torch.int32)
    weight = torch.rand(n, device="cuda", generator=g).to(dtype)
    for w in (None, weight):
        exp = ops.segment_reduce_forward(rows, w, plan.inverse, offsets, "sum")
        got = ops.plan_expand_rows(plan, n, rows=rows, weight=w)
        assert got.dtype == exp.dtype and torch.equal(got, exp)
    # out of a block list, with keys the table does not hold (row -1 reads as zeros)
    bs, nb = 1024, -(-U // 1024) + 1
    blocks = [torch.randn(bs, D, device="cuda", generator=g).to(dtype) for _ in range(nb)]
    index = torch.randperm(bs * nb, device="cuda", generator=g)[:U]
    index[::11] = -1
    exp = ops.segment_reduce_forward_blocks(blocks, bs, index, None, plan.inverse, offsets, "mean")
    got = ops.plan_expand_rows(plan, n, blocks=blocks, block_size=bs, row_index=index)
    assert torch.equal(got, exp)
    # with the step filter's stamps written in the same pass: the rows that are read, and only
    # those, carry the new step; the output is the same
    stamps = [torch.full((bs, 1), -5, dtype=torch.int64, device="cuda") for _ in range(nb)]
    step = torch.tensor([41], dtype=torch.int64, device="cuda")
    got = ops.plan_expand_rows(plan, n, blocks=blocks, block_size=bs, row_index=index, stamp=(stamps, step))
    assert torch.equal(got, exp)
    want = [torch.full((bs, 1), -5, dtype=torch.int64, device="cuda") for _ in range(nb)]
    ops.block_insert(index[index >= 0], step.expand(int((index >= 0).sum()), 1).contiguous(), want, bs)
    for a, b in zip(stamps, want):
        assert torch.equal(a, b)
    assert int(sum((b == 41).sum() for b in stamps)) == int((index >= 0).sum())
    with pytest.raises(ValueError):
        ops.plan_expand_rows(plan, n, rows=rows, stamp=(stamps, step))
    assert _lib.poll_device_errors() == 0


def test_engine_takes_the_expand_path_for_dense_id_columns():
    """Dense [B] id tensors through EmbeddingEngine (one id per sample: the click-through shape)
    against the same ids as RaggedTensors with explicit offsets: same outputs, same gradients."""
    from recis_amd.nn import EmbeddingEngine, EmbeddingOption
    from recis_amd.nn.initializers import NormalInitializer
    from recis_amd.nn.modules.hashtable import HashtableRegister
    from recis_amd.ragged.tensor import RaggedTensor

    def make():
        HashtableRegister().clear()
        torch.manual_seed(0)
        return EmbeddingEngine({f: EmbeddingOption(embedding_dim=16, shared_name=f, combiner="sum", block_size=512,
                                                   initializer=NormalInitializer(0, 0.1), use_weight=False)
                                for f in ("a", "b")})

    g = torch.Generator(device="cuda").manual_seed(1)
    ids = {f: torch.randint(0, 300, (4096,), device="cuda", generator=g) for f in ("a", "b")}
    up = torch.randn(4096, 16, device="cuda", generator=g)
    results = []
    for as_ragged in (False, True):
        eng = make()
        eng.train()
        inputs = {f: RaggedTensor(v, torch.arange(4097, device="cuda", dtype=torch.int32)) if as_ragged else v
                  for f, v in ids.items()}
        out = eng(inputs)
        (out["a"] * up).sum().backward()
        impl = list(eng.hashtables().values())[0]._hashtable_impl
        index, grad = impl.grad_pairs(1)
        order = torch.argsort(index)
        results.append((out["a"].detach().clone(), out["b"].detach().clone(), index[order], grad[order]))
    for x, y in list(zip(*results))[:3]:
        assert torch.equal(x, y)
    # the order in which the occurrences of one id are summed is not fixed from run to run
    torch.testing.assert_close(results[0][3], results[1][3], rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("D", [3, 64, 128, 520])
def test_long_segments_workgroup_path(dtype, D):
    """Segments of hundreds of rows (a workgroup per segment) against a float64 sum, with and
    without reverse indices, int32 and int64, empty and very short segments in between."""
    from recis_amd import _lib, ops

    g = torch.Generator(device="cuda").manual_seed(D)
    lens = torch.randint(100, 900, (300,), generator=torch.Generator().manual_seed(D))
    lens[::17] = 0
    lens[5::29] = 3
    off = torch.cat([torch.zeros(1, dtype=torch.long), lens.cumsum(0)]).cuda()
    n, U = int(off[-1]), 5000
    rows = torch.randn(U, D, device="cuda", generator=g).to(dtype)
    rev = torch.randint(0, U, (n,), device="cuda", generator=g)
    seg = torch.repeat_interleave(torch.arange(300, device="cuda"), lens.cuda())
    for mode in ("sum", "mean"):
        ref = torch.zeros(300, D, device="cuda", dtype=torch.float64).index_add_(0, seg, rows[rev].double())
        mag = torch.zeros(300, device="cuda", dtype=torch.float64).index_add_(0, seg, rows[rev].double().abs().sum(1))
        if mode == "mean":
            ref /= lens.cuda().clamp(min=1).view(-1, 1)
            mag /= lens.cuda().clamp(min=1)
        for r in (rev, rev.int()):
            for o in (off, off.int()):
                got = ops.segment_reduce_forward(rows, None, r, o, mode, out_dtype=torch.float32)
                err = (got.double() - ref).abs().sum(1)
                assert bool((err <= 1e-5 * ref.abs().sum(1) + 1e-6 * mag.clamp(min=1.0)).all()), (mode, r.dtype, o.dtype)
    plain = ops.segment_reduce_forward(rows[rev], None, None, off, "sum", out_dtype=torch.float32)
    ref = torch.zeros(300, D, device="cuda", dtype=torch.float64).index_add_(0, seg, rows[rev].double())
    torch.testing.assert_close(plain.double(), ref, rtol=1e-5, atol=1e-3)
    assert _lib.poll_device_errors() == 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("D", [8, 128])
def test_long_segments_out_of_the_table_blocks(dtype, D):
    """The workgroup-per-segment pooling reading rows straight out of table blocks (row u = row
    row_index[u], some keys absent) equals pooling the gathered copy of the same rows."""
    g = torch.Generator(device="cuda").manual_seed(D)
    lens = torch.randint(100, 700, (200,), generator=torch.Generator().manual_seed(D))
    lens[::13] = 0
    off = torch.cat([torch.zeros(1, dtype=torch.long), lens.cumsum(0)]).int().cuda()
    n, U, block_rows, n_blocks = int(off[-1]), 3000, 512, 9
    blocks = [torch.randn(block_rows, D, device="cuda", generator=g).to(dtype) for _ in range(n_blocks)]
    row_index = torch.randint(0, block_rows * n_blocks, (U,), device="cuda", generator=g)
    row_index[::41] = -1                                     # keys the table does not hold read as zeros
    rev = torch.randint(0, U, (n,), device="cuda", generator=g).int()
    table = torch.cat(blocks)
    rows = torch.where(row_index.view(-1, 1) >= 0, table[row_index.clamp(min=0)], torch.zeros((), dtype=dtype, device="cuda"))
    for mode in ("sum", "mean"):
        direct = ops.segment_reduce_forward_blocks(blocks, block_rows, row_index, None, rev, off, mode,
                                                   out_dtype=torch.float32)
        copied = ops.segment_reduce_forward(rows, None, rev, off, mode, out_dtype=torch.float32)
        assert torch.equal(direct, copied)                   # the same rows summed in the same order
    assert _lib.poll_device_errors() == 0

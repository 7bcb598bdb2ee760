"""The functional layer with the reference's names (recis.nn.functional.{embedding_ops, array_ops,
ragged_ops}): each wrapper runs the HIP operator and is compared with the CPU oracle; gradients of
the autograd functions against the oracle's backward (fp32: rtol 1e-5, atol 1e-6 per unit of
summed magnitude)."""
import numpy as np
import pytest
import torch

import oracle
from conftest import ragged_offsets
from recis_amd import _lib
from recis_amd.nn.functional import array_ops, embedding_ops, ragged_ops

pytestmark = pytest.mark.gpu


def _dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a))
    return (t if dtype is None else t.to(dtype)).cuda()


def _sparse_case(rng, U=400, S=700, D=16, max_len=4):
    off = ragged_offsets(rng, S, 0, max_len, empty_frac=0.2)
    n = int(off[-1])
    rev = rng.integers(0, U, n)
    seg = oracle.gen_segment_indices(off)
    w = rng.random(n).astype(np.float32) + 0.5
    emb = rng.standard_normal((U, D)).astype(np.float32)
    return off, rev, seg, w, emb


@pytest.mark.parametrize("backend", ["recis", "torch"])
def test_segment_sum_sparse_and_weight_norm(rng, backend):
    off, rev, seg, w, emb = _sparse_case(rng)
    S = len(off) - 1
    out = embedding_ops.segment_sum_sparse(_dev(emb), _dev(w), _dev(rev), _dev(seg), S, backend=backend)
    exp = oracle.segment_sum(emb, w, rev, seg, S)
    np.testing.assert_allclose(out.cpu().numpy(), exp, rtol=1e-5, atol=1e-5)
    norm = embedding_ops.weight_norm_sparse(_dev(emb), _dev(w), _dev(seg), S, backend=backend)
    if backend == "recis":     # segment_ops_kernel.cu:74-108: weight / sum of the segment's weights
        exp_norm = oracle.segment_mean_weight(w, seg, S)
    else:                      # embedding_ops.py:108-123: weight / occurrences of the segment
        exp_norm = w / np.maximum(np.bincount(seg, minlength=S), 1)[seg]
    np.testing.assert_allclose(norm.cpu().numpy(), exp_norm, rtol=1e-6)
    with pytest.raises(RuntimeError, match="only support"):
        embedding_ops.segment_sum_sparse(_dev(emb), _dev(w), _dev(rev), _dev(seg), S, backend="x")


@pytest.mark.parametrize("combiner", ["sum", "mean"])
def test_sparse_embedding_segment_reduce_forward_backward(rng, combiner):
    off, rev, seg, w, emb = _sparse_case(rng)
    S, U = len(off) - 1, emb.shape[0]
    e = _dev(emb).requires_grad_()
    out = embedding_ops.sparse_embedding_segment_reduce(e, _dev(w), _dev(rev), _dev(seg), S, combiner)
    wn = oracle.segment_mean_weight(w, seg, S) if combiner == "mean" else w
    np.testing.assert_allclose(out.detach().cpu().numpy(), oracle.segment_sum(emb, wn, rev, seg, S),
                               rtol=1e-5, atol=1e-5)
    g = rng.standard_normal(out.shape).astype(np.float32)
    out.backward(_dev(g))
    exp_g = oracle.segment_sum(g, wn, seg, rev, U)      # the same sum with the two index lists swapped
    np.testing.assert_allclose(e.grad.cpu().numpy(), exp_g, rtol=1e-5, atol=2e-5)
    assert _lib.poll_device_errors() == 0


def test_merge_offsets_ids_partition_ids_encode(rng):
    offs = [ragged_offsets(rng, n, 0, 6).astype(np.int32) for n in (30, 1, 200)]
    merged = embedding_ops.merge_offsets([_dev(o) for o in offs])
    exp = oracle.merge_offsets(offs, [int(o[-1]) for o in offs])
    np.testing.assert_array_equal(merged.cpu().numpy(), exp)
    given = embedding_ops.merge_offsets([_dev(o) for o in offs], torch.tensor([int(o[-1]) for o in offs]))
    assert torch.equal(given, merged)

    ids = rng.integers(0, 500, 4000)
    u, counts, inv = embedding_ops.ids_partition(_dev(ids), 16, 4)
    eu, ec, ei = oracle.ids_partition(ids, 4)
    np.testing.assert_array_equal(np.sort(u.cpu().numpy()), np.sort(eu))
    np.testing.assert_array_equal(counts.cpu().numpy(), ec)
    np.testing.assert_array_equal(u.cpu().numpy()[inv.cpu().numpy()], ids)

    lists = [rng.integers(-(1 << 60), 1 << 60, n) for n in (100, 0, 33)]
    enc = embedding_ops.ids_encode([_dev(a) for a in lists], [3, 0, 4095])
    np.testing.assert_array_equal(enc.cpu().numpy(), oracle.ids_encode(lists, [3, 0, 4095]))
    with pytest.raises(AssertionError):
        embedding_ops.ids_encode(_dev(lists[0]), [3])


def test_array_ops(rng):
    x = rng.standard_normal((40, 7)).astype(np.float32) * 3
    bnd = np.sort(rng.standard_normal(13).astype(np.float32))
    got = array_ops.bucketize(_dev(x), bnd.tolist())
    np.testing.assert_array_equal(got.cpu().numpy(), oracle.bucketize(x.reshape(-1), bnd).reshape(x.shape))
    ids = rng.integers(-(1 << 62), 1 << 62, (9, 11))
    got = array_ops.bucketize_mod(_dev(ids), 1000003)
    np.testing.assert_array_equal(got.cpu().numpy(), oracle.uint64_mod(ids.reshape(-1), 1000003).reshape(ids.shape))
    muls, primes, buckets = [3, 5, 7, 11], [1000003, 999983, 10007, 7919], [20000, 20000, 10000, 500]
    outs = array_ops.multi_hash(_dev(ids), muls, primes, buckets)
    exp = oracle.multi_hash(ids.reshape(-1), muls, primes, buckets)
    assert len(outs) == 4
    for o, e in zip(outs, exp):
        np.testing.assert_array_equal(o.cpu().numpy(), np.asarray(e).reshape(ids.shape))


def test_ragged_tile_function_and_list_form_of_the_tile_combiner(rng):
    batch, seq = [40, 9], [6, 25]
    U, D = 120, 32
    off = np.concatenate([[0], np.cumsum(np.concatenate([rng.integers(0, 30, b) for b in batch]))]).astype(np.int32)
    value = rng.integers(0, U, int(off[-1]))
    table = rng.standard_normal((U, D)).astype(np.float32)
    exp = oracle.ragged_tile(batch, seq, value, off, table)
    dy = rng.standard_normal(exp.shape).astype(np.float32)
    exp_b = oracle.ragged_tile_back(batch, seq, value, off, dy, U)

    t = _dev(table).requires_grad_()
    out = ragged_ops.ragged_tile(batch, seq, _dev(value), _dev(off), t, check_enable=True)
    np.testing.assert_array_equal(out.detach().cpu().numpy(), exp)
    out.backward(_dev(dy))
    np.testing.assert_allclose(t.grad.cpu().numpy(), exp_b, rtol=1e-5, atol=1e-5)

    t2 = _dev(table).requires_grad_()                      # embedding_ops.py:253-271: "bs" + "tile_len" lists
    out2 = embedding_ops.ragged_embedding_segment_reduce(t2, None, _dev(value), _dev(off), "tile",
                                                         {"bs": batch, "tile_len": seq})
    np.testing.assert_array_equal(out2.detach().cpu().numpy(), exp)
    out2.backward(_dev(dy))
    np.testing.assert_allclose(t2.grad.cpu().numpy(), exp_b, rtol=1e-5, atol=1e-5)
    assert _lib.poll_device_errors() == 0

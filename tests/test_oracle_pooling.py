"""Pins the pooling part of the CPU oracle.

Sources of truth: the reference's own known-answer vectors (merge_offsets,
gen_segment_indices, sparse-mode forward and gradient values), the torch
closed form the reference test uses (index + weight + view/sum/mean), torch
library routines (index_add_, segment_reduce, autograd) and brute force.
"""
import numpy as np
import torch

import oracle
from conftest import ragged_offsets


def test_merge_offsets_kat():
    # tests/ops/emb_segment_reduce_test.py:50-55
    out = oracle.merge_offsets([[0, 2, 5], [0, 3, 6]], [5, 8])
    assert out.tolist() == [0, 2, 5, 8, 11]


def test_merge_offsets_three_tensors_bruteforce():
    offs = [np.array([0, 1, 4]), np.array([0, 0, 2, 3]), np.array([0, 5])]
    maxv = [4, 3, 5]
    exp = [0, 1] + [4 + 0, 4 + 0, 4 + 2] + [7 + 0, 7 + 5]
    assert oracle.merge_offsets(offs, maxv).tolist() == exp


def test_gen_segment_indices_kat():
    # tests/ops/emb_segment_reduce_test.py:94-98
    assert oracle.gen_segment_indices([0, 2, 5]).tolist() == [0, 0, 1, 1, 1]
    assert oracle.gen_segment_indices([0, 0, 3, 3, 4]).tolist() == [1, 1, 1, 3]


def test_ragged_forward_reference_test_closed_form():
    # the construction of tests/ops/emb_segment_reduce_test.py:59-90
    g = torch.Generator().manual_seed(0)
    D = 64
    emb = torch.randn(6, D, generator=g)
    rev = torch.tensor([0, 1, 2, 0, 1, 2])
    offsets = torch.tensor([0, 3, 6])
    weight = torch.randn(6, generator=g)
    expanded = emb[rev] * weight.view(-1, 1)
    exp = {"tile": expanded, "sum": expanded.view(-1, 3, D).sum(1),
           "mean": expanded.view(-1, 3, D).mean(1)}
    for mode in ("sum", "mean", "tile"):
        got = oracle.segment_reduce_forward(emb.numpy(), weight.numpy(), rev.numpy(),
                                            offsets.numpy(), mode)
        np.testing.assert_allclose(got, exp[mode].numpy(), rtol=1e-6, atol=1e-6)


def _torch_pool(emb, w, rev, offsets, mode):
    """Independent torch formulation: gather, weight, index_add_ by segment id."""
    lens = offsets[1:] - offsets[:-1]
    seg = torch.repeat_interleave(torch.arange(len(lens)), lens)
    lo, hi = int(offsets[0]), int(offsets[-1])
    rows = emb[rev[lo:hi]]
    if w is not None:
        rows = rows * w[lo:hi].view(-1, 1)
    if mode == "tile":
        out = torch.zeros(rev.numel(), emb.shape[1], dtype=emb.dtype)
        out[lo:hi] = rows
        return out
    if mode == "mean":
        rows = rows / lens[seg].view(-1, 1).to(emb.dtype)
    out = torch.zeros(len(lens), emb.shape[1], dtype=emb.dtype)
    out.index_add_(0, seg, rows)
    return out


def test_ragged_forward_backward_vs_torch_autograd(rng):
    for use_w in (True, False):
        for mode in ("sum", "mean", "tile"):
            S, U, D = 37, 50, 12
            off = ragged_offsets(rng, S, 0, 9, empty_frac=0.2)
            B = int(off[-1]) + 3  # a few trailing occurrences no segment covers
            rev = rng.integers(0, U, size=B)
            emb = torch.tensor(rng.standard_normal((U, D)), dtype=torch.float64, requires_grad=True)
            w = torch.tensor(rng.standard_normal(B), dtype=torch.float64) if use_w else None
            out = _torch_pool(emb, w, torch.tensor(rev), torch.tensor(off), mode)
            gout = torch.tensor(rng.standard_normal(out.shape), dtype=torch.float64)
            out.backward(gout)
            wn = None if w is None else w.numpy()
            got = oracle.segment_reduce_forward(emb.detach().numpy(), wn, rev, off, mode)
            np.testing.assert_allclose(got, out.detach().numpy(), rtol=1e-5, atol=1e-5)
            gb = oracle.segment_reduce_backward(gout.numpy(), wn, rev, off, U, mode)
            np.testing.assert_allclose(gb, emb.grad.numpy(), rtol=1e-5, atol=1e-5)


def test_f64_variant_matches_f32_and_bounds_error(rng):
    S, U, D = 20, 64, 8
    off = ragged_offsets(rng, S, 1, 200)
    rev = rng.integers(0, U, size=int(off[-1]))
    emb = rng.standard_normal((U, D)).astype(np.float32)
    w = rng.standard_normal(int(off[-1])).astype(np.float32)
    for mean in (False, True):
        f32 = oracle.segment_reduce_forward(emb, w, rev, off, "mean" if mean else "sum")
        f64, fabs = oracle.segment_reduce_forward_f64(emb, w, rev, off, mean)
        assert np.all(np.abs(f32 - f64) <= 1e-5 * np.abs(f64) + 1e-6 * np.maximum(1, fabs))
        assert np.all(fabs >= np.abs(f64) - 1e-9)


def test_sparse_mode_kats():
    # tests/nn/segment_ops_test.py:62-74 (mean), :180-229 (gradients)
    data = np.array([[1.0, 1.0], [2.0, 2.0], [3.0, 3.0]], np.float32)
    weight = np.array([2.0, 3.0, 0.5, 1.0], np.float32)
    indices = np.array([2, 0, 1, 0])
    seg = np.array([0, 1, 1, 2])
    s = oracle.segment_sum(data, weight, indices, seg, 4)
    np.testing.assert_allclose(s, [[6, 6], [4, 4], [1, 1], [0, 0]], atol=1e-7)
    wn = oracle.segment_mean_weight(weight, seg, 4)
    m = oracle.segment_sum(data, wn, indices, seg, 4)
    np.testing.assert_allclose(m, [[3, 3], [4 / 3.5, 4 / 3.5], [1, 1], [0, 0]], atol=1e-7)
    # gradient of sum w.r.t. data = segment_sum of grad rows scattered by indices
    grad = np.ones((4, 2), np.float32)
    gsum = oracle.segment_sum(grad, weight, seg, indices, 3)
    np.testing.assert_allclose(gsum, [[4, 4], [0.5, 0.5], [2, 2]], atol=1e-7)
    gmean = oracle.segment_sum(grad, wn, seg, indices, 3)
    np.testing.assert_allclose(gmean, [[1 + 3 / 3.5] * 2, [0.5 / 3.5] * 2, [1, 1]], atol=1e-7)


def test_sparse_mode_out_of_range_segment_keeps_raw_weight():
    w = np.array([2.0, 4.0, 6.0], np.float32)
    wn = oracle.segment_mean_weight(w, np.array([0, 0, 7]), 2)
    np.testing.assert_allclose(wn, [2 / 6, 4 / 6, 6.0], rtol=1e-7)
    wn = oracle.segment_mean_weight(None, np.array([1, 1, 1, 0]), 2)
    np.testing.assert_allclose(wn, [1 / 3, 1 / 3, 1 / 3, 1.0], rtol=1e-7)


def test_max_combiner_vs_torch(rng):
    S, U, D = 25, 30, 7
    off = ragged_offsets(rng, S, 0, 6, empty_frac=0.2)
    B = int(off[-1])
    rev = rng.integers(0, U, size=B)
    emb = np.round(rng.standard_normal((U, D)) * 2).astype(np.float32)  # many ties
    out, arg = oracle.segment_max_forward(emb, rev, off)
    rows = torch.tensor(emb)[torch.tensor(rev)]
    lens = torch.tensor(off[1:] - off[:-1])
    exp = torch.segment_reduce(rows, "max", lengths=lens, initial=None)
    exp = torch.where(lens.view(-1, 1) == 0, torch.zeros_like(exp), exp)
    np.testing.assert_array_equal(out, exp.numpy())
    # argmax: first occurrence attaining the maximum (brute force)
    for s in range(S):
        for d in range(D):
            if off[s] == off[s + 1]:
                assert arg[s, d] == -1
            else:
                col = emb[rev[off[s]:off[s + 1]], d]
                assert arg[s, d] == off[s] + int(np.argmax(col))
    g = rng.standard_normal((S, D)).astype(np.float32)
    gb = oracle.segment_max_backward(g, arg, rev, U)
    exp_g = np.zeros((U, D), np.float32)
    for s in range(S):
        for d in range(D):
            if arg[s, d] >= 0:
                exp_g[rev[arg[s, d]], d] += g[s, d]
    np.testing.assert_allclose(gb, exp_g, rtol=1e-6, atol=1e-6)


def test_ragged_tile_numpy_model(rng):
    # model of tests/nn/test_ragged_tile.py:72-120: per feature, per sample,
    # copy min(len, seq) table rows, pad with zeros
    batch, seq = [3, 2], [4, 2]
    lens = [[2, 5, 0], [1, 3]]
    U, D = 11, 5
    table = rng.standard_normal((U, D)).astype(np.float32)
    flat = [l for f in lens for l in f]
    off = np.concatenate([[0], np.cumsum(flat)])
    value = rng.integers(0, U, size=int(off[-1]))
    out = oracle.ragged_tile(batch, seq, value, off, table)
    exp, k = [], 0
    for f in range(2):
        for b in range(batch[f]):
            for t in range(seq[f]):
                exp.append(table[value[off[k] + t]] if t < flat[k] else np.zeros(D, np.float32))
            k += 1
    np.testing.assert_array_equal(out, np.stack(exp))
    dy = rng.standard_normal(out.shape).astype(np.float32)
    back = oracle.ragged_tile_back(batch, seq, value, off, dy, U)
    exp_b, k, r = np.zeros((U, D), np.float64), 0, 0
    for f in range(2):
        for b in range(batch[f]):
            for t in range(seq[f]):
                if t < flat[k]:
                    exp_b[value[off[k] + t]] += dy[r]
                r += 1
            k += 1
    np.testing.assert_allclose(back, exp_b, rtol=1e-6, atol=1e-6)

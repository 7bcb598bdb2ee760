"""Pins the sequence-truncation part of the CPU oracle. The reference holds no output vectors for
these ops (its own tests compare the fused op with itself), so the pins are: the worked example in
the reference's docstring (recis/nn/functional/ragged_ops.py:225-252), the offsets its feature test
expects (tests/feature_engine/op_test.py:81-93), and a model on Python lists written from the
documented meaning (drop on one side, pad with empty rows on one side)."""
import numpy as np
import pytest

import oracle


def _to_lists_2d(values, offsets):
    return [list(values[offsets[i]:offsets[i + 1]]) for i in range(len(offsets) - 1)]


def _to_lists_3d(values, outer, inner):
    rows = _to_lists_2d(values, inner)
    return [rows[outer[i]:outer[i + 1]] for i in range(len(outer) - 1)]


def _model(seq, keep, drop_left, pad_left, filler):
    """A Python list brought to length ``keep``."""
    if len(seq) >= keep:
        return seq[len(seq) - keep:] if drop_left else seq[:keep]
    fill = [filler() for _ in range(keep - len(seq))]
    return fill + seq if pad_left else seq + fill


def test_docstring_example_3d():
    values = np.arange(10, 20)
    outer = np.array([0, 3, 4, 6], np.int32)
    inner = np.array([0, 1, 4, 4, 8, 8, 10], np.int32)
    v, o, i = oracle.ragged_cutoff_3d(values, outer, inner, 2, True, True)
    assert _to_lists_3d(v, o, i) == [[[11, 12, 13], []], [[], [14, 15, 16, 17]], [[], [18, 19]]]
    assert o.dtype == np.int32 and i.dtype == np.int32 and o.tolist() == [0, 2, 4, 6]


def test_feature_test_offsets_2d():
    values = np.arange(512)
    v, o, d, p = oracle.ragged_cutoff_2d(values, np.array([0, 256, 512], np.int32), 128, True)
    assert o.tolist() == [0, 128, 256] and d.tolist() == [128, 128] and p.tolist() == [0, 0]
    assert v.tolist() == list(range(128, 256)) + list(range(384, 512))   # "left" truncation keeps the tail


@pytest.mark.parametrize("drop_left", [False, True])
@pytest.mark.parametrize("keep", [0, 1, 3, 7])
def test_2d_against_list_model(rng, drop_left, keep):
    lens = rng.integers(0, 9, 50)
    offsets = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
    values = rng.integers(-100, 100, offsets[-1])
    v, o, d, p = oracle.ragged_cutoff_2d(values, offsets, keep, drop_left)
    exp = [(_model(row, keep, drop_left, False, None) if len(row) >= keep else row)
           for row in _to_lists_2d(values, offsets)]
    assert _to_lists_2d(v, o) == exp
    assert d.tolist() == [max(int(n) - keep, 0) for n in lens] and p.tolist() == [max(keep - int(n), 0) for n in lens]


@pytest.mark.parametrize("drop_left,pad_left", [(False, False), (True, False), (False, True), (True, True)])
@pytest.mark.parametrize("keep", [1, 2, 5])
def test_3d_against_list_model(rng, drop_left, pad_left, keep):
    seq_lens = rng.integers(0, 7, 40)
    outer = np.concatenate([[0], np.cumsum(seq_lens)]).astype(np.int32)
    inner_lens = rng.integers(0, 4, outer[-1])
    inner = np.concatenate([[0], np.cumsum(inner_lens)]).astype(np.int32)
    values = rng.standard_normal(inner[-1])
    v, o, i = oracle.ragged_cutoff_3d(values, outer, inner, keep, drop_left, pad_left)
    exp = [_model(seq, keep, drop_left, pad_left, list) for seq in _to_lists_3d(values, outer, inner)]
    assert _to_lists_3d(v, o, i) == exp
    assert o.tolist() == [k * keep for k in range(len(seq_lens) + 1)]


def test_ragged_to_dense_docstring_example():
    # tests/ops/ragged_to_dense_test.py:17-30
    got = oracle.ragged_to_dense(np.array([1, 2, 3, 4, 5, 6, 7, 8, 9, 9, 10, 11, 12]),
                                 [np.array([0, 2, 2, 3, 6]), np.array([0, 2, 4, 6, 9, 11, 13])], 0)
    assert got.tolist() == [[[1, 2, 0], [3, 4, 0], [0, 0, 0]], [[0, 0, 0], [0, 0, 0], [0, 0, 0]],
                            [[5, 6, 0], [0, 0, 0], [0, 0, 0]], [[7, 8, 9], [9, 10, 0], [11, 12, 0]]]


def test_ragged_to_dense_against_nested_lists(rng):
    for levels in (1, 2, 3):
        offsets, n = [], 6
        for _ in range(levels):
            lens = rng.integers(0, 4, n)
            offsets.append(np.concatenate([[0], np.cumsum(lens)]).astype(np.int64))
            n = int(offsets[-1][-1])
        values = rng.integers(1, 1000, n)
        got = oracle.ragged_to_dense(values, offsets, -7)

        def nested(level, at):
            if level == levels:
                return int(values[at])
            return [nested(level + 1, k) for k in range(int(offsets[level][at]), int(offsets[level][at + 1]))]

        def pad(tree, shape):
            if not shape:
                return tree
            rows = [pad(t, shape[1:]) for t in tree]
            filler = np.full(shape[1:], -7).tolist() if len(shape) > 1 else -7
            return rows + [filler] * (shape[0] - len(rows))

        exp = [pad(nested(0, b), got.shape[1:]) for b in range(got.shape[0])]
        assert got.tolist() == exp


def test_dense_to_ragged_kats():
    # tests/ops/dense_to_ragged_test.py:6-27
    v, o = oracle.dense_to_ragged(np.array([[1, 0, 3, 0, 0], [6, 7, 8, 0, 0]], np.float32), 0)
    assert v.tolist() == [1, 0, 3, 6, 7, 8] and o.tolist() == [0, 3, 6] and o.dtype == np.int32
    v, o = oracle.dense_to_ragged(np.array([[1, 2, 3, 0, 0], [6, 7, 8, 0, 0]], np.int64), 0)
    assert v.tolist() == [1, 2, 3, 6, 7, 8] and o.tolist() == [0, 3, 6]
    v, o = oracle.dense_to_ragged(np.zeros((3, 4), np.int32), 0)
    assert v.size == 0 and o.tolist() == [0, 0, 0, 0]


def test_feature_cross_kat():
    # tests/feature_engine/op_test.py:39-63
    ids, offs, w = oracle.feature_cross_ragged(np.array([1001, 1002, 1003]), np.array([0, 1, 2, 3], np.int32),
                                               np.ones(3, np.float32), np.array([1, 2, 3]),
                                               np.array([0, 1, 2, 3], np.int32), np.ones(3, np.float32))
    assert ids.tolist() == [-7808879811642834040, -4967483181219983279, 1752425377096056168]
    assert offs.tolist() == [0, 1, 2, 3] and w.tolist() == [1, 1, 1]


def test_murmur_words_is_murmur64a_over_the_bytes(rng):
    """The word form used by the cross equals the reference's byte-string MurmurHash64A (the one
    compiled from the reference into oracle/_ref and the one the string features use)."""
    for _ in range(50):
        words = rng.integers(-(1 << 63), (1 << 63) - 1, int(rng.integers(1, 5)))
        raw = np.frombuffer(words.astype("<i8").tobytes(), np.uint8)
        got = oracle.hash_strings(raw, np.array([0, raw.size]), "murmur")[0]
        exp = oracle.murmur_hash_64_words(words.tolist())
        assert int(got) == (exp - (1 << 64) if exp >= 1 << 63 else exp)


def test_feature_cross_dedups_and_takes_first_weight():
    ids, offs, w = oracle.feature_cross_ragged(np.array([5, 7, 5, 9]), np.array([0, 3, 4]),
                                               np.array([2.0, 3.0, 100.0, 1.0]), np.array([1, 1, 4, 8]),
                                               np.array([0, 2, 4]), np.array([0.5, 9.0, 1.0, 2.0]))
    assert offs.tolist() == [0, 2, 4]                 # {5,7} x {1} and {9} x {4,8}
    assert w.tolist() == [1.0, 1.5, 1.0, 2.0]
    h = oracle.murmur_hash_64_words
    signed = lambda v: v - (1 << 64) if v >= 1 << 63 else v
    assert ids.tolist() == [signed(h([5, 1])), signed(h([7, 1])), signed(h([9, 4])), signed(h([9, 8]))]


def test_calc_ragged_index_kat():
    # tests/ops/ragged_topk_index_cutoff_test.py:9-22
    idx, offs = oracle.calc_ragged_index(np.array([5, 0, 0]), np.array([0, 8, 10, 13], np.int32),
                                         np.array([[1, 2], [0, 2], [0, 1]]), np.array([0, 1, 2]))
    assert idx.tolist() == [6, 7, 8, 10, 11] and offs.tolist() == [0, 2, 3, 5]
    assert idx.dtype == np.int64 and offs.dtype == np.int32


def test_calc_ragged_index_against_masks(rng):
    """Same selection written as whole-array masks: the kept entries of the [rows, cols] grid in
    row-major order, counts per row as a cumulative sum."""
    for _ in range(20):
        src_rows, rows, cols = int(rng.integers(1, 9)), int(rng.integers(0, 12)), int(rng.integers(0, 7))
        offset = np.concatenate([[0], np.cumsum(rng.integers(0, 9, src_rows))]).astype(np.int64)
        drop = rng.integers(0, 5, src_rows)
        ind = rng.integers(0, src_rows, rows)
        topk = rng.integers(-2, 9, (rows, cols))
        idx, offs = oracle.calc_ragged_index(drop, offset, topk, ind)
        e = topk + (offset[ind] + drop[ind])[:, None]
        keep = (e >= offset[ind][:, None]) & (e < offset[ind + 1][:, None])
        assert idx.tolist() == e[keep].tolist()
        assert offs.tolist() == np.concatenate([[0], np.cumsum(keep.sum(1))]).tolist()


def test_ragged_to_sparse_indices_scatter_into_the_dense_form(rng):
    """The coordinates place every value where ragged_to_dense (pinned by the reference's example)
    puts it, and nowhere else."""
    for levels in (1, 2, 3):
        for _ in range(5):
            offsets, n = [], int(rng.integers(1, 5))
            for _ in range(levels):
                o = np.concatenate([[0], np.cumsum(rng.integers(0, 4, n))]).astype(np.int32)
                offsets.append(o)
                n = int(o[-1])
            values = rng.integers(1, 100, n).astype(np.int64)
            dense = oracle.ragged_to_dense(values, offsets, 0)
            idx = oracle.ragged_to_sparse_indices(offsets)
            assert idx.shape == (levels + 1, n)
            rebuilt = np.zeros_like(dense)
            rebuilt[tuple(idx)] = values
            assert np.array_equal(rebuilt, dense)


def test_ragged_to_sparse_host_function_matches_the_coordinates(rng):
    import torch
    from recis_amd.nn.functional.ragged_ops import ragged_to_sparse
    offsets = [np.array([0, 2, 5, 6], np.int32), np.array([0, 1, 3, 6, 8, 10, 11], np.int32)]
    values = np.arange(1, 12, dtype=np.int64)
    sp = ragged_to_sparse(torch.from_numpy(values), [torch.from_numpy(o) for o in offsets])
    assert list(sp.shape) == [3, 3, 3]
    assert np.array_equal(sp.indices().numpy(), oracle.ragged_to_sparse_indices(offsets))
    assert np.array_equal(sp.to_dense().numpy(), oracle.ragged_to_dense(values, offsets, 0))
    one = ragged_to_sparse(torch.from_numpy(values[:6]), [torch.from_numpy(offsets[0])])
    assert one.indices().tolist() == [[0, 0, 1, 1, 1, 2], [0, 1, 0, 1, 2, 0]]

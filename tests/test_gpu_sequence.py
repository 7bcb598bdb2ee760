"""Sequence ops on the GPU against the CPU oracle, bit for bit: truncation of lists of 2-D / 3-D
ragged tensors, ragged_to_dense, dense_to_ragged (all through the C ABI)."""
import numpy as np
import pytest
import torch

import oracle
from recis_amd import _lib, ops

pytestmark = pytest.mark.gpu

DTYPES = [(np.int64, torch.int64), (np.float32, torch.float32), (np.float64, torch.float64), (np.int32, torch.int32),
          (np.int8, torch.int8), (np.float16, torch.float16)]


def _ragged(rng, rows, max_len, off_dtype, empty_frac=0.2):
    lens = rng.integers(0, max_len + 1, rows)
    lens[rng.random(rows) < empty_frac] = 0
    return np.concatenate([[0], np.cumsum(lens)]).astype(off_dtype)


def _values(rng, n, np_dtype):
    if np.issubdtype(np_dtype, np.integer):
        info = np.iinfo(np_dtype)
        return rng.integers(max(info.min, -(1 << 40)), min(info.max, 1 << 40), n).astype(np_dtype)
    return rng.standard_normal(n).astype(np_dtype)


@pytest.mark.parametrize("off_dtype", [np.int32, np.int64])
@pytest.mark.parametrize("np_dtype,t_dtype", DTYPES)
def test_cutoff_2d_list_matches_oracle(rng, off_dtype, np_dtype, t_dtype):
    n_tensors = 27   # more than one launch of the job table
    rows = [int(r) for r in rng.integers(0, 5000, n_tensors)]
    rows[3] = 0
    offs = [_ragged(rng, r, 12, off_dtype) for r in rows]
    vals = [_values(rng, int(o[-1]), np_dtype) for o in offs]
    keep = [int(k) for k in rng.integers(0, 9, n_tensors)]
    drop = [bool(b) for b in rng.integers(0, 2, n_tensors)]
    pad = [bool(b) for b in rng.integers(0, 2, n_tensors)]
    got = ops.fused_ragged_cutoff([torch.from_numpy(v).cuda() for v in vals], [torch.from_numpy(o).cuda() for o in offs],
                                  torch.tensor(keep, dtype=torch.int32), torch.tensor(drop), torch.tensor(pad))
    for t in range(n_tensors):
        v, o, d, p = oracle.ragged_cutoff_2d(vals[t], offs[t], keep[t], drop[t])
        assert got[0][t].dtype == t_dtype and got[1][t].dtype == torch.from_numpy(offs[t]).dtype
        np.testing.assert_array_equal(got[0][t].cpu().numpy(), v)
        np.testing.assert_array_equal(got[1][t].cpu().numpy(), o)
        np.testing.assert_array_equal(got[2][t].cpu().numpy(), d)
        np.testing.assert_array_equal(got[3][t].cpu().numpy(), p)
    assert _lib.poll_device_errors() == 0


@pytest.mark.parametrize("off_dtype", [np.int32, np.int64])
@pytest.mark.parametrize("drop,pad", [(False, False), (True, False), (False, True), (True, True)])
def test_cutoff_3d_list_matches_oracle(rng, off_dtype, drop, pad):
    n_tensors = 6
    outer = [_ragged(rng, int(r), 9, off_dtype) for r in rng.integers(0, 3000, n_tensors)]
    inner = [_ragged(rng, int(o[-1]), 5, off_dtype) for o in outer]
    vals = [_values(rng, int(i[-1]), np.int64) for i in inner]
    keep = [int(k) for k in rng.integers(1, 8, n_tensors)]
    got = ops.fused_ragged_cutoff_3D([torch.from_numpy(v).cuda() for v in vals],
                                     [torch.from_numpy(o).cuda() for o in outer],
                                     [torch.from_numpy(i).cuda() for i in inner], keep, [drop] * n_tensors,
                                     [pad] * n_tensors)
    for t in range(n_tensors):
        v, o, i = oracle.ragged_cutoff_3d(vals[t], outer[t], inner[t], keep[t], drop, pad)
        np.testing.assert_array_equal(got[0][t].cpu().numpy(), v)
        np.testing.assert_array_equal(got[1][t].cpu().numpy(), o)
        np.testing.assert_array_equal(got[2][t].cpu().numpy(), i)
    assert _lib.poll_device_errors() == 0


def test_cutoff_reference_examples():
    # recis/nn/functional/ragged_ops.py:225-252
    v, o, i = ops.fused_ragged_cutoff_3D([torch.arange(10, 20).cuda()],
                                         [torch.tensor([0, 3, 4, 6], dtype=torch.int32).cuda()],
                                         [torch.tensor([0, 1, 4, 4, 8, 8, 10], dtype=torch.int32).cuda()],
                                         torch.tensor([2], dtype=torch.int32).cuda(), torch.tensor([True]).cuda(),
                                         torch.tensor([True]).cuda())
    assert v[0].tolist() == [11, 12, 13, 14, 15, 16, 17, 18, 19]
    assert o[0].tolist() == [0, 2, 4, 6] and i[0].tolist() == [0, 3, 3, 3, 7, 7, 9]
    # tests/feature_engine/op_test.py:81-93
    out = ops.fused_ragged_cutoff([torch.randn(512).cuda()], [torch.tensor([0, 256, 512], dtype=torch.int32).cuda()],
                                  [128], [True], [False])
    assert out[1][0].tolist() == [0, 128, 256]


def test_cutoff_sequence_workload_properties():
    """The shape of the behaviour-sequence fields (2048 sequences, log-normal lengths, mean 200, cut
    to 100 then to 50): truncation twice equals truncation once to the smaller length; kept
    counts follow from the lengths alone."""
    g = torch.Generator().manual_seed(5)
    lens = torch.clamp(torch.exp(torch.randn(2048, generator=g) * 0.8 + 5.0).long(), 1, 1000)
    off = torch.cat([torch.zeros(1, dtype=torch.long), lens.cumsum(0)]).to(torch.int32).cuda()
    vals = torch.arange(int(off[-1]), dtype=torch.int64).cuda()
    for left in (False, True):
        a = ops.fused_ragged_cutoff([vals] * 4, [off] * 4, [100] * 4, [left] * 4, [False] * 4)
        b = ops.fused_ragged_cutoff(a[0], a[1], [50] * 4, [left] * 4, [False] * 4)
        c = ops.fused_ragged_cutoff([vals] * 4, [off] * 4, [50] * 4, [left] * 4, [False] * 4)
        for t in range(4):
            assert torch.equal(b[0][t], c[0][t]) and torch.equal(b[1][t], c[1][t])
            assert int(a[1][t][-1]) == int(torch.clamp(lens, max=100).sum())
            first = vals[(off[1:].long() - 50).clamp(min=off[:-1].long())] if left else vals[off[:-1].long()]
            assert torch.equal(c[0][t][c[1][t][:-1].long()], first)
    assert _lib.poll_device_errors() == 0


@pytest.mark.parametrize("np_dtype,t_dtype", DTYPES)
def test_ragged_to_dense_matches_oracle(rng, np_dtype, t_dtype):
    for levels in (1, 2, 3):
        offsets, n = [], 40
        for _ in range(levels):
            offsets.append(_ragged(rng, n, 5, np.int32 if levels != 2 else np.int64))
            n = int(offsets[-1][-1])
        values = _values(rng, n, np_dtype)
        got = ops.ragged_to_dense(torch.from_numpy(values).cuda(), [torch.from_numpy(o).cuda() for o in offsets], 3)
        np.testing.assert_array_equal(got.cpu().numpy(), oracle.ragged_to_dense(values, offsets, 3))
    assert _lib.poll_device_errors() == 0


def test_ragged_to_dense_reference_example_and_given_widths():
    vals = torch.tensor([1, 2, 3, 4, 5, 6, 7, 8, 9, 9, 10, 11, 12]).cuda()
    offs = [torch.tensor([0, 2, 2, 3, 6]).cuda(), torch.tensor([0, 2, 4, 6, 9, 11, 13]).cuda()]
    got = ops.ragged_to_dense(vals, offs, 0)
    assert got.tolist() == [[[1, 2, 0], [3, 4, 0], [0, 0, 0]], [[0, 0, 0], [0, 0, 0], [0, 0, 0]],
                            [[5, 6, 0], [0, 0, 0], [0, 0, 0]], [[7, 8, 9], [9, 10, 0], [11, 12, 0]]]
    wide = ops.ragged_to_dense(vals, offs, -1, widths=[4, 2])   # padded / cut to the caller's shape
    assert wide.shape == (4, 4, 2) and wide[3].tolist() == [[7, 8], [9, 10], [11, 12], [-1, -1]]


@pytest.mark.parametrize("np_dtype", [np.float32, np.float64, np.int32, np.int64])
def test_dense_to_ragged_matches_oracle(rng, np_dtype):
    for rows, cols in ((2, 5), (5000, 37), (3, 300), (0, 4), (7, 0)):
        data = rng.integers(0, 3, (rows, cols)).astype(np_dtype)
        if rows > 2:
            data[2] = 0
        for invalid in (0, 1):
            v, o = ops.dense_to_ragged(torch.from_numpy(data).cuda(), True, invalid)
            ev, eo = oracle.dense_to_ragged(data, invalid)
            np.testing.assert_array_equal(v.cpu().numpy(), ev)
            np.testing.assert_array_equal(o.cpu().numpy(), eo)
            assert o.dtype == torch.int32
    # tests/ops/dense_to_ragged_test.py:6-27,58-75
    v, o = ops.dense_to_ragged(torch.tensor([[1.0, 0, 3, 0, 0], [6, 7, 8, 0, 0]]).cuda(), True, 0)
    assert v.tolist() == [1, 0, 3, 6, 7, 8] and o.tolist() == [0, 3, 6]
    d = torch.tensor([[1, 2, 3, 0, 0], [6, 7, 8, 0, 0]], dtype=torch.int32).cuda()
    v, o = ops.dense_to_ragged(d, False, 0)
    assert torch.equal(v, d.view(-1)) and o.tolist() == [0, 5, 10]
    assert _lib.poll_device_errors() == 0


# ------------------------------------------------------------------ feature-engine surface
def test_sequence_truncate_op_and_engine_fusion():
    from recis_amd.features import Feature, FeatureEngine, SelectField, SequenceTruncate
    from recis_amd.ragged.tensor import RaggedTensor

    # tests/feature_engine/op_test.py:66-93
    data = RaggedTensor(torch.randn(512), [torch.tensor([0, 256, 512], dtype=torch.int32),
                                           torch.arange(0, 513, dtype=torch.int32)],
                        dense_shape=(2, 256, 1)).cuda()
    with pytest.raises(AssertionError):
        SequenceTruncate(seq_len=128, check_length=True)(data)
    flat = RaggedTensor(torch.randn(512), [torch.tensor([0, 256, 512], dtype=torch.int32)]).cuda()
    out = SequenceTruncate(seq_len=128, check_length=False, truncate=True, truncate_side="left")(flat)
    assert out.offsets()[-1].tolist() == [0, 128, 256]
    assert torch.equal(out.values(), torch.cat([flat.values()[128:256], flat.values()[384:512]]))
    assert out.dense_shape[1] == 128

    # tests/feature_engine/fused_op_test.py:81-150: several features through the engine (one fused
    # launch per dtype and dimensionality) against each op on its own
    feats, batch, single = [], {}, {}
    for i in range(6):
        dtype = torch.long if i % 2 == 0 else torch.float
        op2 = SequenceTruncate(seq_len=2 + i % 3, check_length=False, truncate_side="left" if i < 3 else "right",
                               n_dims=2, dtype=dtype)
        op3 = SequenceTruncate(seq_len=1 + i % 3, check_length=False, truncate_side="left", n_dims=3, dtype=dtype)
        x2 = RaggedTensor(torch.tensor([1, 2, 3, 4, 5, 6, 7, 8, 9, 10], dtype=dtype),
                          torch.tensor([0, 4, 7, 10]).int()).cuda()
        x3 = RaggedTensor(torch.tensor([1, 2, 3, 4, 5, 6, 7, 8], dtype=dtype),
                          [torch.tensor([0, 2, 3]).int(), torch.tensor([0, 3, 5, 8]).int()]).cuda()
        for tag, op, x in (("a", op2, x2), ("b", op3, x3)):
            name = "%s%d" % (tag, i)
            batch[name] = x
            single[name] = op(x)
            feats.append(Feature(name).add_op(SelectField(name)).add_op(
                SequenceTruncate(**{k: v for k, v in op._get_config().items() if k != "dtype"}, dtype=dtype)))
    outs = FeatureEngine(feats)(batch)
    for name, exp in single.items():
        got = outs[name]
        assert torch.equal(got.values(), exp.values()), name
        assert all(torch.equal(a, b) for a, b in zip(got.offsets(), exp.offsets())), name
        assert got.dense_shape == exp.dense_shape
    x3 = single["b2"]     # keep 3 inner rows of sequences with 2 and 1 rows: padded at the end
    assert x3.offsets()[0].tolist() == [0, 3, 6] and x3.offsets()[1].tolist() == [0, 3, 5, 5, 8, 8, 8]


def test_ragged_tensor_dense_round_trip():
    from recis_amd.ragged.tensor import RaggedTensor

    dense = torch.tensor([[1, 2, 0], [3, 4, 5], [6, 0, 0]]).cuda()
    r = RaggedTensor.from_dense(dense)      # recis/ragged/tensor.py:277-294
    assert r.values().tolist() == [1, 2, 3, 4, 5, 6] and r.offsets()[0].tolist() == [0, 2, 5, 6]
    assert torch.equal(r.to_dense(), dense)
    assert r.to_dense(default_value=-1).tolist() == [[1, 2, -1], [3, 4, 5], [6, -1, -1]]


# ------------------------------------------------------------------ feature cross
@pytest.mark.parametrize("off_dtype", [np.int32, np.int64])
@pytest.mark.parametrize("w_dtype", [np.float32, np.float64, None])
def test_feature_cross_matches_oracle(rng, off_dtype, w_dtype):
    for rows, max_len, key_range in ((2000, 10, 6), (300, 70, 40), (5000, 1, 1000), (50, 0, 5)):
        xo, yo = _ragged(rng, rows, max_len, off_dtype), _ragged(rng, rows + 3, max_len, off_dtype)
        xv, yv = rng.integers(-key_range, key_range, int(xo[-1])), rng.integers(-key_range, key_range, int(yo[-1]))
        xw = None if w_dtype is None else rng.random(int(xo[-1])).astype(w_dtype)
        yw = None if w_dtype is None else rng.random(int(yo[-1])).astype(w_dtype)
        dev = lambda a: None if a is None else torch.from_numpy(a).cuda()
        v, o, w = ops.feature_cross_ragged(dev(xv), dev(xo), dev(xw), dev(yv), dev(yo), dev(yw))
        ev, eo, ew = oracle.feature_cross_ragged(xv, xo, xw, yv, yo, yw)
        np.testing.assert_array_equal(o.cpu().numpy(), eo)
        np.testing.assert_array_equal(v.cpu().numpy(), ev)
        np.testing.assert_array_equal(w.cpu().numpy(), ew)     # one product of two stored weights: exact
        assert o.dtype == torch.from_numpy(xo).dtype
    assert _lib.poll_device_errors() == 0


def test_feature_cross_op_kat():
    # tests/feature_engine/op_test.py:39-63
    from recis_amd.features import FeatureCross
    from recis_amd.ragged.tensor import RaggedTensor

    x = RaggedTensor(torch.tensor([1001, 1002, 1003]), torch.tensor([0, 1, 2, 3]).int(), torch.ones(3)).cuda()
    y = RaggedTensor(torch.tensor([1, 2, 3]), torch.tensor([0, 1, 2, 3]).int(), torch.ones(3)).cuda()
    out = FeatureCross()([x, y])
    assert out.values().tolist() == [-7808879811642834040, -4967483181219983279, 1752425377096056168]
    assert out.offsets()[-1].tolist() == [0, 1, 2, 3] and out.weight().tolist() == [1.0, 1.0, 1.0]


# ------------------------------------------------------------------ top-k index selection
def test_calc_ragged_index_reference_example():
    # tests/ops/ragged_topk_index_cutoff_test.py:9-22
    from recis_amd.nn.functional.ragged_ops import ragged_topk_index_cutoff
    c = lambda t: t.cuda()
    idx, off = ragged_topk_index_cutoff(c(torch.tensor([5, 0, 0])), c(torch.tensor([0, 0, 0])), torch.tensor(True),
                                        torch.tensor(False), c(torch.tensor([0, 8, 10, 13], dtype=torch.int32)),
                                        c(torch.tensor([[1, 2], [0, 2], [0, 1]])), c(torch.tensor([0, 1, 2])))
    assert idx.tolist() == [6, 7, 8, 10, 11] and off.tolist() == [0, 2, 3, 5]
    assert idx.dtype == torch.int64 and off.dtype == torch.int32
    for drop_side, pad_side in ((True, True), (False, True), (False, False)):  # calc_ragged_index.cc:100-127
        with pytest.raises(RuntimeError, match="not supported"):
            ragged_topk_index_cutoff(c(torch.tensor([5, 0, 0])), None, torch.tensor(drop_side), torch.tensor(pad_side),
                                     c(torch.tensor([0, 8, 10, 13])), c(torch.tensor([[1, 2]])), c(torch.tensor([0])))


@pytest.mark.parametrize("off_dtype,topk_dtype,ind_dtype,drop_dtype",
                         [(np.int32, np.int64, np.int64, np.int64), (np.int64, np.int32, np.int32, np.int32),
                          (np.int32, np.int32, np.int64, np.int32), (np.int64, np.int64, np.int32, np.int64)])
def test_calc_ragged_index_matches_oracle(rng, off_dtype, topk_dtype, ind_dtype, drop_dtype):
    side = (torch.tensor(True), torch.tensor(False))
    for src_rows, rows, cols, max_len in ((50, 70, 5, 9), (3000, 5000, 70, 100), (40, 0, 3, 5), (10, 30, 0, 5),
                                          (200, 4100, 1, 3), (500, 300, 200, 150)):
        offset = _ragged(rng, src_rows, max_len, off_dtype)
        drop = rng.integers(0, max_len // 2 + 1, src_rows).astype(drop_dtype)
        ind = rng.integers(0, src_rows, rows).astype(ind_dtype)
        topk = rng.integers(-3, max_len + 3, (rows, cols)).astype(topk_dtype)
        dev = lambda a: torch.from_numpy(a).cuda()
        idx, off = ops.calc_ragged_index(dev(drop), None, *side, dev(offset), dev(topk), dev(ind))
        e_idx, e_off = oracle.calc_ragged_index(drop, offset, topk, ind)
        np.testing.assert_array_equal(off.cpu().numpy(), e_off)
        np.testing.assert_array_equal(idx.cpu().numpy(), e_idx)
        assert idx.cpu().numpy().dtype == topk_dtype and off.cpu().numpy().dtype == off_dtype
    assert _lib.poll_device_errors() == 0


def test_calc_ragged_index_on_a_sequence_batch(rng):
    """Behaviour-sequence shape: 8192 sequences of up to 1000 elements cut to their last 200, top 50
    picked per sequence. Every kept index lies inside its row's kept part, rows are in column order."""
    rows, keep, k = 8192, 200, 50
    lens = np.minimum(rng.lognormal(4.8, 0.9, rows).astype(np.int64) + 1, 1000)
    offset = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    drop = np.maximum(lens - keep, 0)
    topk = np.stack([rng.permutation(keep)[:k] for _ in range(rows)])
    ind = np.arange(rows)
    dev = lambda a: torch.from_numpy(a).cuda()
    idx, off = ops.calc_ragged_index(dev(drop), None, torch.tensor(True), torch.tensor(False), dev(offset), dev(topk),
                                     dev(ind))
    e = topk + (offset[:-1].astype(np.int64) + drop)[:, None]
    keep_mask = e < offset[1:, None]
    np.testing.assert_array_equal(off.cpu().numpy(), np.concatenate([[0], np.cumsum(keep_mask.sum(1))]))
    np.testing.assert_array_equal(idx.cpu().numpy(), e[keep_mask])
    assert _lib.poll_device_errors() == 0


def test_calc_ragged_index_flags_a_bad_indicator():
    dev = lambda *v, dt=torch.int64: torch.tensor(v, dtype=dt).cuda()
    idx, off = ops.calc_ragged_index(dev(0, 0), None, torch.tensor(True), torch.tensor(False), dev(0, 2, 4),
                                     torch.tensor([[0, 1], [0, 1]]).cuda(), dev(1, 7))
    assert idx.tolist() == [2, 3] and off.tolist() == [0, 2, 2]
    assert _lib.poll_device_errors() != 0
    assert _lib.poll_device_errors() == 0


def test_ragged_to_sparse_on_device(rng):
    from recis_amd.nn.functional.ragged_ops import ragged_to_sparse
    from recis_amd.ragged.tensor import RaggedTensor
    for levels in (1, 2):
        offsets, n = [], 300
        for _ in range(levels):
            offsets.append(_ragged(rng, n, 4, np.int32))
            n = int(offsets[-1][-1])
        values = rng.integers(1, 1000, n)
        sp = ragged_to_sparse(torch.from_numpy(values).cuda(), [torch.from_numpy(o).cuda() for o in offsets])
        assert sp.is_cuda
        np.testing.assert_array_equal(sp.indices().cpu().numpy(), oracle.ragged_to_sparse_indices(offsets))
        np.testing.assert_array_equal(sp.to_dense().cpu().numpy(), oracle.ragged_to_dense(values, offsets, 0))
        rt = RaggedTensor(torch.from_numpy(values).cuda(), [torch.from_numpy(o).cuda() for o in offsets])
        assert torch.equal(rt.to_sparse().to_dense(), sp.to_dense())


def test_engine_cross_of_selected_fields_and_topk_after_truncation(rng):
    """Two chains through the FeatureEngine: SelectFields -> FeatureCross, and a fused 2-D
    SequenceTruncate whose recorded drop counts feed the top-k index selection
    (fused_op_impl.py:406-411, ragged_ops.py:717-787)."""
    from recis_amd.features import Feature, FeatureEngine, FeatureCross, SelectField, SelectFields, SequenceTruncate
    from recis_amd.nn.functional.ragged_ops import ragged_topk_index_cutoff
    from recis_amd.ragged import RaggedPadInfo, RaggedTensor

    rows, keep = 300, 6
    xo, yo, so = (_ragged(rng, rows, 12, np.int32) for _ in range(3))
    xv, yv = rng.integers(0, 9, int(xo[-1])), rng.integers(0, 9, int(yo[-1]))
    sv = rng.integers(0, 1 << 40, int(so[-1]))
    dev = lambda a: torch.from_numpy(a).cuda()
    data = {"x": RaggedTensor(dev(xv), dev(xo)), "y": RaggedTensor(dev(yv), dev(yo)), "s": RaggedTensor(dev(sv), dev(so))}
    engine = FeatureEngine([
        Feature("xy").add_op(SelectFields([SelectField("x"), SelectField("y")])).add_op(FeatureCross()),
        Feature("s_cut").add_op(SelectField("s")).add_op(SequenceTruncate(seq_len=keep, check_length=False,
                                                                          truncate=True, truncate_side="left")),
    ])
    out = engine(data)
    ev, eo, _ = oracle.feature_cross_ragged(xv, xo, None, yv, yo, None)
    np.testing.assert_array_equal(out["xy"].values().cpu().numpy(), ev)
    np.testing.assert_array_equal(out["xy"].offsets()[-1].cpu().numpy(), eo)

    cut = out["s_cut"]
    info = cut.pad_info
    assert isinstance(info, RaggedPadInfo) and bool(info.drop_sides) and not bool(info.pad_sides)
    lens = np.diff(so)
    np.testing.assert_array_equal(info.drop_nums.cpu().numpy(), np.maximum(lens - keep, 0))
    # positions 0..keep-1 of the truncated rows, as indices into the ORIGINAL values
    topk = np.tile(np.arange(keep), (rows, 1))
    idx, off = ragged_topk_index_cutoff(info.drop_nums, info.pad_nums, info.drop_sides, info.pad_sides, dev(so),
                                        dev(topk), torch.arange(rows).cuda())
    np.testing.assert_array_equal(off.cpu().numpy(), cut.offsets()[-1].cpu().numpy())
    np.testing.assert_array_equal(sv[idx.cpu().numpy()], cut.values().cpu().numpy())


def test_ragged_tensor_shape_accessors():
    from recis_amd.ragged import RaggedTensor
    rt = RaggedTensor(torch.arange(6), [torch.tensor([0, 2, 5, 6], dtype=torch.int32)]).cuda()
    assert rt.dim == 2 and rt.dense_shape == (3, -1)
    assert rt.shape == (3, 3) and rt.size() == (3, 3) and rt.max_length == 3 and rt.real_shape(0, -1) == (3,)
    rt.set_dim_by_rank(8, 1)
    assert rt.shape == (3, 8) and rt.get_shape(1) == 8
    deep = RaggedTensor(torch.arange(11), [torch.tensor([0, 2, 5, 6]), torch.tensor([0, 1, 3, 6, 8, 10, 11])]).cuda()
    assert deep.dim == 3 and deep.shape == (3, 3, 3) and deep.real_shape(0, -1) == (3, 3)
    host = RaggedTensor.from_numpy(np.arange(6), np.array([0, 2, 5, 6], np.int32))
    assert host.values().tolist() == list(range(6)) and host.pin_memory().values().is_pinned()
    assert "dense_shape=(3, -1)" in str(host)
    from recis_amd.features import SequenceTruncate
    with pytest.raises(AssertionError, match="sequence length"):
        SequenceTruncate(seq_len=2, check_length=True)(RaggedTensor(
            torch.arange(6).cuda(), [torch.tensor([0, 2, 5, 6], dtype=torch.int32).cuda()]))

"""Sequence ops on ragged tensors, the mirror of ``recis.nn.functional.ragged_ops``
(ragged_ops.py:11-420): truncation of lists of 2-D / 3-D ragged tensors and the
dense <-> ragged conversions."""
from typing import List, Optional

import torch

from ... import ops


def dense_to_ragged(tensor: torch.Tensor, check_invalid: bool = True, invalid_value=0):
    """(values, [offsets]) with the trailing ``invalid_value`` run of every row removed
    (ragged_ops.py:11-49)."""
    values, offsets = ops.dense_to_ragged(tensor, check_invalid, invalid_value)
    return values, [offsets]


def ragged_to_dense(values: torch.Tensor, offsets: List[torch.Tensor], default_value=0):
    return ops.ragged_to_dense(values, offsets, default_value)


def fused_ragged_cutoff_2D(values: List[torch.Tensor], offsets: List[torch.Tensor], keep_lengths,
                           drop_sides, pad_sides):
    """ragged_ops.py:305-420. Returns (values, offsets, drop_nums, pad_nums, drop_sides, pad_sides)."""
    if len(values) != len(offsets):
        raise ValueError("Length of 'offsets' list (%d) must match length of 'values' list (%d)"
                         % (len(offsets), len(values)))
    for name, t in (("drop_sides", drop_sides), ("pad_sides", pad_sides)):
        if torch.is_tensor(t) and t.dtype != torch.bool:
            raise ValueError("'%s' must be of type torch.bool, but got %s." % (name, t.dtype))
    return ops.fused_ragged_cutoff(values, offsets, keep_lengths, drop_sides, pad_sides)


def _fused_ragged_cutoff_3D(values: List[torch.Tensor], outer_offsets: List[torch.Tensor],
                            inner_offsets: List[torch.Tensor], keep_lengths,
                            drop_sides: Optional[torch.Tensor] = None, pad_sides: Optional[torch.Tensor] = None):
    """ragged_ops.py:164-302: default drop right, pad right."""
    if drop_sides is None:
        drop_sides = [False] * len(values)
    if pad_sides is None:
        pad_sides = [False] * len(values)
    if len(outer_offsets) != len(values) or len(outer_offsets) != len(inner_offsets):
        raise ValueError("Length of 'offsets' list (%d) must match length of 'values' list (%d) and "
                         "'inner_offsets' (%d)" % (len(outer_offsets), len(values), len(inner_offsets)))
    for name, t in (("drop_sides", drop_sides), ("pad_sides", pad_sides)):
        if torch.is_tensor(t) and t.dtype != torch.bool:
            raise ValueError("'%s' must be of type torch.bool, but got %s." % (name, t.dtype))
    return ops.fused_ragged_cutoff_3D(values, outer_offsets, inner_offsets, keep_lengths, drop_sides, pad_sides)


def fused_ragged_cutoff_3D(values: List[torch.Tensor], offsets: List[List[torch.Tensor]], keep_lengths,
                           drop_sides=None, pad_sides=None):
    """ragged_ops.py:105-161: ``offsets[t] = [outer, inner]``; returns (values, [[outer, inner], ...])."""
    vals, outer, inner = _fused_ragged_cutoff_3D(values, [o[0] for o in offsets], [o[1] for o in offsets],
                                                 keep_lengths, drop_sides, pad_sides)
    return vals, [[outer[i], inner[i]] for i in range(len(outer))]


def feature_cross_ragged(x_value, x_offsets, y_value, y_offsets, x_weight=None, y_weight=None):
    """ragged_ops.py:445-540: (values, offsets, weights) of the per-segment cross of x and y."""
    return ops.feature_cross_ragged(x_value, x_offsets, x_weight, y_value, y_offsets, y_weight)


def ragged_topk_index_cutoff(drop_num, pad_num, drop_side, pad_side, offset, topk_index, indicator):
    """ragged_ops.py:719-787: indices into the values (and their offsets per row) of the elements
    that ``topk_index`` picks out of rows truncated on the left by ``drop_num``."""
    return ops.calc_ragged_index(drop_num, pad_num, drop_side, pad_side, offset, topk_index, indicator)


def ragged_to_sparse(values: torch.Tensor, row_splits: List[torch.Tensor]):
    """ragged_ops.py:52-100 / csrc/ops/ragged_to_sparse.cc:43-91: the ragged tensor as a coalesced
    sparse COO tensor of shape [rows, longest row of level 0, ..., longest row of the last level];
    coordinate k of a value is its position inside the row of level k - 1 that holds it. Works on
    the device of the inputs (the reference has a CPU operator only)."""
    if not row_splits:
        raise RuntimeError("ragged_to_sparse: needs at least one level of offsets")
    if any(o.dtype != row_splits[0].dtype or o.dtype not in (torch.int32, torch.int64) for o in row_splits):
        raise RuntimeError("ragged_to_sparse: each offset_splits should be torch::kInt32 or torch::kInt64")
    splits = [o.to(torch.int64) for o in row_splits]
    n = int(splits[-1][-1].item()) if splits[-1].numel() else 0
    shape = [splits[0].numel() - 1]
    for o in splits:
        shape.append(int((o[1:] - o[:-1]).max().item()) if o.numel() > 1 else 0)
    coords = []
    child = torch.arange(n, device=values.device, dtype=torch.int64)  # index among the rows of the level below
    for o in reversed(splits):
        parent = torch.searchsorted(o, child, right=True) - 1  # the row of this level that holds `child`
        coords.append(child - o[parent])
        child = parent
    coords.append(child)
    indices = torch.stack(coords[::-1]) if n else torch.empty((len(splits) + 1, 0), dtype=torch.int64,
                                                              device=values.device)
    return torch.sparse_coo_tensor(indices, values[:n], shape + list(values.shape[1:])).coalesce()


class RaggedTile(torch.autograd.Function):
    """ragged_ops.py:623-656: for several features at once, the first ``seq[f]`` rows
    ``table[indices[...]]`` of every sample, zero padded; the backward adds the row gradients up."""

    @staticmethod
    def forward(ctx, batch: List[int], seq: List[int], indices: torch.Tensor, offset: torch.Tensor,
                table: torch.Tensor):
        out, batch_seq = ops.ragged_tile(batch, seq, indices, offset, table)
        ctx.save_for_backward(indices, offset)
        ctx.batch_seq = batch_seq
        ctx.batch_info = (table.shape[0], len(batch), max(batch), min(seq))
        return out

    @staticmethod
    def backward(ctx, dy):
        indices, offset = ctx.saved_tensors
        dx = ops.ragged_tile_back(ctx.batch_seq, ctx.batch_info, indices, offset, dy.contiguous())
        return None, None, None, None, dx


def check_para(batch: List[int], seq: List[int], indices: torch.Tensor, offset: torch.Tensor, table: torch.Tensor,
               check_enable: bool):
    """ragged_ops.py:694-714 (reads two values back when enabled)."""
    if not check_enable:
        return
    assert len(batch) == len(seq)
    assert indices.max().item() < table.shape[0]
    assert offset[-1].item() <= len(indices)
    assert indices.dtype in (torch.int, torch.long)
    assert offset.dtype in (torch.int, torch.long)
    assert table.dtype in (torch.float,)
    assert indices.is_cuda and offset.is_cuda and table.is_cuda
    assert table.is_contiguous()


def ragged_tile(batch: List[int], seq: List[int], indices: torch.Tensor, offset: torch.Tensor, table: torch.Tensor,
                check_enable: bool = False):
    """ragged_ops.py:659-691."""
    check_para(batch, seq, indices, offset, table, check_enable)
    return RaggedTile.apply(batch, seq, indices, offset, table)

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

"""``RaggedTensor``: values + one offsets tensor per ragged dimension (+ optional
per-value weight), the container of ``recis.ragged.tensor`` (tensor.py:41-541)
reduced to what the embedding path reads."""
from dataclasses import dataclass
from typing import List, Optional, Union

import torch


@dataclass
class RaggedPadInfo:
    """What a truncation dropped and padded per row (tensor.py:8-38): the input of the top-k
    index selection that follows a truncated sequence."""

    drop_nums: List[torch.Tensor] = None
    pad_nums: List[torch.Tensor] = None
    drop_sides: torch.Tensor = None
    pad_sides: torch.Tensor = None


class RaggedTensor:
    def __init__(self, values: torch.Tensor, offsets: Union[torch.Tensor, List[torch.Tensor]],
                 weight: Optional[torch.Tensor] = None, dense_shape=None):
        if isinstance(offsets, torch.Tensor):
            offsets = [offsets]
        if not offsets:
            raise ValueError("RaggedTensor needs at least one offsets tensor")
        self._values = values
        self._offsets = list(offsets)
        self._weight = weight
        if dense_shape is None:
            # rows = outermost offsets, one trailing ragged dimension per offsets tensor
            dense_shape = tuple([self._offsets[0].numel() - 1] + [-1] * len(self._offsets))
        self._dense_shape = tuple(dense_shape)
        self._pad_info = None

    @property
    def pad_info(self):
        return self._pad_info

    def set_pad_info(self, pad_info: RaggedPadInfo):
        self._pad_info = pad_info

    def values(self):
        return self._values

    def offsets(self):
        return self._offsets

    def weight(self):
        return self._weight

    def set_values(self, values):
        self._values = values

    def set_weight(self, weight):
        self._weight = weight

    def set_offsets(self, offsets):
        self._offsets = [offsets] if isinstance(offsets, torch.Tensor) else list(offsets)

    @property
    def dense_shape(self):
        return self._dense_shape

    def set_dim_by_rank(self, dim, rank):
        shape = list(self._dense_shape)
        shape[rank] = dim
        self._dense_shape = tuple(shape)

    def get_shape(self, dim):
        """Extent of dimension ``dim``: the stated one, else the row count (dim 0) or the longest
        row of that ragged level, which is read back from the device (tensor.py:205-227). The
        reference resolves every unknown extent when the tensor is built; here that happens on
        demand, so building a RaggedTensor never waits for the device."""
        if self._dense_shape[dim] != -1:
            return self._dense_shape[dim]
        if dim < 0:
            dim += len(self._dense_shape)
        if dim == 0:
            return self._offsets[0].numel() - 1
        off = self._offsets[dim - 1]
        if off.numel() < 2:
            return 0
        return int((off[1:] - off[:-1]).max().item())

    def real_shape(self, start=0, end=None):
        """Extents of dimensions [start, end) with unknown ones resolved (tensor.py:174-203)."""
        n = len(self._dense_shape)
        if end is None:
            end = n
        if end < 0:
            end += n
        return tuple(self.get_shape(i) for i in range(start, end))

    @property
    def max_length(self):
        return self.get_shape(-1)

    @property
    def shape(self):
        return self.real_shape()

    def size(self):
        return self.real_shape()

    @staticmethod
    def from_numpy(values, offsets):
        import numpy as np

        if isinstance(offsets, np.ndarray):
            offsets = [offsets]
        return RaggedTensor(torch.from_numpy(values), [torch.from_numpy(o) for o in offsets])

    def pin_memory(self):
        return RaggedTensor(self._values.pin_memory(), [o.pin_memory() for o in self._offsets],
                            None if self._weight is None else self._weight.pin_memory(), self._dense_shape)

    @property
    def device(self):
        return self._values.device

    @property
    def dtype(self):
        return self._values.dtype

    def to(self, *args, **kwargs):
        return RaggedTensor(self._values.to(*args, **kwargs), [o.to(*args, **kwargs) for o in self._offsets],
                            None if self._weight is None else self._weight.to(*args, **kwargs),
                            self._dense_shape)

    def cuda(self):
        return self.to("cuda")

    def cpu(self):
        return self.to("cpu")

    def clone(self):
        return RaggedTensor(self._values.clone(), [o.clone() for o in self._offsets],
                            None if self._weight is None else self._weight.clone(), self._dense_shape)

    @property
    def dim(self):
        return len(self._dense_shape)

    def to_dense(self, default_value=0):
        """Dense ``[rows, longest row of every ragged level]`` (tensor.py:229-248)."""
        from .. import ops

        return ops.ragged_to_dense(self._values, self._offsets, default_value)

    def to_sparse(self):
        """Coalesced sparse COO tensor of the ragged values (tensor.py:296-309)."""
        from ..nn.functional.ragged_ops import ragged_to_sparse

        return ragged_to_sparse(self._values, self._offsets)

    @staticmethod
    def from_dense(dense: torch.Tensor):
        """Rows up to their last non-zero element (tensor.py:277-294)."""
        from .. import ops

        values, offsets = ops.dense_to_ragged(dense, True, 0)
        return RaggedTensor(values, offsets, dense_shape=tuple(dense.shape))

    def __repr__(self):
        return "RaggedTensor(values=%s, offsets=%s, weight=%s)" % (
            tuple(self._values.shape), [tuple(o.shape) for o in self._offsets],
            None if self._weight is None else tuple(self._weight.shape))

    def __str__(self):
        return ("RaggedTensor(\n  values=%s,\n  offsets=%s,\n  weight=%s,\n  dense_shape=%s,\n  dtype=%s,\n"
                "  device=%s\n)" % (self._values, self._offsets, self._weight, self._dense_shape,
                                    self._values.dtype, self._values.device))

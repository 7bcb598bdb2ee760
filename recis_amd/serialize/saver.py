"""Saver: writes tables and dense tensors as a checkpoint directory
(recis/serialize/saver.py:6-78 over csrc/serialize/{saver,write_block,save_bundle}.cc).

Device side of a table block: the key -> row snapshot is split by child on the GPU, the keys go
to the host once, and every slot is gathered ``RECIS_BLOCK_WRITE_SIZE`` rows at a time
(``block_gather`` by range) into one of two pinned host buffers, so the copy of one piece
overlaps the file write of the piece before it."""
import torch

from . import format as fmt
from .. import _lib


class HTSlotWriteBlock(fmt.WriteBlock):
    """Rows ``index`` of one slot (write_block.cc:150-199)."""

    def __init__(self, tensor_name, slice_info, index, slot):
        shape = [index.numel()] + slot.row_shape()
        super().__init__(tensor_name, slice_info, False, _lib.as_dtype(slot.dtype()), shape)
        self._index, self._slot = index, slot

    def chunks(self):
        n, step = self._index.numel(), fmt.block_write_size()
        if n == 0:
            return
        row_shape = self.shape[1:]
        bufs = [torch.empty([min(step, n)] + row_shape, dtype=self.dtype, pin_memory=True) for _ in range(2)]
        events = [torch.cuda.Event(), torch.cuda.Event()]
        device = self._index.device
        with torch.cuda.device(device):
            pending = None
            for k, beg in enumerate(range(0, n, step)):
                end = min(beg + step, n)
                rows = self._slot.index_select(self._index, beg, end)
                buf = bufs[k & 1][: end - beg]
                buf.copy_(rows, non_blocking=True)
                events[k & 1].record()
                if pending is not None:
                    events[pending[0]].synchronize()
                    yield pending[1].reshape(-1).view(torch.uint8).numpy()
                pending = (k & 1, buf)
            events[pending[0]].synchronize()
            yield pending[1].reshape(-1).view(torch.uint8).numpy()


def make_ht_write_blocks(ht):
    """write_block.cc:33-77: per child, the key block then one block per slot, rows in snapshot
    order. Keys of a coalesced table are split by their 12-bit tag and stored without it."""
    ids, index = ht.ids_map()
    info = ht.children_info()
    children = info.children()
    if info.is_coalesce():
        tag = (ids >> info.id_bits_num()) & ((1 << info.index_bits_num()) - 1)
        order = torch.argsort(tag, stable=True)
        counts = torch.bincount(tag, minlength=len(children)).tolist()
        ids = (ids & info.id_mask())[order]
        index = index[order]
        if len(counts) > len(children) and any(counts[len(children):]):
            raise RuntimeError("table holds keys tagged for a child it does not have")
    else:
        counts = [ids.numel()]
    slice_info = fmt.slice_to_string(*ht.slice_info())
    ids_host = ids.cpu()
    blocks, beg = [], 0
    slots = ht.slot_group().slots()
    for c, name in enumerate(children):
        end = beg + int(counts[c])
        blocks.append(fmt.ArrayWriteBlock(name + fmt.INTRA_SEP + fmt.ID_SLOT, slice_info, ids_host[beg:end]))
        for slot in slots:
            blocks.append(HTSlotWriteBlock(name + fmt.INTRA_SEP + slot.name(), slice_info, index[beg:end], slot))
        beg = end
    return blocks


class Saver:
    def __init__(self, shard_index=0, shard_num=1, parallel=8, path=".", hashtables=None, tensors=None,
                 filter_func=lambda x: x):
        self._shard_index, self._shard_num, self._parallel, self._path = shard_index, shard_num, parallel, path
        self._hashtables = hashtables if hashtables is not None else {}
        self._tensors = tensors if tensors is not None else {}
        self._filter_func = filter_func

    def make_write_blocks(self):
        """saver.cc:38-54: table blocks of every table, then (shard 0 only) the dense tensors."""
        blocks = []
        for ht in self._hashtables.values():
            blocks.extend(make_ht_write_blocks(getattr(ht, "_hashtable_impl", ht)))
        if self._shard_index == 0:
            for name, t in self._tensors.items():
                blocks.append(fmt.TensorWriteBlock(name, t))
        return blocks

    def save(self):
        blocks = self._filter_func(self.make_write_blocks())
        bundle = fmt.SaveBundle(self._path, self._parallel, self._shard_index, self._shard_num)
        for b in blocks:
            bundle.add_block(b)
        bundle.save()
        bundle.merge_meta_info()
        if torch.cuda.is_available():
            _lib.raise_device_errors()   # a row index the gathers had to skip means a checkpoint with holes

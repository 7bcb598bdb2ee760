"""Saver: writes tables and dense tensors as a checkpoint directory
(recis/serialize/saver.py:6-78 over ``torch.classes.recis.Saver``, the counterpart of
csrc/serialize/{saver,write_block,save_bundle}.cc in recis.so)."""
import torch


def _impls(hashtables):
    """name -> HashtableImpl for a dict whose values are tables or the modules that hold them."""
    return {k: getattr(v, "_hashtable_impl", v) for k, v in hashtables.items()}


class Saver:
    def __init__(self, shard_index=0, shard_num=1, parallel=8, path=".", hashtables=None, tensors=None,
                 filter_func=lambda x: x):
        from .. import torch_library
        torch_library.load()
        self._shard_index, self._shard_num, self._parallel, self._path = shard_index, shard_num, parallel, path
        self._hashtables = hashtables if hashtables is not None else {}
        self._tensors = tensors if tensors is not None else {}
        self._filter_func = filter_func
        self._saver_impl = torch.classes.recis.Saver(shard_index, shard_num, parallel, path)

    def make_write_blocks(self):
        """saver.cc:38-54: table blocks of every table, then (shard 0 only) the dense tensors."""
        return self._saver_impl.make_write_blocks(_impls(self._hashtables), dict(self._tensors))

    def save(self):
        write_blocks = self._filter_func(self.make_write_blocks())
        self._saver_impl.save(list(write_blocks))

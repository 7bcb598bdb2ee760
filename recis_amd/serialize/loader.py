"""Loader: fills tables and dense tensors from a checkpoint directory
(recis/serialize/loader.py:7-76 over ``torch.classes.recis.Loader``, the counterpart of
csrc/serialize/{loader,load_info,load_internal,read_block,ht_read_collection}.cc in recis.so)."""
import json

import torch

from .saver import _impls


class Loader:
    def __init__(self, checkpoint_path, hashtables=None, tensors=None, parallel=16, filter_func=lambda x: x):
        from .. import torch_library
        torch_library.load()
        self._path = checkpoint_path
        self._hashtables = hashtables if hashtables is not None else {}
        self._tensors = tensors if tensors is not None else {}
        self._parallel = parallel
        self._filter_func = filter_func
        self._impl = torch.classes.recis.Loader(checkpoint_path, parallel, _impls(self._hashtables),
                                                dict(self._tensors))

    def default_load_info(self):
        return self._impl.default_load_info()

    def load(self):
        load_info = self._filter_func(json.loads(self.default_load_info()))
        self._impl.load(json.dumps(load_info))

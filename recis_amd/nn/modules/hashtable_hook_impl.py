"""Hook implementations (``recis.nn.modules.hashtable_hook_impl``): the ReadOnly
admission hook and the last-seen-step eviction filter."""
from typing import Any, Optional, Tuple

import torch

from ... import ops


class HashtableHookFactory:
    """Process-wide registry: hook name -> implementation class, plus the filter
    instances created so far (so a trainer hook can drive them all)."""

    _instance = None

    def __new__(cls):
        if cls._instance is None:
            cls._instance = super().__new__(cls)
            cls._instance._admit = {}
            cls._instance._filter = {}
            cls._instance._filters = {}
        return cls._instance

    def regist_admit(self, name, impl_cls):
        self._admit[name] = impl_cls

    def regist_filter(self, name, impl_cls):
        self._filter[name] = impl_cls

    def create_admit_hook(self, ht, hook):
        if hook.name not in self._admit:
            raise ValueError("unknown admit hook: %s" % hook.name)
        return self._admit[hook.name](ht, **hook.params)

    def create_filter_hook(self, ht, hook):
        if hook.name not in self._filter:
            raise ValueError("unknown filter hook: %s" % hook.name)
        impl = self._filter[hook.name](ht, **hook.params)
        self._filters.setdefault(ht._name, {})[hook.name] = impl
        return impl

    def get_filters(self):
        return self._filters

    def clear_filters(self):
        self._filters.clear()


class BaseAdmitHookImpl:
    """Base of the admission hooks (hashtable_hook_impl.py:193-210)."""

    def __init__(self, **kwargs) -> None:
        pass


class ReadOnlyHookImpl(BaseAdmitHookImpl):
    """Lookups under this hook return zero rows for unknown keys and admit nothing."""

    def __init__(self, ht: Any, **kwargs):
        super().__init__(**kwargs)
        self._ht = ht._hashtable_impl


class BaseFilterHookImpl(torch.nn.Module):
    def __init__(self, ht: Any, name: Optional[str] = None, **kwargs) -> None:
        super().__init__()
        self._ht = ht._hashtable_impl
        self._name = name

    def update(self, index: torch.Tensor) -> None:
        pass

    def do_filter(self) -> None:
        ids, index = self._ht.ids_map()
        delete_ids, delete_index = self.filter(ids, index)
        self._ht.delete(delete_ids, delete_index, self._name)
        self.after_filter(ids, delete_ids)

    def filter(self, ids, index) -> Tuple[torch.Tensor, torch.Tensor]:
        raise NotImplementedError

    def forward(self, index: torch.Tensor) -> None:
        self.update(index)

    def after_filter(self, ids, delete_ids) -> None:
        pass


class GlobalStepFilterHookImpl(BaseFilterHookImpl):
    """Evicts keys whose last-seen step is older than ``filter_step`` steps
    (recis/nn/modules/hashtable_hook_impl.py:389-551): every training lookup stamps
    the looked-up rows of the int64 slot ``name`` with the current step;
    ``do_filter`` removes rows with stamp < global_step - filter_step."""

    def __init__(self, ht: Any, name: str = "step_filter", filter_step: int = 100, **kwargs) -> None:
        super().__init__(ht, name)
        self.register_buffer("_global_step", torch.tensor([0], dtype=torch.int64, device=ht.device))
        assert filter_step > 0, "GlobalStepFilterHookImpl: filter_step must > 0, but get %s" % filter_step
        self._filter_step = filter_step
        self._ht.append_step_filter_slot(self._name, 0)

    def update(self, index: torch.Tensor) -> None:
        self._ht.update_slot(self._name, index, self._global_step)

    def stamp_target(self):
        """(slot name, step tensor) for a lookup that can write the stamps itself, in the pass that
        reads the rows (``ops.plan_expand_rows(stamp=...)``): the same stores as ``update``."""
        return self._name, self._global_step

    def update_step(self, step_size: int = 1) -> None:
        with torch.no_grad():
            self._global_step += step_size

    def _threshold(self) -> int:
        # the counter lives on the device (it is part of the checkpoint and may be loaded or reset
        # behind this object's back); it is read back only here, when a sweep runs
        return int(self._global_step.item()) - self._filter_step

    def do_filter(self) -> None:
        # one pass over the id map instead of snapshot + filter + delete
        self._ht.evict_older(self._name, self._threshold())

    def filter(self, ids, index):
        slot = self._ht.get_slot(self._name)
        chunks, chunk_rows = slot.kernel_blocks()
        mask = ops.block_filter(index, chunks, chunk_rows, self._threshold())
        return torch.masked_select(ids, mask), torch.masked_select(index, mask)

    def __str__(self) -> str:
        return "GlobalStepFilterHookImpl(filter_step=%d, slot_name=%r)" % (self._filter_step, self._name)


HashtableHookFactory().regist_admit("ReadOnly", ReadOnlyHookImpl)
HashtableHookFactory().regist_filter("GlobalStepFilter", GlobalStepFilterHookImpl)

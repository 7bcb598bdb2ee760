"""Trainer-side driver of the table filters (``recis.hooks.filter_hook``): advances
every filter's step after each training step and runs the eviction every
``filter_interval`` steps (recis/hooks/filter_hook.py:82-117)."""
import torch

from ..nn.modules.hashtable_hook_impl import HashtableHookFactory
from .hook import Hook


class HashTableFilterHook(Hook):
    def __init__(self, filter_interval: int = 100):
        self.filter_interval = filter_interval
        self.ht_filters = HashtableHookFactory().get_filters()
        self.last_filter_step = 0

    def reset_filter_interval(self, interval: int = 100):
        self.filter_interval = interval

    def after_step(self, _, gstep):
        gstep = int(gstep.item()) if isinstance(gstep, torch.Tensor) else int(gstep)
        if self.last_filter_step == 0:
            self.last_filter_step = gstep
        exec_filter = self.filter_interval is not None and gstep - self.last_filter_step >= self.filter_interval
        for hooks in self.ht_filters.values():
            for ft in hooks.values():
                ft.update_step()
                if exec_filter:
                    ft.do_filter()
        if exec_filter:
            self.last_filter_step = gstep

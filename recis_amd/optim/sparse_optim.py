"""Python face of the sparse optimizers (``recis.optim``): gradient-accumulation
gating, learning-rate plumbing and state dicts (recis/optim/sparse_optim.py:13-181)
over ``torch.classes.recis.SparseAdam`` / ``SparseAdamW`` / ``SparseAdamWTF`` / ``SparseAdagrad``."""
from torch.optim.optimizer import Optimizer

import torch

from ..nn.modules.hashtable import split_sparse_dense_state_dict


def _classes():
    """``torch.classes.recis``: the optimizers are the native ones of recis.so
    (recis_amd/csrc/torch/sparse_optim.cc), as the reference's are (csrc/bind.cc:112-143)."""
    from .. import torch_library
    torch_library.load()
    return torch.classes.recis


class SparseOptimizer(Optimizer):
    def __init__(self, lr=0.01) -> None:
        self._imp = None
        self._local_step = 0
        self._grad_accum_steps = 1
        super().__init__([{"initial_lr": lr, "lr": lr, "params": []}], defaults={})

    def add_params(self, params: dict):
        self._imp.add_parameters(params)

    def filter_param_dict(self, param_dict):
        out, seen = {}, []
        for key, value in param_dict.items():
            if any(value is v for v in seen):
                continue
            out[key] = value
            seen.append(value)
        return out

    def step(self):
        assert self._grad_accum_steps > 0
        self._local_step += 1
        if self._local_step % self._grad_accum_steps == 0:
            self._imp.set_lr(self.param_groups[0]["lr"])
            self._imp.step()

    def zero_grad(self):
        assert self._grad_accum_steps > 0
        if self._local_step % self._grad_accum_steps == 0:
            self._imp.zero_grad()

    def state_dict(self) -> dict:
        hashtables, steps = self._imp.state_dict()
        ret = {}
        ret.update(hashtables)
        ret.update(steps)
        return ret

    def load_state_dict(self, state_dict: dict):
        hashtables, steps = split_sparse_dense_state_dict(state_dict.copy())
        self._imp.load_state_dict(hashtables, steps)

    def set_grad_accum_steps(self, steps: int):
        self._grad_accum_steps = steps
        self._imp.set_grad_accum_steps(steps)

    def set_lr(self, lr):
        self.param_groups[0]["lr"] = lr


class SparseAdam(SparseOptimizer):
    def __init__(self, param_dict, lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=1e-2, amsgrad=False):
        super().__init__(lr=lr)
        self._imp = _classes().SparseAdam.make(self.filter_param_dict(param_dict), lr, beta1, beta2, eps,
                                                    weight_decay, amsgrad)


class SparseAdamW(SparseOptimizer):
    def __init__(self, param_dict, lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=1e-2, amsgrad=False):
        super().__init__(lr=lr)
        self._imp = _classes().SparseAdamW.make(self.filter_param_dict(param_dict), lr, beta1, beta2, eps,
                                                     weight_decay, amsgrad)


class SparseAdamWTF(SparseOptimizer):
    def __init__(self, param_dict, lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=1e-2,
                 use_nesterov=False):
        super().__init__(lr=lr)
        if use_nesterov:
            raise ValueError("use_nesterov is not support now")
        self._imp = _classes().SparseAdamWTF.make(self.filter_param_dict(param_dict), lr, beta1, beta2, eps,
                                                       weight_decay, use_nesterov)


class SparseAdagrad(SparseOptimizer):
    """Sparse Adagrad (not in the reference, which ships only the Adam family)."""

    def __init__(self, param_dict, lr=1e-2, eps=1e-8):
        super().__init__(lr=lr)
        self._imp = _classes().SparseAdagrad.make(self.filter_param_dict(param_dict), lr, eps)

"""Counterparts of the native sparse optimizers ``torch.classes.recis.SparseAdam``,
``SparseAdamW`` and ``SparseAdamWTF`` (csrc/embedding/adam.cc:55-229, adamw.cc,
adamw_tf.cc; base csrc/embedding/optim.h:85-167), plus ``SparseAdagrad`` (an
addition that follows the same conventions).

State lives in extra slots of the table (same dtype and row shape as the embedding
slot, zero initialised); one fused HIP row kernel updates the touched rows.
"""
import torch

from .. import ops


class _SparseOptimizerImpl:
    prefix = ""

    def __init__(self, hashtables, lr):
        self._lr = float(lr)
        self._grad_accum_steps = 1
        self._params = {}
        self._state = {}
        for name, ht in hashtables.items():
            self._init_param_state(name, ht)
            self._params[name] = ht

    # -- the bound surface (bind.cc:112-143)
    def add_parameters(self, hashtables):
        for name, ht in hashtables.items():
            self._init_param_state(name, ht)
            self._params[name] = ht

    def zero_grad(self):
        for ht in self._params.values():
            ht.clear_grad()

    def set_grad_accum_steps(self, steps):
        self._grad_accum_steps = int(steps)

    def set_lr(self, lr):
        self._lr = float(lr)

    def load_state_dict(self, hashtables, steps):
        # the reference leaves this empty (adam.cc:210-212): slots are restored with the table
        pass

    def step(self):
        with torch.no_grad():
            for name, ht in self._params.items():
                if not ht.has_grad():
                    continue
                planned = ht.take_planned_grad() if self._grad_accum_steps == 1 and hasattr(self, "apply_planned") else None
                if planned is not None:   # the gradient is still a sum to be taken: sum and update in one launch
                    index, plan, rows, src, coef, cover = planned[0]
                    if len(planned) == 1:
                        self.apply_planned(ht, plan, rows, src, coef, index, cover)
                    else:   # two gradients of one plan
                        self.apply_planned2(ht, plan, (rows, src, coef), planned[1][2:5], index)
                    continue
                index, grad = ht.grad_pairs(self._grad_accum_steps)
                self._update(ht, self._state[id(ht)], index, grad)

    def _init_param_state(self, name, ht):
        if id(ht) in self._state:
            raise RuntimeError("some parameters appear in more than one parameter group.")
        self._state[id(ht)] = self._make_state(ht)


class _AdamFamilyImpl(_SparseOptimizerImpl):
    beta_dtype = torch.float32
    beta_shape = ()

    def __init__(self, hashtables, lr, beta1, beta2, eps, weight_decay, flag):
        self._beta1, self._beta2, self._eps, self._weight_decay = float(beta1), float(beta2), float(eps), float(weight_decay)
        super().__init__(hashtables, lr)

    @classmethod
    def make(cls, hashtables, lr, beta1, beta2, eps, weight_decay, flag=False):
        return cls(dict(hashtables), lr, beta1, beta2, eps, weight_decay, flag)

    def _decay(self):
        raise NotImplementedError

    def _make_state(self, ht):
        sg = ht._slot_group
        emb = sg.emb_slot()
        shape = [1] + emb._row_shape
        dev = ht.device
        return dict(
            beta1=torch.ones(self.beta_shape, dtype=self.beta_dtype, device=dev),
            beta2=torch.ones(self.beta_shape, dtype=self.beta_dtype, device=dev),
            step=torch.zeros(1, dtype=torch.int64, device=dev),
            exp_avg=sg.append_slot(self.prefix + "exp_avg", emb.dtype(), shape),
            exp_avg_sq=sg.append_slot(self.prefix + "exp_avg_sq", emb.dtype(), shape),
        )

    def _update(self, ht, st, index, grad):
        emb = ht._slot_group.emb_slot()
        chunks, chunk_rows = emb.kernel_blocks()
        ops.block_apply_adamw(index, grad, chunks, st["beta1"], st["beta2"], st["step"],
                              st["exp_avg"].kernel_blocks()[0], st["exp_avg_sq"].kernel_blocks()[0],
                              self._lr, self._beta1, self._beta2, self._decay(), self._eps, chunk_rows)

    def apply_planned(self, ht, plan, grad_rows, src, coef, index, cover=None):
        """One optimizer step for ``ht`` straight from the gradients of the lookups: the gradient of
        unique id ``u`` of ``plan`` (sum over its occurrence list of ``coef * grad_rows[src]``) is applied
        to row ``index[u]`` as it is summed (``ops.csr_gather_reduce_adamw``); the ``[U, D]`` gradient is
        never written. Same result, bit for bit, as ``accept_grad(index, csr_gather_reduce(...))`` +
        ``step()`` for a table that receives one gradient in the step and no gradient accumulation."""
        st = self._state[id(ht)]
        chunks, chunk_rows = ht._slot_group.emb_slot().kernel_blocks()
        ops.csr_gather_reduce_adamw(grad_rows, plan, src, coef, index, chunks, st["beta1"], st["beta2"],
                                    st["exp_avg"].kernel_blocks()[0], st["exp_avg_sq"].kernel_blocks()[0], self._lr,
                                    self._beta1, self._beta2, self._decay(), self._eps, chunk_rows, cover=cover)

    def apply_planned2(self, ht, plan, first, second, index):
        """``apply_planned`` for a table whose lookup fed two outputs: ``first`` and ``second`` are
        ``(grad_rows, src, coef)`` of the two gradients, summed per unique id in
        one pass (``ops.csr_gather_reduce2_adamw``)."""
        st = self._state[id(ht)]
        chunks, chunk_rows = ht._slot_group.emb_slot().kernel_blocks()
        ops.csr_gather_reduce2_adamw(plan, first, second, index, chunks, st["beta1"], st["beta2"],
                                     st["exp_avg"].kernel_blocks()[0], st["exp_avg_sq"].kernel_blocks()[0], self._lr,
                                     self._beta1, self._beta2, self._decay(), self._eps, chunk_rows)

    def state_dict(self):
        steps = {}
        for st in self._state.values():
            # in the order the reference's map hands them out (its state-dict test lists the keys:
            # tests/hashtable/ht_state_dict_test.py:44-49)
            steps[self.prefix + "beta2"] = st["beta2"]
            steps[self.prefix + "beta1"] = st["beta1"]
            steps[self.prefix + "step"] = st["step"]
        return {}, steps


class SparseAdamImpl(_AdamFamilyImpl):
    """decay multiplier 1 (its weight_decay option is ignored, adam.cc:70-73); running
    beta powers in float64 (adam.h:37)."""
    prefix = "sparse_adam_"
    beta_dtype = torch.float64
    beta_shape = (1,)

    def _decay(self):
        return 1.0


class SparseAdamWImpl(_AdamFamilyImpl):
    """decay multiplier 1 - lr * weight_decay (adamw.cc:64)."""
    prefix = "sparse_adamw_"

    def _decay(self):
        return 1.0 - self._lr * self._weight_decay


class SparseAdamWTFImpl(_AdamFamilyImpl):
    """decay multiplier 1 - weight_decay (adamw_tf.cc:64)."""
    prefix = "sparse_adamw_tf_"

    def _decay(self):
        return 1.0 - self._weight_decay


class SparseAdagradImpl(_SparseOptimizerImpl):
    """s += g^2; w -= lr * g / (sqrt(s) + eps) on the touched rows; state slot
    ``sparse_adagrad_accum``."""
    prefix = "sparse_adagrad_"

    def __init__(self, hashtables, lr, eps):
        self._eps = float(eps)
        super().__init__(hashtables, lr)

    @classmethod
    def make(cls, hashtables, lr, eps=1e-8):
        return cls(dict(hashtables), lr, eps)

    def _make_state(self, ht):
        sg = ht._slot_group
        emb = sg.emb_slot()
        return dict(accum=sg.append_slot(self.prefix + "accum", emb.dtype(), [1] + emb._row_shape))

    def _update(self, ht, st, index, grad):
        chunks, chunk_rows = ht._slot_group.emb_slot().kernel_blocks()
        ops.block_apply_adagrad(index, grad, chunks, st["accum"].kernel_blocks()[0], self._lr, self._eps, chunk_rows)

    def apply_planned(self, ht, plan, grad_rows, src, coef, index, cover=None):
        """The Adagrad step of ``ht`` fused into the gather-reduce of its gradients (see the Adam family)."""
        st = self._state[id(ht)]
        chunks, chunk_rows = ht._slot_group.emb_slot().kernel_blocks()
        ops.csr_gather_reduce_adagrad(grad_rows, plan, src, coef, index, chunks, st["accum"].kernel_blocks()[0],
                                      self._lr, self._eps, chunk_rows, cover=cover)

    def apply_planned2(self, ht, plan, first, second, index):
        """The Adagrad step of ``ht`` fused into the gather-reduce of two gradients (see the Adam family)."""
        st = self._state[id(ht)]
        chunks, chunk_rows = ht._slot_group.emb_slot().kernel_blocks()
        ops.csr_gather_reduce2_adagrad(plan, first, second, index, chunks, st["accum"].kernel_blocks()[0],
                                       self._lr, self._eps, chunk_rows)

    def state_dict(self):
        return {}, {}

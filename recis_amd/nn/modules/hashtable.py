"""Dynamic hash table: host-side mirror of ``recis.nn.modules.hashtable`` and of the
native classes behind it (``HashtableImpl``, ``SlotGroup``, ``Slot``,
``ChildrenInfo``: csrc/embedding/hashtable.cc:46-313, slot_group.cc:26-201,
children_info.h:12-37, registered at csrc/bind.cc:47-109).

The table lives in GPU memory: the key -> row map is the HIP ``IdMap`` and every
slot (the embedding rows, optimizer state, the last-seen step) is EmbeddingBlocks
storage read and written by the HIP row kernels. There is no CPU-resident mode.

Storage layout. The reference grows every slot one ``[block_size, D]`` tensor at a
time. Here a slot is a short list of large chunks, each a whole number of blocks;
``Slot.values()`` still hands out one aliasing ``[block_size, D]`` view per block,
while the kernels address the chunks directly (a chunk is simply a bigger block,
so the row arithmetic ``row // size, row % size`` is the same). Rows are
initialised by the slot's generator when their chunk is allocated.
"""
import json
import os
from typing import List, Optional, Tuple

import torch

from ... import ops
from ..._lib import RecisHipError
from ..hashtable_hook import AdmitHook, FilterHook
from ..initializers import ConstantInitializer


class Slice:
    def __init__(self, slice_begin, slice_end, slice_size):
        self.slice_begin, self.slice_end, self.slice_size = slice_begin, slice_end, slice_size


_default_slice = Slice(0, 65536, 65536)


def gen_slice(shard_index=0, shard_num=1, slice_size=65536):
    """Key-space range of one shard (recis/nn/modules/hashtable.py:48-92): ``slice_size``
    slots split into ``shard_num`` contiguous ranges, the first ``slice_size % shard_num``
    one longer."""
    base, extra = divmod(slice_size, shard_num)
    begin = shard_index * base + min(shard_index, extra)
    return Slice(begin, begin + base + (1 if shard_index < extra else 0), slice_size)


class HashtableRegister:
    """Process-wide registry that rejects two tables with one name and different
    configuration (recis/nn/modules/hashtable.py:674-731)."""

    _instance = None

    def __new__(cls):
        if cls._instance is None:
            cls._instance = super().__new__(cls)
            cls._instance._tables = {}
        return cls._instance

    def register(self, name, info):
        if name in self._tables:
            raise ValueError("duplicate hashtable name: %s" % name)
        self._tables[name] = info

    def clear(self):
        self._tables.clear()


def _recis():
    from ... import torch_library
    torch_library.load()
    return torch.ops.recis


def make_hashtable(block_size, embedding_shape, dtype, device, coalesce, children, generator,
                   slice_begin=0, slice_end=65536, slice_size=65536, reserve_rows=0):
    """``torch.ops.recis.make_hashtable`` (hashtable.h:36-41, bind.cc:145): a
    ``torch.classes.recis.HashtableImpl``, the table object of recis.so
    (recis_amd/csrc/torch/table.cc). ``reserve_rows`` (an addition) pre-sizes the id map and the
    row storage (``HashtableImpl.reserve``)."""
    device = torch.device(device)
    if device.type != "cuda":
        raise RecisHipError("tables live in GPU memory in this build; got device %s" % device)
    if device.index is None:
        device = torch.device("cuda", torch.cuda.current_device())
    impl = _recis().make_hashtable(block_size, list(embedding_shape), dtype, device, bool(coalesce), list(children),
                                   generator, slice_begin, slice_end, slice_size)
    if reserve_rows > 0:
        impl.reserve(int(reserve_rows))
    return impl


HashtableImpl = make_hashtable  # the table class is the native one; this name builds one


def plan_lookup(impl, ids, wait=False, need_inverse=True, need_pos=False, tags=None):
    """Dedup of ``ids`` and find-or-insert of the distinct ids in table ``impl`` in one pass
    (``HashtableImpl.plan_lookup``): the batch plan with ``index_buf`` = the row of every unique id.
    ``ids`` may be a list of id tensors with their table ``tags`` (see ``ops.ids_unique_plan``).
    Replaces ``ids_partition`` / ``torch.unique`` + ``IdMap::Lookup`` of the training lookup
    (recis/nn/modules/hashtable.py:262-293)."""
    jobs = list(ids) if isinstance(ids, (list, tuple)) else [ids]
    return impl.plan_lookup(jobs, None if tags is None else [int(t) for t in tags], bool(wait), bool(need_inverse),
                            bool(need_pos))


def accept_planned_grad(impl, index, plan, rows, src, coef=None, cover=None, key=None, may_miss=False):
    """A gradient handed to table ``impl`` before it is summed (``HashtableImpl.accept_planned_grad``): the
    gradient of ``plan``'s unique id ``u`` (table row ``index[u]``; negative = the table does not hold the key, no
    gradient) is the sum over u's occurrence list of ``coef * rows[src]``; ``rows`` may be a list of arrays laid
    end to end. If it stays the only gradient of the step, or one of the two gradients of one plan (same ``key``),
    the optimizer's ``step()`` sums it and applies the row update in one launch; anything else that asks for the
    gradient gets it summed first."""
    in_parts = not torch.is_tensor(rows)
    impl.accept_planned_grad(index, plan, list(rows) if in_parts else [rows], in_parts, src, coef, cover,
                             0 if key is None else int(key), bool(may_miss))


def is_hashtable(obj):
    return hasattr(obj, "hashtable_tag")


def filter_out_sparse_param(model):
    """name -> HashtableImpl for every table under ``model`` (what the sparse
    optimizers take), mirroring ``recis.nn.modules.hashtable.filter_out_sparse_param``."""
    out = {}
    for module in model.modules():
        if isinstance(module, HashTable):
            out[module._name] = module._hashtable_impl
    return out


def split_sparse_dense_state_dict(state_dict):
    sparse = {k: v for k, v in state_dict.items() if is_hashtable(v)}
    dense = {k: v for k, v in state_dict.items() if not is_hashtable(v)}
    return sparse, dense


# ----------------------------------------------------------------- autograd
class HashTableLookupHelpFunction(torch.autograd.Function):
    """Lookup of unique ids; backward hands (row index, gradient) to the table
    (recis/nn/modules/hashtable.py:425-481)."""

    @staticmethod
    def forward(ctx, ids, hashtable, backward_holder, admit_hook_impl, grad_key=None):
        from .hashtable_hook_impl import ReadOnlyHookImpl

        ctx.grad_key = grad_key if admit_hook_impl is None else None

        assert admit_hook_impl is None or isinstance(admit_hook_impl, ReadOnlyHookImpl), \
            "admit hook only support ReadOnlyHook yet, but got: %s" % admit_hook_impl
        index, embedding = hashtable.embedding_lookup(ids.detach(), admit_hook_impl is not None)
        ctx.save_for_backward(index)
        ctx.hashtable = hashtable
        ctx.mark_non_differentiable(index)
        return index, embedding

    @staticmethod
    def backward(ctx, grad_output_index, grad_output_emb):
        (index,) = ctx.saved_tensors
        ctx.hashtable.accept_grad_ex(index, grad_output_emb.contiguous(), True,
                                     0 if ctx.grad_key is None else int(ctx.grad_key))
        return None, None, None, None, None


class GradIDMeanFunction(torch.autograd.Function):
    """Expand unique rows to request order; backward = mean over the duplicates of
    each id (recis/nn/modules/hashtable.py:484-537)."""

    @staticmethod
    def forward(ctx, embedding, index, plan=None):
        ctx.save_for_backward(index)
        ctx.unique_size = embedding.shape[0]
        ctx.plan = plan
        return ops.gather(index, embedding)

    @staticmethod
    def backward(ctx, grad_outputs):
        (index,) = ctx.saved_tensors
        summed = _scatter_sum(grad_outputs, index, ctx.unique_size, ctx.plan)
        counts = torch.bincount(index.long(), minlength=ctx.unique_size).clamp_(min=1)
        return (summed / counts.view(-1, 1).to(summed.dtype)).to(grad_outputs.dtype), None, None


class GradWorkerMeanFunction(torch.autograd.Function):
    """Expand unique rows to request order; backward = sum over duplicates divided
    by the number of workers (recis/nn/modules/hashtable.py:540-586)."""

    @staticmethod
    def forward(ctx, embedding, index, slice_num, plan=None):
        ctx.save_for_backward(index)
        ctx.unique_size = embedding.shape[0]
        ctx.slice_num = slice_num
        ctx.plan = plan
        return ops.gather(index, embedding)

    @staticmethod
    def backward(ctx, grad_outputs):
        (index,) = ctx.saved_tensors
        if ctx.slice_num != 1:
            grad_outputs = grad_outputs / ctx.slice_num
        return _scatter_sum(grad_outputs, index, ctx.unique_size, ctx.plan).to(grad_outputs.dtype), None, None, None


class LookupExpandFunction(torch.autograd.Function):
    """Dedup, lookup of the unique ids and one output row per request in one pass over the table
    (what HashTableLookupHelpFunction + GradWorkerMeanFunction give, hashtable.py:425-586, without
    the ``[U, D]`` copy of the rows): every unique row is read once and written to its
    occurrences. Backward: sum over the duplicates of each id, divided by the number of workers."""

    @staticmethod
    def forward(ctx, backward_holder, impl, ids, slice_num, readonly, stamp=None, exact_index=False):
        """``stamp`` = (name of the step filter's slot, its one-element step tensor): the rows read
        are stamped in the same pass (what the filter hook's update would do in a launch of its own).
        ``exact_index``: return the rows proper instead of the full-length buffer (waits for the count)."""
        if readonly:
            plan = ops.ids_unique_plan(ids, wait=False, need_inverse=False, need_pos=False)
            index = impl.lookup_index_readonly(plan.unique)
        else:
            # nothing here waits for the unique count: the lookup rides on the plan, the expansion takes
            # the count from device memory, and backward reads it long after it has arrived
            plan = impl.plan_lookup([ids], None, False, False, False)
            index = plan.index_buf   # full length: its first plan.U entries are the rows
        out = impl.expand_rows(plan, index, None, None if stamp is None else stamp[0],
                               None if stamp is None else stamp[1])
        ctx.settled = readonly
        if exact_index and not readonly:
            impl.settle_count(plan.U, plan)
            index = index[: plan.U]
            ctx.settled = True
        ctx.impl, ctx.plan, ctx.slice_num, ctx.readonly = impl, plan, slice_num, readonly
        ctx.save_for_backward(index)
        ctx.mark_non_differentiable(index)
        return index, out

    @staticmethod
    def backward(ctx, _grad_index, grad):
        (index,) = ctx.saved_tensors
        plan = ctx.plan
        flat = grad.reshape(plan.n, -1).contiguous()
        if ctx.slice_num != 1:
            flat = flat / ctx.slice_num
        if not ctx.settled:
            ctx.impl.settle_count(plan.U, plan)
            index = index[: plan.U]
        # the sum over the duplicates of each id is left to the optimizer step where it can be (one launch
        # sums and updates the row); keys the table does not hold (negative index) take no gradient
        accept_planned_grad(ctx.impl, index, plan, flat, plan.occ, may_miss=ctx.readonly)
        return None, None, None, None, None, None, None


def _scatter_sum(grad_rows, index, unique_size, plan=None):
    """sum of ``grad_rows[i]`` into row ``index[i]`` of a ``[unique_size, D]`` result: a
    gather-reduce over the batch plan's occurrence lists when there is one, fp32 atomics else."""
    n = index.numel()
    flat = grad_rows.reshape(n, -1).contiguous()
    if plan is not None:
        out = ops.csr_gather_reduce(flat, plan, plan.occ)
    else:
        span = torch.tensor([0, n], dtype=torch.int64, device=index.device)
        out = ops.segment_reduce_backward(flat, None, index, span, unique_size, "tile", out_dtype=torch.float32)
    return out.view((unique_size,) + tuple(grad_rows.shape[1:]))


# ------------------------------------------------------------------- module
class HashTable(torch.nn.Module):
    """Dynamic embedding table (recis/nn/modules/hashtable.py:98-423).

    ``dedup`` chooses how ``forward`` removes duplicate ids: ``"hash"`` (default) is the
    HIP hash dedup, whose unique ids come in a fixed, input-determined order (hash bucket, then first occurrence); ``"sorted"`` is
    ``torch.unique`` as in the reference, which also makes the row a new key receives
    identical to the reference's (new keys are ranked in ascending key order).
    ``reserve_rows`` pre-sizes the map and the row storage."""

    def __init__(self, embedding_shape: List, block_size: int = 5, dtype: torch.dtype = torch.float32,
                 device: torch.device = torch.device("cuda"), coalesced: bool = False,
                 children: Optional[List[str]] = None, slice: Slice = _default_slice, initializer=None,
                 name: str = "hashtable", grad_reduce_by: str = "worker",
                 filter_hook: Optional[FilterHook] = None, dedup: str = "hash", reserve_rows: int = 0):
        super().__init__()
        from .hashtable_hook_impl import HashtableHookFactory

        self._initializer = ConstantInitializer(init_val=0) if initializer is None else initializer
        if children is None:
            children = [name]
        self._device = torch.device(device)
        assert grad_reduce_by in ["id", "worker"]
        assert dedup in ["hash", "sorted"]
        self._grad_reduce_by = grad_reduce_by
        self._dedup = dedup
        self._initializer.set_shape([block_size] + list(embedding_shape))
        self._initializer.set_dtype(dtype)
        self._initializer.build()
        self._dtype = dtype
        self._name = name
        for child in children:
            info = json.dumps(dict(shape=list(embedding_shape), dtype=str(dtype),
                                   initializer=str(self._initializer)))
            HashtableRegister().register(child, info)
        self._hashtable_impl = make_hashtable(block_size, list(embedding_shape), dtype, self._device, coalesced,
                                              children, self._initializer.impl(), slice.slice_begin,
                                              slice.slice_end, slice.slice_size, reserve_rows)
        self._embedding_shape = list(embedding_shape)
        self._impl_device = self._hashtable_impl.device()
        self._backward_holder = torch.tensor([0.0], requires_grad=True)
        self._worker_num = int(os.environ.get("WORLD_SIZE", 1))

        def state_dict_hook(module, state_dict, prefix, local_metadata):
            state_dict[module._name] = module._hashtable_impl

        self._register_state_dict_hook(state_dict_hook)
        if filter_hook is not None:
            self._filter_hook_impl = HashtableHookFactory().create_filter_hook(self, filter_hook)
        else:
            self._filter_hook_impl = torch.nn.Identity()

    def _unique(self, ids):
        """(unique ids, inverse, batch plan | None)."""
        if self._dedup == "sorted":
            uniq, inverse = ids.unique(return_inverse=True)
            return uniq, inverse, None
        plan = ops.ids_unique_plan(ids, need_pos=False)
        return plan.unique, plan.inverse, plan

    def forward(self, ids: torch.Tensor, admit_hook: AdmitHook = None) -> torch.Tensor:
        from .hashtable_hook_impl import HashtableHookFactory

        admit_hook_impl = HashtableHookFactory().create_admit_hook(self, admit_hook) if admit_hook else None
        shape = tuple(ids.shape)
        ids = ids.to(self._device).reshape(-1)
        if self.training and self._dedup != "sorted" and self._grad_reduce_by != "id" and len(
                self._embedding_shape) == 1 and self._dtype in (torch.float32, torch.bfloat16, torch.float16):
            from .hashtable_hook_impl import ReadOnlyHookImpl

            assert admit_hook_impl is None or isinstance(admit_hook_impl, ReadOnlyHookImpl), \
                "admit hook only support ReadOnlyHook yet, but got: %s" % admit_hook_impl
            if ids.dtype != torch.int64:
                ids = ids.long()
            # a step filter's stamps ride on the pass that reads the rows
            stamp = getattr(self._filter_hook_impl, "stamp_target", lambda: None)()
            # a hook that cannot stamp in that pass gets the rows proper afterwards, which needs the count
            hooked = stamp is None and not isinstance(self._filter_hook_impl, torch.nn.Identity)
            emb_idx, embedding = LookupExpandFunction.apply(self._backward_holder, self._hashtable_impl, ids,
                                                            self._worker_num, admit_hook_impl is not None, stamp, hooked)
            if hooked:
                self._filter_hook_impl(emb_idx)
            return embedding.view(shape + tuple(embedding.shape[1:])) if len(shape) != 1 else embedding
        uids, index, plan = self._unique(ids)
        if self.training and self._dtype not in (torch.int8, torch.int32, torch.int64):
            emb_idx, embedding = HashTableLookupHelpFunction.apply(uids, self._hashtable_impl,
                                                                   self._backward_holder, admit_hook_impl)
            if self._grad_reduce_by == "id":
                embedding = GradIDMeanFunction.apply(embedding, index, plan)
            else:
                embedding = GradWorkerMeanFunction.apply(embedding, index, self._worker_num, plan)
            self._filter_hook_impl(emb_idx)
        else:
            _, embedding = self._hashtable_impl.embedding_lookup(uids.detach(), True)
            embedding = ops.gather(index, embedding)
        return embedding.view(shape + tuple(embedding.shape[1:])) if len(shape) != 1 else embedding

    def initializer(self):
        return self._initializer

    @property
    def device(self):
        return self._device

    @property
    def coalesce(self):
        return self._hashtable_impl.children_info().is_coalesce()

    @property
    def children_hashtable(self):
        return self._hashtable_impl.children_info().children()

    def accept_grad(self, grad_index, grad) -> None:
        self._hashtable_impl.accept_grad(grad_index, grad)

    def grad(self, acc_step=1) -> torch.Tensor:
        return self._hashtable_impl.grad(acc_step)

    def clear_grad(self) -> None:
        self._hashtable_impl.clear_grad()

    def insert(self, ids, embeddings) -> None:
        self._hashtable_impl.insert(ids, embeddings)

    def clear(self) -> None:
        self._hashtable_impl.clear()

    def ids(self) -> torch.Tensor:
        return self._hashtable_impl.ids()

    def ids_map(self) -> Tuple[torch.Tensor, torch.Tensor]:
        return self._hashtable_impl.ids_map()

    def embeddings(self) -> torch.Tensor:
        return self._hashtable_impl.slot_group().slot_by_name("embedding").value()

    def slot_group(self):
        return self._hashtable_impl.slot_group()

    def children_info(self):
        return self._hashtable_impl.children_info()

    def __str__(self) -> str:
        return "HashTable_%s" % self._name

    __repr__ = __str__

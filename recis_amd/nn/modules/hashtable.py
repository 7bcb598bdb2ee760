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

_CHUNK_BYTES = 8 << 20


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


class ChildrenInfo:
    """12-bit table tag / 52-bit id packing for coalesced tables (children_info.h:12-37)."""

    def __init__(self, coalesce, children):
        self._coalesce = bool(coalesce)
        self._children = list(children)
        if len(self._children) > self.max_children_num():
            raise RuntimeError("too many children: %d" % len(self._children))
        if not self._coalesce and len(self._children) != 1:
            raise RuntimeError("a table that is not coalesced has exactly one child")

    def index_bits_num(self):
        return 12

    def id_bits_num(self):
        return 52

    def index_mask(self):
        return -(1 << 52)

    def id_mask(self):
        return (1 << 52) - 1

    def max_children_num(self):
        return 4095

    def encode_id(self, id_, index):
        v = (id_ & self.id_mask()) | ((index << 52) & 0xFFFFFFFFFFFFFFFF)
        return v - (1 << 64) if v >= (1 << 63) else v

    def children(self):
        return list(self._children)

    def child_index(self, name):
        return self._children.index(name)

    def has_child(self, name):
        return name in self._children

    def child_at(self, index):
        return self._children[index]

    def is_coalesce(self):
        return self._coalesce


class Slot:
    """One named column of the table (slot_group.h:17-58)."""

    def __init__(self, name, block_size, dtype, partial_shape, generator, device, chunk_rows):
        self._name = name
        self._block_size = block_size
        self._dtype = dtype
        self._row_shape = list(partial_shape[1:])
        self._generator = generator
        self._device = device
        self._chunk_rows = chunk_rows
        self._chunks = []
        self._visible_blocks = 0
        generator.set_device(device)

    # -- reference surface
    def block_size(self):
        return self._block_size

    def name(self):
        return self._name

    def flat_size(self):
        n = 1
        for d in self._row_shape:
            n *= d
        return n

    def dtype(self):
        return self._dtype

    def values(self):
        """One ``[block_size, D]`` view per block; the views alias live storage."""
        per = self._chunk_rows // self._block_size
        out = []
        for b in range(self._visible_blocks):
            c, k = divmod(b, per)
            out.append(self._chunks[c][k * self._block_size:(k + 1) * self._block_size])
        return out

    def value(self):
        rows = self._visible_blocks * self._block_size
        if rows == 0:
            return torch.empty([0] + self._row_shape, dtype=self._dtype, device=self._device)
        full, rest = divmod(rows, self._chunk_rows)
        parts = self._chunks[:full] + ([self._chunks[full][:rest]] if rest else [])
        return torch.cat(parts, 0)

    def row_shape(self):
        return list(self._row_shape)

    def index_select(self, index, beg=0, end=None):
        end = index.numel() if end is None else end
        return ops.block_gather_by_range(index, self._chunks, self._chunk_rows, beg, end)

    def index_insert(self, index, value, accept_indicator=None):
        if value.dim() == 0:
            value = value.view(1)
        if value.dim() == 1 and self._row_shape == [1]:
            value = value.view(-1, 1)
        value = value.to(device=self._device, dtype=self._dtype)
        if accept_indicator is None:
            ops.block_insert(index, value, self._chunks, self._chunk_rows)
        else:
            ops.block_insert_with_mask(index, value, accept_indicator, self._chunks, self._chunk_rows)

    def gen_val(self, rows):
        return self._generator.generate([rows] + self._row_shape)

    # -- storage management
    def kernel_blocks(self):
        """(chunk list, rows per chunk): what the row kernels take as (blocks, block_size)."""
        return self._chunks, self._chunk_rows

    def _ensure_chunks(self, n_chunks):
        while len(self._chunks) < n_chunks:
            # one tensor for several blocks; fan-dependent initialisers still see one [block_size, D] block
            self._chunks.append(self._generator.generate([self._chunk_rows] + self._row_shape,
                                                         fan_shape=[self._block_size] + self._row_shape))

    def _clear(self):
        self._chunks = []
        self._visible_blocks = 0


class SlotGroup:
    """All slots of one table; they grow together (slot_group.h:60-90)."""

    def __init__(self, block_size, device, chunk_rows):
        self._block_size = block_size
        self._device = device
        self._chunk_rows = chunk_rows
        self._slots = []
        self._name_to_index = {}
        self._emb_slot_index = -1
        self._n_chunks = 0
        self._block_num = 0

    @staticmethod
    def emb_slot_name():
        return "embedding"

    def append_slot(self, name, dtype, partial_shape, generator=None, init_val=0.0):
        if name in self._name_to_index:
            raise RuntimeError("slot %r already exists" % name)
        if generator is None:
            generator = ConstantInitializer(init_val)
            generator.set_shape([self._block_size] + list(partial_shape[1:]))
            generator.set_dtype(dtype)
            generator = generator.build().impl()
        slot = Slot(name, self._block_size, dtype, partial_shape, generator, self._device, self._chunk_rows)
        slot._ensure_chunks(self._n_chunks)  # a late slot catches up with the table
        slot._visible_blocks = self._block_num
        self._slots.append(slot)
        self._name_to_index[name] = len(self._slots) - 1
        return slot

    def append_emb_slot(self, dtype, partial_shape, generator):
        self.append_slot(self.emb_slot_name(), dtype, partial_shape, generator)
        self._emb_slot_index = len(self._slots) - 1

    def append_step_filter_slot(self, name, init_step):
        return self.append_slot(name, torch.int64, [self._block_size, 1], init_val=int(init_step))

    def slot_by_name(self, name):
        return self._slots[self._name_to_index[name]]

    def slot_by_index(self, index):
        return self._slots[index]

    slot_index = slot_by_index  # the reference binds this name to GetSlotByIndex (bind.cc:70)

    def get_slot_index(self, name):
        return self._name_to_index[name]

    def slots(self):
        return list(self._slots)

    def emb_slot(self):
        return self._slots[self._emb_slot_index]

    def block_size(self):
        return self._block_size

    def block_num(self):
        return self._block_num

    def capacity_rows(self):
        return self._n_chunks * self._chunk_rows

    def chunk_rows(self):
        return self._chunk_rows

    def ensure_rows(self, rows):
        need = (rows + self._chunk_rows - 1) // self._chunk_rows
        if need > self._n_chunks:
            self._n_chunks = need
            for s in self._slots:
                s._ensure_chunks(need)

    def set_block_num(self, block_num):
        if block_num > self._block_num:
            self.ensure_rows(block_num * self._block_size)
            self._block_num = block_num
            for s in self._slots:
                s._visible_blocks = block_num

    def clear(self):
        for s in self._slots:
            s._clear()
        self._n_chunks = 0
        self._block_num = 0


class HashtableImpl:
    """Counterpart of ``torch.classes.recis.HashtableImpl`` (bind.cc:92-109)."""

    hashtable_tag = -1

    def __init__(self, block_size, embedding_shape, dtype, device, coalesce, children, generator,
                 slice_begin=0, slice_end=65536, slice_size=65536, reserve_rows=0):
        device = torch.device(device)
        if device.type != "cuda":
            raise RecisHipError("tables live in GPU memory in this build; got device %s" % device)
        if device.index is None:
            device = torch.device("cuda", torch.cuda.current_device())
        self._device = device
        self._dtype = dtype
        self._embedding_shape = list(embedding_shape)
        row_bytes = torch.empty((), dtype=dtype).element_size()
        for d in embedding_shape:
            row_bytes *= d
        if reserve_rows > 0:
            chunk_rows = -(-int(reserve_rows + 1) // block_size) * block_size
        else:
            chunk_rows = max(1, _CHUNK_BYTES // max(1, row_bytes * block_size)) * block_size
        self._slot_group = SlotGroup(block_size, device, chunk_rows)
        self._slot_group.append_emb_slot(dtype, [block_size] + self._embedding_shape, generator)
        self._children_info = ChildrenInfo(coalesce, children)
        self._slice = Slice(slice_begin, slice_end, slice_size)
        self._idmap = ops.IdMap(device, reserve=reserve_rows)
        self._grad_index, self._grad, self._grad_unique, self._grad_keys = [], [], [], {}
        self._planned = []   # gradients handed over as sums still to be taken (accept_planned_grad): two at most

    # ------------------------------------------------------------- storage
    def _make_room(self, incoming):
        """After a find-or-insert of ``incoming`` keys: rows up to the allocator's
        high-water mark (+1 spare) must exist before any row kernel runs. The map keeps an
        upper bound of the mark on the host (what the last finished call published plus every
        id queued since); the exact mark is read back only when that bound passes the
        capacity."""
        sg = self._slot_group
        ub = self._idmap.id_num_bound()
        if ub + 1 > sg.capacity_rows():
            ub = self._idmap.id_num()  # synchronises
            # Leave room for many calls of this size, unless storage grows in chunks far larger
            # than a batch (a pre-sized table): rows are cheap, pipeline bubbles are not.
            roomy = sg.chunk_rows() <= 32 * max(incoming, 1)
            want = ub + 1 + max((16 if roomy else 2) * incoming, sg.block_size())
            if want > sg.capacity_rows() and (roomy or ub + 1 + incoming > sg.capacity_rows()):
                sg.ensure_rows(want)
        if sg.capacity_rows() == 0:
            sg.ensure_rows(1)

    def _sync_block_num(self):
        """block_num = (id_num + block_size) / block_size (hashtable.cc:255-261)."""
        sg = self._slot_group
        id_num = self._idmap.id_num()
        sg.set_block_num((id_num + sg.block_size()) // sg.block_size())

    # ------------------------------------------------------------- lookups
    def embedding_lookup(self, ids, readonly=False):
        ids = ids.to(self._device)
        if ids.dtype != torch.int64:
            ids = ids.long()
        if readonly:
            index = self._idmap.lookup_readonly(ids)
            self._make_room(0)
        else:
            index = self._idmap.lookup(ids)
            self._make_room(ids.numel())
        chunks, chunk_rows = self._slot_group.emb_slot().kernel_blocks()
        emb = ops.block_gather(index, chunks, chunk_rows, -1, bool(readonly))
        return index, emb

    def insert_lookup_index(self, ids):
        ids = ids.to(self._device)
        index = self._idmap.lookup(ids)
        self._make_room(ids.numel())
        return index

    def insert_lookup_index_with_indicator(self, ids, indicator):
        """hashtable.cc:237-248: rows of the ids whose indicator is set (inserted when new), 0
        for the others."""
        ids, indicator = ids.to(self._device), indicator.to(self._device)
        index = torch.zeros_like(ids)
        index.masked_scatter_(indicator, self.insert_lookup_index(torch.masked_select(ids, indicator)))
        return index

    def insert(self, ids, embedding):
        slot = self._slot_group.emb_slot()
        if embedding.dtype != slot.dtype():
            raise RuntimeError("embeding type must be [%s] but get %s" % (slot.dtype(), embedding.dtype))
        if ids.shape[0] != embedding.shape[0]:
            raise RuntimeError("size of ids and embedding dismatch, ids: %d embedding: %d"
                               % (ids.shape[0], embedding.shape[0]))
        index = self.insert_lookup_index(ids)
        slot.index_insert(index, embedding.to(self._device))

    def lookup_index_readonly(self, ids):
        return self._idmap.lookup_readonly(ids.to(self._device))

    def emb_blocks(self):
        """(chunk list, rows per chunk) of the embedding slot, as the row kernels take them
        (no read-back of the allocator state)."""
        return self._slot_group.emb_slot().kernel_blocks()

    def slot_blocks(self, name):
        """The same for the slot ``name``."""
        return self._slot_group.slot_by_name(name).kernel_blocks()

    def lookup_index_counted(self, plan):
        """Queue the find-or-insert of a plan's unique ids before the host knows how many
        there are; finish with ``settle_lookup`` once ``plan.U`` has been read."""
        index_buf = self._idmap.lookup_counted(plan.unique_buf, plan.counts)
        plan.lookup_calls[id(self)] = self._idmap.last_call()
        return index_buf

    def plan_lookup(self, ids, wait=False, need_inverse=True, need_pos=False, tags=None):
        """Dedup of ``ids`` and find-or-insert of the distinct ids in this table in one pass
        (``recis_unique_plan_lookup``): the batch plan with ``index_buf`` = the row of every unique
        id. ``ids`` may be a list of id tensors with their table ``tags`` (see ``ops.ids_unique_plan``). Replaces ``ids_partition`` / ``torch.unique`` + ``IdMap::Lookup`` of the training
        lookup (recis/nn/modules/hashtable.py:262-293). Room is made for the rows every id of the
        batch could need; settle with ``settle_count(plan.U, plan)`` once the count has been read."""
        plan = ops.ids_unique_plan(ids, wait=wait, need_inverse=need_inverse, need_pos=need_pos, idmap=self._idmap,
                                   tags=tags)
        plan.lookup_calls[id(self)] = self._idmap.last_call()
        self._make_room(plan.n if wait is False else plan.U)
        return plan

    def plan_index(self, plan):
        """The rows of ``plan``'s unique ids if the plan was made by ``plan_lookup`` of THIS table
        (the full-length buffer: its first ``plan.U`` entries count), else None."""
        return plan.index_buf if id(self) in plan.lookup_calls and plan.index_buf is not None else None

    def lookup_index_unsettled(self, plan):
        """``lookup_index_counted`` for consumers that take the unique count from device memory: the
        rows every one of the plan's ids could need are made room for, nothing waits for the count.
        Returns the full-length index buffer (its first ``plan.U`` entries are the rows); settle
        with ``settle_count`` whenever the count has been read."""
        index_buf = self._idmap.lookup_counted(plan.unique_buf, plan.counts)
        plan.lookup_calls[id(self)] = self._idmap.last_call()
        self._make_room(plan.n)
        return index_buf

    def settle_count(self, n_true, plan=None):
        """The true size of the counted lookup queued for ``plan`` (default: of the last one)."""
        self._idmap.settle_count(n_true, None if plan is None else plan.lookup_calls.get(id(self)))

    def settle_lookup(self, index_buf, n_true, plan=None):
        self.settle_count(n_true, plan)
        self._make_room(n_true)
        return index_buf[:n_true]

    def lookup_index(self, ids, readonly=False):
        """Row index of ``ids`` (inserting missing keys unless ``readonly``) without
        gathering the rows: for consumers that read the rows out of the table themselves."""
        if readonly:
            return self.lookup_index_readonly(ids)
        return self.insert_lookup_index(ids)

    # -------------------------------------------------------------- grads
    def accept_grad(self, grad_index, grad, unique=False, key=None):
        """``unique=True``: the caller knows ``grad_index`` has no duplicates (it is the
        row index of unique ids), which spares ``grad()`` a dedup pass. ``key``: two calls of one
        step with the same key hand over gradients for the SAME rows in the same order (the rows
        of one batch plan's unique ids, looked up twice); the second is added onto the first
        instead of being merged by row index later."""
        if grad_index.dtype != torch.int64:
            raise RuntimeError("grad_index must be int64")
        self._sum_planned()   # a gradient waiting to be summed comes first, as it was handed over first
        if grad.dtype != self._dtype and not (grad.dtype == torch.float32 and self._dtype in
                                              (torch.bfloat16, torch.float16)):
            raise RuntimeError("grad dtype %s does not match the table (%s)" % (grad.dtype, self._dtype))
        if key is not None:
            at = self._grad_keys.get(key)
            if at is not None and self._grad[at].shape == grad.shape:
                self._grad[at] = self._grad[at] + grad
                return
            self._grad_keys[key] = len(self._grad)
        self._grad_index.append(grad_index)
        self._grad.append(grad)
        self._grad_unique.append(bool(unique))

    def accept_planned_grad(self, index, plan, rows, src, coef=None, cover=None, key=None, may_miss=False):
        """A gradient handed over before it is summed: the gradient of ``plan``'s unique id ``u`` (table row
        ``index[u]``; negative = the table does not hold the key, no gradient) is the sum over u's occurrence
        list of ``coef * rows[src]`` (``ops.csr_gather_reduce``; ``rows`` may be a list of arrays laid end to
        end, ``ops.csr_gather_reduce_parts``). If it stays the only gradient of the step, or one of the two
        gradients of one plan (a lookup whose rows fed a pooled and a padded output; same ``key``), an optimizer
        that can (``apply_planned`` / ``apply_planned2``) takes the sum and applies the row update in one launch
        and the ``[U, D]`` gradient is never written; anything else that asks for the gradient (``grad``,
        ``grad_pairs``, a further gradient, accumulation over several steps) gets it summed first, as
        ``accept_grad`` would have. ``may_miss``: ``index`` may hold negative entries (a read-only lookup)."""
        entry = (index, plan, rows, src, coef, cover, key, may_miss)
        if not self._grad and len(self._planned) == 1 and self._one_launch_sums(self._planned[0], entry):
            self._planned.append(entry)
            return
        if self._grad or self._planned:
            self._sum_planned()
            self._accept_summed(index, self._sum_of(entry), key, may_miss)
            return
        self._planned = [entry]

    def _one_launch_sums(self, a, b):
        """Whether two unsummed gradients are the two inputs of one ``ops.csr_gather_reduce2*`` launch: of one
        plan and the same rows (one key), whole (no cover), each float32 or of the table's type, at most one
        of them in parts."""
        if a[1] is not b[1] or a[6] is None or a[6] != b[6] or a[7] != b[7] or a[5] is not None or b[5] is not None:
            return False
        if a[0].shape != b[0].shape:
            return False
        in_parts = [not torch.is_tensor(e[2]) for e in (a, b)]
        if all(in_parts) or any(p and (e[4] is not None or not 1 <= len(e[2]) <= 8) for p, e in zip(in_parts, (a, b))):
            return False
        dtype_of = lambda e: e[2].dtype if torch.is_tensor(e[2]) else e[2][0].dtype
        return all(dtype_of(e) in (torch.float32, self._dtype) for e in (a, b))

    @staticmethod
    def _sum_of(entry):
        index, plan, rows, src, coef, cover, key, may_miss = entry
        if torch.is_tensor(rows):
            return ops.csr_gather_reduce(rows, plan, src, coef, cover=cover)
        return ops.csr_gather_reduce_parts(rows, plan, src)

    def _accept_summed(self, index, g, key, may_miss):
        if may_miss:  # keys the table does not hold take no gradient
            keep = index >= 0
            index, g = index[keep], g[keep]
        self.accept_grad(index, g, unique=True, key=key)

    def _sum_planned(self):
        planned, self._planned = self._planned, []
        for entry in planned:
            self._accept_summed(entry[0], self._sum_of(entry), entry[6], entry[7])

    def take_planned_grad(self):
        """The planned gradients if they are all this table received since the last ``clear_grad`` (and
        forgets them), else None: a list of one or two ``(index, plan, rows, src, coef, cover)``; of two, the
        first is one array (the other may be a list of arrays)."""
        if not self._planned or self._grad:
            return None
        if len(self._planned) == 1 and not torch.is_tensor(self._planned[0][2]):
            return None   # parts alone: no fused row update takes them
        planned, self._planned = self._planned, []
        if len(planned) == 2 and not torch.is_tensor(planned[0][2]):
            planned.reverse()
        return [e[:6] for e in planned]

    def has_grad(self):
        return len(self._grad) > 0 or len(self._planned) > 0

    def grad_pairs(self, accumulate_steps=1):
        """(row index, gradient rows) merged over the accepted gradients: what
        ``grad()`` wraps as a sparse tensor (hashtable.cc:90-134), without the host
        round trips. With duplicates the gradients are summed per row."""
        self._sum_planned()
        index = self._grad_index[0] if len(self._grad_index) == 1 else torch.cat(self._grad_index, 0)
        g = self._grad[0] if len(self._grad) == 1 else torch.cat(self._grad, 0)
        if not (len(self._grad_unique) == 1 and self._grad_unique[0]):
            uniq, inverse = torch.unique(index, sorted=False, return_inverse=True)
            if uniq.numel() != index.numel():
                summed = torch.zeros((uniq.numel(),) + tuple(g.shape[1:]), dtype=g.dtype, device=g.device)
                summed.index_add_(0, inverse, g)
                index, g = uniq, summed
        if accumulate_steps != 1:
            g = g / accumulate_steps
        return index, g

    def grad(self, accumulate_steps=1):
        """Sparse COO gradient exactly as the reference builds it (hashtable.cc:90-134),
        including its layout when rows repeat: positions 0..U-1 as indices and an
        N-row value buffer whose first U rows hold the sums."""
        self._sum_planned()
        index = torch.cat(self._grad_index, 0)
        g = torch.cat(self._grad, 0)
        uniq, inverse = torch.unique(index, sorted=False, return_inverse=True)
        emb_shape = list(g.shape[1:])
        if index.numel() == uniq.numel():
            final_indices = index.view(1, -1)
            final_grad = g
            rows = int(index.max().item()) + 1 if index.numel() else 0
        else:
            final_indices = inverse.view(1, -1)
            final_grad = torch.zeros([inverse.numel()] + emb_shape, dtype=g.dtype, device=g.device)
            final_grad.index_add_(0, inverse.view(-1), g)
            rows = int(uniq.max().item()) + 1 if uniq.numel() else 0
        final_grad = final_grad / accumulate_steps
        return torch.sparse_coo_tensor(final_indices, final_grad, [rows] + emb_shape,
                                       check_invariants=False).detach_()

    def clear_grad(self):
        self._grad_index, self._grad, self._grad_unique, self._grad_keys = [], [], [], {}
        self._planned = []

    # ------------------------------------------------------------ bookkeeping
    def clear(self):
        self.clear_grad()
        self._idmap.clear()
        self._slot_group.clear()

    def clear_id(self):
        self._idmap.clear()

    def ids(self):
        return self._idmap.snapshot()[0]

    def ids_map(self):
        return self._idmap.snapshot()

    def ids_num(self):
        return self._idmap.id_num()

    def slot_group(self):
        self._sync_block_num()
        return self._slot_group

    def children_info(self):
        return self._children_info

    def slice_info(self):
        return self._slice

    def append_filter_slot(self, name, dtype, slot_dim, generator):
        self._slot_group.append_slot(name, dtype, [0, slot_dim], generator)

    def append_step_filter_slot(self, name, init_step):
        if torch.is_tensor(init_step):
            init_step = int(init_step.item())
        self._slot_group.append_step_filter_slot(name, init_step)

    def update_slot(self, slot_name, index, value):
        slot = self._slot_group.slot_by_name(slot_name)
        if value.dtype != slot.dtype():
            raise RuntimeError("embedding type must be [%s] but get %s" % (slot.dtype(), value.dtype))
        slot.index_insert(index.to(self._device), value)

    def get_slot(self, name):
        self._sync_block_num()
        return self._slot_group.slot_by_name(name)

    def delete(self, ids, index, preserve_slot=""):
        """Erase keys, free their rows, re-initialise every slot but ``preserve_slot``
        at those rows (hashtable.cc:263-278)."""
        if ids.numel() == 0:
            return
        ids, index = ids.to(self._device), index.to(self._device)
        self._idmap.erase(ids, index)
        sg = self._slot_group
        for i, slot in enumerate(sg.slots()):
            if preserve_slot and sg.get_slot_index(preserve_slot) == i:
                continue
            slot.index_insert(index, slot.gen_val(ids.numel()))

    def evict_older(self, stamp_slot, threshold):
        """Eviction sweep of a step filter in one pass over the map: erase every key whose
        row has ``stamp_slot < threshold``, free the rows and re-initialise every other slot
        there. Same outcome as ``ids_map`` + ``block_filter`` + ``delete``
        (hashtable_hook_impl.py:487-551, hashtable.cc:263-278) without materialising all
        (key, row) pairs. Returns the evicted ``(ids, index)``."""
        chunks, chunk_rows = self.get_slot(stamp_slot).kernel_blocks()
        ids, index = self._idmap.evict_older(chunks, chunk_rows, threshold)
        if ids.numel():
            sg = self._slot_group
            keep = sg.get_slot_index(stamp_slot)
            for i, slot in enumerate(sg.slots()):
                if i != keep:
                    slot.index_insert(index, slot.gen_val(ids.numel()))
        return ids, index

    def id_map(self):
        return self._idmap

    @property
    def device(self):
        return self._device

    @property
    def dtype(self):
        return self._dtype


def make_hashtable(block_size, embedding_shape, dtype, device, coalesce, children, generator,
                   slice_begin=0, slice_end=65536, slice_size=65536, reserve_rows=0):
    """``torch.ops.recis.make_hashtable`` (hashtable.h:36-41, bind.cc:145)."""
    return HashtableImpl(block_size, embedding_shape, dtype, device, coalesce, children, generator,
                         slice_begin, slice_end, slice_size, reserve_rows)


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
        ctx.hashtable.accept_grad(index, grad_output_emb.contiguous(), unique=True, key=ctx.grad_key)
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
    """Lookup of a plan's unique ids and one output row per request in one pass over the table
    (what HashTableLookupHelpFunction + GradWorkerMeanFunction give, hashtable.py:425-586, without
    the ``[U, D]`` copy of the rows): every unique row is read once and written to its
    occurrences. Backward: sum over the duplicates of each id, divided by the number of workers."""

    @staticmethod
    def forward(ctx, backward_holder, impl, plan, slice_num, readonly, stamp=None):
        """``stamp`` = (name of the step filter's slot, its one-element step tensor): the rows read
        are stamped in the same pass (what the filter hook's update would do in a launch of its own)."""
        if readonly:
            index = impl.lookup_index(plan.unique, True)
        else:
            index_buf = impl.lookup_index_counted(plan)   # queued before the host has the unique count
            index = impl.settle_lookup(index_buf, plan.U, plan)
        chunks, chunk_rows = impl.emb_blocks()
        if stamp is not None:   # the slot's blocks as they are now, after the lookup may have grown the table
            stamp = (impl.slot_blocks(stamp[0])[0], stamp[1])
        out = ops.plan_expand_rows(plan, plan.n, blocks=chunks, block_size=chunk_rows, row_index=index, stamp=stamp)
        ctx.impl, ctx.plan, ctx.slice_num, ctx.readonly = impl, plan, slice_num, readonly
        ctx.save_for_backward(index)
        ctx.mark_non_differentiable(index)
        return index, out

    @staticmethod
    def backward(ctx, _grad_index, grad):
        (index,) = ctx.saved_tensors
        n = ctx.plan.n
        flat = grad.reshape(n, -1).contiguous()
        if ctx.slice_num != 1:
            flat = flat / ctx.slice_num
        # the sum over the duplicates of each id is left to the optimizer step where it can be (one launch
        # sums and updates the row); keys the table does not hold (negative index) take no gradient
        ctx.impl.accept_planned_grad(index, ctx.plan, flat, ctx.plan.occ, may_miss=ctx.readonly)
        return None, None, None, None, None, None


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
                self._hashtable_impl._embedding_shape) == 1 and self._dtype in (torch.float32, torch.bfloat16, torch.float16):
            from .hashtable_hook_impl import ReadOnlyHookImpl

            assert admit_hook_impl is None or isinstance(admit_hook_impl, ReadOnlyHookImpl), \
                "admit hook only support ReadOnlyHook yet, but got: %s" % admit_hook_impl
            plan = ops.ids_unique_plan(ids, wait=False, need_pos=False)
            # a step filter's stamps ride on the pass that reads the rows
            stamp = getattr(self._filter_hook_impl, "stamp_target", lambda: None)()
            emb_idx, embedding = LookupExpandFunction.apply(self._backward_holder, self._hashtable_impl, plan,
                                                            self._worker_num, admit_hook_impl is not None, stamp)
            if stamp is None:
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

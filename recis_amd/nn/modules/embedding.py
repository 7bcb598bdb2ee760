"""``EmbeddingOption`` and ``DynamicEmbedding``: the mirror of
``recis.nn.modules.embedding`` (embedding.py:161-624) for one GPU that owns the whole
table (world size 1: the id / row / gradient all-to-alls of the reference are the
identity and are left out)."""
import json
import math
import os
from dataclasses import dataclass, field
from typing import List, Optional, Union

import torch

from ... import ops
from ...ragged.tensor import RaggedTensor
from ..functional.embedding_ops import ragged_embedding_segment_reduce
from ..hashtable_hook import AdmitHook, FilterHook
from ..initializers import ConstantInitializer, Initializer
from .hashtable import (GradIDMeanFunction, HashTable, HashTableLookupHelpFunction, accept_planned_grad, gen_slice,
                        plan_lookup)


class _Done:
    """Stands where the reference keeps the handle of an asynchronous all-to-all: with one GPU
    there is nothing to wait for."""

    def wait(self):
        return None


@dataclass
class ExchangeIDsResults:
    """embedding.py:121-140, for one GPU: ``ids`` are the distinct ids of the batch (what the
    reference receives from its peers), ``parts`` / ``parts_reverse`` their count, ``plan`` the
    batch plan the later stages reuse."""

    ids: torch.Tensor
    ids_await: object
    parts: List[int]
    parts_reverse: List[int]
    reverse_index: torch.Tensor
    offsets: torch.Tensor
    plan: object = None


@dataclass
class ExchangeEmbResults:
    """embedding.py:142-158."""

    emb: torch.Tensor
    reverse_index: torch.Tensor
    emb_shape: List[int]
    offsets: torch.Tensor
    emb_await: Optional[object] = None
    plan: object = None


@dataclass
class EmbeddingOption:
    embedding_dim: int = 16
    block_size: int = 10240
    dtype: torch.dtype = torch.float32
    device: torch.device = torch.device("cuda")
    trainable: bool = True
    pg: object = None
    max_partition_num: int = 65536
    shared_name: str = "embedding"
    children: List[str] = field(default_factory=list)
    coalesced: Optional[bool] = False
    initializer: Optional[Initializer] = None
    use_weight: Optional[bool] = True
    combiner: Optional[str] = "sum"
    combiner_kwargs: Optional[dict] = None
    grad_reduce_by: Optional[str] = "worker"
    filter_hook: Optional[FilterHook] = None
    admit_hook: Optional[AdmitHook] = None
    fp16_enabled: bool = False
    reserve_rows: int = 0  # addition: pre-size the map and the row storage

    def __post_init__(self):
        if not self.children:
            self.children = [self.shared_name]
        if self.initializer is None:
            self.initializer = ConstantInitializer(init_val=0)
        if self.fp16_enabled:
            assert self.dtype in (torch.int8,), "only int8 emb can set fp16_enabled"
        assert self.combiner in ["sum", "mean", "tile", "max"], \
            "Hashtable combiner only support [sum/mean/tile/max], but got %s" % self.combiner
        if self.combiner == "tile":
            if self.combiner_kwargs is None:
                raise RuntimeError("combiner_kwargs must be set when combiner is tile.")
            if "tile_len" not in self.combiner_kwargs:
                raise RuntimeError("tile_len must be in combiner_kwargs when combiner is tile.")

    def coalesced_info(self):
        return json.dumps({
            "dim": self.embedding_dim, "dtype": str(self.dtype), "device": str(torch.device(self.device).type),
            "initializer": str(self.initializer), "grad_reduce_by": self.grad_reduce_by,
            "filter_hook": str(self.filter_hook),
        })

    def runtime_info(self):
        return json.dumps({
            "combiner": self.combiner, "use_weight": self.use_weight, "trainable": self.trainable,
            "admit_hook": str(self.admit_hook), "fp16_enabled": self.fp16_enabled,
        })


def lookup_unique_rows(hashtable: HashTable, unique_ids, admit_hook=None, trainable=True, grad_key=None):
    """Rows of ids that are already unique: the lookup autograd function, the
    last-seen-step stamp, no second dedup. ``grad_key``: see ``HashtableImpl.accept_grad``."""
    from .hashtable_hook_impl import HashtableHookFactory

    impl = hashtable._hashtable_impl
    float_table = hashtable._dtype not in (torch.int8, torch.int32, torch.int64)
    if hashtable.training and trainable and float_table:
        admit_impl = HashtableHookFactory().create_admit_hook(hashtable, admit_hook) if admit_hook else None
        emb_idx, emb = HashTableLookupHelpFunction.apply(unique_ids, impl, hashtable._backward_holder, admit_impl,
                                                         grad_key)
        hashtable._filter_hook_impl(emb_idx)
        return emb
    readonly = (not hashtable.training) or admit_hook is not None or not float_table
    _, emb = impl.embedding_lookup(unique_ids.detach(), readonly)
    if hashtable.training and not readonly:
        hashtable._filter_hook_impl(_)
    return emb


class LookupPoolFunction(torch.autograd.Function):
    """Lookup of a plan's unique ids and sum / mean pooling straight out of the table: the
    ``[U, D]`` copy of the looked-up rows (lookup function + ``ragged_embedding_segment_reduce``,
    recis/nn/modules/embedding.py:592-624) is never made. Backward reduces the pooled
    gradients per unique row over the plan and hands (row index, gradient) to the table."""

    @staticmethod
    def forward(ctx, backward_holder, impl, plan, weight, offsets, combiner, readonly, unit_segments=False,
                split=None):
        """``split``: row counts to cut the pooled output into (one part per feature of a group that is pooled
        in one go); the parts are returned as separate outputs, views of the one buffer, and backward takes
        their gradients as they come: slices of one buffer are used in place, anything else is concatenated."""
        late_count = not readonly
        if readonly:
            index = impl.lookup_index(plan.unique, True)
        else:
            # Nothing in this forward waits for the unique count: the lookup and the expansion take
            # it from device memory, the pooling kernel only follows the plan's inverse (which names
            # rows below the count), and the host reads it in backward, long after it has arrived.
            # `index` is the full-length buffer; its first plan.U entries are the rows. A plan made by
            # make_plan for this table brings them along (dedup and lookup were one pass).
            index = impl.plan_index(plan)
            if index is None:
                index = impl.lookup_index_counted(plan, True)
        if unit_segments:
            # one id per segment (sum == mean == the row itself): every unique row is read once and
            # written to its occurrences, instead of one index chase per output row
            out = impl.expand_rows(plan, index, weight, None, None)
        else:
            chunks, chunk_rows = impl.emb_blocks()
            out = ops.segment_reduce_forward_blocks(chunks, chunk_rows, index, weight, plan.inverse, offsets,
                                                    combiner)
        ctx.impl, ctx.plan, ctx.combiner, ctx.readonly, ctx.late_count = impl, plan, combiner, readonly, late_count
        ctx.split, ctx.out_shape = split, tuple(out.shape)
        ctx.save_for_backward(index, weight, offsets)
        ctx.mark_non_differentiable(index)
        if split is None:
            return index, out
        return (index,) + tuple(torch.split(out, split))

    @staticmethod
    def backward(ctx, _grad_index, *grads):
        index, weight, offsets = ctx.saved_tensors
        if ctx.late_count:
            ctx.impl.settle_count(ctx.plan.U, ctx.plan)
            index = index[: ctx.plan.U]
        grad = grads[0] if ctx.split is None else _joined(grads, ctx.split, ctx.out_shape)
        # sum / mean: the gradient of a unique row is a gather-reduce over its occurrence list; it is handed
        # over unsummed, so that the optimizer step can sum and update the row in one launch (keys the table
        # does not hold carry a negative index and take no gradient)
        src, coef = ctx.plan.src_coef_for_pool(offsets.contiguous(), weight, ctx.combiner == "mean")
        accept_planned_grad(ctx.impl, index, ctx.plan, grad.contiguous(), src, coef,
                            key=None if ctx.readonly else ctx.plan.serial, may_miss=ctx.readonly)
        return (None,) * 9


def _joined(grads, split, shape):
    """The gradients of the parts of one pooled output as one ``shape`` tensor: in place when they are
    consecutive slices of one buffer (what a caller that keeps its gradients in one array hands over),
    concatenated otherwise (a missing gradient counts as zeros)."""
    like = next((g for g in grads if g is not None), None)
    if like is None:
        return torch.zeros(shape, device="cuda")
    first = grads[0]
    if first is not None and first.is_contiguous():
        at = first.data_ptr()
        for g, rows in zip(grads, split):
            if g is None or g.dtype != first.dtype or not g.is_contiguous() or g.data_ptr() != at \
                    or g.untyped_storage().data_ptr() != first.untyped_storage().data_ptr():
                break
            at += rows * shape[1] * g.element_size()
        else:
            whole = torch.as_strided(first, shape, (shape[1], 1), first.storage_offset())
            return whole
    return torch.cat([g if g is not None else like.new_zeros((rows, shape[1])) for g, rows in zip(grads, split)])


class DenseLookupFunction(torch.autograd.Function):
    """Dedup, lookup and pooling of a group of dense id columns (``[B]`` / ``[B, 1]`` int64: one id per
    sample, so sum == mean == the row itself) as ONE native call each way
    (``HashtableImpl.dense_lookup_expand`` forward, ``accept_split_grad`` backward): what the per-feature
    loop of ``EmbeddingEngine.forward`` + ``LookupPoolFunction`` do for such a group, without the Python
    work per feature. One output per column, views of the one ``[N, D]`` buffer; nothing waits for the
    unique count. ``forward`` returns None instead when a column is something else."""

    @staticmethod
    def forward(ctx, backward_holder, impl, cols, tags, stamp):
        res = impl.dense_lookup_expand(cols, tags, None if stamp is None else stamp[0],
                                       None if stamp is None else stamp[1])
        if res is None:
            ctx.mark_non_differentiable()
            return None
        plan, index, out = res
        split = [c.shape[0] for c in cols]
        ctx.impl, ctx.plan, ctx.split = impl, plan, split
        ctx.save_for_backward(index)
        ctx.mark_non_differentiable(index)
        return (index,) + tuple(torch.split(out, split))

    @staticmethod
    def backward(ctx, _grad_index, *grads):
        (index,) = ctx.saved_tensors
        # the gradients of the columns, as they come (slices of one buffer are used in place); the sum per
        # unique row is left to the optimizer step, which then updates the row in the same launch
        ctx.impl.accept_split_grad(index, ctx.plan, list(grads), ctx.split, None, None, ctx.plan.serial, False, True)
        return None, None, None, None, None


class LookupTileFunction(torch.autograd.Function):
    """Lookup of a plan's unique ids and the padded gather of several features at once, ONE output
    per feature (``[bs[f], tile_len[f] * D]``, views of one buffer: the list form of the tile
    combiner, recis/nn/modules/embedding_engine.py:383-411). Backward hands the features' gradients
    to the table unsummed, as separate arrays: no concatenation of the padded gradients, and the
    optimizer step sums them (together with the gradient of a pooled output of the same lookup, if
    there is one) where it updates the rows."""

    @staticmethod
    def forward(ctx, backward_holder, impl, plan, offsets, bs, tile_len, readonly):
        bs, tile_len = [int(b) for b in bs], [int(t) for t in tile_len]
        U = plan.U   # the padded gather reads a dense copy of the rows: this forward needs the count
        if readonly:
            index = impl.lookup_index(plan.unique, True)
        else:
            index = impl.plan_index(plan)   # a plan made for this table brings the rows along
            if index is None:
                index = impl.lookup_index_counted(plan, True)
            index = impl.settle_lookup(index, U, plan)
        chunks, chunk_rows = impl.emb_blocks()
        rows = ops.block_gather(index, chunks, chunk_rows, -1, readonly)
        out, _ = ops.ragged_tile(bs, tile_len, plan.inverse, offsets, rows)
        D = rows.shape[1]
        ctx.impl, ctx.plan, ctx.readonly, ctx.bs, ctx.tile_len, ctx.D = impl, plan, readonly, bs, tile_len, D
        ctx.save_for_backward(index, offsets)
        ctx.mark_non_differentiable(index)
        n_rows = [b * t for b, t in zip(bs, tile_len)]
        return (index,) + tuple(p.view(b, t * D) for p, b, t in zip(torch.split(out, n_rows), bs, tile_len))

    @staticmethod
    def backward(ctx, _grad_index, *grads):
        index, offsets = ctx.saved_tensors
        plan, D = ctx.plan, ctx.D
        n_rows = [b * t for b, t in zip(ctx.bs, ctx.tile_len)]
        like = next((g for g in grads if g is not None), None)
        if like is not None:
            src = plan.src_for_tile(ctx.bs, ctx.tile_len, offsets.contiguous())
            parts = [(g if g is not None else like.new_zeros((n, D))).reshape(n, D) for g, n in zip(grads, n_rows)]
            key = None if ctx.readonly else plan.serial
            if len(parts) <= 8 and len({p.dtype for p in parts}) == 1:
                accept_planned_grad(ctx.impl, index, plan, parts, src, key=key, may_miss=ctx.readonly)
            else:
                accept_planned_grad(ctx.impl, index, plan, torch.cat(parts), src, key=key, may_miss=ctx.readonly)
        return (None,) * 7


def _pools_out_of_the_table(hashtable, opt, n_occ, n_offsets):
    """Whether lookup_and_pool takes the path that pools straight out of the table rows."""
    float_table = hashtable._dtype in (torch.float32, torch.bfloat16, torch.float16)
    sparse_mean = opt.combiner == "mean" and not n_occ / n_offsets > 5
    id_mean = opt.grad_reduce_by == "id" and hashtable.training and opt.trainable
    return opt.combiner in ("sum", "mean") and float_table and not sparse_mean and not id_mean


def make_plan(hashtable: HashTable, ids, offsets, opt, has_weight=False, unit_segments=False, tags=None):
    """The batch plan of ``ids`` for ``lookup_and_pool``. When what follows is the training lookup
    that admits new keys and pools out of the table, dedup and find-or-insert run as one pass
    (``HashtableImpl.plan_lookup``) and the plan carries the rows; ``unit_segments`` plans leave
    out the per-occurrence arrays nobody reads (the expansion and its backward walk the lists).
    ``ids`` may be a list of id tensors with their table ``tags`` (``ops.ids_unique_plan``)."""
    n_occ = sum(t.numel() for t in ids) if isinstance(ids, (list, tuple)) else ids.numel()
    if (hashtable.training and opt.trainable and opt.admit_hook is None
            and _pools_out_of_the_table(hashtable, opt, n_occ, offsets.numel())):
        lean = bool(unit_segments)
        return plan_lookup(hashtable._hashtable_impl, ids, need_inverse=not lean, tags=tags)
    return ops.ids_unique_plan(ids, wait=False, need_pos=False, tags=tags)


def lookup_and_pool(hashtable: HashTable, plan, weight, offsets, opt, unit_segments=False, combiner_kwargs=None,
                    split=None):
    """Rows of the plan's unique ids pooled per segment. Sum / mean over a float table go
    through ``LookupPoolFunction`` (pooling reads the table directly); everything else looks the
    rows up first and pools the copy. ``unit_segments``: the caller built ``offsets`` as
    0, 1, 2, ... (dense ``[B, 1]`` id tensors), so segment i holds exactly occurrence i.
    ``split``: return the pooled rows cut into parts of these row counts (a tuple)."""
    impl = hashtable._hashtable_impl
    id_mean = opt.grad_reduce_by == "id" and hashtable.training and opt.trainable
    if _pools_out_of_the_table(hashtable, opt, plan.n, offsets.numel()):
        if weight is not None and weight.dtype != hashtable._dtype:
            weight = weight.to(hashtable._dtype)
        if hashtable.training and opt.trainable:
            readonly = opt.admit_hook is not None
            if readonly:
                from .hashtable_hook_impl import HashtableHookFactory, ReadOnlyHookImpl
                admit = HashtableHookFactory().create_admit_hook(hashtable, opt.admit_hook)
                assert isinstance(admit, ReadOnlyHookImpl), "admit hook only support ReadOnlyHook yet, but got: %s" % admit
            index, *outs = LookupPoolFunction.apply(hashtable._backward_holder, impl, plan, weight, offsets,
                                                    opt.combiner, readonly, unit_segments, split)
            if not isinstance(hashtable._filter_hook_impl, torch.nn.Identity):
                # a step filter stamps the looked-up rows: it needs the rows proper (the index may
                # be the full-length buffer of the forward that does not wait for the count)
                hashtable._filter_hook_impl(index[: plan.U] if not readonly else index)
            return outs[0] if split is None else tuple(outs)
        readonly = (not hashtable.training) or opt.admit_hook is not None
        index = impl.lookup_index(plan.unique.detach(), readonly)
        if hashtable.training and not readonly:
            hashtable._filter_hook_impl(index)
        chunks, chunk_rows = impl.emb_blocks()
        out = ops.segment_reduce_forward_blocks(chunks, chunk_rows, index, weight, plan.inverse, offsets,
                                                opt.combiner)
        return out if split is None else torch.split(out, split)
    emb = lookup_unique_rows(hashtable, plan.unique, opt.admit_hook, opt.trainable)
    inverse = plan.inverse
    if id_mean:
        # mean over the duplicates of each id: pool the expanded rows instead
        emb = GradIDMeanFunction.apply(emb, inverse, plan)
        inverse, plan = None, None
    if weight is not None and weight.dtype != emb.dtype:
        weight = weight.to(emb.dtype)
    out = ragged_embedding_segment_reduce(emb, weight, inverse, offsets, opt.combiner,
                                          combiner_kwargs if combiner_kwargs is not None else opt.combiner_kwargs,
                                          plan=plan)
    return out if split is None else torch.split(out, split)


class DynamicEmbedding(torch.nn.Module):
    def __init__(self, emb_opt: EmbeddingOption, pg=None):
        super().__init__()
        self._emb_opt = emb_opt
        self._world_size = int(os.environ.get("WORLD_SIZE", 1))
        self._rank = int(os.environ.get("RANK", 0))
        if self._world_size != 1:
            raise NotImplementedError("this build runs one GPU that owns the whole table (WORLD_SIZE=1)")
        self._hashtable = HashTable(
            embedding_shape=[emb_opt.embedding_dim], block_size=emb_opt.block_size, dtype=emb_opt.dtype,
            device=emb_opt.device, initializer=emb_opt.initializer, children=emb_opt.children,
            name=emb_opt.shared_name, coalesced=emb_opt.coalesced,
            slice=gen_slice(shard_index=self._rank, shard_num=self._world_size),
            grad_reduce_by=emb_opt.grad_reduce_by, filter_hook=emb_opt.filter_hook,
            reserve_rows=emb_opt.reserve_rows)

    def deal_with_tensor(self, input_tensor: Union[torch.Tensor, RaggedTensor]):
        self._unit_segments = False
        if isinstance(input_tensor, RaggedTensor):
            val = input_tensor.values()
            weight = input_tensor.weight()
            offsets = input_tensor.offsets()[-1]
            shape = input_tensor.real_shape(0, -1)
            if not math.prod(shape) == (offsets.numel() - 1):
                raise RuntimeError("RaggedTensor must pad before lookup, got: %s" % input_tensor)
        elif isinstance(input_tensor, torch.Tensor):
            if input_tensor.is_sparse:
                raise TypeError("RaggedDynamicEmbedding doesn't support sparse ids")
            val = input_tensor.reshape(-1)
            bs, fea_dim = input_tensor.shape[0], input_tensor.shape[1]
            offsets = torch.arange(bs + 1, device=val.device) * fea_dim
            weight = None
            shape = tuple(input_tensor.shape[:-1])
            self._unit_segments = fea_dim == 1
        else:
            raise TypeError("DynamicEmbedding only support RaggedTensor or dense tensor, got %s" % type(input_tensor))
        return val, offsets, weight, shape

    def forward(self, input_ids, input_weights=None):
        opt = self._emb_opt
        val, offsets, weight, shape = self.deal_with_tensor(input_ids)
        dev = self._hashtable._impl_device
        val, offsets = val.to(dev), offsets.to(dev)
        if input_weights is not None:
            weight = input_weights
        if weight is not None:
            weight = weight.to(dev) if opt.use_weight else None
        plan = make_plan(self._hashtable, val, offsets, opt, weight is not None, self._unit_segments)
        out = lookup_and_pool(self._hashtable, plan, weight, offsets, opt, unit_segments=self._unit_segments)
        if opt.combiner == "tile":
            return out.view(tuple(shape) + (opt.combiner_kwargs["tile_len"] * opt.embedding_dim,))
        return out.view(tuple(shape) + (opt.embedding_dim,))

    # The staged form of forward (embedding.py:498-624), which EmbeddingEngine-style callers drive
    # stage by stage. With one GPU the two all-to-alls are the identity: exchange_ids is the dedup,
    # lookup_exchange_emb the table lookup of the distinct ids, emb_reduce the pooling. forward()
    # above fuses the last two (pooling reads the table rows directly).
    def exchange_ids(self, ids: torch.Tensor, offsets: torch.Tensor):
        plan = ops.ids_unique_plan(ids, wait=True, need_pos=False)
        n = int(plan.U)
        return ExchangeIDsResults(ids=plan.unique, ids_await=_Done(), parts=[n], parts_reverse=[n],
                                  reverse_index=plan.inverse, offsets=offsets, plan=plan)

    def lookup_exchange_emb(self, ids_exchange_result: ExchangeIDsResults, admit_hook=None):
        ids_exchange_result.ids_await.wait()
        emb = lookup_unique_rows(self._hashtable, ids_exchange_result.ids, admit_hook, self._emb_opt.trainable)
        return ExchangeEmbResults(emb=emb, emb_await=_Done(), reverse_index=ids_exchange_result.reverse_index,
                                  emb_shape=list(emb.shape), offsets=ids_exchange_result.offsets,
                                  plan=ids_exchange_result.plan)

    def wait_exchange_emb(self, emb_exchange_result: ExchangeEmbResults):
        emb_exchange_result.emb_await.wait()
        return emb_exchange_result.emb.view(emb_exchange_result.emb_shape)

    def emb_reduce(self, emb_exchange_result: ExchangeEmbResults, weight, combiner, combiner_kwargs,
                   fp16_enable=False):
        emb = self.wait_exchange_emb(emb_exchange_result)
        if emb.dtype in (torch.int8,):
            emb = emb.to(torch.float16 if fp16_enable else torch.float32)
        if weight is not None and weight.dtype != emb.dtype:
            weight = weight.to(emb.dtype)
        return ragged_embedding_segment_reduce(emb, weight, emb_exchange_result.reverse_index,
                                               emb_exchange_result.offsets, combiner, combiner_kwargs,
                                               plan=emb_exchange_result.plan)

    @property
    def hashtable(self):
        return self._hashtable

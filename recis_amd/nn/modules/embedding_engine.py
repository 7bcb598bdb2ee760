"""``EmbeddingEngine``: looks up many features in one go (mirror of
``recis.nn.modules.embedding_engine``, embedding_engine.py:17-832).

Features whose options agree on dim / dtype / device / initializer / gradient
reduction / filter hook are coalesced into ONE physical table, each feature's ids
tagged with a 12-bit table index (embedding_engine.py:607-625, ids_encode). Within a
table, features that also agree on combiner / use_weight / trainable / admit hook
form one runtime group and are processed together:

    ids_encode + merge_offsets  ->  dedup (hash)  ->  find-or-insert + row gather
    ->  segment reduce over all the group's segments  ->  split per feature

which is the reference's group_exchange_ids / group_exchange_embs / group_reduce
pipeline with the all-to-alls removed (one GPU owns the whole table).
"""
import hashlib
from collections import OrderedDict
from typing import Dict, Union

import torch

from ... import ops
from ...ragged.tensor import RaggedTensor
from ..functional.embedding_ops import RaggedTileParts
from .embedding import (DenseLookupFunction, EmbeddingOption, LookupTileFunction, lookup_and_pool, lookup_unique_rows,
                        make_plan)
from .hashtable import HashTable, gen_slice, plan_lookup


def _key(text):
    return hashlib.sha256(text.encode()).hexdigest()[:16]


class _TableGroup:
    def __init__(self, key, first_opt):
        self.key = key
        self.opt = first_opt
        self.children = []          # shared names in order of first appearance
        self.features = OrderedDict()  # feature name -> option


class EmbeddingEngine(torch.nn.Module):
    def __init__(self, emb_options: Dict[str, EmbeddingOption]):
        super().__init__()
        self._emb_options = OrderedDict(emb_options)
        self._groups = OrderedDict()
        for name, opt in self._emb_options.items():
            gkey = _key(opt.coalesced_info())
            grp = self._groups.get(gkey)
            if grp is None:
                grp = self._groups[gkey] = _TableGroup(gkey, opt)
            if opt.shared_name not in grp.children:
                grp.children.append(opt.shared_name)
            grp.features[name] = opt
        # per feature: the key of its runtime group (features of a table that are pooled together)
        self._runtime_key = {name: opt.runtime_info() for name, opt in self._emb_options.items()}
        self._offsets_cache = {}  # offsets of dense id tensors, which depend on their shape only
        self._tags = {}
        self._tables = torch.nn.ModuleDict()
        for gkey, grp in self._groups.items():
            opt = grp.opt
            coalesced = len(grp.children) > 1
            table_name = grp.children[0] if not coalesced else "CoalescedHashtable_" + gkey
            reserve = sum(o.reserve_rows for o in grp.features.values())
            self._tables[gkey] = HashTable(
                embedding_shape=[opt.embedding_dim], block_size=opt.block_size, dtype=opt.dtype,
                device=opt.device, coalesced=coalesced, children=list(grp.children), slice=gen_slice(0, 1),
                initializer=opt.initializer, name=table_name, grad_reduce_by=opt.grad_reduce_by,
                filter_hook=opt.filter_hook, reserve_rows=reserve)

    def hashtables(self):
        return {t._name: t for t in self._tables.values()}

    def _dense_offsets(self, key, build):
        """Offsets that follow from shapes alone (dense id tensors), built once per shape."""
        hit = self._offsets_cache.get(key)
        if hit is None:
            if len(self._offsets_cache) >= 256:
                self._offsets_cache.clear()
            hit = self._offsets_cache[key] = build()
        return hit

    def _format(self, name, opt, data):
        """(values int64 [N], weight | None, offsets int32 [S+1], output shape prefix, whether the
        offsets are 0, 1, 2, ... by construction, the (rows, width) of a dense id tensor | None)."""
        unit = False
        dense = None
        if isinstance(data, RaggedTensor):
            values = data.values()
            offsets = data.offsets()[-1]
            weight = data.weight() if opt.use_weight else None
            shape = tuple(data.real_shape(0, -1))
            prod = 1
            for d in shape:
                prod *= d
            if prod != offsets.numel() - 1:
                raise RuntimeError("RaggedTensor must pad before lookup, got: %s (%s)" % (data, name))
        elif isinstance(data, torch.Tensor):
            if data.dim() == 1:
                data = data.view(-1, 1)
            values = data.reshape(-1)
            width = data.shape[-1]
            rows = values.numel() // width
            dense = (rows, width)
            offsets = self._dense_offsets((rows, width, data.device), lambda: torch.arange(
                rows + 1, device=data.device, dtype=torch.int32) * width)
            weight = None
            shape = tuple(data.shape[:-1])
            unit = width == 1
        else:
            raise TypeError("feature %s: expected RaggedTensor or Tensor, got %s" % (name, type(data)))
        if values.dtype != torch.int64:
            values = values.long()
        return values, weight, offsets.to(torch.int32), shape, unit, dense

    def forward(self, inputs: Dict[str, Union[torch.Tensor, RaggedTensor]]):
        outputs = {}
        # the same input objects under two combiners (a sequence pooled AND kept row by row) are
        # tagged, merged and deduplicated once per call
        plans = {}
        for gkey, grp in self._groups.items():
            table = self._tables[gkey]
            dev = table._impl_device
            info = table._hashtable_impl.children_info()
            tag_of = self._tags.get(gkey)
            if tag_of is None:  # the 12-bit table index of every feature's shared name, fixed after construction
                tag_of = self._tags[gkey] = {n: info.child_index(o.shared_name) for n, o in grp.features.items()}
            runtime = OrderedDict()
            for name in grp.features:
                if name in inputs:
                    runtime.setdefault(self._runtime_key[name], []).append(name)
            for names in runtime.values():
                opt0 = grp.features[names[0]]
                if (table.training and opt0.combiner in ("sum", "mean") and opt0.trainable and opt0.admit_hook is None
                        and opt0.grad_reduce_by != "id" and table._dtype in (torch.float32, torch.bfloat16, torch.float16)
                        and all(type(inputs[n]) is torch.Tensor for n in names)):
                    # dense id columns only: tagging, dedup, lookup and the rows of every column in one native call
                    stamp = getattr(table._filter_hook_impl, "stamp_target", lambda: None)()
                    if stamp is not None or isinstance(table._filter_hook_impl, torch.nn.Identity):
                        res = DenseLookupFunction.apply(table._backward_holder, table._hashtable_impl,
                                                        [inputs[n] for n in names],
                                                        [tag_of[n] for n in names] if info.is_coalesce() else None, stamp)
                        if res is not None:
                            for name, part in zip(names, res[1:]):
                                outputs[name] = part
                            continue
                vals, weights, offs, shapes, dense = [], [], [], [], []
                all_unit = True
                any_weight = opt0.use_weight and any(
                    isinstance(inputs[n], RaggedTensor) and inputs[n].weight() is not None for n in names)
                for name in names:
                    data = inputs[name]
                    if type(data) is torch.Tensor and data.dtype == torch.int64 and data.device == dev \
                            and data.dim() == 2 and data.shape[1] == 1:
                        # the common dense case, a [B, 1] id column: nothing to convert
                        rows = data.shape[0]
                        v, w, shape, d = data.view(-1), None, (rows,), (rows, 1)
                        o = self._offsets_cache.get((rows, 1, dev))
                        if o is None:
                            o = self._dense_offsets((rows, 1, dev), lambda: torch.arange(
                                rows + 1, device=dev, dtype=torch.int32))
                    else:
                        v, w, o, shape, unit, d = self._format(name, grp.features[name], data)
                        all_unit = all_unit and unit
                        v, o = v.to(dev), o.to(dev)
                    dense.append(d)
                    vals.append(v)
                    offs.append(o)
                    if w is None and any_weight:
                        w = torch.ones(v.numel(), device=dev)
                    weights.append(None if w is None else w.to(dev))
                    shapes.append(shape)
                same = (gkey,) + tuple((id(inputs[n]), tag_of[n]) for n in names)
                if same in plans:
                    offsets, plan = plans[same]
                else:
                    # the id tensors go to the plan as they are: it tags (ids_encode) / concatenates them
                    # in its own reads
                    tags = [tag_of[n] for n in names] if info.is_coalesce() else None
                    ids = vals if (tags is not None or len(vals) > 1) else vals[0]
                    if len(offs) == 1:
                        offsets = offs[0]
                    elif all(d is not None for d in dense):  # dense id tensors only: a function of the shapes
                        offsets = self._dense_offsets((tuple(dense), dev), lambda: ops.merge_offsets(
                            offs, [v.numel() for v in vals]))
                    else:
                        offsets = ops.merge_offsets(offs, [v.numel() for v in vals])
                    if opt0.combiner == "tile":
                        if (table.training and opt0.trainable and opt0.admit_hook is None
                                and table._dtype in (torch.float32, torch.bfloat16, torch.float16)):
                            plan = plan_lookup(table._hashtable_impl, ids, tags=tags)   # dedup + find-or-insert, one pass
                        else:
                            plan = ops.ids_unique_plan(ids, wait=False, need_pos=False, tags=tags)
                    else:  # lean (no per-occurrence arrays) only if no other option can come to share it
                        alone = sum(1 for k in runtime.values() if any(inputs[n] is inputs[names[0]] for n in k)) == 1
                        plan = make_plan(table, ids, offsets, opt0, any_weight, unit_segments=all_unit and alone,
                                         tags=tags)
                    plans[same] = (offsets, plan)
                weight = None
                if all(w is not None for w in weights):
                    weight = weights[0] if len(weights) == 1 else torch.cat(weights)
                seg_counts = [o.numel() - 1 for o in offs]
                if opt0.combiner == "tile":
                    # every feature keeps its own number of rows per sample: the list form of the
                    # padded gather (embedding_engine.py:383-411, 453-455)
                    tile_lens = [int(grp.features[n].combiner_kwargs["tile_len"]) for n in names]
                    if opt0.grad_reduce_by == "id" and table.training and opt0.trainable:
                        pooled = lookup_and_pool(table, plan, weight, offsets, opt0,
                                                 combiner_kwargs={"bs": seg_counts, "tile_len": tile_lens})
                        width = pooled.shape[1]
                        parts = [p.view(b, t * width) for p, b, t in zip(
                            torch.split(pooled, [b * t for b, t in zip(seg_counts, tile_lens)]), seg_counts, tile_lens)]
                    elif (table.training and opt0.trainable and opt0.admit_hook is None
                          and table._dtype in (torch.float32, torch.bfloat16, torch.float16)):
                        # lookup and padded gather as one function: the rows the plan brought along are used
                        # (no second lookup of the same ids) and the gradients reach the table unsummed
                        index, *parts = LookupTileFunction.apply(table._backward_holder, table._hashtable_impl,
                                                                 plan, offsets, seg_counts, tile_lens, False)
                        table._filter_hook_impl(index)
                    else:
                        emb = lookup_unique_rows(table, plan.unique, opt0.admit_hook, opt0.trainable,
                                                 grad_key=plan.serial)
                        parts = RaggedTileParts.apply(emb, plan.inverse, offsets, plan, seg_counts, tile_lens)
                    for name, part, shape in zip(names, parts, shapes):
                        outputs[name] = part if len(shape) == 1 else part.reshape(tuple(shape) + (part.shape[1],))
                    continue
                parts = lookup_and_pool(table, plan, weight, offsets, opt0, unit_segments=all_unit, split=seg_counts)
                for name, part, shape in zip(names, parts, shapes):
                    # [segments, width] already is the answer for a 1-D batch shape: no extra view node
                    outputs[name] = part if len(shape) == 1 else part.reshape(tuple(shape) + (part.shape[1],))
        return outputs

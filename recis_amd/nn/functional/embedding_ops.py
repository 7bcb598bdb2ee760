"""Pooling of looked-up rows with autograd: the mirror of
``recis.nn.functional.embedding_ops`` (embedding_ops.py:133-420).

``ragged_embedding_segment_reduce`` keeps the reference's two semantics of "mean":
ragged mode (more than 5 ids per segment on average, or tile) divides by the segment
length; sparse mode divides by the segment's weight sum. Both run on the same HIP
pooling kernel here (a small team of lanes per short segment replaces the
reference's separate per-occurrence atomic kernel).
"""
from typing import List, Optional, Union

import torch

from ... import ops


def segment_sum_sparse(data, weight, indices, segment_ids, num_segments, backend="recis"):
    """embedding_ops.py:19-71: ``out[segment_ids[i]] += weight[i] * data[indices[i]]``. Backend
    "recis" is the HIP operator; "torch" the reference's gather + ``index_add_`` formulation."""
    if backend == "recis":
        return ops.segment_sum(data, weight, indices, segment_ids, num_segments)
    if backend == "torch":
        src = data[indices]
        if weight is not None:
            src = src * torch.unsqueeze(weight, dim=-1)
        out = torch.zeros([num_segments, data.shape[-1]], dtype=src.dtype, device=data.device)
        out.index_add_(0, segment_ids, src)
        return out
    raise RuntimeError("Segment sum sparse only support ['recis'|'torch'] backend, got: %s" % backend)


def weight_norm_sparse(data, weight, segment_ids, num_segments, backend="recis"):
    """embedding_ops.py:74-130. Backend "recis": every weight divided by the sum of the weights of
    its segment (segment_ops_kernel.cu:74-108); backend "torch": by the number of occurrences of
    its segment, as the reference's torch formulation does."""
    if backend == "recis":
        return ops.segment_mean(data, weight, segment_ids, num_segments)
    if backend == "torch":
        if weight is None:
            weight = torch.ones([segment_ids.numel()], dtype=data.dtype, device=data.device)
        count = torch.zeros([num_segments], dtype=weight.dtype, device=weight.device)
        count.index_add_(0, segment_ids, torch.ones_like(segment_ids, dtype=weight.dtype))
        count = count + (count <= 0).to(count.dtype)
        return weight / count[segment_ids]
    raise RuntimeError("Weight norm sparse only support ['recis'|'torch'] backend, got: %s" % backend)


class EmbeddingSegmentReduceSparse(torch.autograd.Function):
    """embedding_ops.py:133-213: per-occurrence pooling by segment ids. Backend "auto" runs the HIP
    operator in both directions (the reference falls back to torch's ``index_add_`` for the
    backward); the backward is the same operator with ``indices`` and ``segment_ids`` swapped."""

    @staticmethod
    def forward(ctx, unique_emb, weight, reverse_indices, segment_ids, num_segments, combiner, backend):
        backend = "recis" if backend == "auto" else backend
        ctx.backend = backend
        ctx.unique_size = unique_emb.size(0)
        if combiner == "mean":
            weight = weight_norm_sparse(unique_emb, weight, segment_ids, num_segments, backend=backend)
        ctx.save_for_backward(weight, reverse_indices, segment_ids)
        return segment_sum_sparse(unique_emb, weight, reverse_indices, segment_ids, num_segments, backend=backend)

    @staticmethod
    def backward(ctx, grad):
        weight, reverse_indices, segment_ids = ctx.saved_tensors
        g = segment_sum_sparse(grad.contiguous(), weight, segment_ids, reverse_indices, ctx.unique_size,
                               backend=ctx.backend)
        return g, None, None, None, None, None, None


class EmbeddingSegmentReduceRagged(torch.autograd.Function):
    """``combiner`` in sum | mean | max | tile. For tile, ``combiner_kwargs['tile_len']``
    rows are kept per segment (zero padded), returned as ``[S, tile_len * D]``."""

    @staticmethod
    def forward(ctx, unique_emb, weight, reverse_indices, offsets, combiner, combiner_kwargs, plan=None):
        ctx.combiner = combiner
        ctx.plan = plan
        ctx.unique_size = unique_emb.shape[0]
        ctx.emb_dtype = unique_emb.dtype
        if combiner == "tile" and "bs" in combiner_kwargs:
            # the reference's own form (embedding_ops.py:253-271): several tensors in one call,
            # rows per tensor in "bs", rows kept per sample in "tile_len" (two lists); the result
            # is [sum of bs[i] * tile_len[i], D], unreshaped
            bs, tile_len = list(combiner_kwargs["bs"]), list(combiner_kwargs["tile_len"])
            out, batch_seq = ops.ragged_tile(bs, tile_len, reverse_indices, offsets, unique_emb)
            ctx.tile = (batch_seq, [ctx.unique_size, len(bs), max(bs), min(tile_len)], bs, tile_len)
            ctx.save_for_backward(reverse_indices, offsets)
            return out
        if combiner == "tile":
            tile_len = int(combiner_kwargs["tile_len"])
            S = offsets.numel() - 1
            out, batch_seq = ops.ragged_tile([S], [tile_len], reverse_indices, offsets, unique_emb)
            ctx.tile = (batch_seq, [ctx.unique_size, 1, S, tile_len], None, None)
            ctx.save_for_backward(reverse_indices, offsets)
            return out.view(S, tile_len * unique_emb.shape[1])
        if combiner == "max":
            out, argmax = ops.segment_reduce_forward(unique_emb, None, reverse_indices, offsets, "max",
                                                     return_argmax=True)
            ctx.save_for_backward(reverse_indices, offsets, argmax)
            return out
        out = ops.segment_reduce_forward(unique_emb, weight, reverse_indices, offsets, combiner)
        ctx.save_for_backward(reverse_indices, offsets, weight)
        return out

    @staticmethod
    def backward(ctx, grad):
        grad = grad.contiguous()
        if ctx.combiner == "tile":
            rev, offsets = ctx.saved_tensors
            batch_seq, info, bs, tile_len = ctx.tile
            if bs is not None:
                if ctx.plan is not None:
                    g = ops.csr_gather_reduce(grad, ctx.plan, ctx.plan.src_for_tile(bs, tile_len, offsets))
                else:
                    g = ops.ragged_tile_back(batch_seq, info, rev, offsets, grad)
                return g.to(ctx.emb_dtype), None, None, None, None, None, None
            D = grad.shape[1] // info[3]
            if ctx.plan is not None:
                src = ctx.plan.src_for_tile([info[2]], [info[3]], offsets)
                g = ops.csr_gather_reduce(grad.view(-1, D), ctx.plan, src)
            else:
                g = ops.ragged_tile_back(batch_seq, info, rev, offsets, grad.view(-1, D))
            return g.to(ctx.emb_dtype), None, None, None, None, None, None
        if ctx.combiner == "max":
            rev, offsets, argmax = ctx.saved_tensors
            g = ops.segment_reduce_backward(grad, None, rev, offsets, ctx.unique_size, "max", argmax=argmax,
                                            out_dtype=ctx.emb_dtype)
            return g, None, None, None, None, None, None
        rev, offsets, weight = ctx.saved_tensors
        if ctx.plan is not None:
            g = ops.segment_reduce_backward_plan(grad, weight, offsets, ctx.plan, ctx.combiner).to(ctx.emb_dtype)
        else:
            g = ops.segment_reduce_backward(grad, weight, rev, offsets, ctx.unique_size, ctx.combiner,
                                            out_dtype=ctx.emb_dtype)
        return g, None, None, None, None, None, None


class RaggedTileParts(torch.autograd.Function):
    """The padded gather of several features at once with ONE output per feature
    (``[bs[f], tile_len[f] * D]``, views of one buffer). Splitting a single output instead makes
    autograd concatenate the features' gradients again before the backward sees them, a copy of
    the whole padded gradient (2 GB for long behaviour sequences); here every feature's gradient
    goes through its own gather-reduce pass over the plan's occurrence lists."""

    @staticmethod
    def forward(ctx, unique_emb, reverse_indices, offsets, plan, bs, tile_len):
        bs, tile_len = [int(b) for b in bs], [int(t) for t in tile_len]
        out, _ = ops.ragged_tile(bs, tile_len, reverse_indices, offsets, unique_emb)
        D = unique_emb.shape[1]
        ctx.plan, ctx.bs, ctx.tile_len, ctx.D = plan, bs, tile_len, D
        ctx.unique_size, ctx.emb_dtype = unique_emb.shape[0], unique_emb.dtype
        ctx.save_for_backward(offsets)
        rows = [b * t for b, t in zip(bs, tile_len)]
        return tuple(p.view(b, t * D) for p, b, t in zip(torch.split(out, rows), bs, tile_len))

    @staticmethod
    def backward(ctx, *grads):
        (offsets,) = ctx.saved_tensors
        plan, D = ctx.plan, ctx.D
        src = plan.src_for_tile(ctx.bs, ctx.tile_len, offsets)  # row of the whole padded output per list entry
        rows = [b * t for b, t in zip(ctx.bs, ctx.tile_len)]
        if len(grads) <= 8 and all(g is not None for g in grads) and len({g.dtype for g in grads}) == 1 \
                and grads[0].dtype in (torch.float32, torch.bfloat16, torch.float16):
            # one pass: the kernel takes the features' gradients as separate arrays
            g = ops.csr_gather_reduce_parts([grad.reshape(n, D) for grad, n in zip(grads, rows)], plan, src)
            return g.to(ctx.emb_dtype), None, None, None, None, None
        g, lo = None, 0
        for grad, b, t in zip(grads, ctx.bs, ctx.tile_len):
            n = b * t
            if grad is not None and n:
                # this feature's rows only, counted from its own first row; the others are skipped
                mine = torch.where((src >= lo) & (src < lo + n), src - lo, -1)
                g = ops.csr_gather_reduce(grad.reshape(n, D), plan, mine, out=g, accumulate=g is not None)
            lo += n
        if g is None:
            g = torch.zeros((ctx.unique_size, D), dtype=torch.float32, device=offsets.device)
        return g.to(ctx.emb_dtype), None, None, None, None, None


def ragged_embedding_segment_reduce(unique_emb: torch.Tensor, weight: Optional[torch.Tensor],
                                    reverse_indices: torch.Tensor, offsets: torch.Tensor, combiner: str,
                                    combiner_kwargs: Optional[dict] = None, plan=None):
    """``recis.nn.functional.embedding_ops.ragged_embedding_segment_reduce``
    (embedding_ops.py:332-420), plus the ``"max"`` combiner. ``plan`` (the ``BatchPlan`` whose
    ``inverse`` is ``reverse_indices``) switches the backward from atomics to the gather-reduce
    over the plan's occurrence lists."""
    if combiner_kwargs is None:
        combiner_kwargs = {}
    assert combiner in ["sum", "mean", "tile", "max"], "combiner %s is not supported" % combiner
    n_occ = unique_emb.shape[0] if reverse_indices is None else reverse_indices.numel()
    sparse_mode = not (combiner in ("tile", "max") or n_occ / offsets.numel() > 5)
    if sparse_mode and combiner == "mean":
        # sparse-mode mean: w_i / sum of the segment's weights (segment_ops_kernel.cu:92-108)
        seg = ops.gen_segment_indices_by_offset(offsets)
        weight = ops.segment_mean(unique_emb, weight, seg, offsets.numel() - 1)
        combiner = "sum"
    return EmbeddingSegmentReduceRagged.apply(unique_emb, weight, reverse_indices, offsets, combiner,
                                              combiner_kwargs, plan)


def sparse_embedding_segment_reduce(unique_emb: torch.Tensor, weight: torch.Tensor, reverse_indices: torch.Tensor,
                                    segment_ids: torch.Tensor, num_segments: int, combiner: str):
    """embedding_ops.py:423-461."""
    assert combiner in ["sum", "mean"], "combiner %s is not supported" % combiner
    assert weight is not None, "none weight is not supported"
    return EmbeddingSegmentReduceSparse.apply(unique_emb, weight, reverse_indices, segment_ids, num_segments,
                                              combiner, "auto")


def merge_offsets(offsets: List[torch.Tensor], max_value=None) -> torch.Tensor:
    """embedding_ops.py:464-483 over ``torch.ops.recis.merge_offsets(offsets, max_value)``: the
    offsets of several ragged tensors as one. ``max_value`` (list or host tensor: the number of
    values each tensor's offsets run over) defaults to every tensor's last offset, which costs a
    read-back."""
    if max_value is None:
        max_value = torch.stack([o[-1] for o in offsets]).tolist()
    return ops.merge_offsets(offsets, max_value)


def ids_partition(ids: torch.Tensor, max_partition_num: int, world_size: int):
    """embedding_ops.py:486-511: (unique ids in shard order, ids per shard, reverse indices)."""
    return ops.ids_partition(ids, world_size)


def ids_encode(ids_list: List[torch.Tensor], table_ids: Union[torch.Tensor, list]):
    """embedding_ops.py:514-552."""
    assert isinstance(ids_list, list), "ids_list must be a list"
    for ids in ids_list:
        assert isinstance(ids, torch.Tensor), "ids must be a tensor"
        assert ids.device == ids_list[0].device, "ids must be on the same device, %s != %s" % (
            ids.device, ids_list[0].device)
    return ops.ids_encode(ids_list, table_ids)

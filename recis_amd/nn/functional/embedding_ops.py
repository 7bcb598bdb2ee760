"""Pooling of looked-up rows with autograd: the mirror of
``recis.nn.functional.embedding_ops`` (embedding_ops.py:133-420).

``ragged_embedding_segment_reduce`` keeps the reference's two semantics of "mean":
ragged mode (more than 5 ids per segment on average, or tile) divides by the segment
length; sparse mode divides by the segment's weight sum. Both run on the same HIP
pooling kernel here (a small team of lanes per short segment replaces the
reference's separate per-occurrence atomic kernel).
"""
from typing import Optional

import torch

from ... import ops


class EmbeddingSegmentReduceRagged(torch.autograd.Function):
    """``combiner`` in sum | mean | max | tile. For tile, ``combiner_kwargs['tile_len']``
    rows are kept per segment (zero padded), returned as ``[S, tile_len * D]``."""

    @staticmethod
    def forward(ctx, unique_emb, weight, reverse_indices, offsets, combiner, combiner_kwargs, plan=None):
        ctx.combiner = combiner
        ctx.plan = plan
        ctx.unique_size = unique_emb.shape[0]
        ctx.emb_dtype = unique_emb.dtype
        if combiner == "tile":
            tile_len = int(combiner_kwargs["tile_len"])
            S = offsets.numel() - 1
            out, batch_seq = ops.ragged_tile([S], [tile_len], reverse_indices, offsets, unique_emb)
            ctx.tile = (batch_seq, [ctx.unique_size, 1, S, tile_len])
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
            batch_seq, info = ctx.tile
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

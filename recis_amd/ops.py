"""Operator layer: the functions RecIS registers as ``torch.ops.recis.*``
(csrc/bind.cc:172-210), implemented on librecis_hip.so.

Names, argument order and argument meaning follow the reference registrations;
arguments the reference does not have are keyword-only and default to the
reference behaviour. Tensors must live on the GPU: there is no CPU path here.
"""
import ctypes

import torch

from . import _lib
from ._lib import check, dtype_code, i64, lib, ptr, require_cuda, stream_ptr


def _index_kind(t, name):
    if t.dtype == torch.int64:
        return 1
    if t.dtype == torch.int32:
        return 0
    raise TypeError("%s must be int32 or int64, got %s" % (name, t.dtype))


def _contig(t):
    return t if t is None or t.is_contiguous() else t.contiguous()


def _rev_ptr(rev, other):
    """NULL means "identity" to the library; an empty (but given) index tensor has
    a NULL data pointer too, so hand over another valid pointer: with zero
    occurrences it is never dereferenced."""
    if rev is None:
        return ptr(None)
    return ptr(rev) if rev.numel() else ptr(other)


# --------------------------------------------------------------------- pooling
def segment_reduce_forward(unique_emb, weight, reverse_indices, offsets, mode, *,
                           out_dtype=None, return_argmax=False):
    """``torch.ops.recis.segment_reduce_forward`` (embedding_segment_reduce.h:9-12).

    ``mode``: "sum" | "mean" | "tile", plus "max" (an addition). ``reverse_indices``
    may be None for rows that are already materialised per occurrence. With
    ``mode="max"`` and ``return_argmax=True`` returns ``(out, argmax)``.
    """
    require_cuda(unique_emb, weight, reverse_indices, offsets)
    if mode not in _lib.MODES:
        raise ValueError("Invalid mode: %s" % mode)
    unique_emb, weight = _contig(unique_emb), _contig(weight)
    reverse_indices, offsets = _contig(reverse_indices), _contig(offsets)
    U, D = unique_emb.shape
    S = offsets.numel() - 1
    B = reverse_indices.numel() if reverse_indices is not None else U
    out_dtype = out_dtype or unique_emb.dtype
    out = torch.empty((B if mode == "tile" else S, D), dtype=out_dtype, device=unique_emb.device)
    argmax = None
    if mode == "max" and return_argmax:
        argmax = torch.empty((S, D), dtype=torch.int32, device=unique_emb.device)
    check(lib().recis_segment_reduce_forward(
        ptr(unique_emb), dtype_code(unique_emb.dtype),
        ptr(weight), dtype_code(weight.dtype) if weight is not None else 0,
        _rev_ptr(reverse_indices, offsets),
        _index_kind(reverse_indices, "reverse_indices") if reverse_indices is not None else 1,
        ptr(offsets), _index_kind(offsets, "offsets"),
        ptr(out), dtype_code(out_dtype), ptr(argmax),
        i64(B), i64(U), i64(S), i64(D), _lib.MODES[mode], stream_ptr(unique_emb.device)))
    if mode == "max" and return_argmax:
        return out, argmax
    return out


def segment_reduce_backward(grad_output, weight, reverse_indices, offsets, unique_size, mode, *,
                            rev_unique=False, argmax=None, out_dtype=None):
    """``torch.ops.recis.segment_reduce_backward`` (embedding_segment_reduce.h:14-17).

    ``rev_unique=True`` promises that ``reverse_indices`` has no duplicates, which
    lets every gradient row be written once with plain stores; otherwise
    duplicates are accumulated with fp32 atomics (the result is then fp32
    internally and cast to ``out_dtype``).
    """
    require_cuda(grad_output, weight, reverse_indices, offsets, argmax)
    if mode not in _lib.MODES:
        raise ValueError("Invalid mode: %s" % mode)
    grad_output, weight = _contig(grad_output), _contig(weight)
    reverse_indices, offsets = _contig(reverse_indices), _contig(offsets)
    D = grad_output.shape[1]
    S = offsets.numel() - 1
    U = int(unique_size)
    B = reverse_indices.numel() if reverse_indices is not None else U
    out_dtype = out_dtype or grad_output.dtype
    unique = rev_unique or reverse_indices is None
    work_dtype = out_dtype if unique else torch.float32
    out = torch.empty((U, D), dtype=work_dtype, device=grad_output.device)
    check(lib().recis_segment_reduce_backward(
        ptr(grad_output), dtype_code(grad_output.dtype),
        ptr(weight), dtype_code(weight.dtype) if weight is not None else 0,
        _rev_ptr(reverse_indices, offsets),
        _index_kind(reverse_indices, "reverse_indices") if reverse_indices is not None else 1,
        ptr(offsets), _index_kind(offsets, "offsets"), ptr(argmax),
        ptr(out), dtype_code(work_dtype), i64(B), i64(U), i64(S), i64(D), _lib.MODES[mode],
        _lib.FLAG_REV_UNIQUE if unique else 0, stream_ptr(grad_output.device)))
    return out if work_dtype == out_dtype else out.to(out_dtype)

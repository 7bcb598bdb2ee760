"""Operator layer: the functions RecIS registers as ``torch.ops.recis.*``
(csrc/bind.cc:172-210), implemented on librecis_hip.so.

Names, argument order and argument meaning follow the reference registrations;
arguments the reference does not have are keyword-only and default to the
reference behaviour. Tensors must live on the GPU: there is no CPU path here.
"""
import ctypes
import itertools

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


def segment_reduce_forward_blocks(emb_blocks, block_size, row_index, weight, reverse_indices, offsets, mode, *,
                                  out_dtype=None):
    """``segment_reduce_forward`` over rows that stay where the table keeps them: unique row
    ``u`` is row ``row_index[u]`` of ``emb_blocks`` (a negative index reads as zeros). Same
    result as ``segment_reduce_forward(block_gather(row_index, emb_blocks, block_size, -1, True),
    weight, reverse_indices, offsets, mode)`` without the ``[U, D]`` intermediate
    (``recis_segment_reduce_forward_blocks``). ``mode``: "sum" | "mean" | "tile"."""
    if mode not in ("sum", "mean", "tile"):
        raise ValueError("Invalid mode for pooling out of the table: %s" % mode)
    b0 = _check_blocks(emb_blocks, block_size)
    require_cuda(row_index, weight, reverse_indices, offsets)
    row_index = _ids64(row_index)
    weight, reverse_indices, offsets = _contig(weight), _contig(reverse_indices), _contig(offsets)
    U, D = row_index.numel(), b0[0].numel()
    S = offsets.numel() - 1
    B = reverse_indices.numel() if reverse_indices is not None else U
    out_dtype = out_dtype or b0.dtype
    out = torch.empty((B if mode == "tile" else S, D), dtype=out_dtype, device=b0.device)
    tab = block_ptr_table(emb_blocks)
    check(lib().recis_segment_reduce_forward_blocks(
        ptr(tab), i64(len(emb_blocks)), i64(block_size), i64(_pitch_bytes(emb_blocks)), ptr(row_index),
        dtype_code(b0.dtype), ptr(weight), dtype_code(weight.dtype) if weight is not None else 0,
        _rev_ptr(reverse_indices, offsets),
        _index_kind(reverse_indices, "reverse_indices") if reverse_indices is not None else 1,
        ptr(offsets), _index_kind(offsets, "offsets"), ptr(out), dtype_code(out_dtype),
        i64(B), i64(U), i64(S), i64(D), _lib.MODES[mode], stream_ptr(b0.device)))
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


# ------------------------------------------------------------- small helpers
def _host_ptrs(tensors):
    return (ctypes.c_void_p * len(tensors))(*[t.data_ptr() for t in tensors])


def _host_i64(values):
    return (ctypes.c_int64 * len(values))(*[int(v) for v in values])


_PTR_TABLE_CACHE = {}


def block_ptr_table(blocks):
    """Device int64 tensor holding the base pointer of every block.

    Cached on the tuple of pointers, so a slot that does not grow pays the
    host-to-device copy once, not per launch."""
    key = (blocks[0].device.index,) + tuple(b.data_ptr() for b in blocks)
    tab = _PTR_TABLE_CACHE.get(key)
    if tab is None:
        if len(_PTR_TABLE_CACHE) > 256:
            _PTR_TABLE_CACHE.clear()
        tab = torch.tensor(key[1:], dtype=torch.int64).to(blocks[0].device)
        _PTR_TABLE_CACHE[key] = tab
    return tab


def _check_blocks(blocks, block_size):
    if len(blocks) == 0:
        raise ValueError("empty block list")
    b0 = blocks[0]
    for b in blocks:
        require_cuda(b)
        if b.dtype != b0.dtype or b.shape[1:] != b0.shape[1:] or not _rows_dense(b) or b.stride(0) != b0.stride(0):
            raise ValueError("blocks must hold contiguous rows at one pitch and share dtype and row shape")
        if b.shape[0] < block_size:
            raise ValueError("block with %d rows is smaller than block_size %d" % (b.shape[0], block_size))
    return b0


def _rows_dense(block):
    """Every row of ``block`` is contiguous and rows do not overlap (rows may lie a pitch apart: a slot
    that shares its allocation with the optimizer state of the same keys)."""
    if block.is_contiguous():
        return True
    return block.dim() >= 1 and block[0].is_contiguous() and block.stride(0) >= block[0].numel()


def _pitch_bytes(*block_lists):
    """``row_pitch_bytes`` of the C header for block lists that go into one call: 0 when rows lie back to
    back, else the distance between rows, which all the lists must share."""
    b0 = block_lists[0][0]
    for blocks in block_lists:
        if blocks[0].stride(0) != b0.stride(0) or blocks[0].dtype != b0.dtype:
            raise ValueError("slots that are updated together must share dtype and row pitch")
    return 0 if b0.is_contiguous() else b0.stride(0) * b0.element_size()


def _row_bytes(block):
    n = block.element_size()
    for d in block.shape[1:]:
        n *= d
    return n


def _ids64(ids):
    if not ids.is_cuda:
        require_cuda(ids)
    if ids.dtype != torch.int64:
        raise TypeError("ids must be int64, got %s" % ids.dtype)
    if ids.dim() == 1 and ids.is_contiguous():
        return ids
    return _contig(ids).view(-1)


# ---------------------------------------------------------------- row blocks
def gather(ids, emb):
    """``torch.ops.recis.gather`` (block_ops.h:6): ``emb[ids]`` for a flat table."""
    require_cuda(ids, emb)
    ids, emb = _contig(ids).view(-1), _contig(emb)
    out = torch.empty((ids.numel(),) + tuple(emb.shape[1:]), dtype=emb.dtype, device=emb.device)
    check(lib().recis_gather(ptr(ids), _index_kind(ids, "ids"), ptr(emb), i64(emb.shape[0]), ptr(out),
                             i64(ids.numel()), i64(_row_bytes(emb)), stream_ptr(emb.device)))
    return out


def block_gather(ids, emb_blocks, block_size, default_key=-1, readonly=False):
    """``torch.ops.recis.block_gather`` (block_ops.h:8-12)."""
    b0 = _check_blocks(emb_blocks, block_size)
    ids = _ids64(ids)
    out = torch.empty((ids.numel(),) + tuple(b0.shape[1:]), dtype=b0.dtype, device=b0.device)
    tab = block_ptr_table(emb_blocks)
    check(lib().recis_block_gather(ptr(ids), ptr(tab), i64(len(emb_blocks)), i64(block_size),
                                   i64(_pitch_bytes(emb_blocks)), i64(default_key), int(bool(readonly)), ptr(out), i64(ids.numel()),
                                   i64(_row_bytes(b0)), stream_ptr(b0.device)))
    return out


def block_gather_by_range(ids, emb_blocks, block_size, beg, end):
    """``block_gather_by_range`` (block_ops.cc:305-314): rows of ``ids[beg:end]``."""
    return block_gather(_ids64(ids)[beg:end], emb_blocks, block_size, -1, False)


def block_insert(ids, embedding, emb_blocks, block_size):
    """``torch.ops.recis.block_insert`` (block_ops.h:28-30); one embedding row is broadcast."""
    b0 = _check_blocks(emb_blocks, block_size)
    ids = _ids64(ids)
    require_cuda(embedding)
    embedding = _contig(embedding)
    if embedding.dtype != b0.dtype:
        raise TypeError("embedding dtype %s does not match the blocks (%s)" % (embedding.dtype, b0.dtype))
    if not (embedding.shape[0] == ids.numel() or embedding.shape[0] == 1):
        raise ValueError("ids batch_size must = embedding batch size or embedding batch size = 1")
    broadcast = int(embedding.shape[0] == 1 and ids.numel() != 1)
    tab = block_ptr_table(emb_blocks)
    check(lib().recis_block_insert(ptr(ids), ptr(embedding), broadcast, ptr(None), ptr(tab),
                                   i64(len(emb_blocks)), i64(block_size), i64(_pitch_bytes(emb_blocks)),
                                   i64(ids.numel()), i64(_row_bytes(b0)), stream_ptr(b0.device)))


def block_insert_with_mask(ids, embedding, mask, emb_blocks, block_size):
    """``torch.ops.recis.block_insert_with_mask`` (block_ops.h:32-36)."""
    b0 = _check_blocks(emb_blocks, block_size)
    ids = _ids64(ids)
    require_cuda(embedding, mask)
    embedding = _contig(embedding)
    if embedding.dtype != b0.dtype:
        raise TypeError("embedding dtype %s does not match the blocks (%s)" % (embedding.dtype, b0.dtype))
    if mask.dtype != torch.bool:
        raise TypeError("mask must be bool")
    mask = _contig(mask)
    tab = block_ptr_table(emb_blocks)
    check(lib().recis_block_insert(ptr(ids), ptr(embedding), 0, ptr(mask), ptr(tab),
                                   i64(len(emb_blocks)), i64(block_size), i64(_pitch_bytes(emb_blocks)),
                                   i64(ids.numel()), i64(_row_bytes(b0)), stream_ptr(b0.device)))


def block_filter(ids, emb_blocks, block_size, threshold):
    """``torch.ops.recis.block_filter`` (block_ops.h:20-22): ``slot[ids] < threshold``."""
    b0 = _check_blocks(emb_blocks, block_size)
    if b0.dtype not in (torch.int32, torch.int64) or _row_bytes(b0) != b0.element_size():
        raise TypeError("block_filter needs an int32/int64 slot of width 1")
    ids = _ids64(ids)
    out = torch.empty(ids.numel(), dtype=torch.bool, device=b0.device)
    tab = block_ptr_table(emb_blocks)
    check(lib().recis_block_filter(ptr(ids), ptr(tab), i64(len(emb_blocks)), i64(block_size),
                                   i64(threshold), int(b0.dtype == torch.int64), ptr(out),
                                   i64(ids.numel()), stream_ptr(b0.device)))
    return out


# ----------------------------------------------------------------- optimizers
def block_apply_adamw(index, grad, emb_blocks, beta1_t, beta2_t, step, exp_avg, exp_avg_sq, lr,
                      beta1, beta2, weight_decay, eps, block_size):
    """``torch.ops.recis.block_apply_adamw`` (block_apply_adamw_op.h:6-12).

    In place on the three block lists and on ``beta1_t`` / ``beta2_t`` (GPU scalars,
    float32 or float64). ``weight_decay`` is the multiplicative factor applied to the
    row. ``step`` is accepted and left untouched, as in the reference
    (block_apply_adamw_op.cc:121 discards the result of ``step.add(1)``)."""
    b0 = _check_blocks(emb_blocks, block_size)
    _check_blocks(exp_avg, block_size)
    _check_blocks(exp_avg_sq, block_size)
    if len(exp_avg) != len(emb_blocks) or len(exp_avg_sq) != len(emb_blocks):
        raise ValueError("state slots must have as many blocks as the embedding slot")
    index = _ids64(index)
    require_cuda(grad, beta1_t, beta2_t)
    grad = _contig(grad)
    if beta1_t.dtype != beta2_t.dtype or beta1_t.dtype not in (torch.float32, torch.float64):
        raise TypeError("beta1_t / beta2_t must both be float32 or float64")
    D = _row_bytes(b0) // b0.element_size()
    if grad.numel() != index.numel() * D:
        raise ValueError("grad has %d elements, expected %d x %d" % (grad.numel(), index.numel(), D))
    # rows of doubles (the reference's functor is dispatched for them too) go with gradients of doubles
    code = lambda dt: _lib.F64 if dt == torch.float64 and b0.dtype == torch.float64 else dtype_code(dt)
    check(lib().recis_block_apply_adamw(
        ptr(index), ptr(grad), code(grad.dtype), ptr(block_ptr_table(emb_blocks)),
        ptr(block_ptr_table(exp_avg)), ptr(block_ptr_table(exp_avg_sq)), i64(len(emb_blocks)),
        i64(block_size), i64(_pitch_bytes(emb_blocks, exp_avg, exp_avg_sq)), code(b0.dtype), ptr(beta1_t),
        ptr(beta2_t), int(beta1_t.dtype == torch.float64), ctypes.c_double(lr), ctypes.c_double(beta1),
        ctypes.c_double(beta2), ctypes.c_double(weight_decay), ctypes.c_double(eps),
        i64(index.numel()), i64(D), stream_ptr(b0.device)))


def block_apply_adagrad(index, grad, emb_blocks, accum_blocks, lr, eps, block_size):
    """Sparse Adagrad row update (an addition; same conventions as block_apply_adamw)."""
    b0 = _check_blocks(emb_blocks, block_size)
    _check_blocks(accum_blocks, block_size)
    if len(accum_blocks) != len(emb_blocks):
        raise ValueError("state slot must have as many blocks as the embedding slot")
    index = _ids64(index)
    require_cuda(grad)
    grad = _contig(grad)
    D = _row_bytes(b0) // b0.element_size()
    if grad.numel() != index.numel() * D:
        raise ValueError("grad has %d elements, expected %d x %d" % (grad.numel(), index.numel(), D))
    check(lib().recis_block_apply_adagrad(
        ptr(index), ptr(grad), dtype_code(grad.dtype), ptr(block_ptr_table(emb_blocks)),
        ptr(block_ptr_table(accum_blocks)), i64(len(emb_blocks)), i64(block_size),
        i64(_pitch_bytes(emb_blocks, accum_blocks)), dtype_code(b0.dtype),
        ctypes.c_double(lr), ctypes.c_double(eps), i64(index.numel()), i64(D), stream_ptr(b0.device)))


# ------------------------------------------------------------- allocator ops
def generate_ids(gen_num, free_blocks, free_count, cur_count, free_block_size):
    """``torch.ops.recis.generate_ids`` (hashtable_ops.h:17-21)."""
    dev = free_blocks[0].device
    out = torch.empty(gen_num, dtype=torch.int64, device=dev)
    check(lib().recis_generate_ids(i64(gen_num), ptr(block_ptr_table(free_blocks)), i64(free_count),
                                   i64(cur_count), i64(free_block_size), ptr(out), stream_ptr(dev)))
    return out


def free_ids(ids, free_blocks, free_count, free_block_size):
    """``torch.ops.recis.free_ids`` (hashtable_ops.h:23-25); in place on ``free_blocks``."""
    ids = _ids64(ids)
    check(lib().recis_free_ids(ptr(ids), i64(ids.numel()), ptr(block_ptr_table(free_blocks)),
                               i64(free_count), i64(free_block_size), stream_ptr(ids.device)))


def mask_key_index(in_keys, mask, in_out_index, out_size):
    """``torch.ops.recis.mask_key_index`` (hashtable_ops.h:27-30)."""
    in_keys, in_out_index = _ids64(in_keys), _ids64(in_out_index)
    require_cuda(mask)
    if mask.dtype != torch.bool:
        raise TypeError("mask must be bool")
    mask = _contig(mask)
    out_keys = torch.empty(out_size, dtype=torch.int64, device=in_keys.device)
    out_index = torch.empty_like(out_keys)
    check(lib().recis_mask_key_index(ptr(in_keys), ptr(mask), ptr(in_out_index), i64(in_keys.numel()),
                                     i64(out_size), ptr(out_keys), ptr(out_index),
                                     stream_ptr(in_keys.device)))
    return out_keys, out_index


def scatter_ids_with_mask(out_ids, in_ids, mask_index):
    """``torch.ops.recis.scatter_ids_with_mask`` (hashtable_ops.h:32-34); in place, returns ``out_ids``."""
    require_cuda(out_ids, in_ids, mask_index)
    if not out_ids.is_contiguous():
        raise ValueError("out_ids must be contiguous")
    in_ids, mask_index = _ids64(in_ids), _ids64(mask_index)
    check(lib().recis_scatter_ids_with_mask(ptr(out_ids), i64(out_ids.numel()), ptr(in_ids),
                                            ptr(mask_index), i64(in_ids.numel()),
                                            stream_ptr(out_ids.device)))
    return out_ids


# ------------------------------------------------------------ tagging / dedup
def ids_encode(ids_list, table_ids):
    """``torch.ops.recis.ids_encode`` (ids_encode.h:15): tag and concatenate."""
    ids_list = [_ids64(t) for t in ids_list]
    tids = table_ids.tolist() if torch.is_tensor(table_ids) else list(table_ids)
    total = sum(t.numel() for t in ids_list)
    dev = ids_list[0].device
    out = torch.empty(total, dtype=torch.int64, device=dev)
    check(lib().recis_ids_encode(_host_ptrs(ids_list), _host_i64([t.numel() for t in ids_list]),
                                 _host_i64(tids), i64(len(ids_list)), ptr(out), stream_ptr(dev)))
    return out


def merge_offsets(offsets_list, max_value):
    """``torch.ops.recis.merge_offsets`` (embedding_segment_reduce.h:19-20).

    ``max_value`` (host tensor or list): number of values each tensor's offsets run over."""
    offsets_list = [_contig(o) for o in offsets_list]
    require_cuda(*offsets_list)
    dt = offsets_list[0].dtype
    if any(o.dtype != dt for o in offsets_list):
        raise TypeError("offsets must share one integer dtype")
    is64 = _index_kind(offsets_list[0], "offsets")
    mv = max_value.tolist() if torch.is_tensor(max_value) else list(max_value)
    n = len(offsets_list)
    total = sum(o.numel() for o in offsets_list) - (n - 1)
    dev = offsets_list[0].device
    out = torch.empty(total, dtype=dt, device=dev)
    check(lib().recis_merge_offsets(_host_ptrs(offsets_list), _host_i64([o.numel() for o in offsets_list]),
                                    _host_i64(mv), i64(n), is64, ptr(out), stream_ptr(dev)))
    return out


def ids_unique(ids, inverse_dtype=torch.int32):
    """Dedup: ``(unique, inverse, count)`` with the unique ids in order of first
    occurrence. ``unique`` has room for ``len(ids)`` entries, of which the first
    ``count`` (a one-element GPU tensor) are valid: no host synchronisation."""
    ids = _ids64(ids)
    n = ids.numel()
    uniq = torch.empty(n, dtype=torch.int64, device=ids.device)
    inv = torch.empty(n, dtype=inverse_dtype, device=ids.device)
    count = torch.empty(1, dtype=torch.int64, device=ids.device)
    check(lib().recis_unique(ptr(ids), i64(n), ptr(uniq), ptr(inv), int(inverse_dtype == torch.int64),
                             ptr(count), stream_ptr(ids.device)))
    return uniq, inv, count


_SLICE_SIZE = 65536


def ids_partition(ids, num_parts):
    """``torch.ops.recis.ids_partition`` (ids_partition.h:14), device ordering
    (ids_partition_kernel.cu:36-55): unique ids ascending by ``rotr64(id, 16)`` as
    unsigned, per-shard counts, int32 inverse. The dedup is the hash kernel; the
    (much smaller) unique set is ordered by a radix sort of (rotated id, position)
    pairs, and the inverse is a gather of 4-byte rows out of the rank table."""
    if ids.dim() != 1:
        raise ValueError("ids must be 1-dim")
    uniq, inv, count = ids_unique(ids)
    u = uniq[: int(count.item())]
    sorted_u, _, rank = partition_order(u)
    m, r = divmod(_SLICE_SIZE, num_parts)
    slot = torch.bitwise_and(sorted_u, _SLICE_SIZE - 1)
    part = torch.maximum(torch.div(slot, m + 1, rounding_mode="floor"),
                         torch.div(slot - r, m, rounding_mode="trunc"))
    counts = torch.bincount(part, minlength=num_parts).to(torch.int64)
    return sorted_u, counts, gather(inv, rank)


def partition_order(unique_ids):
    """The sort by PartitionKey of ids_partition_kernel.cu:36-55 on ids without duplicates:
    ``(sorted_ids, order, rank)`` with ``sorted_ids == unique_ids[order]`` ascending by
    ``rotr64(id, 16)`` as unsigned and ``rank[order[k]] == k`` (both int32)."""
    require_cuda(unique_ids)
    u = _ids64(unique_ids)
    n = u.numel()
    sorted_u = torch.empty_like(u)
    order = torch.empty(n, dtype=torch.int32, device=u.device)
    rank = torch.empty(n, dtype=torch.int32, device=u.device)
    check(lib().recis_partition_order(ptr(u), i64(n), ptr(sorted_u), ptr(order), ptr(rank), stream_ptr(u.device)))
    return sorted_u, order, rank


# --------------------------------------------------------- sparse-mode pooling
def segment_sum(data, weight, indices, segment_ids, num_segments):
    """``torch.ops.recis.segment_sum`` (segment_ops.h:5-8)."""
    require_cuda(data, weight, indices, segment_ids)
    data, indices, segment_ids = _contig(data), _contig(indices), _contig(segment_ids)
    if indices.dtype != segment_ids.dtype:
        raise TypeError("indices and segment_ids must share a dtype")
    num_segments = int(num_segments)
    D = data.shape[1]
    out = torch.empty((num_segments, D), dtype=torch.float32, device=data.device)
    use_w = weight is not None
    weight = _contig(weight)
    check(lib().recis_segment_sum(ptr(data), dtype_code(data.dtype), i64(data.shape[0]), ptr(weight),
                                  dtype_code(weight.dtype) if use_w else 0, int(use_w), ptr(indices),
                                  ptr(segment_ids), _index_kind(indices, "indices"), ptr(out),
                                  i64(indices.numel()), i64(num_segments), i64(D), stream_ptr(data.device)))
    return out if data.dtype == torch.float32 else out.to(data.dtype)


def segment_mean(data, weight, segment_ids, num_segments):
    """``torch.ops.recis.segment_mean`` (segment_ops.h:10-13): the normalised weights."""
    require_cuda(data, weight, segment_ids)
    segment_ids = _contig(segment_ids)
    num_segments = int(num_segments)
    n = segment_ids.numel()
    use_w = weight is not None
    w = _contig(weight).float() if use_w else torch.ones(1, dtype=torch.float32, device=data.device)
    wsum = torch.empty(num_segments, dtype=torch.float32, device=data.device)
    wnorm = torch.empty(n, dtype=torch.float32, device=data.device)
    check(lib().recis_segment_mean_weight(ptr(w), int(use_w), ptr(segment_ids),
                                          _index_kind(segment_ids, "segment_ids"), ptr(wsum), ptr(wnorm),
                                          i64(n), i64(num_segments), stream_ptr(data.device)))
    return wnorm if data.dtype == torch.float32 else wnorm.to(data.dtype)


def gen_segment_indices_by_offset(offsets):
    """``torch.ops.recis.gen_segment_indices_by_offset`` (embedding_segment_reduce.h:22)."""
    require_cuda(offsets)
    offsets = _contig(offsets)
    S = offsets.numel() - 1
    total = int(offsets[-1].item())  # the reference reads it back too (.item() at :405)
    out = torch.empty(total, dtype=offsets.dtype, device=offsets.device)
    check(lib().recis_gen_segment_indices(ptr(offsets), _index_kind(offsets, "offsets"), i64(S), ptr(out),
                                          i64(total), stream_ptr(offsets.device)))
    return out


# ------------------------------------------------------------ padded gather
def ragged_tile(batch, seq, value, offset, table):
    """``torch.ops.recis.ragged_tile`` (ragged_tile.h:9-13). Returns ``[out, batch_seq]``;
    ``batch_seq`` is the [3 * (n + 1)] bookkeeping tensor the reference's backward expects
    (cumulative batch, cumulative batch*seq, seq per feature)."""
    require_cuda(value, offset, table)
    value, offset, table = _contig(value), _contig(offset), _contig(table)
    batch, seq = [int(b) for b in batch], [int(s) for s in seq]
    D = table.shape[1]
    rows = sum(b * s for b, s in zip(batch, seq))
    out = torch.empty((rows, D), dtype=table.dtype, device=table.device)
    check(lib().recis_ragged_tile(_host_i64(batch), _host_i64(seq), i64(len(batch)), ptr(value),
                                  _index_kind(value, "value"), i64(value.numel()), ptr(offset),
                                  _index_kind(offset, "offset"), ptr(table), i64(table.shape[0]),
                                  dtype_code(table.dtype), ptr(out), i64(D), stream_ptr(table.device)))
    cum = [0, 0, 0]
    ba = bs = 0
    for b, s in zip(batch, seq):
        ba += b
        bs += b * s
        cum += [ba, bs, s]
    return [out, torch.tensor(cum, dtype=torch.int64)]


def ragged_tile_back(batch_seq, batch_info, value, offset, dy):
    """``torch.ops.recis.ragged_tile_back`` (ragged_tile.h:15-18).
    ``batch_info`` = [table_rows, n_features, batch_max, seq_min]."""
    require_cuda(value, offset, dy)
    value, offset, dy = _contig(value), _contig(offset), _contig(dy)
    cum = batch_seq.tolist()
    n = int(batch_info[1])
    batch = [cum[3 * (f + 1)] - cum[3 * f] for f in range(n)]
    seq = [cum[3 * (f + 1) + 2] for f in range(n)]
    table_rows = int(batch_info[0])
    D = dy.shape[1]
    out = torch.empty((table_rows, D), dtype=torch.float32, device=dy.device)
    check(lib().recis_ragged_tile_back(_host_i64(batch), _host_i64(seq), i64(n), ptr(value),
                                       _index_kind(value, "value"), i64(value.numel()), ptr(offset),
                                       _index_kind(offset, "offset"), ptr(dy), dtype_code(dy.dtype),
                                       ptr(out), i64(table_rows), i64(D), stream_ptr(dy.device)))
    return out if dy.dtype == torch.float32 else out.to(dy.dtype)


# ------------------------------------------------------------- feature ops
def fused_uint64_mod(inputs, mods):
    """``torch.ops.recis.fused_uint64_mod`` (fused_uint64_mod.h)."""
    inputs = [_ids64(t) for t in inputs]
    mods = mods.tolist() if torch.is_tensor(mods) else list(mods)
    if not inputs:
        return []
    # one allocation for the whole list (a view per tensor), as fused_bucketized does
    sizes = [t.numel() for t in inputs]
    outs = [o.view(t.shape) for o, t in zip(torch.split(torch.empty(sum(sizes), dtype=torch.int64,
                                                                    device=inputs[0].device), sizes), inputs)]
    check(lib().recis_fused_uint64_mod(_host_ptrs(inputs), _host_i64(sizes), _host_i64(mods), _host_ptrs(outs),
                                       i64(len(inputs)), stream_ptr(inputs[0].device)))
    return outs


def uint64_mod(inputs, num):
    """``torch.ops.recis.uint64_mod`` (uint64_mod.h)."""
    shape = inputs.shape
    return fused_uint64_mod([inputs], [int(num)])[0].view(shape)


def fused_bucketized(inputs, boundaries, mods=None):
    """``torch.ops.recis.fused_bucketized`` (fused_bucketized.h); the outputs are views of one buffer.
    ``mods`` (one positive modulus per tensor): ``fused_uint64_mod`` of the buckets in the same pass."""
    for t in list(inputs) + list(boundaries):
        if t.dtype != torch.float32:
            raise TypeError("fused_bucketized takes float32 values and boundaries")
        if not t.is_cuda:
            require_cuda(t)
    inputs = [t if (t.dim() == 1 and t.is_contiguous()) else _contig(t).view(-1) for t in inputs]
    boundaries = [b if b.is_contiguous() else _contig(b) for b in boundaries]
    if not inputs:
        return []
    sizes = [t.numel() for t in inputs]
    buf = torch.empty(sum(sizes), dtype=torch.int64, device=inputs[0].device)
    outs = list(torch.split(buf, sizes))
    if mods is not None and len(mods) != len(inputs):
        raise ValueError("fused_bucketized: %d mods for %d tensors" % (len(mods), len(inputs)))
    check(lib().recis_fused_bucketized_mod(_host_ptrs(inputs), _host_i64(sizes), _host_ptrs(boundaries),
                                           _host_i64([b.numel() for b in boundaries]),
                                           _host_i64(mods) if mods is not None else None, _host_ptrs(outs),
                                           i64(len(inputs)), stream_ptr(inputs[0].device)))
    return outs


def bucketize_op(values, boundaries):
    """``torch.ops.recis.bucketize_op`` (bucketize_op.h)."""
    if values.dtype != torch.float32:
        values, boundaries = values.float(), boundaries.float()
    return fused_bucketized([values], [boundaries.float()])[0].view(values.shape)


def fused_multi_hash(inputs, muls, primes, bucket_num):
    """``torch.ops.recis.fused_multi_hash`` (multi_hash.h): one output per (tensor, hash)."""
    inputs = [_ids64(t) for t in inputs]
    jobs_in, jobs_out, sizes, m, p, b = [], [], [], [], [], []
    for t, tm, tp, tb in zip(inputs, muls, primes, bucket_num):
        tm = tm.tolist() if torch.is_tensor(tm) else list(tm)
        tp = tp.tolist() if torch.is_tensor(tp) else list(tp)
        tb = tb.tolist() if torch.is_tensor(tb) else list(tb)
        for j in range(len(tm)):
            jobs_in.append(t)
            jobs_out.append(torch.empty_like(t))
            sizes.append(t.numel())
            m.append(tm[j])
            p.append(tp[j])
            b.append(tb[j])
    if jobs_in:
        check(lib().recis_fused_multi_hash(_host_ptrs(jobs_in), _host_i64(sizes), _host_i64(m), _host_i64(p),
                                           _host_i64(b), _host_ptrs(jobs_out), i64(len(jobs_in)),
                                           stream_ptr(inputs[0].device)))
    return jobs_out


def fused_hash(inputs, input_offsets, hash_type):
    """``torch.ops.recis.fused_hash`` (fused_hash.h): "farm" | "murmur" over int8 byte strings."""
    if hash_type not in ("farm", "murmur"):
        raise RuntimeError("Unsupported hash type: %s" % hash_type)
    require_cuda(*inputs)
    require_cuda(*input_offsets)
    inputs = [_contig(t) for t in inputs]
    offs = [_contig(o) for o in input_offsets]
    for t in inputs:
        if t.dtype not in (torch.int8, torch.uint8):
            raise TypeError("hash input must be int8 bytes")
    if not inputs:
        return []
    is64 = _index_kind(offs[0], "offsets")
    if any(_index_kind(o, "offsets") != is64 for o in offs):
        raise TypeError("offsets must share one integer dtype")
    outs = [torch.empty(o.numel() - 1, dtype=torch.int64, device=o.device) for o in offs]
    check(lib().recis_fused_hash(_host_ptrs(inputs), _host_i64([t.numel() for t in inputs]), _host_ptrs(offs),
                                 is64, _host_i64([o.numel() - 1 for o in offs]), _host_ptrs(outs),
                                 i64(len(inputs)), 0 if hash_type == "farm" else 1,
                                 stream_ptr(inputs[0].device)))
    return outs


# ------------------------------------------------------------------- id map
class IdMap:
    """GPU key -> row map with the row-index allocator (``recis_idmap_*``)."""

    def __init__(self, device=None, reserve=0):
        self.device = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
        if self.device.type != "cuda":
            raise _lib.RecisHipError("IdMap lives on the GPU; got device %s" % self.device)
        self._h = ctypes.c_void_p()
        with torch.cuda.device(self.device):
            check(lib().recis_idmap_create(i64(reserve), ctypes.byref(self._h)))

    def __del__(self):
        h = getattr(self, "_h", None)
        if h is not None and h.value:
            try:
                lib().recis_idmap_destroy(h)
            except Exception:
                pass
            self._h = None

    def lookup(self, ids):
        ids = _ids64(ids)
        out = torch.empty(ids.numel(), dtype=torch.int64, device=ids.device)
        check(lib().recis_idmap_lookup(self._h, ptr(ids), i64(ids.numel()), ptr(out), stream_ptr(ids.device)))
        return out

    def lookup_counted(self, ids_buf, n_dev):
        """Find-or-insert of the first ``n_dev[0]`` (device word) ids of ``ids_buf``: queued
        without the host knowing the count. Returns the full-length index buffer; entries
        beyond the count are not written."""
        ids_buf = _ids64(ids_buf)
        out = torch.empty_like(ids_buf)
        check(lib().recis_idmap_lookup_counted(self._h, ptr(ids_buf), i64(ids_buf.numel()), ptr(n_dev), ptr(out),
                                               stream_ptr(self.device)))
        return out

    def last_call(self):
        """Number of the call just queued on this map (for ``settle_count(..., call=)``)."""
        seq = ctypes.c_int64(0)
        check(lib().recis_idmap_last_call(self._h, ctypes.byref(seq)))
        return seq.value

    def settle_count(self, n_true, call=None):
        """Tell the map how many ids counted lookup number ``call`` (default: the last one) held."""
        if call is None:
            check(lib().recis_idmap_settle_count(self._h, i64(n_true)))
        else:
            check(lib().recis_idmap_settle_call(self._h, i64(call), i64(n_true)))

    def id_num_bound(self):
        """Upper bound of ``id_num()`` without waiting for the device."""
        v = ctypes.c_int64(0)
        check(lib().recis_idmap_bounds(self._h, ctypes.byref(v), None))
        return v.value

    def lookup_readonly(self, ids):
        ids = _ids64(ids)
        out = torch.empty(ids.numel(), dtype=torch.int64, device=ids.device)
        check(lib().recis_idmap_lookup_readonly(self._h, ptr(ids), i64(ids.numel()), ptr(out),
                                                stream_ptr(ids.device)))
        return out

    def erase(self, ids, index):
        ids, index = _ids64(ids), _ids64(index)
        if ids.numel() != index.numel():
            raise ValueError("ids and index differ in length")
        check(lib().recis_idmap_erase(self._h, ptr(ids), ptr(index), i64(ids.numel()), stream_ptr(ids.device)))

    def stats(self):
        """(live keys, allocator high-water mark, free-list length, slot capacity); synchronises."""
        vals = [ctypes.c_int64(0) for _ in range(4)]
        check(lib().recis_idmap_stats(self._h, *[ctypes.byref(v) for v in vals], stream_ptr(self.device)))
        _lib.raise_device_errors()   # the call above has waited for the stream already
        return tuple(v.value for v in vals)

    def size(self):
        return self.stats()[0]

    def id_num(self):
        return self.stats()[1]

    def snapshot(self):
        n = self.size()
        ids = torch.empty(n, dtype=torch.int64, device=self.device)
        index = torch.empty(n, dtype=torch.int64, device=self.device)
        count = ctypes.c_int64(0)
        check(lib().recis_idmap_snapshot(self._h, ptr(ids), ptr(index), i64(n), ctypes.byref(count),
                                         stream_ptr(self.device)))
        assert count.value == n, (count.value, n)
        return ids, index

    def evict_older(self, stamp_blocks, block_rows, threshold, max_out=None):
        """One-pass eviction sweep: erase every key whose row has ``stamp < threshold`` and
        free the row; returns the evicted ``(ids, index)`` (``recis_idmap_evict_older``)."""
        b0 = _check_blocks(stamp_blocks, block_rows)
        if b0.dtype not in (torch.int32, torch.int64) or _row_bytes(b0) != b0.element_size():
            raise TypeError("the stamp slot must be int32/int64 of width 1")
        n = self.size() if max_out is None else int(max_out)
        ids = torch.empty(n, dtype=torch.int64, device=self.device)
        index = torch.empty(n, dtype=torch.int64, device=self.device)
        count = ctypes.c_int64(0)
        tab = block_ptr_table(stamp_blocks)
        check(lib().recis_idmap_evict_older(self._h, ptr(tab), i64(len(stamp_blocks)), i64(block_rows),
                                            int(b0.dtype == torch.int64), i64(threshold), ptr(ids), ptr(index),
                                            i64(n), ctypes.byref(count), stream_ptr(self.device)))
        return ids[: count.value], index[: count.value]

    def clear(self):
        check(lib().recis_idmap_clear(self._h, stream_ptr(self.device)))

    def reserve(self, n_keys):
        check(lib().recis_idmap_reserve(self._h, i64(n_keys), stream_ptr(self.device)))


# ------------------------------------------------------------------ batch plan
_HOT_LEN, _HOT_CHUNK = 64, 2048  # RECIS_PLAN_HOT_LEN / RECIS_PLAN_HOT_CHUNK of the library


_RECIS_OPS = None


def recis_ops():
    """``torch.ops.recis`` of recis.so (loaded on first use)."""
    global _RECIS_OPS
    if _RECIS_OPS is None:
        from . import torch_library
        torch_library.load()
        _RECIS_OPS = torch.ops.recis
    return _RECIS_OPS


_recis_ops = recis_ops


def ids_unique_plan(ids, wait=True, need_inverse=True, need_pos=True, idmap=None, tags=None):
    """Dedup + transposed index of a batch of ids: a ``torch.classes.recis.BatchPlan``
    (``recis_unique_plan``; recis_amd/csrc/torch/plan.h). Its attributes: ``unique`` [U], ``inverse``
    int32 [N] (``unique[inverse] == ids``), ``row_start`` int32 [N + 1] and ``occ`` int32 [N] (the
    occurrences of unique id ``u`` are ``occ[row_start[u]:row_start[u + 1]]``), ``pos`` [N] (the
    position of each occurrence in ``occ``), ``hot_items`` / ``hot_cap`` / ``counts`` (device words),
    ``n``, ``serial``, ``U`` (the host copy of the unique count; a plan made with ``wait=False`` fetches
    it on first use) and ``U_bound()``; ``unique_buf`` [N] is there at once, for work that can be
    queued before the host knows ``U``. ``inverse`` and ``pos`` are filled by the plan when asked for
    (``need_inverse`` / ``need_pos``) and otherwise on first use, from the lists.

    ``ids`` may be a list of id tensors: the batch is their concatenation, tagged per tensor with
    ``tags`` as ``ids_encode`` does when given (the kernels read the tensors directly, the tagged
    batch is never written). ``wait=False`` returns without the host copy of the unique count; at
    most one such plan per stream may have its count outstanding. With ``idmap`` (an ``IdMap``) the
    unique ids are found or inserted in that map in the same pass (``recis_unique_plan_lookup``) and
    ``plan.index_buf`` holds their rows; a table does the same through ``HashtableImpl.plan_lookup``."""
    if isinstance(ids, (list, tuple)):
        jobs = list(ids)
        if tags is not None and len(tags) != len(jobs):
            raise ValueError("ids_unique_plan: %d tags for %d id tensors" % (len(tags), len(jobs)))
        if not jobs:
            jobs = [torch.empty(0, dtype=torch.int64, device="cuda")]
            tags = None
    else:
        if tags is not None:
            raise ValueError("ids_unique_plan: tags go with a list of id tensors")
        jobs = [ids]
    for t in jobs:
        if t.dtype != torch.int64:
            raise TypeError("ids must be int64, got %s" % t.dtype)
        require_cuda(t)
    handle = 0 if idmap is None else int(idmap._h.value or 0)
    return _recis_ops().unique_plan(jobs, None if tags is None else [int(t) for t in tags], handle, bool(wait),
                                    bool(need_inverse), bool(need_pos))


def csr_gather_reduce(rows, plan, src, coef=None, out=None, accumulate=False, cover=None, out_rows=None):
    """``out[u] (+)= sum_k coef[k] * rows[src[k]]`` over the list of every unique id of
    ``plan``; returns the fp32 ``[U, D]`` result. With ``out_rows`` (int32 ``[U]``, each row of
    ``out`` named at most once) the sum of unique id ``u`` goes to ``out[out_rows[u]]``."""
    require_cuda(rows, src, coef)
    rows = _contig(rows)
    D = rows.shape[1]
    if out is None:
        out = torch.empty((plan.U, D), dtype=torch.float32, device=rows.device)
        accumulate = False
    head = (ptr(rows), dtype_code(rows.dtype), i64(rows.shape[0]), ptr(src), ptr(coef),
            dtype_code(coef.dtype) if coef is not None else 0, ptr(plan.row_start),
            ptr(plan.hot_items), i64(plan.hot_cap), ptr(plan.counts), ptr(out),
            dtype_code(out.dtype), i64(plan.U), i64(D), int(bool(accumulate)),
            ptr(cover), _index_kind(cover, "offsets") if cover is not None else 0,
            i64(cover.numel() - 1 if cover is not None else 0))
    if out_rows is None:
        check(lib().recis_csr_gather_reduce(*head, stream_ptr(rows.device)))
    else:
        require_cuda(out_rows)
        if out_rows.dtype != torch.int32 or out_rows.numel() < plan.U:
            raise TypeError("out_rows must be int32 with an entry per unique id")
        check(lib().recis_csr_gather_reduce_mapped(*head, ptr(_contig(out_rows)), stream_ptr(rows.device)))
    return out


def csr_gather_reduce_parts(parts, plan, src, out=None, accumulate=False):
    """``csr_gather_reduce`` over rows that live in up to 8 separate ``[rows_f, D]`` arrays (one
    dtype): ``src`` numbers the rows of ``parts[0]``, then those of ``parts[1]``, ..."""
    require_cuda(src, *parts)
    parts = [_contig(p) for p in parts]
    D, dt, dev = parts[0].shape[1], parts[0].dtype, parts[0].device
    if any(p.dtype != dt or p.shape[1] != D for p in parts):
        raise TypeError("csr_gather_reduce_parts: the parts must share dtype and row width")
    if out is None:
        out = torch.empty((plan.U, D), dtype=torch.float32, device=dev)
        accumulate = False
    check(lib().recis_csr_gather_reduce_parts(_host_ptrs(parts), _host_i64([p.shape[0] for p in parts]),
                                              len(parts), dtype_code(dt), ptr(src), ptr(plan.row_start),
                                              ptr(plan.hot_items), i64(plan.hot_cap), ptr(plan.counts), ptr(out),
                                              i64(plan.U), i64(D), int(bool(accumulate)), stream_ptr(dev)))
    return out


def _fused_update_args(rows, plan, src, coef, cover, row_index, emb_blocks, block_size):
    require_cuda(rows, src, coef, row_index)
    rows = _contig(rows)
    b0 = _check_blocks(emb_blocks, block_size)
    D = rows.shape[1]
    if _row_bytes(b0) // b0.element_size() != D:
        raise ValueError("gradient rows have %d columns, the table's rows %d" % (D, _row_bytes(b0) // b0.element_size()))
    row_index = _ids64(row_index)
    if row_index.numel() < plan.U:
        raise ValueError("row_index holds %d rows for %d unique ids" % (row_index.numel(), plan.U))
    head = (ptr(rows), dtype_code(rows.dtype), i64(rows.shape[0]), ptr(src), ptr(coef),
            dtype_code(coef.dtype) if coef is not None else 0, ptr(plan.row_start), ptr(plan.hot_items),
            i64(plan.hot_cap), ptr(plan.counts), i64(plan.U), i64(D), ptr(cover),
            _index_kind(cover, "offsets") if cover is not None else 0,
            i64(cover.numel() - 1 if cover is not None else 0), ptr(row_index))
    return head, b0, rows


def csr_gather_reduce_adamw(rows, plan, src, coef, row_index, emb_blocks, beta1_t, beta2_t, exp_avg, exp_avg_sq, lr,
                            beta1, beta2, weight_decay, eps, block_size, cover=None):
    """``csr_gather_reduce`` + ``block_apply_adamw`` in one launch (``recis_csr_gather_reduce_adamw``): the
    gradient of unique id ``u`` (the sum over its list of ``coef * rows[src]``) is applied to table row
    ``row_index[u]`` by the lanes that summed it; the ``[U, D]`` gradient is never written. Bit for bit
    what the two calls give."""
    head, b0, rows = _fused_update_args(rows, plan, src, coef, cover, row_index, emb_blocks, block_size)
    _check_blocks(exp_avg, block_size)
    _check_blocks(exp_avg_sq, block_size)
    if len(exp_avg) != len(emb_blocks) or len(exp_avg_sq) != len(emb_blocks):
        raise ValueError("state slots must have as many blocks as the embedding slot")
    require_cuda(beta1_t, beta2_t)
    if beta1_t.dtype != beta2_t.dtype or beta1_t.dtype not in (torch.float32, torch.float64):
        raise TypeError("beta1_t / beta2_t must both be float32 or float64")
    check(lib().recis_csr_gather_reduce_adamw(
        *head, ptr(block_ptr_table(emb_blocks)), ptr(block_ptr_table(exp_avg)), ptr(block_ptr_table(exp_avg_sq)),
        i64(len(emb_blocks)), i64(block_size), i64(_pitch_bytes(emb_blocks, exp_avg, exp_avg_sq)), dtype_code(b0.dtype),
        ptr(beta1_t), ptr(beta2_t),
        int(beta1_t.dtype == torch.float64), ctypes.c_double(lr), ctypes.c_double(beta1), ctypes.c_double(beta2),
        ctypes.c_double(weight_decay), ctypes.c_double(eps), stream_ptr(rows.device)))


def csr_gather_reduce_adagrad(rows, plan, src, coef, row_index, emb_blocks, accum_blocks, lr, eps, block_size,
                              cover=None):
    """``csr_gather_reduce`` + ``block_apply_adagrad`` in one launch (``recis_csr_gather_reduce_adagrad``)."""
    head, b0, rows = _fused_update_args(rows, plan, src, coef, cover, row_index, emb_blocks, block_size)
    _check_blocks(accum_blocks, block_size)
    if len(accum_blocks) != len(emb_blocks):
        raise ValueError("state slot must have as many blocks as the embedding slot")
    check(lib().recis_csr_gather_reduce_adagrad(
        *head, ptr(block_ptr_table(emb_blocks)), ptr(block_ptr_table(accum_blocks)), i64(len(emb_blocks)),
        i64(block_size), i64(_pitch_bytes(emb_blocks, accum_blocks)), dtype_code(b0.dtype), ctypes.c_double(lr),
        ctypes.c_double(eps), stream_ptr(rows.device)))


class _CsrInput(ctypes.Structure):
    """``recis_csr_input`` of the C header."""
    _fields_ = [("rows", ctypes.c_void_p), ("rows_dtype", ctypes.c_int), ("n_rows", ctypes.c_int64),
                ("src", ctypes.c_void_p), ("coef", ctypes.c_void_p), ("coef_dtype", ctypes.c_int),
                ("part_rows", ctypes.c_void_p), ("part_counts", ctypes.c_void_p), ("n_parts", ctypes.c_int)]


def _csr_input(rows, src, coef):
    """One input ``(rows, src, coef)`` of a two-input gather-reduce as the C struct, with what it
    points into (to be kept alive over the call). ``rows``: a ``[rows, D]`` tensor, or a list of
    up to 8 such tensors laid end to end in ``src``'s numbering (the second input only)."""
    parts = None
    if isinstance(rows, (list, tuple)):
        parts = [_contig(p) for p in rows]
        require_cuda(src, coef, *parts)
        if any(p.dim() != 2 or p.dtype != parts[0].dtype or p.shape[1] != parts[0].shape[1] for p in parts):
            raise TypeError("the parts of an input must be [rows, D] tensors of one dtype and row width")
        rows = parts[0]
        tables = (_host_ptrs(parts), _host_i64([p.shape[0] for p in parts]))
    else:
        require_cuda(rows, src, coef)
        rows = _contig(rows)
        if rows.dim() != 2:
            raise ValueError("gradient rows must be [rows, D]")
        tables = (None, None)
    c = _CsrInput(rows.data_ptr() if parts is None and rows.numel() else None, dtype_code(rows.dtype),
                  rows.shape[0] if parts is None else 0, src.data_ptr() if src.numel() else None,
                  coef.data_ptr() if coef is not None and coef.numel() else None,
                  dtype_code(coef.dtype) if coef is not None else 0,
                  ctypes.cast(tables[0], ctypes.c_void_p) if parts is not None else None,
                  ctypes.cast(tables[1], ctypes.c_void_p) if parts is not None else None,
                  len(parts) if parts is not None else 0)
    return c, (rows, src, coef, parts, tables)


def _two_inputs(plan, first, second):
    if isinstance(first[0], (list, tuple)):
        if isinstance(second[0], (list, tuple)):
            raise TypeError("only one input of a two-input gather-reduce may come in parts")
        first, second = second, first   # the kernels take the parts as their second input
    a, keep_a = _csr_input(*first)
    b, keep_b = _csr_input(*second)
    D = keep_a[0].shape[1]
    if keep_b[0].shape[1] != D:
        raise ValueError("the two inputs have rows of %d and %d columns" % (D, keep_b[0].shape[1]))
    head = (ctypes.byref(a), ctypes.byref(b), ptr(plan.row_start), ptr(plan.hot_items), i64(plan.hot_cap),
            ptr(plan.counts))
    return head, D, keep_a[0].device, (a, b, keep_a, keep_b)


def csr_gather_reduce2(plan, first, second, out=None, accumulate=False):
    """``csr_gather_reduce`` with two inputs ``(rows, src, coef)`` over the lists of ``plan``
    (``recis_csr_gather_reduce2``): ``out[u] (+)= sum_k coef1[k] * rows1[src1[k]] + coef2[k] *
    rows2[src2[k]]``. Each input float32 or a half type (two half inputs of one type); one of them may
    come as a list of arrays laid end to end in its ``src``'s numbering."""
    head, D, dev, keep = _two_inputs(plan, first, second)
    if out is None:
        out = torch.empty((plan.U, D), dtype=torch.float32, device=dev)
        accumulate = False
    if out.dtype != torch.float32:
        raise TypeError("csr_gather_reduce2 writes float32 rows")
    check(lib().recis_csr_gather_reduce2(*head, ptr(out), i64(plan.U), i64(D), int(bool(accumulate)), stream_ptr(dev)))
    return out


def _two_inputs_table(plan, first, second, row_index, emb_blocks, block_size):
    head, D, dev, keep = _two_inputs(plan, first, second)
    require_cuda(row_index)
    b0 = _check_blocks(emb_blocks, block_size)
    if _row_bytes(b0) // b0.element_size() != D:
        raise ValueError("gradient rows have %d columns, the table's rows %d" % (D, _row_bytes(b0) // b0.element_size()))
    row_index = _ids64(row_index)
    if row_index.numel() < plan.U:
        raise ValueError("row_index holds %d rows for %d unique ids" % (row_index.numel(), plan.U))
    return head + (i64(plan.U), i64(D), ptr(row_index)), b0, dev, (keep, row_index)


def csr_gather_reduce2_adamw(plan, first, second, row_index, emb_blocks, beta1_t, beta2_t, exp_avg, exp_avg_sq, lr,
                             beta1, beta2, weight_decay, eps, block_size):
    """Two-input gather-reduce ending in the Adam-family row update (``recis_csr_gather_reduce2_adamw``)."""
    head, b0, dev, keep = _two_inputs_table(plan, first, second, row_index, emb_blocks, block_size)
    _check_blocks(exp_avg, block_size)
    _check_blocks(exp_avg_sq, block_size)
    if len(exp_avg) != len(emb_blocks) or len(exp_avg_sq) != len(emb_blocks):
        raise ValueError("state slots must have as many blocks as the embedding slot")
    require_cuda(beta1_t, beta2_t)
    if beta1_t.dtype != beta2_t.dtype or beta1_t.dtype not in (torch.float32, torch.float64):
        raise TypeError("beta1_t / beta2_t must both be float32 or float64")
    check(lib().recis_csr_gather_reduce2_adamw(
        *head, ptr(block_ptr_table(emb_blocks)), ptr(block_ptr_table(exp_avg)), ptr(block_ptr_table(exp_avg_sq)),
        i64(len(emb_blocks)), i64(block_size), i64(_pitch_bytes(emb_blocks, exp_avg, exp_avg_sq)), dtype_code(b0.dtype),
        ptr(beta1_t), ptr(beta2_t),
        int(beta1_t.dtype == torch.float64), ctypes.c_double(lr), ctypes.c_double(beta1), ctypes.c_double(beta2),
        ctypes.c_double(weight_decay), ctypes.c_double(eps), stream_ptr(dev)))


def csr_gather_reduce2_adagrad(plan, first, second, row_index, emb_blocks, accum_blocks, lr, eps, block_size):
    """Two-input gather-reduce ending in the Adagrad row update (``recis_csr_gather_reduce2_adagrad``)."""
    head, b0, dev, keep = _two_inputs_table(plan, first, second, row_index, emb_blocks, block_size)
    _check_blocks(accum_blocks, block_size)
    if len(accum_blocks) != len(emb_blocks):
        raise ValueError("state slot must have as many blocks as the embedding slot")
    check(lib().recis_csr_gather_reduce2_adagrad(
        *head, ptr(block_ptr_table(emb_blocks)), ptr(block_ptr_table(accum_blocks)), i64(len(emb_blocks)),
        i64(block_size), i64(_pitch_bytes(emb_blocks, accum_blocks)), dtype_code(b0.dtype), ctypes.c_double(lr),
        ctypes.c_double(eps), stream_ptr(dev)))


def plan_expand_rows(plan, n_out, rows=None, blocks=None, block_size=0, row_index=None, weight=None, out_dtype=None,
                     stamp=None):
    """``out[i] = weight[i] * row(unique id of occurrence i)`` for the ``n_out`` occurrences of
    ``plan``: every unique row is read once and written to all its occurrences. Rows come from
    ``rows`` ``[U, D]`` or from ``blocks`` (row u = row ``row_index[u]``, negative = zeros).
    ``stamp`` = (blocks of an int64 slot of the same table, a one-element int64 device tensor):
    every row that is read also gets that value written into the slot (the step filter's stamp)."""
    if blocks is not None:
        require_cuda(row_index, weight)
        table, dt, D, dev = block_ptr_table(blocks), blocks[0].dtype, blocks[0][0].numel(), blocks[0].device
        n_blocks, rows_arg = len(blocks), None
    else:
        require_cuda(rows, weight)
        rows = _contig(rows)
        table, dt, D, dev, n_blocks, rows_arg = None, rows.dtype, rows.shape[1], rows.device, 0, rows
    stamp_table = stamp_value = None
    if stamp is not None:
        stamp_blocks, stamp_value = stamp
        if blocks is None:
            raise ValueError("rows are stamped in a block list only")
        if (len(stamp_blocks) != n_blocks or stamp_blocks[0].dtype != torch.int64
                or stamp_blocks[0].numel() != blocks[0].shape[0]):
            raise ValueError("the stamp slot must be an int64 slot with the blocks of the embedding's table")
        if stamp_value.dtype != torch.int64 or stamp_value.numel() != 1:
            raise TypeError("the stamp value must be a one-element int64 tensor")
        require_cuda(stamp_value)
        stamp_table = block_ptr_table(stamp_blocks)
    out = torch.empty((n_out, D), dtype=out_dtype or dt, device=dev)
    weight = _contig(weight)
    check(lib().recis_csr_expand_rows_stamped(ptr(rows_arg), ptr(table), i64(n_blocks), i64(block_size),
                                              i64(_pitch_bytes(blocks) if blocks is not None else 0), ptr(row_index),
                                              dtype_code(dt), ptr(weight),
                                              dtype_code(weight.dtype) if weight is not None else 0,
                                              ptr(plan.row_start), ptr(plan.occ), ptr(plan.hot_items), i64(plan.hot_cap),
                                              ptr(plan.counts), ptr(out), dtype_code(out.dtype), i64(plan.U_bound()),
                                              i64(n_out), i64(D), ptr(stamp_table), ptr(stamp_value), stream_ptr(dev)))
    return out


def segment_reduce_backward_plan(grad_output, weight, offsets, plan, mode, out=None, accumulate=False):
    """Backward of the pooling for duplicated ids without atomics on row data: the same
    result as ``segment_reduce_backward(grad, weight, plan.inverse, offsets, plan.U, mode)``
    (sum | mean | tile), computed as a gather-reduce over ``plan``'s occurrence lists."""
    if mode not in ("sum", "mean", "tile"):
        raise ValueError("Invalid mode for the planned backward: %s" % mode)
    grad_output, weight, offsets = _contig(grad_output), _contig(weight), _contig(offsets)
    if mode == "tile":
        src = plan.occ
        coef = None if weight is None else gather(plan.occ, weight.view(-1, 1)).view(-1)
        # occurrences no segment covers are skipped by the kernel (no host read of the offsets)
        return csr_gather_reduce(grad_output, plan, src, coef, out=out, accumulate=accumulate,
                                 cover=offsets if offsets.numel() else None)
    src, coef = plan.src_coef_for_pool(offsets, weight, mode == "mean")
    return csr_gather_reduce(grad_output, plan, src, coef, out=out, accumulate=accumulate)


# ------------------------------------------------------------ sequence truncation


def _host_list(x, n, name):
    """keep_lengths / drop_sides / pad_sides as a host list of n entries (a device tensor is read
    back: pass host values where the step must not wait)."""
    v = x.reshape(-1).tolist() if torch.is_tensor(x) else list(x)
    if len(v) != n:
        raise RuntimeError("%s.numel() = %d but is expected equals fea_num = %d" % (name, len(v), n))
    return v


def _host_u8(values):
    return (ctypes.c_uint8 * len(values))(*[1 if v else 0 for v in values])


def _ragged_cutoff(values, outer, inner, keep_lengths, drop_sides, pad_sides):
    n = len(values)
    if len(outer) != n or (inner is not None and len(inner) != n):
        raise RuntimeError("offsets.numel() = %d but is expected equals fea_num = %d" % (len(outer), n))
    require_cuda(*values)
    require_cuda(*outer)
    values = [_contig(v).reshape(-1) for v in values]
    outer = [_contig(o) for o in outer]
    if any(v.dtype != values[0].dtype for v in values):
        raise RuntimeError("fused_ragged_cutoff: each value should be the same type")
    is64 = _index_kind(outer[0], "offsets")
    every = outer + ([_contig(o) for o in inner] if inner is not None else [])
    if any(_index_kind(o, "offsets") != is64 for o in every):
        raise RuntimeError("fused_ragged_cutoff: each offsets should be torch.int32 or torch.int64")
    if inner is not None:
        require_cuda(*inner)
        inner = every[n:]
    keep = _host_list(keep_lengths, n, "keep_lengths")
    drop = _host_list(drop_sides, n, "drop_sides")
    pad = _host_list(pad_sides, n, "pad_sides")
    dev, odt = values[0].device, outer[0].dtype
    rows = [o.numel() - 1 for o in outer]
    out_rows = [r * k for r, k in zip(rows, keep)] if inner is not None else rows
    # one allocation per kind of output, one view per tensor (as the reference slices its buffers)
    off_buf = torch.empty(sum(out_rows) + n, dtype=odt, device=dev)
    src_buf = torch.empty(max(sum(out_rows), 1), dtype=torch.int64, device=dev)
    cnt_buf = torch.empty(2 * sum(rows), dtype=odt, device=dev)
    totals = torch.empty(n, dtype=torch.int64, device=dev)
    out_off, src, drop_nums, pad_nums, out_outer = [], [], [], [], []
    a = b = 0
    for t in range(n):
        out_off.append(off_buf[a + t: a + t + out_rows[t] + 1])
        src.append(src_buf[a: a + out_rows[t]] if out_rows[t] else src_buf[:0])
        drop_nums.append(cnt_buf[b: b + rows[t]])
        pad_nums.append(cnt_buf[sum(rows) + b: sum(rows) + b + rows[t]])
        a += out_rows[t]
        b += rows[t]
    if inner is not None:
        outer_buf = torch.empty(sum(rows) + n, dtype=odt, device=dev)
        b = 0
        for t in range(n):
            out_outer.append(outer_buf[b + t: b + t + rows[t] + 1])
            b += rows[t]
    sp = stream_ptr(dev)

    def ptrs_or_dummy(ts):   # an empty view has no address: any valid one will do, it is never used
        return (ctypes.c_void_p * len(ts))(*[t.data_ptr() if t.numel() else src_buf.data_ptr() for t in ts])

    check(lib().recis_ragged_cutoff_rows(
        _host_ptrs(outer), _host_ptrs(inner) if inner is not None else None, is64, _host_i64(rows),
        _host_i64([o.numel() - 1 for o in inner]) if inner is not None else None,
        _host_i64([v.numel() for v in values]), _host_i64(keep), _host_u8(drop), _host_u8(pad), i64(n),
        _host_ptrs(out_off), _host_ptrs(out_outer) if inner is not None else None, ptrs_or_dummy(drop_nums),
        ptrs_or_dummy(pad_nums), ptrs_or_dummy(src), ptr(totals), sp))
    total_host = totals.tolist()   # the one wait of this op: the outputs are sized by it
    val_buf = torch.empty(sum(total_host), dtype=values[0].dtype, device=dev)
    out_vals, a = [], 0
    for t in range(n):
        out_vals.append(val_buf[a: a + total_host[t]])
        a += total_host[t]
    check(lib().recis_ragged_cutoff_copy(
        ptrs_or_dummy(values), values[0].element_size(), _host_ptrs(out_off), is64, _host_i64(out_rows),
        ptrs_or_dummy(src), _host_i64(total_host), ptrs_or_dummy(out_vals), i64(n), sp))
    return out_vals, out_off, drop_nums, pad_nums, out_outer


def fused_ragged_cutoff(values, offsets, keep_lengths, drop_sides, pad_sides):
    """``torch.ops.recis.fused_ragged_cutoff`` (fused_ragged_cutoff.cc:10-140): every row of every
    2-D ragged tensor cut to at most keep_lengths[t] elements (the last ones when drop_sides[t]).
    Returns (values, offsets, drop_nums, pad_nums, drop_sides, pad_sides)."""
    if not values:
        return [], [], [], [], drop_sides, pad_sides
    vals, offs, drop_nums, pad_nums, _ = _ragged_cutoff(values, offsets, None, keep_lengths, drop_sides, pad_sides)
    return vals, offs, drop_nums, pad_nums, drop_sides, pad_sides


def fused_ragged_cutoff_3D(values, outer_offsets, inner_offsets, keep_lengths, drop_sides, pad_sides):
    """``torch.ops.recis.fused_ragged_cutoff_3D`` (fused_ragged_cutoff.cc:143-287): every sequence
    of every 3-D ragged tensor brought to exactly keep_lengths[t] inner rows, by dropping inner
    rows or adding empty ones. Returns (values, outer_offsets, inner_offsets)."""
    if not values:
        return [], [], []
    vals, inner, _, _, outer = _ragged_cutoff(values, outer_offsets, inner_offsets, keep_lengths, drop_sides,
                                               pad_sides)
    return vals, outer, inner


# ------------------------------------------------------------ dense <-> ragged

_SEQ_KIND = {torch.float32: 0, torch.float64: 1, torch.int32: 2, torch.int64: 3}


def _scalar_bytes(value, dtype):
    return torch.tensor([value], dtype=dtype).view(torch.uint8).numpy().tobytes()


def ragged_to_dense(values, offsets, default_value=0, widths=None):
    """``torch.ops.recis.ragged_to_dense`` (ragged_to_dense.cc:47-100): dense
    ``[batch, max width of every ragged level]`` with ``default_value`` outside the rows.
    ``widths`` (one per level) skips the read-back of the longest rows."""
    require_cuda(values, *offsets)
    if values.dim() != 1:
        raise RuntimeError("values must dim == 1")
    values = _contig(values)
    offsets = [_contig(o) for o in offsets]
    is64 = _index_kind(offsets[0], "offsets")
    if any(_index_kind(o, "offsets") != is64 for o in offsets):
        raise RuntimeError("ragged_to_dense: each offsets should be torch.int32 or torch.int64")
    if widths is None:
        widths = [int((o[1:] - o[:-1]).max()) if o.numel() > 1 else 0 for o in offsets]
    shape = [offsets[0].numel() - 1] + [int(w) for w in widths]
    out = torch.empty(shape, dtype=values.dtype, device=values.device)
    fill = _scalar_bytes(default_value, values.dtype)
    check(lib().recis_ragged_to_dense(ptr(values), values.element_size(), i64(values.numel()), _host_ptrs(offsets),
                                      _host_i64([o.numel() for o in offsets]), is64, _host_i64(shape[1:]),
                                      len(offsets), ctypes.c_char_p(fill), ptr(out), stream_ptr(values.device)))
    return out


def dense_to_ragged(data, check_invalid=True, invalid_value=0):
    """``torch.ops.recis.dense_to_ragged`` (dense_to_ragged.cc:56-76): (values, int32 offsets) of a
    2-D tensor; with ``check_invalid`` the trailing run of ``invalid_value`` of every row is dropped."""
    if data.dim() != 2:
        raise RuntimeError("Input must be a 2D tensor")
    require_cuda(data)
    rows, cols = data.shape
    if not check_invalid:
        return data.reshape(-1), torch.arange(0, rows * cols + 1, max(cols, 1), dtype=torch.int32,
                                              device=data.device)[: rows + 1]
    if data.dtype not in _SEQ_KIND:
        raise TypeError("dense_to_ragged: float32, float64, int32 or int64 data, got %s" % data.dtype)
    data = _contig(data)
    if torch.is_tensor(invalid_value):
        invalid_value = invalid_value.reshape(-1)[0].item()
    offsets = torch.empty(rows + 1, dtype=torch.int32, device=data.device)
    src = torch.empty(max(rows, 1), dtype=torch.int64, device=data.device)
    total = torch.empty(1, dtype=torch.int64, device=data.device)
    sp = stream_ptr(data.device)
    check(lib().recis_dense_to_ragged_rows(ptr(data), _SEQ_KIND[data.dtype], i64(rows), i64(cols),
                                           ctypes.c_char_p(_scalar_bytes(invalid_value, data.dtype)), ptr(offsets),
                                           ptr(src), ptr(total), sp))
    n = int(total.item())
    values = torch.empty(n, dtype=data.dtype, device=data.device)
    if n:
        check(lib().recis_ragged_cutoff_copy(_host_ptrs([data]), data.element_size(), _host_ptrs([offsets]), 0,
                                             _host_i64([rows]), _host_ptrs([src]), _host_i64([n]),
                                             _host_ptrs([values]), i64(1), sp))
    return values, offsets


def feature_cross_ragged(x_value, x_offsets, x_weight, y_value, y_offsets, y_weight):
    """``torch.ops.recis.feature_cross_ragged`` (feature_cross_ragged.cc:24-98): per segment the
    cross of the distinct ids of x and y. Returns (values, offsets, weights); an empty weight
    tensor (or None) means all ones."""
    require_cuda(x_value, x_offsets, y_value, y_offsets)
    if x_value.dtype != torch.int64 or y_value.dtype != torch.int64:
        raise RuntimeError("feature_cross_ragged: ids for x and y must be torch.int64")
    is64 = _index_kind(x_offsets, "x_offsets")
    if _index_kind(y_offsets, "y_offsets") != is64:
        raise RuntimeError("feature_cross_ragged: each offset should be torch.int32 or torch.int64")
    xv, yv, xo, yo = _contig(x_value), _contig(y_value), _contig(x_offsets), _contig(y_offsets)
    dev = xv.device

    def weight(w):
        return None if w is None or w.numel() == 0 else _contig(w)

    xw, yw = weight(x_weight), weight(y_weight)
    wdt = (xw if xw is not None else yw if yw is not None else torch.empty(0)).dtype
    if wdt not in (torch.float32, torch.float64) or any(w is not None and w.dtype != wdt for w in (xw, yw)):
        raise TypeError("feature_cross_ragged: weights must share float32 or float64")
    n_seg = min(xo.numel(), yo.numel()) - 1
    nx, ny = xv.numel(), yv.numel()
    x_rank = torch.empty(max(nx, 1), dtype=torch.int32, device=dev)
    y_rank = torch.empty(max(ny, 1), dtype=torch.int32, device=dev)
    y_count = torch.empty(max(n_seg, 1), dtype=torch.int32, device=dev)
    out_off = torch.empty(n_seg + 1, dtype=xo.dtype, device=dev)
    total = torch.empty(1, dtype=torch.int64, device=dev)
    sp = stream_ptr(dev)
    check(lib().recis_feature_cross_rows(ptr(xv), ptr(xo), i64(nx), ptr(yv), ptr(yo), i64(ny), is64, i64(n_seg),
                                         ptr(x_rank), ptr(y_rank), ptr(y_count), ptr(out_off), ptr(total), sp))
    n = int(total.item())
    out_val = torch.empty(n, dtype=torch.int64, device=dev)
    out_w = torch.empty(n, dtype=wdt, device=dev)
    check(lib().recis_feature_cross_emit(ptr(xv), ptr(xo), ptr(xw), i64(nx), ptr(yv), ptr(yo), ptr(yw), i64(ny), is64,
                                         int(wdt == torch.float64), i64(n_seg), ptr(x_rank), ptr(y_rank),
                                         ptr(y_count), ptr(out_off), i64(n), ptr(out_val), ptr(out_w), sp))
    return out_val, out_off, out_w


def calc_ragged_index(drop_num, pad_num, drop_side, pad_side, offset, topk_index, indicator):
    """``torch.ops.recis.calc_ragged_index`` (calc_ragged_index.cc:93-131): indices into the
    values of a ragged tensor selected by ``topk_index`` [rows, cols] (positions counted after a
    left truncation by ``drop_num``), and their offsets per row. Only drop left / pad right is
    implemented, as in the reference. Returns (value_index, offsets) on the device of the inputs."""
    require_cuda(drop_num, offset, topk_index, indicator)
    for t, what in ((drop_side, "drop_side"), (pad_side, "pad_side")):
        if not torch.is_tensor(t) or t.dtype != torch.bool:
            raise RuntimeError("drop_side and pad_side must be bool")
    drop_left, pad_left = bool(drop_side.item()), bool(pad_side.item())
    if not drop_left or pad_left:
        raise RuntimeError("drop %s, pad %s is not supported yet" % ("left" if drop_left else "right",
                                                                    "left" if pad_left else "right"))
    if topk_index.dim() != 2:
        raise RuntimeError("calc_ragged_index: topk_index must be [rows, cols]")
    rows, cols = topk_index.shape
    if indicator.numel() != rows:
        raise RuntimeError("indicator==row_num;indicator.numel(): %d; row_num: %d" % (indicator.numel(), rows))
    src_rows = offset.numel() - 1
    if drop_num.numel() < src_rows:
        raise RuntimeError("calc_ragged_index: drop_num is shorter than the rows of offset")
    d, o, t, ind = _contig(drop_num), _contig(offset), _contig(topk_index), _contig(indicator)
    kinds = [_index_kind(x, n) for x, n in ((d, "drop_num"), (o, "offset"), (t, "topk_index"), (ind, "indicator"))]
    dev = t.device
    out_index = torch.empty(max(rows * cols, 1), dtype=t.dtype, device=dev)
    out_off = torch.empty(rows + 1, dtype=o.dtype, device=dev)
    total = torch.empty(1, dtype=torch.int64, device=dev)
    check(lib().recis_ragged_topk_index(ptr(d), kinds[0], ptr(o), kinds[1], i64(src_rows), ptr(t), kinds[2],
                                        ptr(ind), kinds[3], i64(rows), i64(cols), ptr(out_index), ptr(out_off),
                                        ptr(total), stream_ptr(dev)))
    return out_index[: int(total.item())], out_off

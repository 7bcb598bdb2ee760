"""CPU oracle for the sparse-embedding hot path: TEST INFRASTRUCTURE ONLY.

numpy-facing wrappers over ``recis_oracle.c`` (built into
``oracle/_build/liboracle.so`` by ``oracle/Makefile``). Only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import this package; the product (``recis_amd``) never does.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "_build", "liboracle.so")
_lib = None

c_i64 = ctypes.c_int64
c_f32p = ctypes.POINTER(ctypes.c_float)
c_void = ctypes.c_void_p


def build():
    """Compile the oracle with gcc (always recompiles)."""
    subprocess.run(["make", "-C", _HERE, "-B", "-s"], check=True)
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.oracle_idmap_create.restype = c_void
        _lib.oracle_idmap_create.argtypes = [c_i64]
        for name in ("oracle_idmap_size", "oracle_idmap_id_num", "oracle_idmap_free_size",
                     "oracle_idmap_snapshot", "oracle_ids_partition", "oracle_merge_offsets"):
            getattr(_lib, name).restype = c_i64
        _lib.oracle_murmur64.restype = ctypes.c_uint64
        _lib.oracle_farmhash64.restype = ctypes.c_uint64
        _lib.oracle_cal_alpha_f64.restype = ctypes.c_double
        _lib.oracle_cal_alpha_f32.restype = ctypes.c_float
    return _lib


def _p(a):
    """Pointer to a C-contiguous numpy array (None -> NULL)."""
    if a is None:
        return None
    assert a.flags["C_CONTIGUOUS"], "oracle needs contiguous arrays"
    return ctypes.c_void_p(a.ctypes.data)


def _f32(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.float32)


def _i64(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.int64)


MODES = {"sum": 0, "mean": 1, "tile": 2}

# ------------------------------------------------------------------ pooling


def segment_reduce_forward(emb, weight, rev, offsets, mode):
    emb, weight, rev, offsets = _f32(emb), _f32(weight), _i64(rev), _i64(offsets)
    U, D = emb.shape
    S = offsets.shape[0] - 1
    B = rev.shape[0] if rev is not None else U
    out = np.empty(((B if mode == "tile" else S), D), np.float32)
    lib().oracle_segment_reduce_forward(_p(emb), _p(weight), _p(rev), _p(offsets), _p(out),
                                        c_i64(B), c_i64(U), c_i64(S), c_i64(D), MODES[mode])
    return out


def segment_reduce_backward(grad, weight, rev, offsets, unique_size, mode):
    grad, weight, rev, offsets = _f32(grad), _f32(weight), _i64(rev), _i64(offsets)
    D = grad.shape[1]
    S = offsets.shape[0] - 1
    B = rev.shape[0] if rev is not None else unique_size
    out = np.empty((unique_size, D), np.float32)
    lib().oracle_segment_reduce_backward(_p(grad), _p(weight), _p(rev), _p(offsets), _p(out),
                                         c_i64(B), c_i64(unique_size), c_i64(S), c_i64(D),
                                         MODES[mode])
    return out


def segment_reduce_forward_f64(emb, weight, rev, offsets, mean):
    """(sum in double, sum of |terms| in double) for error-bound checks."""
    emb, weight, rev, offsets = _f32(emb), _f32(weight), _i64(rev), _i64(offsets)
    D = emb.shape[1]
    S = offsets.shape[0] - 1
    out = np.empty((S, D), np.float64)
    out_abs = np.empty((S, D), np.float64)
    lib().oracle_segment_reduce_forward_f64(_p(emb), _p(weight), _p(rev), _p(offsets), _p(out),
                                            _p(out_abs), c_i64(S), c_i64(D), int(bool(mean)))
    return out, out_abs


def segment_max_forward(emb, rev, offsets):
    emb, rev, offsets = _f32(emb), _i64(rev), _i64(offsets)
    D = emb.shape[1]
    S = offsets.shape[0] - 1
    out = np.empty((S, D), np.float32)
    arg = np.empty((S, D), np.int32)
    lib().oracle_segment_max_forward(_p(emb), _p(rev), _p(offsets), _p(out), _p(arg),
                                     c_i64(S), c_i64(D))
    return out, arg


def segment_max_backward(grad, argmax, rev, unique_size):
    grad, rev = _f32(grad), _i64(rev)
    argmax = np.ascontiguousarray(argmax, dtype=np.int32)
    S, D = grad.shape
    out = np.empty((unique_size, D), np.float32)
    lib().oracle_segment_max_backward(_p(grad), _p(argmax), _p(rev), _p(out),
                                      c_i64(unique_size), c_i64(S), c_i64(D))
    return out


def merge_offsets(offsets_list, max_value):
    arrs = [_i64(o) for o in offsets_list]
    n = len(arrs)
    ptrs = (ctypes.c_void_p * n)(*[a.ctypes.data for a in arrs])
    sizes = np.array([a.shape[0] for a in arrs], np.int64)
    mv = _i64(max_value)
    out = np.empty(int(sizes.sum()) - (n - 1), np.int64)
    k = lib().oracle_merge_offsets(ptrs, _p(sizes), _p(mv), c_i64(n), _p(out))
    assert k == out.shape[0]
    return out


def gen_segment_indices(offsets):
    offsets = _i64(offsets)
    S = offsets.shape[0] - 1
    out = np.empty(int(offsets[-1]), np.int64)
    lib().oracle_gen_segment_indices(_p(offsets), c_i64(S), _p(out))
    return out


def segment_sum(data, weight, indices, seg_ids, num_segments):
    data, indices, seg_ids = _f32(data), _i64(indices), _i64(seg_ids)
    use_w = weight is not None
    weight = _f32(weight) if use_w else np.ones(1, np.float32)
    D = data.shape[1]
    out = np.empty((num_segments, D), np.float32)
    lib().oracle_segment_sum(_p(data), _p(weight), int(use_w), _p(indices), _p(seg_ids), _p(out),
                             c_i64(indices.shape[0]), c_i64(num_segments), c_i64(D))
    return out


def segment_mean_weight(weight, seg_ids, num_segments):
    """Normalised weights of the sparse-mode mean combiner."""
    seg_ids = _i64(seg_ids)
    use_w = weight is not None
    weight = _f32(weight) if use_w else np.ones(1, np.float32)
    n = seg_ids.shape[0]
    wsum = np.empty(num_segments, np.float32)
    wnorm = np.empty(n, np.float32)
    lib().oracle_segment_mean_weight(_p(weight), int(use_w), _p(seg_ids), _p(wsum), _p(wnorm),
                                     c_i64(n), c_i64(num_segments))
    return wnorm


def ragged_tile(batch, seq, value, offset, table):
    batch, seq, value, offset, table = _i64(batch), _i64(seq), _i64(value), _i64(offset), _f32(table)
    D = table.shape[1]
    rows = int((batch * seq).sum())
    out = np.empty((rows, D), np.float32)
    lib().oracle_ragged_tile(_p(batch), _p(seq), c_i64(batch.shape[0]), _p(value), _p(offset),
                             _p(table), _p(out), c_i64(D))
    return out


def ragged_tile_back(batch, seq, value, offset, dy, table_rows):
    batch, seq, value, offset, dy = _i64(batch), _i64(seq), _i64(value), _i64(offset), _f32(dy)
    D = dy.shape[1]
    out = np.empty((table_rows, D), np.float32)
    lib().oracle_ragged_tile_back(_p(batch), _p(seq), c_i64(batch.shape[0]), _p(value), _p(offset),
                                  _p(dy), _p(out), c_i64(table_rows), c_i64(D))
    return out


# ---------------------------------------------------------------- allocator


def generate_ids(n, free_list, free_count, cur_count):
    free_list = _i64(free_list)
    out = np.empty(n, np.int64)
    lib().oracle_generate_ids(c_i64(n), _p(free_list), c_i64(free_count), c_i64(cur_count), _p(out))
    return out


def mask_key_index(keys, mask, cumsum, out_size):
    keys, cumsum = _i64(keys), _i64(cumsum)
    mask = np.ascontiguousarray(mask, dtype=np.uint8)
    ok = np.empty(out_size, np.int64)
    oi = np.empty(out_size, np.int64)
    lib().oracle_mask_key_index(_p(keys), _p(mask), _p(cumsum), c_i64(keys.shape[0]), _p(ok), _p(oi))
    return ok, oi


def scatter_ids_with_mask(out_ids, in_ids, mask_index):
    out_ids = _i64(out_ids).copy()
    in_ids, mask_index = _i64(in_ids), _i64(mask_index)
    lib().oracle_scatter_ids_with_mask(_p(out_ids), _p(in_ids), _p(mask_index), c_i64(in_ids.shape[0]))
    return out_ids


class IdMap:
    """CPU key -> row map with the reference allocator's assignment order."""

    def __init__(self, reserve=0):
        self._h = c_void(lib().oracle_idmap_create(c_i64(reserve)))

    def __del__(self):
        if getattr(self, "_h", None) and _lib is not None:
            _lib.oracle_idmap_destroy(self._h)
            self._h = None

    def lookup(self, ids):
        ids = _i64(ids)
        out = np.empty(ids.shape[0], np.int64)
        lib().oracle_idmap_lookup(self._h, _p(ids), c_i64(ids.shape[0]), _p(out))
        return out

    def lookup_readonly(self, ids):
        ids = _i64(ids)
        out = np.empty(ids.shape[0], np.int64)
        lib().oracle_idmap_lookup_readonly(self._h, _p(ids), c_i64(ids.shape[0]), _p(out))
        return out

    def delete(self, ids, index):
        ids, index = _i64(ids), _i64(index)
        lib().oracle_idmap_delete(self._h, _p(ids), _p(index), c_i64(ids.shape[0]))

    def size(self):
        return int(lib().oracle_idmap_size(self._h))

    def id_num(self):
        return int(lib().oracle_idmap_id_num(self._h))

    def free_size(self):
        return int(lib().oracle_idmap_free_size(self._h))

    def snapshot(self):
        n = self.size()
        ids = np.empty(n, np.int64)
        index = np.empty(n, np.int64)
        k = lib().oracle_idmap_snapshot(self._h, _p(ids), _p(index))
        assert k == n
        return ids, index

    def clear(self):
        lib().oracle_idmap_clear(self._h)


# ---------------------------------------------------------------- row blocks


def _block_ptrs(blocks):
    return (ctypes.c_void_p * len(blocks))(*[b.ctypes.data for b in blocks])


def gather(ids, emb):
    ids = _i64(ids)
    emb = np.ascontiguousarray(emb)
    out = np.empty((ids.shape[0], emb.shape[1]), emb.dtype)
    lib().oracle_gather(_p(ids), c_i64(ids.shape[0]), _p(emb), _p(out), c_i64(emb.shape[1]),
                        c_i64(emb.itemsize))
    return out


def block_gather(ids, blocks, block_size, default_key=-1, readonly=False):
    ids = _i64(ids)
    D = blocks[0].shape[1]
    out = np.empty((ids.shape[0], D), blocks[0].dtype)
    lib().oracle_block_gather(_p(ids), c_i64(ids.shape[0]), _block_ptrs(blocks), c_i64(block_size),
                              c_i64(default_key), int(readonly), _p(out), c_i64(D),
                              c_i64(blocks[0].itemsize))
    return out


def block_insert(ids, emb, blocks, block_size, mask=None):
    """In place on ``blocks``; emb with one row is broadcast."""
    ids = _i64(ids)
    emb = np.ascontiguousarray(emb, dtype=blocks[0].dtype)
    D = blocks[0].shape[1]
    m = None if mask is None else np.ascontiguousarray(mask, dtype=np.uint8)
    lib().oracle_block_insert(_p(ids), c_i64(ids.shape[0]), _p(emb),
                              int(emb.shape[0] == 1 and ids.shape[0] != 1), _p(m),
                              _block_ptrs(blocks), c_i64(block_size), c_i64(D),
                              c_i64(blocks[0].itemsize))


def block_filter(ids, blocks, block_size, threshold):
    ids = _i64(ids)
    out = np.empty(ids.shape[0], np.uint8)
    lib().oracle_block_filter(_p(ids), c_i64(ids.shape[0]), _block_ptrs(blocks), c_i64(block_size),
                              c_i64(threshold), int(blocks[0].dtype == np.int64), _p(out))
    return out.astype(bool)


# ---------------------------------------------------------------- optimizers


def cal_alpha(b1_t, b2_t, lr, beta1, beta2):
    """Advances the running beta powers in place (1-element arrays) and returns alpha."""
    if b1_t.dtype == np.float64:
        return float(lib().oracle_cal_alpha_f64(_p(b1_t), _p(b2_t), ctypes.c_double(lr),
                                                ctypes.c_double(beta1), ctypes.c_double(beta2)))
    assert b1_t.dtype == np.float32
    return float(lib().oracle_cal_alpha_f32(_p(b1_t), _p(b2_t), ctypes.c_double(lr),
                                            ctypes.c_double(beta1), ctypes.c_double(beta2)))


def block_apply_adamw(index, grad, emb_blocks, b1_t, b2_t, exp_avg, exp_avg_sq, lr, beta1, beta2,
                      weight_decay, eps, block_size):
    """The op as registered: advances b1_t/b2_t, then updates the rows in place.
    ``weight_decay`` is the multiplicative decay factor applied to the row."""
    index, grad = _i64(index), _f32(grad)
    alpha = cal_alpha(b1_t, b2_t, lr, beta1, beta2)
    D = emb_blocks[0].shape[1]
    lib().oracle_block_apply_adamw(_p(index), c_i64(index.shape[0]), _p(grad),
                                   _block_ptrs(emb_blocks), _block_ptrs(exp_avg),
                                   _block_ptrs(exp_avg_sq), ctypes.c_double(alpha),
                                   ctypes.c_double(beta1), ctypes.c_double(beta2),
                                   ctypes.c_double(weight_decay), ctypes.c_double(eps),
                                   c_i64(block_size), c_i64(D))
    return alpha


def block_apply_adamw_f16(index, grad, emb_blocks, b1_t, b2_t, exp_avg, exp_avg_sq, lr, beta1, beta2,
                          weight_decay, eps, block_size):
    """block_apply_adamw on float16 rows and gradients, as the reference's CPU functor computes it
    when TEmb = at::Half (block_apply_adamw_op.cc:32-58): every product and sum in double (a Half
    operand meets a double), every assignment rounds double -> float -> half, sqrtf of the Half in
    float, and `emb_elem += <double>` converts the step to Half first and adds the two Halves in
    float (c10::Half defines += for Half operands only). numpy, vectorised over the rows of a call;
    ``index`` holds no duplicates. Pinned bit for bit against the compiled reference
    (tests/test_oracle_ref_ops.py)."""
    g = np.asarray(grad, dtype=np.float16).astype(np.float64)
    return _block_apply_adamw_16(index, g, emb_blocks, b1_t, b2_t, exp_avg, exp_avg_sq, lr, beta1, beta2, weight_decay,
                                 eps, block_size, lambda x: x.astype(np.float32).astype(np.float16))


def _block_apply_adamw_16(index, g, emb_blocks, b1_t, b2_t, exp_avg, exp_avg_sq, lr, beta1, beta2, weight_decay, eps,
                          block_size, r16):
    """The functor of block_apply_adamw_op.cc:32-58 with a 16-bit TEmb; ``r16`` is the rounding of a
    float to that type (the result in an array type that holds its values exactly), ``g`` the
    gradient in float64."""
    index = _i64(index)
    alpha = cal_alpha(b1_t, b2_t, lr, beta1, beta2)
    blk, row = index // block_size, index % block_size
    for b in np.unique(blk):
        sel = blk == b
        r = row[sel]
        w = r16(emb_blocks[b][r].astype(np.float64) * weight_decay)
        m = r16(exp_avg[b][r].astype(np.float64) * beta1 + g[sel] * (1 - beta1))
        v = r16(exp_avg_sq[b][r].astype(np.float64) * beta2 + (1 - beta2) * g[sel] * g[sel])
        step = r16(alpha * (m.astype(np.float64) / (np.sqrt(v.astype(np.float32)).astype(np.float64) + eps)))
        emb_blocks[b][r] = r16(w.astype(np.float32) + step.astype(np.float32))
        exp_avg[b][r] = m
        exp_avg_sq[b][r] = v
    return alpha


def round_bf16(x):
    """float -> bfloat16 as c10::BFloat16(float) rounds (round to nearest even on the upper 16 bits
    of the float32 pattern, NaN stays NaN), returned as float32 (which holds every bfloat16 value).
    Pinned against torch's own conversion on the CPU (tests/test_oracle_ref_ops.py)."""
    f = np.ascontiguousarray(np.asarray(x).astype(np.float32))
    u = f.view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    out = (r & 0xFFFFFFFF).astype(np.uint32).view(np.float32).copy()
    out[np.isnan(f)] = np.nan
    return out


def block_apply_adamw_bf16(index, grad, emb_blocks, b1_t, b2_t, exp_avg, exp_avg_sq, lr, beta1, beta2,
                           weight_decay, eps, block_size):
    """block_apply_adamw on bfloat16 rows (held as float32 arrays of bfloat16 values). The reference
    dispatches its functor for float, double and Half only (block_apply_adamw_op.cc:96-102), so this
    is that functor with TEmb = c10::BFloat16, which has the operators of c10::Half: the same
    statements as block_apply_adamw_f16 (pinned by the compiled reference) with the rounding of
    round_bf16 (pinned by torch's conversion). ``grad``: bfloat16 values, or float32 (the library
    also takes full-precision gradients for 16-bit rows: the functor with a float gradient)."""
    g = np.asarray(grad, dtype=np.float32).astype(np.float64)
    return _block_apply_adamw_16(index, g, emb_blocks, b1_t, b2_t, exp_avg, exp_avg_sq, lr, beta1, beta2, weight_decay,
                                 eps, block_size, lambda x: round_bf16(x.astype(np.float32)))


def block_apply_adamw_f64(index, grad, emb_blocks, b1_t, b2_t, exp_avg, exp_avg_sq, lr, beta1, beta2,
                          weight_decay, eps, block_size):
    """block_apply_adamw on float64 rows and gradients (the functor with TEmb = double,
    block_apply_adamw_op.cc:32-58): everything in double, nothing rounded but the argument of
    sqrtf, which is converted to float first. numpy; ``index`` holds no duplicates. Pinned bit for
    bit against the compiled reference (tests/test_oracle_ref_ops.py)."""
    index = _i64(index)
    alpha = cal_alpha(b1_t, b2_t, lr, beta1, beta2)
    g = np.asarray(grad, dtype=np.float64)
    blk, row = index // block_size, index % block_size
    for b in np.unique(blk):
        sel = blk == b
        r = row[sel]
        w = emb_blocks[b][r] * weight_decay
        m = exp_avg[b][r] * beta1 + g[sel] * (1 - beta1)
        v = exp_avg_sq[b][r] * beta2 + (1 - beta2) * g[sel] * g[sel]
        emb_blocks[b][r] = w + alpha * (m / (np.sqrt(v.astype(np.float32)).astype(np.float64) + eps))
        exp_avg[b][r] = m
        exp_avg_sq[b][r] = v
    return alpha


def block_apply_adagrad(index, grad, emb_blocks, accum, lr, eps, block_size):
    index, grad = _i64(index), _f32(grad)
    D = emb_blocks[0].shape[1]
    lib().oracle_block_apply_adagrad(_p(index), c_i64(index.shape[0]), _p(grad),
                                     _block_ptrs(emb_blocks), _block_ptrs(accum),
                                     ctypes.c_float(lr), ctypes.c_float(eps), c_i64(block_size),
                                     c_i64(D))


def block_apply_adagrad_exact(index, grad, emb_blocks, accum, lr, eps, block_size, bf16=False):
    """The Adagrad row update operation by operation, every one rounded once in float32 and the two
    results rounded to the rows' storage type (float32, or bfloat16 with ``bf16``: float32 arrays of
    bfloat16 values) when they are assigned:  s = r(s + g * g);  w = r(w - lr * (g / (sqrt(s) + eps))).
    The reference has no sparse Adagrad; the formula is torch.optim.Adagrad's (lr_decay 0, initial
    accumulator 0) on the rows that received a gradient, and this function is held to
    block_apply_adagrad above (which tests/test_oracle_table.py holds to torch.optim.Adagrad) within
    float32 rounding (tests/test_oracle_table.py). What it adds is the order and place of the
    roundings, so that the kernels can be compared bit for bit, bfloat16 rows included."""
    index = _i64(index)
    g = np.asarray(grad, dtype=np.float32)
    lr, eps = np.float32(lr), np.float32(eps)
    r = round_bf16 if bf16 else (lambda x: x)
    blk, row = index // block_size, index % block_size
    for b in np.unique(blk):
        sel = blk == b
        rr, gg = row[sel], g[sel]
        s = r(accum[b][rr].astype(np.float32) + gg * gg)
        w = r(emb_blocks[b][rr].astype(np.float32) - lr * (gg / (np.sqrt(s) + eps)))
        accum[b][rr] = s
        emb_blocks[b][rr] = w


# ----------------------------------------------------------- dedup / tagging


def ids_encode(ids_list, table_ids):
    outs = []
    for ids, t in zip(ids_list, table_ids):
        ids = _i64(ids)
        out = np.empty_like(ids)
        lib().oracle_ids_encode(_p(ids), c_i64(ids.shape[0]), c_i64(int(t)), _p(out))
        outs.append(out)
    return np.concatenate(outs) if outs else np.empty(0, np.int64)


def ids_partition(ids, num_parts):
    ids = _i64(ids)
    n = ids.shape[0]
    uniq = np.empty(n, np.int64)
    counts = np.empty(num_parts, np.int64)
    inv = np.empty(n, np.int32)
    u = lib().oracle_ids_partition(_p(ids), c_i64(n), int(num_parts), _p(uniq), _p(counts), _p(inv))
    return uniq[:u].copy(), counts, inv


# ------------------------------------------------------------- feature ops


def uint64_mod(x, mod):
    x = _i64(x)
    out = np.empty_like(x)
    lib().oracle_uint64_mod(_p(x), c_i64(x.size), c_i64(int(mod)), _p(out))
    return out


def bucketize(values, boundaries):
    v, b = _f32(values), _f32(boundaries)
    out = np.empty(v.shape, np.int64)
    lib().oracle_bucketize(_p(v), c_i64(v.size), _p(b), ctypes.c_int32(b.size), _p(out))
    return out


def multi_hash(x, muls, primes, buckets):
    x = _i64(x)
    outs = []
    for m, p, b in zip(muls, primes, buckets):
        out = np.empty_like(x)
        lib().oracle_multi_hash(_p(x), c_i64(x.size), c_i64(int(m)), c_i64(int(p)), c_i64(int(b)),
                                _p(out))
        outs.append(out)
    return outs


def hash_strings(values, offsets, kind):
    """values: int8/uint8 bytes; offsets: [n+1]; kind 'farm' | 'murmur'."""
    values = np.ascontiguousarray(values).view(np.int8)
    offsets = _i64(offsets)
    n = offsets.shape[0] - 1
    out = np.empty(n, np.int64)
    lib().oracle_hash_strings(_p(values), _p(offsets), c_i64(n), {"farm": 0, "murmur": 1}[kind],
                              _p(out))
    return out


# ------------------------------------------------------- sequence truncation


def ragged_cutoff_2d(values, offsets, keep, drop_left):
    """One 2-D ragged tensor cut to at most ``keep`` elements per row
    (csrc/ops/fused_ragged_cutoff_kernel.cu:55-69 lengths, :706-727 which elements stay).
    Returns (values, offsets, drop_nums, pad_nums)."""
    values, offsets = np.asarray(values), np.asarray(offsets)
    out_v, out_o, drops, pads = [], [0], [], []
    for r in range(len(offsets) - 1):
        beg, end = int(offsets[r]), int(offsets[r + 1])
        n = end - beg
        dropped = n >= keep
        k = keep if dropped else n
        drop = n - keep if dropped else 0
        drops.append(drop)
        pads.append(0 if dropped else keep - n)
        first = beg + (drop if drop_left else 0)
        out_v.append(values[first:first + k])
        out_o.append(out_o[-1] + k)
    vals = np.concatenate(out_v) if out_v else values[:0]
    return vals, np.asarray(out_o, offsets.dtype), np.asarray(drops, offsets.dtype), np.asarray(pads, offsets.dtype)


def ragged_cutoff_3d(values, outer, inner, keep, drop_left, pad_left):
    """One 3-D ragged tensor with every sequence brought to exactly ``keep`` inner rows
    (csrc/ops/fused_ragged_cutoff_kernel.cu:300-337 which inner row lands where, :513-550 the values).
    Returns (values, outer_offsets, inner_offsets)."""
    values, outer, inner = np.asarray(values), np.asarray(outer), np.asarray(inner)
    out_v, out_inner = [], [0]
    n_seq = len(outer) - 1
    for s in range(n_seq):
        beg, end = int(outer[s]), int(outer[s + 1])
        n = end - beg
        drop = n - keep if n >= keep else 0
        pad = 0 if n >= keep else keep - n
        for col in range(keep):
            row, padded = col, False
            if drop > 0:
                if drop_left:
                    row += drop
            elif pad > 0:
                if pad_left:
                    padded = col < pad
                    row -= pad
                else:
                    padded = keep <= pad + col
            if padded:
                out_inner.append(out_inner[-1])
            else:
                b, e = int(inner[beg + row]), int(inner[beg + row + 1])
                out_v.append(values[b:e])
                out_inner.append(out_inner[-1] + (e - b))
    vals = np.concatenate(out_v) if out_v else values[:0]
    return vals, (np.arange(n_seq + 1) * keep).astype(outer.dtype), np.asarray(out_inner, inner.dtype)


def ragged_to_dense(values, offsets, default_value=0):
    """Dense ``[batch, longest row of every level]`` of a ragged tensor with several levels of
    offsets, ``default_value`` outside the rows (csrc/ops/ragged_to_dense.cc:6-45; the walk of
    ragged_common.cuh:36-64)."""
    values = np.asarray(values)
    offsets = [np.asarray(o) for o in offsets]
    widths = [int((o[1:] - o[:-1]).max()) if len(o) > 1 else 0 for o in offsets]
    out = np.full([len(offsets[0]) - 1] + widths, default_value, values.dtype)
    for coord in np.ndindex(*out.shape):
        at = coord[0]
        for d, o in enumerate(offsets):
            beg, end = int(o[at]), int(o[at + 1])
            if coord[d + 1] >= end - beg:
                break
            at = beg + coord[d + 1]
        else:
            out[coord] = values[at]
    return out


def dense_to_ragged(data, invalid_value):
    """(values, int32 offsets): every row up to its last element that differs from
    ``invalid_value`` (csrc/ops/dense_to_ragged.cc:6-53)."""
    data = np.asarray(data)
    vals, offs = [], [0]
    for row in data:
        keep = np.nonzero(row != invalid_value)[0]
        n = int(keep[-1]) + 1 if len(keep) else 0
        vals.append(row[:n])
        offs.append(offs[-1] + n)
    return (np.concatenate(vals) if vals else data.reshape(-1)[:0]), np.asarray(offs, np.int32)


# ------------------------------------------------------------ feature cross


def murmur_hash_64_words(words, seed=0):
    """MurmurHash64A over 8-byte words (csrc/ops/ragged_common.cuh:105-125), as a Python int."""
    mask = (1 << 64) - 1
    m = 0xc6a4a7935bd1e995
    h = (seed ^ (len(words) * 8 * m)) & mask
    for k in words:
        k = (int(k) & mask) * m & mask
        k ^= k >> 47
        k = k * m & mask
        h = ((h ^ k) * m) & mask
    h ^= h >> 47
    h = h * m & mask
    h ^= h >> 47
    return h


def feature_cross_ragged(x_val, x_off, x_w, y_val, y_off, y_w):
    """Per segment: distinct ids of x crossed with distinct ids of y, each with the weight of its
    first occurrence (csrc/ops/feature_cross_ragged.cc:7-20,60-92). Entries in first-occurrence
    order, x outermost. Returns (ids int64, offsets, weights)."""
    x_val, y_val, x_off, y_off = (np.asarray(a) for a in (x_val, y_val, x_off, y_off))
    wdt = np.asarray(x_w if x_w is not None else y_w if y_w is not None else np.zeros(0, np.float32)).dtype
    ids, ws, offs = [], [], [0]

    def distinct(val, w, beg, end):
        seen = {}
        for i in range(beg, end):
            if int(val[i]) not in seen:
                seen[int(val[i])] = wdt.type(1) if w is None else w[i]
        return seen

    for s in range(min(len(x_off), len(y_off)) - 1):
        ux = distinct(x_val, x_w, int(x_off[s]), int(x_off[s + 1]))
        uy = distinct(y_val, y_w, int(y_off[s]), int(y_off[s + 1]))
        for a, wa in ux.items():
            for b, wb in uy.items():
                h = murmur_hash_64_words([a, b])
                ids.append(h - (1 << 64) if h >= 1 << 63 else h)
                ws.append(wa * wb)
        offs.append(len(ids))
    return np.asarray(ids, np.int64), np.asarray(offs, x_off.dtype), np.asarray(ws, wdt)


def calc_ragged_index(drop_num, offset, topk_index, indicator):
    """Drop left / pad right of csrc/ops/calc_ragged_index.cc:55-76: for row r of topk_index
    [rows, cols] and src = indicator[r], the kept elements offset[src] + drop_num[src] +
    topk_index[r, c] that fall inside [offset[src], offset[src + 1]), in column order, and the
    running count per row. Returns (value_index of topk_index's dtype, offsets of offset's dtype)."""
    drop_num, offset, topk_index, indicator = (np.asarray(a) for a in (drop_num, offset, topk_index, indicator))
    out, offs = [], [0]
    for r in range(topk_index.shape[0]):
        src = int(indicator[r])
        beg, end, drop = int(offset[src]), int(offset[src + 1]), int(drop_num[src])
        for c in range(topk_index.shape[1]):
            e = int(topk_index[r, c]) + beg + drop
            if beg <= e < end:
                out.append(e)
        offs.append(len(out))
    return np.asarray(out, topk_index.dtype), np.asarray(offs, offset.dtype)


def ragged_to_sparse_indices(offsets):
    """COO coordinates [levels + 1, n_values] of the values of a ragged tensor with the given
    list of offsets, outermost level first (csrc/ops/ragged_to_sparse.cc:8-40): coordinate 0 is
    the outermost row, coordinate k the position inside the row of level k - 1."""
    offsets = [np.asarray(o).astype(np.int64) for o in offsets]
    n = int(offsets[-1][-1]) if len(offsets[-1]) else 0
    idx = np.zeros((len(offsets) + 1, n), np.int64)
    for v in range(n):
        child = v
        for k in range(len(offsets) - 1, -1, -1):
            o = offsets[k]
            row = 0
            while not (o[row] <= child < o[row + 1]):
                row += 1
            idx[k + 1, v] = child - o[row]
            child = row
        idx[0, v] = child
    return idx

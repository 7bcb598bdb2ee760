"""Feature-engine ops on the hot path: the mirror of ``recis.features.op`` for
``SelectField``, ``Mod``, ``Bucketize``, ``Hash``, ``IDMultiHash`` and ``SequenceTruncate``
and ``FeatureCross`` (recis/features/op.py:129-686).

Every op works on a ``RaggedTensor`` (its values) or a plain tensor; the engine
batches same-typed ops of one step into a single fused HIP launch.
"""
import hashlib
import json
from typing import Dict, List, Union

import torch
from torch import nn

from .. import ops
from ..ragged.tensor import RaggedPadInfo, RaggedTensor


def _values(x):
    return x.values() if isinstance(x, RaggedTensor) else x


def _with_values(x, values):
    if isinstance(x, RaggedTensor):
        return RaggedTensor(values, x.offsets(), x.weight(), x.dense_shape)
    return values


class DataValueProcessor:
    """The values an op works on, whatever container carries them, and the container rebuilt
    around the op's result (op.py:22-84)."""

    def __init__(self, data: Union[RaggedTensor, torch.Tensor]):
        self._data = data

    def get_input_value(self):
        if isinstance(self._data, RaggedTensor):
            return self._data.values()
        if isinstance(self._data, torch.Tensor):
            return self._data._values() if self._data.is_sparse else self._data
        raise ValueError("Unsupported data type: %s" % type(self._data))

    def get_output_value(self, result):
        if isinstance(self._data, RaggedTensor):
            return RaggedTensor(result, self._data.offsets(), self._data.weight(), self._data.dense_shape)
        if isinstance(self._data, torch.Tensor):
            if self._data.is_sparse:
                return torch.sparse_coo_tensor(self._data._indices(), result, self._data.shape)
            return result.reshape(self._data.shape)
        raise ValueError("Unsupported data type: %s" % type(self._data))


class _OP(nn.Module):
    def get_hash(self) -> int:
        text = json.dumps({"type": type(self).__name__, "config": self._get_config()}, sort_keys=True)
        return int(hashlib.sha256(text.encode()).hexdigest()[:16], 16)

    def _get_config(self) -> Dict:
        raise NotImplementedError


class SelectField(_OP):
    def __init__(self, name: str, dtype=torch.long, dim=None, from_dict=True):
        super().__init__()
        self._name, self._dtype, self._dim, self._from_dict = name, dtype, dim, from_dict

    def forward(self, data):
        if self._from_dict:
            assert isinstance(data, dict), "data must be a dict, fn:%s" % self._name
            return data[self._name]
        return data

    def _get_config(self):
        return {"name": self._name, "dtype": str(self._dtype), "dim": self._dim, "from_dict": self._from_dict}


class SelectFields(_OP):
    """Several fields at once, as a list (op.py:198-245)."""

    def __init__(self, input_list: List[SelectField]):
        super().__init__()
        self.input_list = nn.ModuleList(input_list)

    def forward(self, data):
        return [op(data) for op in self.input_list]

    def _get_config(self):
        return {"input_hashes": [op.get_hash() for op in self.input_list]}


class Mod(_OP):
    """``(int64)((uint64) x % mod)``."""

    def __init__(self, mod_value):
        super().__init__()
        self.mod_value = int(mod_value)

    def forward(self, x: Union[RaggedTensor, torch.Tensor]):
        return _with_values(x, ops.uint64_mod(_values(x).cuda(), self.mod_value))

    def _get_config(self):
        return {"mod": self.mod_value}


class Bucketize(_OP):
    """Number of boundaries <= value (int64)."""

    def __init__(self, boundary):
        super().__init__()
        b = torch.tensor(boundary, dtype=torch.float) if isinstance(boundary, list) else boundary.float()
        self.register_buffer("boundary", b)
        self._on_device = None

    def boundary_on(self, device):
        """The boundaries on ``device``: the buffer itself when it lives there, else a copy made once (and
        again if the buffer is replaced or written to)."""
        b = self.boundary
        if b.device == device:
            return b
        hit = self._on_device
        if hit is None or hit[0] is not b or hit[1] != b._version or hit[2].device != device:
            hit = self._on_device = (b, b._version, b.to(device))
        return hit[2]

    def forward(self, x):
        v = _values(x).cuda().float()
        return _with_values(x, ops.bucketize_op(v, self.boundary_on(v.device)))

    def _get_config(self):
        return {"boundary": self.boundary.tolist()}


class Hash(_OP):
    """64-bit hash ("farm" | "murmur") of the byte strings of a two-level ragged tensor: the
    innermost offsets delimit the strings, the hashed values replace them (one per string)."""

    def __init__(self, hash_type: str):
        super().__init__()
        assert hash_type in ("farm", "murmur"), "hash_type must be farm or murmur"
        self.hash_type = hash_type

    def forward(self, x: RaggedTensor):
        assert isinstance(x, RaggedTensor), "Hash takes a RaggedTensor of bytes"
        values = x.values().cuda()
        out = ops.fused_hash([values], [x.offsets()[-1].cuda()], self.hash_type)[0]
        rest = [o.cuda() for o in x.offsets()[:-1]]
        if not rest:
            rest = [torch.arange(out.numel() + 1, device=out.device)]
        return RaggedTensor(out, rest, None)

    def _get_config(self):
        return {"hash_type": self.hash_type}


def _largest_prime_le(n):
    def is_prime(k):
        if k < 2:
            return False
        d = 2
        while d * d <= k:
            if k % d == 0:
                return False
            d += 1
        return True
    while not is_prime(n):
        n -= 1
    return n


class IDMultiHash(_OP):
    """``multi_hash_j = (((x * mul_j) % p_j + p_j) % p_j) % bucket_j`` with mul = [1, 3, 5, 7] and
    p_j the largest prime <= [29, 47, 67, 83][j] * bucket_j (recis/features/op.py:520-577)."""

    _MULS = [1, 3, 5, 7]
    _MODS = [29, 47, 67, 83]

    def __init__(self, num_buckets: List[int], prefix: str = "multi_hash"):
        super().__init__()
        assert 1 <= len(num_buckets) <= 4, "IDMultiHash supports 1 to 4 hashes"
        self.num_buckets = [int(b) for b in num_buckets]
        self.prefix = prefix
        n = len(self.num_buckets)
        self.muls = self._MULS[:n]
        self.primes = [_largest_prime_le(m * b) for m, b in zip(self._MODS[:n], self.num_buckets)]

    def forward(self, x):
        outs = ops.fused_multi_hash([_values(x).cuda()], [self.muls], [self.primes], [self.num_buckets])
        return {"%s_%d" % (self.prefix, j): _with_values(x, o) for j, o in enumerate(outs)}

    def _get_config(self):
        return {"num_buckets": self.num_buckets, "prefix": self.prefix}


class FeatureCross(_OP):
    """Cross of two id features, segment by segment (recis/features/op.py:357-405)."""

    def forward(self, data: List[RaggedTensor]):
        x, y = data
        assert isinstance(x, RaggedTensor) and isinstance(y, RaggedTensor)
        val, offsets, weight = ops.feature_cross_ragged(x.values(), x.offsets()[-1], x.weight(), y.values(),
                                                        y.offsets()[-1], y.weight())
        return RaggedTensor(val, offsets, weight, x.dense_shape)

    def _get_config(self):
        return {}


class SequenceTruncate(_OP):
    """Cuts every sequence to ``seq_len`` (recis/features/op.py:408-517): a 2-D ragged tensor
    keeps at most ``seq_len`` elements per row; a 3-D one comes out with exactly ``seq_len`` inner
    rows per sequence (missing ones empty, added at the end). ``truncate_side`` "left" drops the
    oldest entries (the start of the row)."""

    def __init__(self, seq_len=64, check_length=True, truncate=True, truncate_side="left", n_dims=2,
                 dtype=torch.long):
        super().__init__()
        assert n_dims in [2, 3]
        self.n_dims, self.seq_len, self.check_length = n_dims, int(seq_len), check_length
        self.truncate, self.truncate_side, self.dtype = truncate, truncate_side, dtype

    def forward(self, x: RaggedTensor):
        if self.check_length:
            # x.shape resolves an unstated extent by reading the longest row back, as the reference does
            assert x.shape[1] <= self.seq_len, "sequence length must be less than %d" % self.seq_len
        if not self.truncate:
            return None  # as the reference (op.py:489-507 has no other branch)
        return sequence_truncate([self], [x])[0]

    def _get_config(self):
        return {"seq_len": self.seq_len, "check_length": self.check_length, "truncate": self.truncate,
                "truncate_side": self.truncate_side, "n_dims": self.n_dims, "dtype": str(self.dtype)}


def sequence_truncate(op_list, inputs):
    """One fused launch per (value dtype, dimensionality) group (FusedCutoffOP, fused_op_impl.py:274-390)."""
    from ..nn.functional import ragged_ops

    results = [None] * len(inputs)
    groups = {}
    for i, (op, x) in enumerate(zip(op_list, inputs)):
        groups.setdefault((x.values().dtype, op.n_dims), []).append(i)
    for (_, n_dims), idx in groups.items():
        keep = [op_list[i].seq_len for i in idx]
        drop = [op_list[i].truncate_side == "left" for i in idx]
        pad = [False] * len(idx)
        vals = [inputs[i].values().cuda() for i in idx]
        if n_dims == 2:
            out = ragged_ops.fused_ragged_cutoff_2D(vals, [inputs[i].offsets()[-1].cuda() for i in idx], keep, drop, pad)
            new_vals, new_offs = out[0], [[o] for o in out[1]]
            pad_infos = [RaggedPadInfo(out[2][k], out[3][k], torch.tensor(drop[k]), torch.tensor(pad[k]))
                         for k in range(len(idx))]
        else:
            new_vals, new_offs = ragged_ops.fused_ragged_cutoff_3D(
                vals, [[o.cuda() for o in inputs[i].offsets()] for i in idx], keep, drop, pad)
            pad_infos = None  # as in the reference, only the 2-D truncation records what it dropped
        for k, i in enumerate(idx):
            shape = list(inputs[i].dense_shape)
            shape[1] = op_list[i].seq_len
            results[i] = RaggedTensor(new_vals[k], new_offs[k], inputs[i].weight(), shape)
            if pad_infos is not None:  # fused_op_impl.py:406-411
                results[i].set_pad_info(pad_infos[k])
    return results

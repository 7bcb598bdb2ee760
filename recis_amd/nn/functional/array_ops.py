"""``recis.nn.functional.array_ops`` (array_ops.py:4-127): single-tensor forms of the feature ops."""
import torch

from ... import ops


def bucketize(input, boundaries):
    """Index of the bucket of every element: the number of boundaries <= the element."""
    if not isinstance(boundaries, torch.Tensor):
        boundaries = torch.tensor(boundaries)
    boundaries = boundaries.to(device=input.device, dtype=input.dtype)
    return ops.bucketize_op(input.reshape([-1]), boundaries).reshape(input.shape)


def bucketize_mod(input, bucket):
    """``(uint64) input % bucket`` as int64."""
    assert input.dtype == torch.int64
    return ops.uint64_mod(input.reshape([-1]), bucket).reshape(input.shape)


def multi_hash(input, muls, primes, bucket_num):
    """Four hashes ``(((x * mul) % prime + prime) % prime) % bucket`` of every id. (The reference
    calls an operator ``multi_hash`` that its extension does not register; this runs the fused
    operator on one tensor.)"""
    assert input.dtype == torch.int64

    def as_i64(v):
        v = v if isinstance(v, torch.Tensor) else torch.tensor(v)
        return v.to(device=input.device, dtype=torch.int64)

    muls, primes, bucket_num = as_i64(muls), as_i64(primes), as_i64(bucket_num)
    assert muls.numel() == 4
    assert primes.numel() == 4
    outs = ops.fused_multi_hash([input.reshape([-1])], [muls], [primes], [bucket_num])
    return [out.reshape(input.shape) for out in outs]

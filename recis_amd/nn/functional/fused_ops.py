"""Thin wrappers with the names of ``recis.nn.functional.fused_ops`` over the fused
multi-tensor HIP ops."""
import torch

from ... import ops


def fused_ids_encode_gpu(ids_list, table_ids):
    return ops.ids_encode(ids_list, table_ids)


def fused_bucketize_gpu(values, boundaries):
    return ops.fused_bucketized(values, boundaries)


def fused_uint64_mod_gpu(values, mods):
    if torch.is_tensor(mods):
        mods = mods.tolist()
    return ops.fused_uint64_mod(values, mods)


def fused_multi_hash(inputs, muls, primes, bucket_nums):
    return ops.fused_multi_hash(inputs, muls, primes, bucket_nums)

"""``recis.nn.functional.hash_ops``: 64-bit string hashes over lists of byte tensors."""
from ... import ops


def farmhash(inputs, offsets):
    return ops.fused_hash(inputs, offsets, "farm")


def murmurhash(inputs, offsets):
    return ops.fused_hash(inputs, offsets, "murmur")

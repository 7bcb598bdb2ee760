from . import embedding_ops, fused_ops, hash_ops, ragged_ops  # noqa: F401

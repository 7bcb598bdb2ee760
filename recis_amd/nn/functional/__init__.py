from . import embedding_ops, fused_ops, hash_ops  # noqa: F401

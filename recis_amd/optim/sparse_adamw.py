"""``recis.optim.sparse_adamw`` (the class lives in ``sparse_optim``)."""
from .sparse_optim import SparseAdamW  # noqa: F401

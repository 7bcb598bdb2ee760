"""``recis.optim.sparse_adam`` (the class lives in ``sparse_optim``)."""
from .sparse_optim import SparseAdam  # noqa: F401

"""``recis.optim.sparse_adamw_tf`` (the class lives in ``sparse_optim``)."""
from .sparse_optim import SparseAdamWTF  # noqa: F401

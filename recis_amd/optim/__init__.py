from .sparse_optim import SparseAdagrad, SparseAdam, SparseAdamW, SparseAdamWTF, SparseOptimizer  # noqa: F401

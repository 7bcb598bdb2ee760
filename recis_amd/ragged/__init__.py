from .tensor import RaggedTensor  # noqa: F401

from .tensor import RaggedPadInfo, RaggedTensor  # noqa: F401

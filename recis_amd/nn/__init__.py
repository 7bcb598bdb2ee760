from . import functional, hashtable_hook, initializers  # noqa: F401
from .modules import hashtable_hook_impl  # noqa: F401
from .modules.embedding import DynamicEmbedding, EmbeddingOption  # noqa: F401
from .modules.embedding_engine import EmbeddingEngine  # noqa: F401
from .modules.hashtable import HashTable, filter_out_sparse_param  # noqa: F401

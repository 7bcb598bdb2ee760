from . import hashtable_hook_impl  # noqa: F401  (registers the built-in hooks)
from .hashtable import HashTable, gen_slice, filter_out_sparse_param  # noqa: F401

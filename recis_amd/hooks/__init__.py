from .filter_hook import HashTableFilterHook  # noqa: F401
from .hook import Hook  # noqa: F401

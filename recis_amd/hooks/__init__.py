from .filter_hook import HashTableFilterHook  # noqa: F401

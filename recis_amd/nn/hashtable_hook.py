"""Hook descriptors (``recis.nn.hashtable_hook``): a name plus parameters; the table
turns them into implementations through ``HashtableHookFactory``."""
from typing import Optional


class BaseHook:
    def __init__(self, name: str, params: Optional[dict] = None):
        self._name = name
        self._params = {} if params is None else dict(params)

    @property
    def name(self) -> str:
        return self._name

    @property
    def params(self) -> dict:
        return self._params

    def __str__(self):
        return "%s(name=%s, params=%s)" % (type(self).__name__, self._name, self._params)


class AdmitHook(BaseHook):
    """Controls whether a lookup may admit new keys; ``"ReadOnly"`` never admits."""

    @property
    def type(self) -> str:
        return "admit"


class FilterHook(BaseHook):
    """Controls eviction; ``"GlobalStepFilter"`` (params ``filter_step``) evicts keys not
    seen for more than ``filter_step`` steps."""

    @property
    def type(self) -> str:
        return "filter"

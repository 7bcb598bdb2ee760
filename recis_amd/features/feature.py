"""``Feature``: a named chain of ops (mirror of ``recis.features.feature``)."""
import hashlib
from typing import List

from torch import nn


class Feature(nn.Module):
    def __init__(self, name: str):
        super().__init__()
        self._name = name
        self._ops = nn.ModuleList()
        self._compiled = False

    @property
    def name(self):
        return self._name

    @property
    def compiled(self):
        return self._compiled

    def compiled_(self, value: bool):
        self._compiled = value

    @property
    def ops(self) -> List[nn.Module]:
        return list(self._ops)

    def add_op(self, op):
        self._ops.append(op)
        return self

    def get_hash(self) -> int:
        text = ",".join(str(op.get_hash()) for op in self._ops)
        return int(hashlib.sha256(text.encode()).hexdigest()[:16], 16)

    def forward(self, data):
        for op in self._ops:
            data = op(data)
        return data

"""Loader of ``recis_amd/lib/recis.so``: the ``TORCH_LIBRARY(recis)`` registration
(csrc/bind.cc:46-211 of the reference) on top of librecis_hip.so.

After ``load()``, ``torch.ops.recis.<op>`` and ``torch.classes.recis.<Class>`` exist with the
reference's names and schemas, exactly as after the reference's
``torch.classes.load_library(<pkg>/lib/recis.so)`` (recis/__init__.py:8-16).
"""
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "recis.so")
_loaded = False


def load():
    global _loaded
    if _loaded:
        return
    if not os.path.exists(LIB_PATH):
        from . import build as _build

        if not os.path.exists(_build.LIB_PATH):
            _build.build(verbose=False)
        else:
            _build.build_torch_library(verbose=False)
    torch.classes.load_library(LIB_PATH)
    _loaded = True

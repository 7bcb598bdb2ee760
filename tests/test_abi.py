"""The C-ABI library loads without a GPU and exports every symbol the header declares."""
import os
import re

from recis_amd import _lib


def test_library_exports_every_declared_symbol():
    with open(_lib.HEADER_PATH) as f:
        text = f.read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = re.findall(r"\b(recis_[a-z0-9_]+)\s*\(", text)
    assert len(names) >= 36
    lib = _lib.lib()
    for n in sorted(set(names)):
        assert hasattr(lib, n), "missing export: %s" % n
    assert lib.recis_hip_abi_version() == _lib.ABI_VERSION == 2
    assert isinstance(lib.recis_hip_last_error(), bytes)


def test_header_is_plain_c():
    import subprocess

    r = subprocess.run(["gcc", "-std=c99", "-fsyntax-only", "-x", "c", _lib.HEADER_PATH],
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    assert "torch" not in open(_lib.HEADER_PATH).read().split("*/", 1)[1].lower().replace("torch.unique", "")


def test_product_package_does_not_import_the_oracle():
    root = os.path.dirname(os.path.abspath(_lib.__file__))
    for dirpath, _, files in os.walk(root):
        for fn in files:
            if fn.endswith((".py", ".hip", ".cuh", ".cpp", ".h")):
                src = open(os.path.join(dirpath, fn)).read()
                assert "import oracle" not in src and "liboracle" not in src, fn

"""The C-ABI library loads without a GPU and exports every symbol include/deepep_amd.h declares."""

import os
import re

from deepep_amd import _lib

HEADER = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include", "deepep_amd.h")


def _declared():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(dpep_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree():
    assert _declared() == sorted(_lib.SIGNATURES)


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    for name in _declared():
        assert hasattr(lib, name), name
    assert lib.dpep_version() >= 1
    assert lib.dpep_layout_workspace_bytes(4096, 8, 256) >= 256 * 4
    assert lib.dpep_layout_workspace_bytes(-1, 8, 256) == 0

"""The C-ABI library loads without a GPU and exports every symbol include/scn_hip.h declares,
and the ctypes table binds exactly those symbols."""
import os
import re

from sparseconvnet_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "scn_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(scn_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_exported_and_bound():
    names = declared_symbols()
    assert len(names) >= 24
    lib = _lib.lib()
    for n in names:
        assert hasattr(lib, n), n
    assert sorted(_lib.SIGNATURES) == names


def test_error_reporting_without_gpu():
    lib = _lib.lib()
    assert lib.scn_rulebook_bits() == 32
    assert not lib.scn_md_create(0)
    assert b"dimension" in lib.scn_last_error()
    h = lib.scn_md_create(3)
    assert h
    lib.scn_md_destroy(h)

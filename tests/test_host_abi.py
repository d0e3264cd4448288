"""C-ABI library: loads without a GPU and exports every symbol the header declares."""
import ctypes
import os
import re

from helpers import ROOT, mil


def _declared():
    names = set()
    for header in sorted(os.listdir(os.path.join(ROOT, "include"))):
        text = open(os.path.join(ROOT, "include", header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names |= set(re.findall(r"\b(mi_[a-z0-9_]+)\s*\(", text))
    return sorted(names)


def test_library_exports_every_declared_symbol():
    names = _declared()
    assert len(names) >= 35
    lib = ctypes.CDLL(mil.LIB_PATH)
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing


def test_binding_covers_every_declared_symbol():
    assert sorted(mil._SIGNATURES) == _declared()


def test_register_argument_checks_need_no_gpu(capfd):
    L = mil.lib()
    # null / non-positive arguments -> false (LF/src/utils.cpp:358, 585)
    assert L.mi_register_int8_weight(None, 0x1000, 4, 4) == 0
    assert L.mi_register_int8_weight(0x1000, None, 4, 4) == 0
    assert L.mi_register_int8_weight(0x1000, 0x2000, 0, 4) == 0
    assert L.mi_register_q4_weight(0x1000, 0x2000, 4, -1) == 0
    # Q4 with a K that is not a whole number of 32-blocks is refused, as the quantizer does
    assert L.mi_register_q4_weight(0x1000, 0x2000, 4, 48) == 0
    assert "ERROR:" in capfd.readouterr().err
    # registry bookkeeping
    assert L.mi_register_int8_weight(0x1000, 0x2000, 8, 64) == 1
    assert L.mi_weight_kind(0x1000) == 8
    assert L.mi_register_q4_weight(0x1000, 0x2000, 8, 64) == 1       # re-registration overwrites
    assert L.mi_weight_kind(0x1000) == 4
    assert L.mi_unregister_weight(0x1000) == 1
    assert L.mi_weight_kind(0x1000) == 0
    assert L.mi_unregister_weight(0x1000) == 0

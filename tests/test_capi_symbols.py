"""The C-ABI library loads and exports every symbol include/coalsack_moe.h
declares (no compute: runs without a GPU)."""
import ctypes
import os
import re

from coalsack_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "coalsack_moe.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(csk_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree():
    assert declared_symbols() == sorted(capi.SIGNATURES)


def test_library_exports_every_declared_symbol():
    dll = ctypes.CDLL(capi.lib_path())
    for name in declared_symbols():
        assert hasattr(dll, name), name


def test_calls_before_init_fail_cleanly():
    lib = capi.Library()
    if lib.dll.csk_init(0) == capi.OK:
        return  # a GPU is present: nothing to check here
    assert lib.dll.csk_last_error()  # a message, not a crash
    h = ctypes.c_void_p()
    assert lib.dll.csk_layer_create(4, 2, 64, 64, ctypes.byref(h)) == capi.ERR_STATE
    assert b"csk_init" in lib.dll.csk_last_error()
    assert lib.dll.csk_synchronize() == capi.ERR_STATE
    assert not lib.dll.csk_dev_alloc(16)

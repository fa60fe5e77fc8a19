"""MI355X (gfx950) implementation of coalsack's mixture-of-experts path.

The product is the C-ABI shared library ``libcoalsack_moe.so`` (sources under
``csrc/``, declarations in ``include/coalsack_moe.h``) and the C++ node classes
under ``host/``.  This Python package is only the loader the tests and the
benchmark use to reach that library through ctypes; it contains no compute.
"""
from .capi import Library, CskError, load, lib_path  # noqa: F401

"""MI355X-native worker-side logistic regression for Paracel.

The package wraps ``libplr.so`` (hand-written HIP kernels for gfx950 behind the
C ABI of ``include/plr.h``).  There is no CPU fallback: if the library is not
built, importing :mod:`paracel_amd.capi` raises.
"""
from .capi import Plr, PlrError, lib_path, load_library  # noqa: F401

__all__ = ["Plr", "PlrError", "lib_path", "load_library"]

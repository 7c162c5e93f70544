"""blackforge_amd: an MI355X (gfx950) operator backend for BlackForge.

The product is the C-ABI library built from ``csrc/`` (``lib/libbf_hip.so``, declared in
``include/bf_hip.h``) and the C++ operator layer in ``include/blackforge/backend/hip/`` on top of it.
This Python package only binds the C ABI with ctypes (``capi``) and mirrors the operator interface
(``ops``: same function names and argument meaning as the reference's free functions) so that
parity tests and the benchmark can drive the library from Python.
"""
from . import capi  # noqa: F401
from .tensor import DeviceTensor, Stream, Event  # noqa: F401
from . import ops  # noqa: F401

__all__ = ["capi", "ops", "DeviceTensor", "Stream", "Event"]

"""MI355X-native implementation of Tracea's dense-contraction path.

The product is ``lib/libtracea.so`` (hand-written HIP kernels for gfx950 behind
Tracea's C ABI, see ``include/tracea.h``).  This package is the thin Python
caller above that ABI: ``tracea_amd.capi`` binds the C entry points with
ctypes, ``tracea_amd.ops`` mirrors the operator front end of the reference's
Python layer (``tracea.ops`` in tracea-python/python/tracea/ops.py) on torch
tensors.  torch is used for device memory and streams only.
"""
from . import capi  # noqa: F401

__version__ = "0.1.0"

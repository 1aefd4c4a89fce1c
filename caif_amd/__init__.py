"""MI355X (gfx950) implementation of CAIF's frozen quantized linear.

The product is the C-ABI library ``caif_amd/lib/libcaifx.so`` (hand-written HIP
kernels, declared in ``include/caifx.h``) and the C++ host layer under
``caif_amd/host`` that mirrors the reference's layer / ops API on top of it.
This Python package is the ctypes plumbing that tests and ``bench.py`` use to
reach the same entry points with torch-owned device memory.  There is no CPU
fallback: loading fails loudly when the library has not been built.
"""
from . import capi  # noqa: F401

__all__ = ["capi"]

"""rocmforge_amd -- MI355X (gfx950) kernels for ROCmForge's quantized-weight path.

The product is ``librfq.so`` (``csrc/``, C ABI in ``include/rfq.h``).  This
package holds the ctypes binding used by the tests and the bench, a host-side
mirror of the ROCmForge operator surface for this path (``loader``, ``ops``)
and the seeded block generators (``quantize``).
"""
from . import quantize  # noqa: F401
from ._lib import RfqError, lib, lib_path  # noqa: F401

__all__ = ["quantize", "RfqError", "lib", "lib_path"]

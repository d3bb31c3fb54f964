"""MI355X (gfx950) implementation of the GPU operator layer behind Minerva's NArray
engine.  The product is native: `lib/libmnv_hip.so` (HIP kernels behind the C ABI of
include/mnv_hip.h) and `lib/libmnv_host.so` (C++ mirror of Minerva's operator / device
interface).  This package only loads them; there is no Python or CPU fallback."""
from . import capi  # noqa: F401

__all__ = ["capi"]

"""MI355X (gfx950) implementation of the TOSA reference model's tensor-op hot path.

The product is the HIP library ``libtosa_mi355.so`` behind the C ABI of ``include/tosa_mi355.h``;
``capi`` binds it with ctypes and ``ops`` mirrors the reference's operator interface on top of it.
"""
from . import capi  # noqa: F401
from .capi import Context, DeviceTensor, TmiError  # noqa: F401

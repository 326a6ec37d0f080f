"""MI355X (gfx950) implementation of the TOSA reference model's tensor-op hot path.

The product is the HIP library ``libtosa_mi355.so`` behind the C ABI of ``include/tosa_mi355.h``;
``capi`` binds it with ctypes, ``build`` compiles it in-tree with hipcc, ``sut_run`` plugs the command-line
runner (``tosa_mi355_run``, the C++ mirror of the reference's operator classes under ``csrc/host``) into the
reference's conformance test runner.
"""
from . import capi  # noqa: F401
from .capi import Context, DeviceTensor, TmiError  # noqa: F401

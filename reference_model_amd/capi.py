"""ctypes binding of the C ABI declared in include/tosa_mi355.h.

The shared library is loaded from this package directory; there is no CPU fall-back: if the library is
missing or a call fails, an exception is raised.
"""
from __future__ import annotations

import ctypes
import os
from typing import Optional, Sequence

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libtosa_mi355.so")

VALID, UNPREDICTABLE, ERROR = 0, 1, 2
INT8, INT16, INT32, INT48, FP32, FP16, BF16 = 3, 4, 5, 6, 7, 8, 9
ROUND_SINGLE, ROUND_INEXACT, ROUND_DOUBLE = 1, 2, 3
FLAG_SCALE_MULTIPLIER, FLAG_SCALE_SHIFT, FLAG_SCALE_VALUE, FLAG_SCALE_RESULT, FLAG_ZP_RESULT = 1, 2, 4, 8, 16
KERNEL_AUTO, KERNEL_DIRECT, KERNEL_MFMA, KERNEL_GEMM, KERNEL_SLAB, KERNEL_POINTWISE, KERNEL_STREAM = 0, 1, 2, 3, 4, 5, 6

F64 = -64  # host-side tag of the fp64 buffers of the precise / bounds passes (not a TOSA element type)
DTYPE_SIZE = {INT8: 1, INT16: 2, INT32: 4, INT48: 8, FP32: 4, FP16: 2, BF16: 2, F64: 8}
_NP_TO_TMI = {np.dtype(np.int8): INT8, np.dtype(np.uint8): INT8, np.dtype(np.int16): INT16,
              np.dtype(np.uint16): INT16, np.dtype(np.int32): INT32, np.dtype(np.int64): INT48,
              np.dtype(np.float32): FP32,
              np.dtype(np.float16): FP16}

EXPORTS = [
    "tmi_version", "tmi_ctx_create", "tmi_ctx_destroy", "tmi_ctx_set_stream", "tmi_ctx_sync", "tmi_ctx_flags",
    "tmi_last_error", "tmi_last_kernel", "tmi_buf_alloc", "tmi_buf_free", "tmi_upload", "tmi_download",
    "tmi_conv2d", "tmi_depthwise_conv2d", "tmi_matmul", "tmi_rescale", "tmi_clamp", "tmi_conv2d_rescale_clamp",
    "tmi_depthwise_conv2d_rescale_clamp", "tmi_ctx_set_kernel_choice", "tmi_conv2d_check", "tmi_rescale_check",
    "tmi_transpose_conv2d", "tmi_conv3d", "tmi_transpose_conv2d_check", "tmi_conv3d_check",
    "tmi_avg_pool2d", "tmi_max_pool2d", "tmi_pool2d_check",
    "tmi_conv2d_precise", "tmi_depthwise_conv2d_precise", "tmi_matmul_precise", "tmi_dot_product_check",
    "tmi_ctx_reserve_workspace", "tmi_transpose_conv2d_noalloc", "tmi_ctx_set_level", "tmi_clamp_fp",
    "tmi_ctx_set_precise_mode", "tmi_ctx_workspace_bytes", "tmi_ctx_trim_workspace",
    "tmi_debug_launch_empty", "tmi_debug_tile_decode", "tmi_debug_last_launch_shape", "tmi_debug_stream",
]

NOALLOC_SCRATCH_BYTES = 16 << 20  # TMI_NOALLOC_SCRATCH_BYTES


class ConvDesc(ctypes.Structure):
    _fields_ = [
        ("in_dtype", ctypes.c_int32), ("out_dtype", ctypes.c_int32),
        ("N", ctypes.c_int32), ("IH", ctypes.c_int32), ("IW", ctypes.c_int32), ("IC", ctypes.c_int32),
        ("OC", ctypes.c_int32), ("KH", ctypes.c_int32), ("KW", ctypes.c_int32),
        ("OH", ctypes.c_int32), ("OW", ctypes.c_int32),
        ("pad", ctypes.c_int32 * 4), ("stride", ctypes.c_int32 * 2), ("dilation", ctypes.c_int32 * 2),
        ("bias_len", ctypes.c_int32), ("acc_dtype", ctypes.c_int32),
    ]


class TconvDesc(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int32) for n in ("in_dtype", "out_dtype", "N", "IH", "IW", "IC", "OC", "KH", "KW", "OH",
                                              "OW")] + [
        ("out_pad", ctypes.c_int32 * 4), ("stride", ctypes.c_int32 * 2), ("bias_len", ctypes.c_int32),
        ("acc_dtype", ctypes.c_int32)]

    def __setattr__(self, name, value):
        # the accumulator type follows the operand type unless it is set explicitly afterwards
        super().__setattr__(name, value)
        if name == "in_dtype":
            super().__setattr__("acc_dtype", INT32 if value == INT8 else (INT48 if value == INT16 else FP32))


class Conv3dDesc(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int32) for n in ("in_dtype", "out_dtype", "N", "ID", "IH", "IW", "IC", "OC", "KD", "KH",
                                              "KW", "OD", "OH", "OW")] + [
        ("pad", ctypes.c_int32 * 6), ("stride", ctypes.c_int32 * 3), ("dilation", ctypes.c_int32 * 3),
        ("bias_len", ctypes.c_int32), ("acc_dtype", ctypes.c_int32)]

    def __setattr__(self, name, value):
        super().__setattr__(name, value)
        if name == "in_dtype":
            super().__setattr__("acc_dtype", INT32 if value == INT8 else (INT48 if value == INT16 else FP32))


class PoolDesc(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int32) for n in ("dtype", "acc_dtype", "N", "IH", "IW", "C", "OH", "OW")] + [
        ("kernel", ctypes.c_int32 * 2), ("stride", ctypes.c_int32 * 2), ("pad", ctypes.c_int32 * 4),
        ("nan_mode", ctypes.c_int32)]


class Level(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int32) for n in ("max_rank", "max_kernel", "max_stride", "max_scale",
                                              "max_tensor_list_size")]


LEVEL_NONE = (0, 0, 0, 0, 0)
LEVEL_EIGHTK = (6, 8192, 8192, 256, 64)
FLAG_LEVEL = 32


class DpResult(ctypes.Structure):
    _fields_ = [("err_sum", ctypes.c_double), ("err_sumsq", ctypes.c_double), ("max_abs_err", ctypes.c_double),
                ("failed_elements", ctypes.c_int64), ("elements", ctypes.c_int64), ("abs_bound", ctypes.c_int32),
                ("variance_bound", ctypes.c_double), ("compliant", ctypes.c_int32)]


class RescaleDesc(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int32) for n in (
        "in_dtype", "out_dtype", "scale32", "rounding_mode", "per_channel", "input_unsigned", "output_unsigned",
        "in_zp", "out_zp", "n_multiplier", "n_shift")]


class TmiError(RuntimeError):
    """Raised for TMI_ERROR (the reference's TOSA_ERROR); .status holds the GraphStatus value."""

    def __init__(self, status: int, message: str):
        super().__init__(f"status {status}: {message}")
        self.status = status
        self.message = message


_lib: Optional[ctypes.CDLL] = None


def load_library() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(f"{LIB_PATH} is not built: run `python -m reference_model_amd.build` "
                          "(there is no CPU fall-back)")
    lib = ctypes.CDLL(LIB_PATH)
    vp, i32, i64 = ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64
    lib.tmi_version.restype = ctypes.c_char_p
    lib.tmi_ctx_create.argtypes = [ctypes.POINTER(vp), ctypes.c_int]
    lib.tmi_ctx_destroy.argtypes = [vp]
    lib.tmi_ctx_set_stream.argtypes = [vp, vp]
    lib.tmi_ctx_sync.argtypes = [vp]
    lib.tmi_ctx_flags.argtypes = [vp]
    lib.tmi_ctx_flags.restype = ctypes.c_uint32
    lib.tmi_last_error.argtypes = [vp]
    lib.tmi_last_error.restype = ctypes.c_char_p
    lib.tmi_last_kernel.argtypes = [vp]
    lib.tmi_last_kernel.restype = ctypes.c_char_p
    lib.tmi_ctx_set_kernel_choice.argtypes = [vp, i32]
    lib.tmi_ctx_reserve_workspace.argtypes = [vp, ctypes.c_size_t]
    lib.tmi_ctx_workspace_bytes.argtypes = [vp, ctypes.POINTER(ctypes.c_size_t), ctypes.POINTER(ctypes.c_size_t)]
    lib.tmi_ctx_trim_workspace.argtypes = [vp]
    lib.tmi_buf_alloc.argtypes = [vp, ctypes.c_size_t, ctypes.POINTER(vp)]
    lib.tmi_buf_free.argtypes = [vp, vp]
    lib.tmi_upload.argtypes = [vp, vp, vp, ctypes.c_size_t]
    lib.tmi_download.argtypes = [vp, vp, vp, ctypes.c_size_t]
    conv_args = [vp, ctypes.POINTER(ConvDesc), vp, vp, vp, i32, i32]
    lib.tmi_conv2d.argtypes = conv_args + [vp]
    lib.tmi_depthwise_conv2d.argtypes = conv_args + [vp]
    fused = conv_args + [ctypes.POINTER(RescaleDesc), vp, vp, i32, i32, i32, vp]
    lib.tmi_conv2d_rescale_clamp.argtypes = fused
    lib.tmi_depthwise_conv2d_rescale_clamp.argtypes = fused
    tconv_args = [vp, ctypes.POINTER(TconvDesc), vp, vp, vp, i32, i32, vp]
    lib.tmi_transpose_conv2d.argtypes = tconv_args
    lib.tmi_transpose_conv2d_noalloc.argtypes = tconv_args
    lib.tmi_conv3d.argtypes = [vp, ctypes.POINTER(Conv3dDesc), vp, vp, vp, i32, i32, vp]
    lib.tmi_matmul.argtypes = [vp, i32, i32, i32, i32, i32, vp, vp, i32, i32, vp]
    lib.tmi_rescale.argtypes = [vp, ctypes.POINTER(RescaleDesc), i32, i64, i32, vp, vp, vp, vp]
    lib.tmi_clamp.argtypes = [vp, i32, i64, vp, i32, i32, vp]
    lib.tmi_clamp_fp.argtypes = [vp, i32, i64, vp, ctypes.c_float, ctypes.c_float, i32, vp]
    lib.tmi_ctx_set_level.argtypes = [vp, ctypes.POINTER(Level)]
    lib.tmi_ctx_set_precise_mode.argtypes = [vp, i32, i32, i32]
    lib.tmi_debug_launch_empty.argtypes = [vp, i32, i32, i32]
    lib.tmi_debug_last_launch_shape.argtypes = [ctypes.POINTER(ctypes.c_int32)]
    lib.tmi_debug_last_launch_shape.restype = None
    lib.tmi_debug_stream.argtypes = [vp, i32, vp, vp, i64]
    lib.tmi_debug_tile_decode.argtypes = [i64, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32,
                                          ctypes.POINTER(ctypes.c_int32)]
    lib.tmi_avg_pool2d.argtypes = [vp, ctypes.POINTER(PoolDesc), vp, i32, i32, vp]
    lib.tmi_max_pool2d.argtypes = [vp, ctypes.POINTER(PoolDesc), vp, vp]
    lib.tmi_pool2d_check.argtypes = [vp, ctypes.POINTER(PoolDesc), i32]
    lib.tmi_conv2d_precise.argtypes = [vp, ctypes.POINTER(ConvDesc), vp, vp, vp, i32, i32, vp]
    lib.tmi_depthwise_conv2d_precise.argtypes = [vp, ctypes.POINTER(ConvDesc), vp, vp, vp, i32, i32, vp]
    lib.tmi_matmul_precise.argtypes = [vp, i32, i32, i32, i32, i32, vp, vp, i32, vp]
    lib.tmi_dot_product_check.argtypes = [vp, i32, i64, vp, vp, vp, i32, i32, ctypes.POINTER(DpResult)]
    lib.tmi_conv2d_check.argtypes = [vp, ctypes.POINTER(ConvDesc), i32]
    lib.tmi_rescale_check.argtypes = [vp, ctypes.POINTER(RescaleDesc), i32, i32]
    for name in EXPORTS:
        fn = getattr(lib, name)
        if fn.restype is ctypes.c_int:
            fn.restype = ctypes.c_int
    _lib = lib
    return lib


def _ptr(x) -> ctypes.c_void_p:
    """Device pointer of a DeviceTensor, a torch tensor, an int, or None."""
    if x is None:
        return ctypes.c_void_p(0)
    if isinstance(x, DeviceTensor):
        return ctypes.c_void_p(x.ptr)
    if isinstance(x, int):
        return ctypes.c_void_p(x)
    if hasattr(x, "data_ptr"):
        return ctypes.c_void_p(x.data_ptr())
    raise TypeError(f"not a device tensor: {type(x)!r}")


class DeviceTensor:
    """A packed row-major tensor in HBM owned by a Context."""

    def __init__(self, ctx: "Context", shape: Sequence[int], dtype: int, np_dtype=None):
        self.ctx, self.shape, self.dtype = ctx, tuple(int(s) for s in shape), dtype
        self.np_dtype = np.dtype(np_dtype) if np_dtype is not None else None
        self.size = int(np.prod(self.shape, dtype=np.int64)) if self.shape else 1
        self.nbytes = self.size * DTYPE_SIZE[dtype]
        self.ptr = ctx._alloc(self.nbytes)

    def numpy(self) -> np.ndarray:
        dt = self.np_dtype or {INT8: np.int8, INT16: np.int16, INT32: np.int32, INT48: np.int64, FP32: np.float32,
                               FP16: np.float16, BF16: np.uint16, F64: np.float64}[self.dtype]
        out = np.empty(self.shape, dtype=dt)
        self.ctx._check(self.ctx.lib.tmi_download(self.ctx.handle, out.ctypes.data_as(ctypes.c_void_p),
                                                  ctypes.c_void_p(self.ptr), self.nbytes))
        return out

    def free(self):
        if self.ptr:
            self.ctx._free(self.ptr)
            self.ptr = 0


class Context:
    """One device context = one stream + the latched status word (see tmi_ctx_create)."""

    def __init__(self, device: int = 0):
        self.lib = load_library()
        h = ctypes.c_void_p()
        rc = self.lib.tmi_ctx_create(ctypes.byref(h), device)
        if rc != VALID or not h.value:
            raise RuntimeError(f"tmi_ctx_create(device={device}) failed: no usable MI355X / HIP device")
        self.handle = h
        self._owned = set()

    # -- plumbing ------------------------------------------------------------------------------
    def close(self):
        if getattr(self, "handle", None):
            for p in list(self._owned):
                self._free(p)
            self.lib.tmi_ctx_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def _check(self, rc: int) -> int:
        if rc == ERROR:
            raise TmiError(rc, self.lib.tmi_last_error(self.handle).decode())
        return rc

    def _alloc(self, nbytes: int) -> int:
        p = ctypes.c_void_p()
        self._check(self.lib.tmi_buf_alloc(self.handle, nbytes, ctypes.byref(p)))
        self._owned.add(p.value)
        return p.value

    def _free(self, ptr: int):
        self._owned.discard(ptr)
        self._check(self.lib.tmi_buf_free(self.handle, ctypes.c_void_p(ptr)))

    def set_stream(self, hip_stream: int):
        self._check(self.lib.tmi_ctx_set_stream(self.handle, ctypes.c_void_p(hip_stream)))

    def set_kernel_choice(self, choice: int):
        self._check(self.lib.tmi_ctx_set_kernel_choice(self.handle, choice))

    def sync(self) -> int:
        """Waits for the stream; returns VALID or UNPREDICTABLE (a RESCALE REQUIRE condition fired)."""
        return self._check(self.lib.tmi_ctx_sync(self.handle))

    @property
    def flags(self) -> int:
        return int(self.lib.tmi_ctx_flags(self.handle))

    @property
    def last_kernel(self) -> str:
        return self.lib.tmi_last_kernel(self.handle).decode()

    def empty(self, shape, dtype: int, np_dtype=None) -> DeviceTensor:
        return DeviceTensor(self, shape, dtype, np_dtype)

    def upload(self, array: np.ndarray, dtype: Optional[int] = None) -> DeviceTensor:
        a = np.ascontiguousarray(array)
        t = DeviceTensor(self, a.shape, dtype if dtype is not None else _NP_TO_TMI[a.dtype], a.dtype)
        self._check(self.lib.tmi_upload(self.handle, ctypes.c_void_p(t.ptr), a.ctypes.data_as(ctypes.c_void_p),
                                        a.nbytes))
        return t

    # -- descriptors ---------------------------------------------------------------------------
    @staticmethod
    def conv_desc(in_dtype, out_dtype, in_shape, oc, kh, kw, out_hw, pad, stride, dilation, bias_len,
                  acc_dtype=None) -> ConvDesc:
        d = ConvDesc()
        d.acc_dtype = acc_dtype if acc_dtype is not None else (INT32 if in_dtype == INT8 else (INT48 if in_dtype == INT16 else FP32))
        d.in_dtype, d.out_dtype = in_dtype, out_dtype
        d.N, d.IH, d.IW, d.IC = in_shape
        d.OC, d.KH, d.KW = oc, kh, kw
        d.OH, d.OW = out_hw
        d.pad[:] = list(pad)
        d.stride[:] = list(stride)
        d.dilation[:] = list(dilation)
        d.bias_len = bias_len
        return d

    @staticmethod
    def rescale_desc(in_dtype, out_dtype, n_multiplier, n_shift, in_zp=0, out_zp=0, scale32=True,
                     rounding_mode=ROUND_DOUBLE, per_channel=True, input_unsigned=False,
                     output_unsigned=False) -> RescaleDesc:
        r = RescaleDesc()
        r.in_dtype, r.out_dtype = in_dtype, out_dtype
        r.scale32, r.rounding_mode, r.per_channel = int(scale32), int(rounding_mode), int(per_channel)
        r.input_unsigned, r.output_unsigned = int(input_unsigned), int(output_unsigned)
        r.in_zp, r.out_zp = _stored(in_zp, in_dtype), _stored(out_zp, out_dtype)
        r.n_multiplier, r.n_shift = n_multiplier, n_shift
        return r

    # -- operators (device pointers in, status out) ------------------------------------------
    def conv2d(self, d: ConvDesc, inp, w, bias, in_zp, w_zp, out) -> int:
        return self._check(self.lib.tmi_conv2d(self.handle, ctypes.byref(d), _ptr(inp), _ptr(w), _ptr(bias),
                                               in_zp, w_zp, _ptr(out)))

    def transpose_conv2d(self, d: TconvDesc, inp, w, bias, in_zp, w_zp, out) -> int:
        return self._check(self.lib.tmi_transpose_conv2d(self.handle, ctypes.byref(d), _ptr(inp), _ptr(w),
                                                         _ptr(bias), in_zp, w_zp, _ptr(out)))

    def transpose_conv2d_noalloc(self, d: TconvDesc, inp, w, bias, in_zp, w_zp, out) -> int:
        return self._check(self.lib.tmi_transpose_conv2d_noalloc(self.handle, ctypes.byref(d), _ptr(inp), _ptr(w),
                                                                 _ptr(bias), in_zp, w_zp, _ptr(out)))

    def workspace_bytes(self):
        """(bytes of the scratch buffer in use, bytes of the outgrown blocks still held)"""
        live, retired = ctypes.c_size_t(0), ctypes.c_size_t(0)
        self._check(self.lib.tmi_ctx_workspace_bytes(self.handle, ctypes.byref(live), ctypes.byref(retired)))
        return live.value, retired.value

    def trim_workspace(self) -> int:
        return self._check(self.lib.tmi_ctx_trim_workspace(self.handle))

    def reserve_workspace(self, nbytes: int) -> int:
        return self._check(self.lib.tmi_ctx_reserve_workspace(self.handle, nbytes))

    def conv2d_precise(self, d: ConvDesc, inp, w, bias, bounds_mode, out, depthwise=False, local_bound=True) -> int:
        fn = self.lib.tmi_depthwise_conv2d_precise if depthwise else self.lib.tmi_conv2d_precise
        return self._check(fn(self.handle, ctypes.byref(d), _ptr(inp), _ptr(w), _ptr(bias), int(bounds_mode),
                              int(local_bound), _ptr(out)))

    def matmul_precise(self, in_dtype, n, h, c, w, a, b, bounds_mode, out) -> int:
        return self._check(self.lib.tmi_matmul_precise(self.handle, in_dtype, n, h, c, w, _ptr(a), _ptr(b),
                                                       int(bounds_mode), _ptr(out)))

    def dot_product_check(self, out_dtype, n, imp, ref, bnd, ksb, set_number=-1) -> DpResult:
        r = DpResult()
        self._check(self.lib.tmi_dot_product_check(self.handle, out_dtype, n, _ptr(imp), _ptr(ref), _ptr(bnd), ksb,
                                                   set_number, ctypes.byref(r)))
        return r

    def avg_pool2d(self, d: PoolDesc, inp, in_zp, out_zp, out) -> int:
        return self._check(self.lib.tmi_avg_pool2d(self.handle, ctypes.byref(d), _ptr(inp), in_zp, out_zp, _ptr(out)))

    def max_pool2d(self, d: PoolDesc, inp, out) -> int:
        return self._check(self.lib.tmi_max_pool2d(self.handle, ctypes.byref(d), _ptr(inp), _ptr(out)))

    def conv3d(self, d: Conv3dDesc, inp, w, bias, in_zp, w_zp, out) -> int:
        return self._check(self.lib.tmi_conv3d(self.handle, ctypes.byref(d), _ptr(inp), _ptr(w), _ptr(bias),
                                               in_zp, w_zp, _ptr(out)))

    def depthwise_conv2d(self, d: ConvDesc, inp, w, bias, in_zp, w_zp, out) -> int:
        return self._check(self.lib.tmi_depthwise_conv2d(self.handle, ctypes.byref(d), _ptr(inp), _ptr(w),
                                                         _ptr(bias), in_zp, w_zp, _ptr(out)))

    def conv2d_rescale_clamp(self, d, inp, w, bias, in_zp, w_zp, r: RescaleDesc, mult, shift, out,
                             clamp=None) -> int:
        lo, hi = clamp if clamp is not None else (0, 0)
        return self._check(self.lib.tmi_conv2d_rescale_clamp(
            self.handle, ctypes.byref(d), _ptr(inp), _ptr(w), _ptr(bias), in_zp, w_zp, ctypes.byref(r), _ptr(mult),
            _ptr(shift), int(clamp is not None), lo, hi, _ptr(out)))

    def depthwise_conv2d_rescale_clamp(self, d, inp, w, bias, in_zp, w_zp, r: RescaleDesc, mult, shift, out,
                                       clamp=None) -> int:
        lo, hi = clamp if clamp is not None else (0, 0)
        return self._check(self.lib.tmi_depthwise_conv2d_rescale_clamp(
            self.handle, ctypes.byref(d), _ptr(inp), _ptr(w), _ptr(bias), in_zp, w_zp, ctypes.byref(r), _ptr(mult),
            _ptr(shift), int(clamp is not None), lo, hi, _ptr(out)))

    def matmul(self, in_dtype, n, h, c, w, a, b, a_zp, b_zp, out) -> int:
        return self._check(self.lib.tmi_matmul(self.handle, in_dtype, n, h, c, w, _ptr(a), _ptr(b), a_zp, b_zp,
                                               _ptr(out)))

    def rescale(self, r: RescaleDesc, rank, rows, c, inp, mult, shift, out) -> int:
        return self._check(self.lib.tmi_rescale(self.handle, ctypes.byref(r), rank, rows, c, _ptr(inp), _ptr(mult),
                                                _ptr(shift), _ptr(out)))

    def clamp(self, dtype, n, inp, lo, hi, out) -> int:
        return self._check(self.lib.tmi_clamp(self.handle, dtype, n, _ptr(inp), lo, hi, _ptr(out)))

    def clamp_fp(self, dtype, n, inp, lo, hi, nan_mode, out) -> int:
        return self._check(self.lib.tmi_clamp_fp(self.handle, dtype, n, _ptr(inp), float(lo), float(hi), int(nan_mode),
                                                 _ptr(out)))

    def stream_probe(self, mode, src, dst, nbytes) -> int:
        return self._check(self.lib.tmi_debug_stream(self.handle, mode, _ptr(src), _ptr(dst), nbytes))

    def last_launch_shape(self):
        out = (ctypes.c_int32 * 3)()
        self.lib.tmi_debug_last_launch_shape(out)
        return tuple(out)

    def launch_empty(self, grid, block, lds_bytes) -> int:
        return self._check(self.lib.tmi_debug_launch_empty(self.handle, grid, block, lds_bytes))

    def set_precise_mode(self, precise=False, compliance=False, bounds=False):
        """g_func_config.precise_mode / compliance_mode / bounds_mode as RESCALE's INEXACT_ROUND reads them"""
        self._check(self.lib.tmi_ctx_set_precise_mode(self.handle, int(precise), int(compliance), int(bounds)))

    def set_level(self, level=LEVEL_NONE):
        lv = Level(*level)
        self._check(self.lib.tmi_ctx_set_level(self.handle, ctypes.byref(lv)))


def _stored(zp: int, dtype: int) -> int:
    """Stored (sign-interpreted) value of a zero point given as a mathematical integer."""
    bits = 8 * DTYPE_SIZE[dtype]
    zp = int(zp) & ((1 << bits) - 1)
    return zp - (1 << bits) if zp >= (1 << (bits - 1)) else zp

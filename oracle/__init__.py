"""CPU oracle for the TOSA tensor-op hot path -- TEST INFRASTRUCTURE ONLY.

numpy front end of ``libtosa_oracle.so`` (``tosa_oracle.c``), the plain-C restatement of the TOSA
reference model's CONV2D / DEPTHWISE_CONV2D / MATMUL / RESCALE / CLAMP (and CONV3D / TRANSPOSE_CONV2D) arithmetic.  Only the tests,
the smoke test and the benchmark's CPU-baseline leg may import this package; the shipped library
never does.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libtosa_oracle.so")
_LIB_OMP_PATH = os.path.join(_HERE, "libtosa_oracle_omp.so")   # the same source built with -fopenmp (all host cores)

VALID, UNPREDICTABLE, ERROR = 0, 1, 2
ROUND_SINGLE, ROUND_INEXACT, ROUND_DOUBLE = 1, 2, 3


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (make).  Returns the path of the shared object."""
    if force:
        subprocess.check_call(["make", "-C", _HERE, "clean"], stdout=subprocess.DEVNULL)
    subprocess.check_call(["make", "-C", _HERE], stdout=subprocess.DEVNULL)
    return _LIB_PATH


class ConvShape(ctypes.Structure):
    _fields_ = [
        ("N", ctypes.c_int32), ("IH", ctypes.c_int32), ("IW", ctypes.c_int32), ("IC", ctypes.c_int32),
        ("OC", ctypes.c_int32), ("KH", ctypes.c_int32), ("KW", ctypes.c_int32),
        ("OH", ctypes.c_int32), ("OW", ctypes.c_int32),
        ("pad", ctypes.c_int32 * 4), ("stride", ctypes.c_int32 * 2), ("dilation", ctypes.c_int32 * 2),
        ("bias_len", ctypes.c_int32),
    ]


class RescaleAttr(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int32) for n in (
        "in_bits", "out_bits", "scale32", "rounding_mode", "per_channel",
        "input_unsigned", "output_unsigned", "in_zp", "out_zp")]


_libs = {}
_parallel = False


def set_parallel(on: bool) -> None:
    """Selects the OpenMP build (CONV2D / DEPTHWISE_CONV2D / MATMUL loops over all host cores) for the calls that
    follow; the scalar build, which is the reference-equivalent single-threaded path, is the default."""
    global _parallel
    _parallel = bool(on)


def threads() -> int:
    """host threads the selected build runs CONV2D / DEPTHWISE_CONV2D / MATMUL on"""
    return int(lib().orc_threads())


def lib() -> ctypes.CDLL:
    path = _LIB_OMP_PATH if _parallel else _LIB_PATH
    if path not in _libs:
        if not os.path.exists(path):
            build()
        L = ctypes.CDLL(path)
        L.orc_apply_scale_32.restype = ctypes.c_int32
        L.orc_apply_scale_32.argtypes = [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_int,
                                         ctypes.POINTER(ctypes.c_int)]
        L.orc_apply_scale_16.restype = ctypes.c_int32
        L.orc_apply_scale_16.argtypes = [ctypes.c_int64, ctypes.c_int16, ctypes.c_int32,
                                         ctypes.POINTER(ctypes.c_int)]
        _libs[path] = L
    return _libs[path]


def _ptr(a: np.ndarray):
    return a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dtype) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(a), dtype=dtype)


def conv_out_hw(ih, iw, kh, kw, pad, stride, dilation):
    """Output height/width rule of check_conv_attribute (tensor_ops.cpp:203-223); None if inexact."""
    fh = ih - 1 + pad[0] + pad[1] - (kh - 1) * dilation[0]
    fw = iw - 1 + pad[2] + pad[3] - (kw - 1) * dilation[1]
    if stride[0] < 1 or stride[1] < 1 or fh % stride[0] or fw % stride[1] or fh < 0 or fw < 0:
        return None
    return fh // stride[0] + 1, fw // stride[1] + 1


def _shape(inp, kh, kw, oc, bias, pad, stride, dilation, out_hw=None) -> ConvShape:
    n, ih, iw, ic = inp.shape
    if out_hw is None:
        out_hw = conv_out_hw(ih, iw, kh, kw, pad, stride, dilation) or (-1, -1)
    s = ConvShape()
    s.N, s.IH, s.IW, s.IC = n, ih, iw, ic
    s.OC, s.KH, s.KW = oc, kh, kw
    s.OH, s.OW = out_hw
    s.pad[:] = list(pad)
    s.stride[:] = list(stride)
    s.dilation[:] = list(dilation)
    s.bias_len = int(np.asarray(bias).shape[0])
    return s


class OracleStatus(Exception):
    def __init__(self, status):
        super().__init__(f"oracle status {status}")
        self.status = status


def _check(rc, allow=(VALID,)):
    if rc not in allow:
        raise OracleStatus(rc)
    return rc


_KINDS = {
    "i8": (np.int8, np.int32, np.int32),      # element dtype, bias dtype, output dtype
    "i32": (np.int32, np.int32, np.int32),
    "i16": (np.int16, np.int64, np.int64),    # INT16 x INT8 (MATMUL: x INT16) -> INT48 in its int64 storage
    "f32": (np.float32, np.float32, np.float32),
    "f64": (np.float64, np.float64, np.float64),
}


def _abs_code(abs_mode, local_bound):
    """0: ordinary pass; 1: bounds pass (absolute values); 2: bounds pass of an operator whose local_bound attribute
    is false: the input is replaced by its largest magnitude (tensor_ops.cpp:797-801, 1252-1256)."""
    return 0 if not abs_mode else (1 if local_bound else 2)


def conv2d(kind, inp, w, bias, pad=(0, 0, 0, 0), stride=(1, 1), dilation=(1, 1), in_zp=0, w_zp=0,
           abs_mode=False, out_hw=None, local_bound=True):
    """CONV2D.  inp NHWC, w OHWI, bias [1] or [OC].  kind in i8/i32/i16/f32/f64 (i16: INT8 weights, INT48 results)."""
    et, bt, ot = _KINDS[kind]
    inp, w, bias = _c(inp, et), _c(w, np.int8 if kind == "i16" else et), _c(bias, bt)
    oc, kh, kw, _ = w.shape
    s = _shape(inp, kh, kw, oc, bias, pad, stride, dilation, out_hw)
    if w.shape[3] != inp.shape[3]:
        raise OracleStatus(ERROR)
    out = np.zeros((s.N, max(s.OH, 0), max(s.OW, 0), oc), dtype=ot)
    L = lib()
    if kind in ("i8", "i32", "i16"):
        fn = {"i8": L.orc_conv2d_i8, "i32": L.orc_conv2d_i32, "i16": L.orc_conv2d_i16}[kind]
        rc = fn(ctypes.byref(s), _ptr(inp), _ptr(w), _ptr(bias), ctypes.c_int32(in_zp), ctypes.c_int32(w_zp),
                _ptr(out))
    elif kind == "f32":
        rc = L.orc_conv2d_f32(ctypes.byref(s), _ptr(inp), _ptr(w), _ptr(bias), _ptr(out))
    else:
        rc = L.orc_conv2d_f64(ctypes.byref(s), _ptr(inp), _ptr(w), _ptr(bias),
                              ctypes.c_int(_abs_code(abs_mode, local_bound)), _ptr(out))
    _check(rc)
    return out


def depthwise_conv2d(kind, inp, w, bias, pad=(0, 0, 0, 0), stride=(1, 1), dilation=(1, 1), in_zp=0, w_zp=0,
                     abs_mode=False, out_hw=None, local_bound=True):
    """DEPTHWISE_CONV2D.  inp NHWC, w [KH,KW,C,M], bias [1] or [C*M]."""
    et, bt, ot = _KINDS[kind]
    inp, w, bias = _c(inp, et), _c(w, np.int8 if kind == "i16" else et), _c(bias, bt)
    kh, kw, c, m = w.shape
    if c != inp.shape[3]:
        raise OracleStatus(ERROR)
    s = _shape(inp, kh, kw, c * m, bias, pad, stride, dilation, out_hw)
    out = np.zeros((s.N, max(s.OH, 0), max(s.OW, 0), c * m), dtype=ot)
    L = lib()
    if kind in ("i8", "i32", "i16"):
        fn = {"i8": L.orc_depthwise_i8, "i32": L.orc_depthwise_i32, "i16": L.orc_depthwise_i16}[kind]
        rc = fn(ctypes.byref(s), ctypes.c_int32(m), _ptr(inp), _ptr(w), _ptr(bias), ctypes.c_int32(in_zp),
                ctypes.c_int32(w_zp), _ptr(out))
    elif kind == "f32":
        rc = L.orc_depthwise_f32(ctypes.byref(s), ctypes.c_int32(m), _ptr(inp), _ptr(w), _ptr(bias), _ptr(out))
    else:
        rc = L.orc_depthwise_f64(ctypes.byref(s), ctypes.c_int32(m), _ptr(inp), _ptr(w), _ptr(bias),
                                 ctypes.c_int(_abs_code(abs_mode, local_bound)), _ptr(out))
    _check(rc)
    return out


class Conv3dShape(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int32) for n in ("N", "ID", "IH", "IW", "IC", "OC", "KD", "KH", "KW", "OD", "OH", "OW")] + [
        ("pad", ctypes.c_int32 * 6), ("stride", ctypes.c_int32 * 3), ("dilation", ctypes.c_int32 * 3),
        ("bias_len", ctypes.c_int32)]


class TconvShape(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int32) for n in ("N", "IH", "IW", "IC", "OC", "KH", "KW", "OH", "OW")] + [
        ("out_pad", ctypes.c_int32 * 4), ("stride", ctypes.c_int32 * 2), ("bias_len", ctypes.c_int32)]


def conv3d_out_dhw(idhw, kdhw, pad, stride, dilation):
    """Output depth/height/width rule of check_conv_attribute for three dimensions; None if inexact."""
    out = []
    for i in range(3):
        full = idhw[i] - 1 + pad[2 * i] + pad[2 * i + 1] - (kdhw[i] - 1) * dilation[i]
        if stride[i] < 1 or full < 0 or full % stride[i]:
            return None
        out.append(full // stride[i] + 1)
    return tuple(out)


def _dispatch(prefix, kind, s, inp, w, bias, in_zp, w_zp, abs_mode, out):
    L = lib()
    if kind in ("i8", "i32", "i16"):
        rc = getattr(L, f"{prefix}_{kind}")(ctypes.byref(s), _ptr(inp), _ptr(w), _ptr(bias), ctypes.c_int32(in_zp),
                                            ctypes.c_int32(w_zp), _ptr(out))
    elif kind == "f32":
        rc = getattr(L, f"{prefix}_f32")(ctypes.byref(s), _ptr(inp), _ptr(w), _ptr(bias), _ptr(out))
    else:
        rc = getattr(L, f"{prefix}_f64")(ctypes.byref(s), _ptr(inp), _ptr(w), _ptr(bias),
                                         ctypes.c_int(int(abs_mode)), _ptr(out))
    _check(rc)
    return out


def conv3d(kind, inp, w, bias, pad=(0,) * 6, stride=(1, 1, 1), dilation=(1, 1, 1), in_zp=0, w_zp=0,
           abs_mode=False, out_dhw=None):
    """CONV3D.  inp [N,D,H,W,C], w [OC,KD,KH,KW,C], bias [1] or [OC].  kind i16: INT8 weights, INT48 results."""
    et, bt, ot = _KINDS[kind]
    inp, w, bias = _c(inp, et), _c(w, np.int8 if kind == "i16" else et), _c(bias, bt)
    if w.shape[4] != inp.shape[4]:
        raise OracleStatus(ERROR)
    if out_dhw is None:
        out_dhw = conv3d_out_dhw(inp.shape[1:4], w.shape[1:4], pad, stride, dilation) or (-1, -1, -1)
    s = Conv3dShape()
    s.N, s.ID, s.IH, s.IW, s.IC = inp.shape
    s.OC, s.KD, s.KH, s.KW = w.shape[:4]
    s.OD, s.OH, s.OW = out_dhw
    s.pad[:], s.stride[:], s.dilation[:] = list(pad), list(stride), list(dilation)
    s.bias_len = int(bias.shape[0])
    out = np.zeros((s.N,) + tuple(max(v, 0) for v in out_dhw) + (s.OC,), dtype=ot)
    return _dispatch("orc_conv3d", kind, s, inp, w, bias, in_zp, w_zp, abs_mode, out)


def transpose_conv2d(kind, inp, w, bias, out_pad=(0, 0, 0, 0), stride=(1, 1), in_zp=0, w_zp=0, abs_mode=False,
                     out_hw=None):
    """TRANSPOSE_CONV2D.  inp NHWC, w OHWI, bias [1] or [OC].  kind i16: INT8 weights, INT48 results."""
    et, bt, ot = _KINDS[kind]
    inp, w, bias = _c(inp, et), _c(w, np.int8 if kind == "i16" else et), _c(bias, bt)
    if w.shape[3] != inp.shape[3]:
        raise OracleStatus(ERROR)
    n, ih, iw, ic = inp.shape
    oc, kh, kw, _ = w.shape
    if out_hw is None:
        out_hw = ((ih - 1) * stride[0] + out_pad[0] + out_pad[1] + kh, (iw - 1) * stride[1] + out_pad[2] + out_pad[3] + kw)
    s = TconvShape()
    s.N, s.IH, s.IW, s.IC, s.OC, s.KH, s.KW = n, ih, iw, ic, oc, kh, kw
    s.OH, s.OW = out_hw
    s.out_pad[:], s.stride[:] = list(out_pad), list(stride)
    s.bias_len = int(bias.shape[0])
    out = np.zeros((n, max(out_hw[0], 0), max(out_hw[1], 0), oc), dtype=ot)
    return _dispatch("orc_transpose_conv2d", kind, s, inp, w, bias, in_zp, w_zp, abs_mode, out)


def matmul(kind, a, b, a_zp=0, b_zp=0, abs_mode=False):
    """MATMUL a[N,H,C] x b[N,C,W] -> [N,H,W]."""
    et, _, ot = _KINDS[kind]
    a, b = _c(a, et), _c(b, et)
    n, h, c = a.shape
    if b.shape[0] != n or b.shape[1] != c:
        raise OracleStatus(ERROR)
    w = b.shape[2]
    out = np.zeros((n, h, w), dtype=ot)
    L = lib()
    dims = [ctypes.c_int32(v) for v in (n, h, c, w)]
    if kind in ("i8", "i32", "i16"):
        fn = {"i8": L.orc_matmul_i8, "i32": L.orc_matmul_i32, "i16": L.orc_matmul_i16}[kind]
        rc = fn(*dims, _ptr(a), _ptr(b), ctypes.c_int32(a_zp), ctypes.c_int32(b_zp), _ptr(out))
    elif kind == "f32":
        rc = L.orc_matmul_f32(*dims, _ptr(a), _ptr(b), _ptr(out))
    else:
        rc = L.orc_matmul_f64(*dims, _ptr(a), _ptr(b), ctypes.c_int(int(abs_mode)), _ptr(out))
    _check(rc)
    return out


def apply_scale_32(value, multiplier, shift, double_round=True):
    """Returns (result, status)."""
    st = ctypes.c_int(VALID)
    r = lib().orc_apply_scale_32(int(value), int(multiplier), int(shift), int(bool(double_round)), ctypes.byref(st))
    return int(r), st.value


def apply_scale_16(value, multiplier, shift):
    st = ctypes.c_int(VALID)
    r = lib().orc_apply_scale_16(int(value), int(multiplier), int(shift), ctypes.byref(st))
    return int(r), st.value


_BITS = {np.dtype(np.int8): 8, np.dtype(np.uint8): 8, np.dtype(np.int16): 16, np.dtype(np.uint16): 16,
         np.dtype(np.int32): 32, np.dtype(np.int64): 48}     # int64 is the storage of INT48


def rescale(inp, multiplier, shift, in_zp=0, out_zp=0, out_dtype=np.int8, scale32=True,
            rounding_mode=ROUND_DOUBLE, per_channel=True, input_unsigned=False, output_unsigned=False, inexact_mode=0):
    """RESCALE.  Returns (out, status); out has dtype out_dtype (bit pattern of the stored value).
    inexact_mode: how INEXACT_ROUND is evaluated (0 FP32; 1 precise mode; 2 / 3 precise + compliance, normal / bounds pass)."""
    inp = np.asarray(inp)
    out_dtype = np.dtype(out_dtype)
    a = RescaleAttr()
    a.in_bits, a.out_bits = _BITS[inp.dtype], _BITS[out_dtype]
    a.scale32, a.rounding_mode, a.per_channel = int(scale32), int(rounding_mode), int(per_channel)
    a.input_unsigned, a.output_unsigned = int(input_unsigned), int(output_unsigned)
    # the zero-point tensors hold the stored (sign-interpreted) value of their dtype
    a.in_zp = int(np.array(in_zp).astype(np.int64).astype(_signed(inp.dtype)))
    a.out_zp = int(np.array(out_zp).astype(np.int64).astype(_signed(out_dtype)))
    rank = inp.ndim
    C = inp.shape[-1] if rank > 0 else 1
    rows = int(np.prod(inp.shape[:-1], dtype=np.int64)) if rank > 0 else 1
    i48 = a.in_bits == 48
    stored = _c(inp.view(_signed(inp.dtype)) if inp.dtype.kind == "u" else inp, np.int64 if i48 else np.int32)
    mult = _c(np.atleast_1d(multiplier), np.int32)
    sh = _c(np.atleast_1d(shift), np.int32)
    out = np.zeros(inp.shape, dtype=np.int32)
    fn = lib().orc_rescale_i48 if i48 else lib().orc_rescale
    lib().orc_set_inexact_mode(ctypes.c_int(int(inexact_mode)))
    rc = fn(ctypes.byref(a), ctypes.c_int64(rows), ctypes.c_int32(C), _ptr(stored), _ptr(mult),
            _ptr(sh), ctypes.c_int32(mult.size), ctypes.c_int32(sh.size), ctypes.c_int32(rank), _ptr(out))
    lib().orc_set_inexact_mode(ctypes.c_int(0))
    # narrow to the output dtype keeping the low bits (uint16 32832 is stored as such)
    narrowed = out.astype(np.int64).astype(_signed(out_dtype), casting="unsafe") if out_dtype.kind != "u" else \
        (out.astype(np.int64) & ((1 << (8 * out_dtype.itemsize)) - 1)).astype(out_dtype)
    return narrowed, rc


def _signed(dt):
    dt = np.dtype(dt)
    return {1: np.int8, 2: np.int16, 4: np.int32, 8: np.int64}[dt.itemsize]


def clamp(inp, lo, hi, nan_mode=1):
    """CLAMP; integer dtypes go through the int32 storage path, floats through float32 storage."""
    inp = np.asarray(inp)
    if inp.dtype.kind in "iu":
        x = _c(inp, np.int32)
        out = np.zeros_like(x)
        rc = lib().orc_clamp_i32(ctypes.c_int64(x.size), _ptr(x), ctypes.c_int32(int(lo)), ctypes.c_int32(int(hi)),
                                 _ptr(out))
        _check(rc)
        return out.astype(inp.dtype)
    x = _c(inp, np.float32)
    out = np.zeros_like(x)
    rc = lib().orc_clamp_f32(ctypes.c_int64(x.size), _ptr(x), ctypes.c_float(lo), ctypes.c_float(hi),
                             ctypes.c_int(nan_mode), _ptr(out))
    _check(rc)
    return out.astype(inp.dtype)


class PoolShape(ctypes.Structure):
    _fields_ = [
        ("N", ctypes.c_int32), ("IH", ctypes.c_int32), ("IW", ctypes.c_int32), ("C", ctypes.c_int32),
        ("OH", ctypes.c_int32), ("OW", ctypes.c_int32),
        ("kernel", ctypes.c_int32 * 2), ("stride", ctypes.c_int32 * 2), ("pad", ctypes.c_int32 * 4),
    ]


def pool_out_hw(ih, iw, kernel, stride, pad):
    """Output size the attribute check accepts (tensor_ops.cpp:100-113), or None when there is none."""
    fh, fw = ih + pad[0] + pad[1] - kernel[0], iw + pad[2] + pad[3] - kernel[1]
    if fh < 0 or fw < 0 or fh % stride[0] or fw % stride[1]:
        return None
    return fh // stride[0] + 1, fw // stride[1] + 1


def _pool_shape(inp, kernel, stride, pad, out_hw):
    n, ih, iw, c = inp.shape
    if out_hw is None:
        out_hw = pool_out_hw(ih, iw, kernel, stride, pad) or (0, 0)
    return PoolShape(n, ih, iw, c, out_hw[0], out_hw[1], (ctypes.c_int32 * 2)(*kernel), (ctypes.c_int32 * 2)(*stride),
                     (ctypes.c_int32 * 4)(*pad))


def reciprocal_scale(count):
    m, s = ctypes.c_int32(), ctypes.c_int32()
    lib().orc_reciprocal_scale(ctypes.c_int32(count), ctypes.byref(m), ctypes.byref(s))
    return m.value, s.value


def avg_pool2d(inp, kernel, stride=(1, 1), pad=(0, 0, 0, 0), in_zp=0, out_zp=0, out_hw=None):
    """AVG_POOL2D.  int8 / int16 input: int32 accumulator, result of the input type.  float32 input (holding
    fp16 / bf16 / fp32 values): fp32 accumulator, fp32 result for the caller to narrow."""
    inp = np.asarray(inp)
    s = _pool_shape(inp, kernel, stride, pad, out_hw)
    shape = (s.N, max(s.OH, 0), max(s.OW, 0), s.C)
    if inp.dtype != np.int8 and (in_zp != 0 or out_zp != 0):
        raise OracleStatus(ERROR)    # zero points belong to int8 only (tensor_ops.cpp:568-571)
    if inp.dtype.kind == "i":
        info = np.iinfo(inp.dtype)
        x, out = _c(inp, np.int32), np.zeros(shape, np.int32)
        rc = lib().orc_avg_pool2d_i32(ctypes.byref(s), _ptr(x), ctypes.c_int32(in_zp), ctypes.c_int32(out_zp),
                                      ctypes.c_int32(int(info.min)), ctypes.c_int32(int(info.max)), _ptr(out))
        _check(rc)
        return out.astype(inp.dtype)
    x, out = _c(inp, np.float32), np.zeros(shape, np.float32)
    _check(lib().orc_avg_pool2d_f32(ctypes.byref(s), _ptr(x), _ptr(out)))
    return out


def max_pool2d(inp, kernel, stride=(1, 1), pad=(0, 0, 0, 0), nan_mode=1, out_hw=None):
    """MAX_POOL2D on int8 / int16 (padding = lowest value of the type) or float32 storage (nan_mode 1 = PROPAGATE,
    2 = IGNORE)."""
    inp = np.asarray(inp)
    s = _pool_shape(inp, kernel, stride, pad, out_hw)
    shape = (s.N, max(s.OH, 0), max(s.OW, 0), s.C)
    if inp.dtype.kind == "i":
        x, out = _c(inp, np.int32), np.zeros(shape, np.int32)
        _check(lib().orc_max_pool2d_i32(ctypes.byref(s), _ptr(x), ctypes.c_int32(int(np.iinfo(inp.dtype).min)), _ptr(out)))
        return out.astype(inp.dtype)
    x, out = _c(inp, np.float32), np.zeros(shape, np.float32)
    _check(lib().orc_max_pool2d_f32(ctypes.byref(s), _ptr(x), ctypes.c_int(nan_mode), _ptr(out)))
    return out


_DP_OPS = {"matmul": 0, "conv2d": 1, "depthwise": 2}
_DP_KINDS = {"fp16": 16, "bf16": 17, "fp32": 32}


def dot_product_data(op, data_set, param, ks, shape, kind="fp32", kernel=None, acc16=False):
    """The DOT_PRODUCT test data set `data_set` (0..5) for operand `param` of `op` ("matmul", "conv2d",
    "depthwise"), as float32 values; kind selects the bound parameter B of the operand type."""
    L = lib()
    L.orc_dp_bound_parameter.restype = ctypes.c_float
    B = L.orc_dp_bound_parameter(ctypes.c_int(_DP_KINDS[kind]), ctypes.c_int(int(acc16)))
    out = np.zeros(shape, np.float32)
    shp = (ctypes.c_int32 * len(shape))(*shape)
    ker = (ctypes.c_int32 * 2)(*kernel) if kernel is not None else None
    rc = L.orc_dp_generate(ctypes.c_int(_DP_OPS[op]), ctypes.c_int(data_set), ctypes.c_int(param), ctypes.c_uint32(ks),
                           ctypes.c_float(B), shp, ctypes.c_int(len(shape)), ker, _ptr(out))
    _check(rc)
    return out

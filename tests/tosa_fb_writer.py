"""Minimal FlatBuffers *writer* for TOSA 1.x graphs, for the tests only: builds small graphs (CONV2D,
DEPTHWISE_CONV2D, MATMUL, RESCALE, CLAMP, CONST) that the host runner loads like a file produced by the
reference's serialization library.  Objects are laid out top-down: every offset points forward, each vtable
sits right in front of its table.  Field numbers: see tosa_flatbuffer.py."""
from __future__ import annotations

import struct

import numpy as np

DTYPE_CODE = {np.dtype(np.int8): 3, np.dtype(np.int16): 4, np.dtype(np.int32): 5, np.dtype(np.int64): 6,
              np.dtype(np.float32): 7,
              np.dtype(np.float16): 8}


class _Ref:
    """A child object (table, string or vector) referenced through a forward uoffset."""

    def __init__(self, kind, value, fmt=None):
        self.kind, self.value, self.fmt = kind, value, fmt


def table(fields):
    """fields: list of (index, fmt_or_None, value); fmt is a struct char for scalars, None for children."""
    return _Ref("table", fields)


def string(s):
    return _Ref("string", s)


def vector(fmt, values):
    return _Ref("vector", list(values), fmt)


def vector_of(children):
    return _Ref("refvector", list(children))


class Writer:
    def __init__(self):
        self.buf = bytearray()

    def _align(self, n):
        while len(self.buf) % n:
            self.buf.append(0)

    def _emit(self, ref: _Ref) -> int:
        """Appends the object and (recursively) its children; returns the object's position."""
        if ref.kind == "string":
            self._align(4)
            pos = len(self.buf)
            raw = ref.value.encode()
            self.buf += struct.pack("<I", len(raw)) + raw + b"\0"
            return pos
        if ref.kind == "vector":
            size = struct.calcsize("<" + ref.fmt)
            self._align(4)
            if size == 8 or ref.fmt == "B":
                while (len(self.buf) + 4) % 8:  # payload 8-byte aligned, as the serialization library forces
                    self.buf.append(0)
            pos = len(self.buf)
            self.buf += struct.pack("<I", len(ref.value))
            self.buf += struct.pack("<%d%s" % (len(ref.value), ref.fmt), *ref.value)
            return pos
        if ref.kind == "refvector":
            self._align(4)
            pos = len(self.buf)
            self.buf += struct.pack("<I", len(ref.value)) + b"\0" * (4 * len(ref.value))
            for i, child in enumerate(ref.value):
                cpos = self._emit(child)
                slot = pos + 4 + 4 * i
                struct.pack_into("<I", self.buf, slot, cpos - slot)
            return pos
        # table: vtable then inline fields, children afterwards
        fields = sorted(ref.value, key=lambda f: f[0])
        nslots = (fields[-1][0] + 1) if fields else 0
        inline, off = [], 4
        for idx, fmt, val in fields:
            size = struct.calcsize("<" + fmt) if fmt else 4
            off = (off + size - 1) // size * size
            inline.append((idx, fmt, val, off))
            off += size
        table_len = (off + 3) // 4 * 4
        vt_len = 4 + 2 * nslots
        self._align(4)
        if (len(self.buf) + vt_len) % 4:
            self.buf += b"\0\0"
        vt_pos = len(self.buf)
        vt = [0] * nslots
        for idx, _, _, o in inline:
            vt[idx] = o
        self.buf += struct.pack("<HH%dH" % nslots, vt_len, table_len, *vt)
        tpos = len(self.buf)
        assert tpos % 4 == 0
        self.buf += b"\0" * table_len
        struct.pack_into("<i", self.buf, tpos, tpos - vt_pos)
        for idx, fmt, val, o in inline:
            if fmt:
                struct.pack_into("<" + fmt, self.buf, tpos + o, val)
        for idx, fmt, val, o in inline:
            if not fmt:
                cpos = self._emit(val)
                struct.pack_into("<I", self.buf, tpos + o, cpos - (tpos + o))
        return tpos

    def finish(self, root: _Ref) -> bytes:
        self.buf = bytearray(b"\0\0\0\0TOSA")
        pos = self._emit(root)
        struct.pack_into("<I", self.buf, 0, pos)
        return bytes(self.buf)


def tensor(name, shape, dtype, data=None, int4=False):
    """int4: an INT4 tensor (DType 2) from int8 values of -8 ... 7, two to a byte, the first of a pair in the low half"""
    f = [(0, None, string(name)), (1, None, vector("i", shape)), (2, "I", 2 if int4 else DTYPE_CODE[np.dtype(dtype)])]
    if data is not None:
        arr = np.ascontiguousarray(data, dtype=dtype)
        if int4:
            nib = (arr.reshape(-1).astype(np.int16) & 0xF).astype(np.uint8)
            nib = np.concatenate([nib, np.zeros(len(nib) & 1, np.uint8)])
            raw = (nib[0::2] | (nib[1::2] << 4)).astype(np.uint8).tobytes()
        else:
            # INT48 (int64 here) is serialized as the low 6 bytes of every element
            raw = arr.view(np.uint8).reshape(-1, 8)[:, :6].tobytes() if arr.dtype == np.int64 else arr.tobytes()
        raw += b"\0" * (-len(raw) % 8)
        f.append((3, None, vector("B", raw)))
    return table(f)


def operator(op, inputs, outputs, attr=None):
    f = [(0, "I", op), (3, None, vector_of([string(s) for s in inputs])), (4, None, vector_of([string(s) for s in outputs]))]
    if attr is not None:
        f += [(1, "B", 1), (2, None, attr)]
    return table(f)


def conv_attr(pad, stride, dilation, acc_type=5, local_bound=False):
    return table([(0, None, vector("i", pad)), (1, None, vector("i", stride)), (2, None, vector("i", dilation)),
                  (3, "B", int(local_bound)), (4, "I", acc_type)])


def transpose_conv_attr(out_pad, stride, acc_type=5, local_bound=False):
    return table([(0, None, vector("i", out_pad)), (1, None, vector("i", stride)), (2, "B", int(local_bound)),
                  (3, "I", acc_type)])


def pool_attr(kernel, stride, pad, last):
    """AvgPool2dAttribute (last = acc_type) / MaxPool2dAttribute (last = nan_mode)"""
    return table([(0, None, vector("i", kernel)), (1, None, vector("i", stride)), (2, None, vector("i", pad)),
                  (3, "I", last)])


def rescale_attr(scale32=True, rounding_mode=3, per_channel=True, input_unsigned=False, output_unsigned=False):
    return table([(0, "B", int(scale32)), (1, "I", rounding_mode), (2, "B", int(per_channel)),
                  (3, "B", int(input_unsigned)), (4, "B", int(output_unsigned))])


def clamp_attr(lo, hi, dtype=np.int8):
    enc = lambda v: np.array([v], dtype=dtype).tobytes()
    return table([(0, None, vector("B", enc(lo))), (1, None, vector("B", enc(hi))), (2, "I", 1)])


def graph(tensors, operators, inputs, outputs) -> bytes:
    block = table([(0, None, string("main")), (1, None, vector_of(operators)), (2, None, vector_of(tensors)),
                   (3, None, vector_of([string(s) for s in inputs])), (4, None, vector_of([string(s) for s in outputs]))])
    region = table([(0, None, string("main")), (1, None, vector_of([block]))])
    version = table([(0, "i", 1), (1, "i", 1), (2, "i", 0), (3, "B", 1)])
    return Writer().finish(table([(0, None, version), (1, None, vector_of([region]))]))

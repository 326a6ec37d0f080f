"""Minimal FlatBuffers walker for TOSA 1.x graph files, for the tests only.

No schema compiler is available, so tables are walked generically (root offset -> vtable -> field
offsets).  Field numbers are those observed in the reference's example graphs:

    TosaGraph       0 version, 1 regions[]
    TosaRegion      0 name, 1 blocks[]
    TosaBasicBlock  0 name, 1 operators[], 2 tensors[], 3 inputs[str], 4 outputs[str]
    TosaTensor      0 name, 1 shape[int32], 2 type(uint32), 3 data[ubyte]
    TosaOperator    0 op(uint32), 1 attribute_type(ubyte), 2 attribute(table), 3 inputs[str], 4 outputs[str]
"""
from __future__ import annotations

import struct

import numpy as np

# Op / DType numbers of the TOSA 1.0 serialization schema; ops 3, 15, 57, 61, 66, 67, 68, 71 and dtypes
# 3, 5, 7 are confirmed by the reference's example graphs.
OP_CONV2D, OP_DEPTHWISE_CONV2D, OP_MATMUL, OP_CLAMP, OP_RESCALE, OP_CONST = 3, 5, 7, 11, 66, 67
OP_AVG_POOL2D, OP_CONV3D, OP_MAX_POOL2D, OP_TRANSPOSE_CONV2D = 2, 4, 8, 10
DTYPE_NP = {3: np.int8, 4: np.int16, 5: np.int32, 7: np.float32, 8: np.float16}


class Table:
    def __init__(self, buf: bytes, pos: int):
        self.buf, self.pos = buf, pos
        self.vt = pos - struct.unpack_from("<i", buf, pos)[0]
        self.vt_len = struct.unpack_from("<H", buf, self.vt)[0]

    def _off(self, field: int) -> int:
        o = 4 + 2 * field
        if o >= self.vt_len:
            return 0
        return struct.unpack_from("<H", self.buf, self.vt + o)[0]

    def scalar(self, field: int, fmt: str, default=0):
        o = self._off(field)
        return struct.unpack_from("<" + fmt, self.buf, self.pos + o)[0] if o else default

    def _indirect(self, field: int):
        o = self._off(field)
        if not o:
            return None
        p = self.pos + o
        return p + struct.unpack_from("<I", self.buf, p)[0]

    def table(self, field: int):
        p = self._indirect(field)
        return Table(self.buf, p) if p is not None else None

    def string(self, field: int, default=""):
        p = self._indirect(field)
        if p is None:
            return default
        n = struct.unpack_from("<I", self.buf, p)[0]
        return self.buf[p + 4:p + 4 + n].decode()

    def vector(self, field: int, fmt: str):
        p = self._indirect(field)
        if p is None:
            return []
        n = struct.unpack_from("<I", self.buf, p)[0]
        return list(struct.unpack_from("<%d%s" % (n, fmt), self.buf, p + 4))

    def bytes_(self, field: int) -> bytes:
        p = self._indirect(field)
        if p is None:
            return b""
        n = struct.unpack_from("<I", self.buf, p)[0]
        return self.buf[p + 4:p + 4 + n]

    def tables(self, field: int):
        p = self._indirect(field)
        if p is None:
            return []
        n = struct.unpack_from("<I", self.buf, p)[0]
        out = []
        for i in range(n):
            q = p + 4 + 4 * i
            out.append(Table(self.buf, q + struct.unpack_from("<I", self.buf, q)[0]))
        return out

    def strings(self, field: int):
        p = self._indirect(field)
        if p is None:
            return []
        n = struct.unpack_from("<I", self.buf, p)[0]
        out = []
        for i in range(n):
            q = p + 4 + 4 * i
            s = q + struct.unpack_from("<I", self.buf, q)[0]
            ln = struct.unpack_from("<I", self.buf, s)[0]
            out.append(self.buf[s + 4:s + 4 + ln].decode())
        return out


def load_main_block(path: str):
    """Returns (tensors, operators, inputs, outputs) of region 0 / block 0.

    tensors: name -> dict(shape, type, data: np.ndarray or None)
    operators: list of dict(op, attr: Table or None, inputs, outputs)
    """
    buf = open(path, "rb").read()
    assert buf[4:8] == b"TOSA"
    root = Table(buf, struct.unpack_from("<I", buf, 0)[0])
    block = root.tables(1)[0].tables(1)[0]
    tensors = {}
    for t in block.tables(2):
        shape = t.vector(1, "i")
        ty = t.scalar(2, "I")
        raw = t.bytes_(3)
        data = None
        if raw and ty in DTYPE_NP:
            n = int(np.prod(shape)) if shape else 1
            data = np.frombuffer(raw, dtype=DTYPE_NP[ty], count=n).reshape(shape)
        tensors[t.string(0)] = dict(shape=shape, type=ty, data=data)
    ops = []
    for o in block.tables(1):
        ops.append(dict(op=o.scalar(0, "I"), attr=o.table(2), inputs=o.strings(3), outputs=o.strings(4)))
    return tensors, ops, block.strings(3), block.strings(4)


def conv_attr(t: Table):
    return dict(pad=t.vector(0, "i"), stride=t.vector(1, "i"), dilation=t.vector(2, "i"),
                local_bound=bool(t.scalar(3, "B")), acc_type=t.scalar(4, "I"))


def rescale_attr(t: Table):
    return dict(scale32=bool(t.scalar(0, "B")), rounding_mode=t.scalar(1, "I"), per_channel=bool(t.scalar(2, "B")),
                input_unsigned=bool(t.scalar(3, "B")), output_unsigned=bool(t.scalar(4, "B")))

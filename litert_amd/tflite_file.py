"""Minimal reader of the `.tflite` flatbuffer: just the tables a FULLY_CONNECTED model needs.

Follows the schema in tflite/converter/schema/schema.fbs (Model :1697-1734, SubGraph
:1609-1630, Tensor :249-295, QuantizationParameters :114-138, BlockwiseQuantization :84-93,
Operator :1559-1605, OperatorCode :1522-1538, Buffer :1634-1643, FullyConnectedOptions
:962-982) and, for what becomes of the quantization tables at load time, ParseQuantization in
tflite/core/interpreter_builder.cc:500-519 (blockwise) and :521-600 (affine). Nothing is
generated and no flatbuffers package is needed: a flatbuffer table is a vtable of 16-bit field
offsets, which is all this file decodes.
"""
import struct
from dataclasses import dataclass, field
from typing import List, Optional

import numpy as np

# TensorType (schema.fbs:41-68) -> (name, numpy dtype or None, TfLiteType value of tflite_types.h:43-68)
TENSOR_TYPES = {
    0: ("FLOAT32", np.float32, 1), 1: ("FLOAT16", np.float16, 10), 2: ("INT32", np.int32, 2),
    3: ("UINT8", np.uint8, 3), 4: ("INT64", np.int64, 4), 7: ("INT16", np.int16, 7),
    9: ("INT8", np.int8, 9), 17: ("INT4", None, 18), 19: ("INT2", None, 20),
}
BUILTIN_FULLY_CONNECTED = 9          # BuiltinOperator FULLY_CONNECTED (schema.fbs:312)
OPTIONS_FULLY_CONNECTED = 8          # position of FullyConnectedOptions in union BuiltinOptions (:525-533)
DETAILS_BLOCKWISE = 2                # position of BlockwiseQuantization in union QuantizationDetails (:77-81)


class _Table:
    """One flatbuffer table: field i lives at `pos + vtable[i]` when the vtable lists it."""

    def __init__(self, buf, pos):
        self.buf, self.pos = buf, pos
        vt = pos - struct.unpack_from("<i", buf, pos)[0]
        size = struct.unpack_from("<H", buf, vt)[0]
        self.offsets = struct.unpack_from("<%dH" % ((size - 4) // 2), buf, vt + 4)

    def _at(self, i):
        return self.pos + self.offsets[i] if i < len(self.offsets) and self.offsets[i] else None

    def scalar(self, i, fmt, default=0):
        at = self._at(i)
        return default if at is None else struct.unpack_from("<" + fmt, self.buf, at)[0]

    def _indirect(self, i):
        at = self._at(i)
        return None if at is None else at + struct.unpack_from("<I", self.buf, at)[0]

    def table(self, i):
        at = self._indirect(i)
        return None if at is None else _Table(self.buf, at)

    def string(self, i):
        at = self._indirect(i)
        if at is None:
            return None
        n = struct.unpack_from("<I", self.buf, at)[0]
        return bytes(self.buf[at + 4:at + 4 + n]).decode("utf-8", "replace")

    def vector(self, i, dtype):
        """Vector of scalars as a numpy array (a view of the file), or None when absent."""
        at = self._indirect(i)
        if at is None:
            return None
        n = struct.unpack_from("<I", self.buf, at)[0]
        return np.frombuffer(self.buf, dtype=dtype, count=n, offset=at + 4)

    def tables(self, i):
        at = self._indirect(i)
        if at is None:
            return []
        n = struct.unpack_from("<I", self.buf, at)[0]
        out = []
        for j in range(n):
            slot = at + 4 + 4 * j
            out.append(_Table(self.buf, slot + struct.unpack_from("<I", self.buf, slot)[0]))
        return out


@dataclass
class Quantization:
    """What ParseQuantization leaves on the tensor: kind 'none' | 'affine' | 'blockwise'."""
    kind: str = "none"
    scale: Optional[np.ndarray] = None        # affine: float32 per channel (or one)
    zero_point: Optional[np.ndarray] = None   # affine: int64 as stored
    quantized_dimension: int = 0
    scales_tensor: int = -1                   # blockwise: tensor indices within the subgraph
    zero_points_tensor: int = -1
    block_size: int = 0


@dataclass
class Tensor:
    index: int
    name: str
    shape: tuple
    type_code: int
    buffer_index: int
    data: Optional[np.ndarray]                # raw bytes of a constant tensor, else None
    quantization: Quantization = field(default_factory=Quantization)

    @property
    def type_name(self):
        return TENSOR_TYPES.get(self.type_code, ("TYPE_%d" % self.type_code, None, 0))[0]

    @property
    def tflite_type(self):
        return TENSOR_TYPES[self.type_code][2]

    def array(self):
        """Constant data in the tensor's dtype and shape (INT4/INT2 stay packed bytes)."""
        if self.data is None:
            return None
        dtype = TENSOR_TYPES[self.type_code][1]
        if dtype is None:
            return self.data
        return self.data.view(dtype).reshape(self.shape)


@dataclass
class Operator:
    builtin_code: int
    version: int
    inputs: tuple
    outputs: tuple
    fully_connected: Optional[dict]           # FullyConnectedOptions, for FULLY_CONNECTED ops


@dataclass
class SubGraph:
    name: str
    tensors: List[Tensor]
    inputs: tuple
    outputs: tuple
    operators: List[Operator]


@dataclass
class Model:
    version: int
    description: str
    subgraphs: List[SubGraph]


def _quantization(q):
    if q is None:
        return Quantization()
    if q.scalar(4, "B") == DETAILS_BLOCKWISE:
        d = q.table(5)
        if d is None:
            raise ValueError("Blockwise quantization details are missing.")
        return Quantization(kind="blockwise", scales_tensor=d.scalar(0, "i"),
                            zero_points_tensor=d.scalar(1, "i"), block_size=d.scalar(2, "i"),
                            quantized_dimension=q.scalar(6, "i"))
    scale = q.vector(2, np.float32)
    if scale is None or scale.size == 0:
        return Quantization()
    zp = q.vector(3, np.int64)
    if zp is None:
        raise ValueError("Quantization parameters has non-null scale but null zero_point.")
    if zp.size != scale.size:
        raise ValueError("QuantizationParam has %d zero_point values and %d scale values."
                         % (zp.size, scale.size))
    return Quantization(kind="affine", scale=scale, zero_point=zp,
                        quantized_dimension=q.scalar(6, "i"))


def parse(buf) -> Model:
    buf = memoryview(buf).cast("B") if not isinstance(buf, (bytes, bytearray)) else buf
    if len(buf) < 8:
        raise ValueError("not a flatbuffer: %d bytes" % len(buf))
    root = _Table(buf, struct.unpack_from("<I", buf, 0)[0])
    codes = []
    for oc in root.tables(1):
        # the newer 32-bit field wins over the deprecated byte (schema_utils.cc GetBuiltinCode)
        codes.append((max(oc.scalar(0, "b"), oc.scalar(3, "i")), oc.scalar(2, "i", 1)))
    buffers = []
    for b in root.tables(4):
        data = b.vector(0, np.uint8)
        off, size = b.scalar(1, "Q"), b.scalar(2, "Q")
        if (data is None or data.size == 0) and off > 1 and size:
            data = np.frombuffer(buf, dtype=np.uint8, count=size, offset=off)  # appended buffer
        buffers.append(data if data is not None and data.size else None)
    subgraphs = []
    for sg in root.tables(2):
        tensors = []
        for i, t in enumerate(sg.tables(0)):
            shape = t.vector(0, np.int32)
            bi = t.scalar(2, "I")
            tensors.append(Tensor(index=i, name=t.string(3) or "",
                                  shape=tuple(int(d) for d in shape) if shape is not None else (),
                                  type_code=t.scalar(1, "b"), buffer_index=bi,
                                  data=buffers[bi] if 0 < bi < len(buffers) else None,
                                  quantization=_quantization(t.table(4))))
        ops = []
        for op in sg.tables(3):
            code, version = codes[op.scalar(0, "I")]
            ins, outs = op.vector(1, np.int32), op.vector(2, np.int32)
            fc = None
            if code == BUILTIN_FULLY_CONNECTED:
                o = op.table(4) if op.scalar(3, "B") == OPTIONS_FULLY_CONNECTED else None
                fc = dict(activation=o.scalar(0, "b") if o else 0,
                          weights_format=o.scalar(1, "b") if o else 0,
                          keep_num_dims=bool(o.scalar(2, "B")) if o else False,
                          asymmetric_quantize_inputs=bool(o.scalar(3, "B")) if o else False,
                          quantized_bias_type=o.scalar(4, "b") if o else 0)
            ops.append(Operator(code, version, tuple(int(v) for v in ins) if ins is not None else (),
                                tuple(int(v) for v in outs) if outs is not None else (), fc))
        si, so = sg.vector(1, np.int32), sg.vector(2, np.int32)
        subgraphs.append(SubGraph(sg.string(4) or "", tensors,
                                  tuple(int(v) for v in si) if si is not None else (),
                                  tuple(int(v) for v in so) if so is not None else (), ops))
    return Model(root.scalar(0, "I"), root.string(3) or "", subgraphs)


def load(path) -> Model:
    with open(path, "rb") as f:
        return parse(f.read())

"""Host-side mirror of the reference's EMBEDDING_LOOKUP op for quantized tables
(tflite/kernels/embedding_lookup.cc): the table is uploaded once, calls enqueue one gather
kernel through the C-ABI and leave the rows in device memory, ready to feed FULLY_CONNECTED.

An index outside [0, rows) fails the reference's invoke at the first such lookup (:280-286,
:365-371). The kernel records it in a device status pair; `__call__` reads that pair back (one
stream synchronization) and raises IndexError with the reference's message, unless
`check=False` leaves the check to the caller (`status` holds {0 or 1, position or -1, the
index found there or 0}).
"""
import numpy as np
import torch

from . import capi
from .fully_connected import _dev, _ensure_init, _ptr, _stream


class _Lookup:
    def _output(self, count, out, f16):
        dtype = torch.float16 if f16 else torch.float32
        if out is None:
            return torch.empty((count, self.cols), dtype=dtype, device="cuda")
        if out.dtype != dtype or out.numel() != count * self.cols or not out.is_contiguous():
            raise ValueError("output tensor does not match the lookup")
        return out

    def _finish(self, check):
        if not check:
            return
        flag, _, index = self.status.tolist()  # synchronizes the stream
        if flag:
            raise IndexError("Embedding Lookup: index out of bounds. Got %d, and bounds are [0, %d]"
                             % (index, self.rows - 1))


class EmbeddingLookupBlockwiseInt4(_Lookup):
    """EvalBlockwise, embedding_lookup.cc:194-307. table: uint8 [rows, cols/2] (low nibble = even
    column); scales_f16: [rows, cols/blocksize] float16 (or its bit patterns)."""

    def __init__(self, table, scales_f16, cols, blocksize=32, out_f16=False):
        _ensure_init()
        self.table = _dev(table, torch.uint8)
        self.rows = self.table.shape[0]
        self.cols = int(cols)
        self.blocksize = int(blocksize)
        if isinstance(scales_f16, np.ndarray):
            scales_f16 = scales_f16.view(np.int16)
        elif scales_f16.dtype == torch.float16:
            scales_f16 = scales_f16.view(torch.int16)
        self.scales = _dev(scales_f16, torch.int16)
        self.out_f16 = bool(out_f16)
        self.status = torch.zeros(3, dtype=torch.int32, device="cuda")

    def __call__(self, lookup, out=None, check=True):
        lookup = _dev(lookup, torch.int32)
        out = self._output(lookup.numel(), out, self.out_f16)
        capi.check(capi.load().lrtfc_embedding_lookup_blockwise_int4(
            _ptr(lookup), lookup.numel(), _ptr(self.table), self.rows, self.cols, _ptr(self.scales),
            self.blocksize, capi.OUT_FLOAT16 if self.out_f16 else capi.OUT_FLOAT32, _ptr(out),
            _ptr(self.status), _stream()))
        self._finish(check)
        return out


class EmbeddingLookupHybrid(_Lookup):
    """EvalHybrid, embedding_lookup.cc:309-395. table: int8 [rows, cols], or for value_bits=4
    uint8 [rows, cols/2]; `scale` for the whole table or `row_scales` [rows]."""

    def __init__(self, table, cols, value_bits=8, scale=1.0, row_scales=None, out_f16=False):
        _ensure_init()
        if value_bits not in (4, 8):
            raise ValueError("value_bits must be 4 or 8")
        self.table = _dev(table, torch.uint8 if value_bits == 4 else torch.int8)
        self.rows = self.table.shape[0]
        self.cols = int(cols)
        self.value_bits = value_bits
        self.scale = float(scale)
        self.row_scales = _dev(row_scales, torch.float32)
        self.out_f16 = bool(out_f16)
        self.status = torch.zeros(3, dtype=torch.int32, device="cuda")

    def __call__(self, lookup, out=None, check=True):
        lookup = _dev(lookup, torch.int32)
        out = self._output(lookup.numel(), out, self.out_f16)
        capi.check(capi.load().lrtfc_embedding_lookup_hybrid(
            _ptr(lookup), lookup.numel(), _ptr(self.table), self.value_bits, self.rows, self.cols,
            self.scale, _ptr(self.row_scales),
            capi.OUT_FLOAT16 if self.out_f16 else capi.OUT_FLOAT32, _ptr(out), _ptr(self.status),
            _stream()))
        self._finish(check)
        return out

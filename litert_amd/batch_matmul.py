"""Host-side mirror of the reference's BATCH_MATMUL op for the hybrid case (float32 left
operand, constant int8 right operand): tflite/kernels/batch_matmul.cc. The constructor is
`Prepare` plus the one-time transposition of the constant operand (batch_matmul.cc:776-782);
`__call__` is `Eval` -> EvalHybrid (:454-520)."""
import ctypes as C

import numpy as np
import torch

from . import capi
from .fully_connected import _dev, _ensure_init, _ptr, _stream


class BatchMatMulHybrid:
    """rhs: int8 [..., K, N] (adj_y: [..., N, K]), constant. per_channel_scales: [N] or None
    (then filter_scale). Left operands are float32 [..., M, K]; adj_x is not offered. Batch
    dimensions must be equal, or all 1 on one side."""

    def __init__(self, rhs, per_channel_scales=None, filter_scale=1.0,
                 asymmetric_quantize_inputs=True, adj_y=False, quant_variant=capi.QUANT_PORTABLE):
        _ensure_init()
        lib = capi.load()
        rhs = np.ascontiguousarray(rhs, dtype=np.int8)
        if rhs.ndim < 2 or rhs.ndim > 5:
            raise ValueError("BATCH_MATMUL operands have 2 to 5 dimensions")
        w = rhs if adj_y else np.ascontiguousarray(np.swapaxes(rhs, -1, -2))
        self.rhs_batch_shape = tuple(w.shape[:-2])
        self.units, self.depth = w.shape[-2:]
        self.matrices = int(np.prod(self.rhs_batch_shape, dtype=np.int64))
        w = _dev(w.reshape(self.matrices, self.units, self.depth), torch.int8)
        self.matrix_bytes = lib.lrtfc_packed_int8_filter_bytes(self.units, self.depth)
        self.packed = torch.empty(self.matrices * self.matrix_bytes, dtype=torch.int8, device="cuda")
        self.row_sums = torch.empty((self.matrices, self.units), dtype=torch.int32, device="cuda")
        for m in range(self.matrices):
            capi.check(lib.lrtfc_row_sums_int8(_ptr(w[m]), self.units, self.depth,
                                               _ptr(self.row_sums[m]), _stream()))
            capi.check(lib.lrtfc_pack_int8_filter(
                _ptr(w[m]), self.units, self.depth,
                C.c_void_p(self.packed.data_ptr() + m * self.matrix_bytes), _stream()))
        torch.cuda.current_stream().synchronize()
        self.pcs = _dev(per_channel_scales, torch.float32)
        self.filter_scale = float(filter_scale)
        self.asymmetric = bool(asymmetric_quantize_inputs)
        self.variant = quant_variant
        self._ws = None

    def __call__(self, lhs):
        lhs = lhs.contiguous()
        if lhs.shape[-1] != self.depth:
            raise ValueError("accumulation depths differ")
        rows = lhs.shape[-2]
        lhs_batch_shape = tuple(lhs.shape[:-2])
        lhs_batches = int(np.prod(lhs_batch_shape, dtype=np.int64))
        rank = max(len(lhs_batch_shape), len(self.rhs_batch_shape))
        lb = (1,) * (rank - len(lhs_batch_shape)) + lhs_batch_shape
        rb = (1,) * (rank - len(self.rhs_batch_shape)) + self.rhs_batch_shape
        if not (lb == rb or lhs_batches == 1 or self.matrices == 1):
            raise ValueError("batch dimensions must be equal, or all 1 on one side")
        out_batch = tuple(max(a, b) for a, b in zip(lb, rb))
        out = torch.empty(out_batch + (rows, self.units), dtype=torch.float32, device=lhs.device)
        lib = capi.load()
        need = lib.lrtfc_activation_workspace_bytes(lhs_batches * rows, self.depth)
        if self._ws is None or self._ws.numel() < need:
            self._ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        capi.check(lib.lrtfc_batch_matmul_hybrid_packed(
            _ptr(lhs), lhs_batches, rows, self.depth, _ptr(self.packed), self.matrices, self.units,
            _ptr(self.pcs), self.filter_scale, _ptr(self.row_sums), _ptr(out), int(self.asymmetric),
            self.variant, _ptr(self._ws), self._ws.numel(), _stream()))
        return out

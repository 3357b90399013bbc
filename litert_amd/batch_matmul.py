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
    (then filter_scale). Left operands are float32 [..., M, K] (adj_x: [..., K, M]). Batch
    dimensions broadcast as the op's do: each pair equal, or 1 on either side."""

    def __init__(self, rhs, per_channel_scales=None, filter_scale=1.0,
                 asymmetric_quantize_inputs=True, adj_y=False, quant_variant=capi.QUANT_PORTABLE,
                 adj_x=False):
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
        self.adj_x = bool(adj_x)
        self._ws = None

    def __call__(self, lhs):
        lhs = lhs.contiguous()
        if lhs.dim() < 2 or lhs.dim() > 5:
            raise ValueError("BATCH_MATMUL operands have 2 to 5 dimensions")
        rows, depth = (lhs.shape[-1], lhs.shape[-2]) if self.adj_x else (lhs.shape[-2], lhs.shape[-1])
        if depth != self.depth:
            raise ValueError("accumulation depths differ")
        lhs_batch_shape = tuple(lhs.shape[:-2])
        lhs_batches = int(np.prod(lhs_batch_shape, dtype=np.int64))
        lb = (1,) * (3 - len(lhs_batch_shape)) + lhs_batch_shape
        rb = (1,) * (3 - len(self.rhs_batch_shape)) + self.rhs_batch_shape
        if any(a != b and a != 1 and b != 1 for a, b in zip(lb, rb)):
            raise ValueError("batch dimensions must be equal or 1, pair by pair")
        rank = max(len(lhs_batch_shape), len(self.rhs_batch_shape))
        out_batch = tuple(b if a == 1 else a for a, b in zip(lb, rb))[3 - rank:]
        out = torch.empty(out_batch + (rows, self.units), dtype=torch.float32, device=lhs.device)
        lib = capi.load()
        need = lib.lrtfc_batch_matmul_workspace_bytes(lhs_batches, rows, self.depth, int(self.adj_x))
        if self._ws is None or self._ws.numel() < need:
            self._ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        capi.check(lib.lrtfc_batch_matmul_hybrid_packed_nd(
            _ptr(lhs), (C.c_int * 3)(*lb), rows, self.depth, int(self.adj_x), _ptr(self.packed),
            (C.c_int * 3)(*rb), self.units, _ptr(self.pcs), self.filter_scale, _ptr(self.row_sums),
            _ptr(out), int(self.asymmetric), self.variant, _ptr(self._ws), self._ws.numel(),
            _stream()))
        return out

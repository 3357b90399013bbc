"""Host-side mirror of the reference's quantized FULLY_CONNECTED op for Python callers.

Each class follows the builtin op's two phases (tflite/kernels/fully_connected.cc):
the constructor is `Prepare` (validates the tensor / quantization-parameter
combination, derives multipliers and activation bounds, uploads and pre-reduces the
constant filter) and `__call__` is `Eval` (launches the HIP kernels through the C
ABI on torch's current stream). Tensors handed to `__call__` are torch CUDA tensors;
torch is used only for device memory and streams.
"""
import ctypes as C

import numpy as np
import torch

from . import capi

_ACT = {"none": capi.ACT_NONE, "relu": capi.ACT_RELU, "relu_n1_to_1": capi.ACT_RELU_N1_TO_1,
        "relu6": capi.ACT_RELU6, "sign_bit": capi.ACT_SIGN_BIT}


def _act(a):
    return _ACT[a] if isinstance(a, str) else int(a)


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def _dev(a, dtype):
    if a is None:
        return None
    if isinstance(a, torch.Tensor):
        return a.to(device="cuda", dtype=dtype).contiguous()
    return torch.from_numpy(np.ascontiguousarray(a)).to(device="cuda", dtype=dtype).contiguous()


def _ensure_init():
    capi.init(torch.cuda.current_device())


def _pack_int8(filter_dev):
    """Re-tiles a row-major int8 [N, K] device tensor for the matrix-core GEMV."""
    n, k = filter_dev.shape
    lib = capi.load()
    packed = torch.empty(lib.lrtfc_packed_int8_filter_bytes(n, k), dtype=torch.int8, device="cuda")
    capi.check(lib.lrtfc_pack_int8_filter(_ptr(filter_dev), n, k, _ptr(packed), _stream()))
    return packed


def quantize_multiplier(m):
    q, s = C.c_int32(), C.c_int()
    capi.check(capi.load().lrtfc_quantize_multiplier(float(m), C.byref(q), C.byref(s)))
    return q.value, s.value


def activation_range_int8(activation, out_scale, out_zp):
    lo, hi = C.c_int32(), C.c_int32()
    capi.check(capi.load().lrtfc_activation_range_int8(_act(activation), out_scale, out_zp,
                                                       C.byref(lo), C.byref(hi)))
    return lo.value, hi.value


def prepare_per_channel(in_scale, filter_scales, out_scale):
    fs = np.ascontiguousarray(filter_scales, dtype=np.float32)
    mult = np.empty(fs.size, np.int32)
    shift = np.empty(fs.size, np.int32)
    capi.check(capi.load().lrtfc_prepare_per_channel(
        in_scale, fs.ctypes.data_as(C.POINTER(C.c_float)), fs.size, out_scale,
        mult.ctypes.data_as(C.POINTER(C.c_int32)), shift.ctypes.data_as(C.POINTER(C.c_int32))))
    return mult, shift


def prepare_per_tensor(in_scale, filter_scale, out_scale, bias_scale=None):
    m, s = C.c_int32(), C.c_int32()
    capi.check(capi.load().lrtfc_prepare_per_tensor(
        in_scale, filter_scale, bias_scale is not None,
        0.0 if bias_scale is None else bias_scale, out_scale, C.byref(m), C.byref(s)))
    return m.value, s.value


def batch_quantize_floats(x, asymmetric=True, variant=capi.QUANT_PORTABLE):
    """tensor_utils::BatchQuantizeFloats on the GPU: returns (q int8 [B,K], scale [B], zp [B])."""
    _ensure_init()
    x = x.contiguous()
    B, K = x.shape
    q = torch.empty((B, K), dtype=torch.int8, device=x.device)
    sf = torch.empty(B, dtype=torch.float32, device=x.device)
    zp = torch.zeros(B, dtype=torch.int32, device=x.device)
    capi.check(capi.load().lrtfc_batch_quantize_floats(_ptr(x), B, K, _ptr(q), _ptr(sf), _ptr(zp),
                                                       int(asymmetric), variant, _stream()))
    return q, sf, zp


class FullyConnectedInt8:
    """Full-integer int8 FC: Prepare = fully_connected.cc:526-581, Eval = :1383-1421 / :1254-1284.

    filter: int8 [N,K], or packed int4 (pass int4=True: [N, ceil(K/2)] bytes, unpacked once here
    as fully_connected.cc:1670-1677 does on every call), or packed int2 (int2=True: the flat
    tensor, four values per byte, fully_connected.cc:1678-1685). filter_scales of size N > 1 selects
    the per-channel form, otherwise per-tensor (filter_zero_point then applies).
    """

    def __init__(self, filter, bias, input_scale, input_zero_point, filter_scales,
                 output_scale, output_zero_point, activation="none", filter_zero_point=0,
                 bias_scale=None, int4=False, depth=None, packed=True, int2=False, out_depth=None):
        _ensure_init()
        lib = capi.load()
        fs = np.atleast_1d(np.asarray(filter_scales, dtype=np.float32))
        self.per_channel = fs.size > 1
        if int4:
            nibbles = _dev(filter, torch.uint8)
            n = nibbles.shape[0]
            if depth is None:
                raise ValueError("depth is required for packed int4 filters")
            self.filter = torch.empty((n, depth), dtype=torch.int8, device="cuda")
            capi.check(lib.lrtfc_unpack_int4(_ptr(nibbles), n * depth, _ptr(self.filter), _stream()))
        elif int2:
            fields = _dev(filter, torch.uint8).reshape(-1)
            if depth is None or out_depth is None:
                raise ValueError("depth and out_depth are required for packed int2 filters")
            self.filter = torch.empty((out_depth, depth), dtype=torch.int8, device="cuda")
            capi.check(lib.lrtfc_unpack_int2(_ptr(fields), out_depth * depth, _ptr(self.filter),
                                             _stream()))
        else:
            self.filter = _dev(filter, torch.int8)
        self.out_depth, self.depth = self.filter.shape
        if self.per_channel:
            if fs.size != self.out_depth:
                raise ValueError("per-channel scales must have one entry per output channel")
            if filter_zero_point != 0:
                raise ValueError("per-channel filters are symmetric")
            mult, shift = prepare_per_channel(input_scale, fs, output_scale)
        else:
            m, s = prepare_per_tensor(input_scale, float(fs[0]), output_scale,
                                      bias_scale if bias is not None else None)
            mult, shift = np.array([m], np.int32), np.array([s], np.int32)
        self.multipliers = _dev(mult, torch.int32)
        self.shifts = _dev(shift, torch.int32)
        self.bias = _dev(bias, torch.int32)
        self.input_offset = -int(input_zero_point)
        self.filter_offset = -int(filter_zero_point)
        self.output_offset = int(output_zero_point)
        self.act_min, self.act_max = activation_range_int8(activation, output_scale,
                                                           output_zero_point)
        self.row_sums = torch.empty(self.out_depth, dtype=torch.int32, device="cuda")
        capi.check(lib.lrtfc_row_sums_int8(_ptr(self.filter), self.out_depth, self.depth,
                                           _ptr(self.row_sums), _stream()))
        # packed: every batch size runs on a re-tiled copy of the filter (matrix-core GEMV up
        # to 16 rows, MFMA GEMM above); otherwise the row-major kernels.
        self.packed_filter = None
        if packed and self.filter_offset == 0 and self.depth > 0:
            self.packed_filter = _pack_int8(self.filter)

    def __call__(self, x, out=None):
        x = x.contiguous()
        batches = x.numel() // self.depth if self.depth else 0
        if out is None:
            out = torch.empty((batches, self.out_depth), dtype=torch.int8, device=x.device)
        if self.packed_filter is not None:
            capi.check(capi.load().lrtfc_fc_int8_packed(
                _ptr(x), _ptr(self.packed_filter), _ptr(self.bias), _ptr(self.multipliers),
                _ptr(self.shifts), int(self.per_channel), _ptr(self.row_sums), _ptr(out), batches,
                self.depth, self.out_depth, self.input_offset, self.output_offset, self.act_min,
                self.act_max, _stream()))
            return out
        capi.check(capi.load().lrtfc_fc_int8(
            _ptr(x), _ptr(self.filter), _ptr(self.bias), _ptr(self.multipliers), _ptr(self.shifts),
            int(self.per_channel), _ptr(self.row_sums), _ptr(out), batches, self.depth,
            self.out_depth, self.input_offset, self.filter_offset, self.output_offset,
            self.act_min, self.act_max, _stream()))
        return out


class FullyConnectedUInt8:
    """The legacy full-integer uint8 FC (per-tensor; fully_connected.cc:1607-1626 with
    reference/fully_connected.h:118-166) on the int8 kernels: every uint8 tensor is taken as
    int8 (value - 128, a flip of the top bit: the filter once here, the rows and the result on
    every call) and every zero point lowered by 128, which leaves each term of the sum, the
    multiplier and the clamped result what they were."""

    def __init__(self, filter, bias, input_scale, input_zero_point, filter_scale,
                 filter_zero_point, output_scale, output_zero_point, activation="none",
                 bias_scale=None, packed=True):
        _ensure_init()
        lib = capi.load()
        w = _dev(filter, torch.uint8).contiguous()
        capi.check(lib.lrtfc_xor_sign_bit(_ptr(w), _ptr(w), w.numel(), _stream()))
        self.int8 = FullyConnectedInt8(
            w.view(torch.int8), bias, input_scale, int(input_zero_point) - 128, [filter_scale],
            output_scale, int(output_zero_point) - 128, activation=activation,
            filter_zero_point=int(filter_zero_point) - 128, bias_scale=bias_scale, packed=packed)
        self.out_depth, self.depth = self.int8.out_depth, self.int8.depth

    def __call__(self, x, out=None):
        lib = capi.load()
        x = x.contiguous()
        rows = torch.empty_like(x)
        capi.check(lib.lrtfc_xor_sign_bit(_ptr(x), _ptr(rows), x.numel(), _stream()))
        y = self.int8(rows.view(torch.int8))
        if out is None:
            out = torch.empty(y.shape, dtype=torch.uint8, device=x.device)
        capi.check(lib.lrtfc_xor_sign_bit(_ptr(y), _ptr(out), y.numel(), _stream()))
        return out


class FullyConnectedHybrid:
    """Hybrid FC (float activations, int8 filter): EvalHybridDense, fully_connected.cc:763-858."""

    def __init__(self, filter, per_channel_scales=None, filter_scale=1.0, bias=None,
                 asymmetric_quantize_inputs=True, activation="none",
                 quant_variant=capi.QUANT_PORTABLE, packed=True):
        _ensure_init()
        self.filter = _dev(filter, torch.int8)
        self.out_depth, self.depth = self.filter.shape
        self.pcs = _dev(per_channel_scales, torch.float32)
        self.filter_scale = float(filter_scale)
        self.bias = _dev(bias, torch.float32)
        self.asymmetric = bool(asymmetric_quantize_inputs)
        self.activation = _act(activation)
        self.variant = quant_variant
        self.row_sums = torch.empty(self.out_depth, dtype=torch.int32, device="cuda")
        capi.check(capi.load().lrtfc_row_sums_int8(_ptr(self.filter), self.out_depth, self.depth,
                                                   _ptr(self.row_sums), _stream()))
        self._ws = None
        # packed: one fused kernel (quantize in the prologue, matrix-core GEMV);
        # otherwise the two-kernel form on the row-major filter.
        self.packed_filter = _pack_int8(self.filter) if packed else None

    def _workspace(self, batches):
        need = capi.load().lrtfc_activation_workspace_bytes(batches, self.depth)
        if self._ws is None or self._ws.numel() < need:
            self._ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        return self._ws

    def __call__(self, x, out=None):
        x = x.contiguous()
        batches = x.numel() // self.depth
        if out is None:
            out = torch.empty((batches, self.out_depth), dtype=torch.float32, device=x.device)
        if self.packed_filter is not None and batches > self._fused_max():
            return self.call_split(x, out)
        if self.packed_filter is not None:
            capi.check(capi.load().lrtfc_fc_hybrid_packed(
                _ptr(x), _ptr(self.packed_filter), _ptr(self.pcs), self.filter_scale,
                _ptr(self.row_sums), _ptr(self.bias), _ptr(out), batches, self.depth,
                self.out_depth, int(self.asymmetric), self.activation, self.variant, _stream()))
            return out
        ws = self._workspace(batches)
        capi.check(capi.load().lrtfc_fc_hybrid(
            _ptr(x), _ptr(self.filter), _ptr(self.pcs), self.filter_scale, _ptr(self.row_sums),
            _ptr(self.bias), _ptr(out), batches, self.depth, self.out_depth, int(self.asymmetric),
            self.activation, self.variant, _ptr(ws), ws.numel(), _stream()))
        return out


    # Above this many rows the fused kernel's prologue costs more than a separate quantization
    # launch: None = what the library says for the shape (lrtfc_fc_hybrid_fused_max_batches).
    FUSED_MAX_BATCHES = None

    def _fused_max(self):
        if self.FUSED_MAX_BATCHES is not None:
            return self.FUSED_MAX_BATCHES
        return capi.load().lrtfc_fc_hybrid_fused_max_batches(self.depth, self.out_depth)

    def call_split(self, x, out=None):
        """Two launches on the packed filter: the standalone row quantizer, then the
        matrix-core GEMV (or GEMM) on its int8 output. Same results as the fused call."""
        if self.packed_filter is None:
            raise RuntimeError("call_split needs the packed filter (packed=True)")
        x = x.contiguous()
        batches = x.numel() // self.depth
        if out is None:
            out = torch.empty((batches, self.out_depth), dtype=torch.float32, device=x.device)
        ws = self._workspace(batches)
        capi.check(capi.load().lrtfc_fc_hybrid_packed_workspace(
            _ptr(x), _ptr(self.packed_filter), _ptr(self.pcs), self.filter_scale,
            _ptr(self.row_sums), _ptr(self.bias), _ptr(out), batches, self.depth, self.out_depth,
            int(self.asymmetric), self.activation, self.variant, _ptr(ws), ws.numel(), _stream()))
        return out


class FullyConnectedBlockwiseInt4:
    """Blockwise-int4 hybrid FC: EvalBlockwise4Bit, fully_connected.cc:1014-1086.

    packed_filter: uint8 [N, K/2], low nibble = even k; scales_f16: [N, K/blocksize] as
    float16 (or its uint16 bit patterns).
    """

    def __init__(self, packed_filter, scales_f16, depth, blocksize=32, bias=None,
                 quant_variant=capi.QUANT_PORTABLE, packed=True):
        _ensure_init()
        self.filter = _dev(packed_filter, torch.uint8)
        self.out_depth = self.filter.shape[0]
        self.depth = int(depth)
        self.blocksize = int(blocksize)
        if isinstance(scales_f16, np.ndarray) and scales_f16.dtype == np.float16:
            scales_f16 = scales_f16.view(np.uint16)
        if isinstance(scales_f16, torch.Tensor) and scales_f16.dtype == torch.float16:
            scales_f16 = scales_f16.view(torch.int16)
        if isinstance(scales_f16, np.ndarray):
            scales_f16 = scales_f16.view(np.int16)
        self.scales = _dev(scales_f16, torch.int16)
        self.bias = _dev(bias, torch.float32)
        self.variant = quant_variant
        self.kfsum = torch.empty(self.out_depth, dtype=torch.float32, device="cuda")
        capi.check(capi.load().lrtfc_blockwise_int4_kfsum(
            _ptr(self.filter), _ptr(self.scales), self.out_depth, self.depth, self.blocksize,
            _ptr(self.kfsum), _stream()))
        self._ws = None
        self._gemm_filter = None
        self._nibble_filter = None
        self._gemm_ws = None
        # packed: one fused kernel on the re-tiled filter (block size 32 only); otherwise the
        # two-kernel form on the reference layout.
        self.retiled = None
        if packed and self.blocksize == 32 and self.depth % 32 == 0:
            lib = capi.load()
            self.retiled = torch.empty(
                lib.lrtfc_packed_int4_blockwise_bytes(self.out_depth, self.depth),
                dtype=torch.uint8, device="cuda")
            capi.check(lib.lrtfc_pack_int4_blockwise(_ptr(self.filter), _ptr(self.scales),
                                                     self.out_depth, self.depth, 32,
                                                     _ptr(self.retiled), _stream()))

    def _workspace(self, batches):
        need = capi.load().lrtfc_activation_workspace_bytes(batches, self.depth)
        if self._ws is None or self._ws.numel() < need:
            self._ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        return self._ws

    # From this many rows on a matrix-core GEMM streams the filter once for the whole batch,
    # whatever the shape (lrtfc_fc_blockwise_int4_preferred_form picks the form per shape).
    GEMM_MIN_BATCHES = 16

    def call_gemm(self, x, out=None):
        """Prefill form: row quantizer, row re-tiling and the blockwise GEMM on a filter
        re-tiled for it (made on first use and kept). Same results as the other forms."""
        if self.blocksize != 32 or self.depth % 32:
            raise RuntimeError("call_gemm needs block size 32")
        lib = capi.load()
        x = x.contiguous()
        batches = x.numel() // self.depth
        if out is None:
            out = torch.empty((batches, self.out_depth), dtype=torch.float32, device=x.device)
        if self._gemm_filter is None:
            self._gemm_filter = torch.empty(
                lib.lrtfc_gemm_int4_blockwise_bytes(self.out_depth, self.depth), dtype=torch.uint8,
                device="cuda")
            capi.check(lib.lrtfc_pack_int4_blockwise_gemm(
                _ptr(self.filter), _ptr(self.scales), self.out_depth, self.depth, 32,
                _ptr(self._gemm_filter), _stream()))
        need = lib.lrtfc_fc_blockwise_int4_gemm_workspace_bytes(batches, self.depth)
        if self._gemm_ws is None or self._gemm_ws.numel() < need:
            self._gemm_ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        capi.check(lib.lrtfc_fc_blockwise_int4_gemm(
            _ptr(x), _ptr(self._gemm_filter), _ptr(self.kfsum), _ptr(self.bias), _ptr(out), batches,
            self.depth, self.out_depth, self.variant, _ptr(self._gemm_ws), self._gemm_ws.numel(),
            _stream()))
        return out

    def _nibble_filter_tensor(self):
        """The filter re-tiled at 4 bits per weight for the matrix cores (made once)."""
        if self.blocksize != 32 or self.depth % 32:
            raise RuntimeError("the 4-bit-resident matrix-core form needs block size 32")
        if self._nibble_filter is None:
            lib = capi.load()
            self._nibble_filter = torch.empty(
                lib.lrtfc_gemm_int4_blockwise_nibble_bytes(self.out_depth, self.depth),
                dtype=torch.uint8, device="cuda")
            capi.check(lib.lrtfc_pack_int4_blockwise_gemm_nibbles(
                _ptr(self.filter), _ptr(self.scales), self.out_depth, self.depth, 32,
                _ptr(self._nibble_filter), _stream()))
        return self._nibble_filter

    def call_gemm_nibbles(self, x, out=None):
        """The same GEMM on the filter kept at 4 bits per weight (made on first use and kept):
        the form for batches between decode and prefill. Same results as the other forms."""
        if self.blocksize != 32 or self.depth % 32:
            raise RuntimeError("call_gemm_nibbles needs block size 32")
        lib = capi.load()
        x = x.contiguous()
        batches = x.numel() // self.depth
        if out is None:
            out = torch.empty((batches, self.out_depth), dtype=torch.float32, device=x.device)
        self._nibble_filter_tensor()
        need = lib.lrtfc_fc_blockwise_int4_gemm_workspace_bytes(batches, self.depth)
        if self._gemm_ws is None or self._gemm_ws.numel() < need:
            self._gemm_ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        capi.check(lib.lrtfc_fc_blockwise_int4_gemm_nibbles(
            _ptr(x), _ptr(self._nibble_filter), _ptr(self.kfsum), _ptr(self.bias), _ptr(out),
            batches, self.depth, self.out_depth, self.variant, _ptr(self._gemm_ws),
            self._gemm_ws.numel(), _stream()))
        return out

    def __call__(self, x, out=None):
        x = x.contiguous()
        batches = x.numel() // self.depth
        if self.blocksize == 32 and self.depth % 32 == 0 and self.retiled is not None:
            form = capi.load().lrtfc_fc_blockwise_int4_preferred_form(batches, self.depth,
                                                                      self.out_depth)
            if form == capi.INT4_FORM_GEMM_NIBBLES:
                return self.call_gemm_nibbles(x, out)
            if form == capi.INT4_FORM_GEMM_INT8:
                return self.call_gemm(x, out)
        if out is None:
            out = torch.empty((batches, self.out_depth), dtype=torch.float32, device=x.device)
        if (self.retiled is not None and self.depth > self.FUSED_MAX_DEPTH
                and batches > self.DEEP_FUSED_MAX_BATCHES):
            return self.call_split(x, out)
        if self.retiled is not None:
            capi.check(capi.load().lrtfc_fc_blockwise_int4_packed(
                _ptr(x), _ptr(self.retiled), _ptr(self.kfsum), _ptr(self.bias), _ptr(out), batches,
                self.depth, self.out_depth, self.variant, _stream()))
            return out
        ws = self._workspace(batches)
        capi.check(capi.load().lrtfc_fc_blockwise_int4(
            _ptr(x), _ptr(self.filter), _ptr(self.scales), _ptr(self.kfsum), _ptr(self.bias),
            _ptr(out), batches, self.depth, self.out_depth, self.blocksize, self.variant,
            _ptr(ws), ws.numel(), _stream()))
        return out

    # Rows deeper than FUSED_MAX_DEPTH fuse the quantizer for at most DEEP_FUSED_MAX_BATCHES
    # batch rows (the prologue keeps the float rows in registers); more rows split it off.
    FUSED_MAX_DEPTH = 4096
    DEEP_FUSED_MAX_BATCHES = 2

    def call_split(self, x, out=None):
        """Two launches on the re-tiled filter: the standalone row quantizer, then the
        streaming kernel on its int8 output. Same results as the fused call."""
        if self.retiled is None:
            raise RuntimeError("call_split needs the re-tiled filter (packed=True, block size 32)")
        x = x.contiguous()
        batches = x.numel() // self.depth
        if out is None:
            out = torch.empty((batches, self.out_depth), dtype=torch.float32, device=x.device)
        key = (batches, str(x.device))
        if getattr(self, "_split_key", None) != key:
            self._split_q = torch.empty((batches, self.depth), dtype=torch.int8, device=x.device)
            self._split_sf = torch.empty(batches, dtype=torch.float32, device=x.device)
            self._split_zp = torch.zeros(batches, dtype=torch.int32, device=x.device)
            self._split_key = key
        q, sf, zp = self._split_q, self._split_sf, self._split_zp
        capi.check(capi.load().lrtfc_batch_quantize_floats(_ptr(x), batches, self.depth, _ptr(q),
                                                           _ptr(sf), _ptr(zp), 1, self.variant,
                                                           _stream()))
        capi.check(capi.load().lrtfc_fc_blockwise_int4_packed_quantized(
            _ptr(q), _ptr(sf), _ptr(zp), _ptr(self.retiled), _ptr(self.kfsum), _ptr(self.bias),
            _ptr(out), batches, self.depth, self.out_depth, _stream()))
        return out


class FullyConnectedHybridInt4PerChannel:
    """Per-channel int4 hybrid FC: EvalHybridDense4Bit, fully_connected.cc:1088-1178.

    packed_filter: uint8 [N, K/2] as the model stores it (low nibble = even k); filter_scales:
    [N], or one value for every channel; bias float32 [N] or None."""

    def __init__(self, packed_filter, depth, filter_scales, bias=None, activation="none"):
        _ensure_init()
        lib = capi.load()
        nibbles = _dev(packed_filter, torch.uint8)
        self.out_depth = nibbles.shape[0]
        self.depth = int(depth)
        if self.depth % 2:
            raise ValueError("the 4-bit path needs an even depth")
        # Two device layouts, each made on first use: the nibbles re-tiled (decode batches: half
        # the bytes to stream) and the int8 expansion re-tiled (prefill batches: the MFMA GEMM).
        self._nibbles = nibbles
        self._retiled_nibbles = None
        self._packed_int8 = None
        fs = np.atleast_1d(np.asarray(filter_scales, dtype=np.float32))
        self.pcs = _dev(fs, torch.float32) if fs.size > 1 else None
        self.filter_scale = float(fs[0])
        self.bias = _dev(bias, torch.float32)
        self.activation = _act(activation)
        self._ws = None

    NIBBLE_MAX_BATCHES = 32  # above: one pass of the MFMA GEMM over the int8 copy is cheaper

    def __call__(self, x, out=None, force_int8=False):
        x = x.contiguous()
        batches = x.numel() // self.depth
        if out is None:
            out = torch.empty((batches, self.out_depth), dtype=torch.float32, device=x.device)
        need = capi.load().lrtfc_activation_workspace_bytes(batches, self.depth)
        if self._ws is None or self._ws.numel() < need:
            self._ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        lib = capi.load()
        if batches <= self.NIBBLE_MAX_BATCHES and not force_int8:
            if self._retiled_nibbles is None:
                self._retiled_nibbles = torch.empty(
                    lib.lrtfc_packed_int4_per_channel_bytes(self.out_depth, self.depth),
                    dtype=torch.uint8, device="cuda")
                capi.check(lib.lrtfc_pack_int4_per_channel(
                    _ptr(self._nibbles), self.out_depth, self.depth, _ptr(self._retiled_nibbles),
                    _stream()))
            capi.check(lib.lrtfc_fc_hybrid_int4_per_channel_nibbles(
                _ptr(x), _ptr(self._retiled_nibbles), _ptr(self.pcs), self.filter_scale,
                _ptr(self.bias), _ptr(out), batches, self.depth, self.out_depth, self.activation,
                _ptr(self._ws), self._ws.numel(), _stream()))
            return out
        if self._packed_int8 is None:
            unpacked = torch.empty((self.out_depth, self.depth), dtype=torch.int8, device="cuda")
            capi.check(lib.lrtfc_unpack_int4(_ptr(self._nibbles), self.out_depth * self.depth,
                                             _ptr(unpacked), _stream()))
            self._packed_int8 = _pack_int8(unpacked)
        capi.check(lib.lrtfc_fc_hybrid_int4_per_channel_packed(
            _ptr(x), _ptr(self._packed_int8), _ptr(self.pcs), self.filter_scale, _ptr(self.bias),
            _ptr(out), batches, self.depth, self.out_depth, self.activation, _ptr(self._ws),
            self._ws.numel(), _stream()))
        return out


class GroupedBlockwiseInt4:
    """Several FullyConnectedBlockwiseInt4 nodes of one depth that do not depend on each other
    (q/k/v, gate/up), run as ONE kernel. `bind` fixes the input and output tensors of every
    node (the launch reads their addresses from a table in device memory); `__call__`
    launches. Results are those of the nodes' own calls."""

    MAX_NODES = 128  # LRTFC_INT4_GROUP_MAX

    def __init__(self, ops):
        if not 1 <= len(ops) <= self.MAX_NODES:
            raise ValueError("a group holds 1..%d nodes" % self.MAX_NODES)
        depth = ops[0].depth
        for op in ops:
            if op.retiled is None or op.depth != depth or op.variant != ops[0].variant:
                raise ValueError("grouped nodes need the re-tiled filter, one depth, one variant")
        self.ops = list(ops)
        self.depth = depth
        self.variant = ops[0].variant
        self.table = torch.empty(capi.load().lrtfc_int4_group_table_bytes(), dtype=torch.uint8,
                                 device="cuda")
        self.launch = None
        self._bound = None

    def bind(self, inputs, outputs):
        """inputs[i] [B, depth] float32, outputs[i] [B, out_depth_i] float32, CUDA, contiguous."""
        batches = inputs[0].numel() // self.depth
        nodes = (capi.Int4GroupNode * len(self.ops))()
        # Deep rows beyond two per launch are quantized into per-node workspaces first, so that
        # every filter is streamed once (same rule as FullyConnectedBlockwiseInt4.__call__).
        workspaces = None
        if batches > FullyConnectedBlockwiseInt4.DEEP_FUSED_MAX_BATCHES:
            need = capi.load().lrtfc_activation_workspace_bytes(batches, self.depth)
            workspaces = torch.empty((len(self.ops), (need + 255) // 256 * 256), dtype=torch.uint8,
                                     device="cuda")
        out_depths = (C.c_int * len(self.ops))(*[op.out_depth for op in self.ops])
        nibbles = capi.load().lrtfc_int4_group_preferred_form(
            out_depths, len(self.ops), batches, self.depth) == capi.INT4_FORM_GEMM_NIBBLES
        for i, (op, x, y) in enumerate(zip(self.ops, inputs, outputs)):
            if not (x.is_contiguous() and y.is_contiguous()):
                raise ValueError("grouped inputs and outputs must be contiguous")
            if x.numel() != batches * self.depth or y.numel() != batches * op.out_depth:
                raise ValueError("node %d: tensor sizes do not match the group" % i)
            nodes[i].input = x.data_ptr()
            nodes[i].retiled_filter = op.retiled.data_ptr()
            nodes[i].kfsum = op.kfsum.data_ptr()
            nodes[i].bias = op.bias.data_ptr() if op.bias is not None else None
            nodes[i].output = y.data_ptr()
            nodes[i].out_depth = op.out_depth
            nodes[i].workspace = workspaces[i].data_ptr() if workspaces is not None else None
            # Some shapes run faster on the filters kept at 4 bits per weight for the matrix
            # cores (three or four rows of wide groups deeper than 8192).
            nodes[i].nibble_filter = op._nibble_filter_tensor().data_ptr() if nibbles else None
        launch = capi.Int4GroupLaunch()
        capi.check(capi.load().lrtfc_int4_group_prepare(
            C.byref(nodes), len(self.ops), batches, self.depth, _ptr(self.table),
            C.byref(launch), _stream()))
        self.launch = launch
        self._bound = (list(inputs), list(outputs), workspaces)  # keep the tensors alive
        return self

    def __call__(self):
        if self.launch is None:
            raise RuntimeError("bind() the group's tensors first")
        capi.check(capi.load().lrtfc_fc_blockwise_int4_packed_grouped(
            _ptr(self.table), C.byref(self.launch), self.variant, _stream()))
        return self._bound[1]

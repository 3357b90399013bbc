"""ctypes front end of the CPU oracle (oracle/liboracle.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by
the cpu_baseline leg of bench.py as the checker / reported baseline. The
product path (litert_amd) never imports this package.

Each wrapper takes and returns numpy arrays; the C side (oracle.cc) cites the
reference file:line it restates.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None
_REF = None

ACT_NONE, ACT_RELU, ACT_RELU_N1_TO_1, ACT_RELU6, ACT_TANH, ACT_SIGN_BIT, ACT_SIGMOID = range(7)
QUANT_PORTABLE, QUANT_NEON_V8, QUANT_NEON_LEGACY = range(3)

_i8p = C.POINTER(C.c_int8)
_u8p = C.POINTER(C.c_uint8)
_u16p = C.POINTER(C.c_uint16)
_i32p = C.POINTER(C.c_int32)
_f32p = C.POINTER(C.c_float)
_intp = C.POINTER(C.c_int)


def build(force=False):
    """Compile liboracle.so (and oracle/_ref when the reference tree is there)."""
    target = os.path.join(_HERE, "liboracle.so")
    if force or not os.path.exists(target):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s"])
    return target


def lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "liboracle.so")
        if os.environ.get("LITERT_AMD_SANITIZED") == "1":
            # the build of `make -C oracle san` (tests/test_sanitizers.py runs under it)
            path = os.path.join(_HERE, "_san", "liboracle_san.so")
        elif not os.path.exists(path):
            build()
        L = C.CDLL(path)
        L.orc_quantize_multiplier.argtypes = [C.c_double, _i32p, _intp]
        L.orc_srdhm.argtypes = [C.c_int32, C.c_int32]
        L.orc_srdhm.restype = C.c_int32
        L.orc_rounding_divide_by_pot.argtypes = [C.c_int32, C.c_int]
        L.orc_rounding_divide_by_pot.restype = C.c_int32
        L.orc_mbqm.argtypes = [C.c_int32, C.c_int32, C.c_int]
        L.orc_mbqm.restype = C.c_int32
        L.orc_mbqm_single_rounding.argtypes = [C.c_int32, C.c_int32, C.c_int]
        L.orc_mbqm_single_rounding.restype = C.c_int32
        L.orc_activation_range_int8.argtypes = [C.c_int, C.c_float, C.c_int32, _i32p, _i32p]
        L.orc_half_to_float.argtypes = [C.c_uint16]
        L.orc_half_to_float.restype = C.c_float
        L.orc_unpack_int4.argtypes = [_i8p, C.c_int, _i8p]
        L.orc_unpack_int2.argtypes = [_i8p, C.c_int, _i8p]
        L.orc_fc_prepare_per_channel.argtypes = [C.c_float, _f32p, C.c_int, C.c_float, _i32p, _i32p]
        L.orc_fc_prepare_per_tensor.argtypes = [C.c_float, C.c_float, C.c_int, C.c_float,
                                                C.c_float, _i32p, _i32p]
        pc = [_i8p, _i8p, _i32p, _i32p, _i32p, _i8p, C.c_int, C.c_int, C.c_int, C.c_int32,
              C.c_int32, C.c_int32, C.c_int32]
        L.orc_fc_int8_per_channel.argtypes = pc
        L.orc_fc_int8_per_channel_single_rounding.argtypes = pc
        L.orc_fc_int8_per_channel_float_scale.argtypes = [
            _i8p, _i8p, _i32p, _f32p, C.c_float, C.c_float, _i8p, C.c_int, C.c_int, C.c_int,
            C.c_int32, C.c_int32, C.c_int32, C.c_int32]
        L.orc_fc_int8_per_tensor.argtypes = [
            _i8p, _i8p, _i32p, C.c_int32, C.c_int, _i8p, C.c_int, C.c_int, C.c_int, C.c_int32,
            C.c_int32, C.c_int32, C.c_int32, C.c_int32]
        L.orc_fc_uint8_per_tensor.argtypes = [
            _u8p, _u8p, _i32p, C.c_int32, C.c_int, _u8p, C.c_int, C.c_int, C.c_int, C.c_int32,
            C.c_int32, C.c_int32, C.c_int32, C.c_int32]
        L.orc_activation_range_uint8.argtypes = [C.c_int, C.c_float, C.c_int32, _i32p, _i32p]
        L.orc_fc_int8_per_tensor_float_scale.argtypes = [
            _i8p, _i8p, _i32p, C.c_float, C.c_float, C.c_float, _i8p, C.c_int, C.c_int, C.c_int,
            C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_int32]
        L.orc_asymmetric_quantize_floats.argtypes = [_f32p, C.c_int, _i8p, _f32p, _i32p, C.c_int]
        L.orc_symmetric_quantize_floats.argtypes = [_f32p, C.c_int, _i8p, _f32p, C.c_int]
        L.orc_batch_quantize_floats.argtypes = [_f32p, C.c_int, C.c_int, _i8p, _f32p, _i32p,
                                                C.c_int, C.c_int]
        L.orc_matrix_batch_vector_multiply_accumulate.argtypes = [
            _i8p, C.c_int, C.c_int, _i8p, _f32p, C.c_int, _f32p, _f32p, _i32p, _i32p, C.c_int]
        L.orc_apply_activation.argtypes = [_f32p, C.c_int, C.c_int]
        L.orc_fc_hybrid.argtypes = [_f32p, C.c_int, C.c_int, _i8p, C.c_int, _f32p, C.c_float,
                                    _f32p, C.c_int, C.c_int, C.c_int, _f32p, _i8p, _f32p, _i32p]
        L.orc_fc_hybrid_cached.argtypes = L.orc_fc_hybrid.argtypes + [_i32p, C.c_int]
        L.orc_matrix_batch_vector_multiply_accumulate_sse.argtypes = [
            _i8p, C.c_int, C.c_int, _i8p, _f32p, C.c_int, _f32p, _f32p, _i32p, _i32p]
        L.orc_matrix_batch_vector_multiply_accumulate_sse.restype = None
        L.orc_batch_matmul_hybrid.argtypes = [_f32p, C.c_int, C.c_int, C.c_int, _i8p, C.c_int,
                                              C.c_int, _f32p, C.c_float, C.c_int, C.c_int, _intp,
                                              _intp, C.c_int, _f32p]
        L.orc_fc_blockwise_int4.argtypes = [_f32p, C.c_int, C.c_int, _u8p, C.c_int, _u16p,
                                            C.c_int, _f32p, C.c_int, _f32p]
        L.orc_fc_hybrid_int4_per_channel.argtypes = [_f32p, C.c_int, C.c_int, _u8p, C.c_int, _f32p,
                                                     _f32p, C.c_int, _f32p]
        _LIB = L
    return _LIB


def ref_lib():
    """oracle/_ref/libref_leaf.so (real reference leaf code) or None when absent."""
    global _REF
    if _REF is None:
        path = os.path.join(_HERE, "_ref", "libref_leaf.so")
        if not os.path.exists(path):
            return None
        R = C.CDLL(path)
        R.ref_quantize_multiplier.argtypes = [C.c_double, _i32p, _intp]
        R.ref_unpack_int4.argtypes = [_i8p, C.c_int, _i8p]
        if hasattr(R, "ref_unpack_int2"):
            R.ref_unpack_int2.argtypes = [_i8p, C.c_int, _i8p]
        for name in ("ref_apply_relu", "ref_apply_relu1", "ref_apply_relu6"):
            getattr(R, name).argtypes = [_f32p, C.c_int, _f32p]
        if hasattr(R, "ref_fc_hybrid_int4"):
            R.ref_fc_hybrid_int4.argtypes = [_f32p, C.c_int, C.c_int, _i8p, C.c_int, _f32p, _f32p,
                                             _f32p]
        _REF = R
    return _REF


def _p(a, t):
    return None if a is None else a.ctypes.data_as(t)


def _c(a, dtype):
    return None if a is None else np.ascontiguousarray(a, dtype=dtype)


# ---- scalar helpers ---------------------------------------------------------

def quantize_multiplier(m):
    q, s = C.c_int32(), C.c_int()
    lib().orc_quantize_multiplier(float(m), C.byref(q), C.byref(s))
    return q.value, s.value


def mbqm(x, m, shift):
    return lib().orc_mbqm(int(x), int(m), int(shift))


def mbqm_single_rounding(x, m, shift):
    return lib().orc_mbqm_single_rounding(int(x), int(m), int(shift))


def activation_range_int8(activation, out_scale, out_zp):
    lo, hi = C.c_int32(), C.c_int32()
    rc = lib().orc_activation_range_int8(activation, out_scale, out_zp, C.byref(lo), C.byref(hi))
    if rc:
        raise ValueError("activation range overflows int32")
    return lo.value, hi.value


def activation_range_uint8(activation, out_scale, out_zp):
    lo, hi = C.c_int32(), C.c_int32()
    rc = lib().orc_activation_range_uint8(activation, out_scale, out_zp, C.byref(lo), C.byref(hi))
    if rc:
        raise ValueError("activation range overflows int32")
    return lo.value, hi.value


def half_to_float(bits_u16):
    a = np.ascontiguousarray(bits_u16, dtype=np.uint16)
    out = np.empty(a.shape, dtype=np.float32)
    L = lib()
    flat_in, flat_out = a.ravel(), out.ravel()
    for i in range(flat_in.size):
        flat_out[i] = L.orc_half_to_float(int(flat_in[i]))
    return out


def unpack_int4(packed, num_elements):
    src = _c(packed, np.int8).ravel()
    dst = np.empty(num_elements, dtype=np.int8)
    lib().orc_unpack_int4(_p(src, _i8p), num_elements, _p(dst, _i8p))
    return dst


def unpack_int2(packed, num_elements):
    src = _c(packed, np.int8).ravel()
    dst = np.empty(num_elements, dtype=np.int8)
    lib().orc_unpack_int2(_p(src, _i8p), num_elements, _p(dst, _i8p))
    return dst


def fc_prepare_per_channel(in_scale, filter_scales, out_scale):
    fs = _c(filter_scales, np.float32)
    n = fs.size
    mult = np.empty(n, dtype=np.int32)
    shift = np.empty(n, dtype=np.int32)
    lib().orc_fc_prepare_per_channel(in_scale, _p(fs, _f32p), n, out_scale, _p(mult, _i32p),
                                     _p(shift, _i32p))
    return mult, shift


def fc_prepare_per_tensor(in_scale, filter_scale, out_scale, bias_scale=None):
    m, s = C.c_int32(), C.c_int32()
    rc = lib().orc_fc_prepare_per_tensor(in_scale, filter_scale, bias_scale is not None,
                                         0.0 if bias_scale is None else bias_scale, out_scale,
                                         C.byref(m), C.byref(s))
    if rc:
        raise ValueError("per-tensor scale checks failed")
    return m.value, s.value


# ---- full-integer FC --------------------------------------------------------

def _fc_dims(x, w):
    x = _c(x, np.int8)
    w = _c(w, np.int8)
    out_depth, depth = w.shape
    batches = x.size // depth
    return x, w, batches, depth, out_depth


def fc_int8_per_channel(x, w, bias, mult, shift, input_offset, output_offset, act_min, act_max,
                        single_rounding=False):
    x, w, B, K, N = _fc_dims(x, w)
    bias, mult, shift = _c(bias, np.int32), _c(mult, np.int32), _c(shift, np.int32)
    y = np.empty((B, N), dtype=np.int8)
    fn = (lib().orc_fc_int8_per_channel_single_rounding if single_rounding
          else lib().orc_fc_int8_per_channel)
    fn(_p(x, _i8p), _p(w, _i8p), _p(bias, _i32p), _p(mult, _i32p), _p(shift, _i32p),
       _p(y, _i8p), B, K, N, input_offset, output_offset, act_min, act_max)
    return y


def fc_int8_per_channel_float_scale(x, w, bias, filter_scales, in_scale, out_scale, input_offset,
                                    output_offset, act_min, act_max):
    x, w, B, K, N = _fc_dims(x, w)
    bias, fs = _c(bias, np.int32), _c(filter_scales, np.float32)
    y = np.empty((B, N), dtype=np.int8)
    lib().orc_fc_int8_per_channel_float_scale(
        _p(x, _i8p), _p(w, _i8p), _p(bias, _i32p), _p(fs, _f32p), in_scale, out_scale,
        _p(y, _i8p), B, K, N, input_offset, output_offset, act_min, act_max)
    return y


def fc_int8_per_tensor(x, w, bias, mult, shift, input_offset, filter_offset, output_offset,
                       act_min, act_max):
    x, w, B, K, N = _fc_dims(x, w)
    bias = _c(bias, np.int32)
    y = np.empty((B, N), dtype=np.int8)
    lib().orc_fc_int8_per_tensor(_p(x, _i8p), _p(w, _i8p), _p(bias, _i32p), int(mult), int(shift),
                                 _p(y, _i8p), B, K, N, input_offset, filter_offset, output_offset,
                                 act_min, act_max)
    return y


def fc_uint8_per_tensor(x, w, bias, mult, shift, input_offset, filter_offset, output_offset,
                        act_min, act_max):
    """x [B,K] and w [N,K] uint8; offsets are the negated uint8 zero points."""
    x = _c(x, np.uint8)
    w = _c(w, np.uint8)
    x = x.reshape(-1, w.shape[1])
    B, K, N = x.shape[0], w.shape[1], w.shape[0]
    bias = _c(bias, np.int32)
    y = np.empty((B, N), dtype=np.uint8)
    lib().orc_fc_uint8_per_tensor(_p(x, _u8p), _p(w, _u8p), _p(bias, _i32p), int(mult), int(shift),
                                  _p(y, _u8p), B, K, N, input_offset, filter_offset, output_offset,
                                  act_min, act_max)
    return y


def fc_int8_per_tensor_float_scale(x, w, bias, in_scale, filter_scale, out_scale, input_offset,
                                   filter_offset, output_offset, act_min, act_max):
    x, w, B, K, N = _fc_dims(x, w)
    bias = _c(bias, np.int32)
    y = np.empty((B, N), dtype=np.int8)
    lib().orc_fc_int8_per_tensor_float_scale(
        _p(x, _i8p), _p(w, _i8p), _p(bias, _i32p), in_scale, filter_scale, out_scale,
        _p(y, _i8p), B, K, N, input_offset, filter_offset, output_offset, act_min, act_max)
    return y


# ---- activation quantization ------------------------------------------------

def batch_quantize_floats(x, asymmetric=True, variant=QUANT_PORTABLE):
    x = _c(x, np.float32)
    B, K = x.shape
    q = np.empty((B, K), dtype=np.int8)
    sf = np.empty(B, dtype=np.float32)
    zp = np.zeros(B, dtype=np.int32)
    lib().orc_batch_quantize_floats(_p(x, _f32p), B, K, _p(q, _i8p), _p(sf, _f32p),
                                    _p(zp, _i32p), int(asymmetric), variant)
    return q, sf, zp


# ---- hybrid -----------------------------------------------------------------

def matrix_batch_vector_multiply_accumulate(matrix, vectors, scaling_factors, result,
                                            per_channel_scale=None, input_offset=None):
    m = _c(matrix, np.int8)
    v = _c(vectors, np.int8)
    rows, cols = m.shape
    n_batch = v.size // cols
    sf = _c(scaling_factors, np.float32)
    res = np.array(result, dtype=np.float32).reshape(n_batch, rows).copy()
    pcs = _c(per_channel_scale, np.float32)
    off = _c(input_offset, np.int32)
    row_sums = np.zeros(rows, dtype=np.int32)
    lib().orc_matrix_batch_vector_multiply_accumulate(
        _p(m, _i8p), rows, cols, _p(v, _i8p), _p(sf, _f32p), n_batch, _p(res, _f32p),
        _p(pcs, _f32p), _p(off, _i32p), _p(row_sums, _i32p), 1)
    return res


def have_sse():
    return bool(lib().orc_have_sse())


def matrix_batch_vector_multiply_accumulate_sse(matrix, vectors, scaling_factors, result,
                                                per_channel_scale=None, input_offset=None,
                                                row_sums=None):
    """The optimized-x86 tier (sse_tensor_utils.cc:308-379); row_sums are computed here when an
    input_offset is given and none are passed (the op caches them after its first Eval)."""
    m = _c(matrix, np.int8)
    v = _c(vectors, np.int8)
    rows, cols = m.shape
    n_batch = v.size // cols
    sf = _c(scaling_factors, np.float32)
    res = np.array(result, dtype=np.float32).reshape(n_batch, rows).copy()
    pcs = _c(per_channel_scale, np.float32)
    off = _c(input_offset, np.int32)
    if off is not None and row_sums is None:
        row_sums = m.astype(np.int32).sum(1).astype(np.int32)
    rs = _c(row_sums, np.int32)
    lib().orc_matrix_batch_vector_multiply_accumulate_sse(
        _p(m, _i8p), rows, cols, _p(v, _i8p), _p(sf, _f32p), n_batch, _p(res, _f32p),
        _p(pcs, _f32p), _p(off, _i32p), _p(rs, _i32p))
    return res


def fc_hybrid_sse(x, w, per_channel_scales, row_sums, asymmetric=True, variant=QUANT_PORTABLE):
    """EvalHybridDense with the optimized-x86 product (no bias, no activation: the form the CPU
    baseline times): BatchQuantizeFloats, then the SSE kernel on a zeroed output."""
    x = _c(x, np.float32)
    w = _c(w, np.int8)
    q, sf, zp = batch_quantize_floats(x.reshape(-1, w.shape[1]), asymmetric, variant)
    out = np.zeros((q.shape[0], w.shape[0]), np.float32)
    return matrix_batch_vector_multiply_accumulate_sse(
        w, q, sf, out, per_channel_scales, zp if asymmetric else None, row_sums)


def fc_hybrid(x, w, per_channel_scales=None, filter_scale=1.0, bias=None, asymmetric=True,
              activation=ACT_NONE, variant=QUANT_PORTABLE, return_quant=False, row_sums=None):
    """row_sums: an int32 [N] array already filled by an earlier call (the op's cached
    persistent temporary); None recomputes them."""
    x = _c(x, np.float32)
    w = _c(w, np.int8)
    N, K = w.shape
    B = x.size // K
    pcs = _c(per_channel_scales, np.float32)
    bias = _c(bias, np.float32)
    y = np.empty((B, N), dtype=np.float32)
    q = np.empty((B, K), dtype=np.int8)
    sf = np.empty(B, dtype=np.float32)
    zp = np.empty(B, dtype=np.int32)
    compute = row_sums is None
    if compute:
        row_sums = np.empty(N, dtype=np.int32)
    rc = lib().orc_fc_hybrid_cached(_p(x, _f32p), B, K, _p(w, _i8p), N, _p(pcs, _f32p),
                                    filter_scale, _p(bias, _f32p), int(asymmetric), activation,
                                    variant, _p(y, _f32p), _p(q, _i8p), _p(sf, _f32p),
                                    _p(zp, _i32p), _p(row_sums, _i32p), int(compute))
    if rc:
        raise ValueError("activation not restated in the oracle")
    return (y, q, sf, zp) if return_quant else y


# ---- BATCH_MATMUL hybrid ------------------------------------------------------

def batch_matmul_broadcast(lhs_shape, rhs_shape, adj_y=False):
    """Shapes and batch pairing of BATCH_MATMUL (tflite/kernels/batch_matmul.cc:356-391 and
    reference/batch_matmul.h:120-146): returns (rows, depth, units, output shape, lhs batch
    index per output batch, rhs batch index per output batch). lhs_shape is the left operand's
    shape after the op's adj_x transposition, [..., rows, depth]."""
    rank = max(len(lhs_shape), len(rhs_shape))
    le = (1,) * (rank - len(lhs_shape)) + tuple(lhs_shape)
    re = (1,) * (rank - len(rhs_shape)) + tuple(rhs_shape)
    rows, depth = le[-2], le[-1]
    units = re[-2] if adj_y else re[-1]
    assert (re[-1] if adj_y else re[-2]) == depth
    lb, rb = le[:-2], re[:-2]
    ob = []
    for a, b in zip(lb, rb):
        assert a == b or a == 1 or b == 1
        ob.append(max(a, b))
    li = np.arange(int(np.prod(lb, dtype=np.int64))).reshape(lb) if lb else np.zeros((), np.int64)
    ri = np.arange(int(np.prod(rb, dtype=np.int64))).reshape(rb) if rb else np.zeros((), np.int64)
    li = np.broadcast_to(li, ob).ravel().astype(np.int32)
    ri = np.broadcast_to(ri, ob).ravel().astype(np.int32)
    return rows, depth, units, tuple(ob) + (rows, units), li, ri


def batch_matmul_hybrid(lhs, rhs, per_channel_scales=None, filter_scale=1.0, asymmetric=True,
                        adj_y=False, variant=QUANT_PORTABLE, adj_x=False):
    """lhs float32 [..., M, K] (adj_x: [..., K, M]); rhs int8 [..., K, N] (adj_y: [..., N, K]);
    float32 [..., M, N]. adj_x is the op's own first step: the left operand's last two dimensions
    are transposed into a temporary (TransposeRowsColumns, batch_matmul.cc:811-813), and nothing
    after that knows of it."""
    lhs = _c(lhs, np.float32)
    if adj_x:
        lhs = np.ascontiguousarray(np.swapaxes(lhs, -1, -2))
    rhs = _c(rhs, np.int8)
    rows, depth, units, out_shape, li, ri = batch_matmul_broadcast(lhs.shape, rhs.shape, adj_y)
    w = rhs if adj_y else np.ascontiguousarray(np.swapaxes(rhs, -1, -2))  # the op's transposition
    pcs = _c(per_channel_scales, np.float32)
    out = np.empty(out_shape, np.float32)
    lib().orc_batch_matmul_hybrid(
        _p(lhs, _f32p), lhs.size // (rows * depth), rows, depth, _p(w, _i8p),
        w.size // (units * depth), units, _p(pcs, _f32p), filter_scale, int(asymmetric), variant,
        _p(li, _intp), _p(ri, _intp), li.size, _p(out, _f32p))
    return out


# ---- blockwise int4 ---------------------------------------------------------

def fc_blockwise_int4(x, packed_w, out_depth, scales_f16_bits, blocksize, bias=None,
                      variant=QUANT_PORTABLE):
    x = _c(x, np.float32)
    B, K = x.shape
    pw = _c(packed_w, np.uint8).ravel()
    sc = _c(scales_f16_bits, np.uint16).ravel()
    bias = _c(bias, np.float32)
    y = np.empty((B, out_depth), dtype=np.float32)
    lib().orc_fc_blockwise_int4(_p(x, _f32p), B, K, _p(pw, _u8p), out_depth, _p(sc, _u16p),
                                blocksize, _p(bias, _f32p), variant, _p(y, _f32p))
    return y


# ---- per-channel int4 hybrid --------------------------------------------------

def fc_hybrid_int4_per_channel(x, packed_w, out_depth, filter_scales, bias=None,
                               activation=ACT_NONE):
    """EvalHybridDense4Bit: x [B,K] float32, packed_w [N, K/2] nibbles (low = even k),
    filter_scales [N] (or one value, broadcast as the op does)."""
    x = _c(x, np.float32)
    B, K = x.shape
    pw = _c(packed_w, np.uint8).ravel()
    fs = np.ascontiguousarray(np.broadcast_to(np.asarray(filter_scales, np.float32).ravel(),
                                              (out_depth,)) if np.size(filter_scales) == 1
                              else np.asarray(filter_scales, np.float32))
    bias = _c(bias, np.float32)
    y = np.empty((B, out_depth), dtype=np.float32)
    lib().orc_fc_hybrid_int4_per_channel(_p(x, _f32p), B, K, _p(pw, _u8p), out_depth,
                                         _p(fs, _f32p), _p(bias, _f32p), activation,
                                         _p(y, _f32p))
    return y


# ---- EMBEDDING_LOOKUP from quantized tables ------------------------------------

class LookupOutOfBounds(ValueError):
    """A lookup index outside [0, rows); `position` is its place in the lookup vector."""

    def __init__(self, position):
        super().__init__(f"lookup {position} out of bounds")
        self.position = position


def float_to_half_bits(values):
    v = _c(values, np.float32).ravel()
    L = lib()
    L.orc_float_to_half.argtypes = [C.c_float]
    L.orc_float_to_half.restype = C.c_uint16
    return np.array([L.orc_float_to_half(float(f)) for f in v], dtype=np.uint16)


def _lookup_output(count, cols, out_f16):
    return np.zeros((count, cols), dtype=np.uint16 if out_f16 else np.float32)


def embedding_lookup_blockwise_int4(lookup, packed_table, rows, cols, scales_f16_bits, blocksize,
                                    out_f16=False):
    """EvalBlockwise: packed_table [rows, cols/2] nibbles (low = even column), scales
    [rows, cols/blocksize] as binary16 bit patterns. Returns float32 [count, cols], or binary16
    bit patterns (uint16) when out_f16."""
    lk = _c(lookup, np.int32).ravel()
    tb = _c(packed_table, np.uint8).ravel()
    sc = _c(scales_f16_bits, np.uint16).ravel()
    y = _lookup_output(lk.size, cols, out_f16)
    rc = lib().orc_embedding_lookup_blockwise_int4(
        _p(lk, _i32p), lk.size, _p(tb, _u8p), rows, cols, _p(sc, _u16p), blocksize, int(out_f16),
        y.ctypes.data_as(C.c_void_p))
    if rc < 0:
        raise LookupOutOfBounds(-rc - 1)
    if rc:
        raise ValueError("columns not divisible by the block size")
    return y


def embedding_lookup_hybrid(lookup, table, value_bits, rows, cols, scale=1.0, row_scales=None,
                            out_f16=False):
    """EvalHybrid: table int8 [rows, cols] (value_bits 8) or nibbles [rows*cols/2] (4)."""
    lk = _c(lookup, np.int32).ravel()
    tb = np.ascontiguousarray(table).view(np.uint8).ravel()
    rs = _c(row_scales, np.float32)
    y = _lookup_output(lk.size, cols, out_f16)
    L = lib()
    L.orc_embedding_lookup_hybrid.argtypes = [_i32p, C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_int,
                                              C.c_float, _f32p, C.c_int, C.c_void_p]
    rc = L.orc_embedding_lookup_hybrid(_p(lk, _i32p), lk.size, tb.ctypes.data_as(C.c_void_p),
                                       value_bits, rows, cols, float(scale), _p(rs, _f32p),
                                       int(out_f16), y.ctypes.data_as(C.c_void_p))
    if rc < 0:
        raise LookupOutOfBounds(-rc - 1)
    return y

"""Quantization-parameter derivation used by the reference's op tests, restated
so that its known-answer vectors can be replayed against the oracle and the HIP
path without the interpreter.

Follows SingleOpModel::QuantizationParams<T> (tflite/kernels/test_util.h:1123-1190)
and Quantize<T> (tflite/kernels/test_util.h:198-222): all arithmetic in float32.
"""
import numpy as np

f32 = np.float32


def _round_half_away(x):
    x = np.asarray(x)
    return np.sign(x) * np.floor(np.abs(x) + 0.5)


def quantization_params(f_min, f_max, qmin=-128, qmax=127):
    f_min, f_max = f32(f_min), f32(f_max)
    if f_min == f_max:
        return f32(0), 0
    qmin_f, qmax_f = f32(qmin), f32(qmax)
    scale = f32(f32(f_max - f_min) / f32(qmax_f - qmin_f))
    zp_from_min = f32(qmin_f - f32(f_min / scale))
    zp_from_max = f32(qmax_f - f32(f_max / scale))
    err_min = f32(abs(qmin_f) + abs(f32(f_min / scale)))
    err_max = f32(abs(qmax_f) + abs(f32(f_max / scale)))
    zp = zp_from_min if err_min < err_max else zp_from_max
    if zp < qmin_f:
        nudged = qmin
    elif zp > qmax_f:
        nudged = qmax
    else:
        nudged = int(_round_half_away(zp))
    return scale, nudged


def quantize(values, scale, zero_point, lo=-128, hi=127, dtype=np.int8):
    v = np.asarray(values, dtype=np.float32)
    q = _round_half_away(f32(zero_point) + v / f32(scale))
    return np.clip(q, lo, hi).astype(dtype)


def quantize_bias(values, scale):
    v = np.asarray(values, dtype=np.float32)
    return _round_half_away(v / f32(scale)).astype(np.int32)


def pack_int4(values_i8):
    """Two signed nibbles per byte, low nibble first (PopulateTensor4bit)."""
    v = np.asarray(values_i8, dtype=np.int8).ravel()
    if v.size % 2:
        v = np.concatenate([v, np.zeros(1, np.int8)])
    lo = v[0::2].astype(np.uint8) & 0xF
    hi = v[1::2].astype(np.uint8) & 0xF
    return (lo | (hi << 4)).astype(np.uint8)


def pack_int2(values_i8):
    """Four signed 2-bit values per byte, the first in bits 0-1 (PopulateTensor2bit; the inverse of
    portable_tensor_utils.cc:128-163)."""
    v = np.asarray(values_i8, dtype=np.int8).ravel()
    if v.size % 4:
        v = np.concatenate([v, np.zeros(4 - v.size % 4, np.int8)])
    u = v.astype(np.uint8) & 0x3
    return (u[0::4] | (u[1::4] << 2) | (u[2::4] << 4) | (u[3::4] << 6)).astype(np.uint8)


def symmetric_quantize_tensor(values):
    """SingleOpModel::QuantizeTensor (tflite/kernels/test_util.h:1407-1430): the whole tensor
    through SymmetricQuantizeFloats (reference/portable_tensor_utils.cc:41-71). Returns
    (int8 values, float32 scale)."""
    v = np.asarray(values, dtype=np.float32)
    rng = f32(np.max(np.abs(v))) if v.size else f32(0)
    if rng == 0:
        return np.zeros(v.shape, np.int8), f32(1)
    scale = f32(rng / f32(127))
    inv = f32(f32(127) / rng)
    q = np.clip(_round_half_away((v * inv).astype(np.float32)), -127, 127).astype(np.int8)
    return q, scale

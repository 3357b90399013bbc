"""ctypes binding of the C-ABI kernel library (include/litert_amd_fc.h).

The library is loaded from litert_amd/lib/liblitert_amd_fc.so, which
`python -m litert_amd.build` (or __graft_entry__.build()) produces. There is no
fallback: if the library is missing, or no gfx950 device is visible, the calls
raise.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "liblitert_amd_fc.so")

OK, INVALID_ARGUMENT, NO_DEVICE, HIP_ERROR, UNSUPPORTED = range(5)
ACT_NONE, ACT_RELU, ACT_RELU_N1_TO_1, ACT_RELU6 = range(4)
ACT_SIGN_BIT = 5
QUANT_PORTABLE, QUANT_NEON_V8, QUANT_NEON_LEGACY = range(3)
OUT_FLOAT32, OUT_FLOAT16 = range(2)
INT4_FORM_DECODE, INT4_FORM_GEMM_NIBBLES, INT4_FORM_GEMM_INT8 = range(3)

# Every symbol include/litert_amd_fc.h declares: (name, restype, argtypes).
_vp, _i, _i32, _i64, _f, _d, _sz = (C.c_void_p, C.c_int, C.c_int32, C.c_int64, C.c_float,
                                    C.c_double, C.c_size_t)
_pi32, _pint, _pf = C.POINTER(C.c_int32), C.POINTER(C.c_int), C.POINTER(C.c_float)
SYMBOLS = [
    ("lrtfc_abi_version", _i, []),
    ("lrtfc_last_error", C.c_char_p, []),
    ("lrtfc_init", _i, [_i]),
    ("lrtfc_quantize_multiplier", _i, [_d, _pi32, _pint]),
    ("lrtfc_prepare_per_channel", _i, [_f, _pf, _i, _f, _pi32, _pi32]),
    ("lrtfc_prepare_per_tensor", _i, [_f, _f, _i, _f, _f, _pi32, _pi32]),
    ("lrtfc_activation_range_int8", _i, [_i, _f, _i32, _pi32, _pi32]),
    ("lrtfc_row_sums_int8", _i, [_vp, _i, _i, _vp, _vp]),
    ("lrtfc_unpack_int4", _i, [_vp, _i64, _vp, _vp]),
    ("lrtfc_unpack_int2", _i, [_vp, _i64, _vp, _vp]),
    ("lrtfc_xor_sign_bit", _i, [_vp, _vp, _sz, _vp]),
    ("lrtfc_blockwise_int4_kfsum", _i, [_vp, _vp, _i, _i, _i, _vp, _vp]),
    ("lrtfc_fc_int8_preferred_layout", _i, [_i, _i, _i, _i]),
    ("lrtfc_fc_blockwise_int4_preferred_layout", _i, [_i, _i]),
    ("lrtfc_fc_hybrid_fused_max_batches", _i, [_i, _i]),
    ("lrtfc_packed_int8_filter_bytes", _sz, [_i, _i]),
    ("lrtfc_pack_int8_filter", _i, [_vp, _i, _i, _vp, _vp]),
    ("lrtfc_fc_int8_packed", _i, [_vp, _vp, _vp, _vp, _vp, _i, _vp, _vp, _i, _i, _i, _i32, _i32,
                                  _i32, _i32, _vp]),
    ("lrtfc_fc_hybrid_packed", _i, [_vp, _vp, _vp, _f, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i,
                                    _vp]),
    ("lrtfc_fc_int8", _i, [_vp, _vp, _vp, _vp, _vp, _i, _vp, _vp, _i, _i, _i, _i32, _i32, _i32,
                           _i32, _i32, _vp]),
    ("lrtfc_batch_quantize_floats", _i, [_vp, _i, _i, _vp, _vp, _vp, _i, _i, _vp]),
    ("lrtfc_fc_hybrid_int8", _i, [_vp, _vp, _vp, _vp, _vp, _f, _vp, _vp, _vp, _i, _i, _i, _i,
                                  _vp]),
    ("lrtfc_fc_hybrid_int8_packed", _i, [_vp, _vp, _vp, _vp, _vp, _f, _vp, _vp, _vp, _i, _i, _i,
                                         _i, _vp]),
    ("lrtfc_activation_workspace_bytes", _sz, [_i, _i]),
    ("lrtfc_fc_hybrid", _i, [_vp, _vp, _vp, _f, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp, _sz,
                             _vp]),
    ("lrtfc_fc_hybrid_packed_workspace", _i, [_vp, _vp, _vp, _f, _vp, _vp, _vp, _i, _i, _i, _i,
                                              _i, _i, _vp, _sz, _vp]),
    ("lrtfc_batch_matmul_hybrid_packed", _i, [_vp, _i, _i, _i, _vp, _i, _i, _vp, _f, _vp, _vp, _i,
                                              _i, _vp, _sz, _vp]),
    ("lrtfc_batch_matmul_workspace_bytes", _sz, [_i, _i, _i, _i]),
    ("lrtfc_batch_matmul_hybrid_packed_nd", _i, [_vp, _vp, _i, _i, _i, _vp, _vp, _i, _vp, _f, _vp,
                                                 _vp, _i, _i, _vp, _sz, _vp]),
    ("lrtfc_static_scratch_bytes", _sz, []),
    ("lrtfc_fc_hybrid_static_scratch", _i, [_vp, _vp, _vp, _f, _vp, _vp, _vp, _i, _i, _i, _i, _i,
                                            _i, _vp]),
    ("lrtfc_fc_blockwise_int4", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp, _sz,
                                     _vp]),
    ("lrtfc_packed_int4_blockwise_bytes", _sz, [_i, _i]),
    ("lrtfc_pack_int4_blockwise", _i, [_vp, _vp, _i, _i, _i, _vp, _vp]),
    ("lrtfc_fc_blockwise_int4_packed", _i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    ("lrtfc_fc_blockwise_int4_packed_quantized", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i,
                                                      _i, _vp]),
    ("lrtfc_batch_quantize_floats_4bit", _i, [_vp, _i, _i, _vp, _vp, _vp, _vp]),
    ("lrtfc_fc_hybrid_int4_per_channel_packed", _i, [_vp, _vp, _vp, _f, _vp, _vp, _i, _i, _i, _i,
                                                     _vp, _sz, _vp]),
    ("lrtfc_packed_int4_per_channel_bytes", _sz, [_i, _i]),
    ("lrtfc_pack_int4_per_channel", _i, [_vp, _i, _i, _vp, _vp]),
    ("lrtfc_fc_hybrid_int4_per_channel_nibbles", _i, [_vp, _vp, _vp, _f, _vp, _vp, _i, _i, _i, _i,
                                                      _vp, _sz, _vp]),
    ("lrtfc_gemm_int4_blockwise_bytes", _sz, [_i, _i]),
    ("lrtfc_pack_int4_blockwise_gemm", _i, [_vp, _vp, _i, _i, _i, _vp, _vp]),
    ("lrtfc_fc_blockwise_int4_gemm_workspace_bytes", _sz, [_i, _i]),
    ("lrtfc_fc_blockwise_int4_gemm", _i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp, _sz, _vp]),
    ("lrtfc_fc_blockwise_int4_preferred_form", _i, [_i, _i, _i]),
    ("lrtfc_gemm_int4_blockwise_nibble_bytes", _sz, [_i, _i]),
    ("lrtfc_pack_int4_blockwise_gemm_nibbles", _i, [_vp, _vp, _i, _i, _i, _vp, _vp]),
    ("lrtfc_fc_blockwise_int4_gemm_nibbles", _i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp, _sz,
                                                  _vp]),
    ("lrtfc_embedding_lookup_blockwise_int4", _i, [_vp, _i, _vp, _i, _i, _vp, _i, _i, _vp, _vp, _vp]),
    ("lrtfc_embedding_lookup_hybrid", _i, [_vp, _i, _vp, _i, _i, _i, _f, _vp, _i, _vp, _vp, _vp]),
    ("lrtfc_mark_completion", _i, [_vp, C.c_uint32, _vp]),
    ("lrtfc_int4_group_table_bytes", _sz, []),
    ("lrtfc_int4_group_preferred_form", _i, [_vp, _i, _i, _i]),
    ("lrtfc_int4_group_prepare", _i, [_vp, _i, _i, _i, _vp, _vp, _vp]),
    ("lrtfc_fc_blockwise_int4_packed_grouped", _i, [_vp, _vp, _i, _vp]),
    ("lrtfc_fc_blockwise_int4_quantized", _i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i,
                                               _i, _vp]),
]

_LIB = None


class LrtFcError(RuntimeError):
    def __init__(self, status, message):
        super().__init__("litert_amd_fc status %d: %s" % (status, message))
        self.status = status


def load():
    """Loads the shared library and binds every declared symbol (no device needed)."""
    global _LIB
    if _LIB is None:
        if not os.path.exists(LIB_PATH):
            raise FileNotFoundError(
                LIB_PATH + " is missing: run `python -m litert_amd.build` (hipcc, gfx950) first")
        lib = C.CDLL(LIB_PATH)
        for name, restype, argtypes in SYMBOLS:
            fn = getattr(lib, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _LIB = lib
    return _LIB


def check(status):
    if status != OK:
        raise LrtFcError(status, load().lrtfc_last_error().decode())


def init(device=0):
    check(load().lrtfc_init(device))


class Int4GroupNode(C.Structure):
    """lrtfc_int4_group_node."""
    _fields_ = [("input", C.c_void_p), ("retiled_filter", C.c_void_p), ("kfsum", C.c_void_p),
                ("bias", C.c_void_p), ("output", C.c_void_p), ("out_depth", C.c_int),
                ("workspace", C.c_void_p), ("nibble_filter", C.c_void_p)]


class Int4GroupLaunch(C.Structure):
    """lrtfc_int4_group_launch."""
    _fields_ = [("count", C.c_int), ("grid_blocks", C.c_int), ("ksplit", C.c_int),
                ("groups_per_wave", C.c_int), ("batches", C.c_int), ("depth", C.c_int),
                ("split_quantize", C.c_int), ("form", C.c_int)]

"""ctypes binding of the benchmark's two measurement aids (bench_probes.h beside this file):
a launch that only streams bytes and a launch that only issues MFMAs. A library of its own,
loaded by bench.py and tests/test_gpu_probes.py; the kernel library and the delegate know
nothing of it."""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(os.path.dirname(_HERE), "lib", "liblitert_amd_bench_probes.so")

_vp, _i, _sz = C.c_void_p, C.c_int, C.c_size_t
SYMBOLS = [
    ("lrtprobe_last_error", C.c_char_p, []),
    ("lrtprobe_stream_read", _i, [_vp, _sz, _vp, _vp]),
    ("lrtprobe_mfma_rate", _i, [_i, _i, _i, _vp, C.POINTER(C.c_double), _vp]),
]

_LIB = None


def load():
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
    if status != 0:
        raise RuntimeError("bench probe status %d: %s" %
                           (status, load().lrtprobe_last_error().decode()))

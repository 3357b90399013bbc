"""The LiteRT accelerator skin: the exported LiteRtAcceleratorImpl object as the LiteRT runtime
would consume it (litert/runtime/accelerators/registration_helper.cc:34-86): ABI header, the
five mandatory callbacks, and create_delegate against a stand-in runtime context whose
wrap_delegate records what it is handed."""
import ctypes as C
import os

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "litert_amd", "lib", "liblitert_amd_delegate.so")


class AbiHeader(C.Structure):
    _fields_ = [("struct_size", C.c_uint16), ("major_version", C.c_uint16),
                ("minor_version", C.c_uint16), ("reserved", C.c_uint16)]


class BufferHandlers(C.Structure):
    _fields_ = [("abi_header", AbiHeader)] + [(n, C.c_void_p) for n in (
        "create_func", "destroy_func", "lock_func", "unlock_func", "clear_func", "import_func")] + [
        ("device_tag", C.c_int), ("queue_tag", C.c_int), ("num_supported_buffer_types", C.c_size_t),
        ("supported_buffer_types", C.c_int * 16)]


class ApiVersion(C.Structure):
    _fields_ = [("major", C.c_int), ("minor", C.c_int), ("patch", C.c_int)]


DELETER = C.CFUNCTYPE(None, C.c_void_p)
WRAP = C.CFUNCTYPE(C.c_int, C.c_void_p, DELETER, C.POINTER(C.c_void_p))
UNWRAP = C.CFUNCTYPE(C.c_int, C.c_void_p, C.POINTER(C.c_void_p))


class RuntimeContext(C.Structure):
    _fields_ = [("abi_header", AbiHeader), ("before", C.c_void_p * 17), ("wrap_delegate", WRAP),
                ("unwrap_delegate", UNWRAP)]


class AcceleratorDef(C.Structure):
    _fields_ = [("abi_header", AbiHeader),
                ("get_name", C.CFUNCTYPE(C.c_int, C.c_void_p, C.POINTER(C.c_char_p))),
                ("get_version", C.CFUNCTYPE(C.c_int, C.c_void_p, C.POINTER(ApiVersion))),
                ("get_hardware_support", C.CFUNCTYPE(C.c_int, C.c_void_p, C.POINTER(C.c_int))),
                ("is_jit", C.CFUNCTYPE(C.c_int, C.c_void_p, C.POINTER(C.c_bool))),
                ("create_delegate", C.CFUNCTYPE(C.c_int, C.POINTER(RuntimeContext), C.c_void_p,
                                                C.c_void_p, C.c_void_p, C.POINTER(C.c_void_p))),
                ("start_metrics_collection", C.CFUNCTYPE(C.c_int, C.POINTER(RuntimeContext),
                                                         C.c_void_p, C.c_int)),
                ("stop_metrics_collection", C.CFUNCTYPE(C.c_int, C.POINTER(RuntimeContext),
                                                        C.c_void_p, C.c_void_p)),
                ("buffer_handlers", BufferHandlers)]


def _impl():
    lib = C.CDLL(LIB)
    return lib, AcceleratorDef.in_dll(lib, "LiteRtAcceleratorImpl")


def test_layout_constants_of_the_reference():
    # litert_accelerator_def.h:74-97, litert_custom_tensor_buffer_handlers_def.h:52-68,
    # litert_runtime_context.h:259-262
    assert C.sizeof(AcceleratorDef) == 200 and AcceleratorDef.buffer_handlers.offset == 64
    assert C.sizeof(BufferHandlers) == 136 and BufferHandlers.supported_buffer_types.offset == 72
    assert RuntimeContext.wrap_delegate.offset == 144 and RuntimeContext.unwrap_delegate.offset == 152


def test_exported_table_is_what_the_runtime_accepts():
    _, d = _impl()
    assert (d.abi_header.struct_size, d.abi_header.major_version) == (200, 1)
    for f in ("get_name", "get_version", "get_hardware_support", "is_jit", "create_delegate",
              "start_metrics_collection", "stop_metrics_collection"):
        assert C.cast(getattr(d, f), C.c_void_p).value, f
    assert d.buffer_handlers.num_supported_buffer_types < 16  # registration_helper.cc:48-49
    name = C.c_char_p()
    assert d.get_name(None, C.byref(name)) == 0 and name.value == b"litert_amd_fc_mi355x"
    v = ApiVersion()
    assert d.get_version(None, C.byref(v)) == 0 and (v.major, v.minor, v.patch) == (0, 1, 0)
    hw = C.c_int()
    assert d.get_hardware_support(None, C.byref(hw)) == 0 and hw.value == 2  # kLiteRtHwAcceleratorGpu
    jit = C.c_bool(True)
    assert d.is_jit(None, C.byref(jit)) == 0 and jit.value is False
    assert d.get_name(None, None) == 1  # kLiteRtStatusErrorInvalidArgument


def _context(record):
    def wrap(delegate, deleter, out):
        record["delegate"] = delegate
        record["deleter"] = deleter
        out[0] = 0xABC0
        return 0
    ctx = RuntimeContext()
    ctx.abi_header = AbiHeader(C.sizeof(RuntimeContext), 1, 0, 0)
    ctx.wrap_delegate = WRAP(wrap)
    record["keepalive"] = ctx.wrap_delegate
    return ctx


def test_create_delegate_rejects_bad_arguments_without_touching_the_device():
    _, d = _impl()
    out = C.c_void_p()
    assert d.create_delegate(None, None, None, None, C.byref(out)) == 1
    rec = {}
    ctx = _context(rec)
    assert d.create_delegate(C.byref(ctx), None, None, None, None) == 1
    short = _context({})
    short.abi_header.struct_size = 100  # a table that ends before wrap_delegate
    assert d.create_delegate(C.byref(short), None, None, None, C.byref(out)) == 1


def test_create_delegate_without_gpu_fails_cleanly():
    torch = pytest.importorskip("torch")
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    _, d = _impl()
    rec, out = {}, C.c_void_p()
    ctx = _context(rec)
    assert d.create_delegate(C.byref(ctx), None, None, None, C.byref(out)) == 3  # runtime failure
    assert "delegate" not in rec


@pytest.mark.gpu
def test_create_delegate_hands_a_working_delegate_to_the_runtime():
    torch = pytest.importorskip("torch")
    if not torch.cuda.is_available():
        pytest.fail("GPU tests need a gfx950 device; none visible")
    _, d = _impl()
    rec, out = {}, C.c_void_p()
    ctx = _context(rec)
    assert d.create_delegate(C.byref(ctx), None, None, None, C.byref(out)) == 0
    assert out.value == 0xABC0 and rec["delegate"]
    # the wrapped object is a TfLiteDelegate whose Prepare is set (tflite/core/c/common.h:1442-1493)
    prepare = C.cast(rec["delegate"] + 8, C.POINTER(C.c_void_p))[0]
    assert prepare
    rec["deleter"](rec["delegate"])  # what the runtime does when the wrapper dies


def test_metrics_callbacks_reject_what_they_cannot_unwrap():
    """start/stop_metrics_collection (litert_accelerator_def.h:57-62) reach the delegate through
    the runtime context's unwrap_delegate; without one, or with a wrapper it refuses, they fail
    with kLiteRtStatusErrorInvalidArgument and touch nothing."""
    lib, d = _impl()
    assert d.start_metrics_collection(None, 0x1, 0) == 1
    ctx = _context({})  # no unwrap_delegate in this table
    assert d.start_metrics_collection(C.byref(ctx), 0x1, 0) == 1
    ctx.unwrap_delegate = UNWRAP(lambda wrapper, out: 1)
    assert d.start_metrics_collection(C.byref(ctx), 0x1, 0) == 1
    lib.litert_amd_metrics_object_new.restype = C.c_void_p
    lib.litert_amd_metrics_object_free.argtypes = [C.c_void_p]
    m = lib.litert_amd_metrics_object_new()
    assert d.stop_metrics_collection(C.byref(ctx), 0x1, m) == 1
    assert d.stop_metrics_collection(C.byref(ctx), 0x1, None) == 1
    lib.litert_amd_metrics_object_free(m)


@pytest.mark.gpu
def test_metrics_collection_reports_what_the_partitions_did():
    torch = pytest.importorskip("torch")
    if not torch.cuda.is_available():
        pytest.fail("GPU tests need a gfx950 device; none visible")
    import numpy as np
    from litert_amd import workloads as wl
    from tests.fake_host import FakeHost, FLOAT32, INT8, OK
    lib, d = _impl()
    lib.litert_amd_metrics_object_new.restype = C.c_void_p
    lib.litert_amd_metrics_object_free.argtypes = [C.c_void_p]
    lib.litert_amd_metrics_object_size.argtypes = [C.c_void_p]
    lib.litert_amd_metrics_object_name.argtypes = [C.c_void_p, C.c_int]
    lib.litert_amd_metrics_object_name.restype = C.c_char_p
    lib.litert_amd_metrics_object_value.argtypes = [C.c_void_p, C.c_int]
    lib.litert_amd_metrics_object_value.restype = C.c_double
    c = wl.hybrid_fc(2, 512, 64)
    with FakeHost() as h:
        x = h.tensor(FLOAT32, (2, 512), data=c["x"])
        w = h.tensor(INT8, (64, 512), data=c["w"], const=True)
        h.affine(w, c["pcs"])
        y = h.tensor(FLOAT32, (2, 64))
        h.fc(x, w, None, y)
        assert h.load_delegate() == 0 and h.modify_graph_with_delegate() == OK, h.errors()
        assert h.allocate_tensors() == OK, h.errors()
        delegate = h.L.fh_delegate(h.h)

        def unwrap(wrapper, out):
            out[0] = delegate if wrapper == 0xABC0 else None
            return 0 if wrapper == 0xABC0 else 1
        ctx = _context({})
        ctx.unwrap_delegate = UNWRAP(unwrap)
        m = lib.litert_amd_metrics_object_new()
        assert d.stop_metrics_collection(C.byref(ctx), 0xABC0, m) == 1  # nothing was started
        assert h.invoke() == OK  # before the collection: not counted
        assert d.start_metrics_collection(C.byref(ctx), 0xABC0, 1) == 0  # level 1: device time too
        for _ in range(3):
            assert h.invoke() == OK, h.errors()
        assert d.stop_metrics_collection(C.byref(ctx), 0xABC0, m) == 0
        got = {lib.litert_amd_metrics_object_name(m, i).decode(): lib.litert_amd_metrics_object_value(m, i)
               for i in range(lib.litert_amd_metrics_object_size(m))}
        lib.litert_amd_metrics_object_free(m)
        m0 = lib.litert_amd_metrics_object_new()
        assert d.start_metrics_collection(C.byref(ctx), 0xABC0, 0) == 0  # level 0: host side only
        assert h.invoke() == OK, h.errors()
        assert d.stop_metrics_collection(C.byref(ctx), 0xABC0, m0) == 0
        got0 = {lib.litert_amd_metrics_object_name(m0, i).decode(): lib.litert_amd_metrics_object_value(m0, i)
                for i in range(lib.litert_amd_metrics_object_size(m0))}
        lib.litert_amd_metrics_object_free(m0)
        assert got0["litert_amd.partition_invokes"] == 1 and got0["litert_amd.device_time_us"] == 0
        assert got0["litert_amd.host_time_us"] > 0
        assert got["litert_amd.partition_invokes"] == 3 and got["litert_amd.nodes_run"] == 3
        assert got["litert_amd.bytes_uploaded"] == 3 * c["x"].nbytes
        assert got["litert_amd.bytes_downloaded"] == 3 * 2 * 64 * 4
        assert 0 < got["litert_amd.device_time_us"] <= got["litert_amd.host_time_us"]
        phases = [got["litert_amd.host_%s_us" % p] for p in ("gather", "enqueue", "wait", "scatter")]
        assert all(v > 0 for v in phases)
        assert abs(sum(phases) - got["litert_amd.host_time_us"]) < 1e-6 * got["litert_amd.host_time_us"] + 1e-3
        assert h.invoke() == OK  # collection is off again

"""CPU-side checks of the product's C ABI: the library loads, exports every symbol the
header declares, does the Prepare-time host math like the oracle, and refuses to
compute without a gfx950 device instead of falling back."""
import ctypes as C
import os
import re

import numpy as np
import pytest

import oracle
from litert_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _header_symbols():
    text = open(os.path.join(ROOT, "include", "litert_amd_fc.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(lrtfc_[a-z0-9_]+)\s*\(", text)))


def test_delegate_plugin_exports_every_declared_symbol():
    """include/litert_amd_delegate.h and the plugin entry points of include/tflite_abi.h."""
    text = open(os.path.join(ROOT, "include", "litert_amd_delegate.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    declared = sorted(set(re.findall(r"\b(litert_amd_[a-z0-9_]+)\s*\(", text)))
    assert len(declared) == 10
    lib = C.CDLL(os.path.join(ROOT, "litert_amd", "lib", "liblitert_amd_delegate.so"))
    for name in declared + ["tflite_plugin_create_delegate", "tflite_plugin_destroy_delegate",
                            "LiteRtAcceleratorImpl"]:
        assert hasattr(lib, name), name


def test_bench_probe_library_is_separate_and_exports_its_header():
    """The measurement aids have their own header and library; the kernel library's header
    declares none of them."""
    from litert_amd import bench_probes as probes
    text = open(os.path.join(ROOT, "litert_amd", "bench_probes", "bench_probes.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    declared = sorted(set(re.findall(r"\b(lrtprobe_[a-z0-9_]+)\s*\(", text)))
    assert declared == ["lrtprobe_last_error", "lrtprobe_mfma_rate", "lrtprobe_stream_read"]
    lib = probes.load()
    for name in declared:
        assert hasattr(lib, name), name
    assert not [n for n in _header_symbols() if "probe" in n]
    fc_lib = capi.load()
    assert not hasattr(fc_lib, "lrtfc_stream_read_probe")
    assert not hasattr(fc_lib, "lrtfc_mfma_rate_probe")


def test_library_exports_every_declared_symbol():
    lib = capi.load()
    declared = _header_symbols()
    assert len(declared) >= 17
    for name in declared:
        assert hasattr(lib, name), name
    assert sorted(n for n, _, _ in capi.SYMBOLS) == declared
    assert lib.lrtfc_abi_version() == 2


def test_host_prepare_math_matches_oracle():
    lib = capi.load()
    rng = np.random.default_rng(1)
    for m in np.concatenate([np.exp(rng.uniform(np.log(1e-11), np.log(50), 3000)), [0.0, 0.5, 1.0]]):
        q, s = C.c_int32(), C.c_int()
        assert lib.lrtfc_quantize_multiplier(float(m), C.byref(q), C.byref(s)) == 0
        assert (q.value, s.value) == oracle.quantize_multiplier(float(m))
    from litert_amd import fully_connected as fc
    ws = np.exp(rng.uniform(np.log(1e-3), np.log(1e-2), 257)).astype(np.float32)
    m1, s1 = fc.prepare_per_channel(0.02, ws, 0.05)
    m2, s2 = oracle.fc_prepare_per_channel(0.02, ws, 0.05)
    assert np.array_equal(m1, m2) and np.array_equal(s1, s2)
    assert fc.prepare_per_tensor(0.5, 0.5, 1.0, 0.25) == oracle.fc_prepare_per_tensor(0.5, 0.5, 1.0, 0.25)
    with pytest.raises(capi.LrtFcError):
        fc.prepare_per_tensor(0.5, 0.5, 1.0, 0.5)  # bias scale off by 0.25 output quanta
    for act in range(4):
        for scale, zp in ((0.05, 5), (1.0, -1), (0.4, 3), (0.01, -128)):
            assert fc.activation_range_int8(act, scale, zp) == oracle.activation_range_int8(act, scale, zp)


def test_no_device_is_an_error_not_a_fallback():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    lib = capi.load()
    assert lib.lrtfc_init(0) == capi.NO_DEVICE
    assert b"HIP device" in lib.lrtfc_last_error()
    # compute entry points refuse to run before a successful init
    rc = lib.lrtfc_row_sums_int8(None, 4, 16, None, None)
    assert rc == capi.NO_DEVICE
    rc = lib.lrtfc_embedding_lookup_blockwise_int4(None, 1, None, 4, 64, None, 32, capi.OUT_FLOAT32,
                                                   None, None, None)
    assert rc == capi.NO_DEVICE
    rc = lib.lrtfc_embedding_lookup_hybrid(None, 1, None, 8, 4, 64, 0.5, None, capi.OUT_FLOAT16, None,
                                           None, None)
    assert rc == capi.NO_DEVICE
    # the host mirrors raise instead of computing anywhere else
    from litert_amd import embedding_lookup as el
    with pytest.raises(Exception):
        el.EmbeddingLookupHybrid(np.zeros((4, 8), np.int8), 8)

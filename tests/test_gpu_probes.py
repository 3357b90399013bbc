"""The library's two measurement aids (no counterpart in the reference): a launch that only
streams bytes and a launch that only issues MFMAs. They compute nothing that is kept; the tests
pin their argument checks and what they report."""
import ctypes as C

import numpy as np
import pytest

from litert_amd import capi

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def lib():
    if not torch.cuda.is_available():
        pytest.fail("GPU tests need a gfx950 device; none visible")
    from litert_amd import fully_connected as fc
    fc._ensure_init()
    return capi.load()


def _stream():
    return torch.cuda.current_stream().cuda_stream


def test_stream_read_probe_reads_without_writing(lib):
    src = torch.randint(0, 256, (1 << 20,), dtype=torch.uint8, device="cuda")
    keep = src.clone()
    sink = torch.zeros(1, dtype=torch.int32, device="cuda")
    for nbytes in (0, 15, 16, 4096, (1 << 20) - 16, 1 << 20):
        capi.check(lib.lrtfc_stream_read_probe(src.data_ptr(), nbytes, sink.data_ptr(), _stream()))
    capi.check(lib.lrtfc_stream_read_probe(src.data_ptr(), 1 << 20, None, _stream()))
    torch.cuda.synchronize()
    assert torch.equal(src, keep) and int(sink.item()) == 0
    assert lib.lrtfc_stream_read_probe(src.data_ptr() + 4, 4096, None, _stream()) != 0
    assert b"16-byte aligned" in lib.lrtfc_last_error()


def test_mfma_rate_probe_reports_its_operations_and_runs(lib):
    sink = torch.full((8 * 256,), -1, dtype=torch.int32, device="cuda")
    ops = C.c_double(0.0)
    for random_operands in (1, 0):
        capi.check(lib.lrtfc_mfma_rate_probe(8, 3, random_operands, sink.data_ptr(), C.byref(ops),
                                             _stream()))
        torch.cuda.synchronize()
        assert ops.value == 65536.0 * 8 * 3 * 4 * 8   # 8 MFMAs x 3 iterations x 4 wavefronts x 8 workgroups
    # constant operands: every accumulator element is 3 iterations x 32 x (5 * 3); the XOR of an
    # even number of equal values is zero
    assert not sink.cpu().numpy().any()
    capi.check(lib.lrtfc_mfma_rate_probe(1, 1, 0, sink.data_ptr(), None, _stream()))
    assert lib.lrtfc_mfma_rate_probe(0, 1, 0, sink.data_ptr(), None, _stream()) != 0
    assert lib.lrtfc_mfma_rate_probe(1, 0, 0, sink.data_ptr(), None, _stream()) != 0
    assert lib.lrtfc_mfma_rate_probe(1, 1, 0, None, None, _stream()) != 0

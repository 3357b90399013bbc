"""The benchmark's two measurement aids (a library of their own) (no counterpart in the reference): a launch that only
streams bytes and a launch that only issues MFMAs. They compute nothing that is kept; the tests
pin their argument checks and what they report."""
import ctypes as C

import numpy as np
import pytest

from litert_amd import bench_probes as probes

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def lib():
    if not torch.cuda.is_available():
        pytest.fail("GPU tests need a gfx950 device; none visible")
    from litert_amd import fully_connected as fc
    fc._ensure_init()
    return probes.load()


def _stream():
    return torch.cuda.current_stream().cuda_stream


def test_stream_read_probe_reads_without_writing(lib):
    src = torch.randint(0, 256, (1 << 20,), dtype=torch.uint8, device="cuda")
    keep = src.clone()
    sink = torch.zeros(1, dtype=torch.int32, device="cuda")
    for nbytes in (0, 15, 16, 4096, (1 << 20) - 16, 1 << 20):
        probes.check(lib.lrtprobe_stream_read(src.data_ptr(), nbytes, sink.data_ptr(), _stream()))
    probes.check(lib.lrtprobe_stream_read(src.data_ptr(), 1 << 20, None, _stream()))
    torch.cuda.synchronize()
    assert torch.equal(src, keep) and int(sink.item()) == 0
    assert lib.lrtprobe_stream_read(src.data_ptr() + 4, 4096, None, _stream()) != 0
    assert b"16-byte aligned" in lib.lrtprobe_last_error()


def test_mfma_rate_probe_reports_its_operations_and_runs(lib):
    sink = torch.full((8 * 256,), -1, dtype=torch.int32, device="cuda")
    ops = C.c_double(0.0)
    for random_operands in (1, 0):
        probes.check(lib.lrtprobe_mfma_rate(8, 3, random_operands, sink.data_ptr(), C.byref(ops),
                                             _stream()))
        torch.cuda.synchronize()
        assert ops.value == 65536.0 * 8 * 3 * 4 * 8   # 8 MFMAs x 3 iterations x 4 wavefronts x 8 workgroups
    # constant operands: every accumulator element is 3 iterations x 32 x (5 * 3); the XOR of an
    # even number of equal values is zero
    assert not sink.cpu().numpy().any()
    probes.check(lib.lrtprobe_mfma_rate(1, 1, 0, sink.data_ptr(), None, _stream()))
    assert lib.lrtprobe_mfma_rate(0, 1, 0, sink.data_ptr(), None, _stream()) != 0
    assert lib.lrtprobe_mfma_rate(1, 0, 0, sink.data_ptr(), None, _stream()) != 0
    assert lib.lrtprobe_mfma_rate(1, 1, 0, None, None, _stream()) != 0
    # One launch is bounded (about 0.1 s of matrix-core time): a careless iteration count is
    # refused instead of occupying the device for minutes.
    assert lib.lrtprobe_mfma_rate(256, 1000000000, 0, sink.data_ptr(), None, _stream()) != 0
    assert b"more than one launch may hold" in lib.lrtprobe_last_error()

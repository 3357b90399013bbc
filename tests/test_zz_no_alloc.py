"""lrtfc_fc_hybrid_static_scratch (the entry point that allocates nothing: its activation
scratch is a static device array) against lrtfc_fc_hybrid with a caller-owned workspace, bit
for bit, on two calls in a row, the second with a smaller input; plus the size limit.

Collected last on purpose: it leaves the shared scratch array written, and a failure here
must not hide the other GPU tests.
"""
import ctypes as C

import numpy as np
import pytest

import oracle
from litert_amd import workloads as wl

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


def _p(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def _cuda(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _both(lib, capi, c, bias, asym, activation):
    """Runs one shape through both entry points; every buffer exists before the calls."""
    B, K = c["x"].shape
    N = c["w"].shape[0]
    x, w, pcs = _cuda(c["x"]), _cuda(c["w"]), _cuda(c["pcs"])
    b = None if bias is None else _cuda(bias)
    rs = torch.empty(N, dtype=torch.int32, device="cuda")
    capi.check(lib.lrtfc_row_sums_int8(_p(w), N, K, _p(rs), None))
    need = lib.lrtfc_activation_workspace_bytes(B, K)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    want = torch.full((B, N), float("nan"), dtype=torch.float32, device="cuda")
    got = torch.full((B, N), float("nan"), dtype=torch.float32, device="cuda")
    torch.cuda.synchronize()
    capi.check(lib.lrtfc_fc_hybrid(_p(x), _p(w), _p(pcs), 1.0, _p(rs), _p(b), _p(want), B, K, N,
                                   int(asym), activation, 0, _p(ws), need, None))
    # Free device memory as the driver sees it (hipMemGetInfo): a hipMalloc inside the entry
    # point would lower it, which torch's own allocator statistics cannot see.
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    free_before = torch.cuda.mem_get_info()[0]
    capi.check(lib.lrtfc_fc_hybrid_static_scratch(_p(x), _p(w), _p(pcs), 1.0, _p(rs), _p(b),
                                                  _p(got), B, K, N, int(asym), activation, 0,
                                                  None))
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.cuda.mem_get_info()[0] == free_before
    return got.cpu().numpy(), want.cpu().numpy()


def test_static_scratch_matches_workspace_entry_point_twice():
    if not torch.cuda.is_available():
        pytest.fail("GPU tests need a gfx950 device; none visible")
    from litert_amd import capi
    capi.init(torch.cuda.current_device())
    lib = capi.load()
    assert lib.lrtfc_static_scratch_bytes() == 1024 * 1024 + 64 * 1024
    bias = np.random.default_rng(5).standard_normal(300).astype(np.float32)
    # First call: 8 rows of depth 4096 (config 2's batch and depth). Second call: smaller in
    # both dimensions, so stale rows of the first call lie behind what it writes.
    for (B, K, N, b, asym, act) in ((8, 4096, 300, bias, True, 0), (3, 520, 77, None, True, 1),
                                    (2, 64, 5, None, False, 3)):
        c = wl.hybrid_fc(B, K, N, seed=100 + B)
        got, want = _both(lib, capi, c, None if b is None else b[:N], asym, act)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (B, K, N)
        ref = oracle.fc_hybrid(c["x"], c["w"], c["pcs"], 1.0, None if b is None else b[:N], asym,
                               act)
        assert np.array_equal(got.view(np.uint32), ref.view(np.uint32)), (B, K, N)


def test_static_scratch_rejects_oversized_rows():
    if not torch.cuda.is_available():
        pytest.fail("GPU tests need a gfx950 device; none visible")
    from litert_amd import capi
    capi.init(torch.cuda.current_device())
    lib = capi.load()
    dummy = torch.zeros(16, dtype=torch.float32, device="cuda")
    # 128 rows of depth 16384 need 2 MiB of quantized rows: over the limit, refused before
    # any pointer is read.
    rc = lib.lrtfc_fc_hybrid_static_scratch(_p(dummy), _p(dummy), None, 1.0, _p(dummy), None,
                                            _p(dummy), 128, 16384, 4, 1, 0, 0, None)
    assert rc == capi.INVALID_ARGUMENT
    assert b"static scratch" in lib.lrtfc_last_error()

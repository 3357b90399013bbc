"""BATCH_MATMUL hybrid (float32 x constant int8) on the GPU against the oracle's restatement of
batch_matmul::EvalHybrid (tflite/kernels/batch_matmul.cc:454-520), bit for bit: every
broadcasting form the entry point offers, adj_y, symmetric and asymmetric inputs, per-channel
and per-tensor scales, row counts on both sides of the GEMV / GEMM switch, and rows deep enough
that the reference kernel's float zero-point correction rounds."""
import json
import os

import numpy as np
import pytest

import oracle

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def bmm():
    if not torch.cuda.is_available():
        pytest.fail("GPU tests need a gfx950 device; none visible")
    from litert_amd import batch_matmul
    return batch_matmul


def _bits_equal(a, b):
    return a.shape == b.shape and np.array_equal(a.view(np.uint32), b.view(np.uint32))


@pytest.mark.parametrize("lhs_shape,rhs_shape,adj_y", [
    ((3, 40), (40, 7), False), ((3, 40), (7, 40), True), ((2, 3, 5, 64), (64, 9), False),
    ((2, 3, 5, 64), (2, 3, 64, 9), False), ((6, 1, 256), (6, 33, 256), True),
    ((1, 4, 48), (5, 48, 6), False), ((4, 48), (2, 2, 48, 6), False),
    ((2, 40, 512), (2, 512, 130), False), ((3, 20, 1040), (1040, 24), False),
    ((1, 4096), (4096, 520), False), ((8, 4096), (300, 4096), True)])
@pytest.mark.parametrize("asym", [True, False])
@pytest.mark.parametrize("per_channel", [True, False])
def test_matches_oracle(bmm, lhs_shape, rhs_shape, adj_y, asym, per_channel):
    rng = np.random.default_rng([len(lhs_shape), lhs_shape[-1], rhs_shape[-1], int(asym)])
    lhs = rng.standard_normal(lhs_shape).astype(np.float32)
    rhs = rng.integers(-127, 128, rhs_shape).astype(np.int8)
    units = rhs_shape[-2] if adj_y else rhs_shape[-1]
    pcs = rng.uniform(2e-3, 8e-3, units).astype(np.float32) if per_channel else None
    op = bmm.BatchMatMulHybrid(rhs, pcs, 0.005, asym, adj_y)
    got = op(torch.from_numpy(lhs).cuda()).cpu().numpy()
    want = oracle.batch_matmul_hybrid(lhs, rhs, pcs, 0.005, asym, adj_y)
    assert _bits_equal(got, want)


@pytest.mark.parametrize("lhs_shape,rhs_shape,adj_x,adj_y", [
    ((40, 3), (40, 7), True, False),                       # adj_x, rank 2
    ((2, 3, 64, 5), (2, 1, 9, 64), True, True),            # adj_x and adj_y, weights broadcast inside
    ((2, 1, 4, 48), (1, 3, 48, 6), False, False),          # 1 on different sides
    ((2, 1, 48, 4), (1, 3, 48, 6), True, False),           # the same under adj_x
    ((3, 1, 2, 5, 16), (1, 4, 1, 16, 6), False, False),    # rank 5, both sides broadcast
    ((1, 2, 3, 16), (4, 1, 16, 6), False, False),          # runs of left matrices per weight matrix
    ((2, 512, 37), (2, 512, 130), True, False),            # tile edges of the transposition
    ((1040, 20), (1040, 24), True, False)])
@pytest.mark.parametrize("asym", [True, False])
def test_adj_x_and_two_sided_broadcasting_match_oracle(bmm, lhs_shape, rhs_shape, adj_x, adj_y, asym):
    rng = np.random.default_rng([len(lhs_shape), lhs_shape[-1], rhs_shape[-1], int(asym)])
    lhs = rng.standard_normal(lhs_shape).astype(np.float32)
    rhs = rng.integers(-127, 128, rhs_shape).astype(np.int8)
    units = rhs_shape[-2] if adj_y else rhs_shape[-1]
    pcs = rng.uniform(2e-3, 8e-3, units).astype(np.float32)
    op = bmm.BatchMatMulHybrid(rhs, pcs, 1.0, asym, adj_y, adj_x=adj_x)
    got = op(torch.from_numpy(lhs).cuda()).cpu().numpy()
    want = oracle.batch_matmul_hybrid(lhs, rhs, pcs, 1.0, asym, adj_y, adj_x=adj_x)
    assert _bits_equal(got, want)


@pytest.mark.parametrize("rows", [3, 40])  # matrix-core GEMV / GEMM
def test_float_zero_point_correction_on_deep_rows(bmm, rows):
    """Dot products beyond 2^24: the reference kernel's `total -= row_sum * batch_offset` in
    float rounds, and so must the GPU."""
    rng = np.random.default_rng(3)
    depth, units = 8192, 48
    lhs = np.abs(rng.standard_normal((rows, depth))).astype(np.float32) + 0.5
    rhs = rng.integers(100, 128, (units, depth)).astype(np.int8)
    pcs = rng.uniform(2e-3, 8e-3, units).astype(np.float32)
    got = bmm.BatchMatMulHybrid(rhs, pcs, 1.0, True, adj_y=True)(torch.from_numpy(lhs).cuda()).cpu().numpy()
    want = oracle.batch_matmul_hybrid(lhs, rhs, pcs, 1.0, True, adj_y=True)
    assert _bits_equal(got, want)
    exact = oracle.fc_hybrid(lhs, rhs, pcs, 1.0, None, True)
    assert not _bits_equal(exact, want)


def test_reference_vectors_through_hip(bmm):
    """batch_matmul_test.cc:504-985 at the tolerance each test states."""
    kats = json.load(open(os.path.join(HERE, "golden", "reference_kats.json")))["batch_matmul_hybrid"]
    for case in kats:
        lhs = np.asarray(case["lhs"], np.float32)
        rhs = np.asarray(case["rhs"], np.int8)
        op = bmm.BatchMatMulHybrid(rhs, None, case["filter_scale"],
                                   case["asymmetric_quantize_inputs"], case["adj_y"],
                                   adj_x=case["adj_x"])
        got = op(torch.from_numpy(lhs).cuda()).cpu().numpy()
        want = np.asarray(case["expected"], np.float32)
        assert np.max(np.abs(got.ravel() - want)) <= case["max_abs_err"], case["source"]
        assert _bits_equal(got, oracle.batch_matmul_hybrid(
            lhs, rhs, None, case["filter_scale"], case["asymmetric_quantize_inputs"], case["adj_y"],
            adj_x=case["adj_x"]))


def test_rejects_shapes_that_do_not_broadcast(bmm):
    rhs = np.zeros((2, 1, 16, 4), np.int8)
    op = bmm.BatchMatMulHybrid(rhs)
    with pytest.raises(ValueError):
        op(torch.zeros((3, 3, 2, 16), device="cuda"))


@pytest.mark.parametrize("lhs_shape,rhs_shape,adj_y,asym,adj_x", [
    ((3, 40), (40, 7), False, True, False), ((2, 3, 5, 64), (2, 3, 9, 64), True, False, False),
    ((4, 48), (5, 48, 6), False, True, False), ((2, 20, 512), (512, 130), False, True, False),
    ((2, 1, 48, 4), (1, 3, 48, 6), False, True, True), ((3, 1, 5, 64), (1, 2, 9, 64), True, True, False)])
def test_node_through_the_delegate(lhs_shape, rhs_shape, adj_y, asym, adj_x):
    """A BATCH_MATMUL node claimed by the plugin, then a FULLY_CONNECTED node fed by it in the
    same partition."""
    if not torch.cuda.is_available():
        pytest.fail("GPU tests need a gfx950 device; none visible")
    from tests.fake_host import FakeHost, FLOAT32, INT8, OK
    rng = np.random.default_rng(11)
    lhs = rng.standard_normal(lhs_shape).astype(np.float32)
    rhs = rng.integers(-127, 128, rhs_shape).astype(np.int8)
    units = rhs_shape[-2] if adj_y else rhs_shape[-1]
    pcs = rng.uniform(2e-3, 8e-3, units).astype(np.float32)
    want = oracle.batch_matmul_hybrid(lhs, rhs, pcs, 1.0, asym, adj_y, adj_x=adj_x)
    w2 = rng.integers(-127, 128, (12, units)).astype(np.int8)
    pcs2 = rng.uniform(2e-3, 8e-3, 12).astype(np.float32)
    with FakeHost() as h:
        x = h.tensor(FLOAT32, lhs_shape, data=lhs)
        w = h.tensor(INT8, rhs_shape, data=rhs, const=True)
        h.affine(w, pcs, quantized_dimension=len(rhs_shape) - (2 if adj_y else 1))
        y = h.tensor(FLOAT32, want.shape)
        node = h.batch_matmul(x, w, y, adj_x=adj_x, adj_y=adj_y, asymmetric=asym)
        f = h.tensor(INT8, w2.shape, data=w2, const=True)
        h.affine(f, pcs2)
        z = h.tensor(FLOAT32, (want.size // units, 12))
        fc_node = h.fc(y, f, None, z)
        h.mark_output(y)
        assert h.load_delegate() == 0, h.errors()
        assert h.modify_graph_with_delegate() == OK, h.errors()
        assert h.plan()[0][:2] == ("delegate", [node, fc_node])
        assert h.allocate_tensors() == OK, h.errors()
        assert h.invoke() == OK, h.errors()
        got = h.read(y)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
        want2 = oracle.fc_hybrid(want.reshape(-1, units), w2, pcs2)
        assert np.array_equal(h.read(z).view(np.uint32), want2.view(np.uint32))

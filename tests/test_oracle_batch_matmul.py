"""Pins the oracle's BATCH_MATMUL hybrid (tflite/kernels/batch_matmul.cc:454-520 over
reference/batch_matmul.h:111-210), CPU only.

(1) The reference's own vectors (batch_matmul_test.cc:504-985, committed as data in
    tests/golden/reference_kats.json) at the tolerance each test states: every broadcasting
    form (weights broadcast, inputs broadcast, adj_y), symmetric and asymmetric inputs.
(2) Where the kernel's float detour (`total -= row_sum * batch_offset`, batch_matmul.h:199-200)
    is exact -- |total| and |row_sum * offset| below 2^24 -- the op must equal the hybrid
    FULLY_CONNECTED of the same rows on the same weights without bias, which is pinned bit for
    bit elsewhere: a transposed operand, a wrong batch pairing or a missing row-sum term fails.
(3) Where it is not exact (deep rows), a numpy replay of the detour in float32, step by step,
    on the oracle's own quantized rows: dropping the detour (exact integer arithmetic) changes
    outputs in that case, and the test checks that it does.
"""
import json
import os

import numpy as np
import pytest

import oracle

HERE = os.path.dirname(os.path.abspath(__file__))
KATS = json.load(open(os.path.join(HERE, "golden", "reference_kats.json")))["batch_matmul_hybrid"]


@pytest.mark.parametrize("case", KATS, ids=[c["source"].split(":")[1] for c in KATS])
def test_reference_vectors(case):
    lhs = np.asarray(case["lhs"], np.float32)
    rhs = np.asarray(case["rhs"], np.int8)
    got = oracle.batch_matmul_hybrid(lhs, rhs, None, case["filter_scale"],
                                     case["asymmetric_quantize_inputs"], case["adj_y"],
                                     adj_x=case["adj_x"])
    want = np.asarray(case["expected"], np.float32)
    assert got.size == want.size
    assert np.max(np.abs(got.ravel() - want)) <= case["max_abs_err"]


@pytest.mark.parametrize("lhs_shape,rhs_shape,adj_y", [
    ((3, 40), (40, 7), False), ((3, 40), (7, 40), True), ((2, 3, 5, 64), (64, 9), False),
    ((2, 3, 5, 64), (2, 3, 64, 9), False), ((2, 3, 5, 64), (2, 1, 9, 64), True),
    ((1, 4, 48), (5, 48, 6), False), ((2, 1, 4, 48), (1, 3, 48, 6), False)])
@pytest.mark.parametrize("asym", [True, False])
@pytest.mark.parametrize("per_channel", [True, False])
def test_equals_hybrid_fully_connected_where_the_float_detour_is_exact(lhs_shape, rhs_shape, adj_y,
                                                                       asym, per_channel):
    rng = np.random.default_rng([len(lhs_shape), lhs_shape[-1], int(adj_y), int(asym)])
    lhs = rng.standard_normal(lhs_shape).astype(np.float32)
    rhs = rng.integers(-127, 128, rhs_shape).astype(np.int8)
    rows, depth, units, out_shape, li, ri = oracle.batch_matmul_broadcast(lhs_shape, rhs_shape, adj_y)
    pcs = rng.uniform(2e-3, 8e-3, units).astype(np.float32) if per_channel else None
    got = oracle.batch_matmul_hybrid(lhs, rhs, pcs, 0.005, asym, adj_y)
    assert got.shape == out_shape
    w = (rhs if adj_y else np.swapaxes(rhs, -1, -2)).reshape(-1, units, depth)
    x = lhs.reshape(-1, rows, depth)
    got = got.reshape(-1, rows, units)
    for b in range(li.size):
        want = oracle.fc_hybrid(x[li[b]], w[ri[b]], pcs, 0.005, None, asym)
        assert np.array_equal(got[b].view(np.uint32), want.view(np.uint32)), b


@pytest.mark.parametrize("lhs_shape,rhs_shape,adj_y", [
    ((40, 3), (40, 7), False), ((2, 3, 64, 5), (2, 1, 9, 64), True),
    ((2, 1, 48, 4), (1, 3, 48, 6), False), ((3, 1, 2, 16, 5), (1, 4, 1, 16, 6), False)])
def test_adj_x_is_the_transposed_left_operand(lhs_shape, rhs_shape, adj_y):
    """adj_x against the same oracle on the left operand transposed beforehand -- and against the
    hybrid FULLY_CONNECTED per output matrix, with the pairing worked out here by numpy
    broadcasting of index arrays (one-sided, two-sided and rank-5 batch shapes)."""
    rng = np.random.default_rng([len(lhs_shape), lhs_shape[-1], int(adj_y)])
    lhs = rng.standard_normal(lhs_shape).astype(np.float32)
    rhs = rng.integers(-127, 128, rhs_shape).astype(np.int8)
    units = rhs_shape[-2] if adj_y else rhs_shape[-1]
    pcs = rng.uniform(2e-3, 8e-3, units).astype(np.float32)
    got = oracle.batch_matmul_hybrid(lhs, rhs, pcs, 1.0, True, adj_y, adj_x=True)
    lhs_t = np.ascontiguousarray(np.swapaxes(lhs, -1, -2))
    same = oracle.batch_matmul_hybrid(lhs_t, rhs, pcs, 1.0, True, adj_y)
    assert np.array_equal(got.view(np.uint32), same.view(np.uint32))
    rows, depth = lhs_t.shape[-2:]
    w = (rhs if adj_y else np.swapaxes(rhs, -1, -2))
    rank = max(lhs.ndim, rhs.ndim) - 2
    lb = (1,) * (rank - (lhs.ndim - 2)) + lhs_t.shape[:-2]
    rb = (1,) * (rank - (rhs.ndim - 2)) + w.shape[:-2]
    ob = np.broadcast_shapes(lb, rb)
    assert got.shape == ob + (rows, units)
    x = np.broadcast_to(lhs_t.reshape(lb + (rows, depth)), ob + (rows, depth))
    wb = np.broadcast_to(w.reshape(rb + (units, depth)), ob + (units, depth))
    for idx in np.ndindex(*ob):
        want = oracle.fc_hybrid(np.ascontiguousarray(x[idx]), np.ascontiguousarray(wb[idx]), pcs,
                                1.0, None, True)
        assert np.array_equal(got[idx].view(np.uint32), want.view(np.uint32)), idx


def test_float_detour_of_the_zero_point_correction_on_deep_rows():
    rng = np.random.default_rng(3)
    depth, units, rows = 8192, 24, 3
    lhs = np.abs(rng.standard_normal((rows, depth))).astype(np.float32) + 0.5  # offset -128
    rhs = rng.integers(100, 128, (units, depth)).astype(np.int8)                 # large sums
    pcs = rng.uniform(2e-3, 8e-3, units).astype(np.float32)
    got = oracle.batch_matmul_hybrid(lhs, rhs, pcs, 1.0, True, adj_y=True)
    q, sf, zp = oracle.batch_quantize_floats(lhs, True)
    total = q.astype(np.int64) @ rhs.astype(np.int64).T                       # exact dots
    row_sum = rhs.astype(np.int64).sum(1)
    assert np.abs(total).max() > 2 ** 24  # the detour rounds here
    f32 = np.float32
    replay = np.empty((rows, units), np.float32)
    for j in range(rows):
        for i in range(units):
            t = f32(total[j, i]) - f32(row_sum[i]) * f32(zp[j])      # float, float, float
            t = int(t)                                               # truncation to int32
            replay[j, i] = f32(0) + f32(sf[j] * pcs[i]) * f32(t)
    assert np.array_equal(got.view(np.uint32), replay.view(np.uint32))
    exact = ((total - row_sum[None, :] * zp[:, None].astype(np.int64)).astype(np.float32) *
             (sf[:, None] * pcs[None, :]).astype(np.float32))
    assert not np.array_equal(exact.view(np.uint32), got.view(np.uint32))

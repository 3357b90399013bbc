"""The oracle's restatement of EvalHybridDense4Bit (per-channel int4 weights, symmetric
activations; tflite/kernels/fully_connected.cc:1088-1178) against what pins it without a
reference build: the op's two known-answer tests (loose by design: abs 1.3), an independent
numpy float32 evaluation of the same chain of operations, a float64 evaluation of the
mathematical value, and the structural properties the reference's unit tests check
(optimized_4bit_test.cc:192-291: scale = max|x| / 127, offsets = -7 * sum(q))."""
import numpy as np
import pytest

import oracle
from tests import kat_harness as kh

f32 = np.float32

# tflite/kernels/fully_connected_4bit_test.cc:102-147
W_ROW_A = [-1, 2, 3, 4, 5, 6, 7, 1, 2, 3] * 4
W_ROW_B = [1, 2, 3, 4, 5, 6, 7, 1, 2, -3] + [-1, 2, 3, 4, 5, 6, 7, 1, 2, 3] * 3
KAT_W = np.array([W_ROW_A[:20] + W_ROW_A[:20],
                  W_ROW_B[:10] + W_ROW_A[:10] + W_ROW_A[:20],
                  W_ROW_B[:10] + W_ROW_A[:10] + W_ROW_A[:20],
                  W_ROW_B[:10] + W_ROW_A[:10] + W_ROW_A[:20],
                  W_ROW_A[:20] + W_ROW_A[:20]], np.int8)
X_A = [1, 2, 3, 4, 5, 6, 7, 8, -9, -10] * 4
X_B = [1, 2, 3, 4, 5, 6, 7, -8, 9, -10] + [1, 2, 3, 4, 5, 6, 7, 8, -9, -10] * 3
KAT_BIAS = np.array([1, 2, 3, 1, 2], np.float32)


def _pack(w):
    return np.stack([kh.pack_int4(r) for r in w])


def test_reference_kat_simple_hybrid_int4():
    """:102-147, weights scale 1.0, RELU; tolerance as in the reference's test."""
    # the weight literal lists 10 rows of 20: five units of 40
    rows = [[-1, 2, 3, 4, 5, 6, 7, 1, 2, 3], [-1, 2, 3, 4, 5, 6, 7, 1, 2, 3],
            [1, 2, 3, 4, 5, 6, 7, 1, 2, -3]]
    a, b = rows[0] + rows[1], rows[2] + rows[1]
    w = np.array([a + a, b + a, b + a, b + a, a + a], np.int8)
    x = np.array([X_A, X_B, X_A, X_A], np.float32)
    y = oracle.fc_hybrid_int4_per_channel(x, _pack(w), 5, [1.0], KAT_BIAS, oracle.ACT_RELU)
    want = np.array([393., 456., 457., 455., 394., 413., 476., 477., 475., 414.,
                     393., 456., 457., 455., 394., 393., 456., 457., 455., 394]).reshape(4, 5)
    assert np.abs(y - want).max() <= 1.3
    # :149-190: an all-zero batch row leaves the bias
    x[3] = 0
    y = oracle.fc_hybrid_int4_per_channel(x, _pack(w), 5, [1.0], KAT_BIAS, oracle.ACT_RELU)
    assert y[3].tolist() == [1, 2, 3, 1, 2]
    assert np.abs(y[:3] - want[:3]).max() <= 1.3


def _numpy_chain(x, w, fs, bias):
    """The same operations, one numpy float32 step at a time (no C++ shared with the oracle)."""
    out = np.empty((x.shape[0], w.shape[0]), f32)
    for m, row in enumerate(x):
        denom = f32(np.abs(row).max()) if np.abs(row).max() != 0 else f32(127.0)
        scale = f32(127.0 / np.float64(denom))
        sf = f32(np.float64(denom) / 127.0)
        q = kh._round_half_away((row * scale).astype(f32)).astype(np.int8)
        offset = np.int32(q.astype(np.int32).sum() * -7)
        val = f32(f32(offset) * sf)
        acc = (w.astype(np.int32) + 7) @ q.astype(np.int32)
        base = (val * fs).astype(f32)
        if bias is not None:
            base = (base + bias).astype(f32)
        term = ((acc.astype(f32) * sf).astype(f32) * fs).astype(f32)
        out[m] = (base + term).astype(f32)
    return out


@pytest.mark.parametrize("B,K,N", [(1, 32, 4), (3, 40, 5), (2, 256, 17), (4, 1024, 64), (1, 4096, 24)])
def test_against_numpy_chain_and_float64(B, K, N):
    rng = np.random.default_rng(B + K + N)
    x = rng.standard_normal((B, K)).astype(f32)
    x[0, :3] = [0.5, -0.5, 1.5]  # exact halves after scaling are likelier here
    w = rng.integers(-7, 8, (N, K)).astype(np.int8)
    fs = rng.uniform(0.01, 0.1, N).astype(f32)
    bias = rng.standard_normal(N).astype(f32) if N % 2 else None
    y = oracle.fc_hybrid_int4_per_channel(x, _pack(w), N, fs, bias)
    assert np.array_equal(y.view(np.uint32), _numpy_chain(x, w, fs, bias).view(np.uint32))
    # the mathematical value: bias + sum_k fs * w * x, up to the 8-bit activation quantization
    exact = (x.astype(np.float64) @ (w.astype(np.float64) * fs[:, None]).T)
    if bias is not None:
        exact += bias
    tol = (np.abs(x).max(1)[:, None] / 127.0) * 0.5 * np.abs(w * fs[:, None]).sum(1)[None, :]
    assert (np.abs(y - exact) <= tol + 1e-4).all()


def test_structure_of_quantized_rows():
    """What RunQuantizeInputTests checks (optimized_4bit_test.cc:192-291), seen through the op:
    with unit filter scale, one channel of weights all equal to c gives
    (c + 7) * sum(q) * sf - 7 * sum(q) * sf = c * sum(q) * sf, q = round(x * 127 / max|x|)."""
    x = np.array([[-127.0 + 2 * i for i in range(64)]], f32)  # max |x| = 127: scale exactly 1
    for c in (-7, -1, 0, 3, 7):
        w = np.full((4, 64), c, np.int8)
        y = oracle.fc_hybrid_int4_per_channel(x, _pack(w), 4, [1.0])
        assert y[0].tolist() == [float(c * x.sum())] * 4
    # all-zero row: scale_denom becomes 127, every q is 0, output is the bias alone
    y = oracle.fc_hybrid_int4_per_channel(np.zeros((1, 64), f32), _pack(np.full((4, 64), 5, np.int8)),
                                          4, [0.3], np.arange(4, dtype=f32))
    assert y[0].tolist() == [0, 1, 2, 3]


def test_activation_and_scalar_scale_broadcast():
    rng = np.random.default_rng(3)
    x = rng.standard_normal((2, 64)).astype(f32)
    w = rng.integers(-7, 8, (8, 64)).astype(np.int8)
    y = oracle.fc_hybrid_int4_per_channel(x, _pack(w), 8, [0.05])
    y_pc = oracle.fc_hybrid_int4_per_channel(x, _pack(w), 8, np.full(8, 0.05, f32))
    assert np.array_equal(y, y_pc)
    assert np.array_equal(oracle.fc_hybrid_int4_per_channel(x, _pack(w), 8, [0.05], None, oracle.ACT_RELU),
                          np.maximum(y, 0))
    assert (y < 0).any()


@pytest.mark.parametrize("B,K,N", [(1, 32, 4), (4, 40, 5), (3, 46, 7), (2, 256, 17), (5, 1000, 33),
                                   (1, 4096, 64), (7, 72, 4)])
def test_bit_identical_to_the_reference_kernels(B, K, N):
    """The reference's own kernels (fully_connected_reference.cc, compiled from where it lies)
    driven in EvalHybridDense4Bit's order: identical bits, ragged shapes included."""
    import ctypes as C
    R = oracle.ref_lib()
    if R is None or not hasattr(R, "ref_fc_hybrid_int4"):
        pytest.skip("oracle/_ref not built (reference tree absent)")
    rng = np.random.default_rng(100 + B + K + N)
    x = rng.standard_normal((B, K)).astype(f32)
    if B > 2:
        x[1] = 0  # all-zero row
    x[0, :4] = [0.5, -0.5, 2.5, -2.5]
    w = rng.integers(-7, 8, (N, K)).astype(np.int8)
    fs = rng.uniform(0.01, 0.1, N).astype(f32)
    for bias in (None, rng.standard_normal(N).astype(f32)):
        want = np.empty((B, N), f32)
        packed = np.ascontiguousarray(_pack(w)).view(np.int8)
        fp = C.POINTER(C.c_float)
        R.ref_fc_hybrid_int4(x.ctypes.data_as(fp), B, K, packed.ctypes.data_as(C.POINTER(C.c_int8)),
                             N, fs.ctypes.data_as(fp),
                             None if bias is None else bias.ctypes.data_as(fp),
                             want.ctypes.data_as(fp))
        got = oracle.fc_hybrid_int4_per_channel(x, _pack(w), N, fs, bias)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))

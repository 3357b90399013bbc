"""The reference holds no vectors for EvalBlockwise4Bit (tflite/kernels/fully_connected.cc:1014-1086),
so the oracle's restatement is pinned through identities a plausible mistake would break:
nibble order, scale indexing, the zero-point correction and the order of the final
scale/bias steps. Bit-level parity with a reference build stays unpinned."""
import numpy as np

import oracle
from tests import kat_harness as kh


def _case(rng, B, K, N, bs, lo=-7, hi=7):
    x = rng.standard_normal((B, K)).astype(np.float32)
    w = rng.integers(lo, hi + 1, (N, K)).astype(np.int8)
    scales = rng.uniform(5e-3, 2e-2, (N, K // bs)).astype(np.float16)
    return x, w, scales


def _pack_rows(w):
    return np.stack([kh.pack_int4(r) for r in w])


def test_blockwise_float64_brute_force():
    rng = np.random.default_rng(31)
    for B, K, N, bs in ((1, 32, 4, 32), (2, 64, 5, 32), (3, 128, 7, 64), (1, 256, 9, 32)):
        x, w, scales = _case(rng, B, K, N, bs, -8, 7)
        bias = rng.standard_normal(N).astype(np.float32)
        y = oracle.fc_blockwise_int4(x, _pack_rows(w), N, scales.view(np.uint16), bs, bias)
        q, sf, zp = oracle.batch_quantize_floats(x, True)
        s64 = np.repeat(scales.astype(np.float64), bs, axis=1)           # [N,K]
        want = np.empty((B, N))
        for b in range(B):
            want[b] = sf[b].astype(np.float64) * ((w * s64) @ (q[b].astype(np.float64) - zp[b])) + bias
        tol = 1e-5 * np.abs(want).max() + 1e-5 * np.abs(want)
        assert np.all(np.abs(y - want) <= tol)


def test_blockwise_reduces_to_per_channel_hybrid():
    """With one scale per row and power-of-two values every float step is exact, so the
    blockwise result must equal the per-channel hybrid formula bit for bit."""
    rng = np.random.default_rng(32)
    B, K, N, bs = 2, 128, 6, 32
    x, w, _ = _case(rng, B, K, N, bs)
    row_scale = np.array([2.0 ** -e for e in range(3, 3 + N)], np.float16)
    scales = np.repeat(row_scale[:, None], K // bs, axis=1)
    y = oracle.fc_blockwise_int4(x, _pack_rows(w), N, scales.view(np.uint16), bs, None)
    q, sf, zp = oracle.batch_quantize_floats(x, True)
    acc = w.astype(np.int64) @ q.astype(np.int64).T - w.astype(np.int64).sum(1)[:, None] * zp[None, :]
    # every partial sum is an integer times a power of two below 2^24: exact in float32
    want = (acc.T.astype(np.float32) * row_scale.astype(np.float32)[None, :]) * sf[:, None]
    assert np.array_equal(y.view(np.uint32), want.astype(np.float32).view(np.uint32))


def test_blockwise_nibble_order_and_scale_index():
    """A single non-zero weight at (n, k) must pick activation k and scale [n, k // bs]."""
    rng = np.random.default_rng(33)
    B, K, N, bs = 1, 96, 5, 32
    x = rng.standard_normal((B, K)).astype(np.float32)
    scales = rng.uniform(5e-3, 2e-2, (N, K // bs)).astype(np.float16)
    q, sf, zp = oracle.batch_quantize_floats(x, True)
    for n, k, v in ((0, 0, 3), (1, 1, -8), (2, 33, 7), (4, 95, -1), (3, 64, 5)):
        w = np.zeros((N, K), np.int8)
        w[n, k] = v
        y = oracle.fc_blockwise_int4(x, _pack_rows(w), N, scales.view(np.uint16), bs, None)
        s = np.float32(scales[n, k // bs])
        out = np.float32(np.float32(int(q[0, k]) * v) * s)
        out = np.float32(out - np.float32(np.float32(zp[0]) * np.float32(s * np.float32(v))))
        out = np.float32(out * sf[0])
        want = np.zeros(N, np.float32)
        want[n] = out
        assert np.array_equal(y[0], want)


def test_blockwise_bias_added_after_input_scale():
    rng = np.random.default_rng(34)
    x, w, scales = _case(rng, 2, 64, 4, 32)
    bias = np.array([100.0, -3.5, 0.25, 7.0], np.float32)
    y0 = oracle.fc_blockwise_int4(x, _pack_rows(w), 4, scales.view(np.uint16), 32, None)
    y1 = oracle.fc_blockwise_int4(x, _pack_rows(w), 4, scales.view(np.uint16), 32, bias)
    assert np.array_equal(y1, (y0 + bias[None, :]).astype(np.float32))

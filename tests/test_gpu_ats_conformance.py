"""The full-integer FULLY_CONNECTED cases of the reference's accelerator test suite, restated:
`litert/ats/register_fully_connected.cc:103-124` registers rank {2, 3} x keep_num_dims x
{NONE, RELU} x bias x per-channel for int8 and for uint8 (the shuffled-weights column and
per-channel uint8 filters, which the builtin's Prepare refuses too (fully_connected.cc:528-531),
are nodes this delegate declines, see test_delegate_cpu.py), and
`litert/test/generators/fully_connected.h`
builds each case: every dimension drawn from [2, 6] (:107-117), weights all 1 and bias all 0
(:122-123), every scale 0.01 with zero point 0 (:344-395), inputs uniform over int8. The suite's
own reference is a float FULLY_CONNECTED on the raw integers, times 0.01, cast to int8
(:181-260, `litert/core/model/ops/matmul.h:220-236`), and its comparator lets integers differ by
one bucket (`inference_fixture.h:315-327`, `bucket_tolerance = 1`).

Each case goes through the delegate as the interpreter would drive it; the output is held to the
suite's comparator against the suite's reference AND bit-exact against the oracle of the builtin.
"""
import itertools

import numpy as np
import pytest

import oracle
from tests.fake_host import FakeHost, INT32, INT8, UINT8, OK

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")

SCALE = 0.01
BIAS_SCALE = 0.0001
NONE, RELU = 0, 1


@pytest.fixture(autouse=True)
def _need_gpu():
    if not torch.cuda.is_available():
        pytest.fail("GPU tests need a gfx950 device; none visible")


def _suite_reference(x, w, bias, activation, dtype=np.int8):
    """ReferenceFullyConnected on the integers as floats, scaled by 0.01, cast to the output type."""
    B = int(np.prod(x.shape[:-1]))
    xf = x.reshape(B, -1).astype(np.float32)
    wf = w.astype(np.float32)
    out = np.empty((B, w.shape[0]), np.float32)
    for b in range(B):
        for o in range(w.shape[0]):
            s = np.float32(bias[o]) if bias is not None else np.float32(0)
            for i in range(w.shape[1]):
                s = np.float32(s + np.float32(xf[b, i] * wf[o, i]))
            out[b, o] = s
    if activation == RELU:
        out = np.maximum(out, np.float32(0))
    return np.trunc(out * np.float32(SCALE)).astype(dtype)


CASES = list(itertools.product((2, 3), (False, True), (NONE, RELU), (False, True), (False, True)))


@pytest.mark.parametrize("rank,keep_num_dims,activation,has_bias,per_channel", CASES)
def test_int8_cases_of_the_accelerator_suite(rank, keep_num_dims, activation, has_bias, per_channel):
    seed = sum(int(v) << i for i, v in enumerate((rank, keep_num_dims, activation, has_bias, per_channel)))
    rng = np.random.default_rng(seed)
    for _ in range(3):
        dims = rng.integers(2, 7, size=rank + 1)
        in_shape = tuple(int(d) for d in dims[:rank])
        K, N = in_shape[-1], int(dims[rank])
        B = int(np.prod(in_shape[:-1]))
        x = rng.integers(-128, 128, in_shape, dtype=np.int8)
        w = np.ones((N, K), np.int8)
        bias = np.zeros(N, np.int32) if has_bias else None
        out_shape = in_shape[:-1] + (N,) if keep_num_dims else (B, N)
        with FakeHost() as h:
            xt = h.tensor(INT8, in_shape, data=x)
            h.affine(xt, [SCALE], [0])
            wt = h.tensor(INT8, (N, K), data=w, const=True)
            h.affine(wt, [SCALE] * (N if per_channel else 1))
            bt = None
            if has_bias:
                bt = h.tensor(INT32, (N,), data=bias, const=True)
                h.affine(bt, [BIAS_SCALE] * (N if per_channel else 1))
            yt = h.tensor(INT8, out_shape)
            h.affine(yt, [SCALE], [0])
            node = h.fc(xt, wt, bt, yt, activation=activation, keep_num_dims=keep_num_dims)
            assert h.classify(node)[0] == "int8"
            assert h.load_delegate() == 0, h.errors()
            assert h.modify_graph_with_delegate() == OK and h.allocate_tensors() == OK, h.errors()
            assert h.plan()[0][:2] == ("delegate", [node])
            assert h.invoke() == OK, h.errors()
            got = h.read(yt)
        assert got.shape == out_shape
        got = got.reshape(B, N)
        # the suite's comparator against the suite's reference
        ref = _suite_reference(x, w, bias, activation)
        assert np.abs(got.astype(np.int64) - ref.astype(np.int64)).max() <= 1, (in_shape, N)
        # and the builtin's arithmetic, bit for bit
        if per_channel:
            mult, shift = oracle.fc_prepare_per_channel(SCALE, np.full(N, SCALE, np.float32), SCALE)
            lo, hi = oracle.activation_range_int8(activation, SCALE, 0)
            want = oracle.fc_int8_per_channel(x.reshape(B, K), w, bias, mult, shift, 0, 0, lo, hi)
        else:
            mult, shift = oracle.fc_prepare_per_tensor(SCALE, SCALE, SCALE,
                                                       BIAS_SCALE if has_bias else None)
            lo, hi = oracle.activation_range_int8(activation, SCALE, 0)
            want = oracle.fc_int8_per_tensor(x.reshape(B, K), w, bias, mult, shift, 0, 0, 0, lo, hi)
        assert np.array_equal(got, want), (in_shape, N)


UINT8_CASES = list(itertools.product((2, 3), (False, True), (NONE, RELU), (False, True)))


@pytest.mark.parametrize("rank,keep_num_dims,activation,has_bias", UINT8_CASES)
def test_uint8_cases_of_the_accelerator_suite(rank, keep_num_dims, activation, has_bias):
    """The suite's uint8 column with a per-tensor filter: inputs uniform over uint8, zero points 0."""
    seed = 100 + sum(int(v) << i for i, v in enumerate((rank, keep_num_dims, activation, has_bias)))
    rng = np.random.default_rng(seed)
    for _ in range(3):
        dims = rng.integers(2, 7, size=rank + 1)
        in_shape = tuple(int(d) for d in dims[:rank])
        K, N = in_shape[-1], int(dims[rank])
        B = int(np.prod(in_shape[:-1]))
        x = rng.integers(0, 256, in_shape).astype(np.uint8)
        w = np.ones((N, K), np.uint8)
        bias = np.zeros(N, np.int32) if has_bias else None
        out_shape = in_shape[:-1] + (N,) if keep_num_dims else (B, N)
        with FakeHost() as h:
            xt = h.tensor(UINT8, in_shape, data=x)
            h.affine(xt, [SCALE], [0])
            wt = h.tensor(UINT8, (N, K), data=w, const=True)
            h.affine(wt, [SCALE])
            bt = None
            if has_bias:
                bt = h.tensor(INT32, (N,), data=bias, const=True)
                h.affine(bt, [BIAS_SCALE])
            yt = h.tensor(UINT8, out_shape)
            h.affine(yt, [SCALE], [0])
            node = h.fc(xt, wt, bt, yt, activation=activation, keep_num_dims=keep_num_dims)
            assert h.classify(node)[0] == "int8"
            assert h.load_delegate() == 0, h.errors()
            assert h.modify_graph_with_delegate() == OK and h.allocate_tensors() == OK, h.errors()
            assert h.plan()[0][:2] == ("delegate", [node])
            assert h.invoke() == OK, h.errors()
            got = h.read(yt)
        assert got.shape == out_shape and got.dtype == np.uint8
        got = got.reshape(B, N)
        ref = _suite_reference(x, w, bias, activation, np.uint8)
        assert np.abs(got.astype(np.int64) - ref.astype(np.int64)).max() <= 1, (in_shape, N)
        mult, shift = oracle.fc_prepare_per_tensor(SCALE, SCALE, SCALE,
                                                   BIAS_SCALE if has_bias else None)
        lo, hi = oracle.activation_range_uint8(activation, SCALE, 0)
        want = oracle.fc_uint8_per_tensor(x.reshape(B, K), w, bias, mult, shift, 0, 0, 0, lo, hi)
        assert np.array_equal(got, want), (in_shape, N)

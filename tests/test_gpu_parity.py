"""Parity of the HIP path (through the C ABI) against the CPU oracle on the same seeded
inputs. Bars: bit-exact for full-integer int8 outputs and for quantized activations
(values, scales and zero points); float outputs of the hybrid and blockwise paths are
held to rtol 1e-5 with atol 1e-5 * max|ref| (the reference's comparator form,
litert/ats/inference_fixture.h:262-286) and are in fact expected bit-identical, which
is asserted where the kernel replays the reference's operation order.
"""
import numpy as np
import pytest

import oracle
from litert_amd import workloads as wl
from tests import kat_harness as kh

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


@pytest.fixture(scope="module")
def fc():
    if not torch.cuda.is_available():
        pytest.fail("GPU tests need a gfx950 device; none visible")
    from litert_amd import fully_connected
    fully_connected._ensure_init()
    return fully_connected


def _cuda(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _close(got, want, rtol=1e-5):
    atol = rtol * float(np.abs(want).max())
    return np.all(np.abs(got - want) <= atol + rtol * np.abs(want))


def _bits_equal(a, b):
    return np.array_equal(a.view(np.uint32), b.view(np.uint32))


# ---- full-integer int8 -------------------------------------------------------------

def _run_int8(fc, c, activation="none", bias=True, packed=True):
    op = fc.FullyConnectedInt8(c["w"], c["bias"] if bias else None, float(c["in_scale"]),
                               c["in_zp"], c["w_scale"], float(c["out_scale"]), c["out_zp"],
                               activation=activation, packed=packed)
    y = op(_cuda(c["x"])).cpu().numpy()
    mult, shift = oracle.fc_prepare_per_channel(float(c["in_scale"]), c["w_scale"],
                                                float(c["out_scale"]))
    lo, hi = oracle.activation_range_int8(fc._act(activation), float(c["out_scale"]), c["out_zp"])
    want = oracle.fc_int8_per_channel(c["x"], c["w"], c["bias"] if bias else None, mult, shift,
                                      -c["in_zp"], c["out_zp"], lo, hi)
    return y, want


@pytest.mark.parametrize("packed", [True, False])
def test_int8_config1_bit_exact(fc, packed):
    """Config 1: [1,2048] x [2048,2048], per-channel, bias, no activation; on the re-tiled
    filter (matrix-core GEMV) and on the row-major one (dot4 GEMV)."""
    y, want = _run_int8(fc, wl.int8_fc(), packed=packed)
    assert np.array_equal(y, want)
    assert len(np.unique(y)) > 100  # the case exercises the whole int8 range, not a clamp


@pytest.mark.parametrize("B,K,N", [(1, 16, 1), (2, 48, 5), (3, 1040, 17), (4, 2048, 256),
                                   (5, 512, 67), (8, 4096, 512), (9, 256, 33), (16, 128, 40),
                                   (1, 16384, 64), (2, 10, 3), (3, 33, 7), (1, 100, 9),
                                   (17, 320, 19), (40, 64, 16), (1, 20000, 5)])
@pytest.mark.parametrize("activation", ["none", "relu6"])
@pytest.mark.parametrize("packed", [True, False])
def test_int8_gemv_shapes_bit_exact(fc, B, K, N, activation, packed):
    """Ragged shapes: depth off the 16-byte grid takes the generic kernel, batches that are
    not a power of two split into tiles, rows that do not fill a pass are clamped."""
    c = wl.int8_fc(B, K, N, seed=100 + B + K + N)
    y, want = _run_int8(fc, c, activation, bias=(N % 2 == 1), packed=packed)
    assert np.array_equal(y, want)


def test_int8_per_tensor_with_filter_zero_point(fc):
    rng = np.random.default_rng(5)
    for B, K, N in ((2, 10, 3), (3, 64, 9), (8, 256, 40)):
        x = rng.integers(-128, 128, (B, K)).astype(np.int8)
        w = rng.integers(-128, 128, (N, K)).astype(np.int8)
        bias = rng.integers(-1000, 1000, N).astype(np.int32)
        op = fc.FullyConnectedInt8(w, bias, 0.5, -1, [0.5], 1.0, -1, activation="relu",
                                   filter_zero_point=-1, bias_scale=0.25)
        y = op(_cuda(x)).cpu().numpy()
        m, s = oracle.fc_prepare_per_tensor(0.5, 0.5, 1.0, 0.25)
        lo, hi = oracle.activation_range_int8(oracle.ACT_RELU, 1.0, -1)
        want = oracle.fc_int8_per_tensor(x, w, bias, m, s, 1, 1, -1, lo, hi)
        assert np.array_equal(y, want)


def test_int8_reference_kats_through_hip(fc):
    """tflite/kernels/fully_connected_test.cc:816-840, :863-888, :1463-1487, :1530-1562."""
    W10 = [1, 2, 3, 4, 5, 6, 7, 8, 9, 10]
    X2 = [1, 2, 3, 4, 5, 6, 7, 8, -9, -10, 1, 2, 3, 4, 5, 6, 7, -8, 9, -10]

    def per_tensor(in_range, out_range, units, x, bias):
        in_s, in_zp = kh.quantization_params(*in_range)
        out_s, out_zp = kh.quantization_params(*out_range)
        w_s, w_zp = kh.quantization_params(-63.5, 64)
        wq = kh.quantize(W10 * units, w_s, w_zp).reshape(units, 10)
        xq = kh.quantize(x, in_s, in_zp).reshape(-1, 10)
        bs = np.float32(in_s * w_s)
        op = fc.FullyConnectedInt8(wq, kh.quantize_bias(bias, bs), float(in_s), in_zp, [float(w_s)],
                                   float(out_s), out_zp, filter_zero_point=w_zp,
                                   bias_scale=float(bs))
        return op(_cuda(xq)).cpu().numpy().ravel().tolist()

    assert per_tensor((-63.5, 64), (-127, 128), 3, X2, [1, 2, 3]) == [23, 24, 25, 57, 58, 59]
    assert per_tensor((-63.5, 64), (-127, 128), 4, X2[10:], [1, 2, 3, 4]) == [57, 58, 59, 60]
    assert per_tensor((-127, 128), (-63.5, 64), 3, X2, [1, 2, 3]) == [47, 49, 51, 115, 117, 119]

    in_s, in_zp = kh.quantization_params(-63.5, 64)
    out_s, out_zp = kh.quantization_params(-127, 128)
    scales = np.array([0.2, 0.25, 0.5], np.float32)
    w = np.array(W10 * 3, np.float32).reshape(3, 10)
    wq = np.clip(kh._round_half_away(w * (np.float32(1) / scales)[:, None]), -127, 127).astype(np.int8)
    bq = kh._round_half_away(np.array([1, 2, 3], np.float32) / (scales * in_s)).astype(np.int32)
    op = fc.FullyConnectedInt8(wq, bq, float(in_s), in_zp, scales, float(out_s), out_zp)
    y = op(_cuda(kh.quantize(X2, in_s, in_zp).reshape(2, 10))).cpu().numpy().ravel().tolist()
    assert y == [23, 24, 25, 57, 58, 59]


def test_int8_int4_weights_kat(fc):
    """fully_connected_test.cc:950-976: packed int4 per-channel weights, unpacked on the GPU."""
    in_s, in_zp = kh.quantization_params(-63.5, 64)
    out_s, out_zp = kh.quantization_params(-127, 128)
    w4 = np.array([1, 2, 3, 4, 5, 6, 7, 6, 5, 4] * 3, np.int8).reshape(3, 10)
    X2 = [1, 2, 3, 4, 5, 6, 7, 8, -9, -10, 1, 2, 3, 4, 5, 6, 7, -8, 9, -10]
    bq = kh._round_half_away(np.array([1, 2, 3], np.float32) / np.float32(in_s)).astype(np.int32)
    op = fc.FullyConnectedInt8(wl.pack_int4(w4), bq, float(in_s), in_zp, [1.0, 1.0, 1.0],
                               float(out_s), out_zp, activation="relu", int4=True, depth=10)
    y = op(_cuda(kh.quantize(X2, in_s, in_zp).reshape(2, 10))).cpu().numpy().ravel().tolist()
    assert y == [103, 104, 105, 97, 98, 99]


@pytest.mark.parametrize("activation", ["none", "relu6"])
def test_int8_prefill_gemm_bit_exact(fc, activation):
    """Config 4 shape class on the MFMA path, at a size the scalar oracle finishes in seconds."""
    c = wl.prefill_int8_fc(256, 512, 512, seed=77)
    for packed in (True, False):  # GEMM on the re-tiled filter / on the row-major one
        y, want = _run_int8(fc, c, activation, packed=packed)
        assert np.array_equal(y, want)
    c = wl.int8_fc(128, 256, 256, in_zp=-3, out_zp=5, seed=78)  # non-zero input offset on the GEMM
    for packed in (True, False):
        y, want = _run_int8(fc, c, activation, packed=packed)
        assert np.array_equal(y, want)


@pytest.mark.parametrize("B,K,N", [(33, 64, 20), (128, 256, 256), (130, 272, 48), (200, 1040, 300),
                                   (64, 16, 4), (257, 192, 513), (40, 4096, 70), (300, 80, 257),
                                   (129, 128, 30), (96, 2048, 64), (1030, 48, 4100),
                                   (2050, 80, 2049), (1152, 96, 4096), (1100, 208, 4112)])
@pytest.mark.parametrize("activation", ["none", "relu6"])
def test_int8_packed_gemm_ragged_shapes_bit_exact(fc, B, K, N, activation):
    """More than 16 rows on the re-tiled filter take the MFMA GEMM: batch and channel counts
    off the tile (64 x 128 for the small launches, 128 x 256 from (1030, 48, 4100) on), depths
    that end inside a 64-deep slab or give an odd slab count, channel counts that rule out vector
    stores; the last two have interior tiles whose int8 outputs leave through LDS in whole
    cache lines (all of them, and beside ragged last rows and columns)."""
    c = wl.int8_fc(B, K, N, in_zp=(-3 if N % 2 else 0), seed=300 + B + K + N)
    y, want = _run_int8(fc, c, activation, bias=(N % 3 != 0))
    assert np.array_equal(y, want)


@pytest.mark.parametrize("B,K,N", [(130, 272, 300), (1030, 48, 4100)])
@pytest.mark.parametrize("case", ["zero_shift", "left_shift", "big_bias", "shift_31", "mixed"])
def test_int8_packed_gemm_requantization_forms_bit_exact(fc, B, K, N, case):
    """The GEMM epilogue has a short form of MultiplyByQuantizedMultiplier for tiles whose
    channels all shift right by 1..31 bits with a small addend, and the general form for the
    rest. Raw multipliers and shifts put single channels, or all of them, outside the short
    form: a shift of zero, left shifts, a bias beyond 2^29, the multiplier INT32_MIN; the
    tiles next to such a channel stay on the short form."""
    c = wl.int8_fc(B, K, N, in_zp=-3, seed=900 + B + len(case))
    rng = np.random.default_rng(len(case) + N)
    mult = rng.integers(1 << 30, (1 << 31) - 1, N, dtype=np.int64).astype(np.int32)
    shift = rng.integers(-13, -9, N).astype(np.int32)
    bias = c["bias"].copy()
    if case == "zero_shift":
        shift[N // 2] = 0
        mult[N // 2] = 1 << 20
    elif case == "left_shift":
        shift[:] = rng.integers(1, 4, N)
        mult[:] = rng.integers(1 << 18, 1 << 21, N)
    elif case == "big_bias":
        bias[5] = (1 << 30) + 12345
        bias[N - 1] = -(1 << 30) - 777
        shift[5] = shift[N - 1] = -24
    elif case == "shift_31":
        shift[:] = rng.integers(-31, -27, N)
        bias[:] = rng.integers(-(1 << 29) + 1, 1 << 29, N)
    else:
        shift[::97] = 0
        mult[::97] = 1 << 20
        shift[3::131] = 2
        mult[3::131] = 1 << 18
        mult[7] = np.iinfo(np.int32).min
    op = fc.FullyConnectedInt8(c["w"], bias, float(c["in_scale"]), c["in_zp"], c["w_scale"],
                               float(c["out_scale"]), c["out_zp"])
    op.multipliers, op.shifts = _cuda(mult), _cuda(shift)
    y = op(_cuda(c["x"])).cpu().numpy()
    want = oracle.fc_int8_per_channel(c["x"], c["w"], bias, mult, shift, -c["in_zp"], c["out_zp"],
                                      -128, 127)
    assert np.array_equal(y, want)
    assert len(np.unique(y)) > 3


@pytest.mark.parametrize("B,K,N", [(33, 64, 20), (128, 256, 256), (130, 272, 48), (65, 1040, 301),
                                   (1025, 96, 4096)])
@pytest.mark.parametrize("asym", [True, False])
@pytest.mark.parametrize("per_channel", [True, False])
def test_hybrid_packed_gemm_matches_oracle(fc, B, K, N, asym, per_channel):
    """Hybrid rows beyond 16 run the same GEMM with the float epilogue (the last shape in its
    128 x 256 tile form)."""
    c = wl.hybrid_fc(B, K, N, seed=17 + B + K)
    bias = np.random.default_rng(3).standard_normal(N).astype(np.float32)
    pcs = c["pcs"] if per_channel else None
    op = fc.FullyConnectedHybrid(c["w"], pcs, filter_scale=0.005, bias=bias,
                                 asymmetric_quantize_inputs=asym, activation="relu6")
    y = op(_cuda(c["x"])).cpu().numpy()
    want = oracle.fc_hybrid(c["x"], c["w"], pcs, 0.005, bias, asym, oracle.ACT_RELU6)
    assert _bits_equal(y, want)


@pytest.mark.parametrize("B,K,N", [(17, 64, 20), (24, 4096, 1024), (32, 4096, 520), (31, 1040, 301),
                                   (32, 512, 14336), (20, 2064, 48), (29, 16, 4), (32, 272, 100),
                                   (17, 8192, 64), (30, 4100, 40)])
@pytest.mark.parametrize("asym", [True, False])
def test_hybrid_17_to_32_rows_in_one_pass_matches_oracle(fc, B, K, N, asym):
    """17 to 32 rows whose LDS image fits a compute unit take the register-resident GEMV with two
    row tiles per weight tile (depth shares of 8 and 16 tiles, depths that end inside a slab, one
    or several channel tiles per workgroup, ragged channel counts); the last two shapes -- too
    deep, and a depth that is no multiple of 16 -- go to the GEMM instead. Same bits either way."""
    c = wl.hybrid_fc(B, K, N, seed=29 + B + K)
    bias = np.random.default_rng(5).standard_normal(N).astype(np.float32)
    bias[::5] = -0.0
    pcs = c["pcs"] if (B + N) % 2 else None
    for activation, code in (("relu6", oracle.ACT_RELU6), ("none", oracle.ACT_NONE)):
        op = fc.FullyConnectedHybrid(c["w"], pcs, filter_scale=0.005, bias=bias,
                                     asymmetric_quantize_inputs=asym, activation=activation)
        y = op(_cuda(c["x"])).cpu().numpy()
        want = oracle.fc_hybrid(c["x"], c["w"], pcs, 0.005, bias, asym, code)
        assert _bits_equal(y, want)
    zeros = np.zeros_like(c["x"])  # the whole-zero input exit keeps the bias bits
    y = op(_cuda(zeros)).cpu().numpy()
    assert _bits_equal(y, oracle.fc_hybrid(zeros, c["w"], pcs, 0.005, bias, asym, oracle.ACT_NONE))


@pytest.mark.parametrize("B,K,N", [(17, 64, 20), (32, 4096, 520), (31, 1040, 301), (24, 2048, 2048)])
@pytest.mark.parametrize("activation", ["none", "relu6"])
def test_int8_17_to_32_rows_in_one_pass_bit_exact(fc, B, K, N, activation):
    c = wl.int8_fc(B, K, N, in_zp=(-3 if N % 2 else 0), seed=310 + B + K + N)
    y, want = _run_int8(fc, c, activation, bias=(N % 3 != 0))
    assert np.array_equal(y, want)


ROWS_33_TO_128 = [(33, 1024, 10225), (40, 4096, 14336), (64, 1040, 10256), (100, 2064, 10240),
                  (128, 1536, 12000), (65, 1024, 10240), (130, 1024, 10240),
                  # 641 and 642 channel tiles: the last workgroup owns one / two real tiles of four
                  (50, 1024, 10250), (100, 1024, 10270)]


@pytest.mark.parametrize("B,K,N", ROWS_33_TO_128)
@pytest.mark.parametrize("asym", [True, False])
def test_hybrid_33_to_128_rows_on_wide_filters_matches_oracle(fc, B, K, N, asym):
    """33 to 128 rows against a filter of 640 or more channel tiles take the kernel that streams
    the filter once and walks the rows through LDS in depth chunks: four and eight row tiles per
    weight tile, odd and even chunk counts, depths that end 16 into a chunk, a ragged last channel
    tile, a ragged last row tile, workgroups whose last tiles lie past the filter; 130 rows stay on
    the GEMM. Same bits either way."""
    c = wl.hybrid_fc(B, K, N, seed=41 + B + K)
    bias = np.random.default_rng(6).standard_normal(N).astype(np.float32)
    bias[::5] = -0.0
    pcs = c["pcs"] if (B + N) % 2 else None
    for activation, code in (("relu6", oracle.ACT_RELU6), ("none", oracle.ACT_NONE)):
        op = fc.FullyConnectedHybrid(c["w"], pcs, filter_scale=0.005, bias=bias,
                                     asymmetric_quantize_inputs=asym, activation=activation)
        y = op(_cuda(c["x"])).cpu().numpy()
        want = oracle.fc_hybrid(c["x"], c["w"], pcs, 0.005, bias, asym, code)
        assert _bits_equal(y, want)
    zeros = np.zeros_like(c["x"])
    zeros[B // 2] = c["x"][B // 2]  # one live row among whole-zero ones
    y = op(_cuda(zeros)).cpu().numpy()
    assert _bits_equal(y, oracle.fc_hybrid(zeros, c["w"], pcs, 0.005, bias, asym, oracle.ACT_NONE))


@pytest.mark.parametrize("B,K,N", [(33, 1024, 10225), (64, 1040, 10256), (100, 2064, 10240),
                                   (128, 1536, 12000), (70, 1024, 10250)])
@pytest.mark.parametrize("activation", ["none", "relu6"])
def test_int8_33_to_128_rows_on_wide_filters_bit_exact(fc, B, K, N, activation):
    c = wl.int8_fc(B, K, N, in_zp=(-3 if N % 2 else 0), seed=510 + B + K + N)
    y, want = _run_int8(fc, c, activation, bias=(N % 3 != 0))
    assert np.array_equal(y, want)


def test_int8_prefill_full_size_properties(fc):
    """Config 4 at full size (2048 x 4096 x 4096), RELU6 on and off, checked through
    size-independent properties: a random sample of outputs against an int64 numpy
    evaluation of the definition, agreement with the GEMV kernel on a slice of rows, and
    clamp(no-activation output) == RELU6 output."""
    c = wl.prefill_int8_fc()
    x = _cuda(c["x"])
    outs = {}
    for activation in ("none", "relu6"):
        op = fc.FullyConnectedInt8(c["w"], c["bias"], float(c["in_scale"]), c["in_zp"],
                                   c["w_scale"], float(c["out_scale"]), c["out_zp"],
                                   activation=activation)
        outs[activation] = op(x).cpu().numpy()
        if activation == "none":
            y_gemv = op(x[:8]).cpu().numpy()  # 8 rows take the GEMV kernel
            assert np.array_equal(outs["none"][:8], y_gemv)
            rowmajor = fc.FullyConnectedInt8(c["w"], c["bias"], float(c["in_scale"]), c["in_zp"],
                                             c["w_scale"], float(c["out_scale"]), c["out_zp"],
                                             packed=False)
            assert np.array_equal(outs["none"], rowmajor(x).cpu().numpy())  # the other GEMM
    lo, hi = oracle.activation_range_int8(oracle.ACT_RELU6, 0.05, 0)
    assert np.array_equal(np.clip(outs["none"], lo, hi), outs["relu6"])
    mult, shift = oracle.fc_prepare_per_channel(0.03, c["w_scale"], 0.05)
    rng = np.random.default_rng(9)
    ms, ns = rng.integers(0, 2048, 4000), rng.integers(0, 4096, 4000)
    acc = np.einsum("ik,ik->i", c["x"][ms].astype(np.int64), c["w"][ns].astype(np.int64)) + c["bias"][ns]
    want = np.array([oracle.mbqm(int(a), int(mult[n]), int(shift[n])) for a, n in zip(acc, ns)])
    assert np.array_equal(outs["none"][ms, ns], np.clip(want, -128, 127).astype(np.int8))


# ---- activation quantization ---------------------------------------------------------

@pytest.mark.parametrize("variant", [0, 1, 2])
@pytest.mark.parametrize("asym", [True, False])
def test_batch_quantize_floats_bit_exact(fc, variant, asym):
    rng = np.random.default_rng(41)
    for B, K in ((1, 4096), (4, 2048), (8, 4096), (3, 1001), (2, 7), (5, 16384), (1, 9)):
        x = rng.standard_normal((B, K)).astype(np.float32)
        if B > 1:
            x[1] = 0.0                      # all-zero row: scale 1, zero point 0
        if B > 2:
            x[2] = np.abs(x[2]) * 1e-4      # rmin clamps to zero
        q, sf, zp = fc.batch_quantize_floats(_cuda(x), asym, variant)
        wq, wsf, wzp = oracle.batch_quantize_floats(x, asym, variant)
        assert np.array_equal(q.cpu().numpy(), wq)
        assert _bits_equal(sf.cpu().numpy(), wsf)
        assert np.array_equal(zp.cpu().numpy(), wzp)


@pytest.mark.parametrize("variant", [0, 1, 2])
@pytest.mark.parametrize("asym", [True, False])
def test_batch_quantize_at_and_beside_every_tie(fc, variant, asym):
    """Rows whose scale is exactly 1 (range [-128, 127], or |max| 127 for the symmetric form), so
    every element reaches the rounding step unchanged: each k + 0.5, the floats just below and
    above it, and the float just below 0.5, where adding one half and truncating goes wrong."""
    ks = np.arange(-127, 127, dtype=np.float32) + np.float32(0.5)
    near = np.concatenate([ks, np.nextafter(ks, np.float32(-1e9)), np.nextafter(ks, np.float32(1e9)),
                           np.array([0.0, -0.0, 0.49999997, -0.49999997, 0.25, -0.25, 1e-30, -1e-30],
                                    np.float32)]).astype(np.float32)
    ends = np.array([-128.0 if asym else -127.0, 127.0], np.float32)
    for pad in (0, 3, 5):   # rows of 772, 775, 777: with and without the NEON builds' scalar tail
        row = np.concatenate([ends, near, np.zeros(pad, np.float32)])
        x = np.stack([row, row[::-1]]).astype(np.float32)
        q, sf, zp = fc.batch_quantize_floats(_cuda(x), asym, variant)
        wq, wsf, wzp = oracle.batch_quantize_floats(x, asym, variant)
        assert wsf.tolist() == [1.0, 1.0] and wzp.tolist() == [0, 0]
        assert np.array_equal(q.cpu().numpy(), wq)
        assert _bits_equal(sf.cpu().numpy(), wsf) and np.array_equal(zp.cpu().numpy(), wzp)


def test_batch_quantize_reference_kats_through_hip(fc):
    """tflite/kernels/internal/tensor_utils_test.cc:220-345."""
    a = np.array([[-640, -635.0, -630, 10.0, 2.0, -5.0, -10.0, 0.0, 1000.0]], np.float32)
    small = np.array([[-1e-5, 3e-5, -7e-6, -9e-5, 1e-6, 4e-5, 9e-6, 2e-4, 0]], np.float32)
    q, _, _ = fc.batch_quantize_floats(_cuda(a), False)
    assert q.cpu().numpy()[0].tolist() == [-81, -81, -80, 1, 0, -1, -1, 0, 127]
    q, _, _ = fc.batch_quantize_floats(_cuda(small), False)
    assert q.cpu().numpy()[0].tolist() == [-6, 19, -4, -57, 1, 25, 6, 127, 0]
    q, _, zp = fc.batch_quantize_floats(_cuda(a), True)
    assert q.cpu().numpy()[0].tolist() == [-128, -127, -126, -26, -28, -29, -30, -28, 127]
    q, sf, zp = fc.batch_quantize_floats(_cuda(np.full((1, 9), 2000, np.float32)), True)
    assert q.cpu().numpy()[0].tolist() == [127] * 9
    q, _, _ = fc.batch_quantize_floats(_cuda(small), True)
    assert q.cpu().numpy()[0].tolist() == [-58, -23, -55, -128, -48, -14, -41, 127, -49]
    q, sf, zp = fc.batch_quantize_floats(_cuda(np.zeros((1, 9), np.float32)), True)
    assert q.cpu().numpy()[0].tolist() == [0] * 9 and sf.item() == 1 and zp.item() == 0


# ---- hybrid ----------------------------------------------------------------------------

def _hybrid_call(op, x, mode):
    """mode: "fused" (one kernel whatever the batch), "split" (quantizer launch + GEMV on the
    packed filter), True (the class's own choice between those two), False (row-major)."""
    if mode == "fused":
        op.FUSED_MAX_BATCHES = 1 << 30
        return op(x)
    if mode == "split":
        return op.call_split(x)
    return op(x)


@pytest.mark.parametrize("B", [1, 4, 8])
@pytest.mark.parametrize("packed", ["fused", "split", True, False])
def test_hybrid_config2_shape(fc, B, packed):
    """Config 2 at its real depth with a reduced number of output channels (the scalar
    oracle needs ~60 ms per 1000 channels per batch row); the fused single-kernel form on
    the re-tiled filter and the two-kernel form on the row-major one."""
    c = wl.hybrid_fc(B, 4096, 2048)
    op = fc.FullyConnectedHybrid(c["w"], c["pcs"], packed=bool(packed))
    y = _hybrid_call(op, _cuda(c["x"]), packed).cpu().numpy()
    want = oracle.fc_hybrid(c["x"], c["w"], c["pcs"])
    assert _close(y, want)
    assert _bits_equal(y, want)


@pytest.mark.parametrize("B,K,N", [(1, 64, 5), (3, 1040, 33), (2, 100, 7), (6, 512, 130),
                                   (19, 257, 21)])
@pytest.mark.parametrize("asym", [True, False])
@pytest.mark.parametrize("per_channel", [True, False])
@pytest.mark.parametrize("activation", ["none", "relu", "relu_n1_to_1", "relu6"])
@pytest.mark.parametrize("packed", ["fused", "split", False])
def test_hybrid_variants(fc, B, K, N, asym, per_channel, activation, packed):
    c = wl.hybrid_fc(B, K, N, seed=7 + B + K)
    bias = np.random.default_rng(3).standard_normal(N).astype(np.float32)
    pcs = c["pcs"] if per_channel else None
    op = fc.FullyConnectedHybrid(c["w"], pcs, filter_scale=0.005, bias=bias,
                                 asymmetric_quantize_inputs=asym, activation=activation,
                                 packed=bool(packed))
    y = _hybrid_call(op, _cuda(c["x"]), packed).cpu().numpy()
    want = oracle.fc_hybrid(c["x"], c["w"], pcs, 0.005, bias, asym, fc._act(activation))
    assert _close(y, want)
    assert _bits_equal(y, want)


@pytest.mark.parametrize("B,K,N", [(1, 16384, 40), (1, 8192, 48), (2, 8192, 24), (1, 10000, 33),
                                   (1, 4100, 20), (2, 16384, 16), (3, 8192, 16), (1, 20000, 8)])
@pytest.mark.parametrize("asym", [True, False])
def test_hybrid_deep_rows(fc, B, K, N, asym):
    """Rows deeper than 4096: one row up to 16384 deep and two rows up to 8192 stay in registers
    through the fused prologue (their own kernel variants); the rest are read twice."""
    c = wl.hybrid_fc(B, K, N, seed=21 + B + K)
    op = fc.FullyConnectedHybrid(c["w"], c["pcs"], asymmetric_quantize_inputs=asym)
    y = _hybrid_call(op, _cuda(c["x"]), "fused").cpu().numpy()
    want = oracle.fc_hybrid(c["x"], c["w"], c["pcs"], 1.0, None, asym, 0)
    assert _bits_equal(y, want)


def test_hybrid_dot_reference_kats_through_hip(fc):
    """tflite/kernels/internal/tensor_utils_test.cc:1214-1231 (per-channel + offsets), exact."""
    from tests.test_oracle_kat import _mv_data
    from litert_amd import capi
    import ctypes as C
    for (rows, cols, batch), idx_want in (
            ((4, 16, 1), {0: 620, 1: 3160, 2: 2540, 3: 7000}),
            ((4, 32, 2), dict(enumerate([5208, 26288, 4245, 23312, 9138, 70756, 18708, 60916]))),
            ((32, 512, 5), {0: 207783, 13: 411552, 39: 835936, 50: 440368, 100: 875192,
                            123: 1775536, 150: 1050930})):
        m, v, sf, _, pcs, offs = _mv_data(rows, cols, batch, per_channel=True)
        dm, dv = _cuda(m), _cuda(v)
        dsf, dpcs, doffs = _cuda(sf[:batch].copy()), _cuda(pcs), _cuda(offs)
        rs = torch.empty(rows, dtype=torch.int32, device="cuda")
        out = torch.empty((batch, rows), dtype=torch.float32, device="cuda")
        lib = capi.load()
        p = lambda t: C.c_void_p(t.data_ptr())
        capi.check(lib.lrtfc_row_sums_int8(p(dm), rows, cols, p(rs), None))
        capi.check(lib.lrtfc_fc_hybrid_int8(p(dv), p(dsf), p(doffs), p(dm), p(dpcs), 1.0, p(rs),
                                            None, p(out), batch, cols, rows, 0, None))
        torch.cuda.synchronize()
        got = out.cpu().numpy().ravel()
        for i, w in idx_want.items():
            assert got[i] == w


@pytest.mark.parametrize("variant", [1, 2])
def test_hybrid_fused_quantizer_variants(fc, variant):
    """The in-kernel quantizer of the fused form reproduces the NEON-flavoured variants too,
    including the scalar tail of a row whose length is not a multiple of 8."""
    c = wl.hybrid_fc(3, 1004, 40, seed=21)
    c["x"][0, :4] = [-125.0, 130.0, 2.5, -2.5]
    op = fc.FullyConnectedHybrid(c["w"], c["pcs"], quant_variant=variant)
    y = op(_cuda(c["x"])).cpu().numpy()
    want = oracle.fc_hybrid(c["x"], c["w"], c["pcs"], variant=variant)
    assert _bits_equal(y, want)


@pytest.mark.parametrize("activation", ["none", "relu", "relu_n1_to_1", "relu6", "sign_bit"])
@pytest.mark.parametrize("packed", ["fused", "split", False])
@pytest.mark.parametrize("B", [1, 3, 19])
def test_hybrid_whole_zero_input_keeps_the_bias_bits(fc, activation, packed, B):
    """tflite/kernels/fully_connected.cc:789-795: a whole-zero input (a -0.0f element counts as
    zero) leaves activation(bias) in the output and skips the product. Adding a zero product
    instead would turn a bias element of -0.0f into +0.0f, so the bias here holds -0.0f, +0.0f
    and ordinary values. Then one row is made non-zero: the exit no longer applies and the zero
    rows go through the product like any other (-0.0f + 0.0f = +0.0f)."""
    K, N = 520, 70
    c = wl.hybrid_fc(B, K, N, seed=31)
    bias = np.random.default_rng(9).standard_normal(N).astype(np.float32)
    bias[::3] = -0.0
    bias[1::7] = 0.0
    op = fc.FullyConnectedHybrid(c["w"], c["pcs"], bias=bias, activation=activation,
                                 packed=bool(packed))
    x = np.zeros((B, K), np.float32)
    x[0, 5] = -0.0
    y = _hybrid_call(op, _cuda(x), packed).cpu().numpy()
    want = oracle.fc_hybrid(x, c["w"], c["pcs"], 1.0, bias, True, fc._act(activation))
    assert _bits_equal(y, want)
    if activation == "none":
        assert _bits_equal(y, np.broadcast_to(bias, (B, N)).copy())
    x[B - 1] = c["x"][B - 1]
    y = _hybrid_call(op, _cuda(x), packed).cpu().numpy()
    want = oracle.fc_hybrid(x, c["w"], c["pcs"], 1.0, bias, True, fc._act(activation))
    assert _bits_equal(y, want)


@pytest.mark.parametrize("packed", ["fused", "split", False])
def test_hybrid_sign_bit_activation(fc, packed):
    """kTfLiteActSignBit on the hybrid path (tensor_utils.h:58-77 ->
    portable_tensor_utils.cc:65-71): 1.0f where the result's sign bit is set."""
    c = wl.hybrid_fc(5, 1040, 33, seed=12)
    op = fc.FullyConnectedHybrid(c["w"], c["pcs"], activation="sign_bit", packed=bool(packed))
    y = _hybrid_call(op, _cuda(c["x"]), packed).cpu().numpy()
    want = oracle.fc_hybrid(c["x"], c["w"], c["pcs"], 1.0, None, True, oracle.ACT_SIGN_BIT)
    assert _bits_equal(y, want)
    assert set(np.unique(y)) == {0.0, 1.0}


def test_hybrid_full_size_properties(fc):
    """Config 2 at full size (14336 x 4096, B = 8): row sums against numpy, a sample of
    output channels against the oracle, and batch-row independence (row b of a B=8 call
    equals the B=1 call on that row)."""
    c = wl.hybrid_fc(8)
    op = fc.FullyConnectedHybrid(c["w"], c["pcs"])
    x = _cuda(c["x"])
    y8 = op(x).cpu().numpy()
    assert np.array_equal(op.row_sums.cpu().numpy(), c["w"].astype(np.int32).sum(1))
    y1 = op(x[3:4]).cpu().numpy()
    assert _bits_equal(y8[3:4], y1)
    pick = np.random.default_rng(2).choice(14336, 256, replace=False)
    want = oracle.fc_hybrid(c["x"], c["w"][pick], c["pcs"][pick])
    assert _bits_equal(np.ascontiguousarray(y8[:, pick]), want)
    # B = 4 at full width (the batch size at which the fused kernel keeps four rows in
    # registers): every channel against the oracle.
    y4 = op(x[:4]).cpu().numpy()
    want4 = oracle.fc_hybrid(c["x"][:4], c["w"], c["pcs"])
    assert _bits_equal(y4, want4)


# ---- blockwise int4 -------------------------------------------------------------------------

def _run_int4(fc, c, bias=None, packed=True):
    N = c["w"].shape[0]
    op = fc.FullyConnectedBlockwiseInt4(c["packed"], c["scales"], c["w"].shape[1], c["blocksize"],
                                        bias, packed=packed)
    y = op(_cuda(c["x"])).cpu().numpy()
    want = oracle.fc_blockwise_int4(c["x"], c["packed"], N, c["scales"].view(np.uint16),
                                    c["blocksize"], bias)
    return y, want


@pytest.mark.parametrize("B,K,N", [(1, 4096, 1024), (4, 2048, 512), (1, 2048, 256), (4, 16384, 64),
                                   (1, 16384, 130), (2, 32, 4), (3, 96, 9), (8, 1024, 77),
                                   (5, 4096, 40), (1, 8192, 31), (9, 2048, 20), (2, 6144, 24),
                                   (3, 16384, 24), (2, 8192, 16), (1, 32768, 12), (2, 20480, 8),
                                   (2, 17408, 10), (4, 16384, 2048), (1, 9216, 520)])
@pytest.mark.parametrize("packed", [True, False])
def test_blockwise_int4_shapes(fc, B, K, N, packed):
    """Config 3 / config 5 depths (2048, 4096, 16384) and ragged sizes, blocksize 32, with the
    full signed nibble range including -8."""
    c = wl.blockwise_int4_fc(B, K, N, seed=11 + B + K + N, lo=-8, hi=7)
    bias = np.random.default_rng(4).standard_normal(N).astype(np.float32) if N % 2 else None
    y, want = _run_int4(fc, c, bias, packed=packed)
    assert _close(y, want)
    assert _bits_equal(y, want)


@pytest.mark.parametrize("B,K,N", [(1, 4096, 72), (4, 2048, 33), (4, 16384, 16), (3, 8192, 9),
                                   (7, 1056, 24), (2, 20480, 8)])
def test_blockwise_int4_split_launch_matches_oracle(fc, B, K, N):
    """Standalone quantizer + streaming kernel on pre-quantized rows (the form used for deep
    rows with more than two batch rows)."""
    c = wl.blockwise_int4_fc(B, K, N, seed=3 + B + K + N, lo=-8, hi=7)
    op = fc.FullyConnectedBlockwiseInt4(c["packed"], c["scales"], K, 32)
    y = op.call_split(_cuda(c["x"])).cpu().numpy()
    want = oracle.fc_blockwise_int4(c["x"], c["packed"], N, c["scales"].view(np.uint16), 32)
    assert _bits_equal(y, want)


@pytest.mark.parametrize("B,K,Ns", [(1, 2048, (64, 8, 24, 130, 520)), (3, 2048, (16, 256, 9)),
                                    (4, 1024, (40,)), (1, 16384, (16, 40)), (2, 8192, (24, 8, 72)),
                                    (9, 2048, (24, 80)), (5, 16384, (8, 16)),
                                    # deep rows beyond two: quantized by the group's own launch
                                    (3, 8192, (24, 40, 8)), (4, 16384, (16, 264)), (9, 8192, (8, 72)),
                                    (1, 64, tuple(range(4, 36))), (2, 64, tuple(range(3, 103))),
                                    # 4096..8191 channels in all: two wavefronts share a channel
                                    # group's depth and four deep rows no longer fit the LDS, so
                                    # the launch falls back to two rows at a time
                                    (4, 16384, (2048, 2056)), (3, 16384, (4100,)),
                                    # wide and deep: the 4-bit-resident matrix-core form
                                    (4, 16384, (2048,) * 8), (3, 16384, (8200, 8200)),
                                    (4, 8224, (9000, 7400, 33)),
                                    # deeper than the register forms: rows re-read, LDS-bound tile
                                    (3, 32768, (16, 24)), (4, 32768, (8,))])
def test_blockwise_int4_grouped_launch_matches_oracle(fc, B, K, Ns):
    """Several filters of one depth in one launch: every node against the oracle, with its
    own input and, for odd channel counts, its own bias; then again after re-binding to new
    inputs (the table is rewritten, the filters are not)."""
    rng = np.random.default_rng(8)
    cs = [wl.blockwise_int4_fc(B, K, n, seed=500 + i + n, lo=-8, hi=7) for i, n in enumerate(Ns)]
    biases = [rng.standard_normal(n).astype(np.float32) if n % 2 else None for n in Ns]
    ops = [fc.FullyConnectedBlockwiseInt4(c["packed"], c["scales"], K, 32, b)
           for c, b in zip(cs, biases)]
    group = fc.GroupedBlockwiseInt4(ops)
    for trial in range(2):
        xs_np = [c["x"] if trial == 0 else rng.standard_normal((B, K)).astype(np.float32) for c in cs]
        xs = [_cuda(x) for x in xs_np]
        ys = [torch.full((B, n), float("nan"), dtype=torch.float32, device="cuda") for n in Ns]
        group.bind(xs, ys)()
        torch.cuda.synchronize()
        # three or four rows deeper than 8192 run on the filters kept at 4 bits per weight for
        # the matrix cores (four blocks per tile); everything else on the decode tiling
        from litert_amd import capi
        wide = sum((n + 15) // 16 for n in Ns) >= 1024  # a wavefront per SIMD at least
        assert group.launch.form == (capi.INT4_FORM_GEMM_NIBBLES
                                     if B in (3, 4) and K > 8192 and wide else capi.INT4_FORM_DECODE)
        for c, b, x, y, n in zip(cs, biases, xs_np, ys, Ns):
            want = oracle.fc_blockwise_int4(x, c["packed"], n, c["scales"].view(np.uint16), 32, b)
            assert _bits_equal(y.cpu().numpy(), want), (trial, n)


@pytest.mark.parametrize("B", [1, 3])
def test_blockwise_int4_wavefronts_spanning_channel_groups(fc, B):
    """Launches large enough that one wavefront works through 8 consecutive channel groups
    (7169 groups of 8 channels, depth 2048): a single node whose last wavefront and last group
    are partial, then three nodes of the same total size in one launch."""
    K = 2048
    c = wl.blockwise_int4_fc(B, K, 57349, seed=77, lo=-8, hi=7)
    bias = np.random.default_rng(3).standard_normal(57349).astype(np.float32)
    op = fc.FullyConnectedBlockwiseInt4(c["packed"], c["scales"], K, 32, bias)
    y = op(_cuda(c["x"])).cpu().numpy()
    want = oracle.fc_blockwise_int4(c["x"], c["packed"], 57349, c["scales"].view(np.uint16), 32, bias)
    assert _bits_equal(y, want)
    Ns = (40000, 264, 17101)
    cs = [wl.blockwise_int4_fc(B, K, n, seed=900 + n, lo=-8, hi=7) for n in Ns]
    ops = [fc.FullyConnectedBlockwiseInt4(ci["packed"], ci["scales"], K, 32) for ci in cs]
    xs = [_cuda(ci["x"]) for ci in cs]
    ys = [torch.full((B, n), float("nan"), dtype=torch.float32, device="cuda") for n in Ns]
    fc.GroupedBlockwiseInt4(ops).bind(xs, ys)()
    torch.cuda.synchronize()
    for ci, yi, n in zip(cs, ys, Ns):
        want = oracle.fc_blockwise_int4(ci["x"], ci["packed"], n, ci["scales"].view(np.uint16), 32)
        assert _bits_equal(yi.cpu().numpy(), want), n


@pytest.mark.parametrize("B,K,N,bias", [(16, 64, 8, False), (33, 128, 20, True), (64, 256, 70, False),
                                        (100, 2048, 264, True), (17, 4096, 130, False),
                                        (128, 1024, 64, True), (65, 96, 5, True), (1, 64, 4, False),
                                        (250, 32, 33, False), (16, 1184, 40, True),
                                        (32, 2080, 24, False), (140, 1056, 48, True),
                                        (300, 4128, 36, False), (8, 32, 20, True), (40, 96, 24, False),
                                        (20, 544, 16, True)])
def test_blockwise_int4_gemm_matches_oracle(fc, B, K, N, bias):
    """Prefill form (matrix-core GEMM, one float accumulator per output walking the blocks in
    order): bit-identical to the oracle, edges in every direction (rows and channels that do
    not fill their tiles, one block, odd block counts that end inside a pair and inside a group
    of 16 scales, odd channel counts with scalar stores) in each of the kernel's tile forms."""
    c = wl.blockwise_int4_fc(B, K, N, seed=11 + B + K + N, lo=-8, hi=7)
    b = np.random.default_rng(B).standard_normal(N).astype(np.float32) if bias else None
    op = fc.FullyConnectedBlockwiseInt4(c["packed"], c["scales"], K, 32, b)
    y = op.call_gemm(_cuda(c["x"])).cpu().numpy()
    want = oracle.fc_blockwise_int4(c["x"], c["packed"], N, c["scales"].view(np.uint16), 32, b)
    assert _bits_equal(y, want)
    if B >= op.GEMM_MIN_BATCHES:  # the op picks a GEMM form by itself from 16 rows on
        assert _bits_equal(op(_cuda(c["x"])).cpu().numpy(), want)
    # The same shapes on the filter kept at 4 bits per weight (quads of blocks, groups of 16
    # scales, one or two row tiles per wavefront).
    assert _bits_equal(op.call_gemm_nibbles(_cuda(c["x"])).cpu().numpy(), want)


@pytest.mark.parametrize("B,K,N,bias", [(1, 32, 16, True), (2, 64, 5, False), (3, 96, 40, True),
                                        (4, 2048, 72, False), (4, 16384, 24, True),
                                        (3, 4128, 33, False), (4, 160, 100, True), (1, 4096, 520, False),
                                        (2, 544, 17, True)])
@pytest.mark.parametrize("variant", [0, 1, 2])
def test_blockwise_int4_nibble_gemm_up_to_four_rows_matches_oracle(fc, B, K, N, bias, variant):
    """One to four rows on the filter kept at 4 bits per weight: the four blocks of a quad share
    one matrix-core tile (columns = block x row), the products of blocks 1..3 reach block 0's
    lanes by row shifts and are added there in block order. Depths that end inside a quad and
    inside a group of 16 scales, fewer than four rows (the clamped copies are not stored),
    ragged channel counts, every quantizer variant."""
    c = wl.blockwise_int4_fc(B, K, N, seed=21 + B + K + N, lo=-8, hi=7)
    b = np.random.default_rng(B).standard_normal(N).astype(np.float32) if bias else None
    op = fc.FullyConnectedBlockwiseInt4(c["packed"], c["scales"], K, 32, b, quant_variant=variant)
    y = op.call_gemm_nibbles(_cuda(c["x"])).cpu().numpy()
    want = oracle.fc_blockwise_int4(c["x"], c["packed"], N, c["scales"].view(np.uint16), 32, b,
                                    variant=variant)
    assert _bits_equal(y, want)


def test_blockwise_int4_nibble_gemm_full_width_and_dispatch(fc):
    """The nibble-resident GEMM on config 3's filter at 5, 8 and 24 rows: what the op picks by
    itself for this shape (lrtfc_fc_blockwise_int4_preferred_form), bit-identical to the decode
    kernel on the same rows and, on a sample of channels, to the oracle; with the two NEON
    quantizer flavours on the way."""
    from litert_amd import capi
    lib = capi.load()
    assert lib.lrtfc_fc_blockwise_int4_preferred_form(4, 4096, 14336) == capi.INT4_FORM_DECODE
    assert lib.lrtfc_fc_blockwise_int4_preferred_form(5, 4096, 14336) == capi.INT4_FORM_GEMM_NIBBLES
    assert lib.lrtfc_fc_blockwise_int4_preferred_form(32, 4096, 14336) == capi.INT4_FORM_GEMM_NIBBLES
    assert lib.lrtfc_fc_blockwise_int4_preferred_form(33, 4096, 14336) == capi.INT4_FORM_GEMM_INT8
    assert lib.lrtfc_fc_blockwise_int4_preferred_form(8, 16384, 2048) == capi.INT4_FORM_DECODE
    assert lib.lrtfc_fc_blockwise_int4_preferred_form(16, 16384, 2048) == capi.INT4_FORM_GEMM_INT8
    c = wl.blockwise_int4_fc(4)
    sample = np.arange(0, 14336, 449)
    for rows, variant in ((5, 0), (8, 1), (24, 2)):
        x = np.random.default_rng(rows).standard_normal((rows, 4096)).astype(np.float32)
        x[0, :4] = [-125.0, 130.0, 2.5, -2.5]
        op = fc.FullyConnectedBlockwiseInt4(c["packed"], c["scales"], 4096, 32,
                                            quant_variant=variant)
        xd = _cuda(x)
        got = op(xd).cpu().numpy()
        assert op._nibble_filter is not None and op._gemm_filter is None
        decode = torch.cat([fc.FullyConnectedBlockwiseInt4.__call__(op, xd[i:i + 4])
                            for i in range(0, rows, 4)]).cpu().numpy()
        assert _bits_equal(got, decode)
        want = oracle.fc_blockwise_int4(x, c["packed"][sample], sample.size,
                                        c["scales"][sample].view(np.uint16), 32,
                                        variant=variant)
        assert _bits_equal(got[:, sample], want)


def test_blockwise_int4_gemm_full_width_agrees_with_decode_kernel(fc):
    """256 rows against the full-size filter of config 3 (14336 x 4096): the GEMM and the
    decode kernel (64 passes of four rows) must agree bit for bit; a sample of channels is
    also checked against the oracle."""
    c = wl.blockwise_int4_fc(4)
    x = np.random.default_rng(12).standard_normal((256, 4096)).astype(np.float32)
    op = fc.FullyConnectedBlockwiseInt4(c["packed"], c["scales"], 4096, 32)
    xd = _cuda(x)
    gemm = op.call_gemm(xd).cpu().numpy()
    decode = torch.cat([op(xd[i:i + 4]) for i in range(0, 256, 4)]).cpu().numpy()
    assert _bits_equal(gemm, decode)
    rows = [0, 100, 255]
    sample = np.arange(0, 14336, 449)
    want = oracle.fc_blockwise_int4(x[rows], c["packed"][sample], sample.size,
                                    c["scales"][sample].view(np.uint16), 32)
    assert _bits_equal(gemm[rows][:, sample], want)


@pytest.mark.parametrize("variant", [1, 2])
def test_blockwise_int4_grouped_deep_rows_quantizer_variants(fc, variant):
    """The group's row quantizer launch (deep rows, more than two per node, filters too large in
    all for the side-by-side form of small groups) in the two NEON flavours, with elements on
    rounding ties."""
    B, K, Ns = 4, 8200 - 8, (4104, 2056)
    cs = [wl.blockwise_int4_fc(B, K, n, seed=40 + n) for n in Ns]
    for c in cs:
        c["x"][0, :4] = [-125.0, 130.0, 2.5, -2.5]
    ops = [fc.FullyConnectedBlockwiseInt4(c["packed"], c["scales"], K, 32, quant_variant=variant)
           for c in cs]
    ys = [torch.empty((B, n), dtype=torch.float32, device="cuda") for n in Ns]
    group = fc.GroupedBlockwiseInt4(ops).bind([_cuda(c["x"]) for c in cs], ys)
    assert group.launch.split_quantize == 1
    group()
    torch.cuda.synchronize()
    for c, y, n in zip(cs, ys, Ns):
        want = oracle.fc_blockwise_int4(c["x"], c["packed"], n, c["scales"].view(np.uint16), 32,
                                        variant=variant)
        assert _bits_equal(y.cpu().numpy(), want), n


@pytest.mark.parametrize("B,K,Ns,variant", [(4, 2048, (2048,), 0), (3, 2048, (2048, 256, 256), 1),
                                            (4, 16384, (264,), 2), (3, 8192, (24, 40, 8), 0),
                                            (4, 4096 + 64, (72,), 0)])
def test_blockwise_int4_small_groups_run_row_pairs_side_by_side(fc, B, K, Ns, variant):
    """Three or four rows of a small group (a decoder stage) go as two fused pairs in one launch:
    rows 2 and 3 from the second slice of the grid, a third row alone in its slice."""
    cs = [wl.blockwise_int4_fc(B, K, n, seed=90 + i + n, lo=-8, hi=7) for i, n in enumerate(Ns)]
    for c in cs:
        c["x"][B - 1, :4] = [-125.0, 130.0, 2.5, -2.5]
    ops = [fc.FullyConnectedBlockwiseInt4(c["packed"], c["scales"], K, 32, quant_variant=variant)
           for c in cs]
    ys = [torch.full((B, n), float("nan"), dtype=torch.float32, device="cuda") for n in Ns]
    group = fc.GroupedBlockwiseInt4(ops).bind([_cuda(c["x"]) for c in cs], ys)
    assert group.launch.split_quantize == 2
    group()
    torch.cuda.synchronize()
    for c, y, n in zip(cs, ys, Ns):
        want = oracle.fc_blockwise_int4(c["x"], c["packed"], n, c["scales"].view(np.uint16), 32,
                                        variant=variant)
        assert _bits_equal(y.cpu().numpy(), want), n


def test_blockwise_int4_grouped_launch_needs_bind(fc):
    c = wl.blockwise_int4_fc(1, 64, 8, seed=2, lo=-8, hi=7)
    op = fc.FullyConnectedBlockwiseInt4(c["packed"], c["scales"], 64, 32)
    with pytest.raises(RuntimeError):
        fc.GroupedBlockwiseInt4([op])()
    with pytest.raises(ValueError):
        fc.GroupedBlockwiseInt4([])
    with pytest.raises(ValueError):
        fc.GroupedBlockwiseInt4([op] * (fc.GroupedBlockwiseInt4.MAX_NODES + 1))


@pytest.mark.parametrize("B,K,N,bs", [(2, 128, 6, 64), (1, 64, 5, 16), (3, 256, 4, 128), (2, 96, 8, 8)])
def test_blockwise_int4_other_block_sizes(fc, B, K, N, bs):
    c = wl.blockwise_int4_fc(B, K, N, blocksize=bs, seed=5 + bs, lo=-8, hi=7)
    y, want = _run_int4(fc, c)
    assert _close(y, want)
    assert _bits_equal(y, want)


@pytest.mark.parametrize("variant", [1, 2])
def test_blockwise_int4_fused_quantizer_variants(fc, variant):
    c = wl.blockwise_int4_fc(3, 1056, 24, seed=8)
    c["x"][0, :4] = [-125.0, 130.0, 2.5, -2.5]
    op = fc.FullyConnectedBlockwiseInt4(c["packed"], c["scales"], 1056, 32, quant_variant=variant)
    y = op(_cuda(c["x"])).cpu().numpy()
    want = oracle.fc_blockwise_int4(c["x"], c["packed"], 24, c["scales"].view(np.uint16), 32,
                                    variant=variant)
    assert _bits_equal(y, want)


@pytest.mark.parametrize("packed", [True, False])
def test_blockwise_int4_subnormal_and_large_scales(fc, packed):
    c = wl.blockwise_int4_fc(2, 256, 16, seed=3)
    s = c["scales"].view(np.uint16).copy()
    s[0, :] = [0x0001, 0x03FF, 0x0400, 0x7BFF, 0x8001, 0x0000, 0x3C00, 0xBC00]  # subnormals, max, -0...
    c["scales"] = s.view(np.float16)
    y, want = _run_int4(fc, c, packed=packed)
    assert _bits_equal(y, want)


def test_blockwise_int4_config3_full_size_properties(fc):
    """Config 3 at full size (14336 x 4096): a sample of output channels against the oracle
    and batch-row independence between B=4 and B=1 calls."""
    c = wl.blockwise_int4_fc(4)
    op = fc.FullyConnectedBlockwiseInt4(c["packed"], c["scales"], 4096, 32)
    x = _cuda(c["x"])
    y4 = op(x).cpu().numpy()
    y1 = op(x[2:3]).cpu().numpy()
    assert _bits_equal(y4[2:3], y1)
    pick = np.random.default_rng(6).choice(14336, 192, replace=False)
    want = oracle.fc_blockwise_int4(c["x"], c["packed"][pick], pick.size,
                                    c["scales"][pick].view(np.uint16), 32)
    assert _bits_equal(np.ascontiguousarray(y4[:, pick]), want)


# ---- edge cases of the op contract ------------------------------------------------------------

def test_empty_and_zero_depth(fc):
    """NumElements(output) == 0 is a no-op and depth 0 zero-fills
    (tflite/kernels/fully_connected.cc:1966-1973)."""
    import ctypes as C
    from litert_amd import capi
    lib = capi.load()
    out = torch.full((2, 3), 7, dtype=torch.int8, device="cuda")
    one = torch.ones(1, dtype=torch.int32, device="cuda")
    p = lambda t: C.c_void_p(t.data_ptr())
    capi.check(lib.lrtfc_fc_int8(None, None, None, p(one), p(one), 0, None, p(out), 0, 16, 3, 0, 0,
                                 0, -128, 127, None))
    torch.cuda.synchronize()
    assert out.eq(7).all()
    capi.check(lib.lrtfc_fc_int8(None, None, None, p(one), p(one), 0, None, p(out), 2, 0, 3, 0, 0,
                                 0, -128, 127, None))
    torch.cuda.synchronize()
    assert out.eq(0).all()
    rc = lib.lrtfc_fc_int8(p(out), p(out), None, p(one), p(one), 0, None, p(out), 2, 16, 3, 5, 0, 0,
                           -128, 127, None)
    assert rc == capi.INVALID_ARGUMENT and b"filter_row_sums" in lib.lrtfc_last_error()


# ---- per-channel int4 hybrid (EvalHybridDense4Bit) ----------------------------------------

@pytest.mark.parametrize("B,K,N", [(1, 32, 4), (4, 40, 5), (3, 46, 7), (2, 256, 17), (1, 4096, 512),
                                   (8, 2048, 130), (16, 1000, 33), (40, 512, 72), (130, 272, 48),
                                   # 17..32 rows: on the int8 expansion they take the one-pass GEMV
                                   (20, 2048, 130), (32, 4096, 40), (17, 1008, 33),
                                   # 33..128 rows on a wide filter: the chunked one-pass kernel
                                   (48, 1040, 10240), (100, 1536, 10255),
                                   # GEMM tiles whose outputs leave through LDS, beside ragged ones
                                   (200, 512, 384)])
@pytest.mark.parametrize("activation", ["none", "relu", "relu6"])
def test_hybrid_int4_per_channel_matches_oracle(fc, B, K, N, activation):
    """Bit-identical floats against the oracle (itself bit-identical to the reference's 4-bit
    kernels): decode batches on the GEMV, more than 32 rows on the GEMM, ragged shapes, an
    all-zero row, per-channel scales with and without bias."""
    from tests import kat_harness as kh
    rng = np.random.default_rng(700 + B + K + N)
    x = rng.standard_normal((B, K)).astype(np.float32)
    if B > 2:
        x[1] = 0
    w = rng.integers(-7, 8, (N, K)).astype(np.int8)
    packed = np.stack([kh.pack_int4(r) for r in w])
    fs = rng.uniform(0.01, 0.1, N).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32) if N % 2 else None
    op = fc.FullyConnectedHybridInt4PerChannel(packed, K, fs, bias, activation)
    y = op(_cuda(x)).cpu().numpy()
    want = oracle.fc_hybrid_int4_per_channel(x, packed, N, fs, bias, fc._act(activation))
    assert _bits_equal(y, want)
    # both device layouts (nibbles for decode batches, int8 expansion for prefill) agree
    assert _bits_equal(op(_cuda(x), force_int8=True).cpu().numpy(), want)


def test_hybrid_int4_per_channel_nibble_layout_shapes(fc):
    """The 4-bit-resident GEMV on its own entry point: a depth split over several wavefronts
    (few channels, deep rows), 17..32 rows (two passes over the filter), a depth that is not a
    multiple of 16 or 128, one filter scale for every channel."""
    from tests import kat_harness as kh
    rng = np.random.default_rng(99)
    for B, K, N, per_channel in ((1, 8192, 24, True), (20, 640, 40, True), (32, 1024, 16, False),
                                 (3, 34, 5, True), (2, 130, 9, False), (5, 16384, 8, True)):
        x = rng.standard_normal((B, K)).astype(np.float32)
        w = rng.integers(-7, 8, (N, K)).astype(np.int8)
        packed = np.stack([kh.pack_int4(r) for r in w])
        fs = rng.uniform(0.01, 0.1, N).astype(np.float32) if per_channel else np.array([0.03], np.float32)
        op = fc.FullyConnectedHybridInt4PerChannel(packed, K, fs)
        y = op(_cuda(x)).cpu().numpy()
        assert op._retiled_nibbles is not None and op._packed_int8 is None
        want = oracle.fc_hybrid_int4_per_channel(x, packed, N, np.broadcast_to(fs, (N,)).copy(), None, 0)
        assert _bits_equal(y, want), (B, K, N)


@pytest.mark.parametrize("B,K,N", [
    # fused rows (1..4) on the register-resident form: shares of 8 / 16 / 32 tiles, a depth that
    # ends inside a lane's eight values, inside a slab, at one slab, at the form's limit
    (1, 4096, 1040), (2, 4092, 520), (4, 4096, 300), (3, 2000, 700), (4, 1028, 100), (1, 100, 50),
    (2, 4, 16), (4, 2048, 8200),
    # few channel groups: the depth is split over the wavefronts of a workgroup
    (1, 4096, 16), (3, 4096, 100), (2, 2048, 40),
    # rows that arrive quantized: 4 and 16 chunks per thread, depth not a multiple of 128
    (5, 1024, 300), (8, 4096, 520), (16, 4096, 1040), (16, 2000, 130), (12, 4080, 64), (9, 16, 20)])
def test_hybrid_int4_per_channel_register_resident_form(fc, B, K, N):
    from tests import kat_harness as kh
    rng = np.random.default_rng(B * 7 + K + N)
    x = (rng.standard_normal((B, K)) * rng.uniform(0.1, 30, (B, 1))).astype(np.float32)
    if B > 2:
        x[1] = 0
    w = rng.integers(-7, 8, (N, K)).astype(np.int8)
    packed = np.stack([kh.pack_int4(r) for r in w])
    fs = rng.uniform(0.01, 0.1, N).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32) if N % 8 else None
    op = fc.FullyConnectedHybridInt4PerChannel(packed, K, fs, bias, "relu" if K % 3 else "none")
    flat = torch.empty(B * N + 1, device="cuda")
    y = (flat[1:] if (B + N) % 2 else flat[:-1]).view(B, N)   # every other case: rows off 16 bytes
    got = op(_cuda(x), out=y).cpu().numpy()
    want = oracle.fc_hybrid_int4_per_channel(x, packed, N, fs, bias, op.activation)
    assert _bits_equal(got, want), (B, K, N)


def test_hybrid_int4_per_channel_seeded_random_shapes(fc):
    """Forty seeded draws over row counts, even depths and channel counts that cross every launch
    rule of the 4-bit-resident GEMV (fused rows or not, register-resident or ring, depth shares,
    16-row passes), each bit-identical to the oracle."""
    from tests import kat_harness as kh
    rng = np.random.default_rng(20240607)
    for case in range(40):
        B = int(rng.integers(1, 21))
        K = int(rng.choice([2, 4, 16]) * rng.integers(1, 300))
        N = int(rng.integers(1, 600))
        x = (rng.standard_normal((B, K)) * rng.uniform(0.05, 50)).astype(np.float32)
        w = rng.integers(-7, 8, (N, K)).astype(np.int8)
        packed = np.stack([kh.pack_int4(r) for r in w])
        fs = rng.uniform(0.01, 0.1, N).astype(np.float32)
        bias = rng.standard_normal(N).astype(np.float32) if case % 3 else None
        op = fc.FullyConnectedHybridInt4PerChannel(packed, K, fs, bias, ("none", "relu", "relu6")[case % 3])
        got = op(_cuda(x)).cpu().numpy()
        want = oracle.fc_hybrid_int4_per_channel(x, packed, N, fs, bias, op.activation)
        assert _bits_equal(got, want), (case, B, K, N)


def test_hybrid_int4_per_channel_reference_kat_and_scalar_scale(fc):
    """tflite/kernels/fully_connected_4bit_test.cc:102-190 through the HIP path (the test's own
    tolerance), with the single filter scale the test model uses."""
    from tests import kat_harness as kh
    a = [-1, 2, 3, 4, 5, 6, 7, 1, 2, 3] * 2
    b = [1, 2, 3, 4, 5, 6, 7, 1, 2, -3] + [-1, 2, 3, 4, 5, 6, 7, 1, 2, 3]
    w = np.array([a + a, b + a, b + a, b + a, a + a], np.int8)
    xa = [1, 2, 3, 4, 5, 6, 7, 8, -9, -10] * 4
    xb = [1, 2, 3, 4, 5, 6, 7, -8, 9, -10] + [1, 2, 3, 4, 5, 6, 7, 8, -9, -10] * 3
    x = np.array([xa, xb, xa, [0] * 40], np.float32)
    packed = np.stack([kh.pack_int4(r) for r in w])
    op = fc.FullyConnectedHybridInt4PerChannel(packed, 40, [1.0], np.array([1, 2, 3, 1, 2], np.float32),
                                               "relu")
    y = op(_cuda(x)).cpu().numpy()
    want = np.array([[393., 456., 457., 455., 394.], [413., 476., 477., 475., 414.],
                     [393., 456., 457., 455., 394.]])
    assert np.abs(y[:3] - want).max() <= 1.3
    assert y[3].tolist() == [1, 2, 3, 1, 2]

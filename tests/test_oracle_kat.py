"""Pins the CPU oracle to every known-answer vector the reference's own tests hold
for the quantized FULLY_CONNECTED path, to the real reference leaf code where it
builds (oracle/_ref), and to exact rational arithmetic where neither reaches."""
import ctypes as C
from fractions import Fraction

import numpy as np
import pytest

import oracle
from tests import kat_harness as kh

INT32_MIN, INT32_MAX = -(2 ** 31), 2 ** 31 - 1


# ---- QuantizeMultiplier: tflite/kernels/internal/quantization_util_test.cc:358-423

@pytest.mark.parametrize("m,expect", [
    (0.25, (1073741824, -1)), (0.50 - 5e-9, (2147483627, -1)), (0.50 - 1e-10, (1073741824, 0)),
    (0.50, (1073741824, 0)), (0.75, (1610612736, 0)), (1 - 1e-9, (2147483646, 0)),
    (1 + 1e-11, (1073741824, 1)), (1.25, (1342177280, 1)), (1.50, (1610612736, 1)),
    (1.75, (1879048192, 1)), (2 - 1e-9, (2147483647, 1)), (2 - 1e-11, (1073741824, 2)),
    (2.0, (1073741824, 2)),
    (float(np.ldexp(np.float32(1.0), -31)), (1073741824, -30)),
    (float(np.ldexp(np.float32(1.0), -32)), (1073741824, -31)),
    (float(np.ldexp(np.float32(0.99), -32)), (0, 0)),
    (float(np.ldexp(np.float32(1.0), -33)), (0, 0)),
    (0.0, (0, 0)),
])
def test_quantize_multiplier_kat(m, expect):
    assert oracle.quantize_multiplier(m) == expect


def test_quantize_multiplier_matches_reference_build():
    R = oracle.ref_lib()
    if R is None:
        pytest.skip("oracle/_ref not built (reference tree absent)")
    rng = np.random.default_rng(7)
    ms = np.concatenate([np.exp(rng.uniform(np.log(1e-12), np.log(1e3), 20000)),
                         -np.exp(rng.uniform(np.log(1e-6), np.log(10), 2000)),
                         [0.5, 1.0, 2.0, 2 ** -31, 2 ** -32, 1 - 2 ** -33, 0.5 - 2 ** -34]])
    for m in ms:
        q, s = C.c_int32(), C.c_int()
        R.ref_quantize_multiplier(float(m), C.byref(q), C.byref(s))
        assert oracle.quantize_multiplier(float(m)) == (q.value, s.value), m


# ---- MultiplyByQuantizedMultiplier: quantization_util_test.cc:447-485

def _quant_and_multiply(x, m):
    q, s = oracle.quantize_multiplier(m)
    return oracle.mbqm(x, q, s)


@pytest.mark.parametrize("x,m,expect", [
    (0, 0.1, 0), (1, 0, 0), (10000, 0.00097656, 10), (-10000, 0.00097656, -10),
    (INT32_MIN, 0.00001, -21475), (INT32_MAX, 0.00001, 21475),
    (10000, -0.00097656, -10), (-10000, -0.00097656, 10),
    (INT32_MIN, -0.00001, 21475), (INT32_MAX, -0.00001, -21475),
])
def test_mbqm_kat(x, m, expect):
    assert _quant_and_multiply(x, m) == expect


def test_mbqm_kat_max_operands():
    x = m = INT32_MAX
    expect = int(kh._round_half_away(np.float64(x * m) / float(1 << 34)))
    assert oracle.mbqm(x, m, -3) == expect
    assert oracle.mbqm(-x, m, -3) == -expect


def _srdhm_exact(a, b):
    if a == b == INT32_MIN:
        return INT32_MAX
    # nearest; the nudge 1 - 2^30 for negative products sends exact halves upward
    return (Fraction(a * b, 2 ** 31) + Fraction(1, 2)).__floor__()


def _rdbp_exact(x, e):
    v = Fraction(x, 2 ** e)
    n = int(abs(v) + Fraction(1, 2))
    return n if v >= 0 else -n


def test_mbqm_against_exact_rationals():
    """The doubling high multiply is floor(ab / 2^31 + 1/2) and the power-of-two
    division is round-to-nearest, ties away from zero: checked with Python big
    rationals, which share no code with the C implementation (a wrong nudge sign,
    threshold or shift fails here)."""
    rng = np.random.default_rng(11)
    L = oracle.lib()
    xs = rng.integers(INT32_MIN, INT32_MAX, 4000, endpoint=True)
    ms = rng.integers(1 << 30, INT32_MAX, 4000, endpoint=True)
    shifts = rng.integers(-31, 3, 4000)
    for x, m, s in zip(xs.tolist(), ms.tolist(), shifts.tolist()):
        assert L.orc_srdhm(x, m) == _srdhm_exact(x, m)
        e = max(-s, 0)
        assert L.orc_rounding_divide_by_pot(x, e) == _rdbp_exact(x, e)
        if s <= 0:
            assert oracle.mbqm(x, m, s) == _rdbp_exact(_srdhm_exact(x, m), e)
    # ties: odd multiples of 2^(e-1)
    for e in range(1, 31):
        for k in (-5, -3, -1, 1, 3, 5):
            x = k * (1 << (e - 1))
            if INT32_MIN <= x <= INT32_MAX:
                assert L.orc_rounding_divide_by_pot(x, e) == _rdbp_exact(x, e)
    assert L.orc_srdhm(INT32_MIN, INT32_MIN) == INT32_MAX
    # exact halves of the high multiply: a * b = (2j + 1) * 2^30
    for j in (-7, -2, -1, 0, 1, 5):
        for a, b in (((2 * j + 1), 1 << 30), ((2 * j + 1) << 10, 1 << 20), (-(2 * j + 1), -(1 << 30))):
            assert L.orc_srdhm(a, b) == _srdhm_exact(a, b) == j + 1
    # accumulator-sized inputs with a left shift (multiplier > 1)
    for x in rng.integers(-(1 << 27), 1 << 27, 2000).tolist():
        for s in (1, 2, 3):
            m = int(rng.integers(1 << 30, INT32_MAX))
            assert oracle.mbqm(x, m, s) == _srdhm_exact(x << s, m)


def test_mbqm_single_rounding_closed_form():
    rng = np.random.default_rng(12)
    for _ in range(3000):
        x = int(rng.integers(-(1 << 28), 1 << 28))
        m = int(rng.integers(1 << 30, INT32_MAX))
        s = int(rng.integers(-20, 2))
        exact = Fraction(x * m, 2 ** (31 - s))
        # floor(v + 1/2): ties toward +inf (common.cc:33-47)
        expect = (exact + Fraction(1, 2)).__floor__()
        assert oracle.mbqm_single_rounding(x, m, s) == expect


# ---- activation range: kernel_util.cc:354-412

def test_activation_range():
    assert oracle.activation_range_int8(oracle.ACT_NONE, 0.05, 5) == (-128, 127)
    assert oracle.activation_range_int8(oracle.ACT_RELU, 1.0, -1) == (-1, 127)
    assert oracle.activation_range_int8(oracle.ACT_RELU6, 0.05, 5) == (5, 125)
    assert oracle.activation_range_int8(oracle.ACT_RELU6, 0.01, -128) == (-128, 127)
    assert oracle.activation_range_int8(oracle.ACT_RELU_N1_TO_1, 0.5, 0) == (-2, 2)
    assert oracle.activation_range_int8(oracle.ACT_RELU_N1_TO_1, 0.4, 3) == (0, 6)  # 2.5 -> 3 away


# ---- fp16: every bit pattern against numpy's IEEE conversion

def test_half_to_float_all_patterns():
    bits = np.arange(65536, dtype=np.uint16)
    got = oracle.half_to_float(bits)
    want = bits.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    # NaN payloads do not survive the float return through ctypes (signalling NaNs are
    # quietened on the way); every other pattern must match bit for bit.
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got.view(np.uint32)[~nan], want.view(np.uint32)[~nan])


# ---- int4 unpack: tflite/kernels/internal/tensor_utils_test.cc:2110-2129 + reference build

def test_unpack_int4_kat():
    packed = kh.pack_int4(np.array([1, 2, 3, -8, -1, 7, 0, -5, 4], np.int8))
    got = oracle.unpack_int4(packed.view(np.int8), 9)
    assert got.tolist() == [1, 2, 3, -8, -1, 7, 0, -5, 4]


def test_unpack_int4_matches_reference_build():
    R = oracle.ref_lib()
    if R is None:
        pytest.skip("oracle/_ref not built (reference tree absent)")
    rng = np.random.default_rng(3)
    for n in (1, 2, 7, 64, 1001):
        src = rng.integers(-128, 128, (n + 1) // 2).astype(np.int8)
        want = np.empty(n, np.int8)
        R.ref_unpack_int4(src.ctypes.data_as(C.POINTER(C.c_int8)), n,
                          want.ctypes.data_as(C.POINTER(C.c_int8)))
        assert np.array_equal(oracle.unpack_int4(src, n), want)


# ---- int2 unpack: tflite/kernels/internal/tensor_utils_test.cc:2131-2150 + reference build

def test_unpack_int2_kat():
    # UnpackInt2Basic: 0x6C = fields 0, 3, 2, 1 -> 0, -1, -2, 1; UnpackInt2OddLength: 0xD8, 3 values
    assert oracle.unpack_int2(np.array([0x6C], np.uint8).view(np.int8), 4).tolist() == [0, -1, -2, 1]
    assert oracle.unpack_int2(np.array([0xD8], np.uint8).view(np.int8), 3).tolist() == [0, -2, 1]
    values = np.array([1, -2, 0, -1, 1, 1, -2, 0, -1], np.int8)
    assert oracle.unpack_int2(kh.pack_int2(values).view(np.int8), 9).tolist() == values.tolist()


def test_unpack_int2_matches_reference_build():
    R = oracle.ref_lib()
    if R is None or not hasattr(R, "ref_unpack_int2"):
        pytest.skip("oracle/_ref not built (reference tree absent)")
    rng = np.random.default_rng(4)
    for n in (1, 2, 3, 4, 5, 7, 64, 1001, 1002, 1003):
        src = rng.integers(-128, 128, (n + 3) // 4).astype(np.int8)
        want = np.empty(n, np.int8)
        R.ref_unpack_int2(src.ctypes.data_as(C.POINTER(C.c_int8)), n,
                          want.ctypes.data_as(C.POINTER(C.c_int8)))
        assert np.array_equal(oracle.unpack_int2(src, n), want)


def test_relu_matches_reference_build():
    R = oracle.ref_lib()
    if R is None:
        pytest.skip("oracle/_ref not built (reference tree absent)")
    x = np.array([-7.5, -1.0, -0.25, -0.0, 0.0, 0.5, 1.0, 5.9, 6.0, 6.1, 1e30, -1e30], np.float32)
    fp = C.POINTER(C.c_float)
    for act, fn in ((oracle.ACT_RELU, R.ref_apply_relu), (oracle.ACT_RELU_N1_TO_1, R.ref_apply_relu1),
                    (oracle.ACT_RELU6, R.ref_apply_relu6)):
        want = np.empty_like(x)
        fn(x.ctypes.data_as(fp), x.size, want.ctypes.data_as(fp))
        got = x.copy()
        assert oracle.lib().orc_apply_activation(got.ctypes.data_as(fp), got.size, act) == 0
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


# ---- activation quantizers: tensor_utils_test.cc:220-345

KAT_IN_A = [-640, -635.0, -630, 10.0, 2.0, -5.0, -10.0, 0.0, 1000.0]
KAT_IN_SMALL = [-1e-5, 3e-5, -7e-6, -9e-5, 1e-6, 4e-5, 9e-6, 2e-4, 0]
VARIANTS = [oracle.QUANT_PORTABLE, oracle.QUANT_NEON_V8, oracle.QUANT_NEON_LEGACY]


@pytest.mark.parametrize("variant", VARIANTS)
def test_symmetric_quantize_kat(variant):
    x = np.array([KAT_IN_A], np.float32)
    q, sf, _ = oracle.batch_quantize_floats(x, asymmetric=False, variant=variant)
    assert q[0].tolist() == [-81, -81, -80, 1, 0, -1, -1, 0, 127]
    assert abs(sf[0] - 1000 / 127.0) < 1e-6 * 10
    q, sf, _ = oracle.batch_quantize_floats(np.zeros((1, 9), np.float32), False, variant)
    assert q[0].tolist() == [0] * 9 and sf[0] == 1
    q, sf, _ = oracle.batch_quantize_floats(np.array([KAT_IN_SMALL], np.float32), False, variant)
    assert q[0].tolist() == [-6, 19, -4, -57, 1, 25, 6, 127, 0]
    assert abs(sf[0] - 1.57e-6) < 1e-6


@pytest.mark.parametrize("variant", VARIANTS)
def test_asymmetric_quantize_kat(variant):
    q, sf, zp = oracle.batch_quantize_floats(np.array([KAT_IN_A], np.float32), True, variant)
    assert q[0].tolist() == [-128, -127, -126, -26, -28, -29, -30, -28, 127]
    assert zp[0] == -28 and abs(sf[0] - 1640 / 255.0) < 1e-6
    q, sf, zp = oracle.batch_quantize_floats(np.zeros((1, 9), np.float32), True, variant)
    assert q[0].tolist() == [0] * 9 and sf[0] == 1 and zp[0] == 0
    q, sf, zp = oracle.batch_quantize_floats(np.full((1, 9), 2000, np.float32), True, variant)
    assert q[0].tolist() == [127] * 9 and zp[0] == -128 and abs(sf[0] - 2000 / 255.0) < 1e-5
    q, sf, zp = oracle.batch_quantize_floats(np.array([KAT_IN_SMALL], np.float32), True, variant)
    assert q[0].tolist() == [-58, -23, -55, -128, -48, -14, -41, 127, -49]
    assert zp[0] == -49


def _asym_numpy(row):
    """Independent float64/float32 re-derivation of the portable asymmetric quantizer."""
    rmin = np.float64(min(np.float32(0), row.min()))
    rmax = np.float64(max(np.float32(0), row.max()))
    scale = (rmax - rmin) / 255.0
    zmin, zmax = -128.0 - rmin / scale, 127.0 - rmax / scale
    zp = zmin if (128.0 + abs(rmin / scale)) < (127.0 + abs(rmax / scale)) else zmax
    zp = -128 if zp <= -128 else 127 if zp >= 127 else int(kh._round_half_away(zp))
    sf = np.float32(scale)
    inv = np.float32(1.0) / sf
    t = (np.float32(zp) + row * inv).astype(np.float32)
    q = np.clip(kh._round_half_away(t), -128, 127).astype(np.int8)
    return q, sf, zp


def test_asymmetric_quantize_vs_numpy_rederivation():
    rng = np.random.default_rng(5)
    x = rng.standard_normal((6, 4096)).astype(np.float32)
    x[1] *= 1e-3
    x[2] = np.abs(x[2])          # rmin clamps to 0
    x[3] = -np.abs(x[3])         # rmax clamps to 0
    x[4, 17] = 250.0             # one outlier
    q, sf, zp = oracle.batch_quantize_floats(x, True)
    for b in range(x.shape[0]):
        wq, wsf, wzp = _asym_numpy(x[b])
        assert np.array_equal(q[b], wq) and sf[b] == wsf and zp[b] == wzp


def test_quantize_variants_differ_only_on_ties():
    """zp=-3, v*inv=2.5: portable rounds (-3+2.5)=-0.5 -> -1; the NEON forms round
    2.5 -> 3 first, giving 0."""
    # rmin=-125*s, rmax=130*s with s=1 -> scale 1, zero point -3
    row = np.array([-125.0, 130.0, 2.5, 0.0, 0, 0, 0, 0], np.float32)
    qp, _, zpp = oracle.batch_quantize_floats(row[None], True, oracle.QUANT_PORTABLE)
    qn, _, zpn = oracle.batch_quantize_floats(row[None], True, oracle.QUANT_NEON_V8)
    ql, _, _ = oracle.batch_quantize_floats(row[None], True, oracle.QUANT_NEON_LEGACY)
    assert zpp[0] == zpn[0] == -3
    assert qp[0, 2] == -1 and qn[0, 2] == 0 and ql[0, 2] == 0
    assert np.array_equal(np.delete(qp[0], 2), np.delete(qn[0], 2))


# ---- hybrid dot: tensor_utils_test.cc:1064-1231 (exact, integer-valued floats)

def _mv_data(rows, cols, batch, negative=False, per_channel=False, init_to_one=False):
    i = np.arange(rows * cols)
    sign = np.where((i % 3 == 0) & negative, -1, 1)
    matrix = (sign * (i % 70)).astype(np.int8).reshape(rows, cols)
    j = np.arange(cols * batch)
    sign = np.where((j % 5 == 0) & negative, -1, 1)
    vectors = (sign * (j % 50)).astype(np.int32).reshape(batch, cols)
    scale_factors = np.tile(np.arange(1, 9, dtype=np.float32), batch)[:max(batch, 8)]
    results = np.full((batch, rows), 1.0 if init_to_one else 0.0, np.float32)
    pcs = offs = None
    if per_channel:
        pcs = np.where(np.arange(rows) % 2 == 0, 0.5, 1.0).astype(np.float32)
        vectors = vectors + np.arange(batch)[:, None]
        offs = np.arange(batch, dtype=np.int32)
    return matrix, vectors.astype(np.int8), scale_factors, results, pcs, offs


DOT_KERNELS = {"portable": oracle.matrix_batch_vector_multiply_accumulate,
               "sse": oracle.matrix_batch_vector_multiply_accumulate_sse}
_dot_kernel = "portable"


@pytest.fixture(params=sorted(DOT_KERNELS))
def dot_kernel(request):
    """The reference runs these vectors against every build of the kernel (portable, NEON, SSE:
    tensor_utils_test.cc is linked against each); so do the two tiers restated here."""
    global _dot_kernel
    if request.param == "sse" and not oracle.have_sse():
        pytest.skip("not an x86 host")
    _dot_kernel = request.param
    yield request.param
    _dot_kernel = "portable"


def _dot(rows, cols, batch, negative=False, init_to_one=False, per_channel=False):
    m, v, sf, res, pcs, offs = _mv_data(rows, cols, batch, negative, per_channel, init_to_one)
    return DOT_KERNELS[_dot_kernel](m, v, sf, res, pcs, offs).ravel()


def test_sse_dot_is_bit_identical_to_portable():
    """The optimized-x86 tier of the CPU baseline (oracle_sse.cc) against the portable kernel on
    ragged depths (vector body, 16-byte step, scalar tail), with and without input offsets,
    activations over the whole int8 range, weights over [-127, 127] (the range symmetric weight
    quantization produces; at -128 the kernel's sign transfer wraps, in the reference too)."""
    if not oracle.have_sse():
        pytest.skip("not an x86 host")
    rng = np.random.default_rng(12)
    for rows, cols, batch in ((3, 1, 1), (5, 15, 2), (4, 16, 1), (7, 31, 3), (2, 33, 1), (9, 100, 2),
                              (6, 4096, 2)):
        m = rng.integers(-127, 128, (rows, cols)).astype(np.int8)
        v = rng.integers(-128, 128, (batch, cols)).astype(np.int8)
        sf = rng.uniform(0.01, 0.1, batch).astype(np.float32)
        pcs = rng.uniform(1e-3, 1e-2, rows).astype(np.float32)
        res = rng.standard_normal((batch, rows)).astype(np.float32)
        offsets = rng.integers(-128, 128, batch).astype(np.int32)
        # the portable kernel's short form (no offsets) has no per-channel scale, so that
        # pairing is not a call the op makes
        for use_pcs, offs in ((None, None), (None, offsets), (pcs, offsets)):
            a = oracle.matrix_batch_vector_multiply_accumulate(m, v, sf, res, use_pcs, offs)
            b = oracle.matrix_batch_vector_multiply_accumulate_sse(m, v, sf, res, use_pcs, offs)
            assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), (rows, cols, batch)
    x = rng.standard_normal((3, 200)).astype(np.float32)
    w = rng.integers(-127, 128, (11, 200)).astype(np.int8)
    pcs = rng.uniform(1e-3, 1e-2, 11).astype(np.float32)
    for asym in (True, False):
        assert np.array_equal(oracle.fc_hybrid(x, w, pcs, asymmetric=asym).view(np.uint32),
                              oracle.fc_hybrid_sse(x, w, pcs, None, asymmetric=asym).view(np.uint32))


def test_hybrid_dot_kat(dot_kernel):
    assert _dot(4, 16, 1).tolist() == [1240, 3160, 5080, 7000]
    assert _dot(4, 32, 2).tolist() == [10416, 26288, 8490, 23312, 18276, 70756, 37416, 60916]
    r = _dot(32, 512, 5)
    for idx, want in ((0, 415566), (50, 880736), (72, 1312062), (100, 1750384), (120, 1776224),
                      (150, 2101860)):
        assert r[idx] == want
    assert _dot(4, 64, 1, True).tolist() == [13696, 6904, 7764, 11806]
    assert _dot(4, 32, 2, True).tolist() == [3436, 3522, 1590, 6972, 2516, 20520, 456, 10628]
    assert _dot(4, 32, 2, True, True).tolist() == [3437, 3523, 1591, 6973, 2517, 20521, 457, 10629]


def test_hybrid_dot_per_channel_kat(dot_kernel):
    assert _dot(4, 16, 1, per_channel=True).tolist() == [620, 3160, 2540, 7000]
    assert _dot(4, 32, 2, per_channel=True).tolist() == [5208, 26288, 4245, 23312, 9138, 70756,
                                                         18708, 60916]
    r = _dot(32, 512, 5, per_channel=True)
    for idx, want in ((0, 207783), (13, 411552), (39, 835936), (50, 440368), (100, 875192),
                      (123, 1775536), (150, 1050930)):
        assert r[idx] == want


# ---- int8 FC end to end: tflite/kernels/fully_connected_test.cc

W10 = [1, 2, 3, 4, 5, 6, 7, 8, 9, 10]
X2 = [1, 2, 3, 4, 5, 6, 7, 8, -9, -10, 1, 2, 3, 4, 5, 6, 7, -8, 9, -10]


def _per_tensor_case(in_range, out_range, weights, bias, x, units, filter_range=(-63.5, 64),
                     act=oracle.ACT_NONE, int4=False):
    in_s, in_zp = kh.quantization_params(*in_range)
    out_s, out_zp = kh.quantization_params(*out_range)
    if int4:
        w_s, w_zp = kh.quantization_params(-7.0, 7.0, -7, 7)
        wq = kh.quantize(weights, w_s, w_zp, -7, 7).reshape(units, -1)
        wq = oracle.unpack_int4(kh.pack_int4(wq).view(np.int8), wq.size).reshape(units, -1)
    else:
        w_s, w_zp = kh.quantization_params(*filter_range)
        wq = kh.quantize(weights, w_s, w_zp).reshape(units, -1)
    xq = kh.quantize(x, in_s, in_zp).reshape(-1, wq.shape[1])
    bias_scale = np.float32(in_s * w_s)
    bq = None if bias is None else kh.quantize_bias(bias, bias_scale)
    m, s = oracle.fc_prepare_per_tensor(float(in_s), float(w_s), float(out_s),
                                        None if bias is None else float(bias_scale))
    lo, hi = oracle.activation_range_int8(act, float(out_s), out_zp)
    y = oracle.fc_int8_per_tensor(xq, wq, bq, m, s, -in_zp, -w_zp, out_zp, lo, hi)
    yf = oracle.fc_int8_per_tensor_float_scale(xq, wq, bq, float(in_s), float(w_s), float(out_s),
                                               -in_zp, -w_zp, out_zp, lo, hi)
    return y.ravel().tolist(), yf.ravel().tolist()


def test_fc_int8_per_tensor_kats():
    # :816-840 SimpleTestQuantizedInt8
    y, yf = _per_tensor_case((-63.5, 64), (-127, 128), W10 * 3, [1, 2, 3], X2, 3)
    assert y == yf == [23, 24, 25, 57, 58, 59]
    # :1319-1347 no bias, fused RELU
    y, yf = _per_tensor_case((-63.5, 64), (-127, 128), W10 * 3, None, X2, 3, act=oracle.ACT_RELU)
    assert y == yf == [22, 22, 22, 56, 56, 56]
    # :1463-1487 GEMV, batch 1
    y, yf = _per_tensor_case((-63.5, 64), (-127, 128), W10 * 4, [1, 2, 3, 4], X2[10:], 4)
    assert y == yf == [57, 58, 59, 60]
    # :1530-1562 real multiplier 2
    y, yf = _per_tensor_case((-127, 128), (-63.5, 64), W10 * 3, [1, 2, 3], X2, 3)
    assert y == yf == [47, 49, 51, 115, 117, 119]
    # :756-782 int4 weights, RELU
    w4 = [1, 2, 3, 4, 5, 6, 7, 6, 5, 4] * 3
    y, yf = _per_tensor_case((-63.5, 64), (-127, 128), w4, [1, 2, 3], X2, 3, act=oracle.ACT_RELU,
                             int4=True)
    assert y == yf == [103, 104, 105, 97, 98, 99]


def _per_channel_case(in_range, out_range, scales, weights, bias, x, units, depth,
                      act=oracle.ACT_NONE, int4=False):
    in_s, in_zp = kh.quantization_params(*in_range)
    out_s, out_zp = kh.quantization_params(*out_range)
    scales = np.asarray(scales, np.float32)
    w = np.asarray(weights, np.float32).reshape(units, depth)
    inv = (np.float32(1.0) / scales).astype(np.float32)
    lim = 7 if int4 else 127
    wq = np.clip(kh._round_half_away(w * inv[:, None]), -lim, lim).astype(np.int8)
    if int4:
        wq = oracle.unpack_int4(kh.pack_int4(wq).view(np.int8), wq.size).reshape(units, depth)
    xq = kh.quantize(x, in_s, in_zp).reshape(-1, depth)
    bq = None
    if bias is not None:
        bscale = (scales * in_s).astype(np.float32)
        bq = kh._round_half_away(np.asarray(bias, np.float32) / bscale).astype(np.int32)
    mult, shift = oracle.fc_prepare_per_channel(float(in_s), scales, float(out_s))
    lo, hi = oracle.activation_range_int8(act, float(out_s), out_zp)
    y = oracle.fc_int8_per_channel(xq, wq, bq, mult, shift, -in_zp, out_zp, lo, hi)
    yf = oracle.fc_int8_per_channel_float_scale(xq, wq, bq, scales, float(in_s), float(out_s),
                                                -in_zp, out_zp, lo, hi)
    ys = oracle.fc_int8_per_channel(xq, wq, bq, mult, shift, -in_zp, out_zp, lo, hi,
                                    single_rounding=True)
    return y.ravel().tolist(), yf.ravel().tolist(), ys.ravel().tolist()


def test_fc_int8_per_channel_kats():
    # :863-888
    y, yf, ys = _per_channel_case((-63.5, 64), (-127, 128), [0.2, 0.25, 0.5], W10 * 3, [1, 2, 3],
                                  X2, 3, 10)
    assert y == yf == ys == [23, 24, 25, 57, 58, 59]
    # :890-948 3-D input, keep_num_dims, RELU
    x3 = [1, 2, 3, 4, -5, 1, 2, 3, -4, 5, 1, 2, -3, 4, 5, 1, -2, 3, 4, 5]
    y, yf, ys = _per_channel_case((-63.5, 64), (-127, 128), [0.2, 0.25, 0.5], [1, 2, 3, 4, 5] * 3,
                                  [1, 2, 3], x3, 3, 5, act=oracle.ACT_RELU)
    assert y == yf == ys == [5, 6, 7, 23, 24, 25, 37, 38, 39, 47, 48, 49]
    # :950-976 int4 per-channel
    w4 = [1, 2, 3, 4, 5, 6, 7, 6, 5, 4] * 3
    y, yf, ys = _per_channel_case((-63.5, 64), (-127, 128), [1.0, 1.0, 1.0], w4, [1, 2, 3], X2, 3,
                                  10, act=oracle.ACT_RELU, int4=True)
    assert y == yf == ys == [103, 104, 105, 97, 98, 99]


def test_fc_int8_brute_force_and_invariants():
    """Tiny shapes against a numpy int64 evaluation of the definition, plus the
    zero-point identity sum w*(x+off) == sum w*x + off*sum w that the HIP path uses."""
    rng = np.random.default_rng(21)
    for B, K, N in ((1, 1, 1), (2, 7, 3), (3, 33, 5), (4, 130, 9)):
        x = rng.integers(-128, 128, (B, K)).astype(np.int8)
        w = rng.integers(-127, 128, (N, K)).astype(np.int8)
        bias = rng.integers(-2 ** 14, 2 ** 14, N).astype(np.int32)
        ws = np.exp(rng.uniform(np.log(1e-3), np.log(1e-2), N)).astype(np.float32)
        mult, shift = oracle.fc_prepare_per_channel(0.02, ws, 0.05)
        off = 3
        y = oracle.fc_int8_per_channel(x, w, bias, mult, shift, off, 5, -128, 127)
        acc = w.astype(np.int64) @ (x.astype(np.int64) + off).T  # [N,B]
        acc2 = w.astype(np.int64) @ x.astype(np.int64).T + off * w.astype(np.int64).sum(1)[:, None]
        assert np.array_equal(acc, acc2)
        acc = acc + bias[:, None]
        want = np.empty((B, N), np.int64)
        for n in range(N):
            for b in range(B):
                want[b, n] = oracle.mbqm(int(acc[n, b]), int(mult[n]), int(shift[n])) + 5
        assert np.array_equal(y, np.clip(want, -128, 127).astype(np.int8))
        # clamp idempotence under a tighter activation range
        y6 = oracle.fc_int8_per_channel(x, w, bias, mult, shift, off, 5, 5, 125)
        assert np.array_equal(y6, np.clip(y, 5, 125))


# ---- hybrid FC end to end (loose goldens): fully_connected_test.cc:1728-1758

def test_fc_hybrid_kat_loose():
    w = np.array(W10 * 3, np.float32).reshape(3, 10)
    # SymmetricQuantizeAndPopulate: per-tensor symmetric int8, scale = max|w| / 127
    w_scale = np.float32(10.0 / 127.0)
    wq = np.clip(kh._round_half_away(w / w_scale), -127, 127).astype(np.int8)
    x = np.array(X2, np.float32).reshape(2, 10)
    bias = np.array([1, 2, 3], np.float32)
    for asym in (False, True):
        y = oracle.fc_hybrid(x, wq, None, float(w_scale), bias, asymmetric=asym)
        assert np.allclose(y.ravel(), [24, 25, 26, 58, 59, 60], atol=1.3)

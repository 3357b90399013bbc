"""Replays tests/golden/reference_kats.json -- the known-answer vectors of the reference's own
tests, stored as data -- against the CPU oracle (no GPU needed) and against the HIP path through
the C ABI (gpu). Integer results must be equal; scales are compared as the reference's tests do."""
import json
import os

import numpy as np
import pytest

import oracle

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "reference_kats.json")) as f:
    KATS = json.load(f)


def _fc_ids():
    return [c["source"].split(":", 1)[1] for c in KATS["fully_connected_int8"]]


def _filter_int8(case):
    w = np.array(case["filter"], np.int8)
    if case["int4"]:  # stored two per byte in the model; what the kernels see after unpacking
        from tests import kat_harness as kh
        w = oracle.unpack_int4(kh.pack_int4(w).view(np.int8), w.size).reshape(w.shape)
    if case.get("int2"):  # four per byte
        from tests import kat_harness as kh
        w = oracle.unpack_int2(kh.pack_int2(w).view(np.int8), w.size).reshape(w.shape)
    return w


# ---- oracle (CPU) ----------------------------------------------------------------------------

@pytest.mark.parametrize("case", KATS["quantize_multiplier"], ids=lambda c: repr(c["real"]))
def test_oracle_quantize_multiplier(case):
    assert oracle.quantize_multiplier(case["real"]) == (case["quantized"], case["shift"])


@pytest.mark.parametrize("case", KATS["multiply_by_quantized_multiplier"],
                         ids=lambda c: "%d*%g" % (c["x"], c["real_multiplier"]))
def test_oracle_multiply_by_quantized_multiplier(case):
    q, s = oracle.quantize_multiplier(case["real_multiplier"])
    assert oracle.mbqm(case["x"], q, s) == case["expected"]


@pytest.mark.parametrize("case", KATS["batch_quantize_floats"], ids=lambda c: c["source"][-7:])
@pytest.mark.parametrize("variant", [oracle.QUANT_PORTABLE, oracle.QUANT_NEON_V8,
                                     oracle.QUANT_NEON_LEGACY])
def test_oracle_batch_quantize_floats(case, variant):
    x = np.array([case["values"]], np.float32)
    q, sf, zp = oracle.batch_quantize_floats(x, case["asymmetric"], variant)
    assert q[0].tolist() == case["expected"]
    if "expected_scale" in case:
        assert sf[0] == case["expected_scale"]
    if "expected_zero_point" in case:
        assert zp[0] == case["expected_zero_point"]


@pytest.mark.parametrize("case", KATS["unpack_int4"], ids=lambda c: str(c["count"]))
def test_oracle_unpack_int4(case):
    got = oracle.unpack_int4(np.array(case["packed"], np.uint8).view(np.int8), case["count"])
    assert got.tolist() == case["expected"]


@pytest.mark.parametrize("case", KATS["unpack_int2"], ids=lambda c: str(c["count"]))
def test_oracle_unpack_int2(case):
    got = oracle.unpack_int2(np.array(case["packed"], np.uint8).view(np.int8), case["count"])
    assert got.tolist() == case["expected"]


@pytest.mark.parametrize("case", KATS["hybrid_dot_per_channel"], ids=lambda c: str(len(c["expected"])))
def test_oracle_hybrid_dot(case):
    m = np.array(case["matrix"], np.int8)
    v = np.array(case["vectors"], np.int8)
    res = np.zeros((v.shape[0], m.shape[0]), np.float32)
    got = oracle.matrix_batch_vector_multiply_accumulate(
        m, v, np.array(case["scaling_factors"], np.float32), res,
        np.array(case["per_channel_scales"], np.float32), np.array(case["input_offsets"], np.int32))
    assert got.ravel().tolist() == case["expected"]


def _oracle_fc(case):
    x = np.array(case["input"], np.int8)
    w = _filter_int8(case)
    bias = None if case["bias"] is None else np.array(case["bias"], np.int32)
    lo, hi = oracle.activation_range_int8(case["activation"], case["output_scale"],
                                          case["output_zero_point"])
    if case["per_channel"]:
        mult, shift = oracle.fc_prepare_per_channel(case["input_scale"],
                                                    np.array(case["filter_scales"], np.float32),
                                                    case["output_scale"])
        return oracle.fc_int8_per_channel(x, w, bias, mult, shift, -case["input_zero_point"],
                                          case["output_zero_point"], lo, hi)
    m, s = oracle.fc_prepare_per_tensor(case["input_scale"], case["filter_scales"][0],
                                        case["output_scale"], case["bias_scale"])
    return oracle.fc_int8_per_tensor(x, w, bias, m, s, -case["input_zero_point"],
                                     -case["filter_zero_point"], case["output_zero_point"], lo, hi)


@pytest.mark.parametrize("case", KATS["fully_connected_int8"], ids=_fc_ids())
def test_oracle_fully_connected_int8(case):
    assert _oracle_fc(case).ravel().tolist() == case["expected_output"]


def _uint8_case(case):
    x = np.array(case["input"], np.uint8)
    w = np.array(case["filter"], np.uint8)
    bias = None if case["bias"] is None else np.array(case["bias"], np.int32)
    return x, w, bias


@pytest.mark.parametrize("case", KATS["fully_connected_uint8"],
                         ids=lambda c: c["source"].split(":", 1)[1])
def test_oracle_fully_connected_uint8(case):
    """The legacy uint8 op's vectors (the same for every kernel type the reference's test is
    instantiated with), and the change of representation the HIP path rests on: the int8 oracle on
    the tensors taken as value - 128, every zero point lowered by 128, gives the same bytes + 128."""
    x, w, bias = _uint8_case(case)
    m, s = oracle.fc_prepare_per_tensor(case["input_scale"], case["filter_scale"],
                                        case["output_scale"], case["bias_scale"])
    lo, hi = oracle.activation_range_uint8(case["activation"], case["output_scale"],
                                           case["output_zero_point"])
    got = oracle.fc_uint8_per_tensor(x, w, bias, m, s, -case["input_zero_point"],
                                     -case["filter_zero_point"], case["output_zero_point"], lo, hi)
    assert got.ravel().tolist() == case["expected_output"]
    lo8, hi8 = oracle.activation_range_int8(case["activation"], case["output_scale"],
                                            case["output_zero_point"] - 128)
    assert (lo8, hi8) == (lo - 128, hi - 128)
    moved = oracle.fc_int8_per_tensor((x ^ 0x80).view(np.int8), (w ^ 0x80).view(np.int8), bias, m, s,
                                      -(case["input_zero_point"] - 128),
                                      -(case["filter_zero_point"] - 128),
                                      case["output_zero_point"] - 128, lo8, hi8)
    assert np.array_equal(moved.view(np.uint8) ^ 0x80, got)


@pytest.mark.parametrize("seed", range(6))
def test_oracle_uint8_equals_int8_on_moved_tensors(seed):
    """The same identity on random tensors, zero points and activations (clamps that bite)."""
    rng = np.random.default_rng(seed)
    B, K, N = int(rng.integers(1, 5)), int(rng.integers(1, 70)), int(rng.integers(1, 9))
    x = rng.integers(0, 256, (B, K)).astype(np.uint8)
    w = rng.integers(0, 256, (N, K)).astype(np.uint8)
    bias = rng.integers(-2000, 2000, N).astype(np.int32)
    zx, zw, zy = (int(v) for v in rng.integers(0, 256, 3))
    in_s, w_s, out_s = 0.02, 0.01, float(rng.uniform(0.05, 0.5))
    m, s = oracle.fc_prepare_per_tensor(in_s, w_s, out_s, None)
    act = int(rng.integers(0, 4))
    lo, hi = oracle.activation_range_uint8(act, out_s, zy)
    lo8, hi8 = oracle.activation_range_int8(act, out_s, zy - 128)
    assert (lo8, hi8) == (lo - 128, hi - 128)
    got = oracle.fc_uint8_per_tensor(x, w, bias, m, s, -zx, -zw, zy, lo, hi)
    moved = oracle.fc_int8_per_tensor((x ^ 0x80).view(np.int8), (w ^ 0x80).view(np.int8), bias, m, s,
                                      -(zx - 128), -(zw - 128), zy - 128, lo8, hi8)
    assert np.array_equal(moved.view(np.uint8) ^ 0x80, got)


# ---- HIP path through the C ABI (gpu) ----------------------------------------------------------

@pytest.fixture(scope="module")
def fc():
    torch = pytest.importorskip("torch")
    if not torch.cuda.is_available():
        pytest.fail("GPU tests need a gfx950 device; none visible")
    from litert_amd import fully_connected
    return fully_connected


def _cuda(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.gpu
@pytest.mark.parametrize("case", KATS["fully_connected_int8"], ids=_fc_ids())
@pytest.mark.parametrize("packed", [True, False])
def test_hip_fully_connected_int8(fc, case, packed):
    w = _filter_int8(case)
    scales = case["filter_scales"] if case["per_channel"] else [case["filter_scales"][0]]
    op = fc.FullyConnectedInt8(
        w, None if case["bias"] is None else np.array(case["bias"], np.int32),
        case["input_scale"], case["input_zero_point"], np.array(scales, np.float32),
        case["output_scale"], case["output_zero_point"], activation=case["activation"],
        filter_zero_point=case["filter_zero_point"], bias_scale=case["bias_scale"], packed=packed)
    y = op(_cuda(np.array(case["input"], np.int8))).cpu().numpy()
    assert y.ravel().tolist() == case["expected_output"]


@pytest.mark.gpu
@pytest.mark.parametrize("case", KATS["fully_connected_uint8"],
                         ids=lambda c: c["source"].split(":", 1)[1])
@pytest.mark.parametrize("packed", [True, False])
def test_hip_fully_connected_uint8(fc, case, packed):
    x, w, bias = _uint8_case(case)
    op = fc.FullyConnectedUInt8(w, bias, case["input_scale"], case["input_zero_point"],
                                case["filter_scale"], case["filter_zero_point"],
                                case["output_scale"], case["output_zero_point"],
                                activation=case["activation"], bias_scale=case["bias_scale"],
                                packed=packed)
    y = op(_cuda(x)).cpu().numpy()
    assert y.dtype == np.uint8 and y.ravel().tolist() == case["expected_output"]


@pytest.mark.gpu
@pytest.mark.parametrize("B,K,N,zw", [(1, 64, 40, 128), (4, 1000, 33, 128), (3, 272, 130, 121),
                                     (40, 512, 72, 128), (130, 96, 300, 7), (2, 17, 5, 255)])
@pytest.mark.parametrize("activation", [0, 1, 3])
def test_hip_uint8_shapes_match_oracle(fc, B, K, N, zw, activation):
    """Filter zero point 128 (0 once moved: the re-tiled filter, GEMV and GEMM) and other values
    (the row-major kernels), input and output zero points at both ends of the range where the
    filter is centred."""
    rng = np.random.default_rng(B + K + N + zw)
    x = rng.integers(0, 256, (B, K)).astype(np.uint8)
    w = rng.integers(0, 256, (N, K)).astype(np.uint8)
    bias = rng.integers(-5000, 5000, N).astype(np.int32)
    # one of the two factors stays centred, or every sum lands beyond a clamp
    zx, zy = (127, 130) if zw != 128 else ((0, 255) if (B + N) % 2 else (250, 3))
    in_s, w_s = 0.02, 0.01
    out_s = float(0.02 * 0.01 * np.sqrt(K) * 60)
    op = fc.FullyConnectedUInt8(w, bias, in_s, zx, w_s, zw, out_s, zy, activation=activation)
    y = op(_cuda(x)).cpu().numpy()
    m, s = oracle.fc_prepare_per_tensor(in_s, w_s, out_s, None)
    lo, hi = oracle.activation_range_uint8(activation, out_s, zy)
    want = oracle.fc_uint8_per_tensor(x, w, bias, m, s, -zx, -zw, zy, lo, hi)
    assert np.array_equal(y, want)
    if activation == 0:  # (a ReLU under an output zero point of 255 leaves one value: 255)
        assert len(np.unique(want)) > 3


@pytest.mark.gpu
@pytest.mark.parametrize("case", [c for c in KATS["fully_connected_int8"] if c.get("int2")],
                         ids=lambda c: c["source"].split(":", 1)[1])
def test_hip_fully_connected_int2_filter_unpacked_on_the_device(fc, case):
    """The two Int2 cases with the filter handed over as the model holds it (four values per
    byte) and unpacked by lrtfc_unpack_int2."""
    from tests import kat_harness as kh
    w = np.array(case["filter"], np.int8)
    scales = case["filter_scales"] if case["per_channel"] else [case["filter_scales"][0]]
    op = fc.FullyConnectedInt8(
        kh.pack_int2(w), np.array(case["bias"], np.int32), case["input_scale"],
        case["input_zero_point"], np.array(scales, np.float32), case["output_scale"],
        case["output_zero_point"], activation=case["activation"],
        filter_zero_point=case["filter_zero_point"], bias_scale=case["bias_scale"], int2=True,
        depth=w.shape[1], out_depth=w.shape[0])
    y = op(_cuda(np.array(case["input"], np.int8))).cpu().numpy()
    assert y.ravel().tolist() == case["expected_output"]


@pytest.mark.gpu
@pytest.mark.parametrize("count", [1, 2, 3, 4, 5, 7, 64, 1001, 1002, 1003, 70000])
def test_hip_unpack_int2_matches_oracle(fc, count):
    import torch
    from litert_amd import capi
    rng = np.random.default_rng(count)
    packed = rng.integers(0, 256, (count + 3) // 4).astype(np.uint8)
    src = _cuda(packed)
    dst = torch.full((count + 8,), 99, dtype=torch.int8, device="cuda")
    capi.check(capi.load().lrtfc_unpack_int2(src.data_ptr(), count, dst.data_ptr(), None))
    got = dst.cpu().numpy()
    assert np.array_equal(got[:count], oracle.unpack_int2(packed.view(np.int8), count))
    assert (got[count:] == 99).all()  # nothing written past the last element
    for case in KATS["unpack_int2"]:
        src = _cuda(np.array(case["packed"], np.uint8))
        dst = torch.empty(case["count"], dtype=torch.int8, device="cuda")
        capi.check(capi.load().lrtfc_unpack_int2(src.data_ptr(), case["count"], dst.data_ptr(), None))
        assert dst.cpu().numpy().tolist() == case["expected"]


@pytest.mark.gpu
@pytest.mark.parametrize("case", KATS["batch_quantize_floats"], ids=lambda c: c["source"][-7:])
@pytest.mark.parametrize("variant", [0, 1, 2])
def test_hip_batch_quantize_floats(fc, case, variant):
    q, sf, zp = fc.batch_quantize_floats(_cuda(np.array([case["values"]], np.float32)),
                                         case["asymmetric"], variant)
    assert q.cpu().numpy()[0].tolist() == case["expected"]
    if "expected_scale" in case:
        assert sf.item() == case["expected_scale"]
    if "expected_zero_point" in case:
        assert zp.item() == case["expected_zero_point"]


@pytest.mark.gpu
@pytest.mark.parametrize("case", KATS["quantize_multiplier"], ids=lambda c: repr(c["real"]))
def test_capi_quantize_multiplier(fc, case):
    assert fc.quantize_multiplier(case["real"]) == (case["quantized"], case["shift"])

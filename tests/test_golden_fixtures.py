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

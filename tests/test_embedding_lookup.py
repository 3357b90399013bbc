"""EMBEDDING_LOOKUP from quantized tables (tflite/kernels/embedding_lookup.cc:140-159, 194-395).

CPU part: the oracle against the reference's own known-answer vectors
(tests/golden/reference_kats.json, from embedding_lookup_test.cc), against what the arithmetic
fixes (moving a nibble to the top of a byte and dividing the scale by 16 are both exact, so
every output must be THE correctly rounded product value x scale), and its float -> binary16
conversion against numpy's. GPU part: the HIP path through the C-ABI, bit-identical to the
oracle on the vectors, on seeded shapes of both kernel forms, and at the size of a real
vocabulary."""
import json
import os

import numpy as np
import pytest

import oracle

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "reference_kats.json")) as f:
    KATS = json.load(f)["embedding_lookup"]


def _ids(cases):
    return [c["source"].rsplit(":", 1)[1] + ("-f16" if c["out_f16"] else "") for c in cases]


def _oracle_case(c):
    table = np.asarray(c["table"], np.uint8 if c["value_bits"] == 4 else np.int8)
    if c["kind"] == "blockwise":
        return oracle.embedding_lookup_blockwise_int4(
            c["lookup"], table, c["rows"], c["cols"], np.asarray(c["scales_f16_bits"], np.uint16),
            c["blocksize"], c["out_f16"])
    return oracle.embedding_lookup_hybrid(c["lookup"], table, c["value_bits"], c["rows"], c["cols"],
                                          row_scales=c["row_scales"], out_f16=c["out_f16"])


def _as_float(y):
    return y.view(np.float16).astype(np.float32) if y.dtype == np.uint16 else y


@pytest.mark.parametrize("case", KATS, ids=_ids(KATS))
def test_oracle_against_reference_vectors(case):
    got = _as_float(_oracle_case(case)).ravel()
    assert np.abs(got - np.asarray(case["expected"], np.float32)).max() <= case["tolerance"]


def _unpack(table_u8, count):
    out = np.empty(table_u8.size * 2, np.int8)
    out[0::2] = (table_u8.astype(np.int8) << 4) >> 4
    out[1::2] = table_u8.astype(np.int8) >> 4
    return out[:count]


def _random_blockwise(rng, rows, cols, bs, full_range=True):
    table = rng.integers(0, 256, (rows, cols // 2), dtype=np.uint8)
    scales = (rng.random((rows, cols // bs), dtype=np.float32) * 0.05 + 1e-3).astype(np.float16)
    if full_range:  # subnormal, tiny and large block scales
        flat = scales.reshape(-1)
        flat[:: 7] = np.float16(6e-8)
        flat[3:: 11] = np.float16(3.1e-5)
        flat[5:: 13] = np.float16(900.0)
    return table, scales.view(np.uint16)


def test_oracle_is_the_correctly_rounded_product():
    rng = np.random.default_rng(11)
    rows, cols, bs = 37, 96, 16
    table, sbits = _random_blockwise(rng, rows, cols, bs)
    lookup = rng.integers(0, rows, 50).astype(np.int32)
    got = oracle.embedding_lookup_blockwise_int4(lookup, table, rows, cols, sbits, bs)
    values = _unpack(table.ravel(), rows * cols).reshape(rows, cols).astype(np.float64)
    scales = np.repeat(sbits.view(np.float16).astype(np.float64), bs, axis=1)
    want = (values * scales)[lookup].astype(np.float32)  # exact in double, rounded once
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # binary16 output: the same product rounded to float32 and then to binary16
    got16 = oracle.embedding_lookup_blockwise_int4(lookup, table, rows, cols, sbits, bs, out_f16=True)
    with np.errstate(over="ignore"):
        assert np.array_equal(got16, want.astype(np.float16).view(np.uint16))
    # per-row and per-table scales, Int8 and Int4
    rs = (rng.random(rows, dtype=np.float32) * 0.1 + 1e-4).astype(np.float32)
    t8 = rng.integers(-128, 128, (rows, cols), dtype=np.int8)
    got = oracle.embedding_lookup_hybrid(lookup, t8, 8, rows, cols, row_scales=rs)
    want = (t8.astype(np.float64) * rs.astype(np.float64)[:, None])[lookup].astype(np.float32)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    got = oracle.embedding_lookup_hybrid(lookup, table, 4, rows, cols, scale=0.0371)
    want = (values * float(np.float32(0.0371)))[lookup].astype(np.float32)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_oracle_float_to_half_is_round_to_nearest_even():
    rng = np.random.default_rng(0)
    v = (rng.standard_normal(20000) * 10.0 ** rng.integers(-9, 6, 20000)).astype(np.float32)
    halves = np.arange(0, 0x7C00, dtype=np.uint16).view(np.float16).astype(np.float32)
    mid = ((halves[:-1].astype(np.float64) + halves[1:].astype(np.float64)) / 2).astype(np.float32)
    edge = np.array([0.0, -0.0, 65504, 65519.99, 65520, 65536, 1e9, -1e9, np.inf, -np.inf,
                     2.9802322e-8, 2.9802326e-8, 1e-10], np.float32)
    v = np.concatenate([v, edge, mid[::9], -mid[::9], halves[::9],
                        np.nextafter(mid[::9], np.float32(0)), np.nextafter(mid[::9], np.float32(1e9))])
    with np.errstate(over="ignore"):
        want = v.astype(np.float16).view(np.uint16)
    assert np.array_equal(oracle.float_to_half_bits(v), want)


def test_oracle_lookup_errors():
    table = np.zeros((4, 8), np.uint8)
    scales = np.ones((4, 1), np.float16).view(np.uint16)
    with pytest.raises(oracle.LookupOutOfBounds) as e:
        oracle.embedding_lookup_blockwise_int4([0, 3, 4, -1], table, 4, 16, scales, 16)
    assert e.value.position == 2
    with pytest.raises(oracle.LookupOutOfBounds) as e:
        oracle.embedding_lookup_hybrid([-1], table, 8, 4, 8)
    assert e.value.position == 0
    with pytest.raises(ValueError):
        oracle.embedding_lookup_blockwise_int4([0], table, 4, 16, scales, 12)


# ---- GPU -----------------------------------------------------------------------------------

def _gpu():
    torch = pytest.importorskip("torch")
    if not torch.cuda.is_available():
        pytest.fail("GPU tests need a gfx950 device; none visible")
    from litert_amd import embedding_lookup as el
    return torch, el


def _bits(t):
    """Device result as the oracle returns it: float32 array, or binary16 bit patterns."""
    a = t.cpu().numpy()
    return a.view(np.uint16) if a.dtype == np.float16 else a


@pytest.mark.gpu
@pytest.mark.parametrize("case", KATS, ids=_ids(KATS))
def test_hip_against_reference_vectors(case):
    torch, el = _gpu()
    table = np.asarray(case["table"], np.uint8 if case["value_bits"] == 4 else np.int8)
    if case["kind"] == "blockwise":
        op = el.EmbeddingLookupBlockwiseInt4(table.reshape(case["rows"], -1),
                                             np.asarray(case["scales_f16_bits"], np.uint16),
                                             case["cols"], case["blocksize"], case["out_f16"])
    else:
        op = el.EmbeddingLookupHybrid(table.reshape(case["rows"], -1), case["cols"],
                                      case["value_bits"], row_scales=case["row_scales"],
                                      out_f16=case["out_f16"])
    got = _bits(op(np.asarray(case["lookup"], np.int32)))
    want = _oracle_case(case)
    assert np.array_equal(got.view(want.dtype), want)
    assert np.abs(_as_float(got).ravel() - np.asarray(case["expected"], np.float32)).max() <= case["tolerance"]


@pytest.mark.gpu
@pytest.mark.parametrize("out_f16", [False, True])
@pytest.mark.parametrize("rows,cols,bs,count", [
    (64, 2048, 32, 1),       # one decode token, 8 columns per thread
    (300, 2048, 32, 77),
    (50, 640, 128, 9),
    (41, 24, 4, 13),         # blocks narrower than 8 columns: 2 columns per thread
    (17, 36, 6, 5),
    (9, 4096 + 64, 32, 3),   # rows that do not fill their last thread group
])
def test_hip_blockwise_int4_matches_oracle(rows, cols, bs, count, out_f16):
    torch, el = _gpu()
    rng = np.random.default_rng(rows * 1000 + cols + count)
    table, sbits = _random_blockwise(rng, rows, cols, bs)
    lookup = rng.integers(0, rows, count).astype(np.int32)
    lookup[0] = rows - 1
    op = el.EmbeddingLookupBlockwiseInt4(table, sbits, cols, bs, out_f16)
    got = _bits(op(lookup))
    want = oracle.embedding_lookup_blockwise_int4(lookup, table, rows, cols, sbits, bs, out_f16)
    assert np.array_equal(got.view(want.dtype), want)


@pytest.mark.gpu
@pytest.mark.parametrize("out_f16", [False, True])
@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("rows,cols,count,per_row", [
    (128, 1024, 40, True), (128, 1024, 40, False), (33, 50, 7, True), (5, 6, 11, False),
    (20, 8, 3, True),
])
def test_hip_hybrid_matches_oracle(rows, cols, count, per_row, bits, out_f16):
    torch, el = _gpu()
    rng = np.random.default_rng(rows + cols + count + bits)
    if bits == 4:
        table = rng.integers(0, 256, (rows, cols // 2), dtype=np.uint8)
    else:
        table = rng.integers(-128, 128, (rows, cols), dtype=np.int8)
    rs = (rng.random(rows, dtype=np.float32) * 0.05 + 1e-6) if per_row else None
    if rs is not None:
        rs[::5] = 1e-9  # products that are subnormal as binary16
    lookup = rng.integers(0, rows, count).astype(np.int32)
    op = el.EmbeddingLookupHybrid(table, cols, bits, scale=0.0173, row_scales=rs, out_f16=out_f16)
    got = _bits(op(lookup))
    want = oracle.embedding_lookup_hybrid(lookup, table, bits, rows, cols, scale=0.0173,
                                          row_scales=rs, out_f16=out_f16)
    assert np.array_equal(got.view(want.dtype), want)


@pytest.mark.gpu
def test_hip_lookup_out_of_bounds_and_empty():
    torch, el = _gpu()
    rng = np.random.default_rng(3)
    rows, cols, bs = 16, 64, 32
    table, sbits = _random_blockwise(rng, rows, cols, bs, full_range=False)
    op = el.EmbeddingLookupBlockwiseInt4(table, sbits, cols, bs)
    lookup = np.array([3, 15, 16, 2, -4, 1], np.int32)
    out = torch.full((6, cols), 7.0, device="cuda")
    with pytest.raises(IndexError, match=r"Got 16, and bounds are \[0, 15\]"):
        op(lookup, out=out)
    assert op.status.tolist() == [1, 2, 16]
    got = out.cpu().numpy()
    good = [0, 1, 3, 5]
    want = oracle.embedding_lookup_blockwise_int4(lookup[good], table, rows, cols, sbits, bs)
    assert np.array_equal(got[good], want)
    assert np.all(got[[2, 4]] == 7.0)  # rows of offending lookups are left alone
    # the next good call rewrites the status pair
    op(lookup[good])
    assert op.status.tolist() == [0, -1, 0]
    # the failing position may lie beyond the first 256 lookups
    many = np.zeros(1000, np.int32)
    many[[700, 900]] = rows
    with pytest.raises(IndexError):
        op(many)
    assert op.status.tolist() == [1, 700, 16]
    # empty lookup vector: nothing written, status cleared
    assert op(np.zeros(0, np.int32)).shape == (0, cols)
    assert op.status.tolist() == [0, -1, 0]
    hy = el.EmbeddingLookupHybrid(np.zeros((4, 8), np.int8), 8, 8, scale=0.5)
    with pytest.raises(IndexError, match=r"Got -1, and bounds are \[0, 3\]"):
        hy(np.array([-1], np.int32))


@pytest.mark.gpu
def test_hip_rejects_what_the_reference_rejects():
    torch, el = _gpu()
    from litert_amd import capi
    table = np.zeros((4, 24), np.uint8)
    scales = np.ones((4, 4), np.float16)
    op = el.EmbeddingLookupBlockwiseInt4(table, scales, 48, 10)  # 10 does not divide 48
    with pytest.raises(capi.LrtFcError, match="divisible by blocksize"):
        op(np.zeros(1, np.int32))
    odd = el.EmbeddingLookupHybrid(np.zeros((4, 3), np.uint8), 5, 4)
    with pytest.raises(capi.LrtFcError, match="even number of columns"):
        odd(np.zeros(1, np.int32))


@pytest.mark.gpu
def test_hip_vocabulary_sized_table():
    """A 256000 x 2048 Int4 table with block size 32 (the embedding of a 2B-parameter decoder):
    a prefill batch of 2048 lookups against the oracle, and invariance of a row's result to its
    position in the lookup vector."""
    torch, el = _gpu()
    rows, cols, bs = 256000, 2048, 32
    g = torch.Generator(device="cuda").manual_seed(9)
    table = torch.randint(0, 256, (rows, cols // 2), dtype=torch.uint8, device="cuda", generator=g)
    scales = (torch.rand((rows, cols // bs), device="cuda", generator=g) * 2e-2 + 1e-3).half()
    op = el.EmbeddingLookupBlockwiseInt4(table, scales, cols, bs)
    rng = np.random.default_rng(4)
    lookup = rng.integers(0, rows, 2048).astype(np.int32)
    lookup[:3] = [0, rows - 1, rows // 2]
    got = op(lookup).cpu().numpy()
    # the oracle on the looked-up rows only (re-indexed), so the host never holds the table
    uniq, inverse = np.unique(lookup, return_inverse=True)
    idx = torch.from_numpy(uniq.astype(np.int64)).cuda()
    sub_table = table[idx].cpu().numpy()
    sub_scales = scales[idx].cpu().numpy().view(np.uint16)
    want = oracle.embedding_lookup_blockwise_int4(inverse.astype(np.int32), sub_table, uniq.size,
                                                  cols, sub_scales, bs)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    again = op(lookup[::-1].copy()).cpu().numpy()
    assert np.array_equal(again[::-1], got)

"""Writes tests/golden/reference_kats.json: the known-answer vectors that the reference's own
tests hold for the quantized FULLY_CONNECTED path, as plain data (inputs and expected outputs).

The numbers are transcribed from the reference's test sources (cited per entry); nothing of the
reference is imported or executed. Float tensors of the op tests are quantized here with the
restated test harness (tests/kat_harness.py, after tflite/kernels/test_util.h:198-222,
1123-1190), so that a fixture holds exactly the integer tensors the kernels see.

    python tests/golden/make_reference_kats.py
"""
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from tests import kat_harness as kh  # noqa: E402

W10 = [1, 2, 3, 4, 5, 6, 7, 8, 9, 10]
X2 = [1, 2, 3, 4, 5, 6, 7, 8, -9, -10, 1, 2, 3, 4, 5, 6, 7, -8, 9, -10]
W4 = [1, 2, 3, 4, 5, 6, 7, 6, 5, 4] * 3
W2 = [1, 0, 1, 0, 1, 0, 1, 0, -1, 0] * 3
ACT = {"none": 0, "relu": 1}


def per_tensor(source, in_range, out_range, weights, bias, x, units, act="none", int4=False,
               int2=False):
    in_s, in_zp = kh.quantization_params(*in_range)
    out_s, out_zp = kh.quantization_params(*out_range)
    if int2:
        # An Int2 filter takes the range [-1, 1] (fully_connected_test.cc:189-192), its scale is
        # derived for quantized values -1 .. 1 (test_util.h:1133-1135) and the values are
        # clamped to -2 .. 1 (test_util.h:209-211).
        w_s, w_zp = kh.quantization_params(-1.0, 1.0, -1, 1)
        wq = kh.quantize(weights, w_s, w_zp, -2, 1).reshape(units, -1)
    elif int4:
        w_s, w_zp = kh.quantization_params(-7.0, 7.0, -7, 7)
        wq = kh.quantize(weights, w_s, w_zp, -7, 7).reshape(units, -1)
    else:
        w_s, w_zp = kh.quantization_params(-63.5, 64)
        wq = kh.quantize(weights, w_s, w_zp).reshape(units, -1)
    xq = kh.quantize(x, in_s, in_zp).reshape(-1, wq.shape[1])
    bias_scale = np.float32(in_s * w_s)
    bq = None if bias is None else kh.quantize_bias(bias, bias_scale)
    return dict(source=source, per_channel=False, int4=int4, int2=int2, activation=ACT[act],
                input=xq.tolist(), filter=wq.tolist(), bias=None if bq is None else bq.tolist(),
                input_scale=float(in_s), input_zero_point=int(in_zp),
                filter_scales=[float(w_s)], filter_zero_point=int(w_zp),
                bias_scale=None if bias is None else float(bias_scale),
                output_scale=float(out_s), output_zero_point=int(out_zp))


def per_tensor_uint8(source, in_range, out_range, weights, bias, x, units, act="none"):
    """QuantizedFullyConnectedOpModel with uint8 tensors: a UINT8 filter takes the INPUT's range
    (fully_connected_test.cc:182-203: no case of its own), every tensor is quantized to 0 .. 255
    (test_util.h:1123-1190), the bias with input scale x filter scale."""
    in_s, in_zp = kh.quantization_params(*in_range, 0, 255)
    out_s, out_zp = kh.quantization_params(*out_range, 0, 255)
    w_s, w_zp = in_s, in_zp
    wq = kh.quantize(weights, w_s, w_zp, 0, 255, np.uint8).reshape(units, -1)
    xq = kh.quantize(x, in_s, in_zp, 0, 255, np.uint8).reshape(-1, wq.shape[1])
    bias_scale = np.float32(in_s * w_s)
    bq = None if bias is None else kh.quantize_bias(bias, bias_scale)
    return dict(source=source, activation=ACT[act], input=xq.tolist(), filter=wq.tolist(),
                bias=None if bq is None else bq.tolist(),
                input_scale=float(in_s), input_zero_point=int(in_zp),
                filter_scale=float(w_s), filter_zero_point=int(w_zp),
                bias_scale=None if bias is None else float(bias_scale),
                output_scale=float(out_s), output_zero_point=int(out_zp))


def per_channel(source, scales, weights, bias, x, units, depth, act="none", int4=False,
                int2=False):
    in_s, in_zp = kh.quantization_params(-63.5, 64)
    out_s, out_zp = kh.quantization_params(-127, 128)
    scales = np.asarray(scales, np.float32)
    w = np.asarray(weights, np.float32).reshape(units, depth)
    inv = (np.float32(1.0) / scales).astype(np.float32)
    lim = 7 if int4 else 127
    lo, hi = (-2, 1) if int2 else (-lim, lim)  # quantization_utils.cc:428-431 for Int2
    wq = np.clip(kh._round_half_away(w * inv[:, None]), lo, hi).astype(np.int8)
    xq = kh.quantize(x, in_s, in_zp).reshape(-1, depth)
    bscale = (scales * in_s).astype(np.float32)
    bq = kh._round_half_away(np.asarray(bias, np.float32) / bscale).astype(np.int32)
    return dict(source=source, per_channel=True, int4=int4, int2=int2, activation=ACT[act],
                input=xq.tolist(), filter=wq.tolist(), bias=bq.tolist(),
                input_scale=float(in_s), input_zero_point=int(in_zp),
                filter_scales=[float(s) for s in scales], filter_zero_point=0, bias_scale=None,
                output_scale=float(out_s), output_zero_point=int(out_zp))


def embedding_lookup_cases():
    """tflite/kernels/embedding_lookup_test.cc: tables quantized as its harness does
    (test_util.h:705-750 per block, :753-800 per row; round half away of value x float(1 / scale),
    clamped to +-7 for Int4 and +-127 for Int8, quantization_utils.cc:394-437, 440-475), the
    lookups and the float outputs the tests expect within their tolerances (7.41e-3, 1e-2 for
    Float16 outputs, :35-36)."""
    e = "tflite/kernels/embedding_lookup_test.cc"
    small = [0.00, 0.007, 0.006, 0.005, 0.004, 0.003, 0.002, 0.001,
             0.02, -0.02, 0.04, 0.06, 0.08, -0.04, -0.08, -0.06,
             0.3, 0.6, 0.9, 1.2, 1.5, -0.3, -0.6, -0.9]
    wide = [0.00, 0.01, 0.02, 0.03, 0.10, 0.11, 0.12, 0.13,
            1.00, -1.01, 1.02, 1.03, 1.10, 1.11, 1.12, 1.13,
            2.00, 2.01, 2.02, 2.03, 2.10, 2.11, 2.12, 2.13]
    lookup = [1, 0, 2]

    def rows_of(data, order):
        d = np.asarray(data, np.float32).reshape(3, 8)
        return d[order].ravel().tolist()

    def quantize(data, scales_per_element, limit):
        inv = (np.float32(1.0) / scales_per_element).astype(np.float32)
        q = kh._round_half_away(np.asarray(data, np.float32) * inv)
        return np.clip(q, -limit, limit).astype(np.int8)

    cases = []
    for lines, f16 in ((":509-534", False), (":569-596", True)):
        bits16 = np.asarray([0.001, 0.001, 0.02, 0.02, 0.3, 0.3], np.float16)
        per_element = np.repeat(bits16.astype(np.float32), 4)
        q = quantize(small, per_element, 7)
        cases.append(dict(source=e + lines, kind="blockwise", value_bits=4, rows=3, cols=8,
                          blocksize=4, lookup=lookup, table=kh.pack_int4(q).tolist(),
                          scales_f16_bits=bits16.view(np.uint16).tolist(), out_f16=f16,
                          expected=rows_of(small, lookup), tolerance=1e-2 if f16 else 7.41e-3))
    for lines, data, scales, bits, shape in (
            (":420-440", wide, [0.00102, 0.0089, 0.016772], 8, [3, 8]),
            (":442-462", wide, [0.00102, 0.0089, 0.016772], 8, [3, 2, 4]),
            (":633-656", small, [0.001, 0.02, 0.3], 4, [3, 8]),
            (":658-679", small, [0.001, 0.02, 0.3], 4, [3, 2, 4])):
        sc = np.asarray(scales, np.float32)
        q = quantize(data, np.repeat(sc, 8), 7 if bits == 4 else 127)
        table = kh.pack_int4(q).tolist() if bits == 4 else q.tolist()
        cases.append(dict(source=e + lines, kind="per_row", value_bits=bits, rows=3, cols=8,
                          value_shape=shape, lookup=lookup, table=table,
                          row_scales=[float(v) for v in sc], out_f16=False,
                          expected=rows_of(data, lookup), tolerance=7.41e-3))
    return cases


def batch_matmul_hybrid_cases():
    """tflite/kernels/batch_matmul_test.cc:504-985: float inputs, weights quantized per tensor
    by the harness (SetSignedWeights -> QuantizeTensor), expected float outputs with the
    tolerance each test states."""
    b = "tflite/kernels/batch_matmul_test.cc"
    w3 = [1, 1, 1, 2, 2, 2, 3, 3, 3, 4, 4, 4, 5, 5, 5, 6, 6, 6, 7, 7, 7, 8, 8, 8, 9, 9, 9, 10, 10, 10]
    w9 = [v for r in range(10) for v in [r + 1] * 3 + [r + 17] * 3 + [r + 26] * 3]
    w_two = ([v for r in range(10) for v in (r + 1, r - 3, r + 1)] +
             [v for r in range(10) for v in (r + 1,) * 3])
    w10 = [1] * 5 + [2] * 5 + [3] * 5 + [1] * 5 + [2] * 5 + [3] * 5
    x_small = [1, 2, 3, 4, 5, 6, 7, 8, -9, -10, 1, 2, 3, 4, 5, 6, 7, -8, 9, -10]
    x_big = [11, 12, 13, 14, 15, 16, 17, 18, -19, -20, 11, 12, 13, 14, 15, 16, 17, -18, 19, -20]
    big_want = [23, 23, 23, 295, 295, 295, 448, 448, 448, 57, 57, 57, 361, 361, 361, 532, 532, 532,
                193, 193, 193, 1425, 1425, 1425, 2118, 2118, 2118,
                247, 247, 247, 1511, 1511, 1511, 2222, 2222, 2222]
    cases = []

    def add(source, lhs_shape, rhs_shape, weights, x, want, tol, asym=True, adj_y=False,
            adj_x=False):
        q, scale = kh.symmetric_quantize_tensor(weights)
        cases.append(dict(source=source, lhs_shape=lhs_shape, rhs_shape=rhs_shape,
                          rhs=q.reshape(rhs_shape).tolist(), filter_scale=float(scale),
                          lhs=np.asarray(x, np.float32).reshape(lhs_shape).tolist(),
                          asymmetric_quantize_inputs=asym, adj_y=adj_y, adj_x=adj_x,
                          expected=want, max_abs_err=tol))

    add(b + ":504-533", [2, 10], [10, 3], w3, x_big, [193] * 3 + [247] * 3, 3.0)
    add(b + ":535-565", [1, 2, 2, 3], [3, 10], w10, [11, 12, 13] * 4, [73] * 40, 0.64)
    add(b + ":567-592", [2, 3], [3, 10], w10, [11, 12, 13] * 2, [73] * 20, 0.64)
    add(b + ":600-631", [6, 3], [3, 8], [1] * 8 + [2] * 8 + [3] * 8, [11, 12, 13] * 6, [74] * 48, 0.15)
    add(b + ":633-661", [3, 6], [3, 8], [1] * 8 + [2] * 8 + [3] * 8, [11] * 6 + [12] * 6 + [13] * 6,
        [74] * 48, 0.15, adj_x=True)
    add(b + ":663-698", [6, 3], [8, 3], [1, 2, 3] * 8, [11, 12, 13] * 6, [74] * 48, 0.15,
        adj_y=True)
    add(b + ":700-727", [3, 6], [8, 3], [1, 2, 3] * 8, [11] * 6 + [12] * 6 + [13] * 6, [74] * 48,
        0.15, adj_x=True, adj_y=True)
    add(b + ":729-758", [2, 2, 10], [10, 3], w3, x_small + x_big,
        [23] * 3 + [57] * 3 + [193] * 3 + [247] * 3, 3.0)
    add(b + ":760-798", [2, 2, 10], [10, 9], w9, x_small + x_big, big_want, 10.0)
    add(b + ":800-846", [2, 10], [2, 10, 3], w_two, x_small,
        [23, -45, 23, 57, -19, 57, 23, 23, 23, 57, 57, 57], 1.5)
    add(b + ":848-878", [2, 10], [10, 3], w3, x_big, [193] * 3 + [247] * 3, 1.5, asym=False)
    add(b + ":880-910", [2, 2, 10], [10, 3], w3, x_small + x_big,
        [23] * 3 + [57] * 3 + [193] * 3 + [247] * 3, 1.5, asym=False)
    add(b + ":912-951", [2, 2, 10], [10, 9], w9, x_small + x_big, big_want, 10.0, asym=False)
    add(b + ":953-985", [2, 10], [2, 10, 3], w_two, x_small,
        [23, -45, 23, 57, -19, 57, 23, 23, 23, 57, 57, 57], 1.5, asym=False)
    return cases


def main():
    t = "tflite/kernels/fully_connected_test.cc"
    fc = []
    for case, want in (
            (per_tensor(t + ":816-840", (-63.5, 64), (-127, 128), W10 * 3, [1, 2, 3], X2, 3),
             [23, 24, 25, 57, 58, 59]),
            (per_tensor(t + ":1319-1347", (-63.5, 64), (-127, 128), W10 * 3, None, X2, 3, "relu"),
             [22, 22, 22, 56, 56, 56]),
            (per_tensor(t + ":1463-1487", (-63.5, 64), (-127, 128), W10 * 4, [1, 2, 3, 4], X2[10:], 4),
             [57, 58, 59, 60]),
            (per_tensor(t + ":1530-1562", (-127, 128), (-63.5, 64), W10 * 3, [1, 2, 3], X2, 3),
             [47, 49, 51, 115, 117, 119]),
            (per_tensor(t + ":756-782", (-63.5, 64), (-127, 128), W4, [1, 2, 3], X2, 3, "relu", True),
             [103, 104, 105, 97, 98, 99]),
            (per_channel(t + ":863-888", [0.2, 0.25, 0.5], W10 * 3, [1, 2, 3], X2, 3, 10),
             [23, 24, 25, 57, 58, 59]),
            (per_channel(t + ":890-948", [0.2, 0.25, 0.5], [1, 2, 3, 4, 5] * 3, [1, 2, 3],
                         [1, 2, 3, 4, -5, 1, 2, 3, -4, 5, 1, 2, -3, 4, 5, 1, -2, 3, 4, 5], 3, 5, "relu"),
             [5, 6, 7, 23, 24, 25, 37, 38, 39, 47, 48, 49]),
            (per_channel(t + ":950-976", [1.0, 1.0, 1.0], W4, [1, 2, 3], X2, 3, 10, "relu", True),
             [103, 104, 105, 97, 98, 99]),
            (per_tensor(t + ":784-814", (-63.5, 64), (-127, 128), W2, [1, 2, 3], X2, 3, "relu",
                        int2=True),
             [25, 26, 27, 7, 8, 9]),
            (per_channel(t + ":978-1004", [1.0, 1.0, 1.0], W2, [1, 2, 3], X2, 3, 10, "relu",
                         int2=True),
             [25, 26, 27, 7, 8, 9])):
        case["expected_output"] = want
        fc.append(case)

    # The legacy uint8 op. The 4-D inputs {4, 1, 5, 1} of :2079-2158 flatten to the same [2, 10].
    fc_u8 = []
    for case, want in (
            (per_tensor_uint8(t + ":674-712", (-63.5, 64), (-127, 128), W10 * 3, [1, 2, 3], X2, 3, "relu"),
             [151, 152, 153, 185, 186, 187]),
            (per_tensor_uint8(t + ":714-752", (-63.5, 64), (-127, 128), W10 * 3, None, X2, 3, "relu"),
             [150, 150, 150, 184, 184, 184]),
            (per_tensor_uint8(t + ":1489-1528", (-127, 128), (-63.5, 64), W10 * 3, [1, 2, 3], X2, 3, "relu"),
             [175, 177, 179, 243, 245, 247]),
            (per_tensor_uint8(t + ":2079-2117", (-63.5, 64), (-127, 128), W10 * 3, [1, 2, 3], X2, 3, "relu"),
             [151, 152, 153, 185, 186, 187]),
            (per_tensor_uint8(t + ":2119-2158", (-127, 128), (-63.5, 64), W10 * 3, [1, 2, 3], X2, 3, "relu"),
             [175, 177, 179, 243, 245, 247])):
        case["expected_output"] = want
        fc_u8.append(case)

    u = "tflite/kernels/internal/tensor_utils_test.cc"
    a = [-640, -635.0, -630, 10.0, 2.0, -5.0, -10.0, 0.0, 1000.0]
    small = [-1e-5, 3e-5, -7e-6, -9e-5, 1e-6, 4e-5, 9e-6, 2e-4, 0]
    quantize = [
        dict(source=u + ":220-236", asymmetric=False, values=a,
             expected=[-81, -81, -80, 1, 0, -1, -1, 0, 127]),
        dict(source=u + ":238-251", asymmetric=False, values=[0.0] * 9, expected=[0] * 9,
             expected_scale=1.0),
        dict(source=u + ":253-268", asymmetric=False, values=small,
             expected=[-6, 19, -4, -57, 1, 25, 6, 127, 0]),
        dict(source=u + ":270-290", asymmetric=True, values=a,
             expected=[-128, -127, -126, -26, -28, -29, -30, -28, 127], expected_zero_point=-28),
        dict(source=u + ":292-303", asymmetric=True, values=[0.0] * 9, expected=[0] * 9,
             expected_scale=1.0, expected_zero_point=0),
        dict(source=u + ":305-324", asymmetric=True, values=[2000.0] * 9, expected=[127] * 9,
             expected_zero_point=-128),
        dict(source=u + ":326-345", asymmetric=True, values=small,
             expected=[-58, -23, -55, -128, -48, -14, -41, 127, -49], expected_zero_point=-49),
    ]

    q = "tflite/kernels/internal/quantization_util_test.cc"
    multiplier = [dict(source=q + ":358-423", real=m, quantized=qm, shift=s) for m, qm, s in (
        (0.25, 1073741824, -1), (0.50 - 5e-9, 2147483627, -1), (0.50 - 1e-10, 1073741824, 0),
        (0.50, 1073741824, 0), (0.75, 1610612736, 0), (1 - 1e-9, 2147483646, 0),
        (1 + 1e-11, 1073741824, 1), (1.25, 1342177280, 1), (1.50, 1610612736, 1),
        (1.75, 1879048192, 1), (2 - 1e-9, 2147483647, 1), (2 - 1e-11, 1073741824, 2),
        (2.0, 1073741824, 2), (2.0 ** -31, 1073741824, -30), (2.0 ** -32, 1073741824, -31),
        (2.0 ** -33, 0, 0), (0.0, 0, 0))]
    mbqm = [dict(source=q + ":447-485", x=x, real_multiplier=m, expected=e) for x, m, e in (
        (0, 0.1, 0), (1, 0, 0), (10000, 0.00097656, 10), (-10000, 0.00097656, -10),
        (-2 ** 31, 0.00001, -21475), (2 ** 31 - 1, 0.00001, 21475),
        (10000, -0.00097656, -10), (-10000, -0.00097656, 10),
        (-2 ** 31, -0.00001, 21475), (2 ** 31 - 1, -0.00001, -21475))]

    # Hybrid dot goldens with per-channel scales and input offsets (u:1214-1231); the tensors
    # are the test's generated data (u:1064-1150) for the 4 x 16 x 1 and 4 x 32 x 2 cases.
    def mv(rows, cols, batch):
        i = np.arange(rows * cols)
        matrix = (i % 70).astype(np.int8).reshape(rows, cols)
        j = np.arange(cols * batch)
        vectors = (j % 50).astype(np.int32).reshape(batch, cols) + np.arange(batch)[:, None]
        return dict(matrix=matrix.tolist(), vectors=vectors.astype(np.int8).tolist(),
                    scaling_factors=[float(v) for v in np.arange(1, 9, dtype=np.float32)[:batch]],
                    per_channel_scales=[0.5 if r % 2 == 0 else 1.0 for r in range(rows)],
                    input_offsets=list(range(batch)))
    hybrid_dot = []
    for (rows, cols, batch), want in (((4, 16, 1), [620, 3160, 2540, 7000]),
                                      ((4, 32, 2), [5208, 26288, 4245, 23312, 9138, 70756, 18708, 60916])):
        case = mv(rows, cols, batch)
        case.update(source=u + ":1214-1231", expected=want)
        hybrid_dot.append(case)

    lookups = embedding_lookup_cases()

    out = dict(embedding_lookup=lookups, fully_connected_int8=fc, fully_connected_uint8=fc_u8,
               batch_quantize_floats=quantize,
               quantize_multiplier=multiplier, multiply_by_quantized_multiplier=mbqm,
               hybrid_dot_per_channel=hybrid_dot,
               batch_matmul_hybrid=batch_matmul_hybrid_cases(),
               unpack_int2=[dict(source=u + ":2131-2140", packed=[0x6C], count=4,
                                 expected=[0, -1, -2, 1]),
                            dict(source=u + ":2142-2150", packed=[0xD8], count=3,
                                 expected=[0, -2, 1])],
               unpack_int4=[dict(source=u + ":2110-2119", packed=[0x38, 0xBE], count=4,
                                 expected=[-8, 3, -2, -5]),
                            dict(source=u + ":2121-2130", packed=[0x21, 0x43], count=3,
                                 expected=[1, 2, 3])])
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_kats.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=1)
    print("wrote", path)


if __name__ == "__main__":
    main()

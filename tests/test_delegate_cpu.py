"""Host-side behaviour of the delegate plugin that needs no GPU: exported entry points,
option handling, the node-claim predicate (same accept/decline decisions as the builtin
kernel's type and shape checks), and loud failure when no gfx950 device exists."""
import ctypes as C

import numpy as np
import pytest

from tests import fake_host as fhm
from tests.fake_host import FakeHost, FLOAT32, INT32, UINT8, INT8, FLOAT16, INT4, INT16, INT2


def test_plugin_exports_entry_points():
    lib = C.CDLL(fhm.DELEGATE_LIB)
    for name in ("tflite_plugin_create_delegate", "tflite_plugin_destroy_delegate",
                 "litert_amd_classify_node", "litert_amd_describe_partition",
                 "litert_amd_register_device_buffer", "LiteRtAcceleratorImpl"):
        assert hasattr(lib, name)
    # no delegate, no handle (kTfLiteNullBufferHandle)
    lib.litert_amd_register_device_buffer.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
    assert lib.litert_amd_register_device_buffer(None, None, 16) == -1


def _int8_node(h, B=2, K=32, N=8, per_channel=True, filter_type=INT8, in_type=INT8, out_type=INT8,
               const_filter=True, w_zp=0, bias=True, **kw):
    x = h.tensor(in_type, (B, K), scale=0.02, zero_point=-3)
    h.affine(x, [0.02], [-3])
    wbytes = {INT4: N * K // 2, INT2: N * K // 4}.get(filter_type, N * K)
    w = h.tensor(filter_type, (N, K), data=np.zeros(wbytes, np.int8), const=const_filter)
    if per_channel:
        h.affine(w, np.full(N, 0.005), np.full(N, w_zp))
    else:
        h.affine(w, [0.005], [w_zp])
    b = h.tensor(INT32, (N,), data=np.zeros(N, np.int32), const=True) if bias else None
    y = h.tensor(out_type, (B, N), scale=0.05, zero_point=5)
    h.affine(y, [0.05], [5])
    return h.fc(x, w, b, y, **kw)


def test_claim_predicate_int8():
    with FakeHost() as h:
        assert h.classify(_int8_node(h))[0] == "int8"
        assert h.classify(_int8_node(h, per_channel=False, w_zp=-1))[0] == "int8"
        assert h.classify(_int8_node(h, filter_type=INT4))[0] == "int8"
        # Int2 filters are unpacked to int8 like Int4 ones (fully_connected.cc:1678-1685)
        assert h.classify(_int8_node(h, filter_type=INT2))[0] == "int8"
        assert h.classify(_int8_node(h, filter_type=INT2, per_channel=False))[0] == "int8"
        assert h.classify(_int8_node(h, per_channel=False, filter_type=INT2, w_zp=1)) == (
            None, "non-zero filter zero point")
        assert h.classify(_int8_node(h, bias=False))[0] == "int8"
        assert h.classify(_int8_node(h, bias=False, optional_bias_slot=True))[0] == "int8"
        for act in (0, 1, 2, 3):
            assert h.classify(_int8_node(h, activation=act))[0] == "int8"
        # declined: left to the CPU kernels
        # the legacy uint8 op: per-tensor only, claimed (it runs on the int8 kernels, value - 128)
        assert h.classify(_int8_node(h, in_type=UINT8, out_type=UINT8, filter_type=UINT8,
                                     per_channel=False, w_zp=131))[0] == "int8"
        assert h.classify(_int8_node(h, in_type=UINT8, out_type=UINT8, filter_type=UINT8)) == (
            None, "uint8 filter is not per-tensor")
        assert h.classify(_int8_node(h, in_type=UINT8, out_type=UINT8, filter_type=UINT8,
                                     per_channel=False, activation=4)) == (None, "activation not a clamp")
        assert h.classify(_int8_node(h, in_type=UINT8, out_type=INT8, filter_type=UINT8,
                                     per_channel=False)) == (None, "tensor type combination not handled")
        assert h.classify(_int8_node(h, in_type=INT16, out_type=INT16))[0] is None
        assert h.classify(_int8_node(h, const_filter=False)) == (None, "filter is not a constant tensor")
        assert h.classify(_int8_node(h, weights_format=1)) == (None, "shuffled weights format")
        assert h.classify(_int8_node(h, w_zp=3)) == (None, "non-zero filter zero point")
        assert h.classify(_int8_node(h, per_channel=False, filter_type=INT4, w_zp=1))[0] is None
        assert h.classify(_int8_node(h, activation=4)) == (None, "activation not a clamp")
        assert h.classify(_int8_node(h, version=15)) == (None, "op version newer than 14")
        a, b = h.tensor(FLOAT32, (2, 4)), h.tensor(FLOAT32, (2, 4))
        assert h.classify(h.other(0, a, b)) == (None, "not FULLY_CONNECTED")


def _float_node(h, B=2, K=64, N=8, filter_type=INT8, blockwise=False, bs=32, per_channel=True,
                scale_type=FLOAT16, quantized_dimension=0, **kw):
    x = h.tensor(FLOAT32, (B, K))
    if blockwise:
        w = h.tensor(INT4, (N, K), data=np.zeros(N * K // 2, np.uint8), const=True)
        s = h.tensor(scale_type, (N, K // bs), data=np.ones((N, K // bs), np.float16 if scale_type == FLOAT16 else np.float32), const=True)
        h.blockwise(w, s, bs)
    else:
        nbytes = {INT8: N * K, INT2: N * K // 4}.get(filter_type, N * K // 2)
        w = h.tensor(filter_type, (N, K), data=np.zeros(nbytes, np.int8), const=True)
        h.affine(w, np.full(N if per_channel else 1, 0.004), quantized_dimension=quantized_dimension)
    y = h.tensor(FLOAT32, (B, N))
    return h.fc(x, w, None, y, **kw)


def test_claim_predicate_float_activations():
    with FakeHost() as h:
        assert h.classify(_float_node(h))[0] == "hybrid"
        assert h.classify(_float_node(h, per_channel=False, asymmetric=False))[0] == "hybrid"
        assert h.classify(_float_node(h, activation=3))[0] == "hybrid"
        # the hybrid path takes every activation in the reference; the sign bit is exact and
        # claimed, tanh (4) and sigmoid (6) go through Eigen there and stay on the CPU
        assert h.classify(_float_node(h, activation=5))[0] == "hybrid"
        assert h.classify(_float_node(h, activation=4)) == (None, "activation is tanh or sigmoid")
        assert h.classify(_float_node(h, activation=6)) == (None, "activation is tanh or sigmoid")
        assert h.classify(_float_node(h, blockwise=True))[0] == "int4_blockwise"
        assert h.classify(_float_node(h, blockwise=True, K=128, bs=64))[0] == "int4_blockwise"
        # the builtin's 4-bit gate: N >= 4, K >= 32, K even, blocksize | K
        assert h.classify(_float_node(h, blockwise=True, N=2)) == (None, "shape outside 4-bit gate")
        assert h.classify(_float_node(h, blockwise=True, K=16, bs=16)) == (None, "shape outside 4-bit gate")
        assert h.classify(_float_node(h, blockwise=True, K=96, bs=64)) == (None, "bad blocksize")
        assert h.classify(_float_node(h, blockwise=True, scale_type=FLOAT32)) == (None, "scales not const fp16")
        # per-channel int4 hybrid (EvalHybridDense4Bit): claimed inside the builtin's 4-bit gate
        assert h.classify(_float_node(h, filter_type=INT4))[0] == "int4_per_channel"
        assert h.classify(_float_node(h, filter_type=INT4, per_channel=False))[0] == "int4_per_channel"
        # outside that gate the builtin unpacks the nibbles and runs the ordinary hybrid kernels
        # (fully_connected.cc:805-814): claimed as a hybrid node
        assert h.classify(_float_node(h, filter_type=INT4, N=2))[0] == "hybrid"
        assert h.classify(_float_node(h, filter_type=INT4, K=16))[0] == "hybrid"
        assert h.classify(_float_node(h, filter_type=INT4, K=16, activation=4)) == (
            None, "activation is tanh or sigmoid")
        assert h.classify(_float_node(h, filter_type=INT4, activation=4)) == (None, "activation is tanh or sigmoid")
        assert h.classify(_float_node(h, filter_type=INT4, activation=5))[0] == "int4_per_channel"
        # an Int2 filter under float activations: unpacked, then EvalHybridDense
        # (fully_connected.cc:812-818): claimed as a hybrid node, whatever the shape
        assert h.classify(_float_node(h, filter_type=INT2))[0] == "hybrid"
        assert h.classify(_float_node(h, filter_type=INT2, per_channel=False, N=2, K=16))[0] == "hybrid"
        assert h.classify(_float_node(h, filter_type=INT2, activation=6)) == (
            None, "activation is tanh or sigmoid")
        # scales along the depth are not per-output-channel scales
        assert h.classify(_float_node(h, filter_type=INT4, N=8, K=8 * 8, quantized_dimension=1)) == (
            None, "per-channel scales do not match output channels")


def _bmm_node(h, lhs_shape=(2, 5, 64), rhs_shape=(64, 8), lhs_type=FLOAT32, const=True,
              scales=None, qdim=0, **kw):
    x = h.tensor(lhs_type, lhs_shape)
    w = h.tensor(INT8, rhs_shape, data=np.zeros(rhs_shape, np.int8), const=const)
    h.affine(w, [0.004] if scales is None else scales, quantized_dimension=qdim)
    y = h.tensor(FLOAT32, (2, 5, 8))
    return h.batch_matmul(x, w, y, **kw)


def test_claim_predicate_batch_matmul():
    """The hybrid form of BATCH_MATMUL (tflite/kernels/batch_matmul.cc:363-374): float32 left
    operand, constant int8 right operand, adj_x / adj_y and the op's broadcasting of up to three
    batch dimensions included."""
    with FakeHost() as h:
        assert h.classify(_bmm_node(h))[0] == "batch_matmul"
        assert h.classify(_bmm_node(h, rhs_shape=(8, 64), adj_y=True))[0] == "batch_matmul"
        assert h.classify(_bmm_node(h, rhs_shape=(2, 64, 8)))[0] == "batch_matmul"
        assert h.classify(_bmm_node(h, scales=np.full(8, 0.01), qdim=1))[0] == "batch_matmul"
        assert h.classify(_bmm_node(h, scales=np.full(8, 0.01), qdim=0)) == (
            None, "per-channel scales do not run along the output units")
        assert h.classify(_bmm_node(h, lhs_shape=(2, 64, 5), adj_x=True))[0] == "batch_matmul"
        assert h.classify(_bmm_node(h, adj_x=True)) == (None, "accumulation depths differ")
        # register.cc:327-329 registers versions 1..4; a newer one may mean other arithmetic
        assert h.classify(_bmm_node(h, version=4))[0] == "batch_matmul"
        assert h.classify(_bmm_node(h, version=5)) == (None, "op version newer than 4")
        assert h.classify(_bmm_node(h, const=False)) == (None, "right operand is not a constant tensor")
        assert h.classify(_bmm_node(h, lhs_type=INT8)) == (None, "not the float32 x int8 form")
        assert h.classify(_bmm_node(h, rhs_shape=(32, 8))) == (None, "accumulation depths differ")
        assert h.classify(_bmm_node(h, lhs_shape=(2, 1, 5, 64), rhs_shape=(1, 3, 64, 8)))[0] == "batch_matmul"
        assert h.classify(_bmm_node(h, lhs_shape=(2, 5, 64), rhs_shape=(3, 64, 8))) == (
            None, "batch dimensions do not broadcast")


def test_bad_options_are_rejected_before_touching_the_device():
    with FakeHost() as h:
        assert h.load_delegate({"no_such_option": "1"}) == 1
        assert "unknown option 'no_such_option'" in h.errors()
    with FakeHost() as h:
        assert h.load_delegate({"quant_variant": "fast"}) == 1
        assert "quant_variant must be" in h.errors()
    with FakeHost() as h:
        assert h.load_delegate({"claim": "int8,float"}) == 1
        assert "claim accepts" in h.errors()
    with FakeHost() as h:
        assert h.load_delegate({"direct_inputs": "yes"}) == 1
        assert "direct_inputs must be 0 or 1" in h.errors()
    with FakeHost() as h:
        assert h.load_delegate({"completion": "spin"}) == 1
        assert "completion must be poll or sync" in h.errors()


def test_no_gpu_means_no_delegate():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    with FakeHost() as h:
        _int8_node(h)
        assert h.load_delegate() == 1  # create_delegate returned NULL
        assert "HIP device" in h.errors()
        # the graph is untouched: every node still belongs to the CPU
        assert [kind for kind, _, _ in h.plan()] == ["cpu"]


def _lookup_node(h, rows=16, cols=64, count=3, value_type=INT4, blockwise=True, bs=32, per_row=True,
                 out_type=FLOAT32, lookup_type=INT32, const_table=True, zero_point=0,
                 scale_type=FLOAT16, value_shape=None):
    lk = h.tensor(lookup_type, (count,))
    shape = value_shape or (rows, cols)
    nbytes = rows * cols // 2 if value_type == INT4 else rows * cols
    v = h.tensor(value_type, shape, data=np.zeros(nbytes, np.uint8), const=const_table)
    if blockwise:
        s = h.tensor(scale_type, (rows, cols // bs),
                     data=np.ones((rows, cols // bs), np.float16 if scale_type == FLOAT16 else np.float32),
                     const=True)
        h.blockwise(v, s, bs)
    else:
        h.affine(v, np.full(rows if per_row else 1, 0.01), np.full(rows if per_row else 1, zero_point))
    y = h.tensor(out_type, (count,) + tuple(shape[1:]))
    return h.embedding_lookup(lk, v, y)


def test_claim_predicate_embedding_lookup():
    """What EvalBlockwise / EvalHybrid accept for Int4 and Int8 tables
    (tflite/kernels/embedding_lookup.cc:49-100, 194-225, 397-412), nothing else."""
    with FakeHost() as h:
        assert h.classify(_lookup_node(h))[0] == "embedding_lookup"
        assert h.classify(_lookup_node(h, out_type=FLOAT16))[0] == "embedding_lookup"
        assert h.classify(_lookup_node(h, blockwise=False))[0] == "embedding_lookup"
        assert h.classify(_lookup_node(h, blockwise=False, per_row=False))[0] == "embedding_lookup"
        assert h.classify(_lookup_node(h, blockwise=False, value_type=INT8))[0] == "embedding_lookup"
        assert h.classify(_lookup_node(h, blockwise=False, value_type=INT8,
                                       value_shape=(16, 4, 16)))[0] == "embedding_lookup"
        # declined: left to the CPU kernel
        assert h.classify(_lookup_node(h, bs=24)) == (None, "bad blocksize")
        assert h.classify(_lookup_node(h, scale_type=FLOAT32)) == (None, "scales not const fp16")
        assert h.classify(_lookup_node(h, const_table=False)) == (None, "table is not a constant tensor")
        assert h.classify(_lookup_node(h, lookup_type=FLOAT32))[1] == "lookup is not a rank-1 int32 tensor"
        assert h.classify(_lookup_node(h, out_type=INT8))[1] == "output is not float32 or float16"
        assert h.classify(_lookup_node(h, blockwise=False, value_type=UINT8))[1] == (
            "table type is left to the CPU kernels")
        assert h.classify(_lookup_node(h, blockwise=False, zero_point=3))[1] == "non-zero table zero point"
        assert h.classify(_lookup_node(h, blockwise=False, cols=7, rows=2))[1] == "odd row length"
        assert h.load_delegate({"claim": "int8,lookup"}) == 1
        assert "batch_matmul; got 'lookup'" in h.errors()

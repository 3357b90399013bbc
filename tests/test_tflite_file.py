"""`.tflite` files: the reader (litert_amd/tflite_file.py) on model files the reference's own
tests load (tests/golden/models), with the assertions those tests make about their contents,
and their FULLY_CONNECTED nodes through the delegate against the oracle."""
import os

import numpy as np
import pytest

import oracle
from litert_amd import tflite_file
from tests.fake_host import FakeHost, OK

MODELS = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "models")


def _load(name):
    return tflite_file.load(os.path.join(MODELS, name))


def test_qwen_blockwise_model_contents():
    """litert/core/model/model_file_test.cc:562-590 and litert/c/litert_model_test.cc:409-455:
    one FULLY_CONNECTED op whose weights are Int4 with blockwise quantization, block size 32,
    scales present."""
    m = _load("qwen_fc_blockwise_quantized.tflite")
    sg = m.subgraphs[0]
    assert len(sg.operators) == 1
    op = sg.operators[0]
    assert op.builtin_code == tflite_file.BUILTIN_FULLY_CONNECTED and len(op.inputs) >= 2
    w = sg.tensors[op.inputs[1]]
    assert w.type_name == "INT4" and w.quantization.kind == "blockwise"
    assert w.quantization.block_size == 32 and w.quantization.scales_tensor >= 0
    # what the FC kernel itself requires of such a filter (fully_connected.cc:254-308, 1006-1030)
    s = sg.tensors[w.quantization.scales_tensor]
    assert s.type_name == "FLOAT16" and s.shape == (w.shape[0], w.shape[1] // 32)
    assert w.quantization.zero_points_tensor == -1 and w.quantization.quantized_dimension == 0
    assert w.data.size == w.shape[0] * w.shape[1] // 2 and s.data.size == 2 * int(np.prod(s.shape))
    assert op.fully_connected["asymmetric_quantize_inputs"] and op.fully_connected["keep_num_dims"]


def test_blockwise_quantized_model_contents():
    """litert/c/litert_model_test.cc:340-404: an ADD whose input "quantized_tensor" is Int8,
    blockwise with block size 32, scales tensor "scales", zero points tensor "zps"."""
    m = _load("blockwise_quantized.tflite")
    sg = m.subgraphs[0]
    assert len(sg.operators) == 1 and sg.operators[0].builtin_code == 0
    assert len(sg.operators[0].inputs) == 2
    q = [sg.tensors[i] for i in sg.operators[0].inputs if sg.tensors[i].name == "quantized_tensor"]
    assert len(q) == 1 and q[0].type_name == "INT8" and q[0].quantization.kind == "blockwise"
    assert q[0].quantization.block_size == 32
    assert sg.tensors[q[0].quantization.scales_tensor].name == "scales"
    assert sg.tensors[q[0].quantization.zero_points_tensor].name == "zps"


def test_fc_qat_model_contents():
    m = _load("fc_qat.bin")
    sg = m.subgraphs[0]
    fcs = [op for op in sg.operators if op.fully_connected is not None]
    assert len(fcs) == 1 and fcs[0].version == 4 and len(fcs[0].inputs) == 3
    x, w, b = (sg.tensors[i] for i in fcs[0].inputs)
    assert (x.type_name, w.type_name, b.type_name) == ("INT8", "INT8", "INT32")
    assert w.shape == (10, 784) and w.quantization.kind == "affine" and w.quantization.scale.size == 1
    # the bias scale a converter writes is input scale x filter scale (kernel_util.cc:275-352)
    assert np.isclose(b.quantization.scale[0], x.quantization.scale[0] * w.quantization.scale[0],
                      rtol=1e-6)


def test_reader_rejects_garbage():
    with pytest.raises(ValueError):
        tflite_file.parse(b"\x00\x01")


def test_delegate_claims_the_file_models_nodes():
    """No GPU needed: the claim predicate on the nodes as the files describe them."""
    for name, kind in (("qwen_fc_blockwise_quantized.tflite", "int4_blockwise"),
                       ("fc_qat.bin", "int8")):
        sg = _load(name).subgraphs[0]
        with FakeHost() as h:
            h.add_fc_nodes_of(sg)
            assert h.classify(0)[0] == kind, (name, h.classify(0))


@pytest.mark.gpu
@pytest.mark.parametrize("seed", [0, 1])
def test_qwen_blockwise_model_through_delegate(seed):
    """The file's one node (float [1, 1, 1024] in, Int4 blockwise [1024, 1024] filter, no bias
    slot, keep_num_dims) run by the delegate; bit-identical to the oracle of EvalBlockwise4Bit."""
    sg = _load("qwen_fc_blockwise_quantized.tflite").subgraphs[0]
    op = sg.operators[0]
    w = sg.tensors[op.inputs[1]]
    scales = sg.tensors[w.quantization.scales_tensor]
    x = np.random.default_rng(seed).standard_normal(sg.tensors[op.inputs[0]].shape).astype(np.float32)
    with FakeHost() as h:
        made = h.add_fc_nodes_of(sg, {op.inputs[0]: x})
        assert h.load_delegate() == 0, h.errors()
        assert h.modify_graph_with_delegate() == OK and h.allocate_tensors() == OK, h.errors()
        assert len(h.plan()) == 1  # the node was replaced by one delegate kernel
        h.write(made[op.inputs[0]], x)
        assert h.invoke() == OK, h.errors()
        got = h.read(made[op.outputs[0]])
    want = oracle.fc_blockwise_int4(x.reshape(1, 1024), w.data.reshape(1024, 512), 1024,
                                    scales.data.view(np.uint16).reshape(1024, 32), 32)
    assert got.shape == (1, 1, 1024)
    assert np.array_equal(got.reshape(1, 1024).view(np.uint32), want.view(np.uint32))


@pytest.mark.gpu
def test_fc_qat_model_node_through_delegate():
    """The int8 FULLY_CONNECTED of fc_qat.bin (per-tensor scale, int32 bias) on a random int8
    input; bit-exact against the integer reference path."""
    sg = _load("fc_qat.bin").subgraphs[0]
    op = [o for o in sg.operators if o.fully_connected is not None][0]
    xt, wt, bt = (sg.tensors[i] for i in op.inputs)
    yt = sg.tensors[op.outputs[0]]
    x = np.random.default_rng(5).integers(-128, 128, xt.shape, dtype=np.int8)
    with FakeHost() as h:
        made = h.add_fc_nodes_of(sg, {op.inputs[0]: x})
        assert h.load_delegate() == 0, h.errors()
        assert h.modify_graph_with_delegate() == OK and h.allocate_tensors() == OK, h.errors()
        h.write(made[op.inputs[0]], x)
        assert h.invoke() == OK, h.errors()
        got = h.read(made[op.outputs[0]])
    in_s, w_s, out_s = (float(t.quantization.scale[0]) for t in (xt, wt, yt))
    in_zp, w_zp, out_zp = (int(t.quantization.zero_point[0]) for t in (xt, wt, yt))
    mult, shift = oracle.fc_prepare_per_tensor(in_s, w_s, out_s, float(bt.quantization.scale[0]))
    lo, hi = oracle.activation_range_int8(op.fully_connected["activation"], out_s, out_zp)
    want = oracle.fc_int8_per_tensor(x, wt.array(), bt.array(), mult, shift, -in_zp, -w_zp, out_zp,
                                     lo, hi)
    assert np.array_equal(got, want)

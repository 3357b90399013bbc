"""The delegate plugin end to end on the GPU, driven by the fake TFLite host exactly as
the interpreter drives an external delegate: Prepare -> ReplaceNodeSubsetsWithDelegateKernels
-> init -> prepare -> invoke. Outputs are compared with the CPU oracle on the same
seeded inputs: bit-exact for int8, bit-identical floats for the hybrid and blockwise paths."""
import numpy as np
import pytest

import oracle
from litert_amd import workloads as wl
from tests.fake_host import (FakeHost, FLOAT32, INT32, UINT8, INT8, FLOAT16, INT4, INT2, OK,
                             DELEGATE_ERROR)

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")


@pytest.fixture(autouse=True)
def _need_gpu():
    if not torch.cuda.is_available():
        pytest.fail("GPU tests need a gfx950 device; none visible")


def _add_int8_fc(h, c, x=None, activation=0, bias=True, out_scale=None, out_zp=None):
    B, K = c["x"].shape
    N = c["w"].shape[0]
    if x is None:
        x = h.tensor(INT8, (B, K), data=c["x"])
        h.affine(x, [c["in_scale"]], [c["in_zp"]])
    w = h.tensor(INT8, (N, K), data=c["w"], const=True)
    h.affine(w, c["w_scale"])
    b = h.tensor(INT32, (N,), data=c["bias"], const=True) if bias else None
    y = h.tensor(INT8, (B, N))
    h.affine(y, [c["out_scale"] if out_scale is None else out_scale],
             [c["out_zp"] if out_zp is None else out_zp])
    return h.fc(x, w, b, y, activation=activation), x, y


def _oracle_int8(c, x, activation=0, bias=True, in_scale=None, in_zp=None):
    in_scale = float(c["in_scale"]) if in_scale is None else in_scale
    in_zp = c["in_zp"] if in_zp is None else in_zp
    mult, shift = oracle.fc_prepare_per_channel(in_scale, c["w_scale"], float(c["out_scale"]))
    lo, hi = oracle.activation_range_int8(activation, float(c["out_scale"]), c["out_zp"])
    return oracle.fc_int8_per_channel(x, c["w"], c["bias"] if bias else None, mult, shift, -in_zp,
                                      c["out_zp"], lo, hi)


# kernels read the host's rows / a copy of them; the invoke polls for its end / synchronizes
BOUNDARY_OPTIONS = [{}, {"direct_inputs": "0"}, {"completion": "sync"},
                    {"direct_inputs": "0", "completion": "sync"}]


@pytest.mark.parametrize("options", BOUNDARY_OPTIONS, ids=lambda o: ",".join(o.values()) or "default")
def test_int8_node_config1_through_delegate(options):
    c = wl.int8_fc()
    with FakeHost() as h:
        node, x, y = _add_int8_fc(h, c)
        assert h.load_delegate(options) == 0, h.errors()
        assert h.modify_graph_with_delegate() == OK, h.errors()
        assert h.plan()[0][:2] == ("delegate", [node])
        assert h.allocate_tensors() == OK, h.errors()
        assert h.invoke() == OK, h.errors()
        assert np.array_equal(h.read(y), _oracle_int8(c, c["x"]))
        # the arena may hand out new addresses between invokes
        h.write(x, np.roll(c["x"], 7, axis=1))
        h.move(x)
        h.move(y)
        assert h.invoke() == OK, h.errors()
        assert np.array_equal(h.read(y), _oracle_int8(c, np.roll(c["x"], 7, axis=1)))


@pytest.mark.parametrize("options", BOUNDARY_OPTIONS, ids=lambda o: ",".join(o.values()) or "default")
@pytest.mark.parametrize("B", [1, 4, 8, 19])  # up to 8 rows fuse the quantizer, more split it off
def test_hybrid_node_through_delegate(B, options):
    c = wl.hybrid_fc(B, 4096, 1024)
    bias = np.random.default_rng(1).standard_normal(1024).astype(np.float32)
    with FakeHost() as h:
        x = h.tensor(FLOAT32, (B, 4096), data=c["x"])
        w = h.tensor(INT8, (1024, 4096), data=c["w"], const=True)
        h.affine(w, c["pcs"])
        b = h.tensor(FLOAT32, (1024,), data=bias, const=True)
        y = h.tensor(FLOAT32, (B, 1024))
        h.fc(x, w, b, y, activation=1, asymmetric=True)
        assert h.load_delegate(options) == 0, h.errors()
        assert h.modify_graph_with_delegate() == OK and h.allocate_tensors() == OK, h.errors()
        assert h.invoke() == OK, h.errors()
        want = oracle.fc_hybrid(c["x"], c["w"], c["pcs"], 1.0, bias, True, oracle.ACT_RELU)
        assert np.array_equal(h.read(y).view(np.uint32), want.view(np.uint32))
        x2 = np.roll(c["x"], 3, axis=1)  # a second invoke sees the new rows, not the first ones
        h.write(x, x2)
        assert h.invoke() == OK, h.errors()
        want = oracle.fc_hybrid(x2, c["w"], c["pcs"], 1.0, bias, True, oracle.ACT_RELU)
        assert np.array_equal(h.read(y).view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("B", [2, 8])  # fused prologue / quantizer launch of its own
def test_hybrid_sign_bit_and_whole_zero_input_through_delegate(B):
    """kTfLiteActSignBit on a hybrid node, and the builtin's early exit for a whole-zero input
    (fully_connected.cc:789-795): a -0.0f bias element must come out with its sign bit set."""
    c = wl.hybrid_fc(B, 512, 96)
    bias = np.random.default_rng(1).standard_normal(96).astype(np.float32)
    bias[::4] = -0.0
    with FakeHost() as h:
        x = h.tensor(FLOAT32, (B, 512), data=c["x"])
        w = h.tensor(INT8, (96, 512), data=c["w"], const=True)
        h.affine(w, c["pcs"])
        b = h.tensor(FLOAT32, (96,), data=bias, const=True)
        y = h.tensor(FLOAT32, (B, 96))
        h.fc(x, w, b, y, activation=5, asymmetric=True)
        assert h.load_delegate() == 0, h.errors()
        assert h.modify_graph_with_delegate() == OK and h.allocate_tensors() == OK, h.errors()
        assert h.plan()[0][0] == "delegate"
        assert h.invoke() == OK, h.errors()
        want = oracle.fc_hybrid(c["x"], c["w"], c["pcs"], 1.0, bias, True, oracle.ACT_SIGN_BIT)
        assert np.array_equal(h.read(y).view(np.uint32), want.view(np.uint32))
        zeros = np.zeros((B, 512), np.float32)
        h.write(x, zeros)
        assert h.invoke() == OK, h.errors()
        want = oracle.fc_hybrid(zeros, c["w"], c["pcs"], 1.0, bias, True, oracle.ACT_SIGN_BIT)
        assert np.array_equal(h.read(y).view(np.uint32), want.view(np.uint32))
        assert want[0, 0] == 1.0 and want[0, 1] == (1.0 if bias[1] < 0 else 0.0)


@pytest.mark.parametrize("B,K,N", [(2, 2048, 512), (1, 16384, 40), (3, 8192, 24), (5, 1024, 16),
                                   (8, 160, 8200), (20, 96, 8192)])
def test_blockwise_int4_node_through_delegate(B, K, N):
    """Shallow rows and up to two deep rows run the fused kernel on the re-tiled filter; three
    or more deep rows are quantized by a launch of their own first; five to 32 rows on a wide
    filter take the GEMM that keeps the filter at 4 bits per weight."""
    c = wl.blockwise_int4_fc(B, K, N, lo=-8, hi=7)
    bias = np.random.default_rng(2).standard_normal(N).astype(np.float32)
    with FakeHost() as h:
        x = h.tensor(FLOAT32, (B, K), data=c["x"])
        w = h.tensor(INT4, (N, K), data=c["packed"], const=True)
        s = h.tensor(FLOAT16, (N, K // 32), data=c["scales"], const=True)
        h.blockwise(w, s, 32)
        b = h.tensor(FLOAT32, (N,), data=bias, const=True)
        y = h.tensor(FLOAT32, (B, N))
        h.fc(x, w, b, y, activation=1)  # the reference ignores the fused activation on this path
        assert h.load_delegate() == 0, h.errors()
        assert h.modify_graph_with_delegate() == OK and h.allocate_tensors() == OK, h.errors()
        assert h.invoke() == OK, h.errors()
        want = oracle.fc_blockwise_int4(c["x"], c["packed"], N, c["scales"].view(np.uint16), 32, bias)
        assert np.array_equal(h.read(y).view(np.uint32), want.view(np.uint32))
        assert (want < 0).any()  # so an applied RELU would have shown


def test_chain_stays_on_device_and_splits_around_cpu_nodes():
    """FC -> FC -> (other op) -> FC: the first two share one partition (their link never
    goes back to the host), the third sits in its own after the CPU node."""
    c1 = wl.int8_fc(3, 256, 128, seed=1)
    c2 = wl.int8_fc(3, 128, 64, in_scale=float(c1["out_scale"]), in_zp=c1["out_zp"], seed=2)
    c3 = wl.int8_fc(3, 64, 32, in_scale=float(c2["out_scale"]), in_zp=c2["out_zp"], seed=3)
    with FakeHost() as h:
        n1, x, y1 = _add_int8_fc(h, c1, activation=3)
        n2, _, y2 = _add_int8_fc(h, c2, x=y1)
        mid = h.tensor(INT8, (3, 64))
        h.affine(mid, [c2["out_scale"]], [c2["out_zp"]])
        other = h.other(0, y2, mid)  # builtin ADD: not ours
        n3, _, y3 = _add_int8_fc(h, c3, x=mid, bias=False)
        ran_on_cpu = []

        def cpu(node):
            ran_on_cpu.append(node)
            h.write(mid, h.read(y2))  # identity stand-in for the foreign op
            return 0
        from tests.fake_host import CPU_CB
        cb = CPU_CB(cpu)
        h.L.fh_set_cpu_callback(h.h, cb)
        assert h.load_delegate() == 0, h.errors()
        assert h.modify_graph_with_delegate() == OK, h.errors()
        plan = h.plan()
        assert [(k, r) for k, r, _ in plan] == [("delegate", [n1, n2]), ("cpu", [other]), ("delegate", [n3])]
        ins, outs = h.node_io(plan[0][2])
        assert outs == [y2] and x in ins and y1 not in ins and y1 not in outs
        assert h.L.fh_tensor_has_delegate(h.h, y2) and not h.L.fh_tensor_has_delegate(h.h, y1)
        assert h.allocate_tensors() == OK and h.invoke() == OK, h.errors()
        w1 = _oracle_int8(c1, c1["x"], activation=3)
        w2 = _oracle_int8(c2, w1)
        w3 = _oracle_int8(c3, w2, bias=False)
        assert ran_on_cpu == [other]
        assert np.array_equal(h.read(y2), w2) and np.array_equal(h.read(y3), w3)


def test_link_that_is_also_a_graph_output_is_copied_not_written_to_the_host():
    """FC -> FC in one partition. Host outputs that no node of the partition reads are written by
    the kernels straight into page-locked host memory; once the link tensor is a graph output as
    well, the second node reads a downloaded tensor, so the partition keeps its outputs in device
    memory and copies them out. Both forms give the oracle's bits, on repeated invokes with new
    inputs."""
    c1 = wl.int8_fc(3, 256, 128, seed=11)
    c2 = wl.int8_fc(3, 128, 64, in_scale=float(c1["out_scale"]), in_zp=c1["out_zp"], seed=12)
    for link_is_output in (False, True):
        with FakeHost() as h:
            n1, x, y1 = _add_int8_fc(h, c1, activation=3)
            n2, _, y2 = _add_int8_fc(h, c2, x=y1)
            if link_is_output:
                h.mark_output(y1)
            assert h.load_delegate() == 0 and h.modify_graph_with_delegate() == OK, h.errors()
            plan = h.plan()
            assert [(k, r) for k, r, _ in plan] == [("delegate", [n1, n2])]
            _, outs = h.node_io(plan[0][2])
            assert sorted(outs) == sorted([y1, y2] if link_is_output else [y2])
            assert h.allocate_tensors() == OK, h.errors()
            rng = np.random.default_rng(3)
            for trial in range(3):
                xin = c1["x"] if trial == 0 else rng.integers(-128, 128, c1["x"].shape).astype(np.int8)
                h.write(x, xin)
                assert h.invoke() == OK, h.errors()
                w1 = _oracle_int8(c1, xin, activation=3)
                assert np.array_equal(h.read(y2), _oracle_int8(c2, w1))
                if link_is_output:
                    assert np.array_equal(h.read(y1), w1)


@pytest.mark.parametrize("streams", [1, 2, 4])
def test_decoder_shaped_partition_on_several_streams(streams):
    """x -> up -> {a, b, c} (three consumers of one tensor, on different streams) plus two
    nodes fed straight from the host and a node that consumes `a`: every cross-stream edge
    (upload -> node, node -> node, node -> download) carries data, so a missing wait shows
    as a wrong result. Repeated invokes with new inputs check that events are re-armed."""
    rng = np.random.default_rng(31)
    B = 2
    cu = wl.hybrid_fc(B, 256, 512, seed=41)
    heads = [wl.hybrid_fc(B, 512, n, seed=42 + i) for i, n in enumerate((96, 64, 200))]
    tail = wl.hybrid_fc(B, 96, 40, seed=50)
    roots = [wl.hybrid_fc(B, 1024, 72, seed=60), wl.blockwise_int4_fc(B, 2048, 24, seed=61, lo=-8, hi=7)]
    with FakeHost() as h:
        def hybrid(x, c, n, k):
            w = h.tensor(INT8, (n, k), data=c["w"], const=True)
            h.affine(w, c["pcs"])
            y = h.tensor(FLOAT32, (B, n))
            h.fc(x, w, None, y, asymmetric=True)
            return y
        x = h.tensor(FLOAT32, (B, 256), data=cu["x"])
        up = hybrid(x, cu, 512, 256)
        ys = [hybrid(up, c, c["w"].shape[0], 512) for c in heads]
        yt = hybrid(ys[0], tail, 40, 96)
        xr0 = h.tensor(FLOAT32, (B, 1024), data=roots[0]["x"])
        yr0 = hybrid(xr0, roots[0], 72, 1024)
        xr1 = h.tensor(FLOAT32, (B, 2048), data=roots[1]["x"])
        w4 = h.tensor(INT4, (24, 2048), data=roots[1]["packed"], const=True)
        s4 = h.tensor(FLOAT16, (24, 64), data=roots[1]["scales"], const=True)
        h.blockwise(w4, s4, 32)
        yr1 = h.tensor(FLOAT32, (B, 24))
        h.fc(xr1, w4, None, yr1)
        assert h.load_delegate({"streams": streams}) == 0, h.errors()
        assert h.modify_graph_with_delegate() == OK and h.allocate_tensors() == OK, h.errors()
        assert len(h.plan()) == 1  # one partition holds all seven nodes
        for trial in range(3):
            xin = cu["x"] if trial == 0 else rng.standard_normal((B, 256)).astype(np.float32)
            h.write(x, xin)
            assert h.invoke() == OK, h.errors()
            w_up = oracle.fc_hybrid(xin, cu["w"], cu["pcs"])
            wants = [oracle.fc_hybrid(w_up, c["w"], c["pcs"]) for c in heads]
            want_tail = oracle.fc_hybrid(wants[0], tail["w"], tail["pcs"])
            for y, want in zip(ys[1:] + [yt], wants[1:] + [want_tail]):
                assert np.array_equal(h.read(y).view(np.uint32), want.view(np.uint32))
            assert np.array_equal(h.read(yr0).view(np.uint32),
                                  oracle.fc_hybrid(roots[0]["x"], roots[0]["w"], roots[0]["pcs"]).view(np.uint32))
            assert np.array_equal(
                h.read(yr1).view(np.uint32),
                oracle.fc_blockwise_int4(roots[1]["x"], roots[1]["packed"], 24,
                                         roots[1]["scales"].view(np.uint16), 32).view(np.uint32))


@pytest.mark.parametrize("streams", [1, 3])
@pytest.mark.parametrize("B", [1, 5])
def test_int4_nodes_share_grouped_launches(streams, B):
    """Blockwise-int4 nodes of one depth that do not depend on each other run as one kernel:
    {a, b, c} read the same host tensor; d reads a's output and forms a second group with two
    more host-fed nodes. Every output is compared with the oracle, over two invokes."""
    K = 64
    rng = np.random.default_rng(77)
    shapes = {"a": 64, "b": 40, "c": 8, "d": 16, "e": 24, "f": 72}
    cs = {k: wl.blockwise_int4_fc(B, K, n, seed=90 + i, lo=-8, hi=7) for i, (k, n) in enumerate(shapes.items())}
    with FakeHost() as h:
        def int4(x, c, n, bias=None):
            w = h.tensor(INT4, (n, K), data=c["packed"], const=True)
            s_ = h.tensor(FLOAT16, (n, K // 32), data=c["scales"], const=True)
            h.blockwise(w, s_, 32)
            b_ = h.tensor(FLOAT32, (n,), data=bias, const=True) if bias is not None else None
            y = h.tensor(FLOAT32, (B, n))
            h.fc(x, w, b_, y)
            return y
        bias_b = rng.standard_normal(40).astype(np.float32)
        x = h.tensor(FLOAT32, (B, K), data=cs["a"]["x"])
        ya = int4(x, cs["a"], 64)
        yb = int4(x, cs["b"], 40, bias_b)
        yc = int4(x, cs["c"], 8)
        yd = int4(ya, cs["d"], 16)
        xe = h.tensor(FLOAT32, (B, K), data=cs["e"]["x"])
        ye = int4(xe, cs["e"], 24)
        yf = int4(xe, cs["f"], 72)
        assert h.load_delegate({"streams": streams}) == 0, h.errors()
        assert h.modify_graph_with_delegate() == OK and h.allocate_tensors() == OK, h.errors()
        assert len(h.plan()) == 1
        groups, text = h.describe_partition(h.plan()[0][2])
        # a, b, c, e, f have no producer inside the partition: one launch; d follows on its own
        assert groups == 1 and text.count("/g0") == 5, text

        def ref(xin, c, n, bias=None):
            return oracle.fc_blockwise_int4(xin, c["packed"], n, c["scales"].view(np.uint16), 32, bias)
        for trial in range(2):
            xin = cs["a"]["x"] if trial == 0 else rng.standard_normal((B, K)).astype(np.float32)
            h.write(x, xin)
            assert h.invoke() == OK, h.errors()
            wa = ref(xin, cs["a"], 64)
            for y, want in ((yb, ref(xin, cs["b"], 40, bias_b)), (yc, ref(xin, cs["c"], 8)),
                            (yd, ref(wa, cs["d"], 16)), (ye, ref(cs["e"]["x"], cs["e"], 24)),
                            (yf, ref(cs["e"]["x"], cs["f"], 72))):
                assert np.array_equal(h.read(y).view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("streams", [1, 4])
def test_int4_groups_follow_dependency_levels(streams):
    """Plan order a, c(a), b, d(b), e(c): the launches are {a, b}, then {c, d}, then e --
    grouping goes by distance from the partition's inputs, not by position in the plan."""
    B, K = 2, 64
    shapes = {"a": 64, "c": 64, "b": 64, "d": 24, "e": 8}
    cs = {k: wl.blockwise_int4_fc(B, K, n, seed=40 + i, lo=-8, hi=7) for i, (k, n) in enumerate(shapes.items())}
    with FakeHost() as h:
        def int4(x, c, n):
            w = h.tensor(INT4, (n, K), data=c["packed"], const=True)
            s_ = h.tensor(FLOAT16, (n, K // 32), data=c["scales"], const=True)
            h.blockwise(w, s_, 32)
            y = h.tensor(FLOAT32, (B, n))
            h.fc(x, w, None, y)
            return y
        x = h.tensor(FLOAT32, (B, K), data=cs["a"]["x"])
        ya = int4(x, cs["a"], 64)
        yc = int4(ya, cs["c"], 64)
        yb = int4(x, cs["b"], 64)
        yd = int4(yb, cs["d"], 24)
        ye = int4(yc, cs["e"], 8)
        assert h.load_delegate({"streams": streams}) == 0, h.errors()
        assert h.modify_graph_with_delegate() == OK and h.allocate_tensors() == OK, h.errors()
        assert len(h.plan()) == 1
        groups, text = h.describe_partition(h.plan()[0][2])
        assert groups == 2 and text.count("/g0") == 2 and text.count("/g1") == 2, text

        def ref(xin, c, n):
            return oracle.fc_blockwise_int4(xin, c["packed"], n, c["scales"].view(np.uint16), 32)
        rng = np.random.default_rng(4)
        for trial in range(2):
            xin = cs["a"]["x"] if trial == 0 else rng.standard_normal((B, K)).astype(np.float32)
            h.write(x, xin)
            assert h.invoke() == OK, h.errors()
            wa, wb = ref(xin, cs["a"], 64), ref(xin, cs["b"], 64)
            wc = ref(wa, cs["c"], 64)
            # ya, yb, yc stay inside the partition (device arena); d and e are its outputs
            for y, want in ((yd, ref(wb, cs["d"], 24)), (ye, ref(wc, cs["e"], 8))):
                assert np.array_equal(h.read(y).view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("B,per_channel", [(1, True), (4, False), (40, True)])
def test_int4_per_channel_hybrid_node_through_delegate(B, per_channel):
    """EvalHybridDense4Bit: float in/out, int4 filter with affine (not blockwise) quantization."""
    from tests import kat_harness as kh
    rng = np.random.default_rng(5 + B)
    K, N = 256, 24
    x_np = rng.standard_normal((B, K)).astype(np.float32)
    w_np = rng.integers(-7, 8, (N, K)).astype(np.int8)
    packed = np.stack([kh.pack_int4(r) for r in w_np])
    fs = rng.uniform(0.01, 0.1, N).astype(np.float32) if per_channel else np.array([0.05], np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    with FakeHost() as h:
        x = h.tensor(FLOAT32, (B, K), data=x_np)
        w = h.tensor(INT4, (N, K), data=packed, const=True)
        h.affine(w, fs)
        b = h.tensor(FLOAT32, (N,), data=bias, const=True)
        y = h.tensor(FLOAT32, (B, N))
        node = h.fc(x, w, b, y, activation=1)
        assert h.classify(node)[0] == "int4_per_channel"
        assert h.load_delegate() == 0, h.errors()
        assert h.modify_graph_with_delegate() == OK and h.allocate_tensors() == OK, h.errors()
        assert h.plan()[0][:2] == ("delegate", [node])
        assert h.invoke() == OK, h.errors()
        want = oracle.fc_hybrid_int4_per_channel(x_np, packed, N, fs, bias, oracle.ACT_RELU)
        assert np.array_equal(h.read(y).view(np.uint32), want.view(np.uint32))


def test_profiling_string_names_the_partition():
    """TfLiteRegistration::profiling_string (tflite/core/c/common.h:1264-1270), which the
    profiler's summary groups executions by (profile_summarizer.cc:84-88): the node kinds of the
    partition with their counts, and its launch units."""
    c8 = wl.int8_fc(1, 128, 64, seed=3)
    ch = wl.hybrid_fc(2, 64, 32, seed=4)
    with FakeHost() as h:
        x = h.tensor(INT8, (1, 128), data=c8["x"])
        h.affine(x, [c8["in_scale"]], [c8["in_zp"]])
        w = h.tensor(INT8, (64, 128), data=c8["w"], const=True)
        h.affine(w, c8["w_scale"])
        b = h.tensor(INT32, (64,), data=c8["bias"], const=True)
        y = h.tensor(INT8, (1, 64))
        h.affine(y, [c8["out_scale"]], [c8["out_zp"]])
        n0 = h.fc(x, w, b, y)
        xs, ys = [], []
        for i in range(2):
            xf = h.tensor(FLOAT32, (2, 64), data=ch["x"])
            wf = h.tensor(INT8, (32, 64), data=ch["w"], const=True)
            h.affine(wf, ch["pcs"])
            yf = h.tensor(FLOAT32, (2, 32))
            h.fc(xf, wf, None, yf)
        assert h.profiling_string(n0) is None      # a builtin node's own registration has none here
        assert h.load_delegate() == 0, h.errors()
        assert h.modify_graph_with_delegate() == OK and h.allocate_tensors() == OK, h.errors()
        kind, replaced, node = h.plan()[0]
        assert kind == "delegate" and len(replaced) == 3
        assert h.profiling_string(node) == "int8:1 hybrid:2 launches:3"
        assert h.invoke() == OK, h.errors()
        assert h.profiling_string(node) == "int8:1 hybrid:2 launches:3"


@pytest.mark.parametrize("B,N,K,per_channel,asymmetric", [
    (1, 2, 64, True, True),      # fewer than 4 output channels
    (3, 8, 16, False, True),     # depth below 32
    (2, 5, 33, True, False),     # odd depth: nibbles packed over the flat tensor, rows not byte-aligned
    (20, 3, 48, True, True),     # prefill-sized batch on a narrow filter
])
def test_int4_affine_filter_outside_the_4bit_gate_runs_the_int8_hybrid_path(B, N, K, per_channel,
                                                                            asymmetric):
    """fully_connected.cc:609-613 keeps such shapes off EvalHybridDense4Bit; EvalHybridDense then
    unpacks the nibbles to int8 (:805-814) and runs the ordinary hybrid kernels. Oracle:
    unpack_int4 followed by fc_hybrid, both pinned on their own."""
    from tests import kat_harness as kh
    rng = np.random.default_rng(50 + N + K)
    x_np = rng.standard_normal((B, K)).astype(np.float32)
    w_np = rng.integers(-8, 8, (N, K)).astype(np.int8)
    packed = kh.pack_int4(w_np.ravel())
    fs = rng.uniform(0.01, 0.1, N).astype(np.float32) if per_channel else np.array([0.05], np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    with FakeHost() as h:
        x = h.tensor(FLOAT32, (B, K), data=x_np)
        w = h.tensor(INT4, (N, K), data=packed, const=True)
        h.affine(w, fs)
        b = h.tensor(FLOAT32, (N,), data=bias, const=True)
        y = h.tensor(FLOAT32, (B, N))
        node = h.fc(x, w, b, y, activation=3, asymmetric=asymmetric)
        assert h.classify(node)[0] == "hybrid"
        assert h.load_delegate() == 0, h.errors()
        assert h.modify_graph_with_delegate() == OK and h.allocate_tensors() == OK, h.errors()
        assert h.plan()[0][:2] == ("delegate", [node])
        assert h.invoke() == OK, h.errors()
        unpacked = oracle.unpack_int4(packed, N * K).reshape(N, K)
        assert np.array_equal(unpacked, w_np)
        want = oracle.fc_hybrid(x_np, unpacked, fs if per_channel else None,
                                1.0 if per_channel else float(fs[0]), bias, asymmetric,
                                oracle.ACT_RELU6)
        assert np.array_equal(h.read(y).view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("B,N,K,per_channel", [(1, 8, 64, True), (3, 5, 33, False), (20, 130, 272, True)])
def test_int2_filter_runs_the_int8_paths_after_unpacking(B, N, K, per_channel):
    """An Int2 filter (four values per byte over the flat tensor, rows not byte-aligned when the
    depth is odd) under float activations and under int8 ones: unpacked once at prepare
    (fully_connected.cc:812-818, 1678-1685), then the hybrid and the full-integer kernels. Oracle:
    unpack_int2 followed by fc_hybrid / fc_int8, each pinned on its own."""
    from tests import kat_harness as kh
    rng = np.random.default_rng(60 + N + K)
    w_np = rng.integers(-2, 2, (N, K)).astype(np.int8)
    packed = kh.pack_int2(w_np.ravel())
    unpacked = oracle.unpack_int2(packed.view(np.int8), N * K).reshape(N, K)
    assert np.array_equal(unpacked, w_np)
    fs = rng.uniform(0.01, 0.1, N).astype(np.float32) if per_channel else np.array([0.05], np.float32)
    # float activations
    x_np = rng.standard_normal((B, K)).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    with FakeHost() as h:
        x = h.tensor(FLOAT32, (B, K), data=x_np)
        w = h.tensor(INT2, (N, K), data=packed, const=True)
        h.affine(w, fs)
        b = h.tensor(FLOAT32, (N,), data=bias, const=True)
        y = h.tensor(FLOAT32, (B, N))
        node = h.fc(x, w, b, y, activation=1, asymmetric=True)
        assert h.classify(node)[0] == "hybrid"
        assert h.load_delegate() == 0, h.errors()
        assert h.modify_graph_with_delegate() == OK and h.allocate_tensors() == OK, h.errors()
        assert h.plan()[0][:2] == ("delegate", [node])
        assert h.invoke() == OK, h.errors()
        want = oracle.fc_hybrid(x_np, unpacked, fs if per_channel else None,
                                1.0 if per_channel else float(fs[0]), bias, True, oracle.ACT_RELU)
        assert np.array_equal(h.read(y).view(np.uint32), want.view(np.uint32))
    # int8 activations
    c = wl.int8_fc(B, K, N, in_zp=-3, seed=61 + N)
    w_scale = fs if per_channel else np.full(N, fs[0], np.float32)  # per-channel scales either way
    with FakeHost() as h:
        x = h.tensor(INT8, (B, K), data=c["x"])
        h.affine(x, [c["in_scale"]], [c["in_zp"]])
        w = h.tensor(INT2, (N, K), data=packed, const=True)
        h.affine(w, w_scale)
        b = h.tensor(INT32, (N,), data=c["bias"], const=True)
        y = h.tensor(INT8, (B, N))
        h.affine(y, [c["out_scale"]], [c["out_zp"]])
        node = h.fc(x, w, b, y, activation=1)
        assert h.classify(node)[0] == "int8"
        assert h.load_delegate() == 0, h.errors()
        assert h.modify_graph_with_delegate() == OK and h.allocate_tensors() == OK, h.errors()
        assert h.invoke() == OK, h.errors()
        c2 = dict(c, w=unpacked, w_scale=w_scale)
        assert np.array_equal(h.read(y), _oracle_int8(c2, c["x"], activation=1))


def _uint8_fc(h, rng, x, B, K, N, in_s, zx, w_s, zw, out_s, zy, activation=0, bias=True):
    """Adds a uint8 FULLY_CONNECTED node reading tensor `x`; returns (node, output tensor, weights,
    bias values)."""
    w_np = rng.integers(0, 256, (N, K)).astype(np.uint8)
    b_np = rng.integers(-3000, 3000, N).astype(np.int32) if bias else None
    w = h.tensor(UINT8, (N, K), data=w_np, const=True)
    h.affine(w, [w_s], [zw])
    b = None
    if bias:
        b = h.tensor(INT32, (N,), data=b_np, const=True)
        h.affine(b, [np.float32(in_s) * np.float32(w_s)])
    y = h.tensor(UINT8, (B, N))
    h.affine(y, [out_s], [zy])
    return h.fc(x, w, b, y, activation=activation), y, w_np, b_np


def _oracle_uint8(x, w, bias, in_s, zx, w_s, zw, out_s, zy, activation=0):
    m, s = oracle.fc_prepare_per_tensor(in_s, w_s, out_s, None)
    lo, hi = oracle.activation_range_uint8(activation, out_s, zy)
    return oracle.fc_uint8_per_tensor(x, w, bias, m, s, -zx, -zw, zy, lo, hi)


@pytest.mark.parametrize("options", [{}, {"direct_inputs": "0", "completion": "sync"}],
                         ids=["default", "copied,sync"])
@pytest.mark.parametrize("B,K,N,zw", [(1, 4096, 2048, 128), (5, 272, 130, 119), (40, 512, 72, 128)])
def test_uint8_nodes_through_delegate(B, K, N, zw, options):
    """The legacy uint8 op, one node and a chain of two whose link stays on the device as uint8:
    filter zero point 128 (the re-tiled filter once the tensors are taken as int8) and another
    (the row-major kernels), decode and prefill batches, a second invoke on new rows."""
    rng = np.random.default_rng(B + K + N)
    x_np = rng.integers(0, 256, (B, K)).astype(np.uint8)
    in_s, w_s, zx = 0.02, 0.01, 131
    s1 = float(in_s * w_s * np.sqrt(K) * 60)
    s2 = float(s1 * 0.01 * np.sqrt(N) * 60)
    with FakeHost() as h:
        x = h.tensor(UINT8, (B, K), data=x_np)
        h.affine(x, [in_s], [zx])
        n1, y1, w1, b1 = _uint8_fc(h, rng, x, B, K, N, in_s, zx, w_s, zw, s1, 7, activation=1)
        n2, y2, w2, b2 = _uint8_fc(h, rng, y1, B, N, 24, s1, 7, 0.01, 128, s2, 200, bias=False)
        assert h.classify(n1)[0] == "int8" and h.classify(n2)[0] == "int8"
        assert h.load_delegate(options) == 0, h.errors()
        assert h.modify_graph_with_delegate() == OK and h.allocate_tensors() == OK, h.errors()
        assert h.plan()[0][:2] == ("delegate", [n1, n2])
        for rows in (x_np, np.roll(x_np, 5, axis=1)):
            h.write(x, rows)
            assert h.invoke() == OK, h.errors()
            t = _oracle_uint8(rows, w1, b1, in_s, zx, w_s, zw, s1, 7, activation=1)
            want = _oracle_uint8(t, w2, None, s1, 7, 0.01, 128, s2, 200)
            assert np.array_equal(h.read(y2), want)
            assert len(np.unique(want)) > 3


def test_int4_per_channel_node_switches_layout_with_the_batch():
    """Decode batches run on the filter kept as nibbles, prefill batches on its int8 expansion;
    a resize moves the node from one to the other and back (prepare runs after every resize)."""
    from tests import kat_harness as kh
    rng = np.random.default_rng(21)
    K, N = 512, 40
    x_all = rng.standard_normal((48, K)).astype(np.float32)
    w_np = rng.integers(-7, 8, (N, K)).astype(np.int8)
    packed = np.stack([kh.pack_int4(r) for r in w_np])
    fs = rng.uniform(0.01, 0.1, N).astype(np.float32)
    with FakeHost() as h:
        x = h.tensor(FLOAT32, (1, K), data=x_all[:1])
        w = h.tensor(INT4, (N, K), data=packed, const=True)
        h.affine(w, fs)
        y = h.tensor(FLOAT32, (1, N))
        h.fc(x, w, None, y)
        assert h.load_delegate() == 0, h.errors()
        assert h.modify_graph_with_delegate() == OK and h.allocate_tensors() == OK, h.errors()
        for rows in (1, 48, 3, 20):
            h.resize(x, (rows, K))
            h.resize(y, (rows, N))
            h.write(x, x_all[:rows])
            assert h.allocate_tensors() == OK, h.errors()
            assert h.invoke() == OK, h.errors()
            want = oracle.fc_hybrid_int4_per_channel(x_all[:rows], packed, N, fs, None, 0)
            assert np.array_equal(h.read(y).view(np.uint32), want.view(np.uint32)), rows


def test_streams_option_is_validated():
    with FakeHost() as h:
        assert h.load_delegate({"streams": 9}) != 0
        assert "streams" in h.errors()


def test_shared_input_and_unclaimed_node_fall_back_to_cpu():
    """q/k/v-style fan-out from one input, plus a uint8 FC the delegate must leave alone."""
    c = wl.hybrid_fc(2, 512, 96, seed=9)
    rng = np.random.default_rng(3)
    with FakeHost() as h:
        x = h.tensor(FLOAT32, (2, 512), data=c["x"])
        outs = []
        for i in range(3):
            w = h.tensor(INT8, (32, 512), data=c["w"][32 * i:32 * i + 32], const=True)
            h.affine(w, c["pcs"][32 * i:32 * i + 32])
            y = h.tensor(FLOAT32, (2, 32))
            h.fc(x, w, None, y, asymmetric=(i != 1))
            outs.append(y)
        xu = h.tensor(UINT8, (2, 16), data=rng.integers(0, 255, (2, 16)).astype(np.uint8))
        wu = h.tensor(UINT8, (4, 16), data=rng.integers(0, 255, (4, 16)).astype(np.uint8), const=True)
        h.affine(wu, [0.01], [128])
        yu = h.tensor(UINT8, (2, 4))
        nu = h.fc(xu, wu, None, yu)
        ran = []
        from tests.fake_host import CPU_CB
        cb = CPU_CB(lambda n: (ran.append(n), 0)[1])
        h.L.fh_set_cpu_callback(h.h, cb)
        assert h.load_delegate() == 0, h.errors()
        assert h.modify_graph_with_delegate() == OK and h.allocate_tensors() == OK, h.errors()
        assert [k for k, _, _ in h.plan()] == ["delegate", "cpu"]
        assert h.invoke() == OK, h.errors()
        assert ran == [nu]
        for i, y in enumerate(outs):
            want = oracle.fc_hybrid(c["x"], c["w"][32 * i:32 * i + 32], c["pcs"][32 * i:32 * i + 32],
                                    asymmetric=(i != 1))
            assert np.array_equal(h.read(y).view(np.uint32), want.view(np.uint32))


def test_claim_option_and_quant_variant_option():
    c = wl.int8_fc(2, 64, 16, seed=4)
    ch = wl.hybrid_fc(1, 72, 8, seed=5)  # 72 = 8 * 9: no ragged tail, ties still differ by variant
    ch["x"][0, :4] = [-125.0, 130.0, 2.5, 0.0]  # scale 1, zero point -3, one exact tie
    ch["x"][0, 4:] = np.clip(ch["x"][0, 4:], -100, 100)
    with FakeHost() as h:
        n_int8, _, _ = _add_int8_fc(h, c)
        x = h.tensor(FLOAT32, (1, 72), data=ch["x"])
        w = h.tensor(INT8, (8, 72), data=ch["w"], const=True)
        h.affine(w, ch["pcs"])
        y = h.tensor(FLOAT32, (1, 8))
        n_h = h.fc(x, w, None, y)
        ran = h.use_oracle_for_cpu_nodes()
        assert h.load_delegate({"claim": "hybrid", "quant_variant": "neon_v8"}) == 0, h.errors()
        assert h.modify_graph_with_delegate() == OK and h.allocate_tensors() == OK, h.errors()
        assert [(k, r) for k, r, _ in h.plan()] == [("cpu", [n_int8]), ("delegate", [n_h])]
        assert h.invoke() == OK, h.errors()
        assert ran == [n_int8]
        want_v8 = oracle.fc_hybrid(ch["x"], ch["w"], ch["pcs"], variant=oracle.QUANT_NEON_V8)
        want_p = oracle.fc_hybrid(ch["x"], ch["w"], ch["pcs"], variant=oracle.QUANT_PORTABLE)
        got = h.read(y)
        assert np.array_equal(got.view(np.uint32), want_v8.view(np.uint32))
        assert not np.array_equal(want_v8, want_p)  # the option is observable


def test_resize_then_reprepare():
    c = wl.hybrid_fc(4, 256, 64, seed=6)
    with FakeHost() as h:
        x = h.tensor(FLOAT32, (1, 256), data=c["x"][:1])
        w = h.tensor(INT8, (64, 256), data=c["w"], const=True)
        h.affine(w, c["pcs"])
        y = h.tensor(FLOAT32, (1, 64))
        h.fc(x, w, None, y)
        assert h.load_delegate() == 0, h.errors()
        assert h.modify_graph_with_delegate() == OK and h.allocate_tensors() == OK, h.errors()
        assert h.invoke() == OK
        assert np.array_equal(h.read(y), oracle.fc_hybrid(c["x"][:1], c["w"], c["pcs"]))
        h.resize(x, (4, 256))
        h.resize(y, (4, 64))
        h.write(x, c["x"])
        assert h.allocate_tensors() == OK, h.errors()  # prepare runs again after a resize
        assert h.invoke() == OK, h.errors()
        assert np.array_equal(h.read(y), oracle.fc_hybrid(c["x"], c["w"], c["pcs"]))


def test_blockwise_int4_other_block_size_keeps_model_layout():
    c = wl.blockwise_int4_fc(2, 256, 24, blocksize=64, lo=-8, hi=7)
    with FakeHost() as h:
        x = h.tensor(FLOAT32, (2, 256), data=c["x"])
        w = h.tensor(INT4, (24, 256), data=c["packed"], const=True)
        s = h.tensor(FLOAT16, (24, 4), data=c["scales"], const=True)
        h.blockwise(w, s, 64)
        y = h.tensor(FLOAT32, (2, 24))
        h.fc(x, w, None, y)
        assert h.load_delegate() == 0, h.errors()
        assert h.modify_graph_with_delegate() == OK and h.allocate_tensors() == OK, h.errors()
        assert h.invoke() == OK, h.errors()
        want = oracle.fc_blockwise_int4(c["x"], c["packed"], 24, c["scales"].view(np.uint16), 64)
        assert np.array_equal(h.read(y).view(np.uint32), want.view(np.uint32))


def test_int8_resize_between_decode_and_prefill():
    """One row runs the GEMV, 128 rows the MFMA GEMM, 3 rows the GEMV again, all on the same
    re-tiled filter; prepare runs after every resize. Each step is checked against the oracle."""
    c = wl.int8_fc(128, 256, 256, seed=9)
    with FakeHost() as h:
        B, K = c["x"].shape
        N = c["w"].shape[0]
        x = h.tensor(INT8, (1, K), data=c["x"][:1])
        h.affine(x, [c["in_scale"]], [c["in_zp"]])
        w = h.tensor(INT8, (N, K), data=c["w"], const=True)
        h.affine(w, c["w_scale"])
        b = h.tensor(INT32, (N,), data=c["bias"], const=True)
        y = h.tensor(INT8, (1, N))
        h.affine(y, [c["out_scale"]], [c["out_zp"]])
        h.fc(x, w, b, y)
        assert h.load_delegate() == 0, h.errors()
        assert h.modify_graph_with_delegate() == OK and h.allocate_tensors() == OK, h.errors()
        for rows in (1, 128, 3):
            h.resize(x, (rows, K))
            h.resize(y, (rows, N))
            h.write(x, c["x"][:rows])
            assert h.allocate_tensors() == OK, h.errors()
            assert h.invoke() == OK, h.errors()
            assert np.array_equal(h.read(y), _oracle_int8(c, c["x"][:rows])), rows


def test_wide_hybrid_node_resized_through_every_row_regime():
    """A hybrid node wide enough for every kernel the row count can select (10240 channels): the
    fused GEMV (1, 8 rows), quantizer + register-resident GEMV (16, 24 rows), the GEMV that walks
    the rows through LDS in depth chunks (40, 100 rows), the MFMA GEMM (150 rows), then back to one
    row; all on one re-tiled filter, each against the oracle bit for bit."""
    K, N = 1040, 10240
    c = wl.hybrid_fc(150, K, N, seed=77)
    bias = np.random.default_rng(2).standard_normal(N).astype(np.float32)
    with FakeHost() as h:
        x = h.tensor(FLOAT32, (1, K), data=c["x"][:1])
        w = h.tensor(INT8, (N, K), data=c["w"], const=True)
        h.affine(w, c["pcs"])
        b = h.tensor(FLOAT32, (N,), data=bias, const=True)
        y = h.tensor(FLOAT32, (1, N))
        h.fc(x, w, b, y, activation=1, asymmetric=True)
        assert h.load_delegate() == 0, h.errors()
        assert h.modify_graph_with_delegate() == OK and h.allocate_tensors() == OK, h.errors()
        for rows in (1, 8, 16, 24, 40, 100, 150, 1):
            h.resize(x, (rows, K))
            h.resize(y, (rows, N))
            h.write(x, c["x"][:rows])
            assert h.allocate_tensors() == OK, h.errors()
            assert h.invoke() == OK, h.errors()
            want = oracle.fc_hybrid(c["x"][:rows], c["w"], c["pcs"], 1.0, bias, True, oracle.ACT_RELU)
            assert np.array_equal(h.read(y).view(np.uint32), want.view(np.uint32)), rows


def test_prepare_failure_is_reported_not_hidden():
    """An output tensor whose shape cannot hold batches x channels makes the delegate
    kernel's prepare fail with a message, like a builtin kernel's Prepare would."""
    c = wl.hybrid_fc(2, 64, 8, seed=7)
    with FakeHost() as h:
        x = h.tensor(FLOAT32, (2, 64), data=c["x"])
        w = h.tensor(INT8, (8, 64), data=c["w"], const=True)
        h.affine(w, c["pcs"])
        y = h.tensor(FLOAT32, (2, 7))
        h.fc(x, w, None, y)
        assert h.load_delegate() == 0
        assert h.modify_graph_with_delegate() == OK
        assert h.allocate_tensors() != OK
        assert "output shape does not hold" in h.errors()


def test_empty_graph_and_nothing_to_claim():
    with FakeHost() as h:
        a, b = h.tensor(FLOAT32, (1, 4)), h.tensor(FLOAT32, (1, 4))
        h.other(0, a, b)
        assert h.load_delegate() == 0
        assert h.modify_graph_with_delegate() == OK
        assert [k for k, _, _ in h.plan()] == ["cpu"]


# ---- EMBEDDING_LOOKUP from quantized tables ---------------------------------------------------

def _lookup_table(rng, rows, cols, bs):
    packed = rng.integers(0, 256, (rows, cols // 2), dtype=np.uint8)
    scales = (rng.random((rows, cols // bs), dtype=np.float32) * 2e-2 + 1e-3).astype(np.float16)
    return packed, scales


@pytest.mark.parametrize("out_f16", [False, True])
@pytest.mark.parametrize("count", [1, 37])
def test_blockwise_embedding_lookup_node_through_delegate(count, out_f16):
    rng = np.random.default_rng(21 + count)
    rows, cols, bs = 500, 2048, 32
    packed, scales = _lookup_table(rng, rows, cols, bs)
    lookup = rng.integers(0, rows, count).astype(np.int32)
    with FakeHost() as h:
        lk = h.tensor(INT32, (count,), data=lookup)
        v = h.tensor(INT4, (rows, cols), data=packed, const=True)
        s = h.tensor(FLOAT16, (rows, cols // bs), data=scales, const=True)
        h.blockwise(v, s, bs)
        y = h.tensor(FLOAT16 if out_f16 else FLOAT32, (count, cols))
        node = h.embedding_lookup(lk, v, y)
        assert h.load_delegate() == 0, h.errors()
        assert h.modify_graph_with_delegate() == OK and h.allocate_tensors() == OK, h.errors()
        assert h.plan()[0][:2] == ("delegate", [node])
        assert h.invoke() == OK, h.errors()
        want = oracle.embedding_lookup_blockwise_int4(lookup, packed, rows, cols,
                                                      scales.view(np.uint16), bs, out_f16)
        assert np.array_equal(h.read(y).view(want.dtype), want)
        # other tokens on the next invoke; a token outside the table fails it as the builtin does
        lookup2 = rng.integers(0, rows, count).astype(np.int32)
        h.write(lk, lookup2)
        assert h.invoke() == OK, h.errors()
        want = oracle.embedding_lookup_blockwise_int4(lookup2, packed, rows, cols,
                                                      scales.view(np.uint16), bs, out_f16)
        assert np.array_equal(h.read(y).view(want.dtype), want)
        lookup2[-1] = rows
        h.write(lk, lookup2)
        assert h.invoke() != OK
        assert "Embedding Lookup: index out of bounds. Got 500, and bounds are [0, 499]" in h.errors()
        lookup2[-1] = 0
        h.write(lk, lookup2)
        assert h.invoke() == OK, h.errors()


@pytest.mark.parametrize("bits,per_row,shape", [(8, True, (40, 96)), (8, False, (40, 4, 24)),
                                                (4, True, (40, 96)), (4, False, (40, 50))])
def test_affine_embedding_lookup_node_through_delegate(bits, per_row, shape):
    rng = np.random.default_rng(bits + shape[-1])
    rows, cols = shape[0], int(np.prod(shape[1:]))
    table = (rng.integers(0, 256, (rows, cols // 2), dtype=np.uint8) if bits == 4
             else rng.integers(-128, 128, (rows, cols), dtype=np.int8))
    scales = (rng.random(rows if per_row else 1, dtype=np.float32) * 0.02 + 1e-3)
    lookup = rng.integers(0, rows, 9).astype(np.int32)
    with FakeHost() as h:
        lk = h.tensor(INT32, (9,), data=lookup)
        v = h.tensor(INT4 if bits == 4 else INT8, shape, data=table, const=True)
        h.affine(v, scales)
        y = h.tensor(FLOAT32, (9,) + shape[1:])
        h.embedding_lookup(lk, v, y)
        assert h.load_delegate() == 0, h.errors()
        assert h.modify_graph_with_delegate() == OK and h.allocate_tensors() == OK, h.errors()
        assert h.invoke() == OK, h.errors()
        got = h.read(y)
    want = oracle.embedding_lookup_hybrid(lookup, table, bits, rows, cols, scale=float(scales[0]),
                                          row_scales=scales if per_row else None)
    assert got.shape == (9,) + shape[1:]
    assert np.array_equal(got.reshape(9, cols).view(np.uint32), want.view(np.uint32))


def test_embedding_lookup_feeds_projections_inside_one_partition():
    """Token ids -> embedding rows -> the q/k/v projections of a decoder's first layer, all
    blockwise Int4: one partition, the rows never leave the device, results as the oracle's
    chain of the two builtins."""
    rng = np.random.default_rng(77)
    rows, K, bs, B = 1000, 2048, 32, 4
    packed, scales = _lookup_table(rng, rows, K, bs)
    lookup = rng.integers(0, rows, B).astype(np.int32)
    projections = [wl.blockwise_int4_fc(B, K, n, seed=5 + i) for i, n in enumerate((2048, 256, 256))]
    with FakeHost() as h:
        lk = h.tensor(INT32, (B,), data=lookup)
        v = h.tensor(INT4, (rows, K), data=packed, const=True)
        s = h.tensor(FLOAT16, (rows, K // bs), data=scales, const=True)
        h.blockwise(v, s, bs)
        x = h.tensor(FLOAT32, (B, K))
        h.embedding_lookup(lk, v, x)
        outs = []
        for c in projections:
            n = c["packed"].shape[0]
            w = h.tensor(INT4, (n, K), data=c["packed"], const=True)
            ws = h.tensor(FLOAT16, (n, K // 32), data=c["scales"], const=True)
            h.blockwise(w, ws, 32)
            y = h.tensor(FLOAT32, (B, n))
            h.fc(x, w, None, y)
            h.mark_output(y)
            outs.append(y)
        assert h.load_delegate() == 0, h.errors()
        assert h.modify_graph_with_delegate() == OK and h.allocate_tensors() == OK, h.errors()
        assert len(h.plan()) == 1 and h.plan()[0][0] == "delegate"
        assert h.invoke() == OK, h.errors()
        rows_f32 = oracle.embedding_lookup_blockwise_int4(lookup, packed, rows, K,
                                                          scales.view(np.uint16), bs)
        for c, y in zip(projections, outs):
            want = oracle.fc_blockwise_int4(rows_f32, c["packed"], c["packed"].shape[0],
                                            c["scales"].view(np.uint16), 32)
            assert np.array_equal(h.read(y).view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("B,K", [(3, 8192), (4, 2048)])
def test_int4_grouped_nodes_with_more_than_two_rows(B, K):
    """Independent blockwise-int4 nodes with three or four batch rows share one launch as well;
    above depth 4096 the group quantizes all its rows in a launch of its own (per-node
    workspaces owned by the partition). Outputs bit-identical to the oracle over two invokes."""
    Ns = (16, 24, 8)
    cs = [wl.blockwise_int4_fc(B, K, n, seed=300 + n, lo=-8, hi=7) for n in Ns]
    rng = np.random.default_rng(5)
    with FakeHost() as h:
        xs, ys = [], []
        for c, n in zip(cs, Ns):
            x = h.tensor(FLOAT32, (B, K), data=c["x"])
            w = h.tensor(INT4, (n, K), data=c["packed"], const=True)
            s_ = h.tensor(FLOAT16, (n, K // 32), data=c["scales"], const=True)
            h.blockwise(w, s_, 32)
            y = h.tensor(FLOAT32, (B, n))
            h.fc(x, w, None, y)
            xs.append(x)
            ys.append(y)
        assert h.load_delegate() == 0, h.errors()
        assert h.modify_graph_with_delegate() == OK and h.allocate_tensors() == OK, h.errors()
        groups, text = h.describe_partition(h.plan()[0][2])
        assert groups == 1 and text.count("/g0") == 3, text
        for trial in range(2):
            ins = [c["x"] if trial == 0 else rng.standard_normal((B, K)).astype(np.float32) for c in cs]
            for x, v in zip(xs, ins):
                h.write(x, v)
            assert h.invoke() == OK, h.errors()
            for c, n, y, v in zip(cs, Ns, ys, ins):
                want = oracle.fc_blockwise_int4(v, c["packed"], n, c["scales"].view(np.uint16), 32)
                assert np.array_equal(h.read(y).view(np.uint32), want.view(np.uint32)), (trial, n)


def test_int4_wide_deep_group_runs_on_the_4bit_resident_form_and_leaves_it_on_resize():
    """Two independent nodes of 8200 channels and depth 8224 at four rows: a group wide and deep
    enough for the library to prefer the filters kept at 4 bits per weight for the matrix cores
    (lrtfc_int4_group_preferred_form); the partition packs that form for the group's members
    ("n" behind the group in the description). At two rows the same group runs on the decode
    tiling. Bit-identical to the oracle both ways."""
    K, Ns = 8224, (8200, 8200)
    cs = [wl.blockwise_int4_fc(4, K, n, seed=700 + i, lo=-8, hi=7) for i, n in enumerate(Ns)]
    with FakeHost() as h:
        xs, ys = [], []
        for c, n in zip(cs, Ns):
            x = h.tensor(FLOAT32, (4, K), data=c["x"])
            w = h.tensor(INT4, (n, K), data=c["packed"], const=True)
            s_ = h.tensor(FLOAT16, (n, K // 32), data=c["scales"], const=True)
            h.blockwise(w, s_, 32)
            y = h.tensor(FLOAT32, (4, n))
            h.fc(x, w, None, y)
            xs.append(x)
            ys.append(y)
        assert h.load_delegate() == 0, h.errors()
        assert h.modify_graph_with_delegate() == OK and h.allocate_tensors() == OK, h.errors()
        for rows in (4, 2, 3):
            for c, n, x, y in zip(cs, Ns, xs, ys):
                h.resize(x, (rows, K))
                h.resize(y, (rows, n))
                h.write(x, c["x"][:rows])
            assert h.allocate_tensors() == OK, h.errors()
            groups, text = h.describe_partition(h.plan()[0][2])
            assert groups == 1 and text.count("/g0n") == (2 if rows >= 3 else 0), (rows, text)
            assert h.invoke() == OK, h.errors()
            for c, n, y in zip(cs, Ns, ys):
                want = oracle.fc_blockwise_int4(c["x"][:rows], c["packed"], n,
                                                c["scales"].view(np.uint16), 32)
                assert np.array_equal(h.read(y).view(np.uint32), want.view(np.uint32)), (rows, n)


def test_blockwise_int4_resize_between_decode_and_prefill():
    """Two rows run the streaming kernel, 40 rows the matrix-core GEMM (the filter is re-tiled
    for it at that prepare), 3 rows the streaming kernel again. Every step bit-identical to the
    oracle; two independent nodes, so the decode steps share a grouped launch."""
    K, Ns = 256, (24, 72)
    cs = [wl.blockwise_int4_fc(40, K, n, seed=60 + n, lo=-8, hi=7) for n in Ns]
    with FakeHost() as h:
        xs, ys = [], []
        for c, n in zip(cs, Ns):
            x = h.tensor(FLOAT32, (2, K), data=c["x"][:2])
            w = h.tensor(INT4, (n, K), data=c["packed"], const=True)
            s_ = h.tensor(FLOAT16, (n, K // 32), data=c["scales"], const=True)
            h.blockwise(w, s_, 32)
            y = h.tensor(FLOAT32, (2, n))
            h.fc(x, w, None, y)
            xs.append(x)
            ys.append(y)
        assert h.load_delegate() == 0, h.errors()
        assert h.modify_graph_with_delegate() == OK and h.allocate_tensors() == OK, h.errors()
        for rows in (2, 40, 3, 16):
            for c, n, x, y in zip(cs, Ns, xs, ys):
                h.resize(x, (rows, K))
                h.resize(y, (rows, n))
                h.write(x, c["x"][:rows])
            assert h.allocate_tensors() == OK, h.errors()
            groups, _ = h.describe_partition(h.plan()[0][2])
            assert groups == (0 if rows >= 16 else 1), rows
            assert h.invoke() == OK, h.errors()
            for c, n, y in zip(cs, Ns, ys):
                want = oracle.fc_blockwise_int4(c["x"][:rows], c["packed"], n,
                                                c["scales"].view(np.uint16), 32)
                assert np.array_equal(h.read(y).view(np.uint32), want.view(np.uint32)), (rows, n)


def test_completion_mark_follows_the_work_enqueued_before_it():
    """lrtfc_mark_completion: the word turns into the value only after the kernel in front of it
    on the stream has written its output, so a host that has seen the value reads the output."""
    import time
    from litert_amd import capi
    lib = capi.load()
    capi.init(0)
    c = wl.hybrid_fc(1, 4096, 1024)
    x = torch.from_numpy(c["x"]).cuda()
    w = torch.from_numpy(c["w"]).cuda()
    pcs = torch.from_numpy(c["pcs"]).cuda()
    sums = torch.from_numpy(c["w"].astype(np.int32).sum(1).astype(np.int32)).cuda()
    y = torch.zeros((1, 1024), dtype=torch.float32).pin_memory()
    word = torch.zeros(16, dtype=torch.int32).pin_memory()
    ws = torch.empty(lib.lrtfc_activation_workspace_bytes(1, 4096), dtype=torch.uint8, device="cuda")
    torch.cuda.synchronize()
    stream = torch.cuda.current_stream().cuda_stream
    want = oracle.fc_hybrid(c["x"], c["w"], c["pcs"])
    for serial in (7, 8, 0x7FFFFFFF):
        y.zero_()
        rc = lib.lrtfc_fc_hybrid(x.data_ptr(), w.data_ptr(), pcs.data_ptr(), 1.0, sums.data_ptr(), None,
                                 y.data_ptr(), 1, 4096, 1024, 1, 0, capi.QUANT_PORTABLE,
                                 ws.data_ptr(), ws.numel(), stream)
        capi.check(rc)
        capi.check(lib.lrtfc_mark_completion(word.data_ptr(), serial, stream))
        deadline = time.perf_counter() + 5.0
        while int(word[0]) != serial and time.perf_counter() < deadline:
            pass
        assert int(word[0]) == serial
        assert np.array_equal(y.numpy().view(np.uint32), want.view(np.uint32))
    torch.cuda.synchronize()
    assert lib.lrtfc_mark_completion(None, 1, stream) != 0
    assert lib.lrtfc_mark_completion(word.data_ptr() + 2, 1, stream) != 0

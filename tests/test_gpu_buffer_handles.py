"""Buffer handles of the delegate (TfLiteDelegate::CopyFromBufferHandle / CopyToBufferHandle /
FreeBufferHandle, tflite/core/c/common.h:1458-1479) driven the way the runtime drives them
(Interpreter::SetBufferHandle subgraph.cc:2784-2800, EnsureTensorDataIsReadable :876-889, the
stale-input check before each node :1724-1734): tensors bound to registered device memory stay
in HBM, and the host copy is only refreshed when somebody asks for it."""
import numpy as np
import pytest

import oracle
from litert_amd import workloads as wl
from tests.fake_host import CPU_CB, FLOAT16, FLOAT32, INT4, INT8, OK, FakeHost

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _need_gpu():
    if not torch.cuda.is_available():
        pytest.fail("GPU tests need a gfx950 device; none visible")


def _hybrid_node(h, c, x=None):
    B, K = c["x"].shape
    N = c["w"].shape[0]
    if x is None:
        x = h.tensor(FLOAT32, (B, K), data=c["x"])
    w = h.tensor(INT8, (N, K), data=c["w"], const=True)
    h.affine(w, c["pcs"])
    y = h.tensor(FLOAT32, (B, N))
    node = h.fc(x, w, None, y, asymmetric=True)
    return node, x, y


def _hybrid_ref(c, x):
    return oracle.fc_hybrid(x, c["w"], c["pcs"], 1.0, None, True, 0)


def _bits(a):
    return np.ascontiguousarray(a).view(np.uint32)


def test_bound_output_stays_on_device_until_asked_for():
    c = wl.hybrid_fc(3, 256, 72, seed=5)
    want = _hybrid_ref(c, c["x"])
    with FakeHost() as h:
        _, x, y = _hybrid_node(h, c)
        assert h.load_delegate() == 0, h.errors()
        assert h.modify_graph_with_delegate() == OK and h.allocate_tensors() == OK, h.errors()
        dev = torch.zeros(3 * 72, dtype=torch.float32, device="cuda")
        handle = h.register_device_buffer(dev.data_ptr(), dev.numel() * 4)
        assert handle == 0 and h.set_buffer_handle(y, handle) == OK
        h.write(y, np.full((3, 72), 7.0, np.float32))
        assert h.invoke() == OK, h.errors()
        assert h.data_is_stale(y)                            # the kernel said: host copy is old
        assert np.all(h.read(y) == 7.0)                      # ... and did not touch it
        assert np.array_equal(_bits(dev.cpu().numpy().reshape(3, 72)), _bits(want))
        assert h.ensure_readable(y) == OK and not h.data_is_stale(y)
        assert np.array_equal(_bits(h.read(y)), _bits(want))
        # a second invoke with new input refreshes the device copy and marks stale again
        x2 = np.random.default_rng(2).standard_normal((3, 256)).astype(np.float32)
        h.write(x, x2)
        assert h.invoke() == OK and h.data_is_stale(y)
        assert np.array_equal(_bits(dev.cpu().numpy().reshape(3, 72)), _bits(_hybrid_ref(c, x2)))


def test_bound_input_is_read_from_device_memory():
    c = wl.hybrid_fc(2, 128, 40, seed=6)
    with FakeHost() as h:
        _, x, y = _hybrid_node(h, c)
        assert h.load_delegate() == 0, h.errors()
        assert h.modify_graph_with_delegate() == OK and h.allocate_tensors() == OK, h.errors()
        x_dev_np = np.random.default_rng(9).standard_normal((2, 128)).astype(np.float32)
        dev = torch.from_numpy(x_dev_np).cuda()
        assert h.set_buffer_handle(x, h.register_device_buffer(dev.data_ptr(), dev.numel() * 4)) == OK
        h.set_data_is_stale(x)                               # host copy (c["x"]) is not the input
        assert h.invoke() == OK, h.errors()
        assert np.array_equal(_bits(h.read(y)), _bits(_hybrid_ref(c, x_dev_np)))
        # CopyToBufferHandle pushes the host copy into the bound memory
        assert h.copy_to_buffer_handle(x) == OK
        assert np.array_equal(dev.cpu().numpy(), c["x"])
        assert h.invoke() == OK
        assert np.array_equal(_bits(h.read(y)), _bits(_hybrid_ref(c, c["x"])))


def test_partitions_chained_through_a_device_buffer():
    """FC_a | foreign op (unrelated) | FC_b(FC_a's output): two partitions. The link tensor is
    bound to device memory: partition 1 leaves it there, partition 2 reads it from there, and
    its host copy is never written; the CPU node in between reads another stale tensor, which
    the host fetches through CopyFromBufferHandle first."""
    ca = wl.hybrid_fc(2, 128, 64, seed=11)
    cb = wl.hybrid_fc(2, 64, 24, seed=12)
    cc = wl.hybrid_fc(2, 128, 16, seed=13)
    with FakeHost() as h:
        na, x, link = _hybrid_node(h, ca)
        nc, _, side = _hybrid_node(h, cc, x=x)
        side_copy = h.tensor(FLOAT32, (2, 16))
        other = h.other(0, side, side_copy)
        nb, _, y = _hybrid_node(h, cb, x=link)
        seen = []

        def cpu(node):
            seen.append(h.read(side).copy())
            h.write(side_copy, h.read(side))
            return 0
        cb_ = CPU_CB(cpu)
        h.L.fh_set_cpu_callback(h.h, cb_)
        assert h.load_delegate() == 0, h.errors()
        assert h.modify_graph_with_delegate() == OK, h.errors()
        assert [(k, r) for k, r, _ in h.plan()] == [("delegate", [na, nc]), ("cpu", [other]),
                                                    ("delegate", [nb])]
        assert h.allocate_tensors() == OK, h.errors()
        link_dev = torch.zeros(2 * 64, dtype=torch.float32, device="cuda")
        side_dev = torch.zeros(2 * 16, dtype=torch.float32, device="cuda")
        assert h.set_buffer_handle(link, h.register_device_buffer(link_dev.data_ptr(), 2 * 64 * 4)) == OK
        assert h.set_buffer_handle(side, h.register_device_buffer(side_dev.data_ptr(), 2 * 16 * 4)) == OK
        h.write(link, np.full((2, 64), -3.0, np.float32))
        assert h.invoke() == OK, h.errors()
        wa = _hybrid_ref(ca, ca["x"])
        assert np.array_equal(_bits(h.read(y)), _bits(_hybrid_ref(cb, wa)))
        assert np.all(h.read(link) == -3.0) and h.data_is_stale(link)   # never came back to the host
        assert np.array_equal(_bits(seen[0]), _bits(_hybrid_ref(cc, ca["x"])))  # fetched for the CPU node
        assert not h.data_is_stale(side)


def test_handles_are_freed_and_slots_reused():
    c = wl.hybrid_fc(1, 64, 8, seed=3)
    with FakeHost() as h:
        _, x, y = _hybrid_node(h, c)
        assert h.load_delegate() == 0, h.errors()
        assert h.modify_graph_with_delegate() == OK and h.allocate_tensors() == OK, h.errors()
        a = torch.zeros(8, dtype=torch.float32, device="cuda")
        b = torch.zeros(8, dtype=torch.float32, device="cuda")
        small = torch.zeros(2, dtype=torch.float32, device="cuda")
        h0 = h.register_device_buffer(a.data_ptr(), 32)
        h1 = h.register_device_buffer(b.data_ptr(), 32)
        assert (h0, h1) == (0, 1)
        assert h.set_buffer_handle(y, h0) == OK
        assert h.set_buffer_handle(y, h1) == OK             # frees h0 (subgraph.cc:2792-2796)
        assert h.register_device_buffer(small.data_ptr(), 8) == 0   # the freed slot is reused
        assert h.invoke() == OK, h.errors()
        assert np.array_equal(_bits(b.cpu().numpy().reshape(1, 8)), _bits(_hybrid_ref(c, c["x"])))
        assert a.eq(0).all()
        # a registered range smaller than the tensor is an error, not an overrun
        assert h.set_buffer_handle(y, 0) == OK
        assert h.invoke() != OK and "holds 8 bytes" in h.errors()
        assert h.register_device_buffer(None, 16) == -1


def _int4_nodes(h, rng, shapes, b):
    nodes = []
    for k, n in shapes:
        x_np = rng.standard_normal((b, k)).astype(np.float32)
        packed = rng.integers(0, 256, (n, k // 2), dtype=np.uint8)
        scales = rng.uniform(5e-3, 2e-2, (n, k // 32)).astype(np.float16)
        x = h.tensor(FLOAT32, (b, k), data=x_np)
        w = h.tensor(INT4, (n, k), const=True, data=packed)
        s = h.tensor(FLOAT16, (n, k // 32), const=True, data=scales)
        h.blockwise(w, s, 32)
        y = h.tensor(FLOAT32, (b, n))
        h.fc(x, w, None, y)
        nodes.append((x, y, x_np, packed, scales, n))
    return nodes


@pytest.mark.parametrize("b", [1, 4])
def test_grouped_launch_works_in_place_on_bound_tensors_and_follows_rebinding(b):
    """A partition of independent blockwise-int4 nodes runs as one grouped launch whose address
    table names each member's tensors. Bound tensors are used where they are (no copy into the
    partition's own memory): the table must name the registered memory, and name the new
    memory after a tensor is bound to another buffer between two invokes."""
    rng = np.random.default_rng(40 + b)
    with FakeHost() as h:
        nodes = _int4_nodes(h, rng, [(2048, 256), (2048, 512), (2048, 64)], b)
        assert h.load_delegate() == 0, h.errors()
        assert h.modify_graph_with_delegate() == OK and h.allocate_tensors() == OK, h.errors()
        plan = h.plan()
        assert len(plan) == 1 and h.describe_partition(plan[0][2])[0] >= 1
        want = [oracle.fc_blockwise_int4(x_np, packed, n, scales.view(np.uint16), 32)
                for _, _, x_np, packed, scales, n in nodes]
        x_dev = [torch.from_numpy(x_np).cuda() for _, _, x_np, _, _, _ in nodes]
        y_dev = [torch.full((b, n), float("nan"), dtype=torch.float32, device="cuda")
                 for *_, n in nodes]
        for (x, y, *_), xd, yd in zip(nodes, x_dev, y_dev):
            assert h.set_buffer_handle(x, h.register_device_buffer(xd.data_ptr(), xd.numel() * 4)) == OK
            h.set_data_is_stale(x)
            h.write(x, np.zeros_like(xd.cpu().numpy()))      # the host copy is not the input
            assert h.set_buffer_handle(y, h.register_device_buffer(yd.data_ptr(), yd.numel() * 4)) == OK
        assert h.invoke() == OK, h.errors()
        for (x, y, *_), yd, w in zip(nodes, y_dev, want):
            assert h.data_is_stale(y)
            assert np.array_equal(_bits(yd.cpu().numpy()), _bits(w))
        # the second node's output moves to other memory, its input too
        y_new = torch.full_like(y_dev[1], float("nan"))
        x_new_np = rng.standard_normal(x_dev[1].shape).astype(np.float32)
        x_new = torch.from_numpy(x_new_np).cuda()
        y_dev[1].fill_(float("nan"))
        assert h.set_buffer_handle(nodes[1][1], h.register_device_buffer(y_new.data_ptr(), y_new.numel() * 4)) == OK
        assert h.set_buffer_handle(nodes[1][0], h.register_device_buffer(x_new.data_ptr(), x_new.numel() * 4)) == OK
        assert h.invoke() == OK, h.errors()
        _, _, _, packed, scales, n = nodes[1]
        assert np.array_equal(_bits(y_new.cpu().numpy()),
                              _bits(oracle.fc_blockwise_int4(x_new_np, packed, n, scales.view(np.uint16), 32)))
        assert torch.isnan(y_dev[1]).all()                    # the old memory is no longer written
        assert np.array_equal(_bits(y_dev[0].cpu().numpy()), _bits(want[0]))
        assert np.array_equal(_bits(y_dev[2].cpu().numpy()), _bits(want[2]))
        # host tensors still work beside bound ones: read a stale output back through the runtime
        assert h.ensure_readable(nodes[0][1]) == OK
        assert np.array_equal(_bits(h.read(nodes[0][1])), _bits(want[0]))


def test_output_bound_over_an_input_is_refused():
    c = wl.hybrid_fc(2, 64, 64, seed=8)
    with FakeHost() as h:
        _, x, y = _hybrid_node(h, c)
        assert h.load_delegate() == 0, h.errors()
        assert h.modify_graph_with_delegate() == OK and h.allocate_tensors() == OK, h.errors()
        dev = torch.from_numpy(c["x"]).cuda()
        assert h.set_buffer_handle(x, h.register_device_buffer(dev.data_ptr(), dev.numel() * 4)) == OK
        h.set_data_is_stale(x)
        assert h.set_buffer_handle(y, h.register_device_buffer(dev.data_ptr(), dev.numel() * 4)) == OK
        assert h.invoke() != OK and "overlapping device memory" in h.errors()

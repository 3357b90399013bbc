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

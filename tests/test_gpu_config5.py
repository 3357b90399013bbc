"""Parity at the geometry of the Gemma-2B-shaped FC chain: 18 layers x 7 FULLY_CONNECTED nodes
(q 2048->2048, k/v 2048->256, o 2048->2048, gate/up 2048->16384, down 16384->2048), blockwise
int4 weights (block 32, fp16 scales), float32 activations from N(0,1), decode batch 1 and 4.

Every output of every node is compared bit for bit with the oracle's restatement of
EvalBlockwise4Bit (tflite/kernels/fully_connected.cc:1014-1086), for the two ways the chain is
run: (1) as one 126-node partition through the delegate plugin, driven by the stand-in
interpreter, host tensors in and out; (2) as the grouped launches the benchmark times: the 108
nodes of depth 2048 in one launch and the 18 down projections in another, each node with its
own input. Weights use the full nibble range (-8 included).
"""
import numpy as np
import pytest

import oracle
from litert_amd import workloads as wl
from tests.fake_host import FakeHost, FLOAT32, FLOAT16, INT4, OK

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")

NODES = [(layer, name, k, n) for layer in range(wl.GEMMA2B_LAYERS)
         for name, k, n in wl.GEMMA2B_LAYER_FCS]


@pytest.fixture(scope="module")
def chain():
    """Seeded weights of the 126 nodes (about 1.1 GB on the host) and one input per node and
    batch size."""
    if not torch.cuda.is_available():
        pytest.fail("GPU tests need a gfx950 device; none visible")
    rng = np.random.default_rng(wl.SEED)
    packed, scales, xs = [], [], {1: [], 4: []}
    for _, _, k, n in NODES:
        packed.append(rng.integers(0, 256, (n, k // 2), dtype=np.uint8))
        scales.append(rng.uniform(5e-3, 2e-2, (n, k // 32)).astype(np.float16))
        for b in xs:
            xs[b].append(rng.standard_normal((b, k)).astype(np.float32))
    return packed, scales, xs


def _want(chain, b, i):
    packed, scales, xs = chain
    _, _, k, n = NODES[i]
    return oracle.fc_blockwise_int4(xs[b][i], packed[i], n, scales[i].view(np.uint16), 32)


@pytest.mark.parametrize("b", [1, 4])
def test_chain_through_the_delegate_matches_oracle(chain, b):
    packed, scales, xs = chain
    with FakeHost() as h:
        outs = []
        for i, (_, _, k, n) in enumerate(NODES):
            x = h.tensor(FLOAT32, (b, k), data=xs[b][i])
            w = h.tensor(INT4, (n, k), const=True, data=packed[i])
            s = h.tensor(FLOAT16, (n, k // 32), const=True, data=scales[i])
            h.blockwise(w, s, 32)
            y = h.tensor(FLOAT32, (b, n))
            h.fc(x, w, None, y)
            outs.append(y)
        assert h.load_delegate() == 0, h.errors()
        assert h.modify_graph_with_delegate() == OK, h.errors()
        plan = h.plan()
        assert len(plan) == 1 and plan[0][0] == "delegate" and len(plan[0][1]) == len(NODES)
        assert h.allocate_tensors() == OK, h.errors()
        for trial in range(2):  # the second invoke replays the partition's recorded launches
            assert h.invoke() == OK, h.errors()
            for i, y in enumerate(outs):
                got = h.read(y)
                want = _want(chain, b, i)
                assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (trial, NODES[i])


@pytest.mark.parametrize("b", [1, 4])
def test_chain_in_two_grouped_launches_matches_oracle(chain, b):
    from litert_amd import fully_connected as fc
    fc._ensure_init()
    packed, scales, xs = chain
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    ops = [fc.FullyConnectedBlockwiseInt4(packed[i], scales[i], k, 32)
           for i, (_, _, k, n) in enumerate(NODES)]
    shallow = [i for i, node in enumerate(NODES) if node[2] == 2048]
    deep = [i for i, node in enumerate(NODES) if node[2] != 2048]
    assert (len(shallow), len(deep)) == (108, 18)
    ys = {}
    groups = []
    for part in (shallow, deep):
        x_dev = [dev(xs[b][i]) for i in part]
        y_dev = [torch.full((b, NODES[i][3]), float("nan"), dtype=torch.float32, device="cuda")
                 for i in part]
        groups.append(fc.GroupedBlockwiseInt4([ops[i] for i in part]).bind(x_dev, y_dev))
        ys.update(zip(part, y_dev))
    for g in groups:
        g()
    torch.cuda.synchronize()
    for i in range(len(NODES)):
        want = _want(chain, b, i)
        assert np.array_equal(ys[i].cpu().numpy().view(np.uint32), want.view(np.uint32)), NODES[i]

"""Two interpreters, two threads, one device: the library's process-wide state (initialisation,
per-kernel LDS grants, per-device scratch addresses) and the delegate's per-instance state must
hold up when two plugin instances are prepared and invoked at the same time (the threading rule
of a TfLiteDelegate, tflite/core/c/common.h:1442-1493: one interpreter drives a delegate from one
thread at a time, but a process may run several interpreters). Every output of every invoke is
compared with the oracle; the first mismatch stops the test."""
import threading

import numpy as np
import pytest

import oracle
from litert_amd import workloads as wl
from tests.fake_host import FakeHost, FLOAT32, INT8, FLOAT16, INT4, OK

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

INVOKES = 12


def _hybrid_graph(h, rng):
    """Three hybrid nodes: a decode row, a four-row batch, and a chained pair."""
    K, N = 512, 192
    c = wl.hybrid_fc(4, K, N, seed=71)
    c2 = wl.hybrid_fc(4, N, 64, seed=72)
    x1 = h.tensor(FLOAT32, (1, K), data=c["x"][:1])
    x4 = h.tensor(FLOAT32, (4, K), data=c["x"])
    w = h.tensor(INT8, (N, K), data=c["w"], const=True)
    h.affine(w, c["pcs"])
    w2 = h.tensor(INT8, (64, N), data=c2["w"], const=True)
    h.affine(w2, c2["pcs"])
    y1 = h.tensor(FLOAT32, (1, N))
    y4 = h.tensor(FLOAT32, (4, N))
    y42 = h.tensor(FLOAT32, (4, 64))
    h.fc(x1, w, None, y1)
    h.fc(x4, w, None, y4, activation=1)
    h.fc(y4, w2, None, y42)
    h.mark_output(y4)  # read back by the test although a node of the partition consumes it

    def feed():
        a = rng.standard_normal((4, K)).astype(np.float32)
        h.write(x1, a[:1])
        h.write(x4, a)
        return a

    def check(a):
        want1 = oracle.fc_hybrid(a[:1], c["w"], c["pcs"])
        want4 = oracle.fc_hybrid(a, c["w"], c["pcs"], activation=oracle.ACT_RELU)
        want42 = oracle.fc_hybrid(want4, c2["w"], c2["pcs"])
        for y, want in ((y1, want1), (y4, want4), (y42, want42)):
            if not np.array_equal(h.read(y).view(np.uint32), want.view(np.uint32)):
                return False
        return True
    return feed, check


def _int4_graph(h, rng):
    """Three independent blockwise-int4 nodes of one depth (one grouped launch) and a consumer."""
    B, K = 2, 256
    widths = {"q": 64, "k": 24, "v": 24}
    cs = {k: wl.blockwise_int4_fc(B, K, n, seed=80 + i, lo=-8, hi=7)
          for i, (k, n) in enumerate(widths.items())}
    co = wl.blockwise_int4_fc(B, 64, 32, seed=90, lo=-8, hi=7)
    x = h.tensor(FLOAT32, (B, K), data=cs["q"]["x"])

    def int4(xin, c, n, k):
        w = h.tensor(INT4, (n, k), data=c["packed"], const=True)
        s_ = h.tensor(FLOAT16, (n, k // 32), data=c["scales"], const=True)
        h.blockwise(w, s_, 32)
        y = h.tensor(FLOAT32, (B, n))
        h.fc(xin, w, None, y)
        return y
    ys = {k: int4(x, cs[k], n, K) for k, n in widths.items()}
    yo = int4(ys["q"], co, 32, 64)
    for k in ("k", "v"):
        h.mark_output(ys[k])

    def feed():
        a = rng.standard_normal((B, K)).astype(np.float32)
        h.write(x, a)
        return a

    def ref(xin, c, n):
        return oracle.fc_blockwise_int4(xin, c["packed"], n, c["scales"].view(np.uint16), 32)

    def check(a):
        wq = ref(a, cs["q"], 64)
        for y, want in ((ys["k"], ref(a, cs["k"], 24)), (ys["v"], ref(a, cs["v"], 24)),
                        (yo, ref(wq, co, 32))):
            if not np.array_equal(h.read(y).view(np.uint32), want.view(np.uint32)):
                return False
        return True
    return feed, check


def _worker(build, seed, start, failures, name):
    try:
        rng = np.random.default_rng(seed)
        with FakeHost() as h:
            feed, check = build(h, rng)
            start.wait(timeout=60)
            if h.load_delegate() != 0:
                raise AssertionError("load_delegate: " + h.errors())
            if h.modify_graph_with_delegate() != OK or h.allocate_tensors() != OK:
                raise AssertionError("prepare: " + h.errors())
            if not all(kind == "delegate" for kind, _, _ in h.plan()):
                raise AssertionError("not every node was claimed: %r" % (h.plan(),))
            for i in range(INVOKES):
                a = feed()
                if h.invoke() != OK:
                    raise AssertionError("invoke %d: %s" % (i, h.errors()))
                if not check(a):
                    raise AssertionError("invoke %d differs from the oracle" % i)
    except Exception as e:  # noqa: BLE001 -- reported by the main thread
        failures.append("%s: %s" % (name, e))


def test_two_plugin_instances_in_two_threads_match_the_oracle():
    if not torch.cuda.is_available():
        pytest.fail("GPU tests need a gfx950 device; none visible")
    for round_ in range(3):
        start = threading.Barrier(2)
        failures = []
        threads = [
            threading.Thread(target=_worker, args=(_hybrid_graph, 100 + round_, start, failures, "hybrid")),
            threading.Thread(target=_worker, args=(_int4_graph, 200 + round_, start, failures, "int4")),
        ]
        for t in threads:
            t.start()
        for t in threads:
            t.join(timeout=120)
        assert not any(t.is_alive() for t in threads), "a worker did not finish"
        assert not failures, failures

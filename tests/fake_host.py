"""The stand-in TFLite host of litert_amd.standin_host with the CPU oracle installed as the
"builtin CPU kernels": FULLY_CONNECTED nodes the delegate declines run through the oracle."""
from litert_amd.standin_host import *  # noqa: F401,F403
from litert_amd.standin_host import CPU_CB, DELEGATE_LIB, HOST_LIB, INT8, KIND, lib  # noqa: F401
from litert_amd import standin_host as _sh


class FakeHost(_sh.FakeHost):
    def use_oracle_for_cpu_nodes(self):
        import oracle
        ran = []

        def run(node):
            try:
                f = self.fc_nodes[node]
                x, w = self.read(f["input"]), self.read(f["filter"])
                fm, om, im = self.meta[f["filter"]], self.meta[f["output"]], self.meta[f["input"]]
                bias = None if f["bias"] is None else self.read(f["bias"])
                K = w.shape[1]
                if im["type"] == INT8:
                    lo, hi = oracle.activation_range_int8(f["activation"], om["scale"], om["zero_point"])
                    scales = fm["scales"]
                    if scales.size > 1:
                        mult, shift = oracle.fc_prepare_per_channel(im["scale"], scales, om["scale"])
                        y = oracle.fc_int8_per_channel(x.reshape(-1, K), w, bias, mult, shift,
                                                       -im["zero_point"], om["zero_point"], lo, hi)
                    else:
                        m, s = oracle.fc_prepare_per_tensor(im["scale"], float(scales[0]), om["scale"])
                        y = oracle.fc_int8_per_tensor(x.reshape(-1, K), w, bias, m, s, -im["zero_point"],
                                                      -fm["zero_point"], om["zero_point"], lo, hi)
                else:
                    scales = fm["scales"]
                    y = oracle.fc_hybrid(x.reshape(-1, K), w, scales if scales.size > 1 else None,
                                         float(scales[0]), bias, f["asymmetric"], f["activation"])
                self.write(f["output"], y)
                ran.append(node)
                return 0
            except Exception as e:  # surfaced through fh_invoke's status
                print("cpu node %d failed: %r" % (node, e))
                return 1

        self.set_cpu_callback(run)
        return ran

"""Python front end of the stand-in TFLite host (fake_tflite_host.cc beside this file): builds
small graphs of FULLY_CONNECTED nodes, applies the delegate plugin to them the way the
interpreter would (Prepare -> ReplaceNodeSubsetsWithDelegateKernels -> init -> prepare ->
invoke), and runs them. It exists because the interpreter itself cannot be built without the
reference's build system; the benchmark and the tests both drive the plugin through it. Nodes
the delegate declines go to a callback the caller installs (the tests install the CPU oracle)."""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
HOST_LIB = os.path.join(HERE, "libfake_tflite_host.so")
DELEGATE_LIB = os.path.join(os.path.dirname(HERE), "lib", "liblitert_amd_delegate.so")
if os.environ.get("LITERT_AMD_SANITIZED") == "1":  # the builds of `make san` beside this file
    HOST_LIB = os.path.join(HERE, "libfake_tflite_host_san.so")
    DELEGATE_LIB = os.path.join(os.path.dirname(HERE), "lib", "liblitert_amd_delegate_san.so")

# TfLiteType / TfLiteAllocationType values (include/tflite_abi.h)
FLOAT32, INT32, UINT8, INT8, FLOAT16, INT4, INT16, INT2 = 1, 2, 3, 9, 10, 18, 7, 20
MMAP_RO, ARENA_RW = 1, 2
OK, ERROR, DELEGATE_ERROR = 0, 1, 2
KIND = {0: None, 1: "int8", 2: "hybrid", 3: "int4_blockwise", 4: "int4_per_channel",
        5: "embedding_lookup", 6: "batch_matmul"}

_NP = {FLOAT32: np.float32, INT32: np.int32, UINT8: np.uint8, INT8: np.int8, FLOAT16: np.float16,
       INT16: np.int16, INT4: np.uint8, INT2: np.uint8}
_lib = None
CPU_CB = C.CFUNCTYPE(C.c_int, C.c_int)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(HOST_LIB):
            subprocess.check_call(["make", "-s", "-C", HERE])
        L = C.CDLL(HOST_LIB)
        L.fh_create.restype = C.c_void_p
        L.fh_destroy.argtypes = [C.c_void_p]
        L.fh_add_tensor.argtypes = [C.c_void_p, C.c_int, C.c_int, C.POINTER(C.c_int), C.c_int,
                                    C.c_void_p, C.c_size_t, C.c_float, C.c_int]
        L.fh_set_affine_quantization.argtypes = [C.c_void_p, C.c_int, C.c_int, C.POINTER(C.c_float),
                                                 C.POINTER(C.c_int), C.c_int]
        L.fh_set_blockwise_quantization.argtypes = [C.c_void_p] + [C.c_int] * 5
        L.fh_add_fc_node.argtypes = [C.c_void_p] + [C.c_int] * 10
        L.fh_add_other_node.argtypes = [C.c_void_p] + [C.c_int] * 3
        L.fh_add_embedding_lookup_node.argtypes = [C.c_void_p] + [C.c_int] * 3
        L.fh_add_batch_matmul_node.argtypes = [C.c_void_p] + [C.c_int] * 7
        L.fh_mark_graph_output.argtypes = [C.c_void_p, C.c_int]
        L.fh_set_cpu_callback.argtypes = [C.c_void_p, CPU_CB]
        L.fh_load_delegate.argtypes = [C.c_void_p, C.c_char_p, C.POINTER(C.c_char_p),
                                       C.POINTER(C.c_char_p), C.c_size_t]
        for name in ("fh_modify_graph_with_delegate", "fh_allocate_tensors", "fh_invoke",
                     "fh_plan_size", "fh_replace_calls"):
            getattr(L, name).argtypes = [C.c_void_p]
        L.fh_tensor_data.argtypes = [C.c_void_p, C.c_int]
        L.fh_tensor_data.restype = C.c_void_p
        L.fh_tensor_bytes.argtypes = [C.c_void_p, C.c_int]
        L.fh_tensor_bytes.restype = C.c_size_t
        L.fh_move_tensor_data.argtypes = [C.c_void_p, C.c_int]
        L.fh_resize_tensor.argtypes = [C.c_void_p, C.c_int, C.c_int, C.POINTER(C.c_int), C.c_size_t]
        for name in ("fh_plan_node", "fh_node_is_delegate_kernel", "fh_node_num_replaced",
                     "fh_node_num_inputs", "fh_node_num_outputs", "fh_tensor_has_delegate"):
            getattr(L, name).argtypes = [C.c_void_p, C.c_int]
        for name in ("fh_node_replaced", "fh_node_input", "fh_node_output"):
            getattr(L, name).argtypes = [C.c_void_p, C.c_int, C.c_int]
        L.fh_node_user_data.argtypes = [C.c_void_p, C.c_int]
        L.fh_node_user_data.restype = C.c_void_p
        L.fh_errors.argtypes = [C.c_void_p]
        L.fh_errors.restype = C.c_char_p
        L.fh_clear_errors.argtypes = [C.c_void_p]
        L.fh_classify.argtypes = [C.c_void_p, C.c_char_p, C.c_int, C.c_char_p, C.c_size_t]
        L.fh_set_buffer_handle.argtypes = [C.c_void_p, C.c_int, C.c_int]
        L.fh_set_data_is_stale.argtypes = [C.c_void_p, C.c_int, C.c_int]
        for name in ("fh_data_is_stale", "fh_buffer_handle", "fh_ensure_tensor_data_is_readable",
                     "fh_copy_to_buffer_handle"):
            getattr(L, name).argtypes = [C.c_void_p, C.c_int]
        L.fh_delegate.argtypes = [C.c_void_p]
        L.fh_delegate.restype = C.c_void_p
        _lib = L
    return _lib


def _dims(shape):
    return (C.c_int * len(shape))(*shape), len(shape)


class FakeHost:
    def __init__(self):
        self.L = lib()
        self.h = C.c_void_p(self.L.fh_create())
        self.meta = {}      # tensor index -> dict(type, shape)
        self.fc_nodes = {}  # node index -> dict describing the FC (for the CPU callback)
        self._cb = None

    def close(self):
        if self.h:
            self.L.fh_destroy(self.h)
            self.h = None

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.close()

    # ---- graph building ----------------------------------------------------------------
    def tensor(self, ttype, shape, data=None, const=False, scale=0.0, zero_point=0, nbytes=None):
        d, n = _dims(shape)
        arr = None
        if data is not None:
            arr = np.ascontiguousarray(data)
            nbytes = arr.nbytes
        elif nbytes is None:
            nbytes = int(np.prod(shape)) * np.dtype(_NP[ttype]).itemsize
        idx = self.L.fh_add_tensor(self.h, ttype, n, d, MMAP_RO if const else ARENA_RW,
                                   None if arr is None else arr.ctypes.data_as(C.c_void_p),
                                   nbytes, scale, zero_point)
        self.meta[idx] = dict(type=ttype, shape=tuple(shape), scale=scale, zero_point=zero_point)
        return idx

    def affine(self, tensor, scales, zero_points=None, quantized_dimension=0):
        s = np.ascontiguousarray(scales, np.float32)
        z = np.zeros(s.size, np.int32) if zero_points is None else np.ascontiguousarray(zero_points, np.int32)
        self.L.fh_set_affine_quantization(self.h, tensor, s.size, s.ctypes.data_as(C.POINTER(C.c_float)),
                                          z.ctypes.data_as(C.POINTER(C.c_int)), quantized_dimension)
        self.meta[tensor].update(scales=s.copy(), zero_points=z.copy(), scale=float(s[0]),
                                 zero_point=int(z[0]))

    def blockwise(self, tensor, scale_tensor, blocksize, zero_point_tensor=-1):
        self.L.fh_set_blockwise_quantization(self.h, tensor, scale_tensor, zero_point_tensor,
                                             blocksize, 0)
        self.meta[tensor].update(block_scales=scale_tensor, blocksize=blocksize)

    def fc(self, inp, filt, bias, out, activation=0, keep_num_dims=False, asymmetric=True,
           weights_format=0, version=9, optional_bias_slot=False):
        three = bias is not None or optional_bias_slot
        node = self.L.fh_add_fc_node(self.h, inp, filt, -1 if bias is None else bias, int(three),
                                     out, activation, int(keep_num_dims), int(asymmetric),
                                     weights_format, version)
        self.fc_nodes[node] = dict(input=inp, filter=filt, bias=bias, output=out,
                                   activation=activation, asymmetric=asymmetric)
        return node

    def other(self, builtin_code, inp, out):
        return self.L.fh_add_other_node(self.h, builtin_code, inp, out)

    def embedding_lookup(self, lookup, value, out):
        return self.L.fh_add_embedding_lookup_node(self.h, lookup, value, out)

    def batch_matmul(self, lhs, rhs, out, adj_x=False, adj_y=False, asymmetric=True, version=4):
        return self.L.fh_add_batch_matmul_node(self.h, lhs, rhs, out, int(adj_x), int(adj_y),
                                               int(asymmetric), version)

    def mark_output(self, tensor):
        self.L.fh_mark_graph_output(self.h, tensor)

    def add_fc_nodes_of(self, subgraph, inputs=None):
        """Builds the FULLY_CONNECTED nodes of a parsed `.tflite` subgraph
        (litert_amd.tflite_file.SubGraph): their tensors with the quantization the runtime would
        attach (interpreter_builder.cc:500-519 for blockwise, :521-600 for affine) and the nodes
        with the file's options. `inputs` maps a model tensor index to the data it starts with.
        Returns {model tensor index: host tensor index}."""
        inputs = inputs or {}
        made = {}

        def make(ti):
            if ti < 0 or ti in made:
                return made.get(ti, -1)
            t = subgraph.tensors[ti]
            const = t.data is not None
            data = t.data if const else inputs.get(ti)
            nbytes = None
            if data is None and t.type_name in ("INT4",):
                nbytes = (int(np.prod(t.shape)) + 1) // 2
            made[ti] = self.tensor(t.tflite_type, t.shape, data=data, const=const, nbytes=nbytes)
            q = t.quantization
            if q.kind == "affine":
                self.affine(made[ti], q.scale, q.zero_point.astype(np.int32), q.quantized_dimension)
            elif q.kind == "blockwise":
                self.blockwise(made[ti], make(q.scales_tensor), q.block_size,
                               make(q.zero_points_tensor))
            return made[ti]

        for op in subgraph.operators:
            if op.fully_connected is None:
                continue
            o = op.fully_connected
            ins = [make(i) for i in op.inputs]
            out = make(op.outputs[0])
            self.fc(ins[0], ins[1], ins[2] if len(ins) > 2 and ins[2] >= 0 else None, out,
                    activation=o["activation"], keep_num_dims=o["keep_num_dims"],
                    asymmetric=o["asymmetric_quantize_inputs"], weights_format=o["weights_format"],
                    version=op.version, optional_bias_slot=len(ins) > 2)
        return made

    # ---- buffer handles (Interpreter::SetBufferHandle, EnsureTensorDataIsReadable) -----------
    def register_device_buffer(self, device_ptr, nbytes, path=DELEGATE_LIB):
        """litert_amd_register_device_buffer on the loaded delegate; returns the handle."""
        d = C.CDLL(path)
        d.litert_amd_register_device_buffer.restype = C.c_int
        d.litert_amd_register_device_buffer.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
        return d.litert_amd_register_device_buffer(self.L.fh_delegate(self.h), device_ptr, nbytes)

    def set_buffer_handle(self, tensor, handle):
        return self.L.fh_set_buffer_handle(self.h, tensor, handle)

    def buffer_handle(self, tensor):
        return self.L.fh_buffer_handle(self.h, tensor)

    def set_data_is_stale(self, tensor, stale=True):
        self.L.fh_set_data_is_stale(self.h, tensor, int(stale))

    def data_is_stale(self, tensor):
        return bool(self.L.fh_data_is_stale(self.h, tensor))

    def ensure_readable(self, tensor):
        return self.L.fh_ensure_tensor_data_is_readable(self.h, tensor)

    def copy_to_buffer_handle(self, tensor):
        return self.L.fh_copy_to_buffer_handle(self.h, tensor)

    # ---- delegate application --------------------------------------------------------------
    def load_delegate(self, options=None, path=DELEGATE_LIB):
        options = options or {}
        keys = (C.c_char_p * max(len(options), 1))(*[k.encode() for k in options])
        vals = (C.c_char_p * max(len(options), 1))(*[str(v).encode() for v in options.values()])
        return self.L.fh_load_delegate(self.h, path.encode(), keys, vals, len(options))

    def modify_graph_with_delegate(self):
        return self.L.fh_modify_graph_with_delegate(self.h)

    def allocate_tensors(self):
        return self.L.fh_allocate_tensors(self.h)

    def invoke(self):
        return self.L.fh_invoke(self.h)

    METRIC_FIELDS = ("invokes", "nodes_run", "bytes_uploaded", "bytes_downloaded", "host_time_us",
                     "device_time_us", "host_gather_us", "host_enqueue_us", "host_wait_us",
                     "host_scatter_us")

    def start_metrics(self, path=DELEGATE_LIB):
        """litert_amd_start_metrics on the loaded delegate (0 on success)."""
        d = C.CDLL(path)
        d.litert_amd_start_metrics.argtypes = [C.c_void_p, C.c_int]
        return d.litert_amd_start_metrics(self.L.fh_delegate(self.h), 0)

    def stop_metrics(self, path=DELEGATE_LIB):
        """litert_amd_stop_metrics: the totals since start_metrics, as a dict keyed by the fields
        of struct litert_amd_metrics."""
        class Metrics(C.Structure):
            _fields_ = ([(n, C.c_int64) for n in self.METRIC_FIELDS[:4]] +
                        [(n, C.c_double) for n in self.METRIC_FIELDS[4:]])
        d = C.CDLL(path)
        d.litert_amd_stop_metrics.argtypes = [C.c_void_p, C.POINTER(Metrics)]
        m = Metrics()
        if d.litert_amd_stop_metrics(self.L.fh_delegate(self.h), C.byref(m)) != 0:
            raise RuntimeError("litert_amd_stop_metrics: no collection was running")
        return {n: getattr(m, n) for n in self.METRIC_FIELDS}

    def classify(self, node, path=DELEGATE_LIB):
        buf = C.create_string_buffer(256)
        kind = self.L.fh_classify(self.h, path.encode(), node, buf, 256)
        return KIND.get(kind, kind), buf.value.decode()

    # ---- inspection ------------------------------------------------------------------------
    def errors(self):
        return self.L.fh_errors(self.h).decode()

    def plan(self):
        out = []
        for i in range(self.L.fh_plan_size(self.h)):
            n = self.L.fh_plan_node(self.h, i)
            if self.L.fh_node_is_delegate_kernel(self.h, n):
                out.append(("delegate", [self.L.fh_node_replaced(self.h, n, j)
                                         for j in range(self.L.fh_node_num_replaced(self.h, n))], n))
            else:
                out.append(("cpu", [n], n))
        return out

    def describe_partition(self, node, path=DELEGATE_LIB):
        """The delegate's own account of how it will run the partition behind `node`."""
        lib = C.CDLL(path)
        lib.litert_amd_describe_partition.argtypes = [C.c_void_p, C.c_char_p, C.c_size_t]
        buf = C.create_string_buffer(4096)
        n = lib.litert_amd_describe_partition(self.L.fh_node_user_data(self.h, node), buf, 4096)
        return n, buf.value.decode()

    def profiling_string(self, node):
        """TfLiteRegistration::profiling_string of the node, or None."""
        self.L.fh_node_profiling_string.restype = C.c_char_p
        self.L.fh_node_profiling_string.argtypes = [C.c_void_p, C.c_int]
        text = self.L.fh_node_profiling_string(self.h, node)
        return None if text is None else text.decode()

    def node_io(self, node):
        ins = [self.L.fh_node_input(self.h, node, i) for i in range(self.L.fh_node_num_inputs(self.h, node))]
        outs = [self.L.fh_node_output(self.h, node, i) for i in range(self.L.fh_node_num_outputs(self.h, node))]
        return ins, outs

    def read(self, tensor):
        m = self.meta[tensor]
        nbytes = self.L.fh_tensor_bytes(self.h, tensor)
        buf = (C.c_char * nbytes).from_address(self.L.fh_tensor_data(self.h, tensor))
        a = np.frombuffer(buf, dtype=_NP[m["type"]]).copy()
        return a.reshape(m["shape"]) if a.size == int(np.prod(m["shape"])) else a

    def write(self, tensor, data):
        arr = np.ascontiguousarray(data)
        assert arr.nbytes == self.L.fh_tensor_bytes(self.h, tensor)
        C.memmove(self.L.fh_tensor_data(self.h, tensor), arr.ctypes.data, arr.nbytes)

    def move(self, tensor):
        self.L.fh_move_tensor_data(self.h, tensor)

    def resize(self, tensor, shape):
        d, n = _dims(shape)
        nbytes = int(np.prod(shape)) * np.dtype(_NP[self.meta[tensor]["type"]]).itemsize
        self.L.fh_resize_tensor(self.h, tensor, n, d, nbytes)
        self.meta[tensor]["shape"] = tuple(shape)

    def set_cpu_callback(self, fn):
        """fn(node index) -> 0 on success: runs a node the delegate left on the host."""
        self._cb = CPU_CB(fn)
        self.L.fh_set_cpu_callback(self.h, self._cb)

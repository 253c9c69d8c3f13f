"""Python mirror of the Saga C++ interface (Graph / Node / Tensor / Context / Program).

A thin ctypes binding of include/saga_capi.h over saga_amd/lib/libsaga.so, which holds the
C++ front end and the hip engine.  Names and argument meaning follow the C++ API so that the
tests read like the reference's own harnesses.  There is no fallback: a missing library raises.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libsaga.so")

# Tensor::DataType
U8, HALF, FLOAT, INT64, I32, I16 = range(6)
_NP = {U8: np.uint8, HALF: np.float16, FLOAT: np.float32, INT64: np.int64, I32: np.int32, I16: np.int16}
_CODE = {np.dtype(v): k for k, v in _NP.items()}

BATCH, UNCHANGED, REDUCE = -1, -2, -3
PRE, POST = 1, 2
LAYOUT_AUTO, LAYOUT_NHWC, LAYOUT_NCHW = 0, 1, 2


class SagaError(RuntimeError):
    pass


class _Attr(C.Structure):
    _fields_ = [("name", C.c_char_p), ("kind", C.c_int), ("i", C.c_int64), ("f", C.c_double),
                ("ints", C.POINTER(C.c_int)), ("n_ints", C.c_int)]


class _ProfileRow(C.Structure):
    _fields_ = [("kind", C.c_char * 48), ("launches", C.c_long), ("ms", C.c_double), ("flops", C.c_double),
                ("bytes", C.c_double)]


class _Config(C.Structure):
    _fields_ = [("learning_rate", C.c_float), ("l2_lambda", C.c_float), ("bn_expavg", C.c_float),
                ("tensor_layout", C.c_int), ("anomaly_detect", C.c_int), ("disable_op_fusing", C.c_int),
                ("initial_loss_scale", C.c_float)]


_lib = None
_VP = C.c_void_p
SIGNATURES = {
    "saga_last_error": (C.c_char_p, []),
    "saga_tensor_create": (_VP, [C.c_int, C.c_int, C.POINTER(C.c_int64), C.c_char_p, C.c_int]),
    "saga_tensor_release": (None, [_VP]),
    "saga_tensor_grad": (_VP, [_VP]),
    "saga_tensor_rank": (C.c_int, [_VP]),
    "saga_tensor_dtype": (C.c_int, [_VP]),
    "saga_tensor_dims": (C.c_int, [_VP, C.POINTER(C.c_int64)]),
    "saga_tensor_write": (C.c_int, [_VP, _VP, C.c_size_t]),
    "saga_tensor_read": (C.c_int, [_VP, _VP, C.c_size_t]),
    "saga_tensor_save": (C.c_int, [_VP, C.c_char_p]),
    "saga_tensor_load": (_VP, [C.c_char_p, C.c_char_p]),
    "saga_tensor_sse": (C.c_double, [_VP, _VP]),
    "saga_graph_create": (_VP, []),
    "saga_graph_release": (None, [_VP]),
    "saga_graph_add_node": (_VP, [_VP, C.c_char_p, C.c_int, C.POINTER(C.c_char_p), C.POINTER(_VP), C.c_int,
                                  C.POINTER(_Attr), C.c_char_p]),
    "saga_graph_add_resnet_bottleneck": (_VP, [_VP, _VP, C.c_int, C.c_int, C.c_int, C.c_char_p]),
    "saga_graph_add_resnet": (_VP, [_VP, _VP, C.c_int, C.c_int, C.c_char_p]),
    "saga_graph_node_count": (C.c_int, [_VP]),
    "saga_graph_load": (_VP, [C.c_char_p]),
    "saga_graph_io_count": (C.c_int, [_VP, C.c_int]),
    "saga_graph_io": (_VP, [_VP, C.c_int, C.c_int]),
    "saga_graph_describe": (C.c_int, [_VP, C.c_char_p, C.c_size_t]),
    "saga_tensor_load_protobuf": (_VP, [C.c_char_p]),
    "saga_graph_save_tensors": (C.c_int, [_VP, C.c_char_p, _VP]),
    "saga_graph_load_tensors": (C.c_int, [_VP, C.c_char_p]),
    "saga_graph_named_tensor": (_VP, [_VP, C.c_char_p]),
    "saga_node_release": (None, [_VP]),
    "saga_node_output": (_VP, [_VP, C.c_char_p]),
    "saga_node_input": (_VP, [_VP, C.c_char_p]),
    "saga_context_create": (_VP, []),
    "saga_context_release": (None, [_VP]),
    "saga_context_reset": (C.c_int, [_VP]),
    "saga_context_resolve": (_VP, [_VP, _VP]),
    "saga_context_memory": (C.c_int, [_VP, C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]),
    "saga_program_create": (_VP, [_VP, _VP, C.c_int, C.c_int, C.POINTER(_Config), C.c_int, C.POINTER(_VP),
                                  C.POINTER(C.c_int)]),
    "saga_program_release": (None, [_VP]),
    "saga_program_finalize": (C.c_int, [_VP]),
    "saga_program_run": (C.c_int, [_VP, C.c_long]),
    "saga_program_loss_scale": (C.c_double, [_VP]),
    "saga_program_dump": (C.c_int, [_VP, C.c_char_p, C.c_int]),
    "saga_program_save_optimizer": (C.c_int, [_VP, C.c_char_p]),
    "saga_program_load_optimizer": (C.c_int, [_VP, C.c_char_p]),
    "saga_program_set_profiling": (C.c_int, [_VP, C.c_int]),
    "saga_program_profile": (C.c_int, [_VP, C.POINTER(_ProfileRow), C.c_int]),
}


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise SagaError(f"{LIB_PATH} is missing: build it with `make -C saga_amd/src` (or __graft_entry__.build())")
        _lib = C.CDLL(LIB_PATH, mode=C.RTLD_GLOBAL)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(_lib, name)
            fn.restype = res
            fn.argtypes = args
    return _lib


def _err(what):
    return SagaError(f"{what}: {lib().saga_last_error().decode()}")


def _name(n):
    return n.encode() if n is not None else None


class Tensor:
    def __init__(self, handle):
        if not handle:
            raise _err("tensor")
        self._h = handle

    @classmethod
    def cpu(cls, dtype, dims, name=None, data=None):
        """makeCPUTensor: host tensor with storage (row-major)."""
        d = (C.c_int64 * len(dims))(*dims)
        t = cls(lib().saga_tensor_create(dtype, len(dims), d, _name(name), 1))
        if data is not None:
            t.write(data)
        return t

    @classmethod
    def placeholder(cls, dtype, dims, name=None):
        """makeTensor: no storage; BATCH marks the batch dimension."""
        d = (C.c_int64 * len(dims))(*dims)
        return cls(lib().saga_tensor_create(dtype, len(dims), d, _name(name), 0))

    @classmethod
    def from_numpy(cls, a, dtype=None, name=None):
        a = np.asarray(a)
        code = dtype if dtype is not None else _CODE[a.dtype]
        return cls.cpu(code, list(a.shape), name, a)

    def __del__(self):
        try:
            lib().saga_tensor_release(self._h)
        except Exception:
            pass

    @property
    def dtype(self):
        return lib().saga_tensor_dtype(self._h)

    @property
    def dims(self):
        r = lib().saga_tensor_rank(self._h)
        out = (C.c_int64 * max(r, 1))()
        lib().saga_tensor_dims(self._h, out)
        return [int(out[i]) for i in range(r)]

    def grad(self):
        return Tensor(lib().saga_tensor_grad(self._h))

    def write(self, a):
        a = np.ascontiguousarray(np.asarray(a).astype(_NP[self.dtype], copy=False))
        if lib().saga_tensor_write(self._h, a.ctypes.data_as(C.c_void_p), a.nbytes):
            raise _err("tensor write")

    def read(self):
        a = np.empty(self.dims, _NP[self.dtype])
        if lib().saga_tensor_read(self._h, a.ctypes.data_as(C.c_void_p), a.nbytes):
            raise _err("tensor read")
        return a

    def save(self, path):
        if lib().saga_tensor_save(self._h, path.encode()):
            raise SagaError("tensor save failed: " + path)

    @classmethod
    def load(cls, path, name=None):
        return cls(lib().saga_tensor_load(path.encode(), _name(name)))

    @classmethod
    def load_protobuf(cls, path):
        """Tensor::loadProtoBuf: a file holding one ONNX TensorProto."""
        h = lib().saga_tensor_load_protobuf(path.encode())
        if not h:
            raise _err("loadProtoBuf")
        return cls(h)

    def sse(self, other):
        return lib().saga_tensor_sse(self._h, other._h)


class Node:
    def __init__(self, handle):
        if not handle:
            raise _err("node")
        self._h = handle

    def __del__(self):
        try:
            lib().saga_node_release(self._h)
        except Exception:
            pass

    def output(self, slot="y"):
        h = lib().saga_node_output(self._h, slot.encode())
        return Tensor(h) if h else None

    def input(self, slot):
        h = lib().saga_node_input(self._h, slot.encode())
        return Tensor(h) if h else None

    def y(self):
        return self.output("y")


def _attrs(attrs):
    keep = []
    arr = (_Attr * max(len(attrs), 1))()
    for i, (k, v) in enumerate(attrs.items()):
        a = arr[i]
        a.name = k.encode()
        if isinstance(v, bool):
            a.kind, a.i = 2, int(v)
        elif isinstance(v, (int, np.integer)):
            a.kind, a.i = 0, int(v)
        elif isinstance(v, float):
            a.kind, a.f = 1, v
        elif isinstance(v, Dims):
            buf = (C.c_int * len(v))(*v)
            keep.append(buf)
            a.kind, a.ints, a.n_ints = 4, buf, len(v)
        elif isinstance(v, (list, tuple)):
            buf = (C.c_int * len(v))(*v)
            keep.append(buf)
            a.kind, a.ints, a.n_ints = 3, buf, len(v)
        else:
            raise TypeError(f"attribute {k}: unsupported value {v!r}")
    return arr, keep


class Dims(list):
    """A Dims-valued attribute (reshape's "shape"); may hold UNCHANGED / REDUCE / BATCH."""


class Graph:
    def __init__(self, handle=None):
        self._h = handle or lib().saga_graph_create()

    @classmethod
    def load(cls, path):
        """Graph::load: an ONNX model file."""
        h = lib().saga_graph_load(path.encode())
        if not h:
            raise _err("Graph::load")
        return cls(h)

    def inputs(self):
        """Graph inputs (tensors no node produces and no initializer fills), in name order."""
        return [Tensor(lib().saga_graph_io(self._h, 0, i)) for i in range(lib().saga_graph_io_count(self._h, 0))]

    def outputs(self):
        return [Tensor(lib().saga_graph_io(self._h, 1, i)) for i in range(lib().saga_graph_io_count(self._h, 1))]

    def describe(self):
        """One line per node: type | inputs | attributes | outputs."""
        n = lib().saga_graph_describe(self._h, None, 0)
        buf = C.create_string_buffer(n + 1)
        lib().saga_graph_describe(self._h, buf, n + 1)
        return buf.value.decode().splitlines()

    def __del__(self):
        try:
            lib().saga_graph_release(self._h)
        except Exception:
            pass

    def add_node(self, type_, inputs, attrs=None, name=None):
        """Graph::addNode; `inputs` is a Tensor (slot "x"), a Node (its y) or a {slot: Tensor} dict."""
        if isinstance(inputs, Node):
            inputs = {"x": inputs.y()}
        elif isinstance(inputs, Tensor):
            inputs = {"x": inputs}
        names = (C.c_char_p * len(inputs))(*[k.encode() for k in inputs])
        handles = (_VP * len(inputs))(*[t._h for t in inputs.values()])
        arr, keep = _attrs(attrs or {})
        h = lib().saga_graph_add_node(self._h, type_.encode(), len(inputs), names, handles, len(attrs or {}), arr,
                                      _name(name))
        if not h:
            raise _err(f"addNode({type_})")
        return Node(h)

    def add_resnet_bottleneck(self, x, squeeze, output, downsample, name):
        h = lib().saga_graph_add_resnet_bottleneck(self._h, x._h, squeeze, output, int(downsample), name.encode())
        if not h:
            raise _err("addResNetBottleNeck")
        return Node(h)

    def add_resnet(self, x, output, downsample, name):
        h = lib().saga_graph_add_resnet(self._h, x._h, output, int(downsample), name.encode())
        if not h:
            raise _err("addResNet")
        return Node(h)

    def node_count(self):
        return lib().saga_graph_node_count(self._h)

    def named_tensor(self, name):
        h = lib().saga_graph_named_tensor(self._h, name.encode())
        return Tensor(h) if h else None

    def save_tensors(self, path, ctx=None):
        if lib().saga_graph_save_tensors(self._h, path.encode(), ctx._h if ctx else None):
            raise SagaError("saveTensors failed")

    def load_tensors(self, path):
        if lib().saga_graph_load_tensors(self._h, path.encode()):
            raise _err("loadTensors")


class Context:
    def __init__(self):
        self._h = lib().saga_context_create()
        if not self._h:
            raise _err("createContext")

    def __del__(self):
        try:
            lib().saga_context_release(self._h)
        except Exception:
            pass

    def reset(self):
        if lib().saga_context_reset(self._h):
            raise _err("reset")

    def memory(self):
        """(arena bytes, total bytes of the storages laid out in the arena)."""
        a, b = C.c_size_t(0), C.c_size_t(0)
        if lib().saga_context_memory(self._h, C.byref(a), C.byref(b)):
            raise _err("memory")
        return a.value, b.value

    def resolve(self, t):
        """Context::resolveTensor: the device tensor behind front-end tensor t (None if unused)."""
        h = lib().saga_context_resolve(self._h, t._h)
        return Tensor(h) if h else None

    def create_program(self, graph, batch_size, training, learning_rate=1e-4, l2_lambda=0.0, bn_expavg=0.1,
                       tensor_layout=LAYOUT_AUTO, anomaly_detect=False, disable_op_fusing=False,
                       initial_loss_scale=0.0, batched=None):
        cfg = _Config(learning_rate, l2_lambda, bn_expavg, tensor_layout, int(anomaly_detect),
                      int(disable_op_fusing), initial_loss_scale)
        batched = batched or {}
        hs = (_VP * max(len(batched), 1))(*[t._h for t in batched])
        ph = (C.c_int * max(len(batched), 1))(*batched.values())
        h = lib().saga_program_create(self._h, graph._h, batch_size, int(training), C.byref(cfg), len(batched), hs, ph)
        if not h:
            raise _err("createProgram")
        return Program(h, graph, self)


class Program:
    def __init__(self, handle, graph, ctx):
        self._h, self._graph, self._ctx = handle, graph, ctx  # keep the graph and context alive

    def __del__(self):
        try:
            lib().saga_program_release(self._h)
        except Exception:
            pass

    def finalize(self):
        if lib().saga_program_finalize(self._h):
            raise _err("finalize")

    def run(self, batches=1):
        rc = lib().saga_program_run(self._h, batches)
        if rc < 0:
            raise _err("run")
        return rc

    def loss_scale(self):
        return lib().saga_program_loss_scale(self._h)

    def save_optimizer(self, path):
        """Adam moments, step counts, fp32 master weights and loss scale -> a sagaO001 file."""
        if lib().saga_program_save_optimizer(self._h, str(path).encode()):
            raise _err("save_optimizer")

    def load_optimizer(self, path):
        if lib().saga_program_load_optimizer(self._h, str(path).encode()):
            raise _err("load_optimizer")

    def set_profiling(self, on=True):
        """Time every operation with HIP events on the program's stream (cleared when switched on)."""
        if lib().saga_program_set_profiling(self._h, int(on)):
            raise _err("set_profiling")

    def profile(self):
        """[{kind, launches, ms, flops, bytes}] accumulated since set_profiling(True)."""
        rows = (_ProfileRow * 1024)()
        n = lib().saga_program_profile(self._h, rows, 1024)
        if n < 0:
            raise _err("profile")
        return [{"kind": rows[i].kind.decode(), "launches": rows[i].launches, "ms": rows[i].ms,
                 "flops": rows[i].flops, "bytes": rows[i].bytes} for i in range(n)]

    def dump(self, path=None, detailed=False):
        if lib().saga_program_dump(self._h, _name(path), int(detailed)):
            raise _err("dump")

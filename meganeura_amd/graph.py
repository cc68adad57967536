"""Python face of the Graph / Session mirror (csrc/session.cpp), shaped after
meganeura's own API so that tests read like the reference's:

    g = Graph()
    a = g.input("a", [1, k]); b = g.parameter_q4("b", [k, n])
    g.set_outputs([g.matmul(a, b)])
    s = build_inference_session(g)
    s.set_input("a", x); s.set_parameter("b", w); s.step(); s.wait()
    y = s.read_output(n)

Everything here forwards to the C ABI; nothing is computed in Python.
"""
import ctypes as C
from enum import IntEnum

import numpy as np

from . import capi


class ShaderEntry(IntEnum):
    MatMul = 0
    MatMulGemv = 1
    FusedMatMulAdd = 2
    MatMulGemvAdd = 3
    Add = 4
    SwiGLU = 5
    SwiGLUConcat = 6
    RmsNorm = 7
    MatMulBT = 8
    MatMulGemvBT = 9
    Relu = 10
    Sigmoid = 11
    Neg = 12
    Silu = 13
    MatMulAT = 14
    FusedMatMulATAdd = 15
    FusedMatMulBTAdd = 16


class EpilogueOp(IntEnum):
    """compile::EpilogueOp (src/compile.rs:382-391), the unary ones."""
    Relu = 1
    Sigmoid = 2
    Neg = 3
    Silu = 4


class WeightFormat(IntEnum):
    F32 = 0
    Q4 = 1
    Q8 = 2


class Dispatch:
    def __init__(self, info):
        self.shader = ShaderEntry(info.shader)
        self.workgroups = list(info.workgroups)
        self.params = list(info.params)
        self.weight_format = WeightFormat(info.weight_format)
        self.epilogue = []
        e = info.epilogue
        while e:
            self.epilogue.append(EpilogueOp(e & 15))
            e >>= 4

    def __repr__(self):
        return (f"Dispatch({self.shader.name}, wg={self.workgroups}, params={self.params}, {self.weight_format.name}, "
                f"epilogue={[o.name for o in self.epilogue]})")


def _shape2(shape):
    shape = list(shape)
    if len(shape) == 1:
        return shape[0], 0
    if len(shape) != 2:
        raise ValueError("this path handles 1-D and 2-D shapes")
    return shape[0], shape[1]


class Graph:
    def __init__(self):
        self.lib = capi.load()
        self.h = C.c_void_p(self.lib.mgn_graph_new())

    def __del__(self):
        if getattr(self, "h", None):
            self.lib.mgn_graph_free(self.h)
            self.h = None

    def _node(self, rc):
        if rc < 0:
            raise ValueError(self.lib.mgn_graph_last_error(self.h).decode())
        return rc

    def input(self, name, shape):
        return self._node(self.lib.mgn_graph_input(self.h, name.encode(), *_shape2(shape)))

    def parameter(self, name, shape):
        return self._node(self.lib.mgn_graph_parameter(self.h, name.encode(), *_shape2(shape)))

    def parameter_q4(self, name, shape):
        return self._node(self.lib.mgn_graph_parameter_q4(self.h, name.encode(), *_shape2(shape)))

    def parameter_q8(self, name, shape):
        return self._node(self.lib.mgn_graph_parameter_q8(self.h, name.encode(), *_shape2(shape)))

    def matmul(self, a, b):
        return self._node(self.lib.mgn_graph_matmul(self.h, a, b))

    def matmul_bt(self, a, b):
        """a[M,K] x b[N,K]^T (src/graph.rs:809-817)."""
        return self._node(self.lib.mgn_graph_matmul_bt(self.h, a, b))

    def matmul_at(self, a, b):
        """a[K,M]^T x b[K,N] (src/graph.rs:798-806)."""
        return self._node(self.lib.mgn_graph_matmul_at(self.h, a, b))

    def add(self, a, b):
        return self._node(self.lib.mgn_graph_add(self.h, a, b))

    def swiglu(self, gate, up):
        return self._node(self.lib.mgn_graph_swiglu(self.h, gate, up))

    def rms_norm(self, x, weight, eps):
        return self._node(self.lib.mgn_graph_rms_norm(self.h, x, weight, eps))

    def relu(self, x):
        return self._node(self.lib.mgn_graph_unary(self.h, int(EpilogueOp.Relu), x))

    def sigmoid(self, x):
        return self._node(self.lib.mgn_graph_unary(self.h, int(EpilogueOp.Sigmoid), x))

    def neg(self, x):
        return self._node(self.lib.mgn_graph_unary(self.h, int(EpilogueOp.Neg), x))

    def silu(self, x):
        return self._node(self.lib.mgn_graph_unary(self.h, int(EpilogueOp.Silu), x))

    def set_outputs(self, ids):
        arr = (C.c_int32 * len(ids))(*ids)
        if self.lib.mgn_graph_set_outputs(self.h, arr, len(ids)) != capi.OK:
            raise ValueError(self.lib.mgn_graph_last_error(self.h).decode())

    def compile(self):
        """optimize + compile without touching a GPU; returns the dispatch list."""
        n = C.c_size_t()
        cap = 256
        infos = (capi.DispatchInfo * cap)()
        if self.lib.mgn_graph_compile(self.h, infos, cap, C.byref(n)) != capi.OK:
            raise ValueError(self.lib.mgn_graph_last_error(None).decode())
        return [Dispatch(infos[i]) for i in range(min(n.value, cap))]


class Session:
    def __init__(self, lib, h):
        self.lib, self.h = lib, h

    def close(self):
        if self.h:
            self.lib.mgn_session_free(self.h)
            self.h = None

    def __del__(self):
        self.close()

    def _check(self, st):
        if st == capi.ENOTFOUND:
            raise KeyError(self.lib.mgn_session_last_error(self.h).decode())
        if st != capi.OK:
            raise capi.MgnError(st, self.lib.mgn_session_last_error(self.h).decode())

    def plan(self):
        out = []
        for i in range(self.lib.mgn_session_num_dispatches(self.h)):
            info = capi.DispatchInfo()
            self._check(self.lib.mgn_session_dispatch_info(self.h, i, C.byref(info)))
            out.append(Dispatch(info))
        return out

    def set_parameter(self, name, data):
        data = np.ascontiguousarray(data, dtype=np.float32).reshape(-1)
        self._check(self.lib.mgn_session_set_parameter(self.h, name.encode(), data.ctypes.data_as(C.c_void_p), data.size))

    def set_input(self, name, data):
        data = np.ascontiguousarray(data, dtype=np.float32).reshape(-1)
        self._check(self.lib.mgn_session_set_input(self.h, name.encode(), data.ctypes.data_as(C.c_void_p), data.size))

    def step(self):
        self._check(self.lib.mgn_session_step(self.h))

    def wait(self):
        self._check(self.lib.mgn_session_wait(self.h))

    def set_graph_replay(self, enable):
        """Steps replay one captured HIP graph (default) or launch dispatch by dispatch."""
        self._check(self.lib.mgn_session_set_graph_replay(self.h, 1 if enable else 0))

    def set_fusion(self, enable):
        """Fold RmsNorm / SwiGLUConcat dispatches into the decode matmuls reading them (default on)."""
        self._check(self.lib.mgn_session_set_fusion(self.h, 1 if enable else 0))

    def set_chains(self, enable):
        """Runs of one-row Q4 matmul launches as one launch each (default on)."""
        self._check(self.lib.mgn_session_set_chains(self.h, 1 if enable else 0))

    def num_launches(self):
        return int(self.lib.mgn_session_num_launches(self.h))

    def graph_active(self):
        return bool(self.lib.mgn_session_graph_active(self.h))

    def context(self):
        """The session's context as a capi.Context view (timers, sync); not owned."""
        return capi.Context.borrowed(self.lib.mgn_session_ctx(self.h))

    def read_output(self, length):
        out = np.empty(length, dtype=np.float32)
        self._check(self.lib.mgn_session_read_output(self.h, out.ctypes.data_as(C.c_void_p), length))
        return out

    def read_output_by_index(self, index, length):
        out = np.empty(length, dtype=np.float32)
        self._check(self.lib.mgn_session_read_output_by_index(self.h, index, out.ctypes.data_as(C.c_void_p), length))
        return out


def build_inference_session(graph, device_id=0):
    lib = capi.load()
    h = C.c_void_p()
    st = lib.mgn_build_inference_session(graph.h, device_id, C.byref(h))
    if st != capi.OK:
        raise capi.MgnError(st, lib.mgn_session_last_error(None).decode())
    return Session(lib, h)

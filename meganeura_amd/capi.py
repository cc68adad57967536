"""ctypes binding of libmgn_hip.so (include/mgn_hip.h, include/mgn_session.h).

The shared library is the product; this module only declares its entry points.
There is no fallback: if the library has not been built, loading raises.
"""
import ctypes as C
import os

import numpy as np

_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_DIR, "libmgn_hip.so")

OK, EINVAL, ENOMEM, EHIP, ENOTFOUND, ENODEVICE, EUNSUPPORTED, ERANGE, ETIMEOUT = range(9)
FMT_Q4, FMT_Q8 = 0, 1
ACT_ANY, ACT_FP16_RANGE = 0, 1
STATIC_WORKSPACE_BYTES = 4 << 20  # MGN_STATIC_WORKSPACE_BYTES
ROUTE_AUTO, ROUTE_GENERIC, ROUTE_GEMV_VALU, ROUTE_GEMV_MFMA, ROUTE_GEMM_MFMA, ROUTE_TILE_MFMA = range(6)

# every symbol include/mgn_hip.h, include/mgn_bench.h and include/mgn_session.h declare
BENCH_SYMBOLS = ["mgn_ctx_set_route", "mgn_ctx_set_spin_limit", "mgn_engine_clock_mhz", "mgn_matmul_q_loop", "mgn_weight_read_loop"]
HIP_SYMBOLS = [
    "mgn_ctx_create", "mgn_ctx_destroy", "mgn_last_error", "mgn_sync", "mgn_ctx_set_activation_range", "mgn_ctx_set_shared_device",
    "mgn_buf_alloc", "mgn_buf_free", "mgn_buf_size", "mgn_buf_device_ptr", "mgn_buf_upload",
    "mgn_buf_download", "mgn_buf_copy", "mgn_packed_size", "mgn_quantize_ref", "mgn_dequantize_ref",
    "mgn_weight_create", "mgn_weight_create_nk", "mgn_quantize_ref_nk", "mgn_weight_create_packed", "mgn_weight_create_device", "mgn_weight_free",
    "mgn_weight_info", "mgn_weight_dequantize", "mgn_weight_export_ref", "mgn_weight_save", "mgn_weight_load", "mgn_matmul_q",
    "mgn_matmul_q_f16a", "mgn_matmul_q_static", "mgn_matmul_q_epilogue", "mgn_matmul_q_at", "mgn_matmul_q_plan", "mgn_matmul_q_rms_norm", "mgn_matmul_q_swiglu", "mgn_matmul_q_can_fuse", "mgn_matmul_q_batch",
    "mgn_chain_create", "mgn_chain_run", "mgn_chain_free",
    "mgn_timer_start", "mgn_timer_stop", "mgn_version", "mgn_built_for",
]
SESSION_SYMBOLS = [
    "mgn_graph_new", "mgn_graph_free", "mgn_graph_last_error", "mgn_graph_input", "mgn_graph_parameter",
    "mgn_graph_parameter_q4", "mgn_graph_parameter_q8", "mgn_graph_matmul", "mgn_graph_matmul_bt", "mgn_graph_matmul_at", "mgn_graph_add",
    "mgn_graph_swiglu", "mgn_graph_rms_norm", "mgn_graph_unary", "mgn_graph_set_outputs", "mgn_graph_compile",
    "mgn_build_inference_session", "mgn_session_free", "mgn_session_last_error",
    "mgn_session_num_dispatches", "mgn_session_dispatch_info", "mgn_session_set_parameter",
    "mgn_session_set_input", "mgn_session_step", "mgn_session_wait", "mgn_session_read_output",
    "mgn_session_read_output_by_index", "mgn_session_ctx", "mgn_session_set_graph_replay",
    "mgn_session_graph_active", "mgn_session_set_fusion", "mgn_session_set_chains", "mgn_session_num_launches",
]


class MatmulItem(C.Structure):
    _fields_ = [("w", C.c_void_p), ("d", C.c_void_p), ("c", C.c_void_p)]


PROLOGUE_NONE, PROLOGUE_RMS_NORM, PROLOGUE_SWIGLU = range(3)


class ChainStage(C.Structure):
    _fields_ = [("w", C.c_void_p), ("a", C.c_void_p), ("prologue", C.c_int), ("norm_weight", C.c_void_p), ("eps", C.c_float),
                ("d", C.c_void_p), ("c", C.c_void_p), ("ops", C.POINTER(C.c_int)), ("n_ops", C.c_size_t)]


class DispatchInfo(C.Structure):
    _fields_ = [
        ("shader", C.c_int32),
        ("workgroups", C.c_uint32 * 3),
        ("params", C.c_uint32 * 4),
        ("weight_format", C.c_int32),
        ("epilogue", C.c_uint32),
    ]


class MgnError(RuntimeError):
    def __init__(self, status, message):
        super().__init__(f"mgn status {status}: {message}")
        self.status = status


_lib = None


def load():
    """Load libmgn_hip.so and declare signatures.  Raises if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
            "or `make -C meganeura_amd/csrc`; there is no fallback path"
        )
    lib = C.CDLL(LIB_PATH)
    vp, sz, u8p, f32p = C.c_void_p, C.c_size_t, C.POINTER(C.c_uint8), C.POINTER(C.c_float)
    sig = {
        "mgn_ctx_create": (C.c_int, [C.c_int, C.POINTER(vp)]),
        "mgn_ctx_destroy": (None, [vp]),
        "mgn_last_error": (C.c_char_p, [vp]),
        "mgn_sync": (C.c_int, [vp]),
        "mgn_ctx_set_route": (C.c_int, [vp, C.c_int]),
        "mgn_ctx_set_spin_limit": (C.c_int, [vp, C.c_uint32]),
        "mgn_engine_clock_mhz": (C.c_int, [vp, C.c_int, C.POINTER(C.c_float), C.POINTER(C.c_float)]),
        "mgn_ctx_set_activation_range": (C.c_int, [vp, C.c_int]),
        "mgn_ctx_set_shared_device": (C.c_int, [vp, C.c_int]),
        "mgn_buf_alloc": (C.c_int, [vp, sz, C.POINTER(vp)]),
        "mgn_buf_free": (None, [vp, vp]),
        "mgn_buf_size": (sz, [vp]),
        "mgn_buf_device_ptr": (vp, [vp]),
        "mgn_buf_upload": (C.c_int, [vp, vp, sz, vp, sz]),
        "mgn_buf_download": (C.c_int, [vp, vp, sz, vp, sz]),
        "mgn_buf_copy": (C.c_int, [vp, vp, vp, sz]),
        "mgn_packed_size": (sz, [C.c_int, sz, sz]),
        "mgn_quantize_ref": (C.c_int, [C.c_int, vp, sz, sz, vp]),
        "mgn_dequantize_ref": (C.c_int, [C.c_int, vp, sz, sz, vp]),
        "mgn_weight_create": (C.c_int, [vp, C.c_int, vp, sz, sz, C.POINTER(vp)]),
        "mgn_weight_create_nk": (C.c_int, [vp, C.c_int, vp, sz, sz, C.POINTER(vp)]),
        "mgn_quantize_ref_nk": (C.c_int, [C.c_int, vp, sz, sz, vp]),
        "mgn_weight_create_packed": (C.c_int, [vp, C.c_int, vp, sz, sz, C.POINTER(vp)]),
        "mgn_weight_create_device": (C.c_int, [vp, C.c_int, vp, sz, sz, C.POINTER(vp)]),
        "mgn_weight_free": (None, [vp, vp]),
        "mgn_weight_dequantize": (C.c_int, [vp, vp, vp]),
        "mgn_weight_export_ref": (C.c_int, [vp, vp, vp]),
        "mgn_weight_save": (C.c_int, [vp, vp, C.c_char_p]),
        "mgn_weight_load": (C.c_int, [vp, C.c_char_p, C.POINTER(vp)]),
        "mgn_weight_info": (C.c_int, [vp, C.POINTER(C.c_int), C.POINTER(sz), C.POINTER(sz)]),
        "mgn_matmul_q": (C.c_int, [vp, vp, vp, vp, vp, C.c_uint32]),
        "mgn_matmul_q_f16a": (C.c_int, [vp, vp, vp, vp, vp, C.c_uint32]),
        "mgn_matmul_q_static": (C.c_int, [vp, vp, vp, vp, vp, C.c_uint32]),
        "mgn_matmul_q_epilogue": (C.c_int, [vp, vp, vp, vp, vp, C.c_uint32, vp, C.c_size_t]),
        "mgn_matmul_q_at": (C.c_int, [vp, vp, vp, vp, vp, C.c_uint32, vp, C.c_size_t]),
        "mgn_matmul_q_plan": (C.c_int, [C.c_int, C.c_uint32, C.c_uint64, C.c_uint64, C.c_int, C.c_int, vp]),
        "mgn_matmul_q_loop": (C.c_int, [vp, vp, C.c_int, vp, C.c_size_t, vp, vp, C.c_uint32, C.c_uint32]),
        "mgn_weight_read_loop": (C.c_int, [vp, vp, C.c_size_t, C.c_uint32, C.c_int]),
        "mgn_matmul_q_rms_norm": (C.c_int, [vp, vp, vp, C.c_float, vp, vp, vp, C.c_uint32]),
        "mgn_matmul_q_swiglu": (C.c_int, [vp, vp, vp, vp, vp, C.c_uint32]),
        "mgn_matmul_q_can_fuse": (C.c_int, [vp, vp, C.c_uint32]),
        "mgn_matmul_q_batch": (C.c_int, [vp, vp, C.c_int, vp, C.c_float, C.POINTER(MatmulItem), sz, C.c_uint32]),
        "mgn_chain_create": (C.c_int, [vp, C.POINTER(ChainStage), sz, C.c_uint32, C.POINTER(vp)]),
        "mgn_chain_run": (C.c_int, [vp, vp]),
        "mgn_chain_free": (None, [vp, vp]),
        "mgn_timer_start": (C.c_int, [vp]),
        "mgn_timer_stop": (C.c_int, [vp, C.POINTER(C.c_float)]),
        "mgn_version": (C.c_char_p, []),
        "mgn_built_for": (C.c_char_p, []),
        "mgn_graph_new": (vp, []),
        "mgn_graph_free": (None, [vp]),
        "mgn_graph_last_error": (C.c_char_p, [vp]),
        "mgn_graph_input": (C.c_int32, [vp, C.c_char_p, sz, sz]),
        "mgn_graph_parameter": (C.c_int32, [vp, C.c_char_p, sz, sz]),
        "mgn_graph_parameter_q4": (C.c_int32, [vp, C.c_char_p, sz, sz]),
        "mgn_graph_parameter_q8": (C.c_int32, [vp, C.c_char_p, sz, sz]),
        "mgn_graph_matmul": (C.c_int32, [vp, C.c_int32, C.c_int32]),
        "mgn_graph_matmul_bt": (C.c_int32, [vp, C.c_int32, C.c_int32]),
        "mgn_graph_matmul_at": (C.c_int32, [vp, C.c_int32, C.c_int32]),
        "mgn_graph_add": (C.c_int32, [vp, C.c_int32, C.c_int32]),
        "mgn_graph_swiglu": (C.c_int32, [vp, C.c_int32, C.c_int32]),
        "mgn_graph_rms_norm": (C.c_int32, [vp, C.c_int32, C.c_int32, C.c_float]),
        "mgn_graph_unary": (C.c_int32, [vp, C.c_int32, C.c_int32]),
        "mgn_graph_set_outputs": (C.c_int, [vp, C.POINTER(C.c_int32), sz]),
        "mgn_graph_compile": (C.c_int, [vp, C.POINTER(DispatchInfo), sz, C.POINTER(sz)]),
        "mgn_build_inference_session": (C.c_int, [vp, C.c_int, C.POINTER(vp)]),
        "mgn_session_free": (None, [vp]),
        "mgn_session_last_error": (C.c_char_p, [vp]),
        "mgn_session_num_dispatches": (sz, [vp]),
        "mgn_session_dispatch_info": (C.c_int, [vp, sz, C.POINTER(DispatchInfo)]),
        "mgn_session_set_parameter": (C.c_int, [vp, C.c_char_p, vp, sz]),
        "mgn_session_set_input": (C.c_int, [vp, C.c_char_p, vp, sz]),
        "mgn_session_step": (C.c_int, [vp]),
        "mgn_session_wait": (C.c_int, [vp]),
        "mgn_session_read_output": (C.c_int, [vp, vp, sz]),
        "mgn_session_read_output_by_index": (C.c_int, [vp, sz, vp, sz]),
        "mgn_session_ctx": (vp, [vp]),
        "mgn_session_set_graph_replay": (C.c_int, [vp, C.c_int]),
        "mgn_session_graph_active": (C.c_int, [vp]),
        "mgn_session_set_fusion": (C.c_int, [vp, C.c_int]),
        "mgn_session_set_chains": (C.c_int, [vp, C.c_int]),
        "mgn_session_num_launches": (sz, [vp]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def _ptr(arr):
    return arr.ctypes.data_as(C.c_void_p)


# ---- host quantizers (no GPU needed) -------------------------------------------

def packed_size(fmt, rows, cols):
    return int(load().mgn_packed_size(fmt, rows, cols))


UNARY_RELU, UNARY_SIGMOID, UNARY_NEG, UNARY_SILU = 1, 2, 3, 4


class PlanInfo(C.Structure):
    _fields_ = [("route", C.c_int), ("grid", C.c_uint32 * 3), ("threads", C.c_uint32), ("lds_bytes", C.c_uint32),
                ("waves_n", C.c_uint32), ("k_splits", C.c_uint32), ("k_parts", C.c_uint32), ("steps", C.c_uint32),
                ("quads_per_wave", C.c_uint32), ("full_steps", C.c_uint32), ("tail_blocks", C.c_uint32),
                ("workspace_bytes", C.c_uint64)]


def matmul_plan(fmt, m, k, n, a_is_f16=False, num_cus=256, fp16_range=False):
    """What mgn_matmul_q would launch for this shape (no device needed).  fp16_range: f32
    activations on a context set to ACT_FP16_RANGE."""
    info = PlanInfo()
    st = load().mgn_matmul_q_plan(fmt, m, k, n, 1 if a_is_f16 else 2 if fp16_range else 0, num_cus, C.byref(info))
    if st != OK:
        raise MgnError(st, "matmul_plan: no weight has this shape")
    return info


def quantize_ref(fmt, w):
    w = np.ascontiguousarray(w, dtype=np.float32)
    rows, cols = w.shape
    out = np.zeros(packed_size(fmt, rows, cols), dtype=np.uint8)
    st = load().mgn_quantize_ref(fmt, _ptr(w), rows, cols, _ptr(out))
    if st != OK:
        raise MgnError(st, "quantize_ref: rows (K dim) must be a multiple of 32")
    return out


def quantize_ref_nk(fmt, w_nk):
    """Packed bytes (reference layout for rows = K, cols = N) of a weight stored [N, K]."""
    w_nk = np.ascontiguousarray(w_nk, dtype=np.float32)
    n, k = w_nk.shape
    out = np.zeros(packed_size(fmt, k, n), dtype=np.uint8)
    st = load().mgn_quantize_ref_nk(fmt, _ptr(w_nk), n, k, _ptr(out))
    if st != OK:
        raise MgnError(st, "quantize_ref_nk: K must be a multiple of 32")
    return out


def dequantize_ref(fmt, packed, rows, cols):
    packed = np.ascontiguousarray(packed, dtype=np.uint8)
    out = np.empty((rows, cols), dtype=np.float32)
    st = load().mgn_dequantize_ref(fmt, _ptr(packed), rows, cols, _ptr(out))
    if st != OK:
        raise MgnError(st, "dequantize_ref: bad arguments")
    return out


# ---- thin object wrappers over the handles -----------------------------------------

class Context:
    def __init__(self, device_id=0):
        self.lib = load()
        h = C.c_void_p()
        st = self.lib.mgn_ctx_create(device_id, C.byref(h))
        if st != OK:
            raise MgnError(st, self.lib.mgn_last_error(None).decode())
        self.h = h
        self.owned = True

    @classmethod
    def borrowed(cls, handle):
        """View of a context owned by someone else (a session's): never destroyed here."""
        self = cls.__new__(cls)
        self.lib = load()
        self.h = C.c_void_p(handle)
        self.owned = False
        return self

    def check(self, st):
        if st != OK:
            raise MgnError(st, self.lib.mgn_last_error(self.h).decode())

    def close(self):
        if self.h and self.owned:
            self.lib.mgn_ctx_destroy(self.h)
        self.h = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def set_activation_range(self, fp16_range):
        """f32 activations of M >= 5: False (default, ACT_ANY) takes any value; True (ACT_FP16_RANGE)
        promises |x| < 65504 and lets the faster unscaled tiled kernel run."""
        self.check(self.lib.mgn_ctx_set_activation_range(self.h, ACT_FP16_RANGE if fp16_range else ACT_ANY))

    def set_shared_device(self, shared):
        """True: other work runs on the device beside this context; launches whose workgroups all
        wait for each other (chains, K parts added up by shares) are not used."""
        self.check(self.lib.mgn_ctx_set_shared_device(self.h, 1 if shared else 0))

    def set_route(self, route):
        self.check(self.lib.mgn_ctx_set_route(self.h, route))

    def set_spin_limit(self, polls):
        """Polls a wave makes for another workgroup's partial sums before it gives up (tests only)."""
        self.check(self.lib.mgn_ctx_set_spin_limit(self.h, polls))

    def engine_clock_mhz(self, loaded=False):
        mhz = C.c_float()
        self.check(self.lib.mgn_engine_clock_mhz(self.h, 1 if loaded else 0, C.byref(mhz), None))
        return float(mhz.value)

    def engine_probe(self):
        """(MHz under the matrix-instruction load, shader cycles per round of that load)."""
        mhz, cyc = C.c_float(), C.c_float()
        self.check(self.lib.mgn_engine_clock_mhz(self.h, 1, C.byref(mhz), C.byref(cyc)))
        return float(mhz.value), float(cyc.value)

    def sync(self):
        self.check(self.lib.mgn_sync(self.h))

    def timer_start(self):
        self.check(self.lib.mgn_timer_start(self.h))

    def timer_stop(self):
        ms = C.c_float()
        self.check(self.lib.mgn_timer_stop(self.h, C.byref(ms)))
        return ms.value

    def buffer(self, nbytes):
        return Buffer(self, nbytes)

    def copy(self, dst, src, nbytes):
        self.check(self.lib.mgn_buf_copy(self.h, dst.h, src.h, nbytes))

    def upload(self, arr):
        arr = np.ascontiguousarray(arr)
        b = Buffer(self, arr.nbytes)
        b.upload(arr)
        return b

    def weight(self, fmt, w):
        w = np.ascontiguousarray(w, dtype=np.float32)
        h = C.c_void_p()
        self.check(self.lib.mgn_weight_create(self.h, fmt, _ptr(w), w.shape[0], w.shape[1], C.byref(h)))
        return Weight(self, h, fmt, w.shape[0], w.shape[1])

    def weight_nk(self, fmt, w_nk):
        """Weight from an [N, K] matrix (matmul_bt operand); the handle is a [K, N] weight."""
        w_nk = np.ascontiguousarray(w_nk, dtype=np.float32)
        h = C.c_void_p()
        self.check(self.lib.mgn_weight_create_nk(self.h, fmt, _ptr(w_nk), w_nk.shape[0], w_nk.shape[1], C.byref(h)))
        return Weight(self, h, fmt, w_nk.shape[1], w_nk.shape[0])

    def load_weight(self, path):
        """Weight from a file written by Weight.save."""
        h = C.c_void_p()
        self.check(self.lib.mgn_weight_load(self.h, str(path).encode(), C.byref(h)))
        fmt, rows, cols = C.c_int(), C.c_size_t(), C.c_size_t()
        self.lib.mgn_weight_info(h, C.byref(fmt), C.byref(rows), C.byref(cols))
        return Weight(self, h, fmt.value, rows.value, cols.value)

    def weight_from_packed(self, fmt, packed, rows, cols):
        packed = np.ascontiguousarray(packed, dtype=np.uint8)
        assert packed.size == packed_size(fmt, rows, cols)
        h = C.c_void_p()
        self.check(self.lib.mgn_weight_create_packed(self.h, fmt, _ptr(packed), rows, cols, C.byref(h)))
        return Weight(self, h, fmt, rows, cols)

    def weight_from_device(self, fmt, buf, rows, cols):
        h = C.c_void_p()
        self.check(self.lib.mgn_weight_create_device(self.h, fmt, buf.h, rows, cols, C.byref(h)))
        return Weight(self, h, fmt, rows, cols)

    def matmul_q(self, a, w, c, m, d=None):
        self.check(self.lib.mgn_matmul_q(self.h, a.h, w.h, d.h if d is not None else None, c.h, m))

    def matmul_q_static(self, a, w, c, m, d=None):
        """mgn_matmul_q on the library's static workspace: no device allocation in the call."""
        self.check(self.lib.mgn_matmul_q_static(self.h, a.h, w.h, d.h if d is not None else None, c.h, m))

    def matmul_q_f16a(self, a, w, c, m, d=None):
        self.check(self.lib.mgn_matmul_q_f16a(self.h, a.h, w.h, d.h if d is not None else None, c.h, m))

    def matmul_q_epilogue(self, a, w, c, m, ops, d=None):
        """C = f_n(...f_1(A x W + D)) with ops a sequence of UNARY_* codes."""
        arr = (C.c_int * max(1, len(ops)))(*ops)
        self.check(self.lib.mgn_matmul_q_epilogue(self.h, a.h, w.h, d.h if d is not None else None, c.h, m, arr, len(ops)))

    def matmul_q_at(self, a_t, w, c, m, d=None, ops=()):
        """C = f(A^T x W + D) with A stored [K, M]; ops as in matmul_q_epilogue."""
        arr = (C.c_int * max(1, len(ops)))(*ops)
        self.check(self.lib.mgn_matmul_q_at(self.h, a_t.h, w.h, d.h if d is not None else None, c.h, m,
                                            arr if len(ops) else None, len(ops)))

    @staticmethod
    def rotation(weights):
        """The handles of `weights`, twice over, as a C array: a rotation that starts at copy `first`
        is the `len(weights)` entries from there, with nothing to build when a timed loop starts."""
        n = len(weights)
        return (C.c_void_p * (2 * n))(*([w.h for w in weights] * 2)), n

    def matmul_q_loop(self, a, weights, c, m, steps, d=None, a_is_f16=False, first=0):
        """`steps` matmuls enqueued back to back from C, call i on weights[(first + i) % len(weights)];
        `weights` is a list of weights or what rotation() made of one."""
        arr, n = weights if isinstance(weights, tuple) else self.rotation(weights)
        start = C.cast(C.byref(arr, (first % n) * C.sizeof(C.c_void_p)), C.c_void_p) if n else None
        self.check(self.lib.mgn_matmul_q_loop(self.h, a.h, 1 if a_is_f16 else 0, start, n,
                                              d.h if d is not None else None, c.h, m, steps))

    def weight_read_loop(self, weights, steps, first=0, pattern=0):
        """`steps` launches of a kernel that only reads the packed bytes of weights[(first + i) % len(weights)]."""
        arr, n = weights if isinstance(weights, tuple) else self.rotation(weights)
        start = C.cast(C.byref(arr, (first % n) * C.sizeof(C.c_void_p)), C.c_void_p) if n else None
        self.check(self.lib.mgn_weight_read_loop(self.h, start, n, steps, pattern))

    def matmul_q_rms_norm(self, x, norm_weight, eps, w, c, m, d=None):
        """C = rms_norm(x; norm_weight, eps) x W (+ D) in one launch."""
        self.check(self.lib.mgn_matmul_q_rms_norm(self.h, x.h, norm_weight.h, eps, w.h, d.h if d is not None else None, c.h, m))

    def matmul_q_swiglu(self, gate_up, w, c, m, d=None):
        """C = (silu(gate) * up) x W (+ D) in one launch; gate_up is [m, 2K]."""
        self.check(self.lib.mgn_matmul_q_swiglu(self.h, gate_up.h, w.h, d.h if d is not None else None, c.h, m))

    def matmul_q_batch(self, a, items, m, prologue=PROLOGUE_NONE, norm_weight=None, eps=0.0):
        """items: (weight, c, d-or-None) tuples sharing the activations `a`; one launch."""
        arr = (MatmulItem * len(items))()
        for j, (w, c, d) in enumerate(items):
            arr[j].w, arr[j].c, arr[j].d = w.h, c.h, (d.h if d is not None else None)
        self.check(self.lib.mgn_matmul_q_batch(self.h, a.h, prologue, norm_weight.h if norm_weight is not None else None,
                                               eps, arr, len(items), m))

    def can_fuse(self, w, m):
        return bool(self.lib.mgn_matmul_q_can_fuse(self.h, w.h, m))

    def chain(self, stages, m=1):
        """One launch for a chain of dependent one-row matmuls.  stages: dicts with w, a, c and
        optionally prologue, norm_weight, eps, d, ops (mgn_chain_stage)."""
        return Chain(self, stages, m)


class Chain:
    def __init__(self, ctx, stages, m=1):
        self.ctx = ctx
        arr = (ChainStage * len(stages))()
        self._keep = []
        for s, st in zip(arr, stages):
            s.w, s.a, s.c = st["w"].h, st["a"].h, st["c"].h
            s.prologue = st.get("prologue", PROLOGUE_NONE)
            s.norm_weight = st["norm_weight"].h if st.get("norm_weight") is not None else None
            s.eps = st.get("eps", 0.0)
            s.d = st["d"].h if st.get("d") is not None else None
            ops = list(st.get("ops", ()))
            if ops:
                o = (C.c_int * len(ops))(*ops)
                self._keep.append(o)
                s.ops = C.cast(o, C.POINTER(C.c_int))
            s.n_ops = len(ops)
        h = C.c_void_p()
        ctx.check(ctx.lib.mgn_chain_create(ctx.h, arr, len(stages), m, C.byref(h)))
        self.h = h

    def run(self):
        self.ctx.check(self.ctx.lib.mgn_chain_run(self.ctx.h, self.h))

    def free(self):
        if self.h:
            self.ctx.lib.mgn_chain_free(self.ctx.h, self.h)
            self.h = None


class Buffer:
    def __init__(self, ctx, nbytes):
        self.ctx = ctx
        h = C.c_void_p()
        ctx.check(ctx.lib.mgn_buf_alloc(ctx.h, nbytes, C.byref(h)))
        self.h = h
        self.nbytes = nbytes

    def upload(self, arr, offset=0):
        arr = np.ascontiguousarray(arr)
        self.ctx.check(self.ctx.lib.mgn_buf_upload(self.ctx.h, self.h, offset, _ptr(arr), arr.nbytes))

    def download(self, dtype, count, offset=0):
        out = np.empty(count, dtype=dtype)
        self.ctx.check(self.ctx.lib.mgn_buf_download(self.ctx.h, self.h, offset, _ptr(out), out.nbytes))
        return out

    def free(self):
        if self.h:
            self.ctx.lib.mgn_buf_free(self.ctx.h, self.h)
            self.h = None


class Weight:
    def __init__(self, ctx, h, fmt, rows, cols):
        self.ctx, self.h, self.fmt, self.rows, self.cols = ctx, h, fmt, rows, cols

    def dequantize(self):
        out = np.empty((self.rows, self.cols), dtype=np.float32)
        self.ctx.check(self.ctx.lib.mgn_weight_dequantize(self.ctx.h, self.h, _ptr(out)))
        return out

    def save(self, path):
        """Write the weight (format, shape, reference-layout bytes) to a file."""
        self.ctx.check(self.ctx.lib.mgn_weight_save(self.ctx.h, self.h, str(path).encode()))

    def export_ref(self):
        out = np.empty(packed_size(self.fmt, self.rows, self.cols), dtype=np.uint8)
        self.ctx.check(self.ctx.lib.mgn_weight_export_ref(self.ctx.h, self.h, _ptr(out)))
        return out

    def free(self):
        if self.h:
            self.ctx.lib.mgn_weight_free(self.ctx.h, self.h)
            self.h = None

"""ctypes front end of liboracle.so (see mgn_oracle.c for what pins each function).

Test infrastructure only: never imported by the shipped package.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_DIR = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_DIR, "liboracle.so")

Q4, Q8 = 0, 1


def build(force=False):
    """Compile liboracle.so with the Makefile beside this file."""
    args = ["make", "-C", _DIR] + (["-B"] if force else [])
    subprocess.run(args, check=True, stdout=subprocess.DEVNULL)


def _load():
    if not os.path.exists(_SO):
        build()
    lib = C.CDLL(_SO)
    f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
    u8p = np.ctypeslib.ndpointer(np.uint8, flags="C_CONTIGUOUS")
    sz = C.c_size_t
    lib.orc_f32_to_f16.restype = C.c_uint16
    lib.orc_f32_to_f16.argtypes = [C.c_float]
    lib.orc_f16_to_f32.restype = C.c_float
    lib.orc_f16_to_f32.argtypes = [C.c_uint16]
    for name in ("orc_quantize_q4", "orc_quantize_q8"):
        fn = getattr(lib, name)
        fn.restype = C.c_int
        fn.argtypes = [f32p, sz, sz, u8p]
    for name in ("orc_dequantize_q4", "orc_dequantize_q8"):
        fn = getattr(lib, name)
        fn.restype = C.c_int
        fn.argtypes = [u8p, sz, sz, f32p]
    for name in ("orc_matmul_f32", "orc_matmul_f64"):
        fn = getattr(lib, name)
        fn.restype = None
        fn.argtypes = [f32p, f32p, C.c_void_p, f32p, sz, sz, sz]
    for name in ("orc_matmul_packed_f32", "orc_matmul_q_tiled"):
        fn = getattr(lib, name)
        fn.restype = C.c_int
        fn.argtypes = [C.c_int, f32p, u8p, C.c_void_p, f32p, sz, sz, sz]
    lib.orc_num_threads.restype = C.c_int
    return lib


_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = _load()
    return _lib


def f32_to_f16_bits(x):
    return int(lib().orc_f32_to_f16(float(np.float32(x))))


def f16_bits_to_f32(bits):
    return np.float32(lib().orc_f16_to_f32(int(bits)))


def packed_size(fmt, rows, cols):
    return (rows // 32) * cols * (20 if fmt == Q4 else 36)


def quantize(fmt, w, rows=None, cols=None):
    """f32 [rows, cols] row-major -> the reference's packed bytes."""
    w = np.ascontiguousarray(w, dtype=np.float32)
    if rows is None:
        rows, cols = w.shape
    if rows % 32 != 0:
        raise ValueError("rows (K dim) must be a multiple of 32")
    out = np.zeros(packed_size(fmt, rows, cols), dtype=np.uint8)
    fn = lib().orc_quantize_q4 if fmt == Q4 else lib().orc_quantize_q8
    rc = fn(w.reshape(-1), rows, cols, out)
    assert rc == 0
    return out


def dequantize(fmt, packed, rows, cols):
    packed = np.ascontiguousarray(packed, dtype=np.uint8)
    assert packed.size == packed_size(fmt, rows, cols)
    out = np.empty(rows * cols, dtype=np.float32)
    fn = lib().orc_dequantize_q4 if fmt == Q4 else lib().orc_dequantize_q8
    rc = fn(packed, rows, cols, out)
    assert rc == 0
    return out.reshape(rows, cols)


def _dptr(d):
    return None if d is None else d.ctypes.data_as(C.c_void_p)


def matmul_f32(a, b, d=None):
    a = np.ascontiguousarray(a, dtype=np.float32)
    b = np.ascontiguousarray(b, dtype=np.float32)
    m, k = a.shape
    k2, n = b.shape
    assert k == k2
    if d is not None:
        d = np.ascontiguousarray(d, dtype=np.float32).reshape(m, n)
    c = np.empty((m, n), dtype=np.float32)
    lib().orc_matmul_f32(a.reshape(-1), b.reshape(-1), _dptr(d), c.reshape(-1), m, k, n)
    return c


def matmul_f64(a, b, d=None):
    a = np.ascontiguousarray(a, dtype=np.float32)
    b = np.ascontiguousarray(b, dtype=np.float32)
    m, k = a.shape
    k2, n = b.shape
    assert k == k2
    if d is not None:
        d = np.ascontiguousarray(d, dtype=np.float32).reshape(m, n)
    c = np.empty((m, n), dtype=np.float32)
    lib().orc_matmul_f64(a.reshape(-1), b.reshape(-1), _dptr(d), c.reshape(-1), m, k, n)
    return c


def matmul_packed(fmt, a, packed, n, d=None, tiled=False):
    """C = A x dequant(packed) (+ D) without materialising the f32 weight."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    m, k = a.shape
    packed = np.ascontiguousarray(packed, dtype=np.uint8)
    assert packed.size == packed_size(fmt, k, n)
    if d is not None:
        d = np.ascontiguousarray(d, dtype=np.float32).reshape(m, n)
    c = np.empty((m, n), dtype=np.float32)
    fn = lib().orc_matmul_q_tiled if tiled else lib().orc_matmul_packed_f32
    rc = fn(fmt, a.reshape(-1), packed, _dptr(d), c.reshape(-1), m, k, n)
    assert rc == 0
    return c


def unary(kind, v):
    """The reference's unary epilogue operations in f32 (src/codegen.rs:85-96):
    relu max(v, 0); sigmoid 1 / (1 + exp(-v)); neg -v; silu v / (1 + exp(-v))."""
    v = np.asarray(v, dtype=np.float32)
    one = np.float32(1.0)
    if kind == "relu":
        return np.maximum(v, np.float32(0.0))
    if kind == "neg":
        return -v
    with np.errstate(over="ignore"):
        e = np.exp(-v).astype(np.float32)
    if kind == "sigmoid":
        return (one / (one + e)).astype(np.float32)
    if kind == "silu":
        return (v / (one + e)).astype(np.float32)
    raise ValueError(kind)


def num_threads():
    return int(lib().orc_num_threads())


def assert_close(got, want, rel_tol=1e-3, abs_tol=1e-4):
    """The reference's tolerance helper (tests/gemv_parity.rs:61-72): an element
    passes if abs <= abs_tol OR rel <= rel_tol, rel = |x-y| / max(|x|,|y|,1e-6)."""
    got = np.asarray(got, dtype=np.float32).reshape(-1)
    want = np.asarray(want, dtype=np.float32).reshape(-1)
    assert got.shape == want.shape, (got.shape, want.shape)
    diff = np.abs(got.astype(np.float64) - want.astype(np.float64))
    scale = np.maximum(np.maximum(np.abs(got), np.abs(want)), 1e-6)
    ok = (diff <= abs_tol) | (diff / scale <= rel_tol)
    ok &= np.isfinite(got)
    if not ok.all():
        i = int(np.argmin(ok))
        raise AssertionError(
            f"{(~ok).sum()} of {ok.size} mismatches; first at [{i}]: got={got[i]!r} "
            f"want={want[i]!r} abs={diff[i]:.3e} rel={diff[i] / scale[i]:.3e}"
        )

"""ctypes binding of oracle/c/oracle.c (test infrastructure only)."""

from __future__ import annotations

import ctypes as C
import subprocess
from pathlib import Path

import numpy as np

_HERE = Path(__file__).resolve().parent
_LIB_PATH = _HERE / "_build" / "liboracle.so"


def build() -> Path:
    """Compile oracle/c/oracle.c with the Makefile next to it."""
    subprocess.run(["make", "-C", str(_HERE), "-B"], check=True,
                   capture_output=True)
    return _LIB_PATH


def _load() -> C.CDLL:
    if not _LIB_PATH.exists():
        build()
    lib = C.CDLL(str(_LIB_PATH))
    sz, p = C.c_size_t, C.c_void_p
    lib.oracle_half_to_float.restype = C.c_float
    lib.oracle_half_to_float.argtypes = [C.c_uint16]
    lib.oracle_float_to_half.restype = C.c_uint16
    lib.oracle_float_to_half.argtypes = [C.c_float]
    lib.oracle_bf16_to_float.restype = C.c_float
    lib.oracle_bf16_to_float.argtypes = [C.c_uint16]
    lib.oracle_float_to_bf16.restype = C.c_uint16
    lib.oracle_float_to_bf16.argtypes = [C.c_float]
    for name in ("oracle_half_to_float_n", "oracle_float_to_half_n",
                 "oracle_float_to_bf16_n"):
        getattr(lib, name).argtypes = [p, p, sz]
    lib.oracle_add_f32.argtypes = [p, p, p, sz]
    lib.oracle_fma_f16.argtypes = [p, sz, p, sz, p, sz, p, sz, sz, sz]
    lib.oracle_copy2d.argtypes = [sz, p, sz, sz, C.c_ssize_t, C.c_ssize_t,
                                  p, sz, sz, C.c_ssize_t, C.c_ssize_t]
    lib.oracle_softmax_f32.argtypes = [p, sz, p, sz, sz, sz]
    lib.oracle_softmax_f64.argtypes = [p, sz, p, sz, sz, sz]
    lib.oracle_quantize_f16_i8.argtypes = [p, sz, p, sz, p, sz, sz]
    lib.oracle_quotient_shortcut_mismatches.restype = C.c_uint64
    lib.oracle_quotient_shortcut_mismatches.argtypes = [
        C.c_uint32, C.c_uint32, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64),
        C.POINTER(C.c_uint64), C.POINTER(C.c_float)]
    for name in ("oracle_gemm_bf16_f32acc", "oracle_gemm_bf16_f64acc"):
        getattr(lib, name).argtypes = [p, sz, p, sz, p, p, sz, sz, sz, sz]
    lib.oracle_suggest_block_size.restype = C.c_int
    lib.oracle_suggest_block_size.argtypes = [p, p, sz]
    lib.oracle_launch_geometry.argtypes = [p, p, sz, p, p]
    return lib


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        _lib = _load()
    return _lib


def _ptr(a: np.ndarray) -> int:
    assert a.flags.c_contiguous
    return a.ctypes.data


def half_to_float(bits: np.ndarray) -> np.ndarray:
    h = np.ascontiguousarray(bits, np.uint16)
    f = np.empty(h.shape, np.float32)
    lib().oracle_half_to_float_n(_ptr(h), _ptr(f), h.size)
    return f


def float_to_half(x: np.ndarray) -> np.ndarray:
    f = np.ascontiguousarray(x, np.float32)
    h = np.empty(f.shape, np.uint16)
    lib().oracle_float_to_half_n(_ptr(f), _ptr(h), f.size)
    return h


def float_to_bf16(x: np.ndarray) -> np.ndarray:
    f = np.ascontiguousarray(x, np.float32)
    b = np.empty(f.shape, np.uint16)
    lib().oracle_float_to_bf16_n(_ptr(f), _ptr(b), f.size)
    return b


def copy2d(src: np.ndarray, dst: np.ndarray) -> None:
    """Masked window copy in place: dst[:r, :c] = src[:r, :c] over the common
    window; both may be strided 2-D views.  Nothing else of dst is written."""
    assert src.ndim == 2 and dst.ndim == 2 and src.dtype == dst.dtype
    e = src.itemsize
    assert all(s % e == 0 for s in src.strides + dst.strides)
    lib().oracle_copy2d(e, src.ctypes.data, src.shape[0], src.shape[1],
                        src.strides[0] // e, src.strides[1] // e,
                        dst.ctypes.data, dst.shape[0], dst.shape[1],
                        dst.strides[0] // e, dst.strides[1] // e)


def add_f32(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    a = np.ascontiguousarray(a, np.float32)
    b = np.ascontiguousarray(b, np.float32)
    c = np.empty_like(a)
    lib().oracle_add_f32(_ptr(a), _ptr(b), _ptr(c), a.size)
    return c


def fma_f16(a: np.ndarray, b: np.ndarray, c: np.ndarray) -> np.ndarray:
    a, b, c = (np.ascontiguousarray(v, np.float16) for v in (a, b, c))
    rows = a.shape[0] if a.ndim == 2 else 1
    cols = a.shape[-1]
    d = np.empty_like(a)
    lib().oracle_fma_f16(_ptr(a), cols, _ptr(b), cols, _ptr(c), cols, _ptr(d),
                         cols, rows, cols)
    return d


def softmax(x: np.ndarray, f64: bool = False) -> np.ndarray:
    x = np.ascontiguousarray(x, np.float32)
    y = np.empty_like(x)
    fn = lib().oracle_softmax_f64 if f64 else lib().oracle_softmax_f32
    fn(_ptr(x), x.shape[1], _ptr(y), x.shape[1], x.shape[0], x.shape[1])
    return y


def quantize(x: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
    x = np.ascontiguousarray(x, np.float16)
    q = np.empty(x.shape, np.int8)
    s = np.empty(x.shape[0], np.float32)
    lib().oracle_quantize_f16_i8(_ptr(x), x.shape[1], _ptr(q), x.shape[1],
                                 _ptr(s), x.shape[0], x.shape[1])
    return q, s


def quotient_shortcut_mismatches(lo: int, hi: int):
    """(value mismatches, sign-of-zero-only mismatches, integer mismatches,
    pairs checked, max |rint(q)|) for absmax bit patterns in [lo, hi)."""
    zero, bad_int, checked, maxq = (C.c_uint64(), C.c_uint64(), C.c_uint64(),
                                    C.c_float())
    bad = lib().oracle_quotient_shortcut_mismatches(
        lo, hi, C.byref(zero), C.byref(bad_int), C.byref(checked),
        C.byref(maxq))
    return (int(bad), int(zero.value), int(bad_int.value), int(checked.value),
            float(maxq.value))


def gemm_bf16(a_bits: np.ndarray, bt_bits: np.ndarray, f64: bool = False):
    """Returns (c_bf16_bits, c_fp32) for A[M,K], Bt[N,K] given as uint16."""
    a = np.ascontiguousarray(a_bits, np.uint16)
    bt = np.ascontiguousarray(bt_bits, np.uint16)
    m, k = a.shape
    n = bt.shape[0]
    c16 = np.empty((m, n), np.uint16)
    c32 = np.empty((m, n), np.float32)
    fn = lib().oracle_gemm_bf16_f64acc if f64 else lib().oracle_gemm_bf16_f32acc
    fn(_ptr(a), k, _ptr(bt), k, _ptr(c16), _ptr(c32), n, m, n, k)
    return c16, c32


def suggest_block_size(global_sizes):
    g = (C.c_size_t * len(global_sizes))(*global_sizes)
    b = (C.c_size_t * max(len(global_sizes), 1))()
    rc = lib().oracle_suggest_block_size(g, b, len(global_sizes))
    return rc, tuple(b[i] for i in range(len(global_sizes)))


def launch_geometry(work, group):
    w = (C.c_size_t * len(work))(*work)
    g = (C.c_size_t * len(group))(*group)
    grid, block = (C.c_size_t * 3)(), (C.c_size_t * 3)()
    lib().oracle_launch_geometry(w, g, len(work), grid, block)
    return tuple(grid), tuple(block)

"""Thin Python layer over the C ABI of libhc_amd_runtime.so.

Everything that touches the GPU goes through the exported C functions declared
in include/hc_amd_runtime.h: device memory (olAllocDevice), copies
(hcamdMemcpy), the typed kernel launchers (hcamdLaunch*), events and the
generic module/kernel/launch calls.  There is no CPU fallback here: without the
native library the import of hc_amd.py_runtime fails, and without a GPU the
first call raises HcRuntimeError.
"""

from __future__ import annotations

import ctypes as C
from dataclasses import dataclass

import numpy as np

from . import py_runtime

_rt = py_runtime.runtime_lib
_py = py_runtime.pyabi_lib


class HcRuntimeError(RuntimeError):
    """An ol*/hcamd* call reported failure; carries the runtime's message."""


# ---------------------------------------------------------------------------
# ctypes signatures (one place, mirrors include/hc_amd_runtime.h)
# ---------------------------------------------------------------------------
_vp, _sz, _ssz, _int = C.c_void_p, C.c_size_t, C.c_ssize_t, C.c_int
ERROR_CALLBACK = C.CFUNCTYPE(None, _vp, _int, C.c_char_p)


def _sig(lib, name, restype, *argtypes):
    fn = getattr(lib, name)
    fn.restype = restype
    fn.argtypes = list(argtypes)
    return fn


_sz_p = C.POINTER(_sz)
olCreateDevice = _sig(_rt, "olCreateDevice", _vp, C.c_char_p, ERROR_CALLBACK, _vp)
olReleaseDevice = _sig(_rt, "olReleaseDevice", None, _vp)
olCreateModule = _sig(_rt, "olCreateModule", _vp, _vp, _vp, _sz)
olReleaseModule = _sig(_rt, "olReleaseModule", None, _vp)
olGetKernel = _sig(_rt, "olGetKernel", _vp, _vp, C.c_char_p)
olReleaseKernel = _sig(_rt, "olReleaseKernel", None, _vp)
olSuggestBlockSize = _sig(_rt, "olSuggestBlockSize", _int, _vp, _sz_p, _sz_p, _sz)
olCreateQueue = _sig(_rt, "olCreateQueue", _vp, _vp)
olReleaseQueue = _sig(_rt, "olReleaseQueue", None, _vp)
olSyncQueue = _sig(_rt, "olSyncQueue", _int, _vp)
olAllocDevice = _sig(_rt, "olAllocDevice", _vp, _vp, _sz, _sz)
olDeallocDevice = _sig(_rt, "olDeallocDevice", None, _vp, _vp)
olLaunchKernel = _sig(_rt, "olLaunchKernel", _int, _vp, _vp, _sz_p, _sz_p, _sz,
                      C.POINTER(_vp), _sz, _sz)
hcgpuGetKernel = _sig(_rt, "hcgpuGetKernel", _vp, C.POINTER(_vp), C.c_char_p, _vp,
                      _sz, C.c_char_p)
hcgpuSuggestBlockSize = _sig(_rt, "hcgpuSuggestBlockSize", None, _vp, _sz_p, _sz_p, _sz)
hcgpuLaunchKernel = _sig(_rt, "hcgpuLaunchKernel", None, _vp, _sz_p, _sz_p, _sz,
                         C.POINTER(_vp), _sz, _sz)
hcamdGetDefaultQueue = _sig(_rt, "hcamdGetDefaultQueue", _vp, C.c_char_p)
hcamdGetDefaultDevice = _sig(_rt, "hcamdGetDefaultDevice", _vp, C.c_char_p)
hcamdQueueDevice = _sig(_rt, "hcamdQueueDevice", _vp, _vp)
hcamdBuiltinModuleCount = _sig(_rt, "hcamdBuiltinModuleCount", _sz)
hcamdGetBuiltinModule = _sig(_rt, "hcamdGetBuiltinModule", _int, _sz,
                             C.POINTER(C.c_char_p), C.POINTER(_vp), _sz_p)
hcamdGetBuiltinKernel = _sig(_rt, "hcamdGetBuiltinKernel", _vp, _vp, C.c_char_p,
                             C.c_char_p)
hcamdMemcpy = _sig(_rt, "hcamdMemcpy", _int, _vp, _vp, _vp, _sz, _int)
hcamdFill32 = _sig(_rt, "hcamdFill32", _int, _vp, _vp, C.c_uint32, _sz)
hcamdEventCreate = _sig(_rt, "hcamdEventCreate", _vp, _vp)
hcamdEventDestroy = _sig(_rt, "hcamdEventDestroy", None, _vp)
hcamdEventRecord = _sig(_rt, "hcamdEventRecord", _int, _vp)
hcamdEventSynchronize = _sig(_rt, "hcamdEventSynchronize", _int, _vp)
hcamdEventElapsedMs = _sig(_rt, "hcamdEventElapsedMs", _int, _vp, _vp,
                           C.POINTER(C.c_float))
hcamdDeviceInfo = _sig(_rt, "hcamdDeviceInfo", _int, _vp, C.POINTER(_int),
                       C.POINTER(_int), C.POINTER(_int), C.POINTER(_int), _sz_p,
                       C.c_char_p, _sz)
hcamdSetVariant = _sig(_rt, "hcamdSetVariant", _int, C.c_char_p, _int)
hcamdSetThreadVariant = _sig(_rt, "hcamdSetThreadVariant", _int, C.c_char_p, _int)
hcamdLastKernelName = _sig(_rt, "hcamdLastKernelName", C.c_char_p)
hcamdLaunchTranspose2D = _sig(_rt, "hcamdLaunchTranspose2D", _int, _vp, _sz, _vp, _sz, _vp, _sz, _sz, _sz)
hcamdLaunchCopy2D = _sig(_rt, "hcamdLaunchCopy2D", _int, _vp, _sz, _vp, _sz, _sz,
                         _ssz, _ssz, _vp, _sz, _sz, _ssz, _ssz)
hcamdLaunchCopy2DTiled = _sig(_rt, "hcamdLaunchCopy2DTiled", _int, _vp, _sz, _vp, _vp,
                              _sz, _sz, _ssz, _ssz, _sz, _sz, _sz)
class AffineId(C.Structure):
    """HcamdAffineId of include/hc_amd_runtime.h."""
    _fields_ = [("c", C.c_int64), ("g", C.c_int64 * 3), ("l", C.c_int64 * 3)]


hcamdLaunchIdScatter = _sig(_rt, "hcamdLaunchIdScatter", _int, _vp, _vp, _int, _sz, _sz_p,
                            C.POINTER(_ssz), C.POINTER(AffineId), C.POINTER(AffineId), _sz, _sz_p,
                            _sz_p, _int)
# (the measurement entry points of include/hc_amd_bench.h)
hcamdLaunchStream = _sig(_rt, "hcamdLaunchStream", _int, _vp, _int, _int, C.POINTER(_vp), _vp, _sz)
hcamdProbesBuilt = _sig(_rt, "hcamdProbesBuilt", _int)
hcamdLaunchAddF32 = _sig(_rt, "hcamdLaunchAddF32", _int, _vp, _vp, _vp, _vp, _sz)
hcamdLaunchFmaF16 = _sig(_rt, "hcamdLaunchFmaF16", _int, _vp, _vp, _sz, _vp, _sz, _vp,
                         _sz, _vp, _sz, _sz, _sz)
hcamdLaunchSoftmaxF32 = _sig(_rt, "hcamdLaunchSoftmaxF32", _int, _vp, _vp, _sz, _vp,
                             _sz, _sz, _sz)
hcamdLaunchQuantizeF16I8 = _sig(_rt, "hcamdLaunchQuantizeF16I8", _int, _vp, _vp, _sz,
                                _vp, _sz, _vp, _sz, _sz)
hcamdLaunchGemmBF16 = _sig(_rt, "hcamdLaunchGemmBF16", _int, _vp, _vp, _sz, _vp, _sz,
                           _vp, _sz, _sz, _sz, _sz)
hcamdLaunchGemmF16 = _sig(_rt, "hcamdLaunchGemmF16", _int, _vp, _vp, _sz, _vp, _sz,
                          _vp, _sz, _sz, _sz, _sz)


class MapInstr(C.Structure):
    """HcamdMapInstr of include/hc_amd_runtime.h."""
    _fields_ = [("op", C.c_uint16), ("arg", C.c_uint16), ("imm", C.c_float)]


hcamdLaunchMap = _sig(_rt, "hcamdLaunchMap", _int, _vp, C.POINTER(MapInstr), _sz,
                      C.POINTER(_vp), C.POINTER(_int), _sz_p, _sz, _vp, _int, _sz, _sz, _sz)
hcamdLaunchPairwiseDistF32 = _sig(_rt, "hcamdLaunchPairwiseDistF32", _int, _vp, _vp, _sz, _vp,
                                  _sz, _vp, _sz, _sz, _sz, _sz)
hcamdLaunchMapSum = _sig(_rt, "hcamdLaunchMapSum", _int, _vp, C.POINTER(MapInstr), _sz,
                         C.POINTER(_vp), C.POINTER(_int), _sz_p, _sz, _vp, _sz, _sz)

hcamdLaunchIMap = _sig(_rt, "hcamdLaunchIMap", _int, _vp, C.POINTER(MapInstr), _sz, C.POINTER(_vp),
                       _sz_p, _sz, _vp, _int, _sz, _sz, _sz)
hcamdLaunchFMap = _sig(_rt, "hcamdLaunchFMap", _int, _vp, C.POINTER(MapInstr), _sz, C.POINTER(_vp),
                       C.POINTER(_int), _sz_p, _sz, _vp, _int, _sz, _sz, _sz, _int)
hcamdMapReduceColsWorkspace = _sig(_rt, "hcamdMapReduceColsWorkspace", _sz, _sz, _sz)
hcamdLaunchMapReduceCols = _sig(_rt, "hcamdLaunchMapReduceCols", _int, _vp, _int,
                                C.POINTER(MapInstr), _sz, C.POINTER(MapInstr), _sz,
                                C.POINTER(_vp), C.POINTER(_int), _sz_p, _sz, _vp, _int, _sz, _sz,
                                _vp, _sz)
# The same launch without a workspace: the bands meet in the library's static
# device scratch array (for callers that cannot allocate device memory).
NOALLOC_SCRATCH_BYTES = 4 << 20
hcamdLaunchMapReduceColsNoAlloc = _sig(_rt, "hcamdLaunchMapReduceColsNoAlloc", _int, _vp, _int,
                                       C.POINTER(MapInstr), _sz, C.POINTER(MapInstr), _sz,
                                       C.POINTER(_vp), C.POINTER(_int), _sz_p, _sz, _vp, _int,
                                       _sz, _sz)


class RowStage(C.Structure):
    """HcamdRowStage of include/hc_amd_runtime.h."""
    _fields_ = [("kind", C.c_uint32), ("nInstr", C.c_uint32), ("dst", C.c_uint32)]


hcamdLaunchRowProgram = _sig(_rt, "hcamdLaunchRowProgram", _int, _vp, C.POINTER(MapInstr),
                             C.POINTER(RowStage), _sz, C.POINTER(_vp), C.POINTER(_int), _sz_p,
                             _sz, C.POINTER(_vp), C.POINTER(_int), _sz, _vp, _int, _sz, _sz, _sz)


class GatherOperand(C.Structure):
    """HcamdGatherOperand of include/hc_amd_runtime.h."""
    _fields_ = [("ndim", _int), ("shape", _sz * 4), ("strides", _sz * 4),
                ("starts", C.POINTER(C.c_int32)), ("rowIndex", C.POINTER(C.c_int32)),
                ("colIndex", C.POINTER(C.c_int32))]


hcamdGatherGemmCreate = _sig(_rt, "hcamdGatherGemmCreate", _vp, _vp, C.POINTER(GatherOperand),
                             C.POINTER(GatherOperand), C.POINTER(GatherOperand), _sz, _sz,
                             _sz, _sz)
hcamdGatherGemmLaunchF32 = _sig(_rt, "hcamdGatherGemmLaunchF32", _int, _vp, _vp, _vp, _vp, _vp)
hcamdGatherGemmLaunch = _sig(_rt, "hcamdGatherGemmLaunch", _int, _vp, _vp, _int, _vp, _vp, _vp)
hcamdGatherGemmRelease = _sig(_rt, "hcamdGatherGemmRelease", None, _vp)
class GatherMapOperand(C.Structure):
    """HcamdGatherMapOperand of include/hc_amd_runtime.h."""
    _fields_ = [("ndim", _int), ("shape", _sz * 4), ("strides", _sz * 4),
                ("starts", C.POINTER(C.c_int32)), ("index", C.POINTER(C.c_int32))]


hcamdGatherMapCreate = _sig(_rt, "hcamdGatherMapCreate", _vp, _vp, C.POINTER(GatherMapOperand), _sz, _sz, _sz)
hcamdGatherMapLaunch = _sig(_rt, "hcamdGatherMapLaunch", _int, _vp, _vp, _vp, _sz, C.POINTER(_vp),
                            C.POINTER(_int), _vp, _int, _int, _sz)
hcamdGatherMapRelease = _sig(_rt, "hcamdGatherMapRelease", None, _vp)
hcamdConvertPyArray = _sig(_py, "hcamdConvertPyArray", _int, C.py_object, _int, _vp,
                           _sz_p, C.c_char_p, _sz)
hcamdConvertPyInt64 = _sig(_py, "hcamdConvertPyInt64", _int, C.py_object,
                           C.POINTER(C.c_int64), C.c_char_p, _sz)

H2D, D2H, D2D = 0, 1, 2


# ---------------------------------------------------------------------------
# Device / queue with a Python error callback
# ---------------------------------------------------------------------------
class Context:
    """One device and one queue (stream).  Error messages from the runtime's
    callback are collected and raised as HcRuntimeError."""

    def __init__(self, desc: str = "hip:0"):
        self.desc = desc
        self.messages: list[str] = []

        def on_error(_ctx, _sev, text):
            self.messages.append(text.decode(errors="replace").rstrip())

        self._cb = ERROR_CALLBACK(on_error)     # keep alive
        self.device = olCreateDevice(desc.encode(), self._cb, None)
        if not self.device:
            raise HcRuntimeError(self._drain() or f"olCreateDevice({desc!r}) failed")
        self.queue = olCreateQueue(self.device)
        if not self.queue:
            msg = self._drain()
            olReleaseDevice(self.device)
            raise HcRuntimeError(msg or "olCreateQueue failed")

    def _drain(self) -> str:
        msg = "; ".join(self.messages)
        self.messages.clear()
        return msg

    def check(self, rc: int, what: str) -> None:
        if rc:
            raise HcRuntimeError(f"{what}: {self._drain() or 'failed'}")

    def synchronize(self) -> None:
        self.check(olSyncQueue(self.queue), "olSyncQueue")

    def info(self) -> dict:
        cu, clk, mclk, bus = _int(), _int(), _int(), _int()
        mem = _sz()
        arch = C.create_string_buffer(64)
        self.check(hcamdDeviceInfo(self.device, C.byref(cu), C.byref(clk), C.byref(mclk),
                                   C.byref(bus), C.byref(mem), arch, 64), "hcamdDeviceInfo")
        return {"compute_units": cu.value, "clock_khz": clk.value,
                "mem_clock_khz": mclk.value, "mem_bus_bits": bus.value,
                "total_mem": mem.value, "arch": arch.value.decode()}


_default: Context | None = None


def default_context(desc: str = "hip:0") -> Context:
    """Process-wide context; the first device description wins, as in the
    reference (python/cpp/py-runtime/src/GpuRuntime.cpp:31-39)."""
    global _default
    if _default is None:
        _default = Context(desc)
    return _default


# ---------------------------------------------------------------------------
# Arrays
# ---------------------------------------------------------------------------
@dataclass
class Memref:
    """ptr / shape / strides (elements) / itemsize of any array-like, obtained
    through the PyObject* half of the C ABI (hcamdConvertPyArray)."""
    ptr: int
    shape: tuple
    strides: tuple
    itemsize: int

    @property
    def size(self) -> int:
        return int(np.prod(self.shape, dtype=np.int64)) if self.shape else 1

    def is_contiguous(self) -> bool:
        acc = 1
        for n, s in zip(reversed(self.shape), reversed(self.strides)):
            if n != 1 and s != acc:
                return False
            acc *= n
        return True


def as_memref(obj, rank: int | None = None) -> Memref:
    if rank is None:
        rank = len(obj.shape)
    words = (C.c_int64 * (3 + 2 * max(rank, 1)))()
    item = _sz()
    err = C.create_string_buffer(256)
    if hcamdConvertPyArray(obj, rank, C.cast(words, _vp), C.byref(item), err, 256):
        raise HcRuntimeError(err.value.decode(errors="replace"))
    return Memref(ptr=int(words[1]) & (2 ** 64 - 1),
                  shape=tuple(int(words[3 + i]) for i in range(rank)),
                  strides=tuple(int(words[3 + rank + i]) for i in range(rank)),
                  itemsize=int(item.value))


_TYPESTR = {"float32": "<f4", "float16": "<f2", "int8": "|i1", "uint8": "|u1",
            "int16": "<i2", "uint16": "<u2", "int32": "<i4", "uint32": "<u4",
            "int64": "<i8", "uint64": "<u8", "float64": "<f8", "bool": "|b1"}


class DeviceArray:
    """Dense row-major array in device memory owned by this object.  bf16 data
    is held as uint16 bit patterns with `bf16=True` (NumPy has no bfloat16)."""

    def __init__(self, shape, dtype, ctx: Context | None = None, bf16: bool = False):
        self.ctx = ctx or default_context()
        self.shape = tuple(int(s) for s in (shape if hasattr(shape, "__iter__") else (shape,)))
        self.dtype = np.dtype(dtype)
        self.bf16 = bool(bf16)
        self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * self.dtype.itemsize
        self.ptr = olAllocDevice(self.ctx.queue, max(self.nbytes, 16), 256)
        if not self.ptr:
            raise HcRuntimeError(self.ctx._drain() or "olAllocDevice failed")

    # dense row-major strides in elements
    @property
    def strides(self):
        out, acc = [], 1
        for n in reversed(self.shape):
            out.append(acc)
            acc *= n
        return tuple(reversed(out))

    @property
    def __cuda_array_interface__(self):
        return {"shape": self.shape, "typestr": _TYPESTR[self.dtype.name],
                "data": (int(self.ptr), False), "strides": None, "version": 2}

    def copy_from_host(self, host: np.ndarray) -> "DeviceArray":
        host = np.ascontiguousarray(host)
        if host.nbytes != self.nbytes:
            raise ValueError("size mismatch in copy_from_host")
        self.ctx.check(hcamdMemcpy(self.ctx.queue, self.ptr, host.ctypes.data, self.nbytes, H2D),
                       "hcamdMemcpy(H2D)")
        self.ctx.synchronize()
        return self

    def to_host(self) -> np.ndarray:
        out = np.empty(self.shape, self.dtype)
        self.ctx.synchronize()
        self.ctx.check(hcamdMemcpy(self.ctx.queue, out.ctypes.data, self.ptr, self.nbytes, D2H),
                       "hcamdMemcpy(D2H)")
        self.ctx.synchronize()
        return out

    def fill_bytes32(self, word: int) -> "DeviceArray":
        self.ctx.check(hcamdFill32(self.ctx.queue, self.ptr, word & 0xFFFFFFFF,
                                   (self.nbytes + 3) // 4), "hcamdFill32")
        return self

    def free(self) -> None:
        if getattr(self, "ptr", None):
            olDeallocDevice(self.ctx.queue, self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def to_device(host: np.ndarray, ctx: Context | None = None, bf16: bool = False) -> DeviceArray:
    host = np.ascontiguousarray(host)
    return DeviceArray(host.shape, host.dtype, ctx, bf16).copy_from_host(host)


def empty_like(a: DeviceArray) -> DeviceArray:
    return DeviceArray(a.shape, a.dtype, a.ctx, a.bf16)


# ---------------------------------------------------------------------------
# Typed launchers
# ---------------------------------------------------------------------------
def _ctx_of(*arrays) -> Context:
    for a in arrays:
        ctx = getattr(a, "ctx", None)
        if isinstance(ctx, Context):
            return ctx
    return default_context()


class Plan:
    """A validated launch: the C entry point and its argument values.  Building
    a plan does the Python-side checks and pointer extraction once; launch()
    is then a single foreign call, which keeps the host out of the way when the
    same kernel is enqueued many times."""

    __slots__ = ("ctx", "fn", "args", "what", "keep")

    def __init__(self, ctx, fn, args, what, keep=()):
        self.ctx, self.fn, self.args, self.what, self.keep = ctx, fn, args, what, keep

    def launch(self, sync: bool = False) -> None:
        rc = self.fn(*self.args)
        if rc:
            self.ctx.check(rc, self.what)
        if sync:
            self.ctx.synchronize()


def _rows_cols(m: Memref):
    if len(m.shape) == 1:
        if m.shape[0] > 1 and m.strides[0] != 1:
            raise HcRuntimeError("a 1-D operand must be contiguous (stride 1)")
        return 1, m.shape[0], m.shape[0]
    if len(m.shape) == 2:
        if m.strides[1] != 1 and m.shape[1] > 1:
            raise HcRuntimeError("rows must be contiguous (last stride 1)")
        return m.shape[0], m.shape[1], (m.strides[0] if m.shape[0] > 1 else m.shape[1])
    raise HcRuntimeError("expected a 1-D or 2-D array")


def _expect(m: Memref, itemsize: int, name: str):
    if m.itemsize != itemsize:
        raise HcRuntimeError(f"{name}: element size {m.itemsize}, expected {itemsize}")


def plan_copy2d(src, dst) -> Plan:
    ctx = _ctx_of(src, dst)
    s, d = as_memref(src), as_memref(dst)
    if s.itemsize != d.itemsize or len(s.shape) != len(d.shape) or len(s.shape) not in (1, 2):
        raise HcRuntimeError("copy2d: element size / rank mismatch")
    if len(s.shape) == 1:
        s = Memref(s.ptr, (1,) + s.shape, (0,) + s.strides, s.itemsize)
        d = Memref(d.ptr, (1,) + d.shape, (0,) + d.strides, d.itemsize)
    return Plan(ctx, hcamdLaunchCopy2D,
                (ctx.queue, s.itemsize, s.ptr, s.shape[0], s.shape[1], s.strides[0],
                 s.strides[1], d.ptr, d.shape[0], d.shape[1], d.strides[0], d.strides[1]),
                "hcamdLaunchCopy2D", (src, dst))


def plan_transpose2d(src, dst) -> Plan:
    """dst[c, r] = src[r, c] over the part of src that fits dst transposed (see
    hcamdLaunchTranspose2D); unit inner strides, equal element sizes."""
    ctx = _ctx_of(src, dst)
    s, d = as_memref(src, 2), as_memref(dst, 2)
    if s.itemsize != d.itemsize or s.strides[1] != 1 or d.strides[1] != 1:
        raise HcRuntimeError("transpose2d: unit inner stride and equal element size required")
    rows, cols = min(s.shape[0], d.shape[1]), min(s.shape[1], d.shape[0])
    return Plan(ctx, hcamdLaunchTranspose2D,
                (ctx.queue, s.itemsize, s.ptr, s.strides[0], d.ptr, d.strides[0], rows, cols),
                "hcamdLaunchTranspose2D", (src, dst))


def plan_copy2d_tiled(src, dst, block_x: int, block_y: int, unroll: int = 1) -> Plan:
    ctx = _ctx_of(src, dst)
    s, d = as_memref(src, 2), as_memref(dst, 2)
    if s.itemsize != d.itemsize or s.strides[1] != 1 or d.strides[1] != 1:
        raise HcRuntimeError("copy2d_tiled: unit inner stride and equal element size required")
    rows, cols = min(s.shape[0], d.shape[0]), min(s.shape[1], d.shape[1])
    return Plan(ctx, hcamdLaunchCopy2DTiled,
                (ctx.queue, s.itemsize, s.ptr, d.ptr, rows, cols, s.strides[0], d.strides[0],
                 block_x, block_y, unroll), "hcamdLaunchCopy2DTiled", (src, dst))


I32, I64 = 3, 4


def plan_id_scatter(out, index, value, group_count, group_shape, per_item=True, out_type=None) -> Plan:
    """out[index] = value for every work-item (or once per group), index (one
    (c, g, l) triple per dimension of out) and value affine in group id and
    local id: c + sum(g[k] * group_id[k]) + sum(l[k] * local_id[k]) (see
    hcamdLaunchIdScatter)."""
    ctx = _ctx_of(out)
    m = as_memref(out)
    if out_type is None:
        name = getattr(getattr(out, "dtype", None), "name", None) or str(getattr(out, "dtype", ""))
        out_type = {"int32": I32, "int64": I64, "float32": F32}.get(name.replace("torch.", ""))
        if out_type is None:
            raise HcRuntimeError(f"id_scatter: output type {name!r} (int32, int64, float32 only)")
    rank = len(group_shape)

    def pack(t):
        c, g, l = t
        a = AffineId()
        a.c = int(c)
        for k in range(3):
            a.g[k] = int(g[k]) if k < len(g) else 0
            a.l[k] = int(l[k]) if k < len(l) else 0
        return a
    if len(index) != len(m.shape):
        raise HcRuntimeError("id_scatter: one index per dimension of the output")
    idx = (AffineId * len(index))(*[pack(t) for t in index])
    val = pack(value)
    shape = (_sz * len(m.shape))(*m.shape)
    strides = (_ssz * len(m.shape))(*m.strides)
    counts = (_sz * rank)(*group_count)
    gshape = (_sz * rank)(*group_shape)
    return Plan(ctx, hcamdLaunchIdScatter,
                (ctx.queue, m.ptr, out_type, len(m.shape), shape, strides, idx, C.byref(val), rank,
                 counts, gshape, 1 if per_item else 0), "hcamdLaunchIdScatter",
                (out, idx, val, shape, strides, counts, gshape))


STREAM_WRITE = {"none": 0, "full": 1, "half": 2}


def plan_stream(inputs, out, write="full") -> Plan:
    """Stream calibration (see hcamdLaunchStream): the inputs (0..3 contiguous
    arrays of equal byte size, a multiple of 16 KiB) are added in 32-bit lanes;
    `write` is "full" (the sum), "half" (xor of each sum word's halves, half the
    bytes) or "none" (one 32-bit total per 16 KiB)."""
    inputs = list(inputs)
    ctx = _ctx_of(*inputs, out)
    ms = [as_memref(x) for x in inputs]
    mo = as_memref(out)
    if any(not m.is_contiguous() for m in ms + [mo]):
        raise HcRuntimeError("stream: contiguous arrays only")
    sizes = {m.size * m.itemsize for m in ms}
    if len(sizes) > 1:
        raise HcRuntimeError("stream: inputs of different sizes")
    out_bytes = mo.size * mo.itemsize
    nbytes = sizes.pop() if sizes else out_bytes
    need = {"full": nbytes, "half": nbytes // 2, "none": nbytes // 4096}[write]
    if out_bytes < need:
        raise HcRuntimeError(f"stream: the output holds {out_bytes} bytes, {need} needed")
    ptrs = (_vp * 3)(*[m.ptr for m in ms])
    return Plan(ctx, hcamdLaunchStream, (ctx.queue, len(ms), STREAM_WRITE[write], ptrs, mo.ptr,
                                         nbytes), "hcamdLaunchStream", (inputs, out, ptrs))


def plan_add_f32(a, b, c) -> Plan:
    ctx = _ctx_of(a, b, c)
    ma, mb, mc = as_memref(a), as_memref(b), as_memref(c)
    for m, n in ((ma, "a"), (mb, "b"), (mc, "c")):
        _expect(m, 4, n)
        if not m.is_contiguous():
            raise HcRuntimeError("add_f32: arrays must be contiguous")
    if not (ma.size == mb.size == mc.size):
        raise HcRuntimeError("add_f32: size mismatch")
    return Plan(ctx, hcamdLaunchAddF32, (ctx.queue, ma.ptr, mb.ptr, mc.ptr, ma.size),
                "hcamdLaunchAddF32", (a, b, c))


def plan_fma_f16(a, b, c, d) -> Plan:
    ctx = _ctx_of(a, b, c, d)
    ms = [as_memref(v) for v in (a, b, c, d)]
    geo = []
    for m, n in zip(ms, "abcd"):
        _expect(m, 2, n)
        geo.append(_rows_cols(m))
    rows, cols = geo[0][0], geo[0][1]
    if any(g[0] != rows or g[1] != cols for g in geo):
        raise HcRuntimeError("fma_f16: shape mismatch")
    return Plan(ctx, hcamdLaunchFmaF16,
                (ctx.queue, ms[0].ptr, geo[0][2], ms[1].ptr, geo[1][2], ms[2].ptr, geo[2][2],
                 ms[3].ptr, geo[3][2], rows, cols), "hcamdLaunchFmaF16", (a, b, c, d))


# Opcodes of the fused elementwise map (enum HcamdMapOp)
MAP_OPS = {"in": 1, "const": 2, "add": 3, "sub": 4, "mul": 5, "div": 6, "max": 7, "min": 8,
           "rsub": 9, "rdiv": 10, "addi": 11, "subi": 12, "muli": 13, "divi": 14, "maxi": 15,
           "mini": 16, "rsubi": 17, "rdivi": 18, "neg": 19, "abs": 20, "sqrt": 21, "rint": 22,
           "exp": 23, "log": 24, "tanh": 25, "r16": 26, "add_in": 27, "sub_in": 28,
           "mul_in": 29, "div_in": 30, "max_in": 31, "min_in": 32, "rsub_in": 33,
           "rdiv_in": 34,
           # the tile operator `/` under numpy.ma's rule, ** and the domain functions
           "mdiv": 35, "rmdiv": 36, "mdivi": 37, "rmdivi": 38, "mdiv_in": 39, "rmdiv_in": 40,
           "clear": 41, "powchk": 42, "msqrt": 43, "mlog": 44}
MAP_MAX_INPUTS, MAP_MAX_INSTRS, MAP_STACK_DEPTH = 4, 32, 4
# Row programs (hcamdLaunchRowProgram): opcodes that read row scalars, stage kinds, limits
MAP_OPS.update({"red": 45, "add_red": 46, "sub_red": 47, "mul_red": 48, "div_red": 49,
                "max_red": 50, "min_red": 51, "rsub_red": 52, "rdiv_red": 53,
                "mdiv_red": 54, "rmdiv_red": 55,
                # push a row scalar as a value, deactivated or not; numpy.ma.sqrt;
                # (last in a stage) the result is active iff row scalar `arg` is positive
                "red0": 56, "masqrt": 57, "livepos": 58,
                # (last in a STORE stage) every element is stored, a deactivated
                # one with the value numpy.ma leaves in it
                "frozen": 59})
ROW_KINDS = {"sum": 0, "max": 1, "min": 2, "scalar": 3, "store": 4, "store_col": 5, "count": 6}
ROW_MAX_STAGES, ROW_MAX_SCALARS, ROW_MAX_INSTRS = 16, 16, 128
F32, F16, BF16 = 0, 1, 2


def plan_map(program, inputs, out, types=None) -> Plan:
    """out = f(inputs...) element by element; `program` is a sequence of
    (opname, arg, imm) triples in postfix order (see MAP_OPS).  Arrays are
    fp32 or fp16 (by element size, or `types` = list of F32/F16 for inputs
    followed by the output), 1-D or 2-D with contiguous rows, all of one
    shape."""
    arrays = list(inputs) + [out]
    ctx = _ctx_of(*arrays)
    ms = [as_memref(v) for v in arrays]
    geo = [_rows_cols(m) for m in ms]
    rows, cols = geo[-1][0], geo[-1][1]
    if any(g[0] != rows or g[1] != cols for g in geo):
        raise HcRuntimeError("map: shape mismatch")
    if types is None:
        types = []
        for m in ms:
            if m.itemsize not in (2, 4):
                raise HcRuntimeError(f"map: element size {m.itemsize} (fp32 and fp16 only)")
            types.append(F16 if m.itemsize == 2 else F32)
    n_in = len(inputs)
    prog = (MapInstr * max(len(program), 1))()
    for i, (name, arg, imm) in enumerate(program):
        prog[i].op, prog[i].arg, prog[i].imm = MAP_OPS[name], int(arg), float(imm)
    ptrs = (_vp * max(n_in, 1))(*[m.ptr for m in ms[:-1]])
    tys = (_int * max(n_in, 1))(*types[:n_in])
    lds = (_sz * max(n_in, 1))(*[g[2] for g in geo[:-1]])
    return Plan(ctx, hcamdLaunchMap,
                (ctx.queue, prog, len(program), ptrs, tys, lds, n_in, ms[-1].ptr, types[-1],
                 geo[-1][2], rows, cols), "hcamdLaunchMap", (arrays, prog, ptrs, tys, lds))


def plan_map_sum(program, inputs, cell, index: int = 0, types=None) -> Plan:
    """cell[index] += sum of f(inputs...) over all elements (fp32 atomic
    accumulation); `cell` is an fp32 array, the inputs are as for plan_map."""
    arrays = list(inputs)
    ctx = _ctx_of(*arrays, cell)
    ms = [as_memref(v) for v in arrays]
    mc = as_memref(cell)
    _expect(mc, 4, "cell")
    n_cells = 1
    for s in mc.shape:
        n_cells *= s
    if not mc.is_contiguous() or not 0 <= index < n_cells:
        raise HcRuntimeError("map_sum: the accumulator must be a contiguous fp32 array and "
                             "the index inside it")
    geo = [_rows_cols(m) for m in ms]
    rows, cols = geo[0][0], geo[0][1]
    if any(g[0] != rows or g[1] != cols for g in geo):
        raise HcRuntimeError("map_sum: shape mismatch")
    if types is None:
        types = []
        for m in ms:
            if m.itemsize not in (2, 4):
                raise HcRuntimeError(f"map_sum: element size {m.itemsize} (fp32 and fp16 only)")
            types.append(F16 if m.itemsize == 2 else F32)
    n_in = len(arrays)
    prog = (MapInstr * max(len(program), 1))()
    for i, (name, arg, imm) in enumerate(program):
        prog[i].op, prog[i].arg, prog[i].imm = MAP_OPS[name], int(arg), float(imm)
    ptrs = (_vp * n_in)(*[m.ptr for m in ms])
    tys = (_int * n_in)(*types[:n_in])
    lds = (_sz * n_in)(*[g[2] for g in geo])
    return Plan(ctx, hcamdLaunchMapSum,
                (ctx.queue, prog, len(program), ptrs, tys, lds, n_in, mc.ptr + 4 * index,
                 rows, cols), "hcamdLaunchMapSum", (arrays, cell, prog, ptrs, tys, lds))


U8 = 5
IMAP_OPS = {"in": 1, "const": 2, "add": 3, "sub": 4, "mul": 5, "floordiv": 6, "mod": 7, "min": 8,
            "max": 9, "and": 10, "or": 11, "xor": 12, "shl": 13, "shr": 14, "lt": 15, "le": 16,
            "eq": 17, "ne": 18, "ge": 19, "gt": 20, "neg": 21, "abs": 22, "not": 23, "lnot": 24,
            "active": 25, "select": 26}


def plan_imap(program, inputs, out, out_bool=False) -> Plan:
    """out = f(inputs...) over int32 windows (see hcamdLaunchIMap).  `program` is
    a postfix list of (opname, arg, int immediate); `out` is an int32 array, or
    with out_bool a one-byte-per-element array that receives 0 / 1."""
    inputs = list(inputs)
    ctx = _ctx_of(*inputs, out)
    mo = as_memref(out)
    _expect(mo, 1 if out_bool else 4, "imap output")
    rows, cols, ldo = _rows_cols(mo)
    ms = []
    for x in inputs:
        m = as_memref(x)
        _expect(m, 4, "imap operand")
        r, c, _ = _rows_cols(m)
        if (r, c) != (rows, cols):
            raise HcRuntimeError("imap: shape mismatch")
        ms.append(m)
    n_in = len(ms)
    prog = (MapInstr * max(len(program), 1))()
    for i, (name, arg, imm) in enumerate(program):
        prog[i].op, prog[i].arg = IMAP_OPS[name], int(arg)
        # the float field carries the int32 bit pattern
        C.memmove(C.addressof(prog[i]) + MapInstr.imm.offset,
                  C.byref(C.c_int32(((int(imm) + 2 ** 31) % 2 ** 32) - 2 ** 31)), 4)
    ptrs = (_vp * max(n_in, 1))(*[m.ptr for m in ms])
    lds = (_sz * max(n_in, 1))(*[_rows_cols(m)[2] for m in ms])
    return Plan(ctx, hcamdLaunchIMap,
                (ctx.queue, prog, len(program), ptrs, lds, n_in, mo.ptr, U8 if out_bool else I32,
                 ldo, rows, cols), "hcamdLaunchIMap", (inputs, out, prog, ptrs, lds))


FMAP_OPS = {"in": 1, "const": 2, "add": 3, "sub": 4, "mul": 5, "div": 6, "floordiv": 7, "mod": 8,
            "min": 9, "max": 10, "udiv": 11, "lt": 12, "le": 13, "eq": 14, "ne": 15, "ge": 16,
            "gt": 17, "neg": 18, "abs": 19, "sqrt": 20, "rint": 21, "exp": 22, "log": 23, "r16": 24,
            "psqrt": 25, "powchk": 26, "active": 27, "tanh": 28, "select": 29,
            "floor": 30, "ceil": 31, "trunc": 32, "sign": 33, "exp2": 34, "log2": 35, "log10": 36,
            "log1p": 37, "expm1": 38, "sin": 39, "cos": 40, "reciprocal": 41, "merge": 42}
FMAP_MAX_INSTRS = 48


def plan_fmap(program, inputs, out, types, store_all=False) -> Plan:
    """out = f(inputs...) over fp32 / fp16 windows with numpy.ma's activity rules
    (see hcamdLaunchFMap).  `program` is a postfix list of (opname, arg, float
    immediate); `types` lists F32 / F16 / I32 (converted when read) for the inputs
    followed by F32, F16 or U8 (a one-byte-per-element array that receives 0 / 1) for the output;
    store_all writes inactive elements too."""
    inputs = list(inputs)
    ctx = _ctx_of(*inputs, out)
    mo = as_memref(out)
    _expect(mo, {F32: 4, F16: 2, U8: 1}[types[-1]], "fmap output")
    rows, cols, ldo = _rows_cols(mo)
    ms = []
    for x, ty in zip(inputs, types):
        m = as_memref(x)
        _expect(m, {F32: 4, F16: 2, I32: 4}[ty], "fmap operand")
        r, c, _ = _rows_cols(m)
        if (r, c) != (rows, cols):
            raise HcRuntimeError("fmap: shape mismatch")
        ms.append(m)
    n_in = len(ms)
    prog = (MapInstr * max(len(program), 1))()
    for i, (name, arg, imm) in enumerate(program):
        prog[i].op, prog[i].arg, prog[i].imm = FMAP_OPS[name], int(arg), float(imm)
    ptrs = (_vp * max(n_in, 1))(*[m.ptr for m in ms])
    tys = (_int * max(n_in, 1))(*types[:n_in])
    lds = (_sz * max(n_in, 1))(*[_rows_cols(m)[2] for m in ms])
    return Plan(ctx, hcamdLaunchFMap,
                (ctx.queue, prog, len(program), ptrs, tys, lds, n_in, mo.ptr, types[-1], ldo, rows,
                 cols, int(bool(store_all))), "hcamdLaunchFMap", (inputs, out, prog, ptrs, tys, lds))


COLS_KINDS = {"sum": 0, "max": 1, "min": 2}
COLS_MAX_POST = 8


def plan_map_reduce_cols(kind, program, inputs, out, post=(), types=None) -> Plan:
    """out[c] = post(fold over the rows of f(inputs...)) (see
    hcamdLaunchMapReduceCols).  `kind` is "sum", "max" or "min"; `program` and
    `post` are map programs ((opname, arg, imm) triples; `post` reads the folded
    value as operand 0).  `inputs` are rows x cols arrays, or 1-D arrays of
    cols elements that every row uses; `out` holds cols contiguous elements.
    The workspace the launch needs is allocated here, once, with the plan."""
    inputs = list(inputs)
    ctx = _ctx_of(*inputs, out)
    mo = as_memref(out)
    cols = 1
    for n in mo.shape:
        cols *= n
    if not mo.is_contiguous():
        raise HcRuntimeError("map_reduce_cols: the result must be contiguous")
    ms, lds, rows = [], [], None
    for x in inputs:
        m = as_memref(x)
        if len(m.shape) == 1:
            if m.shape[0] > 1 and m.strides[0] != 1:
                raise HcRuntimeError("map_reduce_cols: row vectors must be contiguous")
            r, c, ld = None, m.shape[0], 0
        else:
            r, c, ld = _rows_cols(m)
        if c != cols or (r is not None and rows is not None and r != rows):
            raise HcRuntimeError("map_reduce_cols: shape mismatch")
        rows = r if r is not None else rows
        ms.append(m)
        lds.append(ld)
    if rows is None:
        raise HcRuntimeError("map_reduce_cols: at least one rows x cols operand is needed")
    if types is None:
        types = []
        for m in ms + [mo]:
            if m.itemsize not in (2, 4):
                raise HcRuntimeError(f"map_reduce_cols: element size {m.itemsize} "
                                     "(fp32 and fp16 only)")
            types.append(F16 if m.itemsize == 2 else F32)
    n_in = len(inputs)

    def instrs(p):
        arr = (MapInstr * max(len(p), 1))()
        for i, (name, arg, imm) in enumerate(p):
            arr[i].op, arr[i].arg, arr[i].imm = MAP_OPS[name], int(arg), float(imm)
        return arr
    prog, post_prog = instrs(program), instrs(post)
    ptrs = (_vp * max(n_in, 1))(*[m.ptr for m in ms])
    tys = (_int * max(n_in, 1))(*types[:n_in])
    ldv = (_sz * max(n_in, 1))(*lds)
    need = hcamdMapReduceColsWorkspace(rows, cols)
    work = DeviceArray((need // 4,), np.float32, ctx) if need else None
    return Plan(ctx, hcamdLaunchMapReduceCols,
                (ctx.queue, COLS_KINDS[kind], prog, len(program), post_prog, len(post), ptrs, tys,
                 ldv, n_in, mo.ptr, types[-1], rows, cols, work.ptr if work else None, need),
                "hcamdLaunchMapReduceCols", (inputs, out, prog, post_prog, ptrs, tys, ldv, work))


def plan_row_program(stages, inputs, out, columns=(), types=None) -> Plan:
    """Runs a row program (see hcamdLaunchRowProgram) over a rows x cols tile.

    `stages` is a list of (kind, dst, program) with kind one of ROW_KINDS and
    program a list of (opname, arg, imm).  `inputs` are rows x cols arrays, or
    1-D arrays of cols elements that every row uses; `columns` are 1-D arrays
    of rows elements that fill row scalars 0, 1, ...; `out` is rows x cols for a
    final "store" stage, or holds one value per row (1-D, or rows x 1) for
    "store_col".  `types` = F32/F16 per input, then per column, then the
    output's (default: by element size)."""
    inputs, columns = list(inputs), list(columns)
    ctx = _ctx_of(*inputs, *columns, out)
    mo = as_memref(out)
    col_out = stages[-1][0] == "store_col"
    if col_out:
        if len(mo.shape) == 2 and mo.shape[1] == 1:
            rows, ldo = mo.shape[0], (mo.strides[0] if mo.shape[0] > 1 else 1)
        elif len(mo.shape) == 1:
            rows, ldo = mo.shape[0], (mo.strides[0] if mo.shape[0] > 1 else 1)
        else:
            raise HcRuntimeError("row_program: a per-row result needs a 1-D or rows x 1 output")
        cols = None
    else:
        rows, cols, ldo = _rows_cols(mo)
        if len(mo.shape) == 1:
            rows, cols, ldo = 1, mo.shape[0], mo.shape[0]
    ms, lds = [], []
    for x in inputs:
        m = as_memref(x)
        if len(m.shape) == 1 and (rows != 1 or col_out):    # one vector for every row
            if m.shape[0] > 1 and m.strides[0] != 1:
                raise HcRuntimeError("row_program: row vectors must be contiguous")
            r, c, ld = None, m.shape[0], 0
        else:
            r, c, ld = _rows_cols(m)
        if cols is None:
            cols = c
        if c != cols or (r is not None and r != rows):
            raise HcRuntimeError("row_program: shape mismatch")
        ms.append(m)
        lds.append(ld)
    if cols is None:
        raise HcRuntimeError("row_program: no operand gives the row length")
    mc = [as_memref(x) for x in columns]
    for m in mc:
        n = 1
        for d in m.shape:
            n *= d
        if n != rows or not m.is_contiguous():
            raise HcRuntimeError("row_program: a column operand needs one contiguous value per row")
    everything = ms + mc + [mo]
    if types is None:
        types = []
        for m in everything:
            if m.itemsize not in (2, 4):
                raise HcRuntimeError(f"row_program: element size {m.itemsize} (fp32 and fp16 only)")
            types.append(F16 if m.itemsize == 2 else F32)
    n_in, n_col = len(ms), len(mc)
    flat = [ins for _, _, program in stages for ins in program]
    prog = (MapInstr * max(len(flat), 1))()
    for i, (name, arg, imm) in enumerate(flat):
        prog[i].op, prog[i].arg, prog[i].imm = MAP_OPS[name], int(arg), float(imm)
    st = (RowStage * max(len(stages), 1))()
    for i, (kind, dst, program) in enumerate(stages):
        st[i].kind, st[i].nInstr, st[i].dst = ROW_KINDS[kind], len(program), int(dst)
    ptrs = (_vp * max(n_in, 1))(*[m.ptr for m in ms])
    tys = (_int * max(n_in, 1))(*types[:n_in])
    ldv = (_sz * max(n_in, 1))(*lds)
    cptrs = (_vp * max(n_col, 1))(*[m.ptr for m in mc])
    ctys = (_int * max(n_col, 1))(*types[n_in:n_in + n_col])
    return Plan(ctx, hcamdLaunchRowProgram,
                (ctx.queue, prog, st, len(stages), ptrs, tys, ldv, n_in, cptrs, ctys, n_col,
                 mo.ptr, types[-1], ldo, rows, cols), "hcamdLaunchRowProgram",
                (inputs, columns, out, prog, st, ptrs, tys, ldv, cptrs, ctys))


def plan_pairwise_dist_f32(a, b, out) -> Plan:
    """out[i, j] = ||a[i, :] - b[j, :]||_2 for fp32 a[m, d], b[n, d], out[m, n]."""
    ctx = _ctx_of(a, b, out)
    ma, mb, mo = as_memref(a, 2), as_memref(b, 2), as_memref(out, 2)
    for m, n in ((ma, "a"), (mb, "b"), (mo, "out")):
        _expect(m, 4, n)
    (m, d, lda), (n, d2, ldb), (mo_r, mo_c, ldo) = _rows_cols(ma), _rows_cols(mb), _rows_cols(mo)
    if d != d2 or (mo_r, mo_c) != (m, n):
        raise HcRuntimeError("pairwise_dist_f32: shape mismatch")
    return Plan(ctx, hcamdLaunchPairwiseDistF32,
                (ctx.queue, ma.ptr, lda, mb.ptr, ldb, mo.ptr, ldo, m, n, d),
                "hcamdLaunchPairwiseDistF32", (a, b, out))


class GatherGemm:
    """Device tables of a product of gathered tiles (hcamdGatherGemmCreate).

    Each operand is described by (shape, strides, starts, row_index,
    col_index): shape / strides of the whole buffer in elements, starts an
    int array [n_groups, ndim] with the window start of every group, row_index
    [tile rows, ndim] and col_index [tile cols, ndim] the index each tile
    coordinate contributes inside the window."""

    def __init__(self, ctx, a, b, out, n_groups: int, tm: int, tn: int, k: int):
        import numpy as np
        self.ctx, self.handle = ctx, None
        self.layouts = [(tuple(int(v) for v in o[0]), tuple(int(v) for v in o[1]))
                        for o in (a, b, out)]
        ops, keep = [], []
        for shape, strides, starts, rows, cols in (a, b, out):
            op = GatherOperand()
            op.ndim = len(shape)
            if not 1 <= op.ndim <= 4:
                raise HcRuntimeError("gathered operands have 1 to 4 dimensions")
            for d in range(op.ndim):
                op.shape[d], op.strides[d] = int(shape[d]), int(strides[d])
            tabs = []
            for t in (starts, rows, cols):
                t = np.ascontiguousarray(t, dtype=np.int64).reshape(-1, op.ndim)
                if t.size and (t.max() > 0x7fffffff or t.min() < -0x80000000):
                    raise HcRuntimeError("gather index out of the 32-bit range")
                t = t.astype(np.int32)
                keep.append(t)
                tabs.append(t.ctypes.data_as(C.POINTER(C.c_int32)))
            op.starts, op.rowIndex, op.colIndex = tabs
            ops.append(op)
        h = hcamdGatherGemmCreate(ctx.queue, C.byref(ops[0]), C.byref(ops[1]), C.byref(ops[2]),
                                  n_groups, tm, tn, k)
        if not h:
            ctx.check(1, "hcamdGatherGemmCreate")
        self.handle = h

    def __del__(self):
        handle, self.handle = getattr(self, "handle", None), None
        if handle:
            try:
                hcamdGatherGemmRelease(handle)
            except Exception:       # interpreter shutdown: the library may be gone
                pass


class GatherMap:
    """Device tables of an elementwise expression of gathered tiles
    (hcamdGatherMapCreate).  `operands`: the inputs, then the output, each
    (shape, strides, starts [n_groups, ndim], index [tile elements, ndim]);
    shape / strides of the whole buffer in elements."""

    def __init__(self, ctx, operands, n_groups: int, tile_elems: int):
        self.ctx, self.handle = ctx, None
        self.layouts = [(tuple(int(v) for v in o[0]), tuple(int(v) for v in o[1])) for o in operands]
        ops, keep = (GatherMapOperand * len(operands))(), []
        for op, (shape, strides, starts, index) in zip(ops, operands):
            op.ndim = len(shape)
            if not 1 <= op.ndim <= 4:
                raise HcRuntimeError("gathered operands have 1 to 4 dimensions")
            for d in range(op.ndim):
                op.shape[d], op.strides[d] = int(shape[d]), int(strides[d])
            tabs = []
            for t in (starts, index):
                t = np.ascontiguousarray(t, dtype=np.int64).reshape(-1, op.ndim)
                if t.size and (t.max() > 0x7fffffff or t.min() < -0x80000000):
                    raise HcRuntimeError("gather index out of the 32-bit range")
                t = t.astype(np.int32)
                keep.append(t)
                tabs.append(t.ctypes.data_as(C.POINTER(C.c_int32)))
            op.starts, op.index = tabs
        h = hcamdGatherMapCreate(ctx.queue, ops, len(operands) - 1, n_groups, tile_elems)
        if not h:
            ctx.check(1, "hcamdGatherMapCreate")
        self.handle = h

    def __del__(self):
        handle, self.handle = getattr(self, "handle", None), None
        if handle:
            try:
                hcamdGatherMapRelease(handle)
            except Exception:       # interpreter shutdown: the library may be gone
                pass


def plan_gather_map(tables: GatherMap, program, inputs, out, types, out_type, store_all=False,
                    copy_bytes=0) -> Plan:
    """One launch of a GatherMap: `program` is a program of the general float map
    ((opname, arg, imm) triples), or empty with copy_bytes the element size of a
    gathered / scattered copy."""
    inputs = list(inputs)
    ctx = _ctx_of(*inputs, out)
    ms = [as_memref(x) for x in inputs] + [as_memref(out)]
    for m, lay in zip(ms, tables.layouts):
        if (tuple(m.shape), tuple(m.strides)) != lay:
            raise HcRuntimeError(f"gather_map: an operand has shape {m.shape} strides {m.strides}, "
                                 f"the tables were built for {lay[0]} {lay[1]}")
    n_in = len(inputs)
    prog = (MapInstr * max(len(program), 1))()
    for i, (name, arg, imm) in enumerate(program):
        prog[i].op, prog[i].arg, prog[i].imm = FMAP_OPS[name], int(arg), float(imm)
    ptrs = (_vp * max(n_in, 1))(*[m.ptr for m in ms[:-1]])
    tys = (_int * max(n_in, 1))(*types[:n_in])
    return Plan(ctx, hcamdGatherMapLaunch,
                (ctx.queue, tables.handle, prog, len(program), ptrs, tys, ms[-1].ptr, int(out_type),
                 int(store_all), int(copy_bytes)), "hcamdGatherMapLaunch",
                (tables, inputs, out, prog, ptrs, tys))


def plan_gather_gemm(tables: GatherGemm, a, b, out, dtype: str = "float32") -> Plan:
    """One launch of a GatherGemm on buffers of the shapes it was built for;
    dtype ('float32', 'float16' or 'bfloat16') is the storage type of all three."""
    ctx = _ctx_of(a, b, out)
    ma, mb, mo = as_memref(a), as_memref(b), as_memref(out)
    code, size = {"float32": (F32, 4), "float16": (F16, 2), "bfloat16": (BF16, 2)}[dtype]
    for m, n, lay in zip((ma, mb, mo), ("a", "b", "out"), tables.layouts):
        _expect(m, size, n)
        if (tuple(m.shape), tuple(m.strides)) != lay:
            raise HcRuntimeError(f"gather_gemm: {n} has shape {m.shape} strides {m.strides}, "
                                 f"the tables were built for {lay[0]} {lay[1]}")
    if code == F32:
        return Plan(ctx, hcamdGatherGemmLaunchF32, (ctx.queue, tables.handle, ma.ptr, mb.ptr, mo.ptr),
                    "hcamdGatherGemmLaunchF32", (tables, a, b, out))
    return Plan(ctx, hcamdGatherGemmLaunch, (ctx.queue, tables.handle, code, ma.ptr, mb.ptr, mo.ptr),
                "hcamdGatherGemmLaunch", (tables, a, b, out))


def plan_gather_gemm_f32(tables: GatherGemm, a, b, out) -> Plan:
    return plan_gather_gemm(tables, a, b, out, "float32")


def plan_softmax_f32(x, y) -> Plan:
    ctx = _ctx_of(x, y)
    mx, my = as_memref(x, 2), as_memref(y, 2)
    _expect(mx, 4, "x")
    _expect(my, 4, "y")
    rx, cx, ldx = _rows_cols(mx)
    ry, cy, ldy = _rows_cols(my)
    if (rx, cx) != (ry, cy):
        raise HcRuntimeError("softmax_f32: shape mismatch")
    return Plan(ctx, hcamdLaunchSoftmaxF32, (ctx.queue, mx.ptr, ldx, my.ptr, ldy, rx, cx),
                "hcamdLaunchSoftmaxF32", (x, y))


def plan_quantize_f16_i8(x, q, scale) -> Plan:
    ctx = _ctx_of(x, q, scale)
    mx, mq, ms = as_memref(x, 2), as_memref(q, 2), as_memref(scale, 1)
    _expect(mx, 2, "x")
    _expect(mq, 1, "q")
    _expect(ms, 4, "scale")
    rx, cx, ldx = _rows_cols(mx)
    rq, cq, ldq = _rows_cols(mq)
    if (rx, cx) != (rq, cq) or ms.shape[0] != rx or not ms.is_contiguous():
        raise HcRuntimeError("quantize_f16_i8: shape mismatch")
    return Plan(ctx, hcamdLaunchQuantizeF16I8,
                (ctx.queue, mx.ptr, ldx, mq.ptr, ldq, ms.ptr, rx, cx),
                "hcamdLaunchQuantizeF16I8", (x, q, scale))


def plan_gemm_bf16(a, bt, c) -> Plan:
    """C[M,N] = A[M,K] @ Bt[N,K].T, bf16 bit patterns in 2-byte arrays."""
    ctx = _ctx_of(a, bt, c)
    ma, mb, mc = as_memref(a, 2), as_memref(bt, 2), as_memref(c, 2)
    for m, n in ((ma, "a"), (mb, "bt"), (mc, "c")):
        _expect(m, 2, n)
    m_, k_, lda = _rows_cols(ma)
    n_, k2, ldb = _rows_cols(mb)
    m2, n2, ldc = _rows_cols(mc)
    if k_ != k2 or m_ != m2 or n_ != n2:
        raise HcRuntimeError("gemm_bf16: shape mismatch")
    return Plan(ctx, hcamdLaunchGemmBF16,
                (ctx.queue, ma.ptr, lda, mb.ptr, ldb, mc.ptr, ldc, m_, n_, k_),
                "hcamdLaunchGemmBF16", (a, bt, c))


def plan_gemm_f16(a, bt, c) -> Plan:
    """C[M,N] = A[M,K] @ Bt[N,K].T with fp16 storage and fp32 accumulation."""
    ctx = _ctx_of(a, bt, c)
    ma, mb, mc = as_memref(a, 2), as_memref(bt, 2), as_memref(c, 2)
    for m, n in ((ma, "a"), (mb, "bt"), (mc, "c")):
        _expect(m, 2, n)
    m_, k_, lda = _rows_cols(ma)
    n_, k2, ldb = _rows_cols(mb)
    m2, n2, ldc = _rows_cols(mc)
    if k_ != k2 or m_ != m2 or n_ != n2:
        raise HcRuntimeError("gemm_f16: shape mismatch")
    return Plan(ctx, hcamdLaunchGemmF16,
                (ctx.queue, ma.ptr, lda, mb.ptr, ldb, mc.ptr, ldc, m_, n_, k_),
                "hcamdLaunchGemmF16", (a, bt, c))


# Call-and-wait forms: a kernel call is synchronous on return by default, as in
# the reference (python/cpp/py-runtime/src/GpuRuntime.cpp:60-69).
def copy2d(src, dst, sync: bool = True) -> None:
    plan_copy2d(src, dst).launch(sync)


def copy2d_tiled(src, dst, block_x: int, block_y: int, unroll: int = 1, sync: bool = True) -> None:
    plan_copy2d_tiled(src, dst, block_x, block_y, unroll).launch(sync)


def add_f32(a, b, c, sync: bool = True) -> None:
    plan_add_f32(a, b, c).launch(sync)


def fma_f16(a, b, c, d, sync: bool = True) -> None:
    plan_fma_f16(a, b, c, d).launch(sync)


def softmax_f32(x, y, sync: bool = True) -> None:
    plan_softmax_f32(x, y).launch(sync)


def quantize_f16_i8(x, q, scale, sync: bool = True) -> None:
    plan_quantize_f16_i8(x, q, scale).launch(sync)


def gemm_bf16(a, bt, c, sync: bool = True) -> None:
    plan_gemm_bf16(a, bt, c).launch(sync)


def probes_built() -> bool:
    """The library holds the measurement builds of the GEMM (built with
    `python -m hc_amd.build --probes`); see hc_amd_bench.h."""
    return bool(hcamdProbesBuilt())


def _variant_error(family: str, variant: int) -> HcRuntimeError:
    if family == "gemm" and (17 <= variant <= 22 or variant in (26, 28, 29, 30, 31, 32, 33, 34)) and not probes_built():
        return HcRuntimeError(f"gemm variant {variant} is a measurement build whose output is not the "
                              "product; this library was built without them (python -m hc_amd.build "
                              "--probes builds them)")
    return HcRuntimeError(f"unknown kernel family {family!r}")


def set_variant(family: str, variant: int) -> None:
    if hcamdSetVariant(family.encode(), int(variant)):
        raise _variant_error(family, int(variant))


def set_thread_variant(family: str, variant: int) -> None:
    """The choice for this thread only (variant < 0 removes it)."""
    if hcamdSetThreadVariant(family.encode(), int(variant)):
        raise _variant_error(family, int(variant))


def last_kernel_name() -> str:
    return (hcamdLastKernelName() or b"").decode()


# ---------------------------------------------------------------------------
# Events
# ---------------------------------------------------------------------------
class Event:
    def __init__(self, ctx: Context | None = None):
        self.ctx = ctx or default_context()
        self.handle = hcamdEventCreate(self.ctx.queue)
        if not self.handle:
            raise HcRuntimeError(self.ctx._drain() or "hcamdEventCreate failed")

    def record(self):
        self.ctx.check(hcamdEventRecord(self.handle), "hcamdEventRecord")

    def synchronize(self):
        self.ctx.check(hcamdEventSynchronize(self.handle), "hcamdEventSynchronize")

    def elapsed_ms(self, stop: "Event") -> float:
        ms = C.c_float()
        self.ctx.check(hcamdEventElapsedMs(self.handle, stop.handle, C.byref(ms)),
                       "hcamdEventElapsedMs")
        return float(ms.value)

    def __del__(self):
        try:
            if self.handle:
                hcamdEventDestroy(self.handle)
                self.handle = None
        except Exception:
            pass


def builtin_modules() -> dict[str, tuple[int, int]]:
    """name -> (address, length) of the embedded gfx950 code objects."""
    out = {}
    for i in range(hcamdBuiltinModuleCount()):
        name, data, n = C.c_char_p(), _vp(), _sz()
        hcamdGetBuiltinModule(i, C.byref(name), C.byref(data), C.byref(n))
        out[name.value.decode()] = (int(data.value), int(n.value))
    return out

"""Matches a traced per-group program against the hand-written gfx950 kernels.

The reference lowers a kernel body through its compiler; this build has a fixed
set of hand-written kernels instead, so a traced body is recognised
structurally:

    copy       store(load a)
    add        store(load a + load b)                                  fp32
    fma        store((f32 a * f32 b + f32 c) -> f16)                   fp16 storage
    softmax    store(exp(x - max_row x) / sum_row exp(x - max_row x))  fp32 rows
    quantize   store(int8 clip(rint(f32 x / s), -127, 127)), s = max_row|x| / 127
    gemm       store(sum_k dot(load A[m, k-chunk], load Bt[n, k-chunk].T))   bf16 / fp16
    map        store(f(load a, load b, ...)) for any other elementwise f over up to
               four fp32 / fp16 operands: compiled to a postfix program for the
               fused map kernel
    sum        atomic_ref(r)[i] += f(load a, ...).sum(): the same programs, reduced
               with one fp32 atomic addition per workgroup
    distance   store(norm(a[:, None, :] - b[None, :, :], axis=2))          fp32

Every load and the store must walk their buffers tile by tile: the start along a
dimension is either 0 or group_id[i] * tile_extent, so that the tiles of all
groups are disjoint and their union is a window [0, rows) x [0, cols) of the
buffer.  That window, not the user's tile shape, is what the native kernel
receives: it re-tiles the window for the hardware (16-byte accesses, wave64
reductions, MFMA blocks).  A body that matches nothing raises NoNativeKernel;
there is no interpreter or CPU path behind it.
"""

from __future__ import annotations

import math
from dataclasses import dataclass

from . import runtime as rt
from .kernel_api import (Affine, BufferProxy, BufferView, ItemIndex, Tile, TraceError, same_index,
                         same_starts)


class NoNativeKernel(RuntimeError):
    """The traced kernel body does not correspond to a hand-written kernel."""


# ---------------------------------------------------------------------------
# Windows
# ---------------------------------------------------------------------------
@dataclass
class Window:
    """Union over all groups of one tiled access: [0, extent[d]) per dim."""
    buffer: int          # argument index
    extent: tuple        # elements per dim
    driver: tuple        # group dim that walks each buffer dim, or None
    tile: tuple


def _coeffs(a: Affine, rank: int):
    return tuple(a.coeffs) + (0,) * (rank - len(a.coeffs))


def window_of(view: BufferView, tile_shape, n_groups) -> Window:
    rank = len(n_groups)
    extent, driver = [], []
    used = set()
    for d, (start, t) in enumerate(zip(view.starts, tile_shape)):
        co = _coeffs(start, rank)
        nz = [i for i, c in enumerate(co) if c]
        size = view.base.shape[d]
        if not nz:
            if start.const != 0:
                raise NoNativeKernel(f"{view.base.name}: constant offset {start.const} along "
                                     f"dim {d} (only whole-extent or tiled access is bound)")
            extent.append(min(t, size))
            driver.append(None)
        elif len(nz) == 1 and start.const == 0 and co[nz[0]] == t and nz[0] not in used:
            used.add(nz[0])
            extent.append(min(n_groups[nz[0]] * t, size))
            driver.append(nz[0])
        else:
            raise NoNativeKernel(
                f"{view.base.name}: offset {start!r} along dim {d} with tile extent {t} is "
                "not a disjoint tiling (need group_id * tile_extent)")
    return Window(view.base.index, tuple(extent), tuple(driver), tuple(tile_shape))


# ---------------------------------------------------------------------------
# Tiny structural matcher
# ---------------------------------------------------------------------------
def _is(t: Tile, op: str, n: int | None = None) -> bool:
    return isinstance(t, Tile) and t.op == op and (n is None or len(t.args) == n)


def _const(t: Tile, value=None) -> bool:
    if not (_is(t, "const") or _is(t, "full")):
        return False
    return value is None or t.attrs.get("value") == float(value)


def _strip_cast(t: Tile, to: str) -> Tile:
    return t.args[0] if _is(t, "astype", 1) and t.dtype_name == to else t


def _f32(t: Tile):
    """The load behind `x.astype(float32)` (or x itself if already fp32)."""
    if _is(t, "astype", 1) and t.dtype_name == "float32" and _is(t.args[0], "load"):
        return t.args[0]
    if _is(t, "load") and t.dtype_name == "float32":
        return t
    return None


def _same(a: Tile, b: Tile) -> bool:
    """Structural equality of two expression trees (loads by identity of the
    window they read)."""
    if a is b:
        return True
    if a.op != b.op or a.shape != b.shape or a.dtype_name != b.dtype_name:
        return False
    if a.op == "load":
        va, vb = a.attrs["view"], b.attrs["view"]
        return va.base.index == vb.base.index and same_starts(va.starts, vb.starts)
    if {k: v for k, v in a.attrs.items()} != {k: v for k, v in b.attrs.items()}:
        return False
    return len(a.args) == len(b.args) and all(_same(x, y) for x, y in zip(a.args, b.args))


def _row_reduce(t: Tile, op: str):
    """x if t == x.<op>(axis=1, keepdims=True) on a 2-D tile."""
    if _is(t, op, 1) and t.attrs.get("axes") == (1,) and t.attrs.get("keepdims") \
            and len(t.args[0].shape) == 2:
        return t.args[0]
    return None


# ---------------------------------------------------------------------------
# Patterns.  Each returns a function(memrefs, ctx) -> list[rt.Plan] or None.
# ---------------------------------------------------------------------------
def _check_same_window(wins, value: Tile = None):
    """The window every operand and the output walk.  With `value` (what is
    stored) a tile -- operators of loads, stored where active -- the arrays may
    end at different places: an element is active only where every load was
    inside its array, and stored only where the output has it, so the common
    part of the windows is the whole of the work.  (A bare array is written in
    full, with the 0 a load puts outside its array: the windows must agree.)"""
    w0 = wins[0]
    shrink = value is not None and not value.attrs.get("plain")
    extent = w0.extent
    for w in wins[1:]:
        if w.driver != w0.driver or len(w.extent) != len(extent) or (w.extent != extent and not shrink):
            raise NoNativeKernel("loads and the store walk different windows")
        extent = tuple(min(a, b) for a, b in zip(extent, w.extent))
    return Window(w0.buffer, extent, w0.driver, w0.tile) if extent != w0.extent else w0


def _region2d(extent):
    if len(extent) == 1:
        return 1, extent[0]
    if len(extent) == 2:
        return extent
    raise NoNativeKernel("only 1-D and 2-D buffers have native kernels")


def _sub(m: rt.Memref, extent) -> rt.Memref:
    return rt.Memref(m.ptr, tuple(extent), m.strides, m.itemsize)


class _Arr:
    """Memref wrapper accepted by the runtime's plan_* functions."""

    def __init__(self, m: rt.Memref, ctx):
        self.shape, self.ctx = m.shape, ctx
        code = {1: "|u1", 2: "<u2", 4: "<u4", 8: "<u8", 16: "|V16"}[m.itemsize]
        self.__cuda_array_interface__ = {
            "shape": m.shape, "typestr": code, "data": (m.ptr, False),
            "strides": tuple(s * m.itemsize for s in m.strides), "version": 2}


def match_copy(dst_view, value, n_groups):
    if not _is(value, "load"):
        return None
    src = value.attrs["view"]
    if src.base.dtype_name != dst_view.base.dtype_name:
        return None
    ws = window_of(src, value.shape, n_groups)
    wd = window_of(dst_view, value.shape, n_groups)
    if ws.driver != wd.driver:
        raise NoNativeKernel("load and store walk different windows")
    extent = tuple(min(a, b) for a, b in zip(ws.extent, wd.extent))
    if len(extent) > 2:
        raise NoNativeKernel("only 1-D and 2-D copies have a native kernel")

    def make(mem, ctx):
        return [rt.plan_copy2d(_Arr(_sub(mem[ws.buffer], extent), ctx),
                               _Arr(_sub(mem[wd.buffer], extent), ctx))]
    return make


def match_transpose(dst_view, value, n_groups):
    """store(out[j:, i:], load(x[i:, j:], shape).T): a tile's `.T` written to the
    transposed window.  The tiles of all groups add up to one transposed copy
    of the window, whatever the group shape.  `.T` of a tile is a bare numpy.ma
    array in the reference (python/hckernel/kernel_api.py:150-151) and is stored
    in full, so the window must not reach past what was loaded."""
    if not (_is(value, "transpose", 1) and _is(value.args[0], "load") and len(value.shape) == 2):
        return None
    load = value.args[0]
    src = load.attrs["view"]
    if src.base.dtype_name != dst_view.base.dtype_name or \
            getattr(src.base.dtype, "itemsize", 2) not in (1, 2, 4, 8):
        return None
    ws = window_of(src, load.shape, n_groups)
    wd = window_of(dst_view, value.shape, n_groups)
    if wd.driver != ws.driver[::-1]:
        raise NoNativeKernel("the transposed tile is stored to a window that is not the loaded one transposed")
    if wd.extent[0] > ws.extent[1] or wd.extent[1] > ws.extent[0]:
        raise NoNativeKernel(
            f"{dst_view.base.name}: the transposed tile is a bare array, written in full, and its window reaches "
            f"past what was loaded from {src.base.name}; the reference writes its fill value there")
    rows, cols = wd.extent[1], wd.extent[0]          # of the source window

    def make(mem, ctx):
        return [rt.plan_transpose2d(_Arr(_sub(mem[ws.buffer], (rows, cols)), ctx),
                                    _Arr(_sub(mem[wd.buffer], (cols, rows)), ctx))]
    return make


def match_add(dst_view, value, n_groups):
    value = _strip_cast(value, dst_view.base.dtype_name)
    if not (_is(value, "add", 2) and all(_is(a, "load") for a in value.args)):
        return None
    if {a.dtype_name for a in value.args} | {dst_view.base.dtype_name} != {"float32"}:
        return None
    wins = [window_of(a.attrs["view"], a.shape, n_groups) for a in value.args]
    wins.append(window_of(dst_view, value.shape, n_groups))
    w = _check_same_window(wins, value)

    general = match_map(dst_view, value, n_groups)

    def make(mem, ctx):
        ms = [mem[x.buffer] for x in wins]
        if all(m.shape == w.extent and m.is_contiguous() for m in ms):
            return [rt.plan_add_f32(*[_Arr(m, ctx) for m in ms])]
        return general(mem, ctx)        # windows of larger or strided arrays
    return make


def match_fma(dst_view, value, n_groups):
    if dst_view.base.dtype_name != "float16":
        return None
    value = _strip_cast(value, "float16")
    if not (_is(value, "add", 2) and value.dtype_name == "float32"):
        return None
    for prod, addend in (value.args, value.args[::-1]):
        c = _f32(addend)
        if c is None or not _is(prod, "mul", 2):
            continue
        a, b = _f32(prod.args[0]), _f32(prod.args[1])
        if a is None or b is None:
            continue
        if {a.dtype_name, b.dtype_name, c.dtype_name} != {"float16"}:
            return None
        wins = [window_of(t.attrs["view"], t.shape, n_groups) for t in (a, b, c)]
        wins.append(window_of(dst_view, value.shape, n_groups))
        w = _check_same_window(wins)
        if len(w.extent) > 2:
            raise NoNativeKernel("only 1-D and 2-D buffers have native kernels")

        def make(mem, ctx):
            return [rt.plan_fma_f16(*[_Arr(_sub(mem[x.buffer], w.extent), ctx) for x in wins])]
        return make
    return None


def match_softmax(dst_view, value, n_groups):
    if dst_view.base.dtype_name != "float32" or not _is(value, "div", 2):
        return None
    e, s = value.args
    if _row_reduce(s, "sum") is None or not _same(_row_reduce(s, "sum"), e):
        return None
    if not (_is(e, "exp", 1) and _is(e.args[0], "sub", 2)):
        return None
    x, m = e.args[0].args
    if not (_is(x, "load") and x.dtype_name == "float32" and _row_reduce(m, "max") is x):
        return None
    wx = window_of(x.attrs["view"], x.shape, n_groups)
    wy = window_of(dst_view, value.shape, n_groups)
    w = _check_same_window([wx, wy])
    if len(w.extent) != 2 or w.driver[1] is not None or w.extent[1] != x.attrs["view"].base.shape[1]:
        raise NoNativeKernel("row softmax needs tiles that hold whole rows")

    def make(mem, ctx):
        return [rt.plan_softmax_f32(_Arr(_sub(mem[wx.buffer], w.extent), ctx),
                                    _Arr(_sub(mem[wy.buffer], w.extent), ctx))]
    return make


def _quant_parts(value):
    """(x load, scale tile) if value == int8(clip(rint(f32 x / scale), -127, 127))."""
    v = _strip_cast(value, "int8")
    if not (_is(v, "clip", 1) and v.attrs["lo"] == -127.0 and v.attrs["hi"] == 127.0):
        return None
    r = v.args[0]
    if not (_is(r, "rint", 1) and _is(r.args[0], "div", 2)):
        return None
    xf, scale = r.args[0].args
    x = _f32(xf)
    if x is None or x.dtype_name != "float16":
        return None
    if not (_is(scale, "div", 2) and _const(scale.args[1], 127) and scale.dtype_name == "float32"):
        return None
    amax = _row_reduce(scale.args[0], "max")
    if amax is None or not (_is(amax, "abs", 1) and _f32(amax.args[0]) is x):
        return None
    return x, scale


def match_quantize(stores, n_groups):
    """Two stores: the int8 matrix and the per-row scale vector."""
    if len(stores) != 2:
        return None
    for (qv, qval), (sv, sval) in (stores, stores[::-1]):
        if qv.base.dtype_name != "int8" or sv.base.dtype_name != "float32":
            continue
        parts = _quant_parts(qval)
        if parts is None:
            continue
        x, scale = parts
        # the scale may be stored as (rows, 1), or flattened to (rows,)
        s = sval
        while _is(s, "slice", 1) or _is(s, "reshape", 1):
            s = s.args[0]
        if not _same(s, scale):
            continue
        wx = window_of(x.attrs["view"], x.shape, n_groups)
        wq = window_of(qv, qval.shape, n_groups)
        w = _check_same_window([wx, wq])
        if len(w.extent) != 2 or w.driver[1] is not None or \
                w.extent[1] != x.attrs["view"].base.shape[1]:
            raise NoNativeKernel("row quantisation needs tiles that hold whole rows")
        ws = window_of(sv, (x.shape[0],) + (1,) * (sv.base.ndim - 1), n_groups)
        if ws.extent[0] != w.extent[0] or ws.driver[0] != w.driver[0]:
            raise NoNativeKernel("scale vector and matrix walk different rows")

        def make(mem, ctx, wx=wx, wq=wq, ws=ws, w=w):
            sm = mem[ws.buffer]
            scale_arr = rt.Memref(sm.ptr, (w.extent[0],), (sm.strides[0],), sm.itemsize)
            return [rt.plan_quantize_f16_i8(_Arr(_sub(mem[wx.buffer], w.extent), ctx),
                                            _Arr(_sub(mem[wq.buffer], w.extent), ctx),
                                            _Arr(scale_arr, ctx))]
        return make
    return None


def _flatten_sum(t: Tile, out: list):
    if _is(t, "add", 2):
        _flatten_sum(t.args[0], out)
        _flatten_sum(t.args[1], out)
    else:
        out.append(t)


def match_gemm(dst_view, value, n_groups):
    elem = dst_view.base.dtype_name
    if elem not in ("bfloat16", "float16"):
        return None
    value = _strip_cast(value, elem)
    terms: list = []
    _flatten_sum(value, terms)
    dots = [t for t in terms if not _const(t, 0)]
    if not dots or not all(_is(d, "dot", 2) or
                           (_is(d, "astype", 1) and _is(d.args[0], "dot", 2)) for d in dots):
        return None
    chunks, wa0, wb0, a_idx, b_idx = [], None, None, None, None
    for d in dots:
        d = d.args[0] if d.op == "astype" else d
        la, lbt = d.args
        # operands may be widened to fp32 first (`load(...).astype(float32)`): the
        # MFMA multiplies the stored values exactly and accumulates in fp32 anyway
        if _leaf(la) is not None:
            la = _leaf(la)
        if _is(lbt, "transpose", 1) and _leaf(lbt.args[0]) is not None:
            lbt = Tile("transpose", (_leaf(lbt.args[0]),), lbt.shape, lbt.dtype_name)
        elif _is(lbt, "astype", 1) and lbt.dtype_name == "float32" and \
                _is(lbt.args[0], "transpose", 1):
            lbt = lbt.args[0]
        if not (_is(la, "load") and _is(lbt, "transpose", 1) and _is(lbt.args[0], "load")):
            raise NoNativeKernel("GEMM is bound for dot(load A[m, k], load Bt[n, k].T): B must "
                                 "be column-major, passed as Bt[N, K]")
        lb = lbt.args[0]
        if la.dtype_name != elem or lb.dtype_name != elem:
            return None
        va, vb = la.attrs["view"], lb.attrs["view"]
        ka, kb = va.starts[1], vb.starts[1]
        if not (ka.is_const and kb.is_const and ka.const == kb.const and
                la.shape[1] == lb.shape[1]):
            raise NoNativeKernel("A and Bt tiles of one dot must cover the same K range")
        chunks.append((ka.const, la.shape[1]))
        # windows along M and N: evaluate with the K offset removed
        va0 = BufferView(va.base, (va.starts[0], Affine(0, ka.coeffs)))
        vb0 = BufferView(vb.base, (vb.starts[0], Affine(0, kb.coeffs)))
        wa = window_of(va0, (la.shape[0], va.base.shape[1]), n_groups)
        wb = window_of(vb0, (lb.shape[0], vb.base.shape[1]), n_groups)
        if wa0 is None:
            wa0, wb0, a_idx, b_idx = wa, wb, va.base.index, vb.base.index
        elif (wa.extent, wa.driver, wb.extent, wb.driver, va.base.index, vb.base.index) != \
                (wa0.extent, wa0.driver, wb0.extent, wb0.driver, a_idx, b_idx):
            raise NoNativeKernel("dot terms walk different A / Bt windows")
    k_total = wa0.extent[1]
    if wb0.extent[1] != k_total:
        raise NoNativeKernel("A and Bt have different K extents")
    chunks.sort()
    pos = 0
    for start, length in chunks:
        if start != pos:
            raise NoNativeKernel("K chunks of the dot terms are not contiguous")
        pos += length
    if pos < k_total:
        raise NoNativeKernel("the dot terms do not cover all of K")
    wc = window_of(dst_view, value.shape, n_groups)
    if wc.driver != (wa0.driver[0], wb0.driver[0]) or wc.driver[0] == wc.driver[1]:
        raise NoNativeKernel("C tiles must be walked by the A-row and Bt-row group dims")
    m, n = min(wc.extent[0], wa0.extent[0]), min(wc.extent[1], wb0.extent[0])

    plan = rt.plan_gemm_bf16 if elem == "bfloat16" else rt.plan_gemm_f16

    def make(mem, ctx):
        return [plan(_Arr(_sub(mem[a_idx], (m, k_total)), ctx),
                     _Arr(_sub(mem[b_idx], (n, k_total)), ctx),
                     _Arr(_sub(mem[wc.buffer], (m, n)), ctx))]
    return make


# ---------------------------------------------------------------------------
# Products of gathered tiles (mapped loads / stores)
# ---------------------------------------------------------------------------
class _Operand:
    """One side of the product: the tile all dot terms read their chunks from.
    `view` is the window it is loaded from, `func` maps (row, col) of the tile
    to an index tuple inside the window (None: the identity of a plain 2-D
    load), `shape` is the tile shape."""

    def __init__(self, view, func, shape):
        self.view, self.func, self.shape = view, func, tuple(shape)

    def same_as(self, o):
        return (self.view.base.index == o.view.base.index and self.func is o.func
                and all(_same_index(a, b) for a, b in zip(self.view.starts, o.view.starts)))


def _same_index(a, b):
    return same_index(a, b)


def _region(t: Tile, axis_k: int):
    """Follows slice / window nodes down to a load.  Returns (operand, origin,
    limit): element e of `t` along each axis is element origin[axis] + e of the
    operand tile, and holds data only while origin + e < limit[axis] (beyond that
    it is an inactive zero).  A plain load whose K start is a constant is turned
    into a chunk of the load with K start 0."""
    if _is(t, "mapped_load"):
        if len(t.shape) != 2:
            raise NoNativeKernel("mapped loads are bound for 2-D tiles")
        return _Operand(t.attrs["view"], t.attrs["mapping"], t.shape), [0, 0], list(t.shape)
    if _is(t, "load"):
        view = t.attrs["view"]
        if view.base.ndim != 2 or len(t.shape) != 2:
            raise NoNativeKernel("the operands of a dot are 2-D tiles")
        k0 = view.starts[axis_k]
        if not k0.is_const or k0.const < 0:
            raise NoNativeKernel("the K offset of a dot operand must not depend on the group")
        starts = list(view.starts)
        starts[axis_k] = Affine(0, k0.coeffs)
        shape = list(t.shape)
        shape[axis_k] = None                       # filled in from the chunks
        op = _Operand(BufferView(view.base, tuple(starts)), None, shape)
        origin, limit = [0, 0], list(t.shape)
        origin[axis_k] = k0.const
        limit[axis_k] = k0.const + t.shape[axis_k]
        return op, origin, limit
    if _is(t, "astype", 1) and t.dtype_name == t.args[0].dtype_name:
        return _region(t.args[0], axis_k)
    if _is(t, "window", 1):
        op, origin, limit = _region(t.args[0], axis_k)
        limit = [min(l, o + n) for l, o, n in zip(limit, origin, t.shape)]
        return op, origin, limit
    if _is(t, "slice", 1):
        src = t.args[0]
        op, origin, limit = _region(src, axis_k)
        key = t.attrs["key"]
        if len(key) != 2 or any(not isinstance(k, tuple) for k in key):
            raise NoNativeKernel("dot operands are sliced as tile[r0:r1, c0:c1]")
        for ax, k in enumerate(key):
            start, stop, step = slice(*k).indices(src.shape[ax])
            if step != 1:
                raise NoNativeKernel("strided slices of tiles have no native kernel")
            limit[ax] = min(limit[ax], origin[ax] + max(stop, start))
            origin[ax] += start
        return op, origin, limit
    raise NoNativeKernel(f"operand of a dot is {t!r}: bound for (slices of) loads")


def _mapping_tables(func, rows, cols, ndim, name):
    """Evaluates an index mapping on the whole tile.  Returns (row_index
    [rows, ndim], col_index [cols, ndim]); every dimension must depend on one
    tile coordinate only."""
    import numpy as np
    if func is None:
        if ndim != 2:
            raise NoNativeKernel(f"{name}: plain tiles of a product are 2-D")
        r = np.zeros((rows, 2), np.int64)
        c = np.zeros((cols, 2), np.int64)
        r[:, 0] = np.arange(rows)
        c[:, 1] = np.arange(cols)
        return r, c
    i = np.arange(rows, dtype=np.int64).reshape(rows, 1)
    j = np.arange(cols, dtype=np.int64).reshape(1, cols)
    try:
        mapped = func(i, j)
    except TraceError:
        raise
    except Exception as exc:
        raise NoNativeKernel(f"{name}: the mapping cannot be evaluated on index arrays "
                             f"({type(exc).__name__}: {exc})") from exc
    if not isinstance(mapped, tuple) or len(mapped) != ndim:
        raise NoNativeKernel(f"{name}: the mapping must return {ndim} indices")
    r = np.zeros((rows, ndim), np.int64)
    c = np.zeros((cols, ndim), np.int64)
    for d, m in enumerate(mapped):
        try:
            full = np.broadcast_to(np.asarray(m), (rows, cols))
            if full.dtype == object or full.dtype.kind == "f":
                as_int = np.array([[int(v) for v in row] for row in full], dtype=np.int64)
                if not all(v == w for v, w in zip(full.ravel(), as_int.ravel())):
                    raise NoNativeKernel(f"{name}: the mapping gives fractional indices")
                full = as_int
            full = full.astype(np.int64)
        except (TypeError, ValueError) as exc:
            raise NoNativeKernel(f"{name}: mapping result of dimension {d} is not an integer "
                                 f"array ({exc})") from exc
        by_col = rows and cols and bool((full != full[:, :1]).any())
        by_row = rows and cols and bool((full != full[:1, :]).any())
        if by_col and by_row:
            raise NoNativeKernel(f"{name}: index {d} of the mapping depends on both tile "
                                 "coordinates (each index must follow the row or the column)")
        if by_col:
            c[:, d] = full[0, :]
        elif rows and cols:
            r[:, d] = full[:, 0]
    return r, c


def _group_starts(view, n_groups):
    """Window start of every group, [n_groups, ndim], groups in row-major order."""
    import numpy as np
    from .kernel_api import evaluate_index
    total = 1
    for n in n_groups:
        total *= n
    ids = [g.reshape(-1) for g in np.indices(n_groups, dtype=np.int64)]
    out = np.zeros((total, view.base.ndim), np.int64)
    for d, s in enumerate(view.starts):
        v = np.broadcast_to(np.asarray(evaluate_index(s, ids)), (total,))
        if v.dtype == object:
            if any(x != int(x) for x in v):
                raise NoNativeKernel(f"{view.base.name}: fractional window start along dim {d}")
            v = np.array([int(x) for x in v], dtype=np.int64)
        if (v < 0).any():
            raise NoNativeKernel(f"{view.base.name}: negative window start along dim {d}")
        out[:, d] = v
    return out


_MERGED_EDGE = 64         # merged tiles grow up to the kernel's largest block


def _merge_groups(tables, grid, tm, tn):
    """Joins neighbouring groups into larger tiles where that changes nothing
    but the tiling: along a group axis on which the b window stays put and the a
    and out windows advance by a fixed step in dimensions their tile rows drive,
    m groups are one group with m times the rows (row tables repeated with the
    step added).  The same with a and b exchanged grows the columns.  A user's
    8 x 8 tiles thus reach the kernel as 64 x 64 ones.  Exactness: a row that was
    active in its own group is active in the merged one and the other way round,
    because window start plus index is unchanged; that needs indices >= 0 (a
    negative index could become a valid element of the neighbouring window), so
    tables with negative entries are left alone.  tables: [(shape, strides,
    starts, rows, cols)] for a, b, out.  Returns (tables, grid, tm, tn)."""
    import numpy as np
    grid = list(grid)
    ops = [list(t) for t in tables]
    # (operands whose tile rows / columns grow, table slot, the operand that must not move)
    plans = (("rows", (0, 2), 3, 1), ("cols", (1, 2), 4, 0))
    for axis in range(len(grid)):
        for kind, moving, slot, fixed in plans:
            extent = tm if kind == "rows" else tn
            if grid[axis] < 2 or extent >= _MERGED_EDGE:
                continue
            m = max((d for d in range(1, grid[axis] + 1)
                     if grid[axis] % d == 0 and d * extent <= _MERGED_EDGE), default=1)
            if m < 2:
                continue
            starts = [np.asarray(o[2]).reshape(*grid, -1) for o in ops]
            if np.diff(starts[fixed], axis=axis).any():
                continue
            deltas, ok = {}, True
            for o in moving:
                d = np.diff(starts[o], axis=axis).reshape(-1, starts[o].shape[-1])
                step = d[0]
                other = ops[o][4] if slot == 3 else ops[o][3]     # the other coordinate's table
                ok = ok and not (d != step).any() and (step >= 0).all() \
                    and not (other[:, step != 0] != 0).any() \
                    and (ops[o][slot] >= 0).all()
                deltas[o] = step
            if not ok:
                continue
            for o in moving:
                table = ops[o][slot]
                ops[o][slot] = np.concatenate([table + j * deltas[o] for j in range(m)], axis=0)
            for o in range(3):
                ops[o][2] = np.take(starts[o], np.arange(0, grid[axis], m), axis=axis) \
                    .reshape(-1, starts[o].shape[-1])
            grid[axis] //= m
            if kind == "rows":
                tm *= m
            else:
                tn *= m
    return [tuple(o) for o in ops], tuple(grid), tm, tn


def match_gather_gemm(dst_view, value, n_groups, out_func=None, plain=True):
    """store(sum_k dot(A chunk, B chunk)) where the chunks are slices of one A
    tile and one B tile, any of them loaded or stored through a mapping."""
    value = _strip_cast(value, dst_view.base.dtype_name)
    terms: list = []
    _flatten_sum(value, terms)
    dots = [t for t in terms if not _const(t, 0)]
    if not dots or not all(_is(d, "dot", 2) for d in dots):
        if plain:
            return None
        raise NoNativeKernel("a mapped store is bound for a sum of dot products")
    if len(value.shape) != 2:
        raise NoNativeKernel("the product tile must be 2-D")
    tm, tn = value.shape
    a_op = b_op = None
    chunks = []
    for d in dots:
        oa, origin_a, limit_a = _region(d.args[0], 1)
        ob, origin_b, limit_b = _region(d.args[1], 0)
        if a_op is None:
            a_op, b_op = oa, ob
        elif not (a_op.same_as(oa) and b_op.same_as(ob)):
            raise NoNativeKernel("the dot terms read different A / B tiles")
        if origin_a[0] != 0 or origin_b[1] != 0 or d.args[0].shape[0] != tm or \
                d.args[1].shape[1] != tn:
            raise NoNativeKernel("dot terms must use all rows of A and all columns of B")
        for op, got, ax in ((a_op, limit_a[0], 0), (b_op, limit_b[1], 1)):
            if op.shape[ax] is not None and got < min(op.shape[ax], (tm, tn)[ax]):
                raise NoNativeKernel("dot terms must use all rows of A and all columns of B")
        if origin_a[1] != origin_b[0]:
            raise NoNativeKernel("A and B chunks of one dot start at different K")
        # beyond the shorter of the two chunks one factor is an inactive zero
        length = min(limit_a[1] - origin_a[1], limit_b[0] - origin_b[0])
        if length > 0:
            chunks.append((origin_a[1], length))
    chunks.sort()
    pos = 0
    for start, length in chunks:
        if start != pos:
            raise NoNativeKernel("K chunks of the dot terms are not contiguous from 0")
        pos += length
    k_total = pos
    for op, ax in ((a_op, 1), (b_op, 0)):
        if op.shape[ax] is None:
            op.shape = tuple(k_total if i == ax else v for i, v in enumerate(op.shape))
        elif op.shape[ax] != k_total:
            raise NoNativeKernel("the dot terms do not cover all of K")
    if a_op.shape[0] < tm or b_op.shape[1] < tn:
        raise NoNativeKernel("the product tile is larger than its operands")
    o_op = _Operand(dst_view, out_func, (tm, tn))
    ops = (a_op, b_op, o_op)
    names = tuple(o.view.base.name for o in ops)
    elem = ops[0].view.base.dtype_name
    if elem not in ("float32", "float16", "bfloat16") or \
            any(o.view.base.dtype_name != elem for o in ops):
        raise NoNativeKernel("products of gathered tiles are bound for three float32, float16 or "
                             f"bfloat16 buffers of one type "
                             f"({', '.join(o.view.base.dtype_name for o in ops)} given)")
    dims = ((tm, k_total), (k_total, tn), (tm, tn))
    tables = []
    for o, (rows, cols), name in zip(ops, dims, names):
        r, c = _mapping_tables(o.func, rows, cols, o.view.base.ndim, name)
        tables.append((tuple(o.view.base.shape), tuple(o.view.base.strides),
                       _group_starts(o.view, n_groups), r, c))
    # two active elements of the out tile must not land on the same address
    import numpy as np
    so = np.asarray(o_op.view.base.strides, np.int64)
    size = np.asarray(o_op.view.base.shape, np.int64)
    ro, co = tables[2][3], tables[2][4]
    ro = ro[((ro >= 0) & (ro < size)).all(axis=1)]          # rows / columns that can be active
    co = co[((co >= 0) & (co < size)).all(axis=1)]
    dest = (ro @ so)[:, None] + (co @ so)[None, :]
    if len(np.unique(dest)) != dest.size:
        raise NoNativeKernel(f"{names[2]}: the store mapping sends two tile elements to one "
                             "destination")
    tables, n_groups, tm, tn = _merge_groups(tables, n_groups, tm, tn)
    total = 1
    for n in n_groups:
        total *= n
    idx = tuple(o.view.base.index for o in ops)
    cache = {}

    def make(mem, ctx):
        g = cache.get(id(ctx))
        if g is None:
            g = cache[id(ctx)] = rt.GatherGemm(ctx, *tables, total, tm, tn, k_total)
        return [rt.plan_gather_gemm(g, *[_Arr(mem[i], ctx) for i in idx], elem)]
    return make


# ---------------------------------------------------------------------------
# Generic elementwise expressions -> postfix program for the fused map kernel
# ---------------------------------------------------------------------------
_MAP_BINARY = {"add": ("add", "add", True), "mul": ("mul", "mul", True),
               "maximum": ("max", "max", True), "minimum": ("min", "min", True),
               "sub": ("sub", "rsub", False), "div": ("div", "rdiv", False)}
_MAP_UNARY = {"neg": "neg", "abs": "abs", "sqrt": "sqrt", "rint": "rint", "exp": "exp",
              "log": "log", "tanh": "tanh", "masqrt": "masqrt"}
_MAP_EXACT = {"neg", "abs", "maximum", "minimum", "clip"}   # fp16 in -> fp16 out, no rounding
_MAP_FLOATS = ("float16", "float32")


_REDUCTIONS = ("sum", "max", "min", "count", "norm")


def _is_reduction(t: Tile) -> bool:
    return t.op in _REDUCTIONS and "axes" in t.attrs and len(t.args) == 1


def _masks(t: Tile) -> bool:
    """t itself can deactivate elements at run time.  The tile operators / // %
    and ** go through numpy.ma, which deactivates failed divisions and results
    of ** that are not finite; NumPy functions with a domain (sqrt, log, divide)
    called on tiles deactivate where the domain fails.  The division of a mean
    is numpy.ma's too; a variance is inactive where fewer than ddof + 1 elements
    were active; numpy.ma.sqrt (the standard deviation's) deactivates results
    that are not finite."""
    if t.attrs.get("ieee"):
        return False                         # plain NumPy arrays: NumPy's own arithmetic
    if t.op == "masqrt":
        return True
    if t.op == "vardiv":
        return not _const(t.args[1])
    if t.attrs.get("func"):
        return t.op in ("sqrt", "log", "log2", "log10", "div", "floordiv", "mod")
    return t.op in ("div", "floordiv", "mod") or bool(t.attrs.get("pow"))


def _maybe_masked(t: Tile, memo=None) -> bool:
    """Some element of t may be inactive for a reason only the data knows.  (A
    fold over elements of which every one may be inactive may be inactive itself;
    their number never is.)"""
    memo = {} if memo is None else memo
    if t.uid not in memo:
        if _is(t, "load") or _const(t) or t.op in ("count", "where", "active", "activated"):
            memo[t.uid] = False                  # (numpy.where and tile.mask return plain arrays)
        elif _is(t, "merge", 2):
            memo[t.uid] = _maybe_masked(t.args[0], memo)     # active wherever the tile was
        else:
            memo[t.uid] = _masks(t) or any(_maybe_masked(a, memo) for a in t.args if isinstance(a, Tile))
    return memo[t.uid]


def _fails_on_finite_data(t: Tile) -> bool:
    """t can deactivate elements whose operands are ordinary finite numbers: a
    zero divisor, an argument outside a function's domain, a variance over too
    few active elements.  (A division by a non-zero constant or by a count, a
    square and numpy.ma.sqrt of a variance only fail on values that are not
    finite already, or by overflow.)"""
    if not _masks(t):
        return False
    if t.op == "masqrt" or (t.attrs.get("pow") and t.op != "sqrt"):
        return False                         # (x ** 0.5 fails on every negative x)
    if t.op == "div" and not t.attrs.get("func"):
        d = t.args[1]
        if t.attrs.get("ma") or (_const(d) and d.attrs.get("value") != 0.0):
            return False
    return True


# Operations that compute from their operands' values and change nothing about
# which elements are active: NumPy functions without a domain, negation, abs,
# conversions.  (The tile operators + - * are not: numpy.ma gives the first
# operand's value where an operand is inactive.)
_TRANSPARENT_FUNCS = ("exp", "rint", "tanh", "maximum", "minimum", "add", "sub", "mul", "clip", "neg", "abs")


def _values_flow_plainly(t: Tile, clean: bool = True, finite: bool = False) -> bool:
    """Every operation that can deactivate elements has only transparent
    operations above it: then the value stored for a deactivated element is
    what plain arithmetic on the value numpy.ma left there gives.  `finite`:
    only operations that can fail on finite data count."""
    if _is(t, "load") or _const(t):
        return True
    if _is_reduction(t):
        # a fold's value does not depend on what its deactivated elements hold;
        # the fold itself is inactive where all of them are
        return clean or not _can_fail(t, finite)
    if (_fails_on_finite_data(t) if finite else _masks(t)) and not clean:
        return False
    transparent = _is(t, "astype", 1) or t.op in ("neg", "abs") or bool(t.attrs.get("ieee")) or \
        (bool(t.attrs.get("func")) and t.op in _TRANSPARENT_FUNCS)
    return all(_values_flow_plainly(a, clean and transparent, finite) for a in t.args if isinstance(a, Tile))


def _can_fail(t: Tile, finite: bool, memo=None) -> bool:
    """_maybe_masked, or (finite) the same restricted to failures on finite data."""
    if not finite:
        return _maybe_masked(t)
    memo = {} if memo is None else memo
    if t.uid not in memo:
        if _is(t, "load") or _const(t) or t.op in ("count", "where", "active", "activated"):
            memo[t.uid] = False                  # (numpy.where returns a plain array)
        elif _is(t, "merge", 2):
            memo[t.uid] = _can_fail(t.args[0], True, memo)
        else:
            memo[t.uid] = _fails_on_finite_data(t) or \
                any(_can_fail(a, True, memo) for a in t.args if isinstance(a, Tile))
    return memo[t.uid]


class _NeedsEntryMasks(Exception):
    """The expression needs activity tracked per operand and numpy.ma's values
    under deactivated elements: the general float map has both, the fast map
    kernel one flag per element."""


def _round_to(value: float, dtype: str) -> float:
    import numpy as np
    return float(np.float16(value)) if dtype == "float16" else float(np.float32(value))


def _leaf(t: Tile):
    """The load behind t if pushing t is just reading an operand: a load, or a
    load widened to fp32 (no rounding involved)."""
    if _is(t, "load"):
        return t
    if _is(t, "astype", 1) and t.dtype_name == "float32" and _is(t.args[0], "load"):
        return t.args[0]
    return None


# Flags in `arg` of the instructions of a stage that computes with row scalars
# (bit 8 is the fp16 flag of the numpy.ma quotients).  What a deactivated row
# scalar holds is part of the result when it is stored, and numpy.ma leaves the
# first operand's value there for the tile operators + - * / while NumPy
# functions compute on the values regardless.
_FUNC_FORM = 0x200            # the operation was called as a NumPy function
_SWAPPED = 0x400              # a commutative operation whose running value is the second operand
_KEEP_DEAD = 0x800            # a unary operation that leaves a deactivated value as it is (x ** 0.5)


class _MapCompiler:
    """Sethi-Ullman ordering: the operand that needs the deeper stack is
    evaluated first, constants become immediates, so an expression with up to
    eight distinct leaves in a balanced tree fits the four-entry stack."""

    masked = False                # emit numpy.ma's division rule (element-wise map and its sum only)
    _scalar_mode = False          # the program computes with row scalars (row programs only)
    _frozen = False               # the stage keeps what numpy.ma leaves in deactivated elements

    def _form(self, t: Tile, swapped: bool = False) -> int:
        if not (self._scalar_mode or self._frozen):
            return 0
        return (_FUNC_FORM if t.attrs.get("func") else 0) | (_SWAPPED if swapped else 0)

    def __init__(self, n_groups):
        self.n_groups = n_groups
        self.inputs = []          # (buffer index, starts, Tile)
        self.need_cache = {}

    def operand(self, t: Tile) -> int:
        v = t.attrs["view"]
        for i, (b, st, _) in enumerate(self.inputs):
            if b == v.base.index and same_starts(st, v.starts):
                return i
        self.inputs.append((v.base.index, v.starts, t))
        return len(self.inputs) - 1

    def supported(self, t: Tile) -> bool:
        if _const(t):
            return True
        if t.dtype_name not in _MAP_FLOATS:
            return False
        if _is(t, "load"):
            return True
        if _is(t, "astype", 1) or t.op in _MAP_UNARY or _is(t, "clip", 1):
            return len(t.args) == 1 and self.supported(t.args[0])
        if t.op in _MAP_BINARY and len(t.args) == 2:
            if all(_const(a) for a in t.args):
                return False
            if t.op in ("maximum", "minimum") and t.dtype_name == "float16":
                # NumPy's fp16 maximum / minimum return the first of two equal values
                # (+0 and -0), the fp32 ones, which this kernel has, the second:
                # the general float map has both
                return False
            if not all(self.supported(a) and (_const(a) or a.shape == t.shape) for a in t.args):
                return False
            # of two equal values (+0 and -0) NumPy's maximum / minimum return the second:
            # the operands must reach the kernel in the order they were written
            return t.op not in ("maximum", "minimum") or self._keeps_order(t)
        if _is(t, "vardiv", 2):                  # a variance whose count is a number
            return _const(t.args[1]) and self.supported(t.args[0])
        return False

    def _keeps_order(self, t: Tile) -> bool:
        """emit() hands t's operands to the kernel in the order they were written
        (it evaluates the deeper side first and has operand and immediate forms
        that take the running value as the first operand)."""
        a, b = t.args
        if self._scalar_mode or self._frozen:
            return True                               # (those stages say which operand came first)
        if _const(b):
            return True
        if _const(a):
            return a.attrs.get("value") != 0          # only zeros of two signs are equal and differ
        if _leaf(b) is not None:
            return True
        if _leaf(a) is not None:
            return False
        return self.need(a) >= self.need(b)

    def need(self, t: Tile) -> int:
        if t.uid in self.need_cache:
            return self.need_cache[t.uid]
        if _is(t, "load") or _const(t):
            n = 1
        elif len(t.args) == 1 or _is(t, "vardiv", 2):
            n = self.need(t.args[0])
        else:
            a, b = t.args
            if _const(a) or _const(b):
                n = self.need(b if _const(a) else a)
            elif _leaf(b) is not None or _leaf(a) is not None:
                n = self.need(a if _leaf(b) is not None else b)
            else:
                na, nb = self.need(a), self.need(b)
                n = max(na, nb) if na != nb else na + 1
        self.need_cache[t.uid] = n
        return n

    def emit(self, t: Tile, out: list):
        self._emit_node(t, out)
        if self.masked and t.attrs.get("pow"):
            out.append(("powchk", 0, 0.0))
            if t.dtype_name == "float16":
                out.append(("r16", 0, 0.0))        # numpy.ma's fill value 1e20 is infinite as fp16

    def emit_whole(self, t: Tile, out: list):
        """The program of a whole expression where no other kernel can take
        over: numpy.ma's forms where this kernel has them, plain arithmetic for
        what it lacks (numpy.divide called as a function)."""
        try:
            self.emit(t, out)
        except _NeedsEntryMasks:
            raise NoNativeKernel("numpy.divide called as a function next to a reduction has no "
                                 "native code (the / operator has)") from None

    def _emit_node(self, t: Tile, out: list):
        half = t.dtype_name == "float16"
        if _is(t, "load"):
            out.append(("in", self.operand(t), 0.0))
            return
        if _const(t):
            out.append(("const", 0, t.attrs["value"]))
            return
        if _is(t, "astype", 1):
            self.emit(t.args[0], out)
            if half and t.args[0].dtype_name != "float16":
                out.append(("r16", 0, 0.0))
            return
        if _is(t, "clip", 1):
            self.emit(t.args[0], out)
            out.append(("maxi", 0, _round_to(t.attrs["lo"], t.dtype_name)))
            out.append(("mini", 0, _round_to(t.attrs["hi"], t.dtype_name)))
            return
        if _is(t, "vardiv", 2):
            # the sum of the centred squares over a count that is a number: the
            # variance is active whatever the quotient is
            self.emit(t.args[0], out)
            out.append(("divi", 0, _round_to(t.args[1].attrs["value"], t.dtype_name)))
            return
        mdiv = self.masked and t.op == "div" and not t.attrs.get("ieee")
        if mdiv and t.attrs.get("func"):
            raise _NeedsEntryMasks()           # numpy.divide as a function: the general map has it
        if t.op in _MAP_UNARY:
            self.emit(t.args[0], out)
            name = _MAP_UNARY[t.op]
            if self.masked and t.attrs.get("func") and name in ("sqrt", "log") and not t.attrs.get("ieee"):
                name = "m" + name              # numpy.sqrt / numpy.log of a tile: domain fill
            if name == "masqrt" and not self.masked:
                name = "sqrt"                  # stored in full: the same values
            keep = _KEEP_DEAD if (self._scalar_mode or self._frozen) and t.op == "sqrt" and \
                t.attrs.get("pow") else 0      # x ** 0.5: numpy.ma.power keeps an inactive operand's value
            out.append((name, keep, 0.0))
            if self.masked and t.op == "sqrt" and t.attrs.get("pow"):
                out.append(("addi", 0, 0.0))   # x ** 0.5 of -0 is +0 (the square root's is -0)
        else:
            fwd, rev, _ = _MAP_BINARY[t.op]
            if mdiv:
                fwd, rev = "mdiv", "rmdiv"
            flag = int(half) if mdiv else 0              # the quotient is tested as fp16
            a, b = t.args
            same = fwd == rev                       # commutative: the name does not say which side runs
            if _const(b):
                self.emit(a, out)
                out.append((fwd + "i", flag << 8 | self._form(t), _round_to(b.attrs["value"], t.dtype_name)))
            elif _const(a):
                self.emit(b, out)
                out.append((rev + "i", flag << 8 | self._form(t, same), _round_to(a.attrs["value"], t.dtype_name)))
            elif _leaf(b) is not None:              # operand forms: one dispatch, no push
                self.emit(a, out)
                out.append((fwd + "_in", self.operand(_leaf(b)) | (flag << 8) | self._form(t), 0.0))
            elif _leaf(a) is not None:
                self.emit(b, out)
                out.append((rev + "_in", self.operand(_leaf(a)) | (flag << 8) | self._form(t, same), 0.0))
            elif self.need(a) >= self.need(b):
                self.emit(a, out)
                self.emit(b, out)
                out.append((fwd, flag | self._form(t), 0.0))
            else:
                self.emit(b, out)
                self.emit(a, out)
                out.append((rev, flag | self._form(t, same), 0.0))
        if half and t.op not in _MAP_EXACT and not mdiv:
            out.append(("r16", 0, 0.0))


def match_map(dst_view, value, n_groups):
    if dst_view.base.dtype_name not in _MAP_FLOATS:
        return None
    comp = _MapCompiler(n_groups)
    comp.masked = True
    if _const(value) or not comp.supported(value):
        return None
    if comp.need(value) > rt.MAP_STACK_DEPTH:
        if _maybe_masked(value):
            return None                    # the general float map may still take it
        raise NoNativeKernel(f"elementwise expression stored to {dst_view.base.name} needs an "
                             f"evaluation stack deeper than {rt.MAP_STACK_DEPTH}")
    masked = _maybe_masked(value)
    stored_in_full = bool(value.attrs.get("plain"))    # a bare numpy.ma array: every value is written
    if masked and stored_in_full and not _values_flow_plainly(value):
        return None                        # the general float map keeps numpy.ma's values
    program: list = []
    try:
        comp.emit(value, program)
    except _NeedsEntryMasks:
        return None
    if masked and stored_in_full:
        program.append(("clear", 0, 0.0))
    if len(program) > rt.MAP_MAX_INSTRS:
        raise NoNativeKernel(f"elementwise expression stored to {dst_view.base.name} compiles to "
                             f"{len(program)} operations (at most {rt.MAP_MAX_INSTRS})")
    if len(comp.inputs) > rt.MAP_MAX_INPUTS:
        raise NoNativeKernel(f"elementwise expression stored to {dst_view.base.name} reads "
                             f"{len(comp.inputs)} arrays (at most {rt.MAP_MAX_INPUTS})")
    if not comp.inputs:
        return None
    wins = [window_of(t.attrs["view"], t.shape, n_groups) for _, _, t in comp.inputs]
    wins.append(window_of(dst_view, value.shape, n_groups))
    w = _check_same_window(wins, value)
    if len(w.extent) > 2:
        raise NoNativeKernel("only 1-D and 2-D buffers have native kernels")
    types = [rt.F16 if t.dtype_name == "float16" else rt.F32 for _, _, t in comp.inputs]
    types.append(rt.F16 if dst_view.base.dtype_name == "float16" else rt.F32)

    def make(mem, ctx):
        arrays = [_Arr(_sub(mem[x.buffer], w.extent), ctx) for x in wins]
        return [rt.plan_map(program, arrays[:-1], arrays[-1], types)]
    make.program = program
    return make


# ---------------------------------------------------------------------------
# Row programs: elementwise arithmetic mixed with reductions along rows
# ---------------------------------------------------------------------------
_ROW_REDUCE = {"sum": "sum", "max": "max", "min": "min", "count": "count"}


# ---------------------------------------------------------------------------
# Integer tiles: elementwise expressions over int32 loads -> hcamdLaunchIMap
# ---------------------------------------------------------------------------
_IMAP_BINARY = {"add": "add", "sub": "sub", "mul": "mul", "floordiv": "floordiv", "mod": "mod",
                "minimum": "min", "maximum": "max", "and": "and", "or": "or", "xor": "xor",
                "shl": "shl", "shr": "shr", "lt": "lt", "le": "le", "eq": "eq", "ne": "ne",
                "ge": "ge", "gt": "gt"}
_IMAP_UNARY = {"neg": "neg", "abs": "abs"}


def match_imap(dst_view, value, n_groups):
    """An expression of int32 loads of one window, int32 constants and the
    integer operators, stored to an int32 (or, for a comparison, bool) buffer."""
    out_dt = dst_view.base.dtype_name
    if out_dt not in ("int32", "bool"):
        return None
    loads, program = [], []

    def const_of(t):
        v = t.attrs.get("exact")
        if v is None and t.op == "full":
            v = t.args[0].attrs.get("exact")
            if v is None and float(t.attrs["value"]).is_integer():
                v = int(t.attrs["value"])
        if v is None or not -2 ** 31 <= v < 2 ** 31:
            raise NoNativeKernel(f"constant {t.attrs.get('value')} is not an int32")
        return int(v)

    mirrored = {"add": "add", "mul": "mul", "min": "min", "max": "max", "and": "and", "or": "or",
                "xor": "xor", "eq": "eq", "ne": "ne", "lt": "gt", "gt": "lt", "le": "ge", "ge": "le"}
    needs = {}

    def need(t):
        """Stack entries the evaluation of t takes (Sethi-Ullman numbers; an
        operation whose operands may be exchanged evaluates the deeper one first)."""
        if id(t) in needs:
            return needs[id(t)]
        if _is(t, "astype", 1) or _is(t, "active", 1) or (t.op in _IMAP_UNARY and len(t.args) == 1):
            n = need(t.args[0])
        elif _is(t, "where", 3):
            n = max(need(t.args[0]), 1 + need(t.args[1]), 2 + need(t.args[2]))
        elif t.op in _IMAP_BINARY and len(t.args) == 2:
            a, b = need(t.args[0]), need(t.args[1])
            if _IMAP_BINARY[t.op] in mirrored:
                n = max(a, b) if a != b else a + 1
            else:
                n = max(a, b + 1)
        else:
            n = 1
        needs[id(t)] = n
        return n

    def emit(t):
        """Appends the code for t; returns False if t is not an int32 expression."""
        if _is(t, "load"):
            if t.dtype_name != "int32":
                return False
            for i, u in enumerate(loads):
                if _same(u, t):
                    program.append(("in", i, 0))
                    return True
            if len(loads) == 4:
                raise NoNativeKernel("integer expressions read at most four arrays")
            loads.append(t)
            program.append(("in", len(loads) - 1, 0))
            return True
        if _const(t):
            program.append(("const", 0, const_of(t)))
            return True
        if t.op in _IMAP_UNARY and len(t.args) == 1:
            ok = emit(t.args[0])
            program.append((_IMAP_UNARY[t.op], 0, 0))
            return ok
        if t.op in _IMAP_BINARY and len(t.args) == 2:
            a, b = t.args
            if t.attrs.get("operand_dtype", t.dtype_name) != "int32":
                return False
            op = _IMAP_BINARY[t.op]
            if t.attrs.get("right_values") and _maybe_masked(b):
                raise NoNativeKernel("a NumPy function's result on the left of % & | ^ << >> sees the values "
                                     "of the tile on the right, whatever their activity: no native code for "
                                     "integer tiles that can be inactive")
            if op in mirrored and need(b) > need(a):
                a, b, op = b, a, mirrored[op]
            ok = emit(a) and emit(b)
            program.append((op, 0, 0))
            return ok
        if _is(t, "astype", 1) and t.dtype_name == "int32" and t.args[0].dtype_name == "bool":
            return emit(t.args[0])                 # 0 / 1 as int32: the same bits
        if _is(t, "where", 3) and t.dtype_name == "int32":
            # numpy.where picks from the values and returns a plain array.  The kernel
            # keeps one activity flag per element and, under a failed // or %, the
            # value numpy.ma leaves (the dividend, 1): enough for the selection of a
            # whole stored value from operands that are such a quotient or cannot fail
            # (`numpy.where(b != 0, a // b, 0)`), not for arithmetic on top of them.
            def leaves_numpy_mas_value(x):
                return not _maybe_masked(x) or (x.op in ("floordiv", "mod") and not x.attrs.get("func") and
                                                not any(_maybe_masked(z) for z in x.args))
            if t is not value or _maybe_masked(t.args[0]) or not all(leaves_numpy_mas_value(x) for x in t.args[1:]):
                raise NoNativeKernel("numpy.where of integer tiles: only as the whole stored value, chosen by a "
                                     "condition that cannot be deactivated from operands that are a // or % "
                                     "of such values or cannot be deactivated either")
            ok = all([emit(x) for x in t.args])
            program.append(("select", 0, 0))
            return ok
        if _is(t, "active", 1):
            # tile.mask: the kernel keeps one activity flag per element, that of
            # the whole expression so far, so the mask is taken of a whole expression
            if t is not top_active:
                raise NoNativeKernel("tile.mask inside a larger integer expression has no native code "
                                     "(the mask of the stored expression has)")
            ok = emit(t.args[0])
            program.append(("active", 0, 0))
            return ok
        return False

    top_active = value.args[0] if _is(value, "astype", 1) and _is(value.args[0], "active", 1) else value
    is_cmp = value.dtype_name == "bool"
    if value.dtype_name not in ("int32", "bool") or (out_dt == "bool") != is_cmp and out_dt == "bool":
        return None
    if not emit(value) or not loads:
        return None
    depth = need(value)
    if value.attrs.get("plain") and _maybe_masked(value) and not _is(value, "where", 3):
        # A bare numpy.ma array is written in full, with what numpy.ma leaves under a
        # deactivated element.  The kernel keeps one activity flag per element and the
        # leftovers of // and % (the dividend, 1): where only NumPy functions, negation
        # and abs sit above them the plain arithmetic gives numpy.ma's values, and an
        # always-true selection makes every element active again.
        if not _values_flow_plainly(value):
            raise NoNativeKernel(f"{dst_view.base.name}: the stored value is a bare array (a NumPy function of "
                                 "integer tiles), written in full, with an operator above a // or % that can "
                                 "fail: what numpy.ma leaves there has no native code for integer tiles")
        program[:] = [("const", 0, 1)] + program + [("const", 0, 0), ("select", 0, 0)]
        depth += 1
    if depth > 4:
        raise NoNativeKernel("integer expression too deep for the four-entry stack")
    if len(program) > 32:
        raise NoNativeKernel(f"integer expression too long ({len(program)} operations, at most 32)")
    if _is(value, "load"):
        return None                                # a plain copy
    wins = [window_of(t.attrs["view"], t.shape, n_groups) for t in loads]
    wins.append(window_of(dst_view, value.shape, n_groups))
    w = _check_same_window(wins, value)
    if len(w.extent) > 2:
        raise NoNativeKernel("only 1-D and 2-D buffers have native kernels")
    prog = list(program)

    def make(mem, ctx):
        arrays = [_Arr(_sub(mem[x.buffer], w.extent), ctx) for x in wins]
        return [rt.plan_imap(prog, arrays[:-1], arrays[-1], out_bool=out_dt == "bool")]
    make.program = prog
    return make


# ---------------------------------------------------------------------------
# General float expressions -> hcamdLaunchFMap (numpy.ma's activity rules, // %,
# comparisons); what the fast map kernel does not take
# ---------------------------------------------------------------------------
_FMAP_BINARY = {"add": "add", "sub": "sub", "mul": "mul", "div": "div", "floordiv": "floordiv",
                "mod": "mod", "maximum": "max", "minimum": "min", "lt": "lt", "le": "le", "eq": "eq",
                "ne": "ne", "ge": "ge", "gt": "gt"}
_FMAP_UNARY = {"neg": "neg", "abs": "abs", "sqrt": "sqrt", "rint": "rint", "exp": "exp", "log": "log",
               "tanh": "tanh", "floor": "floor", "ceil": "ceil", "trunc": "trunc", "sign": "sign",
               "exp2": "exp2", "log2": "log2", "log10": "log10", "log1p": "log1p", "expm1": "expm1",
               "sin": "sin", "cos": "cos", "reciprocal": "reciprocal"}
_FMAP_MIRROR = {"add": "add", "mul": "mul", "max": "max", "min": "min", "eq": "eq", "ne": "ne",
                "lt": "gt", "gt": "lt", "le": "ge", "ge": "le"}
_FMAP_COMPARE = ("lt", "le", "eq", "ne", "ge", "gt")


def _compile_fmap(value, mapped=False):
    """The program of the general float map for `value`: (loads, program), or
    None if value is not a float expression that kernel takes.  Leaves are
    loads (with `mapped`, loads through a mapping too)."""
    loads, program, needs, memo = [], [], {}, {}

    def fdtype(t):
        return t.attrs.get("operand_dtype", t.dtype_name) if t.op in _FMAP_COMPARE else t.dtype_name

    def int_leaf(t):
        """The int32 load behind `load.astype(float32)`: converted when it is read."""
        if _is(t, "astype", 1) and t.dtype_name == "float32" and t.args[0].dtype_name == "int32" and \
                (_is(t.args[0], "load") or (mapped and _is(t.args[0], "mapped_load"))):
            return t.args[0]
        return None

    def need(t):
        if t.uid in needs:
            return needs[t.uid]
        if _is(t, "load") or _is(t, "mapped_load") or _const(t) or int_leaf(t) is not None:
            n = 1
        elif _is(t, "where", 3):
            n = max(need(t.args[0]), 1 + need(t.args[1]), 2 + need(t.args[2]))
        elif _is(t, "clip", 1):
            n = max(need(t.args[0]), 2)          # the bounds are pushed next to the value
        elif _is(t, "merge", 2):
            n = max(need(t.args[0]), need(t.args[1]) + 1)
        elif _is(t, "activated", 1):
            n = need(t.args[0]) + 1
        elif len(t.args) == 1:
            n = need(t.args[0])
        elif len(t.args) == 2:
            a, b = need(t.args[0]), need(t.args[1])
            if _FMAP_BINARY.get(t.op) in _FMAP_MIRROR and not mapped and not _maybe_masked(t, memo):
                n = max(a, b) if a != b else a + 1
            else:
                n = max(a, b + 1)
        else:
            n = 99
        needs[t.uid] = n
        return n

    def emit(t):
        """Appends the code for t; False if t is not a float expression this kernel takes."""
        half = t.dtype_name == "float16"
        func = bool(t.attrs.get("func"))
        plain_numpy = 4 if t.attrs.get("ieee") else 0      # operands are plain arrays: NumPy's own arithmetic
        if int_leaf(t) is not None:
            t = int_leaf(t)
        if _is(t, "load") or (mapped and _is(t, "mapped_load")):
            if t.dtype_name not in _MAP_FLOATS + ("int32",):
                return False
            for i, u in enumerate(loads):
                if _same(u, t):
                    program.append(("in", i, 0.0))
                    return True
            if len(loads) == 4:
                raise NoNativeKernel("float expressions read at most four arrays")
            loads.append(t)
            program.append(("in", len(loads) - 1, 0.0))
            return True
        if _const(t):
            return False                       # constants are pushed by the operation that uses them
        ok = True
        if _is(t, "astype", 1):
            src = t.args[0]
            if t.dtype_name not in _MAP_FLOATS or src.dtype_name not in _MAP_FLOATS + ("bool",):
                return False
            ok = emit(src)
            if half and src.dtype_name == "float32":
                program.append(("r16", 0, 0.0))
            return ok
        if _is(t, "where", 3):
            if t.dtype_name not in _MAP_FLOATS:
                return False
            for x in t.args:
                if _const(x):
                    program.append(("const", 0, _round_to(x.attrs["value"], t.dtype_name)))
                else:
                    ok = emit(x) and ok
            program.append(("select", 0, 0.0))
            return ok
        if _is(t, "active", 1):
            ok = emit(t.args[0])                   # tile.mask: the entry's activity as 0 / 1
            program.append(("active", 0, 0.0))
            return ok
        if _is(t, "activated", 1):
            # the values whatever their activity, every element active: a selection that always takes them
            if t.dtype_name not in _MAP_FLOATS or _const(t.args[0]):
                return False
            program.append(("const", 0, 1.0))
            ok = emit(t.args[0])
            program.append(("const", 0, 0.0))
            program.append(("select", 0, 0.0))
            return ok
        if _is(t, "merge", 2):
            if t.dtype_name not in _MAP_FLOATS:
                return False
            for x in t.args:
                if _const(x):
                    program.append(("const", 0, _round_to(_const_value(x), t.dtype_name)))
                else:
                    ok = emit(x) and ok
            program.append(("merge", 0, 0.0))
            return ok
        if _is(t, "clip", 1):
            ok = emit(t.args[0])
            program.append(("const", 0, _round_to(t.attrs["lo"], t.dtype_name)))
            program.append(("max", int(half), 0.0))
            program.append(("const", 0, _round_to(t.attrs["hi"], t.dtype_name)))
            program.append(("min", int(half), 0.0))
        elif t.op in _FMAP_UNARY and len(t.args) == 1:
            ok = emit(t.args[0])
            name = _FMAP_UNARY[t.op]
            if name == "sqrt" and t.attrs.get("pow"):
                name = "psqrt"                 # x ** 0.5; numpy.sqrt(x) has a domain instead
            elif name in ("sqrt", "log") and not func:
                return False
            program.append((name, plain_numpy, 0.0))
            if half and t.op not in _MAP_EXACT:
                program.append(("r16", 0, 0.0))
        elif t.op in _FMAP_BINARY and len(t.args) == 2:
            dt = fdtype(t)
            if dt not in _MAP_FLOATS:
                return False
            op = _FMAP_BINARY[t.op]
            if func and op == "floordiv" and not plain_numpy:
                raise NoNativeKernel("numpy.floor_divide called as a function has no native code "
                                     "(the // operator has)")
            a, b = t.args
            # (operands are only exchanged where no element can be inactive: the first
            # operand's value is what numpy.ma leaves in a deactivated result)
            swapped = 0
            if op in _FMAP_MIRROR and not mapped and not _maybe_masked(t, memo) and need(b) > need(a):
                a, b, op = b, a, _FMAP_MIRROR[op]
                swapped = 8                    # which of two equal values min / max return depends on the order
            for x in (a, b):
                if _const(x):
                    program.append(("const", 0, _round_to(x.attrs["value"], dt)))
                else:
                    ok = emit(x) and ok
            half_op = dt == "float16"
            # a bare numpy.ma array % tile: the tile's values, whatever their activity
            values_only = 16 if t.attrs.get("right_values") else 0
            if plain_numpy and op in ("div", "floordiv", "mod"):
                program.append((op, plain_numpy, 0.0))
            elif op == "div" and func:
                program.append(("udiv", 0, 0.0))
            elif op in ("div", "floordiv"):
                program.append((op, int(half_op), 0.0))
            elif op in ("add", "sub", "mul"):
                program.append((op, 2 if func else 0, 0.0))
            elif op in ("min", "max"):
                program.append((op, int(half_op) | swapped, 0.0))
            else:
                program.append((op, values_only | (2 if func else 0), 0.0))
            if half_op and t.op not in _MAP_EXACT and t.op not in _FMAP_COMPARE and \
                    not (op in ("div", "floordiv") and not func and not plain_numpy):
                program.append(("r16", 0, 0.0))
        else:
            return False
        if t.attrs.get("pow"):
            program.append(("powchk", 0, 0.0))
            if half:
                program.append(("r16", 0, 0.0))    # numpy.ma's fill value 1e20 is infinite as fp16
        return ok

    if _is(value, "load") or _is(value, "mapped_load") or _const(value):
        return None
    if not emit(value) or not loads:
        return None
    # (the estimate, then the program as emitted: merges and selections of shared
    # subexpressions can hold more entries than the tree's shape says)
    depth = deepest = 0
    for name, _, _ in program:
        depth += 1 if name in ("in", "const") else -2 if name == "select" else \
            -1 if name == "merge" or rt.FMAP_OPS[name] < rt.FMAP_OPS["neg"] else 0
        deepest = max(deepest, depth)
    if need(value) > 4 or deepest > 4:
        raise NoNativeKernel("float expression too deep for the four-entry stack of the general map")
    if len(program) > rt.FMAP_MAX_INSTRS:
        raise NoNativeKernel(f"float expression too long ({len(program)} operations, at most "
                             f"{rt.FMAP_MAX_INSTRS})")
    return loads, list(program)


def match_fmap(dst_view, value, n_groups):
    """An expression of fp32 / fp16 loads of one window, constants, the tile
    operators and NumPy functions, stored to an fp32, fp16 or (for a
    comparison) bool buffer, with activity tracked per operand."""
    out_dt = dst_view.base.dtype_name
    if out_dt not in _MAP_FLOATS + ("bool",):
        return None
    if (value.dtype_name == "bool") != (out_dt == "bool") or \
            (value.dtype_name != "bool" and value.dtype_name not in _MAP_FLOATS):
        return None
    compiled = _compile_fmap(value)
    if compiled is None:
        return None
    loads, prog = compiled
    wins = [window_of(t.attrs["view"], t.shape, n_groups) for t in loads]
    wins.append(window_of(dst_view, value.shape, n_groups))
    w = _check_same_window(wins, value)
    if len(w.extent) > 2:
        raise NoNativeKernel("only 1-D and 2-D buffers have native kernels")
    types = [{"float16": rt.F16, "int32": rt.I32}.get(t.dtype_name, rt.F32) for t in loads]
    types.append({"float32": rt.F32, "float16": rt.F16, "bool": rt.U8}[out_dt])
    store_all = bool(value.attrs.get("plain"))     # a bare numpy.ma array is written in full

    def make(mem, ctx):
        arrays = [_Arr(_sub(mem[x.buffer], w.extent), ctx) for x in wins]
        return [rt.plan_fmap(prog, arrays[:-1], arrays[-1], types, store_all)]
    make.program = prog
    return make


class _Table:
    """The index table of a load that the binder derived itself: [elements,
    ndim] indices inside the window (compared by identity)."""

    def __init__(self, array):
        self.array = array


def _element_tables(func, shape, ndim, name):
    """An index mapping evaluated on a whole tile: [elements, ndim] int64, the
    index inside the window of every tile element in row-major order (None:
    the identity of an unmapped load or store)."""
    import numpy as np
    if isinstance(func, _Table):
        return func.array
    grids = np.indices(shape, dtype=np.int64)
    if func is None:
        if ndim != len(shape):
            raise NoNativeKernel(f"{name}: a tile of rank {len(shape)} on a buffer of rank {ndim}")
        mapped = tuple(grids)
    else:
        try:
            mapped = func(*grids)
        except TraceError:
            raise
        except Exception as exc:
            raise NoNativeKernel(f"{name}: the mapping cannot be evaluated on index arrays "
                                 f"({type(exc).__name__}: {exc})") from exc
        if not isinstance(mapped, tuple):
            mapped = (mapped,)
        if len(mapped) != ndim:
            raise NoNativeKernel(f"{name}: the mapping must return {ndim} indices")
    out = np.zeros((math.prod(shape), ndim), np.int64)
    for d, m in enumerate(mapped):
        try:
            full = np.broadcast_to(np.asarray(m), shape)
            if full.dtype == object or full.dtype.kind == "f":
                as_int = np.array([int(v) for v in full.ravel()], dtype=np.int64).reshape(shape)
                if not all(v == w for v, w in zip(full.ravel(), as_int.ravel())):
                    raise NoNativeKernel(f"{name}: the mapping gives fractional indices")
                full = as_int
            out[:, d] = full.astype(np.int64).ravel()
        except (TypeError, ValueError) as exc:
            raise NoNativeKernel(f"{name}: mapping result of dimension {d} is not an integer "
                                 f"array ({exc})") from exc
    return out


_GATHER_MAP_MAX_DESTS = 1 << 24


def match_gather_map(dst_view, value, n_groups, out_func=None, force=False):
    """store(f(tiles...)) where a tile is loaded through a mapping, or the store
    goes through one: gathered copies, elementwise expressions of gathered
    tiles, scattered stores (python/hckernel/kernel_api.py:304-310,319-335)."""
    import numpy as np

    def has_mapped(t, seen):
        if t.uid in seen:
            return False
        seen.add(t.uid)
        return _is(t, "mapped_load") or any(has_mapped(a, seen) for a in t.args)

    if not force and not has_mapped(value, set()):
        return None
    if len(value.shape) not in (1, 2, 3):
        raise NoNativeKernel("tiles loaded or stored through a mapping have 1 to 3 dimensions")
    out_dt = dst_view.base.dtype_name
    leaf = value.args[0] if _is(value, "astype", 1) and value.dtype_name == value.args[0].dtype_name else value
    copy_bytes = 0
    # A bare numpy.ma array stored through a mapping goes element by element
    # (python/hckernel/kernel_api.py:331-334): a deactivated element is the
    # masked constant, which NumPy converts to NaN in a float array, to False
    # in a bool array and refuses to convert to an integer.
    masked_constants = out_func is not None and bool(value.attrs.get("plain"))
    if masked_constants and out_dt not in _MAP_FLOATS + ("bool",):
        raise NoNativeKernel(f"{dst_view.base.name}: a numpy.ma array stored through a mapping writes its "
                             "deactivated elements as masked constants, which only float and bool arrays take")
    if (_is(leaf, "load") or _is(leaf, "mapped_load")) and leaf.dtype_name == out_dt and not masked_constants:
        # a gathered / scattered copy: any element type
        loads, program = [leaf], []
        copy_bytes = leaf.attrs["view"].base.dtype.itemsize if hasattr(leaf.attrs["view"].base.dtype, "itemsize") else 2
        if copy_bytes not in (1, 2, 4, 8):
            raise NoNativeKernel(f"copies through a mapping move elements of 1, 2, 4 or 8 bytes")
    else:
        if out_dt not in _MAP_FLOATS + ("bool",) or (value.dtype_name == "bool") != (out_dt == "bool") or \
                (value.dtype_name != "bool" and value.dtype_name not in _MAP_FLOATS):
            raise NoNativeKernel("expressions of tiles loaded or stored through a mapping are bound "
                                 "for float32 / float16 tiles (copies for every type)")
        compiled = _compile_fmap(value, mapped=True)
        if compiled is None:
            raise NoNativeKernel(f"{value!r}: not an elementwise float expression of tiles")
        loads, program = compiled
    shape = value.shape
    for t in loads:
        if t.shape != shape:
            raise NoNativeKernel("the tiles of an expression with mapped loads must have one shape")
    total = math.prod(n_groups)
    operands = []
    for t, func in [(t, t.attrs.get("mapping")) for t in loads] + [(None, out_func)]:
        view = dst_view if t is None else t.attrs["view"]
        base = view.base
        operands.append((tuple(int(v) for v in base.shape), tuple(int(v) for v in base.strides),
                         _group_starts(view, n_groups), _element_tables(func, shape, base.ndim, base.name)))
    # two active elements of the output must not land on one address: the
    # reference stores them one after the other, a launch in no order
    o_shape, o_strides, o_starts, o_index = operands[-1]
    disjoint = False
    if out_func is None:
        # an unmapped store whose windows tile the destination: every element has a place of its own
        try:
            window_of(dst_view, shape, n_groups)
            disjoint = True
        except NoNativeKernel:
            pass
    if not disjoint:
        if total * o_index.shape[0] > _GATHER_MAP_MAX_DESTS:
            raise NoNativeKernel(f"{dst_view.base.name}: {total} groups of {o_index.shape[0]} elements are "
                                 "too many to check that no two of them are stored to one place")
        idx = o_starts[:, None, :] + o_index[None, :, :]
        inside = ((o_index[None, :, :] >= 0) & (idx < np.asarray(o_shape, np.int64))).all(axis=2)
        dest = (idx * np.asarray(o_strides, np.int64)).sum(axis=2)[inside]
        if len(np.unique(dest)) != dest.size:
            raise NoNativeKernel(f"{dst_view.base.name}: two tile elements (of one group or of two) are "
                                 "stored to one place; their order is the reference's group order, which "
                                 "a launch does not keep")
    indices = [t.attrs["view"].base.index for t in loads] + [dst_view.base.index]
    types = [{"float16": rt.F16, "int32": rt.I32}.get(t.dtype_name, rt.F32) for t in loads]
    out_type = {"float32": rt.F32, "float16": rt.F16, "bool": rt.U8}.get(out_dt, rt.F32)
    store_all = 0 if copy_bytes or not value.attrs.get("plain") else 2 if masked_constants else 1
    cache = {}

    def make(mem, ctx):
        g = cache.get(id(ctx))
        if g is None:
            g = cache[id(ctx)] = rt.GatherMap(ctx, operands, total, math.prod(shape))
        arrays = [_Arr(mem[i], ctx) for i in indices]
        return [rt.plan_gather_map(g, program, arrays[:-1], arrays[-1], types, out_type, store_all, copy_bytes)]
    make.program = program
    return make


def _gathered_form(value):
    """`value` rewritten so that every leaf is a load of value's own shape
    through an index table, with the shape-changing nodes between the loads and
    the result (broadcasts of smaller tiles, transposes, slices, reshapes)
    folded into the tables; None if value is not such an expression."""
    import numpy as np
    root = tuple(value.shape)
    elems = math.prod(root)
    memo = {}

    def rebuild(t, args):
        return Tile(t.op, tuple(args), root, t.dtype_name, **t.attrs)

    def go(t, coords):
        # coords[d][e]: along dimension d of t, the element of t that element e of the result reads
        key = (t.uid, coords.tobytes())
        if key in memo:
            return memo[key]
        out = None
        if _is(t, "const"):
            out = t
        elif _is(t, "full"):
            out = Tile("full", t.args, root, t.dtype_name, **t.attrs)
        elif _is(t, "load") or _is(t, "mapped_load"):
            view = t.attrs["view"]
            if _is(t, "load"):
                mapped = tuple(coords)
            else:
                func = t.attrs["mapping"]
                if isinstance(func, _Table):
                    flat = np.ravel_multi_index(tuple(coords), t.shape)
                    mapped = tuple(func.array[flat, d] for d in range(func.array.shape[1]))
                else:
                    mapped = tuple(_element_tables(func, t.shape, view.base.ndim, view.base.name).T)
                    flat = np.ravel_multi_index(tuple(coords), t.shape)
                    mapped = tuple(m[flat] for m in mapped)
            table = np.stack([np.asarray(m, np.int64).reshape(elems) for m in mapped], axis=1)
            out = Tile("mapped_load", (), root, t.dtype_name, view=view, mapping=_Table(table))
        elif _is(t, "transpose", 1):
            out = go(t.args[0], coords[::-1])
        elif _is(t, "reshape", 1):
            flat = np.ravel_multi_index(tuple(coords), t.shape)
            out = go(t.args[0], np.stack(np.unravel_index(flat, t.args[0].shape)))
        elif _is(t, "slice", 1):
            src = t.args[0]
            child, at, dim = [], 0, 0
            for k in t.attrs["key"]:
                if k == "new":
                    at += 1                            # a new axis of t: no axis of the source
                elif isinstance(k, tuple):
                    start, _, step = slice(*k).indices(src.shape[dim])
                    child.append(start + step * coords[at])
                    at += 1
                    dim += 1
                else:
                    child.append(np.full(elems, k % src.shape[dim], np.int64))
                    dim += 1
            out = go(src, np.stack(child)) if len(child) == len(src.shape) else None
        elif t.op in _REDUCTIONS or t.op in ("dot", "norm", "window", "update"):
            out = None
        elif len(t.args) in (1, 2, 3) and all(isinstance(a, Tile) for a in t.args):
            args = []
            for a in t.args:
                if a.shape == ():
                    args.append(go(a, np.zeros((0, elems), np.int64)) if not _const(a) else a)
                    continue
                lead = len(t.shape) - len(a.shape)
                if lead < 0:
                    return None
                sub = [coords[lead + d] if a.shape[d] == t.shape[lead + d] else np.zeros(elems, np.int64)
                       for d in range(len(a.shape))]
                args.append(go(a, np.stack(sub)))
            out = None if any(a is None for a in args) else rebuild(t, args)
        memo[key] = out
        return out

    return go(value, np.indices(root, dtype=np.int64).reshape(len(root), elems))


def _strip_views(t: Tile) -> Tile:
    while (_is(t, "transpose", 1) or _is(t, "slice", 1) or _is(t, "reshape", 1)) and isinstance(t.args[0], Tile):
        t = t.args[0]
    return t


def match_general_windows(dst_view, value, n_groups):
    """The last resort for an elementwise expression whose loads do not walk
    the store's window the way the tiled kernels need: windows shifted by a
    constant (stencils), smaller tiles broadcast over larger ones (a row or a
    column vector next to a 2-D tile), transposed, sliced or reshaped tiles.
    Every load becomes a gathered operand of hcamdGatherMap with the index
    table the expression implies (python/hckernel/kernel_api.py:297-342: the
    same bounds test per element)."""
    import numpy as np
    if len(value.shape) not in (1, 2, 3) or len(value.shape) != dst_view.base.ndim:
        return None
    out_dt = dst_view.base.dtype_name
    copy = _is(_strip_views(value), "load") and value.dtype_name == out_dt
    if not copy and (out_dt not in _MAP_FLOATS + ("bool",) or
                     any(_is(t, "load") and t.dtype_name not in _MAP_FLOATS + ("int32",) for t in _walk(value))):
        return None                              # (copies move any element type)
    lowered = _gathered_form(value)
    if lowered is None:
        return None
    if copy and (value.attrs.get("plain") or lowered.attrs.get("plain")):
        # A bare numpy.ma array is stored in full: where a load was outside its
        # buffer the reference writes the value it initialises tiles with (0), which
        # the copying form of the kernel, that moves elements, does not.  (A computed
        # value is computed from that 0 by the kernel as by the reference.)
        total = math.prod(n_groups)
        elems = math.prod(value.shape)
        if total * elems > 16 * _GATHER_MAP_MAX_DESTS:
            raise NoNativeKernel(f"{dst_view.base.name}: too many elements to check that the stored array "
                                 "has no element that was loaded from outside its buffer")
        d_starts = _group_starts(dst_view, n_groups)
        d_index = np.indices(value.shape, dtype=np.int64).reshape(len(value.shape), elems).T
        d_shape = np.asarray(dst_view.base.shape, np.int64)
        loads = [t for t in _walk(lowered) if _is(t, "mapped_load")]
        starts = [_group_starts(t.attrs["view"], n_groups) for t in loads]
        step = max(1, (1 << 21) // elems)               # groups at a time: a few tens of MB of indices
        for g0 in range(0, total, step):
            g1 = min(total, g0 + step)
            stored = ((d_starts[g0:g1, None, :] + d_index[None, :, :]) < d_shape).all(axis=2)
            for t, st in zip(loads, starts):
                view, table = t.attrs["view"], t.attrs["mapping"].array
                idx = st[g0:g1, None, :] + table[None, :, :]
                inside = ((table[None, :, :] >= 0) & (idx < np.asarray(view.base.shape, np.int64))).all(axis=2)
                if (stored & ~inside).any():
                    raise NoNativeKernel(
                        f"{dst_view.base.name}: the stored value is a bare array (a NumPy function or "
                        f"attribute of a tile), written in full, and some of its elements were loaded from "
                        f"outside {view.base.name}; the reference writes its fill value there")
    return match_gather_map(dst_view, lowered, n_groups, force=True)


class _RowCompiler(_MapCompiler):
    """Splits an expression over (rows, N) tiles that contains reductions along
    axis 1 into the stages of hcamdLaunchRowProgram.

    Every node is one of: E, an elementwise value of shape (rows, N); S, a row
    scalar of shape (rows, 1) or (rows,); V, a vector of shape (N,) or (1, N)
    that every row uses (loads only); or a constant.  A reduction of an E
    expression, a column load and an arithmetic expression of S nodes each get
    a row scalar slot; E programs read slots through the RED instructions."""

    def __init__(self, n_groups, rows, n):
        super().__init__(n_groups)
        self.rows, self.n = rows, n
        self.kinds = {}            # operand index -> "tile" | "vector"
        self.columns = []          # (buffer index, starts, load Tile)
        self.stages = []           # (kind, slot, program)
        self.slots = {}            # uid of an S node -> slot
        self.n_slots = 0

    # -- classification ----------------------------------------------------------
    def klass(self, t: Tile) -> str:
        if _const(t):
            return "C"
        if t.shape == (self.rows, self.n) and len(t.shape) == 2 and not self._is_scalar_node(t):
            return "E"
        if self._is_scalar_node(t):
            return "S"
        if t.shape in ((self.n,), (1, self.n)):
            return "V"
        return "?"

    def _is_scalar_node(self, t: Tile) -> bool:
        """Shape (rows, 1) or (rows,), and made of reductions along axis 1,
        1-D loads of `rows` elements, constants and arithmetic on those."""
        if t.shape not in ((self.rows, 1), (self.rows,)):
            return False
        if (t.op in _ROW_REDUCE or t.op == "norm") and t.attrs.get("axes") == (1,):
            return True
        if _is(t, "load") or _is(t, "slice", 1) or _is(t, "reshape", 1):
            if self.column_load(t) is not None:
                return True
            return not _is(t, "load") and self._is_scalar_node(t.args[0])
        if _is(t, "astype", 1) or t.op in _MAP_UNARY or _is(t, "clip", 1):
            return self._is_scalar_node(t.args[0])
        if (t.op in _MAP_BINARY or t.op == "vardiv") and len(t.args) == 2:
            return all(_const(a) or self._is_scalar_node(a) for a in t.args) and \
                not all(_const(a) for a in t.args)
        return False

    def column_load(self, t: Tile):
        """The load behind t if t is a per-row operand: a 1-D load of `rows`
        elements, as it is (when that cannot be mistaken for a vector of N
        elements) or viewed as (rows, 1)."""
        base = self._strip_views(t)
        if not _is(base, "load") or base.shape not in ((self.rows,), (self.rows, 1)):
            return None
        if base.shape == (self.rows, 1) and self.n == 1:
            return None                                    # a one-column tile is still a tile
        if t.shape == (self.rows, 1):
            return base
        if t.shape == (self.rows,) and self.rows != self.n:
            return base
        return None

    @staticmethod
    def _strip_views(t: Tile) -> Tile:
        while _is(t, "slice", 1) or _is(t, "reshape", 1):
            t = t.args[0]
        return t

    # -- row scalars --------------------------------------------------------------
    def _new_slot(self, t: Tile) -> int:
        if self.n_slots >= rt.ROW_MAX_SCALARS:
            raise NoNativeKernel(f"the expression needs more than {rt.ROW_MAX_SCALARS} row "
                                 "scalars (reductions, per-row operands and expressions of them)")
        self.slots[t.uid] = self.n_slots
        self.n_slots += 1
        return self.slots[t.uid]

    def find_columns(self, t: Tile, seen=None):
        """Per-row operands take the first slots, in the order they are met."""
        seen = set() if seen is None else seen
        if t.uid in seen:
            return
        seen.add(t.uid)
        if self.column_load(t) is not None:
            t = self.column_load(t)
            v = t.attrs["view"]
            if t.dtype_name not in _MAP_FLOATS:
                raise NoNativeKernel(f"{v.base.name}: per-row operands must be float32 or float16")
            for i, (b, st, _) in enumerate(self.columns):
                if b == v.base.index and same_starts(st, v.starts):
                    self.slots[t.uid] = i
                    return
            if len(self.columns) >= rt.MAP_MAX_INPUTS:
                raise NoNativeKernel(f"more than {rt.MAP_MAX_INPUTS} per-row operands")
            self.columns.append((v.base.index, v.starts, t))
            self._new_slot(t)
            return
        for a in t.args:
            self.find_columns(a, seen)

    def scalar(self, t: Tile) -> int:
        """The slot that holds S node t, adding the stages that compute it."""
        t = self._strip_views(t)
        if t.uid in self.slots:
            return self.slots[t.uid]
        for uid_t, slot in self._same_reductions:
            if _same(uid_t, t):
                self.slots[t.uid] = slot
                return slot
        if t.op == "norm" and t.attrs.get("axes") == (1,) and not _maybe_masked(t.args[0]):
            # numpy.linalg.norm along an axis is sqrt(add.reduce(x * x))
            body = t.args[0]
            total = (body * body)._reduce("sum", 1, t.attrs.get("keepdims", False))
            slot = self.scalar(Tile("sqrt", (total,), total.shape, total.dtype_name))
            self.slots[t.uid] = slot
            return slot
        if _is(t, "vardiv", 2):
            # numpy.ma's variance: the sum of the centred squares (0 where every
            # one of them is inactive, whatever made them so) over the count less
            # ddof; active wherever that is positive, whatever the division did
            total, count = t.args
            program = [("red0", self.scalar(total), 0.0)]
            if _const(count):
                program.append(("divi", 0, _round_to(count.attrs["value"], "float32")))
            else:
                c = self.scalar(count)
                program += [("mdiv_red", c, 0.0), ("livepos", c, 0.0)]
            slot = self._new_slot(t)
            self.stages.append(("scalar", slot, program))
            self._same_reductions.append((t, slot))
            return slot
        if t.op == "norm" and t.attrs.get("axes") == (1,) and _maybe_masked(t.args[0]):
            raise NoNativeKernel("numpy.linalg.norm of a tile whose elements a division or a domain "
                                 "function may deactivate: the norm adds up what such elements hold, "
                                 "which has no native code (use (x * x).sum(axis=1) for the active ones)")
        if t.op in _ROW_REDUCE and t.attrs.get("axes") == (1,):
            body = t.args[0]
            if self.klass(body) != "E":
                raise NoNativeKernel(f"{t!r}: only reductions of (rows, N) tiles along axis 1 "
                                     "have native code")
            if t.op == "sum" and body.dtype_name != "float32":
                raise NoNativeKernel("row sums are computed in float32: cast the tile with "
                                     ".astype(np.float32) before adding it up")
            program = self.program(body)
            slot = self._new_slot(t)
            self.stages.append((_ROW_REDUCE[t.op], slot, program))
            self._same_reductions.append((t, slot))
            return slot
        if _is(t, "astype", 1) and t.dtype_name == "float32" and self._is_scalar_node(t.args[0]) \
                and self._strip_views(t.args[0]).uid in self.slots:
            return self.slots[self._strip_views(t.args[0]).uid]     # widening changes nothing
        program = self.program(t, scalar=True)
        slot = self._new_slot(t)
        self.stages.append(("scalar", slot, program))
        self._same_reductions.append((t, slot))
        return slot

    _same_reductions: list

    # -- programs -------------------------------------------------------------------
    def prepare(self, t: Tile, scalar: bool):
        """Makes sure every row scalar an expression reads has its slot (and
        the stages that fill it come first)."""
        if _const(t) or _is(t, "load") and not self._is_scalar_node(t):
            return
        k = self.klass(t)
        if not scalar and k == "S":
            self.scalar(t)
            return
        if scalar:
            base = self._strip_views(t)
            if base.uid in self.slots:
                return
            if base.op in (*_ROW_REDUCE, "norm") and base.attrs.get("axes") == (1,) or \
                    _is(base, "load") or _is(base, "vardiv", 2):
                self.scalar(base)
                return
            t = base
        for a in t.args:
            self.prepare(a, scalar)

    def program(self, t: Tile, scalar: bool = False, frozen: bool = False) -> list:
        self.prepare(t, scalar)
        self._scalar_mode = scalar
        self._frozen = frozen
        # numpy.ma's rules for / ** sqrt log: in the element-wise stages stores
        # skip, and folds leave out, what they deactivate; a row scalar that they
        # deactivate deactivates every element and every row scalar computed from it
        self.masked = True
        self.need_cache = {}
        if not self.supported(t):
            raise NoNativeKernel(f"{t!r} is not an expression of float32 / float16 tiles, row "
                                 "reductions, per-row operands and constants")
        if self.need(t) > rt.MAP_STACK_DEPTH:
            raise NoNativeKernel("expression needs an evaluation stack deeper than "
                                 f"{rt.MAP_STACK_DEPTH}")
        out: list = []
        try:
            self.emit(t, out)
        except _NeedsEntryMasks:
            raise NoNativeKernel("numpy.divide called as a function next to a reduction along rows "
                                 "has no native code (the / operator has)") from None
        return out

    def slot_of(self, t: Tile):
        """Slot of t if pushing t means reading a row scalar."""
        if not isinstance(t, Tile) or _const(t):
            return None
        base = self._strip_views(t)
        if base.uid in self.slots:
            return self.slots[base.uid]
        if _is(base, "astype", 1) and base.dtype_name == "float32":
            inner = self._strip_views(base.args[0])
            if inner.uid in self.slots:
                return self.slots[inner.uid]
        return None

    def operand(self, t: Tile) -> int:
        i = super().operand(t)
        kind = "vector" if self.klass(t) == "V" else "tile"
        if self.kinds.setdefault(i, kind) != kind:
            raise NoNativeKernel("one window is used both as a tile and as a vector")
        return i

    def supported(self, t: Tile) -> bool:
        if _const(t) or self.slot_of(t) is not None:
            return True
        if t.dtype_name not in _MAP_FLOATS:
            return False
        if _is(t, "slice", 1) or _is(t, "reshape", 1):
            # views are transparent on row scalars and on (N,) -> (1, N) vectors
            inner = t.args[0]
            ok_shape = self.klass(t) in ("S", "V") and self.klass(inner) == self.klass(t)
            return ok_shape and self.supported(inner)
        if _is(t, "load"):
            return self.klass(t) in ("E", "V") and not self._scalar_mode
        if _is(t, "astype", 1) or t.op in _MAP_UNARY or _is(t, "clip", 1):
            return len(t.args) == 1 and self.supported(t.args[0])
        if t.op in _MAP_BINARY and len(t.args) == 2:
            if all(_const(a) for a in t.args):
                return False
            return all(self.supported(a) for a in t.args)
        return False

    def need(self, t: Tile) -> int:
        if self.slot_of(t) is not None:
            return 1
        if _is(t, "slice", 1) or _is(t, "reshape", 1):
            return self.need(t.args[0])
        if t.uid in self.need_cache:
            return self.need_cache[t.uid]
        if t.op in _MAP_BINARY and len(t.args) == 2:
            a, b = t.args
            if not (_const(a) or _const(b)):
                # a row scalar on one side is read by the operation itself
                if self.slot_of(b) is not None or self.slot_of(a) is not None:
                    n = self.need(a if self.slot_of(b) is not None else b)
                    self.need_cache[t.uid] = n
                    return n
        return super().need(t)

    def emit(self, t: Tile, out: list):
        slot = self.slot_of(t)
        if slot is not None:
            out.append(("red", slot, 0.0))
            return
        if _is(t, "slice", 1) or _is(t, "reshape", 1):
            self.emit(t.args[0], out)
            return
        if t.op in _MAP_BINARY and len(t.args) == 2 and not (_const(t.args[0]) or _const(t.args[1])):
            fwd, rev, _ = _MAP_BINARY[t.op]
            a, b = t.args
            sa, sb = self.slot_of(a), self.slot_of(b)
            if sb is not None or sa is not None:
                if self.masked and t.op == "div" and t.attrs.get("func") and not t.attrs.get("ieee"):
                    raise _NeedsEntryMasks()       # numpy.divide as a function: its own domain and fill value
                mdiv = self.masked and t.op == "div" and not t.attrs.get("func") and not t.attrs.get("ieee")
                if mdiv:
                    fwd, rev = "mdiv", "rmdiv"
                flag = (0x100 if t.dtype_name == "float16" else 0) if mdiv else 0
                if sb is not None:
                    self.emit(a, out)
                    out.append((fwd + "_red", sb | flag | self._form(t), 0.0))
                else:
                    self.emit(b, out)
                    out.append((rev + "_red", sa | flag | self._form(t, fwd == rev), 0.0))
                if t.dtype_name == "float16" and t.op not in _MAP_EXACT and not mdiv:
                    out.append(("r16", 0, 0.0))
                if self.masked and t.attrs.get("pow"):
                    out.append(("powchk", 0, 0.0))
                    if t.dtype_name == "float16":
                        out.append(("r16", 0, 0.0))
                return
        super().emit(t, out)


_PUSHES = ("in", "const", "red", "red0")
_STACK_BINARY = {n for fwd, rev, _ in _MAP_BINARY.values() for n in (fwd, rev)} | {"mdiv", "rmdiv"}


def _is_chain(program) -> bool:
    """A push, then operations that change that one value in place."""
    return bool(program) and program[0][0] in _PUSHES and all(
        name not in _PUSHES and name not in _STACK_BINARY for name, _, _ in program[1:])


def match_rows(dst_view, value, n_groups):
    """Elementwise expressions with reductions along the rows, e.g.
    (x - x.mean(axis=1, keepdims=True)) / x.std(axis=1, keepdims=True) or
    x.sum(axis=1): python/hckernel/tests/test_examples.py:304-336 is the
    softmax instance of the pattern.  Tiles must hold whole rows."""
    if dst_view.base.dtype_name not in _MAP_FLOATS:
        return None

    def has_row_reduce(t, seen):
        if t.uid in seen:
            return False
        seen.add(t.uid)
        if (t.op in _ROW_REDUCE or t.op == "norm") and t.attrs.get("axes") == (1,) \
                and len(t.args[0].shape) == 2:
            return True
        return any(has_row_reduce(a, seen) for a in t.args)

    def first_tile(t):
        if _is(t, "load") and len(t.shape) == 2:
            return t
        for a in t.args:
            r = first_tile(a)
            if r is not None:
                return r
        return None

    # Without a reduction the same stages serve a 2-D tile next to a row vector
    # or a per-row operand (a bias, a per-row scale): nothing then ties a tile to
    # whole rows, and the groups may cut the columns too.
    broadcast_only = not has_row_reduce(value, set())
    if broadcast_only and not (len(value.shape) == 2 and
                               any(_is(t, "load") and len(t.shape) == 1 for t in _walk(value))):
        return None
    x = first_tile(value)
    if x is None:
        return None
    rows, n = x.shape
    comp = _RowCompiler(n_groups, rows, n)
    comp._same_reductions = []
    comp.find_columns(value)
    per_row = comp._is_scalar_node(value)
    if not per_row and value.shape != (rows, n):
        return None
    if per_row:
        # A per-row result is a bare numpy.ma array: every row is written, a
        # deactivated one with what numpy.ma left in it, which the stages that
        # compute with row scalars reproduce (the tile operators leave their
        # first operand's value, NumPy functions compute regardless; the
        # instructions say which is which).
        comp.prepare(value, True)
        slot = comp.slot_of(value)
        program = [("red", slot, 0.0)] if slot is not None else comp.program(value, scalar=True)
        # (a tile instead -- a per-row operand on the left of the tile operators -- keeps
        # its deactivated rows out of the store: dst 1)
        comp.stages.append(("store_col", 0 if value.attrs.get("plain") else 1, program))
    else:
        program = comp.program(value)
        if value.attrs.get("plain") and _maybe_masked(value):
            # a bare numpy.ma array: every value is written, a deactivated one
            # with what numpy.ma left in it
            if _values_flow_plainly(value):
                program.append(("clear", 0, 0.0))      # plain arithmetic gives those values
            else:
                # a tile operator follows an operation that can deactivate: it
                # leaves its first operand's value there, which a stage that
                # changes one running value in place can do element by element
                frozen = comp.program(value, frozen=True)
                if _is_chain(frozen):
                    program = frozen + [("frozen", 0, 0.0)]
                elif _values_flow_plainly(value, finite=True):
                    # (exact wherever the operands are finite: what can fail here
                    # fails on values that are not finite already, or by overflow)
                    program.append(("clear", 0, 0.0))
                else:
                    raise NoNativeKernel("the stored value is a bare numpy.ma array, written in full, "
                                         "and a tile operator follows an operation that can deactivate "
                                         "elements: what numpy.ma leaves in those is only reproduced "
                                         "for expressions that update one running value")
        comp.stages.append(("store", 0, program))
    if len(comp.stages) > rt.ROW_MAX_STAGES:
        raise NoNativeKernel(f"the expression needs {len(comp.stages)} passes over the rows "
                             f"(at most {rt.ROW_MAX_STAGES})")
    if sum(len(p) for _, _, p in comp.stages) > rt.ROW_MAX_INSTRS:
        raise NoNativeKernel(f"the expression compiles to more than {rt.ROW_MAX_INSTRS} operations")
    if len(comp.inputs) > rt.MAP_MAX_INPUTS:
        raise NoNativeKernel(f"the expression reads {len(comp.inputs)} arrays "
                             f"(at most {rt.MAP_MAX_INPUTS})")
    # windows: tiles and the output walk the same whole rows; vectors are read
    # whole by every group; per-row operands walk the same rows
    wins, tile_win = [], None
    for i, (_, _, t) in enumerate(comp.inputs):
        w = window_of(t.attrs["view"], t.shape, n_groups)
        if comp.kinds[i] == "tile":
            if len(w.extent) != 2 or (not broadcast_only and (
                    w.driver[1] is not None or w.extent[1] != t.attrs["view"].base.shape[1] or
                    w.extent[1] != n)):
                raise NoNativeKernel("row reductions need tiles that hold whole rows")
            if tile_win is not None and (w.extent != tile_win.extent or w.driver != tile_win.driver):
                raise NoNativeKernel("the tiles of a row expression must walk the same rows")
            tile_win = tile_win or w
        wins.append(w)
    if tile_win is None:
        return None
    width = tile_win.extent[1]                 # columns of the window (n when tiles hold whole rows)
    for i, w in enumerate(wins):
        if comp.kinds[i] != "tile":
            # a vector every row uses: loaded whole by every group, or cut along the
            # columns exactly as the tiles are
            one_d = [d for d, e in enumerate(w.extent) if e != 1]
            if math.prod(w.extent) != width or len(one_d) > 1 or \
                    any(w.driver[d] is not None for d in range(len(w.extent)) if d not in one_d) or \
                    (one_d and w.driver[one_d[0]] != tile_win.driver[1]):
                raise NoNativeKernel("a vector used by every row must cover the columns of the tiles: loaded "
                                     "whole by every group, or cut along the columns as the tiles are")
    col_wins = []
    for _, _, t in comp.columns:
        w = window_of(t.attrs["view"], t.shape, n_groups)
        if w.extent[0] != tile_win.extent[0] or w.driver[0] != tile_win.driver[0] or \
                math.prod(w.extent) != w.extent[0]:
            raise NoNativeKernel("per-row operands and tiles walk different rows")
        col_wins.append(w)
    if per_row:
        out_shape = (rows,) + (1,) * (dst_view.base.ndim - 1)
        wo = window_of(dst_view, out_shape, n_groups)
        if wo.extent[0] != tile_win.extent[0] or wo.driver[0] != tile_win.driver[0] or \
                math.prod(wo.extent) != wo.extent[0]:
            raise NoNativeKernel("the per-row result and the tiles walk different rows")
    else:
        wo = window_of(dst_view, value.shape, n_groups)
        if wo.extent != tile_win.extent or wo.driver != tile_win.driver:
            raise NoNativeKernel("loads and the store walk different windows")
    ftype = lambda name: rt.F16 if name == "float16" else rt.F32
    types = [ftype(t.dtype_name) for _, _, t in comp.inputs] + \
            [ftype(t.dtype_name) for _, _, t in comp.columns] + [ftype(dst_view.base.dtype_name)]
    stages = list(comp.stages)
    n_rows = tile_win.extent[0]

    def make(mem, ctx):
        ins = []
        for i, w in enumerate(wins):
            m = mem[w.buffer]
            if comp.kinds[i] == "tile":
                ins.append(_Arr(_sub(m, w.extent), ctx))
            else:
                ins.append(_Arr(rt.Memref(m.ptr, (width,), (m.strides[-1],), m.itemsize), ctx))
        cols = []
        for w in col_wins:
            m = mem[w.buffer]
            cols.append(_Arr(rt.Memref(m.ptr, (n_rows,), (m.strides[0],), m.itemsize), ctx))
        mo = mem[wo.buffer]
        if per_row:
            out = _Arr(rt.Memref(mo.ptr, (n_rows,), (mo.strides[0],), mo.itemsize), ctx)
        else:
            out = _Arr(_sub(mo, wo.extent), ctx)
        return [rt.plan_row_program(stages, ins, out, cols, types)]
    make.stages = stages
    return make


# ---------------------------------------------------------------------------
# Reductions along columns: x.sum(axis=0) and friends of an elementwise expression
# ---------------------------------------------------------------------------
class _PostCompiler(_MapCompiler):
    """Compiles what is done to a reduction's result (a chain of unary
    operations, casts and operations with constants) with that result as
    operand 0.  numpy.ma's forms: the result is a bare array, written whatever
    its activity, with numpy.ma's fill values and dividends where an operation
    fails."""

    masked = True

    def __init__(self, n_groups, root: Tile):
        super().__init__(n_groups)
        self.root = root

    def supported(self, t: Tile) -> bool:
        return t is self.root or super().supported(t)

    def need(self, t: Tile) -> int:
        return 1 if t is self.root else super().need(t)

    def emit(self, t: Tile, out: list):
        if t is self.root:
            out.append(("in", 0, 0.0))
        elif _is(t, "masqrt", 1):
            # the standard deviation's numpy.ma.sqrt: where it fails (a variance that is
            # not finite) it leaves its argument, which is what the root of that is
            self.emit(t.args[0], out)
            out.append(("sqrt", 0, 0.0))
        else:
            super().emit(t, out)


def _is_col_reduce(t: Tile) -> bool:
    return (t.op in _ROW_REDUCE or t.op == "norm") and t.attrs.get("axes") == (0,) \
        and len(t.args) == 1 and len(t.args[0].shape) == 2


class _ColBodyCompiler(_MapCompiler):
    """The expression under a column reduction.  Besides (rows, N) tiles it may
    read per-column vectors of shape (1, N): the results of earlier column
    reductions (`temps`: uid of the reduction -> operand slot), which every row
    uses."""

    masked = True                     # numpy.ma's rules: the folds leave out what / ** sqrt log deactivate

    def __init__(self, n_groups, temps):
        super().__init__(n_groups)
        self.temps = temps            # uid -> index into the list of temporaries
        self.temp_operand = {}        # index of a temporary -> operand number

    def supported(self, t: Tile) -> bool:
        if t.uid in self.temps:
            return True
        if t.op in _MAP_BINARY and len(t.args) == 2 and not all(_const(a) for a in t.args) \
                and t.dtype_name in _MAP_FLOATS and len(t.shape) == 2:
            return all(self.supported(a) and (_const(a) or a.shape in (t.shape, (1, t.shape[1])))
                       for a in t.args)
        return super().supported(t)

    def need(self, t: Tile) -> int:
        return 1 if t.uid in self.temps else super().need(t)

    def emit(self, t: Tile, out: list):
        if t.uid in self.temps:
            k = self.temps[t.uid]
            if k not in self.temp_operand:
                self.inputs.append((None, k, t))
                self.temp_operand[k] = len(self.inputs) - 1
            out.append(("in", self.temp_operand[k], 0.0))
        else:
            super().emit(t, out)


def _compile_col_reduce(red: Tile, root: Tile, n_groups, temps):
    """(kind, program, post, compiler) of root = post(red), red a reduction
    along axis 0."""
    body = red.args[0]
    if red.op == "count":
        raise NoNativeKernel("the number of active elements down the columns (the mean, var or std of an "
                             "expression whose elements can be deactivated) has no native code")
    if red.op == "norm":          # numpy.linalg.norm along an axis is sqrt(add.reduce(x * x))
        body = body * body
    if red.op in ("sum", "norm") and body.dtype_name != "float32":
        raise NoNativeKernel("column sums are computed in float32: cast the tile with "
                             ".astype(np.float32) before adding it up")
    if red.op == "norm" and _maybe_masked(red.args[0]):
        raise NoNativeKernel("numpy.linalg.norm of a tile whose elements a division or a domain "
                             "function may deactivate: the norm adds up what such elements hold, "
                             "which has no native code (use (x * x).sum(axis=0) for the active ones)")
    if root is not red and red.op != "sum" and _maybe_masked(red.args[0]):
        # a maximum / minimum over no active element is deactivated and holds
        # numpy.ma's fill value: the kernel stores that, but computes nothing from it
        raise NoNativeKernel(f"arithmetic on the {red.op} down the columns of an expression whose "
                             "elements may be deactivated has no native code (the fold itself has)")
    comp = _ColBodyCompiler(n_groups, temps)
    if _const(body) or not comp.supported(body):
        raise NoNativeKernel(f"{body!r} is not an elementwise expression of float32 / float16 "
                             "tiles, earlier column reductions and constants")
    if comp.need(body) > rt.MAP_STACK_DEPTH:
        raise NoNativeKernel("expression needs an evaluation stack deeper than "
                             f"{rt.MAP_STACK_DEPTH}")
    program: list = []
    comp.emit_whole(body, program)
    if len(program) > rt.MAP_MAX_INSTRS or not 1 <= len(comp.inputs) <= rt.MAP_MAX_INPUTS:
        raise NoNativeKernel(f"the reduced expression compiles to {len(program)} operations on "
                             f"{len(comp.inputs)} arrays (at most {rt.MAP_MAX_INSTRS} on "
                             f"{rt.MAP_MAX_INPUTS})")
    post: list = []
    if red.op == "norm":
        post = [("in", 0, 0.0), ("sqrt", 0, 0.0)]
    if root is not red:
        pc = _PostCompiler(n_groups, red)
        if not pc.supported(root):
            raise NoNativeKernel(f"{root!r}: what follows a column reduction must be float32 / "
                                 "float16 arithmetic with constants")
        if not _values_flow_plainly(root, finite=True):      # (as for rows: overflow and inf / NaN data aside)
            raise NoNativeKernel(f"{root!r}: an operator follows an operation on a column reduction that "
                                 "can fail (a division, a root, a logarithm); the stored value would be what "
                                 "numpy.ma leaves under the deactivated result, which has no native code")
        tail: list = []
        pc.emit(root, tail)
        post = post + tail[1:] if post else tail
    if len(post) > rt.COLS_MAX_POST:
        raise NoNativeKernel(f"{len(post)} operations follow the column reduction "
                             f"(at most {rt.COLS_MAX_POST})")
    kind = "sum" if red.op == "norm" else _ROW_REDUCE[red.op]
    return kind, program, post, comp


def _no_fold_read_back_if_it_can_be_deactivated(red: Tile):
    """A fold down a column whose elements are all inactive is deactivated, and
    so is everything computed from it; the temporary vectors of the column
    kernels carry values only."""
    if _can_fail(red.args[0], finite=True):
        raise NoNativeKernel("an expression reads back a reduction down the columns of elements that "
                             "a zero divisor or a domain function may deactivate: a column without "
                             "active elements would have to deactivate what is computed from it, "
                             "which has no native code (reductions along rows have)")


def match_cols(dst_view, value, n_groups):
    """value = post(reduce(f(tiles...), axis=0)): sums, maxima, minima, means,
    variances, standard deviations and 2-norms down the columns of (rows, N)
    tiles that hold whole columns of their arrays, one group per block of
    columns.  The tile methods are the ones the simulator forwards to NumPy
    (python/hckernel/kernel_api.py:150-151).  A reduction whose expression
    reads an earlier one (the centred squares of a variance read the mean) runs
    after it, the earlier result in a temporary vector that every row uses."""
    if dst_view.base.dtype_name not in _MAP_FLOATS:
        return None
    # walk down from the stored value to the reduction
    t = value
    while not _is_col_reduce(t):
        if len(t.args) == 1 and (_is(t, "astype", 1) or t.op in _MAP_UNARY or _is(t, "clip", 1)):
            t = t.args[0]
        elif t.op in _MAP_BINARY and len(t.args) == 2 and _const(t.args[0]) != _const(t.args[1]):
            t = t.args[0] if _const(t.args[1]) else t.args[1]
        elif _is(t, "vardiv", 2) and _const(t.args[1]):
            t = t.args[0]
        else:
            return None
    outer = t
    # reductions inside the reduced expression, innermost first
    order, seen = [], set()

    def inner(t):
        if t.uid in seen:
            return
        seen.add(t.uid)
        for a in t.args:
            inner(a)
        if _is_col_reduce(t) and t is not outer:
            if not t.attrs.get("keepdims"):
                raise NoNativeKernel("a column reduction that an expression reads back needs "
                                     "keepdims=True")
            order.append(t)
    inner(outer.args[0])
    temps, steps = {}, []
    for red in order:
        _no_fold_read_back_if_it_can_be_deactivated(red)
        steps.append(_compile_col_reduce(red, red, n_groups, dict(temps)))
        temps[red.uid] = len(temps)
    steps.append(_compile_col_reduce(outer, value, n_groups, dict(temps)))
    # windows: every tile of every step walks the same whole columns
    w, step_wins = None, []
    for _, _, _, comp in steps:
        wins = []
        for b, _, tl in comp.inputs:
            if b is None:
                wins.append(None)
                continue
            x = window_of(tl.attrs["view"], tl.shape, n_groups)
            w = w or x
            if len(x.extent) != 2 or x.extent != w.extent or x.driver != w.driver:
                raise NoNativeKernel("the tiles of a column reduction must walk the same columns")
            if x.driver[0] is not None or tl.shape[0] != tl.attrs["view"].base.shape[0]:
                raise NoNativeKernel("column reductions need tiles that hold whole columns "
                                     "(as many rows as the array has)")
            wins.append(x)
        step_wins.append(wins)
    if w is None:
        return None
    wo = window_of(dst_view, value.shape, n_groups)
    if wo.extent[-1] != w.extent[1] or wo.driver[-1] != w.driver[1] or \
            math.prod(wo.extent) != wo.extent[-1]:
        raise NoNativeKernel("the per-column result and the tiles walk different columns")
    ftype = lambda name: rt.F16 if name == "float16" else rt.F32
    n_cols = w.extent[1]

    def make(mem, ctx, into=None):
        import numpy as np
        mo = mem[wo.buffer]
        if n_cols > 1 and mo.strides[-1] != 1 and into is None:
            raise NoNativeKernel("the per-column result must be contiguous")
        vectors = [rt.DeviceArray((n_cols,), np.float32, ctx) for _ in order]
        plans = []
        for i, ((kind, program, post, comp), wins) in enumerate(zip(steps, step_wins)):
            ins, types = [], []
            for (b, k, tl), x in zip(comp.inputs, wins):
                if b is None:
                    ins.append(vectors[k])
                    types.append(rt.F32)
                else:
                    ins.append(_Arr(_sub(mem[x.buffer], x.extent), ctx))
                    types.append(ftype(tl.dtype_name))
            if i < len(order):
                out, out_type = vectors[i], rt.F32
            elif into is not None:
                out, out_type = into, rt.F32
            else:
                out = _Arr(rt.Memref(mo.ptr, (n_cols,), (1,), mo.itemsize), ctx)
                out_type = ftype(dst_view.base.dtype_name)
            plans.append(rt.plan_map_reduce_cols(kind, program, ins, out, post, types + [out_type]))
        return plans
    make.program, make.post, make.kind = steps[-1][1], steps[-1][2], steps[-1][0]
    make.steps = [(k, pr, po) for k, pr, po, _ in steps]
    make.columns = (w.extent[1], w.driver[1])
    return make


def _cols_chain_root(t: Tile):
    """The column reduction under t if only what match_cols takes as a post program
    sits between them (operations with constants, functions of one operand)."""
    while not _is_col_reduce(t):
        if len(t.args) == 1 and (_is(t, "astype", 1) or t.op in _MAP_UNARY or _is(t, "clip", 1)):
            t = t.args[0]
        elif t.op in _MAP_BINARY and len(t.args) == 2 and _const(t.args[0]) != _const(t.args[1]):
            t = t.args[0] if _const(t.args[1]) else t.args[1]
        elif _is(t, "vardiv", 2) and _const(t.args[1]):
            t = t.args[0]
        else:
            return None
    return t


def match_cols_combined(dst_view, value, n_groups):
    """An elementwise expression of several reductions down the columns
    (`x.sum(axis=0) / y.sum(axis=0)`, `(x * x).mean(axis=0) - x.mean(axis=0) ** 2`):
    every reduction with what follows it alone runs as match_cols would run it,
    into a temporary vector of one element per column, and the general float map
    combines the vectors.  The reductions' results are bare numpy.ma arrays, so
    the combination follows numpy.ma's rules and is written in full; a fold that
    the data could deactivate (a column without active elements) has no activity
    to hand on and is refused."""
    if dst_view.base.dtype_name not in _MAP_FLOATS or len(value.shape) != 1 or \
            value.dtype_name not in _MAP_FLOATS or _cols_chain_root(value) is not None:
        return None
    units, fakes = [], {}

    def split(t: Tile) -> Tile:
        """t with every unit replaced by a load of its temporary vector."""
        if _const(t):
            return t
        if t.shape != value.shape:
            raise NoNativeKernel(f"{t!r} inside an expression of column reductions: only per-column values "
                                 "combine")
        if _cols_chain_root(t) is not None:
            for u, fake in units:
                if _same(u, t):
                    return fake
            proxy = type("TemporaryVector", (), {"index": -1 - len(units), "name": f"column vector {len(units)}",
                                                 "shape": t.shape, "dtype_name": "float32", "ndim": 1})()
            view = type("TemporaryView", (), {"base": proxy, "starts": ()})()
            fake = Tile("load", (), t.shape, "float32", view=view)
            if t.dtype_name != "float32":
                fake = Tile("astype", (fake,), t.shape, t.dtype_name, plain=True)
            units.append((t, fake))
            return fake
        if _is(t, "load") or not t.args:
            raise NoNativeKernel(f"{t!r} next to column reductions: only reductions down the columns and "
                                 "numbers combine")
        args = tuple(split(a) if isinstance(a, Tile) else a for a in t.args)
        return Tile(t.op, args, t.shape, t.dtype_name, **t.attrs)

    if not any(_is_col_reduce(t) for t in _walk(value)):
        return None
    combined = split(value)
    if len(units) < 2:
        return None
    makers = []
    for u, _ in units:
        for red in (t for t in _walk(u) if _is_col_reduce(t)):
            _no_fold_read_back_if_it_can_be_deactivated(red)
        mk = match_cols(dst_view, u, n_groups)
        if mk is None:
            raise NoNativeKernel(f"{u!r}: not a reduction down the columns that has a native kernel")
        makers.append(mk)
    if len({mk.columns for mk in makers}) != 1:
        raise NoNativeKernel("the column reductions of one expression must walk the same columns")
    compiled = _compile_fmap(combined)
    if compiled is None:
        raise NoNativeKernel(f"{value!r}: not an expression of column reductions that the general float map takes")
    loads, prog = compiled
    order = [next(i for i, (_, fake) in enumerate(units)
                  if (fake if _is(fake, "load") else fake.args[0]) is ld) for ld in loads]
    wo = window_of(dst_view, value.shape, n_groups)
    n_cols = makers[0].columns[0]
    out_type = {"float32": rt.F32, "float16": rt.F16}[dst_view.base.dtype_name]

    def make(mem, ctx):
        import numpy as np
        mo = mem[wo.buffer]
        if n_cols > 1 and mo.strides[-1] != 1:
            raise NoNativeKernel("the per-column result must be contiguous")
        vectors = [rt.DeviceArray((n_cols,), np.float32, ctx) for _ in units]
        plans = []
        for mk, vec in zip(makers, vectors):
            plans += mk(mem, ctx, into=vec)
        out = _Arr(rt.Memref(mo.ptr, (n_cols,), (1,), mo.itemsize), ctx)
        plans.append(rt.plan_fmap(prog, [vectors[i] for i in order], out, [rt.F32] * len(order) + [out_type],
                                  store_all=True))
        return plans
    make.program = prog
    return make


def match_cols_tile(dst_view, value, n_groups):
    """A stored (rows, N) tile expression that reads reductions down its own
    columns, e.g. (x - x.mean(axis=0, keepdims=True)) / x.std(axis=0,
    keepdims=True): the reductions run first, each into a temporary vector, and
    the tile is then one elementwise pass in which every row uses those
    vectors."""
    if dst_view.base.dtype_name not in _MAP_FLOATS or len(value.shape) != 2:
        return None
    order, seen = [], set()

    def inner(t):
        if t.uid in seen:
            return
        seen.add(t.uid)
        for a in t.args:
            inner(a)
        if _is_col_reduce(t):
            if not t.attrs.get("keepdims"):
                raise NoNativeKernel("a column reduction that an expression reads back needs "
                                     "keepdims=True")
            order.append(t)
    inner(value)
    if not order:
        return None
    temps, steps = {}, []
    for red in order:
        _no_fold_read_back_if_it_can_be_deactivated(red)
        steps.append(_compile_col_reduce(red, red, n_groups, dict(temps)))
        temps[red.uid] = len(temps)
    final = _ColBodyCompiler(n_groups, dict(temps))
    if not final.supported(value):
        raise NoNativeKernel(f"{value!r} is not an elementwise expression of float32 / float16 "
                             "tiles, column reductions and constants")
    if final.need(value) > rt.MAP_STACK_DEPTH:
        raise NoNativeKernel("expression needs an evaluation stack deeper than "
                             f"{rt.MAP_STACK_DEPTH}")
    program: list = []
    final.emit_whole(value, program)
    if value.attrs.get("plain") and _maybe_masked(value):
        if not _values_flow_plainly(value, finite=True):
            raise NoNativeKernel("the stored value is a bare numpy.ma array, written in full, and a "
                                 "tile operator follows an operation that can deactivate elements: "
                                 "what numpy.ma leaves in those has no native code here")
        program.append(("clear", 0, 0.0))      # a bare numpy.ma array: every value is written
    if len(program) > rt.MAP_MAX_INSTRS or len(final.inputs) > rt.MAP_MAX_INPUTS:
        raise NoNativeKernel(f"the stored expression compiles to {len(program)} operations on "
                             f"{len(final.inputs)} arrays (at most {rt.MAP_MAX_INSTRS} on "
                             f"{rt.MAP_MAX_INPUTS})")
    w, step_wins = None, []
    for comp in [st[3] for st in steps] + [final]:
        wins = []
        for b, _, tl in comp.inputs:
            if b is None:
                wins.append(None)
                continue
            x = window_of(tl.attrs["view"], tl.shape, n_groups)
            w = w or x
            if len(x.extent) != 2 or x.extent != w.extent or x.driver != w.driver:
                raise NoNativeKernel("the tiles of a column reduction must walk the same columns")
            if x.driver[0] is not None or tl.shape[0] != tl.attrs["view"].base.shape[0]:
                raise NoNativeKernel("column reductions need tiles that hold whole columns "
                                     "(as many rows as the array has)")
            wins.append(x)
        step_wins.append(wins)
    if w is None or all(x is None for x in step_wins[-1]):
        return None
    wo = window_of(dst_view, value.shape, n_groups)
    if wo.extent != w.extent or wo.driver != w.driver:
        raise NoNativeKernel("loads and the store walk different windows")
    ftype = lambda name: rt.F16 if name == "float16" else rt.F32
    n_cols = w.extent[1]

    def make(mem, ctx):
        import numpy as np
        vectors = [rt.DeviceArray((n_cols,), np.float32, ctx) for _ in order]

        def operands(comp, wins):
            ins, types = [], []
            for (b, k, tl), x in zip(comp.inputs, wins):
                if b is None:
                    ins.append(vectors[k])
                    types.append(rt.F32)
                else:
                    ins.append(_Arr(_sub(mem[x.buffer], x.extent), ctx))
                    types.append(ftype(tl.dtype_name))
            return ins, types
        plans = []
        for i, (kind, prog, post, comp) in enumerate(steps):
            ins, types = operands(comp, step_wins[i])
            plans.append(rt.plan_map_reduce_cols(kind, prog, ins, vectors[i], post,
                                                 types + [rt.F32]))
        ins, types = operands(final, step_wins[-1])
        out = _Arr(_sub(mem[wo.buffer], wo.extent), ctx)
        plans.append(rt.plan_row_program([("store", 0, program)], ins, out, (),
                                         types + [ftype(dst_view.base.dtype_name)]))
        return plans
    make.program = program
    make.steps = [(k, pr, po) for k, pr, po, _ in steps]
    return make


def match_pairwise(dst_view, value, n_groups):
    """out[m, n] = ||a[m, :] - b[n, :]||: the body of
    python/hckernel/tests/test_examples.py:270-301."""
    if not (_is(value, "norm", 1) and value.attrs.get("axes") == (2,) and
            not value.attrs.get("keepdims") and _is(value.args[0], "sub", 2)):
        return None
    ea, eb = value.args[0].args
    if not (_is(ea, "slice", 1) and _is(eb, "slice", 1) and
            ea.attrs["key"] == ((None, None, None), "new", (None, None, None)) and
            eb.attrs["key"] == ("new", (None, None, None), (None, None, None))):
        return None
    la, lb = ea.args[0], eb.args[0]
    if not (_is(la, "load") and _is(lb, "load")):
        return None
    if {la.dtype_name, lb.dtype_name, dst_view.base.dtype_name} != {"float32"}:
        raise NoNativeKernel("pairwise distances have a native kernel for float32 only")
    wa = window_of(la.attrs["view"], la.shape, n_groups)
    wb = window_of(lb.attrs["view"], lb.shape, n_groups)
    wo = window_of(dst_view, value.shape, n_groups)
    d = wa.extent[1]
    if wa.driver[1] is not None or wb.driver[1] is not None or wb.extent[1] != d or \
            d != la.attrs["view"].base.shape[1] or d != lb.attrs["view"].base.shape[1]:
        raise NoNativeKernel("pairwise distances need tiles that hold whole rows of a and b")
    if wo.driver != (wa.driver[0], wb.driver[0]) or wo.driver[0] == wo.driver[1]:
        raise NoNativeKernel("the output tiles must be walked by the a-row and b-row group dims")
    m, n = min(wo.extent[0], wa.extent[0]), min(wo.extent[1], wb.extent[0])

    def make(mem, ctx):
        return [rt.plan_pairwise_dist_f32(_Arr(_sub(mem[wa.buffer], (m, d)), ctx),
                                          _Arr(_sub(mem[wb.buffer], (n, d)), ctx),
                                          _Arr(_sub(mem[wo.buffer], (m, n)), ctx))]
    return make


# ---------------------------------------------------------------------------
# atomic_ref(result)[i] += <elementwise expression>.sum()
# ---------------------------------------------------------------------------
def _merge_strided_loads(terms, n_groups):
    """The idiom of python/hckernel/tests/test_examples.py:50-71: a group adds up
    N tiles of `size` elements that start at g*N*size + i*size.  Together the N
    loads tile the window [g*N*size, (g+1)*N*size); they are replaced by one
    load of N*size elements.  Returns the new list of terms."""
    loads = [t for t in terms if _is(t, "load") and len(t.shape) == 1]
    rest = [t for t in terms if not (_is(t, "load") and len(t.shape) == 1)]
    by_key = {}
    for t in loads:
        v = t.attrs["view"]
        st = v.starts[0]
        by_key.setdefault((v.base.index, tuple(st.coeffs), t.shape[0]), []).append(t)
    out = list(rest)
    for (_, coeffs, size), group in by_key.items():
        consts = sorted(t.attrs["view"].starts[0].const for t in group)
        nz = [c for c in coeffs if c]
        n = len(group)
        if n > 1 and len(nz) == 1 and nz[0] == n * size and \
                consts == [i * size for i in range(n)]:
            v = group[0].attrs["view"]
            merged = BufferView(v.base, (Affine(0, coeffs),))
            out.append(Tile("load", (), (n * size,), group[0].dtype_name, view=merged))
        else:
            out.extend(group)
    return out


def match_sum(proxy, index, value, n_groups):
    if proxy.dtype_name != "float32":
        raise NoNativeKernel(f"atomic accumulation into {proxy.name}: only float32 cells have "
                             "a native kernel")
    if not (value.op == "sum" and len(value.args) == 1 and
            value.attrs.get("axes") == tuple(range(len(value.args[0].shape)))):
        raise NoNativeKernel(f"atomic accumulation into {proxy.name}: the value must be "
                             "`<tile expression>.sum()` over all axes")
    n_cells = 1
    for s in proxy.shape:
        n_cells *= s
    if not 0 <= index < n_cells:
        raise NoNativeKernel(f"atomic accumulation into {proxy.name}: index {index} out of range")
    # sum(x + y) = sum(x) + sum(y): every term of a top-level sum gets its own
    # pass, which also covers tiles that were added up one by one
    terms: list = []
    if _maybe_masked(value.args[0]):
        # an element that a division deactivated in one term is skipped as a whole
        terms.append(value.args[0])
    else:
        _flatten_sum(value.args[0], terms)
    terms = [t for t in terms if not _const(t, 0)]
    terms = _merge_strided_loads(terms, n_groups)
    if not terms:
        raise NoNativeKernel("nothing to accumulate")
    makers = []
    for term in terms:
        comp = _MapCompiler(n_groups)
        comp.masked = True
        if not comp.supported(term):
            raise NoNativeKernel(f"atomic accumulation into {proxy.name}: {term!r} is not an "
                                 "elementwise expression over fp32 / fp16 loads")
        if comp.need(term) > rt.MAP_STACK_DEPTH:
            raise NoNativeKernel("elementwise expression needs an evaluation stack deeper than "
                                 f"{rt.MAP_STACK_DEPTH}")
        program: list = []
        try:
            comp.emit(term, program)
        except _NeedsEntryMasks:
            raise NoNativeKernel("numpy.divide called as a function inside a sum has no native "
                                 "code (the / operator has)") from None
        if len(program) > rt.MAP_MAX_INSTRS or len(comp.inputs) > rt.MAP_MAX_INPUTS or \
                not comp.inputs:
            raise NoNativeKernel("elementwise expression too large for the map kernel")
        wins = [window_of(t.attrs["view"], t.shape, n_groups) for _, _, t in comp.inputs]
        w = _check_same_window(wins)
        if len(w.extent) > 2:
            raise NoNativeKernel("only 1-D and 2-D buffers have native kernels")
        types = [rt.F16 if t.dtype_name == "float16" else rt.F32 for _, _, t in comp.inputs]

        def make(mem, ctx, program=program, wins=wins, w=w, types=types):
            arrays = [_Arr(_sub(mem[x.buffer], w.extent), ctx) for x in wins]
            return [rt.plan_map_sum(program, arrays, _Arr(mem[proxy.index], ctx), index, types)]
        make.program = program
        makers.append(make)
    return makers


# ---------------------------------------------------------------------------
# Per-subgroup partial results folded back into whole-row reductions
# ---------------------------------------------------------------------------
_FOLDS = ("max", "min", "sum")


def _slice_ranges(node: Tile):
    """(T, per-dim index or (start, stop)) if node == T[key] with unit steps."""
    if not _is(node, "slice", 1):
        return None
    src = node.args[0]
    out = []
    dims = iter(src.shape)
    for k in node.attrs["key"]:
        if k == "new":
            return None
        n = next(dims)
        if isinstance(k, tuple):
            start, stop, step = slice(*k).indices(n)
            if step != 1:
                return None
            out.append((start, max(stop, start)))
        else:
            out.append(int(k) % n)
    return src, tuple(out)


def _assembled_reduce(t: Tile):
    """t = fold(U) where the workgroup tile U was filled, element by element,
    with the same fold of disjoint pieces of one tile T that together cover T's
    rows (what subgroup-scope bodies leave behind: `partial[i, k] =
    x[i, a_k:b_k].max()` per subgroup, then `partial.max(axis=1)` after the
    barrier).  Returns the fold over T's rows, or None."""
    if t.op not in _FOLDS or len(t.args) != 1 or not _is(t.args[0], "update"):
        return None
    u = t.args[0]
    two_d = len(u.shape) == 2
    if len(u.shape) not in (1, 2):
        return None
    axes = t.attrs.get("axes")
    rows = u.shape[0] if two_d else 1
    if two_d and not (axes == (1,) or (axes == (0, 1) and rows == 1)):
        return None
    if not two_d and axes != (0,):
        return None
    pieces = {}
    node = u
    while _is(node, "update"):
        key, value = node.attrs["key"], node.args[1]
        if any(isinstance(k, tuple) for k in key):
            return None                          # a slice was assigned, not an element
        pieces.setdefault(key, value)            # the newest assignment wins
        node = node.args[0]
    if len(pieces) != math.prod(u.shape):
        return None                              # some element still holds the initial value
    source = None
    spans = {}
    for key, value in pieces.items():
        if not (_is(value, t.op, 1) and value.shape == ()):
            return None
        got = _slice_ranges(value.args[0])
        if got is None:
            return None
        src, ranges = got
        if source is None:
            source = src
        elif src is not source and not _same(src, source):
            return None
        if len(src.shape) != len(u.shape):
            return None
        if two_d:
            if not (isinstance(ranges[0], int) and ranges[0] == key[0] and isinstance(ranges[1], tuple)):
                return None
            spans.setdefault(key[0], []).append(ranges[1])
        else:
            if not isinstance(ranges[0], tuple):
                return None
            spans.setdefault(0, []).append(ranges[0])
    if source is None or (two_d and source.shape[0] != rows):
        return None
    n = source.shape[-1]
    for row in range(rows):
        at = 0
        for a, b in sorted(spans.get(row, [])):
            if a != at:
                return None
            at = b
        if at != n:
            return None
    keep = bool(t.attrs.get("keepdims"))
    if two_d and axes == (1,):
        return source._reduce(t.op, 1, keep)
    return source._reduce(t.op, None, keep)


def simplify(t: Tile, memo=None) -> Tile:
    """The traced expression with per-subgroup partial folds replaced by the
    whole-row folds they add up to; everything else unchanged."""
    memo = {} if memo is None else memo
    if id(t) in memo:
        return memo[id(t)]
    args = tuple(simplify(a, memo) for a in t.args)
    out = t
    if any(a is not b for a, b in zip(args, t.args)):
        out = Tile(t.op, args, t.shape, t.dtype_name, **t.attrs)
    folded = _assembled_reduce(out)
    if folded is not None:
        out = folded
    if _is(out, "slice", 1) and _const(out.args[0]) and _const_value(out.args[0]) is not None:
        # part of an allocated tile (CurrentGroup.vec with a shape): the same constant
        out = _const_tile(out.shape, out.dtype_name, out.args[0])
    elif _is(out, "update", 2) and all(k == (0, n) for k, n in zip(out.attrs["key"], out.shape)):
        # `tile[:] = value`, which is also what the in-place operators do
        # (python/hckernel/kernel_api.py:123-145): a tile's active elements are taken
        # and become active, the rest of the tile stays as it is; anything else (a number,
        # a bare array) overwrites the whole tile and activates it.
        old, value = out.args
        if _const(value) and _const_value(value) is not None:
            out = _const_tile(out.shape, out.dtype_name, value)
        elif value.shape == out.shape:
            filled = value if value.dtype_name == out.dtype_name else \
                Tile("astype", (value,), out.shape, out.dtype_name, **value._plain_kw())
            if value.attrs.get("plain"):
                if not _const(old) and out.dtype_name in _MAP_FLOATS:
                    # every element is overwritten with the bare array's value, whatever its
                    # activity there, and is active: a selection that always takes the value
                    out = Tile("activated", (filled,), out.shape, out.dtype_name)
            elif _maybe_masked(value):
                # elements the data can deactivate keep what the tile held (the general float
                # map has that; integer tiles stay an assignment, which no kernel takes)
                if out.dtype_name in _MAP_FLOATS:
                    if filled.op in ("add", "sub", "mul", "div", "floordiv") and not filled.attrs.get("func") \
                            and len(filled.args) == 2 and _same(filled.args[0], old) and not _maybe_masked(old) \
                            and any(_is_reduction(x) for x in _walk(filled)):
                        # tile op= x on a tile that is active everywhere: numpy.ma leaves the first
                        # operand (the dividend) under a deactivated result, which is the tile's
                        # own element, so the merged tile is the result's values, all active.
                        # (Only where a reduction keeps the general map, which has the merge
                        # itself, away: numpy.ma leaves 0 + dividend, so a kept -0 becomes +0.)
                        out = Tile("activated", (filled,), out.shape, out.dtype_name)
                    else:
                        out = Tile("merge", (old, filled), out.shape, out.dtype_name)
            elif _const(old):
                # on a freshly allocated tile: value where it is active, the allocator's fill
                # elsewhere, every element active (a load that reaches past its array is what
                # can be inactive: the store's window must not reach further than the loads')
                if _has_elementwise_load(filled):
                    memo.setdefault("overlays", []).append(filled)
                out = filled
            else:
                out = filled                     # active wherever the tile was: nothing is kept
    if out.op == "count" and _is_reduction(out) and not _maybe_masked(out.args[0]):
        # nothing can deactivate an element: the number of active elements is the
        # number of elements (tiles hold whole rows / columns of their arrays)
        n = math.prod(out.args[0].shape[a] for a in out.attrs["axes"])
        out = Tile("const", (), (), "float32", value=float(n), weak=False, exact=n, counted=True)
    elif out.op == "sub" and len(out.args) == 2 and out.args[0].attrs.get("counted") and \
            _is(out.args[1], "const"):
        n = out.args[0].attrs["value"] - out.args[1].attrs["value"]       # count - ddof
        if n <= 0:
            raise NoNativeKernel("var/std with ddof: fewer than ddof + 1 elements")
        out = Tile("const", (), (), "float32", value=float(n), weak=False, exact=int(n), counted=True)
    memo[id(t)] = out
    return out


def _without_activations_for_data_that_is_not_finite(t: Tile, memo=None) -> Tile:
    """t with `activated(x)` replaced by x wherever only overflow or data that is
    not finite can deactivate an element of x: what the kernels for reductions,
    which cannot represent the activation, compute instead (elsewhere they give
    plain arithmetic on such data too)."""
    memo = {} if memo is None else memo
    if id(t) not in memo:
        args = tuple(_without_activations_for_data_that_is_not_finite(a, memo) if isinstance(a, Tile) else a
                     for a in t.args)
        out = t if all(a is b for a, b in zip(args, t.args)) else Tile(t.op, args, t.shape, t.dtype_name, **t.attrs)
        if _is(out, "activated", 1) and not _can_fail(out.args[0], True):
            out = out.args[0]
        memo[id(t)] = out
    return memo[id(t)]


def _stored_in_full_if_activated(value: Tile) -> Tile:
    """A stored tile all of whose elements an assignment activated, with the values
    numpy.ma left in them, is to the kernels what a bare array is: written in full."""
    if _is(value, "activated", 1) and not _const(value.args[0]):
        inner = value.args[0]
        return Tile(inner.op, inner.args, inner.shape, inner.dtype_name, **{**inner.attrs, "plain": True})
    return value


def _has_elementwise_load(t: Tile) -> bool:
    """A load whose activity reaches t element by element (not through a matrix
    product, numpy.where, tile.mask or a reduction, whose results are active
    everywhere)."""
    if _is(t, "load") or _is(t, "mapped_load"):
        return True
    if t.op in ("dot", "where", "active") or _is_reduction(t):
        return False
    return any(_has_elementwise_load(a) for a in t.args if isinstance(a, Tile))


def _const_value(t: Tile):
    """The number a constant tile holds (exactly, for integers), or None."""
    if _is(t, "full") and t.args:
        t = t.args[0]
    v = t.attrs.get("exact")
    return t.attrs.get("value") if v is None else v


def _const_tile(shape, dtype, like: Tile) -> Tile:
    v = _const_value(like)
    c = Tile("const", (), (), dtype, value=float(v), weak=False,
             **({"exact": int(v)} if float(v).is_integer() else {}))
    return Tile("full", (c,), tuple(shape), dtype, value=float(v))


def _overlay_guard(view, value, overlays, n_groups):
    """A tile filled by `tile[:] = loaded` is active everywhere and holds the
    allocator's fill where the loaded tile is not; that is the loaded tile
    itself as long as the store's window is no larger than the loads'."""
    if not any(_contains(value, o) for o in overlays):
        return
    dst = window_of(view, value.shape, n_groups)
    for t in _walk(value):
        if _is(t, "load"):
            w = window_of(t.attrs["view"], t.shape, n_groups)
            if w.extent != dst.extent or w.driver != dst.driver:
                raise NoNativeKernel(
                    f"{view.base.name}: a tile filled by assignment is stored to a window larger than "
                    "what was loaded into it; the elements beyond would receive the allocator's "
                    "initial value, which no native kernel writes")


def _walk(t: Tile, seen=None):
    seen = set() if seen is None else seen
    if id(t) in seen:
        return
    seen.add(id(t))
    yield t
    for a in t.args:
        if isinstance(a, Tile):
            yield from _walk(a, seen)


def _contains(t: Tile, node: Tile) -> bool:
    return any(u is node for u in _walk(t))


_FILL_TYPES = {"float32": 4, "float16": 2, "int32": 4, "bool": 1}


def match_fill(dst_view, value, n_groups):
    """A constant tile (CurrentGroup.full / zeros / ones / empty, or arithmetic
    on constants that folded to one) stored to a window: a program that only
    pushes the constant, with no operand."""
    if not _const(value) or value.shape == ():
        return None
    v = _const_value(value)
    out_dt = dst_view.base.dtype_name
    if v is None or out_dt not in _FILL_TYPES:
        return None
    w = window_of(dst_view, value.shape, n_groups)
    if len(w.extent) > 2:
        raise NoNativeKernel("only 1-D and 2-D buffers have native kernels")
    if out_dt in ("int32", "bool"):
        iv = int(bool(v)) if out_dt == "bool" else int(v)
        if float(v) != iv and out_dt == "int32":
            raise NoNativeKernel(f"constant {v} stored to an int32 buffer")
        if not -2 ** 31 <= iv < 2 ** 31:
            raise NoNativeKernel(f"constant {v} is not an int32")
        program = [("const", 0, iv)]

        def make(mem, ctx):
            return [rt.plan_imap(program, [], _Arr(_sub(mem[w.buffer], w.extent), ctx), out_bool=out_dt == "bool")]
    else:
        program = [("const", 0, _round_to(float(v), out_dt))]
        types = [rt.F16 if out_dt == "float16" else rt.F32]

        def make(mem, ctx):
            return [rt.plan_map(program, [], _Arr(_sub(mem[w.buffer], w.extent), ctx), types)]
    make.program = program
    return make


def match_id_store(proxy, index, value, per_item, n_groups, group_shape):
    if proxy.dtype_name not in ("int32", "int64", "float32"):
        raise NoNativeKernel(f"ids can be stored to int32, int64 and float32 buffers, "
                             f"{proxy.name} is {proxy.dtype_name}")
    if math.prod(group_shape) > 1024:
        raise NoNativeKernel("a scope whose ids are stored needs groups of at most 1024 work-items")
    out_type = {"int32": rt.I32, "int64": rt.I64, "float32": rt.F32}[proxy.dtype_name]
    idx = [(i.const, i.g, i.l) for i in index]
    val = (value.const, value.g, value.l)
    rank = len(group_shape)
    # (the last Python dimension is the launch's x; the others are y and z)
    for d in range(rank - 1):
        if n_groups[d] > 65535:
            raise NoNativeKernel(f"{n_groups[d]} groups along dimension {d}: a launch takes at most 65535 "
                                 "along every dimension but the last")
    extents = [(n, s if per_item else 1) for n, s in zip(n_groups, group_shape)]

    def span(c, g, l):
        """Smallest and largest value of c + sum g[k] * gid[k] + sum l[k] * lid[k]."""
        lo = hi = c
        for k in range(rank):
            for coef, n in ((g[k], extents[k][0]), (l[k], extents[k][1])):
                lo += min(0, coef * (n - 1))
                hi += max(0, coef * (n - 1))
        return lo, hi

    for d, (c, g, l) in enumerate(idx):
        if span(c, g, l)[0] < 0:
            raise NoNativeKernel(f"{proxy.name}: the index along dimension {d} goes below 0 for some "
                                 "work-item; NumPy counts such an index from the end, the kernel does not")
    # Two work-items that store different values to one element: the simulator
    # keeps the last one's, a launch whichever comes last.
    import numpy as np
    stores = math.prod(n * s for n, s in extents)
    if stores <= 1 << 22:
        ids = np.indices([n for n, _ in extents] + [s for _, s in extents], dtype=np.int64).reshape(2 * rank, -1)

        def values(c, g, l):
            return c + sum(g[k] * ids[k] + l[k] * ids[rank + k] for k in range(rank))
        dest = np.zeros(stores, np.int64)
        for (c, g, l), n in zip(idx, proxy.shape):
            dest = dest * int(n) + np.clip(values(c, g, l), 0, int(n) - 1)
        order = np.argsort(dest, kind="stable")
        same = dest[order][1:] == dest[order][:-1]
        v = values(*val)[order]
        if (same & (v[1:] != v[:-1])).any():
            raise NoNativeKernel(f"{proxy.name}: two work-items store different values to one element; "
                                 "the simulator keeps the last one's, a launch whichever finishes last")
    else:
        # too many to enumerate: every (group id, local id) pair must walk a
        # dimension of its own as a global id does (coefficients s * n, s)
        used = set()
        ok = True
        for c, g, l in idx:
            nz = [k for k in range(rank) if g[k] or l[k]]
            if len(nz) > 1 or (nz and nz[0] in used):
                ok = False
            for k in nz:
                used.add(k)
                lk = extents[k][1]
                if not ((l[k] != 0 and g[k] == l[k] * lk) or (lk == 1 and g[k] != 0)):
                    ok = False
        moving = [k for k in range(rank) if extents[k][0] > 1 or extents[k][1] > 1]
        if not ok or any(k not in used for k in moving):
            raise NoNativeKernel(f"{proxy.name}: {stores} stores are too many to check that no two of them "
                                 "put different values into one element, and the index is not a global id")

    def make(mem, ctx):
        return [rt.plan_id_scatter(_Arr(mem[proxy.index], ctx), idx, val, n_groups, group_shape,
                                   per_item, out_type)]
    return make


_CELL_FOLDS = ("sum", "max", "min")


def match_group_cells(proxy, index, value, accumulate, n_groups):
    """`out[c + k * group_id] = f(tile.sum(), tile.max(), ...)`, or `+=` through
    atomic_ref: one number per group, from reductions of whole 1-D tiles that cut
    their arrays into consecutive pieces (the first stage of a two-stage
    reduction).  The groups' tiles are the rows of a (groups, tile) view of the
    arrays, the results a per-row output of a row program; a last tile that its
    array does not fill is a second launch over the shorter row."""
    if len(n_groups) != 1 or proxy.ndim != 1 or len(index) != 1:
        raise NoNativeKernel("one result per group is bound for 1-D work shapes and 1-D result arrays")
    if proxy.dtype_name not in _MAP_FLOATS:
        raise NoNativeKernel(f"{proxy.name}: per-group results are stored to float32 / float16 arrays")
    (at,) = index
    co = _coeffs(at, 1)[0]
    groups = n_groups[0]
    if co != 1 or at.const < 0 or at.const + groups > proxy.shape[0] or proxy.strides[0] != 1:
        raise NoNativeKernel(f"{proxy.name}[{at!r}]: per-group results go to consecutive elements inside a "
                             "dense array (the group id plus a constant)")
    loads = [t for t in _walk(value) if _is(t, "load")]
    if not loads or any(len(t.shape) != 1 or t.shape != loads[0].shape for t in loads):
        raise NoNativeKernel("per-group results are bound for reductions of 1-D tiles of one length")
    tile = loads[0].shape[0]
    n = None
    for t in loads:
        v = t.attrs["view"]
        st = v.starts[0]
        if not (isinstance(st, Affine) and st.const == 0 and _coeffs(st, 1)[0] == tile):
            raise NoNativeKernel(f"{v.base.name}: the tiles of a per-group reduction must cut the array into "
                                 "consecutive pieces (group_id * tile_length)")
        if n is not None and v.base.shape[0] != n:
            raise NoNativeKernel("the arrays of a per-group reduction must have one length")
        n = v.base.shape[0]
    full, rest = divmod(n, tile)
    if groups != full + (1 if rest else 0):
        raise NoNativeKernel(f"{groups} groups of {tile} elements over arrays of {n}: a group without an element "
                             "has nothing to reduce (numpy.ma gives it a masked value)")

    def lifted(width, rows):
        """The expression over (1, width) row tiles of (rows, width) views; the
        views are what `views` maps argument indices to."""
        memo, views = {}, {}

        def view_of(base, shape, strides, start):
            p2 = BufferProxy(base.index, base.name, shape, strides, base.dtype_name, None)
            views[base.index] = (shape, strides)
            return BufferView(p2, start)

        def go(t):
            if t.uid in memo:
                return memo[t.uid]
            if _const(t):
                out = t if t.shape == () else _const_tile((1, width), t.dtype_name, t)
            elif _is(t, "load"):
                base = t.attrs["view"].base
                v2 = view_of(base, (rows, width), (tile * base.strides[0], base.strides[0]),
                             (Affine(0, (1,)), Affine(0, (0,))))
                out = Tile("load", (), (1, width), t.dtype_name, view=v2)
            elif t.op in _CELL_FOLDS and len(t.args) == 1 and len(t.args[0].shape) == 1 and t.shape == ():
                out = Tile(t.op, (go(t.args[0]),), (1,), t.dtype_name,
                           **{**t.attrs, "axes": (1,), "keepdims": False})
            elif t.op in _REDUCTIONS or t.op in ("norm", "dot", "slice", "reshape", "transpose", "update", "window"):
                raise NoNativeKernel(f"{t!r}: per-group results are built from sum, max and min of whole 1-D "
                                     "tiles and arithmetic on them")
            else:
                args = tuple(go(a) if isinstance(a, Tile) else a for a in t.args)
                shape = (1,) if t.shape == () else (1, width)
                out = Tile(t.op, args, shape, t.dtype_name, **t.attrs)
            memo[t.uid] = out
            return out

        v2 = go(value)
        out_stride = co * proxy.strides[0]
        dst = view_of(proxy, (rows,), (out_stride,), (Affine(0, (1,)),))
        if accumulate:
            old = Tile("load", (), (1,), proxy.dtype_name, view=dst)
            v2 = Tile("add", (old, v2), (1,), proxy.dtype_name, plain=True)
        mk = match_rows(dst, v2, (rows,))
        if mk is None:
            raise NoNativeKernel(f"{value!r}: not a reduction of tiles that a row program computes")
        return mk, views

    parts = []                                    # (maker, views, first row)
    if full:
        parts.append(lifted(tile, full) + (0,))
    if rest:
        parts.append(lifted(rest, 1) + (full,))

    def make(mem, ctx):
        plans = []
        for mk, views, row0 in parts:
            patched = list(mem)
            for i, (shape, strides) in views.items():
                m = mem[i]
                if i == proxy.index and len(shape) == 1:
                    offset = at.const * m.strides[0] + row0 * strides[0]
                else:
                    offset = row0 * tile * m.strides[0]
                patched[i] = rt.Memref(m.ptr + offset * m.itemsize, shape, strides, m.itemsize)
            plans += mk(patched, ctx)
        return plans
    return make


def _has_dot(t: Tile, seen=None) -> bool:
    seen = set() if seen is None else seen
    if t.uid in seen:
        return False
    seen.add(t.uid)
    return t.op == "dot" or any(_has_dot(a, seen) for a in t.args)


def bind(stores, n_groups, atomics=(), mapped_stores=(), id_stores=(), group_shape=(), cell_stores=()):
    """stores: list of (BufferView, Tile) from one traced execution; atomics:
    list of (BufferProxy, index, Tile) atomic additions; mapped_stores: list of
    (BufferView, Tile, index function); id_stores: (BufferProxy, index, value,
    per work-item?) element stores of ids.  Returns a list of plan makers;
    raises NoNativeKernel when nothing matches."""
    if not stores and not atomics and not mapped_stores and not id_stores and not cell_stores:
        raise NoNativeKernel("the kernel body stores nothing")
    memo = {}
    stores = [(view, _stored_in_full_if_activated(simplify(value, memo))) for view, value in stores]
    stores = [(view, _without_activations_for_data_that_is_not_finite(value)
               if any(_is_reduction(t) for t in _walk(value)) else value) for view, value in stores]
    for view, value in stores:
        _overlay_guard(view, value, memo.get("overlays", ()), n_groups)
    id_makers = [match_id_store(p, i, v, per, n_groups, group_shape) for p, i, v, per in id_stores]
    if id_stores and not (stores or atomics or mapped_stores or cell_stores):
        return id_makers
    try:
        if atomics:
            if stores or mapped_stores or cell_stores:
                raise NoNativeKernel("a body that both stores tiles and accumulates "
                                     "atomically has no native kernel")
            return [mk for proxy, index, value in atomics
                    for mk in match_sum(proxy, index, simplify(value, memo), n_groups)]
        makers = list(id_makers)
        for proxy, index, value, accumulate in cell_stores:
            makers.append(match_group_cells(proxy, index, simplify(value, memo), accumulate, n_groups))
        for view, value, func in mapped_stores:
            value = simplify(value, memo)
            if _has_dot(value):
                makers.append(match_gather_gemm(view, value, n_groups, func, plain=False))
            else:
                makers.append(match_gather_map(view, value, n_groups, func, force=True))
        q = match_quantize(stores, n_groups)
        if q is not None:
            return makers + [q]
        for view, value in stores:
            try:
                for matcher in (match_fill, match_copy, match_transpose, match_imap, match_add, match_fma, match_softmax,
                                match_gemm, match_gather_gemm, match_gather_map, match_pairwise, match_cols,
                                match_cols_combined, match_cols_tile, match_rows, match_map, match_fmap, match_general_windows):
                    mk = matcher(view, value, n_groups)
                    if mk is not None:
                        makers.append(mk)
                        break
                else:
                    mk = None
            except NoNativeKernel as refusal:
                # a kernel that walks one window refused the shape of the accesses
                # (shifted, broadcast or transposed tiles): the gathered form may take it
                mk = None
                for fallback in (match_rows, match_general_windows):
                    try:
                        mk = fallback(view, value, n_groups)
                    except NoNativeKernel:
                        mk = None
                    if mk is not None:
                        break
                if mk is None:
                    raise
                makers.append(mk)
            if mk is None:
                raise NoNativeKernel(
                    f"no hand-written kernel matches the value stored to {view.base.name} "
                    f"({value!r}); bound patterns: copy, a+b (fp32), a*b+c (fp16 storage, fp32 "
                    "math), row softmax (fp32), row absmax int8 quantisation, bf16 GEMM, elementwise "
                    "expressions over fp32 / fp16 arrays, with reductions along whole rows or down "
                    "whole columns")
        return makers
    except TraceError as exc:
        raise NoNativeKernel(str(exc)) from exc

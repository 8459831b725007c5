"""GPU parity: every kernel, called through the C ABI (hc_amd.runtime is a ctypes
shim over libhc_amd_runtime.so), against the CPU oracle on the same seeded
inputs.  Integer / byte / fp16 results are compared bit for bit; fp32 softmax
within rtol 1e-5; bf16 GEMM within rtol 1e-2 of an fp32 accumulation (and bit
for bit where the arithmetic is exact).  Full benchmark sizes are covered by
the NumPy closed forms and by size-independent properties."""

import ctypes as C
import sys

import numpy as np
import pytest
from numpy.testing import assert_allclose, assert_array_equal

from hc_amd import runtime as rt
from oracle import c_oracle as co
from oracle import closed_forms as cf

pytestmark = pytest.mark.gpu

POISON32 = 0xA5A5A5A5


def say(*a):
    print(*a, file=sys.stderr, flush=True)


@pytest.fixture(scope="module")
def ctx():
    c = rt.default_context("hip:0")
    say("device:", c.info())
    return c


@pytest.fixture(autouse=True)
def default_variants():
    for fam in ("add", "fma", "softmax", "quantize", "gemm", "copy", "map", "rows", "stream", "cols", "gather", "gather_fuse"):
        rt.set_variant(fam, 0)
    yield
    for fam in ("add", "fma", "softmax", "quantize", "gemm", "copy", "map", "rows", "stream", "cols", "gather", "gather_fuse"):
        rt.set_variant(fam, 0)


def dev(a, **kw):
    return rt.to_device(a, **kw)


def poisoned(shape, dtype):
    return rt.DeviceArray(shape, dtype).fill_bytes32(POISON32)


def poison_value(dtype):
    return np.frombuffer(np.array([POISON32] * 4, np.uint32).tobytes(), dtype)[0]


class _View:
    """A window of a DeviceArray, exposed through __cuda_array_interface__."""

    def __init__(self, base, shape, offset_elems=0, strides=None):
        self.shape = tuple(shape)
        self.ctx = base.ctx
        item = base.dtype.itemsize
        self.__cuda_array_interface__ = {
            "shape": self.shape, "typestr": rt._TYPESTR[base.dtype.name],
            "data": (int(base.ptr) + offset_elems * item, False),
            "strides": None if strides is None else tuple(s * item for s in strides),
            "version": 2}


def _view(base, n, offset=0):
    return _View(base, (n,), offset)


# ---------------------------------------------------------------------------
# runtime plumbing
# ---------------------------------------------------------------------------
def test_device_is_gfx950(ctx):
    info = ctx.info()
    assert info["arch"].startswith("gfx950"), info
    assert info["compute_units"] >= 200


def test_memcpy_round_trip_and_fill(ctx):
    a = np.random.default_rng(0).integers(0, 255, 1_000_003, dtype=np.uint8)
    d = dev(a)
    assert_array_equal(d.to_host(), a)
    p = poisoned((1000,), np.uint32)
    assert_array_equal(p.to_host(), np.full(1000, POISON32, np.uint32))


def test_generic_module_kernel_launch_path(ctx):
    """olCreateModule / olGetKernel / olLaunchKernel with an embedded code
    object, the way the reference's generated host code drives the runtime
    (hcgpuGetKernel / hcgpuLaunchKernel), using the reference's kernel argument
    list for a 2-D copy: (i64, i64 stride, ptr, i64 rows, i64 cols, i64 stride,
    ptr)."""
    rows, cols = 111, 813
    a = np.arange(rows * cols, dtype=np.int32).reshape(rows, cols)
    src, dst = dev(a), poisoned((rows, cols), np.int32)
    addr, n = rt.builtin_modules()["copy"]
    mod = rt.olCreateModule(ctx.device, addr, n)
    assert mod
    k = rt.olGetKernel(mod, b"hcamd_copy2d_tiled_b4")
    assert k
    # geometry exactly as the reference derives it: block from the suggestion
    # for the reversed work shape, grid = reversed group counts
    g = (C.c_size_t * 2)(cols, rows)
    b = (C.c_size_t * 2)()
    assert rt.olSuggestBlockSize(k, g, b, 2) == 0
    assert tuple(b) == (813, 1)
    grid = (C.c_size_t * 3)(-(-cols // b[0]), -(-rows // b[1]), 1)
    block = (C.c_size_t * 3)(b[0], b[1], 1)
    vals = [C.c_int64(1), C.c_int64(cols), C.c_void_p(src.ptr), C.c_int64(rows),
            C.c_int64(cols), C.c_int64(cols), C.c_void_p(dst.ptr)]
    args = (C.c_void_p * len(vals))(*[C.cast(C.pointer(v), C.c_void_p) for v in vals])
    assert rt.olLaunchKernel(ctx.queue, k, grid, block, 3, args, len(vals), 0) == 0
    ctx.synchronize()
    assert_array_equal(dst.to_host(), a)
    # nDims != 3 is rejected with the reference's message
    assert rt.olLaunchKernel(ctx.queue, k, grid, block, 2, args, len(vals), 0) == 1
    assert "Invalid launch dims: 2" in ctx._drain()
    # unknown kernel name
    assert rt.olGetKernel(mod, b"no_such_kernel") is None
    assert "hipModuleGetFunction" in ctx._drain()
    rt.olReleaseKernel(k)
    rt.olReleaseModule(mod)


def test_hcgpu_entry_points_cache_and_launch_synchronously(ctx):
    rows, cols = 10, 20
    a = np.arange(rows * cols, dtype=np.int32).reshape(rows, cols)
    src, dst = dev(a), poisoned((rows, cols), np.int32)
    addr, n = rt.builtin_modules()["copy"]
    handle = C.c_void_p()
    k = rt.hcgpuGetKernel(C.byref(handle), b"hip:0", addr, n, b"hcamd_copy2d_tiled_b4")
    assert k and handle.value == k
    assert rt.hcgpuGetKernel(C.byref(handle), b"hip:0", None, 0, b"ignored") == k   # cached
    grid = (C.c_size_t * 3)(1, rows, 1)
    block = (C.c_size_t * 3)(cols, 1, 1)
    vals = [C.c_int64(1), C.c_int64(cols), C.c_void_p(src.ptr), C.c_int64(rows),
            C.c_int64(cols), C.c_int64(cols), C.c_void_p(dst.ptr)]
    args = (C.c_void_p * len(vals))(*[C.cast(C.pointer(v), C.c_void_p) for v in vals])
    rt.hcgpuLaunchKernel(k, grid, block, 3, args, len(vals), 0)
    # no explicit synchronisation: the call returns after the kernel finished
    out = np.empty_like(a)
    assert rt.hcamdMemcpy(ctx.queue, out.ctypes.data, dst.ptr, out.nbytes, rt.D2H) == 0
    ctx.synchronize()
    assert_array_equal(out, a)


# ---------------------------------------------------------------------------
# W0 masked tile copy (python/hckernel/tests/test_e2e.py:46-136)
# ---------------------------------------------------------------------------
E2E_SHAPES = [(1, 27), (1, 72), (1, 128), (10, 20), (111, 813), (256, 64), (256, 1024)]


@pytest.mark.parametrize("shape", E2E_SHAPES)
def test_copy_e2e_shapes_flat_path(ctx, shape):
    a = np.arange(shape[0] * shape[1], dtype=np.int32).reshape(shape)
    src, dst = dev(a), dev(np.zeros_like(a))
    rt.copy2d(src, dst)
    assert rt.last_kernel_name().startswith("hcamd_copy_flat")
    assert_array_equal(dst.to_host(), a)


@pytest.mark.parametrize("shape", E2E_SHAPES)
@pytest.mark.parametrize("unroll", [1, 2, 4])
def test_copy_e2e_shapes_reference_geometry(ctx, shape, unroll):
    """Tile decomposition of the reference: work_shape (W, ceil(H/V)), group
    shape from olSuggestBlockSize, each group copies a (gs0, gs1*V) tile."""
    rows, cols = shape
    a = np.arange(rows * cols, dtype=np.int32).reshape(shape)
    src, dst = dev(a), poisoned(shape, np.int32)
    work = (rows, -(-cols // unroll))
    gs = cf.default_group_shape(work)
    rt.copy2d_tiled(src, dst, block_x=gs[1], block_y=gs[0], unroll=unroll)
    assert_array_equal(dst.to_host(), a)


@pytest.mark.parametrize("itemsize,dtype", [(1, np.uint8), (2, np.uint16), (4, np.int32),
                                            (8, np.int64)])
def test_copy_window_smaller_than_destination_leaves_rest_untouched(ctx, itemsize, dtype):
    rng = np.random.default_rng(itemsize)
    a = rng.integers(0, 200, (37, 101)).astype(dtype)
    src, dst = dev(a), poisoned((50, 130), dtype)
    rt.copy2d(src, dst)                       # window 37 x 101 of a 50 x 130 array
    assert rt.last_kernel_name() == "hcamd_copy2d_rows_any"     # rows of 101 and of 130 elements
    assert_array_equal(dst.to_host(), cf.np_copy_window(a, np.full((50, 130), poison_value(dtype), dtype)))
    rt.set_variant("copy", 10)                # the element-wise kernel
    dst = poisoned((50, 130), dtype)
    rt.copy2d(src, dst)
    assert rt.last_kernel_name() == f"hcamd_copy2d_b{itemsize}"
    rt.set_variant("copy", 0)
    want = cf.np_copy_window(a, np.full((50, 130), poison_value(dtype), dtype))
    assert_array_equal(dst.to_host(), want)
    big = dev(rng.integers(0, 200, (64, 140)).astype(dtype))
    small = poisoned((5, 9), dtype)
    rt.copy2d(big, small)                     # source larger than destination
    assert_array_equal(small.to_host(), big.to_host()[:5, :9])


@pytest.mark.parametrize("cols,lds,ldd,off,kernel,pieces", [
    (100, 132, 136, 0, "b16", True), (100, 132, 136, 2, "b8", True), (100, 132, 136, 1, "b4", True),
    (102, 132, 136, 0, "b8", True), (100, 130, 136, 0, "b8", False), (101, 132, 136, 0, "b4", True),
    (128, 129, 128, 0, "b4", False)])
def test_copy_windows_use_the_widest_element_their_rows_allow(ctx, cols, lds, ldd, off, kernel, pieces):
    """`pieces`: the rows lie the same way against 16-byte boundaries in both arrays,
    so aligned 16-byte pieces with ragged ends move them; otherwise the pieces of the
    destination are read from wherever they lie in the source (variant 10 of "copy":
    the widest element the rows are aligned for)."""
    rows = 37
    rng = np.random.default_rng(cols + off)
    a = rng.integers(0, 1 << 30, (rows * lds + 8,)).astype(np.int32)
    want = np.full((rows * ldd + 8,), poison_value(np.int32), np.int32)
    want[off:off + rows * ldd].reshape(rows, ldd)[:, :cols] = \
        a[off:off + rows * lds].reshape(rows, lds)[:, :cols]
    for variant in (0, 10):
        rt.set_variant("copy", variant)
        src, dst = dev(a), poisoned((rows * ldd + 8,), np.int32)
        rt.copy2d(_View(src, (rows, cols), off, (lds, 1)), _View(dst, (rows, cols), off, (ldd, 1)))
        assert rt.last_kernel_name() == "hcamd_copy2d_" + (
            kernel if variant == 10 else "rows" if pieces else "rows_any")
        assert_array_equal(dst.to_host(), want)


@pytest.mark.parametrize("dtype", [np.uint8, np.int16, np.int32, np.int64])
@pytest.mark.parametrize("rows,cols,ld,soff,pieces_apart", [
    (1, 1000, 1000, 3, 1), (5, 64, 80, 1, 0), (300, 1001, 1040, 5, 1), (70_000, 67, 80, 7, 0),
    (33, 4097, 4112, 0, 1), (9, 100, 112, 15, 1)])
def test_copy_windows_in_aligned_pieces_with_ragged_ends(ctx, dtype, rows, cols, ld, soff, pieces_apart):
    """Source and destination offsets that differ by a multiple of 16 bytes, strides
    that are multiples of 16 bytes, odd widths: every byte of the window arrives and
    no byte outside it is touched, for every element size."""
    item = np.dtype(dtype).itemsize
    doff = soff + pieces_apart * (16 // item)
    rng = np.random.default_rng(rows + cols)
    a = rng.integers(0, 120, (rows * ld + 64,)).astype(dtype)
    src, dst = dev(a), poisoned((rows * ld + 64,), dtype)
    rt.copy2d(_View(src, (rows, cols), soff, (ld, 1)), _View(dst, (rows, cols), doff, (ld, 1)))
    if cols * item >= 64 and (rows == 1 or (ld * item) % 16 == 0):
        assert rt.last_kernel_name() == "hcamd_copy2d_rows"
    want = np.full((rows * ld + 64,), poison_value(dtype), dtype)
    want[doff:doff + rows * ld].reshape(rows, ld)[:, :cols] = a[soff:soff + rows * ld].reshape(rows, ld)[:, :cols]
    assert_array_equal(dst.to_host(), want)


@pytest.mark.parametrize("dtype", [np.uint8, np.int16, np.int32, np.int64])
@pytest.mark.parametrize("rows,cols,lds,ldd,soff,doff", [(1, 1000, 1000, 1000, 3, 8), (300, 1001, 1037, 1040, 5, 2),
                                                         (20_000, 67, 71, 80, 0, 7), (33, 4097, 4100, 4111, 9, 0)])
def test_copy_windows_whose_rows_lie_differently_in_the_two_arrays(ctx, dtype, rows, cols, lds, ldd, soff, doff):
    item = np.dtype(dtype).itemsize
    rng = np.random.default_rng(rows + cols)
    a = rng.integers(0, 120, (rows * lds + 64,)).astype(dtype)
    src, dst = dev(a), poisoned((rows * ldd + 64,), dtype)
    rt.copy2d(_View(src, (rows, cols), soff, (lds, 1)), _View(dst, (rows, cols), doff, (ldd, 1)))
    if cols * item >= 64:
        assert rt.last_kernel_name() in ("hcamd_copy2d_rows", "hcamd_copy2d_rows_any")
    want = np.full((rows * ldd + 64,), poison_value(dtype), dtype)
    want[doff:doff + rows * ldd].reshape(rows, ldd)[:, :cols] = a[soff:soff + rows * lds].reshape(rows, lds)[:, :cols]
    assert_array_equal(dst.to_host(), want)


@pytest.mark.parametrize("dtype", [np.uint8, np.float16, np.float32, np.int64])
@pytest.mark.parametrize("rows,cols,lds,ldd,soff,doff", [(1, 1, 1, 1, 0, 0), (64, 64, 64, 64, 0, 0), (37, 50, 50, 37, 0, 0),
                                                          (100, 130, 141, 107, 3, 5), (5, 1000, 1000, 8, 0, 1),
                                                          (1000, 3, 4, 1000, 1, 0)])
def test_transposed_copy_of_windows(ctx, dtype, rows, cols, lds, ldd, soff, doff):
    """hcamdLaunchTranspose2D: every element size, windows of larger arrays,
    extents that do not fill the 64 x 64 tiles; everything outside the window
    keeps the poison."""
    rng = np.random.default_rng(rows + cols)
    src = rng.integers(0, 200, (rows, lds)).astype(dtype)
    dsrc = dev(np.concatenate([np.zeros(soff, dtype), src.reshape(-1)]))
    ddst = poisoned((cols * ldd + doff,), dtype)
    rt.plan_transpose2d(_View(dsrc, (rows, cols), soff, (lds, 1)), _View(ddst, (cols, rows), doff, (ldd, 1))).launch()
    assert rt.last_kernel_name() == f"hcamd_transpose2d_b{np.dtype(dtype).itemsize}"
    got = ddst.to_host()
    want = np.full(cols * ldd + doff, poison_value(dtype), dtype)
    body = want[doff:].reshape(cols, ldd)
    body[:, :rows] = src[:, :cols].T
    assert_array_equal(got.view(np.uint8), want.view(np.uint8))


@pytest.mark.parametrize("variant", [0, 10])
def test_copy_from_rows_in_reverse_order(ctx, variant):
    """A source window whose row stride is negative (the rows of an array bottom up)."""
    rows, cols, ld = 61, 203, 208
    a = np.random.default_rng(3).integers(0, 1 << 30, (rows, ld)).astype(np.int32)
    src, dst = dev(a), poisoned((rows, ld), np.int32)
    rt.set_variant("copy", variant)
    rt.copy2d(_View(src, (rows, cols), (rows - 1) * ld + 1, (-ld, 1)), _View(dst, (rows, cols), 2, (ld, 1)))
    assert rt.last_kernel_name() == ("hcamd_copy2d_rows_any" if variant == 0 else "hcamd_copy2d_b4")
    want = np.full((rows * ld,), poison_value(np.int32), np.int32)
    for r in range(rows):
        want[2 + r * ld:2 + r * ld + cols] = a[rows - 1 - r, 1:1 + cols]
    assert_array_equal(dst.to_host().reshape(-1), want)


def test_copy_large_flat_all_variants(ctx):
    a = np.random.default_rng(1).integers(0, 2 ** 31, 4_000_037, dtype=np.int32)[None, :]
    src = dev(a)
    for v in range(0, 9):
        rt.set_variant("copy", v)
        dst = poisoned((1, a.size + 16), np.int32)
        rt.copy2d(src, dst)
        out = dst.to_host()
        assert_array_equal(out[:, :a.size], a)
        assert (out[:, a.size:] == np.int32(poison_value(np.int32))).all(), rt.last_kernel_name()


# ---------------------------------------------------------------------------
# integer map (hcamdLaunchIMap)
# ---------------------------------------------------------------------------
def _np_floor_shift(op, a, b):
    a64, b64 = a.astype(np.int64), b.astype(np.int64)
    if op == "shl":
        return np.where((b64 >= 0) & (b64 < 32), (a64 << np.clip(b64, 0, 31)), 0).astype(np.int64) \
            .astype(np.uint64).astype(np.uint32).view(np.int32)
    return np.where((b64 >= 0) & (b64 < 32), a64 >> np.clip(b64, 0, 31), np.where(a64 < 0, -1, 0)) \
        .astype(np.int32)


@pytest.mark.parametrize("shape,pad,off", [((1, 5000), 0, 0), ((37, 130), 6, 0), ((16, 256), 0, 0),
                                           ((9, 33), 3, 1)])
def test_imap_every_operation_against_numpy(ctx, shape, pad, off):
    """One program per opcode, int32 wrap-around semantics, aligned (16-byte) and
    unaligned / padded windows, poison outside the window."""
    rng = np.random.default_rng(shape[1])
    rows, cols = shape
    ld = cols + pad
    a = rng.integers(-2 ** 31, 2 ** 31, (rows, cols)).astype(np.int32)
    b = rng.integers(-40, 41, (rows, cols)).astype(np.int32)
    b[b == 0] = 7
    a[0, :3] = [-2 ** 31, 2 ** 31 - 1, -1]

    def padded(x):
        buf = np.full(rows * ld + off + 4, 0x0BADBEEF, np.int32)
        buf[off:off + rows * ld].reshape(rows, ld)[:, :cols] = x
        return dev(buf)
    da, dbb = padded(a), padded(b)
    wrap = lambda v: (v & 0xFFFFFFFF).astype(np.uint32).view(np.int32)
    a64, b64 = a.astype(np.int64), b.astype(np.int64)
    cases = {"add": wrap(a64 + b64), "sub": wrap(a64 - b64), "mul": wrap(a64 * b64),
             "floordiv": wrap(a64 // b64), "mod": (a64 % b64).astype(np.int32),
             "min": np.minimum(a, b), "max": np.maximum(a, b), "and": a & b, "or": a | b, "xor": a ^ b,
             "shl": _np_floor_shift("shl", a, b), "shr": _np_floor_shift("shr", a, b),
             "lt": (a < b).astype(np.int32), "le": (a <= b).astype(np.int32),
             "eq": (a == b).astype(np.int32), "ne": (a != b).astype(np.int32),
             "ge": (a >= b).astype(np.int32), "gt": (a > b).astype(np.int32)}
    view = lambda d: _View(d, (rows, cols), off, (ld, 1))
    for name, want in cases.items():
        out = poisoned((rows * ld + off + 4,), np.int32)
        rt.plan_imap([I("in", 0), I("in", 1), I(name)], [view(da), view(dbb)], view(out)).launch(sync=True)
        got = out.to_host()
        win = got[off:off + rows * ld].reshape(rows, ld)
        assert_array_equal(win[:, :cols], want, err_msg=name)
        assert (win[:, cols:].view(np.uint32) == POISON32).all(), name
        assert (got[:off].view(np.uint32) == POISON32).all() and (got[off + rows * ld:].view(np.uint32) == POISON32).all()
    for name, want in {"neg": wrap(-a64), "abs": wrap(np.abs(a64)), "not": ~a,
                       "lnot": (a == 0).astype(np.int32)}.items():
        out = poisoned((rows * ld + off + 4,), np.int32)
        rt.plan_imap([I("in", 0), I(name)], [view(da)], view(out)).launch(sync=True)
        assert_array_equal(out.to_host()[off:off + rows * ld].reshape(rows, ld)[:, :cols], want, err_msg=name)
    # a constant, and a 0 / 1 result into a one-byte buffer
    flags = poisoned((rows, cols), np.uint8)
    rt.plan_imap([I("in", 0), ("const", 0, -5), I("gt")], [view(da)], flags, out_bool=True).launch(sync=True)
    assert_array_equal(flags.to_host(), (a > -5).astype(np.uint8))


def test_imap_zero_divisors_are_left_alone_and_bad_programs_refused(ctx):
    a = np.arange(-8, 8, dtype=np.int32)
    b = np.array([0, 1, 2, 0] * 4, np.int32)
    out = poisoned((16,), np.int32)
    rt.plan_imap([I("in", 0), I("in", 1), I("floordiv"), ("const", 0, 100), I("add")],
                 [dev(a), dev(b)], out).launch(sync=True)
    got = out.to_host()
    assert (got[b == 0].view(np.uint32) == POISON32).all()
    assert_array_equal(got[b != 0], a[b != 0] // b[b != 0] + 100)
    x = dev(a)
    for prog, msg in (([I("in", 0), I("in", 0)], "leaves 2 values"), ([I("add")], "underflow"),
                      ([I("in", 1)], "operand 1"),
                      ([I("in", 0)] * 5 + [I("add")] * 4, "deeper than 4")):
        with pytest.raises(rt.HcRuntimeError, match=msg):
            rt.plan_imap(prog, [x], out).launch(sync=True)


def test_imap_and_fmap_take_more_rows_than_one_grid_dimension_holds(ctx):
    """blockIdx.y numbers the rows (at most 65535 per launch): taller windows are walked in blocks."""
    rows, cols, ld = 70_001, 3, 5
    rng = np.random.default_rng(9)
    ai = rng.integers(-1000, 1000, (rows, ld)).astype(np.int32)
    bi = rng.integers(1, 50, (rows, ld)).astype(np.int32)
    out = poisoned((rows, ld), np.int32)
    view = lambda d: _View(d, (rows, cols), 0, (ld, 1))
    dai, dbi = dev(ai), dev(bi)                      # (a view does not keep its array alive)
    rt.plan_imap([I("in", 0), I("in", 1), I("floordiv")], [view(dai), view(dbi)], view(out)).launch(sync=True)
    got = out.to_host()
    assert_array_equal(got[:, :cols], ai[:, :cols] // bi[:, :cols])
    assert (got[:, cols:].view(np.uint32) == POISON32).all()
    af = rng.standard_normal((rows, ld)).astype(np.float32)
    bf = rng.integers(-2, 3, (rows, ld)).astype(np.float32)
    outf = poisoned((rows, ld), np.float32)
    daf, dbf = dev(af), dev(bf)
    rt.plan_fmap([("in", 0, 0.0), ("in", 1, 0.0), ("div", 0, 0.0)], [view(daf), view(dbf)], view(outf),
                 [rt.F32, rt.F32, rt.F32]).launch(sync=True)
    gotf = outf.to_host()
    ok = bf[:, :cols] != 0
    with np.errstate(all="ignore"):
        want = af[:, :cols] / bf[:, :cols]
    assert_array_equal(gotf[:, :cols][ok], (want + np.float32(0) * af[:, :cols])[ok])
    assert (gotf[:, :cols][~ok].view(np.uint32) == POISON32).all() and (~ok).sum() > 10_000
    assert (gotf[:, cols:].view(np.uint32) == POISON32).all()


def _ma_special(rng, n, dtype):
    big, tiny = (3.0e38, 1.5e-38) if dtype == np.float32 else (60000.0, 6.2e-5)
    x = (rng.standard_normal(n) * 4).astype(dtype)
    special = np.array([0.0, -0.0, 1.0, -1.0, 2.5, -7.25, big, -big, tiny, np.inf, -np.inf, np.nan], dtype)
    pick = rng.random(n) < 0.4
    x[pick] = special[rng.integers(0, len(special), int(pick.sum()))]
    return x


def test_imap_select_picks_from_values_numpy_ma_leaves(ctx):
    """hcamdLaunchIMap, SELECT (numpy.where): the three top entries, condition
    deepest; the element is active again, and under a failed // or % it finds
    what numpy.ma leaves there (the dividend, 1; INT_MIN // 0 stays NumPy's 0)."""
    I = np.int32
    a = np.array([7, -7, 0, 5, np.iinfo(I).min, 9, -3, 4, 11], I)
    b = np.array([0, 0, 0, 2, 0, -4, 3, 0, 5], I)
    F = lambda name, arg=0, imm=0: (name, arg, imm)
    da, db = dev(a), dev(b)
    for op, left in (("floordiv", np.array([7, -7, 0, 2, 0, -3, -1, 4, 2], I)),
                     ("mod", np.array([1, 1, 1, 1, 0, -3, 0, 1, 1], I))):
        out = poisoned((9,), I)
        # where(1, a op b, -5): everything comes from the quotient / remainder
        rt.plan_imap([F("const", 0, 1), F("in", 0), F("in", 1), F(op), F("const", 0, -5), F("select")],
                     [da, db], out).launch(sync=True)
        assert_array_equal(out.to_host(), left, err_msg=op)
    out = poisoned((9,), I)
    rt.plan_imap([F("in", 1), F("const", 0, 0), F("ne"), F("in", 0), F("in", 1), F("floordiv"), F("const", 0, 0),
                  F("select")], [da, db], out).launch(sync=True)
    assert_array_equal(out.to_host(), np.array([0, 0, 0, 2, 0, -3, -1, 0, 2], I))
    with pytest.raises(rt.HcRuntimeError, match="underflow"):
        rt.plan_imap([F("in", 0), F("in", 1), F("select")], [da, db], out).launch(sync=True)


def test_fmap_select_tanh_and_int32_operands(ctx):
    """hcamdLaunchFMap: SELECT takes its values whatever their activity and gives an
    active result (numpy.where returns a plain array), an int32 operand is
    converted when it is read, TANH keeps the activity; a ragged 2-D window, the
    rest of the output untouched."""
    rng = np.random.default_rng(99)
    rows, cols, ld = 13, 1001, 1010
    a = rng.standard_normal((rows, ld)).astype(np.float32)
    b = rng.integers(-2, 3, (rows, ld)).astype(np.float32)
    k = rng.integers(-(2 ** 31), 2 ** 31 - 1, (rows, ld), dtype=np.int64).astype(np.int32)
    F = lambda name, arg=0, imm=0.0: (name, arg, imm)
    da, db, dk = dev(a), dev(b), dev(k)
    win = lambda d: _View(d, (rows, cols), 0, (ld, 1))
    # where(b != 0, a / b, float(k)): the quotient's deactivated elements are not taken anyway
    prog = [F("in", 1), F("const", 0, 0.0), F("ne"), F("in", 0), F("in", 1), F("div"), F("in", 2), F("select")]
    out = poisoned((rows, ld), np.float32)
    rt.plan_fmap(prog, [win(da), win(db), win(dk)], win(out), [rt.F32, rt.F32, rt.I32, rt.F32]).launch()
    got = out.to_host()
    with np.errstate(all="ignore"):
        want = np.where(b != 0, a / b, k.astype(np.float32))
    assert_array_equal(got[:, :cols].view(np.uint32), want[:, :cols].view(np.uint32))
    assert (got[:, cols:].view(np.uint32) == POISON32).all()
    # where(a / b > 0, 1, 2) on a deactivated condition: NumPy sees the value numpy.ma left (the dividend)
    prog = [F("in", 0), F("in", 1), F("div"), F("const", 0, 0.0), F("gt"), F("const", 0, 1.0), F("const", 0, 2.0),
            F("select")]
    out = poisoned((rows, ld), np.float32)
    rt.plan_fmap(prog, [win(da), win(db)], win(out), [rt.F32, rt.F32, rt.F32]).launch()
    import numpy.ma as ma
    with np.errstate(all="ignore"):
        q = ma.array(a) / ma.array(b)
        want = np.where(np.asarray(q > 0), np.float32(1), np.float32(2))
    assert_array_equal(out.to_host()[:, :cols], want[:, :cols])
    # tanh(a / b): deactivated elements are not stored
    prog = [F("in", 0), F("in", 1), F("div"), F("tanh")]
    out = poisoned((rows, ld), np.float32)
    rt.plan_fmap(prog, [win(da), win(db)], win(out), [rt.F32, rt.F32, rt.F32]).launch()
    got = out.to_host()[:, :cols]
    live = b[:, :cols] != 0
    assert (got[~live].view(np.uint32) == POISON32).all()
    assert_allclose(got[live], np.tanh(a[:, :cols][live] / b[:, :cols][live]), rtol=4e-7, atol=1e-7)
    # a program that pops more than the stack holds is refused
    with pytest.raises(rt.HcRuntimeError, match="underflow"):
        rt.plan_fmap([F("in", 0), F("in", 1), F("select")], [win(da), win(db)], win(out), [rt.F32, rt.F32, rt.F32]).launch()


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_fmap_every_operation_against_numpy_ma(ctx, dtype):
    """hcamdLaunchFMap, one program per opcode, against numpy.ma itself on data full
    of zeros, infinities and NaNs: the values, and which elements are stored.  The
    second operand is partly inactive already (a failed division in front of the
    operation under test), so the rules for inactive operands are covered too."""
    import numpy.ma as ma
    rng = np.random.default_rng(321)
    n = 20_003
    a, b, c = (_ma_special(rng, n, dtype) for _ in range(3))
    ty = rt.F32 if dtype == np.float32 else rt.F16
    half = int(dtype == np.float16)
    F = lambda name, arg=0, imm=0.0: (name, arg, imm)
    u = np.uint32 if dtype == np.float32 else np.uint16
    r16 = [F("r16")] if half else []

    def run(prog, n_in, store_all, out_dtype=None):
        out = poisoned((n,), out_dtype or dtype)
        types = [ty] * n_in + [rt.U8 if out_dtype == np.uint8 else ty]
        rt.plan_fmap(prog, [dev(a), dev(b), dev(c)][:n_in], out, types, store_all).launch(sync=True)
        return out.to_host()

    def check(name, got, want_ma, store_all):
        data, mask = ma.getdata(want_ma).astype(dtype), ma.getmaskarray(want_ma)
        poison = np.full(1, POISON32 if dtype == np.float32 else POISON32 & 0xFFFF, u).view(dtype)[0]
        want = data.copy() if store_all else np.where(mask, poison, data)
        nan = np.isnan(want)
        assert_array_equal(np.isnan(got), nan, err_msg=name)
        assert_array_equal(got.view(u)[~nan], want.view(u)[~nan], err_msg=name)

    am, bm, cm = (ma.masked_array(x) for x in (a, b, c))
    with np.errstate(all="ignore"):
        cases = {
            "add": am + bm, "sub": am - bm, "mul": am * bm, "div": am / bm, "floordiv": am // bm,
            "mod": am % bm, "min": np.minimum(am, bm), "max": np.maximum(am, bm), "udiv": np.divide(am, bm)}
        for name, want in cases.items():
            arg = half if name in ("div", "floordiv", "min", "max") else 0
            tail = [] if name in ("div", "floordiv", "min", "max") else r16
            for store_all in (False, True):
                check(name, run([F("in", 0), F("in", 1), F(name, arg)] + tail, 2, store_all), want, store_all)
        # the same operations on a second operand that a division has partly deactivated: b / c
        q = bm / cm
        cases2 = {"add": am + q, "sub": am - q, "mul": am * q, "div": am / q, "floordiv": am // q,
                  "mod": am % q, "max": np.maximum(am, q), "udiv": np.divide(am, q),
                  "add|2": np.add(am, q), "mul|2": np.multiply(am, q)}
        for name, want in cases2.items():
            op, _, fn = name.partition("|")
            arg = (half if op in ("div", "floordiv", "max") else 0) | (2 if fn else 0)
            tail = [] if op in ("div", "floordiv", "max") else r16
            prog = [F("in", 0), F("in", 1), F("in", 2), F("div", half), F(op, arg)] + tail
            for store_all in (False, True):
                check("a " + name + " (b/c)", run(prog, 3, store_all), want, store_all)
        unary = {"neg": -q, "abs": abs(q), "sqrt": np.sqrt(q), "log": None, "rint": np.rint(q),
                 "psqrt": None}
        for name, want in unary.items():
            if want is None:
                continue
            prog = [F("in", 1), F("in", 2), F("div", half), F(name)] + ([] if name in ("neg", "abs") else r16)
            for store_all in (False, True):
                check(name + "(b/c)", run(prog, 3, store_all), want, store_all)
        # x ** 2 as numpy.ma.power computes and checks it
        want = ma.power(am, dtype(2))
        check("pow2", run([F("in", 0), F("in", 0), F("mul")] + r16 + [F("powchk")], 1, False), want, False)
        check("pow2", run([F("in", 0), F("in", 0), F("mul")] + r16 + [F("powchk")], 1, True), want, True)
        # comparisons into a one-byte buffer; inactive elements are left alone
        for name, want in {"lt": am < q, "le": am <= q, "ge": am >= q, "gt": am > q, "ne": am != bm,
                           "eq": am == bm}.items():
            second = [F("in", 1)] if name in ("ne", "eq") else [F("in", 1), F("in", 2), F("div", half)]
            got = run([F("in", 0)] + second + [F(name)], 3, False, np.uint8)
            data, mask = ma.getdata(want).astype(np.uint8), ma.getmaskarray(want)
            assert_array_equal(got, np.where(mask, POISON32 & 0xFF, data), err_msg=name)
    with pytest.raises(rt.HcRuntimeError, match="underflow"):
        rt.plan_fmap([F("add")], [dev(a)], poisoned((n,), dtype), [ty, ty]).launch(sync=True)
    with pytest.raises(rt.HcRuntimeError, match="leaves 2 values"):
        rt.plan_fmap([F("in", 0), F("in", 0)], [dev(a)], poisoned((n,), dtype), [ty, ty]).launch(sync=True)


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_fmap_every_opcode_and_flag_against_its_numpy_restatement(ctx, dtype):
    """hcamdLaunchFMap against tests/fmap_emulator.py (the rules of the kernel's
    header in NumPy, which the CPU tests run the binder's programs with), for
    every opcode under every flag it reads: bit 0 fp16, bit 1 called as a
    function, bit 2 plain arrays, bit 3 operands evaluated in the other order,
    bit 4 the second operand's activity does not count.  Operands are quotients
    with zero divisors, so both carry inactive elements; stored where active and
    in full."""
    from fmap_emulator import run_fmap
    rng = np.random.default_rng(77)
    n = 6_007
    a, b, c = (_ma_special(rng, n, dtype) for _ in range(3))
    ty = rt.F32 if dtype == np.float32 else rt.F16
    half = int(dtype == np.float16)
    u = np.uint32 if dtype == np.float32 else np.uint16
    F = lambda name, arg=0, imm=0.0: (name, arg, imm)
    r16 = [F("r16")] if half else []
    left = [F("in", 0), F("in", 1), F("div", half)]            # a / b: inactive where b == 0 ...
    right = [F("in", 2), F("in", 0), F("div", half)]           # c / a
    inexact = {"exp", "log", "tanh", "exp2", "log2", "log10", "log1p", "expm1", "sin", "cos"}
    binary = ["add", "sub", "mul", "div", "floordiv", "mod", "min", "max", "udiv", "lt", "le", "eq", "ne", "ge", "gt",
              "merge"]
    unary = [k for k in rt.FMAP_OPS if k not in binary + ["end", "in", "const", "select"]]
    programs = []
    for name in binary:
        for arg in (0, 1, 2, 4, 8, 16, 2 | 16, 1 | 8):
            programs.append((f"{name}|{arg}", left + right + [F(name, arg)] + r16))
    for name in unary:
        for arg in (0, 4):
            programs.append((f"{name}|{arg}", left + [F(name, arg)] + r16))
            programs.append((f"{name}|{arg} of an operand", [F("in", 0), F(name, arg)] + r16))
    programs.append(("select", left + right + [F("lt")] + left + right + [F("select")]))
    da, db, dc = dev(a), dev(b), dev(c)
    for label, prog in programs:
        for store_all in (False, True):
            say("fmap", np.dtype(dtype).name, label, store_all)
            out = poisoned((n,), dtype)
            rt.plan_fmap(prog, [da, db, dc], out, [ty, ty, ty, ty], store_all).launch(sync=True)
            got = out.to_host()
            want = np.full(1, POISON32 if dtype == np.float32 else POISON32 & 0xFFFF, u).view(dtype).repeat(n)
            run_fmap(prog, [a, b, c], store_all, want)
            nan = np.isnan(want)
            assert_array_equal(np.isnan(got), nan, err_msg=label)
            if label.split("|")[0] in inexact:
                assert_allclose(got[~nan].astype(np.float64), want[~nan].astype(np.float64),
                                rtol=2e-3 if half else 1e-6, atol=2e-3 if half else 1e-7, err_msg=label)
            else:
                assert_array_equal(got.view(u)[~nan], want.view(u)[~nan], err_msg=label)


# ---------------------------------------------------------------------------
# stream calibration kernels (the yardstick of the memory-bound kernels)
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("n_reads,write", [(1, "full"), (2, "full"), (3, "full"), (0, "full"),
                                            (1, "half"), (1, "none")])
@pytest.mark.parametrize("variant", [0, 1, 2, 3, 4, 5])
def test_stream_mixes_compute_what_they_say(ctx, n_reads, write, variant):
    rt.set_variant("stream", variant)
    try:
        _stream_mix(n_reads, write, variant)
    finally:
        rt.set_variant("stream", 0)


def _stream_mix(n_reads, write, variant):
    nbytes = 5 * 16384
    rng = np.random.default_rng(60 + n_reads)
    ins = [rng.integers(0, 2 ** 32, nbytes // 4, dtype=np.uint32) for _ in range(n_reads)]
    words = {"full": nbytes // 4, "half": nbytes // 8, "none": nbytes // 16384}[write]
    pad = 8
    out = poisoned((words + pad,), np.uint32)
    rt.plan_stream([dev(x) for x in ins], _View(out, (words,), 0), write).launch(sync=True)
    say("stream", n_reads, write, rt.last_kernel_name())
    plain = "hcamd_stream_r%dw%d%s" % (n_reads, write != "none", "h" if write == "half" else "")
    both = n_reads > 0 and write != "none"
    suffix = {0: "_w4_d6" if n_reads == 3 else "", 1: "", 2: "_w4_d6", 3: "_w4_d0", 4: "_w4_d12",
              5: "_w8"}[variant] if both else ""
    assert rt.last_kernel_name() == plain + suffix
    total = np.zeros(nbytes // 4, np.uint32)
    for x in ins:
        total += x
    if n_reads == 0:
        total = np.repeat(np.arange(nbytes // 16, dtype=np.uint32), 4)
    want = {"full": total, "half": total[0::2] ^ total[1::2],
            "none": total.reshape(-1, 4096).sum(axis=1, dtype=np.uint32)}[write]
    got = out.to_host()
    assert_array_equal(got[:words], want)
    assert (got[words:] == POISON32).all()


def test_stream_refusals(ctx):
    x = dev(np.zeros(16384 // 4, np.uint32))
    y = rt.DeviceArray((16384 // 4,), np.uint32)
    with pytest.raises(rt.HcRuntimeError, match="multiple of 16 KiB"):
        rt.plan_stream([_View(x, (1000,), 0)], _View(y, (1000,), 0)).launch(sync=True)
    with pytest.raises(rt.HcRuntimeError, match="no kernel"):
        rt.plan_stream([x, x], y, "half").launch(sync=True)
    with pytest.raises(rt.HcRuntimeError, match="needed"):
        rt.plan_stream([x], _View(y, (100,), 0), "full")


# ---------------------------------------------------------------------------
# W1 c = a + b
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("n", [1, 3, 4, 255, 1024, 4099, 262_144, 1_000_003])
def test_add_bit_exact_with_untouched_tail(ctx, n):
    a, b = cf.inputs_c1(n)
    want = cf.np_add(a, b)
    assert_array_equal(want.view(np.uint32), co.add_f32(a, b).view(np.uint32))
    da, db = dev(a), dev(b)
    for v in range(0, 10):
        rt.set_variant("add", v)
        dc = poisoned((n + 8,), np.float32)
        rt.add_f32(da, db, _view(dc, n))
        out = dc.to_host()
        assert_array_equal(out[:n].view(np.uint32), want.view(np.uint32))
        assert (out[n:].view(np.uint32) == POISON32).all(), (v, rt.last_kernel_name())


def test_add_misaligned_pointers_take_the_scalar_kernel(ctx):
    n = 10_001
    a, b = cf.inputs_c1(n + 1)
    da, db, dc = dev(a), dev(b), poisoned((n + 9,), np.float32)
    rt.add_f32(_view(da, n, 1), _view(db, n, 1), _view(dc, n, 1))
    assert rt.last_kernel_name() == "hcamd_add_f32_scalar"
    out = dc.to_host()
    assert_array_equal(out[1:n + 1].view(np.uint32), (a[1:] + b[1:]).view(np.uint32))
    assert out.view(np.uint32)[0] == POISON32 and (out.view(np.uint32)[n + 1:] == POISON32).all()


def test_add_full_benchmark_size(ctx):
    a, b = cf.inputs_c1()
    assert a.size == 16_777_259
    dc = rt.DeviceArray(a.shape, np.float32)
    rt.add_f32(dev(a), dev(b), dc)
    assert_array_equal(dc.to_host().view(np.uint32), cf.np_add(a, b).view(np.uint32))


def test_add_special_values(ctx):
    f = np.float32
    a = np.array([np.inf, -np.inf, np.inf, 1e-45, -0.0, 3e38, 1.0, 16777216.0], f)
    b = np.array([1.0, 1.0, -np.inf, 1e-45, 0.0, 3e38, 2.0 ** -24, 1.0], f)
    dc = rt.DeviceArray(a.shape, f)
    rt.add_f32(dev(a), dev(b), dc)
    with np.errstate(all="ignore"):
        want = a + b
    out = dc.to_host()
    assert_array_equal(np.isnan(out), np.isnan(want))
    ok = ~np.isnan(want)
    assert_array_equal(out[ok].view(np.uint32), want[ok].view(np.uint32))   # denormals kept


# ---------------------------------------------------------------------------
# W2 d = a * b + c (fp16 storage, fp32 arithmetic)
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("shape", [(1, 1), (3, 5), (1, 4099), (17, 4099), (129, 1031)])
def test_fma_bit_exact_all_variants(ctx, shape):
    a, b, c = cf.inputs_c2(shape)
    want = cf.np_fma_f16(a, b, c)
    assert_array_equal(want.view(np.uint16), co.fma_f16(a, b, c).view(np.uint16))
    da, db, dc = dev(a), dev(b), dev(c)
    for v in range(0, 13):                              # 0: the paced kernel, 8..12: other paces
        rt.set_variant("fma", v)
        dd = poisoned((shape[0] * shape[1] + 16,), np.float16)
        out_view = _View(dd, shape)
        rt.fma_f16(da, db, dc, out_view)
        out = dd.to_host()
        assert_array_equal(out[:want.size].view(np.uint16), want.ravel().view(np.uint16))
        assert (out[want.size:].view(np.uint16) == 0xA5A5).all(), (v, rt.last_kernel_name())


@pytest.mark.parametrize("cols,ld,off,kernel", [
    (1000, 1024, 0, "rows_v8"), (1003, 1024, 0, "rows_v8"), (1003, 1024, 8, "rows_v8"),
    (1001, 1028, 0, "rows_v4"), (1001, 1028, 4, "rows_v4"), (999, 1002, 0, "rows_v2"),
    (999, 1002, 2, "rows_v2"), (1000, 1001, 0, "2d"), (1000, 1024, 1, "2d"), (5, 1024, 0, "rows_v8")])
def test_fma_strided_rows(ctx, cols, ld, off, kernel):
    """Windows of larger arrays: the widest access the rows are aligned for, the
    leftover elements of a row one by one, nothing written outside the window."""
    rows = 33
    a, b, c = cf.inputs_c2((rows, ld + 1))
    flat = [x.ravel()[:rows * ld + 16].copy() for x in (a, b, c)]
    da, db, dc = (dev(x) for x in flat)
    dd = poisoned((rows * ld + 16,), np.float16)
    views = [_View(x, (rows, cols), off, (ld, 1)) for x in (da, db, dc, dd)]
    rt.fma_f16(*views)
    assert rt.last_kernel_name() == "hcamd_fma_f16_" + kernel
    win = [x[off:off + rows * ld].reshape(rows, ld)[:, :cols] for x in flat]
    raw = dd.to_host()
    out = raw[off:off + rows * ld].reshape(rows, ld)
    assert_array_equal(out[:, :cols].view(np.uint16), cf.np_fma_f16(*win).view(np.uint16))
    assert (out[:-1, cols:].view(np.uint16) == 0xA5A5).all()
    assert (raw[:off].view(np.uint16) == 0xA5A5).all()
    assert (raw[off + (rows - 1) * ld + cols:].view(np.uint16) == 0xA5A5).all()


def test_fma_special_values(ctx):
    h = np.float16
    a = np.array([[6e-8, 6e-8, 300, -300, 0.0, 1.0, 2.0 ** -14, 65504, 1.0]], h)
    b = np.array([[1.0, 0.5, 300, 300, -1.0, 1.0, 0.5, 1.0, 1.0]], h)
    c = np.array([[0.0, 0.0, 0.0, 0.0, 0.0, 2.0 ** -11, 0.0, 15.9, 2.0 ** -10]], h)
    dd = rt.DeviceArray(a.shape, h)
    rt.fma_f16(dev(a), dev(b), dev(c), dd)
    with np.errstate(over="ignore"):
        want = cf.np_fma_f16(a, b, c)
    assert_array_equal(dd.to_host().view(np.uint16), want.view(np.uint16))


def test_fma_full_benchmark_size(ctx):
    a, b, c = cf.inputs_c2()
    assert a.shape == (8191, 8193)
    dd = rt.DeviceArray(a.shape, np.float16)
    rt.fma_f16(dev(a), dev(b), dev(c), dd)
    assert rt.last_kernel_name().startswith("hcamd_fma_f16_v")
    assert_array_equal(dd.to_host().view(np.uint16), cf.np_fma_f16(a, b, c).view(np.uint16))


# ---------------------------------------------------------------------------
# pairwise distances
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("mnd", [(1, 1, 1), (5, 7, 3), (64, 64, 32), (65, 130, 33), (300, 200, 128),
                                 (1000, 1, 500)])
def test_pairwise_distances_against_fp64(ctx, mnd):
    m, n, d = mnd
    rng = np.random.default_rng(sum(mnd))
    a = rng.standard_normal((m, d)).astype(np.float32)
    b = rng.standard_normal((n, d)).astype(np.float32)
    out = poisoned((m + 3, n + 5), np.float32)
    rt.plan_pairwise_dist_f32(dev(a), dev(b), _View(out, (m, n), 0, (n + 5, 1))).launch(sync=True)
    got = out.to_host()
    want = np.sqrt(((a[:, None, :].astype(np.float64) - b[None, :, :]) ** 2).sum(axis=2))
    # d fused multiply-adds in fp32, then a correctly rounded square root
    assert_allclose(got[:m, :n], want, rtol=(d + 2) * 2.0 ** -24)
    p = poison_value(np.float32)
    assert (got[m:].view(np.uint32) == p.view(np.uint32)).all()
    assert (got[:, n:].view(np.uint32) == p.view(np.uint32)).all()
    # what NumPy itself computes in fp32 is equally close to the exact result
    ref32 = np.linalg.norm(a[:, None, :] - b[None, :, :], axis=2)
    assert_allclose(ref32, want, rtol=(d + 2) * 2.0 ** -24)


# ---------------------------------------------------------------------------
# product of gathered tiles
# ---------------------------------------------------------------------------
def _operand(arr_shape, starts, rows, cols, strides=None):
    if strides is None:
        strides = tuple(int(np.prod(arr_shape[d + 1:])) for d in range(len(arr_shape)))
    return (tuple(arr_shape), strides, np.asarray(starts, np.int64).reshape(-1, len(arr_shape)),
            np.asarray(rows, np.int64).reshape(-1, len(arr_shape)),
            np.asarray(cols, np.int64).reshape(-1, len(arr_shape)))


def _gather_reference(ops, n_groups, tm, tn, k, a, b, out):
    from test_kernel_frontend import TablesOnly
    t = TablesOnly(None, *ops, n_groups, tm, tn, k)
    t.run(a, b, out)
    return out


_GATHER_KERNELS = ([(v, 1) for v in range(7)] + [(v, 2) for v in range(5)] + [(0, 4), (1, 4), (0, 16), (1, 16)])


@pytest.mark.parametrize("variant,fuse", _GATHER_KERNELS)
@pytest.mark.parametrize("case", ["plain", "tails", "blocks", "transposed", "k0"])
def test_gathered_product_against_the_table_semantics(ctx, case, variant, fuse):
    """variant 0: block shape chosen by tile size; 1-6: every block shape
    (matrix-core and vector-ALU kernels) on every tile size; fuse: records per
    workgroup (runs of groups that read one b window, padded to a multiple)."""
    rt.set_variant("gather", variant)
    rt.set_variant("gather_fuse", fuse)
    rng = np.random.default_rng(len(case))
    # a[M, K] x b[K, N] walked by gm x gn groups of tm x tn tiles, written as tables
    M, N, K, tm, tn = {"plain": (64, 64, 32, 64, 64), "tails": (70, 45, 37, 16, 24),
                       "blocks": (150, 140, 70, 130, 70), "transposed": (33, 50, 19, 20, 20),
                       "k0": (9, 9, 0, 8, 8)}[case]
    gm, gn = -(-M // tm), -(-N // tn)
    a = rng.standard_normal((M, max(K, 1))).astype(np.float32)[:, :K]
    a = np.ascontiguousarray(a) if K else np.zeros((M, 1), np.float32)
    kk = max(K, 1)
    if case == "transposed":                       # b stored as [N, K], out as [N, M]
        b = rng.standard_normal((N, kk)).astype(np.float32)
        b_op = _operand(b.shape, [[gj * tn, 0] for gi in range(gm) for gj in range(gn)],
                        [[0, r] for r in range(K)], [[c, 0] for c in range(tn)])
        out_shape = (N, M)
        o_op = _operand(out_shape, [[gj * tn, gi * tm] for gi in range(gm) for gj in range(gn)],
                        [[0, r] for r in range(tm)], [[c, 0] for c in range(tn)])
    else:
        b = rng.standard_normal((kk, N)).astype(np.float32)
        b_op = _operand(b.shape, [[0, gj * tn] for gi in range(gm) for gj in range(gn)],
                        [[r, 0] for r in range(K)], [[0, c] for c in range(tn)])
        out_shape = (M, N)
        o_op = _operand(out_shape, [[gi * tm, gj * tn] for gi in range(gm) for gj in range(gn)],
                        [[r, 0] for r in range(tm)], [[0, c] for c in range(tn)])
    a_op = _operand(a.shape, [[gi * tm, 0] for gi in range(gm) for gj in range(gn)],
                    [[r, 0] for r in range(tm)], [[0, c] for c in range(K)])
    ops = (a_op, b_op, o_op)
    tables = rt.GatherGemm(ctx, *ops, gm * gn, tm, tn, K)
    out = poisoned(out_shape, np.float32)
    say("gather", case, variant, fuse, M, N, K, tm, tn)
    rt.plan_gather_gemm_f32(tables, dev(a), dev(b), out).launch(sync=True)
    assert rt.last_kernel_name().endswith(f"_g{fuse}")
    got = out.to_host()
    want = _gather_reference(ops, gm * gn, tm, tn, K, a, b, np.full(out_shape, np.nan, np.float32))
    assert not np.isnan(want).any()
    full = a[:, :K].astype(np.float64) @ (b[:, :K].T if case == "transposed" else b[:K]).astype(np.float64)
    assert_allclose(want, full.T if case == "transposed" else full, rtol=1e-6, atol=1e-6)
    assert_allclose(got, want, rtol=1e-5, atol=(K + 2) * 2.0 ** -22)


@pytest.mark.parametrize("fuse", [1, 2, 4, 16])
def test_gathered_product_inactive_elements_and_untouched_memory(ctx, fuse):
    """Windows that leave the buffer, negative and too-large indices, a start
    beyond the end: inactive operands count as zero, inactive outputs keep
    their bytes."""
    rng = np.random.default_rng(77)
    a = rng.standard_normal((3, 10, 7)).astype(np.float32)        # [batch, rows, k]
    b = rng.standard_normal((7, 12)).astype(np.float32)
    out_shape = (3, 12, 11)                                         # [batch, cols, rows + 1]
    tm, tn, k = 6, 8, 9
    rt.set_variant("gather_fuse", fuse)
    groups = [(g0, g1) for g0 in range(4) for g1 in range(2)]       # batch 3 does not exist
    a_op = _operand(a.shape, [[g0, 5 * g1, 0] for g0, g1 in groups],
                    [[0, r - 1, 0] for r in range(tm)],             # row -1 is inactive
                    [[0, 0, c] for c in range(k)])                  # k = 7, 8 are inactive
    b_op = _operand(b.shape, [[0, 0] for _ in groups], [[r, 0] for r in range(k)],
                    [[0, 2 * c] for c in range(tn)])                # every other column, 14 is inactive
    o_op = _operand(out_shape, [[g0, 0, 6 * g1] for g0, g1 in groups],      # row 11 is inactive
                    [[0, 0, r] for r in range(tm)], [[0, 11 - 2 * c, 0] for c in range(tn)])
    ops = (a_op, b_op, o_op)
    tables = rt.GatherGemm(ctx, *ops, len(groups), tm, tn, k)
    out = poisoned(out_shape, np.float32)
    rt.plan_gather_gemm_f32(tables, dev(a), dev(b), out).launch(sync=True)
    got = out.to_host()
    p = poison_value(np.float32)
    want = _gather_reference(ops, len(groups), tm, tn, k, a, b, np.full(out_shape, p, np.float32))
    written = want.view(np.uint32) != POISON32
    assert written.any() and not written.all()
    assert_array_equal(got.view(np.uint32)[~written], want.view(np.uint32)[~written])
    assert_allclose(got[written], want[written], rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("dtype", ["float16", "bfloat16"])
@pytest.mark.parametrize("fuse", [1, 2, 4, 16])
def test_gathered_product_on_16_bit_storage(ctx, dtype, fuse):
    """Elements are widened to fp32, multiplied and summed in fp32 and rounded
    once when stored: the result is the rounding of an fp32-accurate product."""
    rng = np.random.default_rng(fuse)
    M, N, K, tm, tn = 150, 140, 70, 40, 70
    gm, gn = -(-M // tm), -(-N // tn)

    def store(x):                                   # device array + the values it holds
        if dtype == "float16":
            h = x.astype(np.float16)
            return dev(h), h.astype(np.float32)
        bits = cf.f32_to_bf16_bits(x)
        return dev(bits, bf16=True), cf.bf16_bits_to_f32(bits)

    da, a = store(rng.standard_normal((M, K)).astype(np.float32))
    db, b = store(rng.standard_normal((K, N)).astype(np.float32))
    groups = [(gi, gj) for gi in range(gm) for gj in range(gn)]
    ops = (_operand(a.shape, [[gi * tm, 0] for gi, gj in groups], [[r, 0] for r in range(tm)],
                    [[0, c] for c in range(K)]),
           _operand(b.shape, [[0, gj * tn] for gi, gj in groups], [[r, 0] for r in range(K)],
                    [[0, c] for c in range(tn)]),
           _operand((M, N), [[gi * tm, gj * tn] for gi, gj in groups], [[r, 0] for r in range(tm)],
                    [[0, c] for c in range(tn)]))
    rt.set_variant("gather_fuse", fuse)
    tables = rt.GatherGemm(ctx, *ops, len(groups), tm, tn, K)
    out = rt.DeviceArray((M, N), np.float16 if dtype == "float16" else np.uint16, ctx,
                         dtype == "bfloat16").fill_bytes32(POISON32)
    rt.plan_gather_gemm(tables, da, db, out, dtype).launch(sync=True)
    assert rt.last_kernel_name().startswith(f"hcamd_gather_gemm_{'f16' if dtype == 'float16' else 'bf16'}_")
    raw = out.to_host()
    got = raw.astype(np.float32) if dtype == "float16" else cf.bf16_bits_to_f32(raw)
    want = a.astype(np.float64) @ b.astype(np.float64)
    # one rounding to 11 (fp16) or 8 (bf16) significant bits on top of the fp32 sum
    eps = 2.0 ** -11 if dtype == "float16" else 2.0 ** -8
    assert_allclose(got, want, rtol=1.01 * eps, atol=(K + 2) * 2.0 ** -22)
    with pytest.raises(rt.HcRuntimeError, match="element size"):
        rt.plan_gather_gemm(tables, da, db, out, "float32")


def test_gathered_product_rejects_bad_descriptions(ctx):
    ok = _operand((8, 8), [[0, 0]], [[r, 0] for r in range(4)], [[0, c] for c in range(4)])
    both = _operand((8, 8), [[0, 0]], [[r, r] for r in range(4)], [[0, c] for c in range(4)])
    neg = _operand((8, 8), [[-1, 0]], [[r, 0] for r in range(4)], [[0, c] for c in range(4)])
    big = ((1 << 20, 1 << 12), (1 << 12, 1), ok[2], ok[3], ok[4])
    for what, ops in {"both tile coordinates": (both, ok, ok), "negative window start": (ok, neg, ok),
                      "2\\^31": (ok, ok, big)}.items():
        with pytest.raises(rt.HcRuntimeError, match=what):
            rt.GatherGemm(ctx, *ops, 1, 4, 4, 4)
    with pytest.raises(rt.HcRuntimeError, match="invalid sizes"):
        rt.GatherGemm(ctx, ok, ok, ok, 0, 4, 4, 4)
    tables = rt.GatherGemm(ctx, ok, ok, ok, 1, 4, 4, 4)
    x = dev(np.zeros((8, 8), np.float32))
    with pytest.raises(rt.HcRuntimeError, match="built for"):
        rt.plan_gather_gemm_f32(tables, x, x, dev(np.zeros((8, 9), np.float32)))
    assert rt.hcamdGatherGemmLaunchF32(ctx.queue, tables.handle, x.ptr, None, x.ptr) == 1
    with pytest.raises(rt.HcRuntimeError, match="null pointer"):
        ctx.check(1, "hcamdGatherGemmLaunchF32")


# ---------------------------------------------------------------------------
# fused elementwise map (postfix programs)
# ---------------------------------------------------------------------------
def I(name, arg=0, imm=0.0):
    return (name, arg, imm)


def assert_same_floats(got, want, what=""):
    """Bit for bit, except that any NaN matches any NaN (an invalid operation
    yields a NaN whose sign differs between the host CPU and the GPU)."""
    assert got.dtype == want.dtype and got.shape == want.shape
    nan = np.isnan(want)
    assert_array_equal(np.isnan(got), nan, what)
    u = {2: np.uint16, 4: np.uint32}[got.dtype.itemsize]
    assert_array_equal(got.view(u)[~nan], want.view(u)[~nan], what)


FMA_PROGRAM = [I("in", 0), I("in", 1), I("mul"), I("in", 2), I("add")]


@pytest.mark.parametrize("shape", [(1, 1), (3, 5), (1, 4099), (17, 4099), (129, 1031)])
@pytest.mark.parametrize("variant", [0, 1])
def test_map_fma_program_equals_the_fma_kernel(ctx, shape, variant):
    a, b, c = cf.inputs_c2(shape)
    want = cf.np_fma_f16(a, b, c)
    rt.set_variant("map", variant)                      # 1: always the strided kernel
    d = poisoned(shape, np.float16)
    rt.plan_map(FMA_PROGRAM, [dev(a), dev(b), dev(c)], d).launch(sync=True)
    say("map", shape, rt.last_kernel_name())
    assert rt.last_kernel_name() == ("hcamd_map_flat" if variant == 0 else "hcamd_map_strided")
    assert_array_equal(d.to_host().view(np.uint16), want.view(np.uint16))
    assert_array_equal(want.view(np.uint16), co.fma_f16(a, b, c).view(np.uint16))


@pytest.mark.parametrize("n", [4096, 4097, 3 * 4096 + 4095, 1 << 20])
@pytest.mark.parametrize("types", [(np.float16,) * 5, (np.float32,) * 5,
                                   (np.float16, np.float32, np.float32, np.float16, np.float16),
                                   (np.float32, np.float16, np.float16, np.float32, np.float32)])
@pytest.mark.parametrize("n_in", [1, 2, 4])
def test_map_chains_equal_the_general_interpreter(ctx, n, types, n_in):
    """A program that never holds two values at once runs on the chain kernels
    (sixteen elements of a lane to a dispatch) on dense arrays: bit for bit what
    the general interpreter stores, the same elements left alone (zero divisors
    of the numpy.ma division, roots and logarithms outside their domain), and
    nothing written past the end."""
    rng = np.random.default_rng(n + n_in)
    ins = [rng.integers(-3, 4, n + 8).astype(np.float64) * 0.5 for _ in range(4)]
    program = [I("in", 0), I("mul_in", (1) % n_in), I("add_in", (2) % n_in), I("abs"), I("sqrt"),
               I("mdiv_in", (3) % n_in | (0x100 if types[4] == np.float16 else 0)), I("sub_in", 0), I("maxi", 0, -1.5),
               I("msqrt"), I("muli", 0, 0.5), I("rsubi", 0, 2.0), I("exp")]
    devs = [dev(x.astype(t)) for x, t in zip(ins, types)]
    views = [_View(d, (n,), 0, (1,)) for d in devs[:n_in]]
    got = {}
    for variant, prefix in ((0, "hcamd_map_chain_n"), (5, "hcamd_map_flat")):
        out = poisoned((n + 8,), types[4])
        rt.set_variant("map", variant)
        try:
            rt.plan_map(program, views, _View(out, (n,), 0, (1,))).launch(sync=True)
        finally:
            rt.set_variant("map", 0)
        assert rt.last_kernel_name().startswith(prefix), rt.last_kernel_name()
        if variant == 0:
            all_half = all(t == np.float16 for t in types[:n_in] + types[4:])
            assert rt.last_kernel_name() == f"hcamd_map_chain_n{2 if n_in <= 2 else 4}{'h' if all_half else ''}"
        got[variant] = out.to_host()
    bits = np.uint16 if types[4] == np.float16 else np.uint32
    assert_array_equal(got[0].view(bits), got[5].view(bits))
    p = poison_value(types[4])
    assert (got[0][n:].view(bits) == p.view(bits)).all()
    left_alone = got[0][:n].view(bits) == p.view(bits)
    assert left_alone.any() and not left_alone.all()


def test_map_window_of_larger_arrays_leaves_the_rest_untouched(ctx):
    rows, cols = 37, 1031
    a, b, c = cf.inputs_c2((rows, cols))
    big = [np.zeros((40, 1100), np.float16) for _ in range(3)]
    for dst, src in zip(big, (a, b, c)):
        dst[:rows, :cols] = src
    dbig = [dev(x) for x in big]
    out = poisoned((40, 1040), np.float16)
    views = [_View(x, (rows, cols), 0, (1100, 1)) for x in dbig]
    # fp16 rows that do not start on 16-byte boundaries: the row-program kernel
    # with interleaved lanes by default, the element-wise kernel as variant 1
    for variant, name in ((0, "hcamd_row_program_w64"), (1, "hcamd_map_strided")):
        rt.set_variant("map", variant)
        out = poisoned((40, 1040), np.float16)
        try:
            rt.plan_map(FMA_PROGRAM, views, _View(out, (rows, cols), 0, (1040, 1))).launch(sync=True)
        finally:
            rt.set_variant("map", 0)
        assert rt.last_kernel_name() == name
        got = out.to_host()
        assert_array_equal(got[:rows, :cols].view(np.uint16), cf.np_fma_f16(a, b, c).view(np.uint16))
        p = poison_value(np.float16)
        assert (got[rows:].view(np.uint16) == p.view(np.uint16)).all()
        assert (got[:, cols:].view(np.uint16) == p.view(np.uint16)).all()


@pytest.mark.parametrize("cols", [1, 5, 8, 9, 1031, 1032, 2049])
@pytest.mark.parametrize("types", [(np.float16,) * 4, (np.float32,) * 4,
                                   (np.float16, np.float32, np.float16, np.float32)])
def test_map_windows_with_aligned_rows_take_16_byte_accesses(ctx, cols, types):
    """Rows that start on 16-byte boundaries: the row kernel, bit for bit the
    element-wise kernel's results, nothing written outside the window, nothing
    read from outside it (the surroundings hold NaN)."""
    rows, ld = 37, 2064
    rng = np.random.default_rng(cols)
    ins = [rng.standard_normal((rows, cols)).astype(t) for t in types[:3]]
    big = [np.full((rows + 2, ld), np.nan, t) for t in types[:3]]
    for dst, src in zip(big, ins):
        dst[1:rows + 1, 8:8 + cols] = src
    dbig = [dev(x) for x in big]
    views = [_View(x, (rows, cols), ld + 8, (ld, 1)) for x in dbig]
    got = {}
    for variant in (0, 1):
        rt.set_variant("map", variant)
        out = poisoned((rows + 2, ld), types[3])
        rt.plan_map(FMA_PROGRAM, views, _View(out, (rows, cols), ld + 8, (ld, 1))).launch(sync=True)
        say("map window", cols, [np.dtype(t).name for t in types], rt.last_kernel_name())
        assert rt.last_kernel_name() == ("hcamd_map_rows" if variant == 0 else "hcamd_map_strided")
        got[variant] = out.to_host()
    rt.set_variant("map", 0)
    assert_array_equal(got[0].view(np.uint8), got[1].view(np.uint8))
    want = (ins[0].astype(np.float32) * ins[1].astype(np.float32)
            + ins[2].astype(np.float32)).astype(types[3])
    assert_same_floats(np.ascontiguousarray(got[0][1:rows + 1, 8:8 + cols]), want)
    mask = np.ones((rows + 2, ld), bool)
    mask[1:rows + 1, 8:8 + cols] = False
    p = poison_value(types[3])
    u = {2: np.uint16, 4: np.uint32}[np.dtype(types[3]).itemsize]
    assert (got[0].view(u)[mask] == p.view(u)).all()


@pytest.mark.parametrize("rows,cols", [(2, 3), (37, 1031), (5000, 40), (3, 70_001)])
def test_map_sum_over_windows_with_aligned_rows(ctx, rows, cols):
    ld = (cols + 8 + 7) // 8 * 8
    rng = np.random.default_rng(rows)
    a = rng.standard_normal((rows, cols)).astype(np.float16)
    b = rng.standard_normal((rows, cols)).astype(np.float32)
    big_a, big_b = np.full((rows, ld), np.nan, np.float16), np.full((rows, ld), np.nan, np.float32)
    big_a[:, 8:8 + cols], big_b[:, 4:4 + cols] = a, b
    terms = (a.astype(np.float32) * b).astype(np.float64)
    bound = 64 * 2.0 ** -24 * np.abs(terms).sum()
    da, db = dev(big_a), dev(big_b)
    views = [_View(da, (rows, cols), 8, (ld, 1)), _View(db, (rows, cols), 4, (ld, 1))]
    for variant, name in ((0, "hcamd_map_sum_rows"), (1, "hcamd_map_sum_strided")):
        rt.set_variant("map", variant)
        cell = dev(np.array([3.0, 0.0], np.float32))
        rt.plan_map_sum([I("in", 0), I("mul_in", 1)], views, cell).launch(sync=True)
        assert rt.last_kernel_name() == name
        got = cell.to_host()
        assert got[1] == 0.0 and abs(float(got[0]) - 3.0 - terms.sum()) <= bound + 3.0 * 2.0 ** -23
    rt.set_variant("map", 0)


def test_map_every_operation_against_numpy(ctx):
    rng = np.random.default_rng(11)
    n = 50_001
    f = np.float32
    x = rng.uniform(0.5, 2.0, n).astype(f) * rng.choice([-1, 1], n).astype(f)
    y = rng.uniform(0.5, 2.0, n).astype(f) * rng.choice([-1, 1], n).astype(f)
    x[:4] = [np.nan, 1.0, np.inf, -0.0]
    y[:4] = [1.0, np.nan, -np.inf, 1.0]
    dx, dy = dev(x), dev(y)
    k = f(0.75)
    exact = {
        "add": x + y, "sub": x - y, "mul": x * y, "div": x / y,
        "max": np.maximum(x, y), "min": np.minimum(x, y), "rsub": y - x, "rdiv": y / x,
    }
    with np.errstate(all="ignore"):
        for name, want in exact.items():
            out = poisoned((n,), f)
            rt.plan_map([I("in", 0), I("in", 1), I(name)], [dx, dy], out).launch(sync=True)
            assert_same_floats(out.to_host(), want.astype(f), name)
        for name, want in exact.items():                 # operand forms of the same
            out = poisoned((n,), f)
            rt.plan_map([I("in", 0), I(name + "_in", 1)], [dx, dy], out).launch(sync=True)
            assert_same_floats(out.to_host(), want.astype(f), name + "_in")
        imm = {"addi": x + k, "subi": x - k, "muli": x * k, "divi": x / k,
               "maxi": np.maximum(x, k), "mini": np.minimum(x, k), "rsubi": k - x,
               "rdivi": k / x}
        for name, want in imm.items():
            out = poisoned((n,), f)
            rt.plan_map([I("in", 0), I(name, 0, k)], [dx], out).launch(sync=True)
            assert_same_floats(out.to_host(), want.astype(f), name)
        unary = {"neg": -x, "abs": np.abs(x), "rint": np.rint(x * f(3)),
                 "r16": x.astype(np.float16).astype(f)}
        for name, want in unary.items():
            pre = [I("muli", 0, 3.0)] if name == "rint" else []
            out = poisoned((n,), f)
            rt.plan_map([I("in", 0)] + pre + [I(name)], [dx], out).launch(sync=True)
            assert_same_floats(out.to_host(), want, name)
        # correctly rounded square root, bit for bit
        out = poisoned((n,), f)
        rt.plan_map([I("in", 0), I("abs"), I("sqrt")], [dx], out).launch(sync=True)
        assert_same_floats(out.to_host(), np.sqrt(np.abs(x)), "sqrt")
        # transcendental functions: within 2 ulp of NumPy's fp32 results
        for name, fn, arg in (("exp", np.exp, x), ("log", np.log, np.abs(x)), ("tanh", np.tanh, x)):
            out = poisoned((n,), f)
            pre = [I("abs")] if name == "log" else []
            rt.plan_map([I("in", 0)] + pre + [I(name)], [dx], out).launch(sync=True)
            got, want = out.to_host(), fn(arg).astype(f)
            ok = np.isfinite(want)
            assert_array_equal(np.isnan(got), np.isnan(want), name)
            assert_allclose(got[ok], want[ok], rtol=3e-7, atol=1e-45, err_msg=name)
    # a constant pushed on the stack, and the deepest legal stack
    out = poisoned((n,), f)
    rt.plan_map([I("const", 0, 2.0), I("in", 0), I("const", 0, 3.0), I("in", 1), I("mul"),
                 I("add"), I("mul")], [dx, dy], out).launch(sync=True)
    with np.errstate(all="ignore"):
        assert_same_floats(out.to_host(), f(2) * (x + f(3) * y), "stack")


def test_map_no_contraction_two_roundings_in_fp32(ctx):
    # a*b+c where the fused result differs from the twice-rounded one
    rng = np.random.default_rng(12)
    n = 1 << 20
    a, b, c = (rng.standard_normal(n).astype(np.float32) for _ in range(3))
    want = a * b + c
    fused = (a.astype(np.float64) * b.astype(np.float64) + c.astype(np.float64)).astype(np.float32)
    assert (want != fused).any()                      # the inputs do tell the two apart
    out = poisoned((n,), np.float32)
    rt.plan_map(FMA_PROGRAM, [dev(a), dev(b), dev(c)], out).launch(sync=True)
    assert_array_equal(out.to_host().view(np.uint32), want.view(np.uint32))


def test_map_mixed_storage_types(ctx):
    rng = np.random.default_rng(13)
    shape = (33, 517)
    a = rng.standard_normal(shape).astype(np.float16)
    b = rng.standard_normal(shape).astype(np.float32)
    want32 = a.astype(np.float32) * b
    for out_dtype in (np.float32, np.float16):
        out = poisoned(shape, out_dtype)
        rt.plan_map([I("in", 0), I("in", 1), I("mul")], [dev(a), dev(b)], out).launch(sync=True)
        assert_array_equal(out.to_host(), want32.astype(out_dtype))


def test_map_rejects_malformed_programs(ctx):
    x = dev(np.ones(64, np.float32))
    out = poisoned((64,), np.float32)
    bad = {
        "underflow": [I("in", 0), I("add")],
        "leaves 2": [I("in", 0), I("in", 0)],
        "deeper": [I("in", 0)] * 5 + [I("add")] * 4,
        "operand 1": [I("in", 1)],
    }
    for what, prog in bad.items():
        with pytest.raises(rt.HcRuntimeError, match=what):
            rt.plan_map(prog, [x], out).launch(sync=True)
    with pytest.raises(rt.HcRuntimeError, match="instructions"):
        rt.plan_map([I("in", 0)] + [I("neg")] * 32, [x], out).launch(sync=True)
    prog = (rt.MapInstr * 1)()
    prog[0].op = 99
    ptrs, tys, lds = (C.c_void_p * 1)(x.ptr), (C.c_int * 1)(0), (C.c_size_t * 1)(64)
    assert rt.hcamdLaunchMap(ctx.queue, prog, 1, ptrs, tys, lds, 1, out.ptr, 0, 64, 1, 64) == 1
    with pytest.raises(rt.HcRuntimeError, match="unknown opcode"):
        ctx.check(1, "hcamdLaunchMap")
    assert (out.to_host().view(np.uint32) == POISON32).all()      # nothing was launched
    # empty windows are not an error
    rt.plan_map([I("in", 0)], [_view(x, 0)], _view(out, 0)).launch(sync=True)


def test_map_sum_flat_strided_and_accumulation(ctx):
    rng = np.random.default_rng(14)
    shape = (37, 1031)
    a = rng.standard_normal(shape).astype(np.float16)
    b = rng.standard_normal(shape).astype(np.float32)
    terms = (a.astype(np.float32) * b).astype(np.float64)          # fp32 products
    bound = 64 * 2.0 ** -24 * np.abs(terms).sum()
    prog = [I("in", 0), I("mul_in", 1)]
    cell = dev(np.array([0.0, 10.0], np.float32))
    rt.plan_map_sum(prog, [dev(a), dev(b)], cell, 1).launch(sync=True)
    assert rt.last_kernel_name() == "hcamd_map_sum_flat_n2u2"
    got = cell.to_host()
    assert got[0] == 0.0 and abs(float(got[1]) - 10.0 - terms.sum()) <= bound
    # a window of larger arrays goes through the strided kernel; adds on top
    big_a, big_b = np.zeros((40, 1100), np.float16), np.zeros((40, 1100), np.float32)
    big_a[:37, :1031], big_b[:37, :1031] = a, b
    big_a[37:], big_b[:, 1031:] = 9.0, 9.0                          # must not be read as data
    da, db = dev(big_a), dev(big_b)
    views = [_View(da, shape, 0, (1100, 1)), _View(db, shape, 0, (1100, 1))]
    rt.plan_map_sum(prog, views, cell, 1).launch(sync=True)
    assert rt.last_kernel_name() == "hcamd_map_sum_strided"
    assert abs(float(cell.to_host()[1]) - 10.0 - 2 * terms.sum()) <= 2 * bound
    # constants survive the tail handling: sum(x * 0 + 1) counts the elements
    for n in (1, 5, 8, 4099, 70_001):
        x = dev(np.ones(n, np.float32))
        c = dev(np.zeros(1, np.float32))
        rt.plan_map_sum([I("in", 0), I("muli", 0, 0.0), I("addi", 0, 1.0)], [x], c).launch(sync=True)
        assert c.to_host()[0] == n
    with pytest.raises(rt.HcRuntimeError, match="underflow"):
        rt.plan_map_sum([I("add")], [da], cell).launch(sync=True)


@pytest.mark.parametrize("n", [1, 3, 4, 1023, 4096 * 4, 1_000_003, cf.C1_N])
def test_sum_and_dot_of_fp32_vectors_have_their_own_kernels(ctx, n):
    rng = np.random.default_rng(n)
    x = rng.standard_normal(n).astype(np.float32)
    y = rng.standard_normal(n).astype(np.float32)
    dx, dy = dev(x), dev(y)
    cases = {"hcamd_sum_f32": ([I("in", 0)], [dx], x.astype(np.float64)),
             "hcamd_dot_f32": ([I("in", 1), I("mul_in", 0)], [dx, dy], (x * y).astype(np.float64)),
             "hcamd_dot_f32 ": ([I("in", 0), I("mul_in", 0)], [dx], (x * x).astype(np.float64))}
    for kernel, (prog, ins, terms) in cases.items():
        bound = 64 * 2.0 ** -24 * np.abs(terms).sum()
        for variant, name in ((0, kernel.strip()), (2, None)):     # 2: the interpreter
            rt.set_variant("map", variant)
            cell = dev(np.array([7.0], np.float32))
            rt.plan_map_sum(prog, ins, cell).launch(sync=True)
            if name:
                assert rt.last_kernel_name() == name
            else:
                assert rt.last_kernel_name().startswith("hcamd_map_sum_flat")
            assert abs(float(cell.to_host()[0]) - 7.0 - terms.sum()) <= bound + 7.0 * 2.0 ** -23
    # a misaligned operand keeps the general kernel
    rt.set_variant("map", 0)
    if n > 8:
        cell = dev(np.zeros(1, np.float32))
        rt.plan_map_sum([I("in", 0)], [_view(dx, n - 1, 1)], cell).launch(sync=True)
        assert rt.last_kernel_name() == "hcamd_map_sum_strided"
        assert abs(float(cell.to_host()[0]) - x[1:].astype(np.float64).sum()) <= \
            64 * 2.0 ** -24 * np.abs(x).sum()


@pytest.mark.parametrize("n", [8, 2049, 8192 + 5, 3 * 8192 * 4 + 123])
def test_map_of_one_or_two_fp16_operands_takes_four_chunks_per_lane(ctx, n):
    """Dense fp16 maps with one or two operands: four chunks of 8 per lane in
    flight (hcamd_map_flat_n2u4h), bit for bit what one chunk per lane gives
    (variant 3 of "map") and what NumPy gives in fp32 rounded once; fewer than a
    chunk, a ragged tail, several workgroups."""
    rng = np.random.default_rng(n)
    x = rng.standard_normal(n).astype(np.float16)
    y = rng.standard_normal(n).astype(np.float16)
    dx, dy = dev(x), dev(y)
    x32, y32 = x.astype(np.float32), y.astype(np.float32)
    cases = {"one": ([I("in", 0), I("muli", 0, 2.5), I("addi", 0, 1.0)], [dx],
                     (x32 * np.float32(2.5) + np.float32(1.0)).astype(np.float16)),
             "two": ([I("in", 0), I("mul_in", 1), I("sub_in", 0)], [dx, dy],
                     (x32 * y32 - x32).astype(np.float16))}
    for name, (program, inputs, want) in cases.items():
        got = {}
        for variant in (0, 3):
            rt.set_variant("map", variant)
            out = poisoned((n,), np.float16)
            rt.plan_map(program, inputs, out).launch(sync=True)
            assert rt.last_kernel_name() == ("hcamd_map_flat_n2u4h" if variant == 0 else "hcamd_map_flat"), name
            got[variant] = out.to_host()
        rt.set_variant("map", 0)
        assert_array_equal(got[0].view(np.uint16), got[3].view(np.uint16), err_msg=name)
        assert_array_equal(got[0].view(np.uint16), want.view(np.uint16), err_msg=name)


@pytest.mark.parametrize("n", [8, 511, 512 * 3 + 8 * 7 + 3, 1 << 20])
@pytest.mark.parametrize("types", [(np.float32, np.float32, np.float32), (np.float16, np.float32, np.float16),
                                   (np.float16, np.float16, np.float32), (np.float32, np.float16, np.float32),
                                   (np.float32, np.float32, np.float16)])
def test_map_of_flat_arrays_of_mixed_types(ctx, n, types):
    """a * b + a over dense vectors of fp16 and fp32 in every combination (the
    kernel deals elements to lanes differently as soon as one of the three is
    fp32): bit for bit the fp32 arithmetic of NumPy, rounded once to the output's
    type; whole waves, a partial last wave, a ragged tail; and with every third
    divisor zero in a / b under numpy.ma's rule, the poison stays where the
    quotient is not finite."""
    ta, tb, to = types
    rng = np.random.default_rng(n)
    a = rng.standard_normal(n).astype(ta)
    b = rng.standard_normal(n).astype(tb)
    a32, b32 = a.astype(np.float32), b.astype(np.float32)
    out = poisoned((n,), to)
    rt.plan_map([I("in", 0), I("mul_in", 1), I("add_in", 0)], [dev(a), dev(b)], out).launch(sync=True)
    assert rt.last_kernel_name() == "hcamd_map_flat"
    want = (a32 * b32 + a32).astype(to)
    bits = np.uint32 if to == np.float32 else np.uint16
    assert_array_equal(out.to_host().view(bits), want.view(bits))
    b[::3] = 0
    b32 = b.astype(np.float32)
    out = poisoned((n,), to)
    rt.plan_map([I("in", 0), I("mdiv_in", 1 | (0x100 if to == np.float16 else 0))], [dev(a), dev(b)],
                out).launch(sync=True)
    got = out.to_host()
    with np.errstate(all="ignore"):
        q = (a32 / b32).astype(to)
    dead = ~np.isfinite(q.astype(np.float32))
    assert dead[::3].all()
    assert (got.view(bits)[dead] == poison_value(to).view(bits)).all()
    assert_array_equal(got.view(bits)[~dead], (q + np.float32(0) * a32.astype(to)).astype(to).view(bits)[~dead])


def test_map_full_benchmark_size_fma(ctx):
    a, b, c = cf.inputs_c2()
    d = rt.DeviceArray(a.shape, np.float16)
    rt.plan_map(FMA_PROGRAM, [dev(a), dev(b), dev(c)], d).launch(sync=True)
    assert rt.last_kernel_name() == "hcamd_map_flat"
    assert_array_equal(d.to_host().view(np.uint16), cf.np_fma_f16(a, b, c).view(np.uint16))


# ---------------------------------------------------------------------------
# W3 row softmax
# ---------------------------------------------------------------------------
SOFTMAX_RTOL = 1e-5      # the tolerance the task states for fp32 results
SOFTMAX_ATOL = 1e-9


@pytest.mark.parametrize("shape", [(1, 1), (5, 7), (33, 256), (7, 257), (64, 1000), (16, 1024),
                                   (8, 2048), (9, 4097), (12, 8192), (5, 8190), (3, 16384),
                                   (3, 12345), (2, 20000), (1030, 512), (4, 1001), (3, 2047),
                                   (2, 16383), (2, 16385), (3, 50257), (2, 131072)])
def test_softmax_against_both_oracles(ctx, shape):
    (x,) = cf.inputs_c3(shape)
    dy = poisoned(shape, np.float32)
    rt.softmax_f32(dev(x), dy)
    say("softmax", shape, rt.last_kernel_name())
    y = dy.to_host()
    assert_allclose(y, cf.np_softmax(x), rtol=SOFTMAX_RTOL, atol=SOFTMAX_ATOL)
    assert_allclose(y, co.softmax(x, f64=True), rtol=4e-6, atol=SOFTMAX_ATOL)
    assert_allclose(y.astype(np.float64).sum(1), 1.0, atol=2e-6)


def test_softmax_variants_and_strided_rows(ctx):
    rows, cols, ld = 19, 8192, 8200
    (x,) = cf.inputs_c3((rows, ld))
    want = cf.np_softmax(x[:, :cols])
    dx = dev(x)
    for v in (0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11):
        rt.set_variant("softmax", v)
        dy = poisoned((rows, ld), np.float32)
        rt.softmax_f32(_View(dx, (rows, cols), 0, (ld, 1)), _View(dy, (rows, cols), 0, (ld, 1)))
        say("softmax variant", v, rt.last_kernel_name())
        out = dy.to_host()
        assert_allclose(out[:, :cols], want, rtol=SOFTMAX_RTOL, atol=SOFTMAX_ATOL)
        assert (out[:, cols:].view(np.uint32) == POISON32).all()
    # unaligned base pointer -> register-resident kernel with 4-byte accesses
    rt.set_variant("softmax", 0)
    for width, kernel in ((1000, "hcamd_softmax_f32_s256_e4"), (8190, "hcamd_softmax_f32_s256_e32")):
        dy = poisoned((rows, ld), np.float32)
        rt.softmax_f32(_View(dx, (rows, width), 1, (ld, 1)), _View(dy, (rows, width), 1, (ld, 1)))
        assert rt.last_kernel_name() == kernel
        out = dy.to_host()
        assert_allclose(out[:, 1:1 + width], cf.np_softmax(x[:, 1:1 + width]), rtol=SOFTMAX_RTOL,
                        atol=SOFTMAX_ATOL)
        assert (out[:, 0].view(np.uint32) == POISON32).all()
        assert (out[:, 1 + width:].view(np.uint32) == POISON32).all()


@pytest.mark.parametrize("cols,variant", [(1024, 0), (8192, 0), (8192, 5), (8192, 11), (1023, 0), (8191, 0),
                                          (12345, 0), (20000, 0), (50257, 0), (70001, 0), (20000, 2), (8192, 1)])
def test_softmax_extreme_and_special_rows(ctx, cols, variant):
    f = np.float32
    x = np.zeros((6, cols), f)
    x[0, :] = 1.25                                   # constant row: exactly 1/cols
    x[1, :] = np.linspace(-80, 80, cols)             # wide range, tiny tails
    x[2, 5] = np.nan                                 # NaN anywhere -> NaN row
    x[3, 7] = np.inf                                 # +inf -> NaN row (inf - inf)
    x[4, :] = -np.inf                                # all -inf -> NaN row
    x[5, :] = -1e30
    x[5, 3] = 0.0                                    # one-hot
    dy = rt.DeviceArray(x.shape, f)
    rt.set_variant("softmax", variant)
    rt.softmax_f32(dev(x), dy)
    say("softmax special rows", cols, variant, rt.last_kernel_name())
    y = dy.to_host()
    assert_array_equal(y[0], np.full(cols, 1 / cols, f))
    with np.errstate(all="ignore"):
        want = cf.np_softmax(x)
    assert_allclose(y[1], want[1], rtol=SOFTMAX_RTOL, atol=1e-30)
    assert np.isnan(y[2]).all() and np.isnan(y[3]).all() and np.isnan(y[4]).all()
    assert np.isnan(want[2]).all() and np.isnan(want[3]).all() and np.isnan(want[4]).all()
    assert y[5, 3] == 1.0 and y[5].sum() == 1.0


@pytest.mark.parametrize("cols,variant", [(1000, 0), (4096, 0), (8192, 0), (8192, 5), (8192, 11), (4095, 0),
                                          (20001, 0), (40000, 0), (66000, 0)])
def test_softmax_rows_of_huge_magnitude(ctx, cols, variant):
    # a row's maximum may be far from 0: only differences matter
    f = np.float32
    rng = np.random.default_rng(cols)
    base = rng.standard_normal((8, cols)).astype(f)
    x = base.copy()
    x[0] += f(1e30)                 # absorbed: every element becomes the same 1e30
    x[1] = f(3e38)                  # constant, near the top of the range
    x[2] = -x[1]
    x[3] = base[3] * f(1e9)         # spread over +-4e9
    x[4] = base[4] + f(2.5e7)       # fp32 spacing 2 at this magnitude
    x[5] = base[5] - f(7e10)
    rt.set_variant("softmax", variant)
    dy = rt.DeviceArray(x.shape, f)
    rt.softmax_f32(dev(x), dy)
    say("softmax huge rows", cols, variant, rt.last_kernel_name())
    with np.errstate(all="ignore"):
        want = cf.np_softmax(x)
    assert np.isfinite(want).all()
    assert_allclose(dy.to_host(), want, rtol=SOFTMAX_RTOL, atol=1e-30)


def test_softmax_reference_test_input(ctx):
    # python/hckernel/tests/test_examples.py:322-335 (float64 there)
    m, n = 30, 25
    a = (2 * np.arange(m * n).reshape(m, n) / (m * n)).astype(np.float32)
    dy = rt.DeviceArray(a.shape, np.float32)
    rt.softmax_f32(dev(a), dy)
    assert_allclose(dy.to_host(), cf.np_softmax(a.astype(np.float64)), rtol=2e-6)


def test_softmax_full_benchmark_size(ctx):
    (x,) = cf.inputs_c3()
    assert x.shape == (4096, 8192)
    dy = rt.DeviceArray(x.shape, np.float32)
    rt.softmax_f32(dev(x), dy)
    assert rt.last_kernel_name() == "hcamd_softmax_f32_g1024_v2_full_nt"
    y = dy.to_host()
    assert_allclose(y, cf.np_softmax(x), rtol=SOFTMAX_RTOL, atol=SOFTMAX_ATOL)
    assert_allclose(y.astype(np.float64).sum(1), 1.0, atol=2e-6)
    assert_array_equal(y.argmax(1), x.argmax(1))


# ---------------------------------------------------------------------------
# W4 row absmax int8 quantisation
# ---------------------------------------------------------------------------
def run_quantize(x, ld=None):
    rows, cols = x.shape
    ld = ld or cols
    ldq = ld if ld == cols else (ld + 15) // 16 * 16
    xp = np.zeros((rows, ld), np.float16)
    xp[:, :cols] = x
    dq = poisoned((rows, ldq), np.int8)
    ds = poisoned((rows,), np.float32)
    dx = dev(xp)
    rt.quantize_f16_i8(_View(dx, (rows, cols), 0, (ld, 1)), _View(dq, (rows, cols), 0, (ldq, 1)), ds)
    q = dq.to_host()
    assert (q[:, cols:].view(np.uint8) == 0xA5).all(), "wrote past the row"
    return q[:, :cols], ds.to_host()


@pytest.mark.parametrize("shape", [(1, 1), (3, 15), (5, 16), (7, 1000), (33, 1024), (9, 2047),
                                   (64, 4096), (11, 4100), (6, 8192), (3, 16400), (2, 32768),
                                   (2, 40000), (1027, 64)])
def test_quantize_bit_exact(ctx, shape):
    (x,) = cf.inputs_c4(shape)
    q, s = run_quantize(x)
    say("quantize", shape, rt.last_kernel_name())
    q_np, s_np = cf.np_quantize(x)
    assert_array_equal(q, q_np)
    assert_array_equal(s.view(np.uint32), s_np.view(np.uint32))
    if x.size < 200_000:
        q_c, s_c = co.quantize(x)
        assert_array_equal(q, q_c)


@pytest.mark.parametrize("shape,ld,kernel", [
    ((64, 4096), None, "c256x2_w2_full_nt"), ((63, 4096), None, "c256x2_w2_nt"),
    ((7, 2056), None, "c256x2_w2_nt"), ((5, 3000), 3008, "c256x2_w2_nt"),
    ((1, 4096), None, "c256x2_w2_nt"), ((2, 4096), 4160, "c256x2_w2_full_nt"),
    ((9, 4088), 4096, "c256x2_w2_nt")])
def test_quantize_word_layout_kernel(ctx, shape, ld, kernel):
    """Rows of 2049..4096 columns (a multiple of 8) take the kernel that deals
    16-byte words to the lanes: whole and ragged widths, odd row counts, padded
    leading dimensions, zero / inf / NaN rows through its per-element path."""
    rows, cols = shape
    (x,) = cf.inputs_c4(shape)
    x[0, ::5] = 0
    if rows > 3:
        x[1] = 0
        x[2, cols - 1] = np.float16(np.inf)
        x[3, 17] = np.float16(np.nan)
    with np.errstate(all="ignore"):
        q_np, s_np = cf.np_quantize(x)
    q, s = run_quantize(x, ld)
    say("quantize words", shape, ld, rt.last_kernel_name())
    assert rt.last_kernel_name().endswith(kernel)
    assert_array_equal(q, q_np)
    assert_array_equal(s.view(np.uint32), s_np.view(np.uint32))
    if rows > 3:
        q_c, s_c = co.quantize(x)
        assert_array_equal(q, q_c)


@pytest.mark.parametrize("shape,ld,off,kernel", [
    ((37, 4100), None, 0, "s4_e8"), ((19, 1000), None, 0, "s4_e4"), ((7, 4088), None, 0, "c256x2_w2_nt"),
    ((5, 20004), None, 0, "s4_e32"), ((9, 4094), None, 0, "s2_e8"), ((6, 10002), None, 0, "s2_e32"), ((6, 6002), None, 0, "s2_e16"), ((6, 6001), None, 0, "s1_e32"),
    ((3, 30002), None, 0, "s2_e64"), ((11, 4095), None, 0, "s1_e16"), ((5, 15001), None, 0, "s1_e64"),
    ((4, 1), None, 0, "s1_e16"), ((4, 2), None, 0, "s2_e8"), ((4, 3), None, 0, "s1_e16"),
    ((8, 1003), 1004, 0, "s4_e4"), ((8, 1001), 1002, 0, "s2_e8"), ((8, 512), 520, 1, "s1_e16"),
    ((8, 512), 520, 2, "s2_e8"), ((8, 512), 520, 4, "s4_e4"), ((3, 20001), None, 0, "stream")])
def test_quantize_rows_that_are_not_16_byte_aligned(ctx, shape, ld, off, kernel):
    """Column counts, leading dimensions and base addresses that rule out 16-byte
    accesses: register-resident kernels with 8-, 4- or 2-byte loads, bit for bit
    like the aligned ones, nothing written outside the rows."""
    rows, cols = shape
    ld = ld or cols
    (x,) = cf.inputs_c4(shape)
    x[0, ::7] = 0                                        # some exact zeros
    if rows > 2:
        x[1] = 0                                         # an all-zero row
        x[2, cols // 2] = np.float16(np.inf) if cols > 1 else x[2, 0]
    xp = np.full((rows * ld + off + 8,), 7, np.float16)
    xv = xp[off:off + rows * ld].reshape(rows, ld)
    xv[:, :cols] = x
    dx = dev(xp)
    dq = poisoned((rows * ld + off + 8,), np.int8)
    ds = poisoned((rows,), np.float32)
    rt.quantize_f16_i8(_View(dx, (rows, cols), off, (ld, 1)), _View(dq, (rows, cols), off, (ld, 1)), ds)
    say("quantize unaligned", shape, ld, off, rt.last_kernel_name())
    assert rt.last_kernel_name().endswith(kernel)
    with np.errstate(all="ignore"):
        q_np, s_np = cf.np_quantize(x)
    raw = dq.to_host()
    got = raw[off:off + rows * ld].reshape(rows, ld)
    assert_array_equal(got[:, :cols], q_np)
    assert (got[:, cols:].view(np.uint8) == 0xA5).all()
    assert (raw[:off].view(np.uint8) == 0xA5).all() and (raw[off + rows * ld:].view(np.uint8) == 0xA5).all()
    assert_array_equal(ds.to_host().view(np.uint32), s_np.view(np.uint32))


def test_quantize_variants_and_strides(ctx):
    (x,) = cf.inputs_c4((301, 4096))
    q_np, s_np = cf.np_quantize(x)
    for v in range(0, 12):
        rt.set_variant("quantize", v)
        for ld in (4096, 4096 + 64):
            q, s = run_quantize(x, ld)
            say("quantize variant", v, ld, rt.last_kernel_name())
            assert_array_equal(q, q_np)
            assert_array_equal(s.view(np.uint32), s_np.view(np.uint32))


def test_quantize_every_fp16_value_against_many_scales(ctx):
    """Each row holds an absmax and 4095 arbitrary finite fp16 values below it,
    drawn from the bit patterns directly so that every exponent (subnormals
    included) and rounding position is hit; 4096 rows, 16.7 M quotients, bit for
    bit against the IEEE-division statement."""
    rng = np.random.default_rng(44)
    rows, cols = 4096, 4096
    amax_bits = rng.integers(1, 0x7C00, rows).astype(np.uint16)
    frac = rng.random((rows, cols))
    bits = (frac * (amax_bits[:, None].astype(np.float64) + 1)).astype(np.uint16)
    bits = np.minimum(bits, amax_bits[:, None])
    bits[:, 0] = amax_bits
    bits |= (rng.integers(0, 2, (rows, cols)).astype(np.uint16) << 15)
    x = bits.view(np.float16)
    q_np, s_np = cf.np_quantize(x)
    for v in (0, 2, 3):
        rt.set_variant("quantize", v)
        q, s = run_quantize(x)
        assert_array_equal(q, q_np)
        assert_array_equal(s.view(np.uint32), s_np.view(np.uint32))


def test_quantize_ties_and_special_rows(ctx):
    h = np.float16
    for e in (-3, 0, 2):
        ks = np.array([0, 1, 2, 3, 4, 125, 126], np.float32)
        x = (np.concatenate([ks + 0.5, -(ks + 0.5), [127.0]]) * 2.0 ** e).astype(h)[None, :]
        q, s = run_quantize(np.repeat(x, 3, 0))
        assert s[0] == np.float32(2.0 ** e)
        assert_array_equal(q[0], [0, 2, 2, 4, 4, 126, 126, 0, -2, -2, -4, -4, -126, -126, 127])
    rows = np.zeros((4, 64), h)
    rows[1, 3], rows[1, 5] = np.nan, 2.0
    rows[2, 0], rows[2, 1], rows[2, 2] = np.inf, 1.0, -np.inf
    rows[3, :3] = [6e-8, -6e-8, 3e-8]
    q, s = run_quantize(rows)
    q_np, s_np = cf.np_quantize(rows)
    assert s[0] == 0 and np.isnan(s[1]) and np.isinf(s[2])
    assert_array_equal(q, q_np)
    assert_array_equal(q[3, :3], [127, -127, 127])


def test_quantize_full_benchmark_size(ctx):
    (x,) = cf.inputs_c4()
    assert x.shape == (16384, 4096)
    q, s = run_quantize(x)
    q_np, s_np = cf.np_quantize(x)
    assert_array_equal(q, q_np)
    assert_array_equal(s.view(np.uint32), s_np.view(np.uint32))
    # size-independent property: dequantisation error is at most half a step
    # (plus the rounding of q * scale itself)
    err = np.abs(q.astype(np.float64) * s[:, None].astype(np.float64) - x.astype(np.float64))
    assert (err <= 0.5001 * s[:, None]).all()


# ---------------------------------------------------------------------------
# W5 GEMM
# ---------------------------------------------------------------------------
GEMM_RTOL = 1e-2


def run_gemm(ab, bb, ldc_pad=0):
    m, n = ab.shape[0], bb.shape[0]
    dc = poisoned((m, n + ldc_pad), np.uint16)
    rt.gemm_bf16(dev(ab), dev(bb), _View(dc, (m, n), 0, (n + ldc_pad, 1)))
    out = dc.to_host()
    if ldc_pad:
        assert (out[:, n:] == 0xA5A5).all()
    return out[:, :n]


@pytest.mark.parametrize("mnk", [(256, 256, 64), (256, 512, 128), (512, 256, 256), (128, 128, 64),
                                 (384, 128, 192), (33, 47, 96), (100, 200, 300), (1, 1, 1),
                                 (64, 64, 8), (257, 255, 130)])
def test_gemm_exact_integer_matrices_bit_for_bit(ctx, mnk):
    m, n, k = mnk
    rng = np.random.default_rng(m * 7 + n)
    a = rng.integers(-4, 5, (m, k)).astype(np.float32)
    bt = rng.integers(-4, 5, (n, k)).astype(np.float32)
    want = cf.f32_to_bf16_bits((a.astype(np.int64) @ bt.astype(np.int64).T).astype(np.float32))
    got = run_gemm(cf.f32_to_bf16_bits(a), cf.f32_to_bf16_bits(bt))
    say("gemm", mnk, rt.last_kernel_name())
    assert_array_equal(got, want)


@pytest.mark.parametrize("mnk", [(256, 256, 256), (512, 768, 1024), (128, 384, 512),
                                 (100, 200, 300), (77, 33, 4097)])
def test_gemm_random_within_tolerance(ctx, mnk):
    ab, bb = cf.inputs_c5(mnk)
    got = cf.bf16_bits_to_f32(run_gemm(ab, bb))
    want = cf.np_gemm_bf16(ab, bb, np.float32)
    sigma = 0.02 * 0.02 * np.sqrt(mnk[2])
    assert_allclose(got, want, rtol=GEMM_RTOL, atol=1e-2 * sigma)
    # the result is the fp64 product rounded to bf16, give or take one bf16 ulp
    exact = cf.np_gemm_bf16(ab, bb, np.float64)
    assert np.abs(got - exact).max() <= 2.0 ** -8 * np.abs(exact).max()
    if mnk[0] * mnk[1] * mnk[2] <= 256 ** 3:
        _, c32 = co.gemm_bf16(ab, bb)
        assert_allclose(got, c32, rtol=GEMM_RTOL, atol=1e-2 * sigma)


@pytest.mark.parametrize("mnk", [(256, 256, 128), (512, 256, 320), (128, 384, 192), (100, 70, 50),
                                 (256, 256, 64)])
def test_gemm_fp16_against_fp32_accumulation(ctx, mnk):
    m, n, k = mnk
    rng = np.random.default_rng(sum(mnk))
    a = (0.5 * rng.standard_normal((m, k))).astype(np.float16)
    bt = (0.5 * rng.standard_normal((n, k))).astype(np.float16)
    c = poisoned((m, n + 8), np.float16)
    rt.plan_gemm_f16(dev(a), dev(bt), _View(c, (m, n), 0, (n + 8, 1))).launch(sync=True)
    say("gemm f16", mnk, rt.last_kernel_name())
    got = c.to_host()
    want = a.astype(np.float32) @ bt.astype(np.float32).T
    # fp32 accumulation, one rounding to fp16 at the end
    assert_allclose(got[:, :n].astype(np.float32), want, rtol=2.0 ** -10, atol=2.0 ** -10 * np.sqrt(k) * 0.25)
    assert (got[:, n:].view(np.uint16) == poison_value(np.float16).view(np.uint16)).all()
    # small integers: every product and partial sum is exact, so the result is too
    ai = rng.integers(-3, 4, (m, k)).astype(np.float16)
    bi = rng.integers(-3, 4, (n, k)).astype(np.float16)
    c2 = rt.DeviceArray((m, n), np.float16)
    rt.plan_gemm_f16(dev(ai), dev(bi), c2).launch(sync=True)
    assert_array_equal(c2.to_host().astype(np.float32), ai.astype(np.float32) @ bi.astype(np.float32).T)


@pytest.mark.parametrize("half", [False, True])
@pytest.mark.parametrize("mnk", [(300, 200, 136), (257, 255, 72), (1000, 1000, 1000), (129, 640, 192),
                                 (1, 1, 128), (513, 7, 4096 + 8)])
def test_gemm_ragged_shapes_take_the_edge_kernel(ctx, mnk, half):
    """M and N off the tile, K a multiple of 8 only: rows past the end are never
    stored, the K chunks past the end are zeros, and the result equals the
    whole-tile kernel's arithmetic (fp32 accumulation, one rounding)."""
    m, n, k = mnk
    rng = np.random.default_rng(sum(mnk))
    a32 = (0.5 * rng.standard_normal((m, k))).astype(np.float32)
    b32 = (0.5 * rng.standard_normal((n, k))).astype(np.float32)
    pad = 3                                       # odd leading dimension of C: scalar stores
    if half:
        a, bt = a32.astype(np.float16), b32.astype(np.float16)
        c = poisoned((m + 2, n + pad), np.float16)
        rt.plan_gemm_f16(dev(a), dev(bt), _View(c, (m, n), 0, (n + pad, 1))).launch(sync=True)
        got = c.to_host().astype(np.float32)
        av, bv, eps = a.astype(np.float32), bt.astype(np.float32), 2.0 ** -10
    else:
        a, bt = cf.f32_to_bf16_bits(a32), cf.f32_to_bf16_bits(b32)
        c = rt.DeviceArray((m + 2, n + pad), np.uint16, ctx, True).fill_bytes32(POISON32)
        rt.plan_gemm_bf16(dev(a, bf16=True), dev(bt, bf16=True),
                          _View(c, (m, n), 0, (n + pad, 1))).launch(sync=True)
        got = cf.bf16_bits_to_f32(c.to_host())
        av, bv, eps = cf.bf16_bits_to_f32(a), cf.bf16_bits_to_f32(bt), 2.0 ** -7
    say("gemm ragged", mnk, half, rt.last_kernel_name())
    assert rt.last_kernel_name().endswith("_edge")
    want = av.astype(np.float64) @ bv.astype(np.float64).T
    assert_allclose(got[:m, :n], want, rtol=eps, atol=eps * np.sqrt(k) * 0.25)
    raw = c.to_host().view(np.uint16)
    assert (raw[m:] == (POISON32 & 0xFFFF)).all() and (raw[:, n:] == (POISON32 & 0xFFFF)).all()
    # the general kernel (variant 6) agrees to the last bit: same products, fp32 sums in
    # another order would differ, so compare within one rounding instead
    rt.set_variant("gemm", 6)
    if half:
        c2 = rt.DeviceArray((m, n), np.float16)
        rt.plan_gemm_f16(dev(a), dev(bt), c2).launch(sync=True)
        got2 = c2.to_host().astype(np.float32)
    else:
        c2 = rt.DeviceArray((m, n), np.uint16, ctx, True)
        rt.plan_gemm_bf16(dev(a, bf16=True), dev(bt, bf16=True), c2).launch(sync=True)
        got2 = cf.bf16_bits_to_f32(c2.to_host())
    assert rt.last_kernel_name().endswith("_general")
    assert_allclose(got[:m, :n], got2, rtol=2 * eps, atol=eps * np.sqrt(k) * 0.25)


def test_gemm_all_variants_and_padded_output(ctx):
    ab, bb = cf.inputs_c5((512, 512, 256))
    want = cf.np_gemm_bf16(ab, bb, np.float32)
    sigma = 0.02 * 0.02 * 16
    bits0 = None
    # (17..22, 26, 28, 29, 33 and 34 are measurement builds whose output is not the product; 30..32 exist with them only)
    for v in list(range(0, 17)) + [23, 24, 25, 27] + ([30, 31, 32] if rt.probes_built() else []):
        rt.set_variant("gemm", v)
        bits = run_gemm(ab, bb, ldc_pad=8)
        got = cf.bf16_bits_to_f32(bits)
        say("gemm variant", v, rt.last_kernel_name())
        assert_allclose(got, want, rtol=GEMM_RTOL, atol=1e-2 * sigma)
        if v == 0:
            bits0 = bits
        if v in (7, 14, 15, 16, 23, 24, 25, 27, 30, 31, 32):   # the same sums with other epilogues / priorities / load paths / orders
            assert_array_equal(bits, bits0)


def test_gemm_full_benchmark_size_and_linearity(ctx):
    ab, bb = cf.inputs_c5()
    assert ab.shape == (4096, 4096) and bb.shape == (4096, 4096)
    got_bits = run_gemm(ab, bb)
    assert rt.last_kernel_name().startswith("hcamd_gemm_bf16_p256x256")
    got = cf.bf16_bits_to_f32(got_bits)
    want = cf.np_gemm_bf16(ab, bb, np.float32)
    assert_allclose(got, want, rtol=GEMM_RTOL, atol=2.6e-4)
    # linearity: scaling A by 2 is exact in bf16 and in every partial sum
    a2 = cf.f32_to_bf16_bits(cf.bf16_bits_to_f32(ab) * np.float32(2))
    got2 = cf.bf16_bits_to_f32(run_gemm(a2, bb))
    assert_array_equal(got2, got * np.float32(2))
    # identity: A @ I = A exactly
    eye = cf.f32_to_bf16_bits(np.eye(4096, dtype=np.float32))
    # (compared as numbers: -0 * 1 + 0 * 0 + ... is +0)
    assert_array_equal(cf.bf16_bits_to_f32(run_gemm(ab, eye)), cf.bf16_bits_to_f32(ab))

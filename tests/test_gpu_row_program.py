"""Row programs (hcamdLaunchRowProgram) on the GPU against NumPy formulas.

Expected values are written as plain NumPy expressions in float64 (not as an
emulation of the stage programs), so a wrong stage order, a reduction that
misses elements, or a row scalar read from the wrong row fails them.  Sums are
compared within the fp32 bound of a sum of n terms; max/min and everything
after them within a few ulp of fp32.
"""
import sys

import numpy as np
import pytest
from numpy.testing import assert_allclose, assert_array_equal

from hc_amd import runtime as rt

pytestmark = pytest.mark.gpu

POISON32 = 0xA5A5A5A5


def I(name, arg=0, imm=0.0):
    return (name, arg, imm)


def say(*a):
    print(*a, file=sys.stderr, flush=True)


@pytest.fixture(scope="module")
def ctx():
    return rt.default_context("hip:0")


def poisoned(shape, dtype):
    return rt.DeviceArray(shape, dtype).fill_bytes32(POISON32)


class _View:
    def __init__(self, base, shape, offset_elems=0, strides=None):
        self.shape = tuple(shape)
        self.ctx = base.ctx
        item = base.dtype.itemsize
        self.__cuda_array_interface__ = {
            "shape": self.shape, "typestr": rt._TYPESTR[base.dtype.name],
            "data": (int(base.ptr) + offset_elems * item, False),
            "strides": None if strides is None else tuple(s * item for s in strides),
            "version": 2}


SOFTMAX = [("max", 0, [I("in", 0)]),
           ("sum", 1, [I("in", 0), I("sub_red", 0), I("exp")]),
           ("store", 0, [I("in", 0), I("sub_red", 0), I("exp"), I("div_red", 1)])]


def np_softmax(x):
    x = x.astype(np.float64)
    e = np.exp(x - x.max(axis=1, keepdims=True))
    return e / e.sum(axis=1, keepdims=True)


def kernel_for(cols, general=False):
    """The kernel hcamdLaunchRowProgram picks for dense, 16-byte aligned rows whose
    stages are all chains: a chain kernel for whole chunks up to 4096 of them (one,
    two or four chunks per lane of a wave, then four on 128 ... 1024 lanes), else the
    general one (a wave per row up to 4096 columns, else a workgroup)."""
    per_row = cols // 8
    if not general and cols % 8 == 0 and per_row <= 4096:
        p = 1 if per_row <= 64 else 2 if per_row <= 128 else 4
        lanes = 64
        while lanes * p < per_row:
            lanes *= 2
        return f"hcamd_row_program_chain_w{lanes}_p{p}"
    return "hcamd_row_program_w64" if cols <= 4096 else "hcamd_row_program_w256"


@pytest.fixture(params=[0, 1], ids=["chain", "general"])
def rows_variant(request):
    """Variant 1 of "rows" keeps every program on the general kernel."""
    rt.set_variant("rows", request.param)
    yield request.param
    rt.set_variant("rows", 0)


# cols: one wave per row, one workgroup per row, one and several chunks per lane,
# whole chunks and not; rows: fewer than the chain kernels' workgroups, and more
# (their workgroups then take several rows in turns, fetching the next row early)
@pytest.mark.parametrize("rows,cols", [(1, 1), (30, 25), (7, 8), (5, 512), (9, 513), (33, 2048),
                                       (17, 4099), (64, 8192), (3, 16384), (2, 16392), (2, 40_001),
                                       (4501, 512), (4203, 1000), (2051, 2048), (1101, 4096),
                                       (603, 8192), (301, 16384), (5, 32768), (300, 32768)])
def test_softmax_as_a_row_program(ctx, rows, cols, rows_variant):
    rng = np.random.default_rng(cols)
    x = (rng.standard_normal((rows, cols)) * 3).astype(np.float32)
    out = poisoned((rows, cols), np.float32)
    say("row program softmax", rows, cols, rows_variant)
    rt.plan_row_program(SOFTMAX, [rt.to_device(x)], out).launch(sync=True)
    say("  ", rt.last_kernel_name())
    assert rt.last_kernel_name() == kernel_for(cols, general=rows_variant == 1)
    assert_allclose(out.to_host(), np_softmax(x), rtol=1e-5, atol=1e-30)


@pytest.mark.parametrize("cols,dtype", [(300, np.float32), (1000, np.float16), (8192, np.float32),
                                        (4104, np.float16)])
def test_layer_normalisation_with_weight_and_bias_vectors(ctx, cols, dtype, rows_variant):
    rows = 50 if cols != 1000 else 4100      # 4100 rows of 1000: several rows to a workgroup, in turns
    rng = np.random.default_rng(cols)
    x = (rng.standard_normal((rows, cols)) * 2 + 0.5).astype(dtype)
    g = rng.standard_normal(cols).astype(np.float32)
    b = rng.standard_normal(cols).astype(np.float32)
    eps = 1e-5
    n = float(cols)
    stages = [
        ("sum", 0, [I("in", 0)]),
        ("scalar", 0, [I("red", 0), I("divi", 0, n)]),                                   # mean
        ("sum", 1, [I("in", 0), I("sub_red", 0), I("in", 0), I("sub_red", 0), I("mul")]),
        ("scalar", 1, [I("red", 1), I("divi", 0, n), I("addi", 0, eps), I("sqrt")]),     # std
        ("store", 0, [I("in", 0), I("sub_red", 0), I("div_red", 1), I("mul_in", 1), I("add_in", 2)]),
    ]
    out = poisoned((rows, cols), np.float32)
    rt.plan_row_program(stages, [rt.to_device(x), rt.to_device(g), rt.to_device(b)], out).launch(sync=True)
    assert rt.last_kernel_name() == kernel_for(cols, general=rows_variant == 1)   # `x x mul` is a chain too
    x64 = x.astype(np.float64)
    want = (x64 - x64.mean(axis=1, keepdims=True)) / np.sqrt(x64.var(axis=1, keepdims=True) + eps) * g + b
    assert_allclose(out.to_host(), want, rtol=2e-5, atol=2e-5)


def layer_norm_stages(n, eps):
    """The six stages the front-end emits for (x - mean) / sqrt(var + eps) * w + b
    written with mean and var along axis 1: the mean's division and the last one
    are numpy.ma's, the variance reads the sum of the centred squares as a value
    (0 where the mean, and with it every centred square, is deactivated)."""
    return [("sum", 0, [I("in", 0)]),
            ("scalar", 1, [I("red", 0), I("mdivi", 0, n)]),
            ("sum", 2, [I("in", 0), I("sub_red", 1), I("in", 0), I("sub_red", 1), I("mul")]),
            ("scalar", 3, [I("red0", 2), I("divi", 0, n)]),
            ("scalar", 4, [I("red", 3), I("addi", 0, eps), I("msqrt")]),
            ("store", 0, [I("in", 0), I("sub_red", 1), I("mdiv_red", 4), I("mul_in", 1), I("add_in", 2)])]


def layer_norm_kernel(cols, per_chunk=4):
    chunks = cols // per_chunk
    lpr = 64
    while lpr < 512 and lpr * 2 < chunks:
        lpr *= 2
    if chunks > 2048:
        lpr = 1024
    e = 1 if chunks <= 64 else 2
    while lpr * e < chunks:
        e *= 2
    return f"hcamd_layer_norm_f32_w{lpr}_e{e}"


# every kernel of the family, rows that leave lanes and chunk slots idle, more rows
# than a workgroup holds, a window of a wider array
@pytest.mark.parametrize("rows,cols,ld", [(33, 12, 12), (1001, 256, 256), (77, 300, 300), (515, 1000, 1008),
                                          (130, 2048, 2048), (67, 4096, 4100), (4096, 8192, 8192),
                                          (9, 8200, 8200), (5, 20_480, 20_480), (6, 32_768, 32_768)])
def test_layer_normalisation_as_the_front_end_writes_it_takes_its_own_kernel(ctx, rows, cols, ld):
    rng = np.random.default_rng(rows + cols)
    big = np.full((rows, ld), np.nan, np.float32)
    x = (rng.standard_normal((rows, cols)) * 2 + 0.5).astype(np.float32)
    if rows > 8:
        x[3, cols // 2] = np.inf       # the row's mean is not finite: numpy.ma stores nothing of it
        x[5] = 1.25                    # no variance: eps alone under the root
    big[:, :cols] = x
    dbig = rt.to_device(big)
    dx = _View(dbig, (rows, cols), 0, (ld, 1))
    g = rng.standard_normal(cols).astype(np.float32)
    b = rng.standard_normal(cols).astype(np.float32)
    dg, db = rt.to_device(g), rt.to_device(b)
    eps = 1e-5
    stages = layer_norm_stages(float(cols), eps)
    x64 = x.astype(np.float64)
    with np.errstate(invalid="ignore"):
        want = (x64 - x64.mean(axis=1, keepdims=True)) / np.sqrt(x64.var(axis=1, keepdims=True) + eps) * g + b
    stored = np.isfinite(want)
    results = {}
    say("layer norm", rows, cols, ld)
    for variant in (1, 2, 0):
        rt.set_variant("rows", variant)
        try:
            out = poisoned((rows, cols), np.float32)
            rt.plan_row_program(stages, [dx, dg, db], out).launch(sync=True)
            name = rt.last_kernel_name()
        finally:
            rt.set_variant("rows", 0)
        # (a program whose row scalars the data can deactivate: the general kernel, or its own)
        assert name == (layer_norm_kernel(cols) if variant == 0 else kernel_for(cols, general=True))
        got = out.to_host()
        assert_allclose(got[stored], want[stored], rtol=2e-5, atol=2e-5)
        assert (got[~stored].view(np.uint32) == POISON32).all()
        results[variant] = got
    # the same operations per element: only the order of a row's sums differs
    assert_allclose(results[0][stored], results[2][stored], rtol=3e-6, atol=3e-6)


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("rows,cols,ld", [(33, 24, 24), (77, 304, 304), (515, 1000, 1008), (4096, 8192, 8192),
                                          (9, 8200, 8200), (6, 32_768, 32_768)])
def test_rms_normalisation_as_the_front_end_writes_it_takes_its_own_kernel(ctx, rows, cols, ld, dtype):
    """x / sqrt(mean(x * x) + eps) * w in the three stages the front-end emits, on
    fp32 rows and on fp16 rows (computed in fp32, stored as fp16: the program then
    ends in r16)."""
    half = dtype == np.float16
    rng = np.random.default_rng(rows + cols)
    big = np.full((rows, ld), np.nan, dtype)
    x = (rng.standard_normal((rows, cols)) * 2 + 0.5).astype(dtype)
    if rows > 8:
        x[3, cols // 2] = np.inf       # the mean of the squares is not finite: numpy.ma stores nothing of the row
        x[5] = 0.0
    big[:, :cols] = x
    dbig = rt.to_device(big)
    dx = _View(dbig, (rows, cols), 0, (ld, 1))
    g = rng.standard_normal(cols).astype(np.float32)
    dg = rt.to_device(g)
    eps = 1e-6
    stages = [("sum", 0, [I("in", 0), I("mul_in", 0)]),
              ("scalar", 1, [I("red", 0), I("mdivi", 0, float(cols)), I("addi", 0, eps), I("msqrt")]),
              ("store", 0, [I("in", 0), I("mdiv_red", 1), I("mul_in", 1)] + ([I("r16")] if half else []))]
    x64 = x.astype(np.float64)
    with np.errstate(invalid="ignore", over="ignore"):
        q = x64 / np.sqrt((x64 * x64).mean(axis=1, keepdims=True) + eps)
        want = q * g
    stored = np.isfinite(q) & np.isfinite((x64 * x64).mean(axis=1, keepdims=True))
    tol = dict(rtol=1.1e-3, atol=1e-4) if half else dict(rtol=2e-5, atol=2e-5)
    results = {}
    for variant in (1, 2, 0):
        rt.set_variant("rows", variant)
        try:
            out = poisoned((rows, cols), dtype)
            rt.plan_row_program(stages, [dx, dg], out).launch(sync=True)
            name = rt.last_kernel_name()
        finally:
            rt.set_variant("rows", 0)
        own = layer_norm_kernel(cols, 8 if half else 4).replace("layer", "rms").replace("f32", "f16" if half else "f32")
        assert name == (own if variant == 0 else kernel_for(cols, general=True))
        got = out.to_host()
        assert_allclose(got[stored].astype(np.float64), want[stored], **tol)
        raw = got.view(np.uint16 if half else np.uint32)
        assert (raw[~stored] == (POISON32 & 0xFFFF if half else POISON32)).all()
        results[variant] = got.astype(np.float64)
    assert_allclose(results[0][stored], results[2][stored], **(dict(rtol=1e-3, atol=1e-4) if half else
                                                               dict(rtol=3e-6, atol=3e-6)))


def test_rms_normalisation_divides_exactly_where_quotients_leave_the_normal_range(ctx):
    """The normalisation kernels divide by the row's scale through one
    double-precision reciprocal and go the long way for quotients below the
    normal range, where that shortcut can break a tie the wrong way.  Rows built
    so that the scale is exactly 3 * 2^34 whatever the order of the sums (one
    element 3 * 2^40, every other square underflows to nothing), with elements
    3 * m * 2^-120 whose quotients m * 2^-154 need rounding to multiples of
    2^-149, half of them exact ties; zeros of both signs keep their sign.  Every
    kernel must store the IEEE quotient bit for bit."""
    rows, cols = 6, 4096
    m = np.arange(cols, dtype=np.float64)
    x = np.empty((rows, cols), np.float32)
    for r in range(rows):
        x[r] = (3.0 * (m * (2 * r + 1) % 4099) * 2.0 ** -120).astype(np.float32)
        x[r, 1::7] *= -1
        x[r, 5] = 0.0
        x[r, 6] = -0.0
        x[r, 0] = 3.0 * 2.0 ** 40
    s = np.float32(3.0 * 2.0 ** 34)
    assert np.sqrt((x.astype(np.float64) ** 2).sum(axis=1) / cols).astype(np.float32).tolist() == [float(s)] * rows
    want = x / s
    assert (np.abs(want[:, 1:]) < np.float32(1.17549435e-38)).all() and (want[:, 1:] != 0).sum() > rows * 4000
    # some quotients are exact ties between two subnormal numbers
    assert ((x[:, 1:].astype(np.float64) / float(s) / 2.0 ** -150) % 2 == 1).sum() > 100
    stages = [("sum", 0, [I("in", 0), I("mul_in", 0)]),
              ("scalar", 1, [I("red", 0), I("mdivi", 0, float(cols)), I("addi", 0, 0.0), I("msqrt")]),
              ("store", 0, [I("in", 0), I("mdiv_red", 1), I("mul_in", 1)])]
    dx, dg = rt.to_device(x), rt.to_device(np.ones(cols, np.float32))
    for variant in (1, 2, 0):
        rt.set_variant("rows", variant)
        try:
            out = poisoned((rows, cols), np.float32)
            rt.plan_row_program(stages, [dx, dg], out).launch(sync=True)
            name = rt.last_kernel_name()
        finally:
            rt.set_variant("rows", 0)
        assert name.startswith("hcamd_rms_norm_f32") == (variant == 0)
        assert_array_equal(out.to_host().view(np.uint32), want.view(np.uint32), err_msg=name)


@pytest.mark.parametrize("rows,cols", [(1000, 7), (129, 1031), (4, 70_001), (5000, 264), (1300, 3000)])
def test_row_sums_maxima_and_minima_as_per_row_results(ctx, rows, cols, rows_variant):
    rng = np.random.default_rng(rows)
    x = rng.standard_normal((rows, cols)).astype(np.float32)
    dx = rt.to_device(x)
    x64 = x.astype(np.float64)
    cases = {"sum": ((x64 * x64).sum(axis=1), [I("in", 0), I("mul_in", 0)]),
             "max": (x64.max(axis=1), [I("in", 0)]),
             "min": (np.abs(x64).min(axis=1), [I("in", 0), I("abs")])}
    for kind, (want, program) in cases.items():
        for shape in ((rows,), (rows, 1)):
            out = poisoned(shape, np.float32)
            rt.plan_row_program([(kind, 2, program), ("store_col", 0, [I("red", 2)])], [dx], out).launch(sync=True)
            got = out.to_host().reshape(rows)
            if kind == "sum":
                assert_allclose(got, want, rtol=0, atol=cols * 2.0 ** -24 * np.abs(x64 * x64).sum(axis=1).max())
            else:
                assert_array_equal(got, want.astype(np.float32))


@pytest.mark.parametrize("rows", [77, 4300])
def test_column_operands_fill_row_scalars_and_fp16_results_round_once(ctx, rows, rows_variant):
    cols = 1000
    rng = np.random.default_rng(5)
    q = rng.integers(-127, 128, (rows, cols)).astype(np.float16)
    scale = rng.uniform(0.01, 2.0, rows).astype(np.float32)
    shift = rng.standard_normal(rows).astype(np.float16)
    out = poisoned((rows, cols), np.float16)
    rt.plan_row_program([("store", 0, [I("in", 0), I("mul_red", 0), I("add_red", 1)])],
                        [rt.to_device(q)], out,
                        columns=[rt.to_device(scale), rt.to_device(shift)]).launch(sync=True)
    want = ((q.astype(np.float32) * scale[:, None]) + shift.astype(np.float32)[:, None]).astype(np.float16)
    assert_array_equal(out.to_host().view(np.uint16), want.view(np.uint16))


@pytest.mark.parametrize("cols", [1003, 1000])        # 1000: whole chunks, the chain kernel where rows are aligned
def test_windows_of_larger_arrays_and_untouched_surroundings(ctx, cols, rows_variant):
    rows = 19
    rng = np.random.default_rng(6)
    x = rng.standard_normal((rows, cols)).astype(np.float32)
    for ld, off in ((1024, 4), (1011, 3)):            # 16-byte aligned rows, and not
        big = np.full((rows + 2, ld), np.nan, np.float32)
        big[1:rows + 1, off:off + cols] = x
        dbig = rt.to_device(big)
        out = poisoned((rows + 2, ld), np.float32)
        rt.plan_row_program(SOFTMAX, [_View(dbig, (rows, cols), ld + off, (ld, 1))],
                            _View(out, (rows, cols), ld + off, (ld, 1))).launch(sync=True)
        got = out.to_host()
        assert_allclose(got[1:rows + 1, off:off + cols], np_softmax(x), rtol=1e-5)
        mask = np.ones(got.shape, bool)
        mask[1:rows + 1, off:off + cols] = False
        assert (got.view(np.uint32)[mask] == POISON32).all()


@pytest.mark.parametrize("cols,ld", [(7, 9), (513, 515), (1003, 1011), (5001, 5003), (70_001, 70_003)])
def test_fp16_rows_off_16_byte_boundaries_interleave_the_lanes(ctx, cols, ld):
    """Rows of fp16 that start on odd multiples of 2 bytes: columns are dealt to
    the lanes one by one (one pass and several, one wave per row and four).  A
    stored tile and a per-row sum, bit for bit / within the fp32 sum bound, and
    nothing touched outside the window."""
    rows = 11
    rng = np.random.default_rng(cols)
    x = rng.standard_normal((rows, cols)).astype(np.float16)
    y = rng.standard_normal((rows, cols)).astype(np.float16)
    bigs = []
    for src in (x, y):
        big = np.full((rows + 2, ld), np.nan, np.float16)
        big[1:rows + 1, 1:1 + cols] = src
        bigs.append(rt.to_device(big))
    views = [_View(b, (rows, cols), ld + 1, (ld, 1)) for b in bigs]
    out = poisoned((rows + 2, ld + 1), np.float16)
    tile = [I("in", 0), I("mul_in", 1), I("add_in", 0)]
    rt.plan_row_program([("store", 0, tile)], views,
                        _View(out, (rows, cols), ld + 2, (ld + 1, 1))).launch(sync=True)
    say("fp16 interleaved", cols, rt.last_kernel_name())
    x32, y32 = x.astype(np.float32), y.astype(np.float32)
    prod = x32 * y32                                   # fp32 arithmetic, one rounding at the store
    want = (prod + x32).astype(np.float16)
    flat = out.to_host().reshape(-1)
    starts = [(r + 1) * (ld + 1) + 1 for r in range(rows)]
    got = np.stack([flat[s0:s0 + cols] for s0 in starts])
    assert_array_equal(got.view(np.uint16), want.view(np.uint16))
    mask = np.ones(flat.shape, bool)
    for s0 in starts:
        mask[s0:s0 + cols] = False
    assert (flat.view(np.uint16)[mask] == (POISON32 & 0xFFFF)).all()
    sums = poisoned((rows,), np.float32)
    rt.plan_row_program([("sum", 0, [I("in", 0), I("mul_in", 1)]), ("store_col", 0, [I("red", 0)])],
                        views, sums).launch(sync=True)
    p64 = prod.astype(np.float64)
    assert_allclose(sums.to_host(), p64.sum(axis=1), rtol=0,
                    atol=cols * 2.0 ** -24 * np.abs(p64).sum(axis=1).max() + 1e-30)


def test_special_values_follow_numpy(ctx, rows_variant):
    x = np.zeros((6, 600), np.float32)
    x[0, 5] = np.nan                    # NaN reaches every result of its row only
    x[1, :] = -np.inf                   # exp(-inf - -inf) = NaN in NumPy too
    x[2, 7] = np.inf
    x[3, :] = 1e30
    x[4, 100] = -np.inf
    out = poisoned(x.shape, np.float32)
    rt.plan_row_program(SOFTMAX, [rt.to_device(x)], out).launch(sync=True)
    with np.errstate(all="ignore"):
        want = np_softmax(x)
    got = out.to_host()
    assert_array_equal(np.isnan(got), np.isnan(want))
    ok = ~np.isnan(want)
    assert_allclose(got[ok], want[ok], rtol=1e-5)


def test_malformed_programs_are_refused_before_anything_runs(ctx):
    x = rt.to_device(np.ones((4, 16), np.float32))
    out = poisoned((4, 16), np.float32)
    bad = {
        "before it is written": [("store", 0, [I("in", 0), I("sub_red", 3)])],
        "must store": [("sum", 0, [I("in", 0)])],
        "only the last": [("store", 0, [I("in", 0)]), ("store", 0, [I("in", 0)])],
        "scalar stages read none": [("scalar", 0, [I("in", 0)]), ("store", 0, [I("in", 0)])],
        "underflow": [("store", 0, [I("add")])],
        "leaves 2 values": [("store", 0, [I("in", 0), I("in", 0)])],
        "operand 1": [("store", 0, [I("in", 1)])],
    }
    for message, stages in bad.items():
        with pytest.raises(rt.HcRuntimeError, match=message):
            rt.plan_row_program(stages, [x], out).launch(sync=True)
    assert (out.to_host().view(np.uint32) == POISON32).all()
    with pytest.raises(rt.HcRuntimeError, match="shape mismatch"):
        rt.plan_row_program(SOFTMAX, [rt.to_device(np.ones((4, 17), np.float32))], out)


def test_numpy_ma_forms_and_partly_empty_lanes_on_the_chain_kernels(ctx, rows_variant):
    """x / (row sum of y * y) with rows whose sum is zero (numpy.ma leaves such a
    row as it was), the maximum of log(x) over the positive elements only, and a
    row length that leaves some lanes of the chain kernel with one chunk or none:
    both kernels against NumPy, including which elements are written."""
    rows, cols = 4200, 1112                       # 139 chunks: w128_p2 with 117 idle chunk slots
    rng = np.random.default_rng(9)
    x = rng.standard_normal((rows, cols)).astype(np.float32)
    y = rng.standard_normal((rows, cols)).astype(np.float32)
    y[::7] = 0.0
    dx, dy = rt.to_device(x), rt.to_device(y)
    out = poisoned((rows, cols), np.float32)
    rt.plan_row_program([("sum", 0, [I("in", 1), I("mul_in", 1)]),
                         ("store", 0, [I("in", 0), I("mdiv_red", 0)])], [dx, dy], out).launch(sync=True)
    assert rt.last_kernel_name() == kernel_for(cols, general=rows_variant == 1)
    got = out.to_host()
    s = (y.astype(np.float64) ** 2).sum(axis=1)
    dead = s == 0
    assert dead.sum() == 600
    assert (got[dead].view(np.uint32) == POISON32).all()
    assert_allclose(got[~dead], x[~dead] / s[~dead, None], rtol=3e-6)
    tops = poisoned((rows,), np.float32)
    rt.plan_row_program([("max", 0, [I("in", 0), I("mlog")]), ("store_col", 0, [I("red", 0)])],
                        [dx], tops).launch(sync=True)
    want = np.log(np.where(x > 0, x, np.float32(1e-30)).astype(np.float64)).max(axis=1)
    assert_allclose(tops.to_host(), want, rtol=2e-6, atol=1e-6)


def _every_chain_instruction():
    """One stored tile per instruction a chain may hold: `in(0)` followed by the
    instruction (operand 1 for the *_in forms, column 0 for the *_red forms), the
    numpy.ma forms with and without the fp16 flag, and a program that ends after
    a form that deactivates elements followed by more arithmetic."""
    progs = {}
    for name in ("neg", "abs", "sqrt", "rint", "exp", "log", "tanh", "r16", "clear", "powchk",
                 "msqrt", "mlog"):
        progs[name] = [I("in", 0), I(name)]
    for name in ("add", "sub", "mul", "div", "max", "min", "rsub", "rdiv"):
        progs[name + "_in"] = [I("in", 0), I(name + "_in", 1)]
        progs[name + "i"] = [I("in", 0), I(name + "i", 0, 0.75)]
        progs[name + "_red"] = [I("in", 0), I(name + "_red", 0)]
    for flag in (0, 0x100):
        tag = "_h" if flag else ""
        progs["mdivi" + tag] = [I("in", 0), I("mdivi", flag, 0.0)]           # every element deactivated
        progs["rmdivi" + tag] = [I("in", 0), I("rmdivi", flag, 2.0)]         # where x is 0
        progs["mdiv_in" + tag] = [I("in", 0), I("mdiv_in", 1 | flag)]
        progs["rmdiv_in" + tag] = [I("in", 0), I("rmdiv_in", 1 | flag)]
        progs["mdiv_red" + tag] = [I("in", 0), I("mdiv_red", flag)]
        progs["rmdiv_red" + tag] = [I("in", 0), I("rmdiv_red", flag)]
    progs["square"] = [I("in", 0), I("sub_red", 0), I("in", 0), I("sub_red", 0), I("mul")]
    progs["after_mask"] = [I("in", 1), I("rmdiv_in", 0), I("addi", 0, 1.0), I("msqrt"), I("mul_in", 1)]
    progs["const_first"] = [I("const", 0, 3.0), I("sub_in", 0), I("mlog"), I("clear")]
    return progs


@pytest.mark.parametrize("rows,cols,dtype", [(70, 512, np.float32), (300, 1000, np.float16),
                                             (50, 4096, np.float32), (9, 16384, np.float16)])
def test_every_instruction_of_a_chain_computes_what_the_general_kernel_computes(ctx, rows, cols, dtype):
    """Element-wise stages do the same arithmetic on both kernels: the stored tiles
    are equal bit for bit, including which elements the numpy.ma forms leave
    untouched, on one, two and four chunks per lane and both storage types."""
    rng = np.random.default_rng(rows)
    x = (rng.standard_normal((rows, cols)) * 3).astype(dtype)
    y = (rng.standard_normal((rows, cols)) * 3).astype(dtype)
    for a in (x, y):                                   # zeros, negatives are there; add specials
        a[::3, ::5] = 0
        a[1, 7], a[2, 9], a[3, 11] = np.inf, -np.inf, np.nan
    col = rng.standard_normal(rows).astype(np.float32)
    col[::4] = 0
    dx, dy, dcol = rt.to_device(x), rt.to_device(y), rt.to_device(col)
    for name, program in _every_chain_instruction().items():
        results = []
        for variant in (0, 1):
            rt.set_variant("rows", variant)
            out = poisoned((rows, cols), dtype)
            rt.plan_row_program([("store", 0, program)], [dx, dy], out, columns=[dcol]).launch(sync=True)
            assert rt.last_kernel_name() == kernel_for(cols, general=variant == 1), name
            results.append(out.to_host())
        rt.set_variant("rows", 0)
        bits = np.uint32 if dtype == np.float32 else np.uint16
        assert_array_equal(results[0].view(bits), results[1].view(bits), err_msg=name)

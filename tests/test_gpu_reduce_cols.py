"""Reductions along columns (hcamdLaunchMapReduceCols) on the GPU against NumPy.

Expected values are plain NumPy expressions in float64: sums are held to the
fp32 bound of a sum of `rows` terms, maxima and minima are exact, and what a
`post` program computes from them is held to a few ulp of fp32.
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


def sum_bound(terms64):
    """fp32 error bound of rounding the rows of `terms64` and adding them up in
    any order."""
    return (terms64.shape[0] + 1) * 2.0 ** -24 * np.abs(terms64).sum(axis=0) + 1e-30


def within(got, want, bound):
    err = np.abs(got.astype(np.float64) - want)
    worst = int(np.argmax(err - bound))
    assert (err <= bound).all(), (worst, got[worst], want[worst], err[worst], np.broadcast_to(bound, err.shape)[worst])


# one launch and several bands of rows, whole and ragged chunks of columns
SHAPES = [(1, 1), (5, 7), (100, 513), (4097, 1031), (8192, 64), (20_000, 24), (64, 70_001),
          (3000, 4096)]


@pytest.mark.parametrize("rows,cols", SHAPES)
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_sums_maxima_and_minima_of_expressions_down_the_columns(ctx, rows, cols, dtype):
    rng = np.random.default_rng(rows * 31 + cols)
    x = rng.standard_normal((rows, cols)).astype(dtype)
    y = rng.standard_normal((rows, cols)).astype(dtype)
    dx, dy = rt.to_device(x), rt.to_device(y)
    x64, y64 = x.astype(np.float64), y.astype(np.float64)
    say("reduce_cols", rows, cols, np.dtype(dtype).name)
    out = poisoned((cols + 8,), np.float32)
    res = _View(out, (cols,), 0)

    rt.plan_map_reduce_cols("sum", [I("in", 0), I("mul_in", 1)], [dx, dy], res).launch(sync=True)
    got = out.to_host()
    within(got[:cols], (x64 * y64).sum(axis=0), sum_bound(x64 * y64))
    assert (got[cols:].view(np.uint32) == POISON32).all()
    again = poisoned((cols + 8,), np.float32)
    rt.plan_map_reduce_cols("sum", [I("in", 0), I("mul_in", 1)], [dx, dy],
                            _View(again, (cols,), 0)).launch(sync=True)
    assert_array_equal(again.to_host()[:cols].view(np.uint32), got[:cols].view(np.uint32))

    rt.plan_map_reduce_cols("max", [I("in", 0), I("abs")], [dx], res).launch(sync=True)
    assert_array_equal(out.to_host()[:cols], np.abs(x).max(axis=0).astype(np.float32))
    rt.plan_map_reduce_cols("min", [I("in", 0), I("sub_in", 1)], [dx, dy], res).launch(sync=True)
    want = (x.astype(np.float32) - y.astype(np.float32)).min(axis=0)
    assert_array_equal(out.to_host()[:cols], want)

    # the mean: the division runs on the folded value
    rt.plan_map_reduce_cols("sum", [I("in", 0)], [dx], res, post=[I("in", 0), I("divi", 0, rows)]
                            ).launch(sync=True)
    within(out.to_host()[:cols], x64.mean(axis=0), sum_bound(x64) / rows + 1e-6 * np.abs(x64.mean(axis=0)))


@pytest.mark.parametrize("ld,off", [(1040, 8), (1037, 3)])
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_windows_of_larger_arrays_vectors_and_fp16_results(ctx, ld, off, dtype):
    """Rows on and off 16-byte boundaries, NaN around the window, a vector that
    every row uses, a square root of the folded value as an fp16 result."""
    rows, cols = 777, 1001
    rng = np.random.default_rng(ld)
    x = rng.standard_normal((rows, cols)).astype(dtype)
    v = rng.standard_normal(cols).astype(np.float32)
    big = np.full((rows + 2, ld), np.nan, dtype)
    big[1:rows + 1, off:off + cols] = x
    dbig, dv = rt.to_device(big), rt.to_device(v)
    out = poisoned((cols + 9,), np.float16)
    rt.plan_map_reduce_cols("sum", [I("in", 0), I("sub_in", 1), I("abs")],
                            [_View(dbig, (rows, cols), ld + off, (ld, 1)), dv],
                            _View(out, (cols,), 1), post=[I("in", 0), I("sqrt")]).launch(sync=True)
    got = out.to_host()
    d = x.astype(np.float32) - v
    want = np.sqrt(np.abs(d.astype(np.float64)).sum(axis=0))
    assert_allclose(got[1:cols + 1].astype(np.float64), want, rtol=2.0 ** -11 + 1e-5)
    assert (got[:1].view(np.uint16) == POISON32 & 0xFFFF).all()
    assert (got[cols + 1:].view(np.uint16) == POISON32 & 0xFFFF).all()


# rows that fill the turns of the waves and rows that do not,
# column counts on and off the 256 columns of a wave, a window of a wider array
@pytest.mark.parametrize("rows,cols,ld", [(4096, 8192, 8192), (4100, 256, 256), (1031, 264, 272),
                                          (2999, 1000, 1000), (517, 4096, 4104), (70_000, 256, 256)])
def test_sum_and_sum_of_squares_of_a_dense_fp32_window_take_their_own_kernel(ctx, rows, cols, ld):
    rng = np.random.default_rng(rows + cols)
    big = np.full((rows, ld), np.nan, np.float32)
    x = (rng.standard_normal((rows, cols)) + 0.25).astype(np.float32)
    big[:, :cols] = x
    dbig = rt.to_device(big)
    dx = _View(dbig, (rows, cols), 0, (ld, 1))
    x64 = x.astype(np.float64)
    sq64 = (x * x).astype(np.float64)  # the product is rounded to fp32 before it is added
    say("cols_sum", rows, cols, ld)
    programs = {"sum": ([I("in", 0)], x64), "sumsq": ([I("in", 0), I("in", 0), I("mul")], sq64),
                "sumsq2": ([I("in", 0), I("mul_in", 0)], sq64)}
    results = {}
    for variant in (1, 2, 0):
        rt.set_variant("cols", variant)
        try:
            for name, (prog, terms) in programs.items():
                out = poisoned((cols + 8,), np.float32)
                rt.plan_map_reduce_cols("sum", prog, [dx], _View(out, (cols,), 0),
                                        post=[I("in", 0), I("divi", 0, 2.0)]).launch(sync=True)
                kernel = rt.last_kernel_name()
                got = out.to_host()
                within(got[:cols], terms.sum(axis=0) / 2, sum_bound(terms) / 2)
                assert (got[cols:].view(np.uint32) == POISON32).all()
                results[variant, name] = got
                # the bands of a sum with such a post program fold on a kernel of their own
                assert kernel == ("hcamd_map_reduce_cols_n1u4" if variant == 1 else "hcamd_cols_fold_f32")
                if variant == 0:
                    again = poisoned((cols + 8,), np.float32)
                    rt.plan_map_reduce_cols("sum", prog, [dx], _View(again, (cols,), 0),
                                            post=[I("in", 0), I("divi", 0, 2.0)]).launch(sync=True)
                    assert_array_equal(again.to_host().view(np.uint32), got.view(np.uint32))
        finally:
            rt.set_variant("cols", 0)
    assert_array_equal(results[0, "sumsq"].view(np.uint32), results[0, "sumsq2"].view(np.uint32))


def test_the_bands_of_a_sum_fold_with_every_simple_post_instruction(ctx):
    """The general kernel fills the bands (two operands, fp16), the fold kernel adds
    them up and runs the post program; variant 1 of "cols" runs the same on the
    general kernel alone, and the two agree bit for bit where the sums do."""
    rows, cols = 3000, 1028
    rng = np.random.default_rng(5)
    x = rng.standard_normal((rows, cols)).astype(np.float16)
    y = rng.standard_normal((rows, cols)).astype(np.float16)
    dx, dy = rt.to_device(x), rt.to_device(y)
    posts = {"none": [], "mean": [I("in", 0), I("divi", 0, rows)],
             "all": [I("in", 0), I("rsubi", 0, 2.0), I("abs"), I("sqrt"), I("rdivi", 0, 3.0)],
             "more": [I("in", 0), I("muli", 0, 0.5), I("subi", 0, 1.0), I("neg"), I("addi", 0, 0.25)],
             "long": [I("in", 0), I("abs"), I("sqrt"), I("abs"), I("sqrt"), I("neg")],     # five: the general kernel
             "other": [I("in", 0), I("exp")]}                                             # not simple: the general kernel
    for name, post in posts.items():
        got = {}
        for variant in (1, 0):
            rt.set_variant("cols", variant)
            try:
                out = poisoned((cols + 8,), np.float32)
                rt.plan_map_reduce_cols("sum", [I("in", 0), I("mul_in", 1)], [dx, dy], _View(out, (cols,), 0),
                                        post=post).launch(sync=True)
                kernel = rt.last_kernel_name()
            finally:
                rt.set_variant("cols", 0)
            simple = variant == 0 and name not in ("long", "other")
            assert kernel == ("hcamd_cols_fold_f32" if simple else "hcamd_map_reduce_cols_n1u4"), name
            got[variant] = out.to_host()
            assert (got[variant][cols:].view(np.uint32) == POISON32).all()
        # the bands are the same; the fold adds them in another order
        assert_allclose(got[0][:cols], got[1][:cols], rtol=2e-5, atol=1e-5, err_msg=name)
    terms = (x.astype(np.float32) * y.astype(np.float32)).astype(np.float64)
    rt.plan_map_reduce_cols("sum", [I("in", 0), I("mul_in", 1)], [dx, dy], _View(out, (cols,), 0),
                            post=posts["more"]).launch(sync=True)
    within(out.to_host()[:cols], -(terms.sum(axis=0) * 0.5 - 1.0) + 0.25, sum_bound(terms) + 1e-6)


def test_nan_and_infinities_follow_numpy(ctx):
    rows, cols = 300, 40
    x = np.random.default_rng(1).standard_normal((rows, cols)).astype(np.float32)
    x[17, 3] = np.nan
    x[250, 5] = np.inf
    x[0, 6] = -np.inf
    dx = rt.to_device(x)
    out = rt.DeviceArray((cols,), np.float32)
    with np.errstate(invalid="ignore"):
        for kind, want in (("max", x.max(axis=0)), ("min", x.min(axis=0)), ("sum", x.sum(axis=0))):
            rt.plan_map_reduce_cols(kind, [I("in", 0)], [dx], out).launch(sync=True)
            got = out.to_host()
            assert_array_equal(np.isnan(got), np.isnan(want))
            assert_array_equal(np.isinf(got), np.isinf(want))
            if kind != "sum":
                assert_array_equal(got[~np.isnan(want)], want[~np.isnan(want)])


def test_malformed_requests_are_refused_before_anything_runs(ctx):
    x = rt.to_device(np.ones((8, 8), np.float32))
    out = rt.DeviceArray((8,), np.float32)
    with pytest.raises(rt.HcRuntimeError, match="leaves 2 values"):
        rt.plan_map_reduce_cols("sum", [I("in", 0), I("in", 0)], [x], out).launch(sync=True)
    with pytest.raises(rt.HcRuntimeError, match="operand 1"):
        rt.plan_map_reduce_cols("sum", [I("in", 0)], [x], out,
                                post=[I("in", 1)]).launch(sync=True)
    # a window that needs bands of rows, launched without its workspace
    rows, cols = 100_000, 16
    big = rt.to_device(np.ones((rows, cols), np.float32))
    assert rt.hcamdMapReduceColsWorkspace(rows, cols) > 0
    p = rt.plan_map_reduce_cols("sum", [I("in", 0)], [big], rt.DeviceArray((cols,), np.float32))
    args = list(p.args)
    args[-2], args[-1] = None, 0
    with pytest.raises(rt.HcRuntimeError, match="workspace"):
        rt.Plan(ctx, p.fn, tuple(args), "hcamdLaunchMapReduceCols", p.keep).launch(sync=True)

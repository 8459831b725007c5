"""Small kernel bodies whose results follow from numpy.ma internals rather than
from any test or document of the reference simulator: in-place operators on
partially active tiles, loads from tiles that are already masked, domain
masking of divide / floordiv / mod / pow, NumPy functions applied to tiles,
compressed() / repr, Python scalars next to a tile, and the 19 binary + 4 unary
operators the simulator installs (python/hckernel/kernel_api.py:106-211).

Every case takes `api`, a namespace with the simulator's public names (`kernel`,
`sym`, `CurrentGroup`, ...), runs one or more kernels through it and returns a
flat dict name -> ndarray.  tests/golden/make_sim_golden.py runs them with the
reference's simulator and writes the results; tests/test_oracle_sim_golden.py
runs them with oracle.hcsim and compares.  This file holds inputs and recording
code only, no expected values.
"""

import operator
import warnings

import numpy as np

POISON = -77


def _text(s):
    return np.frombuffer(s.encode(), dtype=np.uint8).copy()


class Recorder:
    def __init__(self):
        self.out = {}

    def tile(self, name, t):
        """A tile: type tag, dtype, active flags, data where active."""
        try:
            has_mask = hasattr(t, "mask") and hasattr(t, "data") and not isinstance(t, np.ndarray)
        except AssertionError:
            # the reference's mask property cannot invert numpy.ma's scalar
            # "no mask" (kernel_api.py:93-103,117-119): such a tile cannot be
            # stored either, so there is no result to record
            self.out[name + ".raises"] = _text("AssertionError:mask")
            return
        if has_mask:
            m = np.asarray(t.mask)
            d = np.asarray(t.data)
            if m.shape != d.shape:              # numpy.ma's scalar "nomask"
                m = np.broadcast_to(m, d.shape)
            kind = "masked_array" if isinstance(t, np.ma.MaskedArray) else "tile"
            self.out[name + ".kind"] = _text(kind)
            self.out[name + ".active"] = m.astype(np.uint8)
            if kind == "masked_array":          # numpy.ma's own polarity: True = masked
                act = ~m
            else:
                act = m
            self.out[name + ".dtype"] = _text(str(d.dtype))
            self.out[name + ".value"] = np.where(act, d, np.zeros((), d.dtype))
        else:
            a = np.asarray(t)
            self.out[name + ".kind"] = _text("ndarray" if isinstance(t, np.ndarray) else type(t).__name__)
            self.out[name + ".dtype"] = _text(str(a.dtype))
            self.out[name + ".value"] = a

    def array(self, name, a):
        self.out[name] = np.asarray(a).copy()

    def attempt(self, name, fn):
        """Records fn()'s tile, or the name of the exception it raises."""
        try:
            t = fn()
        except Exception as e:                  # noqa: BLE001  the type is the datum
            self.out[name + ".raises"] = _text(type(e).__name__)
            return None
        self.tile(name, t)
        return None if name + ".raises" in self.out else t


def _one_group(api, body, *args, group=8):
    # The symbol parameter is there because the reference's launcher needs at
    # least one annotated parameter (kernel_sim.py:144-157).
    def entry(gr, n: api.sym.N, *rest):
        body(gr, *rest)

    api.kernel(work_shape=api.sym.N, group_shape=group)(entry)(group, *args)


def case_inplace_partial(api):
    rec = Recorder()
    x = np.arange(1, 9, dtype=np.float32)
    y = np.array([2, 0, 4, 0.5, -1, 3, 7, 9], dtype=np.float32)
    dst = np.full((4, 8), POISON, np.float32)

    def body(gr, x, y, dst):
        a = gr.load(x[:5], shape=8)             # 5 active
        b = gr.load(y[:3], shape=8)             # 3 active
        acc = gr.zeros(8, np.float32)           # all active
        acc += a
        rec.tile("full_plus_partial", acc)
        gr.store(dst[0], acc)
        acc2 = gr.load(x[:5], shape=8)
        acc2 += b
        rec.tile("partial_plus_narrower", acc2)
        acc2 *= b
        acc2 -= 1.5
        rec.tile("after_mul_sub", acc2)
        gr.store(dst[1], acc2)
        acc3 = gr.load(y[:3], shape=8)
        acc3 += a                               # wider operand: does activity grow?
        rec.tile("narrow_plus_wider", acc3)
        gr.store(dst[2], acc3)
        acc4 = gr.load(x[:6], shape=8)
        acc4 /= gr.load(y[:8], shape=8)         # y[1] == 0
        rec.tile("inplace_div_by_zero", acc4)
        gr.store(dst[3], acc4)

    with np.errstate(all="ignore"):
        _one_group(api, body, x, y, dst)
    rec.array("dst", dst)
    return rec.out


def case_load_from_masked(api):
    rec = Recorder()
    x = np.arange(18, dtype=np.int32).reshape(3, 6) + 1
    dst = np.full((2, 4, 4), POISON, np.int32)

    def body(gr, x, dst):
        t = gr.load(x, shape=(4, 8))            # 3 x 6 active
        rec.tile("outer", t)
        u = gr.load(t[:, 2:], shape=(4, 4))     # window of a masked tile
        rec.tile("load_window", u)
        gr.store(dst[0], u)
        v = gr.vload(t[1:, 4:], shape=(4, 4))   # source smaller than the request
        rec.tile("vload_window", v)
        gr.store(dst[1], v)
        rec.attempt("vec_of_tile", lambda: gr.vec(t, (2, 3)))
        rec.attempt("vec_whole", lambda: gr.vec(u))

    _one_group(api, body, x, dst)
    rec.array("dst", dst)
    return rec.out


def case_domain_masking(api):
    rec = Recorder()
    num = np.array([4, -9, 0, 7, 5, -3, 8, 1], dtype=np.float32)
    den = np.array([2, 0, 0, -2, 0.5, 3, 0, 4], dtype=np.float32)
    inum = np.array([7, -7, 0, 9, 5, -3, 8, 1], dtype=np.int32)
    iden = np.array([2, 0, 0, -2, 3, 3, 0, 4], dtype=np.int32)
    dst = np.full((8, 8), POISON, np.float32)
    idst = np.full((2, 8), POISON, np.int32)
    pdst = np.full(8, POISON, np.int32)

    def body(gr, num, den, inum, iden, dst, idst, pdst):
        a, b = gr.load(num, shape=8), gr.load(den[:7], shape=8)
        ia, ib = gr.load(inum, shape=8), gr.load(iden[:7], shape=8)
        for row, (name, fn) in enumerate([
                ("truediv", lambda: a / b),
                ("floordiv", lambda: a // b),
                ("mod", lambda: a % b),
                ("pow_half", lambda: a ** 0.5),
                ("pow_tile", lambda: a ** b),
                ("int_truediv", lambda: ia / ib)]):
            t = rec.attempt(name, fn)
            if t is not None:
                gr.store(dst[row], t)
        for row, (name, fn) in enumerate([
                ("int_floordiv", lambda: ia // ib),
                ("int_mod", lambda: ia % ib)]):
            t = rec.attempt(name, fn)
            if t is not None:
                gr.store(idst[row], t)
        t = rec.attempt("int_pow", lambda: ia ** 2)
        if t is not None:
            gr.store(pdst, t)
            rec.array("int_pow.dst", pdst)
        # NumPy functions see a tile through __array__
        for row, (name, fn) in enumerate([("np_sqrt", lambda: np.sqrt(a)),
                                           ("np_log", lambda: np.log(b))]):
            t = rec.attempt(name, fn)
            if t is not None:
                gr.store(dst[6 + row], t)

    with np.errstate(all="ignore"), warnings.catch_warnings():
        warnings.simplefilter("ignore")
        _one_group(api, body, num, den, inum, iden, dst, idst, pdst)
    rec.array("dst", dst)
    rec.array("idst", idst)
    return rec.out


def case_numpy_functions(api):
    rec = Recorder()
    rng = np.random.default_rng(7)
    x = rng.integers(-4, 5, (3, 5)).astype(np.float64)
    y = rng.integers(-4, 5, (5, 2)).astype(np.float64)
    dst = np.full((4, 4), POISON, np.float64)
    dsum = np.full((3, 4), POISON, np.float64)

    def body(gr, x, y, dst, dsum):
        a = gr.load(x, shape=(4, 6))            # 3 x 5 active of 4 x 6
        b = gr.load(y, shape=(6, 4))            # 5 x 2 active of 6 x 4
        rec.attempt("np_dot", lambda: np.dot(a, b))
        rec.attempt("matmul", lambda: a @ b)
        rec.attempt("norm_rows", lambda: np.linalg.norm(a, axis=-1))
        rec.attempt("np_exp", lambda: np.exp(a))
        rec.attempt("sum_all", lambda: a.sum())
        rec.attempt("max_all", lambda: a.max())
        rec.attempt("sum_rows", lambda: a.sum(axis=1))
        rec.attempt("max_cols", lambda: a.max(axis=0))
        rec.attempt("mean_cols", lambda: a.mean(axis=0))
        rec.attempt("astype", lambda: a.astype(np.float32))
        rec.attempt("reshape", lambda: a.reshape(6, 4))
        rec.attempt("transpose", lambda: a.T)
        rec.attempt("np_sum_function", lambda: np.sum(a))
        t = rec.attempt("acc_dot", lambda: _acc_dot(gr, a, b))
        if t is not None:
            gr.store(dst, t)
        for row, fn in enumerate([lambda: a.sum(axis=1), lambda: a.max(axis=1),
                                  lambda: a.min(axis=1)]):
            gr.store(dsum[row], fn())

    def _acc_dot(gr, a, b):
        r = gr.zeros((4, 4), np.float64)
        r += np.dot(a, b)
        return r

    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        _one_group(api, body, x, y, dst, dsum)
    rec.array("dst", dst)
    rec.array("dsum", dsum)
    return rec.out


def case_compressed_repr(api):
    rec = Recorder()
    x = np.arange(10, dtype=np.int64) * 3

    def body(gr, x):
        t = gr.load(x[2:7], shape=8)
        rec.array("compressed", t.compressed())
        rec.array("repr", _text(repr(t)))
        rec.array("str", _text(str(t)))
        e = gr.load(x[:0], shape=4)
        rec.array("compressed_empty", e.compressed())
        rec.array("repr_all_inactive", _text(repr(e)))
        z = gr.ones((2, 3), np.float32)
        rec.array("repr_all_active", _text(repr(z)))
        rec.array("shape", np.array(t.shape))
        rec.attempt("len", lambda: np.array(len(z)))

    _one_group(api, body, x)
    return rec.out


def case_scalar_promotion(api):
    rec = Recorder()
    xs = {"f32": np.array([1.5, -2.25, 3, 0.1, 7, 8, 9, 10], np.float32),
          "f16": np.array([1.5, -2.25, 3, 0.1, 7, 8, 9, 10], np.float16),
          "i32": np.array([1, -2, 3, 4, 7, 8, 9, 10], np.int32)}
    dst = {k: np.full((4, 8), POISON, v.dtype) for k, v in xs.items()}

    def body(gr, x, dst, tag):
        t = gr.load(x[:6], shape=8)
        for row, (name, fn) in enumerate([
                ("mul_pyfloat", lambda: t * 0.5),
                ("add_pyint", lambda: t + 1),
                ("mul_npf32", lambda: t * np.float32(0.5)),
                ("div_pyint", lambda: t / 2)]):
            r = rec.attempt(f"{tag}.{name}", fn)
            if r is not None:
                gr.store(dst[row], r)

    with np.errstate(all="ignore"):
        for tag, x in xs.items():
            _one_group(api, lambda gr, x, d, _t=tag: body(gr, x, d, _t), x, dst[tag])
    for tag in xs:
        rec.array(f"dst.{tag}", dst[tag])
    return rec.out


BINARY = ["add", "sub", "mul", "matmul", "truediv", "floordiv", "pow", "mod", "lt", "le",
          "eq", "ne", "ge", "gt", "and_", "or_", "xor", "rshift", "lshift"]
UNARY = ["abs", "neg", "not_", "inv"]


def case_operators(api):
    rec = Recorder()
    xs = {"i32": (np.array([5, -3, 12, 0, 7, -8, 9, 2], np.int32),
                  np.array([2, 3, 1, 4, 0, 2, 3, 1], np.int32)),
          "f32": (np.array([5.5, -3, 12, 0, 7, -8.25, 9, 2], np.float32),
                  np.array([2, 3, 0.5, 4, 0, 2, 3, 1], np.float32)),
          "bool": (np.array([1, 0, 1, 1, 0, 0, 1, 0], np.bool_),
                   np.array([1, 1, 0, 1, 0, 1, 0, 0], np.bool_))}

    def body(gr, x, y, tag):
        a = gr.load(x[:7], shape=8)
        b = gr.load(y[1:], shape=8)             # 7 elements, shifted by one
        for name in BINARY:
            op = getattr(operator, name)
            rec.attempt(f"{tag}.{name}", lambda: op(a, b))
            stem = name.rstrip("_")

            def inplace():
                c = gr.load(x[:7], shape=8)
                c = getattr(c, f"__i{stem}__")(b)
                return c

            rec.attempt(f"{tag}.i{stem}", inplace)
        for name in UNARY:
            # the simulator installs __not__ and __inv__ (kernel_api.py:180-201),
            # names the interpreter never looks up: the operator form and the
            # method called by name are different things
            stem = name.rstrip("_")
            rec.attempt(f"{tag}.{stem}.operator", lambda: getattr(operator, name)(a))
            rec.attempt(f"{tag}.{stem}.dunder", lambda: getattr(a, f"__{stem}__")())
        one = gr.load(x[2:3], shape=1)
        rec.attempt(f"{tag}.not_single.dunder", lambda: one.__not__())
        # operands on the left that are not tiles
        rec.attempt(f"{tag}.pyscalar_left_mul", lambda: 2 * a)
        rec.attempt(f"{tag}.pyscalar_left_sub", lambda: 2 - a)
        rec.attempt(f"{tag}.npscalar_left_mul", lambda: x.dtype.type(2) * a)
        rec.attempt(f"{tag}.ndarray_left_add", lambda: x + a)
        rec.attempt(f"{tag}.ndarray_right_add", lambda: a + x)

    with np.errstate(all="ignore"), warnings.catch_warnings():
        warnings.simplefilter("ignore")
        for tag, (x, y) in xs.items():
            _one_group(api, lambda gr, x, y, _t=tag: body(gr, x, y, _t), x, y)
    return rec.out


def case_store_forms(api):
    """Stores whose source is not a tile of the simulator: numpy.ma arrays that
    reductions return, plain arrays, scalars broadcast by a window."""
    rec = Recorder()
    x = (np.arange(24, dtype=np.float32).reshape(4, 6) - 7)
    dst = np.full((5, 4), POISON, np.float32)
    wide = np.full((2, 4, 8), POISON, np.float32)

    def body(gr, x, dst, wide):
        t = gr.load(x[:3, :5], shape=(4, 8))
        gr.store(dst[0], t.sum(axis=1))          # numpy.ma result, last row fully inactive
        gr.store(dst[1], t.max(axis=1))
        gr.store(dst[2], np.exp(t).sum(axis=1))  # plain ndarray: unconditional
        s = t - t.max(axis=1, keepdims=True)
        rec.tile("centred", s)
        gr.store(wide[0], s)
        e = np.exp(s)
        rec.tile("exp_of_centred", e)
        q = e / e.sum(axis=1, keepdims=True)
        rec.tile("normalised", q)
        gr.store(wide[1], q)
        gr.store(dst[3], gr.load(x[0, :2], shape=4) * 2)
        gr.store(dst[4, 1:], gr.load(x[1], shape=8))   # destination narrower than the tile

    with np.errstate(all="ignore"), warnings.catch_warnings():
        warnings.simplefilter("ignore")
        _one_group(api, body, x, dst, wide)
    rec.array("dst", dst)
    rec.array("wide", wide)
    return rec.out


def case_float_activity(api):
    """What the GPU path's float operators are held to: which elements a failed
    division, remainder or power deactivates, what value numpy.ma leaves there,
    what NumPy functions make of such tiles, and what a store writes for each
    kind of result (a tile: active elements only; what a NumPy function or an
    operator with such a result on its left returns: everything)."""
    rec = Recorder()
    dsts = {}
    for tag, dt, big, tiny in (("f32", np.float32, 3.0e38, 1.5e-38), ("f16", np.float16, 60000.0, 6.2e-5)):
        a = np.array([4, -9, 0, -0.0, 7, 5.5, -5.5, big, -big, tiny, np.inf, -np.inf, np.nan, 3, -3, 1,
                      2.5, -7.25, 0, 1e-3], dt)
        b = np.array([2, 0, 0, 3, -0.0, -2, 2, 1e-3, big, big, 2, 0, 1, np.nan, np.inf, -np.inf,
                      0.5, 3, -4, tiny], dt)
        n = len(a)
        K = dt
        bodies = [
            ("div", lambda x, y: x / y), ("floordiv", lambda x, y: x // y), ("mod", lambda x, y: x % y),
            ("div_chain", lambda x, y: x / y * K(2) + K(1)),
            ("pow2", lambda x, y: x ** K(2)), ("pow_half", lambda x, y: x ** K(0.5)),
            ("pow2_div", lambda x, y: x ** K(2) / y),
            ("neg_div", lambda x, y: -(x / y)), ("abs_builtin_div", lambda x, y: abs(x / y)),
            ("np_divide", lambda x, y: np.divide(x, y)), ("np_remainder", lambda x, y: np.remainder(x, y)),
            ("np_abs_div", lambda x, y: np.abs(x / y)), ("np_sqrt", lambda x, y: np.sqrt(x)),
            ("np_log", lambda x, y: np.log(x)), ("np_sqrt_div", lambda x, y: np.sqrt(x / y)),
            ("np_maximum_divs", lambda x, y: np.maximum(x / y, y / x)),
            ("np_minimum", lambda x, y: np.minimum(x, y)), ("np_maximum", lambda x, y: np.maximum(x, y)),
            ("np_add_div", lambda x, y: np.add(x / y, y)),
            ("np_abs_div_times2", lambda x, y: np.abs(x / y * K(2))),
            ("bare_left_sub", lambda x, y: np.abs(x / y) - y / x),
            ("bare_left_mul", lambda x, y: np.abs(x) * (y / x)),
            ("bare_left_div", lambda x, y: np.abs(x) / y),
            ("bare_right_add", lambda x, y: x / y + np.abs(y / x)),
            ("tile_times_np_sqrt", lambda x, y: x * np.sqrt(y)),
            ("np_sqrt_times_tile", lambda x, y: np.sqrt(x) * y),
            ("bare_plus_scalar", lambda x, y: np.abs(x / y) + K(1)),
            ("npscalar_left_mul", lambda x, y: K(2) * (x / y)),
            ("floordiv_mod", lambda x, y: (x // y) * y + x % y),
            ("rint_floordiv_minus_mod", lambda x, y: np.rint(x // y) - x % y),
            ("lt", lambda x, y: x < y), ("le", lambda x, y: x <= y), ("eq", lambda x, y: x == y),
            ("ne", lambda x, y: x != y), ("ge", lambda x, y: x >= y), ("gt", lambda x, y: x > y),
            ("div_gt", lambda x, y: x / y > K(0.5)),
            ("lt_as_factor", lambda x, y: (x < y).astype(dt) * x),
            ("sum_div", lambda x, y: (x / y).sum()), ("np_abs_div_sum", lambda x, y: np.abs(x / y).sum()),
        ]
        # tiles four elements wider than the arrays: every tile has a real mask
        # (the reference cannot read or store a comparison of two tiles that
        # numpy.ma gave its scalar "no mask", kernel_api.py:93-103,117-119)
        dst = np.full((len(bodies), n + 4), 7.5, dt)
        flags = np.zeros((len(bodies), n + 4), bool)
        flags[:, ::3] = True

        def body(gr, a, b, dst, flags, bodies=bodies, tag=tag, n=n):
            x, y = gr.load(a, shape=n + 4), gr.load(b, shape=n + 4)
            for row, (name, fn) in enumerate(bodies):
                t = rec.attempt(f"{tag}.{name}", lambda: fn(x, y))
                if t is None or np.ndim(t) == 0 or "_left_" in name:
                    continue                    # (the reference has no reflected operators)
                try:
                    gr.store(flags[row] if np.asarray(t).dtype == bool else dst[row], t)
                except Exception as e:                  # noqa: BLE001
                    rec.out[f"{tag}.{name}.store_raises"] = _text(type(e).__name__)

        with np.errstate(all="ignore"), warnings.catch_warnings():
            warnings.simplefilter("ignore")
            _one_group(api, body, a, b, dst, flags, group=n)
        rec.array(f"{tag}.dst", dst)
        rec.array(f"{tag}.flags", flags)
    return rec.out


def case_masked_reductions(api):
    """Reductions along rows and down columns over elements that a zero divisor
    deactivated, row / column scalars that are deactivated themselves (a
    quotient of two sums with a zero divisor, numpy.sqrt of a negative sum, a
    mean that is not finite), arithmetic on those, and what a store then writes:
    tiles skip deactivated elements, per-row results (bare numpy.ma arrays) are
    written in full with what numpy.ma left under the mask."""
    rec = Recorder()
    f = np.float32
    rng = np.random.default_rng(11)
    a = rng.integers(-6, 7, (6, 5)).astype(f) / f(2)
    b = rng.integers(-3, 4, (6, 5)).astype(f)
    b[1, :] = 0                                     # every quotient of the row is deactivated
    b[4, :] = [1.5, -1.5, 2, -2, 0]                 # adds up to zero
    b[2, :] = -np.abs(b[2, :]) - f(1)               # a negative sum
    a[5, 2] = np.inf                                # a mean that is not finite
    tiles = {
        "ratio": lambda ta, tb: ta * (ta.sum(axis=1, keepdims=True) / tb.sum(axis=1, keepdims=True)),
        "centre": lambda ta, tb: (ta / tb) - (ta / tb).mean(axis=1, keepdims=True),
        "divsqrt": lambda ta, tb: ta / np.sqrt(tb.sum(axis=1, keepdims=True)),
        "mullog": lambda ta, tb: ta * np.log(tb.sum(axis=1, keepdims=True)),
        "xvar": lambda ta, tb: tb * ta.var(axis=1, keepdims=True),
        "xstd": lambda ta, tb: tb * ta.std(axis=1, keepdims=True),
        "xmaskedvar": lambda ta, tb: tb * (ta / tb).var(axis=1, keepdims=True, ddof=2),
        "rms": lambda ta, tb: ta / np.sqrt(np.mean(np.square(ta), axis=1, keepdims=True) + f(1e-6)) * tb,
        "layernorm": lambda ta, tb: (ta - ta.mean(axis=1, keepdims=True)) /
        np.sqrt(ta.var(axis=1, keepdims=True) + f(1e-5)) * tb,
        "over_max": lambda ta, tb: ta / (ta / tb).max(axis=1, keepdims=True),
        # tile.astype gives a bare numpy.ma array: what is computed from it is
        # stored in full, deactivated elements with what numpy.ma leaves in them
        "bare_scaled_quotient": lambda ta, tb: (ta.astype(f) / tb.astype(f)) * f(3) - f(1),
        "bare_rms": lambda ta, tb: ta.astype(f) / np.sqrt(np.mean(np.square(ta.astype(f)), axis=1, keepdims=True)
                                                          + f(1e-6)) * tb.astype(f),
        "bare_centre_over_sum": lambda ta, tb: (ta.astype(f) - ta.astype(f).mean(axis=1, keepdims=True)) /
        tb.astype(f).sum(axis=1, keepdims=True),
        "bare_one_minus_quotient": lambda ta, tb: f(1) - ta.astype(f) / tb.astype(f),
        "bare_python_one_minus_quotient": lambda ta, tb: 1.0 - ta.astype(f) / tb.astype(f),
        "bare_sqrt_of_quotient": lambda ta, tb: np.sqrt(ta.astype(f) / tb.astype(f)) + f(2),
        "col_centre": lambda ta, tb: ta - ta.mean(axis=0, keepdims=True),
        "col_over_sum": lambda ta, tb: ta / tb.sum(axis=0, keepdims=True),
    }
    rows = {
        "mean": lambda ta, tb: (ta / tb).mean(axis=1),
        "sum": lambda ta, tb: (ta / tb).sum(axis=1),
        "max": lambda ta, tb: (ta / tb).max(axis=1),
        "min": lambda ta, tb: (ta / tb).min(axis=1),
        "var": lambda ta, tb: (ta / tb).var(axis=1),
        "std1": lambda ta, tb: (ta / tb).std(axis=1, ddof=1),
        "plain_mean": lambda ta, tb: ta.mean(axis=1),
        "plain_var": lambda ta, tb: ta.var(axis=1),
        "plain_std": lambda ta, tb: ta.std(axis=1),
        "sqrt_sum": lambda ta, tb: np.sqrt(tb.sum(axis=1)),
        "sum_ratio": lambda ta, tb: ta.sum(axis=1) / tb.sum(axis=1),
        "one_plus_ratio": lambda ta, tb: f(1) + ta.sum(axis=1) / tb.sum(axis=1),
        "python_one_plus_ratio": lambda ta, tb: 1.0 + ta.sum(axis=1) / tb.sum(axis=1),
        "ratio_times_two": lambda ta, tb: ta.sum(axis=1) / tb.sum(axis=1) * f(2),
        "two_ratios": lambda ta, tb: (ta.sum(axis=1) / tb.sum(axis=1) + f(1)) *
        (tb.max(axis=1) / ta.sum(axis=1) - f(2)),
        "neg_sqrt_ratio": lambda ta, tb: -np.sqrt(ta.sum(axis=1) / tb.sum(axis=1)),
        "max_plus_log": lambda ta, tb: ta.max(axis=1) + np.log(tb.sum(axis=1)),
        "log_plus_max": lambda ta, tb: np.log(tb.sum(axis=1)) + ta.max(axis=1),
        "exp_of_mean": lambda ta, tb: np.exp((ta / tb).mean(axis=1)),
    }
    cols = {
        "col_sum": lambda ta, tb: (ta / tb).sum(axis=0),
        "col_max": lambda ta, tb: (ta / tb).max(axis=0),
        "col_min_log": lambda ta, tb: np.log(ta * tb).min(axis=0),
        "col_mean": lambda ta, tb: ta.mean(axis=0),
        "col_var": lambda ta, tb: ta.var(axis=0),
        "col_std": lambda ta, tb: ta.std(axis=0, ddof=1),
    }
    bt = b.copy()
    bt[:, 3] = 0                                    # a column without an active quotient
    dst_t = np.full((len(tiles), 6, 5), POISON, f)
    dst_r = np.full((len(rows), 6), POISON, f)
    dst_c = np.full((len(cols), 5), POISON, f)

    def body(gr, a, b, bt, dst_t, dst_r, dst_c):
        for i, (name, fn) in enumerate(tiles.items()):
            ta, tb = gr.load(a, shape=(8, 5)), gr.load(b, shape=(8, 5))
            t = rec.attempt("tile." + name, lambda: fn(ta, tb))
            if t is not None:
                gr.store(dst_t[i], t)
        for i, (name, fn) in enumerate(rows.items()):
            ta, tb = gr.load(a, shape=(8, 5)), gr.load(b, shape=(8, 5))
            t = rec.attempt("row." + name, lambda: fn(ta, tb))
            if t is not None:
                gr.store(dst_r[i], t)
        for i, (name, fn) in enumerate(cols.items()):
            ta, tb = gr.load(a, shape=(6, 8)), gr.load(bt, shape=(6, 8))
            t = rec.attempt("col." + name, lambda: fn(ta, tb))
            if t is not None:
                gr.store(dst_c[i], t)

    with np.errstate(all="ignore"), warnings.catch_warnings():
        warnings.simplefilter("ignore")
        _one_group(api, body, a, b, bt, dst_t, dst_r, dst_c)
    rec.array("dst_tiles", dst_t)
    rec.array("dst_rows", dst_r)
    rec.array("dst_cols", dst_c)
    return rec.out


def case_shapes_and_selections(api):
    """What a store writes for tiles whose shape was changed on the way (a
    transposed tile, a row vector and a per-row operand broadcast over a 2-D
    tile, a matrix times a vector), for numpy.where and numpy.tanh of tiles, for
    an int32 tile converted with astype, and for one result per group assigned
    to a buffer element; loads reach past their arrays, divisors hold zeros."""
    rec = Recorder()
    f = np.float32
    rng = np.random.default_rng(13)
    x = rng.integers(-4, 5, (5, 6)).astype(f)
    y = rng.integers(-2, 3, (5, 6)).astype(f)
    row = rng.integers(-2, 3, 6).astype(f)
    col = rng.integers(-2, 3, 5).astype(f)
    xi = rng.integers(-9, 10, (5, 6)).astype(np.int32)
    vec = rng.integers(-3, 4, 6).astype(f)
    forms = {
        "where_of_tiles": lambda a, b, r, c, ai: np.where(a > b, a, b),
        "where_with_numbers": lambda a, b, r, c, ai: np.where(a * b >= f(0), a, f(-1)),
        "where_of_quotient": lambda a, b, r, c, ai: np.where(b != f(0), a / b, f(9)),
        "tanh_of_quotient": lambda a, b, r, c, ai: np.tanh(a / b),
        "tanh_times_tile": lambda a, b, r, c, ai: a * np.tanh(b),
        "row_vector": lambda a, b, r, c, ai: a + r,
        "col_vector": lambda a, b, r, c, ai: a * c[:, None],
        "both_vectors": lambda a, b, r, c, ai: (a + r) / c[:, None],
        "vector_first": lambda a, b, r, c, ai: r / a,
        "int_astype": lambda a, b, r, c, ai: ai.astype(f) * f(0.5),
        "int_astype_plus_tile": lambda a, b, r, c, ai: a + ai.astype(f),
    }
    dst = np.full((len(forms), 7, 7), POISON, f)
    dst_t = np.full((2, 8, 7), POISON, f)              # taller than the transposed tile's active part
    dst_v = np.full((2, 7), POISON, f)
    cells = np.full(6, POISON, f)

    def body(gr, x, y, row, col, xi, vec, dst, dst_t, dst_v, cells):
        for i, (name, fn) in enumerate(forms.items()):
            a, b = gr.load(x, shape=(7, 8)), gr.load(y, shape=(7, 8))
            r, c = gr.load(row, shape=8), gr.load(col, shape=7)
            ai = gr.load(xi, shape=(7, 8))
            t = rec.attempt(name, lambda: fn(a, b, r, c, ai))
            if t is not None:
                gr.store(dst[i], t)
        a = gr.load(x, shape=(7, 8))
        t = rec.attempt("transposed", lambda: a.T)
        if t is not None:
            gr.store(dst_t[0], t)
        t = rec.attempt("transposed_sum", lambda: a.T + gr.load(y, shape=(7, 8)).T)
        if t is not None:
            gr.store(dst_t[1], t)
        v = gr.load(vec, shape=8)
        t = rec.attempt("matrix_times_vector", lambda: np.dot(a, v))
        if t is not None:
            gr.store(dst_v[0], t)
        t = rec.attempt("rows_sum_of_products", lambda: (a * v).sum(axis=1))
        if t is not None:
            gr.store(dst_v[1], t)
        cells[gr.id[0] + 1] = (a * a).sum()
        cells[gr.id[0] + 3] += a.max() - a.min()

    with np.errstate(all="ignore"), warnings.catch_warnings():
        warnings.simplefilter("ignore")
        _one_group(api, body, x, y, row, col, xi, vec, dst, dst_t, dst_v, cells)
    rec.array("dst", dst)
    rec.array("dst_transposed", dst_t)
    rec.array("dst_vectors", dst_v)
    rec.array("cells", cells)
    return rec.out


def case_more_functions(api):
    """NumPy functions of one operand on tiles, on values and on quotients with
    deactivated elements: what numpy.ma gives (the function of the values, the
    activity kept; its fill value where a domain fails) and what a store writes."""
    rec = Recorder()
    f = np.float32
    x = np.array([[-2.5, -1.0, -0.5, -0.0, 0.0, 0.5, 1.0, 2.5], [3.75, -3.25, 100.0, -100.0, 1e-3, -1e-3, 7.0, -7.0]], f)
    y = np.array([[1.0, 0.0, 2.0, 0.0, -1.0, 4.0, 0.0, 0.5], [2.0, -2.0, 0.0, 8.0, 0.0, 1.0, -0.5, 0.0]], f)
    names = ["floor", "ceil", "trunc", "sign", "exp2", "log2", "log10", "log1p", "expm1", "sin", "cos", "reciprocal"]
    dst = np.full((2 * len(names), 3, 9), POISON, f)

    def body(gr, x, y, dst):
        for i, name in enumerate(names):
            fn = getattr(np, name)
            a, b = gr.load(x, shape=(3, 9)), gr.load(y, shape=(3, 9))
            t = rec.attempt(name + "_of_tile", lambda: fn(a))
            if t is not None:
                gr.store(dst[2 * i], t)
            t = rec.attempt(name + "_of_quotient", lambda: fn(a / b) + a)
            if t is not None:
                gr.store(dst[2 * i + 1], t)

    with np.errstate(all="ignore"), warnings.catch_warnings():
        warnings.simplefilter("ignore")
        _one_group(api, body, x, y, dst)
    rec.array("dst", dst)
    return rec.out


def case_numpy_scalar_on_the_left(api):
    """`numpy.float32(2) / tile` and the like: the tile type has no reflected
    operators, so the NumPy scalar's own operator decides what happens."""
    rec = Recorder()
    f = np.float32
    x = np.array([1.0, 0.0, -0.0, np.inf, np.nan, 4.0, -2.0, 0.5], f)
    y = np.array([2.0, 0.0, 1.0, 1.0, 1.0, 0.0, 0.0, -1.0], f)
    forms = {
        "div": lambda a, b: f(2.0) / a,
        "mul": lambda a, b: f(2.0) * a,
        "sub": lambda a, b: f(2.0) - a,
        "add": lambda a, b: f(1.0) + a,
        "floordiv": lambda a, b: f(2.0) // a,
        "mod": lambda a, b: f(2.0) % a,
        "pow": lambda a, b: f(2.0) ** a,
        "lt": lambda a, b: f(1.0) < a,
        "div_quotient": lambda a, b: f(2.0) / (a / b),
        "mul_quotient": lambda a, b: f(2.0) * (a / b),
        "add_quotient_then_tile": lambda a, b: (f(1.0) + (a / b)) * a,
        "div_then_tile_op": lambda a, b: (f(2.0) / a) + a,
        "tile_then_div": lambda a, b: a + (f(2.0) / a),
    }
    dst = np.full((len(forms), 8), POISON, f)
    dstb = np.full(8, True)

    def body(gr, x, y, dst, dstb):
        for i, (name, fn) in enumerate(forms.items()):
            a, b = gr.load(x[:7], shape=8), gr.load(y[:7], shape=8)
            t = rec.attempt(name, lambda: fn(a, b))
            if t is not None:
                gr.store(dstb if name == "lt" else dst[i], t)

    with np.errstate(all="ignore"), warnings.catch_warnings():
        warnings.simplefilter("ignore")
        _one_group(api, body, x, y, dst, dstb)
    rec.array("dst_bool", dstb)          # (the arithmetic forms raise in the reference: nothing to compare)
    return rec.out


def _w(a, b):
    return np.where(a < b, a, b)

def _v(a, b):
    return np.where(a < b, b, a)

PLAIN_AND_BARE_FORMS = {
    # plain arrays and numbers
    "w_div_number": lambda a, b: _w(a, b) / np.float32(-0.125),
    "w_div_zero": lambda a, b: _w(a, b) / np.float32(0),
    "w_floordiv_v": lambda a, b: _w(a, b) // _v(a, b),
    "w_mod_number": lambda a, b: _w(a, b) % np.float32(2),
    "w_mod_v": lambda a, b: _w(a, b) % _v(a, b),
    "sqrt_w": lambda a, b: np.sqrt(_w(a, b)),
    "log_w": lambda a, b: np.log(_w(a, b)),
    "w_pow_half": lambda a, b: _w(a, b) ** np.float32(0.5),
    "w_pow_two": lambda a, b: _w(a, b) ** np.float32(2),
    "number_div_w": lambda a, b: np.float32(2) / _w(a, b),
    "pynumber_minus_w": lambda a, b: 2 - _w(a, b),
    "divide_w_v": lambda a, b: np.divide(_w(a, b), _v(a, b)),
    "neg_abs_w": lambda a, b: -abs(_w(a, b)),
    "w_lt_number": lambda a, b: _w(a, b) < np.float32(0),
    "w_sum": lambda a, b: _w(a, b).sum(),
    "where_of_quotient_then_div": lambda a, b: np.where(a < b, a / b, b) / np.float32(0),
    # plain arrays next to tiles
    "w_add_tile": lambda a, b: _w(a, b) + a,
    "w_div_tile": lambda a, b: _w(a, b) / a,
    "w_floordiv_tile": lambda a, b: _w(a, b) // a,
    "w_mod_tile": lambda a, b: _w(a, b) % a,
    "tile_add_w": lambda a, b: a + _w(a, b),
    "tile_div_w": lambda a, b: a / _w(a, b),
    "tile_floordiv_w": lambda a, b: a // _w(a, b),
    "tile_mod_w": lambda a, b: a % _w(a, b),
    "w_lt_tile": lambda a, b: _w(a, b) < a,
    "tile_lt_w": lambda a, b: a < _w(a, b),
    "divide_tile_w": lambda a, b: np.divide(a, _w(a, b)),
    "divide_w_tile": lambda a, b: np.divide(_w(a, b), a),
    "maximum_w_tile": lambda a, b: np.maximum(_w(a, b), a),
    "where_of_w_and_tile": lambda a, b: np.where(_w(a, b) > a, _w(a, b), a),
    "mask_and_mask": lambda a, b: (a / b).mask & (b / a).mask,
    "where_of_mask": lambda a, b: np.where((a / b).mask, a, b),
    # plain arrays next to bare numpy.ma arrays
    "w_div_bare": lambda a, b: _w(a, b) / np.abs(a),
    "w_mod_bare": lambda a, b: _w(a, b) % np.abs(a),
    "bare_div_w": lambda a, b: np.abs(a) / _w(a, b),
    "bare_mod_w": lambda a, b: np.abs(a) % _w(a, b),
    # bare numpy.ma arrays next to tiles
    "bare_add_tile": lambda a, b: np.abs(a) + b,
    "bare_div_tile": lambda a, b: np.abs(a) / b,
    "bare_floordiv_tile": lambda a, b: np.abs(a) // b,
    "bare_mod_tile": lambda a, b: np.abs(a) % b,
    "sqrt_mod_tile": lambda a, b: np.sqrt(a * a) % b,
    "tile_mod_bare": lambda a, b: a % np.abs(b),
    "tile_floordiv_bare": lambda a, b: a // np.abs(b),
    "bare_lt_tile": lambda a, b: np.abs(a) < b,
    "bare_pow_half": lambda a, b: np.negative(a) ** np.float32(0.5),
    "bare_mod_number": lambda a, b: np.abs(a) % np.float32(2),
    "bare_mod_zero": lambda a, b: np.abs(a) % np.float32(0),
    "tile_mod_zero": lambda a, b: a % np.float32(0),
    "tile_mod_product": lambda a, b: a % (np.float32(0) * b),
    "quotient_mod_tile": lambda a, b: (a / b) % b,
}


def case_plain_and_bare_arrays_next_to_tiles(api):
    """What follows numpy.where (a plain NumPy array) and a NumPy function of a
    tile (a bare numpy.ma array) when they meet numbers, each other and tiles,
    on either side of the operators and in NumPy functions: which arithmetic
    runs (NumPy's own, numpy.ma's operator, numpy.ma's wrapped function), what
    kind of value comes back, what raises, and what a store writes."""
    rec = Recorder()
    f = np.float32
    x = np.array([1.0, 0.0, -0.0, np.inf, np.nan, 4.0, -2.0, 0.5, -1.0, 3.0, -np.inf, 2.5], f)
    y = np.array([2.0, 0.0, 1.0, 1.0, 1.0, 0.0, 0.0, -1.0, 1.0, -2.0, 2.0, 0.0], f)

    forms = PLAIN_AND_BARE_FORMS
    dst = np.full((len(forms), 12), POISON, f)
    dstb = np.full((len(forms), 12), True)

    def body(gr, x, y, dst, dstb):
        for i, (name, fn) in enumerate(forms.items()):
            a, b = gr.load(x[:11], shape=12), gr.load(y[:11], shape=12)
            t = rec.attempt(name, lambda: fn(a, b))
            if t is None or np.ndim(t) != 1:
                continue
            if t.dtype == f:
                gr.store(dst[i], t)
            elif t.dtype == bool:
                gr.store(dstb[i], t)

    with np.errstate(all="ignore"), warnings.catch_warnings():
        warnings.simplefilter("ignore")
        _one_group(api, body, x, y, dst, dstb, group=12)
    rec.array("dst", dst)
    rec.array("dst_bool", dstb)
    return rec.out


def case_mapped_loads_and_stores(api):
    """Tiles loaded and stored through index mappings
    (python/hckernel/kernel_api.py:296-335): which elements a mapped load
    activates, what a mapped store writes for a tile, for a bare numpy.ma array
    (its deactivated elements are numpy.ma's masked constant) and for a plain
    array, into float32, float16, bool and int32 destinations."""
    rec = Recorder()
    x = (np.arange(24, dtype=np.float32).reshape(4, 6) - 7)
    y = np.array([[1, 0, 2, 0, -1, 3]] * 4, np.float32)
    shifted = api.create_mapping(lambda i, j: (i - 1, j + 2))
    transpose = api.create_mapping(lambda i, j: (j, i))
    dst = {n: np.full((5, 8), POISON, np.float32) for n in ("tile", "bare", "bare_unmapped", "plain", "quotient")}
    dst16 = np.full((5, 8), POISON, np.float16)
    dstb = np.full((5, 8), True)
    dsti = np.full((5, 8), POISON, np.int32)

    def body(gr, x, y, tile, bare, bare_unmapped, plain, quotient, dst16, dstb, dsti):
        t = gr.load(x, shape=(4, 8), mapping=transpose)      # rows 0..3 of x's columns: a 4 x 4 part is active
        rec.tile("transposed", t)
        s = gr.load(x, shape=(4, 8), mapping=shifted)
        rec.tile("shifted", s)
        u = gr.load(x, shape=(4, 8))
        gr.store(tile, u, mapping=shifted)
        r = np.sqrt(u)                                     # a bare numpy.ma array: negative and inactive elements masked
        rec.tile("sqrt", r)
        gr.store(bare, r, mapping=shifted)
        gr.store(bare_unmapped, r)
        gr.store(plain, np.where(u.mask, u.data, 5), mapping=shifted)
        q = u / gr.load(y, shape=(4, 8))
        rec.tile("quotient", q)
        gr.store(quotient, q, mapping=shifted)
        gr.store(dst16, r.astype(np.float16), mapping=shifted)
        gr.store(dstb, np.less(r, 2.5), mapping=shifted)
        rec.attempt("int_destination", lambda: gr.store(dsti, r.astype(np.int32), mapping=shifted))

    with np.errstate(all="ignore"), warnings.catch_warnings():
        warnings.simplefilter("ignore")
        _one_group(api, body, x, y, *dst.values(), dst16, dstb, dsti)
    for n, a in dst.items():
        rec.array("dst_" + n, a)
    rec.array("dst_float16", dst16)
    rec.array("dst_bool", dstb)
    rec.array("dst_int32", dsti)
    return rec.out


CASES = {
    "mapped_loads_and_stores": case_mapped_loads_and_stores,
    "plain_and_bare_arrays_next_to_tiles": case_plain_and_bare_arrays_next_to_tiles,
    "masked_reductions": case_masked_reductions,
    "inplace_partial": case_inplace_partial,
    "load_from_masked": case_load_from_masked,
    "domain_masking": case_domain_masking,
    "numpy_functions": case_numpy_functions,
    "compressed_repr": case_compressed_repr,
    "scalar_promotion": case_scalar_promotion,
    "operators": case_operators,
    "store_forms": case_store_forms,
    "float_activity": case_float_activity,
    "shapes_and_selections": case_shapes_and_selections,
    "more_functions": case_more_functions,
    "numpy_scalar_on_the_left": case_numpy_scalar_on_the_left,
}


def run_all(api):
    out = {}
    for cname, fn in CASES.items():
        for k, v in fn(api).items():
            out[f"{cname}/{k}"] = v
    return out


def dump(entries, path):
    """One entry per line: name -> [dtype, shape, bytes as hex] (exact for NaN,
    inf and signed zeros, and readable in a diff)."""
    import json
    with open(path, "w") as f:
        f.write("{\n")
        rows = []
        for k in sorted(entries):
            a = np.asarray(entries[k])
            rows.append(f"{json.dumps(k)}: {json.dumps([str(a.dtype), list(a.shape), a.tobytes().hex()])}")
        f.write(",\n".join(rows))
        f.write("\n}\n")


def load(path):
    import json
    with open(path) as f:
        raw = json.load(f)
    return {k: np.frombuffer(bytes.fromhex(h), dtype=np.dtype(dt)).reshape(shape)
            for k, (dt, shape, h) in raw.items()}

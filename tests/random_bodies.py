"""Random elementwise kernel bodies that lean on numpy.ma's rules: zero
divisors, domains of functions, numpy.where, bare arrays and plain arrays next
to tiles, signed zeros, NaN and infinities in the data.  Shared by the CPU test
that runs the binder's programs in a NumPy restatement of the kernel and by the
GPU test that runs them on the device; both compare with the host executor."""

import numpy as np

# functions whose results may differ from NumPy's in the last bits (tile ** 0.5
# is numpy.power's powf there, a correctly rounded square root here)
INEXACT = ("exp", "log", "tanh", "sin", "cos", "expm1", "log1p", "exp2", "log2", "log10", "** K(0.5)")


def expression(rng, depth, K):
    """(function of three tiles, its source text); K is the tiles' NumPy type."""
    def gen(d):
        if d == 0 or rng.random() < 0.15:
            return rng.choice(["a", "b", "c"])
        kind = rng.integers(0, 20)
        x = gen(d - 1)
        if kind <= 2:
            return f"({x} {rng.choice(['+', '-', '*'])} {gen(d - 1)})"
        if kind == 3:
            return f"({x} / {gen(d - 1)})"
        if kind == 4:
            return f"({x} // {gen(d - 1)})"
        if kind == 5:
            return f"({x} % {gen(d - 1)})"
        if kind == 6:
            return f"np.{rng.choice(['maximum', 'minimum'])}({x}, {gen(d - 1)})"
        if kind == 7:
            return f"(-{x})"
        if kind == 8:
            return f"np.abs({x})"
        if kind == 9:
            return f"np.sqrt({x})"
        if kind == 10:
            return f"np.log({x})"
        if kind == 11:
            cmp = rng.choice(['<', '<=', '>', '>=', '==', '!='])
            return f"np.where({gen(d - 1)} {cmp} {gen(d - 1)}, {x}, {gen(d - 1)})"
        if kind == 12:
            return f"({x} ** K({rng.choice(['2', '0.5'])}))"
        if kind == 13:
            return f"np.{rng.choice(['floor', 'ceil', 'trunc', 'sign', 'rint', 'reciprocal'])}({x})"
        if kind == 14:
            return f"np.{rng.choice(['tanh', 'sin', 'cos'])}({x})"
        if kind == 15:
            return f"({x} {rng.choice(['//', '%', '/'])} K({rng.choice(['0.5', '2.0', '-1.25', '0.0'])}))"
        if kind == 16:
            return f"np.{rng.choice(['divide', 'multiply', 'add', 'subtract'])}({x}, {gen(d - 1)})"
        if kind == 17:
            return f"np.clip({x}, -1.5, 2.25)"
        if kind == 18:
            return f"np.square({x})"
        return f"({x} {rng.choice(['+', '-', '*', '/'])} K({rng.choice(['0.5', '4.0', '-0.125', '0.0'])}))"

    text = gen(depth)
    while text in ("a", "b", "c"):
        text = gen(depth)
    return eval(f"lambda a, b, c: {text}", {"np": np, "K": K}), text


def special_values(rng, shape, dtype):
    """Small multiples of 0.5 (so that sums and products are exact) with zeros
    of both signs, infinities and NaN sprinkled in."""
    v = (rng.integers(-6, 7, shape) / 2).astype(dtype)
    flat = v.reshape(-1)
    idx = rng.integers(0, flat.size, max(1, flat.size // 50))
    flat[idx] = rng.choice(np.array([np.inf, -np.inf, np.nan, 0.0, -0.0], dtype), idx.size)
    return v


def case(seed):
    """(function, text, dtype, three operand arrays of shape `shape`, shape kind)."""
    rng = np.random.default_rng(seed)
    dtype = [np.float32, np.float16][seed % 2]
    fn, text = expression(rng, int(rng.integers(1, 4)), dtype)
    shape = (1003,) if seed % 3 == 0 else (37, 131)
    return fn, text, dtype, [special_values(rng, shape, dtype) for _ in range(3)], shape


def difference(got, want, text):
    """None if `got` equals `want`: the same NaNs, the same bits elsewhere
    (a few ulp where `text` calls a function whose last bits may differ)."""
    dtype = want.dtype
    nan = np.isnan(want)
    if not (np.isnan(got) == nan).all():
        i = tuple(np.argwhere(np.isnan(got) != nan)[0])
        return f"NaN pattern differs at {i}: got {got[i]} want {want[i]}"
    if any(w in text for w in INEXACT):
        tol = dict(rtol=2e-3, atol=2e-3) if dtype == np.float16 else dict(rtol=2e-6, atol=1e-6)
        ok = np.isclose(got.astype(np.float64), want.astype(np.float64), equal_nan=True, **tol)
        if not ok.all():
            i = tuple(np.argwhere(~ok)[0])
            return f"values differ at {i}: got {got[i]} want {want[i]}"
        return None
    u = np.uint32 if dtype == np.float32 else np.uint16
    bad = (got.view(u) != want.view(u)) & ~nan
    if bad.any():
        i = tuple(np.argwhere(bad)[0])
        return f"bits differ at {i}: got {got[i]} want {want[i]}"
    return None


def row_expression(rng, K, leaves=("ta", "tb")):
    """(function of two 2-D tiles, its text, result is one value per row): an
    elementwise expression of the tiles and of row scalars (sum, max, min, mean,
    var, std along axis 1 of smaller elementwise expressions).  `leaves` may
    name more operands (a row vector `w`, a per-row operand `s[:, None]`)."""
    red_count = [0]

    def scalar(d):
        red = rng.choice(["sum", "max", "min", "mean", "var", "std"])
        inner = elem(d, False)
        while "ta" not in inner and "tb" not in inner:      # (a reduction needs a 2-D tile under it)
            inner = elem(d, False)
        if red in ("var", "std"):
            ddof = rng.choice(["", ", ddof=1"])
            return f"{inner}.{red}(axis=1, keepdims=True{ddof})"
        return f"{inner}.{red}(axis=1, keepdims=True)"

    def elem(d, scalars):
        if d == 0 or rng.random() < 0.2:
            if scalars and red_count[0] < 3 and rng.random() < 0.45:
                red_count[0] += 1
                return scalar(max(d - 1, 0))
            return rng.choice(list(leaves))
        kind = rng.integers(0, 12)
        x = elem(d - 1, scalars)
        if kind <= 2:
            return f"({x} {rng.choice(['+', '-', '*'])} {elem(d - 1, scalars)})"
        if kind <= 4:
            return f"({x} / {elem(d - 1, scalars)})"
        if kind == 5:
            return f"np.{rng.choice(['maximum', 'minimum'])}({x}, {elem(d - 1, scalars)})"
        if kind == 6:
            return f"np.{rng.choice(['sqrt', 'log', 'abs', 'exp', 'tanh', 'square'])}({x})"
        if kind == 7:
            return f"(-{x})"
        if kind == 8:
            return f"({x} ** K({rng.choice(['2', '0.5'])}))"
        if kind == 9:
            return f"({x} {rng.choice(['+', '-', '*', '/'])} K({rng.choice(['0.5', '2.0', '-1.25', '0.0'])}))"
        if kind == 10:
            return f"{x}.astype(K)"
        return f"np.{rng.choice(['divide', 'multiply', 'add', 'subtract'])}({x}, {elem(d - 1, scalars)})"

    per_row = rng.random() < 0.3
    while True:
        red_count[0] = 0
        if per_row:
            inner = elem(int(rng.integers(1, 3)), False)
            if "ta" not in inner and "tb" not in inner:
                continue
            text = f"{inner}.{rng.choice(['sum', 'max', 'min', 'mean', 'var', 'std'])}(axis=1)"
            if rng.random() < 0.4:
                other = elem(1, False)
                if "ta" in other or "tb" in other:
                    text = f"({text} {rng.choice(['+', '*', '/'])} {other}.{rng.choice(['sum', 'max', 'mean'])}(axis=1))"
            if rng.random() < 0.3 and "s[:, None]" in leaves:
                text = f"(s {rng.choice(['+', '*', '/', '-'])} {text})"
            break
        text = elem(int(rng.integers(1, 4)), True)
        if red_count[0]:
            break
    return eval(f"lambda ta, tb, w=None, s=None: {text}", {"np": np, "K": K}), text, per_row


def vector_case(seed):
    """(function of a tile, a second tile, a row vector w and a per-row operand s,
    text, per_row, the four arrays): row_case with operands that broadcast."""
    rng = np.random.default_rng(seed)
    fn, text, per_row = row_expression(rng, np.float32, ("ta", "ta", "tb", "w", "s[:, None]"))
    rows, n = [(9, 5), (13, 200), (6, 1031)][seed % 3]
    vals = [special_values(rng, shape, np.float32) for shape in ((rows, n), (rows, n), (n,), (rows,))]
    if seed % 2 or any(x in text for x in ("mean(", "var(", "std(")):
        for v in vals:
            v[~np.isfinite(v)] = 0.5
    return fn, text, per_row, vals


def row_case(seed):
    """(function, text, per_row, two operand arrays of shape (rows, n))."""
    rng = np.random.default_rng(seed)
    fn, text, per_row = row_expression(rng, np.float32)
    rows, n = [(9, 5), (13, 200), (6, 1031)][seed % 3]
    vals = [special_values(rng, (rows, n), np.float32) for _ in range(2)]
    # numpy.ma's mean / var / std of a bare array take NumPy's own path while no element of
    # the whole tile is masked and numpy.ma's otherwise, which on rows with infinities or NaN
    # gives different values and activity: data-dependent across rows, outside what the row
    # kernels model (a documented deviation), so those bodies get finite data
    if seed % 2 or any(w in text for w in ("mean(", "var(", "std(")):
        for v in vals:
            v[~np.isfinite(v)] = 0.5
    return fn, text, per_row, vals


def col_expression(rng, K):
    """(function of two (M, GN) tiles holding whole columns, its text): reductions
    down the columns of elementwise expressions, combined per column."""
    def elem(d):
        if d == 0 or rng.random() < 0.25:
            return rng.choice(["ta", "tb"])
        kind = rng.integers(0, 9)
        x = elem(d - 1)
        if kind <= 2:
            return f"({x} {rng.choice(['+', '-', '*'])} {elem(d - 1)})"
        if kind == 3:
            return f"({x} / {elem(d - 1)})"
        if kind == 4:
            return f"np.{rng.choice(['maximum', 'minimum'])}({x}, {elem(d - 1)})"
        if kind == 5:
            return f"np.{rng.choice(['sqrt', 'log', 'abs', 'exp', 'square'])}({x})"
        if kind == 6:
            return f"(-{x})"
        if kind == 7:
            return f"({x} ** K({rng.choice(['2', '0.5'])}))"
        return f"({x} {rng.choice(['+', '-', '*', '/'])} K({rng.choice(['0.5', '2.0', '-1.25', '0.0'])}))"

    def fold():
        red = rng.choice(["sum", "max", "min", "mean", "var", "std"])
        extra = rng.choice(["", ", ddof=1"]) if red in ("var", "std") else ""
        return f"{elem(int(rng.integers(0, 3)))}.{red}(axis=0{extra})"

    text = fold()
    bare_fold = text
    shape = rng.integers(0, 6)
    if shape == 0:
        text = f"np.{rng.choice(['sqrt', 'abs', 'log'])}({text})"
    elif shape == 1:
        text = f"({text} {rng.choice(['*', '+', '/'])} K({rng.choice(['0.5', '2.0', '0.0'])}))"
    elif shape == 2:
        text = f"({text} {rng.choice(['+', '-', '*', '/'])} {fold()})"
    elif shape == 3:
        text = f"np.sqrt({text} / K(7) + K(1e-6))"
    return eval(f"lambda ta, tb: {text}", {"np": np, "K": K}), text, text == bare_fold


def col_case(seed):
    """(function, text, two operand arrays (rows, n), columns per group)."""
    rng = np.random.default_rng(seed)
    fn, text, fold_only = col_expression(rng, np.float32)
    (rows, n), gn = [((37, 70), 32), ((300, 200), 64), ((5, 64), 64)][seed % 3]
    vals = [special_values(rng, (rows, n), np.float32) for _ in range(2)]
    # (see row_case; what follows a fold is plain arithmetic where a column holds infinities
    # or NaN and numpy.ma's there: the documented deviation, so those bodies get finite data too)
    if seed % 2 or not fold_only or any(w in text for w in ("mean(", "var(", "std(")):
        for v in vals:
            v[~np.isfinite(v)] = 0.5
    return fn, text, vals, gn


def statement_body(seed, api):
    """(kernel body, its text, decorator arguments, two operand arrays): a short
    random sequence of statements on two loaded tiles and perhaps an allocated
    one -- in-place operators, `tile[:] = value`, rebinding to an expression or a
    NumPy function -- that ends with a store of one of the tiles.  `api` is the
    module that supplies CurrentGroup, Buffer, sym, typename (the kernel API)."""
    rng = np.random.default_rng(seed)
    two_d = seed % 2 == 0
    names = ["x", "y"]
    lines = []
    if rng.random() < 0.6:
        kind = rng.choice(["zeros", "ones", "full", "empty"])
        lines.append(f"z = gr.{kind}(gr.shape, np.float32{', K(0.5)' if kind == 'full' else ''})")
        names.append("z")

    def operand():
        r = rng.random()
        if r < 0.5:
            return rng.choice(names)
        if r < 0.7:
            return f"K({rng.choice(['0.5', '2.0', '-1.25', '0.0'])})"
        return f"({rng.choice(names)} {rng.choice(['+', '-', '*', '/'])} {rng.choice(names)})"

    for _ in range(int(rng.integers(1, 5))):
        v = rng.choice(names)
        r = rng.random()
        if r < 0.45:
            lines.append(f"{v} {rng.choice(['+=', '-=', '*=', '/='])} {operand()}")
        elif r < 0.65:
            lines.append(f"{v}[:] = {operand()}")
        elif r < 0.8:
            lines.append(f"{v} = {operand()} {rng.choice(['+', '*', '-'])} {operand()}")
        else:
            lines.append(f"{v} = np.{rng.choice(['abs', 'exp', 'sqrt'])}({v})")
    out = rng.choice(names)
    M, N, DT = api.sym.M, api.sym.N, api.typename.DT
    if two_d:
        head = ["def body(gr: CurrentGroup, a: Buffer[M, N, DT], b: Buffer[M, N, DT], out: Buffer[M, N, DT]):",
                "    i, j = gr.work_offset",
                "    x = gr.load(a[i:, j:], shape=gr.shape)", "    y = gr.load(b[i:, j:], shape=gr.shape)"]
        tail = [f"    gr.store(out[i:, j:], {out})"]
        shape, deco = (37, 131), dict(work_shape=(M, N), group_shape=(4, 64))
    else:
        head = ["def body(gr: CurrentGroup, a: Buffer[N, DT], b: Buffer[N, DT], out: Buffer[N, DT]):",
                "    o = gr.work_offset[0]",
                "    x = gr.load(a[o:], shape=gr.shape)", "    y = gr.load(b[o:], shape=gr.shape)"]
        tail = [f"    gr.store(out[o:], {out})"]
        shape, deco = (1003,), dict(work_shape=N, group_shape=256)
    env = {"np": np, "K": np.float32, "CurrentGroup": api.CurrentGroup, "Buffer": api.Buffer, "M": M, "N": N,
           "DT": DT}
    exec("\n".join(head + ["    " + line for line in lines] + tail), env)
    vals = [special_values(rng, shape, np.float32) for _ in range(2)]
    if seed % 4 < 2:
        for v in vals:
            v[~np.isfinite(v)] = 0.5
    return env["body"], "; ".join(lines) + f" -> {out}", deco, vals


def int_statement_body(seed, api):
    """(kernel body, its text, decorator arguments, two int32 operand arrays): a
    few statements on two loaded int32 tiles (in-place operators, assignment,
    rebinding) and a stored expression of + - * // % & | ^ << >> minimum maximum
    abs negation and numpy.where; divisors hold zeros, every fifth case INT_MIN
    and INT_MAX."""
    rng = np.random.default_rng(seed)
    I = np.int32
    names = ["x", "y"]

    def expr(d):
        if d == 0 or rng.random() < 0.25:
            return rng.choice(names)
        k = rng.integers(0, 12)
        x = expr(d - 1)
        if k <= 2:
            return f"({x} {rng.choice(['+', '-', '*'])} {expr(d - 1)})"
        if k == 3:
            return f"({x} // {expr(d - 1)})"
        if k == 4:
            return f"({x} % {expr(d - 1)})"
        if k == 5:
            return f"({x} {rng.choice(['&', '|', '^'])} {expr(d - 1)})"
        if k == 6:
            return f"({x} {rng.choice(['<<', '>>'])} ({expr(d - 1)} & I(7)))"
        if k == 7:
            return f"np.{rng.choice(['maximum', 'minimum'])}({x}, {expr(d - 1)})"
        if k == 8:
            return f"{rng.choice(['-', 'abs'])}({x})"
        if k == 9:
            return f"({x} {rng.choice(['+', '*', '//', '%', '-'])} I({rng.choice(['2', '-3', '0', '7'])}))"
        if k == 10:
            cmp = rng.choice(['<', '==', '!=', '>='])
            return f"np.where({expr(d - 1)} {cmp} {expr(d - 1)}, {x}, {expr(d - 1)})"
        return f"np.abs({x})"

    lines = []
    for _ in range(int(rng.integers(0, 3))):
        v = rng.choice(names)
        r = rng.random()
        if r < 0.5:
            lines.append(f"{v} {rng.choice(['+=', '-=', '*=', '//=', '%=', '&='])} {expr(1)}")
        elif r < 0.7:
            lines.append(f"{v}[:] = {expr(1)}")
        else:
            lines.append(f"{v} = {expr(2)}")
    final = expr(int(rng.integers(0, 3)))
    M, N, DT = api.sym.M, api.sym.N, api.typename.DT
    src = ["def body(gr: CurrentGroup, a: Buffer[M, N, DT], b: Buffer[M, N, DT], out: Buffer[M, N, DT]):",
           "    i, j = gr.work_offset", "    x = gr.load(a[i:, j:], shape=gr.shape)",
           "    y = gr.load(b[i:, j:], shape=gr.shape)"] + ["    " + line for line in lines] + \
          [f"    gr.store(out[i:, j:], {final})"]
    env = {"np": np, "I": I, "CurrentGroup": api.CurrentGroup, "Buffer": api.Buffer, "M": M, "N": N, "DT": DT}
    exec("\n".join(src), env)
    shape = (37, 131)
    vals = [rng.integers(-9, 10, shape).astype(I) for _ in range(2)]
    if seed % 5 == 0:
        vals[0][rng.random(shape) < 0.05] = np.iinfo(I).min
        vals[1][rng.random(shape) < 0.05] = np.iinfo(I).max
    return env["body"], "; ".join(lines) + f" -> {final}", dict(work_shape=(M, N), group_shape=(4, 64)), vals


def row_statement_body(seed, api):
    """(kernel body, text, decorator arguments, two operand arrays, group rows): a
    few statements on two tiles that hold whole rows -- in-place operators with row
    scalars (`t -= t.max(axis=1, keepdims=True)`, `t /= u.sum(axis=1, keepdims=True)`),
    rebinding to NumPy functions -- and a store of a tile or of an expression."""
    rng = np.random.default_rng(seed)
    names = ["t", "u"]

    def scalar():
        red = rng.choice(["sum", "max", "min", "mean", "std"])
        return f"{rng.choice(names)}.{red}(axis=1, keepdims=True)"

    def operand():
        r = rng.random()
        if r < 0.45:
            return scalar()
        if r < 0.65:
            return rng.choice(names)
        if r < 0.8:
            return f"K({rng.choice(['0.5', '2.0', '-1.25', '0.0'])})"
        return f"({rng.choice(names)} {rng.choice(['+', '-', '*'])} {scalar()})"

    lines = []
    for _ in range(int(rng.integers(1, 4))):
        v = rng.choice(names)
        r = rng.random()
        if r < 0.6:
            lines.append(f"{v} {rng.choice(['+=', '-=', '*=', '/='])} {operand()}")
        elif r < 0.75:
            lines.append(f"{v} = np.{rng.choice(['exp', 'abs', 'sqrt', 'tanh'])}({v})")
        else:
            lines.append(f"{v} = {v} {rng.choice(['+', '-', '*', '/'])} {operand()}")
    final = rng.choice(names) if rng.random() < 0.6 else f"({rng.choice(names)} {rng.choice(['+', '*', '/'])} {operand()})"
    M, N, GM, DT = api.sym.M, api.sym.N, api.sym.GM, api.typename.DT
    src = ["def body(gr: CurrentGroup, a: Buffer[M, N, DT], b: Buffer[M, N, DT], out: Buffer[M, N, DT], g: GM):",
           "    m0, mb = gr.work_offset[0], gr.shape[0]",
           "    t = gr.load(a[m0:, :], shape=(mb, N))", "    u = gr.load(b[m0:, :], shape=(mb, N))"] + \
          ["    " + line for line in lines] + [f"    gr.store(out[m0:, :], {final})"]
    env = {"np": np, "K": np.float32, "CurrentGroup": api.CurrentGroup, "Buffer": api.Buffer, "M": M, "N": N,
           "GM": GM, "DT": DT}
    exec("\n".join(src), env)
    rows, n = [(9, 5), (13, 200), (6, 1031)][seed % 3]
    vals = [(rng.integers(-6, 7, (rows, n)) / 2).astype(np.float32) for _ in range(2)]   # finite (see row_case)
    return env["body"], "; ".join(lines) + f" -> {final}", dict(work_shape=M, group_shape=GM), vals

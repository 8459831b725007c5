"""A NumPy restatement of the general float map's rules (the comment at the top
of hc_amd/csrc/kernels/fmap.hip), used by CPU tests to run the programs the
binder emits without a GPU.  It states what each instruction is meant to do;
that the kernel does the same is what the GPU parity tests of its opcodes
check."""

import numpy as np

f32 = np.float32


def _r16(x):
    return x.astype(np.float16).astype(f32)


def run_fmap(program, inputs, store_all, out):
    """Runs `program` ((opname, arg, imm) triples) over `inputs` (arrays of one
    shape: float32, float16 or int32) and stores into `out` (float32, float16
    or bool) where the result is active, or everywhere with store_all."""
    vals = [np.asarray(x).astype(f32) for x in inputs]
    shape = out.shape
    stack = []                                # (values as float32, active)
    with np.errstate(all="ignore"):
        for name, arg, imm in program:
            half, as_function, plain = bool(arg & 1), bool(arg & 2), bool(arg & 4)
            if name == "in":
                stack.append((vals[arg].copy(), np.ones(shape, bool)))
            elif name == "const":
                stack.append((np.full(shape, imm, f32), np.ones(shape, bool)))
            elif name == "select":
                (c, _), (a, _), (b, _) = stack[-3:]
                del stack[-3:]
                stack.append((np.where(c != 0, a, b), np.ones(shape, bool)))
            elif name == "merge":             # tile[:] = value: the value where active, the tile's own elsewhere
                (a, ka), (b, kb) = stack[-2:]
                del stack[-2:]
                stack.append((np.where(kb, b, a), ka | kb))
            elif name in _UNARY:
                a, ok = stack.pop()
                stack.append(_UNARY[name](a, ok.copy(), plain))
            else:
                (a, ka), (b, kb) = stack[-2:]
                del stack[-2:]
                if arg & 16:                  # the second operand's activity does not count
                    kb = np.ones(shape, bool)
                if arg & 8 and name in ("min", "max"):     # evaluated in the other order
                    a, b = b, a
                if name in ("eq", "ne") and not as_function:
                    # numpy.ma compares the activity where the result is inactive
                    same = (a == b) if name == "eq" else (a != b)
                    off = (~ka & ~kb) if name == "eq" else (ka != kb)
                    stack.append((np.where(ka & kb, same, off).astype(f32), ka & kb))
                    continue
                stack.append(_binary(name, a, b, ka & kb, half, as_function, plain))
            assert len(stack) <= 4, "the kernel's stack has four entries"
    (v, ok), = stack
    keep = ok | bool(store_all)
    if out.dtype == bool:
        out[keep] = v[keep] != 0
    else:
        out[keep] = v.astype(out.dtype)[keep]


def _binary(name, a, b, ok, half, as_function, plain):
    if name in ("add", "sub", "mul"):
        r = {"add": np.add, "sub": np.subtract, "mul": np.multiply}[name](a, b)
        return (r if as_function else np.where(ok, r, a)), ok
    if name in ("div", "floordiv", "mod", "udiv") and plain:
        fn = {"div": np.divide, "udiv": np.divide, "floordiv": np.floor_divide, "mod": np.remainder}[name]
        return fn(a, b), ok
    if name in ("div", "floordiv"):
        r = np.divide(a, b) if name == "div" else np.floor_divide(a, b)
        if half:
            r = _r16(r)
        bad = ~ok | (b == 0) | ~np.isfinite(r)
        return np.where(bad, f32(0) + a, r + f32(0) * a), ~bad
    if name in ("mod", "udiv"):
        unsafe = (a == a) & (b == b) & ((b == 0) | np.isinf(a))
        r = np.remainder(a, b) if name == "mod" else np.divide(a, b)
        return np.where(unsafe, f32(1), r), ok & ~unsafe
    if name == "min":
        return np.where((a <= b) | (a != a), a, b) if half else np.where((a < b) | (a != a), a, b), ok
    if name == "max":
        return np.where((a >= b) | (a != a), a, b) if half else np.where((a > b) | (a != a), a, b), ok
    cmp = {"lt": np.less, "le": np.less_equal, "eq": np.equal, "ne": np.not_equal,
           "ge": np.greater_equal, "gt": np.greater}[name]
    return cmp(a, b).astype(f32), ok


def _domain(fn, fill, outside):
    def run(a, ok, plain):
        if plain:
            return fn(a), ok
        out = ~ok | outside(a)
        return np.where(out, f32(fill), fn(np.where(out, f32(1), a))), ~out
    return run


def _keeps(fn):
    return lambda a, ok, plain: (fn(a).astype(f32), ok)


def _sign(a):
    return np.where(a > 0, f32(1), np.where(a < 0, f32(-1), np.where(a == 0, f32(0), a)))


def _active(a, ok, plain):
    return ok.astype(f32), np.ones_like(ok)


def _powchk(a, ok, plain):
    bad = ~np.isfinite(a)
    return np.where(bad, f32(1e20), a), ok & ~bad


def _psqrt(a, ok, plain):
    return np.where(ok, np.sqrt(np.where(ok, a, f32(0))) + f32(0), a), ok


_UNARY = {
    "neg": _keeps(np.negative), "abs": _keeps(np.abs), "rint": _keeps(np.rint), "exp": _keeps(np.exp),
    "tanh": _keeps(np.tanh), "floor": _keeps(np.floor), "ceil": _keeps(np.ceil), "trunc": _keeps(np.trunc),
    "sign": _keeps(_sign), "exp2": _keeps(np.exp2), "log1p": _keeps(np.log1p), "expm1": _keeps(np.expm1),
    "sin": _keeps(np.sin), "cos": _keeps(np.cos), "reciprocal": _keeps(lambda a: f32(1) / a),
    "r16": _keeps(_r16),
    "sqrt": _domain(np.sqrt, 0, lambda a: a < 0), "log": _domain(np.log, 1, lambda a: a <= 0),
    "log2": _domain(np.log2, 1, lambda a: a <= 0), "log10": _domain(np.log10, 1, lambda a: a <= 0),
    "psqrt": _psqrt, "active": _active, "powchk": _powchk,
}

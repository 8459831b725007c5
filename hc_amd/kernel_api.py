"""The kernel programming model: group object, buffers, tiles.

Host-side mirror of the reference's python/hckernel/kernel_api.py (the names a
kernel body is written against: CurrentGroup.load/store/vload, allocators,
work_offset, shape, Buffer, TunableParam, atomic_ref, create_mapping).  The
reference compiles the body's source text; here the body is *run once* with a
tracing group.  Group ids are symbolic, buffers are proxies, and tiles record
the operations applied to them, so that one execution yields the whole
per-group program: which windows are loaded, what is computed, what is stored.
hc_amd.binding then matches that program against the hand-written gfx950
kernels.  Nothing in this module computes array values.
"""

from __future__ import annotations

import functools
import itertools
import math
import weakref
import operator
from collections.abc import Iterable
from fractions import Fraction

import numpy as np


class TraceError(RuntimeError):
    """The kernel body did something the tracer cannot express."""


class DynInt(int):
    """An integer that is only known at launch time: the value of a symbol bound
    from a buffer dimension or from a scalar argument that is neither a literal
    nor a tunable.  It behaves like the int it is; arithmetic on it stays
    dynamic.  The one place that cares is vload, whose shape must be static
    (docs/langref.md:226-243 of the reference: "Vector allocation shape must be
    determinable at compile time")."""

    __slots__ = ()


def _dyn_method(name):
    base = getattr(int, name)

    def method(self, *args):
        r = base(self, *args)
        return DynInt(r) if type(r) is int else r
    method.__name__ = name
    return method


for _name in ("__add__", "__radd__", "__sub__", "__rsub__", "__mul__", "__rmul__", "__floordiv__",
              "__rfloordiv__", "__mod__", "__rmod__", "__neg__", "__pos__", "__abs__", "__pow__",
              "__rpow__", "__lshift__", "__rshift__", "__and__", "__or__", "__xor__"):
    setattr(DynInt, _name, _dyn_method(_name))


def is_static(v) -> bool:
    return not isinstance(v, DynInt)


# ---------------------------------------------------------------------------
# Small public types (kernel_api.py:35-40, 214-220, 231-252, 437-451)
# ---------------------------------------------------------------------------
class TunableParam:
    def __init__(self, sym, default, vals, strategy=None):
        self.sym, self.default, self.vals, self.strategy = sym, default, vals, strategy


class Mapping:
    def __init__(self, func):
        self.func = func


def create_mapping(func):
    return Mapping(func)


_ATOMIC_DONE = object()      # what `cell += v` leaves behind for the `ref[i] = ...` that follows


class _AtomicCell:
    def __init__(self, ref, index):
        self.ref, self.index = ref, index

    def __iadd__(self, value):
        self.ref.record(self.index, value)
        return _ATOMIC_DONE

    def _unsupported(self, *_):
        raise TraceError("only `atomic_ref(buffer)[i] += value` is supported on the GPU path")

    __isub__ = __imul__ = __itruediv__ = __add__ = __radd__ = _unsupported


class AtomicRef:
    """`atomic_ref(buffer)`: element updates through it are atomic
    (python/hckernel/kernel_api.py:450-451 returns the array itself because the
    simulator runs the groups one after another).  Traced: `ref[i] += value`
    records an atomic addition of `value` to element i."""

    def __init__(self, proxy):
        self.proxy = proxy

    def __getitem__(self, index):
        if isinstance(index, tuple) and len(index) == 1:
            index = index[0]
        if isinstance(index, Affine):
            if not index.is_const:
                return _AtomicCell(self, index)       # a cell of the group's own: see record()
            index = index.const
        if not isinstance(index, (int, np.integer)):
            raise TraceError("atomic_ref(buffer)[i]: i must be an integer or built from the group id")
        return _AtomicCell(self, int(index))

    def __setitem__(self, index, value):
        if value is not _ATOMIC_DONE:
            raise TraceError("only `atomic_ref(buffer)[i] += value` is supported on the GPU path")

    def record(self, index, value):
        group = getattr(self.proxy, "group", None)
        if group is None:
            raise TraceError("atomic_ref outside a kernel body")
        if isinstance(index, Affine):
            # `ref[f(group id)] += value`: every group adds to an element that the
            # index picks for it
            group.cell_stores.append((self.proxy, (index,), Tile.wrap(value), True))
            return
        group.atomics.append((self.proxy, index, Tile.wrap(value)))


def atomic_ref(a):
    return AtomicRef(a) if isinstance(a, BufferProxy) else a


class Buffer(type):
    """`Buffer[d0, ..., dtype]`: annotation for an array argument; symbolic
    dims are bound to the argument's shape at call time."""

    def __class_getitem__(cls, spec):
        assert len(spec) > 0, "Invalid shape and dtype"
        return type("Buffer", (cls,), {"shape": tuple(spec[:-1]), "dtype": spec[-1]})


class CurrentSubGroup:
    def __init__(self, size, subgroup_id):
        self._size, self._id = size, subgroup_id

    def size(self):
        return self._size

    def subgroup_id(self):
        return self._id


class CurrentWorkitem:
    def __init__(self, local_id, global_id):
        self._lid, self._gid = local_id, global_id

    def local_id(self):
        return self._lid

    def global_id(self):
        return self._gid


# ---------------------------------------------------------------------------
# Affine index expressions in the group id
# ---------------------------------------------------------------------------
def _index_const(v):
    """int or Fraction for a Python, NumPy or sympy rational number, else None."""
    if isinstance(v, (bool, int, np.integer)):
        return int(v)
    if isinstance(v, Fraction):
        return int(v) if v.denominator == 1 else v
    p, q = getattr(v, "p", None), getattr(v, "q", None)      # sympy Integer / Rational
    if isinstance(p, int) and isinstance(q, int) and q:
        return p // q if p % q == 0 else Fraction(p, q)
    return None


class IndexExpr:
    """An integer expression in the group id that is not affine: it contains a
    floor division or a remainder (`w = idx % W_OUT; h = idx // W_OUT`).  Only
    windows of mapped loads and stores may start at such an offset; their
    kernels take the start of every group from a table."""

    __slots__ = ("op", "args")
    _OPS = {"add": operator.add, "sub": operator.sub, "mul": operator.mul,
            "floordiv": operator.floordiv, "mod": operator.mod}

    def __init__(self, op, args):
        self.op, self.args = op, tuple(args)

    @staticmethod
    def _operand(v):
        if isinstance(v, (Affine, IndexExpr)):
            return v
        c = _index_const(v)
        if c is None:
            raise TraceError(f"unsupported index value {v!r}")
        return c

    @classmethod
    def make(cls, op, a, b):
        return cls(op, (cls._operand(a), cls._operand(b)))

    def __add__(self, o): return IndexExpr.make("add", self, o)
    def __radd__(self, o): return IndexExpr.make("add", o, self)
    def __sub__(self, o): return IndexExpr.make("sub", self, o)
    def __rsub__(self, o): return IndexExpr.make("sub", o, self)
    def __mul__(self, o): return IndexExpr.make("mul", self, o)
    def __rmul__(self, o): return IndexExpr.make("mul", o, self)
    def __floordiv__(self, o): return IndexExpr.make("floordiv", self, o)
    def __rfloordiv__(self, o): return IndexExpr.make("floordiv", o, self)
    def __mod__(self, o): return IndexExpr.make("mod", self, o)
    def __rmod__(self, o): return IndexExpr.make("mod", o, self)
    def __neg__(self): return IndexExpr.make("sub", 0, self)

    def __index__(self):
        raise TraceError("a group-id dependent index was used where a number is needed "
                         "(only offsets of loads and stores may depend on the group id)")

    __int__ = __index__

    def _unsupported(self, *_):
        raise TraceError("only + - * // and % are supported on group offsets")

    __truediv__ = __rtruediv__ = __lt__ = __le__ = __gt__ = __ge__ = _unsupported

    def _no_test(self, *_):
        raise TraceError("a group-id dependent index was compared or tested (`==`, `!=`, "
                         "`if idx:`): the body is traced once for all groups, so control flow "
                         "cannot depend on the group")

    __eq__ = __ne__ = __bool__ = _no_test
    __hash__ = object.__hash__

    def same_as(self, o) -> bool:
        return self is o or (isinstance(o, IndexExpr) and self.op == o.op and
                             all(same_index(a, b) for a, b in zip(self.args, o.args)))

    def __repr__(self):
        sign = {"add": "+", "sub": "-", "mul": "*", "floordiv": "//", "mod": "%"}[self.op]
        return f"({self.args[0]!r} {sign} {self.args[1]!r})"


def same_index(a, b) -> bool:
    """Structural equality of two index values (numbers, Affine, IndexExpr)."""
    if a is b:
        return True
    if isinstance(a, (Affine, IndexExpr)):
        return a.same_as(b)
    if isinstance(b, (Affine, IndexExpr)):
        return False
    return a == b


def same_starts(a, b) -> bool:
    return len(a) == len(b) and all(same_index(x, y) for x, y in zip(a, b))


def evaluate_index(e, group_ids):
    """Value of an index expression for many groups at once.  group_ids: one
    integer array per group dimension, all of one shape; returns an array of
    that shape (int64, or Python objects if fractions are involved)."""
    if isinstance(e, Affine):
        out = np.full(np.shape(group_ids[0]) if len(group_ids) else (), e.const, dtype=np.int64)
        for c, g in zip(e.coeffs, group_ids):
            if c:
                out = out + c * g
        return out
    if isinstance(e, IndexExpr):
        a, b = (evaluate_index(x, group_ids) for x in e.args)
        if e.op in ("floordiv", "mod") and np.any(np.equal(b, 0)):
            raise TraceError("division by zero in a group offset")
        return IndexExpr._OPS[e.op](a, b)
    return e


class Affine:
    """const + sum(coeffs[i] * group_id[i]).  The index arithmetic of a tiled
    kernel: offsets are group id times tile size plus constants.  Floor
    division and remainder leave the affine form and give an IndexExpr."""

    __slots__ = ("const", "coeffs")

    def __init__(self, const, coeffs):
        self.const, self.coeffs = int(const), tuple(int(c) for c in coeffs)

    @staticmethod
    def lift(v, rank):
        if isinstance(v, Affine):
            return v
        if isinstance(_index_const(v), Fraction):
            raise TraceError(f"the index value {v} is not an integer")
        try:
            return Affine(int(v), (0,) * rank)
        except (TypeError, ValueError):
            raise TraceError(f"unsupported index value {v!r}") from None

    @property
    def is_const(self):
        return not any(self.coeffs)

    def __add__(self, o):
        if isinstance(o, (IndexExpr, ItemIndex)):
            return NotImplemented
        o = Affine.lift(o, len(self.coeffs))
        return Affine(self.const + o.const, [a + b for a, b in zip(self.coeffs, o.coeffs)])

    __radd__ = __add__

    def __neg__(self):
        return Affine(-self.const, [-c for c in self.coeffs])

    def __sub__(self, o):
        if isinstance(o, (IndexExpr, ItemIndex)):
            return NotImplemented
        return self + (-Affine.lift(o, len(self.coeffs)))

    def __rsub__(self, o):
        if isinstance(o, (IndexExpr, ItemIndex)):
            return NotImplemented
        return Affine.lift(o, len(self.coeffs)) - self

    def __mul__(self, o):
        if isinstance(o, (IndexExpr, ItemIndex)):
            return NotImplemented
        if isinstance(_index_const(o), Fraction):
            return IndexExpr.make("mul", self, o)
        if isinstance(o, Affine):
            if o.is_const:
                o = o.const
            elif self.is_const:
                return o * self.const
            else:
                raise TraceError("product of two group-id dependent indices")
        try:
            k = int(o)
        except (TypeError, ValueError):
            raise TraceError(f"unsupported index factor {o!r}") from None
        return Affine(self.const * k, [c * k for c in self.coeffs])

    __rmul__ = __mul__

    def __index__(self):
        if self.is_const:
            return self.const
        raise TraceError("a group-id dependent index was used where a number is needed "
                         "(only offsets of loads and stores may depend on the group id)")

    __int__ = __index__

    def __floordiv__(self, o): return IndexExpr.make("floordiv", self, o)
    def __rfloordiv__(self, o): return IndexExpr.make("floordiv", o, self)
    def __mod__(self, o): return IndexExpr.make("mod", self, o)
    def __rmod__(self, o): return IndexExpr.make("mod", o, self)

    def _unsupported(self, *_):
        raise TraceError("only + - * // and % are supported on group offsets")

    __truediv__ = __rtruediv__ = __lt__ = __le__ = __gt__ = __ge__ = _unsupported

    # The body is traced once for all groups, so a comparison whose outcome
    # differs from group to group (`if gr.id[0] == 0:`) cannot be answered; it
    # raises instead of picking one branch for every group.  Structural
    # equality of two expressions is same_as().
    def same_as(self, o) -> bool:
        if not isinstance(o, Affine) or self.const != o.const:
            return False
        n = max(len(self.coeffs), len(o.coeffs))
        return self.coeffs + (0,) * (n - len(self.coeffs)) == o.coeffs + (0,) * (n - len(o.coeffs))

    def _compare(self, o):
        if isinstance(o, Affine):
            if self.is_const and o.is_const:
                return self.const, o.const
        elif self.is_const and isinstance(_index_const(o), (int, Fraction)):
            return self.const, _index_const(o)
        raise TraceError("a group id was compared or tested (`==`, `!=`, `if id:`): the body is "
                         "traced once for all groups, so control flow cannot depend on the group")

    def __eq__(self, o):
        a, b = self._compare(o)
        return a == b

    def __ne__(self, o):
        a, b = self._compare(o)
        return a != b

    def __bool__(self):
        a, _ = self._compare(0)
        return bool(a)

    def __hash__(self):
        return hash(self.const) if self.is_const else hash((self.const, self.coeffs))

    def __repr__(self):
        terms = [f"{c}*g{i}" for i, c in enumerate(self.coeffs) if c]
        return " + ".join(terms + ([str(self.const)] if self.const or not terms else []))


class ItemIndex:
    """const + sum(g[i] * group_id[i]) + sum(l[i] * local_id[i]): what a body sees
    inside a work-item scope (python/hckernel/kernel_api.py:397-403: local_id,
    and global_id = group_id * group_shape + local_id).  Integer sums, differences
    and integer multiples stay in this form; it indexes buffer elements
    (`a[i, j]`) and may be stored as a value."""

    __slots__ = ("const", "g", "l")

    def __init__(self, const, g, l):
        self.const, self.g, self.l = int(const), tuple(int(c) for c in g), tuple(int(c) for c in l)

    @staticmethod
    def lift(v, rank):
        if isinstance(v, ItemIndex):
            return v
        if isinstance(v, Affine):
            return ItemIndex(v.const, tuple(v.coeffs) + (0,) * (rank - len(v.coeffs)), (0,) * rank)
        c = _index_const(v)
        if not isinstance(c, int):
            raise TraceError(f"unsupported work-item index value {v!r}")
        return ItemIndex(c, (0,) * rank, (0,) * rank)

    def __add__(self, o):
        o = ItemIndex.lift(o, len(self.g))
        return ItemIndex(self.const + o.const, [a + b for a, b in zip(self.g, o.g)],
                         [a + b for a, b in zip(self.l, o.l)])

    __radd__ = __add__

    def __neg__(self):
        return ItemIndex(-self.const, [-c for c in self.g], [-c for c in self.l])

    def __sub__(self, o):
        return self + (-ItemIndex.lift(o, len(self.g)))

    def __rsub__(self, o):
        return ItemIndex.lift(o, len(self.g)) - self

    def __mul__(self, o):
        if isinstance(o, (Affine, ItemIndex)):
            varies = any(o.coeffs) if isinstance(o, Affine) else any(o.g) or any(o.l)
            if varies:
                if any(self.g) or any(self.l):
                    raise TraceError("product of two ids")
                return ItemIndex.lift(o, len(self.g)) * self.const
            o = o.const
        k = _index_const(o)
        if not isinstance(k, int):
            raise TraceError("a work-item index may only be multiplied by an integer")
        return ItemIndex(self.const * k, [c * k for c in self.g], [c * k for c in self.l])

    __rmul__ = __mul__

    def _unsupported(self, *_):
        raise TraceError("only + - and * by an integer are supported on work-item ids; comparisons "
                         "and data-dependent control flow inside a scope have no native form")

    __truediv__ = __rtruediv__ = __floordiv__ = __rfloordiv__ = __mod__ = __rmod__ = _unsupported
    __lt__ = __le__ = __gt__ = __ge__ = __eq__ = __ne__ = __bool__ = _unsupported
    __hash__ = None

    def __index__(self):
        if not any(self.g) and not any(self.l):
            return self.const
        raise TraceError("a work-item id was used where a number is needed")

    __int__ = __index__

    def key(self):
        return (self.const, self.g, self.l)

    def __repr__(self):
        terms = [f"{c}*g{i}" for i, c in enumerate(self.g) if c]
        terms += [f"{c}*l{i}" for i, c in enumerate(self.l) if c]
        return " + ".join(terms + ([str(self.const)] if self.const or not terms else []))


# ---------------------------------------------------------------------------
# dtypes
# ---------------------------------------------------------------------------
def dtype_name(dt) -> str:
    """Canonical name ('float32', 'float16', 'bfloat16', 'int8', ...) of a
    NumPy dtype, a torch dtype, a type like np.float32, or a string."""
    if isinstance(dt, str):
        return dt.replace("torch.", "")
    name = getattr(dt, "__name__", None)            # np.float32, float, int
    if name in ("float", "int", "bool"):
        return {"float": "float64", "int": "int64", "bool": "bool"}[name]
    s = str(dt)
    if s.startswith("torch."):
        return s[6:]
    try:
        return np.dtype(dt).name
    except TypeError:
        raise TraceError(f"unknown dtype {dt!r}") from None


_RANK = {"bool": 0, "int8": 1, "uint8": 1, "int16": 2, "uint16": 2, "int32": 3, "uint32": 3,
         "int64": 4, "uint64": 4, "float16": 5, "bfloat16": 5, "float32": 6, "float64": 7}


def promote(a: str, b: str) -> str:
    """Result type of a binary operation between tiles (NumPy's rules for the
    types the kernels use; mixing float16 with bfloat16 gives float32)."""
    if a == b:
        return a
    if {a, b} == {"float16", "bfloat16"}:
        return "float32"
    fa, fb = _RANK[a] >= 5, _RANK[b] >= 5
    if fa != fb:                       # int with float: the float wins if wide enough
        f, i = (a, b) if fa else (b, a)
        if _RANK[f] == 5 and _RANK[i] >= 2:
            return "float32" if _RANK[i] == 2 else "float64"
        return f
    return a if _RANK[a] >= _RANK[b] else b


# ---------------------------------------------------------------------------
# Buffers and views
# ---------------------------------------------------------------------------
class BufferProxy:
    """Stands for an array argument while the body is traced."""

    def __init__(self, index, name, shape, strides, dtype, obj):
        self.index, self.name = index, name
        self.shape, self.strides = tuple(shape), tuple(strides)
        self.dtype_name = dtype
        self.obj = obj

    @property
    def dtype(self):
        try:
            return np.dtype(self.dtype_name)
        except TypeError:
            return self.dtype_name

    @property
    def ndim(self):
        return len(self.shape)

    def _element_index(self, key):
        """key as a tuple of ItemIndex if it addresses one element, else None."""
        if len(key) != self.ndim or any(isinstance(k, slice) or k is None for k in key):
            return None
        group = getattr(self, "group", None)
        if group is None:
            raise TraceError("element access to a buffer outside a kernel body")
        rank = len(group.shape)
        out = []
        for k in key:
            if isinstance(k, IndexExpr):
                raise TraceError("element indices with // or % of the group id have no native form")
            out.append(ItemIndex.lift(k, rank))
        return tuple(out)

    def __getitem__(self, key):
        if not isinstance(key, tuple):
            key = (key,)
        if len(key) > self.ndim:
            raise TraceError(f"too many indices for {self.name}")
        index = self._element_index(key)
        if index is not None:
            return self.group.element_load(self, index)
        starts = []
        for k in key:
            if not isinstance(k, slice):
                raise TraceError("buffers are indexed with slices `a[x:, y:]` inside a kernel")
            if k.step not in (None, 1) or k.stop is not None:
                raise TraceError("only `start:` slices are supported on buffers")
            starts.append(0 if k.start is None else k.start)
        starts += [0] * (self.ndim - len(starts))
        rank = max((len(s.coeffs) for s in starts if isinstance(s, Affine)), default=0)
        return BufferView(self, tuple(s if isinstance(s, IndexExpr) else Affine.lift(s, rank)
                                      for s in starts))

    def __setitem__(self, key, value):
        if value is _ATOMIC_DONE:
            return
        if not isinstance(key, tuple):
            key = (key,)
        index = self._element_index(key)
        if index is None:
            raise TraceError("assignment to a window of a buffer is not supported on the GPU "
                             "path; use group.store (single elements may be assigned)")
        self.group.element_store(self, index, value)

    def __repr__(self):
        return f"<buffer {self.name} {self.shape} {self.dtype_name}>"


class BufferView:
    """`buffer[x:, y:]`: a window that starts at an (affine) offset."""

    def __init__(self, base: BufferProxy, starts):
        self.base, self.starts = base, starts

    @property
    def affine(self):
        """False if a start contains // or % of the group id."""
        return all(isinstance(s, Affine) for s in self.starts)

    @property
    def dtype(self):
        return self.base.dtype

    @property
    def shape(self):
        out = []
        for n, s in zip(self.base.shape, self.starts):
            if not (isinstance(s, Affine) and s.is_const):
                raise TraceError("the shape of a window that depends on the group id is "
                                 "not a number")
            out.append(max(n - s.const, 0))
        return tuple(out)


def _as_view(x) -> BufferView:
    if isinstance(x, BufferView):
        return x
    if isinstance(x, BufferProxy):
        return x[tuple(slice(None) for _ in x.shape)]
    raise TraceError(f"expected a buffer window, got {type(x).__name__}")


# ---------------------------------------------------------------------------
# Tiles: nodes of the traced expression DAG
# ---------------------------------------------------------------------------
_UFUNC_OPS = {"floor_divide": "floordiv", "remainder": "mod", "mod": "mod", "bitwise_and": "and",
              "bitwise_or": "or", "bitwise_xor": "xor", "left_shift": "shl", "right_shift": "shr",
              "less": "lt", "less_equal": "le", "greater": "gt", "greater_equal": "ge",
              "equal": "eq", "not_equal": "ne",
              "add": "add", "subtract": "sub", "multiply": "mul", "true_divide": "div",
              "divide": "div", "exp": "exp", "absolute": "abs", "fabs": "abs", "rint": "rint",
              "negative": "neg", "maximum": "maximum", "minimum": "minimum", "sqrt": "sqrt",
              "log": "log", "tanh": "tanh", "square": "square", "power": "power",
              "floor": "floor", "ceil": "ceil", "trunc": "trunc", "sign": "sign", "exp2": "exp2",
              "log2": "log2", "log10": "log10", "log1p": "log1p", "expm1": "expm1", "sin": "sin",
              "cos": "cos", "reciprocal": "reciprocal"}


def _result_dtype(a: "Tile", b: "Tile") -> str:
    """Python scalars are weak (they adopt the tile's type unless that is an
    integer type and the scalar a float); NumPy scalars and tiles promote."""
    aw, bw = bool(a.attrs.get("weak")), bool(b.attrs.get("weak"))
    if aw and not bw:
        a, b, bw = b, a, True
    elif aw and bw:
        return promote(a.dtype_name, b.dtype_name)
    if bw:
        if _RANK[a.dtype_name] >= 5 or b.dtype_name != "float64":
            return a.dtype_name
        return "float64"
    return promote(a.dtype_name, b.dtype_name)


def _broadcast(a, b):
    try:
        return tuple(np.broadcast_shapes(tuple(a), tuple(b)))
    except ValueError:
        raise TraceError(f"shapes {a} and {b} do not broadcast") from None


class Tile:
    """A value in the per-group program.  `op` is 'load', 'const', an
    elementwise operation, a reduction, 'astype', 'dot', 'transpose', 'clip' or
    'slice'; `args` are Tiles; `attrs` holds the rest."""

    __array_priority__ = 1000
    _counter = 0

    # every node made so far, so that `tile[key] = value` (which changes the tile
    # object in place, as the reference does) can leave what was computed from
    # the tile before reading what the tile held then
    _made = weakref.WeakSet()

    def __init__(self, op, args=(), shape=(), dtype="float32", **attrs):
        self.op, self.args, self.shape = op, tuple(args), tuple(int(s) for s in shape)
        self.dtype_name, self.attrs = dtype, attrs
        Tile._counter += 1
        self.uid = Tile._counter
        Tile._made.add(self)

    def snapshot(self) -> "Tile":
        """What the tile holds now, as a node that a later assignment to the tile
        does not change (a store records this)."""
        return Tile(self.op, self.args, self.shape, self.dtype_name, **self.attrs)

    # -- construction helpers ----------------------------------------------------
    @staticmethod
    def wrap(x, like: "Tile | None" = None) -> "Tile":
        if isinstance(x, Tile):
            return x
        if isinstance(x, np.ndarray) and x.ndim == 0:
            x = x[()]                       # a NumPy scalar that went through a ufunc call
        if isinstance(x, (bool, int, float, np.generic)):
            if isinstance(x, np.generic):
                dt, weak = x.dtype.name, False
            else:
                dt, weak = ("float64" if isinstance(x, float) else "int64"), True
            return Tile("const", (), (), dt, value=float(x), weak=weak,
                        exact=int(x) if isinstance(x, (bool, int, np.integer)) else None)
        raise TraceError(f"cannot use {type(x).__name__} in a tile expression")

    def _binary(self, other, op, reflected=False, as_function=False):
        o = Tile.wrap(other)
        a, b = (o, self) if reflected else (self, o)
        r = Tile(op, (a, b), _broadcast(a.shape, b.shape), _result_dtype(a, b))
        if _all_ndarrays(a, b):
            # plain NumPy arrays (numpy.where's result, tile.mask) and numbers:
            # NumPy's own arithmetic, IEEE results, another plain array
            r.attrs.update(plain=True, ndarray=True, ieee=True)
        elif a.attrs.get("ndarray") and not b.attrs.get("plain") and not as_function:
            # NumPy defers to the tile, whose type has no reflected operators
            # (python/hckernel/kernel_api.py:158-206)
            raise TypeError(f"unsupported operand type(s) for {op}: a plain NumPy array (the result of "
                            f"numpy.where or tile.mask) and a tile; write the tile first")
        elif a.attrs.get("plain") or (a.op == "const" and b.attrs.get("plain")):
            if a.attrs.get("plain") and not b.attrs.get("plain") and b.op != "const" and \
                    op in _NOT_NUMPY_MA_OPERATORS and not as_function:
                # numpy.ma does not define this operator itself: ndarray's runs the
                # NumPy function with the tile converted to its values, whatever
                # their activity (python/hckernel/kernel_api.py:150-151)
                r.attrs["right_values"] = True
            # the left operand is what a NumPy function returned: in the reference a
            # bare numpy.ma array, whose operator gives another one (stored in full);
            # so does the reflected operator of a bare array next to a number
            r.attrs["plain"] = True
        return r

    def __add__(self, o): return self._binary(o, "add")
    def __radd__(self, o): return self._binary(o, "add", True)
    def __sub__(self, o): return self._binary(o, "sub")
    def __rsub__(self, o): return self._binary(o, "sub", True)
    def __mul__(self, o): return self._binary(o, "mul")
    def __rmul__(self, o): return self._binary(o, "mul", True)
    def __truediv__(self, o): return self._true_divide(o, False)
    def __rtruediv__(self, o): return self._true_divide(o, True)

    def _true_divide(self, o, reflected):
        r = self._binary(o, "div", reflected)
        if _RANK[r.dtype_name] < 5:
            raise TraceError("tile / tile on integer tiles is float64 in NumPy, for which there is no "
                             "native kernel (use // for the integer quotient)")
        return r

    # In-place operators are `tile[:] = tile op other` in the reference
    # (python/hckernel/kernel_api.py:142-145): the assignment takes the result's
    # active elements only, so an element whose result is inactive (a zero divisor,
    # an operand that is inactive there) keeps its value and its activity.
    def _in_place(self, other, method):
        if self.attrs.get("plain"):
            raise TraceError("an in-place operator on the result of a NumPy function, a reduction or astype "
                             "is numpy.ma's own in-place operator, which has no native code (write x = x op y)")
        self[:] = method(self, other)
        return self

    def __iadd__(self, o): return self._in_place(o, Tile.__add__)
    def __isub__(self, o): return self._in_place(o, Tile.__sub__)
    def __imul__(self, o): return self._in_place(o, Tile.__mul__)
    def __itruediv__(self, o): return self._in_place(o, Tile.__truediv__)
    def __ifloordiv__(self, o): return self._in_place(o, Tile.__floordiv__)
    def __imod__(self, o): return self._in_place(o, Tile.__mod__)
    def __ipow__(self, o): return self._in_place(o, Tile.__pow__)
    def __iand__(self, o): return self._in_place(o, Tile.__and__)
    def __ior__(self, o): return self._in_place(o, Tile.__or__)
    def __ixor__(self, o): return self._in_place(o, Tile.__xor__)
    def __ilshift__(self, o): return self._in_place(o, Tile.__lshift__)
    def __irshift__(self, o): return self._in_place(o, Tile.__rshift__)

    def __neg__(self): return Tile("neg", (self,), self.shape, self.dtype_name, **self._plain_kw())
    def __abs__(self): return Tile("abs", (self,), self.shape, self.dtype_name, **self._plain_kw())

    def _plain_kw(self):
        if self.attrs.get("ndarray"):
            return {"plain": True, "ndarray": True}
        return {"plain": True} if self.attrs.get("plain") else {}

    # The rest of the operators the reference's wrapper forwards to NumPy
    # (python/hckernel/kernel_api.py:157-180).  Comparisons give bool tiles;
    # // % & | ^ << >> keep the operands' type.  Which of them have a native
    # kernel is the binder's business (today: all of them on int32 tiles).
    def __floordiv__(self, o): return self._binary(o, "floordiv")
    def __rfloordiv__(self, o): return self._binary(o, "floordiv", True)
    def __mod__(self, o): return self._binary(o, "mod")
    def __rmod__(self, o): return self._binary(o, "mod", True)
    def __and__(self, o): return self._binary(o, "and")
    def __rand__(self, o): return self._binary(o, "and", True)
    def __or__(self, o): return self._binary(o, "or")
    def __ror__(self, o): return self._binary(o, "or", True)
    def __xor__(self, o): return self._binary(o, "xor")
    def __rxor__(self, o): return self._binary(o, "xor", True)
    def __lshift__(self, o): return self._binary(o, "shl")
    def __rlshift__(self, o): return self._binary(o, "shl", True)
    def __rshift__(self, o): return self._binary(o, "shr")
    def __rrshift__(self, o): return self._binary(o, "shr", True)

    def _compare(self, other, op):
        o = Tile.wrap(other)
        r = Tile(op, (self, o), _broadcast(self.shape, o.shape), "bool",
                 operand_dtype=_result_dtype(self, o))
        if _all_ndarrays(self, o):
            r.attrs.update(plain=True, ndarray=True)
        elif self.attrs.get("ndarray") and not o.attrs.get("plain"):
            pass                                # the tile's mirrored comparison: a tile
        elif self.attrs.get("plain"):
            r.attrs["plain"] = True
        return r

    def __lt__(self, o): return self._compare(o, "lt")
    def __le__(self, o): return self._compare(o, "le")
    def __gt__(self, o): return self._compare(o, "gt")
    def __ge__(self, o): return self._compare(o, "ge")
    def __eq__(self, o): return self._compare(o, "eq")
    def __ne__(self, o): return self._compare(o, "ne")
    __hash__ = object.__hash__

    def __invert__(self):
        raise TraceError("~tile: the reference's tile type has no __invert__ either (its wrapper "
                         "installs __inv__, which Python never calls)")

    @property
    def mask(self):
        """Which elements are active (True = active: the reference inverts
        numpy.ma's polarity, python/hckernel/kernel_api.py:117-119).  A plain
        bool array, every element of which is a value: stored in full."""
        if self.attrs.get("plain"):
            raise TraceError("the mask of a bare numpy.ma array (the result of a NumPy function, a "
                             "reduction or astype) has numpy.ma's polarity, not a tile's: no native code")
        return Tile("active", (self,), self.shape, "bool", plain=True, ndarray=True)

    def compressed(self):
        raise TraceError("tile.compressed(): a 1-D array of the active elements only; its length "
                         "depends on the data, which a traced body cannot express (store the tile "
                         "and tile.mask instead)")

    def __matmul__(self, o):
        return _dot(self, Tile.wrap(o))

    # -- NumPy protocol -----------------------------------------------------------
    def __array_ufunc__(self, ufunc, method, *inputs, **kwargs):
        """A NumPy function of tiles.  In the reference such a call reaches
        numpy.ma through the tile wrapper's forwarded attributes
        (python/hckernel/kernel_api.py:150-151): the function is applied to the
        values, deactivated or not, numpy.ma's __array_wrap__ puts its fill
        value where the function's domain fails (sqrt of a negative number: 0,
        log of a non-positive one: 1, a division by zero: 1), and the result is
        a bare numpy.ma array, which a store writes out in full.  The nodes made
        here carry func=True (called as a function) and plain=True (not a tile:
        stored in full)."""
        op = _UFUNC_OPS.get(ufunc.__name__)
        if method != "__call__" or op is None or kwargs:
            raise TraceError(f"numpy.{ufunc.__name__} ({method}) is not supported in a GPU kernel")

        def plain(t: "Tile") -> "Tile":
            t.attrs["plain"] = t.attrs["func"] = True
            t.attrs.pop("pow", None)
            if _all_ndarrays(*(Tile.wrap(v) for v in inputs)):
                # a NumPy function of plain arrays is plain NumPy: no domains, IEEE results
                t.attrs["ndarray"] = t.attrs["ieee"] = True
            return t

        if len(inputs) == 1:
            x = Tile.wrap(inputs[0])
            if op == "square":
                return plain(x * x)
            return plain(Tile(op, (x,), x.shape, x.dtype_name))
        a, b = inputs
        if isinstance(a, np.ndarray) and a.ndim == 0:
            a = a[()]                           # (a NumPy scalar's comparison arrives as a 0-d array)
        if isinstance(a, np.generic) and isinstance(b, Tile) and not b.attrs.get("plain"):
            # `np.float32(2) * tile`: the scalar's operator arrives here.  The
            # reference's tile type has no reflected operators and is no array, so
            # there the arithmetic operators raise TypeError and the comparisons
            # fall back to the tile's own, mirrored.  (Next to a bare numpy.ma array
            # the scalar's operator is the NumPy function: computed on the values,
            # deactivated or not.)
            refl = {"lt": "__gt__", "le": "__ge__", "gt": "__lt__", "ge": "__le__", "eq": "__eq__",
                    "ne": "__ne__"}.get(op)
            if refl is not None and _called_by_an_operator():
                return getattr(b, refl)(a)
            if _called_by_an_operator():
                    raise TypeError(f"unsupported operand type(s) for numpy.{ufunc.__name__}: "
                                f"'{type(a).__name__}' and a tile (write the tile first, or a Python number)")
        if op == "power":
            r = Tile.wrap(a) ** b
            if r is a:                          # exponent 1: a new node, the same values
                r = Tile.wrap(a) * Tile.wrap(np.dtype(r.dtype_name).type(1))
            return plain(r)
        if op in ("lt", "le", "gt", "ge", "eq", "ne"):
            a, b = Tile.wrap(a), Tile.wrap(b)
            return plain(a._compare(b, op))
        if isinstance(a, Tile):
            return plain(a._binary(b, op, as_function=True))
        return plain(Tile.wrap(b)._binary(a, op, reflected=True, as_function=True))

    def __array_function__(self, func, types, args, kwargs):
        name = func.__name__
        if name == "dot" and len(args) == 2:
            return _dot(Tile.wrap(args[0]), Tile.wrap(args[1]))
        if name == "clip":
            x = Tile.wrap(args[0])
            lo = kwargs.get("a_min", args[1] if len(args) > 1 else None)
            hi = kwargs.get("a_max", args[2] if len(args) > 2 else None)
            return Tile("clip", (x,), x.shape, x.dtype_name, lo=float(lo), hi=float(hi), func=True,
                        **{"plain": True, **x._plain_kw()})
        if name in ("amax", "max", "sum", "amin", "min"):
            x = Tile.wrap(args[0])
            return x._reduce({"amax": "max", "amin": "min"}.get(name, name),
                             kwargs.get("axis", args[1] if len(args) > 1 else None),
                             kwargs.get("keepdims", False))
        if name in ("mean", "var", "std"):
            extra = set(kwargs) - {"axis", "keepdims", "ddof"}
            if extra or len(args) > 2:
                raise TraceError(f"numpy.{name}: only axis, keepdims and ddof are supported")
            if name == "mean" and "ddof" in kwargs:
                raise TraceError("numpy.mean takes no ddof")
            kw = dict(kwargs)
            if len(args) > 1:
                kw["axis"] = args[1]
            return getattr(Tile.wrap(args[0]), name)(**kw)
        if name == "where" and len(args) == 3:
            # numpy.where converts its arguments to plain arrays (the values, whatever
            # their activity) and returns one
            c, a, b = (Tile.wrap(v) for v in args)
            if c.dtype_name != "bool":
                raise TraceError("numpy.where: the condition must be a comparison of tiles")
            shape = _broadcast(_broadcast(c.shape, a.shape), b.shape)
            return Tile("where", (c, a, b), shape, _result_dtype(a, b), plain=True, func=True, ndarray=True)
        if name == "transpose" and len(args) == 1:
            return Tile.wrap(args[0]).T
        if name == "norm" and kwargs.get("ord", args[1] if len(args) > 1 else None) is None:
            x = Tile.wrap(args[0])             # numpy.linalg.norm: the 2-norm along an axis
            return x._reduce("norm", kwargs.get("axis", args[2] if len(args) > 2 else None),
                             kwargs.get("keepdims", False))
        raise TraceError(f"numpy.{name} is not supported in a GPU kernel")

    # -- methods kernels use ---------------------------------------------------------
    def _reduce(self, op, axis, keepdims):
        if axis is None:
            axes = tuple(range(len(self.shape)))
        else:
            axes = (axis,) if isinstance(axis, int) else tuple(axis)
        axes = tuple(a % len(self.shape) for a in axes)
        shape = tuple((1 if i in axes else n) for i, n in enumerate(self.shape)) if keepdims \
            else tuple(n for i, n in enumerate(self.shape) if i not in axes)
        # (plain: a reduction of a tile is a bare numpy.ma array, not a tile,
        # python/hckernel/kernel_api.py:150-151)
        return Tile(op, (self,), shape, self.dtype_name, axes=axes, keepdims=bool(keepdims),
                    **{"plain": True, **self._plain_kw()})

    def max(self, axis=None, keepdims=False): return self._reduce("max", axis, keepdims)
    def min(self, axis=None, keepdims=False): return self._reduce("min", axis, keepdims)
    def sum(self, axis=None, keepdims=False): return self._reduce("sum", axis, keepdims)

    # mean, var and std as numpy.ma computes them on a tile (numpy/ma/core.py:
    # MaskedArray.mean / var / std; a tile's mask is always an array, so the
    # masked branches run): the mean is the sum over the active elements divided
    # by their number, a domained division that deactivates a result that is not
    # finite; the variance divides the sum of the centred squares by that number
    # less ddof and is active wherever that is positive, whatever the division
    # did; the standard deviation is numpy.ma.sqrt of it.  `count` is a
    # reduction node of its own (the number of active elements, as fp32);
    # hc_amd.binding turns it into a constant where nothing can deactivate an
    # element.
    def _count(self, axis, keepdims):
        r = self._reduce("count", axis, keepdims)
        r.dtype_name = "float32"
        return r

    def mean(self, axis=None, keepdims=False):
        half = self.dtype_name == "float16"     # NumPy adds up fp16 data in fp32
        x = self.astype("float32") if half else self
        if x.dtype_name != "float32":
            raise TraceError("mean of a tile: float32 and float16 tiles only (cast first)")
        total = x._reduce("sum", axis, keepdims)
        if self.attrs.get("ndarray"):           # numpy.mean of a plain array: the sum over the number
            r = Tile("div", (total, x._count(axis, keepdims)), total.shape, "float32", plain=True,
                     ndarray=True, ieee=True)
        else:
            r = Tile("div", (total, x._count(axis, keepdims)), total.shape, "float32", ma=True, plain=True)
        return r.astype("float16") if half else r

    def var(self, axis=None, keepdims=False, ddof=0):
        if self.dtype_name != "float32":
            raise TraceError("var/std of a tile: float32 tiles only (cast first)")
        if not isinstance(ddof, (int, np.integer)) or ddof < 0:
            raise TraceError("var/std of a tile: ddof must be a non-negative integer")
        centred = self - self.mean(axis, True)
        total = (centred * centred)._reduce("sum", axis, keepdims)
        count = self._count(axis, keepdims)
        if ddof:
            count = count - np.float32(ddof)
        return Tile("vardiv", (total, count), total.shape, "float32", plain=True)

    def std(self, axis=None, keepdims=False, ddof=0):
        v = self.var(axis, keepdims, ddof)
        return Tile("masqrt", (v,), v.shape, v.dtype_name, plain=True)

    def __pow__(self, e):
        if isinstance(e, (int, float, np.generic)) and not isinstance(e, bool) and self.attrs.get("ndarray"):
            # a plain array: ndarray.__pow__ calls numpy.square, numpy.sqrt for these exponents
            if float(e) == 2.0:
                return self * self
            if float(e) == 0.5:
                return Tile("sqrt", (self,), self.shape, self.dtype_name, func=True, ieee=True,
                            **self._plain_kw())
        if isinstance(e, (int, float, np.generic)) and not isinstance(e, bool):
            # pow=True: numpy.ma.power deactivates results that are not finite
            if float(e) == 2.0:
                r = self * self                 # what numpy.power does for this exponent
                r.attrs["pow"] = True
                return r
            if float(e) == 0.5:
                return Tile("sqrt", (self,), self.shape, self.dtype_name, pow=True, **self._plain_kw())
            if float(e) == 1.0:
                return self
        raise TraceError("tile ** e: only the exponents 2, 1 and 0.5 have native code")

    def astype(self, dt):
        name = dtype_name(dt)
        if name == self.dtype_name and self.attrs.get("plain"):
            return self
        # (a tile's astype is numpy.ma's, python/hckernel/kernel_api.py:150-151:
        # the result is a bare numpy.ma array, not a tile)
        return Tile("astype", (self,), self.shape, name, **{"plain": True, **self._plain_kw()})

    @property
    def T(self):
        if len(self.shape) != 2:
            raise TraceError(".T needs a 2-D tile")
        # (an attribute the reference's wrapper forwards to numpy.ma,
        # python/hckernel/kernel_api.py:150-151: the result is a bare array)
        return Tile("transpose", (self,), self.shape[::-1], self.dtype_name,
                    **{"plain": True, **self._plain_kw()})

    @property
    def dtype(self):
        try:
            return np.dtype(self.dtype_name)
        except TypeError:
            return self.dtype_name

    @property
    def ndim(self):
        return len(self.shape)

    def __getitem__(self, key):
        if not isinstance(key, tuple):
            key = (key,)
        n_old = sum(1 for k in key if k is not None)
        key = key + (slice(None),) * (len(self.shape) - n_old)
        shape, dims = [], iter(self.shape)
        for k in key:
            if k is None:                      # numpy.newaxis
                shape.append(1)
            elif isinstance(k, slice):
                shape.append(len(range(*k.indices(next(dims)))))
            else:
                int(k)
                next(dims)
        norm = tuple("new" if k is None else
                     (k.start, k.stop, k.step) if isinstance(k, slice) else int(k) for k in key)
        return Tile("slice", (self,), shape, self.dtype_name, key=norm, **self._plain_kw())

    def __setitem__(self, key, value):
        """`tile[key] = value` with a static key: the tile object becomes the
        updated tile (python/hckernel/kernel_api.py:125-131 assigns in place and
        marks the elements active).  The old contents stay reachable as the first
        argument of the new node."""
        if not isinstance(key, tuple):
            key = (key,)
        if any(k is None or k is Ellipsis for k in key) or len(key) > len(self.shape):
            raise TraceError("tile assignment: plain integer / slice keys only")
        norm = []
        for k, n in zip(key + (slice(None),) * (len(self.shape) - len(key)), self.shape):
            if isinstance(k, slice):
                start, stop, step = k.indices(n)
                if step != 1:
                    raise TraceError("tile assignment: unit-step slices only")
                norm.append((start, max(stop, start)))
            else:
                i = int(k)                       # raises for ids that are not numbers
                if not -n <= i < n:
                    raise TraceError(f"tile assignment: index {i} out of range for extent {n}")
                norm.append(i % n)
        if self.attrs.get("plain"):
            raise TraceError("assignment into the result of a NumPy function, a reduction or astype (a bare "
                             "numpy.ma array) is numpy.ma's own __setitem__, which has no native code")
        old = self.snapshot()
        for node in list(Tile._made):           # what was computed from the tile so far keeps reading the old contents
            if node is not old and any(a is self for a in node.args):
                node.args = tuple(old if a is self else a for a in node.args)
        value = Tile.wrap(value)
        self.op, self.args = "update", (old, old if value is self else value)
        self.attrs = {"key": tuple(norm)}
        Tile._counter += 1
        self.uid = Tile._counter

    def reshape(self, *shape):
        shape = shape[0] if len(shape) == 1 and isinstance(shape[0], Iterable) else shape
        shape = tuple(int(s) for s in shape)
        if -1 in shape:
            known = -math.prod(shape)
            shape = tuple(math.prod(self.shape) // known if s == -1 else s for s in shape)
        if math.prod(shape) != math.prod(self.shape):
            raise TraceError("reshape changes the number of elements")
        return Tile("reshape", (self,), shape, self.dtype_name, **self._plain_kw())

    def __bool__(self):
        raise TraceError("the value of a tile is not known while the kernel is traced; "
                         "data-dependent control flow is not supported")

    def __iter__(self):
        raise TraceError("tiles cannot be iterated in a GPU kernel")

    def __repr__(self):
        return f"<tile {self.op} {self.shape} {self.dtype_name}>"


def _called_by_an_operator() -> bool:
    """The NumPy function that reached Tile.__array_ufunc__ was started by an
    operator of a NumPy scalar (`numpy.float32(2) * tile`), not written as a
    call (`numpy.multiply(numpy.float32(2), tile)`).  NumPy gives no other way
    to tell the two apart, and the reference raises for the first only: the
    instruction the body's frame is at says which it is."""
    import dis
    import sys
    frame = sys._getframe(2)                   # the caller of __array_ufunc__'s caller (NumPy has no frame)
    name = dis.opname[frame.f_code.co_code[frame.f_lasti]]
    return name.startswith(("BINARY_", "INPLACE_", "COMPARE_OP"))


_NOT_NUMPY_MA_OPERATORS = ("mod", "and", "or", "xor", "shl", "shr")


def _all_ndarrays(*operands: Tile) -> bool:
    """Plain NumPy arrays and numbers only, at least one array: no numpy.ma
    array among them, so NumPy's own arithmetic applies."""
    return any(t.attrs.get("ndarray") for t in operands) and \
        all(t.attrs.get("ndarray") or t.op == "const" for t in operands)


def _dot(a: Tile, b: Tile) -> Tile:
    if len(a.shape) == 2 and len(b.shape) == 1 and a.shape[1] == b.shape[0]:
        # matrix times vector: the rows' sums of products (NumPy computes on the
        # data, where an inactive element is the 0 a load puts there,
        # python/hckernel/kernel_api.py:223-224,301-303: the same sum)
        return a._binary(b, "mul")._reduce("sum", 1, False)
    if len(a.shape) != 2 or len(b.shape) != 2 or a.shape[1] != b.shape[0]:
        raise TraceError(f"dot of shapes {a.shape} and {b.shape}")
    return Tile("dot", (a, b), (a.shape[0], b.shape[1]), promote(a.dtype_name, b.dtype_name))


# ---------------------------------------------------------------------------
# The group object handed to the kernel body
# ---------------------------------------------------------------------------
class CurrentGroup:
    """Tracing group (python/hckernel/kernel_api.py:255-434).  `id` and
    `work_offset` are symbolic; `shape` and `size` are numbers."""

    def __init__(self, group_shape, subgroup_size):
        self._shape = tuple(int(s) for s in group_shape)
        self._subgroup_size = subgroup_size
        rank = len(self._shape)
        self._id = tuple(Affine(0, [1 if j == i else 0 for j in range(rank)])
                         for i in range(rank))
        self.stores = []          # (BufferView, Tile) in program order
        self.atomics = []         # (BufferProxy, element index, Tile) atomic additions
        self.cell_stores = []     # (BufferProxy, index of Affine, scalar Tile, add to the old value?)
        self.mapped_stores = []   # (BufferView, Tile, index function) scattered stores
        self.id_stores = []       # (BufferProxy, ItemIndex per dim, value ItemIndex, per work-item?)
        self._ring = []           # greenlets of the subgroup scope that is running
        self._turn = 0
        self._in_workitems = False

    @property
    def id(self):
        return self._id

    @property
    def shape(self):
        return self._shape

    @property
    def size(self):
        return math.prod(self._shape)

    @property
    def work_offset(self):
        return tuple(g * s for g, s in zip(self._id, self._shape))

    # -- loads and stores ----------------------------------------------------------
    def load(self, array, shape, mapping=None):
        if not isinstance(shape, Iterable):
            shape = (shape,)
        shape = tuple(int(s) for s in shape)
        if isinstance(array, Tile):
            # a tile re-read at another shape: cropped, or padded with inactive
            # (zero) elements, python/hckernel/kernel_api.py:312-314
            if mapping is not None:
                raise TraceError("a mapping on a load from a tile has no native kernel")
            if len(shape) != len(array.shape):
                raise TraceError(f"load shape {shape} does not match the rank of the tile")
            if shape == array.shape:
                return array
            return Tile("window", (array,), shape, array.dtype_name)
        view = _as_view(array)
        if mapping is not None:
            if not isinstance(mapping, Mapping):
                raise TraceError("mapping must come from create_mapping")
            return Tile("mapped_load", (), shape, view.base.dtype_name, view=view,
                        mapping=mapping.func)
        if not view.affine:
            raise TraceError("window offsets that use // or % of the group id are supported "
                             "on mapped loads and stores only")
        if len(shape) != view.base.ndim:
            raise TraceError(f"load shape {shape} does not match the rank of {view.base.name}")
        return Tile("load", (), shape, view.base.dtype_name, view=view)

    def vload(self, array, shape, mapping=None):
        """A load into a vector: same result as load, but the shape has to be
        static (numbers, group.shape, literal symbols and tunables), as the
        reference specifies (docs/langref.md:226-243; a vector is register
        resident, mlir/lib/Transforms/LowerHKernel.cpp:1056-1083)."""
        dims = shape if isinstance(shape, Iterable) else (shape,)
        if not all(is_static(d) for d in dims):
            raise TraceError("vload needs a static shape: numbers, group.shape, literal symbols "
                             "and tunables, not buffer dimensions or other values that are only "
                             "known at launch (use load for those)")
        t = self.load(array, shape, mapping)
        t.attrs["vector"] = True
        return t

    def store(self, dst, src, mapping=None):
        view = _as_view(dst)
        if mapping is not None:
            if not isinstance(mapping, Mapping):
                raise TraceError("mapping must come from create_mapping")
            self.mapped_stores.append((view, Tile.wrap(src).snapshot(), mapping.func))
            return
        if not view.affine:
            raise TraceError("window offsets that use // or % of the group id are supported "
                             "on mapped loads and stores only")
        self.stores.append((view, Tile.wrap(src).snapshot()))

    # -- allocators ------------------------------------------------------------------
    def _alloc(self, shape, dtype, value):
        if not isinstance(shape, Iterable):
            shape = (shape,)
        t = Tile("const", (), (), dtype_name(dtype), value=float(value), weak=False)
        return Tile("full", (t,), shape, dtype_name(dtype), value=float(value))

    def empty(self, shape, dtype): return self._alloc(shape, dtype, 0)
    def zeros(self, shape, dtype): return self._alloc(shape, dtype, 0)
    def ones(self, shape, dtype): return self._alloc(shape, dtype, 1)
    def full(self, shape, dtype, fill_value): return self._alloc(shape, dtype, fill_value)
    vempty, vzeros, vones, vfull = empty, zeros, ones, full

    def vec(self, src, shape=None):
        src = Tile.wrap(src)
        if shape is None or tuple(shape) == src.shape:
            return src
        return src[tuple(slice(0, s) for s in shape)]

    # -- nested scopes -----------------------------------------------------------------
    # A subgroup scope is run as the reference's simulator runs it
    # (python/hckernel/kernel_api.py:378-395,420-431): the number of subgroups of
    # a group is a number at trace time, so the body is executed once per
    # subgroup id, in order, each as a greenlet, and barrier() hands over to the
    # next one.  What the bodies do to tiles (slices, reductions, element
    # assignment into workgroup tiles, stores) lands in the same traced program;
    # hc_amd.binding then folds per-subgroup partial results back into whole-row
    # operations where a hand-written kernel does the same work.
    #
    # A work-item scope is traced once with symbolic local ids: a per-work-item
    # value is the element of a group-shaped tile that belongs to the work-item,
    # `a[wi.global_id()]` is that element of the group's tile of `a`, and
    # `out[wi.global_id()] = v` stores the tile.  Statements execute for the whole
    # group in program order, which is what barrier() asks for.
    MAX_SUBGROUPS = 4096

    def subgroups(self, func):
        ranges = [range(v) for v in self._shape[:-1]]
        ranges.append(range(-(-self._shape[-1] // self._subgroup_size)))

        def run():
            from greenlet import greenlet
            if self._ring or self._in_workitems:
                raise TraceError("nested scopes are not supported")
            ids = list(itertools.product(*ranges))
            if len(ids) > self.MAX_SUBGROUPS:
                raise TraceError(f"{len(ids)} subgroups per group: too many to trace one by one")

            def task(sgid):
                func(CurrentSubGroup(self._subgroup_size, sgid))

            self._ring = [greenlet(functools.partial(task, i)) for i in ids]
            self._turn = 0
            try:
                for t in list(self._ring):
                    t.switch()
            finally:
                self._ring, self._turn = [], 0

        return run

    def workitems(self, func):
        rank = len(self._shape)

        def unit(d):
            return tuple(1 if j == d else 0 for j in range(rank))

        def run():
            if self._ring or self._in_workitems:
                raise TraceError("nested scopes are not supported")
            zero = (0,) * rank
            lid = tuple(ItemIndex(0, zero, unit(d)) for d in range(rank))
            gid = tuple(ItemIndex(0, tuple(self._shape[d] * c for c in unit(d)), unit(d))
                        for d in range(rank))
            self._in_workitems = True
            try:
                func(CurrentWorkitem(lid, gid))
            finally:
                self._in_workitems = False

        return run

    def barrier(self):
        n = len(self._ring)
        if n <= 1:
            return None
        self._turn = (self._turn + 1) % n
        self._ring[self._turn].switch()
        return None

    # -- single elements of buffers ------------------------------------------------------
    def _is_global_id(self, index, proxy):
        """index addresses, per buffer dim d, global id d (buffer rank == work rank)."""
        rank = len(self._shape)
        if proxy.ndim != rank:
            return False
        for d, ix in enumerate(index):
            want_g = tuple(self._shape[d] if j == d else 0 for j in range(rank))
            want_l = tuple(1 if j == d else 0 for j in range(rank))
            if ix.const != 0 or ix.g != want_g or ix.l != want_l:
                return False
        return True

    def element_load(self, proxy, index):
        if not self._in_workitems:
            raise TraceError("reading single buffer elements is supported inside a work-item "
                             "scope only (use group.load elsewhere)")
        if not self._is_global_id(index, proxy):
            raise TraceError(f"{proxy.name}[{', '.join(map(repr, index))}]: inside a work-item "
                             "scope a buffer is read at wi.global_id() only")
        return self.load(proxy[tuple(slice(o, None) for o in self.work_offset)], self._shape)

    def element_store(self, proxy, index, value):
        if isinstance(value, Tile) and value.shape == self._shape and self._in_workitems:
            if not self._is_global_id(index, proxy):
                raise TraceError(f"{proxy.name}[...] = value: inside a work-item scope a value "
                                 "is stored at wi.global_id() only")
            self.store(proxy[tuple(slice(o, None) for o in self.work_offset)], value)
            return
        if isinstance(value, Tile) and value.shape == () and not self._in_workitems and \
                all(not any(i.l) for i in index):
            # `out[f(group id)] = tile.sum()`: one result per group
            rank = len(self._shape)
            self.cell_stores.append((proxy, tuple(Affine(i.const, i.g[:rank]) for i in index), value, False))
            return
        if isinstance(value, Tile):
            raise TraceError("only ids, numbers, per-work-item values and (at group level) reductions "
                             "of whole tiles may be assigned to a buffer element")
        rank = len(self._shape)
        if isinstance(value, (float, np.floating)) and float(value) != int(value):
            raise TraceError("only integers and ids may be assigned to a buffer element")
        if isinstance(value, (float, np.floating)):
            value = int(value)
        self.id_stores.append((proxy, index, ItemIndex.lift(value, rank), self._in_workitems))


class CurrentGroup1(CurrentGroup):
    pass


class CurrentGroup2(CurrentGroup):
    pass


class CurrentGroup3(CurrentGroup):
    pass

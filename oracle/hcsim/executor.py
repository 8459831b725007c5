"""Host executor: runs a kernel body group by group on NumPy arrays
(test infrastructure only).

Restates python/hckernel/kernel_sim.py (decorator, symbol binding, group loop)
and the group object of python/hckernel/kernel_api.py:231-434.
"""

from __future__ import annotations

import functools
import inspect
import itertools
import math
import types
import typing
from collections.abc import Iterable

import numpy as np
import sympy
from greenlet import greenlet

from .tiles import Mapping, Tile

DEFAULT_GROUP_LAST_DIM = 64   # kernel_sim.py:9
DEFAULT_SUBGROUP_SIZE = 16    # kernel_sim.py:10


# ---------------------------------------------------------------------------
# Symbols, type names, annotations (indexing.py:14-38, typename.py:12-29,
# kernel_api.py:35-40,437-447)
# ---------------------------------------------------------------------------
class _SymbolSpace:
    def __getattr__(self, name):
        return sympy.Symbol(name, integer=True)


sym = _SymbolSpace()


class Typename:
    def __init__(self, name):
        self.name = name


class _TypenameSpace:
    def __init__(self):
        self._known = {}

    def __getattr__(self, name):
        return self._known.setdefault(name, Typename(name))


typename = _TypenameSpace()


class TunableParam:
    def __init__(self, sym, default, vals, strategy=None):
        self.sym, self.default, self.vals, self.strategy = sym, default, vals, strategy


class Buffer(type):
    """Buffer[d0, ..., dtype] -> annotation class carrying shape and dtype."""

    def __class_getitem__(cls, spec):
        assert len(spec) > 0, "Invalid shape and dtype"
        return type("Buffer", (cls,), {"shape": tuple(spec[:-1]), "dtype": spec[-1]})


def atomic_ref(a):
    # Groups run one after another, so a plain read-modify-write is atomic
    # (kernel_api.py:450-451).
    return a


# ---------------------------------------------------------------------------
# Scopes
# ---------------------------------------------------------------------------
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


def _ceil_div(a, b):
    return (a + b - 1) // b


class CurrentGroup:
    def __init__(self, group_shape, subgroup_size):
        self._shape = tuple(group_shape)
        self._sg = subgroup_size
        self._group_id = None
        self._ring = []      # greenlets of the scope that is running
        self._turn = 0

    # -- geometry (kernel_api.py:278-295) -------------------------------------
    @property
    def id(self):
        return self._group_id

    @property
    def shape(self):
        return self._shape

    @property
    def size(self):
        return math.prod(self._shape)

    @property
    def work_offset(self):
        return tuple(s * g for s, g in zip(self._shape, self._group_id))

    # -- masked tile load / store (kernel_api.py:297-345) -----------------------
    def load(self, array, shape, mapping=None):
        if not isinstance(shape, Iterable):
            shape = (shape,)
        shape = tuple(int(s) for s in shape)
        tile = Tile(np.zeros(shape, dtype=array.dtype), active=False)
        if mapping is not None:
            bounds = array.shape
            for idx in np.ndindex(*shape):
                src = mapping.func(*idx)
                if all(0 <= i < b for i, b in zip(src, bounds)):
                    tile[idx] = array[src]
        else:
            win = tuple(slice(0, min(a, s)) for a, s in zip(array.shape, shape))
            tile[win] = array[win]
        return tile

    def vload(self, array, shape, mapping=None):
        return self.load(array, shape, mapping)

    def store(self, dst, src, mapping=None):
        masked = isinstance(src, Tile)
        if mapping is not None:
            bounds = dst.shape
            for idx in np.ndindex(*src.shape):
                to = mapping.func(*idx)
                if not all(0 <= i < b for i, b in zip(to, bounds)):
                    continue
                if masked:
                    if src.mask[idx]:
                        dst[to] = src.data[idx]
                else:
                    dst[to] = src[idx]
            return
        win = tuple(slice(0, min(a, b)) for a, b in zip(src.shape, dst.shape))
        if masked:
            dst[win] = np.where(src.mask[win], src.data[win], dst[win])
        else:
            dst[win] = src[win]

    # -- allocators: all elements active (kernel_api.py:347-376,433-434) --------
    def _alloc(self, shape, dtype, value):
        return Tile(np.full(shape, value, dtype=dtype), active=True)

    def empty(self, shape, dtype):
        return self._alloc(shape, dtype, 0)

    def zeros(self, shape, dtype):
        return self._alloc(shape, dtype, 0)

    def ones(self, shape, dtype):
        return self._alloc(shape, dtype, 1)

    def full(self, shape, dtype, fill_value):
        return self._alloc(shape, dtype, fill_value)

    vempty, vzeros, vones, vfull = empty, zeros, ones, full

    def vec(self, src, shape=None):
        shape = src.shape if shape is None else shape
        return src.copy()[tuple(slice(0, s) for s in shape)]

    # -- nested scopes and barrier (kernel_api.py:378-431) ----------------------
    def _run_scope(self, ids, make_arg, body):
        assert not self._ring and self._turn == 0
        self._ring = [greenlet(functools.partial(body, make_arg(i))) for i in ids]
        for task in list(self._ring):
            task.switch()
        self._ring = []
        self._turn = 0

    def subgroups(self, func):
        ranges = [range(v) for v in self._shape[:-1]]
        ranges.append(range(_ceil_div(self._shape[-1], self._sg)))

        def run():
            self._run_scope(itertools.product(*ranges),
                            lambda sgid: CurrentSubGroup(self._sg, sgid), func)

        return run

    def workitems(self, func):
        def make(lid):
            gid = tuple(g * s + l for g, s, l in zip(self._group_id, self._shape, lid))
            return CurrentWorkitem(lid, gid)

        def run():
            self._run_scope(itertools.product(*(range(v) for v in self._shape)),
                            make, func)

        return run

    def barrier(self):
        # Hand control to the next task of the ring: every task reaches phase k
        # before any enters k+1 (test_kernel_sim.py:287-320,347-379).
        n = len(self._ring)
        if n <= 1:
            return
        self._turn = (self._turn + 1) % n
        self._ring[self._turn].switch()


class CurrentGroup1(CurrentGroup):
    pass


class CurrentGroup2(CurrentGroup):
    pass


class CurrentGroup3(CurrentGroup):
    pass


# ---------------------------------------------------------------------------
# Symbol binding from annotations (kernel_sim.py:34-127)
# ---------------------------------------------------------------------------
def _bind(subs, symbol, value):
    if symbol in subs:
        assert subs[symbol] == value, (
            f"Symbol value conflict for {symbol}: {subs[symbol]} and {value}")
    else:
        subs[symbol] = value


def _binder_for(position, ann):
    """Returns f(subs, args) for one annotated parameter, or None."""
    # Scope annotations bind nothing.  They are recognised by name as well as
    # by identity so that a body annotated with another package's classes of
    # the same names (the GPU front-end's) runs here unchanged.
    if ann in (CurrentGroup, CurrentSubGroup, CurrentWorkitem) or \
            getattr(ann, "__name__", "").startswith(("CurrentGroup", "CurrentSubGroup",
                                                     "CurrentWorkitem")):
        return None
    if isinstance(ann, sympy.Symbol):
        return lambda subs, args: _bind(subs, ann, args[position])
    is_tuple = typing.get_origin(ann) is tuple or isinstance(ann, tuple)
    if is_tuple:
        parts = typing.get_args(ann) if typing.get_origin(ann) is tuple else ann

        def bind_tuple(subs, args):
            val = args[position]
            assert isinstance(val, Iterable) and len(val) == len(parts)
            for s, v in zip(parts, val):
                if isinstance(s, sympy.Symbol):
                    _bind(subs, s, v)

        return bind_tuple
    if isinstance(ann, type) and (issubclass(ann, Buffer) or
                                  (ann.__name__ == "Buffer" and hasattr(ann, "shape"))):
        def bind_buffer(subs, args):
            val = args[position]
            assert len(val.shape) == len(ann.shape)
            for s, v in zip(ann.shape, val.shape):
                if isinstance(s, sympy.Symbol):
                    _bind(subs, s, v)

        return bind_buffer
    raise AssertionError(f"Unsupported annotation: {type(ann)} {ann}")


def _collect_binders(func):
    ann = inspect.get_annotations(func)
    binders = []
    # the first parameter is the group: argument i of the call is parameter i+1
    for i, name in enumerate(inspect.signature(func).parameters):
        if name in ann and ann[name] is not None:
            b = _binder_for(i - 1, ann[name])
            if b is not None:
                binders.append(b)
    return binders


def _to_int_dims(expr, subs):
    if isinstance(expr, Iterable):
        return tuple(_to_int_dims(e, subs) for e in expr)
    if isinstance(expr, sympy.Expr):
        expr = expr.subs(subs)
    return int(expr)


def resolve_symbols(func, subs):
    """Clone `func` with every sympy symbol / expression / Mapping found in its
    closure cells and globals replaced by its bound value
    (kernel_api.py:43-90)."""

    def resolved(val):
        if isinstance(val, sympy.Symbol):
            return subs.get(val)
        if isinstance(val, sympy.Expr):
            return val.subs(subs)
        if isinstance(val, Mapping):
            return Mapping(resolve_symbols(val.func, subs))
        return None

    closure = None
    if func.__closure__ is not None:
        cells = []
        for cell in func.__closure__:
            new = resolved(cell.cell_contents)
            cells.append(cell if new is None else types.CellType(new))
        closure = tuple(cells)
    new_globals = {}
    for k, v in func.__globals__.items():
        new = resolved(v)
        new_globals[k] = v if new is None else new
    clone = types.FunctionType(func.__code__, new_globals, func.__name__,
                               func.__defaults__, closure)
    clone = functools.update_wrapper(clone, func)
    clone.__kwdefaults__ = func.__kwdefaults__
    return clone


class Kernel:
    def __init__(self, func, work_shape, group_shape, subgroup_size, literals,
                 tunables, tuned=None):
        self.func = func
        self.work_shape, self.group_shape = work_shape, group_shape
        self.subgroup_size, self.literals = subgroup_size, literals
        self.tunables = tunables
        self.tuned = dict(tuned or {})
        self._binders = _collect_binders(func)
        # (by attribute, so that the GPU front-end's own TunableParam class,
        # used by kernels written once and run on both sides, is accepted)
        if isinstance(tunables, TunableParam) or (hasattr(tunables, "sym") and
                                                  hasattr(tunables, "default")):
            tunables = (tunables,)
        assert isinstance(tunables, Iterable), "Unsupported tunables"
        self._defaults = {t.sym: t.default for t in tunables}

    def __call__(self, *args, **kwargs):
        subs = {}
        for b in self._binders:
            b(subs, args)
        subs = {**subs, **self._defaults, **self.tuned}
        items = list(subs.items())
        work = _to_int_dims(self.work_shape, items)
        group = _to_int_dims(self.group_shape, items)
        sg = _to_int_dims(self.subgroup_size, items)
        body = resolve_symbols(self.func, subs)
        counts = [_ceil_div(w, g) for w, g in zip(work, group)]
        cg = CurrentGroup(group, sg)
        # kernel_sim.py:161-163: row-major over the group grid
        for gid in itertools.product(*(range(c) for c in counts)):
            cg._group_id = gid
            body(cg, *args, **kwargs)

    def parametrize(self, tuned):
        return Kernel(self.func, self.work_shape, self.group_shape,
                      self.subgroup_size, self.literals, self.tunables,
                      {**self.tuned, **tuned})


def kernel(work_shape, group_shape=None, subgroup_size=None, literals=(),
           tunables=()):
    """kernel_sim.py:177-203."""
    assert (subgroup_size is None or isinstance(subgroup_size, int)
            or subgroup_size in literals), "Subgroup size must be const or literal"
    assert isinstance(literals, Iterable), f"literals must iterable, got {literals}"
    if subgroup_size is None:
        subgroup_size = DEFAULT_SUBGROUP_SIZE
    if not isinstance(work_shape, Iterable):
        work_shape = (work_shape,)
    if group_shape is None:
        group_shape = (1,) * (len(work_shape) - 1) + (DEFAULT_GROUP_LAST_DIM,)
    if not isinstance(group_shape, Iterable):
        group_shape = (group_shape,)
    assert len(work_shape) <= 3
    assert len(work_shape) == len(group_shape)

    def wrap(func):
        return Kernel(func, work_shape, group_shape, subgroup_size, literals,
                      tunables)

    return wrap

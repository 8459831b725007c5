"""`@kernel(work_shape=...)`: the GPU decorator.

Host-side mirror of the reference's python/hckernel/kernel.py:134-173 (same
signature: work_shape, group_shape, subgroup_size, literals, tunables, backend,
device) and of the symbol binding rules of python/hckernel/kernel_sim.py:34-127
(a `Symbol` annotation binds the argument's value, `tuple[S1, ...]` binds element
by element, `Buffer[d0, ..., DT]` binds symbolic dims to the array's shape;
conflicting values are an error).

Calling a kernel
    1. binds the symbols, evaluates work_shape / group_shape to integers (a
       missing group_shape is chosen by the runtime's block-size suggestion for
       the reversed work shape, mlir/lib/Transforms/LowerHKernel.cpp:293-312),
    2. runs the body once with a tracing group (hc_amd.kernel_api),
    3. matches the traced program to a hand-written gfx950 kernel
       (hc_amd.binding) and launches it through the C ABI,
    4. waits for completion: a call is synchronous on return, as in the
       reference (python/cpp/py-runtime/src/GpuRuntime.cpp:60-69).
Array arguments must live in device memory (torch tensors on the GPU,
hc_amd.runtime.DeviceArray, or anything exposing __cuda_array_interface__).
"""

from __future__ import annotations

import ctypes as C
import functools
import inspect
import types
import typing
from collections.abc import Iterable

import sympy

from . import runtime as rt
from .autotune import TunedParams, autotune
from .binding import NoNativeKernel, bind
from .indexing import sym
from .kernel_api import (Buffer, BufferProxy, CurrentGroup, CurrentGroup1, CurrentGroup2,
                         CurrentGroup3, CurrentSubGroup, CurrentWorkitem, DynInt, Mapping, TraceError,
                         TunableParam, atomic_ref, create_mapping, dtype_name)
from .typename import Typename, typename

__all__ = ["kernel", "sym", "typename", "Buffer", "CurrentGroup", "CurrentGroup1",
           "CurrentGroup2", "CurrentGroup3", "CurrentSubGroup", "CurrentWorkitem",
           "TunableParam", "atomic_ref", "create_mapping", "NoNativeKernel", "TraceError",
           "autotune", "TunedParams"]

DEFAULT_SUBGROUP_SIZE = 64      # mlir/lib/Transforms/LowerHKernel.cpp:539-544


def _verify_kernel_params(work_shape, group_shape, subgroup_size, literals, tunables):
    # python/hckernel/kernel_api.py:26-32
    assert (subgroup_size is None or isinstance(subgroup_size, int)
            or subgroup_size in literals), "Subgroup size must be const or literal"
    assert isinstance(literals, Iterable), f"literals must iterable, got {literals}"


# ---------------------------------------------------------------------------
# symbol binding
# ---------------------------------------------------------------------------
def _bind(subs, symbol, value):
    if symbol in subs and subs[symbol] != value:
        raise RuntimeError(f"Symbol value conflict for {symbol}: {subs[symbol]} and {value}")
    subs[symbol] = value


def _is_array(x) -> bool:
    return hasattr(x, "shape") and (hasattr(x, "__cuda_array_interface__")
                                    or hasattr(x, "__dlpack__")
                                    or hasattr(x, "__array_interface__"))


def _binders(func):
    ann = inspect.get_annotations(func)
    out = []
    for i, name in enumerate(inspect.signature(func).parameters):
        a = ann.get(name)
        pos = i - 1                      # the first parameter is the group
        if isinstance(a, str):
            raise RuntimeError(
                f"parameter {name!r} of {func.__name__}: the annotation is the string {a!r}; "
                "kernel bodies need evaluated annotations (define them in a module without "
                "`from __future__ import annotations`)")
        if a is None or a in (CurrentGroup, CurrentGroup1, CurrentGroup2, CurrentGroup3,
                              CurrentSubGroup, CurrentWorkitem):
            continue
        if isinstance(a, sympy.Symbol):
            out.append(lambda subs, args, a=a, pos=pos: _bind(subs, a, args[pos]))
        elif typing.get_origin(a) is tuple or isinstance(a, tuple):
            parts = typing.get_args(a) if typing.get_origin(a) is tuple else a

            def bind_tuple(subs, args, parts=parts, pos=pos, name=name):
                val = args[pos]
                if not isinstance(val, Iterable) or len(val) != len(parts):
                    raise RuntimeError(f"argument {name!r}: expected {len(parts)} values")
                for s, v in zip(parts, val):
                    if isinstance(s, sympy.Symbol):
                        _bind(subs, s, v)
            out.append(bind_tuple)
        elif isinstance(a, type) and issubclass(a, Buffer):
            def bind_buffer(subs, args, a=a, pos=pos, name=name):
                val = args[pos]
                if len(val.shape) != len(a.shape):
                    raise RuntimeError(f"argument {name!r}: Invalid rank (expected "
                                       f"{len(a.shape)}, got {len(val.shape)})")
                for s, v in zip(a.shape, val.shape):
                    if isinstance(s, sympy.Symbol):
                        _bind(subs, s, int(v))
            out.append(bind_buffer)
        else:
            raise RuntimeError(f"Unsupported annotation: {type(a)} {a}")
    return out


def _to_ints(expr, subs):
    if isinstance(expr, Iterable):
        return tuple(_to_ints(e, subs) for e in expr)
    if isinstance(expr, sympy.Expr):
        expr = expr.subs(subs)
        if expr.free_symbols:
            raise RuntimeError(f"unresolved symbols in {expr}: {sorted(map(str, expr.free_symbols))}")
    return int(expr)


def _resolve_symbols(func, subs, _memo=None, dynamic=frozenset()):
    """Clone func with sympy symbols / expressions in its closure and globals
    replaced by their values (python/hckernel/kernel_api.py:43-90); index
    mappings found there are resolved the same way.  Each function is cloned
    once per call (_memo), and a mapping that is reached again while it is being
    cloned is left as it is, so module-level mappings that see each other
    through their globals do not recurse."""
    memo = {} if _memo is None else _memo
    if id(func) in memo:
        return memo[id(func)] or func
    memo[id(func)] = None                       # in progress

    def value_of(v):
        # values of symbols in `dynamic` (known at launch only) are marked as such
        if isinstance(v, sympy.Symbol):
            r = subs.get(v)
            return DynInt(r) if v in dynamic and type(r) is int else r
        if isinstance(v, sympy.Expr):
            r = v.subs(subs)
            if not r.is_Integer:
                return r
            return DynInt(int(r)) if v.free_symbols & dynamic else int(r)
        if isinstance(v, Mapping):
            if memo.get(id(v.func), 0) is None:
                return None
            return Mapping(_resolve_symbols(v.func, subs, memo, dynamic))
        return None

    closure = None
    if func.__closure__ is not None:
        cells = []
        for c in func.__closure__:
            r = value_of(c.cell_contents)
            cells.append(c if r is None else types.CellType(r))
        closure = tuple(cells)
    new_globals = {}
    for k, v in func.__globals__.items():
        r = value_of(v)
        new_globals[k] = v if r is None else r
    clone = types.FunctionType(func.__code__, new_globals, func.__name__,
                               func.__defaults__, closure)
    clone = functools.update_wrapper(clone, func)
    clone.__kwdefaults__ = func.__kwdefaults__
    memo[id(func)] = clone
    return clone


def suggest_group_shape(work_shape):
    """Default group shape: the runtime's block-size suggestion applied to the
    reversed work shape (x = last Python dim), reversed back."""
    n = len(work_shape)
    g = (C.c_size_t * n)(*reversed(work_shape))
    b = (C.c_size_t * n)()
    rt.hcgpuSuggestBlockSize(None, g, b, n)
    return tuple(reversed(tuple(b)))


def _array_dtype(obj) -> str:
    if getattr(obj, "bf16", False):
        return "bfloat16"
    return dtype_name(obj.dtype)


class GpuKernel:
    def __init__(self, func, work_shape, group_shape, subgroup_size, literals, tunables,
                 backend, device, tuned=None):
        self.func = func
        self.work_shape, self.group_shape = work_shape, group_shape
        self.subgroup_size, self.literals, self.tunables = subgroup_size, literals, tunables
        self.backend, self.device = backend, device
        self.tuned = dict(tuned or {})
        self._binders = _binders(func)
        tun = (tunables,) if isinstance(tunables, TunableParam) else tunables
        assert isinstance(tun, Iterable), "Unsupported tunables"
        self._defaults = {t.sym: t.default for t in tun}
        self._cache = {}
        self.last_plans = []
        self.variants = {}              # {kernel family: variant number}

    def parametrize(self, tuned):
        """A copy of the kernel with tunable symbols fixed ({symbol: value},
        python/hckernel/kernel_sim.py:165-175).  The result of
        hc_amd.autotune.autotune() also carries the variants of the hand-written
        kernels to use; they are selected around every call."""
        k = GpuKernel(self.func, self.work_shape, self.group_shape, self.subgroup_size,
                      self.literals, self.tunables, self.backend, self.device,
                      {**self.tuned, **tuned})
        k.variants = {**self.variants, **getattr(tuned, "variants", {})}
        return k

    # -- the work ------------------------------------------------------------------
    def _signature(self, args, memrefs):
        sig = []
        for a, m in zip(args, memrefs):
            if m is None:
                sig.append(("v", a if isinstance(a, (int, float, tuple)) else repr(a)))
            else:
                sig.append(("a", m.shape, m.strides, m.itemsize, _array_dtype(a)))
        return tuple(sig)

    def _trace(self, args, memrefs, subs):
        work = _to_ints(self.work_shape, subs)
        if self.group_shape is None:
            group = suggest_group_shape(work)
        else:
            group = _to_ints(self.group_shape, subs)
        sg = _to_ints(self.subgroup_size, subs)
        if len(work) != len(group):
            raise RuntimeError("work_shape and group_shape have different ranks")
        n_groups = tuple(-(-w // g) for w, g in zip(work, group))
        names = list(inspect.signature(self.func).parameters)[1:]
        # Symbols whose value is only known at launch: everything bound from the
        # arguments except literals and tunables.
        static_syms = set(self.literals) | set(self._defaults) | set(self.tuned)
        dynamic = frozenset(k for k in subs if isinstance(k, sympy.Symbol) and k not in static_syms)
        ann = inspect.get_annotations(self.func)

        def dims_of(name, shape):
            a = ann.get(name)
            spec = getattr(a, "shape", None) if isinstance(a, type) and issubclass(a, Buffer) else None
            out = []
            for d, n in enumerate(shape):
                s = spec[d] if spec is not None and d < len(spec) else None
                static = isinstance(s, int) or (isinstance(s, sympy.Symbol) and s in static_syms)
                out.append(int(n) if static else DynInt(n))
            return tuple(out)

        proxies = []
        for i, (a, m) in enumerate(zip(args, memrefs)):
            name = names[i] if i < len(names) else f"arg{i}"
            if m is None:
                s = ann.get(name)
                if type(a) is int and isinstance(s, sympy.Symbol) and s in dynamic:
                    a = DynInt(a)
                proxies.append(a)
            else:
                proxies.append(BufferProxy(i, name, dims_of(name, m.shape), m.strides,
                                           _array_dtype(a), a))
        group_obj = [CurrentGroup1, CurrentGroup2, CurrentGroup3][len(work) - 1](group, sg)
        for p in proxies:
            if isinstance(p, BufferProxy):
                p.group = group_obj
        body = _resolve_symbols(self.func, subs, dynamic=dynamic)
        try:
            body(group_obj, *proxies)
        except TraceError as exc:
            raise NoNativeKernel(f"{self.func.__name__}: {exc}") from exc
        finally:
            # the plan makers take their arrays from the memrefs of each call; the
            # arrays of the call that was traced must not live on in the cache
            for p in proxies:
                if isinstance(p, BufferProxy):
                    p.obj = None
        return bind(group_obj.stores, n_groups, group_obj.atomics, group_obj.mapped_stores,
                    group_obj.id_stores, group, group_obj.cell_stores)

    def plan(self, *args, ctx=None):
        """Everything a call does short of launching: returns the list of
        hc_amd.runtime.Plan objects (C entry point + argument values)."""
        if self.backend != "rocm":
            raise RuntimeError(f"backend {self.backend!r} is not available: this build "
                               "targets gfx950 through HIP only")
        if ctx is None:
            ctx = rt.default_context(self.device)
        memrefs = []
        for a in args:
            if _is_array(a):
                if not hasattr(a, "__cuda_array_interface__") and \
                        getattr(getattr(a, "device", None), "type", "cpu") == "cpu":
                    raise RuntimeError("host array passed to a GPU kernel: move it to the "
                                       "device first (hc_amd.runtime.to_device or tensor.cuda())")
                memrefs.append(rt.as_memref(a))
            else:
                memrefs.append(None)
        subs = {}
        for b in self._binders:
            b(subs, args)
        subs = {**subs, **self._defaults, **self.tuned}
        key = (self._signature(args, memrefs), tuple(sorted((str(k), v) for k, v in subs.items())))
        makers = self._cache.get(key)
        if makers is None:
            makers = self._trace(args, memrefs, subs)
            self._cache[key] = makers
        return [p for mk in makers for p in mk(memrefs, ctx)]

    def __call__(self, *args, sync: bool = True):
        plans = self.plan(*args)
        # this kernel's tuned variants apply to this thread's launches only and
        # leave a process-wide hcamdSetVariant choice untouched
        for family, v in self.variants.items():
            rt.set_thread_variant(family, v)
        try:
            for p in plans:
                p.launch()
        finally:
            for family in self.variants:
                rt.set_thread_variant(family, -1)
        self.last_plans = plans
        if sync and plans:
            plans[0].ctx.synchronize()


def kernel(work_shape, group_shape=None, subgroup_size=None, literals=(), tunables=(),
           backend="rocm", device="hip:0"):
    _verify_kernel_params(work_shape, group_shape, subgroup_size, literals, tunables)
    if subgroup_size is None:
        subgroup_size = DEFAULT_SUBGROUP_SIZE
    if not isinstance(work_shape, Iterable):
        work_shape = (work_shape,)
    if group_shape is not None and not isinstance(group_shape, Iterable):
        group_shape = (group_shape,)
    assert len(work_shape) <= 3
    assert group_shape is None or len(work_shape) == len(group_shape)

    def wrap(func):
        return GpuKernel(func, tuple(work_shape), group_shape, subgroup_size, literals,
                         tunables, backend, device)

    return wrap

"""Masked tiles of the host executor (test infrastructure only).

Restates the tensor model of the reference simulator
(python/hckernel/kernel_api.py:106-211): a tile is data plus a per-element
"active" flag.  The reference wraps numpy.ma with the public mask inverted
(True = active, kernel_api.py:117-119); so does this class, because the
arithmetic of partially active tiles is by definition whatever numpy.ma does
(result active iff all inputs active; numpy.ma also deactivates results of
division by zero and of out-of-domain sqrt/log).
"""

from __future__ import annotations

import operator

import numpy as np
from numpy import ma


def _as_ma(x):
    return x._m if isinstance(x, Tile) else x


class Tile:
    """data + active flags.  `.mask` is True where the element is active."""

    __slots__ = ("_m",)
    # NumPy must not try to broadcast a Tile as a sequence of rows when it
    # appears on the right of an ndarray operator.
    __array_priority__ = 100

    def __init__(self, data, active=True):
        if isinstance(data, ma.MaskedArray):
            self._m = data
        else:
            data = np.asarray(data)
            inactive = ~np.broadcast_to(np.asarray(active, bool), data.shape)
            self._m = ma.masked_array(data, mask=inactive.copy())

    # -- views ---------------------------------------------------------------
    @property
    def mask(self):
        """True = active (kernel_api.py:117-119)."""
        return ~ma.getmaskarray(self._m)

    @property
    def data(self):
        return self._m.data

    def __getitem__(self, key):
        return Tile(self._m[key])

    def __setitem__(self, key, value):
        # kernel_api.py:123-131: a tile assigns only its active elements and
        # activates them; anything else overwrites and activates the window.
        if isinstance(value, Tile):
            cur = self.data[key]
            self.data[key] = np.where(value.mask, value.data, cur)
            mk = ma.getmaskarray(self._m)
            mk[key] = mk[key] & ~value.mask
            self._m.mask = mk
        else:
            self.data[key] = value
            mk = ma.getmaskarray(self._m)
            mk[key] = False
            self._m.mask = mk

    # -- NumPy interop ---------------------------------------------------------
    def __array__(self, dtype=None, copy=None):
        # np.exp(tile), np.dot(tile, tile), np.linalg.norm(tile) see the raw
        # data with inactive elements at their fill value 0: the reference's
        # wrapper reaches NumPy through numpy.ma's __array__ the same way
        # (kernel_api.py:150-151; test_examples.py:109,291,320).
        d = self._m.data
        return d.astype(dtype) if dtype is not None else d

    def __getattr__(self, name):
        # shape, dtype, sum, max, compressed, astype ... come from numpy.ma, so
        # reductions skip inactive elements (kernel_api.py:150-151).
        return getattr(self._m, name)

    def __len__(self):
        return len(self._m)

    def __repr__(self):
        return str(self._m)


def _install_operators():
    binary = ["add", "sub", "mul", "matmul", "truediv", "floordiv", "pow",
              "mod", "lt", "le", "eq", "ne", "ge", "gt", "and_", "or_", "xor",
              "rshift", "lshift"]
    unary = ["abs", "neg", "not_", "inv"]
    compare = {"lt", "le", "eq", "ne", "ge", "gt"}

    def make_binary(fn):
        def forward(self, other):
            return Tile(fn(self._m, _as_ma(other)))

        def reflected(self, other):
            # The reference's wrapper has no reflected operators
            # (kernel_api.py:158-206).  What is on the left decides:
            #  * a Python number: an extension of this executor (a TypeError there);
            #  * a NumPy scalar or a plain ndarray (numpy.where's result): NumPy
            #    defers to the wrapper, finds no reflected operator: TypeError;
            #  * a bare numpy.ma array arrives here only for the operators
            #    numpy.ma does not define itself (% & | ^ << >>): there ndarray's
            #    operator runs the ufunc with the wrapper converted through
            #    numpy.ma's __array__ (kernel_api.py:150-151), that is on the
            #    tile's values, whatever their activity, and the result is a
            #    bare numpy.ma array again.
            if isinstance(other, ma.MaskedArray):
                return fn(other, self._m.data)
            if isinstance(other, (np.generic, np.ndarray)):
                raise TypeError(f"unsupported operand type(s): '{type(other).__name__}' and a tile")
            return Tile(fn(_as_ma(other), self._m))

        def inplace(self, other):
            # kernel_api.py:142-145: a[:] = a op b
            self[:] = forward(self, other)
            return self

        return forward, reflected, inplace

    for name in binary:
        fn = getattr(operator, name)
        stem = name.rstrip("_")
        fwd, ref, inp = make_binary(fn)
        setattr(Tile, f"__{stem}__", fwd)
        setattr(Tile, f"__i{stem}__", inp)
        if name not in compare:
            setattr(Tile, f"__r{stem}__", ref)
    for name in unary:
        fn = getattr(operator, name)
        # kernel_api.py:180-201 names the methods __abs__, __neg__, __not__ and
        # __inv__; the last two are reachable by name only (`~tile` and
        # `not tile` never look them up), and so they are here.
        setattr(Tile, f"__{name.rstrip('_')}__", lambda self, _fn=fn: Tile(_fn(self._m)))
    Tile.__hash__ = None


_install_operators()


class Mapping:
    """Index mapping for gathered loads / scattered stores
    (kernel_api.py:214-220)."""

    def __init__(self, func):
        self.func = func


def create_mapping(func):
    return Mapping(func)

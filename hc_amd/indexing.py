"""Index symbols: `sym.X` is an integer sympy symbol named "X".

Host-side mirror of python/hckernel/indexing.py:14-38.  Symbols name array
dimensions and scalar parameters in `@kernel(work_shape=...)` expressions and
in `Buffer[...]` annotations; they are bound to integers at call time.
"""

import sympy

IndexSymbol = sympy.Symbol
IndexExpr = sympy.Expr


def index_symbol(name: str) -> sympy.Symbol:
    return sympy.Symbol(name, integer=True)


def index_expr(value) -> sympy.Expr:
    return sympy.sympify(value)


class _SymbolNamespace:
    def __getattr__(self, name: str) -> sympy.Symbol:
        return index_symbol(name)


sym = _SymbolNamespace()

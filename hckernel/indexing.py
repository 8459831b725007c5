from hc_amd.indexing import IndexExpr, IndexSymbol, index_expr, index_symbol, sym  # noqa: F401

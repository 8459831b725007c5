from hc_amd.py_runtime import (JIT_SYMBOLS, enable_func_tracing, pyabi_lib,  # noqa: F401
                               register_cfunc, runtime_lib)

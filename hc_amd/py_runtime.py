"""Loads the native runtime with ctypes and publishes its entry points.

Host-side mirror of the reference's python/hckernel/py_runtime.py:9-28 (CDLL of
the runtime library, registration of the four hcgpu* functions whose addresses
JIT'd host code binds, search paths, call tracing) and of load_lib in
python/hckernel/utils.py:38-59.  The libraries live in hc_amd/_native/, the
directory the reference also searches first (utils.py:26-27); they are built by
`python -m hc_amd.build`.  There is no fallback: a missing library is an error.
"""

from __future__ import annotations

import ctypes
import os

_NATIVE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "_native")


def get_runtime_search_paths() -> list[str]:
    paths = [_NATIVE]
    paths += [p for p in os.environ.get("PYTHONPATH", "").split(os.pathsep) if p]
    return paths


def load_lib(name: str) -> ctypes.CDLL:
    errors = []
    for path in get_runtime_search_paths():
        full = os.path.join(path, f"lib{name}.so")
        if not os.path.exists(full):
            errors.append(f"{full}: not found")
            continue
        try:
            return ctypes.CDLL(full, mode=ctypes.RTLD_GLOBAL)
        except OSError as exc:  # pragma: no cover - depends on the machine
            errors.append(f'CDLL("{full}"): {exc}')
    raise ImportError(
        f'native library "lib{name}.so" is not available; build it with '
        f"`python -m hc_amd.build` (needs hipcc).\n" + "\n".join(errors))


# RTLD_GLOBAL: the PyObject* half looks setGPULoaderSearchPaths up at run time,
# and a loader of the reference's design finds the backend with RTLD_NOLOAD
# (gpu-runtime/loader/src/SharedLib.cpp:22), i.e. only if it is already
# resident in the process.
runtime_lib = load_lib("hc_amd_runtime")
pyabi_lib = load_lib("hc_amd_pyabi")

# name -> address, the table the reference hands to its JIT
# (python/hckernel/settings.py:31-37)
JIT_SYMBOLS: dict[str, int] = {}


def register_cfunc(lib: ctypes.CDLL, name: str) -> None:
    JIT_SYMBOLS[name] = int(ctypes.cast(getattr(lib, name), ctypes.c_void_p).value)


register_cfunc(pyabi_lib, "hcgpuConvertPyArray")
register_cfunc(pyabi_lib, "hcgpuConvertPyInt64")
register_cfunc(runtime_lib, "hcgpuGetKernel")
register_cfunc(runtime_lib, "hcgpuSuggestBlockSize")
register_cfunc(runtime_lib, "hcgpuLaunchKernel")

_enable_tracing = runtime_lib.hcgpuEnableTraceFunctions
_enable_tracing.argtypes = [ctypes.c_int]
_enable_tracing.restype = None
_enable_loader_tracing = runtime_lib.enableFuncTracing
_enable_loader_tracing.argtypes = [ctypes.c_int]
_enable_loader_tracing.restype = None

_set_runtime_search_paths = pyabi_lib.hcgpuSetRuntimeSearchPaths
_set_runtime_search_paths.argtypes = [ctypes.py_object]
_set_runtime_search_paths.restype = None
_search_paths = [p.encode() for p in get_runtime_search_paths()]
_set_runtime_search_paths(ctypes.py_object(_search_paths))


def enable_func_tracing(val, loader: bool = False) -> None:
    """Print "<fn> enter/exit" for hcgpu* calls (and ol* calls with loader=True)."""
    _enable_tracing(ctypes.c_int(int(bool(val))))
    if loader:
        _enable_loader_tracing(ctypes.c_int(int(bool(val))))

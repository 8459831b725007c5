/*
 * hc_amd_pyabi.h - C ABI of libhc_amd_pyabi.so, the half of the reference's
 * Python runtime that takes PyObject* arguments
 * (python/cpp/py-runtime/src/PyRuntime.cpp:41-71, PyABI.cpp:15-54).
 *
 * The library needs the CPython C API and must be loaded into a process that
 * already hosts an interpreter (ctypes does that).  Every entry point takes
 * the GIL itself, so it may be called with or without it.
 */
#ifndef HC_AMD_PYABI_H
#define HC_AMD_PYABI_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
#include <string>
namespace hc {
/* python/cpp/shared/include/PyRuntimeShared.hpp:9-11.  A C++ type in a C
 * signature: layout-compatible only with callers built against the same
 * libstdc++, which JIT'd host code of the reference is. */
struct ExceptionDesc {
  std::string message;
};
} // namespace hc
typedef hc::ExceptionDesc HcExceptionDesc;
extern "C" {
#define HCAMD_NOEXCEPT noexcept
#else
typedef struct HcExceptionDesc HcExceptionDesc; /* opaque in C */
#define HCAMD_NOEXCEPT
#endif

/* The memref descriptor the reference's generated host code passes to its
 * kernels (tests/Transforms/pyapi-to-llvm.mlir:6-8,21; PyABI.cpp:15-20):
 *   { void *allocated; void *aligned; intptr_t offset;
 *     intptr_t sizes[rank]; intptr_t strides[rank]; }
 * with strides in elements and offset 0.  HCAMD_MEMREF_WORDS(rank) is its size
 * in 8-byte words. */
#define HCAMD_MEMREF_WORDS(rank) (3 + 2 * (rank))

/* PyRuntime.cpp:47-58; PyABI.cpp:23-37.  `obj` is a borrowed PyObject*
 * exposing __cuda_array_interface__ (device tensors), the buffer protocol
 * (NumPy) or __dlpack__ (torch CPU tensors).  Fills the descriptor at `ret`.
 * Returns 0, or 1 with errorDesc->message set ("Invalid rank" when the rank
 * differs). */
int hcgpuConvertPyArray(HcExceptionDesc *errorDesc, void *obj, int rank,
                        void *ret) HCAMD_NOEXCEPT;

/* PyRuntime.cpp:60-71; PyABI.cpp:39-41.  Python int -> int64_t. */
int hcgpuConvertPyInt64(HcExceptionDesc *errorDesc, void *obj,
                        int64_t *ret) HCAMD_NOEXCEPT;

/* PyRuntime.cpp:41-45; PyABI.cpp:45-54.  `obj` is a Python list of bytes;
 * forwards to setGPULoaderSearchPaths of libhc_amd_runtime.so when that
 * library is loaded in the process, otherwise does nothing. */
void hcgpuSetRuntimeSearchPaths(void *obj) HCAMD_NOEXCEPT;

/* The same conversions with a plain character buffer for the message (no
 * counterpart in the reference; for callers that are not C++).  The message
 * is truncated to errLen-1 characters and NUL terminated.  itemSize, when not
 * NULL, receives the element size in bytes. */
int hcamdConvertPyArray(void *obj, int rank, void *ret, size_t *itemSize,
                        char *err, size_t errLen) HCAMD_NOEXCEPT;
int hcamdConvertPyInt64(void *obj, int64_t *ret, char *err,
                        size_t errLen) HCAMD_NOEXCEPT;

#ifdef __cplusplus
}
#endif
#endif /* HC_AMD_PYABI_H */

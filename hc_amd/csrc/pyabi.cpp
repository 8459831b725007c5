// libhc_amd_pyabi.so: PyObject* -> memref descriptor / int64 conversions of the
// Python runtime ABI.  Signatures and the reference interfaces they replace are
// documented in include/hc_amd_pyabi.h.
//
// Three producers are understood, tried in this order:
//   1. __cuda_array_interface__  device tensors (torch on ROCm exposes it);
//                                strides there are in bytes or None;
//   2. the buffer protocol       NumPy arrays, memoryviews;
//   3. __dlpack__                torch CPU tensors and anything else DLPack.
// The descriptor borrows the producer's memory: the caller keeps the Python
// object alive for as long as the descriptor is used, as the reference's
// generated host code does for the duration of one call.
#define PY_SSIZE_T_CLEAN
#include <Python.h>

#include "hc_amd_pyabi.h"

#include <dlfcn.h>

#include <cstdio>
#include <cstring>
#include <stdexcept>
#include <string>
#include <vector>

namespace {

struct Gil {
  Gil() : state(PyGILState_Ensure()) {}
  ~Gil() { PyGILState_Release(state); }
  PyGILState_STATE state;
};

struct Ref { // owned reference
  explicit Ref(PyObject *o = nullptr) : p(o) {}
  Ref(const Ref &) = delete;
  ~Ref() { Py_XDECREF(p); }
  explicit operator bool() const { return p != nullptr; }
  PyObject *p;
};

struct MemrefHeader {
  void *allocated;
  void *aligned;
  intptr_t offset;
  intptr_t sizesAndStrides[1];
};

// DLPack 0.x structures (public specification, dlpack.h).
struct DLDevice {
  int32_t device_type;
  int32_t device_id;
};
struct DLDataType {
  uint8_t code;
  uint8_t bits;
  uint16_t lanes;
};
struct DLTensor {
  void *data;
  DLDevice device;
  int32_t ndim;
  DLDataType dtype;
  int64_t *shape;
  int64_t *strides;
  uint64_t byte_offset;
};
struct DLManagedTensor {
  DLTensor dl_tensor;
  void *manager_ctx;
  void (*deleter)(DLManagedTensor *);
};

[[noreturn]] void fail(const std::string &msg) { throw std::runtime_error(msg); }

std::string pyErrorText() {
  PyObject *type = nullptr, *value = nullptr, *tb = nullptr;
  PyErr_Fetch(&type, &value, &tb);
  std::string text = "Python error";
  if (value) {
    Ref s(PyObject_Str(value));
    if (s) {
      const char *c = PyUnicode_AsUTF8(s.p);
      if (c)
        text = c;
    }
  }
  Py_XDECREF(type);
  Py_XDECREF(value);
  Py_XDECREF(tb);
  PyErr_Clear();
  return text;
}

void fill(void *ret, void *data, int rank, const std::vector<intptr_t> &shape,
          const std::vector<intptr_t> &strides) {
  auto *d = static_cast<MemrefHeader *>(ret);
  d->allocated = data;
  d->aligned = data;
  d->offset = 0;
  for (int i = 0; i < rank; ++i) {
    d->sizesAndStrides[i] = shape[i];
    d->sizesAndStrides[i + rank] = strides[i];
  }
}

std::vector<intptr_t> compactStrides(const std::vector<intptr_t> &shape) {
  std::vector<intptr_t> s(shape.size());
  intptr_t acc = 1;
  for (size_t i = shape.size(); i-- > 0;) {
    s[i] = acc;
    acc *= shape[i];
  }
  return s;
}

bool fromCudaArrayInterface(PyObject *obj, int rank, void *ret, size_t *item) {
  if (!PyObject_HasAttrString(obj, "__cuda_array_interface__"))
    return false;
  Ref iface(PyObject_GetAttrString(obj, "__cuda_array_interface__"));
  if (!iface) { // e.g. a tensor that requires grad: try the next protocol
    PyErr_Clear();
    return false;
  }
  if (!PyDict_Check(iface.p))
    return false;
  PyObject *shapeObj = PyDict_GetItemString(iface.p, "shape");
  PyObject *dataObj = PyDict_GetItemString(iface.p, "data");
  PyObject *typeObj = PyDict_GetItemString(iface.p, "typestr");
  PyObject *stridesObj = PyDict_GetItemString(iface.p, "strides");
  if (!shapeObj || !dataObj || !typeObj || !PyTuple_Check(shapeObj) ||
      !PyTuple_Check(dataObj) || PyTuple_Size(dataObj) < 1)
    fail("Malformed __cuda_array_interface__");
  if (PyTuple_Size(shapeObj) != rank)
    fail("Invalid rank");
  const char *typestr = PyUnicode_AsUTF8(typeObj);
  if (!typestr || std::strlen(typestr) < 3)
    fail("Malformed __cuda_array_interface__ typestr");
  const long itemsize = std::strtol(typestr + 2, nullptr, 10);
  if (itemsize <= 0)
    fail("Malformed __cuda_array_interface__ typestr");
  std::vector<intptr_t> shape(rank), strides(rank);
  for (int i = 0; i < rank; ++i)
    shape[i] = (intptr_t)PyLong_AsSsize_t(PyTuple_GetItem(shapeObj, i));
  if (stridesObj && stridesObj != Py_None) {
    if (!PyTuple_Check(stridesObj) || PyTuple_Size(stridesObj) != rank)
      fail("Malformed __cuda_array_interface__ strides");
    for (int i = 0; i < rank; ++i) {
      const intptr_t b =
          (intptr_t)PyLong_AsSsize_t(PyTuple_GetItem(stridesObj, i));
      if (b % itemsize)
        fail("Stride is not a multiple of the element size");
      strides[i] = b / itemsize;
    }
  } else {
    strides = compactStrides(shape);
  }
  void *data = PyLong_AsVoidPtr(PyTuple_GetItem(dataObj, 0));
  if (PyErr_Occurred())
    fail(pyErrorText());
  fill(ret, data, rank, shape, strides);
  if (item)
    *item = (size_t)itemsize;
  return true;
}

bool fromBuffer(PyObject *obj, int rank, void *ret, size_t *item) {
  if (!PyObject_CheckBuffer(obj))
    return false;
  Py_buffer view;
  if (PyObject_GetBuffer(obj, &view, PyBUF_STRIDES | PyBUF_FORMAT) != 0) {
    PyErr_Clear();
    return false;
  }
  struct Release {
    Py_buffer *v;
    ~Release() { PyBuffer_Release(v); }
  } release{&view};
  if (view.ndim != rank)
    fail("Invalid rank");
  if (view.itemsize <= 0)
    fail("Invalid element size");
  std::vector<intptr_t> shape(rank), strides(rank);
  for (int i = 0; i < rank; ++i) {
    shape[i] = (intptr_t)view.shape[i];
    if (view.strides[i] % view.itemsize)
      fail("Stride is not a multiple of the element size");
    strides[i] = (intptr_t)(view.strides[i] / view.itemsize);
  }
  fill(ret, view.buf, rank, shape, strides);
  if (item)
    *item = (size_t)view.itemsize;
  return true;
}

bool fromDlpack(PyObject *obj, int rank, void *ret, size_t *item) {
  if (!PyObject_HasAttrString(obj, "__dlpack__"))
    return false;
  Ref capsule(PyObject_CallMethod(obj, "__dlpack__", nullptr));
  if (!capsule)
    fail(pyErrorText());
  auto *managed = static_cast<DLManagedTensor *>(
      PyCapsule_GetPointer(capsule.p, "dltensor"));
  if (!managed)
    fail(pyErrorText());
  const DLTensor &t = managed->dl_tensor;
  if (t.ndim != rank)
    fail("Invalid rank");
  if (t.dtype.lanes != 1 || t.dtype.bits % 8)
    fail("Unsupported DLPack element type");
  std::vector<intptr_t> shape(rank), strides(rank);
  for (int i = 0; i < rank; ++i)
    shape[i] = (intptr_t)t.shape[i];
  if (t.strides) {
    for (int i = 0; i < rank; ++i)
      strides[i] = (intptr_t)t.strides[i];
  } else {
    strides = compactStrides(shape);
  }
  fill(ret, static_cast<char *>(t.data) + t.byte_offset, rank, shape, strides);
  if (item)
    *item = t.dtype.bits / 8;
  // The capsule still owns the managed tensor; dropping it runs the producer's
  // deleter.  The memory itself stays alive through `obj`.
  return true;
}

void convertArray(void *pyobj, int rank, void *ret, size_t *item) {
  auto *obj = static_cast<PyObject *>(pyobj);
  if (!obj || !ret)
    fail("Null argument");
  if (rank < 0 || rank > 32)
    fail("Invalid rank");
  if (fromCudaArrayInterface(obj, rank, ret, item))
    return;
  if (fromBuffer(obj, rank, ret, item))
    return;
  if (fromDlpack(obj, rank, ret, item))
    return;
  fail("Object is not an array (no __cuda_array_interface__, buffer or "
       "__dlpack__)");
}

void convertInt64(void *pyobj, int64_t *ret) {
  auto *obj = static_cast<PyObject *>(pyobj);
  if (!obj || !ret)
    fail("Null argument");
  Ref index(PyNumber_Index(obj));
  if (!index)
    fail(pyErrorText());
  const long long v = PyLong_AsLongLong(index.p);
  if (v == -1 && PyErr_Occurred())
    fail(pyErrorText());
  *ret = (int64_t)v;
}

void copyMessage(const char *msg, char *err, size_t errLen) {
  if (!err || errLen == 0)
    return;
  std::snprintf(err, errLen, "%s", msg);
}

} // namespace

extern "C" {

int hcgpuConvertPyArray(HcExceptionDesc *errorDesc, void *obj, int rank,
                        void *ret) noexcept {
  Gil gil;
  try {
    convertArray(obj, rank, ret, nullptr);
    return 0;
  } catch (const std::exception &e) {
    if (errorDesc)
      errorDesc->message = e.what();
    return 1;
  }
}

int hcgpuConvertPyInt64(HcExceptionDesc *errorDesc, void *obj,
                        int64_t *ret) noexcept {
  Gil gil;
  try {
    convertInt64(obj, ret);
    return 0;
  } catch (const std::exception &e) {
    if (errorDesc)
      errorDesc->message = e.what();
    return 1;
  }
}

void hcgpuSetRuntimeSearchPaths(void *obj) noexcept {
  Gil gil;
  auto *list = static_cast<PyObject *>(obj);
  if (!list || !PyList_Check(list))
    return;
  std::vector<std::string> keep;
  for (Py_ssize_t i = 0; i < PyList_Size(list); ++i) {
    PyObject *item = PyList_GetItem(list, i);
    const char *s = PyBytes_Check(item) ? PyBytes_AsString(item) : nullptr;
    if (s)
      keep.emplace_back(s);
  }
  std::vector<const char *> ptrs;
  for (const std::string &s : keep)
    ptrs.push_back(s.c_str());
  using Setter = void (*)(const char *[], size_t);
  if (auto set = reinterpret_cast<Setter>(
          dlsym(RTLD_DEFAULT, "setGPULoaderSearchPaths")))
    set(ptrs.data(), ptrs.size());
}

int hcamdConvertPyArray(void *obj, int rank, void *ret, size_t *itemSize,
                        char *err, size_t errLen) noexcept {
  Gil gil;
  try {
    convertArray(obj, rank, ret, itemSize);
    return 0;
  } catch (const std::exception &e) {
    copyMessage(e.what(), err, errLen);
    return 1;
  }
}

int hcamdConvertPyInt64(void *obj, int64_t *ret, char *err,
                        size_t errLen) noexcept {
  Gil gil;
  try {
    convertInt64(obj, ret);
    return 0;
  } catch (const std::exception &e) {
    copyMessage(e.what(), err, errLen);
    return 1;
  }
}

} // extern "C"

// libnumba-mlir-python-runtime-hip.so: turns a Python object that describes a
// HIP device array into the native array record compiled code takes.
//
// The reference does this for SYCL USM arrays in
// numba_mlir/numba_mlir/python_runtime/lib/Boxing.cpp:45-136
// (nmrtUnboxSyclInterface, bound by mlir/dpctl_interop.py:233-262) with the
// MemInfo helpers of PythonRt.cpp:29-47.  Same three entry points, same
// record and MemInfo layouts (they are Numba's: numba/core/runtime/nrt.h),
// same conventions of the described dict -- `__hip_array_interface__` carries
// the fields of `__sycl_usm_array_interface__`:
//   "data":    (address as int, read-only flag)
//   "shape":   tuple of ints
//   "strides": tuple of ints in ELEMENTS, or None for a C-contiguous array
//   "typestr": NumPy array-interface type string, e.g. "<f4"
// The item size is read from the type string itself, so NumPy's C API is not
// needed.  Errors: -1 with a Python exception set that says what is wrong.
#define PY_SSIZE_T_CLEAN
#include <Python.h>

#include <cstddef>
#include <cstdint>
#include <cstdlib>
#include <cstring>

#define PYRT_EXPORT extern "C" __attribute__((visibility("default")))

namespace {

// Numba's arystruct_t: the fixed fields, then `ndim` extents and `ndim`
// strides in bytes.
struct ArrayRecord {
  void *meminfo;
  PyObject *parent;
  Py_ssize_t nitems;
  Py_ssize_t itemsize;
  void *data;
  Py_ssize_t shape_and_strides[1];
};

// Numba's NRT MemInfo.
using DtorFn = void (*)(void *ptr, size_t size, void *info);
struct MemInfo {
  size_t refct;
  DtorFn dtor;
  void *dtor_info;
  void *data;
  size_t size;
  void *external_allocator;
};

using AllocFn = void *(*)(size_t);
AllocFn memInfoAlloc = nullptr;

int fail(PyObject *type, const char *what) {
  PyErr_Format(type, "__hip_array_interface__: %s", what);
  return -1;
}

// "<f8" -> 8, "|b1" -> 1, "<c16" -> 16; 0 if the string is not a type string.
Py_ssize_t itemSizeOf(PyObject *typestr) {
  if (!PyUnicode_Check(typestr))
    return 0;
  Py_ssize_t n = 0;
  const char *s = PyUnicode_AsUTF8AndSize(typestr, &n);
  if (!s || n < 3 || !std::strchr("<>|=", s[0]) || !std::strchr("biufcmMOSUV", s[1]))
    return 0;
  Py_ssize_t size = 0;
  for (Py_ssize_t k = 2; k < n; ++k) {
    if (s[k] < '0' || s[k] > '9')
      return 0;
    size = size * 10 + (s[k] - '0');
    if (size > (Py_ssize_t(1) << 30))
      return 0;
  }
  return size;
}

bool tupleOfInts(PyObject *obj, Py_ssize_t count, Py_ssize_t *out) {
  if (!PyTuple_Check(obj) || PyTuple_GET_SIZE(obj) != count)
    return false;
  for (Py_ssize_t k = 0; k < count; ++k) {
    PyObject *item = PyTuple_GET_ITEM(obj, k);
    if (!PyLong_Check(item))
      return false;
    out[k] = PyLong_AsSsize_t(item);
    if (out[k] == -1 && PyErr_Occurred())
      return false;
  }
  return true;
}

} // namespace

// Numba hands over NRT_MemInfo's allocator once, at import
// (reference: mlir/python_rt.py:19-24).
PYRT_EXPORT void nmrtSetMemInfoAllocFunc(void *func) {
  memInfoAlloc = reinterpret_cast<AllocFn>(func);
}

// A MemInfo with one reference for `size` bytes at `data`; `dtor(data, size,
// dtorInfo)` runs when the last reference goes (NULL: the memory is owned
// elsewhere).  Aborts if no allocator was set; NULL if it returns none.
PYRT_EXPORT void *nmrtAllocMemInfo(void *data, size_t size, DtorFn dtor, void *dtorInfo) {
  if (!memInfoAlloc)
    std::abort();
  auto *info = static_cast<MemInfo *>(memInfoAlloc(sizeof(MemInfo)));
  if (!info)
    return nullptr;
  info->refct = 1;
  info->dtor = dtor;
  info->dtor_info = dtorInfo;
  info->data = data;
  info->size = size;
  info->external_allocator = nullptr;
  return info;
}

// Fills `record` (with room for 2 * ndim trailing integers) from
// obj.__hip_array_interface__.  The memory stays owned by `obj`, which the
// record names as its parent; the MemInfo has no destructor.
PYRT_EXPORT int nmrtUnboxHipInterface(PyObject *obj, ArrayRecord *record) {
  PyObject *iface = PyObject_GetAttrString(obj, "__hip_array_interface__");
  if (!iface)
    return -1; // AttributeError stays set
  struct Release {
    PyObject *o;
    ~Release() { Py_DECREF(o); }
  } release{iface};
  if (!PyDict_Check(iface))
    return fail(PyExc_TypeError, "not a dict");

  PyObject *dataField = PyDict_GetItemString(iface, "data"); // borrowed
  if (!dataField || !PyTuple_Check(dataField) || PyTuple_GET_SIZE(dataField) < 1 ||
      !PyLong_Check(PyTuple_GET_ITEM(dataField, 0)))
    return fail(PyExc_TypeError, "'data' must be (address, read_only)");
  void *data = PyLong_AsVoidPtr(PyTuple_GET_ITEM(dataField, 0));
  if (!data && PyErr_Occurred())
    return -1;

  PyObject *shape = PyDict_GetItemString(iface, "shape");
  if (!shape || !PyTuple_Check(shape))
    return fail(PyExc_TypeError, "'shape' must be a tuple");
  const Py_ssize_t ndim = PyTuple_GET_SIZE(shape);

  PyObject *typestr = PyDict_GetItemString(iface, "typestr");
  const Py_ssize_t itemsize = typestr ? itemSizeOf(typestr) : 0;
  if (itemsize <= 0)
    return fail(PyExc_TypeError, "'typestr' must be an array-interface type string");

  Py_ssize_t *dims = record->shape_and_strides;
  Py_ssize_t *strides = dims + ndim;
  if (!tupleOfInts(shape, ndim, dims))
    return PyErr_Occurred() ? -1 : fail(PyExc_TypeError, "'shape' must hold ints");
  Py_ssize_t nitems = 1;
  for (Py_ssize_t k = 0; k < ndim; ++k) {
    if (dims[k] < 0)
      return fail(PyExc_ValueError, "negative extent");
    nitems *= dims[k];
  }
  if (!data && nitems != 0)
    return fail(PyExc_ValueError, "null address for a non-empty array");

  PyObject *stridesField = PyDict_GetItemString(iface, "strides");
  if (!stridesField || stridesField == Py_None) {
    Py_ssize_t step = itemsize; // dense, row-major
    for (Py_ssize_t k = ndim; k-- > 0;) {
      strides[k] = step;
      step *= dims[k];
    }
  } else {
    if (!tupleOfInts(stridesField, ndim, strides))
      return PyErr_Occurred()
                 ? -1
                 : fail(PyExc_TypeError, "'strides' must be None or one int per dimension");
    for (Py_ssize_t k = 0; k < ndim; ++k)
      strides[k] *= itemsize; // elements -> bytes
  }

  void *meminfo = nmrtAllocMemInfo(data, size_t(itemsize) * size_t(nitems), nullptr, nullptr);
  if (!meminfo) {
    PyErr_NoMemory();
    return -1;
  }
  record->meminfo = meminfo;
  record->parent = obj;
  record->nitems = nitems;
  record->itemsize = itemsize;
  record->data = data;
  return 0;
}

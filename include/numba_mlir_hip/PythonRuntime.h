/*
 * C-ABI of libnumba-mlir-python-runtime-hip.so: the glue between Python
 * objects and the native array records compiled code works on.
 *
 * Counterpart of the reference's python runtime
 * (numba_mlir/numba_mlir/python_runtime/lib/Boxing.cpp:45-136,
 * PythonRt.cpp:29-47, PythonRt.hpp:11-15); the records are Numba's
 * (numba/core/runtime/nrt.h: arystruct_t, NRT MemInfo).  The library uses the
 * CPython API and nothing of HIP; it must be loaded into a process that runs
 * Python and called with the GIL held.
 */
#ifndef NUMBA_MLIR_HIP_PYTHON_RUNTIME_H
#define NUMBA_MLIR_HIP_PYTHON_RUNTIME_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Destructor of a MemInfo: called with the data pointer, the size and the
 * info pointer given at creation (PythonRt.hpp:11). */
typedef void (*NmrtMemInfoDtor)(void *ptr, size_t size, void *info);

/*
 * Hands over the allocator MemInfo records come from (Numba's NRT
 * "Allocate" helper: mlir/python_rt.py:19-24).  Must be called before the two
 * functions below.                                      PythonRt.cpp:24-27
 */
void nmrtSetMemInfoAllocFunc(void *func);

/*
 * A MemInfo holding one reference to `size` bytes at `data`.  A compiled
 * function that returns a device array creates one whose destructor calls
 * gpuxDeAlloc(queue, ptr) (mlir/lib/Conversion/GpuRuntimeToLlvm.cpp:717-720).
 * Aborts when no allocator was set; NULL when it returns none.
 *                                                        PythonRt.cpp:29-47
 */
void *nmrtAllocMemInfo(void *data, size_t size, NmrtMemInfoDtor dtor,
                       void *dtorInfo);

/*
 * Fills the array record at `arystruct` -- {meminfo, parent, nitems,
 * itemsize, data, shape[ndim], strides[ndim] in bytes}, with room for the
 * object's number of dimensions -- from `pyobj.__hip_array_interface__`
 * ("data": (address, read_only), "shape", "strides" in elements or None,
 * "typestr").  `pyobj` is a PyObject*.  Returns 0, or -1 with a Python
 * exception set.  Replaces nmrtUnboxSyclInterface.       Boxing.cpp:45-136
 */
int nmrtUnboxHipInterface(void *pyobj, void *arystruct);

#ifdef __cplusplus
}
#endif

#endif

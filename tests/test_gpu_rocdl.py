"""GPU: code objects serialised from ROCDL-form LLVM IR (what the compiler's
ROCDL tail stores in "gpu.binary") loaded by gpuxModuleLoad and launched by
gpuxLaunchKernel with the reference's parameter marshalling, against the
goldens of the reference's runner tests."""

import ctypes
import json
import os

import numpy as np
import pytest

from numba_mlir_amd.mlir import rocdl_binary as rb

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
with open(os.path.join(ROOT, "tests", "golden", "reference_vectors.json")) as f:
    GOLD = json.load(f)

NO_DEPS = (ctypes.c_void_p * 1)(None)


@pytest.fixture(scope="module")
def rt(native_libs):
    from numba_mlir_amd.mlir import gpu_runtime
    return gpu_runtime.runtime_lib, gpu_runtime


def _ir(name):
    with open(os.path.join(ROOT, "tests", "rocdl_cases", name + ".ll")) as f:
        return f.read()


def _printed(x):
    return np.array([float("%.6g" % v) for v in np.ravel(x)]).reshape(np.shape(x))


class _Session:
    """queue + module + shared allocations, the calls compiled host code makes."""

    def __init__(self, lib, g, blob):
        self.lib, self.g = lib, g
        self.q = lib.gpuxQueueCreate(None)
        self.mod = lib.gpuxModuleLoad(self.q, blob, len(blob))
        self.ptrs = []

    def shared(self, values):
        res = self.g.GPUAllocResult()
        self.lib.gpuxAlloc(self.q, values.nbytes, 64, 1, NO_DEPS, ctypes.byref(res))
        self.lib.gpuxWait(self.q, res.event)
        self.lib.gpuxDestroyEvent(self.q, res.event)
        self.ptrs.append(res.ptr)
        buf = (ctypes.c_uint8 * values.nbytes).from_address(res.ptr)
        view = np.frombuffer(buf, dtype=values.dtype)
        view[:] = values
        return res.ptr, view

    def launch(self, name, blocks, pointers, block=1, local_bytes=None):
        """``pointers`` as ptr params; ``local_bytes``: one more ptr param with
        no data, the reference's form of a workgroup-memory argument."""
        kern = self.lib.gpuxKernelGet(self.mod, name.encode())
        count = len(pointers) + (local_bytes is not None)
        descs = (self.g.GPUParamDesc * (count + 1))()
        keep = [ctypes.c_void_p(p) for p in pointers]
        for i, val in enumerate(keep):
            descs[i].data = ctypes.cast(ctypes.pointer(val), ctypes.c_void_p)
            descs[i].size = ctypes.sizeof(val)
            descs[i].type = 8
        if local_bytes is not None:
            descs[len(keep)].data, descs[len(keep)].size = None, local_bytes
            descs[len(keep)].type = 8
        ev = self.lib.gpuxLaunchKernel(self.q, kern, blocks, 1, 1, block, 1, 1, NO_DEPS, descs)
        self.lib.gpuxWait(self.q, ev)
        self.lib.gpuxDestroyEvent(self.q, ev)
        self.lib.gpuxKernelDestroy(kern)

    def close(self):
        for p in self.ptrs:
            self.lib.gpuxDeAlloc(self.q, p)
        self.lib.gpuxModuleDestroy(self.mod)
        self.lib.gpuxQueueDestroy(self.q)


def test_addf_module_from_llvm_ir(rt):
    """addf.mlir:32-33: eight blocks of one work-item print 3.3 eight times."""
    lib, g = rt
    s = _Session(lib, g, rb.serialize(_ir("addf")))
    gold = GOLD["addf"]
    a, _ = s.shared(np.array(gold["a"], np.float32))
    b, _ = s.shared(np.array(gold["b"], np.float32))
    c, out = s.shared(np.zeros(8, np.float32))
    s.launch("main_kernel", 8, [a, b, c])
    assert np.array_equal(_printed(out), np.array(gold["printed"]))
    assert np.array_equal(out, np.array(gold["a"], np.float32) + np.array(gold["b"], np.float32))
    s.close()


@pytest.mark.parametrize("dtype,kernel", [(np.float32, "foo_kernel_f32"),
                                          (np.float64, "foo_kernel_f64")])
def test_fused_map_module_with_a_device_library_call(rt, dtype, kernel):
    """linalg_test_f32.mlir:125-182 / linalg_test_f64.mlir: 500 x 1.00002, and
    the value behind the print, 1 + 4 / (e^12 + 1)."""
    lib, g = rt
    s = _Session(lib, g, rb.serialize(_ir("linalg_test")))
    gold = GOLD["linalg_test"]
    a, _ = s.shared(np.full(gold["n"], gold["a"], dtype))
    coeff, _ = s.shared(np.array(gold["s"], dtype))
    o, out = s.shared(np.zeros(gold["n"], dtype))
    s.launch(kernel, gold["n"], [a, coeff, o])
    assert np.array_equal(_printed(out), np.full(gold["n"], gold["printed"]))
    assert np.abs(out - (1 + 4 / (np.exp(12.0) + 1))).max() < (2e-6 if dtype is np.float32 else 1e-14)
    s.close()


def test_workgroup_memory_argument_and_barrier_from_llvm_ir(rt):
    """A ptr param without data (GpuRuntimeToLlvm.cpp:507-536) reaches a
    kernel built from LLVM IR as an offset into dynamic LDS: every group's
    sum in index order, bit for bit."""
    lib, g = rt
    s = _Session(lib, g, rb.serialize(_ir("group_sum")))
    groups = 300
    x = np.random.default_rng(3).standard_normal(groups * 256).astype(np.float32)
    src, _ = s.shared(x)
    dst, out = s.shared(np.zeros(groups, np.float32))
    s.launch("group_sum_f32", groups, [src, dst], block=256, local_bytes=256 * 4)
    expect = np.cumsum(x.reshape(groups, 256), axis=1, dtype=np.float32)[:, -1]
    assert np.array_equal(out, expect)
    s.close()

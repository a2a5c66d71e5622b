"""The C-ABI libraries load on a machine without a GPU and export exactly what
include/numba_mlir_hip/*.h declares (no compute calls here)."""

import ctypes
import os
import re
import subprocess


ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INCLUDE = os.path.join(ROOT, "include", "numba_mlir_hip")
PKG = os.path.join(ROOT, "numba_mlir_amd")

# reference: numba_mlir/numba_mlir/mlir/gpu_runtime.py:35-56
GPUX = ["gpuxAlloc", "gpuxDeAlloc", "gpuxKernelDestroy", "gpuxKernelGet",
        "gpuxLaunchKernel", "gpuxModuleDestroy", "gpuxModuleLoad",
        "gpuxQueueCreate", "gpuxQueueDestroy", "gpuxSuggestBlockSize",
        "gpuxWait", "gpuxDestroyEvent", "gpuxDuplicateQueue"]


def _declared(header):
    text = open(os.path.join(INCLUDE, header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    return sorted(set(re.findall(r"\b((?:gpux|nmhip|mkl_gemm_|nmrt)\w*)\s*\(", text)))


def _exported(lib):
    out = subprocess.run(["nm", "-D", "--defined-only", os.path.join(PKG, lib)],
                         check=True, capture_output=True, text=True).stdout
    return sorted(line.split()[-1] for line in out.splitlines() if " T " in line)


def test_runtime_exports_exactly_the_gpux_entry_points(native_libs):
    exported = _exported("libnumba-mlir-gpu-runtime-hip.so")
    assert exported == sorted(GPUX)              # export map: gpux* only
    assert _declared("GpuRuntime.h") == sorted(GPUX)


def test_math_runtime_exports(native_libs):
    declared = _declared("MathRuntime.h")
    assert set(declared) >= {"mkl_gemm_float32_device", "mkl_gemm_float64_device",
                             "nmrtMathRuntimeInit", "nmrtMathRuntimeFinalize"}
    assert _exported("libnumba-mlir-math-hip-runtime.so") == declared


def test_python_runtime_exports(native_libs):
    declared = _declared("PythonRuntime.h")
    assert declared == ["nmrtAllocMemInfo", "nmrtSetMemInfoAllocFunc", "nmrtUnboxHipInterface"]
    assert _exported("libnumba-mlir-python-runtime-hip.so") == declared
    # CPython API only: no HIP and no libpython of its own
    needed = subprocess.run(["readelf", "-d", os.path.join(
        PKG, "libnumba-mlir-python-runtime-hip.so")], check=True, capture_output=True,
        text=True).stdout
    assert "amdhip64" not in needed and "libpython" not in needed


def test_offload_exports(native_libs):
    declared = _declared("Offload.h")
    assert _exported("libnumba-mlir-hip-offload.so") == declared
    for name in declared:
        assert hasattr(native_libs.lib, name)


def test_offload_library_reaches_the_gpu_only_through_registered_symbols(native_libs):
    """The lowered host code makes no HIP call of its own: it imports no hip*
    symbol and does not link libamdhip64 (the reference's JIT'd host code sees
    the device only through the gpux* functions, export.txt:1-4,
    GpuRuntimeToLlvm.cpp:95-194)."""
    path = os.path.join(PKG, "libnumba-mlir-hip-offload.so")
    undefined = subprocess.run(["nm", "-D", "--undefined-only", path], check=True,
                               capture_output=True, text=True).stdout
    names = [line.split()[-1] for line in undefined.splitlines() if line.strip()]
    assert not [n for n in names if n.lower().startswith(("hip", "hsa", "gpux"))], names
    needed = subprocess.run(["readelf", "-d", path], check=True, capture_output=True,
                            text=True).stdout
    assert "amdhip64" not in needed and "hsa-runtime" not in needed


def test_wire_struct_layouts(native_libs):
    from numba_mlir_amd.mlir.gpu_runtime import GPUAllocResult, GPUParamDesc
    # {ptr, i32, i32} and {ptr, ptr}: mlir/lib/Conversion/GpuRuntimeToLlvm.cpp:87-93
    assert ctypes.sizeof(GPUParamDesc) == 16
    assert (GPUParamDesc.data.offset, GPUParamDesc.size.offset,
            GPUParamDesc.type.offset) == (0, 8, 12)
    assert ctypes.sizeof(GPUAllocResult) == 16


def test_loader_registers_every_symbol(native_libs):
    names = [n for n, _ in native_libs._registered_cfuncs]
    assert names[:13] == GPUX
    assert names[13:] == ["_mlir_ciface_mkl_gemm_float32_device",
                          "_mlir_ciface_mkl_gemm_float64_device"]
    assert all(addr for _, addr in native_libs._registered_cfuncs)
    assert native_libs.lib.nmhipRegisterSymbol(b"not_a_runtime_symbol", 1) == -1


def test_runtime_kind_selection(native_libs):
    env = dict(os.environ, NUMBA_MLIR_GPU_RUNTIME="sycl", PYTHONPATH=ROOT)
    proc = subprocess.run(
        ["python", "-c", "import numba_mlir_amd.mlir.gpu_runtime"],
        env=env, capture_output=True, text=True)
    assert proc.returncode != 0
    assert 'Invalid GPU runtime type: "sycl", expected "hip"' in proc.stderr


def test_embedded_code_objects_are_gfx950_elf(native_libs):
    for family in ("maps", "reduce", "twins"):
        blob = native_libs.kernel_blob(family)
        assert blob[:4] == b"\x7fELF" and len(blob) > 4096
        assert b"gfx950" in blob
    assert b"nmk_map2_rowbcast_add_f64" in native_libs.kernel_blob("maps")
    assert b"nmk_sum_axis0_i32_i64" in native_libs.kernel_blob("reduce")
    assert b"nmk_twin_pairwise_f64_rows" in native_libs.kernel_blob("twins")


def _run_child(code):
    env = dict(os.environ, PYTHONPATH=ROOT)
    return subprocess.run(["python", "-c", code], env=env, capture_output=True,
                          text=True)


def test_missing_library_fails_loudly(tmp_path):
    """No fallback: if the runtime library is absent the import raises."""
    code = (
        "import numba_mlir_amd.mlir.utils as u\n"
        f"import pathlib; u.PACKAGE_DIR = pathlib.Path({str(tmp_path)!r})\n"
        "import os; os.environ.pop('PYTHONPATH', None)\n"
        "import numba_mlir_amd.mlir.gpu_runtime\n")
    proc = _run_child(code)
    assert proc.returncode != 0
    assert "load_lib(\"numba-mlir-gpu-runtime-hip\") failed" in proc.stderr


def test_fatal_paths_abort_with_message_on_stdout(native_libs):
    """Errors print to stdout and abort()
    (reference: numba_mlir_gpu_runtime_sycl/lib/Utils.hpp:8-21).  These paths
    are taken before any HIP call, so they run without a GPU."""
    cases = {
        "from numba_mlir_amd.mlir import gpu_runtime as g\n"
        "g.runtime_lib.gpuxQueueCreate(b'opencl:cpu:0')":
            "only drives GPU devices",
        "from numba_mlir_amd.mlir import gpu_runtime as g\n"
        "g.runtime_lib.gpuxQueueCreate(b'gpu:banana')":
            "unknown token 'banana'",
        "from numba_mlir_amd.mlir import gpu_runtime as g\n"
        "g.runtime_lib.gpuxQueueDestroy(None)":
            "Invalid queue",
        "from numba_mlir_amd.mlir import gpu_runtime as g\n"
        "g.runtime_lib.gpuxKernelGet(None, b'k')":
            "Invalid module",
        "from numba_mlir_amd.mlir import lowered as l\n"
        "l.lib.nmhipKernelBlob(b'nope', None)":
            "Unknown kernel family",
    }
    for code, message in cases.items():
        proc = _run_child(code)
        assert proc.returncode == -6, (code, proc.returncode, proc.stdout)
        assert "An exception was thrown:" in proc.stdout
        assert message in proc.stdout


def test_call_logging_env(native_libs):
    env = dict(os.environ, PYTHONPATH=ROOT, NUMBA_MLIR_LOG_GPU_RUNTIME_CALLS="1")
    proc = subprocess.run(
        ["python", "-c",
         "from numba_mlir_amd.mlir import gpu_runtime as g\n"
         "g.runtime_lib.gpuxQueueDestroy(None)"],
        env=env, capture_output=True, text=True)
    assert proc.stdout.startswith("gpuxQueueDestroy enter\n")


def test_bench_refuses_more_than_one_gpu():
    proc = subprocess.run(["python", os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                          capture_output=True, text=True)
    assert proc.returncode == 2
    assert "one GPU" in proc.stderr and proc.stdout == ""

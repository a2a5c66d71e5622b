"""Builds the native pieces of the HIP backend for gfx950, in-tree.

Outputs, next to this file (the reference keeps its runtime libraries in the
package directory as well and finds them there,
reference: numba_mlir/numba_mlir/mlir/utils.py:17-42):

  libnumba-mlir-gpu-runtime-hip.so    the 13 gpux* entry points
  libnumba-mlir-math-hip-runtime.so   mkl_gemm_<dtype>_device
  libnumba-mlir-hip-offload.so        lowered host code, dispatcher and the
                                      embedded code objects of the kernels
                                      (plain C++, does not link HIP)
  libnumba-mlir-python-runtime-hip.so the unboxer of HIP device arrays and the
                                      MemInfo helpers (CPython API, no HIP)
  libnmhip-bench-timer.so             HIP-event stopwatch used by bench.py
  hip-runner                          standalone runner of the reference's
                                      mlir/test/L0_RUNNER cases against a gpux*
                                      runtime named by -shared-libs
  csrc/build/bench_yardsticks.hsaco   memory-only kernels bench.py times beside
                                      the real ones (loaded by bench.py alone)

The HIP runtime is built by its own hipcc step, separate from everything
else, as the reference builds its SYCL runtime with its own compiler
(reference: numba_mlir/setup_helper.py:34-81).

Run:  python -m numba_mlir_amd.build   (or call build_all()).
"""

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
BUILD = os.path.join(CSRC, "build")
INCLUDE = os.path.join(ROOT, "include")

ARCH = "gfx950"
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")
HIPCC = os.environ.get("HIPCC", os.path.join(ROCM, "bin", "hipcc"))
CXX = os.environ.get("CXX", "g++")

# Packed-FP32 instructions are kept out of all device code.
DEVICE_FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]
HOST_FLAGS = ["-O2", "-fPIC", "-std=c++17", "-fvisibility=hidden", f"-I{INCLUDE}",
              "-Wall"]
# Host-only libraries are plain C++ that call the HIP runtime API.
HIP_HOST_FLAGS = ["-D__HIP_PLATFORM_AMD__", "-I" + os.path.join(ROCM, "include")]
HIP_LINK_FLAGS = ["-L" + os.path.join(ROCM, "lib"), "-lamdhip64",
                  "-Wl,-rpath," + os.path.join(ROCM, "lib")]

KERNEL_FAMILIES = ["maps", "reduce", "twins"]

RUNTIME_LIB = "libnumba-mlir-gpu-runtime-hip.so"
MATH_LIB = "libnumba-mlir-math-hip-runtime.so"
OFFLOAD_LIB = "libnumba-mlir-hip-offload.so"
BENCH_TIMER_LIB = "libnmhip-bench-timer.so"


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                          text=True)
    out = "\n".join(
        line for line in proc.stdout.splitlines()
        if "packed-fp32-ops" not in line and line.strip()
    )
    if proc.returncode != 0:
        raise RuntimeError("build step failed:\n  " + " ".join(cmd) + "\n" + out)
    if out:
        print(out, file=sys.stderr)


def build_code_object(family, variant="", defines=()):
    """One gfx950 ELF code object per kernel family.

    -ffp-contract=off keeps a*b+c as two roundings, matching the reference's
    CPU lowering (no fma without fastmath).
    """
    src = os.path.join(CSRC, "kernels", family + ".hip")
    out = os.path.join(BUILD, family + variant + ".hsaco")
    _run([HIPCC, "--genco", "--no-gpu-bundle-output", *DEVICE_FLAGS,
          "-ffp-contract=off", *["-D" + d for d in defines], "-o", out, src])
    return out


def build_reduce_release():
    """The reduction kernels once more with the hand-off of partial results
    written as the language's memory model asks (release on the ticket,
    acquire in the last block): the code object the default one is checked
    against (tuning knob "handoff_release")."""
    return build_code_object("reduce", "_release", ["NMK_HANDOFF_RELEASE=1"])


def build_runtime():
    srcs = [os.path.join(CSRC, "runtime", f)
            for f in ("GpuRuntime.cpp", "HipApiReal.cpp")]
    _run([CXX, *HOST_FLAGS, *HIP_HOST_FLAGS, "-shared", *srcs,
          "-Wl,--version-script=" + os.path.join(CSRC, "runtime", "export.map"),
          "-o", os.path.join(HERE, RUNTIME_LIB), *HIP_LINK_FLAGS, "-lpthread"])


def build_math():
    _run([HIPCC, *HOST_FLAGS, "-Wno-unused-command-line-argument",
          *DEVICE_FLAGS, "-shared",
          os.path.join(CSRC, "math", "Gemm.hip"),
          "-Wl,--version-script=" + os.path.join(CSRC, "math", "export.map"),
          "-o", os.path.join(HERE, MATH_LIB)])


def build_offload():
    """Plain C++: the lowered host code reaches the GPU only through the
    registered gpux* pointers, so neither HIP headers nor libamdhip64."""
    _run([CXX, *HOST_FLAGS, "-shared",
          os.path.join(CSRC, "offload", "Offload.cpp"),
          os.path.join(CSRC, "offload", "Blobs.S"),
          "-Wa,-I" + BUILD,
          "-Wl,--version-script=" + os.path.join(CSRC, "offload", "export.map"),
          "-o", os.path.join(HERE, OFFLOAD_LIB), "-lpthread"])


def build_bench_timer():
    """HIP-event stopwatch on a gpux queue's stream, for bench.py only."""
    _run([CXX, *HOST_FLAGS, *HIP_HOST_FLAGS, "-shared",
          os.path.join(CSRC, "bench", "StreamTimer.cpp"),
          "-o", os.path.join(HERE, BENCH_TIMER_LIB), *HIP_LINK_FLAGS])


PYTHON_RT_LIB = "libnumba-mlir-python-runtime-hip.so"


def build_python_runtime():
    import sysconfig
    _run([CXX, *HOST_FLAGS, "-I" + sysconfig.get_paths()["include"], "-shared",
          os.path.join(CSRC, "python_runtime", "HipBoxing.cpp"),
          "-o", os.path.join(HERE, PYTHON_RT_LIB)])


BENCH_YARDSTICKS = os.path.join(BUILD, "bench_yardsticks.hsaco")


def build_bench_yardsticks():
    _run([HIPCC, "--genco", "--no-gpu-bundle-output", *DEVICE_FLAGS,
          "-o", BENCH_YARDSTICKS, os.path.join(CSRC, "bench", "yardsticks.hip")])


RUNNER = "hip-runner"


def build_runner():
    """Plain C++ with the code object of its kernels embedded; reaches the
    runtime only through dlopen of the -shared-libs it is given."""
    runner = os.path.join(CSRC, "runner")
    _run([HIPCC, "--genco", "--no-gpu-bundle-output", *DEVICE_FLAGS,
          "-ffp-contract=off", "-o", os.path.join(BUILD, "runner_kernels.hsaco"),
          os.path.join(runner, "runner_kernels.hip")])
    _run([CXX, "-O2", "-std=c++17", f"-I{INCLUDE}", "-Wall",
          os.path.join(runner, "HipRunner.cpp"), os.path.join(runner, "RunnerBlob.S"),
          "-Wa,-I" + BUILD, "-o", os.path.join(HERE, RUNNER), "-ldl"])


def build_all(jobs=4):
    os.makedirs(BUILD, exist_ok=True)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        futures = [pool.submit(build_code_object, f) for f in KERNEL_FAMILIES]
        futures.append(pool.submit(build_reduce_release))
        futures.append(pool.submit(build_runtime))
        futures.append(pool.submit(build_math))
        futures.append(pool.submit(build_bench_timer))
        futures.append(pool.submit(build_bench_yardsticks))
        futures.append(pool.submit(build_runner))
        futures.append(pool.submit(build_python_runtime))
        for f in futures:
            f.result()
    build_offload()  # embeds the code objects built above


def libraries_present():
    return all(os.path.exists(os.path.join(HERE, n))
               for n in (RUNTIME_LIB, MATH_LIB, OFFLOAD_LIB, BENCH_TIMER_LIB, RUNNER,
                         PYTHON_RT_LIB)) \
        and os.path.exists(BENCH_YARDSTICKS)


if __name__ == "__main__":
    build_all()
    print("built:", RUNTIME_LIB, MATH_LIB, OFFLOAD_LIB)

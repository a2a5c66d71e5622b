"""Builds tests/host/_build/libgpux-mock.so: the gpux runtime's own sources
linked against the recording HIP table (HipApiMock.cpp) instead of libamdhip64,
so the C-ABI's host logic can be unit-tested without a GPU."""

import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
OUT = os.path.join(HERE, "_build", "libgpux-mock.so")


def build():
    runtime = os.path.join(ROOT, "numba_mlir_amd", "csrc", "runtime")
    srcs = [os.path.join(runtime, "GpuRuntime.cpp"),
            os.path.join(HERE, "HipApiMock.cpp")]
    if os.path.exists(OUT) and all(
            os.path.getmtime(OUT) >= os.path.getmtime(s) for s in srcs):
        return OUT
    os.makedirs(os.path.dirname(OUT), exist_ok=True)
    subprocess.run(
        ["g++", "-O1", "-g", "-fPIC", "-std=c++17", "-fvisibility=hidden",
         "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include",
         "-I" + os.path.join(ROOT, "include"), "-I" + runtime, "-shared", *srcs,
         "-Wl,--version-script=" + os.path.join(HERE, "export.map"),
         "-o", OUT, "-lpthread"], check=True)
    return OUT


if __name__ == "__main__":
    print(build())

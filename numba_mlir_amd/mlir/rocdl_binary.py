"""LLVM IR of a gpu.module in ROCDL form -> gfx950 code object for gpuxModuleLoad.

The reference ends its GPU pipeline by serialising each gpu.module to SPIR-V
and storing the bytes in the module's "gpu.binary" string attribute
(mlir/lib/Conversion/GpuToGpuRuntime.cpp:1234-1275, pipeline tail at
numba_mlir/numba_mlir/mlir_compiler/lib/pipelines/LowerToGpu.cpp:2204-2217);
the runtime hands those bytes to the driver (GpuModule, gpuxModuleLoad).  For
the HIP runtime the bytes are an AMDGPU code object.  This module is the
serialisation step on its own, run on the textual LLVM IR that
convert-gpu-to-rocdl + translation to LLVM IR give for a gpu.module -- the
same steps MLIR's #rocdl.target serialiser takes inside the compiler:

1. triple and data layout of amdgcn-amd-amdhsa are set on the module;
2. if the IR calls the device library (``__ocml_*``, ``__ockl_*``: math
   functions lower to those), ocml/ockl and the ``oclc`` control constants for
   the chip are linked in, only what is needed;
3. ``opt`` at the requested level;
4. ``llc`` to a relocatable object (packed-FP32 arithmetic off, as every
   kernel of this backend is built);
5. ``ld.lld -shared`` to the code object (an ELF shared object with one
   ``<kernel>.kd`` descriptor per ``amdgpu_kernel`` function).

The tools are the ROCm image's own LLVM (``/opt/rocm/llvm/bin``).
"""

import os
import re
import subprocess
import tempfile

LLVM_BIN = os.environ.get("NUMBA_MLIR_HIP_LLVM_BIN", "/opt/rocm/llvm/bin")
BITCODE_DIR = os.environ.get("NUMBA_MLIR_HIP_BITCODE", "/opt/rocm/amdgcn/bitcode")

TRIPLE = "amdgcn-amd-amdhsa"
DATALAYOUT = ("e-p:64:64-p1:64:64-p2:32:32-p3:32:32-p4:64:64-p5:32:32-p6:32:32-p7:160:256:256:32-"
              "p8:128:128:128:48-p9:192:256:256:32-i64:64-v16:16-v24:32-v32:32-v48:64-v96:128-"
              "v192:256-v256:256-v512:512-v1024:1024-v2048:2048-n32:64-S32-A5-G1-ni:7:8:9")
# Subgroup of a CDNA wavefront (the reference sizes group-reduction buffers for
# 8 lanes, LowerToGpu.cpp:1683-1688).
SUBGROUP_SIZE = 64


class SerializeError(RuntimeError):
    pass


def _tool(name):
    path = os.path.join(LLVM_BIN, name)
    if not os.path.exists(path):
        raise SerializeError(f"{name} not found under {LLVM_BIN} "
                             "(set NUMBA_MLIR_HIP_LLVM_BIN)")
    return path


def _run(cmd):
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise SerializeError(f"{os.path.basename(cmd[0])} failed:\n{r.stderr.strip()}")


def _with_target(ir):
    """The module with this target's triple and data layout (whatever it
    said before: a gpu.module carries none until a target is attached)."""
    lines = [line for line in ir.splitlines()
             if not re.match(r"\s*target\s+(triple|datalayout)\s*=", line)]
    head = [f'target datalayout = "{DATALAYOUT}"', f'target triple = "{TRIPLE}"']
    at = 0
    while at < len(lines) and (lines[at].startswith(";") or lines[at].startswith("source_filename")
                               or not lines[at].strip()):
        at += 1
    return "\n".join(lines[:at] + head + lines[at:]) + "\n"


def device_libraries(ir, chip="gfx950", fast=False):
    """Bitcode files the module needs from the device library, in link order
    (none when it calls nothing from there)."""
    if not re.search(r"@__(ocml|ockl)_", ir):
        return []
    isa = chip[3:] if chip.startswith("gfx") else chip
    names = ["ocml.bc", "ockl.bc",
             f"oclc_isa_version_{isa}.bc", "oclc_abi_version_600.bc",
             "oclc_wavefrontsize64_on.bc",
             "oclc_unsafe_math_on.bc" if fast else "oclc_unsafe_math_off.bc",
             "oclc_finite_only_on.bc" if fast else "oclc_finite_only_off.bc",
             "oclc_daz_opt_off.bc", "oclc_correctly_rounded_sqrt_on.bc"]
    paths = [os.path.join(BITCODE_DIR, n) for n in names]
    missing = [p for p in paths if not os.path.exists(p)]
    if missing:
        raise SerializeError("device library bitcode not found: " + ", ".join(missing))
    return paths


def serialize(ir, chip="gfx950", opt_level=3, fast=False, keep_dir=None):
    """Code object bytes for the LLVM IR text of one gpu.module."""
    if opt_level not in (0, 1, 2, 3):
        raise ValueError("opt_level must be 0..3")
    ir = _with_target(ir)
    with tempfile.TemporaryDirectory(prefix="nmhip-rocdl-") as tmp:
        work = keep_dir or tmp
        src = os.path.join(work, "module.ll")
        linked = os.path.join(work, "module.linked.bc")
        optimised = os.path.join(work, "module.opt.bc")
        obj = os.path.join(work, "module.o")
        out = os.path.join(work, "module.hsaco")
        with open(src, "w") as f:
            f.write(ir)
        libs = device_libraries(ir, chip, fast)
        if libs:
            _run([_tool("llvm-link"), "--only-needed", src] + libs + ["-o", linked])
        else:
            _run([_tool("llvm-link"), src, "-o", linked])
        machine = [f"-mtriple={TRIPLE}", f"-mcpu={chip}", "-mattr=-packed-fp32-ops"]
        _run([_tool("opt"), f"-O{opt_level}"] + machine + [linked, "-o", optimised])
        _run([_tool("llc"), f"-O{opt_level}"] + machine +
             ["-filetype=obj", "-relocation-model=pic", optimised, "-o", obj])
        _run([_tool("ld.lld"), "-shared", obj, "-o", out])
        with open(out, "rb") as f:
            return f.read()


def kernel_names(blob):
    """Names of the kernels of a code object: its ``<name>.kd`` descriptor
    symbols (dynamic symbol table of the ELF)."""
    import struct
    if blob[:4] != b"\x7fELF" or blob[4] != 2:
        raise ValueError("not a 64-bit ELF")
    shoff, = struct.unpack_from("<Q", blob, 0x28)
    shentsize, shnum = struct.unpack_from("<HH", blob, 0x3A)
    sections = [struct.unpack_from("<IIQQQQIIQQ", blob, shoff + k * shentsize)
                for k in range(shnum)]
    names = []
    for sec in sections:
        if sec[1] != 11:                 # SHT_DYNSYM
            continue
        _, _, _, _, off, size, link, _, _, entsize = sec
        stroff = sections[link][4]
        for k in range(size // entsize):
            st_name, = struct.unpack_from("<I", blob, off + k * entsize)
            end = blob.index(b"\0", stroff + st_name)
            name = blob[stroff + st_name:end].decode()
            if name.endswith(".kd"):
                names.append(name[:-3])
    return sorted(names)

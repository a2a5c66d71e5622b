"""Serialisation of a gpu.module's LLVM IR (ROCDL form) to a gfx950 code
object: the HIP counterpart of the reference's SerializeSPIRVPass
(mlir/lib/Conversion/GpuToGpuRuntime.cpp:1234-1275).  CPU only: the tools
cross-compile."""

import os

import pytest

from numba_mlir_amd.mlir import rocdl_binary as rb

CASES = os.path.join(os.path.dirname(os.path.abspath(__file__)), "rocdl_cases")

pytestmark = pytest.mark.skipif(not os.path.exists(os.path.join(rb.LLVM_BIN, "llc")),
                                reason="no LLVM tools in this image")


def _ir(name):
    with open(os.path.join(CASES, name + ".ll")) as f:
        return f.read()


def test_kernels_become_descriptors_of_an_elf_code_object():
    blob = rb.serialize(_ir("addf"))
    assert blob[:4] == b"\x7fELF"
    assert blob[18:20] == (224).to_bytes(2, "little")        # e_machine: EM_AMDGPU
    assert rb.kernel_names(blob) == ["main_kernel"]
    assert b"amdhsa.kernels" in blob and b"gfx950" in blob   # the metadata note names the chip


def test_device_library_is_linked_only_when_called():
    assert rb.device_libraries(_ir("addf")) == []
    libs = [os.path.basename(p) for p in rb.device_libraries(_ir("linalg_test"))]
    assert libs[:2] == ["ocml.bc", "ockl.bc"]
    assert "oclc_isa_version_950.bc" in libs and "oclc_wavefrontsize64_on.bc" in libs
    assert "oclc_unsafe_math_off.bc" in libs and "oclc_finite_only_off.bc" in libs
    fast = [os.path.basename(p) for p in rb.device_libraries(_ir("linalg_test"), fast=True)]
    assert "oclc_unsafe_math_on.bc" in fast
    blob = rb.serialize(_ir("linalg_test"))
    assert rb.kernel_names(blob) == ["foo_kernel_f32", "foo_kernel_f64"]
    # nothing of the library is left to resolve at load time
    assert b"__ocml_exp_f32" not in blob


def test_the_target_is_set_whatever_the_module_said(tmp_path):
    ir = 'target triple = "spirv64-unknown-unknown"\n' + _ir("addf")
    blob = rb.serialize(ir, keep_dir=str(tmp_path))
    text = (tmp_path / "module.ll").read_text()
    assert text.count("target triple") == 1 and rb.TRIPLE in text and rb.DATALAYOUT in text
    assert rb.kernel_names(blob) == ["main_kernel"]


def test_every_optimisation_level_and_errors():
    for level in range(4):
        assert rb.kernel_names(rb.serialize(_ir("addf"), opt_level=level)) == ["main_kernel"]
    with pytest.raises(ValueError):
        rb.serialize(_ir("addf"), opt_level=4)
    with pytest.raises(rb.SerializeError, match="llvm-link failed"):
        rb.serialize("define void @broken( {")
    with pytest.raises(ValueError):
        rb.kernel_names(b"not an elf")


def test_workgroup_memory_stays_dynamic():
    """The external workgroup-memory array takes no static LDS: the launch
    supplies the bytes."""
    blob = rb.serialize(_ir("group_sum"))
    assert rb.kernel_names(blob) == ["group_sum_f32"]
    at = blob.index(b".group_segment_fixed_size")
    # msgpack: the key, then a positive fixint 0
    assert blob[at + len(b".group_segment_fixed_size")] == 0

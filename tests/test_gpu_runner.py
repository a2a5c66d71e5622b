"""GPU: every program of the reference's mlir/test/L0_RUNNER through
hip-runner against the HIP runtime, its output checked by the reference's own
FileCheck directives (tests/golden/l0_runner_checks.json)."""

import json
import os
import subprocess

import pytest

import filecheck_lite

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
with open(os.path.join(ROOT, "tests", "golden", "l0_runner_checks.json")) as f:
    CHECKS = {k: v for k, v in json.load(f).items() if not k.startswith("_")}


@pytest.mark.parametrize("case", sorted(CHECKS))
def test_runner_case_matches_the_reference_checks(hip, case, tmp_path):
    from numba_mlir_amd import build
    runner = os.path.join(build.HERE, build.RUNNER)
    assert os.path.exists(runner), "hip-runner is not built"
    r = subprocess.run(
        [runner, f"mlir/test/L0_RUNNER/{case}.mlir", "-e", "main", "-entry-point-result=void",
         "-shared-libs=" + os.path.join(build.HERE, build.RUNTIME_LIB)],
        capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    directives = [tuple(c) for c in CHECKS[case]["checks"]]
    filecheck_lite.check(r.stdout, directives)
    if os.path.exists(filecheck_lite.LLVM_FILECHECK):     # LLVM's own, as the reference runs it
        accepted, message = filecheck_lite.llvm_filecheck(r.stdout, directives, tmp_path)
        assert accepted, message


# -- the same programs through the decorators ---------------------------------
# What a user of the reference writes in Python for these programs, translated
# and launched through gpuxLaunchKernel; the printed form (six significant
# digits, as printMemrefF32 shows them) is compared with the reference's.

with open(os.path.join(ROOT, "tests", "golden", "reference_vectors.json")) as f:
    GOLD = json.load(f)


def _printed(x):
    import numpy as np
    return np.array([float("%.6g" % v) for v in np.ravel(x)]).reshape(np.shape(x))


def test_addf_golden_as_a_kernel_over_group_ids(hip):
    """addf.mlir:21-28: eight groups of one work-item, indexed by the group id."""
    import numpy as np
    from numba_mlir_amd import kernel as K
    get_group_id = K.get_group_id

    @K.kernel
    def addf(a, b, c):
        i = get_group_id(0)
        c[i] = a[i] + b[i]

    g = GOLD["addf"]
    a, b = (hip.asarray(np.array(g[k], np.float32)) for k in ("a", "b"))
    c = hip.asarray(np.zeros(8, np.float32))
    launch = addf[(8,), (1,)]
    launch(a, b, c)
    assert launch.last_plan.info["grid"][0] == 8 and launch.last_plan.info["block"][0] == 1
    assert np.array_equal(_printed(c.asnumpy()), np.array(g["printed"]))


def test_linalg_gemvf_and_gemmf_goldens_as_kernels(hip):
    """linalg_gemvf.mlir:20-31, linalg_gemmf.mlir:23-34: the parallel
    dimensions are the work-items, the reduction a loop inside each."""
    import numpy as np
    from numba_mlir_amd import kernel as K
    get_global_id = K.get_global_id

    @K.kernel
    def gemv(A, x, y):
        i = get_global_id(0)
        for j in range(A.shape[1]):
            y[i] = y[i] + A[i, j] * x[j]

    @K.kernel
    def gemm(A, B, C):
        i = get_global_id(0)
        j = get_global_id(1)
        for k in range(A.shape[1]):
            C[i, j] = C[i, j] + A[i, k] * B[k, j]

    g = GOLD["linalg_gemvf"]
    A, x = hip.asarray(np.array(g["a"], np.float32)), hip.asarray(np.array(g["x"], np.float32))
    y = hip.asarray(np.array(g["y0"], np.float32))
    gemv[(3,), ()](A, x, y)
    assert np.array_equal(_printed(y.asnumpy()), np.array(g["printed"]))
    g = GOLD["linalg_gemmf"]
    A, B = hip.asarray(np.array(g["a"], np.float32)), hip.asarray(np.array(g["b"], np.float32))
    C = hip.asarray(np.array(g["c0"], np.float32))
    gemm[(3, 3), ()](A, B, C)
    assert np.array_equal(_printed(C.asnumpy()), np.array(g["printed"]))


@pytest.mark.parametrize("dtype", ["float32", "float64"])
def test_linalg_test_golden_as_one_fused_map(hip, dtype):
    """linalg_test_f32.mlir:7-122 (and its f64 twin): @foo's nineteen
    linalg.generic ops are add, sub, neg, mul, exp and div over a tensor<500>
    and five scalars; written as array arithmetic they fuse into one map.
    Expected print: 500 times 1.00002 (126-182)."""
    import numpy as np
    from numba_mlir_amd.decorators import njit

    def foo(a, s0, s1, s2, s3, s4):
        return (s0 + s1) + (s3 + (s4 - s3) / (np.exp((-s2) * (a - s0)) + a)) * (a - s0)

    g = GOLD["linalg_test"]
    t = np.dtype(dtype).type
    a = hip.asarray(np.full(g["n"], g["a"], t))
    f = njit(foo)
    out = f(a, *[t(v) for v in g["s"]])
    assert f.last_launch["path"] == "elementwise"
    got = out.asnumpy()
    assert got.dtype == t and got.shape == (g["n"],)
    assert np.array_equal(_printed(got), np.full(g["n"], g["printed"]))

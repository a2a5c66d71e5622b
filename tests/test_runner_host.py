"""Host-side tests of hip-runner, the standalone runner of the reference's
mlir/test/L0_RUNNER cases: its command line (the reference's RUN lines apply
as they are), its failure modes, the call sequence it replays against the
recording runtime, and the FileCheck subset the GPU test uses."""

import json
import os
import subprocess
import sys

import pytest

import filecheck_lite

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "tests", "host"))

with open(os.path.join(ROOT, "tests", "golden", "l0_runner_checks.json")) as f:
    CHECKS = {k: v for k, v in json.load(f).items() if not k.startswith("_")}


@pytest.fixture(scope="module")
def runner():
    from numba_mlir_amd import build
    path = os.path.join(build.HERE, build.RUNNER)
    if not os.path.exists(path):
        build.build_runner()
    return path


@pytest.fixture(scope="module")
def mock():
    import build_mock
    return build_mock.build()


def _run(runner, *args, env=None):
    full = dict(os.environ)
    full.update(env or {})
    return subprocess.run([runner, *args], capture_output=True, text=True, env=full,
                          timeout=60)


def test_every_reference_runner_test_has_a_case(runner):
    listed = dict(line.split("\t") for line in _run(runner, "--list").stdout.splitlines())
    assert set(listed) == set(CHECKS)
    for name, source in listed.items():
        assert CHECKS[name]["source"].startswith(source + ":")


def test_command_line_errors(runner, mock):
    std = ["-e", "main", "-entry-point-result=void"]
    assert "no -shared-libs" in _run(runner, "addf", *std).stderr
    assert "unknown case 'nosuch'" in _run(runner, "nosuch.mlir", *std,
                                           f"-shared-libs={mock}").stderr
    assert "entry point 'foo' not found" in _run(runner, "addf", "-e", "foo",
                                                 f"-shared-libs={mock}").stderr
    assert "unknown option" in _run(runner, "addf", "--frobnicate").stderr
    assert "cannot load" in _run(runner, "addf", *std, "-shared-libs=/nonexistent.so").stderr
    # a library that is not a gpux* runtime: every missing entry point is named
    r = _run(runner, "addf", *std, "-shared-libs=libm.so.6")
    assert r.returncode == 1 and "do not export gpuxQueueCreate, " in r.stderr
    assert "gpuxDuplicateQueue" in r.stderr
    assert _run(runner).returncode == 1


def test_replays_the_lowered_call_sequence(runner, mock):
    """The reference's own RUN line shape: a path to the .mlir file, several
    -shared-libs (the first ones without gpux* symbols).  Against the
    recording runtime the kernels do not run; the calls and the printed
    metadata are what is checked."""
    r = _run(runner, "/some/dir/addf.mlir", "-e", "main", "-entry-point-result=void",
             "-shared-libs=libm.so.6", f"-shared-libs={mock}",
             env={"NUMBA_MLIR_LOG_GPU_RUNTIME_CALLS": "1"})
    assert r.returncode == 0, r.stderr
    calls = [line.split()[0] for line in r.stdout.splitlines() if line.endswith(" enter")]
    calls = [c for c in calls if c.startswith("gpux")]
    alloc = ["gpuxAlloc", "gpuxWait", "gpuxDestroyEvent"]
    assert calls == (["gpuxQueueCreate", "gpuxModuleLoad"] + alloc * 3 +
                     ["gpuxKernelGet", "gpuxLaunchKernel", "gpuxWait", "gpuxDestroyEvent"] +
                     ["gpuxDeAlloc"] * 3 +
                     ["gpuxKernelDestroy", "gpuxModuleDestroy", "gpuxQueueDestroy"])
    filecheck_lite.check(r.stdout, CHECKS["addf"]["checks"][:1])
    # nineteen linalg.generic ops, fifteen of them launches of their own
    r = _run(runner, "linalg_test_f32", f"--shared-libs={mock}",
             env={"NUMBA_MLIR_LOG_GPU_RUNTIME_CALLS": "1"})
    assert r.returncode == 0, r.stderr
    assert r.stdout.count("gpuxLaunchKernel enter") == 15
    assert r.stdout.count("gpuxKernelGet enter") == 2


def test_filecheck_subset():
    out = "x = 0x1f rank = 1 data =\n[1,  2,   3, 4]\n[5, 6]\n"
    filecheck_lite.check(out, [("CHECK", "x = {{(0x)?[0-9a-f]*}}"), ("CHECK-SAME", "rank = 1"),
                               ("CHECK-NEXT", "[1, 2,"), ("CHECK-SAME", "3, 4]"),
                               ("CHECK-NEXT", "[5, 6]")])
    with pytest.raises(AssertionError, match="CHECK-NEXT"):
        filecheck_lite.check(out, [("CHECK", "rank = 1"), ("CHECK-NEXT", "[5, 6]")])
    with pytest.raises(AssertionError, match="CHECK-SAME"):
        filecheck_lite.check(out, [("CHECK", "[1, 2"), ("CHECK-SAME", "[5")])
    with pytest.raises(AssertionError, match="not found"):
        filecheck_lite.check(out, [("CHECK", "rank = 2")])


def _conforming_output(directives):
    """Printed output that satisfies the directives: each CHECK or CHECK-NEXT
    pattern on a line of its own, CHECK-SAME continuing the line, a regex
    block replaced by text it matches (an address, one digit)."""
    import re
    lines = []
    for kind, text in directives:
        text = re.sub(r"\{\{(.*?)\}\}",
                      lambda m: "2" if m.group(1) == "." else "0xdeadbeef", text)
        if kind == "CHECK-SAME":
            lines[-1] += " " + text
        else:
            lines.append(text)
    return "\n".join(lines) + "\n"


@pytest.mark.skipif(not os.path.exists(filecheck_lite.LLVM_FILECHECK),
                    reason="no LLVM FileCheck in this image")
def test_filecheck_subset_agrees_with_llvm_filecheck(tmp_path):
    """The directives of every runner test of the reference, against output
    that conforms and against the same output with one printed digit changed,
    one line dropped, one line inserted ahead of a CHECK-NEXT: the Python
    subset and LLVM's FileCheck give the same verdict each time."""
    with open(os.path.join(ROOT, "tests", "golden", "l0_runner_checks.json")) as f:
        cases = {k: v for k, v in json.load(f).items() if not k.startswith("_")}
    compared = 0
    for name, case in sorted(cases.items()):
        directives = [tuple(c) for c in case["checks"]]
        good = _conforming_output(directives)
        lines = good.splitlines()
        variants = [good]
        last = lines[-1]
        digit = next((k for k in range(len(last) - 1, -1, -1) if last[k].isdigit()), None)
        if digit is not None:
            changed = last[:digit] + str((int(last[digit]) + 1) % 10) + last[digit + 1:]
            variants.append("\n".join(lines[:-1] + [changed]) + "\n")
        variants.append("\n".join(lines[:-1]) + "\n")
        variants.append("\n".join(lines[:1] + ["something else"] + lines[1:]) + "\n")
        for out in variants:
            try:
                filecheck_lite.check(out, directives)
                mine = True
            except AssertionError:
                mine = False
            theirs, message = filecheck_lite.llvm_filecheck(out, directives, tmp_path)
            assert mine == theirs, (name, out, message)
            compared += 1
        assert filecheck_lite.llvm_filecheck(good, directives, tmp_path)[0], name
    assert compared >= 3 * len(cases)

"""The part of LLVM FileCheck the reference's runner tests use: CHECK,
CHECK-NEXT and CHECK-SAME directives whose patterns are fixed text with
``{{regex}}`` blocks, horizontal whitespace canonicalised on both sides."""

import re


def _canonical(text):
    return re.sub(r"[ \t]+", " ", text)


def _pattern(text):
    parts, pos = [], 0
    for m in re.finditer(r"\{\{(.*?)\}\}", text):
        parts.append(re.escape(_canonical(text[pos:m.start()])))
        parts.append("(?:" + m.group(1) + ")")
        pos = m.end()
    parts.append(re.escape(_canonical(text[pos:])))
    return re.compile("".join(parts).replace(r"\ ", " "))


def check(output, directives):
    """Raises AssertionError naming the first directive that does not match
    ``output``; ``directives`` is a list of (kind, pattern)."""
    lines = [_canonical(line) for line in output.splitlines()]
    line, col = 0, 0          # where the previous match ended
    matched = False
    for kind, text in directives:
        rx = _pattern(text.strip())
        if kind == "CHECK":
            at = None
            for k in range(line, len(lines)):
                m = rx.search(lines[k], col if k == line else 0)
                if m:
                    at = (k, m.end())
                    break
            assert at is not None, f"CHECK: {text!r} not found from line {line + 1} on"
            line, col = at
        elif kind == "CHECK-SAME":
            assert matched, "CHECK-SAME without a previous match"
            m = rx.search(lines[line], col) if line < len(lines) else None
            assert m, f"CHECK-SAME: {text!r} not on line {line + 1} after column {col}: " \
                      f"{lines[line][col:col + 120]!r}"
            col = m.end()
        elif kind == "CHECK-NEXT":
            assert matched, "CHECK-NEXT without a previous match"
            assert line + 1 < len(lines), f"CHECK-NEXT: {text!r}: no next line"
            m = rx.search(lines[line + 1])
            assert m, f"CHECK-NEXT: {text!r} not on line {line + 2}: {lines[line + 1][:120]!r}"
            line, col = line + 1, m.end()
        else:
            raise ValueError(f"unsupported directive {kind}")
        matched = True


LLVM_FILECHECK = "/opt/rocm/llvm/bin/FileCheck"


def llvm_filecheck(output, directives, workdir):
    """The same question put to LLVM's own FileCheck, where the ROCm image has
    one: (accepted, its message)."""
    import os
    import subprocess
    checks = os.path.join(str(workdir), "checks.txt")
    with open(checks, "w") as f:
        for kind, text in directives:
            f.write(f"// {kind}: {text}\n")
    r = subprocess.run([LLVM_FILECHECK, checks], input=output, capture_output=True, text=True,
                       timeout=60)
    return r.returncode == 0, r.stderr

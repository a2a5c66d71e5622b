"""Writes tests/golden/l0_runner_checks.json: the FileCheck directives the
reference's runner tests hold (mlir/test/L0_RUNNER/*.mlir), i.e. the expected
output of each program, as data: per file a list of [directive, pattern].

Run in the container that has the reference checked out:
    python tests/golden/extract_runner_checks.py [/root/reference]
"""

import json
import os
import re
import sys

HERE = os.path.dirname(os.path.abspath(__file__))


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    folder = os.path.join(ref, "mlir", "test", "L0_RUNNER")
    out = {"_comment": "FileCheck directives of the reference's runner tests "
                       "(expected printed output); data only."}
    directive = re.compile(r"//\s*(CHECK(?:-NEXT|-SAME)?):\s?(.*?)\s*$")
    for name in sorted(os.listdir(folder)):
        if not name.endswith(".mlir"):
            continue
        checks = []
        with open(os.path.join(folder, name)) as f:
            for lineno, line in enumerate(f, 1):
                m = directive.search(line)
                if m:
                    if not checks:
                        first = lineno
                    checks.append([m.group(1), m.group(2)])
                    last = lineno
        out[name[:-len(".mlir")]] = {
            "source": f"mlir/test/L0_RUNNER/{name}:{first}-{last}", "checks": checks}
    with open(os.path.join(HERE, "l0_runner_checks.json"), "w") as f:
        json.dump(out, f, indent=1)
        f.write("\n")


if __name__ == "__main__":
    main()

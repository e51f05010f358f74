"""Writes tests/golden/itensorbackend_members.json: the abstract members of the reference's ITensorBackend<'T>
(Tensor/Tensor/TensorBackend.fs:64-146) with the number of tuple arguments each takes.  The reference file is read as text in
the build container; the committed JSON is what the binding cross-check (tests/test_fsharp_binding.py) runs against.

    python tests/golden/extract_backend_members.py [/root/reference]
"""
import json
import os
import re
import sys


def members(path):
    text = open(path, encoding="utf-8-sig").read()
    start = text.index("and ITensorBackend<'T> =")
    end = text.index("/// Base tensor device.", start)
    body = text[start:end]
    # a declaration may run over two lines (SymmetricEigenDecomposition): join continuation lines first
    body = re.sub(r"\*\s*\n\s+", "* ", body)
    out = []
    for line in body.splitlines():
        line = line.strip()
        if line.startswith("//"):
            continue                       # BatchedLU is commented out in the reference
        m = re.match(r"abstract\s+(\w+)\s*:\s*(.*)$", line)
        if not m:
            continue
        name, sig = m.group(1), m.group(2)
        args = sig.rsplit("->", 1)[0]
        # tuple arguments are separated by '*' outside parentheses
        depth, n = 0, 1
        for ch in args:
            if ch == "(":
                depth += 1
            elif ch == ")":
                depth -= 1
            elif ch == "*" and depth == 0:
                n += 1
        out.append({"name": name, "args": n, "property": "with get" in sig})
    return out


if __name__ == "__main__":
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    ms = members(os.path.join(ref, "Tensor", "Tensor", "TensorBackend.fs"))
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "itensorbackend_members.json")
    with open(dst, "w") as f:
        json.dump({"source": "Tensor/Tensor/TensorBackend.fs:64-146", "members": ms}, f, indent=1)
    print(f"{len(ms)} members -> {dst}")

"""Writes tests/golden/print_layout_tables.json: the outputs of print_layout that the reference keeps in
its docstrings (src/layout.jl, the `julia> print_layout(...)` blocks), verbatim, keyed by their first
line (the printed layout).  Data only; run in the build container where /root/reference exists:

    python tests/golden/make_print_fixtures.py
"""
import json
import os
import re

SRC = "/root/reference/src/layout.jl"


def main():
    text = open(SRC).read()
    out = []
    for expr, body in re.findall(r"julia> print_layout\(([^\n]*)\)\n((?:.+\n)+?)\n", text):
        lines = []
        for l in body.splitlines():
            if l.startswith("julia>") or l.startswith("```"):
                break
            lines.append(l.rstrip())
        out.append({"expression": expr, "layout": lines[0], "lines": lines})
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "print_layout_tables.json")
    with open(dst, "w") as fh:
        json.dump(out, fh, indent=0)
    print("wrote", dst, len(out), "tables")


if __name__ == "__main__":
    main()

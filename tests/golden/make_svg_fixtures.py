"""Writes tests/golden/svg_owner_tables.json from the figures the reference's manual ships
(docs/src/assets/*.svg), which are renderings of print_typst(tiled_copy) / print_typst(tiled_mma)
(src/print.jl:46-172, 179-288).  Every table cell of those figures is a 26.5 pt square whose fill
colour is color_map[thr_idx & 31] (src/print.jl:135), so the colours record which thread owns which
element.  The fixture keeps, per figure and per table, the grid of fill colours (hex plus opacity):
data only.  Run in the build container, where /root/reference exists:

    python tests/golden/make_svg_fixtures.py
"""
import json
import os
import re
import xml.etree.ElementTree as ET

ASSETS = "/root/reference/docs/src/assets"
FIGURES = ["tiled_copy.svg", "ldmatrix.svg", "smem_copy_A.svg", "smem_copy_B.svg", "TF32F32.svg"]
NS = "{http://www.w3.org/2000/svg}"
CELL = 26.5


def cells_of(path):
    out = []

    def walk(e, tx, ty):
        t = e.get("transform")
        if t:
            m = re.match(r"translate\(([-\d.]+) ([-\d.]+)\)", t)
            if m:
                tx, ty = tx + float(m.group(1)), ty + float(m.group(2))
        if e.tag == NS + "path" and e.get("class") == "typst-shape" and e.get("fill") not in (None, "none"):
            if re.match(r"M 0 0 L 0 26\.5 L 26\.5 26\.5 L 26\.5 0 Z", e.get("d").strip()):
                colour = e.get("fill") + ("/" + e.get("fill-opacity") if e.get("fill-opacity") else "")
                out.append((int(round(tx / CELL)), int(round(ty / CELL)), colour))
        for c in e:
            walk(c, tx, ty)

    walk(ET.parse(path).getroot(), 0.0, 0.0)
    return out


def tables_of(cells):
    """Connected components of the cell grid (tables are separated by a label column or row)."""
    at = {(x, y): c for x, y, c in cells}
    seen, tables = set(), []
    for start in sorted(at, key=lambda p: (p[1], p[0])):
        if start in seen:
            continue
        comp, todo = [], [start]
        seen.add(start)
        while todo:
            x, y = todo.pop()
            comp.append((x, y))
            for q in ((x + 1, y), (x - 1, y), (x, y + 1), (x, y - 1)):
                if q in at and q not in seen:
                    seen.add(q)
                    todo.append(q)
        x0, y0 = min(p[0] for p in comp), min(p[1] for p in comp)
        w, h = max(p[0] for p in comp) - x0 + 1, max(p[1] for p in comp) - y0 + 1
        assert len(comp) == w * h, "table is not a full rectangle"
        tables.append({"col0": x0, "row0": y0, "rows": h, "cols": w,
                       "colours": [[at[(x0 + c, y0 + r)] for c in range(w)] for r in range(h)]})
    return tables


def main():
    out = {}
    for f in FIGURES:
        out[f] = tables_of(cells_of(os.path.join(ASSETS, f)))
        print(f, [(t["rows"], t["cols"], t["row0"], t["col0"]) for t in out[f]])
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "svg_owner_tables.json")
    with open(dst, "w") as fh:
        json.dump(out, fh, separators=(",", ":"))
    print("wrote", dst, os.path.getsize(dst), "bytes")


if __name__ == "__main__":
    main()

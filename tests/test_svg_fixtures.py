"""Thread ownership recorded in the figures of the reference's manual (docs/src/assets/*.svg,
rendered from print_typst, src/print.jl) against TiledCopy / TiledMMA of the oracle and of the
C++ host library.  A cell's colour is color_map[thr_idx & 31] (src/print.jl:135); the first seven
palette entries are plain rgb values (src/print.jl:100-106), the others are typst colour
expressions whose rendered value is taken from the figure itself, so for those the check is that
colour <-> thread is one bijection across all tables of a figure.

Pins function values of get_layoutS/D_TV, make_tiled_copy_A/B, the ldmatrix traits and
get_layoutA/B/C_TV, for which the reference has no other vector."""
import json
import os

import pytest

import layout_oracle as lo
import tiled_oracle as to
from layout_oracle import S, SL

HERE = os.path.dirname(os.path.abspath(__file__))
FIX = json.load(open(os.path.join(HERE, "golden", "svg_owner_tables.json")))
PALETTE_RGB = {0: "#afafff", 1: "#afffaf", 2: "#ffffaf", 3: "#ffafaf", 4: "#d2d2ff", 5: "#d2ffd2", 6: "#ffd2d2"}


def owners(layout_tv, rows, cols):
    """owner[r][c] = 1-based thread whose (thr, val) -> index layout reaches cell (r, c) of the
    column-major (rows, cols) tile; every cell must be reached exactly once (print.jl:226-233 inverts
    the TV layout, which needs exactly that)."""
    nthr, nval = int(lo.size(layout_tv, 1)), int(lo.size(layout_tv, 2))
    grid = [[None] * cols for _ in range(rows)]
    for t in range(1, nthr + 1):
        for v in range(1, nval + 1):
            idx = int(layout_tv((t, v))) - 1
            r, c = idx % rows, idx // rows
            assert c < cols and grid[r][c] is None, "TV layout is not a bijection onto the tile"
            grid[r][c] = t
    assert all(x is not None for row in grid for x in row)
    return grid


def owners_as_printed(layout_tv, rows, cols):
    """The table print_typst draws (src/print.jl:226-233 with src/atom/copy.jl:175-196): the TV
    layout is inverted with right_inverse and composed with the (rows, cols) tile; cell (m, n) then
    holds a (thr, val) index whose thread part is (idx - 1) % nthr + 1.  Unlike `owners` this is
    defined for the ldmatrix source side too, where half of the threads of LDSM_U32x2 alias the
    other half (stride 0 in traits/ldmatrix.jl:16-17)."""
    nthr = int(lo.size(layout_tv, 1))
    mn = lo.composition(lo.right_inverse(layout_tv), lo.make_layout((S(rows), S(cols))))
    return [[(int(mn((r + 1, c + 1))) - 1) % nthr + 1 for c in range(cols)] for r in range(rows)]


def check_figure(name, expected_tables):
    tables = FIX[name]
    assert len(tables) == len(expected_tables)
    colour_of, thread_of = {}, {}
    for tab, grid in zip(tables, expected_tables):
        assert (tab["rows"], tab["cols"]) == (len(grid), len(grid[0])), name
        for r in range(tab["rows"]):
            for c in range(tab["cols"]):
                key, col = grid[r][c] & 31, tab["colours"][r][c]
                assert colour_of.setdefault(key, col) == col, (name, r, c, "thread shown in two colours")
                assert thread_of.setdefault(col, key) == key, (name, r, c, "colour used by two threads")
    for k, rgb in PALETTE_RGB.items():
        if k in colour_of:
            assert colour_of[k] == rgb, (name, k)
    return len(colour_of)


def transpose(g):
    return [list(r) for r in zip(*g)]


def test_tiled_copy_figure():
    """docs/src/manual/tiled_matmul.md:30-49: thr (2,3):(3,1), val (2,3):(1,2), UniversalCopy{Float64}."""
    tc = to.make_tiled_copy(to.CopyAtom(to.UniversalCopy(64), 64), SL((2, 3), (3, 1)), SL((2, 3), (1, 2)))
    s, d = owners(tc.get_layoutS_TV(), 4, 9), owners(tc.get_layoutD_TV(), 4, 9)
    assert check_figure("tiled_copy.svg", [s, d]) == 6
    # the same table is printed in the text of the manual (tiled_matmul.md:9-14)
    assert s == [[1, 1, 1, 2, 2, 2, 3, 3, 3], [1, 1, 1, 2, 2, 2, 3, 3, 3], [4, 4, 4, 5, 5, 5, 6, 6, 6], [4, 4, 4, 5, 5, 5, 6, 6, 6]]


def test_ldmatrix_figure():
    """tiled_matmul.md:53-58: CopyAtom{LDSM_U32x4_N, UInt16}, thr (16,2), val (2,4): the source side
    is the ldmatrix address pattern, the destination side the register layout."""
    tc = to.make_tiled_copy(to.CopyAtom(to.LDSM["LDSM_U32x4_N"], 16), SL((16, 2)), SL((2, 4)))
    assert tuple(int(x) for x in tc.tiler_MN) == (32, 8)
    s, d = owners(tc.get_layoutS_TV(), 32, 8), owners(tc.get_layoutD_TV(), 32, 8)
    assert check_figure("ldmatrix.svg", [s, d]) == 32
    assert s == owners_as_printed(tc.get_layoutS_TV(), 32, 8) and d == owners_as_printed(tc.get_layoutD_TV(), 32, 8)
    assert s != d


def _tf32_mma():
    return to.make_tiled_mma(to.REFERENCE_MMA_OPS["MMAOP_16x8x8_F32TF32TF32F32_TN"])


def test_tf32_mma_figure():
    """docs/src/manual/tensor_core.md:15-19: print_typst(make_tiled_mma(MMAOP_16x8x8_F32TF32TF32F32_TN())).
    B is drawn as (K, N) above C, A to the left of C (src/print.jl:63-93)."""
    mma = _tf32_mma()
    a = owners(mma.get_layoutA_TV(), 16, 8)
    b = owners(mma.get_layoutB_TV(), 8, 8)      # (N, K)
    c = owners(mma.get_layoutC_TV(), 16, 8)
    assert check_figure("TF32F32.svg", [transpose(b), a, c]) == 32


def test_smem_copy_A_and_B_figures():
    """tensor_core.md:124-145: make_tiled_copy_A/B with ldmatrix atoms over the TF32 mma; the
    destination tables are the mma's A and B ownership (the manual says so at :132)."""
    mma = _tf32_mma()
    ca = to.make_tiled_copy_A(to.CopyAtom(to.LDSM["LDSM_U32x4_N"], 32), mma)
    sa, da = owners_as_printed(ca.get_layoutS_TV(), 16, 8), owners(ca.get_layoutD_TV(), 16, 8)
    assert sa == owners(ca.get_layoutS_TV(), 16, 8)
    assert check_figure("smem_copy_A.svg", [sa, da]) == 32
    assert da == owners(mma.get_layoutA_TV(), 16, 8)
    cb = to.make_tiled_copy_B(to.CopyAtom(to.LDSM["LDSM_U32x2_N"], 32), mma)
    sb, db = owners_as_printed(cb.get_layoutS_TV(), 8, 8), owners(cb.get_layoutD_TV(), 8, 8)
    check_figure("smem_copy_B.svg", [sb, db])
    assert db == owners(mma.get_layoutB_TV(), 8, 8)


def test_host_library_agrees_on_the_mma_figure():
    """The C++ host's layoutA/B/C_TV of the same atom give the same ownership tables."""
    import moye_hip as mh
    from moye_hip import layout as ml
    mma = _tf32_mma()
    host = mh.TiledMMAOp("MMAOP_16x8x8_F32TF32TF32F32_TN")
    tables = []
    for operand, rows, cols, want in (("A", 16, 8, mma.get_layoutA_TV()), ("B", 8, 8, mma.get_layoutB_TV()),
                                      ("C", 16, 8, mma.get_layoutC_TV())):
        got = lo.parse_layout(host.layout_tv(operand).text)
        assert owners(got, rows, cols) == owners(want, rows, cols), operand
        tables.append(owners(got, rows, cols))
    assert check_figure("TF32F32.svg", [transpose(tables[1]), tables[0], tables[2]]) == 32


# ---- the tables themselves: get_layoutX_MK/NK/MN + print_typst's cell rule, as text from the host library ----

def parse_tables(text):
    """{title: [[(thr, val), ...] per row]} from the text the host library prints."""
    import re
    tables, cur = {}, None
    for line in text.splitlines():
        cells = re.findall(r"T(\d+)V(\d+)", line)
        if cells:
            cur.append([(int(t), int(v)) for t, v in cells])
        elif line and not line.startswith(" "):
            cur = tables.setdefault(line.strip(), [])
    return tables


def thread_part(table):
    return [[t for t, _ in row] for row in table]


def check_cells_invert(table, layout_tv, rows):
    """Every cell (m, n) names a (thread, value) that the TV layout sends back to that cell."""
    for m, row in enumerate(table):
        for n, (t, v) in enumerate(row):
            assert int(layout_tv((t, v))) - 1 == m + rows * n, (m, n, t, v)


def test_printed_mma_tables_match_the_figure_and_the_oracle():
    import moye_hip as mh
    mma = _tf32_mma()
    host = mh.TiledMMAOp("MMAOP_16x8x8_F32TF32TF32F32_TN")
    tabs = parse_tables(host.print_tv(file=False))
    assert list(tabs) == ["B (K, N)", "A (M, K)", "C (M, N)"]
    want = {"A (M, K)": to.tv_table(*mma.get_layoutA_MK()), "C (M, N)": to.tv_table(*mma.get_layoutC_MN()),
            "B (K, N)": transpose(to.tv_table(*mma.get_layoutB_NK()))}
    for k in want:
        assert tabs[k] == [list(r) for r in want[k]], k
    # the figure of the manual draws exactly these threads (tensor_core.md:15-19)
    assert check_figure("TF32F32.svg", [thread_part(tabs["B (K, N)"]), thread_part(tabs["A (M, K)"]), thread_part(tabs["C (M, N)"])]) == 32
    check_cells_invert(tabs["A (M, K)"], mma.get_layoutA_TV(), 16)
    check_cells_invert(transpose(tabs["B (K, N)"]), mma.get_layoutB_TV(), 8)
    check_cells_invert(tabs["C (M, N)"], mma.get_layoutC_TV(), 16)


def test_printed_copy_tables_match_the_figures():
    import moye_hip as mh
    from moye_hip import layout as ml
    tc = mh.make_tiled_copy(mh.CopyAtom(64, 64), ml.Layout("(_2,_3):(_3,_1)"), ml.Layout("(_2,_3):(_1,_2)"))
    tabs = parse_tables(tc.print_tv(file=False))
    s, d = tabs["S (_4, _9)"], tabs["D (_4, _9)"]
    assert check_figure("tiled_copy.svg", [thread_part(s), thread_part(d)]) == 6
    otc = to.make_tiled_copy(to.CopyAtom(to.UniversalCopy(64), 64), SL((2, 3), (3, 1)), SL((2, 3), (1, 2)))
    assert s == [list(r) for r in to.tv_table(*otc.get_layoutS_MN())] and d == [list(r) for r in to.tv_table(*otc.get_layoutD_MN())]
    check_cells_invert(s, otc.get_layoutS_TV(), 4)
    # tiled_matmul.md:9-14 prints the thread table of this copy
    assert thread_part(s) == [[1, 1, 1, 2, 2, 2, 3, 3, 3], [1, 1, 1, 2, 2, 2, 3, 3, 3], [4, 4, 4, 5, 5, 5, 6, 6, 6], [4, 4, 4, 5, 5, 5, 6, 6, 6]]
    # make_tiled_copy_A over the TF32 mma: the destination table is the mma's A table (tensor_core.md:132)
    mma = mh.TiledMMAOp("MMAOP_16x8x8_F32TF32TF32F32_TN")
    ca = mh.make_tiled_copy_A(mh.CopyAtom(32, 32), mma)
    tabs = parse_tables(ca.print_tv(file=False))
    a_tab = parse_tables(mma.print_tv(file=False))["A (M, K)"]
    assert thread_part(tabs["D (_16, _8)"]) == thread_part(a_tab)


@pytest.mark.parametrize("atom,atom_layout,perm", [
    ("MFMA_F32_16x16x32_F16", (2, 2, 1), None), ("MFMA_F32_16x16x32_BF16", (2, 4, 1), None),
    ("MFMA_F32_32x32x16_F16", (2, 2, 1), None), ("MFMA_F32_16x16x4_F32", (1, 2, 1), None),
    ("MFMA_F32_16x16x32_F16", (2, 2, 1), (64, 64, 32)), ("MMAOP_16x8x8_F32TF32TF32F32_TN", (2, 2, 1), (32, 32, 8))])
def test_layouts_mn_of_tiled_mfma_agree_with_the_oracle(atom, atom_layout, perm):
    """get_layoutA_MK / B_NK / C_MN (src/atom/mma.jl:235-262) of tiled gfx950 atoms: host library against the oracle,
    and each cell's (thread, value) inverts through get_layoutX_TV."""
    import moye_hip as mh
    from moye_hip import layout as ml
    op = to.MFMA_OPS.get(atom) or to.REFERENCE_MMA_OPS[atom]
    operm = None if perm is None else tuple(S(v) for v in perm)
    omma = to.make_tiled_mma(op, SL(atom_layout), operm)
    host = mh.TiledMMAOp(atom, ml.static_layout(atom_layout), None if perm is None else tuple(ml.StaticInt(v) for v in perm))
    tabs = parse_tables(host.print_tv(file=False))
    for operand, key, fn, tv in (("A", "A (M, K)", omma.get_layoutA_MK, omma.get_layoutA_TV()),
                                 ("B", "B (K, N)", omma.get_layoutB_NK, omma.get_layoutB_TV()),
                                 ("C", "C (M, N)", omma.get_layoutC_MN, omma.get_layoutC_TV())):
        want_l, want_t = fn()
        got_l, got_t = host.layout_mn(operand)
        assert lo.parse_layout(got_l.text) == want_l and lo.parse_layout(got_t.text) == want_t, operand
        want = to.tv_table(want_l, want_t)
        got = transpose(tabs[key]) if operand == "B" else tabs[key]
        assert [list(r) for r in got] == [list(r) for r in want], operand
        check_cells_invert(got, tv, len(got))
        # every (thread, value) pair appears exactly once
        flat = [c for row in got for c in row]
        assert len(set(flat)) == len(flat)

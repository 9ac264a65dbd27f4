"""Pins the layout-algebra oracle (oracle/layout_oracle.py) against the reference's own known
answers and invariant helpers (test/stride.jl, test/int_tuple.jl, test/tuple_alg.jl,
test/layout.jl, test/array.jl of MoYe.jl), transcribed into tests/golden/layout_vectors.json."""
import itertools

import pytest

import layout_oracle as lo
from helpers import canon, load_vectors, split_top
from layout_oracle import COLON, S, SL, Layout, static

V = load_vectors()


def T(text):
    """int tuple / int / colon."""
    return lo.parse_int_tuple(canon(text))


def L(text):
    return lo.parse_layout(canon(text))


def X(text):
    """tile: layout, int, colon or `<...>` tuple of tiles."""
    text = canon(text)
    if text.startswith("<"):
        return tuple(X(p) for p in split_top(text[1:-1]))
    if text == ":":
        return COLON
    if ":" in text or text.startswith("("):
        return lo.parse_layout(text)
    return lo.parse_int_tuple(text)


def B(text):
    return text == "true"


OPS = {
    "coord_to_index": lambda a: lo.coord_to_index(*[T(x) for x in a]),
    "index_to_coord": lambda a: lo.index_to_coord(*[T(x) for x in a]),
    "compact_col_major": lambda a: lo.compact_col_major(T(a[0])),
    "compact_row_major": lambda a: lo.compact_row_major(T(a[0])),
    "make_layout_col": lambda a: lo.make_layout(T(a[0]), lo.GenColMajor),
    "make_layout_row": lambda a: lo.make_layout(T(a[0]), lo.GenRowMajor),
    "make_ordered_layout": lambda a: lo.make_ordered_layout(T(a[0]), T(a[1])),
    "capacity": lambda a: lo.capacity(T(a[0])),
    "shape_div": lambda a: lo.shape_div(T(a[0]), T(a[1])),
    "slice": lambda a: lo.slice_(T(a[0]), T(a[1])),
    "flatten": lambda a: lo.lflatten(L(a[0])),
    "coalesce": lambda a: lo.coalesce(L(a[0])),
    "composition": lambda a: lo.composition(L(a[0]), X(a[1])),
    "complement": lambda a: lo.complement(L(a[0]), T(a[1])),
    "logical_product": lambda a: lo.logical_product(L(a[0]), X(a[1])),
    "blocked_product": lambda a: lo.blocked_product(L(a[0]), L(a[1]), B(a[2])),
    "raked_product": lambda a: lo.raked_product(L(a[0]), L(a[1]), B(a[2])),
    "zipped_product": lambda a: lo.zipped_product(L(a[0]), X(a[1])),
    "tiled_product": lambda a: lo.tiled_product(L(a[0]), X(a[1])),
    "logical_divide": lambda a: lo.logical_divide(L(a[0]), X(a[1])),
    "zipped_divide": lambda a: lo.zipped_divide(L(a[0]), X(a[1])),
    "tiled_divide": lambda a: lo.tiled_divide(L(a[0]), X(a[1])),
    "recast": lambda a: lo.recast_layout(L(a[0]), int(a[1]), int(a[2])),
    "append": lambda a: lo.lappend(L(a[0]), int(a[1])),
    "prepend": lambda a: lo.lprepend(L(a[0]), int(a[1])),
}

LAYOUT_RESULT = {"make_layout_col", "make_layout_row", "make_ordered_layout", "flatten", "coalesce",
                 "composition", "complement", "logical_product", "blocked_product", "raked_product",
                 "zipped_product", "tiled_product", "logical_divide", "zipped_divide", "tiled_divide",
                 "recast", "append", "prepend"}


@pytest.mark.parametrize("case", V["known_answers"], ids=lambda c: "%s[%s]" % (c["op"], c["ref"]))
def test_known_answers(case):
    got = OPS[case["op"]](case["args"])
    if case["op"] in LAYOUT_RESULT:
        want = L(case["expect"])
        assert got == want, "%s: got %r want %r" % (case["ref"], got, want)
        if case.get("identical"):
            assert got.identical(want), "static-ness differs: got %r want %r" % (got, want)
    else:
        want = T(case["expect"])
        assert got == want, "%s: got %r want %r" % (case["ref"], got, want)
        if case.get("identical"):
            assert lo._same_static(got, want)


# ---- test/layout.jl invariant helpers -------------------------------------------------------


@pytest.mark.parametrize("text", V["coalesce_layouts"]["layouts"])
def test_coalesce_invariant(text):
    """test/layout.jl:39-48."""
    l = L(text)
    c = lo.coalesce(l)
    assert lo.ldepth(c) <= 1
    assert lo.size(c) == lo.size(l)
    for i in range(1, int(lo.size(l)) + 1):
        assert c(i) == l(i)


@pytest.mark.parametrize("pair", V["composition_pairs"]["pairs"], ids=lambda p: "%s o %s" % tuple(p))
def test_composition_invariant(pair):
    """test/layout.jl:140-147."""
    a, b = L(pair[0]), L(pair[1])
    c = lo.composition(a, b)
    assert lo.iscompatible(b.shape, c.shape)
    for i in range(1, int(lo.size(c)) + 1):
        assert c(i) == a(b(i))


@pytest.mark.parametrize("case", V["complement_cases"]["cases"], ids=lambda p: "%s|%s" % tuple(p))
def test_complement_invariant(case):
    """test/layout.jl:323-347."""
    l = L(case[0])
    cot = lo.cosize(l) if case[1] is None else T(case[1])
    r = lo.complement(l, cot)
    fl = lo.lfilter(l)
    assert int(lo.size(r)) >= int(cot) // int(lo.size(fl))
    assert int(lo.cosize(r)) <= -(-int(cot) // int(lo.cosize(l))) * int(lo.cosize(l))
    completed = lo.make_layout(l, r)
    assert int(lo.cosize(completed)) >= int(cot)
    lvals = {int(l(j)) for j in range(1, int(lo.size(l)) + 1)}
    for i in range(2, int(lo.size(r)) + 1):
        assert r(i - 1) < r(i)
        assert int(r(i)) not in lvals
    assert int(lo.size(r)) <= int(lo.cosize(r))
    assert int(lo.cosize(r)) >= int(cot) // int(lo.size(fl))
    assert int(lo.cosize(completed)) <= int(lo.cosize(r)) + int(lo.cosize(l))
    if lo.is_static(completed.stride):
        assert int(lo.size(lo.complement(completed))) == 1


@pytest.mark.parametrize("pair", V["logical_product_pairs"]["pairs"], ids=lambda p: "%s x %s" % tuple(p))
def test_logical_product_invariant(pair):
    """test/layout.jl:430-435."""
    a, b = L(pair[0]), L(pair[1])
    c = lo.logical_product(a, b)
    assert lo.lrank(c) == 2
    assert lo.iscompatible(a.shape, c[1].shape)


@pytest.mark.parametrize("pair", V["logical_divide_pairs"]["pairs"], ids=lambda p: "%s / %s" % tuple(p))
def test_logical_divide_invariant(pair):
    """test/layout.jl:536-541."""
    a, b = L(pair[0]), L(pair[1])
    c = lo.logical_divide(a, b)
    assert lo.lrank(c) == 2
    assert lo.iscompatible(b.shape, c[1].shape)
    # what the mathematics fixes: a divide only re-orders the domain
    assert sorted(lo.all_indices(c)) == sorted(lo.all_indices(a))


@pytest.mark.parametrize("text", V["right_inverse_layouts"]["layouts"])
def test_right_inverse_invariant(text):
    """test/layout.jl:624-633."""
    l = L(text)
    inv = lo.right_inverse(l)
    for i in range(1, int(lo.size(inv)) + 1):
        assert l(inv(i)) == i


@pytest.mark.parametrize("tab", V["tables"], ids=lambda t: t["ref"])
def test_printed_tables(tab):
    """The `print_layout` tables in the docstrings of src/layout.jl."""
    l = L(tab["layout"])
    for r in range(tab["rows"]):
        for c in range(tab["cols"]):
            assert l((r + 1, c + 1)) == tab["cells"][r][c]


# ---- test/tuple_alg.jl, test/int_tuple.jl (plain Julia tuples -> Python tuples) --------------


def test_tuple_algorithms():
    """test/tuple_alg.jl:4-85."""
    assert lo.unflatten((1, 2, 3), (0, 0, 0)) == (1, 2, 3)
    assert lo.unflatten((1, 2, 3, 4), (0, (0, (0, 0)))) == (1, (2, (3, 4)))
    assert lo.unflatten((1, 2, 3, 4), ((0, 0), (0, 0))) == ((1, 2), (3, 4))
    assert lo.unflatten((1, 2, 3, 4, 5), (0, (0, 0), 0)) == (1, (2, 3), 4)
    assert lo.unflatten((1, 2, 3, 4, 5, 6), (0, (0, (0, (0, (0, 0)))))) == (1, (2, (3, (4, (5, 6)))))
    assert lo.unflatten((), ()) == ()
    assert lo.front(((2, 3), 4)) == 2
    assert lo.back((2, (3, 4))) == 4
    assert lo.tuple_cat((1, 2), (3, 4)) == (1, 2, 3, 4)
    assert lo.insert((1, 2, 3), 10, 2) == (1, 10, 2, 3)
    assert lo.remove((1, 2, 3), 2) == (1, 3)
    assert lo.replace((1, 2, 3), 10, 2) == (1, 10, 3)
    assert lo.unwrap(((1,),)) == 1
    assert lo.append((1, 2), 3) == (1, 2, 3)
    assert lo.append((1, 2), 3, 4) == (1, 2, 3, 3)
    assert lo.prepend((1, 2), 3) == (3, 1, 2)
    assert lo.prepend((1, 2), 3, 4) == (3, 3, 1, 2)
    assert lo.escan(lambda a, b: a * b, (1, 2, 3, 4, 5), 10) == (10, 10, 20, 60, 240)
    assert lo.zip2_by((("A", "a"), (("B", "b"), ("C", "c")), "d"), (0, (0, 0))) == \
        (("A", ("B", "C")), ("a", ("b", "c"), "d"))
    assert lo.repeat_like((2, 3, 4), 1) == (1, 1, 1)
    assert lo.repeat_like(((2, 3), (4, 5)), 1) == ((1, 1), (1, 1))


def test_comparisons_and_increment():
    """test/int_tuple.jl:46-96."""
    el, cl = lo.elem_less, lo.colex_less
    assert el((1, 2, 3), (1, 2, 4)) and not el((1, 2, 3), (1, 2, 3))
    assert el((1, 2, 3), (1, 2, 3, 1)) and not el((1, 2, 3, 1), (1, 2, 3))
    assert not el(((1, 2, 3),), ((1, 2, 3),)) and el(((1, 2, 3),), ((1, 2, 4),))
    assert el(((1, 2, 3),), ((1, 2, 3), 1)) and el(((1, 2, 3), 1), ((1, 2, 3), 2))
    assert not el(((1, 2, 3), 2), ((1, 2, 4), 1))
    assert el(((1, 2), (3, 4)), ((5, 6), (7, 8))) and el(((1, 2), (3, 4)), ((1, 2), (7, 8)))
    assert not el(((1, 2), (3, 4)), ((1, 2), (1, 8))) and not el(((1, 2), (3, 4)), ((3, 4), (3, 4)))
    assert el(((1, 2), (3, 4)), ((3, 4), (3, 4, 1))) and el(((1, 2), (3, 4)), ((3, 4), (3, 4), 1))
    assert cl((1, 2, 3), (1, 2, 4)) and not cl((1, 2, 3), (1, 2, 3))
    assert cl((1, 2, 3), (1, 1, 2, 3)) and not cl((1, 1, 2, 3), (1, 2, 3))
    assert not cl(((1, 2, 3),), ((1, 2, 3),)) and cl(((0, 2, 3),), ((1, 2, 3),))
    assert cl(((1, 2, 3),), (1, (1, 2, 3))) and cl((1, (1, 2, 3)), (2, (1, 2, 3)))
    assert cl((2, (1, 2, 3)), (1, (2, 2, 3)))
    assert cl(((1, 2), (3, 4)), ((5, 6), (7, 8))) and cl(((1, 2), (3, 4)), ((2, 3), (3, 4)))
    assert cl(((1, 2), (3, 4)), ((1, 3), (3, 4))) and not cl(((5, 4), (3, 4)), ((3, 4), (3, 4)))
    assert cl(((1, 2), (3, 4)), ((1, 1, 2), (3, 4)))
    inc = lo.increment
    assert inc((1, 1), (3, 4)) == (2, 1) and inc((3, 1), (3, 4)) == (1, 2) and inc((3, 4), (3, 4)) == (1, 1)
    assert inc((2, (2, 1), 1), (2, (2, 3), 3)) == (1, (1, 2), 1)
    assert inc((2, (2, 2), 1), (2, (2, 3), 3)) == (1, (1, 3), 1)
    assert inc((2, (2, 3), 1), (2, (2, 3), 3)) == (1, (1, 1), 2)
    assert inc((2, (2, 3), 3), (2, (2, 3), 3)) == (1, (1, 1), 1)


def test_errors():
    """test/stride.jl:54 and the divisibility assert of int_tuple.jl:87-90."""
    with pytest.raises(ValueError):
        lo.index_to_coord(9, (3, 4), (1, 3, 5))
    with pytest.raises(AssertionError):
        lo.shape_div(S(6), S(4))
    assert lo.shape_div(6, 4) == 1
    with pytest.raises(ValueError):
        lo.logical_divide(SL((4, 4)), (S(2), S(2), S(2)))


def test_static_propagation():
    """test/static.jl:4-10 and test/layout.jl:4-12 — static in, static out."""
    l = lo.make_layout(static((3, 4)), static((1, 2)))
    assert isinstance(lo.size(l), S) and isinstance(lo.cosize(l), S)
    assert isinstance(l(S(1)), S) and isinstance(l(static((1, 2))), S)
    assert not isinstance(l(2), S)


# ---- what the mathematics fixes, by brute force ----------------------------------------------


def _all_coords(shape):
    if not isinstance(shape, tuple):
        return list(range(1, int(shape) + 1))
    return [tuple(reversed(c)) for c in itertools.product(*[_all_coords(s) for s in reversed(shape)])]


@pytest.mark.parametrize("text", ["@(3,4):(2,8)", "@(3,(2,2)):(2,(16,8))", "@((2,3),(4,(2,2))):((1,2),(6,(24,48)))",
                                  "(5,3):(7,1)"])
def test_linear_index_is_colex_over_hier_coords(text):
    """l(i) for an integer i must equal l(c_i) where c_i is the i-th hierarchical coordinate in
    colexicographic order, and equal the closed form sum((c-1)*d)+1."""
    l = L(text)
    coords = _all_coords(l.shape)
    fs, fd = lo.flatten(l.shape), lo.flatten(l.stride)
    for i, c in enumerate(coords, start=1):
        assert l(i) == l(c)
        fc = lo.flatten(c)
        assert l(c) == sum((int(a) - 1) * int(d) for a, d in zip(fc, fd)) + 1
    assert len(coords) == int(lo.size(l))
    assert lo.cosize(l) == l(lo.size(l))
    del fs


def test_divide_of_config_shapes():
    """Tile views the kernels are driven by (fp16 4096^3 TN GEMM with a 128x128x32 CTA tile)."""
    a = lo.make_layout(static((4096, 4096)), static((4096, 1)))
    z = lo.zipped_divide(a, static((128, 32)))
    assert z == L("@((128,32),(32,128)):((4096,1),(524288,32))")
    sub, off = lo.slice_and_offset(z, ((COLON, COLON), (3, COLON)))
    assert sub == L("@(128,32,128):(4096,1,32)") and off == 2 * 524288
    # brute force on a small analogue: every element appears in exactly one tile
    small = lo.make_layout(static((8, 12)), static((12, 1)))
    zs = lo.zipped_divide(small, static((4, 3)))
    assert sorted(lo.all_indices(zs)) == sorted(lo.all_indices(small))


def test_text_roundtrip():
    for text in ["(_2, (_1, _6)):(_1, (_6, _2))", "(4,):(2,)", "_12:_1", "((1, (2, 4)), 1):((_1, (1, 2)), 8)"]:
        assert repr(lo.parse_layout(text)) == text


def test_print_layout_matches_the_reference_docstrings():
    """The print_layout outputs the reference keeps in its docstrings (src/layout.jl), verbatim: pins the
    text format of src/print.jl:7-44 and, once more, the index every cell holds."""
    import json
    import os
    tables = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "print_layout_tables.json")))
    assert len(tables) == 10
    for t in tables:
        got = [line.rstrip() for line in lo.print_layout(lo.parse_layout(t["layout"])).split("\n")]
        assert got == t["lines"], t["expression"]


def test_int32_known_answers():
    """test/layout.jl:4-12 of the reference: a layout called with an Int32 gives an Int32, for a static layout
    (promote_rule(StaticInt, Int32) = Int32, src/utilities.jl:4-6) and for a layout made of Int32 shapes; plus what
    Julia's promotion and wrap-around fix for the other combinations."""
    import layout_oracle as lo
    a = lo.parse_layout("(_2,(_2,_2)):(_2,(_1,_4))")
    r = a(lo.I32(2))
    assert type(r) is lo.I32 and int(r) == 3 and repr(r) == "3i32"
    b = lo.make_layout((lo.I32(2), lo.I32(4)))
    assert repr(b) == "(2i32, 4i32):(_1, 2i32)"
    r = b(lo.I32(2))
    assert type(r) is lo.I32 and int(r) == 2
    assert type(b(2)) is int and b(2) == 2                       # Int32 with an Int is an Int
    assert type(a(2)) is int and type(a(lo.S(2))) is lo.S        # static stays static
    assert repr(lo.parse_layout("(2i32,4):(_1,2i32)")(lo.I32(7))) == "7"   # one Int among the inputs: an Int
    # hierarchical coordinates and the way back
    assert repr(a((lo.I32(2), (lo.I32(1), lo.I32(2))))) == "7i32"
    assert repr(lo.index_to_coord(lo.I32(7), a.shape, a.stride)) == "(2i32, (1i32, 2i32))"
    assert repr(lo.index_to_coord(lo.I32(5), (lo.I32(3), lo.I32(4)))) == "(2i32, 2i32)"
    # Int32 arithmetic wraps as Julia's does: (4 - 1) * 2^30 = 3 * 2^30 -> -2^30, plus one
    w = lo.parse_layout("4i32:1073741824i32")
    assert repr(w(lo.I32(4))) == "-1073741823i32" and w(4) == 3 * 2 ** 30 + 1
    assert repr(lo.parse_int_tuple("(2i32, (_3, 4))")) == "(2i32, (_3, 4))"
    # the algebra carries the type: products of Int32 shapes, shape_div, coalesce of dynamic modes
    assert repr(lo.compact_col_major((lo.I32(3), lo.I32(5), lo.S(2)))) == "(_1, 3i32, 15i32)"
    assert repr(lo.shape_div(lo.I32(12), lo.S(4))) == "3i32" and repr(lo.shape_div(lo.I32(12), 4)) == "3"
    assert repr(lo.size(lo.parse_layout("(2i32,_3,4i32):(_1,2i32,6i32)"))) == "24i32"

"""The shipped host-side layout algebra (C++ inside libmoye_hip.so, reached through the C ABI and
the moye_hip Python mirror) against (1) the reference's own known answers and invariant helpers
(tests/golden/layout_vectors.json) and (2) the independent Python oracle on seeded random cases.
No GPU needed."""
import random

import pytest

import layout_oracle as lo
import numpy as np
import moye_hip as mh
import tiled_oracle as to
from helpers import canon, load_vectors, split_top

from moye_hip import layout as ml
from moye_hip import array as ma
from moye_hip import MoyeError
from moye_hip._lib import ERR_RANK, ERR_SHAPE, ERR_PARSE, ERR_UNSUPPORTED

V = load_vectors()


def L(text):
    return ml.Layout(canon(text))


def T(text):
    return ml.parse_tuple(canon(text))


def X(text):
    return canon(text)  # tiles go through as text


def OL(text):
    return lo.parse_layout(canon(text))


def OX(text):
    text = canon(text)
    if text.startswith("<"):
        return tuple(OX(p) for p in split_top(text[1:-1]))
    if text == ":":
        return lo.COLON
    if ":" in text or text.startswith("("):
        return lo.parse_layout(text)
    return lo.parse_int_tuple(text)


OPS = {
    "coord_to_index": lambda a: ml.coord_to_index(*[T(x) for x in a]),
    "index_to_coord": lambda a: ml.index_to_coord(*[T(x) for x in a]),
    "compact_col_major": lambda a: ml.compact_col_major(T(a[0])),
    "compact_row_major": lambda a: ml.compact_row_major(T(a[0])),
    "make_layout_col": lambda a: ml.make_layout(T(a[0]), ml.GenColMajor),
    "make_layout_row": lambda a: ml.make_layout(T(a[0]), ml.GenRowMajor),
    "make_ordered_layout": lambda a: ml.make_ordered_layout(T(a[0]), T(a[1])),
    "capacity": lambda a: ml.tuple_op("capacity", T(a[0])),
    "shape_div": lambda a: ml.shape_div(T(a[0]), T(a[1])),
    "slice": lambda a: ml.tuple_op("slice", T(a[0]), T(a[1])),
    "flatten": lambda a: ml.flatten(L(a[0])),
    "coalesce": lambda a: ml.coalesce(L(a[0])),
    "composition": lambda a: ml.composition(L(a[0]), X(a[1])),
    "complement": lambda a: ml.complement(L(a[0]), T(a[1])),
    "logical_product": lambda a: ml.logical_product(L(a[0]), X(a[1])),
    "blocked_product": lambda a: ml.blocked_product(L(a[0]), L(a[1]), a[2] == "true"),
    "raked_product": lambda a: ml.raked_product(L(a[0]), L(a[1]), a[2] == "true"),
    "zipped_product": lambda a: ml.zipped_product(L(a[0]), X(a[1])),
    "tiled_product": lambda a: ml.tiled_product(L(a[0]), X(a[1])),
    "logical_divide": lambda a: ml.logical_divide(L(a[0]), X(a[1])),
    "zipped_divide": lambda a: ml.zipped_divide(L(a[0]), X(a[1])),
    "tiled_divide": lambda a: ml.tiled_divide(L(a[0]), X(a[1])),
    "recast": lambda a: ml.recast(L(a[0]), int(a[1]), int(a[2])),
    "append": lambda a: ml.append(L(a[0]), int(a[1])),
    "prepend": lambda a: ml.prepend(L(a[0]), int(a[1])),
}
LAYOUT_RESULT = {"make_layout_col", "make_layout_row", "make_ordered_layout", "flatten", "coalesce", "composition",
                 "complement", "logical_product", "blocked_product", "raked_product", "zipped_product",
                 "tiled_product", "logical_divide", "zipped_divide", "tiled_divide", "recast", "append", "prepend"}


def _same_static(a, b):
    if isinstance(a, tuple):
        return isinstance(b, tuple) and len(a) == len(b) and all(_same_static(x, y) for x, y in zip(a, b))
    return isinstance(a, ml.StaticInt) == isinstance(b, ml.StaticInt)


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
            assert _same_static(got, want)


def _values(l):
    return [l(i) for i in range(1, ml.size(l) + 1)]


@pytest.mark.parametrize("text", V["coalesce_layouts"]["layouts"])
def test_coalesce_invariant(text):
    l = L(text)
    c = ml.coalesce(l)
    assert ml.depth(c) <= 1 and ml.size(c) == ml.size(l)
    assert _values(c) == _values(l)
    assert c.identical(ml.Layout(repr(lo.coalesce(OL(text)))))


@pytest.mark.parametrize("pair", V["composition_pairs"]["pairs"], ids=lambda p: "%s o %s" % tuple(p))
def test_composition_invariant(pair):
    a, b = L(pair[0]), L(pair[1])
    c = ml.composition(a, b)
    assert ml.tuple_op("iscompatible", b.shape, c.shape)
    for i in range(1, ml.size(c) + 1):
        assert c(i) == a(b(i))
    assert c.identical(ml.Layout(repr(lo.composition(OL(pair[0]), OL(pair[1])))))


@pytest.mark.parametrize("case", V["complement_cases"]["cases"], ids=lambda p: "%s|%s" % tuple(p))
def test_complement_invariant(case):
    l = L(case[0])
    cot = ml.cosize(l) if case[1] is None else int(T(case[1]))
    r = ml.complement(l, ml.StaticInt(cot))
    fl = ml.filter(l)
    assert ml.size(r) >= cot // ml.size(fl)
    assert ml.cosize(r) <= -(-cot // ml.cosize(l)) * ml.cosize(l)
    completed = ml.make_layout(l, r)
    assert ml.cosize(completed) >= cot
    lvals = set(_values(l))
    rv = _values(r)
    for i in range(1, len(rv)):
        assert rv[i - 1] < rv[i] and rv[i] not in lvals
    assert ml.size(r) <= ml.cosize(r) >= cot // ml.size(fl)
    assert ml.cosize(completed) <= ml.cosize(r) + ml.cosize(l)
    assert ml.size(ml.complement(completed)) == 1
    want = lo.complement(OL(case[0]), lo.S(cot))
    assert r.identical(ml.Layout(repr(want)))


@pytest.mark.parametrize("pair", V["logical_product_pairs"]["pairs"], ids=lambda p: "%s x %s" % tuple(p))
def test_logical_product_invariant(pair):
    a, b = L(pair[0]), L(pair[1])
    c = ml.logical_product(a, b)
    assert ml.rank(c) == 2 and ml.tuple_op("iscompatible", a.shape, c[1].shape)
    assert c.identical(ml.Layout(repr(lo.logical_product(OL(pair[0]), OL(pair[1])))))


@pytest.mark.parametrize("pair", V["logical_divide_pairs"]["pairs"], ids=lambda p: "%s / %s" % tuple(p))
def test_logical_divide_invariant(pair):
    a, b = L(pair[0]), L(pair[1])
    c = ml.logical_divide(a, b)
    assert ml.rank(c) == 2 and ml.tuple_op("iscompatible", b.shape, c[1].shape)
    assert sorted(_values(c)) == sorted(_values(a))
    assert c.identical(ml.Layout(repr(lo.logical_divide(OL(pair[0]), OL(pair[1])))))


@pytest.mark.parametrize("text", V["right_inverse_layouts"]["layouts"])
def test_right_inverse_invariant(text):
    l = L(text)
    inv = ml.right_inverse(l)
    for i in range(1, ml.size(inv) + 1):
        assert l(inv(i)) == i
    assert inv.identical(ml.Layout(repr(lo.right_inverse(OL(text)))))


@pytest.mark.parametrize("tab", V["tables"], ids=lambda t: t["ref"])
def test_printed_tables(tab):
    l = L(tab["layout"])
    for r in range(tab["rows"]):
        for c in range(tab["cols"]):
            assert l((r + 1, c + 1)) == tab["cells"][r][c]


# ---- seeded differential test against the oracle ------------------------------------------------

def _rand_layout(rng, static_prob=0.85):
    """A random injective-ish layout: compact strides of a random nested shape, modes shuffled,
    occasionally a stride-0 mode or a dynamic integer."""
    n = rng.randint(1, 4)
    sizes = [rng.choice([1, 2, 2, 3, 4, 4, 6, 8]) for _ in range(n)]
    order = list(range(n))
    rng.shuffle(order)
    strides, cur = [0] * n, 1
    for k in order:
        strides[k] = cur * rng.choice([1, 1, 1, 2])
        cur = strides[k] * sizes[k]
    if rng.random() < 0.15:
        strides[rng.randrange(n)] = 0

    def I(v, allow_dyn=True):
        return ("_%d" if (rng.random() < static_prob or not allow_dyn) else "%d") % v

    sh = [I(s) for s in sizes]
    st = [I(d) for d in strides]
    if n >= 3 and rng.random() < 0.5:  # nest the first two modes
        return "((%s,%s),%s):((%s,%s),%s)" % (sh[0], sh[1], ",".join(sh[2:]), st[0], st[1], ",".join(st[2:]))
    if n == 1:
        return "%s:%s" % (sh[0], st[0])
    return "(%s):(%s)" % (",".join(sh), ",".join(st))


def _both(fn_m, fn_o):
    """Run the product and the oracle; both must fail, or both succeed with identical text."""
    try:
        want = repr(fn_o())
        o_err = None
    except Exception as e:  # noqa: BLE001 - any oracle failure counts
        want, o_err = None, e
    try:
        got = fn_m().text
        m_err = None
    except MoyeError as e:
        got, m_err = None, e
    assert (o_err is None) == (m_err is None), "oracle: %r / product: %r" % (o_err or want, m_err or got)
    if want is not None:
        assert got == want


def test_random_differential():
    rng = random.Random(20240611)
    n_checked = 0
    for _ in range(400):
        ta, tb = _rand_layout(rng), _rand_layout(rng)
        a, b, oa, ob = ml.Layout(ta), ml.Layout(tb), lo.parse_layout(ta), lo.parse_layout(tb)
        _both(lambda: ml.coalesce(a), lambda: lo.coalesce(oa))
        _both(lambda: ml.filter(a), lambda: lo.lfilter(oa))
        _both(lambda: ml.right_inverse(a), lambda: lo.right_inverse(oa))
        _both(lambda: ml.composition(a, b), lambda: lo.composition(oa, ob))
        _both(lambda: ml.complement(a), lambda: lo.complement(oa))
        _both(lambda: ml.logical_divide(a, b), lambda: lo.logical_divide(oa, ob))
        _both(lambda: ml.logical_product(a, b), lambda: lo.logical_product(oa, ob))
        _both(lambda: ml.raked_product(a, b, True), lambda: lo.raked_product(oa, ob, True))
        _both(lambda: ml.blocked_product(a, b), lambda: lo.blocked_product(oa, ob))
        _both(lambda: ml.recast(a, 4, 2), lambda: lo.recast_layout(oa, 4, 2))
        _both(lambda: ml.recast(a, 2, 4), lambda: lo.recast_layout(oa, 2, 4))
        assert ml.size(a) == int(lo.size(oa)) and ml.cosize(a) == int(lo.cosize(oa))
        for i in range(1, min(ml.size(a), 12) + 1):
            assert a(i) == int(oa(i))
        n_checked += 1
    assert n_checked == 400


# ---- arrays, tiling verbs, TiledMMA, TiledCopy ---------------------------------------------------

@pytest.mark.parametrize("case", V["tiling"], ids=lambda c: c["ref"])
def test_tile_and_parallelize(case):
    lay = L(case["array"])
    x = ma.MoYeArray(0, 7, lay)  # U32 elements at address 0: offsets are readable from .ptr
    tile = X(case["tile"])
    if case["op"] == "local_tile":
        r = ma.local_tile(x, tile, ml.parse_tuple(case["coord"]))
    elif "index" in case:
        r = ma.local_partition(x, tile, case["index"])
    else:
        r = ma.local_partition(x, tile, ml.parse_tuple(case["coord"]))
    if "expect_layout" in case:
        assert r.layout == L(case["expect_layout"])
    if "expect_rank" in case:
        assert ml.rank(r.layout) == case["expect_rank"]
    if "expect_values" in case:  # element k of a 1..N buffer sits at offset k-1
        vals = [r.ptr // 4 + r.layout(i) for i in range(1, ml.size(r.layout) + 1)]
        assert vals == case["expect_values"]


def test_projection_partitions_match_oracle():
    import numpy as np
    lay = "(8,3):(1,8)"
    x = ma.MoYeArray(0, 7, ml.Layout(lay))
    o = to.Array(np.arange(24), lo.parse_layout(lay))
    thr = ml.static_layout((4, 2))
    for tid in range(1, 9):
        for proj_m, proj_o in (((ml.StaticInt(1), ml.COLON), (lo.S(1), lo.COLON)),
                               ((ml.COLON, ml.StaticInt(1)), (lo.COLON, lo.S(1)))):
            r = ma.local_partition(x, thr, tid, proj_m)
            w = to.local_partition(o, lo.SL((4, 2)), tid, proj_o)
            assert r.layout.text == repr(w.layout) and r.ptr // 4 == w.offset


@pytest.mark.parametrize("case", V["tiled_mma"], ids=lambda c: c["ref"])
def test_tiled_mma(case):
    perm = None
    if "permutation" in case:
        perm = tuple(X(p) for p in split_top(canon(case["permutation"])[1:-1]))
    tm = ma.make_tiled_mma(case["atom"], L(case["atom_layout"]), perm)
    assert [int(v) for v in tm.tile_shape()] == case["tile_size"]
    if "thr_layout_vmnk" in case:
        assert tm.thr_layout_vmnk().identical(L(case["thr_layout_vmnk"]))
    if "C" in case:
        thr = tm.get_slice(case["thr"])
        for name, part in (("C", thr.partition_C), ("A", thr.partition_A), ("B", thr.partition_B)):
            p = part(ma.MoYeArray(0, 0, L(case[name])))
            assert [ml.size(p.layout, 2), ml.size(p.layout, 3)] == case[name + "_rest"]


@pytest.mark.parametrize("name", sorted(to.REFERENCE_MMA_OPS) + sorted(to.MFMA_OPS))
def test_mma_partitions_match_oracle(name):
    """partition_A/B/C of every thread: identical layouts and offsets to the oracle, and the
    TV layouts used by make_tiled_copy_A/B/C map to the same tile indices."""
    import numpy as np
    op = to.REFERENCE_MMA_OPS.get(name) or to.MFMA_OPS[name]
    otm = to.make_tiled_mma(op, lo.SL((2, 1, 1)))
    tm = ma.make_tiled_mma(name, ml.static_layout((2, 1, 1)))
    assert tm.thr_layout_vmnk().text == repr(otm.thr_layout_vmnk())
    m, n, k = (int(v) for v in otm.tile_shape())
    assert [int(v) for v in tm.tile_shape()] == [m, n, k]
    tids = lo.all_indices(otm.thr_layout_vmnk())
    for shp, opnd in (((m, n), "C"), ((m, k), "A"), ((n, k), "B")):
        lay = "(_%d,_%d):(_%d,_1)" % (shp[0], shp[1], shp[1])
        oarr = to.Array(np.arange(shp[0] * shp[1]), lo.parse_layout(lay))
        arr = ma.MoYeArray(0, 5, ml.Layout(lay))  # U8: ptr == element offset
        for t in tids[::7]:
            got = getattr(tm.get_slice(t), "partition_" + opnd)(arr)
            want = getattr(otm.get_slice(t), "partition_" + opnd)(oarr)
            assert got.layout.text == repr(want.layout) and got.ptr == want.offset
    for opnd, f in (("A", otm.get_layoutA_TV), ("B", otm.get_layoutB_TV), ("C", otm.get_layoutC_TV)):
        got, want = tm.layout_tv(opnd), f()
        assert _values(got) == lo.all_indices(want)


def test_mfma_descriptor_for_config3():
    tm = ma.make_tiled_mma(1, ml.static_layout((2, 2, 1)), (ml.StaticInt(128), ml.StaticInt(128), ml.StaticInt(32)))
    d = tm.descriptor()
    assert list(d.atom_layout_mnk) == [2, 2, 1] and list(d.tile_mnk) == [128, 128, 32]
    assert list(d.cta_tile_mnk) == [128, 128, 32] and tm.size() == 256
    with pytest.raises(MoyeError) as e:  # the reference's NVIDIA atoms exist as data only
        ma.make_tiled_mma("MMAOP_16x8x8_F16F16F16F16_TN").descriptor()
    assert e.value.status == ERR_UNSUPPORTED


def test_tiled_copy_owner_table_and_partitions():
    import numpy as np
    f = V["tiled_copy_owner_table"]
    tc = ma.make_tiled_copy(ma.CopyAtom(64, 64), L(f["thr_layout"]), L(f["val_layout"]))
    assert [int(v) for v in tc.tiler_MN] == f["tiler"]
    assert tc.tiled_layout_TV == L("@((3,2),(2,3)):((12,2),(1,4))")
    rows, cols = f["tiler"]
    own = [[0] * cols for _ in range(rows)]
    for tid in range(1, 7):
        for v in range(1, 7):
            idx = tc.tiled_layout_TV((tid, v)) - 1
            own[idx % rows][idx // rows] = tid
    assert own == f["owners"]
    assert ma.CopyAtom(128, 32) and ma.make_tiled_copy(ma.CopyAtom(128, 32), L("@(32,8)"), L("@(4,1)")).num_val_src == 4
    with pytest.raises(MoyeError) as e:  # 3 values per thread cannot be moved by a 4-value access
        ma.make_tiled_copy(ma.CopyAtom(128, 32), L("@(32,8)"), L("@(3,1)")).tiled_layout_TV
    assert e.value.status == ERR_SHAPE
    # partition_S/D against the oracle (test/copy.jl:123-145 layouts)
    for smem, thr, val, n in (("@(32,32):(1,32)", "@(16,2)", "@(2,4)", 1024),
                              ("@(32,(2,4)):(2,(1,64))", "@(32,1)", "@(1,8)", 256)):
        otc = to.make_tiled_copy(to.CopyAtom(to.UniversalCopy(16), 16), OL(thr), OL(val))
        mtc = ma.make_tiled_copy(ma.CopyAtom(16, 16), L(thr), L(val))
        assert mtc.tiled_layout_TV.text == repr(otc.tiled_layout_TV)
        oarr = to.Array(np.arange(n, dtype=np.uint16), OL(smem))
        arr = ma.MoYeArray(0, 5, L(smem))
        for tid in range(1, int(otc.size()) + 1):
            for which in ("S", "D"):
                got = getattr(mtc.get_slice(tid), "partition_" + which)(arr)
                want = getattr(otc.get_slice(tid), "partition_" + which)(oarr)
                assert got.layout.text == repr(want.layout) and got.ptr == want.offset


def test_config_descriptors():
    """The tile views the GPU kernels are launched with (fp16 4096^3, 128x128x32 CTA tile)."""
    a = ma.MoYeArray(4096, 1, ml.Layout("(_4096,_4096):(_4096,_1)"))
    g = ma.local_tile(a, (ml.StaticInt(128), ml.StaticInt(32)), (3, ml.COLON))
    assert g.layout == L("@(128,32,128):(4096,1,32)") and g.ptr == 4096 + 2 * 524288 * 2
    t = a.tensor()
    assert (t.rank, list(t.shape)[:2], list(t.stride)[:2]) == (2, [4096, 4096], [4096, 1])
    assert ml.max_common_vector(ml.Layout("(_64,_64):(_1,_64)"), ml.Layout("(_64,_64):(_1,_64)")) == 4096
    assert ml.max_common_vector(ml.Layout("(_64,_64):(_1,_64)"), ml.Layout("(_64,_64):(_64,_1)")) == 1


def test_errors_map_to_status_codes():
    with pytest.raises(MoyeError) as e:
        ml.Layout("(2,3):(1,")
    assert e.value.status == ERR_PARSE
    with pytest.raises(MoyeError) as e:
        ml.Layout("(2,3):(1,2,3)")
    assert e.value.status == ERR_PARSE
    with pytest.raises(MoyeError) as e:  # too many modes in tile -> DimensionMismatch (layout.jl:1062)
        ml.logical_divide(L("@(4,4)"), "<_2,_2,_2>")
    assert e.value.status == ERR_RANK
    with pytest.raises(MoyeError) as e:  # static shape_div assert (int_tuple.jl:87-90)
        ml.shape_div(ml.StaticInt(6), ml.StaticInt(4))
    assert e.value.status == ERR_SHAPE
    assert ml.shape_div(6, 4) == 1
    with pytest.raises(MoyeError) as e:  # complement needs static strides (layout.jl:640)
        ml.complement(ml.Layout("(4,2):(1,8)"))
    assert e.value.status == ERR_UNSUPPORTED
    with pytest.raises(MoyeError) as e:
        ml.index_to_coord(9, (3, 4), (1, 3, 5))
    assert e.value.status == ERR_RANK


# ---------------------------------------------------------------------------------------------
# IntTuple helpers, tile_to_shape, make_layout_like and the TV-based TiledCopy: host vs oracle
# ---------------------------------------------------------------------------------------------
import numpy as np
import moye_hip as mh
import tiled_oracle as to


def _o2t(x):
    """oracle IntTuple -> text the host parses."""
    return lo._fmt(x) if hasattr(lo, "_fmt") else str(x)


def _same(host_value, oracle_value):
    assert ml.tuple_text(host_value).replace(" ", "") == _o2t(oracle_value).replace(" ", ""), (host_value, oracle_value)


def test_more_tuple_helpers_against_the_oracle():
    S = lo.S
    t = (S(2), (3, S(4)), ((5, 6), S(7)))
    h = ml.parse_tuple(_o2t(t))
    _same(ml.unflatten(ml.parse_tuple("(1,2,3,4,5,6)"), ml.parse_tuple("(0,(0,0),((0,0),0))")),
          lo.unflatten((1, 2, 3, 4, 5, 6), (0, (0, 0), ((0, 0), 0))))
    _same(ml.group(h, 2, 3), lo.group(t, 2, 3))
    _same(ml.group(h, 1, 1), lo.group(t, 1, 1))
    _same(ml.tuple_append(h, ml.StaticInt(1)), lo.append(t, S(1)))
    _same(ml.tuple_append(h, ml.StaticInt(1), 5), lo.append(t, S(1), 5))
    _same(ml.tuple_prepend(h, 9, 4), lo.prepend(t, 9, 4))
    with pytest.raises(mh.MoyeError):
        ml.tuple_append(h, 1, 2)
    z = (((1, 2), (3, 4)), ((5, 6), (7, 8)), (9, 10))
    _same(ml.zip2_by(ml.parse_tuple(_o2t(z)), ml.parse_tuple("((0,0),0)")), lo.zip2_by(z, ((0, 0), 0)))
    _same(ml.product_each(h), lo.product_each(t))
    _same(ml.elem_scale(ml.parse_tuple("(2,(3,_4))"), ml.parse_tuple("(5,((6,7),_2))")),
          lo.elem_scale((2, (3, S(4))), (5, ((6, 7), S(2)))))
    _same(ml.filter_zeros(ml.parse_tuple("(_0,(3,_0))"), ml.parse_tuple("(7,(8,9))")),
          lo.filter_zeros((S(0), (3, S(0))), (7, (8, 9))))
    _same(ml.coord_to_coord(ml.parse_tuple("(3,(2,2))"), ml.parse_tuple("(4,(2,3))"), ml.parse_tuple("(2,(6,1))")),
          lo.coord_to_coord((3, (2, 2)), (4, (2, 3)), (2, (6, 1))))
    # orderings and increment: all coordinates of a small hierarchical shape
    shape = (2, (3, 2))
    coords = [lo.index_to_coord(i, shape) for i in range(1, 13)]
    c = coords[0]
    for nxt in coords[1:] + coords[:1]:
        _same(ml.increment(ml.parse_tuple(_o2t(c)), ml.parse_tuple(_o2t(shape))), lo.increment(c, shape))
        assert lo.increment(c, shape) == nxt      # the oracle itself walks the coordinates in order
        c = nxt
    for a in coords[::3]:
        for b in coords[::2]:
            ta, tb = ml.parse_tuple(_o2t(a)), ml.parse_tuple(_o2t(b))
            assert ml.colex_less(ta, tb) == lo.colex_less(a, b)
            assert ml.elem_less(ta, tb) == lo.elem_less(a, b)
    # reference known answers (test/int_tuple.jl:46-96 style)
    assert ml.colex_less(ml.parse_tuple("(1,2,3)"), ml.parse_tuple("(1,2,4)")) is True
    assert ml.elem_less(ml.parse_tuple("(1,2,3)"), ml.parse_tuple("(2,3,4)")) is True
    assert ml.elem_less(ml.parse_tuple("(3,2,3)"), ml.parse_tuple("(2,3,4)")) is False


def test_tile_to_shape_and_make_layout_like_against_the_oracle():
    for text, trg, order in (("(_2,_2):(_1,_2)", "(_8,_6)", None), ("(_4,_2):(_2,_1)", "(_8,_8)", "(_1,_0)"),
                             ("_4:_1", "(_8,_4,_2)", None), ("(_2,_3):(_3,_1)", "(_4,_9)", "(_0,_1)")):
        l = lo.parse_layout(text)
        want = lo.tile_to_shape(l, lo.parse_int_tuple(trg)) if order is None else \
            lo.tile_to_shape(l, lo.parse_int_tuple(trg), lo.parse_int_tuple(order))
        got = ml.tile_to_shape(ml.Layout(text), ml.parse_tuple(trg), None if order is None else ml.parse_tuple(order))
        assert canon(got.text) == canon(str(want)), (text, trg, order)
        # what the function is for: the result covers the target shape with copies of the block
        assert int(lo.size(want)) == int(lo.product(lo.parse_int_tuple(trg)))
    for text in ("(_2,(_3,_4)):(_12,(_1,_3))", "(4,_1,6):(6,_0,1)", "(_8,_8):(_8,_1)"):
        assert canon(ml.make_layout_like(ml.Layout(text)).text) == canon(str(lo.make_layout_like(lo.parse_layout(text))))


def test_make_tiled_copy_ABC_and_retile_against_the_oracle():
    """make_tiled_copy_A/B/C (src/atom/copy.jl:227-240), partition_S/D and retile through the TV form."""
    S = lo.S
    for name, al in (("MMAOP_16x8x8_F32TF32TF32F32_TN", None), ("MMAOP_16x8x8_F16F16F16F16_TN", lo.SL((2, 2, 1))),
                     ("MFMA_F32_16x16x32_F16", lo.SL((2, 2, 1)))):
        op = to.REFERENCE_MMA_OPS.get(name) or to.MFMA_OPS[name]
        omma = to.make_tiled_mma(op, al)
        hmma = mh.TiledMMAOp(name, None if al is None else ml.Layout(str(al)))
        vb = 32 if "TF32" in name else 16
        oatom, hatom = to.CopyAtom(to.UniversalCopy(vb), vb), mh.CopyAtom(vb, vb)
        for which, omake, hmake, tile in (("A", to.make_tiled_copy_A, mh.make_tiled_copy_A, (1, 3)),
                                          ("B", to.make_tiled_copy_B, mh.make_tiled_copy_B, (2, 3)),
                                          ("C", to.make_tiled_copy_C, mh.make_tiled_copy_C, (1, 2))):
            otc, htc = omake(oatom, omma), hmake(hatom, hmma)
            assert canon(htc.tiled_layout_TV.text) == canon(str(otc.tiled_layout_TV))
            assert canon(htc.get_layoutS_TV().text) == canon(str(otc.get_layoutS_TV()))
            assert canon(htc.get_layoutD_TV().text) == canon(str(otc.get_layoutD_TV()))
            rows, cols = int(omma.tile_size(tile[0])), int(omma.tile_size(tile[1]))
            buf = np.arange(rows * cols * 4, dtype=np.float32)
            oarr = to.Array(buf, lo.make_layout((S(2 * rows), S(2 * cols))))
            harr = mh.MoYeArray(0, mh.F32, ml.Layout("(_%d,_%d)" % (2 * rows, 2 * cols)))
            seen = np.zeros(rows * cols * 4, dtype=np.int32)
            for thr in range(1, int(otc.size()) + 1):
                op_, hp_ = otc.get_slice(thr).partition_S(oarr), htc.get_slice(thr).partition_S(harr)
                assert canon(hp_.layout.text) == canon(str(op_.layout)) and hp_.ptr == op_.offset * 4, (name, which, thr)
                seen[op_.offsets()] += 1
            # A is shared by the atoms along N, B by the atoms along M (src/atom/mma.jl:120-169): every element
            # is owned that many times, C exactly once
            mult = 1 if al is None else {"A": int(al.shape[1]), "B": int(al.shape[0]), "C": 1}[which]
            assert (seen == mult).all(), (name, which, mult)
            # retile of a fragment-shaped layout (atom/copy.jl:151-166)
            frag = otc.get_slice(1).partition_D(oarr).layout
            frag_like = lo.make_fragment_like(frag)
            assert canon(htc.retile(ml.Layout(str(frag_like))).text) == canon(str(otc.retile(frag_like))), (name, which)


def test_host_print_layout_matches_the_reference_docstrings():
    import json
    import os
    tables = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "print_layout_tables.json")))
    for t in tables:
        text = ml.print_layout(ml.Layout(t["layout"]), file=False)
        assert [line.rstrip() for line in text.split("\n")] == t["lines"], t["expression"]
        assert text == lo.print_layout(lo.parse_layout(t["layout"]))
    with pytest.raises(MoyeError):
        ml.print_layout(ml.Layout("(_2,_2,_2)"), file=False)


# ---- Int32: the coordinate's integer type survives (test/layout.jl:4-12, src/utilities.jl:1-11) -----------------------

def test_int32_known_answers_through_the_abi():
    a = ml.Layout("(_2,(_2,_2)):(_2,(_1,_4))")
    r = a(ml.Int32(2))
    assert type(r) is ml.Int32 and r == 3
    assert type(a(2)) is int and type(a(ml.StaticInt(2))) is ml.StaticInt
    b = ml.make_layout((ml.Int32(2), ml.Int32(4)))
    assert b.text == "(2i32, 4i32):(_1, 2i32)"
    r = b(ml.Int32(2))
    assert type(r) is ml.Int32 and r == 2
    assert type(b(2)) is int
    assert repr(ml.index_to_coord(ml.Int32(7), a.shape, a.stride)) == "(2i32, (1i32, 2i32))"
    assert repr(ml.coord_to_index((ml.Int32(2), (ml.Int32(1), ml.Int32(2))), a.shape, a.stride)) == "7i32"
    w = ml.Layout("4i32:1073741824i32")
    assert repr(w(ml.Int32(4))) == "-1073741823i32" and w(4) == 3 * 2 ** 30 + 1     # wraps as Julia's Int32 does
    assert repr(ml.compact_col_major((ml.Int32(3), ml.Int32(5), ml.StaticInt(2)))) == "(_1, 3i32, 15i32)"
    with pytest.raises(MoyeError) as e:
        ml.Layout("_4i32:_1")                  # a static integer has no width
    assert e.value.status == ERR_PARSE
    with pytest.raises(MoyeError) as e:
        ml.Layout("4294967296i32:_1")
    assert e.value.status == ERR_PARSE


def test_int32_random_differential():
    """The C++ algebra against the oracle on random layouts whose dynamic integers are a mix of Int32 and Int: the
    printed results agree, widths included."""
    rng = random.Random(77)

    def widen(text):      # every dynamic integer becomes an Int32 with probability 0.7
        import re
        return re.sub(r"(?<![_\d])(\d+)(?![\d])", lambda m: m.group(1) + ("i32" if rng.random() < 0.7 else ""), text)

    n = 0
    for _ in range(300):
        ta, tb = widen(_rand_layout(rng, 0.5)), widen(_rand_layout(rng, 0.5))
        a, b, oa, ob = ml.Layout(ta), ml.Layout(tb), lo.parse_layout(ta), lo.parse_layout(tb)
        assert a.text == repr(oa)
        _both(lambda: ml.coalesce(a), lambda: lo.coalesce(oa))
        _both(lambda: ml.filter(a), lambda: lo.lfilter(oa))
        _both(lambda: ml.composition(a, b), lambda: lo.composition(oa, ob))
        _both(lambda: ml.logical_divide(a, b), lambda: lo.logical_divide(oa, ob))
        _both(lambda: ml.logical_product(a, b), lambda: lo.logical_product(oa, ob))
        _both(lambda: ml.recast(a, 2, 4), lambda: lo.recast_layout(oa, 2, 4))
        _both(lambda: ml.recast(a, 4, 2), lambda: lo.recast_layout(oa, 4, 2))
        for i in range(1, min(ml.size(a), 8) + 1):
            for c, oc in ((ml.Int32(i), lo.I32(i)), (i, i), (ml.StaticInt(i), lo.S(i))):
                assert repr(a(c)) == repr(oa(oc)), (ta, i)
            if "0" not in [t.strip("_i32") for t in ta.split(":")[1].replace("(", "").replace(")", "").split(",")]:  # no stride of 0
                assert repr(ml.index_to_coord(ml.Int32(i), a.shape, a.stride)) == repr(lo.index_to_coord(lo.I32(i), oa.shape, oa.stride))
        n += 1
    assert n == 300

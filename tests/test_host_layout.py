"""The shipped host-side layout algebra (C++ inside libmoye_hip.so, reached through the C ABI and
the moye_hip Python mirror) against (1) the reference's own known answers and invariant helpers
(tests/golden/layout_vectors.json) and (2) the independent Python oracle on seeded random cases.
No GPU needed."""
import random

import pytest

import layout_oracle as lo
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

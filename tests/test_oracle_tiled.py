"""Pins oracle/tiled_oracle.py (arrays, @tile/@parallelize, TiledMMA, TiledCopy, copyto!, gemm!)
against the reference's test vectors: test/tiling.jl, test/tiled_mma.jl, test/copy.jl,
test/host/tiling_matmul.jl, the docstrings of src/algorithm/array_algorithms.jl and
src/atom/mma.jl, and the owner table of docs/src/manual/tiled_matmul.md."""
import numpy as np
import pytest

import layout_oracle as lo
import tiled_oracle as to
from helpers import canon, load_vectors, split_top
from layout_oracle import COLON, S, SL, static

V = load_vectors()


def L(text):
    return lo.parse_layout(canon(text))


def X(text):
    text = canon(text)
    if text.startswith("<"):
        return tuple(X(p) for p in split_top(text[1:-1]))
    if text == ":":
        return COLON
    if ":" in text or text.startswith("("):
        return lo.parse_layout(text)
    return lo.parse_int_tuple(text)


@pytest.mark.parametrize("case", V["tiling"], ids=lambda c: c["ref"])
def test_tile_and_parallelize(case):
    lay = L(case["array"])
    a = to.Array(np.arange(1, int(lo.size(lay)) + 1), lay)
    tile = X(case["tile"])
    if case["op"] == "local_tile":
        r = to.local_tile(a, tile, lo.parse_int_tuple(case["coord"]))
    elif "index" in case:
        r = to.local_partition(a, tile, case["index"])
    else:
        r = to.local_partition(a, tile, lo.parse_int_tuple(case["coord"]))
    if "expect_layout" in case:
        assert r.layout == L(case["expect_layout"])
    if "expect_rank" in case:
        assert lo.lrank(r.layout) == case["expect_rank"]
    if "expect_values" in case:
        assert list(r.values()) == case["expect_values"]


def test_partitions_tile_the_array():
    """Brute force: over all thread indices the raked partitions are disjoint and cover the array."""
    a = to.Array(np.arange(48), SL((6, 8)))
    thr = SL((2, 2), (2, 1))
    seen = np.concatenate([to.local_partition(a, thr, i).values() for i in range(1, 5)])
    assert sorted(seen) == list(range(48))
    tiles = [to.local_tile(a, static((3, 2)), (i, j)).values() for i in (1, 2) for j in (1, 2, 3, 4)]
    assert sorted(np.concatenate(tiles)) == list(range(48))


def test_projection_partitions():
    """test/host/tiling_matmul.jl:25-39 and test/device/matmul.jl:32-33 — `(1,:)` keeps rows of the
    first thread-mode, `(:,1)` of the second."""
    M, K = 8, 3
    a = to.Array(np.arange(M * K), lo.make_layout((M, K)))
    thr = SL((4, 2))
    for tid in range(1, 9):
        tm, tn = (tid - 1) % 4, (tid - 1) // 4
        pa = to.local_partition(a, thr, tid, (S(1), COLON))
        assert pa.layout.shape == (2, 3)
        assert [int(pa[(1, k)]) for k in (1, 2, 3)] == [tm + M * (k - 1) for k in (1, 2, 3)]
        pb = to.local_partition(a, thr, tid, (COLON, S(1)))
        assert pb.layout.shape == (4, 3)
        assert int(pb[(1, 1)]) == tn and int(pb[(2, 1)]) == tn + 2


@pytest.mark.parametrize("case", V["tiled_mma"], ids=lambda c: c["ref"])
def test_tiled_mma(case):
    perm = X(case["permutation"]) if "permutation" in case else None
    tm = to.make_tiled_mma(to.REFERENCE_MMA_OPS[case["atom"]], L(case["atom_layout"]), perm)
    assert [int(v) for v in tm.tile_shape()] == case["tile_size"]
    if "thr_layout_vmnk" in case:
        assert tm.thr_layout_vmnk().identical(L(case["thr_layout_vmnk"]))
    if "C" in case:
        thr = tm.get_slice(case["thr"])
        for name, part, frag in (("C", thr.partition_C, thr.partition_fragment_C),
                                 ("A", thr.partition_A, thr.partition_fragment_A),
                                 ("B", thr.partition_B, thr.partition_fragment_B)):
            lay = L(case[name])
            arr = to.Array(np.arange(1, int(lo.size(lay)) + 1, dtype=np.float32), lay)
            p = part(arr)
            assert [int(lo.size(p.layout, 2)), int(lo.size(p.layout, 3))] == case[name + "_rest"]
            f = frag(arr)
            assert [int(lo.size(f.layout, i)) for i in (1, 2, 3)] == \
                [int(lo.size(p.layout, i)) for i in (1, 2, 3)]


@pytest.mark.parametrize("name", sorted(to.REFERENCE_MMA_OPS) + sorted(to.MFMA_OPS))
def test_mma_partitions_cover_operands(name):
    """Over all threads the A/B/C partitions cover the atom tile, each element held by the number of
    threads the TV layout implies (exactly once for C)."""
    op = to.REFERENCE_MMA_OPS.get(name) or to.MFMA_OPS[name]
    tm = to.make_tiled_mma(op)
    m, n, k = (int(v) for v in tm.tile_shape())
    # hardware thread ids are the image of the thread layout (sm70 quad-pairs are not contiguous)
    tids = lo.all_indices(tm.thr_layout_vmnk())
    for shp, part in (((m, n), "partition_C"), ((m, k), "partition_A"), ((n, k), "partition_B")):
        lay = lo.make_layout(static(shp))
        arr = to.Array(np.arange(shp[0] * shp[1]), lay)
        got = np.concatenate([getattr(tm.get_slice(t), part)(arr).values() for t in tids])
        counts = np.bincount(got, minlength=shp[0] * shp[1])
        assert counts.min() == counts.max() >= 1
        if part == "partition_C":
            assert counts.max() == 1


def test_mfma_tv_layout_closed_form():
    """The gfx950 tables against the lane/register map they encode."""
    op = to.MFMA_OPS["MFMA_F32_16x16x32_F16"]
    for lane in range(64):
        for j in range(8):
            assert op.layout_a((lane + 1, j + 1)) - 1 == (lane % 16) + 16 * (8 * (lane // 16) + j)
        for r in range(4):
            assert op.layout_c((lane + 1, r + 1)) - 1 == (4 * (lane // 16) + r) + 16 * (lane % 16)
    op = to.MFMA_OPS["MFMA_F32_32x32x16_F16"]
    for lane in range(64):
        for j in range(8):
            assert op.layout_a((lane + 1, j + 1)) - 1 == (lane % 32) + 32 * (8 * (lane // 32) + j)
        for r in range(16):
            row = 8 * (r // 4) + 4 * (lane // 32) + r % 4
            assert op.layout_c((lane + 1, r + 1)) - 1 == row + 32 * (lane % 32)


def test_config3_descriptor():
    """fp16 4096^3: MFMA 16x16x32 atoms, 2x2 waves, permutation (128,128,32)."""
    tm = to.make_tiled_mma(to.MFMA_OPS["MFMA_F32_16x16x32_F16"], SL((2, 2, 1)), (S(128), S(128), S(32)))
    assert [int(v) for v in tm.tile_shape()] == [128, 128, 32]
    assert int(tm.size()) == 256
    thr = tm.get_slice(1)
    c = to.Array(np.zeros(128 * 128, np.float32), SL((128, 128)))
    a = to.Array(np.zeros(128 * 32, np.float16), SL((128, 32)))
    pc, pa = thr.partition_C(c), thr.partition_A(a)
    assert [int(lo.size(pc.layout, i)) for i in (1, 2, 3)] == [4, 4, 4]
    assert [int(lo.size(pa.layout, i)) for i in (1, 2, 3)] == [8, 4, 1]


def test_tiled_copy_owner_table():
    """docs/src/manual/tiled_matmul.md:9-14."""
    f = V["tiled_copy_owner_table"]
    tc = to.make_tiled_copy(to.CopyAtom(to.UniversalCopy(64), 64), L(f["thr_layout"]), L(f["val_layout"]))
    assert [int(v) for v in tc.tiler_MN] == f["tiler"]
    assert tc.tiled_layout_TV == L("@((3,2),(2,3)):((12,2),(1,4))")
    rows, cols = f["tiler"]
    own = np.zeros((rows, cols), int)
    for tid in range(1, 7):
        for v in range(1, 7):
            idx = int(tc.tiled_layout_TV((tid, v))) - 1
            assert own[idx % rows, idx // rows] == 0
            own[idx % rows, idx // rows] = tid
    assert own.tolist() == f["owners"]
    # vectorised atom: UniversalCopy{UInt128} over Float64 moves 2 values per instruction
    assert int(to.CopyAtom(to.UniversalCopy(128), 64).num_val_src) == 2
    assert int(to.CopyAtom(to.UniversalCopy(128), 32).num_val_src) == 4


def _tiled_copy_kernel(smem_layout, tc, n):
    """test/copy.jl:102-121 — the CPU twin of the device tiled-copy kernel."""
    g_in = np.arange(1, n + 1, dtype=np.uint16)
    g_out = np.zeros(n, np.uint16)
    smem = to.Array(g_in.copy(), smem_layout, memspace="smem")
    gout = to.Array(g_out, smem_layout)
    for tid in range(1, int(tc.size()) + 1):
        thr = tc.get_slice(tid)
        s, d = thr.partition_S(smem), thr.partition_D(gout)
        r = to.Array.undef(np.uint16, lo.make_layout(d.layout.shape))
        to.copyto(r, s, tc)
        to.copyto(d, r)
    return g_in, g_out


def test_tiled_copy_roundtrips():
    """test/copy.jl:123-145."""
    atom = to.CopyAtom(to.UniversalCopy(16), 16)
    g_in, g_out = _tiled_copy_kernel(SL((32, 32), (1, 32)), to.make_tiled_copy(atom, SL((16, 2)), SL((2, 4))), 1024)
    assert (g_in == g_out).all()
    g_in, g_out = _tiled_copy_kernel(SL((32, (2, 4)), (2, (1, 64))),
                                     to.make_tiled_copy(atom, SL((32, 1)), SL((1, 8))), 256)
    assert (g_in == g_out).all()
    for name in to.LDSM:  # test/copy.jl:154-159: construction only
        to.make_tiled_copy(to.CopyAtom(to.LDSM[name], 16), SL((16, 2)), SL((2, 4)))


def _ldmatrix(nmat, trans, ptrs, mem):
    """What PTX `ldmatrix.sync.aligned.m8n8.x{nmat}[.trans].b16` does for one warp, written from the
    instruction's definition and not from the reference's layouts: thread 8i+r supplies the
    address of row r of matrix i (8 contiguous b16 values); thread t receives from every matrix
    the two values at (row t//4, columns 2(t%4), 2(t%4)+1), or of the transposed matrix."""
    out = np.zeros((32, 2 * nmat), mem.dtype)
    for t in range(32):
        for i in range(nmat):
            for v in range(2):
                r, c = (2 * (t % 4) + v, t // 4) if trans else (t // 4, 2 * (t % 4) + v)
                out[t, 2 * i + v] = mem[ptrs[8 * i + r] + c]
    return out


def _ldmatrix_copy_kernel(smem_layout, tc, n, nmat, trans):
    """test/device/tiled_copy.jl:2-22 for one warp, with the shared->register step done by the
    instruction model above: every thread passes the address of each 8-value source slice of its
    partition_S and stores what it receives through its partition_D."""
    g_in = np.arange(1, n + 1, dtype=np.uint16)
    g_out = np.zeros(n, np.uint16)
    smem = to.Array(g_in.copy(), smem_layout, memspace="smem")
    gout = to.Array(g_out, smem_layout)
    src, dst = [], []
    for tid in range(1, 33):
        thr = tc.get_slice(tid)
        src.append(thr.partition_S(smem).offsets())
        dst.append(thr.partition_D(gout).offsets())
    natoms = len(src[0]) // 8
    assert len(dst[0]) == natoms * 2 * nmat
    for k in range(natoms):
        for t in range(32):  # a row handed to the instruction is 16 contiguous bytes
            assert (np.diff(src[t][8 * k:8 * k + 8]) == 1).all()
        regs = _ldmatrix(nmat, trans, [int(src[t][8 * k]) for t in range(32)], smem.buf)
        for t in range(32):
            g_out[dst[t][2 * nmat * k:2 * nmat * (k + 1)]] = regs[t]
    return g_in, g_out


@pytest.mark.parametrize("name,nmat", [("LDSM_U32x1_N", 1), ("LDSM_U32x2_N", 2), ("LDSM_U32x4_N", 4)])
def test_ldmatrix_tiled_copy_roundtrips(name, nmat):
    """test/device/tiled_copy.jl:56-90: `cu_g_out == cu_g_in` for the three ldmatrix atoms on both
    shared layouts of that file."""
    atom = to.CopyAtom(to.LDSM[name], 16)
    g_in, g_out = _ldmatrix_copy_kernel(SL((32, 32), (1, 32)), to.make_tiled_copy(atom, SL((16, 2)), SL((2, 4))),
                                        1024, nmat, False)
    assert (g_in == g_out).all()
    g_in, g_out = _ldmatrix_copy_kernel(SL((32, (2, 4)), (2, (1, 64))),
                                        to.make_tiled_copy(atom, SL((32, 1)), SL((1, 8))), 256, nmat, False)
    assert (g_in == g_out).all()


@pytest.mark.parametrize("name,nmat", [("LDSM_U16x2_T", 1), ("LDSM_U16x4_T", 2), ("LDSM_U16x8_T", 4)])
def test_ldmatrix_trans_tiled_copy_roundtrips(name, nmat):
    """traits/ldmatrix.jl:22-41 has no test in the reference; the same round trip pins the tables.
    The transposing atoms want the shared tile contiguous along the mode the registers do not
    run along, so the tiles here are row-major and the values run down the rows."""
    tc = to.make_tiled_copy(to.CopyAtom(to.LDSM[name], 16), SL((4, 8)), SL((8, 1)))
    for layout, n in ((SL((32, 8), (8, 1)), 256), (SL((32, 32), (32, 1)), 1024)):
        g_in, g_out = _ldmatrix_copy_kernel(layout, tc, n, nmat, True)
        assert (g_in == g_out).all()


def test_plain_copyto():
    """test/copy.jl:5-99."""
    x = to.Array(np.arange(1, 9, dtype=np.int32), lo.make_layout((4, 2)))
    y = to.Array(np.arange(9, 17, dtype=np.int32), lo.make_layout((4, 2)))
    to.copyto(y, x)
    assert (y.buf == x.buf).all()
    a = to.Array(np.arange(1, 37, dtype=np.int32), SL((6, 6)))
    b = to.Array(np.arange(37, 73, dtype=np.int32), SL((6, 6)))
    thr = SL((2, 3))
    for i in range(1, 7):
        to.copyto(to.local_partition(b, thr, i), to.local_partition(a, thr, i))
    assert (a.buf == b.buf).all()
    # transposed destination: dst[j,i] == src[i,j] (test/host/copy_async.jl:95)
    src = to.Array(np.arange(12, dtype=np.float32), lo.make_layout((3, 4)))
    dst = to.Array(np.zeros(12, np.float32), lo.make_layout((3, 4), (4, 1)))
    to.copyto(dst, src)
    assert (dst.buf.reshape(3, 4) == src.buf.reshape(4, 3).T).all()
    # conversion rule of UniversalCopy{TS,TD}: round to nearest even
    s = to.Array(np.array([1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11, 65520.0], np.float32), SL(3))
    d = to.Array(np.zeros(3, np.float16), SL(3))
    to.copyto(d, s)
    assert d.buf[0] == np.float16(1.0) and d.buf[1] == np.float16(1.0 + 2.0 ** -9) and np.isinf(d.buf[2])


def test_recast_arrays():
    """test/array.jl:84-106,127-143."""
    data = np.arange(1, 13, dtype=np.int64)
    a = to.Array(data, SL((4, 3)))
    b = to.recast(np.int32, a)
    assert b.layout == SL((8, 3)) and int(b[(1, 1)]) == 1 and int(b[(3, 1)]) == 2
    x = to.Array(np.arange(12, dtype=np.float32), SL((4, 3)))
    x2 = to.recast(np.float64, x)
    assert x2.layout == SL((2, 3))
    assert (to.recast(np.float32, x2).values() == x.values()).all()


def test_gemm_universal_fma_matches_reference_host_test():
    """test/host/tiling_matmul.jl:4-41 — partitioned triple loop equals A*B'."""
    rng = np.random.default_rng(7)
    M, N, K = 16, 12, 8
    A = rng.random((M, K)).astype(np.float32)
    B = rng.random((N, K)).astype(np.float32)
    Cbuf = np.zeros(M * N, np.float32)
    mA, mB = to.Array.from_matrix(A), to.Array.from_matrix(B)
    mC = to.Array(Cbuf, lo.make_layout((M, N)))
    thr = SL((4, 4))
    for tid in range(1, 17):
        tA = to.local_partition(mA, thr, tid, (S(1), COLON))
        tB = to.local_partition(mB, thr, tid, (COLON, S(1)))
        tC = to.local_partition(mC, thr, tid)
        to.gemm_arrays(tC, tA, tB, tC)
    C = Cbuf.reshape(N, M).T
    np.testing.assert_allclose(C, A @ B.T, rtol=1e-5)
    # the vectorised restatement is bit-identical to the element loop
    assert (to.gemm_universal_fma(A, B, np.zeros((M, N), np.float32)) == C).all()


def test_gemm_rounding_rule():
    """src/arch/mma/mma.jl:64 — the product is rounded in the input type before the fp32 add, never
    fused.  Inputs chosen so that a fused or an fp32-product evaluation gives a different answer."""
    a = np.array([[1.0 + 2.0 ** -10]], np.float16).astype(np.float32)   # 1 + ulp
    b = np.array([[1.0 + 2.0 ** -10]], np.float16).astype(np.float32)
    c = np.zeros((1, 1), np.float32)
    # exact product = 1 + 2^-9 + 2^-20; fp16 keeps 1 + 2^-9
    assert to.gemm_universal_fma(a, b, c, "f16", "f16")[0, 0] == np.float32(1.0 + 2.0 ** -9)
    assert to.gemm_universal_fma(a, b, c, "f32", "f32")[0, 0] == np.float32(1.0 + 2.0 ** -9 + 2.0 ** -20)
    ab = np.array([[1.0 + 2.0 ** -7]], np.float32)
    assert to.gemm_universal_fma(ab, ab, c, "bf16", "bf16")[0, 0] == np.float32(1.0 + 2.0 ** -6)
    # strict left-to-right sum over k in fp32
    A = np.array([[1.0, 2.0 ** -24, 2.0 ** -24]], np.float32)
    B = np.ones((1, 3), np.float32)
    assert to.gemm_universal_fma(A, B, c)[0, 0] == np.float32(1.0)
    assert to.gemm_universal_fma(A[:, ::-1], B, c)[0, 0] == np.float32(1.0 + 2.0 ** -23)


def test_round_bf16():
    x = np.array([1.0, 1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8, -(1.0 + 2.0 ** -8 + 2.0 ** -20), 3.0e38],
                 np.float32)
    want = np.array([1.0, 1.0, 1.0 + 2.0 ** -6, -(1.0 + 2.0 ** -7), 3.0e38], np.float32)
    got = to.round_bf16(x)
    assert (got[:4] == want[:4]).all()
    assert (got.view(np.uint32) & 0xFFFF == 0).all()
    try:
        import torch
        t = torch.from_numpy(np.random.default_rng(0).standard_normal(4096).astype(np.float32))
        assert (to.round_bf16(t.numpy()) == t.to(torch.bfloat16).to(torch.float32).numpy()).all()
    except ImportError:
        pass


def test_axpby_known_answers():
    """axpby! (src/algorithm/blas.jl:1-9): hand-built cases that separate the reference's arithmetic
    from its plausible mis-statements."""
    f32 = np.float32
    # b == 0 must not read Y: NaN in Y disappears (the iszero(b) branch)
    X = to.Array(np.array([1, 2, 3], f32), lo.make_layout(S(3)))
    Y = to.Array(np.array([np.nan, np.inf, 5], f32), lo.make_layout(S(3)))
    to.axpby(2.0, X, 0.0, Y)
    assert Y.buf.tolist() == [2.0, 4.0, 6.0]
    # unfused: a*x is rounded before the add.  a = x = 1 + 2^-12: a*x = 1 + 2^-11 + 2^-24 rounds (ties to
    # even) to 1 + 2^-11, and y = -(1 + 2^-11) cancels it exactly; an fma would leave 2^-24
    v = f32(1 + 2.0 ** -12)
    X = to.Array(np.array([v], f32), lo.make_layout(S(1)))
    Y = to.Array(np.array([-(1 + 2.0 ** -11)], f32), lo.make_layout(S(1)))
    to.axpby(float(v), X, 1.0, Y)
    assert Y.buf[0] == 0.0
    # fp16: every operation rounded to fp16.  a*x = 3 * 0.1(fp16) is rounded once, then b*y, then the sum
    h = np.float16
    X = to.Array(np.array([0.1], h), lo.make_layout(S(1)))
    Y = to.Array(np.array([1000.0], h), lo.make_layout(S(1)))
    to.axpby(3.0, X, 1.0, Y)
    ax = h(h(3.0) * h(0.1))
    assert Y.buf[0] == h(np.float32(ax) + np.float32(1000.0))
    # through layouts: X column-major, Y row-major views of 2x3
    X = to.Array(np.arange(6, dtype=f32), lo.make_layout((S(2), S(3))))
    Y = to.Array(np.zeros(6, f32), lo.make_layout((S(2), S(3)), (S(3), S(1))))
    to.axpby(1.0, X, 0.0, Y)
    assert Y.buf.reshape(2, 3).tolist() == [[0, 2, 4], [1, 3, 5]]
    # fill!: only the elements the layout reaches
    Z = to.Array(np.zeros(8, f32), lo.make_layout((S(2), S(2)), (S(1), S(4))))
    to.fill(Z, 7)
    assert Z.buf.tolist() == [7, 7, 0, 0, 7, 7, 0, 0]


def test_broadcast_layouts_and_known_answers():
    """test/broadcast.jl:3-17: `x .+ x`, `x .+ 1` and `x .+ y` (y of lower rank) give owning arrays with x's
    layout; values by hand."""
    f32 = np.float32
    x = to.Array(np.arange(1, 7, dtype=f32), lo.make_layout((S(3), S(2))))
    x2 = to.broadcast("add", x, x)
    x3 = to.broadcast("add", x, None, 1)
    assert x2.layout == L("(_3,_2):(_1,_3)") and x3.layout == x2.layout
    assert x2.buf.tolist() == [2, 4, 6, 8, 10, 12] and x3.buf.tolist() == [2, 3, 4, 5, 6, 7]
    assert x2.buf is not x.buf                                      # an owning result (ArrayEngine), x untouched
    y = to.Array(np.array([10, 0, 20, 0, 30, 0], f32), lo.make_layout((S(3),), (S(2),)))
    z = to.broadcast("add", x, y)                                   # test/broadcast.jl:15-17
    assert z.layout == x.layout
    assert z.buf.tolist() == [11, 22, 33, 14, 25, 36]               # y repeats over the second mode
    # through layouts: make_layout_like keeps the order of the strides (a row-major view gives a row-major result),
    # a padded view gives a compact one; operands meet by logical index
    xr = to.Array(np.arange(1, 7, dtype=f32), lo.make_layout((S(3), S(2)), (S(2), S(1))))
    r = to.broadcast("mul", xr, None, 2)
    assert r.layout == L("(_3,_2):(_2,_1)") and r.buf.tolist() == [2, 4, 6, 8, 10, 12]
    xp = to.Array(np.arange(8, dtype=f32), lo.make_layout((S(3), S(2)), (S(1), S(4))))    # pitch 4: 0 1 2 | 4 5 6
    rp = to.broadcast("add", xp, x)
    assert rp.layout == L("(_3,_2):(_1,_3)") and rp.buf.tolist() == [1, 3, 5, 8, 10, 12]
    # device/broadcast.jl:5-9 in numbers: fill!(a, 1); a .= a .* 2; sum(a) == 12
    a = to.Array(np.zeros(6, np.float64), lo.make_layout((S(3), S(2))))
    to.fill(a, 1.0)
    to.broadcast("mul", a, None, 2, out=a)
    assert a.buf.sum() == 12.0
    # Julia's max/min on floats: the NaN operand wins, and the signs of zeros are ordered
    u = to.Array(np.array([np.nan, 1.0, -0.0, 0.0], f32), lo.make_layout(S(4)))
    v = to.Array(np.array([1.0, np.nan, 0.0, -0.0], f32), lo.make_layout(S(4)))
    mx, mn = to.broadcast("max", u, v).buf, to.broadcast("min", u, v).buf
    assert np.isnan(mx[0]) and np.isnan(mx[1]) and np.isnan(mn[0]) and np.isnan(mn[1])
    assert not np.signbit(mx[2]) and not np.signbit(mx[3]) and np.signbit(mn[2]) and np.signbit(mn[3])
    # fp16: one rounding per operation
    h = np.float16
    p = to.Array(np.array([0.1, 1000.0], h), lo.make_layout(S(2)))
    q = to.broadcast("mul", p, None, 3.0)
    assert q.buf[0] == h(np.float32(h(0.1)) * np.float32(3.0)) and q.buf.dtype == h


def test_copyto_if_moves_only_where_the_mask_is_true():
    """algorithm/copy.jl:4-12: `if mask(i) apply(copy_op, pointer(dest, i), pointer(src, i))` over the linear index;
    checked by the element loop written out, on layouts where dst, src and mask all order their elements differently."""
    ls, ld, lm = lo.parse_layout("(4,6):(1,4)"), lo.parse_layout("(4,6):(6,1)"), lo.parse_layout("((2,2),6):((12,1),2)")
    rng = np.random.default_rng(5)
    src = to.Array(rng.integers(-100, 100, 24).astype(np.int32), ls)
    mask = to.Array((rng.random(24) < 0.5).astype(np.uint8), lm)
    dst = to.Array(np.full(24, 7, np.int32), ld)
    want = dst.buf.copy()
    for i in range(1, 25):
        if mask.buf[int(lm(i)) - 1]:
            want[int(ld(i)) - 1] = src.buf[int(ls(i)) - 1]
    to.copyto_if(dst, src, mask)
    assert np.array_equal(dst.buf, want)
    assert 0 < int((want == 7).sum()) < 24            # some moved, some kept
    # an all-true mask is copyto!
    d2, d3 = to.Array(np.full(24, 7, np.int32), ld), to.Array(np.full(24, 7, np.int32), ld)
    to.copyto_if(d2, src, to.Array(np.ones(24, np.uint8), lm))
    to.copyto(d3, src)
    assert np.array_equal(d2.buf, d3.buf)
    with pytest.raises(ValueError):
        to.copyto_if(dst, src, to.Array(np.ones(12, np.uint8), lo.parse_layout("12:1")))


def test_gemm_epilogue_oracle_known_answers():
    """The epilogue oracle (axpby! then one broadcast, then the converting copy): hand-built cases that a fused
    multiply-add, a dropped beta, a transposed operand or a wrong conversion would fail."""
    import tiled_oracle as to
    f32 = np.float32
    # alpha * acc rounds to 1 + 2^-11 (the exact product has a further 2^-24: a tie, to even); adding -(1 + 2^-11)
    # gives exactly 0 when the product is rounded first and 2^-24 when product and sum are fused
    a = f32(1) + f32(2.0 ** -12)
    acc = np.full((2, 3), a, f32)
    C = np.full((2, 3), -(f32(1) + f32(2.0 ** -11)), f32)
    r = to.gemm_epilogue(acc, a, 1.0, C, None, None, 0.0, "f32")
    assert r.dtype == np.float32 and np.all(r == 0.0)
    # beta == 0 leaves C out altogether, NaNs included (axpby!'s iszero(b))
    r = to.gemm_epilogue(np.ones((2, 3), f32), 2.0, 0.0, np.full((2, 3), np.nan, f32), None, None, 0.0, "f32")
    assert np.all(r == 2.0)
    # beta scales C, then the sum: 0.5 * 3 + (-2) * 4 = -6.5; fp16 result
    r = to.gemm_epilogue(np.full((2, 2), 3, f32), 0.5, -2.0, np.full((2, 2), 4, np.float16), None, None, 0.0, "f16")
    assert r.dtype == np.float16 and np.all(r == np.float16(-6.5))
    # a row vector is repeated down the rows, a column vector along them
    acc = np.arange(6, dtype=f32).reshape(2, 3)
    assert np.array_equal(to.gemm_epilogue(acc, 1.0, 0.0, None, "add", np.array([[10, 20, 30]], f32), 0.0, "f32"),
                          np.array([[10, 21, 32], [13, 24, 35]], f32))
    assert np.array_equal(to.gemm_epilogue(acc, 1.0, 0.0, None, "sub", np.array([[10], [20]], f32), 0.0, "f32"),
                          np.array([[-10, -9, -8], [-17, -16, -15]], f32))
    # relu through max with a scalar; Julia's max: NaN wins, +0 > -0
    r = to.gemm_epilogue(np.array([[-1.0, np.nan, -0.0, 2.0]], f32), 1.0, 0.0, None, "max", None, 0.0, "f32")
    assert r[0, 0] == 0 and np.isnan(r[0, 1]) and r[0, 3] == 2 and not np.signbit(r[0, 2])
    # conversion is round-to-nearest-even after the operation: 2049 is a tie in fp16 (-> 2048), 2051 -> 2052; bf16: 257 -> 256, 259 -> 260
    r = to.gemm_epilogue(np.array([[2048.0, 2050.0]], f32), 1.0, 0.0, None, "add", None, 1.0, "f16")
    assert list(r[0].astype(np.float64)) == [2048.0, 2052.0]
    r = to.gemm_epilogue(np.array([[256.0, 258.0]], f32), 1.0, 0.0, None, "add", None, 1.0, "bf16")
    assert list(r[0].astype(np.float64)) == [256.0, 260.0]
    # division and the unary operations
    assert to.gemm_epilogue(np.array([[1.0]], f32), 1.0, 0.0, None, "div", None, 3.0, "f32")[0, 0] == f32(1) / f32(3)
    assert to.gemm_epilogue(np.array([[-2.5]], f32), 1.0, 0.0, None, "abs", None, 0.0, "f32")[0, 0] == 2.5
    assert to.gemm_epilogue(np.array([[-2.5]], f32), 1.0, 0.0, None, "neg", None, 0.0, "f32")[0, 0] == 2.5


def test_vectorised_offsets_match_the_element_loop():
    """Array.offsets() for large arrays decomposes all indices at once; same numbers as layout(i) element by element on
    hierarchical, padded, zero-stride and row-major layouts."""
    import tiled_oracle as to
    from layout_oracle import Layout, make_layout
    for shape, stride in [((4, 6), (1, 4)), ((4, 6), (6, 1)), (((2, 3), (2, 2)), ((1, 4), (2, 12))), ((8, 5), (0, 1)),
                          ((3, (2, 4)), (16, (1, 2))), (12, 3), ((5, 7, 2), (1, 10, 100))]:
        a = to.Array(np.zeros(1), Layout(shape, stride), offset=7)
        want = np.array([a.index0(i) for i in range(1, len(a) + 1)], dtype=np.int64)
        assert np.array_equal(a.offsets_vectorised(), want), (shape, stride)
    big = to.Array(np.zeros(1), make_layout((96, 64)))
    assert len(big) > 4096 and np.array_equal(big.offsets(), np.arange(96 * 64))

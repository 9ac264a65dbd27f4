"""GPU parity of copyto! through the C ABI (moye_copy) against the CPU oracle and against the
closed form the reference's own device tests use (`a == transpose(b)`,
test/host/copy_async.jl:43,95).  Bit-exact: everything is compared as integers."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

import layout_oracle as lo  # noqa: E402
import tiled_oracle as to  # noqa: E402


@pytest.fixture(scope="module")
def mh():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    import moye_hip
    from moye_hip import torch_interop  # noqa: F401
    return moye_hip


def _tens(mh, t, shape, stride):
    from moye_hip.torch_interop import tensor_of
    return tensor_of(t, shape, stride)


def _flat(l):
    f = lo.lflatten(l)
    s, d = f.shape, f.stride
    if not isinstance(s, tuple):
        s, d = (s,), (d,)
    return [int(x) for x in s], [int(x) for x in d]


def _rand_bits(n, seed, device="cuda"):
    g = torch.Generator(device="cpu").manual_seed(seed)
    return torch.randint(-2 ** 31, 2 ** 31 - 1, (n,), dtype=torch.int32, generator=g).to(device)


@pytest.mark.parametrize("M,N", [(64, 64), (128, 256), (192, 64), (1024, 2048)])
def test_transpose_matches_oracle_and_closed_form(mh, M, N):
    """config-2 shape family: column-major src -> row-major dst through the 64x64 LDS tile."""
    src = _rand_bits(M * N, 1002)
    dst = torch.zeros(M * N, dtype=torch.int32, device="cuda")
    tc = mh.tiled_copy_desc(op=mh.COPY_LDS_TILED, vec_bits=128, tiler=(64, 64))
    mh.copyto_(_tens(mh, dst, (M, N), (N, 1)), _tens(mh, src, (M, N), (1, M)), tc)
    torch.cuda.synchronize()
    assert torch.equal(dst.view(M, N), src.view(N, M).t())
    if M * N <= 128 * 256:  # the oracle walks both layouts element by element
        s = to.Array(src.cpu().numpy(), lo.make_layout((M, N), (1, M)))
        d = to.Array(np.zeros(M * N, np.int32), lo.make_layout((M, N), (N, 1)))
        to.copyto(d, s)
        assert np.array_equal(d.buf, dst.cpu().numpy())


def test_transpose_other_orientation_and_pitch(mh):
    """row-major src -> column-major dst, with padded leading dimensions on both sides."""
    M, N, lds, ldd = 128, 192, 200, 136
    src = _rand_bits(M * lds, 7)
    dst = torch.full((N * ldd,), -1, dtype=torch.int32, device="cuda")
    mh.copyto_(_tens(mh, dst, (M, N), (1, ldd)), _tens(mh, src, (M, N), (lds, 1)))
    torch.cuda.synchronize()
    assert torch.equal(dst.view(N, ldd)[:, :M], src.view(M, lds)[:, :N].t())
    assert bool((dst.view(N, ldd)[:, M:] == -1).all())  # padding untouched


@pytest.mark.parametrize("dt", ["float32", "float16"])
@pytest.mark.parametrize("M,N", [(1000, 1032), (72, 4104), (8200, 136), (64, 64 + 8)])
def test_ragged_transpose_interior_and_strips(mh, M, N, dt):
    """Sizes that are not multiples of the 64 x 64 tile: the interior goes through the LDS tiles, the strips through the
    general kernel; together they are the transpose, bit for bit, and nothing outside dst is written."""
    tdt = getattr(torch, dt)
    bits = _rand_bits(M * N, 5).view(torch.int32)
    src = (bits.view(torch.float32) if dt == "float32" else bits.to(torch.int16).view(torch.float16)).clone()   # any bit pattern
    big = torch.full(((N + 2) * M + 16,), 7, dtype=tdt, device="cuda")
    dst = big[8:8 + N * M]
    # src column-major (M, N):(1, M) ... as a row-major (M, N):(N, 1)
    mh.copyto_(_tens(mh, dst, (M, N), (N, 1)), _tens(mh, src, (M, N), (1, M)))
    torch.cuda.synchronize()
    it = torch.int32 if dt == "float32" else torch.int16
    assert torch.equal(dst.view(it).view(M, N), src.view(it).view(N, M).t())
    assert bool((big[:8] == 7).all()) and bool((big[8 + N * M:] == 7).all())


@pytest.mark.parametrize("dt", ["float32", "float16"])
def test_ragged_transpose_with_padded_pitches(mh, dt):
    """Sizes that are not even whole 16-byte pieces, inside aligned pitches: the strips go through the general kernel."""
    tdt = getattr(torch, dt)
    M, N, PM, PN = 1002, 205, 1008, 208
    it = torch.int32 if dt == "float32" else torch.int16
    src = _rand_bits(PM * N, 6).to(it).view(tdt).clone()
    dst = torch.full((M * PN,), 7, dtype=tdt, device="cuda")
    mh.copyto_(_tens(mh, dst, (M, N), (PN, 1)), _tens(mh, src, (M, N), (1, PM)))
    torch.cuda.synchronize()
    got = dst.view(it).view(M, PN)
    assert torch.equal(got[:, :N], src.view(it).view(N, PM)[:, :M].t())
    assert bool((dst.view(M, PN)[:, N:] == 7).all())          # the padding of dst is untouched


def test_transpose_without_swizzle_is_identical(mh):
    M = N = 256
    src = _rand_bits(M * N, 11)
    a = torch.zeros_like(src)
    b = torch.zeros_like(src)
    mh.copyto_(_tens(mh, a, (M, N), (N, 1)), _tens(mh, src, (M, N), (1, M)))
    tc = mh.tiled_copy_desc(op=mh.COPY_LDS_TILED, tiler=(64, 64), flags=mh.GEMM_NO_LDS_SWIZZLE)
    mh.copyto_(_tens(mh, b, (M, N), (N, 1)), _tens(mh, src, (M, N), (1, M)), tc)
    torch.cuda.synchronize()
    assert torch.equal(a, b)


def test_transpose_full_size_involution(mh):
    """Benchmark configuration 2 at full size (16384^2 fp32 bits, 1 GiB each side): closed form on sampled
    tiles, an order-independent checksum, and transpose(transpose(x)) == x."""
    M = N = 16384
    src = _rand_bits(M * N, 1002)
    dst = torch.empty_like(src)
    tc = mh.tiled_copy_desc(op=mh.COPY_LDS_TILED, vec_bits=128, tiler=(64, 64))
    mh.copyto_(_tens(mh, dst, (M, N), (N, 1)), _tens(mh, src, (M, N), (1, M)), tc)
    torch.cuda.synchronize()
    assert int(dst.sum(dtype=torch.int64)) == int(src.sum(dtype=torch.int64))
    # every element against the closed form dst[i, j] == src[j, i] (test/host/copy_async.jl:43,95), 2048 rows at a time
    # so that the comparison's temporaries stay small
    for r in range(0, M, 2048):
        assert torch.equal(dst.view(M, N)[r:r + 2048], src.view(N, M)[:, r:r + 2048].t()), "rows %d.." % r
    rng = np.random.default_rng(0)
    for _ in range(64):
        i, j = int(rng.integers(0, M - 64)), int(rng.integers(0, N - 64))
        assert torch.equal(dst.view(M, N)[i:i + 64, j:j + 64], src.view(N, M)[j:j + 64, i:i + 64].t())
    back = torch.empty_like(src)
    # dst viewed as the column-major matrix of the transposed problem
    mh.copyto_(_tens(mh, back, (N, M), (M, 1)), _tens(mh, dst, (N, M), (1, N)), tc)
    torch.cuda.synchronize()
    assert torch.equal(back, src)


CASES = [
    # (dst layout, src layout) — hierarchical, strided, broadcast-free
    ("(4,6):(6,1)", "(4,6):(1,4)"),
    ("((2,3),(2,4)):((1,16),(2,4))", "(6,8):(1,6)"),
    ("(32,(2,4)):(2,(1,64))", "(32,8):(1,32)"),
    ("(3,5,7):(35,7,1)", "(3,5,7):(1,3,15)"),
    ("(8,9):(1,10)", "(8,9):(11,1)"),
    ("105:1", "(3,5,7):(1,3,15)"),
]


@pytest.mark.parametrize("dl,sl", CASES)
@pytest.mark.parametrize("dtype", ["int8", "int16", "int32", "int64"])
def test_generic_copy_matches_oracle(mh, dl, sl, dtype):
    """Arbitrary layouts go through the gather/scatter kernel; the oracle is the element loop of
    src/algorithm/copy.jl:4-12."""
    ld, ls = lo.parse_layout(dl), lo.parse_layout(sl)
    ns, nd = int(lo.cosize(ls)), int(lo.cosize(ld))
    tdt = getattr(torch, dtype)
    info = torch.iinfo(tdt)
    g = torch.Generator().manual_seed(3)
    src = torch.randint(max(info.min, -2 ** 62), min(info.max, 2 ** 62), (ns,), dtype=tdt, generator=g)
    dst0 = torch.full((nd,), 5, dtype=tdt)
    s_sh, s_st = _flat(ls)
    d_sh, d_st = _flat(ld)
    src_d, dst_d = src.cuda(), dst0.cuda()
    mh.copyto_(_tens(mh, dst_d, d_sh, d_st), _tens(mh, src_d, s_sh, s_st))
    torch.cuda.synchronize()
    o_dst = to.Array(dst0.numpy().copy(), ld)
    to.copyto(o_dst, to.Array(src.numpy(), ls))
    assert np.array_equal(o_dst.buf, dst_d.cpu().numpy())


MASK_LAYOUTS = ["(4,6):(1,4)", "((2,3),(2,4)):((3,1),(6,12))", "(32,8):(8,1)", "(3,5,7):(1,3,15)", "72:1", "105:1"]


@pytest.mark.parametrize("case", range(len(CASES)))
@pytest.mark.parametrize("dtype", ["int8", "int32", "int64", "float16->float32", "float32->bfloat16"])
def test_copy_if_matches_oracle(mh, case, dtype):
    """copyto_if! (src/algorithm/copy.jl:4-16): the mask has a layout of its own; elements whose mask is false keep
    the value dst had.  Plain and converting copies, compared bit for bit with the oracle's element loop."""
    dl, sl = CASES[case]
    ld, ls, lm = lo.parse_layout(dl), lo.parse_layout(sl), lo.parse_layout(MASK_LAYOUTS[case])
    ns, nd, nm = int(lo.cosize(ls)), int(lo.cosize(ld)), int(lo.cosize(lm))
    g = torch.Generator().manual_seed(11 + case)
    if "->" in dtype:
        sdt, ddt = (getattr(torch, x) for x in dtype.split("->"))
        src = (torch.randn(ns, generator=g) * 100).to(sdt)
        dst0 = torch.full((nd,), 5.0, dtype=ddt)
    else:
        sdt = ddt = getattr(torch, dtype)
        info = torch.iinfo(sdt)
        src = torch.randint(max(info.min, -2 ** 62), min(info.max, 2 ** 62), (ns,), dtype=sdt, generator=g)
        dst0 = torch.full((nd,), 5, dtype=ddt)
    mask = (torch.rand(nm, generator=g) < 0.5).to(torch.uint8) * 3          # any nonzero byte is true
    src_d, dst_d, mask_d = src.cuda(), dst0.cuda(), mask.cuda()
    mh.copyto_if_(_tens(mh, dst_d, *_flat(ld)), _tens(mh, src_d, *_flat(ls)), _tens(mh, mask_d, *_flat(lm)))
    torch.cuda.synchronize()
    as_np = lambda t: t.float().numpy().copy() if t.dtype == torch.bfloat16 else t.numpy().copy()
    o_dst = to.Array(as_np(dst0), ld)
    o_src = to.Array(as_np(src), ls)
    if ddt == torch.bfloat16:       # numpy has no bfloat16: convert through torch, element by element as the oracle would
        keep = to.Array(mask.numpy(), lm).values() != 0
        want = dst0.clone()
        want[torch.from_numpy(o_dst.offsets()[keep])] = src[torch.from_numpy(o_src.offsets()[keep])].to(ddt)
        assert torch.equal(want.view(torch.int16), dst_d.cpu().view(torch.int16))
    else:
        to.copyto_if(o_dst, o_src, to.Array(mask.numpy(), lm))
        assert np.array_equal(o_dst.buf.view(np.uint8), dst_d.cpu().numpy().view(np.uint8))
    # all-true and all-false masks: copyto! and nothing
    ones = torch.ones(nm, dtype=torch.uint8, device="cuda")
    d1, d2 = dst0.cuda(), dst0.cuda()
    mh.copyto_if_(_tens(mh, d1, *_flat(ld)), _tens(mh, src_d, *_flat(ls)), _tens(mh, ones, *_flat(lm)))
    mh.copyto_(_tens(mh, d2, *_flat(ld)), _tens(mh, src_d, *_flat(ls)))
    torch.cuda.synchronize()
    assert torch.equal(d1.view(torch.uint8), d2.view(torch.uint8))
    zeros = torch.zeros(nm, dtype=torch.uint8, device="cuda")
    d3 = dst0.cuda()
    mh.copyto_if_(_tens(mh, d3, *_flat(ld)), _tens(mh, src_d, *_flat(ls)), _tens(mh, zeros, *_flat(lm)))
    torch.cuda.synchronize()
    assert torch.equal(d3.cpu().view(torch.uint8), dst0.view(torch.uint8))


def test_copy_if_errors(mh):
    from moye_hip import _lib
    x = torch.zeros(24, dtype=torch.float32, device="cuda")
    m8 = torch.zeros(24, dtype=torch.uint8, device="cuda")
    with pytest.raises(mh.MoyeError) as e:        # mask of the wrong size
        mh.copyto_if_(_tens(mh, x, [24], [1]), _tens(mh, x, [24], [1]), _tens(mh, m8, [12], [1]))
    assert e.value.status == _lib.ERR_SHAPE
    with pytest.raises(mh.MoyeError) as e:        # mask that is not bytes
        mh.copyto_if_(_tens(mh, x, [24], [1]), _tens(mh, x, [24], [1]), _tens(mh, x, [24], [1]))
    assert e.value.status == _lib.ERR_UNSUPPORTED


def test_contiguous_copy_and_odd_sizes(mh):
    for n in (1, 7, 4096, 1000003):
        src = _rand_bits(n, n)
        dst = torch.zeros_like(src)
        mh.copyto_(_tens(mh, dst, (n,), (1,)), _tens(mh, src, (n,), (1,)))
        torch.cuda.synchronize()
        assert torch.equal(dst, src)
    # same dense order expressed with two modes
    src = _rand_bits(96 * 40, 5)
    dst = torch.zeros_like(src)
    mh.copyto_(_tens(mh, dst, (96, 40), (1, 96)), _tens(mh, src, (96 * 40,), (1,)))
    torch.cuda.synchronize()
    assert torch.equal(dst, src)


def test_converting_copy_rounds_to_nearest_even(mh):
    """UniversalCopy{TS,TD} converts with Julia's `convert` (src/arch/copy/copy.jl:38-43)."""
    g = torch.Generator().manual_seed(9)
    x = torch.randn(5000, generator=g) * 3
    x[:6] = torch.tensor([1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11, 65520.0, -65519.0, 2.0 ** -25, 0.0])
    xd = x.cuda()
    h = torch.zeros(5000, dtype=torch.float16, device="cuda")
    b = torch.zeros(5000, dtype=torch.bfloat16, device="cuda")
    mh.copyto_(_tens(mh, h, (5000,), (1,)), _tens(mh, xd, (5000,), (1,)))
    mh.copyto_(_tens(mh, b, (50, 100), (100, 1)), _tens(mh, xd, (50, 100), (1, 50)))
    torch.cuda.synchronize()
    want_h = x.numpy().astype(np.float16)
    assert np.array_equal(h.cpu().numpy().view(np.uint16), want_h.view(np.uint16))
    want_b = to.round_bf16(x.numpy().reshape(100, 50).T.copy()).reshape(-1)
    got_b = b.cpu().float().numpy().reshape(-1)
    assert np.array_equal(got_b.view(np.uint32), want_b.view(np.uint32))
    # and back up, exactly
    up = torch.zeros(5000, dtype=torch.float32, device="cuda")
    mh.copyto_(_tens(mh, up, (5000,), (1,)), _tens(mh, h, (5000,), (1,)))
    torch.cuda.synchronize()
    assert np.array_equal(up.cpu().numpy(), want_h.astype(np.float32))


def test_dense_converting_copy_matches_the_general_kernel(mh):
    """Every pair of floating-point types, sizes that are not a multiple of the group a lane converts: two aligned
    runs take the 16-byte kernel, the same values one element off alignment take the general one; same bits (NaN
    payloads aside), and the same as torch's conversion where torch rounds to nearest even too."""
    types = [torch.float32, torch.float16, torch.bfloat16, torch.float64]
    if hasattr(torch, "float8_e4m3fn"):
        types.append(torch.float8_e4m3fn)
    g = torch.Generator().manual_seed(17)
    for sdt in types:
        for ddt in types:
            if sdt == ddt:
                continue
            for n in (3, 1000, 70001):
                X = (torch.randn(n + 16, generator=g) * 20).to(sdt)
                xa = X[:n].clone().cuda()
                xu_ = X.cuda()
                xu_[1:n + 1] = xa
                d1 = torch.zeros(n, dtype=ddt, device="cuda")
                d2 = torch.zeros(n + 16, dtype=ddt, device="cuda")
                mh.copyto_(_tens(mh, d1, [n], [1]), _tens(mh, xa, [n], [1]))
                mh.copyto_(_tens(mh, d2[1:n + 1], [n], [1]), _tens(mh, xu_[1:n + 1], [n], [1]))
                torch.cuda.synchronize()
                it = {1: torch.uint8, 2: torch.int16, 4: torch.int32, 8: torch.int64}[d1.element_size()]
                a, b = d1.view(it), d2[1:n + 1].view(it)
                nan = torch.isnan(d1.float()) & torch.isnan(d2[1:n + 1].float())
                assert bool(((a == b) | nan).all()), (sdt, ddt, n)
                if ddt != getattr(torch, "float8_e4m3fn", None):         # torch saturates fp8 differently; covered elsewhere
                    want = xa.to(ddt)
                    assert bool(((a == want.view(it)) | (torch.isnan(d1.float()) & torch.isnan(want.float()))).all()), (sdt, ddt, n, "torch")


def test_pitched_converting_copies_and_masked_copies_in_groups(mh):
    """Pitched matrices (row-major inside wider buffers): converting copies between every pair of floating-point types, and
    copyto_if! of bits and with conversion, take a kernel that moves groups of elements along the rows.  Checked element
    by element: against torch's conversion of the same window (fp8 aside: against the library's own dense conversion),
    the masked-out elements and the padding untouched.  Shapes whose rows the group does not divide, or whose windows
    start off alignment, fall back to the element loop and must give the same bits."""
    types = [torch.float32, torch.float16, torch.bfloat16, torch.float64]
    if hasattr(torch, "float8_e4m3fn"):
        types.append(torch.float8_e4m3fn)
    g = torch.Generator().manual_seed(23)
    it_of = {1: torch.uint8, 2: torch.int16, 4: torch.int32, 8: torch.int64}
    for (R, Cn, ps, pd, off) in ((300, 512, 528, 640, 0), (257, 48, 64, 48, 0), (64, 200, 208, 216, 0), (33, 96, 100, 104, 0), (100, 128, 144, 160, 1)):
        for sdt in types:
            for ddt in types:
                X = (torch.randn(R, ps, generator=g) * 20).to(sdt).cuda()
                M = (torch.rand(R, Cn + 16, generator=g) < 0.4).to(torch.uint8).cuda() * 7
                src = X[:, off:off + Cn]
                want_full = src.to(ddt) if ddt != getattr(torch, "float8_e4m3fn", None) or sdt == ddt else None
                if want_full is None:           # the library's own conversion of a dense copy of the window
                    dense = src.contiguous()
                    want_full = torch.zeros(R, Cn, dtype=ddt, device="cuda")
                    mh.copyto_(_tens(mh, want_full, [R * Cn], [1]), _tens(mh, dense, [R * Cn], [1]))
                it = it_of[torch.empty(0, dtype=ddt).element_size()]
                if sdt != ddt:
                    D = torch.full((R, pd), 3.0).to(ddt).cuda()
                    mh.copyto_(_tens(mh, D[:, off:off + Cn], (R, Cn), (pd, 1)), _tens(mh, src, (R, Cn), (ps, 1)))
                    torch.cuda.synchronize()
                    got = D[:, off:off + Cn]
                    same = (got.contiguous().view(it) == want_full.contiguous().view(it)) | (torch.isnan(got.float()) & torch.isnan(want_full.float()))
                    assert bool(same.all()), (sdt, ddt, R, Cn, "converting copy")
                    frame = D.clone()
                    frame[:, off:off + Cn] = 3.0
                    assert bool((frame.float() == 3.0).all()), (sdt, ddt, "padding of dst touched")
                # copyto_if! with a mask that is a window of a wider byte array
                D = torch.full((R, pd), 3.0).to(ddt).cuda()
                mask = M[:, off:off + Cn]
                mh.copyto_if_(_tens(mh, D[:, off:off + Cn], (R, Cn), (pd, 1)), _tens(mh, src, (R, Cn), (ps, 1)), _tens(mh, mask, (R, Cn), (Cn + 16, 1)))
                torch.cuda.synchronize()
                got = D[:, off:off + Cn].contiguous()
                want = torch.where(mask != 0, want_full.float().double(), torch.full((), 3.0, dtype=torch.float64, device="cuda"))
                gotd = got.float().double()
                assert bool(((gotd == want) | (torch.isnan(gotd) & torch.isnan(want))).all()), (sdt, ddt, R, Cn, "copyto_if!")
                frame = D.clone()
                frame[:, off:off + Cn] = 3.0
                assert bool((frame.float() == 3.0).all()), (sdt, ddt, "padding of dst touched by copyto_if!")


def test_fp8_conversion_matches_torch(mh):
    if not hasattr(torch, "float8_e4m3fn"):
        pytest.skip("torch without float8_e4m3fn")
    g = torch.Generator().manual_seed(4)
    x = torch.cat([torch.randn(4000, generator=g) * 40, torch.linspace(-464, 464, 4001),
                   torch.tensor([2.0 ** -9, 2.0 ** -10, 3 * 2.0 ** -10, 0.0156, 448.0, 0.0])])
    n = x.numel()
    xd = x.cuda()
    q = torch.zeros(n, dtype=torch.float8_e4m3fn, device="cuda")
    mh.copyto_(_tens(mh, q, (n,), (1,)), _tens(mh, xd, (n,), (1,)))
    torch.cuda.synchronize()
    want = x.to(torch.float8_e4m3fn)
    assert torch.equal(q.cpu().view(torch.uint8), want.view(torch.uint8))
    back = torch.zeros(n, dtype=torch.float32, device="cuda")
    mh.copyto_(_tens(mh, back, (n,), (1,)), _tens(mh, q, (n,), (1,)))
    torch.cuda.synchronize()
    assert torch.equal(back.cpu(), want.float())


def test_copy_errors(mh):
    a = torch.zeros(64, dtype=torch.int32, device="cuda")
    af = a.float()
    with pytest.raises(mh.MoyeError) as e:
        mh.copyto_(_tens(mh, a, (8, 8), (1, 8)), _tens(mh, a, (8, 4), (1, 8)))
    assert e.value.status == mh._lib.ERR_SHAPE
    with pytest.raises(mh.MoyeError) as e:
        mh.copyto_(_tens(mh, a, (8, 8), (1, 8)), _tens(mh, af, (8, 8), (1, 8)))
    assert e.value.status == mh._lib.ERR_UNSUPPORTED
    tc = mh.tiled_copy_desc(op=mh.COPY_LDS_TILED, tiler=(64, 64))
    with pytest.raises(mh.MoyeError) as e:  # the 64x64 tiler does not divide 8x8 (zipped_divide's assertion)
        mh.copyto_(_tens(mh, a, (8, 8), (8, 1)), _tens(mh, a, (8, 8), (1, 8)), tc)
    assert e.value.status == mh._lib.ERR_SHAPE
    with pytest.raises(mh.MoyeError) as e:  # both sides with the unit stride on the same mode: not what the op is for
        wide = torch.zeros(128, dtype=torch.int32, device="cuda")
        mh.copyto_(_tens(mh, torch.zeros_like(wide), (8, 8), (1, 16)), _tens(mh, wide, (8, 8), (1, 16)),
                   mh.tiled_copy_desc(op=mh.COPY_LDS_TILED, tiler=(8, 8)))
    assert e.value.status == mh._lib.ERR_UNSUPPORTED
    empty = torch.zeros(0, dtype=torch.int32, device="cuda")
    mh.copyto_(_tens(mh, empty, (0,), (1,)), _tens(mh, empty, (0,), (1,)))


# ---------------------------------------------------------------------------------------------
# axpby! and fill! / zeros! (src/algorithm/blas.jl:1-9, src/algorithm/array_algorithms.jl:158-182)
# ---------------------------------------------------------------------------------------------

AXPBY_LAYOUTS = [
    ("(_4096)", "(_4096)"),                                      # both dense
    ("(_64,_48):(_1,_64)", "(_64,_48):(_48,_1)"),                # column-major X into row-major Y
    ("((_4,_8),(_2,_3)):((_1,_8),(_4,_64))", "(_32,_6):(_1,_40)"),  # hierarchical X, padded Y
]


@pytest.mark.parametrize("dt", ["float32", "float16", "bfloat16", "float64"])
def test_axpby_bit_exact_against_the_oracle(mh, dt):
    tdt = getattr(torch, dt)
    g = torch.Generator().manual_seed(7)
    for lx_text, ly_text in AXPBY_LAYOUTS:
        lx, ly = lo.parse_layout(lx_text), lo.parse_layout(ly_text)
        nx, ny = int(lo.cosize(lx)), int(lo.cosize(ly))
        for a, b in ((1.7, 0.0), (-0.3, 2.5), (1.0 + 2.0 ** -12, 1.0)):
            X = (torch.randn(nx, generator=g) * 3).to(tdt)
            Y = (torch.randn(ny, generator=g) * 3).to(tdt)
            if b == 0.0:
                Y[::3] = float("nan")          # must be overwritten, not propagated
            x, y = X.cuda(), Y.cuda()
            sx, dx = _flat(lx)
            sy, dy = _flat(ly)
            mh.axpby_(a, _tens(mh, x, sx, dx), b, _tens(mh, y, sy, dy))
            torch.cuda.synchronize()
            # oracle on the same bits
            if dt == "bfloat16":
                ox = to.Array(X.float().numpy().copy(), lx)
                oy = to.Array(Y.float().numpy().copy(), ly)
                oy.bf16 = True
                to.axpby(a, ox, b, oy)
            else:
                ox, oy = to.Array(X.numpy().copy(), lx), to.Array(Y.numpy().copy(), ly)
                to.axpby(a, ox, b, oy)
            # elements the layout does not reach keep their bits (NaN payloads included)
            reached = torch.from_numpy(np.asarray(oy.offsets(), dtype=np.int64))
            want = Y.clone()
            want[reached] = torch.from_numpy(oy.buf[reached.numpy()]).to(tdt)
            got = y.cpu()
            itype = {2: torch.int16, 4: torch.int32, 8: torch.int64}[got.element_size()]
            assert torch.equal(got.view(itype), want.view(itype)), (dt, lx_text, a, b)


def test_fill_and_zeros(mh):
    for dt, val in ((torch.float32, 3.25), (torch.float16, -1.5), (torch.bfloat16, 0.1), (torch.float64, 1e-300),
                    (torch.int32, 77)):
        y = torch.full((64,), 9, dtype=dt, device="cuda")
        # a strided view: every fourth element of the first 48
        mh.fill_(_tens(mh, y, [12], [4]), val)
        torch.cuda.synchronize()
        want = torch.full((64,), 9, dtype=dt)
        want[0:48:4] = torch.tensor(val, dtype=torch.float64).to(dt) if dt != torch.int32 else 77
        assert torch.equal(y.cpu(), want), dt
        mh.zeros_(_tens(mh, y, [64], [1]))
        torch.cuda.synchronize()
        assert float(y.abs().max()) == 0.0


MAP_LAYOUTS = [("(_4,_6):(_1,_4)", "(_4,_6):(_6,_1)", "(_4,_6):(_1,_8)"),           # dst, a, b
               ("((_2,_3),(_2,_4)):((_1,_16),(_2,_4))", "(_6,_8):(_1,_6)", "(_6):(_2)"),   # b spans the first mode of dst
               ("(_3,_5,_7):(_1,_3,_15)", "(_3,_5,_7):(_35,_7,_1)", "(_3,_5):(_5,_1)")]     # ... and the first two of three


@pytest.mark.parametrize("dt", ["float32", "float64", "float16", "bfloat16"])
def test_map_bit_exact_against_the_oracle(mh, dt):
    """dst .= op.(a, b) for every operation, array, lower-rank and scalar second operands, through
    hierarchical and padded layouts; NaNs and signed zeros included (Julia's max/min rules)."""
    tdt = getattr(torch, dt)
    g = torch.Generator().manual_seed(23)
    for ld_text, la_text, lb_text in MAP_LAYOUTS:
        ld, la, lb = lo.parse_layout(ld_text), lo.parse_layout(la_text), lo.parse_layout(lb_text)
        nd, na, nb = int(lo.cosize(ld)), int(lo.cosize(la)), int(lo.cosize(lb))
        for op in ("identity", "add", "sub", "mul", "div", "max", "min", "neg", "abs"):
            for second in ("array", "scalar"):
                A = (torch.randn(na, generator=g) * 3).to(tdt)
                B = (torch.randn(nb, generator=g) * 3).to(tdt)
                if dt in ("float32", "float64"):
                    A[1], A[3], B[0] = float("nan"), -0.0, 0.0
                    B[2] = float("nan")
                Dst = torch.full((nd,), 9.0, dtype=tdt)
                a, b, d = A.cuda(), B.cuda(), Dst.cuda()
                sd, dd = _flat(ld)
                sa, da = _flat(la)
                sb, db = _flat(lb)
                mh.map_(op, _tens(mh, d, sd, dd), _tens(mh, a, sa, da), _tens(mh, b, sb, db) if second == "array" else None, 1.75)
                torch.cuda.synchronize()
                conv = (lambda t: t.float().numpy().copy()) if dt == "bfloat16" else (lambda t: t.numpy().copy())
                oa, ob, od = to.Array(conv(A), la), to.Array(conv(B), lb), to.Array(conv(Dst), ld)
                if dt == "bfloat16":
                    oa.bf16 = ob.bf16 = od.bf16 = True
                to.broadcast(op, oa, ob if second == "array" else None, 1.75, out=od)
                got, want = d.cpu(), torch.from_numpy(od.buf).to(tdt)
                itype = {2: torch.int16, 4: torch.int32, 8: torch.int64}[got.element_size()]
                same = got.view(itype) == want.view(itype)
                both_nan = torch.isnan(got.float()) & torch.isnan(want.float())     # NaN payloads are not compared
                assert bool((same | both_nan).all()), (dt, op, second, ld_text)


def test_broadcast_returns_a_compact_array_like_the_first_operand(mh):
    """test/broadcast.jl:3-17 on the device: `x .+ x`, `x .+ 1`, `x .+ y` with a lower-rank y."""
    from moye_hip import MoYeArray
    xt = torch.arange(1, 7, dtype=torch.float32, device="cuda")
    x = MoYeArray(xt.data_ptr(), mh.F32, lo_text("(_3,_2):(_1,_3)", mh), keep=xt)
    x2, x3 = mh.broadcast("add", x, x), mh.broadcast("add", x, None, 1.0)
    torch.cuda.synchronize()
    assert str(x2.layout) == str(x.layout) and x2.ptr != x.ptr
    assert x2._keep.tolist() == [2, 4, 6, 8, 10, 12] and x3._keep.tolist() == [2, 3, 4, 5, 6, 7]
    yt = torch.tensor([10, 0, 20, 0, 30, 0], dtype=torch.float32, device="cuda")
    y = MoYeArray(yt.data_ptr(), mh.F32, lo_text("(_3):(_2)", mh), keep=yt)
    z = mh.broadcast("add", x, y)
    torch.cuda.synchronize()
    assert str(z.layout) == str(x.layout) and z._keep.tolist() == [11, 22, 33, 14, 25, 36]
    with pytest.raises(mh.MoyeError):
        w = torch.zeros(4, device="cuda")
        mh.map_("add", x, x, MoYeArray(w.data_ptr(), mh.F32, lo_text("(_4):(_1)", mh), keep=w))


def lo_text(text, mh):
    from moye_hip.layout import Layout
    return Layout(text)


@pytest.mark.parametrize("dt", ["float32", "float64", "float16", "bfloat16"])
def test_dense_elementwise_paths_match_the_general_kernels(mh, dt):
    """Arrays that are one aligned run take 16-byte accesses; the same values behind a pointer that is not 16-byte
    aligned take the general kernels.  Both must give the same bits (axpby!, map! with array and scalar operands,
    fill!), for sizes that are not a multiple of the vector width and sizes beyond one chunk."""
    tdt = getattr(torch, dt)
    g = torch.Generator().manual_seed(31)
    itype = {2: torch.int16, 4: torch.int32, 8: torch.int64}[torch.empty(0, dtype=tdt).element_size()]
    for n in (1, 5, 4099, 1 << 20, (1 << 20) + 7):
        X, Y = (torch.randn(n + 1, generator=g) * 3).to(tdt), (torch.randn(n + 1, generator=g) * 3).to(tdt)
        xa, ya = X[:n].clone().cuda(), Y[:n].clone().cuda()              # aligned
        xu_, yu_ = X.cuda(), Y.cuda()
        xu_[1:] = xa
        yu_[1:] = ya
        xu, yu = xu_[1:], yu_[1:]                                         # the same values, one element off alignment
        def t1(t):
            return _tens(mh, t, [n], [1])
        for b in (0.0, -1.25):
            y1, y2 = ya.clone(), yu_.clone()
            mh.axpby_(0.75, t1(xa), b, t1(y1))
            mh.axpby_(0.75, t1(xu), b, t1(y2[1:]))
            torch.cuda.synchronize()
            assert torch.equal(y1.view(itype), y2[1:].view(itype)), (dt, n, "axpby", b)
        for op in ("add", "mul", "max", "div", "abs"):
            for second in ("array", "scalar"):
                d1, d2 = torch.zeros(n, dtype=tdt, device="cuda"), torch.zeros(n + 1, dtype=tdt, device="cuda")
                mh.map_(op, t1(d1), t1(xa), t1(ya) if second == "array" else None, 1.75)
                mh.map_(op, t1(d2[1:]), t1(xu), t1(yu) if second == "array" else None, 1.75)
                torch.cuda.synchronize()
                same = d1.view(itype) == d2[1:].view(itype)
                assert bool((same | (torch.isnan(d1.float()) & torch.isnan(d2[1:].float()))).all()), (dt, n, op, second)
        if dt == "float32":       # and against torch where the rounding is plain IEEE
            d1 = torch.zeros(n, dtype=tdt, device="cuda")
            mh.map_("add", t1(d1), t1(xa), t1(ya))
            torch.cuda.synchronize()
            assert torch.equal(d1, xa + ya)
        f1, f2 = torch.zeros(n, dtype=tdt, device="cuda"), torch.zeros(n + 1, dtype=tdt, device="cuda")
        mh.fill_(t1(f1), 2.71828)
        mh.fill_(t1(f2[1:]), 2.71828)
        torch.cuda.synchronize()
        assert torch.equal(f1.view(itype), f2[1:].view(itype)) and float(f2[0]) == 0.0
        assert torch.equal(f1, torch.full((n,), 2.71828, dtype=tdt, device="cuda"))
    for idt in (torch.uint8, torch.int16, torch.int32, torch.int64):        # fill! of integer arrays through the dense path
        z = torch.zeros(1037, dtype=idt, device="cuda")
        mh.fill_(_tens(mh, z, [1037], [1]), 93)
        torch.cuda.synchronize()
        assert bool((z == 93).all())


@pytest.mark.parametrize("dt", ["float32", "float64", "float16", "bfloat16"])
def test_elementwise_with_a_transposed_operand_matches_the_dense_kernels(mh, dt):
    """An operand whose unit stride lies on another mode than the destination's goes through LDS tiles: the same bits as the
    dense kernels give on a contiguous copy of that operand.  Ragged extents, a batch mode, a pitched destination inside a
    frame, one or both operands transposed, a scalar second operand, axpby! with and without the old Y."""
    tdt = getattr(torch, dt)
    g = torch.Generator(device="cuda").manual_seed(57)
    itype = {2: torch.int16, 4: torch.int32, 8: torch.int64}[tdt.itemsize]

    def rnd(*shape):
        return (torch.randn(*shape, generator=g, device="cuda") * 3).to(tdt)

    def flat(x):
        return _tens(mh, x, [x.numel()], [1])

    # (extents and pitches that are multiples of two (4-byte elements) or eight (2-byte) take the form with groups per lane)
    for (R, C, Bn) in ((64, 64, 1), (200, 77, 1), (130, 1000, 3), (16, 16, 5), (1025, 129, 2), (258, 130, 2), (128, 384, 1), (1000, 61, 1), (136, 264, 2)):
        # destination d[b][r][c] with c contiguous and a pitch of C + 3 or C + 8 inside a frame; xt[b][c][r] with r contiguous
        pad = 3 if C % 2 else 8           # (extents and pitches that are multiples of two or eight let the lanes take groups)
        frame = torch.full((Bn, R, C + pad), 55.0, device="cuda").to(tdt)
        x_same, xt, yt = rnd(Bn, R, C), rnd(Bn, C, R), rnd(Bn, C, R)
        shape, d_str = (C, R, Bn), (1, C + pad, R * (C + pad))
        same_str, t_str = (1, C, R * C), (R, 1, R * C)
        xt_c, yt_c = xt.transpose(1, 2).contiguous(), yt.transpose(1, 2).contiguous()   # what the transposed views hold, dense
        for op in ("add", "max", "div"):
            for (a_t, b_kind) in ((True, "same"), (False, "t"), (True, "t"), (True, "scalar")):
                a_dense = xt_c if a_t else x_same
                b_dense = {"same": x_same, "t": yt_c, "scalar": None}[b_kind]
                want = torch.zeros(Bn, R, C, device="cuda").to(tdt)
                mh.map_(op, flat(want), flat(a_dense), flat(b_dense) if b_dense is not None else None, 1.75)
                d = frame.clone()
                ta = _tens(mh, xt, shape, t_str) if a_t else _tens(mh, x_same, shape, same_str)
                tb = {"same": lambda: _tens(mh, x_same, shape, same_str), "t": lambda: _tens(mh, yt, shape, t_str), "scalar": lambda: None}[b_kind]()
                mh.map_(op, _tens(mh, d, shape, d_str), ta, tb, 1.75)
                torch.cuda.synchronize()
                got = d[:, :, :C].contiguous()
                same = got.view(itype) == want.view(itype)
                assert bool((same | (torch.isnan(got.float()) & torch.isnan(want.float()))).all()), (dt, R, C, Bn, op, a_t, b_kind)
                assert bool((d[:, :, C:].float() == 55.0).all()), "stores into the padding"
        for b in (0.0, -1.25):
            y0 = rnd(Bn, R, C)
            want = y0.clone()
            mh.axpby_(0.75, flat(xt_c), b, flat(want))
            d = frame.clone()
            d[:, :, :C] = y0
            mh.axpby_(0.75, _tens(mh, xt, shape, t_str), b, _tens(mh, d, shape, d_str))
            torch.cuda.synchronize()
            assert torch.equal(d[:, :, :C].contiguous().view(itype), want.view(itype)), (dt, R, C, Bn, "axpby", b)
            assert bool((d[:, :, C:].float() == 55.0).all()), "stores into the padding"
    if dt == "float32":   # and against torch where the rounding is plain IEEE
        x, y = rnd(300, 500), rnd(500, 300)
        d = torch.zeros(300, 500, device="cuda")
        mh.map_("add", _tens(mh, d, (500, 300), (1, 500)), _tens(mh, x, (500, 300), (1, 500)), _tens(mh, y, (500, 300), (300, 1)))
        torch.cuda.synchronize()
        assert torch.equal(d, x + y.t())


@pytest.mark.parametrize("dt", ["float32", "float16", "float64"])
def test_map_with_operands_that_repeat_along_a_mode(mh, dt):
    """Operands with a zero stride (one value per row or per column of dst), alone and next to a transposed operand, which
    sends the call through the LDS blocks: one rounded operation, so torch's result bit for bit."""
    tdt = getattr(torch, dt)
    g = torch.Generator(device="cuda").manual_seed(3)
    for (R, C) in ((64, 64), (200, 136), (130, 77), (1024, 512)):
        a = torch.randn(R, C, generator=g, device="cuda").to(tdt)
        at = torch.randn(C, R, generator=g, device="cuda").to(tdt)
        col = torch.randn(R, generator=g, device="cuda").to(tdt)
        row = torch.randn(C, generator=g, device="cuda").to(tdt)
        for name, ta, tb, want in (
                ("a + one per row", _tens(mh, a, (R, C), (C, 1)), _tens(mh, col, (R, C), (1, 0)), a + col[:, None]),
                ("a + one per column", _tens(mh, a, (R, C), (C, 1)), _tens(mh, row, (R, C), (0, 1)), a + row[None, :]),
                ("a' + one per row", _tens(mh, at, (R, C), (1, R)), _tens(mh, col, (R, C), (1, 0)), at.t() + col[:, None]),
                ("a' + one per column", _tens(mh, at, (R, C), (1, R)), _tens(mh, row, (R, C), (0, 1)), at.t() + row[None, :]),
                ("one per row + a'", _tens(mh, col, (R, C), (1, 0)), _tens(mh, at, (R, C), (1, R)), col[:, None] + at.t())):
            d = torch.zeros(R, C, device="cuda", dtype=tdt)
            mh.map_("add", _tens(mh, d, (R, C), (C, 1)), ta, tb)
            torch.cuda.synchronize()
            assert torch.equal(d, want.to(tdt)), (dt, R, C, name)


def test_axpby_errors(mh):
    x = torch.zeros(8, device="cuda")
    y = torch.zeros(8, dtype=torch.float16, device="cuda")
    with pytest.raises(mh.MoyeError):
        mh.axpby_(1.0, _tens(mh, x, [8], [1]), 1.0, _tens(mh, y, [8], [1]))
    with pytest.raises(mh.MoyeError):
        mh.axpby_(1.0, _tens(mh, x, [8], [1]), 1.0, _tens(mh, x, [4], [1]))


def test_generic_copy_vectorised_paths_bit_exact(mh):
    """Layouts whose logical neighbours are memory neighbours in runs (padded pitches, a flat source
    into a padded destination, runs of different lengths, misaligned bases, 2-byte elements): the copy
    may use 4..16-byte accesses, the result must not change."""
    cases = [("(_64,_48):(_1,_64)", "(_64,_48):(_1,_80)", 0, 0),
             ("(_3072)", "(_64,_48):(_1,_80)", 0, 0),
             ("(_6,_8):(_1,_6)", "(_4,_12):(_1,_10)", 0, 0),
             ("(_64,_48):(_1,_64)", "(_64,_48):(_1,_80)", 1, 0),      # source base off by one element
             ("(_64,_48):(_1,_64)", "(_64,_48):(_1,_82)", 0, 2),      # pitch and base only 8-byte friendly
             ("((_8,_8),_48):((_1,_16),_128)", "(_64,_48):(_1,_64)", 0, 0)]
    for dt in (torch.int32, torch.int16):
        for sl, dl, soff, doff in cases:
            ls, ld = lo.parse_layout(sl), lo.parse_layout(dl)
            ns, nd = int(lo.cosize(ls)) + soff, int(lo.cosize(ld)) + doff
            src = _rand_bits(ns, 5).to(dt)
            dst = torch.full((nd,), -1, dtype=dt, device="cuda")
            sx, dx = _flat(ls)
            sy, dy = _flat(ld)
            mh.copyto_(_tens(mh, dst[doff:], sy, dy), _tens(mh, src[soff:], sx, dx))
            torch.cuda.synchronize()
            want = np.full(nd, -1, dtype=src.cpu().numpy().dtype)
            o_src = to.Array(src.cpu().numpy()[soff:], ls)
            o_dst = to.Array(want[doff:], ld)
            to.copyto(o_dst, o_src)
            assert np.array_equal(dst.cpu().numpy(), want), (dt, sl, dl, soff, doff)


@pytest.mark.parametrize("M,N", [(64, 64), (128, 192), (512, 64), (192, 128), (256, 1024), (4096, 4096)])
def test_transpose_two_byte_elements(mh, M, N):
    """fp16 / bf16 matrices through the 2-byte LDS tile (1, 2, 4 or 8 tiles per workgroup depending on M):
    both orientations, padded pitches, bits compared as int16; the oracle on the small cases."""
    src = _rand_bits(M * N, 31).to(torch.int16)
    dst = torch.zeros(M * N, dtype=torch.int16, device="cuda")
    tc = mh.tiled_copy_desc(op=mh.COPY_LDS_TILED, vec_bits=128, tiler=(64, 64))
    mh.copyto_(_tens(mh, dst, (M, N), (N, 1)), _tens(mh, src, (M, N), (1, M)), tc)
    torch.cuda.synchronize()
    assert torch.equal(dst.view(M, N), src.view(N, M).t())
    if M * N <= 128 * 256:
        s = to.Array(src.cpu().numpy(), lo.make_layout((M, N), (1, M)))
        d = to.Array(np.zeros(M * N, np.int16), lo.make_layout((M, N), (N, 1)))
        to.copyto(d, s)
        assert np.array_equal(d.buf, dst.cpu().numpy())
    # the other orientation with padded pitches (multiples of 8 elements = 16 bytes)
    lds, ldd = N + 8, M + 24
    src2 = _rand_bits(M * lds, 32).to(torch.int16)
    dst2 = torch.full((N * ldd,), -1, dtype=torch.int16, device="cuda")
    mh.copyto_(_tens(mh, dst2, (M, N), (1, ldd)), _tens(mh, src2, (M, N), (lds, 1)))
    torch.cuda.synchronize()
    assert torch.equal(dst2.view(N, ldd)[:, :M], src2.view(M, lds)[:, :N].t())
    assert bool((dst2.view(N, ldd)[:, M:] == -1).all())


@pytest.mark.parametrize("M,N", [(64, 256), (128, 512), (192, 256), (256, 1024), (512, 256), (768, 1280), (4096, 4096), (8192, 2048), (200, 300), (1088, 784),
                                 (16384, 12288)])
def test_transpose_one_byte_elements(mh, M, N):
    """fp8 matrices / bytes through the 1-byte LDS tiles (256 x 256 bytes in whole 256-byte runs where M is a multiple of 256,
    else 64 x 256 with 1 or 2 sub-tiles per workgroup), sizes
    that are not multiples of the tile through interior + strips or the general kernel: both orientations, padded pitches,
    compared as bytes; the oracle on the small cases."""
    g = torch.Generator().manual_seed(M + N)
    src = torch.randint(0, 256, (M * N,), dtype=torch.uint8, generator=g).cuda()
    dst = torch.zeros(M * N, dtype=torch.uint8, device="cuda")
    mh.copyto_(_tens(mh, dst, (M, N), (N, 1)), _tens(mh, src, (M, N), (1, M)))
    torch.cuda.synchronize()
    assert torch.equal(dst.view(M, N), src.view(N, M).t())
    if M * N <= 128 * 512:
        s = to.Array(src.cpu().numpy(), lo.make_layout((M, N), (1, M)))
        d = to.Array(np.zeros(M * N, np.uint8), lo.make_layout((M, N), (N, 1)))
        to.copyto(d, s)
        assert np.array_equal(d.buf, dst.cpu().numpy())
    # the other orientation with padded pitches (multiples of 16 bytes)
    lds, ldd = N + 16, M + 48
    src2 = torch.randint(0, 256, (M * lds,), dtype=torch.uint8, generator=g).cuda()
    dst2 = torch.full((N * ldd,), 255, dtype=torch.uint8, device="cuda")
    mh.copyto_(_tens(mh, dst2, (M, N), (1, ldd)), _tens(mh, src2, (M, N), (lds, 1)))
    torch.cuda.synchronize()
    assert torch.equal(dst2.view(N, ldd)[:, :M], src2.view(M, lds)[:, :N].t())
    assert bool((dst2.view(N, ldd)[:, M:] == 255).all())
    if hasattr(torch, "float8_e4m3fn") and M % 64 == 0:      # the same through the fp8 element type
        s8, d8 = src.view(torch.float8_e4m3fn), torch.zeros(M * N, dtype=torch.uint8, device="cuda").view(torch.float8_e4m3fn)
        mh.copyto_(_tens(mh, d8, (M, N), (N, 1)), _tens(mh, s8, (M, N), (1, M)))
        torch.cuda.synchronize()
        assert torch.equal(d8.view(torch.uint8), dst)


@pytest.mark.parametrize("M,N", [(64, 128), (128, 256), (192, 384), (4096, 2048), (200, 300), (1088, 896), (8192, 4096)])
def test_transpose_eight_byte_elements(mh, M, N):
    """Float64 / Int64 matrices through the 8-byte LDS tile (64 x 128 elements, destination rows first), sizes that are not
    multiples of the tile through interior + strips or the general kernel: both orientations, padded pitches, a batch of
    matrices in one launch; compared as bits; the oracle on the small cases."""
    g = torch.Generator().manual_seed(M * 3 + N)
    src = torch.randint(-2 ** 62, 2 ** 62, (M * N,), dtype=torch.int64, generator=g).cuda()
    dst = torch.zeros(M * N, dtype=torch.int64, device="cuda")
    mh.copyto_(_tens(mh, dst, (M, N), (N, 1)), _tens(mh, src, (M, N), (1, M)))
    torch.cuda.synchronize()
    assert torch.equal(dst.view(M, N), src.view(N, M).t())
    if M * N <= 128 * 256:
        s = to.Array(src.cpu().numpy(), lo.make_layout((M, N), (1, M)))
        d = to.Array(np.zeros(M * N, np.int64), lo.make_layout((M, N), (N, 1)))
        to.copyto(d, s)
        assert np.array_equal(d.buf, dst.cpu().numpy())
    # the other orientation with padded pitches (multiples of 16 bytes), as Float64
    lds, ldd = N + 2, M + 6
    src2 = torch.randn(M * lds, dtype=torch.float64, generator=g).cuda()
    dst2 = torch.full((N * ldd,), -1.0, dtype=torch.float64, device="cuda")
    mh.copyto_(_tens(mh, dst2, (M, N), (1, ldd)), _tens(mh, src2, (M, N), (lds, 1)))
    torch.cuda.synchronize()
    assert torch.equal(dst2.view(N, ldd)[:, :M], src2.view(M, lds)[:, :N].t())
    assert bool((dst2.view(N, ldd)[:, M:] == -1.0).all())
    # a batch of three such matrices: one launch when they are whole tiles
    if M <= 4096:
        B = 3
        src3 = torch.randint(-2 ** 62, 2 ** 62, (B, N, M), dtype=torch.int64, generator=g).cuda()      # [b][n][m]: m contiguous
        dst3 = torch.zeros(B, M, N, dtype=torch.int64, device="cuda")                                  # [b][m][n]: n contiguous
        mh.copyto_(_tens(mh, dst3, (M, N, B), (N, 1, M * N)), _tens(mh, src3, (M, N, B), (1, M, M * N)))
        torch.cuda.synchronize()
        assert torch.equal(dst3, src3.transpose(1, 2))


@pytest.mark.parametrize("pair", ["float32->float16", "float16->float32", "float32->bfloat16", "bfloat16->float16", "float16->float8_e4m3fn",
                                  "float8_e4m3fn->float32", "float64->float16", "float32->float64", "float64->float8_e4m3fn", "float8_e4m3fn->bfloat16"])
def test_transpose_that_converts(mh, pair):
    """copyto! between matrices of different floating-point types whose unit strides lie on different modes: whole tiles
    through the LDS kernel that converts on the way, other sizes as interior + strips, both orientations, padded pitches.
    Bit for bit what the library's dense conversion makes of the transposed source (that conversion is pinned against the
    oracle elsewhere), values that round differently in every target among them; the frame of the destination untouched."""
    sname, dname = pair.split("->")
    sdt, ddt = getattr(torch, sname), getattr(torch, dname)
    g = torch.Generator().manual_seed(len(pair) * 7)
    bits = {1: torch.uint8, 2: torch.int16, 4: torch.int32, 8: torch.int64}

    def dense(x):       # the library's conversion of a contiguous array
        out = torch.zeros(x.shape, dtype=ddt, device="cuda")
        mh.copyto_(_tens(mh, out, (x.numel(),), (1,)), _tens(mh, x.contiguous(), (x.numel(),), (1,)))
        torch.cuda.synchronize()
        return out

    for (M, N) in ((128, 256), (256, 512), (1024, 768), (200, 300), (1088, 784), (4096, 2048)):
        vals = (torch.randn(M, N, generator=g, dtype=torch.float64) * 3).to(torch.float32)
        vals[0, :8] = torch.tensor([0.0, -0.0, 1e-8, 65520.0, -70000.0, 448.0, 464.0, float("inf")])
        src = vals.to(sdt).cuda()                                   # (M, N) row-major: N contiguous
        lds, ldd = N + 16, M + 32
        sbuf = torch.zeros(M, lds, dtype=sdt, device="cuda")
        sbuf[:, :N] = src
        dbuf = torch.full((N, ldd), 3.0, device="cuda").to(ddt)     # destination (M, N) with M contiguous: stored as (N, ldd)
        mh.copyto_(_tens(mh, dbuf, (M, N), (1, ldd)), _tens(mh, sbuf, (M, N), (lds, 1)))
        torch.cuda.synchronize()
        want = dense(src.t())
        assert torch.equal(dbuf[:, :M].contiguous().view(bits[ddt.itemsize]), want.view(bits[ddt.itemsize])), (pair, M, N)
        assert bool((dbuf[:, M:].float() == 3.0).all()), "stores outside the destination"
        # the other orientation: source with M contiguous, destination row-major
        s2 = src.t().contiguous()                                   # stored (N, M): element (m, n) at n * M + m
        d2 = torch.zeros(M, N, dtype=ddt, device="cuda")
        mh.copyto_(_tens(mh, d2, (M, N), (N, 1)), _tens(mh, s2, (M, N), (1, M)))
        torch.cuda.synchronize()
        assert torch.equal(d2.view(bits[ddt.itemsize]), dense(src).view(bits[ddt.itemsize])), (pair, M, N, "other orientation")


@pytest.mark.parametrize("pair", ["float32->float16", "float16->float32", "bfloat16->float8_e4m3fn", "float64->float32"])
def test_permutations_that_convert(mh, pair):
    """Rank-4 permutations between arrays of different floating-point types: modes merged, then a batch of converting
    transposes in one launch where the matrices are whole tiles (NCHW -> NHWC), counted by two modes ([B, S, H, D] ->
    [B, H, D, S]), the general kernel otherwise.  Bit for bit the library's dense conversion of torch's permuted source."""
    sname, dname = pair.split("->")
    sdt, ddt = getattr(torch, sname), getattr(torch, dname)
    g = torch.Generator().manual_seed(len(pair))
    bits = {1: torch.uint8, 2: torch.int16, 4: torch.int32, 8: torch.int64}[ddt.itemsize]

    def dense(x):
        out = torch.zeros(x.shape, dtype=ddt, device="cuda")
        mh.copyto_(_tens(mh, out, (x.numel(),), (1,)), _tens(mh, x.contiguous(), (x.numel(),), (1,)))
        torch.cuda.synchronize()
        return out

    def check(shape, perm):
        x = (torch.randn(*shape, generator=g) * 4).to(sdt).cuda()
        view = x.permute(*perm)
        want = dense(view.contiguous())
        dst = torch.zeros(want.shape, dtype=ddt, device="cuda")
        lshape = tuple(reversed(want.shape))
        mh.copyto_(_tens(mh, dst, lshape, tuple(reversed(dst.stride()))), _tens(mh, x, lshape, tuple(reversed(view.stride()))))
        torch.cuda.synchronize()
        assert torch.equal(dst.view(bits), want.view(bits)), (pair, shape, perm)

    check((3, 256, 16, 16), (0, 2, 3, 1))      # NCHW -> NHWC, H W = 256
    check((3, 16, 16, 256), (0, 3, 1, 2))      # NHWC -> NCHW
    check((2, 128, 14, 14), (0, 2, 3, 1))      # H W = 196: not whole tiles
    check((2, 256, 3, 128), (0, 2, 3, 1))      # [B, S, H, D] -> [B, H, D, S]
    check((2, 256, 3, 128), (0, 2, 1, 3))      # rows move


@pytest.mark.parametrize("dt", ["uint8", "float16", "float32", "float64"])
def test_permutations_that_are_batches_of_transposes(mh, dt):
    """Rank-4 permutations whose modes merge into a batch of matrices (NCHW <-> NHWC: H and W are neighbours in memory on
    both sides) or that count matrices in two modes ([B, S, H, D] -> [B, H, D, S]); one launch each where the matrices are
    whole tiles, the rank-2 route per matrix otherwise.  Against torch's permute, as bits."""
    tdt = getattr(torch, dt)
    g = torch.Generator().manual_seed(41)

    def rand(*shape):
        n = int(np.prod(shape))
        return torch.randint(0, 256, (n * tdt.itemsize,), dtype=torch.uint8, generator=g).view(tdt).view(*shape).cuda()

    def check(x, perm):
        view = x.permute(*perm)
        want = view.contiguous()
        dst = torch.zeros_like(want)
        shape = tuple(reversed(want.shape))
        mh.copyto_(_tens(mh, dst, shape, tuple(reversed(dst.stride()))), _tens(mh, x, shape, tuple(reversed(view.stride()))))
        torch.cuda.synchronize()
        bits = {1: torch.uint8, 2: torch.int16, 4: torch.int32, 8: torch.int64}[tdt.itemsize]
        assert torch.equal(dst.view(bits), want.view(bits)), (dt, tuple(x.shape), perm)

    x = rand(3, 256, 16, 16)          # NCHW, H W = 256: whole tiles for every element size
    check(x, (0, 2, 3, 1))
    check(x.permute(0, 2, 3, 1).contiguous(), (0, 3, 1, 2))
    x = rand(2, 128, 14, 14)          # H W = 196: ragged matrices
    check(x, (0, 2, 3, 1))
    check(x.permute(0, 2, 3, 1).contiguous(), (0, 3, 1, 2))
    x = rand(2, 256, 3, 128)          # [B, S, H, D] -> [B, H, D, S]: matrices D x S, counted by H and B
    check(x, (0, 2, 3, 1))
    check(x, (0, 2, 1, 3))            # [B, H, S, D]: rows move, nothing is transposed
    x = rand(2, 1, 256, 1, 128)       # modes of extent 1 in between
    check(x, (0, 1, 3, 4, 2))
    x = rand(2, 3, 2, 64, 256)        # three modes that count matrices: not one launch
    check(x, (0, 1, 2, 4, 3))


@pytest.mark.parametrize("dt", ["uint8", "float16", "float32", "int64"])
def test_same_shape_copies_whatever_the_order_of_the_modes(mh, dt):
    """Arrays of one shape whose unit stride sits on the last or the middle mode (row-major with a pitch, a batch of
    padded matrices, permuted rank-3 strides, a source one element off alignment): the library is free to visit the
    coordinates in the order that suits the strides; the result is the element loop's (torch.as_strided + copy_)."""
    tdt = getattr(torch, dt)
    g = torch.Generator().manual_seed(29)

    def rand(n):
        return torch.randint(0, 256, (n * tdt.itemsize,), dtype=torch.uint8, generator=g).view(tdt)

    cases = [
        # shape, dst strides, src strides, dst offset, src offset
        ((96, 200), (256, 1), (208, 1), 0, 0),
        ((96, 200), (256, 1), (208, 1), 0, 1),
        ((96, 200), (1, 96), (208, 1), 0, 0),
        ((5, 24, 64), (24 * 64, 64, 1), (32 * 80, 80, 1), 0, 0),
        ((5, 24, 64), (64, 5 * 64, 1), (1, 5, 120), 0, 0),
        ((16, 3, 40), (1, 16 * 40, 16), (3 * 48, 48, 1), 8, 16),
        ((7, 1, 33), (33, 0, 1), (1, 0, 7), 0, 0),
    ]
    for shape, dstr, sstr, doff, soff in cases:
        extent = lambda st, off: off + 1 + sum((n - 1) * s for n, s in zip(shape, st))
        src, dst0 = rand(extent(sstr, soff)), rand(extent(dstr, doff))
        want = dst0.clone()
        torch.as_strided(want, shape, dstr, doff).copy_(torch.as_strided(src, shape, sstr, soff))
        s_d, d_d = src.cuda(), dst0.cuda()
        mh.copyto_(_tens(mh, d_d[doff:], shape, dstr), _tens(mh, s_d[soff:], shape, sstr))
        torch.cuda.synchronize()
        assert torch.equal(d_d.cpu().view(torch.uint8), want.view(torch.uint8)), (shape, dstr, sstr, doff, soff)
        # with a mask of the same shape in an order of its own
        mask = (torch.rand(shape, generator=g) < 0.5).to(torch.uint8)
        want = dst0.clone()
        wv, sv = torch.as_strided(want, shape, dstr, doff), torch.as_strided(src, shape, sstr, soff)
        wv[mask.bool()] = sv[mask.bool()]
        m_d, d_d = mask.cuda(), dst0.cuda()
        mh.copyto_if_(_tens(mh, d_d[doff:], shape, dstr), _tens(mh, s_d[soff:], shape, sstr), _tens(mh, m_d, shape, tuple(mask.stride())))
        torch.cuda.synchronize()
        assert torch.equal(d_d.cpu().view(torch.uint8), want.view(torch.uint8)), ("masked", shape, dstr, sstr)


@pytest.mark.parametrize("dt", ["float32", "float16"])
def test_elementwise_on_arrays_with_the_unit_stride_on_a_later_mode(mh, dt):
    """axpby!, map! and fill! over row-major arrays with a pitch and over a rank-3 array with permuted strides give
    the bits of the same operation on dense copies, and leave the padding alone."""
    tdt = getattr(torch, dt)
    itype = {2: torch.int16, 4: torch.int32}[tdt.itemsize]
    g = torch.Generator().manual_seed(41)
    cases = [((96, 200), (256, 1), (208, 1)), ((5, 24, 64), (64, 5 * 64, 1), (1, 5, 120)), ((96, 200), (1, 96), (208, 1))]
    for shape, ystr, xstr in cases:
        n = int(np.prod(shape))
        extent = lambda st: 1 + sum((k - 1) * s for k, s in zip(shape, st))
        X, Y = (torch.randn(extent(xstr), generator=g) * 3).to(tdt), (torch.randn(extent(ystr), generator=g) * 3).to(tdt)
        xv, yv = torch.as_strided(X, shape, xstr), torch.as_strided(Y, shape, ystr)
        # dense copies in the order of the logical index (first mode fastest)
        order = tuple(reversed(range(len(shape))))
        xd, yd = xv.permute(order).contiguous().cuda(), yv.permute(order).contiguous().cuda()
        flat = lambda t: _tens(mh, t, [n], [1])
        yd1 = yd.clone()
        mh.axpby_(0.75, flat(xd), -1.25, flat(yd1))
        xs, ys = X.cuda(), Y.cuda()
        mh.axpby_(0.75, _tens(mh, xs, shape, xstr), -1.25, _tens(mh, ys, shape, ystr))
        torch.cuda.synchronize()
        want = Y.clone()
        torch.as_strided(want, shape, ystr).copy_(yd1.cpu().permute(order))
        assert torch.equal(ys.cpu().view(itype), want.view(itype)), ("axpby", shape, ystr, xstr)
        for second in ("array", "scalar"):
            dd = torch.zeros(n, dtype=tdt, device="cuda")
            mh.map_("mul", flat(dd), flat(xd), flat(yd) if second == "array" else None, 1.75)
            D = torch.full((extent(ystr),), 7.0, dtype=tdt)
            ds = D.cuda()
            y2 = Y.cuda()
            mh.map_("mul", _tens(mh, ds, shape, ystr), _tens(mh, xs, shape, xstr), _tens(mh, y2, shape, ystr) if second == "array" else None, 1.75)
            torch.cuda.synchronize()
            want = D.clone()
            torch.as_strided(want, shape, ystr).copy_(dd.cpu().reshape(tuple(reversed(shape))).permute(order))
            assert torch.equal(ds.cpu().view(itype), want.view(itype)), ("map", second, shape, ystr, xstr)
        F = torch.full((extent(ystr),), 7.0, dtype=tdt)
        fs = F.cuda()
        mh.fill_(_tens(mh, fs, shape, ystr), 2.5)
        torch.cuda.synchronize()
        want = F.clone()
        torch.as_strided(want, shape, ystr).fill_(2.5)
        assert torch.equal(fs.cpu(), want), ("fill", shape, ystr)


@pytest.mark.parametrize("dt", ["uint8", "float16", "float32"])
def test_batches_of_transposes(mh, dt):
    """Rank-3 and rank-4 arrays whose two sides have their unit strides on different modes: every other mode counts
    matrices, and each matrix goes through the tiled transpose (whole tiles, ragged edges, padded pitches).  Checked
    against the element loop (torch.as_strided + copy_), padding included."""
    tdt = getattr(torch, dt)
    g = torch.Generator().manual_seed(53)

    def rand(n):
        return torch.randint(0, 256, (n * tdt.itemsize,), dtype=torch.uint8, generator=g).view(tdt)

    M, N = 512, 320
    cases = [
        # shape, dst strides, src strides
        ((3, M, N), (M * N, N, 1), (M * N, 1, M)),                      # batch first
        ((M, N, 3), (N, 1, M * N), (1, M, M * N)),                      # batch last
        ((M, 2, N), (2 * N, N, 1), (1, M * N, M)),                      # batch in the middle, interleaved rows on one side
        ((2, M + 8, N + 16), ((M + 8) * (N + 32), N + 32, 1), ((M + 16) * (N + 16), 1, M + 16)),   # ragged sizes, padded pitches
        ((2, M, 3, N), (3 * M * N, N, M * N, 1), (3 * M * N, 1, M * N, M)),                       # two batch modes
    ]
    for shape, dstr, sstr in cases:
        extent = lambda st: 1 + sum((k - 1) * s for k, s in zip(shape, st))
        src, dst0 = rand(extent(sstr)), rand(extent(dstr))
        want = dst0.clone()
        torch.as_strided(want, shape, dstr).copy_(torch.as_strided(src, shape, sstr))
        s_d, d_d = src.cuda(), dst0.cuda()
        mh.copyto_(_tens(mh, d_d, shape, dstr), _tens(mh, s_d, shape, sstr))
        torch.cuda.synchronize()
        assert torch.equal(d_d.cpu().view(torch.uint8), want.view(torch.uint8)), (shape, dstr, sstr)


@pytest.mark.parametrize("tiler", [(32, 32), (64, 64), (16, 128), (8, 8), (0, 0)])
def test_lds_tiled_copy_takes_any_tiler_that_divides(mh, tiler):
    """The reference's own transpose kernel tiles 32 x 32 with 256 threads (test/host/copy_async.jl:51-76): the tiler
    of the descriptor only has to divide the array; closed form dst[j, i] == src[i, j] bit for bit, for sizes that are
    whole 64 x 64 patches, sizes that leave strips, and an array smaller than a patch."""
    for (M, N) in ((2048, 4096), (4096, 2048), (96, 160), (32, 32), (2048 + 32, 2048)):
        if tiler[0] and (M % tiler[0] or N % tiler[1]):
            continue
        src = _rand_bits(M * N, 31 + M)
        dst = torch.zeros_like(src)
        tc = mh.tiled_copy_desc(op=mh.COPY_LDS_TILED, vec_bits=128, thr_shape=(32, 8), val_shape=(1, 1), tiler=tiler)
        mh.copyto_(_tens(mh, dst, (M, N), (N, 1)), _tens(mh, src, (M, N), (1, M)), tc)
        torch.cuda.synchronize()
        assert torch.equal(dst.view(M, N), src.view(N, M).t()), (M, N, tiler)
    if tiler[0] > 8:
        src = _rand_bits(24 * 24, 5)
        with pytest.raises(mh.MoyeError) as e:
            mh.copyto_(_tens(mh, torch.zeros_like(src), (24, 24), (24, 1)), _tens(mh, src, (24, 24), (1, 24)),
                       mh.tiled_copy_desc(op=mh.COPY_LDS_TILED, tiler=tiler))
        assert e.value.status == mh._lib.ERR_SHAPE


def test_transpose_destination_rows_first_and_source_first_agree(mh):
    """Large matrices take the kernel that completes destination rows first, matrices whose destination rows are the
    longer side the one that walks the source first: both against the closed form, bit for bit, on shapes either side
    of the rule, and on a batch."""
    for (ni, nj) in ((4096, 2048), (2048, 4096), (2048, 2048), (8192, 1024), (1024, 8192), (2304, 2304)):
        src = _rand_bits(ni * nj, ni + nj)
        dst = torch.zeros_like(src)
        mh.copyto_(_tens(mh, dst, (ni, nj), (nj, 1)), _tens(mh, src, (ni, nj), (1, ni)))
        torch.cuda.synchronize()
        assert torch.equal(dst.view(ni, nj), src.view(nj, ni).t()), (ni, nj)
    for (ni, nj) in ((4096, 3072), (3072, 4096), (3072, 3072), (2048, 2048)):      # the same for 2-byte elements
        src = _rand_bits(ni * nj, ni + nj).to(torch.int16)
        dst = torch.zeros_like(src)
        mh.copyto_(_tens(mh, dst, (ni, nj), (nj, 1)), _tens(mh, src, (ni, nj), (1, ni)))
        torch.cuda.synchronize()
        assert torch.equal(dst.view(ni, nj), src.view(nj, ni).t()), (ni, nj, "int16")
    ni = nj = 2048
    src = _rand_bits(ni * nj * 3, 77)
    dst = torch.zeros_like(src)
    mh.copyto_(_tens(mh, dst, (ni, nj, 3), (nj, 1, ni * nj)), _tens(mh, src, (ni, nj, 3), (1, ni, ni * nj)))
    torch.cuda.synchronize()
    assert torch.equal(dst.view(3, ni, nj), src.view(3, nj, ni).transpose(1, 2))


def test_more_than_16_gib_in_one_call(mh):
    """Arrays of more than 2^30 16-byte pieces: the kernels that give every lane one piece then spread their workgroups
    over two grid dimensions (a launch holds fewer than 2^32 work-items per dimension).  fill!, a plain copy, a
    converting copy and axpby! on 17 GiB arrays; every byte checked on the device."""
    free, _ = torch.cuda.mem_get_info()
    if free < 60 * 2 ** 30:
        pytest.skip("needs 60 GiB of free device memory")
    cols = 1 << 20
    rows = 17 * 256 + 3                                   # 17 GiB of int32 and a little more
    n = rows * cols
    x = torch.empty(n, dtype=torch.int32, device="cuda")
    mh.fill_(_tens(mh, x, [n], [1]), 0x01020304)
    torch.cuda.synchronize()
    assert bool((x.view(rows, cols) == 0x01020304).all())
    pat = torch.arange(cols, dtype=torch.int32, device="cuda")
    for r0 in range(0, rows, 512):                        # row r holds (column index) * 3 + r
        r1 = min(rows, r0 + 512)
        x.view(rows, cols)[r0:r1] = pat[None, :] * 3 + torch.arange(r0, r1, dtype=torch.int32, device="cuda")[:, None]
    y = torch.zeros(n, dtype=torch.int32, device="cuda")
    mh.copyto_(_tens(mh, y, [n], [1]), _tens(mh, x, [n], [1]))
    torch.cuda.synchronize()
    assert torch.equal(x, y)
    # axpby! on the same bytes as fp32 values (small integers, exact): y = 2 x + y
    xf, yf = x.view(torch.float32), y.view(torch.float32)
    xf.view(rows, cols)[:] = pat[None, :].float() % 1024
    yf.view(rows, cols)[:] = 1.0
    mh.axpby_(2.0, _tens(mh, xf, [n], [1]), 1.0, _tens(mh, yf, [n], [1]))
    torch.cuda.synchronize()
    assert bool((yf.view(rows, cols) == 2 * (pat[None, :].float() % 1024) + 1).all())
    del y, yf
    # a narrowing conversion: fp32 -> fp16, 2^30 and more pieces on the fp32 side
    h = torch.zeros(n, dtype=torch.float16, device="cuda")
    mh.copyto_(_tens(mh, h, [n], [1]), _tens(mh, xf, [n], [1]))
    torch.cuda.synchronize()
    assert bool((h.view(rows, cols) == (pat[None, :] % 1024).half()).all())

"""GPU parity of gemm! through the C ABI (moye_gemm).

UniversalFMA atom: bit-exact against the CPU restatement of the reference's arithmetic
(oracle/tiled_oracle.py::gemm_universal_fma) — the tolerance is zero.
MFMA atoms: norm-wise relative error  max|C - C64| / max|C64|  against an fp64 product of the
same rounded inputs, tolerance 1e-2 for f16/bf16/fp8 inputs and 1e-5 for fp32, with the error of
the reference's own arithmetic printed alongside."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

import tiled_oracle as to  # noqa: E402

TOL16 = 1e-2
TOL32 = 1e-5


@pytest.fixture(scope="module")
def mh():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    import moye_hip
    return moye_hip


def T(t, shape=None, stride=None):
    from moye_hip.torch_interop import tensor_of
    return tensor_of(t, shape, stride)


def kernels_of(mh, mma, d, a, b, c=None, ep=None):
    """The kernel steps of the plan the library makes for this call (moye_gemm_explain): what a test that means a
    specific kernel instance asserts, so that a changed threshold cannot leave the instance untested while all stays green."""
    return [s for s in mh.gemm_explain(mma, d, a, b, c, ep)["steps"] if s["what"] == "kernel"]


def relerr(c, c64):
    c64 = c64.double()
    return float((c.double() - c64).abs().max() / c64.abs().max())


# ---------------------------------------------------------------------------------------------
# UniversalFMA: exact
# ---------------------------------------------------------------------------------------------

def test_config1_fp32_256_nn_bit_exact(mh):
    """Benchmark configuration 1: fp32 C = A*B, M=N=K=256, A and B column-major, 32x32x8 tiles."""
    rng = np.random.default_rng(1001)
    M = N = K = 256
    A = (rng.random((M, K), dtype=np.float32) * 2 - 1)           # A[m,k]
    Bkn = (rng.random((K, N), dtype=np.float32) * 2 - 1)         # B[k,n]
    a = torch.from_numpy(np.asfortranarray(A).reshape(-1, order="F").copy()).cuda()    # column-major storage
    b = torch.from_numpy(np.asfortranarray(Bkn).reshape(-1, order="F").copy()).cuda()
    c = torch.zeros(M * N, dtype=torch.float32, device="cuda")
    mma = mh.tiled_mma_desc(mh.MMA_UNIVERSAL_FMA, cta_tile=(32, 32, 8))
    # MoYe operands: A (M,K):(1,M); B as (N,K):(K,1); C (M,N):(1,M)
    mh.gemm_(mma, T(c, (M, N), (1, M)), T(a, (M, K), (1, M)), T(b, (N, K), (K, 1)), T(c, (M, N), (1, M)))
    torch.cuda.synchronize()
    got = c.cpu().numpy().reshape(N, M).T
    want = to.gemm_universal_fma(A, Bkn.T.copy(), np.zeros((M, N), np.float32))
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    c64 = A.astype(np.float64) @ Bkn.astype(np.float64)
    err = to.relerr(got, c64)
    print("config1 fp32 256^3: rel err vs fp64 = %.3e (reference arithmetic: identical)" % err)
    assert err <= TOL32
    # every built tiling gives the same bits
    for tile in ((64, 64, 8), (128, 128, 8)):
        c2 = torch.zeros_like(c)
        mh.gemm_(mh.tiled_mma_desc(mh.MMA_UNIVERSAL_FMA, cta_tile=tile), T(c2, (M, N), (1, M)),
                 T(a, (M, K), (1, M)), T(b, (N, K), (K, 1)))
        torch.cuda.synchronize()
        assert torch.equal(c2, c)


@pytest.mark.parametrize("dt", ["f16", "bf16", "f32"])
def test_universal_fma_ragged_bit_exact(mh, dt):
    """Odd sizes, K-major operands, C accumulated: product rounded in the input type (f16/bf16),
    unfused fp32 add, k ascending."""
    rng = np.random.default_rng(5)
    M, N, K = 70, 45, 37
    tdt = {"f16": torch.float16, "bf16": torch.bfloat16, "f32": torch.float32}[dt]
    A = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(tdt)
    B = torch.from_numpy(rng.standard_normal((N, K)).astype(np.float32)).to(tdt)
    C0 = torch.from_numpy(rng.standard_normal((M, N)).astype(np.float32))
    a, b, c = A.cuda(), B.cuda(), C0.cuda()
    d = torch.zeros(M, N, dtype=torch.float32, device="cuda")
    mh.gemm_(mh.tiled_mma_desc(mh.MMA_UNIVERSAL_FMA), T(d), T(a), T(b), T(c))
    torch.cuda.synchronize()
    want = to.gemm_universal_fma(A.float().numpy(), B.float().numpy(), C0.numpy(), dt, dt)
    assert np.array_equal(d.cpu().numpy().view(np.uint32), want.view(np.uint32))


def test_universal_fma_matches_reference_device_test_shape(mh):
    """test/device/matmul.jl:75-81 — C = A*B' with A:(2048,256), B:(2048,256) column-major."""
    rng = np.random.default_rng(6)
    M = N = 2048
    K = 256
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = rng.standard_normal((N, K)).astype(np.float32)
    a = torch.from_numpy(A.reshape(-1, order="F").copy()).cuda()
    b = torch.from_numpy(B.reshape(-1, order="F").copy()).cuda()
    c = torch.zeros(M * N, dtype=torch.float32, device="cuda")
    mh.gemm_(mh.tiled_mma_desc(mh.MMA_UNIVERSAL_FMA, cta_tile=(128, 128, 8)), T(c, (M, N), (1, M)),
             T(a, (M, K), (1, M)), T(b, (N, K), (1, N)))
    torch.cuda.synchronize()
    got = c.cpu().numpy().reshape(N, M).T
    rows = rng.choice(M, 48, replace=False)
    want = to.gemm_universal_fma(A[rows], B, np.zeros((len(rows), N), np.float32))
    assert np.array_equal(got[rows].view(np.uint32), want.view(np.uint32))


# ---------------------------------------------------------------------------------------------
# MFMA kernels: tolerance against fp64
# ---------------------------------------------------------------------------------------------

def _mfma_case(mh, atom, tdt, out_dt, M, N, K, seed, scale, cta=(128, 128, 0), col_major_d=False, with_c=False,
               alpha=1.0):
    g = torch.Generator().manual_seed(seed)
    A = (torch.randn(M, K, generator=g) * scale).to(tdt)
    B = (torch.randn(N, K, generator=g) * scale).to(tdt)
    a, b = A.cuda(), B.cuda()
    if col_major_d:
        d = torch.zeros(N, M, dtype=out_dt, device="cuda")
        dd = T(d, (M, N), (1, M))
    else:
        d = torch.zeros(M, N, dtype=out_dt, device="cuda")
        dd = T(d)
    cc, C0 = None, None
    if with_c:
        C0 = torch.randn(M, N, generator=g).to(out_dt)
        c = C0.cuda()
        cc = T(c)
    mh.gemm_(mh.tiled_mma_desc(atom, atom_layout=(2, 2, 1), cta_tile=cta), dd, T(a), T(b), cc, alpha)
    torch.cuda.synchronize()
    got = d.t() if col_major_d else d
    c64 = alpha * (a.double() @ b.double().t())
    if with_c:
        c64 = c64 + C0.cuda().double()
    return got, c64, A, B


@pytest.mark.parametrize("bk", [32, 64])
@pytest.mark.parametrize("M,N,K", [(128, 128, 64), (256, 384, 512), (512, 256, 1024)])
def test_f16_tn_small(mh, M, N, K, bk):
    got, c64, A, B = _mfma_case(mh, mh.MFMA_F32_16x16x32_F16, torch.float16, torch.float16, M, N, K, 3,
                                K ** -0.5, cta=(128, 128, bk))
    err = relerr(got, c64)
    # the reference's own arithmetic (16-bit rounded products, sequential fp32 sum), fp16 output
    ref = to.gemm_universal_fma(A.float().numpy(), B.float().numpy(), np.zeros((M, N), np.float32), "f16", "f16")
    ref_err = to.relerr(ref.astype(np.float16), c64.cpu().numpy())
    print("f16 %dx%dx%d bk=%d: rel err %.3e (reference arithmetic %.3e)" % (M, N, K, bk, err, ref_err))
    assert err <= TOL16
    # cross-check the GPU fp64 oracle against numpy on the host
    c64_host = A.double().numpy() @ B.double().numpy().T
    assert np.allclose(c64.cpu().numpy(), c64_host, rtol=1e-12, atol=1e-12)


def test_f16_tn_exact_on_integers(mh):
    """Small-integer inputs make every product and partial sum exact in fp32, so any indexing
    mistake (wrong k pairing, transposed tile, swapped fragment) shows as a hard mismatch."""
    M, N, K = 256, 256, 256
    g = torch.Generator().manual_seed(8)
    A = torch.randint(-4, 5, (M, K), generator=g).to(torch.float16)
    B = torch.randint(-4, 5, (N, K), generator=g).to(torch.float16)
    a, b = A.cuda(), B.cuda()
    for out_dt in (torch.float32, torch.float16):
        d = torch.zeros(M, N, dtype=out_dt, device="cuda")
        mh.gemm_(mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, cta_tile=(128, 128, 32)), T(d), T(a), T(b))
        torch.cuda.synchronize()
        want = (A.double() @ B.double().t())
        assert torch.equal(d.cpu().double(), want)


def test_f16_variants(mh):
    """column-major D, C accumulation, alpha, fp32 output."""
    for kw in (dict(col_major_d=True), dict(with_c=True), dict(with_c=True, alpha=0.5, col_major_d=True)):
        for out_dt in (torch.float16, torch.float32):
            got, c64, _, _ = _mfma_case(mh, mh.MFMA_F32_16x16x32_F16, torch.float16, out_dt, 256, 128, 256, 4,
                                        1 / 16, **kw)
            assert relerr(got, c64) <= TOL16, kw


def test_config3_f16_tn_4096(mh):
    """Benchmark configuration 3 at full size: fp16 TN 4096^3, fp32 accumulate, fp16 out, 128x128x32 tile."""
    M = N = K = 4096
    got, c64, A, B = _mfma_case(mh, mh.MFMA_F32_16x16x32_F16, torch.float16, torch.float16, M, N, K, 1003,
                                K ** -0.5, cta=(128, 128, 32))
    err = relerr(got, c64)
    rows = np.random.default_rng(0).choice(M, 64, replace=False)
    host = A[rows].double().numpy() @ B.double().numpy().T
    assert np.allclose(c64[rows].cpu().numpy(), host, rtol=1e-12, atol=1e-12)
    ref = to.gemm_universal_fma(A[rows[:16]].float().numpy(), B.float().numpy(), np.zeros((16, N), np.float32),
                                "f16", "f16").astype(np.float16)
    ref_err = to.relerr(ref, host[:16])
    print("config3 f16 4096^3: rel err %.3e (reference arithmetic on 16 rows: %.3e)" % (err, ref_err))
    assert err <= TOL16


def test_bf16_tn(mh):
    """Benchmark configuration 4 (square), reduced to 1024^3 here; bf16 in, fp32 out, N(0, 0.02)."""
    got, c64, A, B = _mfma_case(mh, mh.MFMA_F32_16x16x32_BF16, torch.bfloat16, torch.float32, 1024, 1024, 1024,
                                1004, 0.02)
    err = relerr(got, c64)
    ref = to.gemm_universal_fma(A[:32].float().numpy(), B.float().numpy(), np.zeros((32, 1024), np.float32),
                                "bf16", "bf16")
    ref_err = to.relerr(ref, c64[:32].cpu().numpy())
    print("bf16 1024^3: rel err %.3e (reference arithmetic on 32 rows: %.3e)" % (err, ref_err))
    assert err <= TOL16


def test_fp8_tn_with_scales(mh):
    """Benchmark configuration 5 reduced to 1024^3: e4m3 inputs quantised per tensor by amax/448, fp32
    accumulate, bf16 out = acc * s_a * s_b."""
    if not hasattr(torch, "float8_e4m3fn"):
        pytest.skip("torch without float8_e4m3fn")
    M = N = K = 1024
    g = torch.Generator().manual_seed(1005)
    X, W = torch.randn(M, K, generator=g), torch.randn(N, K, generator=g)
    sa, sb = float(X.abs().max() / 448), float(W.abs().max() / 448)
    qa, qb = (X / sa).to(torch.float8_e4m3fn), (W / sb).to(torch.float8_e4m3fn)
    a, b = qa.cuda(), qb.cuda()
    d = torch.zeros(M, N, dtype=torch.bfloat16, device="cuda")
    mh.gemm_(mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_FP8, cta_tile=(128, 128, 64)), T(d), T(a), T(b), None, sa * sb)
    torch.cuda.synchronize()
    c64 = (qa.double().cuda() @ qb.double().cuda().t()) * (sa * sb)
    err = relerr(d, c64)
    print("fp8 1024^3: rel err vs fp64 of the quantised inputs %.3e" % err)
    assert err <= TOL16


def test_gemm_errors(mh):
    a = torch.zeros(128, 64, dtype=torch.float16, device="cuda")
    b = torch.zeros(128, 64, dtype=torch.float16, device="cuda")
    d = torch.zeros(128, 128, dtype=torch.float16, device="cuda")
    E = mh._lib
    mma = mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, cta_tile=(128, 128, 32))
    with pytest.raises(mh.MoyeError) as e:  # K mismatch
        mh.gemm_(mma, T(d), T(a), T(b[:, :32]))
    assert e.value.status == E.ERR_SHAPE
    with pytest.raises(mh.MoyeError) as e:  # tile does not divide
        mh.gemm_(mma, T(d[:96]), T(a[:96]), T(b))
    assert e.value.status == E.ERR_SHAPE
    with pytest.raises(mh.MoyeError) as e:  # M-major A is not the TN form, and the workspace is forbidden
        mh.gemm_(mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, cta_tile=(128, 128, 32), flags=E.GEMM_NO_WORKSPACE),
                 T(d), T(a, (128, 64), (1, 128)), T(b))
    assert e.value.status == E.ERR_UNSUPPORTED
    with pytest.raises(mh.MoyeError) as e:  # wrong operand type for the atom
        a32 = a.float()
        mh.gemm_(mma, T(d), T(a32), T(b))
    assert e.value.status == E.ERR_UNSUPPORTED
    with pytest.raises(mh.MoyeError) as e:  # rank
        mh.gemm_(mma, T(d), T(a, (128, 8, 8), (64, 8, 1)), T(b))
    assert e.value.status == E.ERR_RANK


# ---------------------------------------------------------------------------------------------
# 256 x 256 CTA tile schedules (one workgroup per CU)
# ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("waves,stages", [((2, 4, 1), 0), ((2, 2, 1), 0), ((2, 4, 1), 2), ((2, 2, 1), 2), ((2, 4, 1), 4), ((2, 4, 1), 5)])
def test_f16_tn_256_tile_exact_on_integers(mh, waves, stages):
    """Every 256x256 schedule (8 waves, 4 waves; stages 0: the library's choice, the hand-ordered kernel on whole-line
    stages; 2: the compiler-scheduled two-stage kernel; 4- and 5-stage ring) on small-integer inputs:
    all sums are exact in fp32, so the result must equal the integer product exactly."""
    M, N, K = 512, 768, 320
    g = torch.Generator().manual_seed(12)
    A = torch.randint(-4, 5, (M, K), generator=g).to(torch.float16)
    B = torch.randint(-4, 5, (N, K), generator=g).to(torch.float16)
    a, b = A.cuda(), B.cuda()
    bk = 32 if stages >= 3 else 64
    for out_dt in (torch.float32, torch.float16):
        d = torch.zeros(M, N, dtype=out_dt, device="cuda")
        mma = mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, atom_layout=waves, cta_tile=(256, 256, bk), stages=stages)
        mh.gemm_(mma, T(d), T(a), T(b))
        torch.cuda.synchronize()
        assert torch.equal(d.cpu().double(), A.double() @ B.double().t()), (waves, stages, out_dt)


def test_pingpong_schedule_exact_on_integers(mh):
    """MOYE_GEMM_PINGPONG: 64-byte k-tiles in a five-stage ring; K from one k-tile to many (the
    prologue, the steady state and the drain each have their own wait counts), every input type."""
    from moye_hip import _lib
    g = torch.Generator().manual_seed(13)
    cases = [(torch.float16, mh.MFMA_F32_16x16x32_F16, 32), (torch.bfloat16, mh.MFMA_F32_16x16x32_BF16, 32)]
    if hasattr(torch, "float8_e4m3fn"):
        cases.append((torch.float8_e4m3fn, mh.MFMA_F32_16x16x32_FP8, 64))
    for in_dt, atom, bk in cases:
        for (M, N, kt) in ((256, 256, 1), (256, 512, 3), (512, 256, 4), (256, 256, 5), (256, 256, 6), (512, 768, 37)):
            K = kt * bk
            A = torch.randint(-3, 4, (M, K), generator=g).float()
            B = torch.randint(-3, 4, (N, K), generator=g).float()
            C = torch.randint(-8, 9, (M, N), generator=g).float()
            a, b, c = A.to(in_dt).cuda(), B.to(in_dt).cuda(), C.cuda()
            d = torch.zeros(M, N, dtype=torch.float32, device="cuda")
            mma = mh.tiled_mma_desc(atom, atom_layout=(2, 4, 1), cta_tile=(256, 256, bk), flags=_lib.GEMM_PINGPONG)
            mh.gemm_(mma, T(d), T(a), T(b), T(c), 2.0)
            torch.cuda.synchronize()
            assert torch.equal(d.cpu().double(), 2.0 * (A.double() @ B.double().t()) + C.double()), (in_dt, M, N, K)


def test_pingpong_schedule_random(mh):
    from moye_hip import _lib
    M = N = K = 2048
    g = torch.Generator().manual_seed(14)
    A = (torch.randn(M, K, generator=g) * K ** -0.5).half()
    B = (torch.randn(N, K, generator=g) * K ** -0.5).half()
    a, b = A.cuda(), B.cuda()
    d = torch.zeros(M, N, dtype=torch.float16, device="cuda")
    d2 = torch.zeros(M, N, dtype=torch.float16, device="cuda")
    mh.gemm_(mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, atom_layout=(2, 4, 1), cta_tile=(256, 256, 32),
                               flags=_lib.GEMM_PINGPONG), T(d), T(a), T(b))
    mh.gemm_(mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, atom_layout=(2, 4, 1), cta_tile=(256, 256, 64)), T(d2), T(a), T(b))
    torch.cuda.synchronize()
    c64 = a.double() @ b.double().t()
    assert relerr(d, c64) <= TOL16
    # both schedules add the same products in the same k order within a lane
    assert torch.equal(d, d2)


@pytest.mark.parametrize("waves", [(2, 2, 1), (2, 4, 1)])
def test_wave4_schedule_exact_on_integers(mh, waves):
    """MOYE_GEMM_WAVE4: four waves with 128x128 wave tiles or eight with 128x64, fragments refilled in
    place, hand-placed waits.  Small integers make every sum exact, so any fragment read too early, any stage
    overwritten too soon or any misplaced accumulator shows as a wrong integer.  K from one
    k-step to many: the prologue, the steady state and the drain each have their own wait counts."""
    from moye_hip import _lib
    g = torch.Generator().manual_seed(17)
    cases = [(torch.float16, mh.MFMA_F32_16x16x32_F16, 32), (torch.bfloat16, mh.MFMA_F32_16x16x32_BF16, 32),
             (torch.float32, mh.MFMA_F32_16x16x4_F32, 16), (torch.float32, mh.MFMA_F32_16x16x4_F32, 32),
             # the 16-bit types with k-steps of two stages (two MFMAs in a row per accumulator)
             (torch.float16, mh.MFMA_F32_16x16x32_F16, 64), (torch.bfloat16, mh.MFMA_F32_16x16x32_BF16, 64)]
    if hasattr(torch, "float8_e4m3fn"):
        cases.append((torch.float8_e4m3fn, mh.MFMA_F32_16x16x32_FP8, 128))
    for in_dt, atom, bk in cases:
        for (M, N, kt) in ((256, 256, 1), (256, 512, 2), (512, 256, 3), (256, 256, 4), (256, 256, 5), (256, 256, 6),
                           (256, 256, 7), (512, 768, 37)):
            K = kt * bk
            A = torch.randint(-3, 4, (M, K), generator=g).float()
            B = torch.randint(-3, 4, (N, K), generator=g).float()
            C = torch.randint(-8, 9, (M, N), generator=g).float()
            a, b, c = A.to(in_dt).cuda(), B.to(in_dt).cuda(), C.cuda()
            # stages 0: k-steps of 128 bytes run on two whole-line stages; 5: on the ring of five 64-byte-row stages
            for stages in ((0, 5) if bk * a.element_size() == 128 else (0,)):
                d = torch.zeros(M, N, dtype=torch.float32, device="cuda")
                mma = mh.tiled_mma_desc(atom, atom_layout=waves, cta_tile=(256, 256, bk), stages=stages, flags=_lib.GEMM_WAVE4)
                print("wave4", waves, in_dt, M, N, K, stages, flush=True)
                mh.gemm_(mma, T(d), T(a), T(b), T(c), 2.0)
                torch.cuda.synchronize()
                assert torch.equal(d.cpu().double(), 2.0 * (A.double() @ B.double().t()) + C.double()), (in_dt, M, N, K, stages)


def test_hand_ordered_128_tile_exact_on_integers(mh):
    """The 128x128 instance of the hand-ordered kernel: plain f16 / bf16 calls with more tiles than CUs (17 x 17 here) and
    every plain fp8 and fp32 call on whole 128x128 tiles.  K from one k-step of 128 bytes to many (the prologue, the steady state
    and the drain each have their own wait counts), C with alpha, every output type; exact on small integers."""
    g = torch.Generator().manual_seed(23)
    cases = [(torch.float16, mh.MFMA_F32_16x16x32_F16, 64, 2176, 2176), (torch.bfloat16, mh.MFMA_F32_16x16x32_BF16, 64, 2176, 2304),
             (torch.float32, mh.MFMA_F32_16x16x4_F32, 32, 128, 128), (torch.float32, mh.MFMA_F32_16x16x4_F32, 32, 384, 640)]
    if hasattr(torch, "float8_e4m3fn"):
        cases += [(torch.float8_e4m3fn, mh.MFMA_F32_16x16x32_FP8, 128, 128, 128), (torch.float8_e4m3fn, mh.MFMA_F32_16x16x32_FP8, 128, 384, 640),
                  (torch.float8_e4m3fn, mh.MFMA_F32_16x16x32_FP8, 128, 2176, 2176)]
    for in_dt, atom, bk, M, N in cases:
        for kt in (1, 2, 3, 4, 5, 7, 37):
            if M > 1000 and kt in (4, 5):
                continue
            K = kt * bk
            A = torch.randint(-3, 4, (M, K), generator=g).float()
            B = torch.randint(-3, 4, (N, K), generator=g).float()
            C = torch.randint(-8, 9, (M, N), generator=g).float()
            a, b, c = A.to(in_dt).cuda(), B.to(in_dt).cuda(), C.cuda()
            ref = A.double() @ B.double().t()
            for cta in ((0, 0, 0), (128, 128, bk)):
                d = torch.zeros(M, N, dtype=torch.float32, device="cuda")
                if cta != (0, 0, 0):
                    ks = kernels_of(mh, mh.tiled_mma_desc(atom, atom_layout=(2, 2, 1), cta_tile=cta), T(d), T(a), T(b), T(c))
                    assert len(ks) == 1 and ks[0]["family"] == "gemm_mfma_tn_256_w4" and "tile=128" in ks[0]["name"], ks
                mh.gemm_(mh.tiled_mma_desc(atom, atom_layout=(2, 2, 1), cta_tile=cta), T(d), T(a), T(b), T(c), 2.0)
                torch.cuda.synchronize()
                assert torch.equal(d.cpu().double(), 2.0 * ref + C.double()), (in_dt, M, N, K, cta)
            for out_dt in (torch.float16, torch.bfloat16):
                if float(ref.abs().max()) >= (256 if out_dt == torch.bfloat16 else 2048):
                    continue
                d = torch.zeros(M, N, dtype=out_dt, device="cuda")
                mh.gemm_(mh.tiled_mma_desc(atom, atom_layout=(2, 2, 1), cta_tile=(128, 128, bk)), T(d), T(a), T(b))
                torch.cuda.synchronize()
                assert torch.equal(d.cpu().double(), ref), (in_dt, out_dt, M, N, K)


@pytest.mark.parametrize("waves", [(2, 2, 1), (2, 4, 1)])
def test_wave4_schedule_random(mh, waves):
    from moye_hip import _lib
    M = N = K = 2048
    g = torch.Generator().manual_seed(18)
    A = (torch.randn(M, K, generator=g) * K ** -0.5).half()
    B = (torch.randn(N, K, generator=g) * K ** -0.5).half()
    a, b = A.cuda(), B.cuda()
    d = torch.zeros(M, N, dtype=torch.float16, device="cuda")
    d2 = torch.zeros(M, N, dtype=torch.float16, device="cuda")
    mh.gemm_(mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, atom_layout=waves, cta_tile=(256, 256, 32),
                               flags=_lib.GEMM_WAVE4), T(d), T(a), T(b))
    mh.gemm_(mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, atom_layout=(2, 4, 1), cta_tile=(256, 256, 64)), T(d2), T(a), T(b))
    torch.cuda.synchronize()
    c64 = a.double() @ b.double().t()
    assert relerr(d, c64) <= TOL16
    # both schedules add the same products in the same k order within a lane
    assert torch.equal(d, d2)
    if hasattr(torch, "float8_e4m3fn"):
        x = torch.randn(M, K, generator=g)
        w = torch.randn(N, K, generator=g)
        sa, sb = float(x.abs().max()) / 448.0, float(w.abs().max()) / 448.0
        qa, qb = (x / sa).to(torch.float8_e4m3fn).cuda(), (w / sb).to(torch.float8_e4m3fn).cuda()
        o = torch.zeros(M, N, dtype=torch.bfloat16, device="cuda")
        mh.gemm_(mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_FP8, atom_layout=waves, cta_tile=(256, 256, 128),
                                   flags=_lib.GEMM_WAVE4), T(o), T(qa), T(qb), None, sa * sb)
        torch.cuda.synchronize()
        c64 = (qa.double() @ qb.double().t()) * (sa * sb)
        assert relerr(o, c64) <= TOL16


@pytest.mark.parametrize("tdt,atom", [("float16", "MFMA_F32_16x16x32_F16"), ("bfloat16", "MFMA_F32_16x16x32_BF16")])
def test_256_tile_variants(mh, tdt, atom):
    """column-major D, C accumulation and alpha through the 256x256 kernel; one k-tile and many."""
    tdt = getattr(torch, tdt)
    for K in (64, 1024):
        for kw in (dict(), dict(col_major_d=True), dict(with_c=True, alpha=0.5)):
            got, c64, _, _ = _mfma_case(mh, getattr(mh, atom), tdt, torch.float32, 512, 256, K, 21, K ** -0.5,
                                        cta=(256, 256, 64), **kw)
            assert relerr(got, c64) <= TOL16, (K, kw)


def test_library_picks_the_tile(mh):
    """cta_tile = (0,0,0): the library chooses; the result must not depend on the choice."""
    for (M, N, K) in ((4096, 2048, 512), (384, 128, 96)):
        got, c64, _, _ = _mfma_case(mh, mh.MFMA_F32_16x16x32_F16, torch.float16, torch.float16, M, N, K, 5, K ** -0.5,
                                    cta=(0, 0, 0))
        assert relerr(got, c64) <= TOL16


def test_64x64_tile_exact_on_integers(mh):
    """The 64 x 64 CTA tile (what the library picks for problems that leave CUs idle with 128 x 128): every input
    type, both K extents per tile, C and alpha, column-major D, and the library's own choice."""
    cases = [(mh.MFMA_F32_16x16x32_F16, torch.float16, 32), (mh.MFMA_F32_16x16x32_BF16, torch.bfloat16, 32),
             (mh.MFMA_F32_16x16x4_F32, torch.float32, 16)]
    if hasattr(torch, "float8_e4m3fn"):
        cases.append((mh.MFMA_F32_16x16x32_FP8, torch.float8_e4m3fn, 64))
    g = torch.Generator().manual_seed(64)
    for atom, tdt, bk in cases:
        for (M, N, K) in ((64, 64, 2 * bk), (192, 320, 256), (1024, 1024, 512)):
            A = torch.randint(-4, 5, (M, K), generator=g).float()
            B = torch.randint(-4, 5, (N, K), generator=g).float()
            C = torch.randint(-9, 10, (M, N), generator=g).float()
            a, b, c = A.to(tdt).cuda(), B.to(tdt).cuda(), C.cuda()
            ref = A.double() @ B.double().t()
            for cta in ((64, 64, bk), (64, 64, 2 * bk), (0, 0, 0)):
                mma = mh.tiled_mma_desc(atom, atom_layout=(2, 2, 1), cta_tile=cta)
                d = torch.zeros(M, N, device="cuda")
                mh.gemm_(mma, T(d), T(a), T(b))
                torch.cuda.synchronize()
                assert torch.equal(d.cpu().double(), ref), (tdt, M, N, K, cta)
                mh.gemm_(mma, T(d), T(a), T(b), T(c), 2.0)
                torch.cuda.synchronize()
                assert torch.equal(d.cpu().double(), 2 * ref + C.double()), (tdt, M, N, K, cta, "C")
                dt_ = torch.zeros(N, M, device="cuda")
                mh.gemm_(mma, T(dt_, (M, N), (1, M)), T(a), T(b))
                torch.cuda.synchronize()
                assert torch.equal(dt_.t().cpu().double(), ref), (tdt, M, N, K, cta, "column-major D")
            d16 = torch.zeros(M, N, dtype=torch.bfloat16, device="cuda")
            mh.gemm_(mh.tiled_mma_desc(atom, atom_layout=(2, 2, 1), cta_tile=(64, 64, bk)), T(d16), T(a), T(b), None, 2.0 ** -6)
            torch.cuda.synchronize()
            assert torch.equal(d16.cpu().double(), (ref * 2.0 ** -6).to(torch.bfloat16).double()), (tdt, M, N, K, "bf16 out")
    with pytest.raises(mh.MoyeError):          # an explicit 64 x 64 tile keeps the reference's divisibility assertion
        x = torch.zeros(100, 64, dtype=torch.float16, device="cuda")
        mh.gemm_(mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, cta_tile=(64, 64, 32)), T(torch.zeros(100, 100, device="cuda")), T(x), T(x))


def test_config4_bf16_8192(mh):
    """Benchmark configuration 4 (square) at full size: bf16 8192^3, fp32 accumulate and output."""
    M = N = K = 8192
    got, c64, A, B = _mfma_case(mh, mh.MFMA_F32_16x16x32_BF16, torch.bfloat16, torch.float32, M, N, K, 1004, 0.02,
                                cta=(256, 256, 64))
    err = relerr(got, c64)
    rows = np.random.default_rng(1).choice(M, 16, replace=False)
    ref = to.gemm_universal_fma(A[rows].float().numpy(), B.float().numpy(), np.zeros((16, N), np.float32), "bf16", "bf16")
    ref_err = to.relerr(ref, c64[rows].cpu().numpy())
    print("config4 bf16 8192^3: rel err %.3e (reference arithmetic on 16 rows: %.3e)" % (err, ref_err))
    assert err <= TOL16


def test_config5_fp8_8192(mh):
    """Benchmark configuration 5 at full size: e4m3 8192^3, per-tensor scales, bf16 out."""
    if not hasattr(torch, "float8_e4m3fn"):
        pytest.skip("torch without float8_e4m3fn")
    M = N = K = 8192
    g = torch.Generator(device="cuda").manual_seed(1005)
    X = torch.randn(M, K, generator=g, device="cuda")
    W = torch.randn(N, K, generator=g, device="cuda")
    sa, sb = float(X.abs().max() / 448), float(W.abs().max() / 448)
    a, b = (X / sa).to(torch.float8_e4m3fn), (W / sb).to(torch.float8_e4m3fn)
    del X, W
    d = torch.zeros(M, N, dtype=torch.bfloat16, device="cuda")
    mh.gemm_(mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_FP8, atom_layout=(2, 4, 1), cta_tile=(256, 256, 128)), T(d), T(a),
             T(b), None, sa * sb)
    torch.cuda.synchronize()
    rows = torch.randperm(M, device="cuda")[:512]
    c64 = (a[rows].float().double() @ b.float().double().t()) * (sa * sb)
    err = relerr(d[rows], c64)
    print("config5 fp8 8192^3 (512 sampled rows): rel err vs fp64 of the quantised inputs %.3e" % err)
    assert err <= TOL16


def test_moye_array_api_on_device(mh):
    """The MoYe-level calls: MoYeArray views, @tile, make_tiled_mma, gemm!, copyto! on device arrays."""
    from moye_hip import layout as ml
    g = torch.Generator().manual_seed(2)
    M, N, K = 512, 256, 128
    A = (torch.randn(M, K, generator=g) / 8).half().cuda()
    B = (torch.randn(N, K, generator=g) / 8).half().cuda()
    Dt = torch.zeros(M, N, dtype=torch.float16, device="cuda")
    mA = mh.MoYeArray.from_torch(A)          # (M,K):(K,1)
    mB = mh.MoYeArray.from_torch(B)          # (N,K):(K,1)
    mD = mh.MoYeArray.from_torch(Dt)
    S = ml.StaticInt
    mma = mh.make_tiled_mma(mh.MFMA_F32_16x16x32_F16, ml.static_layout((2, 2, 1)), (S(128), S(128), S(32)))
    assert [int(v) for v in mma.tile_shape()] == [128, 128, 32] and mma.size() == 256
    mh.gemm_(mma, mD, mA, mB)
    torch.cuda.synchronize()
    c64 = A.double() @ B.double().t()
    assert relerr(Dt, c64) <= TOL16
    # gemm! on one CTA tile of the problem, selected with @tile as the reference's kernels do
    Dt2 = torch.zeros_like(Dt)
    mD2 = mh.MoYeArray.from_torch(Dt2)
    gA = mh.local_tile(mA, (S(128), S(K)), (2, 1))
    gB = mh.local_tile(mB, (S(128), S(K)), (1, 1))
    gD = mh.local_tile(mD2, (S(128), S(128)), (2, 1))
    mh.gemm_(mma, gD, gA, gB)
    torch.cuda.synchronize()
    assert torch.equal(Dt2[128:256, :128], Dt[128:256, :128]) and float(Dt2[:128].abs().max()) == 0.0
    # copyto! with a tiled copy: transposed destination
    src = torch.randint(-2 ** 31, 2 ** 31 - 1, (256 * 192,), dtype=torch.int32, device="cuda")
    dst = torch.zeros_like(src)
    ms = mh.MoYeArray.from_torch(src, ml.Layout((256, 192), (1, 256)))
    md = mh.MoYeArray.from_torch(dst, ml.Layout((256, 192), (192, 1)))
    tc = mh.make_tiled_copy(mh.CopyAtom(128, 32), ml.static_layout((16, 16)), ml.static_layout((4, 4)),
                            op=mh.COPY_LDS_TILED)
    mh.copyto_(md, ms, tc)
    torch.cuda.synchronize()
    assert torch.equal(dst.view(256, 192), src.view(192, 256).t())


# ---------------------------------------------------------------------------------------------
# short A (M <= 64): the bandwidth-shaped kernel
# ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("M", [16, 32, 48, 64])
def test_short_m_exact_on_integers(mh, M):
    g = torch.Generator().manual_seed(40 + M)
    for (N, K) in ((256, 320), (1024, 4096), (48, 32), (8192, 288), (8192, 512)):
        A = torch.randint(-4, 5, (M, K), generator=g).to(torch.float16)
        B = torch.randint(-4, 5, (N, K), generator=g).to(torch.float16)
        C = torch.randint(-8, 9, (M, N), generator=g).to(torch.float32)
        a, b, c = A.cuda(), B.cuda(), C.cuda()
        ref = A.double() @ B.double().t()
        for explicit in (False, True):
            d = torch.zeros(M, N, dtype=torch.float32, device="cuda")
            mma = mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, cta_tile=(M, 16, 32) if explicit else (0, 0, 0))
            mh.gemm_(mma, T(d), T(a), T(b))
            torch.cuda.synchronize()
            assert torch.equal(d.cpu().double(), ref), (M, N, K, explicit)
        d = torch.zeros(M, N, dtype=torch.float32, device="cuda")
        mh.gemm_(mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, cta_tile=(0, 0, 0)), T(d), T(a), T(b), T(c), 2.0)
        torch.cuda.synchronize()
        assert torch.equal(d.cpu().double(), 2.0 * ref + C.double()), (M, N, K, "C, alpha")
        for split in (-1, 2):          # K ranges: from M = 33 on a workgroup then takes 64 rows of B
            d = torch.zeros(M, N, dtype=torch.float32, device="cuda")
            mh.gemm_(mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, cta_tile=(0, 0, 0), split_k=split), T(d), T(a), T(b), T(c), 2.0)
            torch.cuda.synchronize()
            assert torch.equal(d.cpu().double(), 2.0 * ref + C.double()), (M, N, K, "split_k", split)


@pytest.mark.parametrize("tdt,atom,K", [("float16", "MFMA_F32_16x16x32_F16", 8216), ("bfloat16", "MFMA_F32_16x16x32_BF16", 136),
                                        ("float32", "MFMA_F32_16x16x4_F32", 4100), ("float8_e4m3fn", "MFMA_F32_16x16x32_FP8", 8304)])
def test_short_m_k_tail_inside_nan_frames(mh, tdt, atom, K):
    """A K that ends inside a 128-byte line: the short-M kernel masks the pieces beyond K in registers.  The operands
    are windows of arrays whose other bytes are NaN (Inf), so a piece read past K and not masked shows; every type;
    also as the K ranges of a split (whole lines, the tail in the last)."""
    if not hasattr(torch, tdt):
        pytest.skip("no " + tdt)
    tdt, atom = getattr(torch, tdt), getattr(mh, atom)
    g = torch.Generator().manual_seed(K)
    for (M, N) in ((16, 8192), (5, 100), (64, 8200)):
        A = torch.randint(-3, 4, (M, K), generator=g).float()
        B = torch.randint(-3, 4, (N, K), generator=g).float()
        if K > 4000:
            A[:, 100:K - 100] = 0
        pad = 16 // torch.empty(0, dtype=tdt).element_size()
        Ab = torch.full((M + 1, K + 3 * pad), float("nan"), dtype=torch.float32).to(tdt).cuda()
        Bb = torch.full((N + 1, K + pad), float("nan") if tdt == torch.float8_e4m3fn else float("inf"), dtype=torch.float32).to(tdt).cuda()
        Ab[:M, :K] = A.to(tdt).cuda()
        Bb[:N, :K] = B.to(tdt).cuda()
        ref = A.double() @ B.double().t()
        for split in (0, -1):
            d = torch.zeros(M, N, dtype=torch.float32, device="cuda")
            mma = mh.tiled_mma_desc(atom, cta_tile=(0, 0, 0), split_k=split)
            ks = kernels_of(mh, mma, T(d), T(Ab[:M, :K]), T(Bb[:N, :K]))
            assert ks[0]["family"] == "gemm_mfma_skinny_lds", ks
            mh.gemm_(mma, T(d), T(Ab[:M, :K]), T(Bb[:N, :K]))
            torch.cuda.synchronize()
            assert torch.equal(d.cpu().double(), ref), (tdt, M, N, K, split)


@pytest.mark.parametrize("M", [1, 7, 20, 33, 63])
def test_short_m_any_m_and_n(mh, M):
    """M and N that are not multiples of 16: lanes beyond the operands read the last row and store nothing.
    D is a window of a larger buffer whose frame must stay untouched."""
    g = torch.Generator().manual_seed(90 + M)
    for (N, K) in ((100, 320), (1, 64), (8200, 256), (8191, 96)):
        A = torch.randint(-4, 5, (M, K), generator=g).to(torch.float16)
        B = torch.randint(-4, 5, (N, K), generator=g).to(torch.float16)
        C = torch.randint(-8, 9, (M, N), generator=g).to(torch.float32)
        a, b, c = A.cuda(), B.cuda(), C.cuda()
        ref = A.double() @ B.double().t()
        big = torch.full((M + 2, N + 3), 77.0, device="cuda")
        d = big[1:M + 1, 2:N + 2]
        mh.gemm_(mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, cta_tile=(0, 0, 0)), T(d), T(a), T(b), T(c), 2.0)
        torch.cuda.synchronize()
        assert torch.equal(d.cpu().double(), 2.0 * ref + C.double()), (M, N, K)
        frame = big.clone()
        frame[1:M + 1, 2:N + 2] = 77.0
        assert bool((frame == 77.0).all()), "stores outside D"
        dt_ = torch.zeros(N, M, device="cuda")                 # column-major D: the short side becomes N
        mh.gemm_(mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, cta_tile=(0, 0, 0)), T(dt_, (M, N), (1, M)), T(a), T(b))
        torch.cuda.synchronize()
        assert torch.equal(dt_.t().cpu().double(), ref), (M, N, K, "column-major D")


def test_short_m_small_n_long_k_takes_k_ranges(mh):
    """With split_k < 0 the library cuts K into ranges for a short-M problem whose N is small and K long (its workgroups of
    16 columns would leave most CUs idle): the workspace it asks for tells how many; none when N fills the chip or K is
    short.  Results exact on small integers either way, the same bits as unsplit (integers: every order of the sum)."""
    g = torch.Generator().manual_seed(41)
    for (M, N, K, ranges) in ((16, 1024, 32768, 4), (16, 2048, 16384, 2), (32, 1024, 8192, 4), (64, 2048, 8192, 2), (16, 1000, 32768, 4),
                              (16, 8192, 8192, 1), (16, 2048, 4096, 1), (16, 4096, 8192, 1), (16, 1024, 2048, 1)):
        A = torch.randint(-2, 3, (M, K), generator=g).to(torch.bfloat16)
        B = torch.randint(-2, 3, (N, K), generator=g).to(torch.bfloat16)
        a, b = A.cuda(), B.cuda()
        d = torch.zeros(M, N, device="cuda")
        mma = mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_BF16, split_k=-1)
        need = mh.gemm_workspace_size(mma, T(d), T(a), T(b))
        assert need == (ranges * M * N * 4 if ranges > 1 else 0), (M, N, K, need)
        mh.gemm_(mma, T(d), T(a), T(b))
        torch.cuda.synchronize()
        assert torch.equal(d.cpu().double(), A.double() @ B.double().t()), (M, N, K)


@pytest.mark.parametrize("M", [33, 48, 64])
def test_short_m_sixty_four_rows_of_b_per_workgroup(mh, M):
    """More than 32 rows of A and an N whose workgroups of 32 rows of B would need a second round on the CUs while those of
    64 rows need one: the form with ntw=4 and two stages; N ragged against 64, K with and without a tail, every input
    type, D inside a frame; exact on small integers."""
    g = torch.Generator().manual_seed(700 + M)
    for (tdt, atom) in ((torch.float16, mh.MFMA_F32_16x16x32_F16), (torch.bfloat16, mh.MFMA_F32_16x16x32_BF16),
                        (torch.float8_e4m3fn, mh.MFMA_F32_16x16x32_FP8)):
        eb = tdt.itemsize
        for (N, K) in ((16384, 256 // eb), (16256 + M, 1280 // eb), (12289, 464 // eb)):   # 256, 255 and 193 workgroups of 64 rows
            A = torch.randint(-2, 3, (M, K), generator=g).float()
            B = torch.randint(-2, 3, (N, K), generator=g).float()
            a, b = A.cuda().to(tdt), B.cuda().to(tdt)
            big = torch.full((M + 2, N + 3), 77.0, device="cuda")
            d = big[1:M + 1, 2:N + 2]
            mma = mh.tiled_mma_desc(atom, cta_tile=(0, 0, 0))
            ks = kernels_of(mh, mma, T(d), T(a), T(b))
            assert len(ks) == 1 and "mt=%d,ntw=4,waves=4,stages=2" % ((M + 15) // 16) in ks[0]["name"], ks
            mh.gemm_(mma, T(d), T(a), T(b))
            torch.cuda.synchronize()
            assert torch.equal(d.cpu().double(), A.double() @ B.double().t()), (tdt, M, N, K)
            frame = big.clone()
            frame[1:M + 1, 2:N + 2] = 77.0
            assert bool((frame == 77.0).all()), "stores outside D"


@pytest.mark.parametrize("M", [17, 40, 64])
def test_short_a_with_a_short_k_and_many_columns_runs_on_tiles(mh, M):
    """More than 16 rows of A, K of at most 4096 bytes and columns for 128-wide tiles on three quarters of the CUs: the
    library takes tiles, not the short-M kernel; row- and column-major D inside a frame, exact on small integers."""
    g = torch.Generator().manual_seed(800 + M)
    for (tdt, atom) in ((torch.float16, mh.MFMA_F32_16x16x32_F16), (torch.float8_e4m3fn, mh.MFMA_F32_16x16x32_FP8)):
        for (N, K) in ((24576, 256), (24576 + 40, 1024 // tdt.itemsize), (65536, 128)):
            A = torch.randint(-2, 3, (M, K), generator=g).float()
            B = torch.randint(-2, 3, (N, K), generator=g).float()
            a, b = A.cuda().to(tdt), B.cuda().to(tdt)
            ref = A.double() @ B.double().t()
            mma = mh.tiled_mma_desc(atom, cta_tile=(0, 0, 0))
            big = torch.full((M + 2, N + 8), 77.0, device="cuda")
            d = big[1:M + 1, 4:N + 4]
            ks = kernels_of(mh, mma, T(d), T(a), T(b))
            assert ks[0]["family"] != "gemm_mfma_skinny_lds", ks
            mh.gemm_(mma, T(d), T(a), T(b))
            torch.cuda.synchronize()
            assert torch.equal(d.cpu().double(), ref), (tdt, M, N, K)
            frame = big.clone()
            frame[1:M + 1, 4:N + 4] = 77.0
            assert bool((frame == 77.0).all()), "stores outside D"
            dt_ = torch.zeros(N, M, device="cuda")                 # column-major D
            mh.gemm_(mma, T(dt_, (M, N), (1, M)), T(a), T(b))
            torch.cuda.synchronize()
            assert torch.equal(dt_.t().cpu().double(), ref), (tdt, M, N, K, "column-major D")


@pytest.mark.parametrize("M", [1, 16, 17, 48, 64])
def test_short_m_line_staging_kernel(mh, M):
    """K of whole 128-byte lines runs on the kernel that stages them through LDS: any M <= 64 and any N (16 and
    32 rows of B per workgroup), K ranges of none, one and many lines per wave, even and uneven, row- and column-major D inside a frame, C with alpha,
    every input type; exact on small integers, so a wrong piece, row or K range is a hard mismatch."""
    g = torch.Generator().manual_seed(300 + M)
    # (K of whole 128-byte lines, and K with a tail of one to seven 16-byte pieces: 8, 72, 200, 4152, 56)
    for (N, K) in ((100, 256), (8191, 768), (8200, 2048), (12000, 256), (32, 4096), (8192, 320), (100, 64), (8200, 704), (100, 8), (8191, 72),
                   (8200, 200), (300, 4152), (8192, 56)):
        A = torch.randint(-4, 5, (M, K), generator=g).to(torch.float16)
        B = torch.randint(-4, 5, (N, K), generator=g).to(torch.float16)
        C = torch.randint(-8, 9, (M, N), generator=g).to(torch.float32)
        a, b, c = A.cuda(), B.cuda(), C.cuda()
        ref = A.double() @ B.double().t()
        big = torch.full((M + 2, N + 3), 77.0, device="cuda")
        d = big[1:M + 1, 2:N + 2]
        ks = kernels_of(mh, mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, cta_tile=(0, 0, 0)), T(d), T(a), T(b), T(c))
        assert len(ks) == 1 and ks[0]["family"] == "gemm_mfma_skinny_lds" and "mt=%d," % ((M + 15) // 16) in ks[0]["name"], ks
        mh.gemm_(mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, cta_tile=(0, 0, 0)), T(d), T(a), T(b), T(c), 2.0)
        torch.cuda.synchronize()
        assert torch.equal(d.cpu().double(), 2.0 * ref + C.double()), (M, N, K)
        frame = big.clone()
        frame[1:M + 1, 2:N + 2] = 77.0
        assert bool((frame == 77.0).all()), "stores outside D"
        dt_ = torch.zeros(N, M, device="cuda")
        mh.gemm_(mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, cta_tile=(0, 0, 0)), T(dt_, (M, N), (1, M)), T(a), T(b))
        torch.cuda.synchronize()
        assert torch.equal(dt_.t().cpu().double(), ref), (M, N, K, "column-major D")
        if K % 16:
            continue
        d2 = torch.zeros(M, N, dtype=torch.float32, device="cuda")     # two K ranges on request: each of whole lines or not
        mh.gemm_(mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, cta_tile=(0, 0, 0), split_k=2), T(d2), T(a), T(b), T(c), 2.0)
        torch.cuda.synchronize()
        assert torch.equal(d2.cpu().double(), 2.0 * ref + C.double()), (M, N, K, "split_k 2")
    N, K = 8192, 1024
    A = torch.randint(-3, 4, (M, K), generator=g).float()
    B = torch.randint(-3, 4, (N, K), generator=g).float()
    ref = A.double() @ B.double().t()
    cases = [(torch.bfloat16, mh.MFMA_F32_16x16x32_BF16, torch.bfloat16), (torch.float32, mh.MFMA_F32_16x16x4_F32, torch.float32)]
    if hasattr(torch, "float8_e4m3fn"):
        cases.append((torch.float8_e4m3fn, mh.MFMA_F32_16x16x32_FP8, torch.float16))
    for in_dt, atom, out_dt in cases:
        a, b = A.to(in_dt).cuda(), B.to(in_dt).cuda()
        d = torch.zeros(M, N, dtype=out_dt, device="cuda")
        mh.gemm_(mh.tiled_mma_desc(atom, cta_tile=(0, 0, 0)), T(d), T(a), T(b), None, 1.0 / 64)
        torch.cuda.synchronize()
        want = (ref / 64).to(torch.float32).to(out_dt)
        assert torch.equal(d.cpu(), want), (in_dt, out_dt)


def test_thin_fringes_with_a_d_that_is_not_aligned(mh):
    """At most 64 rows and columns beyond whole 256x256 tiles, D's rows 8 bytes off 16-byte boundaries: the interior
    runs on whole tiles through the guarded instance where there is one (f16 / bf16 / f32 operands), the fringes on the
    short-M kernel; fp8 has no guarded instance and takes the residue kernels.  Exact on small integers; the frame
    around D stays untouched."""
    g = torch.Generator().manual_seed(77)
    cases = [(torch.float16, mh.MFMA_F32_16x16x32_F16, torch.float16, 4100, 4104, 2048),
             (torch.bfloat16, mh.MFMA_F32_16x16x32_BF16, torch.float32, 4160, 4098, 2048),
             (torch.float32, mh.MFMA_F32_16x16x4_F32, torch.float32, 4100, 4104, 64)]
    if hasattr(torch, "float8_e4m3fn"):
        cases.append((torch.float8_e4m3fn, mh.MFMA_F32_16x16x32_FP8, torch.bfloat16, 4100, 4104, 2048))
    for in_dt, atom, out_dt, M, N, K in cases:
        A = torch.randint(-1, 2, (M, K), generator=g).float()
        B = torch.randint(-1, 2, (N, K), generator=g).float()
        A[:, 100:K - 100] = 0                    # keeps every sum small enough for bf16 results
        ref = A.double() @ B.double().t()
        assert float(ref.abs().max()) < 250
        a, b = A.to(in_dt).cuda(), B.to(in_dt).cuda()
        off = 8 // torch.empty(0, dtype=out_dt).element_size()          # elements in 8 bytes
        pitch = (N + 2 * off + 7) // 8 * 8 + off
        big = torch.full((M + 2, pitch), 7.0, dtype=out_dt, device="cuda")
        d = big[1:M + 1, off:off + N]
        assert (d.data_ptr() % 16, (pitch * d.element_size()) % 16) in ((8, 8), (0, 8), (8, 0))
        mh.gemm_(mh.tiled_mma_desc(atom, cta_tile=(0, 0, 0)), T(d), T(a), T(b))
        torch.cuda.synchronize()
        assert torch.equal(d.cpu().double(), ref), (in_dt, out_dt)
        frame = big.clone()
        frame[1:M + 1, off:off + N] = 7.0
        assert bool((frame == 7.0).all()), ("stores outside D", in_dt)


@pytest.mark.parametrize("case", [(4608, 4608, 2048), (2304, 9216, 1024), (6144, 6144, 512), (4608, 4608, 64), (5120, 5120, 1024),
                                  (7168, 7168, 256)])
def test_last_round_on_its_own_launch_exact_on_integers(mh, case):
    """More whole 256x256 tiles than CUs and a last round that fills little of the chip: the library may run the first
    tile rows (columns where N has more tiles) on 256x256 tiles and the rest as a problem of its own, on the same
    stream.  Every element of D belongs to exactly one of the two launches: exact on small integers, with and without
    C, D a window of a larger buffer whose frame stays untouched."""
    M, N, K = case
    g = torch.Generator().manual_seed(M + N + K)
    kinds = [(torch.float16, mh.MFMA_F32_16x16x32_F16, torch.float16, False),
             (torch.bfloat16, mh.MFMA_F32_16x16x32_BF16, torch.float32, True)]
    if hasattr(torch, "float8_e4m3fn") and K >= 128:
        kinds.append((torch.float8_e4m3fn, mh.MFMA_F32_16x16x32_FP8, torch.bfloat16, False))
    if K <= 512:
        kinds.append((torch.float32, mh.MFMA_F32_16x16x4_F32, torch.float32, False))
    for in_dt, atom, out_dt, with_c in kinds:
        A = torch.randint(-1, 2, (M, K), generator=g).float()
        B = torch.randint(-1, 2, (N, K), generator=g).float()
        if K > 200:
            A[:, 100:K - 100] = 0
        Cm = torch.randint(-3, 4, (M, N), generator=g).float()
        ref = 0.5 * (A.double() @ B.double().t()) + (Cm.double() if with_c else 0)
        assert float(ref.abs().max()) < 250
        a, b = A.to(in_dt).cuda(), B.to(in_dt).cuda()
        big = torch.full((M + 2, N + 16), 7.0, dtype=out_dt, device="cuda")
        d = big[1:M + 1, 8:8 + N]
        mma = mh.tiled_mma_desc(atom, cta_tile=(0, 0, 0), split_k=-1)
        cm = T(Cm.to(out_dt).cuda()) if with_c else None
        ks = kernels_of(mh, mma, T(d), T(a), T(b), cm)
        if in_dt in (torch.float16, torch.bfloat16) and case == (4608, 4608, 2048):
            # 324 tiles of 256 x 256: the first eleven tile rows on them, the rest as a problem of its own on 128 x 128 tiles
            assert [k["tile"] for k in ks] == ["256x256x128B", "128x128x128B"] and ks[0]["M"] + ks[1]["M"] == M, ks
        if in_dt in (torch.float16, torch.bfloat16) and case == (5120, 5120, 1024):
            assert len(ks) == 1 and ks[0]["tile"] == "256x256x128B", ks      # 400 tiles: the model sees nothing to gain
        mh.gemm_(mma, T(d), T(a), T(b), cm, 0.5)
        torch.cuda.synchronize()
        assert torch.equal(d.cpu().double(), ref), (in_dt, out_dt)
        frame = big.clone()
        frame[1:M + 1, 8:8 + N] = 7.0
        assert bool((frame == 7.0).all()), ("stores outside D", in_dt)


@pytest.mark.parametrize("shape,kind", [((4608, 4608, 64), "col"), ((2304, 9216, 64), "row"), ((4608, 4608, 128), "full"),
                                        ((2304, 9216, 128), "col"), ((4608, 4608, 64), "row")])
def test_last_round_on_its_own_launch_keeps_the_epilogue_operand_in_step(mh, shape, kind):
    """The same two-launch shapes with a fused epilogue: the second launch reads C and the operand (a vector along
    either mode, or a whole array) from where its part of D begins.  Bit-exact against the oracle's epilogue."""
    M, N, K = shape
    mma = mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, cta_tile=(0, 0, 0), split_k=-1)
    _epilogue_case(mh, mma, M, N, K, "float16", "add", kind, seed=M + K + len(kind))
    _epilogue_case(mh, mma, M, N, K, "float32", "max", kind, seed=N + K + len(kind), beta=0.0)


@pytest.mark.parametrize("case", [(4000, 2200, 328), (3900, 2304, 120), (4096, 2048, 72), (4090, 2203, 40), (2100, 4100, 200),
                                  (4099, 2050, 4096 + 8), (4096, 2048, 128), (1000, 600, 136), (384, 256, 128), (130, 2000, 72),
                                  (4000, 2200, 192), (3841, 2305, 4096), (4100, 2052, 4096),
                                  (3000, 2000, 192), (2100, 2900, 4096), (4000, 4000, 4096), (5000, 3000, 4096), (4000, 4000, 4096 + 48),
                                  (2100, 2900, 4096 + 16)])
def test_ragged_256_tiles_exact_on_integers(mh, case):
    """Problems the library puts on 256x256 tiles (the larger cases) or 128x128 tiles that reach beyond M, N and K: rows beyond the operands are read from
    the last row and never stored, the K tail (1 to 7 pieces of 16 bytes, also with less than one k-tile in all) is
    masked, pieces of D that cross N go out element by element.  D is a window of a larger buffer whose frame must stay
    untouched; small integers make every sum exact.  (The guarded forms of the hand-ordered kernel, K tails included:
    with C the one whose epilogue is the general one.)"""
    M, N, K = case
    g = torch.Generator().manual_seed(M + N + K)
    A = torch.randint(-3, 4, (M, K), generator=g).float()
    B = torch.randint(-3, 4, (N, K), generator=g).float()
    C = torch.randint(-8, 9, (M, N), generator=g).float()
    if K >= 4096:                     # keep |sum| small enough to be exact in fp16 too; both ends of K stay in play
        A[:, 150:K - 150] = 0
    ref = A.double() @ B.double().t()
    assert float(ref.abs().max()) * 2 + 8 < 2048
    pitch = (N + 8 + 7) // 8 * 8
    types = [(torch.float16, mh.MFMA_F32_16x16x32_F16, torch.float16), (torch.bfloat16, mh.MFMA_F32_16x16x32_BF16, torch.float32),
             (torch.float32, mh.MFMA_F32_16x16x4_F32, torch.float32)]
    if hasattr(torch, "float8_e4m3fn") and K % 16 == 0:
        types.append((torch.float8_e4m3fn, mh.MFMA_F32_16x16x32_FP8, torch.float32))
    for in_dt, atom, out_dt in types:
        a, b, c = A.to(in_dt).cuda(), B.to(in_dt).cuda(), C.to(out_dt).cuda()
        big = torch.full((M + 2, pitch), 77.0, dtype=out_dt, device="cuda")
        d = big[1:M + 1, 8:8 + N]
        mh.gemm_(mh.tiled_mma_desc(atom, cta_tile=(0, 0, 0)), T(d), T(a), T(b), T(c), 2.0)
        torch.cuda.synchronize()
        assert torch.equal(d.cpu().double(), 2.0 * ref + C.double()), (case, in_dt, out_dt)
        frame = big.clone()
        frame[1:M + 1, 8:8 + N] = 77.0
        assert bool((frame == 77.0).all()), "stores outside D"
        d.zero_()
        ks = kernels_of(mh, mh.tiled_mma_desc(atom, cta_tile=(0, 0, 0)), T(d), T(a), T(b))
        kc = kernels_of(mh, mh.tiled_mma_desc(atom, cta_tile=(0, 0, 0)), T(d), T(a), T(b), T(c))
        b16 = in_dt in (torch.float16, torch.bfloat16)
        if case == (3841, 2305, 4096) and b16:
            # one row and one column beyond whole tiles: the interior on whole 256 x 256 tiles, each fringe on the short-M kernel
            assert [k["family"] for k in ks] == ["gemm_mfma_tn_256_w4", "gemm_mfma_skinny_lds", "gemm_mfma_skinny_lds"] and "ragged=0" in ks[0]["name"], ks
        if case in ((4000, 4000, 4096), (5000, 3000, 4096)):
            # at least 128 ragged 256 x 256 tiles, K of whole 128-byte rows: the guarded forms of the hand-ordered kernel,
            # with C the one whose epilogue is the general one
            # (fp32, whose pace the matrix pipe sets whatever the fill, is cheaper on 128 x 128 tiles here: the same kernel's guarded 128 x 128 form)
            assert ks[0]["family"] == "gemm_mfma_tn_256_w4" and "ragged=1" in ks[0]["name"] and "ops=0" in ks[0]["name"], ks
            assert "tile=256" in ks[0]["name"] or in_dt == torch.float32, ks
            if in_dt != torch.float32:
                assert kc[0]["family"] == "gemm_mfma_tn_256_w4" and "ragged=1" in kc[0]["name"] and "ops=1" in kc[0]["name"], kc
        if case in ((2100, 2900, 4096), (2100, 2900, 4096 + 16)):     # fewer than 128 tiles of 256 x 256: the hand-ordered kernel's guarded 128 x 128 instance
            assert ks[0]["family"] == "gemm_mfma_tn_256_w4" and "ragged=1" in ks[0]["name"] and "tile=128" in ks[0]["name"], ks
        if (case == (4099, 2050, 4096 + 8) and b16) or case == (4000, 4000, 4096 + 48):     # a K tail on 256 x 256 tiles: the same guarded forms mask it in registers
            assert ks[0]["family"] == "gemm_mfma_tn_256_w4" and "ragged=1" in ks[0]["name"] and ("tile=256" in ks[0]["name"] or in_dt == torch.float32), ks
            if in_dt != torch.float32:
                assert kc[0]["family"] == "gemm_mfma_tn_256_w4" and "ragged=1" in kc[0]["name"] and "ops=1" in kc[0]["name"], kc
        if case == (1000, 600, 136):     # too few tiles for 256 x 256: the 128 x 128 kernel's guarded instance
            assert ks[0]["tile"].startswith("128x128") and "ragged" in ks[0]["flags"], ks
        mh.gemm_(mh.tiled_mma_desc(atom, cta_tile=(0, 0, 0)), T(d), T(a), T(b))
        torch.cuda.synchronize()
        assert torch.equal(d.cpu().double(), ref), (case, in_dt, out_dt, "no C")
    # a D whose rows do not start on 16-byte boundaries (pitch and first element 8 bytes off): the pieces that are not
    # aligned go out element by element
    a, b = A.half().cuda(), B.half().cuda()
    big = torch.full((M + 2, N + 12 + (N % 2)), 77.0, dtype=torch.float16, device="cuda")
    d = big[1:M + 1, 4:4 + N]
    mh.gemm_(mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, cta_tile=(0, 0, 0)), T(d), T(a), T(b))
    torch.cuda.synchronize()
    assert torch.equal(d.cpu().double(), ref), (case, "unaligned D")
    frame = big.clone()
    frame[1:M + 1, 4:4 + N] = 77.0
    assert bool((frame == 77.0).all()), "stores outside an unaligned D"
    # NaN and Inf beyond the operands' K extent and in the rows after them must not reach D: the operands are windows too
    Ab = torch.full((M + 1, K + 8), float("nan"), dtype=torch.float16, device="cuda")
    Bb = torch.full((N + 1, K + 8), float("inf"), dtype=torch.float16, device="cuda")
    Ab[:M, :K] = A.half().cuda()
    Bb[:N, :K] = B.half().cuda()
    d = torch.zeros(M, (N + 7) // 8 * 8, dtype=torch.float16, device="cuda")[:, :N]
    mh.gemm_(mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, cta_tile=(0, 0, 0)), T(d), T(Ab[:M, :K]), T(Bb[:N, :K]))
    torch.cuda.synchronize()
    assert torch.equal(d.cpu().double(), ref), (case, "operands inside NaN / Inf frames")


def test_random_shapes_exact_on_integers(mh):
    """Whatever kernel the library picks for a shape (short-M by registers or by lines, 64 / 128 / 256 tiles, whole,
    predicated or ragged, interior plus thin fringes, K ranges), the result on small integers is exact.  Seeded shapes
    from the ranges where the choice changes; row- and column-major D, with and without C."""
    import random
    rnd = random.Random(20240607)
    pools = ([1, 8, 16, 17, 40, 64, 65, 96, 128, 200, 256, 300, 520], [16, 100, 128, 256, 1000, 2048, 4000, 4096, 4100, 4160, 8192, 8200],
             [8, 32, 64, 72, 128, 256, 264, 512, 1000, 1024, 2048])
    shapes = {(rnd.choice(pools[0]), rnd.choice(pools[1]), rnd.choice(pools[2])) for _ in range(40)}
    shapes |= {(rnd.choice(pools[1]), rnd.choice(pools[1]), rnd.choice(pools[2][:8])) for _ in range(24)}
    g = torch.Generator().manual_seed(5)
    seen = set()
    for (M, N, K) in sorted(shapes):
        if M * N * K > 4096 * 4096 * 300:
            K = 72
        A = torch.randint(-2, 3, (M, K), generator=g).to(torch.float16)
        B = torch.randint(-2, 3, (N, K), generator=g).to(torch.float16)
        C = torch.randint(-8, 9, (M, N), generator=g).to(torch.float16)
        a, b, c = A.cuda(), B.cuda(), C.cuda()
        ref = (a.float() @ b.float().t()).double().cpu()            # exact: |sum| <= 4 K <= 8192 in fp32
        if float(ref.abs().max()) * 2 + 8 >= 2048:                  # ... and representable in fp16 after alpha and C
            continue
        for split in (0, -1):
            d = torch.full((M, N), 9.0, dtype=torch.float16, device="cuda")
            for k in kernels_of(mh, mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, cta_tile=(0, 0, 0), split_k=split), T(d), T(a), T(b), T(c)):
                seen.add((k["family"], k["tile"].rsplit("x", 1)[0], "ragged" in k["flags"], k["split"] > 1))
            mh.gemm_(mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, cta_tile=(0, 0, 0), split_k=split), T(d), T(a), T(b), T(c), 2.0)
            torch.cuda.synchronize()
            assert torch.equal(d.cpu().double(), 2.0 * ref + C.double()), (M, N, K, "split_k", split)
        dt_ = torch.full((N, M), 9.0, dtype=torch.float16, device="cuda")
        mh.gemm_(mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, cta_tile=(0, 0, 0)), T(dt_, (M, N), (1, M)), T(a), T(b))
        torch.cuda.synchronize()
        assert torch.equal(dt_.t().cpu().double(), ref), (M, N, K, "column-major D")
    # the seeded shapes do reach the kernels the docstring names
    fams = {f for f, _, _, _ in seen}
    # (short K keeps these shapes off 256 x 256 tiles; test_ragged_256_tiles_* and test_last_round_* cover those)
    assert {"gemm_mfma_skinny_lds", "gemm_mfma_tn", "gemm_mfma_tn_128"} <= fams, sorted(fams)
    assert any(t == "64x64" for _, t, _, _ in seen) and any(r for _, _, r, _ in seen) and any(sp for _, _, _, sp in seen), sorted(seen)


def test_one_row_operands_with_any_stride_on_the_unit_mode(mh):
    """A 1 x K operand described as (1, K):(1, 1) (what an M-major view of a one-row A looks like) and a 1 x N result
    described the same way: the stride of the mode of extent 1 is never used and must not be taken for a pitch."""
    g = torch.Generator().manual_seed(3)
    for (N, K) in ((1000, 264), (8192, 512), (8, 32)):
        A = torch.randint(-3, 4, (1, K), generator=g).half()
        B = torch.randint(-3, 4, (N, K), generator=g).half()
        ref = A.double() @ B.double().t()
        a, b = A.cuda(), B.cuda()
        d = torch.zeros(1, N, dtype=torch.float32, device="cuda")
        mh.gemm_(mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, cta_tile=(0, 0, 0)), T(d, (1, N), (1, 1)), T(a, (1, K), (1, 1)), T(b))
        torch.cuda.synchronize()
        assert torch.equal(d.cpu().double(), ref), (N, K)


def test_short_m_other_types(mh):
    g = torch.Generator().manual_seed(77)
    M, N, K = 16, 512, 1024
    A = torch.randint(-3, 4, (M, K), generator=g).float()
    B = torch.randint(-3, 4, (N, K), generator=g).float()
    ref = A.double() @ B.double().t()
    cases = [(torch.bfloat16, mh.MFMA_F32_16x16x32_BF16, torch.bfloat16), (torch.bfloat16, mh.MFMA_F32_16x16x32_BF16, torch.float32)]
    if hasattr(torch, "float8_e4m3fn"):
        cases.append((torch.float8_e4m3fn, mh.MFMA_F32_16x16x32_FP8, torch.bfloat16))
    for in_dt, atom, out_dt in cases:
        a, b = A.to(in_dt).cuda(), B.to(in_dt).cuda()
        d = torch.zeros(M, N, dtype=out_dt, device="cuda")
        mh.gemm_(mh.tiled_mma_desc(atom, cta_tile=(0, 0, 0)), T(d), T(a), T(b), None, 1.0 / 64)
        torch.cuda.synchronize()
        # |sum| <= 9 * 1024 / 64 = 144 in steps of 1/64: exact in fp32, and in bf16 after the 1/64 scaling
        # only when it fits 8 bits of mantissa, so compare against the same rounding
        want = (ref / 64).to(torch.float32).to(out_dt)
        assert torch.equal(d.cpu(), want), (in_dt, out_dt)


def test_config4_skinny_bf16(mh):
    """Benchmark configuration 4, skinny case: bf16 16 x 8192 x 8192, fp32 out; run twice, results identical."""
    M, N, K = 16, 8192, 8192
    got, c64, A, B = _mfma_case(mh, mh.MFMA_F32_16x16x32_BF16, torch.bfloat16, torch.float32, M, N, K, 1004, 0.02,
                                cta=(0, 0, 0))
    again, _, _, _ = _mfma_case(mh, mh.MFMA_F32_16x16x32_BF16, torch.bfloat16, torch.float32, M, N, K, 1004, 0.02,
                                cta=(0, 0, 0))
    assert torch.equal(got, again)
    err = relerr(got, c64)
    ref = to.gemm_universal_fma(A.float().numpy()[:, :], B[:64].float().numpy(), np.zeros((M, 64), np.float32), "bf16", "bf16")
    ref_err = to.relerr(ref, c64[:, :64].cpu().numpy())
    print("config4 bf16 16x8192x8192: rel err %.3e (reference arithmetic on 64 columns: %.3e)" % (err, ref_err))
    assert err <= TOL16


# ---------------------------------------------------------------------------------------------
# the MFMA atoms' (thr,val) tables against the instruction itself
# ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("atom,m,n,k,dt", [
    ("MFMA_F32_16x16x32_F16", 16, 16, 32, "float16"), ("MFMA_F32_32x32x16_F16", 32, 32, 16, "float16"),
    ("MFMA_F32_16x16x32_BF16", 16, 16, 32, "bfloat16"), ("MFMA_F32_32x32x16_BF16", 32, 32, 16, "bfloat16"),
    ("MFMA_F32_16x16x32_FP8", 16, 16, 32, "float8_e4m3fn"), ("MFMA_F32_32x32x16_FP8", 32, 32, 16, "float8_e4m3fn"),
    ("MFMA_F32_16x16x4_F32", 16, 16, 4, "float32"), ("MFMA_F32_32x32x2_F32", 32, 32, 2, "float32")])
def test_mfma_atom_tables_on_hardware(mh, atom, m, n, k, dt):
    """layout_a/b/c of every gfx950 atom: one wave gathers A and B through the tables, executes the
    instruction once, scatters D through the C table; D must equal A*B' exactly on small integers.
    A wrong lane->row, lane->k-group or accumulator-register mapping breaks the equality."""
    if not hasattr(torch, dt):
        pytest.skip("torch without " + dt)
    tdt = getattr(torch, dt)
    g = torch.Generator().manual_seed(m * 1000 + k)
    for trial in range(3):
        A = torch.randint(-4, 5, (m, k), generator=g).float()       # distinct rows and columns
        B = torch.randint(-4, 5, (n, k), generator=g).float()
        # column-major dense tiles: element (i, kk) at i + m*kk
        a = A.t().contiguous().to(tdt).cuda()
        b = B.t().contiguous().to(tdt).cuda()
        d = torch.full((n, m), float("nan"), dtype=torch.float32, device="cuda")   # (M,N) column-major
        mh.mma_atom_probe(getattr(mh, atom), a.data_ptr(), b.data_ptr(), d.data_ptr())
        torch.cuda.synchronize()
        assert torch.equal(d.t().cpu().double(), A.double() @ B.double().t()), (atom, trial)


# ---------------------------------------------------------------------------------------------
# fp32 operands on the matrix cores (v_mfma_f32_16x16x4_f32)
# ---------------------------------------------------------------------------------------------

TOL32 = 1e-5   # rel err bound for fp32 inputs


@pytest.mark.parametrize("cta,flags", [((128, 128, 16), 0), ((128, 128, 32), 0), ((256, 256, 32), 0), ((256, 256, 16), 0x100),
                                       ((0, 0, 0), 0)])
def test_f32_mfma_gemm(mh, cta, flags):
    g = torch.Generator().manual_seed(55)
    for (M, N, K) in ((256, 256, 32), (512, 768, 416)):
        # exact on integers
        A = torch.randint(-50, 51, (M, K), generator=g).float()
        B = torch.randint(-50, 51, (N, K), generator=g).float()
        a, b = A.cuda(), B.cuda()
        d = torch.zeros(M, N, device="cuda")
        mma = mh.tiled_mma_desc(mh.MFMA_F32_16x16x4_F32, atom_layout=(2, 4, 1) if cta[0] == 256 else (2, 2, 1), cta_tile=cta,
                                flags=flags)
        mh.gemm_(mma, T(d), T(a), T(b))
        torch.cuda.synchronize()
        assert torch.equal(d.cpu().double(), A.double() @ B.double().t()), (cta, M, N, K)
        # random data against fp64
        A = torch.rand(M, K, generator=g) * 2 - 1
        B = torch.rand(N, K, generator=g) * 2 - 1
        a, b = A.cuda(), B.cuda()
        mh.gemm_(mma, T(d), T(a), T(b))
        torch.cuda.synchronize()
        assert relerr(d, a.double() @ b.double().t()) <= TOL32


def test_f32_mfma_short_m(mh):
    g = torch.Generator().manual_seed(56)
    A = torch.randint(-50, 51, (16, 2048), generator=g).float()
    B = torch.randint(-50, 51, (512, 2048), generator=g).float()
    a, b = A.cuda(), B.cuda()
    d = torch.zeros(16, 512, device="cuda")
    mh.gemm_(mh.tiled_mma_desc(mh.MFMA_F32_16x16x4_F32, cta_tile=(0, 0, 0)), T(d), T(a), T(b))
    torch.cuda.synchronize()
    assert torch.equal(d.cpu().double(), A.double() @ B.double().t())


def _atoms32(mh):
    out = [(mh.MFMA_F32_32x32x16_F16, mh.MFMA_F32_16x16x32_F16, torch.float16, 4, TOL16),
           (mh.MFMA_F32_32x32x16_BF16, mh.MFMA_F32_16x16x32_BF16, torch.bfloat16, 4, TOL16),
           (mh.MFMA_F32_32x32x2_F32, mh.MFMA_F32_16x16x4_F32, torch.float32, 50, TOL32)]
    if hasattr(torch, "float8_e4m3fn"):
        out.append((mh.MFMA_F32_32x32x16_FP8, mh.MFMA_F32_16x16x32_FP8, torch.float8_e4m3fn, 4, TOL16))
    return out


def test_32x32_atoms_exact_on_integers(mh):
    """The 32x32 MFMA forms in the 128x128 kernel: small-integer inputs make every partial sum exact, so a wrong
    k pairing between the two operands or a misplaced accumulator group is a hard mismatch.  Row-major and
    column-major D, C accumulated with alpha, every output type."""
    g = torch.Generator().manual_seed(32)
    for atom, _, tdt, hi, _ in _atoms32(mh):
        for (M, N, K) in ((128, 128, 64), (256, 384, 448)):
            A = torch.randint(-hi, hi + 1, (M, K), generator=g).float()
            B = torch.randint(-hi, hi + 1, (N, K), generator=g).float()
            C = torch.randint(-9, 10, (M, N), generator=g).float()
            a, b = A.to(tdt).cuda(), B.to(tdt).cuda()
            ref = A.double() @ B.double().t()
            for out_dt in (torch.float32, torch.float16, torch.bfloat16):
                if out_dt != torch.float32 and float(ref.abs().max()) * 2 + 9 > (2048 if out_dt == torch.float16 else 256):
                    continue        # not every integer of that size is a float of that type
                mma = mh.tiled_mma_desc(atom, atom_layout=(2, 2, 1), cta_tile=(128, 128, 0))
                d = torch.zeros(M, N, dtype=out_dt, device="cuda")
                mh.gemm_(mma, T(d), T(a), T(b))
                torch.cuda.synchronize()
                assert torch.equal(d.cpu().double(), ref), (atom, M, N, K, out_dt)
                c = C.to(out_dt).cuda()
                mh.gemm_(mma, T(d), T(a), T(b), T(c), 2.0)
                torch.cuda.synchronize()
                assert torch.equal(d.cpu().double(), 2 * ref + C.double()), (atom, M, N, K, out_dt, "C")
                dt_ = torch.zeros(N, M, dtype=out_dt, device="cuda")          # column-major D
                mh.gemm_(mma, T(dt_, (M, N), (1, M)), T(a), T(b))
                torch.cuda.synchronize()
                assert torch.equal(dt_.t().cpu().double(), ref), (atom, M, N, K, out_dt, "col-major")


def test_32x32_atoms_random_and_residue_tiles(mh):
    from moye_hip import _lib
    g = torch.Generator().manual_seed(33)
    for atom, atom16, tdt, hi, tol in _atoms32(mh):
        M, N, K = 256, 256, 512
        A = (torch.randn(M, K, generator=g) * K ** -0.5).to(tdt)
        B = (torch.randn(N, K, generator=g) * K ** -0.5).to(tdt)
        a, b = A.cuda(), B.cuda()
        d, d16 = torch.zeros(M, N, device="cuda"), torch.zeros(M, N, device="cuda")
        mh.gemm_(mh.tiled_mma_desc(atom, atom_layout=(2, 2, 1), cta_tile=(128, 128, 0)), T(d), T(a), T(b))
        mh.gemm_(mh.tiled_mma_desc(atom16, atom_layout=(2, 2, 1), cta_tile=(128, 128, 0)), T(d16), T(a), T(b))
        torch.cuda.synchronize()
        c64 = A.double().cuda() @ B.double().cuda().t()
        assert relerr(d, c64) <= tol, atom
        assert relerr(d, d16) <= 1e-5, atom            # both forms accumulate in fp32; only the order differs
        # residue tiles: the library's tile, and the explicit tile with the predicate flag
        for (M, N, K) in ((100, 130, 48), (129, 127, 80), (1, 1, 16)):
            A = torch.randint(-hi, hi + 1, (M, K), generator=g).float()
            B = torch.randint(-hi, hi + 1, (N, K), generator=g).float()
            a, b = A.to(tdt).cuda(), B.to(tdt).cuda()
            ref = A.double() @ B.double().t()
            for kw in (dict(cta_tile=(0, 0, 0)), dict(cta_tile=(128, 128, 0), flags=_lib.GEMM_PREDICATE)):
                big = torch.full((M + 2, N + 3), 77.0, device="cuda")
                d = big[1:M + 1, 2:N + 2]
                mh.gemm_(mh.tiled_mma_desc(atom, **kw), T(d), T(a), T(b))
                torch.cuda.synchronize()
                assert torch.equal(d.cpu().double(), ref), (atom, M, N, K, kw)
                frame = big.clone()
                frame[1:M + 1, 2:N + 2] = 77.0
                assert bool((frame == 77.0).all()), "stores outside D"


def test_32x32_atoms_on_256_tiles_exact_on_integers(mh):
    """The 32x32 MFMA forms on the 256x256 CTA tile (eight waves of 4 x 2 MFMA tiles): every operand type, every output
    type, named and left to the library, with C and alpha, with an operation in the epilogue (general form), column-major
    D (the operands swapped); small integers, so a misplaced accumulator group or k pairing is a hard mismatch."""
    from moye_hip import _lib
    g = torch.Generator().manual_seed(3232)
    for atom, _, tdt, hi, _ in _atoms32(mh):
        eb = tdt.itemsize
        for (M, N, K, cta) in ((256, 256, 128 // eb, (256, 256, 128 // eb)), (512, 768, 5 * 128 // eb, (256, 256, 0)), (2816, 3072, 256 // eb, (0, 0, 0))):
            A = torch.randint(-hi, hi + 1, (M, K), generator=g).float()
            B = torch.randint(-hi, hi + 1, (N, K), generator=g).float()
            C = torch.randint(-9, 10, (M, N), generator=g).float()
            X = torch.randint(-3, 4, (N,), generator=g).float()
            a, b = A.to(tdt).cuda(), B.to(tdt).cuda()
            ref = A.double() @ B.double().t()
            for out_dt in (torch.float32, torch.float16, torch.bfloat16):
                if out_dt != torch.float32 and float(ref.abs().max()) * 2 + 12 > (2048 if out_dt == torch.float16 else 256):
                    continue        # not every integer of that size is a float of that type
                mma = mh.tiled_mma_desc(atom, atom_layout=(2, 4, 1), cta_tile=cta)
                d = torch.zeros(M, N, dtype=out_dt, device="cuda")
                c = C.to(out_dt).cuda()
                names = [s["name"] for s in mh.gemm_explain(mma, T(d), T(a), T(b))["steps"]]
                assert names == ["gemm_mfma_tn_256_atom32<%s,%s,ops=0>" % ({2: "InF16" if tdt == torch.float16 else "InBF16", 1: "InFP8", 4: "InF32"}[eb],
                                                                             {torch.float32: "OutF32", torch.float16: "OutF16", torch.bfloat16: "OutBF16"}[out_dt])], names
                mh.gemm_(mma, T(d), T(a), T(b))
                torch.cuda.synchronize()
                assert torch.equal(d.cpu().double(), ref), (atom, M, N, K, out_dt)
                mh.gemm_(mma, T(d), T(a), T(b), T(c), 2.0)
                torch.cuda.synchronize()
                assert torch.equal(d.cpu().double(), 2 * ref + C.double()), (atom, M, N, K, out_dt, "C")
                x = X.cuda()
                ep = mh.gemm_epilogue(alpha=1.0, beta=1.0, op=_lib.MAP_MAX, operand=T(x, (M, N), (0, 1)))
                mh.gemm_ex_(mma, T(d), T(a), T(b), T(c), ep)
                torch.cuda.synchronize()
                assert torch.equal(d.cpu().double(), torch.maximum(ref + C.double(), X.double().expand(M, N))), (atom, M, N, K, out_dt, "max")
                dt_ = torch.zeros(N, M, dtype=out_dt, device="cuda")          # column-major D
                mh.gemm_(mma, T(dt_, (M, N), (1, M)), T(a), T(b))
                torch.cuda.synchronize()
                assert torch.equal(dt_.t().cpu().double(), ref), (atom, M, N, K, out_dt, "col-major")


def test_32x32_atoms_on_256_tiles_random_against_fp64_and_limits(mh):
    g = torch.Generator().manual_seed(3233)
    for atom, atom16, tdt, hi, tol in _atoms32(mh):
        M, N, K = 512, 512, 1024
        A = (torch.randn(M, K, generator=g) * K ** -0.5).to(tdt)
        B = (torch.randn(N, K, generator=g) * K ** -0.5).to(tdt)
        a, b = A.cuda(), B.cuda()
        d, d16 = torch.zeros(M, N, device="cuda"), torch.zeros(M, N, device="cuda")
        mh.gemm_(mh.tiled_mma_desc(atom, atom_layout=(2, 4, 1), cta_tile=(256, 256, 0)), T(d), T(a), T(b))
        mh.gemm_(mh.tiled_mma_desc(atom16, atom_layout=(2, 4, 1), cta_tile=(256, 256, 0)), T(d16), T(a), T(b))
        torch.cuda.synchronize()
        c64 = A.double().cuda() @ B.double().cuda().t()
        assert relerr(d, c64) <= tol, atom
        assert relerr(d, d16) <= 1e-5, atom            # both forms accumulate in fp32; only the order differs
    # whole tiles only, 128 bytes of K per tile row, 2 x 4 waves
    a = torch.zeros(256, 64, dtype=torch.float16, device="cuda")
    d = torch.zeros(256, 256, dtype=torch.float16, device="cuda")
    for kw, word in ((dict(atom_layout=(2, 4, 1), cta_tile=(256, 256, 32)), "32x32"), (dict(atom_layout=(2, 2, 1), cta_tile=(256, 256, 64)), "2 x 4 waves")):
        with pytest.raises(mh.MoyeError) as e:
            mh.gemm_(mh.tiled_mma_desc(mh.MFMA_F32_32x32x16_F16, **kw), T(d), T(a), T(a))
        assert word in str(e.value), str(e.value)
    a = torch.zeros(300, 64, dtype=torch.float16, device="cuda")
    d = torch.zeros(300, 300, dtype=torch.float16, device="cuda")
    with pytest.raises(mh.MoyeError) as e:
        mh.gemm_(mh.tiled_mma_desc(mh.MFMA_F32_32x32x16_F16, atom_layout=(2, 4, 1), cta_tile=(256, 256, 64)), T(d), T(a), T(a))
    assert "whole 256x256" in str(e.value)


def test_persistent_workgroups_on_more_tiles_than_cus_exact_on_integers(mh):
    """More 256x256 tiles than CUs: one workgroup per CU walks over the tiles, and a tile's first loads are
    requested before the epilogue of the tile before.  Every operand type, every output type, tile counts that are and are not
    multiples of the CUs (and of the XCDs), K of one to nine k-steps, with and without C; exact on small integers inside
    NaN frames, and bit-identical to a workgroup per tile."""
    from moye_hip import _lib
    g = torch.Generator(device="cuda").manual_seed(77)
    atoms = {torch.float16: mh.MFMA_F32_16x16x32_F16, torch.bfloat16: mh.MFMA_F32_16x16x32_BF16, torch.float8_e4m3fn: mh.MFMA_F32_16x16x32_FP8}
    for tdt, out_dt in ((torch.float16, torch.float16), (torch.bfloat16, torch.bfloat16), (torch.float8_e4m3fn, torch.bfloat16), (torch.float16, torch.bfloat16),
                        (torch.float8_e4m3fn, torch.float16), (torch.bfloat16, torch.float32), (torch.float16, torch.float32)):
        eb = tdt.itemsize
        for (M, N, K) in ((4352, 4096, 128 // eb), (8192, 8192, 256 // eb), (4352, 4352, 1152 // eb), (16384, 4352, 384 // eb)):
            A = torch.randint(-2, 3, (M, K), generator=g, device="cuda").float() * (torch.rand(M, K, generator=g, device="cuda") < 0.25)
            B = torch.randint(-2, 3, (N, K), generator=g, device="cuda").float() * (torch.rand(N, K, generator=g, device="cuda") < 0.25)
            C = torch.randint(-3, 4, (M, N), generator=g, device="cuda").float()
            a, b, c = A.to(tdt), B.to(tdt), C.to(out_dt)
            ref = A @ B.t()
            assert float(ref.abs().max()) * 2 + 3 <= 256
            got = {}
            for flags in (0, _lib.GEMM_NO_PERSIST):
                mma = mh.tiled_mma_desc(atoms[tdt], atom_layout=(2, 4, 1), cta_tile=(256, 256, 128 // eb), flags=flags)
                big = torch.full((M + 2, N + 16), float("nan"), dtype=out_dt, device="cuda")
                d = big[1:M + 1, 8:8 + N]
                name = mh.gemm_explain(mma, T(d), T(a), T(b))["steps"][0]["name"]
                assert ("persist=1" in name) == (flags == 0), name
                mh.gemm_(mma, T(d), T(a), T(b))
                torch.cuda.synchronize()
                assert torch.equal(d.float(), ref), (tdt, out_dt, M, N, K, flags)
                mh.gemm_(mma, T(d), T(a), T(b), T(c), 2.0)
                torch.cuda.synchronize()
                assert torch.equal(d.float(), 2 * ref + C), (tdt, out_dt, M, N, K, flags, "C")
                frame = big.clone()
                frame[1:M + 1, 8:8 + N] = float("nan")
                assert bool(torch.isnan(frame).all()), "stores outside D"
                got[flags] = d.clone()
            bits = torch.int16 if out_dt.itemsize == 2 else torch.int32
            assert torch.equal(got[0].contiguous().view(bits), got[_lib.GEMM_NO_PERSIST].contiguous().view(bits))
    # random operands: the two forms add in the same order, so they agree bit for bit
    for tdt, out_dt in ((torch.float16, torch.float16), (torch.float8_e4m3fn, torch.bfloat16)):
        M, N, K = 4608, 4352, 2048
        a = (torch.randn(M, K, generator=g, device="cuda") / 8).to(tdt)
        b = (torch.randn(N, K, generator=g, device="cuda") / 8).to(tdt)
        outs = []
        for flags in (0, _lib.GEMM_NO_PERSIST):
            d = torch.zeros(M, N, dtype=out_dt, device="cuda")
            mh.gemm_(mh.tiled_mma_desc(atoms[tdt], cta_tile=(0, 0, 0), flags=flags), T(d), T(a), T(b))
            torch.cuda.synchronize()
            outs.append(d)
        assert torch.equal(outs[0].view(torch.int16), outs[1].view(torch.int16))
        assert relerr(outs[0][:256], a[:256].double() @ b.double().t()) <= TOL16


@pytest.mark.parametrize("M,N", [(4100, 4104), (4096 + 64, 4096), (4096, 4096 + 136), (4352 + 200, 2816 + 248)])
def test_large_ragged_problem_runs_its_interior_on_256_tiles(mh, M, N):
    """Tile left to the library, M or N not a multiple of 256, at least 128 tiles of 256 x 256 inside: interior, right
    fringe and bottom fringe are three launches; exact on integers, with C and alpha, frame around D untouched."""
    K = 512
    g = torch.Generator().manual_seed(M + N)
    A = torch.randint(-4, 5, (M, K), generator=g).to(torch.float16)
    B = torch.randint(-4, 5, (N, K), generator=g).to(torch.float16)
    C = torch.randint(-9, 10, (M, N), generator=g).float()
    a, b, c = A.cuda(), B.cuda(), C.cuda()
    ref = (a.double() @ b.double().t())
    mma = mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, cta_tile=(0, 0, 0))
    big = torch.full((M + 2, N + 8), 77.0, device="cuda")
    d = big[1:M + 1, 4:N + 4]                       # 16-byte aligned window of a larger buffer
    mh.gemm_(mma, T(d), T(a), T(b))
    torch.cuda.synchronize()
    assert torch.equal(d.double(), ref)
    mh.gemm_(mma, T(d), T(a), T(b), T(c), 0.5)
    torch.cuda.synchronize()
    assert torch.equal(d.double(), 0.5 * ref + c.double())
    frame = big.clone()
    frame[1:M + 1, 4:N + 4] = 77.0
    assert bool((frame == 77.0).all()), "stores outside D"
    d16 = torch.zeros(M, N, dtype=torch.float16, device="cuda")
    mh.gemm_(mma, T(d16), T(a), T(b), None, 0.25)
    torch.cuda.synchronize()
    assert torch.equal(d16.double(), (0.25 * ref).half().double())
    dt_ = torch.zeros(N, M, device="cuda")                                  # column-major D
    mh.gemm_(mma, T(dt_, (M, N), (1, M)), T(a), T(b))
    torch.cuda.synchronize()
    assert torch.equal(dt_.t().double(), ref)


@pytest.mark.parametrize("split", [2, 4, 8])
def test_split_k_exact_on_integers(mh, split):
    """split_k > 1: K cut into equal ranges, fp32 partial products summed in ascending order in a second pass.
    Exact on integers whatever the tile, with C and alpha, with a column-major D, with an operand that is not K-major
    (its K-major copy and the partials share the workspace) and for a short A."""
    from moye_hip import _lib
    g = torch.Generator().manual_seed(40 + split)
    M, N, K = 256, 384, 2048
    A = torch.randint(-4, 5, (M, K), generator=g).to(torch.float16)
    B = torch.randint(-4, 5, (N, K), generator=g).to(torch.float16)
    C = torch.randint(-9, 10, (M, N), generator=g).float()
    a, b, c = A.cuda(), B.cuda(), C.cuda()
    ref = A.double() @ B.double().t()
    for cta, waves in (((128, 128, 32), (2, 2, 1)), ((0, 0, 0), (1, 1, 1)), ((128, 128, 64), (2, 2, 1))):
        mma = mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, atom_layout=waves, cta_tile=cta, split_k=split)
        d = torch.zeros(M, N, device="cuda")
        mh.gemm_(mma, T(d), T(a), T(b))
        torch.cuda.synchronize()
        assert torch.equal(d.cpu().double(), ref), (cta, "plain")
        mh.gemm_(mma, T(d), T(a), T(b), T(c), 2.0)
        torch.cuda.synchronize()
        assert torch.equal(d.cpu().double(), 2 * ref + C.double()), (cta, "alpha, C")
        dt_ = torch.zeros(N, M, device="cuda")
        mh.gemm_(mma, T(dt_, (M, N), (1, M)), T(a), T(b))
        torch.cuda.synchronize()
        assert torch.equal(dt_.t().cpu().double(), ref), (cta, "column-major D")
        at = A.t().contiguous().cuda()                      # A stored M-major: (M,K):(1,M)
        d.zero_()
        mh.gemm_(mma, T(d), T(at, (M, K), (1, M)), T(b))
        torch.cuda.synchronize()
        assert torch.equal(d.cpu().double(), ref), (cta, "M-major A")
    # 256x256 tile
    M2 = N2 = 512
    A2 = torch.randint(-4, 5, (M2, K), generator=g).to(torch.bfloat16)
    B2 = torch.randint(-4, 5, (N2, K), generator=g).to(torch.bfloat16)
    d2 = torch.zeros(M2, N2, dtype=torch.bfloat16, device="cuda")
    a2, b2 = A2.cuda(), B2.cuda()
    mh.gemm_(mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_BF16, atom_layout=(2, 4, 1), cta_tile=(256, 256, 64), split_k=split),
             T(d2), T(a2), T(b2), None, 0.125)
    torch.cuda.synchronize()
    assert torch.equal(d2.cpu().double(), (0.125 * (A2.double() @ B2.double().t())).to(torch.bfloat16).double())
    # short A
    d3 = torch.zeros(16, N, device="cuda")
    a16 = a[:16].contiguous()
    mh.gemm_(mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, cta_tile=(0, 0, 0), split_k=split), T(d3), T(a16), T(b))
    torch.cuda.synchronize()
    assert torch.equal(d3.cpu().double(), ref[:16])
    # workspace size is reported; a K that does not split is refused; UniversalFMA keeps its order
    need = mh.gemm_workspace_size(mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, split_k=split), T(d), T(a), T(b))
    assert need == split * M * N * 4
    ak, bk_ = a[:, :K - 8].contiguous(), b[:, :K - 8].contiguous()
    with pytest.raises(mh.MoyeError) as e:
        mh.gemm_(mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, split_k=split), T(d), T(ak), T(bk_))
    assert e.value.status == _lib.ERR_SHAPE
    af, bf = a.float(), b.float()
    with pytest.raises(mh.MoyeError) as e:
        mh.gemm_(mh.tiled_mma_desc(mh.MMA_UNIVERSAL_FMA, cta_tile=(32, 32, 8), split_k=split), T(d), T(af), T(bf))
    assert e.value.status == _lib.ERR_UNSUPPORTED


@pytest.mark.parametrize("out_dt", [torch.float32, torch.float16, torch.bfloat16])
def test_split_k_second_pass_in_pieces_of_four_gives_the_scalar_pass_its_bits(mh, out_dt):
    """The second pass of a K split sums four neighbouring columns per lane when D's rows start on whole pieces of four
    results; a D one element off that, or with an N that is no multiple of four, takes the element-wise pass.  Random
    data, with C, alpha and an operation with a bias row: the same bits from both."""
    from moye_hip import _lib
    g = torch.Generator(device="cuda").manual_seed(61)
    M, N, K = 384, 512, 4096
    a = (torch.randn(M, K, generator=g, device="cuda") * K ** -0.5).half()
    b = (torch.randn(N, K, generator=g, device="cuda") * K ** -0.5).half()
    c = torch.randn(M, N, generator=g, device="cuda").to(out_dt)
    bias = torch.randn(N, generator=g, device="cuda")
    for split in (2, 4):
        for cta, waves in (((128, 128, 64), (2, 2, 1)), ((256, 256, 64), (2, 4, 1))):
            if cta[0] == 256 and M % 256: continue
            mma = mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, atom_layout=waves, cta_tile=cta, split_k=split)
            for ep in (None, mh.gemm_epilogue(alpha=0.75, beta=-0.5, op=_lib.MAP_OPS["add"], operand=T(bias, (M, N), (0, 1)))):
                d1 = torch.zeros(M, N, dtype=out_dt, device="cuda")
                buf = torch.zeros(M, N + 8, dtype=out_dt, device="cuda")
                d2 = buf[:, 1:N + 1]                                    # rows start one element off
                need = mh.gemm_workspace_size(mma, T(d1), T(a), T(b), ep)
                ws = torch.empty(need + 256, dtype=torch.uint8, device="cuda")
                wp = (ws.data_ptr() + 255) // 256 * 256
                mh.gemm_ex_(mma, T(d1), T(a), T(b), T(c) if ep else None, ep, wp, need)
                mh.gemm_ex_(mma, T(d2), T(a), T(b), T(c) if ep else None, ep, wp, need)
                torch.cuda.synchronize()
                assert torch.equal(d1, d2), (out_dt, split, cta, ep is not None)
                assert float(buf[:, 0].abs().max()) == 0.0 and float(buf[:, N + 1:].abs().max()) == 0.0, "stores outside D"
    M = 256
    mma = mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, atom_layout=(2, 2, 1), cta_tile=(128, 128, 64), split_k=2)
    d = torch.zeros(M, N, dtype=out_dt, device="cuda")
    mh.gemm_(mma, T(d), T(a[:M]), T(b))
    torch.cuda.synchronize()
    assert relerr(d, a[:M].double() @ b.double().t()) <= TOL16


def test_split_k_long_k(mh):
    """A small C with a long K leaves most of the chip idle without a split: 256 x 256 x 65536 fp16."""
    g = torch.Generator().manual_seed(77)
    M = N = 256
    K = 65536
    A = (torch.randn(M, K, generator=g) * K ** -0.5).half()
    B = (torch.randn(N, K, generator=g) * K ** -0.5).half()
    a, b = A.cuda(), B.cuda()
    c64 = a.double() @ b.double().t()
    times = {}
    for split in (1, 16, 64, -1):
        d = torch.zeros(M, N, device="cuda")
        mma = mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, atom_layout=(2, 2, 1), cta_tile=(128, 128, 32), split_k=split)
        mh.gemm_(mma, T(d), T(a), T(b))
        torch.cuda.synchronize()
        assert relerr(d, c64) <= TOL16
        times[split] = mh.time_gemm(mma, T(d), T(a), T(b), None, 1.0, None, warmup=2, iters=10)
    print("256x256x65536 f16: " + ", ".join("split_k=%d %.1f us" % (k, v * 1e3) for k, v in times.items()))
    assert times[16] < times[1] and times[-1] < times[1]        # -1: the library chooses
    # the library's choice: tiles that fill the chip are not split (no workspace asked for)
    big = torch.zeros(2048, 2048, dtype=torch.float16, device="cuda")
    assert mh.gemm_workspace_size(mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, split_k=-1), T(big), T(big), T(big)) == 0
    assert mh.gemm_workspace_size(mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, split_k=-1), T(d), T(a), T(b)) > 0


def test_mfma_ceiling_probe(mh):
    """The MFMA-only yardstick: plausible numbers, and zeros never slower than dense random operands."""
    tf_r, ghz_r = mh.mfma_ceiling(mh.F16, True, 0.2)
    tf_z, ghz_z = mh.mfma_ceiling(mh.F16, False, 0.2)
    print("MFMA-only fp16: random %.0f TFLOP/s at %.2f GHz, zeros %.0f TFLOP/s at %.2f GHz" % (tf_r, ghz_r, tf_z, ghz_z))
    assert 500 < tf_r < 2600 and 500 < tf_z < 2600
    assert 0.5 < ghz_r < 2.6 and 0.5 < ghz_z < 2.6
    assert tf_z >= 0.95 * tf_r
    # the rate is the clock times 1024 flop per clock per SIMD (a 16x16x32 MFMA every 16 clocks), to a few per cent
    assert abs(tf_r / (ghz_r * 1e9 * 1024 * 1024 / 1e12) - 1) < 0.1
    for dt, lo_, hi in ((mh.F8E4M3, 1000, 5200), (mh.F32, 50, 160), (mh.BF16, 500, 2600)):
        tf, ghz = mh.mfma_ceiling(dt, True, 0.1)
        assert lo_ < tf < hi and 0.5 < ghz < 2.6, (dt, tf, ghz)
    with pytest.raises(mh.MoyeError):
        mh.mfma_ceiling(mh.F64, True, 0.1)


# ---------------------------------------------------------------------------------------------
# operand majors other than TN: transposed into a K-major workspace first
# ---------------------------------------------------------------------------------------------

def test_operand_majors_nn_nt_tt(mh):
    """A with its unit stride along M and/or B with its unit stride along N (the NN / NT / TT forms of
    src/arch/mma/make_mma_ops.jl:253-265).  Exact on integers; sizes that take the LDS-tiled transpose and
    sizes that take the generic one; the workspace size the query announces."""
    import ctypes as C
    from moye_hip import _lib
    g = torch.Generator().manual_seed(61)
    for (M, N, K) in ((256, 384, 128), (128, 128, 96), (512, 256, 1024)):
        A = torch.randint(-4, 5, (M, K), generator=g).to(torch.float16)
        B = torch.randint(-4, 5, (N, K), generator=g).to(torch.float16)
        ref = A.double() @ B.double().t()
        a_k, b_k = A.cuda(), B.cuda()                                   # K-major
        a_m, b_n = A.t().contiguous().cuda(), B.t().contiguous().cuda()  # M-major / N-major storage
        for a_major, b_major in (("m", "k"), ("k", "n"), ("m", "n")):
            ta = T(a_m, (M, K), (1, M)) if a_major == "m" else T(a_k)
            tb = T(b_n, (N, K), (1, N)) if b_major == "n" else T(b_k)
            d = torch.zeros(M, N, dtype=torch.float32, device="cuda")
            mma = mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, atom_layout=(2, 2, 1), cta_tile=(128, 128, 32))
            nbytes = C.c_size_t(0)
            _lib.check(_lib.lib().moye_gemm_workspace_size(C.byref(mma), C.byref(T(d)), C.byref(ta), C.byref(tb), C.byref(nbytes)))
            want = (M * K * 2 if a_major == "m" else 0) + (N * K * 2 if b_major == "n" else 0)
            assert want <= nbytes.value <= want + 512 + 16 * (M + N)
            mh.gemm_(mma, T(d), ta, tb)
            torch.cuda.synchronize()
            assert torch.equal(d.cpu().double(), ref), (M, N, K, a_major, b_major)
            with pytest.raises(mh.MoyeError) as e:
                mh.gemm_(mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, cta_tile=(128, 128, 32), flags=_lib.GEMM_NO_WORKSPACE),
                         T(d), ta, tb)
            assert "K-major" in str(e.value)


def test_operand_majors_other_element_types(mh):
    """The NN form (A stored M-major, B stored N-major) for fp8, bf16 and fp32 operands: their K-major copies go through
    the 1-, 2- and 4-byte LDS-tiled transposes.  Exact on integers."""
    cases = [(mh.MFMA_F32_16x16x32_BF16, torch.bfloat16), (mh.MFMA_F32_16x16x4_F32, torch.float32)]
    if hasattr(torch, "float8_e4m3fn"):
        cases.append((mh.MFMA_F32_16x16x32_FP8, torch.float8_e4m3fn))
    g = torch.Generator().manual_seed(62)
    for atom, tdt in cases:
        for (M, N, K) in ((256, 512, 256), (320, 192, 448)):
            A = torch.randint(-4, 5, (M, K), generator=g).float()
            B = torch.randint(-4, 5, (N, K), generator=g).float()
            ref = A.double() @ B.double().t()
            a_m, b_n = A.t().contiguous().to(tdt).cuda(), B.t().contiguous().to(tdt).cuda()
            d = torch.zeros(M, N, dtype=torch.float32, device="cuda")
            mh.gemm_(mh.tiled_mma_desc(atom, cta_tile=(0, 0, 0)), T(d), T(a_m, (M, K), (1, M)), T(b_n, (N, K), (1, N)))
            torch.cuda.synchronize()
            assert torch.equal(d.cpu().double(), ref), (tdt, M, N, K)


def test_config1_shape_on_the_matrix_cores(mh):
    """Benchmark configuration 1's operands (fp32 256^3, A and B column-major: the NN form) through the fp32 MFMA
    atom instead of UniversalFMA: tolerance 1e-5 against fp64."""
    M = N = K = 256
    rng = np.random.default_rng(1001)
    A = (rng.random((M, K), dtype=np.float32) * 2 - 1)
    Bkn = (rng.random((K, N), dtype=np.float32) * 2 - 1)
    a = torch.from_numpy(np.asfortranarray(A).T.copy()).cuda()       # column-major A: memory holds A' row-major
    b = torch.from_numpy(np.asfortranarray(Bkn).T.copy()).cuda()     # column-major (K,N): memory holds (N,K) row-major
    d = torch.zeros(N, M, device="cuda")                             # column-major C
    mh.gemm_(mh.tiled_mma_desc(mh.MFMA_F32_16x16x4_F32, atom_layout=(2, 2, 1), cta_tile=(128, 128, 16)),
             T(d, (M, N), (1, M)), T(a, (M, K), (1, M)), T(b, (N, K), (K, 1)))
    torch.cuda.synchronize()
    c64 = A.astype(np.float64) @ Bkn.astype(np.float64)
    err = to.relerr(d.t().cpu().numpy(), c64)
    print("config1 operands on the fp32 MFMA atom: rel err %.3e" % err)
    assert err <= 1e-5


# ---------------------------------------------------------------------------------------------
# residue tiles: M, N, K that the CTA tile does not divide
# ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("M,N,K", [(100, 130, 40), (129, 127, 72), (17, 300, 200), (384, 250, 64), (1, 1, 8), (255, 257, 1032)])
def test_residue_tiles_predicated(mh, M, N, K):
    """cta_tile left to the library (or MOYE_GEMM_PREDICATE with an explicit 128x128 tile): rows beyond M / N
    and k beyond K are read as zeros, stores stay inside D.  Exact on integers; the frame around D untouched."""
    from moye_hip import _lib
    g = torch.Generator().manual_seed(M * 7 + N)
    A = torch.randint(-4, 5, (M, K), generator=g).to(torch.float16)
    B = torch.randint(-4, 5, (N, K), generator=g).to(torch.float16)
    C = torch.randint(-9, 10, (M, N), generator=g).float()
    a, b, c = A.cuda(), B.cuda(), C.cuda()
    ref = A.double() @ B.double().t()
    for kw in (dict(cta_tile=(0, 0, 0)), dict(cta_tile=(128, 128, 32), flags=_lib.GEMM_PREDICATE)):
        for out_dt in (torch.float32, torch.float16):
            big = torch.full((M + 2, N + 3), 77.0, dtype=out_dt, device="cuda")     # D is a window of a larger buffer
            d = big[1:M + 1, 2:N + 2]
            c_out = c.to(out_dt).contiguous()
            mh.gemm_(mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, **kw), T(d), T(a), T(b), T(c_out), 1.0)
            torch.cuda.synchronize()
            assert torch.equal(d.cpu().double(), (ref + C.double()).to(out_dt).double()), (M, N, K, kw, out_dt)
            frame = big.clone()
            frame[1:M + 1, 2:N + 2] = 77.0
            assert bool((frame == 77.0).all()), "stores outside D"
    with pytest.raises(mh.MoyeError) as e:      # an explicit tile without the flag keeps the reference's assertion
        mh.gemm_(mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, cta_tile=(128, 128, 32)),
                 T(torch.zeros(M, N, device="cuda")), T(a), T(b))
    assert e.value.status == _lib.ERR_SHAPE or (M % 128 == 0 and N % 128 == 0 and K % 32 == 0)


# ---------------------------------------------------------------------------------------------
# byte offsets beyond 2^31 and 2^32
# ---------------------------------------------------------------------------------------------

def test_large_offsets_gemm_and_transpose(mh):
    """D of 49152 x 49152 fp16 (4.5 GiB) with K = 64: tile and row offsets exceed 2^32 bytes; and a 2-byte
    transpose of 65536 x 32768 (4 GiB each side).  Sampled against closed forms."""
    M = N = 49152
    K = 64
    g = torch.Generator().manual_seed(3)
    A = torch.randint(-3, 4, (M, K), generator=g).to(torch.float16)
    B = torch.randint(-3, 4, (N, K), generator=g).to(torch.float16)
    a, b = A.cuda(), B.cuda()
    d = torch.empty(M, N, dtype=torch.float16, device="cuda")
    mh.gemm_(mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, atom_layout=(2, 4, 1), cta_tile=(256, 256, 64)), T(d), T(a), T(b))
    torch.cuda.synchronize()
    for r0 in (0, 20000, M - 256):
        ref = A[r0:r0 + 256].double() @ B.double().t()
        assert torch.equal(d[r0:r0 + 256].cpu().double(), ref), r0
    del d
    # an operand whose rows lie 16 MiB apart: 256 rows span 4 GiB, beyond the 32-bit lane offsets of the hand-ordered
    # kernel, so the call stays on the kernel with 64-bit row addresses
    Mp, Kp, pitch = 256, 128, 1 << 23
    abuf = torch.zeros(Mp * pitch, dtype=torch.float16, device="cuda")
    Ap = torch.randint(-3, 4, (Mp, Kp), generator=g).to(torch.float16)
    abuf.view(Mp, pitch)[:, :Kp] = Ap.cuda()
    Bp = torch.randint(-3, 4, (512, Kp), generator=g).to(torch.float16)
    dp = torch.zeros(Mp, 512, dtype=torch.float32, device="cuda")
    mh.gemm_(mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, atom_layout=(2, 4, 1), cta_tile=(256, 256, 64)), T(dp), T(abuf, (Mp, Kp), (pitch, 1)), T(Bp.cuda()))
    torch.cuda.synchronize()
    assert torch.equal(dp.cpu().double(), Ap.double() @ Bp.double().t())
    del abuf, dp
    R, Cn = 65536, 32768
    src = torch.arange(R * Cn, dtype=torch.int64, device="cuda").to(torch.int16)   # wraps: value = index mod 2^16
    dst = torch.empty_like(src)
    mh.copyto_(T(dst, (R, Cn), (Cn, 1)), T(src, (R, Cn), (1, R)))
    torch.cuda.synchronize()
    sv, dv = src.view(Cn, R), dst.view(R, Cn)
    for (i, j) in ((0, 0), (R - 64, Cn - 64), (40000, 17000), (65000, 100)):
        assert torch.equal(dv[i:i + 64, j:j + 64], sv[j:j + 64, i:i + 64].t()), (i, j)


@pytest.mark.parametrize("out_dt", ["float32", "float16", "bfloat16"])
@pytest.mark.parametrize("flags", ["default", "wave4", "128", "64", "128 atom32"])
def test_every_layout_of_c(mh, out_dt, flags):
    """C through the MFMA kernels' epilogues (256x256 tile, lock-step and hand-ordered; 128x128; 64x64; 32x32 atoms): row-major with aligned rows (read in 128-bit pieces of whole rows),
    a row pitch and a base that are not multiples of 16 bytes, column-major, and D itself (in place).  Small integers:
    every result is exact, so a misplaced piece of C shows as a hard mismatch."""
    from moye_hip import _lib
    out_dt = getattr(torch, out_dt)
    M, N, K = 512, 768, 256
    g = torch.Generator().manual_seed(77)
    A = torch.randint(-3, 4, (M, K), generator=g).to(torch.float16)
    B = torch.randint(-3, 4, (N, K), generator=g).to(torch.float16)
    C0 = torch.randint(-8, 9, (M, N), generator=g).to(out_dt)
    a, b = A.cuda(), B.cuda()
    if flags in ("default", "wave4"):
        mma = mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, atom_layout=(2, 4, 1), cta_tile=(256, 256, 64),
                                flags=_lib.GEMM_WAVE4 if flags == "wave4" else 0)
    elif flags == "128 atom32":
        mma = mh.tiled_mma_desc(mh.MFMA_F32_32x32x16_F16, atom_layout=(2, 2, 1), cta_tile=(128, 128, 32))
    else:
        mma = mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, atom_layout=(2, 2, 1), cta_tile=(int(flags), int(flags), 64))
    want = (A.double() @ B.double().t()) * 0.5 + C0.double()
    if out_dt != torch.float32:
        want = want.to(out_dt).double()  # halves of odd sums round to even in the 16-bit types
    forms = {}
    forms["rows"] = (C0.cuda(), (N, 1), 0)
    padded = torch.zeros(M, N + 1, dtype=out_dt)
    padded[:, :N] = C0
    forms["pitch N + 1"] = (padded.cuda(), (N + 1, 1), 0)
    shifted = torch.zeros(M * N + 1, dtype=out_dt)
    shifted[1:] = C0.reshape(-1)
    forms["base off by one element"] = (shifted.cuda(), (N, 1), 1)
    forms["column-major"] = (C0.t().contiguous().cuda(), (1, M), 0)
    for name, (c, strides, off) in forms.items():
        d = torch.zeros(M, N, dtype=out_dt, device="cuda")
        cc = T(c.reshape(-1)[off:], (M, N), strides)
        mh.gemm_(mma, T(d), T(a), T(b), cc, 0.5)
        torch.cuda.synchronize()
        assert torch.equal(d.cpu().double(), want), name
    d = C0.cuda().clone()
    mh.gemm_(mma, T(d), T(a), T(b), T(d), 0.5)
    torch.cuda.synchronize()
    assert torch.equal(d.cpu().double(), want), "in place"


# ---------------------------------------------------------------------------------------------
# moye_gemm_ex: the workspace comes from the caller
# ---------------------------------------------------------------------------------------------

def test_gemm_ex_takes_the_callers_workspace(mh):
    """Split-K partials and K-major copies go into the caller's buffer: same bits as moye_gemm with the library's own
    workspace; a buffer that is too small, misaligned or missing is refused before anything is launched; two streams
    with two workspaces do not disturb each other."""
    from moye_hip import _lib
    g = torch.Generator().manual_seed(90)
    M, N, K = 256, 384, 2048
    A = torch.randint(-4, 5, (M, K), generator=g).to(torch.float16)
    B = torch.randint(-4, 5, (N, K), generator=g).to(torch.float16)
    a, b = A.cuda(), B.cuda()
    a_m = A.t().contiguous().cuda()
    ref = A.double() @ B.double().t()
    mma = mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, atom_layout=(2, 2, 1), cta_tile=(128, 128, 32), split_k=4)
    ta_m = T(a_m, (M, K), (1, M))
    d = torch.zeros(M, N, device="cuda")
    need = mh.gemm_workspace_size(mma, T(d), ta_m, T(b))
    assert need >= 4 * M * N * 4 + M * K * 2
    ws = torch.full((need + 256,), 0x5a, dtype=torch.uint8, device="cuda")
    base = (ws.data_ptr() + 255) // 256 * 256
    mh.gemm_ex_(mma, T(d), ta_m, T(b), None, mh.gemm_epilogue(alpha=0.5), base, need)
    d_lib = torch.zeros(M, N, device="cuda")
    mh.gemm_(mma, T(d_lib), ta_m, T(b), None, 0.5)
    torch.cuda.synchronize()
    assert torch.equal(d.cpu().double(), 0.5 * ref) and torch.equal(d, d_lib)
    # refused: too small, misaligned, missing
    for args in ((base, need - 256), (base + 16, need), (None, 0)):
        with pytest.raises(mh.MoyeError) as e:
            mh.gemm_ex_(mma, T(d), ta_m, T(b), None, None, *args)
        assert e.value.status in (_lib.ERR_ARG, _lib.ERR_ALIGN)
    # a plain TN call needs no workspace and may pass none
    plain = mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, atom_layout=(2, 2, 1), cta_tile=(128, 128, 32))
    d.zero_()
    mh.gemm_ex_(plain, T(d), T(a), T(b))
    torch.cuda.synchronize()
    assert torch.equal(d.cpu().double(), ref)
    # two streams, each with its own workspace (and, through moye_gemm, each with the library's per-stream one)
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    ws2 = torch.zeros(need + 256, dtype=torch.uint8, device="cuda")
    base2 = (ws2.data_ptr() + 255) // 256 * 256
    B2 = torch.randint(-4, 5, (N, K), generator=g).to(torch.float16)
    b2 = B2.cuda()
    ref2 = A.double() @ B2.double().t()
    d1, d2 = torch.zeros(M, N, device="cuda"), torch.zeros(M, N, device="cuda")
    e1, e2 = torch.zeros(M, N, device="cuda"), torch.zeros(M, N, device="cuda")
    torch.cuda.synchronize()
    for _ in range(8):
        mh.gemm_ex_(mma, T(d1), ta_m, T(b), None, None, base, need, stream=s1.cuda_stream)
        mh.gemm_ex_(mma, T(d2), ta_m, T(b2), None, None, base2, need, stream=s2.cuda_stream)
        mh.gemm_(mma, T(e1), ta_m, T(b), stream=s1.cuda_stream)
        mh.gemm_(mma, T(e2), ta_m, T(b2), stream=s2.cuda_stream)
    torch.cuda.synchronize()
    assert torch.equal(d1.cpu().double(), ref) and torch.equal(d2.cpu().double(), ref2)
    assert torch.equal(e1.cpu().double(), ref) and torch.equal(e2.cpu().double(), ref2)
    mh.gemm_release_workspace()
    mh.gemm_(mma, T(e1), ta_m, T(b))        # allocates afresh
    torch.cuda.synchronize()
    assert torch.equal(e1.cpu().double(), ref)


def test_host_threads_with_their_own_streams_and_workspaces(mh):
    """Four host threads call the library at the same time (ctypes drops the interpreter lock during a call), each on its
    own stream with its own workspace: split-K partials, K-major copies of an M-major operand, a ragged problem, a
    transposing copy and an axpby!.  Every thread's results are exact on small integers, every time."""
    import threading
    M, N, K = 256, 384, 2048
    mma = mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, atom_layout=(2, 2, 1), cta_tile=(128, 128, 32), split_k=4)
    lib_choice = mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16)
    errors = []

    def work(seed):
        try:
            g = torch.Generator().manual_seed(seed)
            A = torch.randint(-4, 5, (M, K), generator=g).to(torch.float16)
            B = torch.randint(-4, 5, (N, K), generator=g).to(torch.float16)
            Ar = torch.randint(-4, 5, (300, 520), generator=g).to(torch.float16)
            Br = torch.randint(-4, 5, (1000, 520), generator=g).to(torch.float16)
            S = torch.randint(-1000, 1000, (512, 1024), generator=g, dtype=torch.int32)
            ref, ref_r = A.double() @ B.double().t(), Ar.double() @ Br.double().t()
            st = torch.cuda.Stream()
            with torch.cuda.stream(st):
                a_m, b, ar, br, src = A.t().contiguous().cuda(), B.cuda(), Ar.cuda(), Br.cuda(), S.cuda()
                d, dr = torch.zeros(M, N, device="cuda"), torch.zeros(300, 1000, device="cuda")
                dst = torch.zeros(1024, 512, dtype=torch.int32, device="cuda")
                y = torch.ones(M, N, device="cuda")
                ta_m = T(a_m, (M, K), (1, M))
                need = mh.gemm_workspace_size(mma, T(d), ta_m, T(b))
                ws = torch.zeros(need + 256, dtype=torch.uint8, device="cuda")
                base = (ws.data_ptr() + 255) // 256 * 256
            st.synchronize()
            for it in range(40):
                mh.gemm_ex_(mma, T(d), ta_m, T(b), None, None, base, need, stream=st.cuda_stream)
                mh.gemm_ex_(lib_choice, T(dr), T(ar), T(br), stream=st.cuda_stream)
                mh.copyto_(T(dst, (512, 1024), (1, 512)), T(src), stream=st.cuda_stream)
                mh.axpby_(1.0, T(d), 0.0, T(y), stream=st.cuda_stream)
                st.synchronize()
                with torch.cuda.stream(st):     # (torch's own work on this thread's stream too, so that it is ordered with the calls)
                    got = [t.cpu() for t in (d, dr, dst, y)]
                    d.zero_(), dr.zero_(), dst.zero_(), y.fill_(1.0)
                st.synchronize()
                if not (torch.equal(got[0].double(), ref) and torch.equal(got[1].double(), ref_r)
                        and torch.equal(got[2], S.t()) and torch.equal(got[3].double(), ref)):
                    errors.append("thread %d, pass %d: wrong result (%s)" % (seed, it, [
                        bool(torch.equal(got[0].double(), ref)), bool(torch.equal(got[1].double(), ref_r)),
                        bool(torch.equal(got[2], S.t())), bool(torch.equal(got[3].double(), ref))]))
                    return
        except Exception as e:  # noqa: BLE001 - reported below, in the test's own thread
            errors.append("thread %d: %r" % (seed, e))

    threads = [threading.Thread(target=work, args=(100 + i,)) for i in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not errors, errors


# ---------------------------------------------------------------------------------------------
# exactly what bench.py times, at the size it times
# ---------------------------------------------------------------------------------------------

def _bench_mma(mh):
    """The descriptor of bench.py's headline leg: CTA tile 256x256x64, 2x4 waves, fp16 in and out."""
    return mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, atom_layout=(2, 4, 1), tile=(256, 256, 64), cta_tile=(256, 256, 64))


def test_bench_descriptor_f16_4096_against_fp64(mh):
    """fp16 TN 4096^3, seed 1003, values normal(0,1)/sqrt(K), fp16 out, through the 256x256x64 kernel on all 256 CUs;
    every row against the fp64 product of the rounded inputs: max|D - D64| / max|D64| <= 1e-2."""
    M = N = K = 4096
    g = torch.Generator().manual_seed(1003)
    A = (torch.randn(M, K, generator=g) / K ** 0.5).half()
    B = (torch.randn(N, K, generator=g) / K ** 0.5).half()
    a, b = A.cuda(), B.cuda()
    d = torch.zeros(M, N, dtype=torch.float16, device="cuda")
    mh.gemm_(_bench_mma(mh), T(d), T(a), T(b))
    torch.cuda.synchronize()
    c64 = a.double() @ b.double().t()
    err = relerr(d, c64)
    rows = np.random.default_rng(1).choice(M, 32, replace=False)
    host = A[rows].double().numpy() @ B.double().numpy().T               # the GPU fp64 product checked on the host
    assert np.allclose(c64[rows].cpu().numpy(), host, rtol=1e-12, atol=1e-12)
    ref = to.gemm_universal_fma(A[rows[:8]].float().numpy(), B.float().numpy(), np.zeros((8, N), np.float32),
                                "f16", "f16").astype(np.float16)
    print("bench descriptor f16 4096^3 (256x256x64): rel err %.3e (reference arithmetic on 8 rows: %.3e)"
          % (err, to.relerr(ref, host[:8])))
    assert err <= TOL16
    # the named tile of the baseline's config 3 gives the same product up to the order of the sum
    d128 = torch.zeros_like(d)
    mh.gemm_(mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, atom_layout=(2, 2, 1), cta_tile=(128, 128, 32)), T(d128), T(a), T(b))
    torch.cuda.synchronize()
    assert relerr(d128, c64) <= TOL16
    assert float((d.double() - d128.double()).abs().max()) <= 2 ** -8 * float(c64.abs().max())
    # ... and so does the 128x128x64 tile on the load-to-LDS kernel (bench.py times it too)
    d128l = torch.zeros_like(d)
    mh.gemm_(mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, atom_layout=(2, 2, 1), cta_tile=(128, 128, 64)), T(d128l), T(a), T(b))
    torch.cuda.synchronize()
    assert relerr(d128l, c64) <= TOL16
    assert float((d.double() - d128l.double()).abs().max()) <= 2 ** -8 * float(c64.abs().max())


@pytest.mark.parametrize("out_dt", ["float16", "float32"])
def test_bench_descriptor_every_cta_exact_on_integers(mh, out_dt):
    """4096 x 4096 x 512 on small integers through the bench descriptor: all 256 CTA positions of the XCD-aware
    order, non-temporal stores on, bit for bit (every product and sum is exact in fp32 and in fp16)."""
    out_dt = getattr(torch, out_dt)
    M = N = 4096
    K = 512
    g = torch.Generator().manual_seed(1103)
    A = torch.randint(-2, 3, (M, K), generator=g).half()
    B = torch.randint(-2, 3, (N, K), generator=g).half()
    a, b = A.cuda(), B.cuda()
    d = torch.full((M, N), float("nan"), dtype=out_dt, device="cuda")
    ks = kernels_of(mh, _bench_mma(mh), T(d), T(a), T(b))
    assert len(ks) == 1 and ks[0]["name"].startswith("gemm_mfma_tn_256_w4<W4F16L,") and ks[0]["grid"] == "256x1", ks
    mh.gemm_(_bench_mma(mh), T(d), T(a), T(b))
    torch.cuda.synchronize()
    want = (a.float() @ b.float().t())           # exact: |sum| <= 4 * 512 = 2048, an integer fp16 holds
    assert float(want.abs().max()) <= 2048
    assert torch.equal(d.float(), want)
    # the 1024 workgroups of the 128x128x64 tile on the load-to-LDS kernel, two to a CU
    d.fill_(float("nan"))
    mh.gemm_(mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, atom_layout=(2, 2, 1), cta_tile=(128, 128, 64)), T(d), T(a), T(b))
    torch.cuda.synchronize()
    assert torch.equal(d.float(), want)


@pytest.mark.parametrize("majors", ["mn", "mk", "kn"])
def test_operand_majors_every_cta_exact_on_integers(mh, majors):
    """4096 x 4096 x 512 on small integers with A stored M-major and / or B stored N-major (the reference's own operand
    layout: MoYeArray(Array) is column-major, src/array.jl:101-103), MOYE_GEMM_NO_WORKSPACE: all 256 CTA positions of the
    256 x 256 tile on the transposing fragment reads, for fp16, bf16, fp8 and fp32 operands, named tile and the library's
    choice, bit for bit."""
    from moye_hip import _lib
    M = N = 4096
    K = 512
    g = torch.Generator().manual_seed(1104)
    cases = [(torch.float16, mh.MFMA_F32_16x16x32_F16, 64, torch.float16), (torch.bfloat16, mh.MFMA_F32_16x16x32_BF16, 64, torch.bfloat16),
             (torch.float32, mh.MFMA_F32_16x16x4_F32, 32, torch.float16)]
    if hasattr(torch, "float8_e4m3fn"):
        cases.append((torch.float8_e4m3fn, mh.MFMA_F32_16x16x32_FP8, 128, torch.bfloat16))
    for tdt, atom, bk, out16 in cases:
        A = torch.randint(-2, 3, (M, K), generator=g).float()
        B = torch.randint(-2, 3, (N, K), generator=g).float()
        a_k, b_k = A.to(tdt).cuda(), B.to(tdt).cuda()
        a_m, b_n = A.t().contiguous().to(tdt).cuda(), B.t().contiguous().to(tdt).cuda()
        ta = T(a_m, (M, K), (1, M)) if majors[0] == "m" else T(a_k)
        tb = T(b_n, (N, K), (1, N)) if majors[1] == "n" else T(b_k)
        want = A.cuda() @ B.cuda().t()
        assert float(want.abs().max()) <= 2048
        for cta in ((256, 256, bk), (0, 0, 0)):
            mma = mh.tiled_mma_desc(atom, atom_layout=(2, 4, 1), cta_tile=cta, flags=_lib.GEMM_NO_WORKSPACE)
            for out_dt in (out16, torch.float32):
                d = torch.full((M, N), float("nan"), dtype=out_dt, device="cuda")
                assert mh.gemm_workspace_size(mh.tiled_mma_desc(atom, atom_layout=(2, 4, 1), cta_tile=cta), T(d), ta, tb) == 0
                mh.gemm_(mma, T(d), ta, tb)
                torch.cuda.synchronize()
                assert torch.equal(d.float(), want), (tdt, out_dt, majors, cta)
        # with C, alpha and a column-major D (the kernel then runs the transposed problem: the majors swap with the operands)
        C0 = torch.randint(-8, 9, (M, N), generator=g).float().cuda()
        dt_ = torch.zeros(N, M, dtype=torch.float32, device="cuda")
        mh.gemm_(mh.tiled_mma_desc(atom, atom_layout=(2, 4, 1), cta_tile=(256, 256, bk), flags=_lib.GEMM_NO_WORKSPACE),
                 T(dt_, (M, N), (1, M)), ta, tb, T(C0), 0.5)
        torch.cuda.synchronize()
        assert torch.equal(dt_.t(), 0.5 * want + C0), (tdt, majors, "column-major D, C, alpha")


@pytest.mark.parametrize("majors", ["mk", "kn", "mn"])
def test_operand_majors_on_128_tiles_every_type_exact_on_integers(mh, majors):
    """Mid-size problems with A stored M-major and / or B stored N-major on the 128 x 128 tile of the hand-ordered kernel
    (two workgroups per CU): fp16, bf16, fp8 and fp32 operands read where they lie, the tile named and left to the
    library, MOYE_GEMM_NO_WORKSPACE; 2048 x 2304 x 384 (288 tiles: every CU holds two workgroups for part of the run) on
    small integers, bit for bit; with C, alpha and a column-major D as well."""
    from moye_hip import _lib
    M, N, K = 2048, 2304, 384
    g = torch.Generator().manual_seed(1108)
    cases = [(torch.float16, mh.MFMA_F32_16x16x32_F16, 64, torch.float16), (torch.bfloat16, mh.MFMA_F32_16x16x32_BF16, 64, torch.float32),
             (torch.float32, mh.MFMA_F32_16x16x4_F32, 32, torch.float32)]
    if hasattr(torch, "float8_e4m3fn"):
        cases.append((torch.float8_e4m3fn, mh.MFMA_F32_16x16x32_FP8, 128, torch.bfloat16))
    for tdt, atom, bk, out_dt in cases:
        A = torch.randint(-2, 3, (M, K), generator=g).float()
        B = torch.randint(-2, 3, (N, K), generator=g).float()
        a_k, b_k = A.to(tdt).cuda(), B.to(tdt).cuda()
        a_m, b_n = A.t().contiguous().to(tdt).cuda(), B.t().contiguous().to(tdt).cuda()
        ta = T(a_m, (M, K), (1, M)) if majors[0] == "m" else T(a_k)
        tb = T(b_n, (N, K), (1, N)) if majors[1] == "n" else T(b_k)
        want = A.cuda() @ B.cuda().t()
        assert float(want.abs().max()) <= 256          # exact in bf16 too
        for cta, waves in (((128, 128, bk), (2, 2, 1)), ((0, 0, 0), (1, 1, 1))):
            mma = mh.tiled_mma_desc(atom, atom_layout=waves, cta_tile=cta, flags=_lib.GEMM_NO_WORKSPACE)
            d = torch.full((M, N), float("nan"), dtype=out_dt, device="cuda")
            ks = kernels_of(mh, mma, T(d), ta, tb)
            want_name = ("amaj=%d" % (majors[0] == "m"), "bmaj=%d" % (majors[1] == "n"), "tile=128", "waves=4")
            assert len(ks) == 1 and ks[0]["family"] == "gemm_mfma_tn_256_w4" and all(w in ks[0]["name"] for w in want_name), (tdt, cta, ks)
            mh.gemm_(mma, T(d), ta, tb)
            torch.cuda.synchronize()
            assert torch.equal(d.float(), want), (tdt, majors, cta)
        C0 = torch.randint(-8, 9, (M, N), generator=g).float().cuda()
        dt_ = torch.zeros(N, M, dtype=torch.float32, device="cuda")
        mh.gemm_(mh.tiled_mma_desc(atom, atom_layout=(2, 2, 1), cta_tile=(128, 128, bk), flags=_lib.GEMM_NO_WORKSPACE),
                 T(dt_, (M, N), (1, M)), ta, tb, T(C0), 0.5)
        torch.cuda.synchronize()
        assert torch.equal(dt_.t(), 0.5 * want + C0), (tdt, majors, "column-major D, C, alpha")


def test_operand_majors_wide_types_random_and_workspace_rule(mh):
    """fp8 and fp32 NN (A M-major, B N-major) at 4096^3 on random data against fp64 (tolerances 1e-2 / 1e-5), read where
    they lie; and the one case that still copies: an element-wise epilogue operation, which moye_gemm_ex_workspace_size
    announces and MOYE_GEMM_NO_WORKSPACE refuses."""
    from moye_hip import _lib
    M = N = K = 4096
    g = torch.Generator().manual_seed(1106)
    A = torch.randn(M, K, generator=g) / K ** 0.5
    B = torch.randn(N, K, generator=g) / K ** 0.5
    cases = [(torch.float32, mh.MFMA_F32_16x16x4_F32, 32, 1e-5, 1.0)]
    if hasattr(torch, "float8_e4m3fn"):
        cases.append((torch.float8_e4m3fn, mh.MFMA_F32_16x16x32_FP8, 128, 1e-2, 64.0))
    for tdt, atom, bk, tol, scale in cases:
        a_k, b_k = (A * scale).to(tdt).cuda(), (B * scale).to(tdt).cuda()
        a_m, b_n = a_k.float().t().contiguous().to(tdt), b_k.float().t().contiguous().to(tdt)
        c64 = a_k.double() @ b_k.double().t() if tdt == torch.float32 else a_k.float().double() @ b_k.float().double().t()
        ta, tb = T(a_m, (M, K), (1, M)), T(b_n, (N, K), (1, N))
        mma = mh.tiled_mma_desc(atom, atom_layout=(2, 4, 1), cta_tile=(256, 256, bk), flags=_lib.GEMM_NO_WORKSPACE)
        d = torch.zeros(M, N, dtype=torch.float32, device="cuda")
        mh.gemm_(mma, T(d), ta, tb)
        torch.cuda.synchronize()
        assert relerr(d, c64) <= tol, tdt
        # an operation in the epilogue: the hand-ordered kernel has none, so these operands need their K-major copies
        plain = mh.tiled_mma_desc(atom, atom_layout=(2, 4, 1), cta_tile=(256, 256, bk))
        ep = mh.gemm_epilogue(alpha=1.0, op=_lib.MAP_ABS)
        need = mh.gemm_workspace_size(plain, T(d), ta, tb, ep)
        assert need >= 2 * M * K * a_k.element_size() and mh.gemm_workspace_size(plain, T(d), ta, tb) == 0
        with pytest.raises(mh.MoyeError):
            mh.gemm_ex_(mma, T(d), ta, tb, None, ep)
        ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        mh.gemm_ex_(plain, T(d), ta, tb, None, ep, ws.data_ptr(), need)
        torch.cuda.synchronize()
        assert relerr(d, c64.abs()) <= tol, tdt


def test_fp32_full_grid_exact_on_integers(mh):
    """fp32 operands on the hand-ordered kernel's whole-line form (eight v_mfma_f32_16x16x4_f32 in a row per accumulator
    and k-step): 8192 x 8192 x 256 on small integers, all 1024 CTA positions (four rounds of tiles, the K rotation over
    XCDs on), bit for bit."""
    M = N = 8192
    K = 256
    g = torch.Generator().manual_seed(1105)
    A = torch.randint(-3, 4, (M, K), generator=g).float()
    B = torch.randint(-3, 4, (N, K), generator=g).float()
    a, b = A.cuda(), B.cuda()
    d = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    mh.gemm_(mh.tiled_mma_desc(mh.MFMA_F32_16x16x4_F32, atom_layout=(2, 4, 1), cta_tile=(256, 256, 32)), T(d), T(a), T(b))
    torch.cuda.synchronize()
    want = a.double() @ b.double().t()
    assert torch.equal(d.double(), want)


# ---------------------------------------------------------------------------------------------
# fused epilogue: D = op(alpha * A * B' + beta * C, operand)   (moye_gemm_ex)
# ---------------------------------------------------------------------------------------------

_NP_OF = {"float32": ("f32", np.float32), "float16": ("f16", np.float16), "bfloat16": ("bf16", np.float32)}


def _epilogue_case(mh, mma, M, N, K, out_name, op, operand_kind, seed, col_major_d=False, alpha=0.375, beta=-1.25,
                   operand_in_out_type=False, in_dt=torch.float16, instance=None):
    """Small-integer A and B (the fp32 accumulator is exact whatever the order of the sum), random C and operand:
    every bit of D is then fixed by the epilogue's arithmetic, which the oracle composes from axpby! and broadcast."""
    out_dt = getattr(torch, out_name)
    tag, _ = _NP_OF[out_name]
    g = torch.Generator().manual_seed(seed)
    A = torch.randint(-3, 4, (M, K), generator=g).float().to(in_dt)
    B = torch.randint(-3, 4, (N, K), generator=g).float().to(in_dt)
    C0 = torch.randn(M, N, generator=g).to(out_dt)
    x_dt = out_dt if operand_in_out_type else torch.float32
    if operand_kind == "row":        # one value per column n, repeated down the rows: (M,N):(0,1)
        X0, xs = (torch.randn(N, generator=g) * 4).to(x_dt), (0, 1)
    elif operand_kind == "col":      # one value per row m: (M,N):(1,0)
        X0, xs = (torch.randn(M, generator=g) * 4).to(x_dt), (1, 0)
    elif operand_kind == "full":     # a whole (M,N) array, column-major
        X0, xs = (torch.randn(N, M, generator=g) * 4).to(x_dt), (1, M)
    else:
        X0, xs = None, None
    if op == "div" and X0 is not None:
        X0 = X0 + torch.where(X0 >= 0, 1.0, -1.0).to(x_dt)     # keep away from zero
    acc = (A.float() @ B.float().t()).numpy()
    assert np.abs(acc).max() < 2 ** 20
    a, b, c = A.cuda(), B.cuda(), C0.cuda()
    xd = X0.cuda() if X0 is not None else None
    ep = mh.gemm_epilogue(alpha=alpha, beta=beta, op=mh._lib.MAP_OPS[op],
                          operand=T(xd.reshape(-1), (M, N), xs) if xd is not None else None, scalar=1.5)
    if col_major_d:
        d = torch.zeros(N, M, dtype=out_dt, device="cuda")
        td = T(d, (M, N), (1, M))
    else:
        d = torch.zeros(M, N, dtype=out_dt, device="cuda")
        td = T(d)
    need = mh.gemm_workspace_size(mma, td, T(a), T(b))
    ws = torch.zeros(max(need, 1) + 256, dtype=torch.uint8, device="cuda")
    if instance is not None:      # the test means one kernel instance: the plan must say so
        ks = kernels_of(mh, mma, td, T(a), T(b), T(c) if beta != 0 else None, ep)
        assert len(ks) == 1 and all(part in ks[0]["name"] for part in instance), (instance, ks)
    mh.gemm_ex_(mma, td, T(a), T(b), T(c) if beta != 0 else None, ep, (ws.data_ptr() + 255) // 256 * 256, need)
    torch.cuda.synchronize()
    got = (d.t() if col_major_d else d).cpu()
    cnp = C0.float().numpy().astype(np.float16) if tag == "f16" else C0.float().numpy()
    if X0 is None:
        xnp = None
    else:
        xf = X0.float().numpy()
        xnp = xf[None, :] if operand_kind == "row" else xf[:, None] if operand_kind == "col" else xf.T
    want = to.gemm_epilogue(acc, alpha, beta, cnp if beta != 0 else None, op, xnp, 1.5, tag)
    gb = got.float().numpy().view(np.uint32)
    wb = want.astype(np.float32).view(np.uint32)
    bad = np.argwhere(gb != wb)
    assert bad.size == 0, "%d of %d elements differ, first at %s: got %r want %r" % (
        len(bad), M * N, bad[0], got.float().numpy()[tuple(bad[0])], want.astype(np.float32)[tuple(bad[0])])


@pytest.mark.parametrize("out_name", ["float32", "float16", "bfloat16"])
@pytest.mark.parametrize("op", ["identity", "add", "sub", "mul", "div", "max", "min", "neg", "abs"])
def test_fused_epilogue_every_op_bit_exact(mh, out_name, op):
    """256x256 tile (the default for this size): every operation with a per-column vector, alpha and beta that make
    the products round; bit for bit against the oracle."""
    mma = mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, atom_layout=(2, 4, 1), cta_tile=(256, 256, 64))
    _epilogue_case(mh, mma, 512, 768, 128, out_name, op, "row", 300 + len(op))


@pytest.mark.parametrize("kernel", ["256", "128", "64", "128 atom32", "predicated", "short-M", "split-K", "library", "ragged", "thin fringes"])
@pytest.mark.parametrize("operand_kind", ["row", "col", "full", "scalar"])
def test_fused_epilogue_every_kernel_and_operand(mh, kernel, operand_kind):
    """bias-style add with beta * C through every kernel family that writes D, row-major and column-major D, operands
    as row vector, column vector, whole array and scalar, in fp32 and in D's type."""
    from moye_hip import _lib
    F16 = mh.MFMA_F32_16x16x32_F16
    M, N, K = 512, 512, 128
    if kernel == "256":
        mma = mh.tiled_mma_desc(F16, atom_layout=(2, 4, 1), cta_tile=(256, 256, 64))
    elif kernel == "128":
        mma = mh.tiled_mma_desc(F16, atom_layout=(2, 2, 1), cta_tile=(128, 128, 32))
    elif kernel == "64":
        mma = mh.tiled_mma_desc(F16, atom_layout=(2, 2, 1), cta_tile=(64, 64, 32))
    elif kernel == "128 atom32":
        mma = mh.tiled_mma_desc(mh.MFMA_F32_32x32x16_F16, atom_layout=(2, 2, 1), cta_tile=(128, 128, 32))
    elif kernel == "predicated":
        mma = mh.tiled_mma_desc(F16, cta_tile=(0, 0, 0))
        M, N, K = 200, 136, 72
    elif kernel == "short-M":
        mma = mh.tiled_mma_desc(F16, cta_tile=(0, 0, 0))
        M, N, K = 24, 640, 256
    elif kernel == "split-K":
        mma = mh.tiled_mma_desc(F16, atom_layout=(2, 2, 1), cta_tile=(128, 128, 32), split_k=4)
        M, N, K = 256, 384, 512
    elif kernel == "ragged":     # 256x256 tiles that reach beyond M and N (the guarded instance)
        mma = mh.tiled_mma_desc(F16, cta_tile=(0, 0, 0))
        M, N, K = 4096 + 40, 2048 + 72, 64
    elif kernel == "thin fringes":     # interior on 256x256 tiles, both fringes on the short-M kernel
        mma = mh.tiled_mma_desc(F16, cta_tile=(0, 0, 0))
        M, N, K = 4096 + 40, 2048 + 24, 64
    else:
        mma = mh.tiled_mma_desc(F16, cta_tile=(0, 0, 0))
        M, N, K = 2048, 4096, 64          # the library picks 256x256
    combos = [(c, o, t) for c in (False, True) for o, t in (("float16", False), ("float32", False), ("bfloat16", True))]
    if M * N > 1 << 20:      # the oracle takes seconds on these: one combination per layout of D
        combos = [(False, "float16", False), (True, "bfloat16", True)]
        if operand_kind in ("col", "scalar"):
            combos = combos[:1] if kernel == "library" else combos[1:]
    for col_major_d, out_name, in_out_type in combos:
        _epilogue_case(mh, mma, M, N, K, out_name, "add", operand_kind, 17, col_major_d=col_major_d,
                       operand_in_out_type=in_out_type)
        if kernel in ("256", "library") and operand_kind != "full":
            # a bias and no C (beta = 0): the bias instance of the hand-ordered kernel
            _epilogue_case(mh, mma, M, N, K, out_name, "add", operand_kind, 18, col_major_d=col_major_d, beta=0.0,
                           operand_in_out_type=in_out_type)


@pytest.mark.parametrize("in_name,atom,out_name,K", [("float16", "MFMA_F32_16x16x32_F16", "float16", 128), ("bfloat16", "MFMA_F32_16x16x32_BF16", "float32", 192),
                                                     ("float8_e4m3fn", "MFMA_F32_16x16x32_FP8", "bfloat16", 256), ("float32", "MFMA_F32_16x16x4_F32", "float32", 64)])
def test_fused_epilogue_on_the_hand_ordered_kernel(mh, in_name, atom, out_name, K):
    """The hand-ordered 256 x 256 kernel's two epilogue forms for every operand type.  An operation with a scalar, a
    one-per-column or a one-per-row operand (a ReLU, a scale, a bias), with or without C, is applied in the lanes' own
    accumulators (every such operation, not only the addition); anything else -- a whole-matrix operand, a division, a C
    or an operation on tiles that reach beyond M and N -- goes through the general epilogue behind the same k-loop (fp8
    so keeps its 16x16x128 MFMA).  Bit for bit against the oracle, whole and ragged tiles."""
    in_dt = getattr(torch, in_name)
    mma = mh.tiled_mma_desc(getattr(mh, atom), atom_layout=(2, 4, 1), cta_tile=(256, 256, 128 // in_dt.itemsize))
    lanes = ("gemm_mfma_tn_256_w4", "bias=1", "ops=0")
    general = ("gemm_mfma_tn_256_w4", "bias=0", "ops=1", "ragged=0")
    seed = 900 + K
    for op, kind, beta in (("max", "scalar", 0.0), ("mul", "row", 0.0), ("sub", "col", -1.25), ("min", "row", 0.5), ("abs", "scalar", 0.0), ("neg", "scalar", 0.75),
                           ("add", "col", 0.0), ("add", "row", -1.25)):
        _epilogue_case(mh, mma, 512, 768, K, out_name, op, kind, seed, beta=beta, in_dt=in_dt, instance=lanes)
        seed += 1
    # (a column-major D: the kernel runs the transposed problem, C and the operand are then read through their other stride)
    _epilogue_case(mh, mma, 512, 768, K, out_name, "sub", "row", seed, beta=0.5, in_dt=in_dt, instance=lanes, col_major_d=True)
    seed += 1
    for op, kind, beta in (("div", "row", 0.0), ("mul", "full", 0.0), ("add", "full", -1.25), ("max", "full", 0.5)):
        _epilogue_case(mh, mma, 512, 768, K, out_name, op, kind, seed, beta=beta, in_dt=in_dt, instance=general)
        seed += 1
    # tiles that reach beyond M and N, the tile left to the library: with a C or an operation the guarded general epilogue
    lib = mh.tiled_mma_desc(getattr(mh, atom), cta_tile=(0, 0, 0))
    # (fp32 problems of this size are cheaper on 128 x 128 tiles, whose guarded form with a C or an operation is the
    # compiler-scheduled kernel's: whatever runs must give the same bits)
    ragged = ("gemm_mfma_tn_256_w4", "ragged=1", "ops=1") if in_dt != torch.float32 else ("ragged=1",)
    # (14 x 15 tiles; the row pitch of a 16-bit D is 8 bytes modulo 16; K long enough that the library takes these tiles)
    M, N, Kr = 3400, 3604, {2: 1024, 1: 4096, 4: 256}[in_dt.itemsize]
    _epilogue_case(mh, lib, M, N, Kr, out_name, "identity", "scalar", seed + 1, beta=-1.25, in_dt=in_dt, instance=ragged)
    _epilogue_case(mh, lib, M, N, Kr, out_name, "max", "row", seed + 2, beta=0.0, in_dt=in_dt, instance=ragged, col_major_d=True)


@pytest.mark.parametrize("op", ["max", "min"])
def test_fused_epilogue_max_min_follow_julia_on_nans_and_signed_zeros(mh, op):
    """max / min in the epilogue: NaN if either argument is one, -0.0 below +0.0 (base/math.jl, as `moye_map`), through
    the three places the operation is applied: the lanes' own epilogue, the general epilogue, and the second pass of a
    split-K call.  The product is made +0, -0, NaN and ordinary values by rows (zero rows of A, a negative alpha, a NaN in
    A), the operand carries the same set by columns; bit for bit against the oracle."""
    from moye_hip import _lib
    M, N, K = 256, 512, 128
    g = torch.Generator().manual_seed(77)
    A = torch.randint(-2, 3, (M, K), generator=g).to(torch.float16)
    A[0::4] = 0                      # rows whose product is a zero; its sign is alpha's
    A[1::16, 5] = float("nan")       # rows whose product is NaN
    B = torch.randint(-2, 3, (N, K), generator=g).to(torch.float16)
    B[:, 5] = 1
    xs = torch.tensor([0.0, -0.0, float("nan"), 1.5, -1.5, float("inf"), -float("inf"), 3.0]).repeat(N // 8)
    acc = A.float() @ B.float().t()
    a, b, xd = A.cuda(), B.cuda(), xs.cuda()
    full = xs[None, :].repeat(M, 1).contiguous()
    fd = full.cuda()
    seen = set()
    for alpha in (1.0, -1.0):
        for name, mma, operand, xnp in (
                ("lanes", mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, atom_layout=(2, 4, 1), cta_tile=(256, 256, 64)), T(xd, (M, N), (0, 1)), xs.numpy()[None, :]),
                ("general", mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, atom_layout=(2, 4, 1), cta_tile=(256, 256, 64)), T(fd), full.numpy()),
                ("lanes 128", mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, atom_layout=(2, 2, 1), cta_tile=(128, 128, 64)), T(xd, (M, N), (0, 1)), xs.numpy()[None, :]),
                ("split-K", mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, atom_layout=(2, 2, 1), cta_tile=(128, 128, 32), split_k=2), T(xd, (M, N), (0, 1)), xs.numpy()[None, :])):
            ep = mh.gemm_epilogue(alpha=alpha, beta=0.0, op=_lib.MAP_OPS[op], operand=operand)
            d = torch.zeros(M, N, dtype=torch.float32, device="cuda")
            seen.update(k["name"] for k in kernels_of(mh, mma, T(d), T(a), T(b), None, ep))
            need = mh.gemm_workspace_size(mma, T(d), T(a), T(b), ep)
            ws = torch.zeros(need + 256, dtype=torch.uint8, device="cuda")
            mh.gemm_ex_(mma, T(d), T(a), T(b), None, ep, (ws.data_ptr() + 255) // 256 * 256, need)
            torch.cuda.synchronize()
            want = to.gemm_epilogue(acc.numpy(), alpha, 0.0, None, op, xnp, 0.0, "f32")
            gb, wb = d.cpu().numpy().view(np.uint32), want.astype(np.float32).view(np.uint32)
            nan_both = np.isnan(d.cpu().numpy()) & np.isnan(want)
            bad = np.argwhere((gb != wb) & ~nan_both)
            assert bad.size == 0, (name, alpha, bad[:4], d.cpu().numpy()[tuple(bad[0])], want[tuple(bad[0])])
            assert np.isnan(want).any() and (wb == 0x80000000).any() and (wb == 0).any()     # the cases are in the data
    assert any("gemm_mfma_tn_256_w4" in k and "bias=1" in k for k in seen) and any("gemm_mfma_tn_256_w4" in k and "ops=1" in k for k in seen), seen


def test_fused_epilogue_limits(mh):
    """beta == 0 never reads C (NaNs in it do not reach D); moye_gemm is the beta == 1 case of moye_gemm_ex, bit for
    bit; what is not built says so."""
    from moye_hip import _lib
    g = torch.Generator().manual_seed(5)
    M = N = 256
    K = 128
    A = (torch.randn(M, K, generator=g) / 8).half()
    B = (torch.randn(N, K, generator=g) / 8).half()
    a, b = A.cuda(), B.cuda()
    nan_c = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    mma = mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, cta_tile=(128, 128, 32))
    d0 = torch.zeros(M, N, dtype=torch.float16, device="cuda")
    mh.gemm_ex_(mma, T(d0), T(a), T(b), T(nan_c), mh.gemm_epilogue(alpha=2.0, beta=0.0))
    d1 = torch.zeros_like(d0)
    mh.gemm_(mma, T(d1), T(a), T(b), None, 2.0)
    torch.cuda.synchronize()
    assert not torch.isnan(d0).any() and torch.equal(d0.view(torch.int16), d1.view(torch.int16))
    C0 = torch.randn(M, N, generator=g).half().cuda()
    mh.gemm_ex_(mma, T(d0), T(a), T(b), T(C0), mh.gemm_epilogue(alpha=0.3, beta=1.0))
    mh.gemm_(mma, T(d1), T(a), T(b), T(C0), 0.3)
    torch.cuda.synchronize()
    assert torch.equal(d0.view(torch.int16), d1.view(torch.int16))
    x = torch.zeros(M, N, dtype=torch.float64, device="cuda")
    for bad, status in ((mh.gemm_epilogue(op=99), _lib.ERR_UNSUPPORTED),
                        (mh.gemm_epilogue(op=_lib.MAP_ADD, operand=T(x)), _lib.ERR_UNSUPPORTED),
                        (mh.gemm_epilogue(op=_lib.MAP_ADD, operand=T(d0.float()[:, :128].contiguous())), _lib.ERR_SHAPE)):
        with pytest.raises(mh.MoyeError) as e:
            mh.gemm_ex_(mma, T(d0), T(a), T(b), None, bad)
        assert e.value.status == status
    with pytest.raises(mh.MoyeError) as e:       # the hand-ordered kernel's four-wave schedule has no such epilogue
        mh.gemm_ex_(mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, atom_layout=(2, 2, 1), cta_tile=(256, 256, 64), flags=_lib.GEMM_WAVE4),
                    T(d0), T(a), T(b), None, mh.gemm_epilogue(op=_lib.MAP_ABS))
    assert e.value.status == _lib.ERR_UNSUPPORTED
    af, bf = a.float(), b.float()
    with pytest.raises(mh.MoyeError) as e:       # UniversalFMA keeps the reference's own accumulation
        mh.gemm_ex_(mh.tiled_mma_desc(mh.MMA_UNIVERSAL_FMA, cta_tile=(32, 32, 8)), T(d0.float()), T(af), T(bf), None,
                    mh.gemm_epilogue(op=_lib.MAP_ABS))
    assert e.value.status == _lib.ERR_UNSUPPORTED


# ---------------------------------------------------------------------------------------------
# operands that are not K-major, without a workspace: the transposing fragment reads of the load-to-LDS kernels
# ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("tdt,atom", [("float16", "MFMA_F32_16x16x32_F16"), ("bfloat16", "MFMA_F32_16x16x32_BF16")])
@pytest.mark.parametrize("majors", ["mk", "kn", "mn"])
def test_operand_majors_native_exact_on_integers(mh, tdt, atom, majors):
    """A stored M-major and / or B stored N-major (NN / NT / TT of src/arch/mma/make_mma_ops.jl:253-265) through the
    256x256 and 128x128 tiles with MOYE_GEMM_NO_WORKSPACE: no K-major copy is made, the fragments come out of LDS through the
    transposing read.  Small integers, so every misplaced element shows; named tile and the library's choice, row- and
    column-major D, C and alpha, fp32 and 16-bit results, a padded pitch, and the epilogue operation."""
    from moye_hip import _lib
    tdt = getattr(torch, tdt)
    atom = getattr(mh, atom)
    g = torch.Generator().manual_seed(71)
    cases = [(512, 768, 256, (256, 256, 64), 0), (256, 256, 64, (256, 256, 0), 8), (2048, 4096, 128, (0, 0, 0), 0), (512, 512, 16384, (256, 256, 64), 0),
             # the 128x128 tile of the same schedule: named, and as the library's choice for problems of whole 128x128 tiles
             (384, 640, 256, (128, 128, 64), 8), (128, 128, 64, (128, 128, 64), 0), (1152, 896, 128, (0, 0, 0), 0), (2048, 2048, 192, (0, 0, 0), 8)]
    for (M, N, K, cta, pad) in cases:
        A = torch.randint(-3, 4, (M, K), generator=g).to(tdt)
        B = torch.randint(-3, 4, (N, K), generator=g).to(tdt)
        ref = A.double() @ B.double().t()
        assert float(ref.abs().max()) < 2 ** 24
        a_k, b_k = A.cuda(), B.cuda()
        # M-major / N-major storage with a pitch of M + pad (N + pad) elements between consecutive k
        a_m = torch.zeros(K, M + pad, dtype=tdt)
        a_m[:, :M] = A.t()
        b_n = torch.zeros(K, N + pad, dtype=tdt)
        b_n[:, :N] = B.t()
        a_m, b_n = a_m.cuda(), b_n.cuda()
        ta = T(a_m, (M, K), (1, M + pad)) if majors[0] == "m" else T(a_k)
        tb = T(b_n, (N, K), (1, N + pad)) if majors[1] == "n" else T(b_k)
        mma = mh.tiled_mma_desc(atom, atom_layout=(2, 4, 1), cta_tile=cta, flags=_lib.GEMM_NO_WORKSPACE)
        for out_dt in (torch.float32, tdt):
            d = torch.zeros(M, N, dtype=out_dt, device="cuda")
            assert mh.gemm_workspace_size(mh.tiled_mma_desc(atom, atom_layout=(2, 4, 1), cta_tile=cta), T(d), ta, tb) == 0
            mh.gemm_(mma, T(d), ta, tb)
            torch.cuda.synchronize()
            want = ref if out_dt == torch.float32 else ref.to(out_dt).double()
            assert torch.equal(d.cpu().double(), want), (M, N, K, cta, out_dt, "row-major D")
        C0 = torch.randint(-8, 9, (M, N), generator=g).float()
        dt_ = torch.zeros(N, M, dtype=torch.float32, device="cuda")
        mh.gemm_(mma, T(dt_, (M, N), (1, M)), ta, tb, T(C0.cuda()), 0.5)
        torch.cuda.synchronize()
        assert torch.equal(dt_.t().cpu().double(), 0.5 * ref + C0.double()), (M, N, K, cta, "column-major D, C, alpha")
        if K <= 256:
            bias = torch.randint(-5, 6, (N,), generator=g).float()
            d = torch.zeros(M, N, dtype=torch.float32, device="cuda")
            mh.gemm_ex_(mma, T(d), ta, tb, None,
                        mh.gemm_epilogue(alpha=1.0, op=_lib.MAP_MAX, operand=T(bias.cuda(), (M, N), (0, 1))))
            torch.cuda.synchronize()
            assert torch.equal(d.cpu().double(), torch.maximum(ref, bias.double()[None, :])), (M, N, K, "max with a bias row")


def test_operand_majors_native_random(mh):
    """fp16 NN 4096^3 (A M-major, B N-major) on random data against fp64, and its time beside the TN form's."""
    from moye_hip import _lib
    M = N = K = 4096
    g = torch.Generator().manual_seed(1003)
    A = (torch.randn(M, K, generator=g) / K ** 0.5).half()
    B = (torch.randn(N, K, generator=g) / K ** 0.5).half()
    a_k, b_k = A.cuda(), B.cuda()
    a_m, b_n = A.t().contiguous().cuda(), B.t().contiguous().cuda()
    c64 = a_k.double() @ b_k.double().t()
    mma = mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, atom_layout=(2, 4, 1), cta_tile=(256, 256, 64), flags=_lib.GEMM_NO_WORKSPACE)
    times = {}
    for name, ta, tb in (("TN", T(a_k), T(b_k)), ("NN", T(a_m, (M, K), (1, M)), T(b_n, (N, K), (1, N))),
                         ("A M-major", T(a_m, (M, K), (1, M)), T(b_k)), ("B N-major", T(a_k), T(b_n, (N, K), (1, N)))):
        d = torch.zeros(M, N, dtype=torch.float16, device="cuda")
        mh.gemm_(mma, T(d), ta, tb)
        torch.cuda.synchronize()
        assert relerr(d, c64) <= TOL16, name
        mh.time_gemm(mma, T(d), ta, tb, None, 1.0, None, warmup=20, iters=100)
        times[name] = mh.time_gemm(mma, T(d), ta, tb, None, 1.0, None, warmup=5, iters=100)
    print("fp16 4096^3 by operand major: " + ", ".join("%s %.1f us" % (k, v * 1e3) for k, v in times.items()))
    # (timings are printed, not asserted: a noisy box must not turn a parity suite red; bench.py carries the NN figure)
    # the same on a problem the library puts on 128x128 tiles
    M = N = K = 2048
    a_k, b_k = a_k[:M, :K].contiguous(), b_k[:N, :K].contiguous()
    a_m, b_n = a_k.t().contiguous(), b_k.t().contiguous()
    c64 = a_k.double() @ b_k.double().t()
    mma = mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, cta_tile=(0, 0, 0), flags=_lib.GEMM_NO_WORKSPACE)
    times = {}
    for name, ta, tb in (("TN", T(a_k), T(b_k)), ("NN", T(a_m, (M, K), (1, M)), T(b_n, (N, K), (1, N)))):
        d = torch.zeros(M, N, dtype=torch.float16, device="cuda")
        mh.gemm_(mma, T(d), ta, tb)
        torch.cuda.synchronize()
        assert relerr(d, c64) <= TOL16, name
        mh.time_gemm(mma, T(d), ta, tb, None, 1.0, None, warmup=20, iters=100)
        times[name] = mh.time_gemm(mma, T(d), ta, tb, None, 1.0, None, warmup=5, iters=100)
    print("fp16 2048^3 by operand major: " + ", ".join("%s %.1f us" % (k, v * 1e3) for k, v in times.items()))
    # (printed only; the 128x128 tile reads LDS near its limit already: about 1.4 x TN; with K-major copies about 1.3)

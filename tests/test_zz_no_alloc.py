"""moye_gemm_noalloc (the entry point that allocates nothing: its workspace is a static device array) against
moye_gemm on the same inputs, bit for bit, through the C ABI.  Two calls in a row share the array, the second
smaller than the first, so stale contents of the first call would show."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


@pytest.fixture(scope="module")
def mh():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    import moye_hip
    return moye_hip


def T(t, shape=None, stride=None):
    from moye_hip.torch_interop import tensor_of
    return tensor_of(t, shape, stride)


def _case(mh, M, N, K, split, seed, out_dt=torch.float16, cta=(128, 128, 32), waves=(2, 2, 1)):
    """Random fp16 operands, A stored M-major (needs a K-major copy), split-K (needs partial products), C and alpha.
    moye_gemm runs first (it allocates the library's own workspace); the free device memory is then read on both sides
    of the moye_gemm_noalloc call and must not move."""
    from moye_hip import _lib
    g = torch.Generator().manual_seed(seed)
    A = (torch.randn(M, K, generator=g) * K ** -0.5).half()
    B = (torch.randn(N, K, generator=g) * K ** -0.5).half()
    C0 = torch.randn(M, N, generator=g).to(out_dt)
    a_m, b, c = A.t().contiguous().cuda(), B.cuda(), C0.cuda()
    ta = T(a_m, (M, K), (1, M))
    mma = mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, atom_layout=waves, cta_tile=cta, split_k=split)
    lib = _lib.lib()
    need = C.c_size_t()
    _lib.check(lib.moye_gemm_workspace_size(C.byref(mma), C.byref(T(c)), C.byref(ta), C.byref(T(b)), C.byref(need)))
    # the call does use the scratch: the partial products of every K range and the K-major copy of A, whose rows are
    # rounded up to 16 bytes and whose size to 256; and the plan it runs uses exactly what the query says
    plan = mh.gemm_explain(mma, T(c), ta, T(b), T(c))
    ranges = max(s["split"] for s in plan["steps"] if s["what"] == "kernel")       # (split = -1: the library's own choice)
    assert ranges == split or split == -1
    pitch = (K * 2 + 15) // 16 * 16
    assert need.value >= (ranges * M * N * 4 if ranges > 1 else 0) + (M * pitch + 255) // 256 * 256
    assert plan["workspace"] == need.value and "kmajor_copy" in [s["what"] for s in plan["steps"]]
    assert (ranges > 1) == ("splitk_reduce" in [s["what"] for s in plan["steps"]])
    d_new = torch.full((M, N), float("nan"), dtype=out_dt, device="cuda")
    d_old = torch.full((M, N), float("nan"), dtype=out_dt, device="cuda")
    _lib.check(lib.moye_gemm(C.byref(mma), C.byref(T(d_old)), C.byref(ta), C.byref(T(b)), C.byref(T(c)),
                             C.c_float(0.75), None))
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    _lib.check(lib.moye_gemm_noalloc(C.byref(mma), C.byref(T(d_new)), C.byref(ta), C.byref(T(b)), C.byref(T(c)),
                                     C.c_float(0.75), None))
    torch.cuda.synchronize()
    if getattr(_case, "warm", False):      # (the first call of a process asks for the array's address, which may load code)
        assert torch.cuda.mem_get_info()[0] == free_before, "moye_gemm_noalloc changed the free device memory"
    _case.warm = True
    bits = {torch.float16: torch.int16, torch.float32: torch.int32}[out_dt]
    assert torch.equal(d_new.view(bits), d_old.view(bits)), (M, N, K, split)
    c64 = 0.75 * (A.double() @ B.double().t()) + C0.double()
    err = float((d_new.cpu().double() - c64).abs().max() / c64.abs().max())
    assert err <= 1e-2, err          # fp16 inputs: max|D - D64| / max|D64| <= 1e-2
    return need.value


def test_noalloc_matches_gemm_on_two_calls_in_a_row(mh):
    first = _case(mh, 512, 768, 4096, 4, seed=11)                          # 6 MiB of partials + 4 MiB copy
    second = _case(mh, 128, 256, 1024, 2, seed=12, out_dt=torch.float32)   # smaller: reuses the head of the array
    assert second < first <= mh.device.NOALLOC_SCRATCH_BYTES


def test_noalloc_ragged_shapes_and_the_library_s_own_choices(mh):
    """Shapes that are no multiple of any tile, a K whose rows the K-major copy has to pad, the tile and the K ranges
    left to the library: the same bits as moye_gemm, and no change in free device memory across any of the calls."""
    _case(mh, 256, 256, 512, 1, seed=20)                                         # (warms the process if this test runs alone)
    _case(mh, 200, 136, 72, 1, seed=21, cta=(0, 0, 0), waves=(1, 1, 1))          # residue tiles; copy rows of 144 bytes
    _case(mh, 1000, 520, 1992, 1, seed=22, cta=(0, 0, 0), waves=(1, 1, 1), out_dt=torch.float32)
    _case(mh, 300, 300, 8208, 3, seed=23, cta=(0, 0, 0), waves=(1, 1, 1))        # three K ranges named, ragged in M, N and K
    _case(mh, 128, 384, 16384, -1, seed=24, cta=(0, 0, 0), waves=(1, 1, 1))      # the K ranges left to the library


def test_noalloc_plain_tn_and_limits(mh):
    from moye_hip import _lib
    g = torch.Generator().manual_seed(13)
    M = N = 256
    K = 512
    A = torch.randint(-4, 5, (M, K), generator=g).half()
    B = torch.randint(-4, 5, (N, K), generator=g).half()
    a, b = A.cuda(), B.cuda()
    d = torch.zeros(M, N, device="cuda")
    mh.gemm_noalloc_(mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, cta_tile=(128, 128, 32)), T(d), T(a), T(b))
    torch.cuda.synchronize()
    assert torch.equal(d.cpu().double(), A.double() @ B.double().t())
    # beyond the static array: refused with a clear error, nothing launched
    big = torch.zeros(2048, 2048, device="cuda")
    ah = torch.zeros(2048, 1024, dtype=torch.float16, device="cuda")
    mma = mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, cta_tile=(128, 128, 32), split_k=4)      # 64 MiB of partials
    assert mh.gemm_workspace_size(mma, T(big), T(ah), T(ah)) > mh.device.NOALLOC_SCRATCH_BYTES
    with pytest.raises(mh.MoyeError) as e:
        mh.gemm_noalloc_(mma, T(big), T(ah), T(ah))
    assert e.value.status == _lib.ERR_ARG and "static scratch" in str(e.value)

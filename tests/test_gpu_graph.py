"""The hot-path entry points record into a HIP graph and replay: moye_gemm_noalloc (a split-K call that uses the static
scratch array, and a ragged call), moye_gemm_ex with a fused bias, moye_copy (a transpose) and moye_axpby on one stream
under capture.  Every replay is checked against the eager result of the same calls, with eager work and
synchronisations between the replays; the inputs change between replays (the graph holds pointers, not values)."""
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


def test_hot_path_under_graph_capture_replays_bit_for_bit(mh):
    from moye_hip import _lib
    g = torch.Generator().manual_seed(7)
    M, N, K = 512, 640, 2048
    a = torch.empty(M, K, dtype=torch.float16, device="cuda")
    b = torch.empty(N, K, dtype=torch.float16, device="cuda")
    bias = torch.randn(N, generator=g).cuda()
    ar = torch.empty(300, 520, dtype=torch.float16, device="cuda")     # a ragged problem for the 128x128 tiles
    br = torch.empty(1000, 520, dtype=torch.float16, device="cuda")
    src = torch.empty(2048, 1024, dtype=torch.float32, device="cuda")
    d_split = torch.zeros(M, N, dtype=torch.float16, device="cuda")
    d_bias = torch.zeros(M, N, dtype=torch.float32, device="cuda")
    d_rag = torch.zeros(300, 1000, dtype=torch.float16, device="cuda")
    dst = torch.zeros(1024, 2048, dtype=torch.float32, device="cuda")
    y = torch.zeros(M, N, dtype=torch.float32, device="cuda")
    outs = (d_split, d_bias, d_rag, dst, y)
    m_split = mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, atom_layout=(2, 2, 1), cta_tile=(128, 128, 64), split_k=4)
    m_auto = mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16, cta_tile=(0, 0, 0))
    ep = mh.gemm_epilogue(alpha=0.5, op=_lib.MAP_ADD, operand=T(bias, (M, N), (0, 1)))

    def fill_inputs(seed):
        gg = torch.Generator().manual_seed(seed)
        a.copy_((torch.randn(M, K, generator=gg) * K ** -0.5).half())
        b.copy_((torch.randn(N, K, generator=gg) * K ** -0.5).half())
        ar.copy_(torch.randint(-3, 4, (300, 520), generator=gg).half())
        br.copy_(torch.randint(-3, 4, (1000, 520), generator=gg).half())
        src.copy_(torch.randn(2048, 1024, generator=gg))
        for o in outs:
            o.zero_()

    def work(stream):
        mh.gemm_noalloc_(m_split, T(d_split), T(a), T(b), None, 1.0, stream)
        mh.gemm_ex_(m_auto, T(d_bias), T(a), T(b), None, ep, None, 0, stream)
        mh.gemm_noalloc_(m_auto, T(d_rag), T(ar), T(br), None, 1.0, stream)
        mh.copyto_(T(dst), T(src, (1024, 2048), (1, 1024)), stream=stream)        # dst = src'
        mh.axpby_(2.0, T(d_bias), 0.0, T(y), stream=stream)

    side = torch.cuda.Stream()
    fill_inputs(100)
    torch.cuda.synchronize()
    with torch.cuda.stream(side):                # first use outside capture: LDS caps, the scratch array's address
        work(side.cuda_stream)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        work(side.cuda_stream)
    for seed in (101, 102, 103):
        fill_inputs(seed)
        torch.cuda.synchronize()
        with torch.cuda.stream(side):
            work(side.cuda_stream)
        torch.cuda.synchronize()
        want = [o.clone() for o in outs]
        assert float(want[0].float().abs().max()) > 0 and float(want[3].abs().max()) > 0
        assert torch.equal(want[3], src.t())
        assert torch.equal(want[2].double().cpu(), ar.double().cpu() @ br.double().cpu().t())
        for o in outs:
            o.zero_()
        (a.float() @ b.float().t()).sum().item()            # eager work of the program's own between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, w in zip(outs, want):
            assert torch.equal(got.view(torch.int32 if got.element_size() == 4 else torch.int16),
                               w.view(torch.int32 if w.element_size() == 4 else torch.int16)), seed

"""Pins the C oracle (oracle/gemm_oracle.c): bit-exact against the numpy restatement, against
numpy's float16 conversion, and against hand-built rounding cases that a fused multiply-add, an
unrounded product or a reordered sum would fail."""
import numpy as np
import pytest

import c_oracle as co
import tiled_oracle as to


def test_round_f16_matches_numpy_everywhere_it_matters():
    rng = np.random.default_rng(0)
    x = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * np.float32(10.0) ** rng.integers(-8, 5, 20000),
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e6, 2.0 ** -24, 2.0 ** -25, 1.5 * 2.0 ** -24,
                  2.0 ** -14, 2.0 ** -14 - 2.0 ** -25, 1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11, np.inf, -np.inf],
                 np.float32)]).astype(np.float32)
    got = np.array([co.lib().moye_ref_round_f16(float(v)) for v in x], np.float32)
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).astype(np.float32)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    gb = np.array([co.lib().moye_ref_round_bf16(float(v)) for v in x[:5000]], np.float32)
    assert np.array_equal(gb.view(np.uint32), to.round_bf16(x[:5000]).view(np.uint32))


@pytest.mark.parametrize("prod", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("threads", [1, 4])
def test_c_gemm_equals_numpy_restatement(prod, threads):
    rng = np.random.default_rng(1)
    M, N, K = 45, 38, 29
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = rng.standard_normal((N, K)).astype(np.float32)
    if prod == "f16":
        A, B = A.astype(np.float16).astype(np.float32), B.astype(np.float16).astype(np.float32)
    if prod == "bf16":
        A, B = to.round_bf16(A), to.round_bf16(B)
    C0 = rng.standard_normal((M, N)).astype(np.float32)
    want = to.gemm_universal_fma(A, B, C0, prod, prod)
    got = co.gemm(A, B, C0, prod, (32, 32, 8), threads)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # column-major A (the "NN" operand form of config 1) and another tiling: same bits
    got2 = co.gemm(np.asfortranarray(A), B, C0, prod, (16, 8, 4), threads)
    assert np.array_equal(got2.view(np.uint32), want.view(np.uint32))


def test_c_gemm_rounding_rule():
    one = np.zeros((1, 1), np.float32)
    a = np.array([[1.0 + 2.0 ** -10]], np.float32)
    assert co.gemm(a, a, one, "f16")[0, 0] == np.float32(1.0 + 2.0 ** -9)
    assert co.gemm(a, a, one, "f32")[0, 0] == np.float32(1.0 + 2.0 ** -9 + 2.0 ** -20)
    # unfused: fl(fl(a*b) + c) with a*b = 1 + 2^-12 + 2^-26 -> product rounds to 1 + 2^-12;
    # a fused multiply-add would keep the 2^-26 and round the sum differently
    a = np.array([[1.0 + 2.0 ** -13]], np.float32)
    c = np.array([[-1.0]], np.float32)
    assert co.gemm(a, a, c, "f32")[0, 0] == np.float32(2.0 ** -12)
    A = np.array([[1.0, 2.0 ** -24, 2.0 ** -24]], np.float32)
    B = np.ones((1, 3), np.float32)
    assert co.gemm(A, B, one)[0, 0] == np.float32(1.0)
    assert co.gemm(A[:, ::-1].copy(), B, one)[0, 0] == np.float32(1.0 + 2.0 ** -23)


def test_c_copy_matches_layout_oracle():
    import layout_oracle as lo
    ls, ld = lo.parse_layout("(6,8):(1,6)"), lo.parse_layout("((2,3),(2,4)):((1,16),(2,4))")
    src = np.arange(48, dtype=np.int32)
    d1 = to.Array(np.zeros(48, np.int32), ld)
    to.copyto(d1, to.Array(src, ls))
    f = lo.lflatten(ld)
    d2 = co.copy(np.zeros(48, np.int32), f.shape, f.stride, src, (6, 8), (1, 6))
    assert np.array_equal(d1.buf, d2)

"""The host side of gemm!: which launches a call becomes (moye_gemm_explain).  No device is needed: building a plan is
pure arithmetic on the descriptors, so the whole dispatcher is exercised here -- a few hundred (dtype, shape, strides,
alignment, epilogue, flags) cases, each checked for what its kernel instances require of the sub-problem they get, for
covering D exactly once, and for agreeing with the workspace query; known shapes are pinned to their instance."""
import itertools
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "moye.jl_amd"))

import moye_hip as mh  # noqa: E402
from moye_hip import _lib  # noqa: E402

EB = {mh.F16: 2, mh.BF16: 2, mh.F8E4M3: 1, mh.F32: 4}
ATOM = {mh.F16: mh.MFMA_F32_16x16x32_F16, mh.BF16: mh.MFMA_F32_16x16x32_BF16, mh.F8E4M3: mh.MFMA_F32_16x16x32_FP8,
        mh.F32: mh.MFMA_F32_16x16x4_F32}
ATOM32 = {mh.F16: mh.MFMA_F32_32x32x16_F16, mh.BF16: mh.MFMA_F32_32x32x16_BF16, mh.F8E4M3: mh.MFMA_F32_32x32x16_FP8,
          mh.F32: mh.MFMA_F32_32x32x2_F32}
DT_NAME = {mh.F32: "f32", mh.F16: "f16", mh.BF16: "bf16", mh.F8E4M3: "f8e4m3"}
# addresses that are only compared, never dereferenced
PA, PB, PD, PC, PX = 0x1000_0000_0000, 0x2000_0000_0000, 0x3000_0000_0000, 0x4000_0000_0000, 0x5000_0000_0000


def tensor(ptr, dt, shape, stride):
    return _lib.make_tensor(ptr, dt, shape, stride)


def operands(M, N, K, in_dt, out_dt, a_major="k", b_major="k", d_major="n", pad=(0, 0, 0), offs=(0, 0, 0)):
    """A (M,K), B (N,K), D (M,N) descriptors; *_major names the mode with the unit stride; pad widens the pitches (in
    elements), offs shifts the base addresses (in bytes)."""
    A = tensor(PA + offs[0], in_dt, (M, K), (K + pad[0], 1) if a_major == "k" else (1, M + pad[0]))
    B = tensor(PB + offs[1], in_dt, (N, K), (K + pad[1], 1) if b_major == "k" else (1, N + pad[1]))
    D = tensor(PD + offs[2], out_dt, (M, N), (N + pad[2], 1) if d_major == "n" else (1, M + pad[2]))
    return A, B, D


def check_kernel_step(s, eb, ob, cus=256, xcds=8):
    """What every kernel instance requires of the sub-problem it was given (the launchers' own documented conditions)."""
    fam, name, flags = s["family"], s["name"], s["flags"]
    M, N, K = s["M"], s["N"], s["K"]
    kb = K * eb
    tm, tn = s["tile"].split("x")[0], s["tile"].split("x")[1]
    tm, tn = int(tm), int(tn)
    assert s["A"] != "?" and s["B"] != "?" and s["D"] != "?" and s["C"] != "?", s   # every pointer lies in an array of the call
    assert M > 0 and N > 0 and K > 0
    assert 0 < s["grid"].count("x") and all(0 < int(g) < 2 ** 31 for g in s["grid"].split("x"))
    gx, gy = (int(g) for g in s["grid"].split("x"))
    assert gy == s["split"]
    ragged = "ragged" in flags
    if fam in ("gemm_mfma_tn_256_w4", "gemm_mfma_tn_256", "gemm_mfma_tn_128", "gemm_mfma_tn_256_ring", "gemm_mfma_tn_256_pp", "gemm_mfma_tn"):
        if "persist=1" in name:
            # one workgroup per CU (a whole number per XCD) that walks over more tiles than there are CUs
            assert fam == "gemm_mfma_tn_256_w4" and gx == cus // xcds * xcds and gx < (M // tm) * (N // tn) and gy == 1, s
            assert "tile=256" in name and "waves=8" in name and "bias=0" in name and "ragged=0" in name and "amaj=0" in name and "bmaj=0" in name and "ops=0" in name, s
            assert s["lds"] == 163840 and name.split("<")[1].split(",")[0] in ("W4F16L", "W4BF16L", "W4FP8L"), s
        else:
            assert gx == -(-M // tm) * -(-N // tn), s
        assert s["a16"] == 1 and s["b16"] == 1, s
        a_m, b_n = "a_m_major" in flags, "b_n_major" in flags
        assert (s["lda"] * eb) % 16 == 0 and (s["ldb"] * eb) % 16 == 0, s
        if fam != "gemm_mfma_tn":
            assert tm * s["lda"] * eb < 2 ** 32 and tn * s["ldb"] * eb < 2 ** 32, s     # 32-bit lane offsets over a tile's rows
    if fam == "gemm_mfma_tn_256_w4":
        assert ("ragged=1" in name) == ragged
        assert ("amaj=1" in name) == ("a_m_major" in flags) and ("bmaj=1" in name) == ("b_n_major" in flags)
        step_bytes = int(s["tile"].split("x")[2][:-1])
        assert kb % (16 if ragged else step_bytes) == 0, s       # (the guarded instances mask a K tail of whole 16-byte pieces)
        if not ragged:
            assert M % tm == 0 and N % tn == 0 and s["d16"] == 1 and (s["ldd"] * ob) % 16 == 0, s
        else:
            assert "amaj=0" in name and "bmaj=0" in name, s
            assert "ops=1" in name or (s["C"] == "null" and s["op"] == 0), s
        if "bias=1" in name:
            assert "lane_op" in flags and s["op"] not in (0, _lib.MAP_DIV) and not ragged and "waves=8" in name and "tile=256" in name, s
        elif "ops=1" in name:
            assert "waves=8" in name and "tile=256" in name and "amaj=0" in name and "bmaj=0" in name and step_bytes == 128, s
            assert name.split("<")[1].split(",")[0] in ("W4F16L", "W4BF16L", "W4FP8L", "W4F32L"), s
        else:
            assert s["op"] == 0, s                       # the other instances have no element-wise operation
        if "amaj=1" in name or "bmaj=1" in name:
            assert (("tile=256" in name and "waves=8" in name) or ("tile=128" in name and "waves=4" in name)) and not ragged, s
            assert "bias=0" in name and "ops=0" in name and s["op"] == 0 and step_bytes == 128, s
    elif fam in ("gemm_mfma_tn_256", "gemm_mfma_tn_128"):
        assert ("ragged=1" in name) == ragged
        assert ("amaj=1" in name) == ("a_m_major" in flags) and ("bmaj=1" in name) == ("b_n_major" in flags)
        if "amaj=1" in name or "bmaj=1" in name:
            assert eb == 2 and not ragged, s
        if ragged:
            assert kb % 16 == 0, s
        else:
            assert M % tm == 0 and N % tn == 0 and kb % 128 == 0 and s["d16"] == 1 and (s["ldd"] * ob) % 16 == 0, s
        if s["op"] != 0 and "bias=1" not in name:
            assert "ops=1" in name, s
        if "bias=1" in name:
            assert "lane_op" in flags and s["op"] not in (0, _lib.MAP_DIV), s
    elif fam == "gemm_mfma_tn_256_atom32":
        assert gx == (M // 256) * (N // 256) and s["a16"] == 1 and s["b16"] == 1 and "atom32" in flags, s
        assert (s["lda"] * eb) % 16 == 0 and (s["ldb"] * eb) % 16 == 0, s
        assert M % 256 == 0 and N % 256 == 0 and kb % 128 == 0 and s["d16"] == 1 and (s["ldd"] * ob) % 16 == 0 and not ragged, s
        assert "a_m_major" not in flags and "b_n_major" not in flags, s
        assert ("ops=1" in name) == (s["op"] != 0), s
    elif fam in ("gemm_mfma_tn_256_ring", "gemm_mfma_tn_256_pp"):
        assert M % 256 == 0 and N % 256 == 0 and kb % 64 == 0 and s["d16"] == 1 and s["op"] == 0 and not ragged, s
    elif fam == "gemm_mfma_tn":
        bkb = int(s["tile"].split("x")[2][:-1])
        if "edge=1" in name:
            assert kb % 16 == 0, s
        else:
            assert M % tm == 0 and N % tn == 0 and kb % bkb == 0 and s["d16"] == 1 and (s["ldd"] * ob) % 16 == 0, s
    elif fam == "gemm_mfma_skinny_lds":
        assert 1 <= M <= 64 and s["a16"] == 1 and s["b16"] == 1, s
        assert (s["lda"] * eb) % 16 == 0 and (s["ldb"] * eb) % 16 == 0, s
        assert kb % 16 == 0, s                          # whole 128-byte lines plus a masked tail of 16-byte pieces
        mt = int(name.split("mt=")[1].split(",")[0])
        assert 16 * mt >= M, s
    else:
        raise AssertionError("unknown kernel family in a plan: " + name)


def d_rectangles(plan, M, N, ob, pitch):
    """The parts of a row-major D (M x N, row pitch `pitch` elements) that the kernel steps write, as (row0, col0, rows, cols)."""
    out = []
    for s in plan["steps"]:
        if s["what"] != "kernel" or not str(s["D"]).startswith("D+"):
            continue
        off = int(s["D"][2:])
        r0, c0 = off // (pitch * ob), (off % (pitch * ob)) // ob
        if s["ldd_n"] in (0, 1) and s["ldd"] == pitch:
            out.append((r0, c0, s["M"], s["N"]))
        else:                       # the short-M kernel on a transposed fringe: its m runs along the caller's n
            assert s["ldd"] == 1 and s["ldd_n"] == pitch, s
            out.append((r0, c0, s["N"], s["M"]))
    return out


def covers_exactly_once(rects, M, N):
    area = 0
    for i, (r, c, h, w) in enumerate(rects):
        assert 0 <= r and r + h <= M and 0 <= c and c + w <= N, rects
        area += h * w
        for (r2, c2, h2, w2) in rects[i + 1:]:
            assert r + h <= r2 or r2 + h2 <= r or c + w <= c2 or c2 + w2 <= c, ("overlap", rects)
    assert area == M * N, (rects, M, N)


SHAPES = [(4096, 4096, 4096), (8192, 8192, 8192), (6144, 6144, 6144), (5120, 5120, 5120), (4608, 4608, 512), (4000, 4000, 4096),
          (4100, 4104, 4096), (4100, 4100, 4096), (5000, 3000, 2048), (4096, 4096, 4000), (2048, 2048, 2048), (1024, 1024, 1024),
          (512, 512, 512), (256, 256, 65536), (256, 8192, 8192), (200, 8192, 8192), (96, 8192, 8192), (1000, 1000, 8192),
          (300, 16384, 4096), (3000, 3000, 3072), (130, 32768, 4096), (4096, 2304, 4096), (4096, 2048, 4096), (16, 8192, 8192),
          (16, 8192, 8224), (16, 1024, 32768), (64, 2048, 8192), (33, 4096, 4160), (1, 1, 64), (7, 130, 200), (129, 127, 72),
          (384, 250, 64), (2304, 9216, 4096), (12288, 12288, 4096), (128, 128, 96), (17, 300, 200)]
SEEN = set()


def run_case(in_dt, out_dt, M, N, K, **kw):
    eb, ob = EB[in_dt], EB[out_dt]
    cta = kw.get("cta", (0, 0, 0))
    mma = mh.tiled_mma_desc(kw.get("atom", ATOM[in_dt]), atom_layout=kw.get("waves", (2, 4, 1)), cta_tile=cta, stages=kw.get("stages", 0),
                            split_k=kw.get("split_k", 0), flags=kw.get("flags", 0))
    A, B, D = operands(M, N, K, in_dt, out_dt, kw.get("a_major", "k"), kw.get("b_major", "k"), kw.get("d_major", "n"), kw.get("pad", (0, 0, 0)),
                       kw.get("offs", (0, 0, 0)))
    C = tensor(PC, out_dt, (M, N), (N, 1)) if kw.get("with_c") else None
    ep = kw.get("ep")
    try:
        plan = mh.gemm_explain(mma, D, A, B, C, ep, kw.get("cus", 256))
    except mh.MoyeError as e:
        return e
    # the workspace the plan uses is what the query announces
    assert plan["workspace"] == mh.gemm_workspace_size(mh.tiled_mma_desc(kw.get("atom", ATOM[in_dt]), atom_layout=kw.get("waves", (2, 4, 1)), cta_tile=cta,
                                                                      stages=kw.get("stages", 0), split_k=kw.get("split_k", 0), flags=kw.get("flags", 0)),
                                                   D, A, B, ep) or kw.get("cus", 256) != 256
    ws_used = 0
    kernels = [s for s in plan["steps"] if s["what"] == "kernel"]
    reduces = [s for s in plan["steps"] if s["what"] == "splitk_reduce"]
    for s in plan["steps"]:
        SEEN.add(s.get("family", s["what"]))
        if s["what"] == "kernel":
            if s["family"].startswith("gemm_universal"):
                continue
            SEEN.add(s["name"].split(",")[0] + (",ragged" if "ragged" in s["flags"] else ""))
            for key in ("ragged=1", "bias=1", "amaj=1", "bmaj=1", "ops=1", "edge=1", "atom=32", "tile=128"):
                if key in s["name"]:
                    SEEN.add(s["family"] + ":" + key)
            check_kernel_step(s, eb, 4 if reduces else ob, plan["cus"], plan["xcds"])
            if str(s["D"]).startswith("ws+"):
                ws_used = max(ws_used, int(s["D"][3:]) + s["split"] * s["M"] * s["N"] * 4)
        elif s["what"] == "kmajor_copy":
            pass
    assert ws_used <= plan["workspace"], plan["text"]
    if reduces:
        assert len(reduces) == 1 and reduces[0]["split"] == kernels[-1]["split"] > 1 and plan["steps"][-1] is reduces[0], plan["text"]
        assert reduces[0]["M"] * reduces[0]["N"] == M * N
        if kw.get("split_k", 0) < 0 and cta == (0, 0, 0):
            # tile and K ranges are one decision: 256 x 256 tiles in K ranges only to bring the workgroups up to one per CU
            assert all(not s["tile"].startswith("256x") or (M // 256) * (N // 256) * s["split"] <= plan["cus"] for s in kernels), plan["text"]
    elif kw.get("d_major", "n") == "n" and M > 1 and kernels and not kernels[0]["family"].startswith("gemm_universal"):
        covers_exactly_once(d_rectangles(plan, M, N, ob, N + kw.get("pad", (0, 0, 0))[2]), M, N)
    return plan


@pytest.mark.parametrize("in_dt", [mh.F16, mh.BF16, mh.F8E4M3, mh.F32])
def test_every_plan_meets_its_kernels_conditions(in_dt):
    """Shapes x result types x (tile left to the library | named) x (K ranges none | library's | named) x alignment."""
    n = 0
    for (M, N, K), out_dt in itertools.product(SHAPES, (mh.F32, mh.F16 if in_dt != mh.BF16 else mh.BF16)):
        for kw in ({}, {"split_k": -1}, {"with_c": True}, {"pad": (8, 16, 8)}, {"pad": (0, 0, 4 // EB[out_dt] or 1)}, {"offs": (0, 0, 8)},
                   {"d_major": "m"}, {"flags": _lib.GEMM_NO_WORKSPACE}, {"cus": 64}, {"cus": 304}, {"split_k": 2},
                   {"ep": mh.gemm_epilogue(alpha=0.5, op=_lib.MAP_ADD, scalar=1.0)},
                   {"ep": mh.gemm_epilogue(alpha=0.5, op=_lib.MAP_MAX, scalar=0.0)}):
            if (K * EB[in_dt]) % 16:
                continue
            r = run_case(in_dt, out_dt, M, N, K, **kw)
            n += 1
            if isinstance(r, mh.MoyeError):
                # the library may refuse (a split that does not divide K, a misaligned operand ...) but only with a reason
                assert r.status in (_lib.ERR_SHAPE, _lib.ERR_ALIGN, _lib.ERR_UNSUPPORTED), (M, N, K, kw, str(r))
    assert n > 300


def test_named_tiles_schedules_and_majors():
    """The descriptors that name a tile, a schedule, an atom or operand majors, on shapes they divide."""
    for in_dt in (mh.F16, mh.BF16, mh.F8E4M3, mh.F32):
        eb = EB[in_dt]
        out_dt = mh.F32
        for cta, waves in (((256, 256, 128 // eb), (2, 4, 1)), ((256, 256, 128 // eb), (2, 2, 1)), ((256, 256, 64 // eb), (2, 4, 1)),
                           ((128, 128, 128 // eb), (2, 2, 1)), ((128, 128, 64 // eb), (2, 2, 1)), ((64, 64, 64 // eb), (2, 2, 1))):
            for (M, N, K) in ((4096, 4096, 4096), (512, 768, 1024), (8192, 8192, 512)):
                for kw in ({}, {"stages": 2}, {"stages": 3}, {"flags": _lib.GEMM_PINGPONG}, {"flags": _lib.GEMM_WAVE4}, {"flags": _lib.GEMM_PREDICATE},
                           {"a_major": "m"}, {"b_major": "n"}, {"a_major": "m", "b_major": "n", "flags": _lib.GEMM_NO_WORKSPACE},
                           {"a_major": "m", "b_major": "n", "d_major": "m"}, {"atom": ATOM32[in_dt]}, {"with_c": True, "d_major": "m"},
                           {"ep": mh.gemm_epilogue(alpha=1.0, op=_lib.MAP_ADD, operand=tensor(PX, mh.F32, (M, N), (0, 1)))},
                           {"ep": mh.gemm_epilogue(alpha=1.0, op=_lib.MAP_MUL, operand=tensor(PX, mh.F32, (M, N), (N, 1)))},
                           {"a_major": "m", "ep": mh.gemm_epilogue(alpha=1.0, op=_lib.MAP_MAX, scalar=0.0)}):
                    r = run_case(in_dt, out_dt, M, N, K, cta=cta, waves=waves, **kw)
                    if isinstance(r, mh.MoyeError):
                        assert r.status in (_lib.ERR_SHAPE, _lib.ERR_ALIGN, _lib.ERR_UNSUPPORTED), (cta, M, N, K, kw, str(r))


def test_predicated_named_tiles():
    """MOYE_GEMM_PREDICATE with a named tile that does not divide the problem: the guarded forms of the 128 x 128 kernels
    (the load-to-LDS one for 128-byte k-tiles, the register-staged one for 64-byte k-tiles and the 32 x 32 atoms)."""
    for in_dt in (mh.F16, mh.F8E4M3, mh.F32):
        eb = EB[in_dt]
        for (M, N, K) in ((1000, 1000, 8192), (129, 257, 16 // eb * 5)):
            p = run_case(in_dt, mh.F32, M, N, K, cta=(128, 128, 64 // eb), waves=(2, 2, 1), flags=_lib.GEMM_PREDICATE)
            assert "edge=1" in p["steps"][0]["name"], p["text"]
            p = run_case(in_dt, mh.F32, M, N, K, cta=(128, 128, 128 // eb), waves=(2, 2, 1), flags=_lib.GEMM_PREDICATE)
            assert p["steps"][0]["family"] in ("gemm_mfma_tn_128", "gemm_mfma_tn_256_w4") and "ragged" in p["steps"][0]["flags"], p["text"]
            p = run_case(in_dt, mh.F32, M, N, K, atom=ATOM32[in_dt], cta=(128, 128, 64 // eb), waves=(2, 2, 1), flags=_lib.GEMM_PREDICATE)
            assert "edge=1" in p["steps"][0]["name"] and "atom=32" in p["steps"][0]["name"], p["text"]
            # without the flag the reference's assertion: the tile must divide the problem
            r = run_case(in_dt, mh.F32, M, N, K, cta=(128, 128, 64 // eb), waves=(2, 2, 1))
            assert isinstance(r, mh.MoyeError) and r.status == _lib.ERR_SHAPE


def step_names(plan):
    return [s.get("name", s["what"]) for s in plan["steps"]]


def test_known_shapes_run_on_the_instances_they_are_meant_for():
    """The benchmark's descriptors and the shapes the design documents name, pinned to their kernel instances."""
    f16, bf16, f8, f32 = mh.F16, mh.BF16, mh.F8E4M3, mh.F32
    # the headline: fp16 4096^3 on the hand-ordered whole-line kernel, one launch of 256 workgroups
    p = run_case(f16, f16, 4096, 4096, 4096, cta=(256, 256, 64))
    assert step_names(p) == ["gemm_mfma_tn_256_w4<W4F16L,OutF16,waves=8,bias=0,ragged=0,tile=256,amaj=0,bmaj=0,ops=0>"]
    assert p["steps"][0]["grid"] == "256x1" and {"hand_ordered", "stream_d", "xcd_order"} <= p["steps"][0]["flags"] and "rotate_k" not in p["steps"][0]["flags"]
    # the same left to the library
    assert step_names(run_case(f16, f16, 4096, 4096, 4096)) == step_names(p)
    # bf16 8192^3 fp32 out, fp8 8192^3 bf16 out, fp32 8192^3: the same kernel's other operand types; K rotation on
    p = run_case(bf16, f32, 8192, 8192, 8192, cta=(256, 256, 64))
    assert step_names(p) == ["gemm_mfma_tn_256_w4<W4BF16L,OutF32,waves=8,bias=0,ragged=0,tile=256,amaj=0,bmaj=0,ops=0,persist=1>"] and "rotate_k" in p["steps"][0]["flags"]
    p = run_case(f8, bf16, 8192, 8192, 8192, cta=(256, 256, 128))
    # (more tiles than CUs: one workgroup per CU that walks over the tiles; not when the caller asks for a workgroup per tile)
    assert step_names(p) == ["gemm_mfma_tn_256_w4<W4FP8L,OutBF16,waves=8,bias=0,ragged=0,tile=256,amaj=0,bmaj=0,ops=0,persist=1>"] and p["steps"][0]["grid"] == "256x1"
    p = run_case(f8, bf16, 8192, 8192, 8192, cta=(256, 256, 128), flags=_lib.GEMM_NO_PERSIST)
    assert step_names(p) == ["gemm_mfma_tn_256_w4<W4FP8L,OutBF16,waves=8,bias=0,ragged=0,tile=256,amaj=0,bmaj=0,ops=0>"] and p["steps"][0]["grid"] == "1024x1"
    assert "persist" not in step_names(run_case(f16, f16, 4096, 4096, 4096))[0]
    assert step_names(run_case(f16, f16, 4096, 8192, 4096))[0].endswith("ops=0,persist=1>")
    assert step_names(run_case(f16, f16, 4096, 4096, 4096, cus=64))[0].endswith("ops=0,persist=1>")
    p = run_case(f32, f32, 8192, 8192, 8192, cta=(256, 256, 32))
    assert step_names(p) == ["gemm_mfma_tn_256_w4<W4F32L,OutF32,waves=8,bias=0,ragged=0,tile=256,amaj=0,bmaj=0,ops=0>"]
    # the reference's own operand layout (A M-major, B N-major) needs no workspace for any operand type
    for dt, bk in ((f16, 64), (bf16, 64), (f8, 128), (f32, 32)):
        p = run_case(dt, f32, 4096, 4096, 4096, cta=(256, 256, bk), a_major="m", b_major="n", flags=_lib.GEMM_NO_WORKSPACE)
        assert p["workspace"] == 0 and len(p["steps"]) == 1 and "amaj=1,bmaj=1" in p["steps"][0]["name"] and p["steps"][0]["family"] == "gemm_mfma_tn_256_w4"
    # ... also on 128 x 128 tiles (a small problem left to the library; a named tile)
    p = run_case(f8, f32, 256, 512, 256, a_major="m", b_major="n")
    assert p["workspace"] == 0 and step_names(p) == ["gemm_mfma_tn_256_w4<W4FP8L,OutF32,waves=4,bias=0,ragged=0,tile=128,amaj=1,bmaj=1,ops=0>"]
    p = run_case(f16, f16, 2048, 2048, 2048, cta=(128, 128, 64), waves=(2, 2, 1), a_major="m")
    assert p["workspace"] == 0 and step_names(p) == ["gemm_mfma_tn_256_w4<W4F16L,OutF16,waves=4,bias=0,ragged=0,tile=128,amaj=1,bmaj=0,ops=0>"]
    # ... and a K-major copy where no kernel reads the operand as it lies (tiles that reach beyond M, fp8)
    p = run_case(f8, f32, 200, 512, 256, a_major="m", b_major="n")
    assert [s["what"] for s in p["steps"]][:2] == ["kmajor_copy", "kmajor_copy"] and p["workspace"] >= 200 * 256 + 512 * 256
    # short M: whole 128-byte lines of K through LDS, a K tail as a masked trip of the same kernel
    assert step_names(run_case(bf16, f32, 16, 8192, 8192))[0].startswith("gemm_mfma_skinny_lds<InBF16,OutF32,mt=1,ntw=2,waves=4,stages=3>")
    assert step_names(run_case(bf16, f32, 16, 8192, 8224))[0].startswith("gemm_mfma_skinny_lds<InBF16,OutF32,mt=1,ntw=2,")   # a K tail too
    # more than 32 rows of A: 64 rows of B per workgroup where 32 rows would need more rounds on the CUs
    assert step_names(run_case(bf16, bf16, 64, 28672, 8192))[0].startswith("gemm_mfma_skinny_lds<InBF16,OutBF16,mt=4,ntw=4,waves=4,stages=2>")
    assert step_names(run_case(bf16, bf16, 48, 16384, 4096))[0].startswith("gemm_mfma_skinny_lds<InBF16,OutBF16,mt=3,ntw=4,waves=4,stages=2>")
    assert ",ntw=2," in step_names(run_case(bf16, bf16, 64, 8192, 8192))[0]
    assert ",ntw=4," in step_names(run_case(bf16, bf16, 64, 12288, 8192))[0] and ",ntw=2," in step_names(run_case(bf16, bf16, 16, 6144, 8192))[0]
    assert ",ntw=1," in step_names(run_case(bf16, bf16, 16, 4096, 8192))[0]
    # K ranges count against the CUs as well: 256 workgroups of 16 rows stay whole, 128 of 32 rows take two ranges
    p = run_case(bf16, f32, 64, 4096, 14336, split_k=-1)
    assert p["steps"][0]["split"] == 2 and ",ntw=2," in p["steps"][0]["name"], p["text"]
    # more than 16 rows and more 128-wide tiles than CUs (a very short K: three quarters of the CUs): tiles, not the short-M kernel
    for (M, N, K, fam) in ((64, 65536, 2048, "gemm_mfma_tn_256_w4"), (17, 24576, 512, "gemm_mfma_tn_128"), (64, 65536, 3072, "gemm_mfma_tn_256_w4"),
                           (64, 131072, 4096, "gemm_mfma_tn_256_w4"), (64, 65536, 4096, "gemm_mfma_tn_256_w4"), (64, 24448, 512, "gemm_mfma_skinny_lds"),
                           (64, 65536, 8192, "gemm_mfma_tn_256_w4"), (48, 49152, 8192, "gemm_mfma_skinny_lds"), (64, 32768, 2048, "gemm_mfma_skinny_lds"),
                           (64, 32768, 1024, "gemm_mfma_tn_128"), (16, 65536, 512, "gemm_mfma_skinny_lds"), (64, 32768, 2056, "gemm_mfma_skinny_lds")):
        assert run_case(bf16, bf16, M, N, K)["steps"][0]["family"] == fam, (M, N, K)
    assert run_case(mh.F32, mh.F32, 64, 65536, 512)["steps"][0]["family"] == "gemm_mfma_skinny_lds"   # fp32 operands stay on the short-M kernel
    # small N and a long K: the library's own K ranges for the line kernel, then the reduction
    p = run_case(bf16, f32, 16, 1024, 32768, split_k=-1)
    assert p["steps"][0]["family"] == "gemm_mfma_skinny_lds" and p["steps"][0]["split"] == 4 and p["steps"][-1]["what"] == "splitk_reduce"
    # ragged problems: the guarded forms of the hand-ordered kernel (K of whole lines; with a C the instance whose
    # epilogue is the general one)
    assert "ragged=1" in step_names(run_case(f16, f16, 4000, 4000, 4096))[0] and step_names(run_case(f16, f16, 4000, 4000, 4096))[0].startswith("gemm_mfma_tn_256_w4<W4F16L")
    # (a K that ends inside a 128-byte row: the same guarded form, the tail masked in registers; the compiler-scheduled
    # kernel when the call names it)
    assert step_names(run_case(f16, f16, 4096, 4096, 4000))[0] == "gemm_mfma_tn_256_w4<W4F16L,OutF16,waves=8,bias=0,ragged=1,tile=256,amaj=0,bmaj=0,ops=0>"
    assert step_names(run_case(f8, bf16, 4000, 4096, 4080))[0] == "gemm_mfma_tn_256_w4<W4FP8L,OutBF16,waves=8,bias=0,ragged=1,tile=256,amaj=0,bmaj=0,ops=0>"
    assert step_names(run_case(f16, f16, 4096, 4096, 4000, stages=2))[0].startswith("gemm_mfma_tn_256<InF16,OutF16,waves=8,ops=0,amaj=0,bmaj=0,ragged=1")
    assert step_names(run_case(f16, f16, 4000, 4000, 4096, with_c=True))[0] == "gemm_mfma_tn_256_w4<W4F16L,OutF16,waves=8,bias=0,ragged=1,tile=256,amaj=0,bmaj=0,ops=1>"
    # an element-wise operation with a whole-matrix operand: the same k-loop with the general epilogue, every operand type
    # (fp8 keeps its 16x16x128 MFMA)
    def gate(m, n):
        return mh.gemm_epilogue(alpha=0.5, op=_lib.MAP_MUL, operand=tensor(PX, f32, (m, n), (n, 1)))
    assert step_names(run_case(f16, f16, 4096, 4096, 4096, ep=gate(4096, 4096)))[0] == "gemm_mfma_tn_256_w4<W4F16L,OutF16,waves=8,bias=0,ragged=0,tile=256,amaj=0,bmaj=0,ops=1>"
    assert step_names(run_case(f8, bf16, 8192, 8192, 8192, ep=gate(8192, 8192)))[0] == "gemm_mfma_tn_256_w4<W4FP8L,OutBF16,waves=8,bias=0,ragged=0,tile=256,amaj=0,bmaj=0,ops=1>"
    assert step_names(run_case(f32, f32, 4096, 4096, 4096, ep=gate(4096, 4096)))[0] == "gemm_mfma_tn_256_w4<W4F32L,OutF32,waves=8,bias=0,ragged=0,tile=256,amaj=0,bmaj=0,ops=1>"
    assert step_names(run_case(f16, f16, 4096, 4096, 4096, ep=gate(4096, 4096), a_major="m"))[0].startswith("gemm_mfma_tn_256<InF16,OutF16,waves=8,ops=1,amaj=1")
    # a ReLU, a scale, a bias (a scalar, one-per-column or one-per-row operand): applied in the lanes' own epilogue of the
    # hand-ordered kernel, every operand type, with or without C; a division goes through the general epilogue
    relu = mh.gemm_epilogue(alpha=0.5, op=_lib.MAP_MAX, scalar=0.0)
    relu_c = mh.gemm_epilogue(alpha=0.5, beta=1.0, op=_lib.MAP_MAX, scalar=0.0)
    assert step_names(run_case(f16, f16, 4096, 4096, 4096, ep=relu))[0] == "gemm_mfma_tn_256_w4<W4F16L,OutF16,waves=8,bias=1,ragged=0,tile=256,amaj=0,bmaj=0,ops=0>"
    assert step_names(run_case(f16, f16, 4096, 4096, 4096, ep=relu_c, with_c=True))[0] == "gemm_mfma_tn_256_w4<W4F16L,OutF16,waves=8,bias=1,ragged=0,tile=256,amaj=0,bmaj=0,ops=0>"
    assert step_names(run_case(f8, bf16, 8192, 8192, 8192, ep=relu))[0] == "gemm_mfma_tn_256_w4<W4FP8L,OutBF16,waves=8,bias=1,ragged=0,tile=256,amaj=0,bmaj=0,ops=0>"
    assert step_names(run_case(f32, f32, 4096, 4096, 4096, ep=relu_c, with_c=True))[0] == "gemm_mfma_tn_256_w4<W4F32L,OutF32,waves=8,bias=1,ragged=0,tile=256,amaj=0,bmaj=0,ops=0>"
    assert "ops=1" in step_names(run_case(f16, f16, 4096, 4096, 4096, ep=mh.gemm_epilogue(op=_lib.MAP_DIV, scalar=3.0)))[0]
    # ... and on the compiler-scheduled kernel where a call names it
    assert step_names(run_case(f16, f16, 4096, 4096, 4096, ep=relu_c, with_c=True, stages=2))[0].startswith("gemm_mfma_tn_256<InF16,OutF16,waves=8,ops=0,amaj=0,bmaj=0,ragged=0,bias=1")
    # thin fringes: whole tiles for the interior, the short-M kernel for each fringe (the right-hand one transposed)
    p = run_case(f16, f16, 4100, 4104, 4096)
    fams = [s["family"] for s in p["steps"]]
    assert fams == ["gemm_mfma_tn_256_w4", "gemm_mfma_skinny_lds", "gemm_mfma_skinny_lds"], p["text"]
    assert p["steps"][1]["ldd"] == 1 and p["steps"][1]["ldd_n"] == 4104 and p["steps"][1]["M"] == 8
    # a last round that fills little of the chip goes to a launch of its own, on 128 x 128 tiles two to a CU
    p = run_case(f16, f16, 6144, 6144, 6144, waves=(1, 1, 1))
    assert [s["name"].split(",")[5] for s in p["steps"]] == ["tile=256", "tile=128"] and p["steps"][0]["M"] + p["steps"][1]["M"] == 6144
    assert len(run_case(f16, f16, 5120, 5120, 5120, waves=(1, 1, 1))["steps"]) == 1
    # a bias row in the epilogue: the bias instance of the hand-ordered kernel
    bias = mh.gemm_epilogue(alpha=1.0, op=_lib.MAP_ADD, operand=tensor(PX, f32, (4096, 4096), (0, 1)))
    assert "bias=1" in step_names(run_case(f16, f16, 4096, 4096, 4096, cta=(256, 256, 64), ep=bias))[0]
    assert step_names(run_case(f16, f16, 4096, 4096, 4096, cta=(256, 256, 64), ep=bias))[0].startswith("gemm_mfma_tn_256_w4")
    # the tile config 3 names (128 x 128 x 32)
    p = run_case(f16, f16, 4096, 4096, 4096, cta=(128, 128, 32), waves=(2, 2, 1))
    # (stages of 128 x 32 in a ring of four, k-steps of two stages, two workgroups to a CU)
    assert p["steps"][0]["name"].startswith("gemm_mfma_tn_256_w4<W4F16x2R4,OutF16,waves=4,") and p["steps"][0]["lds"] == 65536, p["text"]
    # mid-size problems: 128 x 128 tiles with K ranges, or 64 x 64 tiles, by the cost model; never 256 x 256 tiles with a split
    assert run_case(f16, f16, 1024, 1024, 1024, split_k=-1)["steps"][0]["tile"].startswith("64x64")
    assert run_case(f16, f16, 256, 256, 65536, split_k=-1)["steps"][0]["split"] > 1
    # the 32 x 32 atoms: the register-staged 128 x 128 kernel, or whole 256 x 256 tiles (named, or chosen when they fill
    # half the chip)
    assert "atom=32" in step_names(run_case(f16, f32, 512, 512, 512, atom=mh.MFMA_F32_32x32x16_F16, cta=(128, 128, 32), waves=(2, 2, 1)))[0]
    assert step_names(run_case(f16, f32, 512, 512, 512, atom=mh.MFMA_F32_32x32x16_F16, cta=(256, 256, 64)))[0] == "gemm_mfma_tn_256_atom32<InF16,OutF32,ops=0>"
    assert step_names(run_case(f16, f16, 4096, 4096, 4096, atom=mh.MFMA_F32_32x32x16_F16))[0] == "gemm_mfma_tn_256_atom32<InF16,OutF16,ops=0>"
    assert step_names(run_case(f16, f16, 4096, 4096, 4096, atom=mh.MFMA_F32_32x32x16_F16, ep=mh.gemm_epilogue(op=_lib.MAP_MAX, scalar=0.0)))[0] == "gemm_mfma_tn_256_atom32<InF16,OutF16,ops=1>"
    assert "atom=32" in step_names(run_case(f16, f16, 1024, 1024, 1024, atom=mh.MFMA_F32_32x32x16_F16))[0]
    assert isinstance(run_case(f16, f32, 500, 512, 512, atom=mh.MFMA_F32_32x32x16_F16, cta=(256, 256, 64)), mh.MoyeError)
    assert isinstance(run_case(f16, f32, 512, 512, 512, atom=mh.MFMA_F32_32x32x16_F16, cta=(256, 256, 32)), mh.MoyeError)
    # a partitioned part (64 CUs in 2 XCDs): the same kernel, planned for fewer CUs
    p = run_case(f16, f16, 4096, 4096, 4096, cus=64)
    assert p["cus"] == 64 and p["xcds"] == 2 and p["steps"][0]["family"] == "gemm_mfma_tn_256_w4"


def test_every_branch_of_the_dispatcher_is_reached():
    """Run after the enumerations above (pytest keeps file order): every kernel family and instance kind the dispatcher can
    emit was emitted at least once, so no branch is dead and none is untested."""
    if len(SEEN) < 10:
        pytest.skip("the enumerating tests did not run in this process")
    want = {"gemm_mfma_tn_256_w4", "gemm_mfma_tn_256", "gemm_mfma_tn_128", "gemm_mfma_tn", "gemm_mfma_tn_256_ring", "gemm_mfma_tn_256_pp",
            "gemm_mfma_skinny_lds", "kmajor_copy", "splitk_reduce",
            "gemm_mfma_tn_256_w4:ragged=1", "gemm_mfma_tn_256_w4:bias=1", "gemm_mfma_tn_256_w4:ops=1", "gemm_mfma_tn_256_w4:amaj=1", "gemm_mfma_tn_256_w4:bmaj=1",
            "gemm_mfma_tn_256_w4:tile=128", "gemm_mfma_tn_256:ragged=1", "gemm_mfma_tn_256:ops=1", "gemm_mfma_tn_256:bias=1",
            "gemm_mfma_tn_256:amaj=1", "gemm_mfma_tn_128:ragged=1", "gemm_mfma_tn_128:ops=1", "gemm_mfma_tn_128:amaj=1", "gemm_mfma_tn_128:bias=1",
            "gemm_mfma_tn:edge=1", "gemm_mfma_tn:atom=32"}
    assert want <= SEEN, sorted(want - SEEN)


def test_universal_fma_plan_and_errors():
    A, B, D = operands(256, 256, 256, mh.F32, mh.F32, "m", "k")
    p = mh.gemm_explain(mh.tiled_mma_desc(mh.MMA_UNIVERSAL_FMA, cta_tile=(32, 32, 8)), D, A, B)
    assert p["steps"][0]["name"] == "gemm_universal<32,32,8>" and p["workspace"] == 0
    with pytest.raises(mh.MoyeError):           # K of A and B differ
        mh.gemm_explain(mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16), tensor(PD, mh.F32, (64, 64), (64, 1)),
                        tensor(PA, mh.F16, (64, 32), (32, 1)), tensor(PB, mh.F16, (64, 64), (64, 1)))
    import ctypes as C
    buf = C.create_string_buffer(8)              # a buffer too small for the text
    A, B, D = operands(256, 256, 256, mh.F16, mh.F32)
    st = _lib.lib().moye_gemm_explain(C.byref(mh.tiled_mma_desc(mh.MFMA_F32_16x16x32_F16)), C.byref(D), C.byref(A), C.byref(B), None, None, 0, buf, 8)
    assert st == _lib.ERR_BUFFER

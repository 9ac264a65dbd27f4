"""Host-side model of the load-to-LDS addressing of the 256 x 256 MFMA kernels (csrc/gemm_mfma256.hip,
csrc/gemm_mfma256w4.hip): for every wave, lane, instruction, ring stage and k-stage, the global byte range against
the operand tile and the LDS byte range against the kernel's dynamic LDS, both 16-byte aligned, and every LDS chunk of
a stage written exactly once.  No GPU: this is the bounds check that runs before such a kernel may.

`global_load_lds_dwordx4 v_off, s[base], offset:imm` reads 16 bytes per lane at base + zext(v_off) + imm and writes
them to LDS at M0 + imm + 16 * lane (the instruction offset is applied to BOTH addresses; imm is a signed 13-bit
field).  The shipped kernels use imm = 0 and one M0 write per instruction.  An earlier variant of the hand-ordered
kernel used imm = 0, 1024, 2048, 3072 behind one M0 write (each lane offset lowered by imm so that the global address
stays put) and faulted the GPU; it is not in the tree.  The model below shows that variant's arithmetic in bounds under
the semantics above, and out of bounds on the GLOBAL side (below the tile's first byte for its first rows, beyond its
last for negative immediates: a page fault where the tile touches the end of an allocation) if the hardware did not
apply imm to the global address of this instruction form.  So no mistake in the variant's own arithmetic explains the
faults; what the instruction does with imm is the open question, which only the hardware can answer, and until it is
answered the variant stays out."""
import itertools

LDS_BYTES = 160 * 1024


def swz4(row):  # swz<4>: chunk permutation of a 64-byte LDS row (mfma_common.hpp)
    return (row // 2) & 3


def w4_plan(waves, pitch, nstages, imm_variant=False):
    """(global offset from the operand tile, LDS byte address, imm) of every lane of every load-to-LDS instruction of
    gemm_mfma_tn_256_w4: ring of five 32 KiB stages, 64-byte rows, A tile then B tile."""
    BM, CPR, STAGES = 256, 4, 5
    stage_bytes, a_tile_bytes = (BM + BM) * CPR * 16, BM * CPR * 16
    RW = BM // waves
    LD = RW // 16
    for g, wave, q, lane in itertools.product(range(nstages), range(waves), range(2 * LD), range(64)):
        slot = g % STAGES
        lrow, lch = wave * RW + (lane >> 2), (lane & 3) ^ swz4(lane >> 2)
        voff = (lrow + 16 * (q % LD)) * pitch + lch * 16
        lds_first = slot * stage_bytes + (0 if q < LD else a_tile_bytes) + (wave * RW + 16 * (q % LD)) * 64
        imm = 0
        if imm_variant:       # one M0 write for the LD instructions of an operand: M0 = first block, imm = 1024 * (q % LD)
            imm = 1024 * (q % LD)
            lds_first -= imm
            voff -= imm
        yield dict(g=g, wave=wave, q=q, lane=lane, operand="A" if q < LD else "B", base=g * 64, voff=voff, imm=imm, m0=lds_first,
                   row=lrow + 16 * (q % LD), chunk=lch)


def check(plan, pitch, apply_imm_to_global=True, apply_imm_to_lds=True):
    """Bounds and coverage of a plan; returns the list of violations (empty = safe)."""
    bad, seen = [], {}
    for p in plan:
        if not (0 <= p["voff"] < 2 ** 32) or not (-4096 <= p["imm"] <= 4095):
            bad.append(("field range", p))
            continue
        gaddr = p["base"] + p["voff"] + (p["imm"] if apply_imm_to_global else 0)       # relative to the tile's first byte
        want = p["row"] * pitch + p["g"] * 64 + p["chunk"] * 16
        lo, hi = 0, 255 * pitch + pitch                                                   # the tile's 256 rows
        if gaddr % 16 or not (lo <= gaddr and gaddr + 16 <= hi):
            bad.append(("global out of the tile", p))
        elif gaddr != want:
            bad.append(("global address is not the element's", p))
        laddr = p["m0"] + (p["imm"] if apply_imm_to_lds else 0) + 16 * p["lane"]
        if laddr % 16 or not (0 <= laddr and laddr + 16 <= LDS_BYTES):
            bad.append(("LDS out of the allocation", p))
        key = (p["g"], laddr)
        if key in seen:
            bad.append(("LDS chunk written twice", p))
        seen[key] = True
    return bad


def test_shipped_load_to_lds_addressing_is_in_bounds():
    for waves, pitch, nstages in ((8, 8192, 7), (4, 8192, 7), (8, 128, 2), (4, 64 * 5, 5), (8, 1 << 20, 6)):
        plan = list(w4_plan(waves, pitch, nstages))
        assert check(plan, pitch) == []
        per_stage = {}
        for p in plan:
            per_stage[p["g"]] = per_stage.get(p["g"], 0) + 1
        assert all(n == 2 * 256 * 4 for n in per_stage.values())          # every 16-byte chunk of both tiles, once


def test_immediate_offset_variant_under_three_readings_of_the_instruction():
    pitch = 8192
    for waves in (4, 8):
        plan = list(w4_plan(waves, pitch, 6, imm_variant=True))
        assert any(p["imm"] for p in plan)
        assert check(plan, pitch) == []                                    # as documented: in bounds, right elements
        g = check(plan, pitch, apply_imm_to_global=False)
        assert g and {k for k, _ in g} <= {"global out of the tile", "global address is not the element's"}
    # the first form of the variant, negative immediates (M0 = last block): the lane offsets grow instead; same verdict
    plan = []
    for p in w4_plan(8, pitch, 6):
        k = p["q"] % 2
        plan.append(dict(p, imm=-1024 * (1 - k), voff=p["voff"] + 1024 * (1 - k), m0=p["m0"] + 1024 * (1 - k)))
    assert check(plan, pitch) == [] and check(plan, pitch, apply_imm_to_global=False)


# ---------------------------------------------------------------------------------------------------------------------
# gemm_mfma_tn_256 with ragged tiles (csrc/gemm_mfma256.hip, kRagged): rows clamped to the operand's last row, pieces
# beyond K swapped for the row's first piece in the last k-tile.  The guarded instances of the hand-ordered kernel
# (csrc/gemm_mfma_w4_kernel.hpp) address their stages the same way: wave w brings rows 32 w + 8 i + lane / 8 (clamped),
# lane l logical piece (l % 8) ^ (l / 8 % 8), a lane beyond K in the last stage minus its piece offset (tail_cut).
# ---------------------------------------------------------------------------------------------------------------------

def ragged256_plan(rows, k_bytes, pitch, tile):
    """(byte offset from the operand's first byte, LDS byte address, row, piece) of every lane of every load-to-LDS
    instruction that fills one operand's 256-row tile `tile`, for every k-tile; rows = M (or N)."""
    waves, WROWS, LD = 8, 32, 4
    ktiles = (k_bytes + 127) // 128
    k_rem = (k_bytes % 128) // 16
    k_valid = k_rem if k_rem else 8
    for kt, wave, i, lane in itertools.product(range(ktiles), range(waves), range(LD), range(64)):
        lrow, lch = wave * WROWS + (lane >> 3), (lane & 7) ^ (lane >> 3)
        row0 = tile * 256 + lrow
        base = min(row0, rows - 1) * pitch + lch * 16
        more = max(rows - 1 - row0, 0)
        tail_delta = 0 if lch < k_valid else -lch * 16
        off = base + min(8 * i, more) * pitch + kt * 128 + (tail_delta if kt == ktiles - 1 else 0)
        lds = (kt & 1) * (512 * 128) + (wave * WROWS * 8 + 8 * 8 * i) * 16 + 16 * lane
        yield dict(kt=kt, off=off, lds=lds, row=min(row0 + 8 * i, rows - 1), want_row=row0 + 8 * i, piece=lch,
                   masked=kt == ktiles - 1 and lch >= k_valid)


def test_ragged_256_tile_addressing_stays_inside_the_operand():
    for rows, k_elems, pad in ((4000, 4000, 0), (300, 8, 8), (257, 72, 0), (4099, 4104, 24), (256, 64, 0), (1, 40, 0)):
        k_bytes = k_elems * 2
        pitch = k_bytes + pad * 2
        assert pitch % 16 == 0 and k_bytes % 16 == 0
        for tile in range((rows + 255) // 256):
            seen = set()
            for p in ragged256_plan(rows, k_bytes, pitch, tile):
                r, c = divmod(p["off"], pitch)
                assert 0 <= p["off"] and p["off"] % 16 == 0
                assert r < rows and c + 16 <= k_bytes, (rows, k_elems, tile, p)         # inside the operand's own bytes
                assert r == p["row"]
                if not p["masked"]:
                    assert c == p["kt"] * 128 + p["piece"] * 16                          # the piece the fragment reads expect
                assert 0 <= p["lds"] and p["lds"] + 16 <= 2 * 512 * 128 and p["lds"] % 16 == 0
                key = (p["kt"], p["lds"])
                assert key not in seen
                seen.add(key)
            assert len(seen) == ((k_bytes + 127) // 128) * 256 * 8                       # every piece of every stage, once


# ---------------------------------------------------------------------------------------------------------------------
# gemm_mfma_skinny_lds (csrc/gemm_mfma_skinny.hip): per-wave rings of whole 128-byte lines
# ---------------------------------------------------------------------------------------------------------------------

def skinny_lines_plan(M, N, k_bytes, MT, NTW, block, waves=4, stages=3):
    ROWS = 16 * NTW + 16 * MT
    LD, STAGE = ROWS // 8, ROWS * 8
    lines = k_bytes // 128
    n0 = block * 16 * NTW
    for wave, j, lane in itertools.product(range(waves), range(LD), range(64)):
      s0 = lines * wave // waves
      length = lines * (wave + 1) // waves - s0          # the waves' K ranges: as even as whole lines come
      first = (block // 8) % length if length else 0
      for t in range(length):
        r = 8 * j + (lane >> 3)
        lch = (lane & 7) ^ (lane >> 3)
        line = s0 + (t + first) % length
        if j < 2 * NTW:
            operand, row = "B", min(n0 + r, N - 1)
        else:
            operand, row = "A", min(r - 16 * NTW, M - 1)
        lds = (wave * stages * STAGE + (t % stages) * STAGE + 64 * j) * 16 + 16 * lane
        yield dict(operand=operand, row=row, col=line * 128 + lch * 16, lds=lds, wave=wave, t=t, line=line)


def test_short_m_line_staging_addressing():
    for M, N, k_bytes, MT, NTW in ((16, 8192, 16384, 1, 2), (64, 100, 512, 4, 1), (33, 8191, 1536, 3, 2), (1, 32, 2048, 1, 1),
                                   (48, 12000, 512, 3, 2), (16, 8192, 640, 1, 2), (7, 64, 128, 1, 1), (64, 8192, 1408, 4, 2)):
        assert k_bytes % 128 == 0 and (M + 15) // 16 == MT
        lds_bytes = 4 * 3 * (16 * NTW + 16 * MT) * 128
        assert lds_bytes <= LDS_BYTES
        blocks = (N + 16 * NTW - 1) // (16 * NTW)
        for block in {0, 1, 9, blocks // 2, blocks - 1}:
            seen, lines_of_wave = set(), {}
            for p in skinny_lines_plan(M, N, k_bytes, MT, NTW, block):
                rows = N if p["operand"] == "B" else M
                assert 0 <= p["row"] < rows and 0 <= p["col"] and p["col"] + 16 <= k_bytes
                assert 0 <= p["lds"] and p["lds"] + 16 <= lds_bytes
                key = (p["wave"], p["t"], p["lds"])
                assert key not in seen
                seen.add(key)
                lines_of_wave.setdefault(p["wave"], set()).add(p["line"])
            # the waves' K ranges are disjoint and together cover K
            allv = sorted(x for v in lines_of_wave.values() for x in v)
            assert allv == list(range(k_bytes // 128))

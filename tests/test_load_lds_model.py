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
    # the 2.1 form of the variant, negative immediates (M0 = last block): the lane offsets grow instead; same verdict
    plan = []
    for p in w4_plan(8, pitch, 6):
        k = p["q"] % 2
        plan.append(dict(p, imm=-1024 * (1 - k), voff=p["voff"] + 1024 * (1 - k), m0=p["m0"] + 1024 * (1 - k)))
    assert check(plan, pitch) == [] and check(plan, pitch, apply_imm_to_global=False)

"""The build's check on kernels whose MFMAs and LDS fragment reads are inline assembly (moye.jl_amd/build.py,
asm_mfma_hazards): the compiler does not know that those results are still in flight, so nothing of its own may name an
accumulator or a fragment register between the MFMAs.  Synthetic listings: what must pass and what must be caught."""
import os
import sys

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "moye.jl_amd"))
import build  # noqa: E402

LOOP = """_Z4kernv:
\ts_load_dwordx2 s[0:1], s[4:5], 0x0
.LBB0_1:
\tds_read_b128 v[10:13], v1 offset:0
\ts_waitcnt lgkmcnt(0)
\tv_mfma_f32_16x16x32_f16 a[0:3], v[10:13], v[14:17], a[0:3]
\tds_read_b128 v[14:17], v1 offset:2048
%s
\ts_cbranch_scc1 .LBB0_1
\ts_nop 15
\t; MOYE_ACC_SETTLED
\tv_accvgpr_read_b32 v20, a1
\tv_mov_b32 v21, v11
\ts_endpgm
"""


def scan(extra):
    return build.asm_mfma_hazards((LOOP % extra).splitlines(), "t.s")


def test_clean_loop_passes():
    acc, frag = scan("\tv_add_u32 v3, v2, v4")
    assert acc == [] and frag == []


def test_a_register_that_was_given_a_new_owner_is_no_fragment_any_more():
    acc, frag = scan("\tv_mov_b32 v10, v2\n\tv_add_u32 v3, v10, v4")
    assert acc == [] and frag == []


def test_a_copy_of_a_fragment_between_the_mfmas_is_caught():
    acc, frag = scan("\tv_mov_b32 v20, v15")
    assert acc == [] and len(frag) == 1 and "v_mov_b32 v20, v15" in frag[0]
    # a register range that overlaps a fragment, and a store that reads one
    assert len(scan("\tv_lshl_add_u64 v[30:31], v[12:13], 0, s[2:3]")[1]) == 1
    assert len(scan("\tglobal_store_dwordx4 v[2:3], v[10:13], off")[1]) == 1


def test_the_fragment_reads_of_operands_that_are_not_k_major_count_too():
    # the transposing reads (16-bit and 8-bit operands) and the single-value reads (fp32 operands) fill fragments as well
    for read in ("ds_read_b64_tr_b16 v[40:41], v1 offset:64", "ds_read_b64_tr_b8 v[40:41], v1 offset:64", "ds_read_b32 v40, v1 offset:64"):
        assert scan("\t" + read)[1] == []
        acc, frag = scan("\t" + read + "\n\tv_mov_b32 v20, v40")
        assert acc == [] and len(frag) == 1 and "v_mov_b32 v20, v40" in frag[0], read
        assert scan("\t" + read + "\n\tv_mov_b32 v40, v2\n\tv_add_u32 v3, v40, v4")[1] == []


def test_an_accumulator_named_by_anything_but_an_mfma_is_caught():
    acc, frag = scan("\tv_accvgpr_read_b32 v20, a2")
    assert len(acc) == 1 and "a2" in acc[0] and frag == []
    assert len(scan("\tv_accvgpr_write_b32 a3, v2")[0]) == 1


def test_the_shipped_listing_is_checked_at_build_time():
    # build() runs the check for every source with inline-assembly MFMAs; the hand-ordered GEMM kernel is one
    with open(os.path.join(build.CSRC, "gemm_mfma_w4_kernel.hpp")) as f:
        assert "v_mfma" in f.read()
    users = [s for s in build.SOURCES if s.endswith(".hip") and "gemm_mfma_w4_kernel.hpp" in open(os.path.join(build.CSRC, s)).read()]
    assert users and set(users) == set(build.ASM_MFMA_SOURCES)

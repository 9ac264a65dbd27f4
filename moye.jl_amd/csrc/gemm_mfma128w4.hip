// The hand-ordered kernel (gemm_mfma_w4_kernel.hpp) on the 128 x 128 tile: four waves, two workgroups per CU.
#include "gemm_mfma_w4_kernel.hpp"

namespace moye {

// The 128 x 128 tile on the same kernel: plain f16 / bf16 calls on whole tiles, K a whole number of 128-byte rows; the
// caller has checked divisibility and alignment.
// `stage64`: the tile is named with 64 bytes of K per stage (128 x 128 x 32 for the 16-bit types, the tile the baseline's
// config 3 names): a ring of four such stages, k-steps of two stages, two workgroups per CU.
int32_t gemm_mfma_tn_128_w4_dispatch(int32_t in_dt, int32_t out_dt, GemmArgs a, GemmPlan& plan, bool stage64) {
    a.tiles_m = (a.M + 127) / 128;  // (beyond whole tiles only with kGemmRagged: the caller has checked; then no C either)
    a.tiles_n = (a.N + 127) / 128;
    if (stage64) {
        if ((a.flags & kGemmRagged) || !row_offsets_fit(a, 128, dtype_bytes(in_dt)))
            return fail(MOYE_ERR_UNSUPPORTED, "gemm!: the 128x128 ring of 64-byte-row stages takes whole tiles with rows that span less than 4 GiB");
        if (in_dt == MOYE_F16) {
            switch (out_dt) {
                case MOYE_F32: return launch256_w4<W4F16x2R4, OutF32, 2, false, false, 128>(a, plan);
                case MOYE_F16: return launch256_w4<W4F16x2R4, OutF16, 2, false, false, 128>(a, plan);
                case MOYE_BF16: return launch256_w4<W4F16x2R4, OutBF16, 2, false, false, 128>(a, plan);
                default: break;
            }
        } else if (in_dt == MOYE_BF16) {
            switch (out_dt) {
                case MOYE_F32: return launch256_w4<W4BF16x2R4, OutF32, 2, false, false, 128>(a, plan);
                case MOYE_F16: return launch256_w4<W4BF16x2R4, OutF16, 2, false, false, 128>(a, plan);
                case MOYE_BF16: return launch256_w4<W4BF16x2R4, OutBF16, 2, false, false, 128>(a, plan);
                default: break;
            }
        }
        return fail(MOYE_ERR_UNSUPPORTED, "gemm!: the 128x128 ring of 64-byte-row stages takes f16 or bf16 operands and writes f32, f16 or bf16");
    }
    if (a.flags & kGemmRagged) {
        if (a.C || a.ep_op != MOYE_MAP_IDENTITY) return fail(MOYE_ERR_UNSUPPORTED, "gemm!: ragged tiles of the hand-ordered kernel take no C and no epilogue operation");
        if (in_dt == MOYE_F32) {
            switch (out_dt) {
                case MOYE_F32: return launch256_w4<W4F32L, OutF32, 2, false, true, 128>(a, plan);
                case MOYE_F16: return launch256_w4<W4F32L, OutF16, 2, false, true, 128>(a, plan);
                case MOYE_BF16: return launch256_w4<W4F32L, OutBF16, 2, false, true, 128>(a, plan);
                default: break;
            }
        }
        if (in_dt == MOYE_F8E4M3) {
            switch (out_dt) {
                case MOYE_F32: return launch256_w4<W4FP8L, OutF32, 2, false, true, 128>(a, plan);
                case MOYE_F16: return launch256_w4<W4FP8L, OutF16, 2, false, true, 128>(a, plan);
                case MOYE_BF16: return launch256_w4<W4FP8L, OutBF16, 2, false, true, 128>(a, plan);
                default: break;
            }
        }
        if (in_dt == MOYE_F16) {
            switch (out_dt) {
                case MOYE_F32: return launch256_w4<W4F16L, OutF32, 2, false, true, 128>(a, plan);
                case MOYE_F16: return launch256_w4<W4F16L, OutF16, 2, false, true, 128>(a, plan);
                case MOYE_BF16: return launch256_w4<W4F16L, OutBF16, 2, false, true, 128>(a, plan);
                default: break;
            }
        } else if (in_dt == MOYE_BF16) {
            switch (out_dt) {
                case MOYE_F32: return launch256_w4<W4BF16L, OutF32, 2, false, true, 128>(a, plan);
                case MOYE_F16: return launch256_w4<W4BF16L, OutF16, 2, false, true, 128>(a, plan);
                case MOYE_BF16: return launch256_w4<W4BF16L, OutBF16, 2, false, true, 128>(a, plan);
                default: break;
            }
        }
        return fail(MOYE_ERR_UNSUPPORTED, "gemm!: the hand-ordered 128x128 kernel takes f16 or bf16 operands and writes f32, f16 or bf16");
    }
    if (!row_offsets_fit(a, 128, dtype_bytes(in_dt))) return fail(MOYE_ERR_SHAPE, "gemm!: row pitch too large for the hand-ordered 128x128 MFMA kernel");
    if (a.flags & (kGemmAMajorM | kGemmBMajorN)) return launch128_w4_majors_dispatch(in_dt, out_dt, a, plan);  // (plain calls on whole tiles)
    if (in_dt == MOYE_F32) {
        switch (out_dt) {
            case MOYE_F32: return launch256_w4<W4F32L, OutF32, 2, false, false, 128>(a, plan);
            case MOYE_F16: return launch256_w4<W4F32L, OutF16, 2, false, false, 128>(a, plan);
            case MOYE_BF16: return launch256_w4<W4F32L, OutBF16, 2, false, false, 128>(a, plan);
            default: break;
        }
    }
    if (in_dt == MOYE_F8E4M3) {  // (the 16x16x128 MFMA: twice the rate of the 16x16x32 one the other 128 x 128 kernels issue)
        switch (out_dt) {
            case MOYE_F32: return launch256_w4<W4FP8L, OutF32, 2, false, false, 128>(a, plan);
            case MOYE_F16: return launch256_w4<W4FP8L, OutF16, 2, false, false, 128>(a, plan);
            case MOYE_BF16: return launch256_w4<W4FP8L, OutBF16, 2, false, false, 128>(a, plan);
            default: break;
        }
    }
    if (in_dt == MOYE_F16) {
        switch (out_dt) {
            case MOYE_F32: return launch256_w4<W4F16L, OutF32, 2, false, false, 128>(a, plan);
            case MOYE_F16: return launch256_w4<W4F16L, OutF16, 2, false, false, 128>(a, plan);
            case MOYE_BF16: return launch256_w4<W4F16L, OutBF16, 2, false, false, 128>(a, plan);
            default: break;
        }
    } else if (in_dt == MOYE_BF16) {
        switch (out_dt) {
            case MOYE_F32: return launch256_w4<W4BF16L, OutF32, 2, false, false, 128>(a, plan);
            case MOYE_F16: return launch256_w4<W4BF16L, OutF16, 2, false, false, 128>(a, plan);
            case MOYE_BF16: return launch256_w4<W4BF16L, OutBF16, 2, false, false, 128>(a, plan);
            default: break;
        }
    }
    return fail(MOYE_ERR_UNSUPPORTED, "gemm!: the hand-ordered 128x128 kernel takes f16, bf16 or fp8 operands and writes f32, f16 or bf16");
}

}  // namespace moye

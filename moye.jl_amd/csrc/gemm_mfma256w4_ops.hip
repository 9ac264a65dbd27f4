// The hand-ordered kernel (gemm_mfma_w4_kernel.hpp) with an element-wise operation in its epilogue: the eight-wave
// whole-line instances on the 256 x 256 tile, K-major operands, with or without C.  kBias: the operation in the lanes' own
// epilogue (a scalar, one-per-column or one-per-row operand; whole tiles).  kOps: the general epilogue (any operand, whole
// or ragged tiles; also a ragged call with C and no operation).
#include "gemm_mfma_w4_kernel.hpp"

namespace moye {

template <typename In>
static int32_t launch256_w4_ops(int32_t out_dt, const GemmArgs& a, GemmPlan& plan) {
    if ((a.flags & kGemmEpiLaneOp) && !(a.flags & kGemmRagged)) {
        if (!a.C) {  // (the form without C's read paths)
            switch (out_dt) {
                case MOYE_F32: return launch256_w4<In, OutF32, 4, true, false, 256, 0, 0, false, true>(a, plan);
                case MOYE_F16: return launch256_w4<In, OutF16, 4, true, false, 256, 0, 0, false, true>(a, plan);
                case MOYE_BF16: return launch256_w4<In, OutBF16, 4, true, false, 256, 0, 0, false, true>(a, plan);
                default: return fail(MOYE_ERR_UNSUPPORTED, "gemm!: MFMA kernels write f32, f16 or bf16, not %s", dtype_name(out_dt));
            }
        }
        switch (out_dt) {
            case MOYE_F32: return launch256_w4<In, OutF32, 4, true>(a, plan);
            case MOYE_F16: return launch256_w4<In, OutF16, 4, true>(a, plan);
            case MOYE_BF16: return launch256_w4<In, OutBF16, 4, true>(a, plan);
            default: return fail(MOYE_ERR_UNSUPPORTED, "gemm!: MFMA kernels write f32, f16 or bf16, not %s", dtype_name(out_dt));
        }
    }
    if (a.flags & kGemmRagged) {
        switch (out_dt) {
            case MOYE_F32: return launch256_w4<In, OutF32, 4, false, true, 256, 0, 0, true>(a, plan);
            case MOYE_F16: return launch256_w4<In, OutF16, 4, false, true, 256, 0, 0, true>(a, plan);
            case MOYE_BF16: return launch256_w4<In, OutBF16, 4, false, true, 256, 0, 0, true>(a, plan);
            default: return fail(MOYE_ERR_UNSUPPORTED, "gemm!: MFMA kernels write f32, f16 or bf16, not %s", dtype_name(out_dt));
        }
    }
    switch (out_dt) {
        case MOYE_F32: return launch256_w4<In, OutF32, 4, false, false, 256, 0, 0, true>(a, plan);
        case MOYE_F16: return launch256_w4<In, OutF16, 4, false, false, 256, 0, 0, true>(a, plan);
        case MOYE_BF16: return launch256_w4<In, OutBF16, 4, false, false, 256, 0, 0, true>(a, plan);
        default: return fail(MOYE_ERR_UNSUPPORTED, "gemm!: MFMA kernels write f32, f16 or bf16, not %s", dtype_name(out_dt));
    }
}

// the caller has checked: K-major operands, K of whole 128-byte rows, eight waves; tiles beyond M or N with kGemmRagged
int32_t launch256_w4_ops_dispatch(int32_t in_dt, int32_t out_dt, const GemmArgs& a, GemmPlan& plan) {
    switch (in_dt) {
        case MOYE_F16: return launch256_w4_ops<W4F16L>(out_dt, a, plan);
        case MOYE_BF16: return launch256_w4_ops<W4BF16L>(out_dt, a, plan);
        case MOYE_F8E4M3: return launch256_w4_ops<W4FP8L>(out_dt, a, plan);
        case MOYE_F32: return launch256_w4_ops<W4F32L>(out_dt, a, plan);
        default: return fail(MOYE_ERR_UNSUPPORTED, "gemm!: no MFMA atom for %s inputs", dtype_name(in_dt));
    }
}

}  // namespace moye

// The hand-ordered kernel (gemm_mfma_w4_kernel.hpp) on the 256 x 256 tile with K-major operands: plain and guarded
// instances of every operand type and schedule (those with an element-wise operation: gemm_mfma256w4_ops.hip).
#include "gemm_mfma_w4_kernel.hpp"

namespace moye {

template <typename In, int WGN>
static int32_t launch256_w4_out(int32_t out_dt, const GemmArgs& a, GemmPlan& plan) {
    if (a.flags & (kGemmAMajorM | kGemmBMajorN)) {
        if constexpr (In::kRow == 128 && WGN == 4) {
            if ((a.flags & (kGemmRagged | kGemmEpiLaneOp)) || a.ep_op != MOYE_MAP_IDENTITY)
                return fail(MOYE_ERR_UNSUPPORTED, "gemm!: the hand-ordered kernel takes operands that are not K-major in plain calls on whole tiles only");
            return launch256_w4_majors_dispatch(In::kDt, out_dt, a, plan);
        } else {
            return fail(MOYE_ERR_UNSUPPORTED, "gemm!: this schedule of the hand-ordered kernel takes K-major operands only");
        }
    }
    // An element-wise operation, or a C on ragged tiles: gemm_mfma256w4_ops.hip (the operation in the lanes' own epilogue
    // where its operand is a scalar, one per column or one per row and the tiles are whole; the general epilogue otherwise)
    if (a.ep_op != MOYE_MAP_IDENTITY || ((a.flags & kGemmRagged) && a.C)) {
        if constexpr (In::kRow == 128 && WGN == 4)
            return launch256_w4_ops_dispatch(In::kDt, out_dt, a, plan);
        else
            return fail(MOYE_ERR_UNSUPPORTED, "gemm!: this schedule of the hand-ordered kernel takes no element-wise epilogue operation");
    }
    if (a.flags & kGemmRagged) {  // tiles that reach beyond M or N: the eight-wave whole-line forms
        if constexpr (In::kRow == 128 && WGN == 4) {
            switch (out_dt) {
                case MOYE_F32: return launch256_w4<In, OutF32, WGN, false, true>(a, plan);
                case MOYE_F16: return launch256_w4<In, OutF16, WGN, false, true>(a, plan);
                case MOYE_BF16: return launch256_w4<In, OutBF16, WGN, false, true>(a, plan);
                default: return fail(MOYE_ERR_UNSUPPORTED, "gemm!: MFMA kernels write f32, f16 or bf16, not %s", dtype_name(out_dt));
            }
        } else {
            return fail(MOYE_ERR_UNSUPPORTED, "gemm!: this schedule of the hand-ordered kernel takes whole tiles only");
        }
    }
    // more tiles than CUs: one workgroup per CU that walks over the tiles (gemm_mfma256w4_persist.hip)
    if constexpr (In::kRow == 128 && WGN == 4 && In::kBytes <= 2) {
        if (a.split <= 1 && (int64_t)a.tiles_m * a.tiles_n > plan.shape.cus && !(a.flags & MOYE_GEMM_NO_PERSIST))
            return launch256_w4_persist_dispatch(In::kDt, out_dt, a, plan);
    }
    switch (out_dt) {
        case MOYE_F32: return launch256_w4<In, OutF32, WGN>(a, plan);
        case MOYE_F16: return launch256_w4<In, OutF16, WGN>(a, plan);
        case MOYE_BF16: return launch256_w4<In, OutBF16, WGN>(a, plan);
        default: return fail(MOYE_ERR_UNSUPPORTED, "gemm!: MFMA kernels write f32, f16 or bf16, not %s", dtype_name(out_dt));
    }
}

template <int WGN>
static int32_t launch256_w4_in(int32_t in_dt, int32_t out_dt, const GemmArgs& a, bool two_stage_steps, bool ring, GemmPlan& plan) {
    switch (in_dt) {
        case MOYE_F16:
            if (two_stage_steps && !ring) return launch256_w4_out<W4F16L, WGN>(out_dt, a, plan);
            return two_stage_steps ? launch256_w4_out<W4F16x2, WGN>(out_dt, a, plan) : launch256_w4_out<W4F16, WGN>(out_dt, a, plan);
        case MOYE_BF16:
            if (two_stage_steps && !ring) return launch256_w4_out<W4BF16L, WGN>(out_dt, a, plan);
            return two_stage_steps ? launch256_w4_out<W4BF16x2, WGN>(out_dt, a, plan) : launch256_w4_out<W4BF16, WGN>(out_dt, a, plan);
        case MOYE_F8E4M3: return ring ? launch256_w4_out<W4FP8, WGN>(out_dt, a, plan) : launch256_w4_out<W4FP8L, WGN>(out_dt, a, plan);
        case MOYE_F32: return two_stage_steps && !ring ? launch256_w4_out<W4F32L, WGN>(out_dt, a, plan) : launch256_w4_out<W4F32, WGN>(out_dt, a, plan);
        default: return fail(MOYE_ERR_UNSUPPORTED, "gemm!: no MFMA atom for %s inputs", dtype_name(in_dt));
    }
}

// 256 x 256 tile, four or eight waves; K a multiple of kstep_bytes = 64 or 128 bytes (fp8: always 128; fp32: always
// 64); the caller has checked divisibility of M and N and alignment.
int32_t gemm_mfma_tn_256_w4_dispatch(int32_t in_dt, int32_t out_dt, GemmArgs a, int waves, int kstep_bytes, bool ring, GemmPlan& plan) {
    a.tiles_m = (a.M + 255) / 256;  // (beyond whole tiles only with kGemmRagged: the caller has checked)
    a.tiles_n = (a.N + 255) / 256;
    // the load-to-LDS addresses are a uniform base plus a 32-bit lane offset
    if (!row_offsets_fit(a, 256, dtype_bytes(in_dt))) return fail(MOYE_ERR_SHAPE, "gemm!: row pitch too large for the 256x256 MFMA kernel");
    const bool two = kstep_bytes == 128;
    return waves == 4 ? launch256_w4_in<2>(in_dt, out_dt, a, two, ring, plan) : launch256_w4_in<4>(in_dt, out_dt, a, two, ring, plan);
}

}  // namespace moye

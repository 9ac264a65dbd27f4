// The hand-ordered kernel (gemm_mfma_w4_kernel.hpp) on the 128 x 128 tile with operands that keep their M- (N-) major form:
// four waves, two workgroups per CU, plain calls on whole tiles (its AMAJ / BMAJ).
#include "gemm_mfma_w4_kernel.hpp"

namespace moye {

template <typename In, int AMAJ, int BMAJ>
static int32_t launch128_w4_majors(int32_t out_dt, const GemmArgs& a, GemmPlan& plan) {
    switch (out_dt) {
        case MOYE_F32: return launch256_w4<In, OutF32, 2, false, false, 128, AMAJ, BMAJ>(a, plan);
        case MOYE_F16: return launch256_w4<In, OutF16, 2, false, false, 128, AMAJ, BMAJ>(a, plan);
        case MOYE_BF16: return launch256_w4<In, OutBF16, 2, false, false, 128, AMAJ, BMAJ>(a, plan);
        default: return fail(MOYE_ERR_UNSUPPORTED, "gemm!: MFMA kernels write f32, f16 or bf16, not %s", dtype_name(out_dt));
    }
}

template <typename In>
static int32_t launch128_w4_majors_in(int32_t out_dt, const GemmArgs& a, GemmPlan& plan) {
    const bool am = a.flags & kGemmAMajorM, bm = a.flags & kGemmBMajorN;
    return am && bm ? launch128_w4_majors<In, 1, 1>(out_dt, a, plan) : am ? launch128_w4_majors<In, 1, 0>(out_dt, a, plan) : launch128_w4_majors<In, 0, 1>(out_dt, a, plan);
}

// the caller has checked: whole 128 x 128 tiles, K of whole 128-byte rows, a plain call, at least one operand not K-major
int32_t launch128_w4_majors_dispatch(int32_t in_dt, int32_t out_dt, const GemmArgs& a, GemmPlan& plan) {
    switch (in_dt) {
        case MOYE_F16: return launch128_w4_majors_in<W4F16L>(out_dt, a, plan);
        case MOYE_BF16: return launch128_w4_majors_in<W4BF16L>(out_dt, a, plan);
        case MOYE_F8E4M3: return launch128_w4_majors_in<W4FP8L>(out_dt, a, plan);
        case MOYE_F32: return launch128_w4_majors_in<W4F32L>(out_dt, a, plan);
        default: return fail(MOYE_ERR_UNSUPPORTED, "gemm!: no MFMA atom for %s inputs", dtype_name(in_dt));
    }
}

}  // namespace moye

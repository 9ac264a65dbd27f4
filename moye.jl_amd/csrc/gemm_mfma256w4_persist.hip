// The hand-ordered kernel (gemm_mfma_w4_kernel.hpp) as one workgroup per CU that walks over the tiles of a launch
// (kPersist): plain calls on whole 256 x 256 tiles with K-major operands, for problems with more tiles than the chip has
// CUs.  A tile's first two stages are requested before the epilogue of the tile before it.
#include "gemm_mfma_w4_kernel.hpp"

namespace moye {

template <typename In>
static int32_t launch256_w4_persist(int32_t out_dt, const GemmArgs& a, GemmPlan& plan) {
    switch (out_dt) {
        case MOYE_F32: return launch256_w4<In, OutF32, 4, false, false, 256, 0, 0, false, false, true>(a, plan);
        case MOYE_F16: return launch256_w4<In, OutF16, 4, false, false, 256, 0, 0, false, false, true>(a, plan);
        case MOYE_BF16: return launch256_w4<In, OutBF16, 4, false, false, 256, 0, 0, false, false, true>(a, plan);
        default: return fail(MOYE_ERR_UNSUPPORTED, "gemm!: MFMA kernels write f32, f16 or bf16, not %s", dtype_name(out_dt));
    }
}

int32_t launch256_w4_persist_dispatch(int32_t in_dt, int32_t out_dt, const GemmArgs& a, GemmPlan& plan) {
    switch (in_dt) {
        case MOYE_F16: return launch256_w4_persist<W4F16L>(out_dt, a, plan);
        case MOYE_BF16: return launch256_w4_persist<W4BF16L>(out_dt, a, plan);
        case MOYE_F8E4M3: return launch256_w4_persist<W4FP8L>(out_dt, a, plan);
        default: return fail(MOYE_ERR_UNSUPPORTED, "gemm!: the persistent form of the hand-ordered kernel takes f16, bf16 or fp8 operands, not %s", dtype_name(in_dt));
    }
}

}  // namespace moye

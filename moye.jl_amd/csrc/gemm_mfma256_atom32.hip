// gemm! with the 32 x 32 MFMA atoms (v_mfma_f32_32x32x16_{f16,bf16,fp8_fp8}, v_mfma_f32_32x32x2_f32) on the 256 x 256 CTA
// tile: the reference's make_tiled_mma takes any atom with any atom layout (src/atom/mma.jl:80-107), and so does the
// 256 x 256 x (128 bytes of K) tile here.  The kernel is gemm_mfma_tn_lds_tile (gemm_mfma_lds_tile.hpp) with AT = 32:
// eight waves as 2 x 4, wave tile 128 x 64 = 4 x 2 MFMA tiles of sixteen accumulators per lane, the LDS stages, loads
// and tile order of the 16 x 16 forms.  Whole tiles, K-major operands; with or without C; an element-wise operation runs
// the general epilogue.
#include "gemm_mfma_lds_tile.hpp"

namespace moye {

template <typename In, typename Out, bool kOps>
__global__ __launch_bounds__(512) void gemm_mfma_tn_256_atom32(GemmArgs p) {
    gemm_mfma_tn_lds_tile<In, Out, 256, 256, 2, 4, kOps, 0, 0, false, false, 32>(p);
}

template <typename In, typename Out, bool kOps>
static int32_t launch256_atom32(const GemmArgs& a, GemmPlan& plan) {
    constexpr int kLds = 2 * (256 + 256) * 128;  // two operand stages, 128 KiB
    static LdsCap cap;
    plan.add_kernel(gemm_mfma_tn_256_atom32<In, Out, kOps>, a, (unsigned)(a.tiles_m * a.tiles_n), (unsigned)(a.split > 1 ? a.split : 1), 512, kLds, &cap,
                    256, 256, 128, In::kDt, Out::kDt, "gemm_mfma_tn_256_atom32<%s,%s,ops=%d>", In::kName, Out::kName, (int)kOps);
    return MOYE_OK;
}

template <typename In>
static int32_t launch256_atom32_out(int32_t out_dt, const GemmArgs& a, GemmPlan& plan) {
    const bool ops = a.ep_op != MOYE_MAP_IDENTITY;
    switch (out_dt) {
        case MOYE_F32: return ops ? launch256_atom32<In, OutF32, true>(a, plan) : launch256_atom32<In, OutF32, false>(a, plan);
        case MOYE_F16: return ops ? launch256_atom32<In, OutF16, true>(a, plan) : launch256_atom32<In, OutF16, false>(a, plan);
        case MOYE_BF16: return ops ? launch256_atom32<In, OutBF16, true>(a, plan) : launch256_atom32<In, OutBF16, false>(a, plan);
        default: return fail(MOYE_ERR_UNSUPPORTED, "gemm!: MFMA kernels write f32, f16 or bf16, not %s", dtype_name(out_dt));
    }
}

// The caller has checked whole tiles, K-major operands and alignment.
int32_t gemm_mfma_tn_256_atom32_dispatch(int32_t in_dt, int32_t out_dt, GemmArgs a, GemmPlan& plan) {
    a.tiles_m = a.M / 256;
    a.tiles_n = a.N / 256;
    switch (in_dt) {
        case MOYE_F16: return launch256_atom32_out<InF16>(out_dt, a, plan);
        case MOYE_BF16: return launch256_atom32_out<InBF16>(out_dt, a, plan);
        case MOYE_F8E4M3: return launch256_atom32_out<InFP8>(out_dt, a, plan);
        case MOYE_F32: return launch256_atom32_out<InF32>(out_dt, a, plan);
        default: return fail(MOYE_ERR_UNSUPPORTED, "gemm!: no MFMA atom for %s inputs", dtype_name(in_dt));
    }
}

}  // namespace moye

// gemm! on the matrix cores, 128 x 128 x (128 bytes of K) CTA tile with the load-to-LDS schedule of
// gemm_mfma_lds_tile.hpp: four waves as 2 x 2 (wave tile 64 x 64, 64 accumulator registers per lane), 64 KiB of LDS, so
// two workgroups share a CU and cover each other's barriers and load stalls.  For problems that do not fill the chip
// with 256 x 256 tiles; against the kernel of gemm_mfma.hip, which stages its operands through registers (fp16,
// same box): 4096^3 156 -> 123 us, 2048^3 29.5 -> 22.9 us, 256 x 8192 x 8192 98 -> 68 us, 8192 x 1024 x 4096 80 -> 63 us.
//
// kOps: element-wise operation in the epilogue; kRagged (with kOps): tiles that reach beyond M, N or K (rows clamped to
// the operand's last row, the K tail masked in registers, guarded stores) -- the predication the reference's copyto_if!
// is meant for (src/algorithm/copy.jl:4-16).
#include "gemm_mfma_lds_tile.hpp"

namespace moye {

template <typename In, typename Out, bool kOps = false, bool kRagged = false, int AMAJ = 0, int BMAJ = 0, bool kBias = false>
__global__ __launch_bounds__(256, 2) void gemm_mfma_tn_128(GemmArgs p) {
    gemm_mfma_tn_lds_tile<In, Out, 128, 128, 2, 2, kOps, AMAJ, BMAJ, kRagged, kBias>(p);
}

template <typename In, typename Out, bool kOps, bool kRagged, int AMAJ = 0, int BMAJ = 0, bool kBias = false>
static int32_t launch128_instance(const GemmArgs& a, GemmPlan& plan) {
    constexpr int kLds = 2 * (128 + 128) * 128;  // two operand stages, 64 KiB
    static LdsCap cap;
    plan.add_kernel(gemm_mfma_tn_128<In, Out, kOps, kRagged, AMAJ, BMAJ, kBias>, a, (unsigned)(a.tiles_m * a.tiles_n), (unsigned)(a.split > 1 ? a.split : 1), 256,
                    kLds, &cap, 128, 128, 128, In::kDt, Out::kDt, "gemm_mfma_tn_128<%s,%s,ops=%d,ragged=%d,amaj=%d,bmaj=%d,bias=%d>", In::kName, Out::kName,
                    (int)kOps, (int)kRagged, AMAJ, BMAJ, (int)kBias);
    return MOYE_OK;
}

template <typename In, typename Out>
static int32_t launch128(const GemmArgs& a, GemmPlan& plan) {
    const bool am = a.flags & kGemmAMajorM, bm = a.flags & kGemmBMajorN;
    if (am || bm) {
        // operands that are not K-major (AMAJ / BMAJ of gemm_mfma_lds_tile.hpp): 16-bit types, whole tiles (the host checked)
        if constexpr (In::kBytes == 2) {
            if (a.flags & kGemmRagged) return fail(MOYE_ERR_UNSUPPORTED, "gemm!: ragged tiles take K-major operands");
            const bool ops = a.ep_op != MOYE_MAP_IDENTITY;
            if (am && bm) return ops ? launch128_instance<In, Out, true, false, 1, 1>(a, plan) : launch128_instance<In, Out, false, false, 1, 1>(a, plan);
            if (am) return ops ? launch128_instance<In, Out, true, false, 1, 0>(a, plan) : launch128_instance<In, Out, false, false, 1, 0>(a, plan);
            return ops ? launch128_instance<In, Out, true, false, 0, 1>(a, plan) : launch128_instance<In, Out, false, false, 0, 1>(a, plan);
        } else {
            return fail(MOYE_ERR_UNSUPPORTED, "gemm!: operands that are not K-major run natively with 16-bit types only");
        }
    }
    if (a.flags & kGemmRagged)
        return a.ep_op != MOYE_MAP_IDENTITY ? launch128_instance<In, Out, true, true>(a, plan) : launch128_instance<In, Out, false, true>(a, plan);
    if (a.flags & kGemmEpiLaneOp) return launch128_instance<In, Out, false, false, 0, 0, true>(a, plan);  // a bias, a ReLU, a scale: in the lanes
    if (a.ep_op != MOYE_MAP_IDENTITY) return launch128_instance<In, Out, true, false>(a, plan);
    return launch128_instance<In, Out, false, false>(a, plan);
}

template <typename In>
static int32_t launch128_out(int32_t out_dt, const GemmArgs& a, GemmPlan& plan) {
    switch (out_dt) {
        case MOYE_F32: return launch128<In, OutF32>(a, plan);
        case MOYE_F16: return launch128<In, OutF16>(a, plan);
        case MOYE_BF16: return launch128<In, OutBF16>(a, plan);
        default: return fail(MOYE_ERR_UNSUPPORTED, "gemm!: MFMA kernels write f32, f16 or bf16, not %s", dtype_name(out_dt));
    }
}

// K-major operands, 16-byte aligned pointers and pitches (D's too); whole tiles (M, N multiples of 128, K of 128 bytes)
// unless kGemmRagged is set in a.flags, in which case K only has to be a multiple of 16 bytes.  The caller checks.
int32_t gemm_mfma_tn_128_dispatch(int32_t in_dt, int32_t out_dt, GemmArgs a, GemmPlan& plan) {
    a.tiles_m = (a.M + 127) / 128;
    a.tiles_n = (a.N + 127) / 128;
    switch (in_dt) {
        case MOYE_F16: return launch128_out<InF16>(out_dt, a, plan);
        case MOYE_BF16: return launch128_out<InBF16>(out_dt, a, plan);
        case MOYE_F8E4M3: return launch128_out<InFP8>(out_dt, a, plan);
        case MOYE_F32: return launch128_out<InF32>(out_dt, a, plan);
        default: return fail(MOYE_ERR_UNSUPPORTED, "gemm!: no MFMA atom for %s inputs", dtype_name(in_dt));
    }
}

}  // namespace moye

// gemm! on the matrix cores, large-tile schedule: one 256 x 256 x (128 bytes of K) CTA tile per
// compute unit; 2 x 4 waves with 128 x 64 wave tiles (the default: 128 accumulator registers per
// lane, two waves per SIMD) or 2 x 2 waves with 128 x 128 wave tiles (256 accumulators).
//
// Why this shape on gfx950: with 64 x 64 wave tiles the fragment reads need about as many LDS
// clocks as the MFMAs need SIMD clocks; larger wave tiles cut the LDS bytes per flop, and the
// 256 x 256 CTA tile halves the L2 bytes per flop of a 128 x 128 one.  4096 / 256 = 16, so a
// 4096^2 problem is exactly 256 workgroups: one per CU, no tail.
//
// The k-loop and the epilogue are gemm_mfma_tn_lds_tile (gemm_mfma_lds_tile.hpp), shared with the 128 x 128 kernel of
// gemm_mfma128.hip; the ring schedule below is a second k-loop for the same tile.  This k-loop is scheduled by the
// compiler under sched_group_barrier hints.  Plain f16 / bf16 calls now run the hand-ordered kernel of
// gemm_mfma256w4.hip instead (same tile, same LDS layout, 4 % faster), and so do calls with fp8 and fp32 operands, with
// operands that are not K-major and with an element-wise operation; this one keeps what that kernel has no instance for:
// a bias, ReLU or scale together with C, an operation on operands that are not K-major, a K tail, and calls that name it
// (stages = 2).
#include "gemm_mfma_lds_tile.hpp"

namespace moye {
// The kernel body lives in gemm_mfma_lds_tile.hpp (kOps, AMAJ / BMAJ, kRagged are described there).
template <typename In, typename Out, int WGM, int WGN, bool kOps = false, int AMAJ = 0, int BMAJ = 0, bool kRagged = false, bool kBias = false>
__global__ __launch_bounds__(64 * WGM * WGN) void gemm_mfma_tn_256(GemmArgs p) {
    gemm_mfma_tn_lds_tile<In, Out, 256, 256, WGM, WGN, kOps, AMAJ, BMAJ, kRagged, kBias>(p);
}

// ------------------------------------------------------------------------------------------------
// Ring schedule: the same 256 x 256 CTA tile, but the K extent per tile is 64 bytes (one k-step)
// and the operand tiles live in a ring of STAGES LDS buffers filled by load-to-LDS instructions
// issued STAGES-1 tiles ahead, so HBM/L2 latency has (STAGES-1) k-steps to hide in.
// Per k-step: issue the loads of tile t+STAGES-1 | first half of the MFMAs of tile t |
// s_waitcnt vmcnt(loads younger than tile t+1) | barrier | ds_read fragments of tile t+1 |
// second half of the MFMAs of tile t.
// ------------------------------------------------------------------------------------------------
template <typename In, typename Out, int WGM, int WGN, int STAGES>
__global__ __launch_bounds__(64 * WGM * WGN) void gemm_mfma_tn_256_ring(GemmArgs p) {
    constexpr int BM = 256, BN = 256, CPR = 4;  // 4 chunks of 16 bytes per tile row
    constexpr int A_CH = BM * CPR, B_CH = BN * CPR, STAGE = A_CH + B_CH;
    constexpr int NWAVES = WGM * WGN;
    constexpr int WROWS = BM / NWAVES;  // operand rows each wave brings in per tile
    constexpr int LD = WROWS / 16;      // load-to-LDS instructions per wave per operand (16 rows each)
    constexpr int WM = BM / WGM, WN = BN / WGN, MI = WM / 16, NI = WN / 16;
    static_assert(LD >= 1 && STAGES >= 3, "ring shape");

    extern __shared__ u32x4 smem[];

    int tm, tn;
    split_of_block(p);
    tile_of_block(p, &tm, &tn);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm0 = (wave / WGN) * WM, wn0 = (wave % WGN) * WN;
    const int r16 = lane & 15, kq = lane >> 4;

    const int64_t pitch_a = (int64_t)p.lda * In::kBytes, pitch_b = (int64_t)p.ldb * In::kBytes;
    // lane l of a load-to-LDS instruction lands in physical chunk l % 4 of row l / 4 of a 16-row block
    const int lrow = wave * WROWS + (lane >> 2), lch = (lane & 3) ^ swz<CPR>(lane >> 2);
    const char* gA = static_cast<const char*>(p.A) + ((int64_t)tm * BM + lrow) * pitch_a + lch * 16;
    const char* gB = static_cast<const char*>(p.B) + ((int64_t)tn * BN + lrow) * pitch_b + lch * 16;
    const int dma_slot = __builtin_amdgcn_readfirstlane(wave * WROWS * CPR);

    const int fa_slot = (wm0 + r16) * CPR + (kq ^ swz<CPR>(r16));
    const int fb_slot = A_CH + (wn0 + r16) * CPR + (kq ^ swz<CPR>(r16));

    f32x4 acc[MI][NI];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int ktiles = (int)(((int64_t)p.K * In::kBytes) / 64);
    u32x4 fa[2][MI], fb[2][NI];

    typedef __attribute__((address_space(1))) const void* gptr_t;
    typedef __attribute__((address_space(3))) void* lptr_t;
#define MOYE_DMA(T)                                                                                    \
    {                                                                                                  \
        u32x4* const base_ = smem + ((T) % STAGES) * STAGE + dma_slot;                                 \
        const int64_t koff_ = (int64_t)(T) * 64;                                                       \
        _Pragma("unroll") for (int i = 0; i < LD; ++i) {                                               \
            __builtin_amdgcn_global_load_lds((gptr_t)(gA + (int64_t)(16 * i) * pitch_a + koff_),       \
                                             (lptr_t)(base_ + 16 * CPR * i), 16, 0, 0);                \
            __builtin_amdgcn_global_load_lds((gptr_t)(gB + (int64_t)(16 * i) * pitch_b + koff_),       \
                                             (lptr_t)(base_ + A_CH + 16 * CPR * i), 16, 0, 0);         \
        }                                                                                              \
    }
#define MOYE_VMCNT(N) __builtin_amdgcn_s_waitcnt(((N) & 0xF) | (((N) >> 4) << 14) | 0x0F70)
    // Wait until at most N of this wave's load-to-LDS instructions are still in flight (the ones for
    // tiles younger than t+1) and its own LDS reads have returned, then meet the other waves.  A
    // plain s_barrier: __syncthreads() would add a release fence, which waits for ALL outstanding
    // loads and so would drain the ring every k-step.
#define MOYE_WAIT_BARRIER(N) \
    { asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(N) : "memory"); }
#define MOYE_FRAGS(T, BUF)                                                                             \
    {                                                                                                  \
        const u32x4* const base_ = smem + ((T) % STAGES) * STAGE;                                      \
        _Pragma("unroll") for (int i = 0; i < MI; ++i) fa[BUF][i] = base_[fa_slot + 16 * CPR * i];     \
        _Pragma("unroll") for (int j = 0; j < NI; ++j) fb[BUF][j] = base_[fb_slot + 16 * CPR * j];     \
    }
#define MOYE_MMA(BUF, I0, I1)                                                                         \
    _Pragma("unroll") for (int i = I0; i < I1; ++i)                                                   \
        _Pragma("unroll") for (int jj = 0; jj < NI; ++jj) {                                           \
            const int j = (i & 1) ? NI - 1 - jj : jj;                                                 \
            In::mma(fb[BUF][j], fa[BUF][i], acc[i][j]);                                               \
        }
    // one k-step; BUF is the fragment buffer that holds tile T
#define MOYE_STEP(T, BUF)                                                                              \
    {                                                                                                  \
        const bool ahead_ = (T) + STAGES - 1 < ktiles;                                                 \
        if (ahead_) MOYE_DMA((T) + STAGES - 1)                                                         \
        MOYE_MMA(BUF, 0, MI / 2)                                                                       \
        __builtin_amdgcn_sched_barrier(0);                                                             \
        if (ahead_) MOYE_WAIT_BARRIER(2 * LD * (STAGES - 2)) else MOYE_WAIT_BARRIER(0)                 \
        __builtin_amdgcn_sched_barrier(0);                                                             \
        if ((T) + 1 < ktiles) MOYE_FRAGS((T) + 1, (BUF) ^ 1)                                           \
        MOYE_MMA(BUF, MI / 2, MI)                                                                      \
    }

    // prologue: fill STAGES-1 buffers, wait for the first
#pragma unroll
    for (int s = 0; s < STAGES - 1; ++s)
        if (s < ktiles) MOYE_DMA(s)
    MOYE_VMCNT(0);
    __syncthreads();
    MOYE_FRAGS(0, 0)

    for (int kt = 0; kt < ktiles; kt += 2) {
        MOYE_STEP(kt, 0)
        if (kt + 1 < ktiles) MOYE_STEP(kt + 1, 1)
    }
#undef MOYE_DMA
#undef MOYE_VMCNT
#undef MOYE_WAIT_BARRIER
#undef MOYE_FRAGS
#undef MOYE_MMA
#undef MOYE_STEP
    __syncthreads();  // every wave is done with the operand ring before it becomes C patches

    // --- epilogue (mfma_epilogue.hpp): alpha*acc + C -> OutT -> this wave's LDS patch -> 128-bit row stores
    static_assert(NWAVES * 32 * WN * 4 <= STAGES * STAGE * 16, "C patches (32 rows per wave and pass) fit in the operand ring");
    store_c_tile<Out, MI, NI>(p, acc, smem, wave, lane, (int64_t)tm * BM + wm0, (int64_t)tn * BN + wn0);
}

template <typename In, typename Out, int STAGES>
static int32_t launch256_ring(const GemmArgs& a, GemmPlan& plan) {
    constexpr int kLds = STAGES * (256 + 256) * 64;
    static LdsCap cap;
    plan.add_kernel(gemm_mfma_tn_256_ring<In, Out, 2, 4, STAGES>, a, (unsigned)(a.tiles_m * a.tiles_n), (unsigned)(a.split > 1 ? a.split : 1), 512, kLds, &cap,
                    256, 256, 64, In::kDt, Out::kDt, "gemm_mfma_tn_256_ring<%s,%s,stages=%d>", In::kName, Out::kName, STAGES);
    return MOYE_OK;
}

template <typename In, typename Out, int WGM, int WGN, bool kOps, int AMAJ, int BMAJ, bool kRagged = false, bool kBias = false>
static int32_t launch256_instance(const GemmArgs& a, GemmPlan& plan) {
    constexpr int kLds = 2 * (256 + 256) * 128;  // two operand stages, 128 KiB
    static LdsCap cap;
    plan.add_kernel(gemm_mfma_tn_256<In, Out, WGM, WGN, kOps, AMAJ, BMAJ, kRagged, kBias>, a, (unsigned)(a.tiles_m * a.tiles_n),
                    (unsigned)(a.split > 1 ? a.split : 1), 64 * WGM * WGN, kLds, &cap, 256, 256, 128, In::kDt, Out::kDt,
                    "gemm_mfma_tn_256<%s,%s,waves=%d,ops=%d,amaj=%d,bmaj=%d,ragged=%d,bias=%d>", In::kName, Out::kName, WGM * WGN, (int)kOps, AMAJ, BMAJ,
                    (int)kRagged, (int)kBias);
    return MOYE_OK;
}

template <typename In, typename Out, int WGM, int WGN>
static int32_t launch256(const GemmArgs& a, GemmPlan& plan) {
    const bool am = a.flags & kGemmAMajorM, bm = a.flags & kGemmBMajorN;
    if (a.flags & kGemmRagged) {
        if constexpr (WGM * WGN == 8 && !std::is_same<In, InFP8>::value) {
            if (am || bm) return fail(MOYE_ERR_UNSUPPORTED, "gemm!: ragged 256 x 256 tiles take K-major operands");
            return a.ep_op != MOYE_MAP_IDENTITY ? launch256_instance<In, Out, WGM, WGN, true, 0, 0, true>(a, plan)
                                                : launch256_instance<In, Out, WGM, WGN, false, 0, 0, true>(a, plan);
        } else {
            return fail(MOYE_ERR_UNSUPPORTED, "gemm!: ragged 256 x 256 tiles run on eight waves with f16, bf16 or f32 operands");
        }
    }
    if (am || bm) {
        // operands that are not K-major: eight waves, 16-bit types (the host checked)
        if constexpr (WGM * WGN == 8 && In::kBytes == 2) {
            const bool ops = a.ep_op != MOYE_MAP_IDENTITY;
            if (am && bm) return ops ? launch256_instance<In, Out, WGM, WGN, true, 1, 1>(a, plan) : launch256_instance<In, Out, WGM, WGN, false, 1, 1>(a, plan);
            if (am) return ops ? launch256_instance<In, Out, WGM, WGN, true, 1, 0>(a, plan) : launch256_instance<In, Out, WGM, WGN, false, 1, 0>(a, plan);
            return ops ? launch256_instance<In, Out, WGM, WGN, true, 0, 1>(a, plan) : launch256_instance<In, Out, WGM, WGN, false, 0, 1>(a, plan);
        } else {
            return fail(MOYE_ERR_UNSUPPORTED, "gemm!: operands that are not K-major run natively with 16-bit types on eight waves only");
        }
    }
    if constexpr (WGM * WGN == 8) {
        if (a.flags & kGemmEpiLaneOp) return launch256_instance<In, Out, WGM, WGN, false, 0, 0, false, true>(a, plan);  // a bias, a ReLU, a scale: in the lanes
        if (a.ep_op != MOYE_MAP_IDENTITY) return launch256_instance<In, Out, WGM, WGN, true, 0, 0>(a, plan);
    }
    return launch256_instance<In, Out, WGM, WGN, false, 0, 0>(a, plan);
}

template <typename In>
static int32_t launch256_out(int32_t out_dt, const GemmArgs& a, int waves, int stages, GemmPlan& plan) {
    if (stages >= 3 && a.ep_op != MOYE_MAP_IDENTITY)
        return fail(MOYE_ERR_UNSUPPORTED, "gemm!: the ring schedules (stages >= 3) take no element-wise epilogue operation; leave stages at 0");
    if (stages >= 3) {
        const bool five = stages >= 5;
        switch (out_dt) {
            case MOYE_F32: return five ? launch256_ring<In, OutF32, 5>(a, plan) : launch256_ring<In, OutF32, 4>(a, plan);
            case MOYE_F16: return five ? launch256_ring<In, OutF16, 5>(a, plan) : launch256_ring<In, OutF16, 4>(a, plan);
            case MOYE_BF16: return five ? launch256_ring<In, OutBF16, 5>(a, plan) : launch256_ring<In, OutBF16, 4>(a, plan);
            default: break;
        }
    }
    if (waves == 4 && a.ep_op == MOYE_MAP_IDENTITY) {  // (with an element-wise operation the eight-wave form runs: 256 accumulators leave it no registers)
        switch (out_dt) {
            case MOYE_F32: return launch256<In, OutF32, 2, 2>(a, plan);
            case MOYE_F16: return launch256<In, OutF16, 2, 2>(a, plan);
            case MOYE_BF16: return launch256<In, OutBF16, 2, 2>(a, plan);
            default: break;
        }
    }
    switch (out_dt) {
        case MOYE_F32: return launch256<In, OutF32, 2, 4>(a, plan);
        case MOYE_F16: return launch256<In, OutF16, 2, 4>(a, plan);
        case MOYE_BF16: return launch256<In, OutBF16, 2, 4>(a, plan);
        default: return fail(MOYE_ERR_UNSUPPORTED, "gemm!: MFMA kernels write f32, f16 or bf16, not %s", dtype_name(out_dt));
    }
}

// 256 x 256 x (128 bytes of K) tile; the caller has checked divisibility and alignment.
int32_t gemm_mfma_tn_256_dispatch(int32_t in_dt, int32_t out_dt, GemmArgs a, int waves, int stages, GemmPlan& plan) {
    a.tiles_m = (a.M + 255) / 256;  // (whole tiles unless kGemmRagged)
    a.tiles_n = (a.N + 255) / 256;
    switch (in_dt) {
        case MOYE_F16: return launch256_out<InF16>(out_dt, a, waves, stages, plan);
        case MOYE_BF16: return launch256_out<InBF16>(out_dt, a, waves, stages, plan);
        case MOYE_F8E4M3: return launch256_out<InFP8>(out_dt, a, waves, stages, plan);
        case MOYE_F32: return launch256_out<InF32>(out_dt, a, waves, stages, plan);
        default: return fail(MOYE_ERR_UNSUPPORTED, "gemm!: no MFMA atom for %s inputs", dtype_name(in_dt));
    }
}

}  // namespace moye

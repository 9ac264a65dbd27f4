// gemm! on the matrix cores, ping-pong schedule: one 256 x 256 CTA tile per compute unit, eight
// waves as 2 x 4 (wave tile 128 x 64), two waves on every SIMD, k-tiles of 64 bytes (one MFMA
// k-step) in a ring of five 32 KiB LDS stages (all 160 KiB).
//
// The two waves of a SIMD (w and w+4) never do the same thing at the same time.  Time is cut into
// slots by workgroup barriers; in every slot one wave of each SIMD issues the 32 MFMAs of a k-tile
// back to back while its partner does its memory work (12 ds_read_b128 for the fragments of its
// next k-tile, four load-to-LDS instructions); in the next slot they swap.
//
//   slot        0        1        2        3        4
//   waves 0-3   MEM(0)   MMA(0)   MEM(1)   MMA(1)   MEM(2) ...
//   waves 4-7   -        MEM(0)   MMA(0)   MEM(1)   MMA(1) ...
// Both groups run the same code; the second enters one barrier late, the first leaves one late.
// Letting the two waves merely drift half a k-tile apart (one barrier per k-tile, the matrix pipe
// arbitrating) measured 10 % slower: the older wave wins the pipe and the younger one's fragment
// reads end up exposed.
//
// Operand traffic: a compute unit's texture-address path moves 64 bytes per clock, so the 32 KiB
// of a k-tile keep it busy for half of the 1024 clocks the MFMAs of that k-tile take.  The
// load-to-LDS instructions are issued at a constant rate, four per wave per k-tile in the MEM slot
// (never in the MMA slot, where a full queue would hold up the MFMAs behind them): tile j+4 is
// requested in MEM(j) and awaited with s_waitcnt vmcnt(12) in MEM(j+3), which leaves the twelve
// younger loads of three k-tiles in flight: about 3000 clocks of latency cover.
//
// Operand conventions as in gemm_mfma256.hip: K-major A and B, N-contiguous D, MFMA issued with B
// rows as its first operand so a lane holds four consecutive n of one m; LDS rows of 64 bytes with
// the 16-byte chunk index XORed with (row / 2) % 4, applied on the global side of the load-to-LDS.
#include "mfma_epilogue.hpp"

namespace moye {

template <typename In, typename Out>
__global__ __launch_bounds__(512) void gemm_mfma_tn_256_pp(GemmArgs p) {
    constexpr int BM = 256, BN = 256, CPR = 4, STAGES = 5;
    constexpr int A_CH = BM * CPR, B_CH = BN * CPR, STAGE = A_CH + B_CH;  // in 16-byte chunks
    constexpr int WGM = 2, WGN = 4, NWAVES = 8;
    constexpr int WROWS = BM / NWAVES, LD = WROWS / 16;  // load-to-LDS instructions per wave per operand
    constexpr int WM = BM / WGM, WN = BN / WGN, MI = WM / 16, NI = WN / 16;
    static_assert(LD == 2, "two loads per operand per wave per k-tile");

    extern __shared__ u32x4 smem[];

    int tm, tn;
    split_of_block(p);
    tile_of_block(p, &tm, &tn);
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int group = wave >> 2;  // wave-uniform: the waits below are scalar instructions
    const int wm0 = (wave / WGN) * WM, wn0 = (wave % WGN) * WN;
    const int r16 = lane & 15, kq = lane >> 4;

    const int64_t pitch_a = (int64_t)p.lda * In::kBytes, pitch_b = (int64_t)p.ldb * In::kBytes;
    // lane l of a load-to-LDS instruction lands in physical chunk l % 4 of row l / 4 of a 16-row block
    const int lrow = wave * WROWS + (lane >> 2), lch = (lane & 3) ^ swz<CPR>(lane >> 2);
    const char* gA = static_cast<const char*>(p.A) + ((int64_t)tm * BM + lrow) * pitch_a + lch * 16;
    const char* gB = static_cast<const char*>(p.B) + ((int64_t)tn * BN + lrow) * pitch_b + lch * 16;
    const int dma_slot = wave * WROWS * CPR;

    const int fa_slot = (wm0 + r16) * CPR + (kq ^ swz<CPR>(r16));
    const int fb_slot = A_CH + (wn0 + r16) * CPR + (kq ^ swz<CPR>(r16));

    f32x4 acc[MI][NI];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int ktiles = (int)(((int64_t)p.K * In::kBytes) / 64);
    u32x4 fa[MI], fb[NI];

    typedef __attribute__((address_space(1))) const void* gptr_t;
    typedef __attribute__((address_space(3))) void* lptr_t;
    // the A half / the B half of this wave's share of tile T (two instructions each)
#define MOYE_DMA_A(T, STG)                                                                             \
    _Pragma("unroll") for (int i = 0; i < LD; ++i)                                                     \
        __builtin_amdgcn_global_load_lds((gptr_t)(gA + (int64_t)(16 * i) * pitch_a + (int64_t)(T) * 64), \
                                         (lptr_t)(smem + (STG) * STAGE + dma_slot + 16 * CPR * i), 16, 0, 0);
#define MOYE_DMA_B(T, STG)                                                                             \
    _Pragma("unroll") for (int i = 0; i < LD; ++i)                                                     \
        __builtin_amdgcn_global_load_lds((gptr_t)(gB + (int64_t)(16 * i) * pitch_b + (int64_t)(T) * 64), \
                                         (lptr_t)(smem + (STG) * STAGE + A_CH + dma_slot + 16 * CPR * i), 16, 0, 0);
    // bare s_barrier: __syncthreads() would add a fence that drains the prefetch
#define MOYE_BARRIER()                        \
    {                                         \
        __builtin_amdgcn_sched_barrier(0);    \
        asm volatile("" ::: "memory");        \
        __builtin_amdgcn_s_barrier();         \
        asm volatile("" ::: "memory");        \
        __builtin_amdgcn_sched_barrier(0);    \
    }
#define MOYE_VMCNT(N) (((N) & 0xF) | (((N) >> 4) << 14))
#define MOYE_FRAGS(STG)                                                                              \
    {                                                                                                \
        const u32x4* const base_ = smem + (STG) * STAGE;                                             \
        _Pragma("unroll") for (int i = 0; i < MI; ++i) fa[i] = base_[fa_slot + 16 * CPR * i];        \
        _Pragma("unroll") for (int j = 0; j < NI; ++j) fb[j] = base_[fb_slot + 16 * CPR * j];        \
    }
#define MOYE_MMA()                                   \
    _Pragma("unroll") for (int i = 0; i < MI; ++i)   \
        _Pragma("unroll") for (int j = 0; j < NI; ++j) In::mma(fb[j], fa[i], acc[i][j]);

    // prologue: tiles 0..3 requested by everybody (16 loads per wave); wait for tile 0
#pragma unroll
    for (int t = 0; t < STAGES - 1; ++t)
        if (t < ktiles) {
            MOYE_DMA_A(t, t)
            MOYE_DMA_B(t, t)
        }
    // fewer than four tiles: simply wait for all of them
    if (ktiles >= STAGES - 1) __builtin_amdgcn_s_waitcnt(MOYE_VMCNT(12) | 0x0F70);
    else __builtin_amdgcn_s_waitcnt(0x0F70);
    MOYE_BARRIER()
    if (group == 1) MOYE_BARRIER()  // the late group starts one slot later

    // Both groups run the same loop; "slot" boundaries are the barriers.
    //   MEM(j): read the fragments of tile j, request tile j+4 into the stage tile j-1 lived in (every
    //           wave finished reading it before the previous barrier), wait for the fragments and for
    //           this wave's share of tile j+1 (vmcnt(12) leaves tiles j+2..j+4 in flight)
    //   MMA(j): 32 MFMAs.  The barrier that ends the slot is issued TAIL MFMAs early, so that its
    //           latency and the partner's start-up are hidden behind this wave's last MFMAs.
    // Every barrier is preceded, on the MEM side, by the waits that make LDS reuse safe, so the
    // partner may overwrite tile j-1's stage and read tile j+1 right after it.
    constexpr int TAIL = 0;
    int s_cur = 0, s_p4 = STAGES - 1;  // stage of tile j and of tile j+4 (= tile j-1's)
    for (int j = 0; j < ktiles; ++j) {
        MOYE_FRAGS(s_cur)
        if (j + 4 < ktiles) {
            MOYE_DMA_A(j + 4, s_p4)
            MOYE_DMA_B(j + 4, s_p4)
            __builtin_amdgcn_s_waitcnt(MOYE_VMCNT(12) | 0x0070);  // and lgkmcnt(0)
        } else {
            __builtin_amdgcn_s_waitcnt(0x0070);  // tail: no younger loads to leave in flight
        }
        MOYE_BARRIER()
#pragma unroll
        for (int q = 0; q < MI * NI - TAIL; ++q) In::mma(fb[q % NI], fa[q / NI], acc[q / NI][q % NI]);
        MOYE_BARRIER()
#pragma unroll
        for (int q = MI * NI - TAIL; q < MI * NI; ++q) In::mma(fb[q % NI], fa[q / NI], acc[q / NI][q % NI]);
        __builtin_amdgcn_sched_barrier(0);
        s_p4 = s_cur;
        s_cur = s_cur + 1 == STAGES ? 0 : s_cur + 1;
    }
    if (group == 0) MOYE_BARRIER()
#undef MOYE_DMA_A
#undef MOYE_DMA_B
#undef MOYE_BARRIER
#undef MOYE_VMCNT
#undef MOYE_FRAGS
#undef MOYE_MMA
    __syncthreads();  // every wave is done with the operand stages before they become C patches

    store_c_tile<Out, MI, NI>(p, acc, smem, wave, lane, (int64_t)tm * BM + wm0, (int64_t)tn * BN + wn0);
}

template <typename In, typename Out>
static int32_t launch256_pp(const GemmArgs& a, GemmPlan& plan) {
    constexpr int kLds = 5 * (256 + 256) * 64;  // all 160 KiB
    static LdsCap cap;
    plan.add_kernel(gemm_mfma_tn_256_pp<In, Out>, a, (unsigned)(a.tiles_m * a.tiles_n), (unsigned)(a.split > 1 ? a.split : 1), 512, kLds, &cap, 256, 256, 64,
                    In::kDt, Out::kDt, "gemm_mfma_tn_256_pp<%s,%s>", In::kName, Out::kName);
    return MOYE_OK;
}

template <typename In>
static int32_t launch256_pp_out(int32_t out_dt, const GemmArgs& a, GemmPlan& plan) {
    switch (out_dt) {
        case MOYE_F32: return launch256_pp<In, OutF32>(a, plan);
        case MOYE_F16: return launch256_pp<In, OutF16>(a, plan);
        case MOYE_BF16: return launch256_pp<In, OutBF16>(a, plan);
        default: return fail(MOYE_ERR_UNSUPPORTED, "gemm!: MFMA kernels write f32, f16 or bf16, not %s", dtype_name(out_dt));
    }
}

// 256 x 256 x (64 bytes of K) tile, ping-pong schedule; the caller has checked divisibility and alignment.
int32_t gemm_mfma_tn_256_pp_dispatch(int32_t in_dt, int32_t out_dt, GemmArgs a, GemmPlan& plan) {
    a.tiles_m = a.M / 256;
    a.tiles_n = a.N / 256;
    switch (in_dt) {
        case MOYE_F16: return launch256_pp_out<InF16>(out_dt, a, plan);
        case MOYE_BF16: return launch256_pp_out<InBF16>(out_dt, a, plan);
        case MOYE_F8E4M3: return launch256_pp_out<InFP8>(out_dt, a, plan);
        case MOYE_F32: return launch256_pp_out<InF32>(out_dt, a, plan);
        default: return fail(MOYE_ERR_UNSUPPORTED, "gemm!: no MFMA atom for %s inputs", dtype_name(in_dt));
    }
}

}  // namespace moye

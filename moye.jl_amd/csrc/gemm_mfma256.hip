// gemm! on the matrix cores, large-tile schedule: one 256 x 256 x (128 bytes of K) CTA tile per
// compute unit, 2 x 2 waves, each wave a 128 x 128 block of C held in 256 accumulator registers.
//
// Why this shape on gfx950: the LDS delivers 128 bytes per clock per CU while the four SIMDs
// retire one 16x16x32 MFMA each every 16 clocks.  With 64 x 64 wave tiles the fragment reads
// alone need as many LDS clocks as the MFMAs need SIMD clocks; 128 x 128 wave tiles halve the
// LDS bytes per flop (and the L2 bytes per flop of the workgroup).  4096 / 256 = 16, so a 4096^2
// problem is exactly 256 workgroups: one per CU, no tail.
//
// Schedule per k-tile (two k-steps of 32 halves / 64 fp8), operand tiles double-buffered in LDS:
//   ds_read fragments of step 1                      (fragments are double-buffered in registers)
//   global_load_lds_dwordx4 of tile t+1 -> the other LDS stage (no registers, no ds_write)
//   MFMAs of step 0, first half of the MFMAs of step 1
//   s_waitcnt vmcnt(0), barrier, ds_read fragments of step 0 of tile t+1
//   second half of the MFMAs of step 1               (covers the LDS latency after the barrier)
// A load-to-LDS instruction writes lane l's 16 bytes at base + 16 l, so the XOR swizzle is
// applied on the global side: lane l of a 64-chunk block fetches chunk (l%8)^(l/8) of row l/8.
//
// Same operand conventions as gemm_mfma.hip: K-major A and B, N-contiguous D, the MFMA issued
// with B rows as its first operand so a lane holds four consecutive n of one m.
#include "mfma_common.hpp"

namespace moye {

template <typename In, typename Out, int WGM, int WGN>
__global__ __launch_bounds__(64 * WGM * WGN) void gemm_mfma_tn_256(GemmArgs p) {
    constexpr int BM = 256, BN = 256, CPR = 8;  // 8 chunks of 16 bytes per tile row
    constexpr int A_CH = BM * CPR, B_CH = BN * CPR, STAGE = A_CH + B_CH;
    constexpr int NWAVES = WGM * WGN;
    constexpr int WROWS = BM / NWAVES;  // operand rows each wave brings in per tile
    constexpr int LD = WROWS / 8;       // load-to-LDS instructions per wave per operand (8 rows each)
    constexpr int WM = BM / WGM, WN = BN / WGN, MI = WM / 16, NI = WN / 16;
    typedef typename Out::type OutT;

    extern __shared__ u32x4 smem[];

    int tm, tn;
    tile_of_block(p, &tm, &tn);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm0 = (wave / WGN) * WM, wn0 = (wave % WGN) * WN;
    const int r16 = lane & 15, kq = lane >> 4;

    const int64_t pitch_a = (int64_t)p.lda * In::kBytes, pitch_b = (int64_t)p.ldb * In::kBytes;
    // load-to-LDS: wave w fills rows WROWS w + 8 i + l/8 (i < LD) of each operand tile; lane l brings
    // the chunk that belongs in physical slot l % 8 of its row
    const int lrow = wave * WROWS + (lane >> 3), lch = (lane & 7) ^ (lane >> 3);
    const char* gA = static_cast<const char*>(p.A) + ((int64_t)tm * BM + lrow) * pitch_a + lch * 16;
    const char* gB = static_cast<const char*>(p.B) + ((int64_t)tn * BN + lrow) * pitch_b + lch * 16;
    const int dma_slot = __builtin_amdgcn_readfirstlane(wave * WROWS * CPR);  // + 8 rows * CPR per i

    // fragment slots: row = w?0 + 16 i + r16, chunk = 4 ks + kq
    int fa_slot[2], fb_slot[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
        const int ch = 4 * ks + kq;
        fa_slot[ks] = (wm0 + r16) * CPR + (ch ^ swz<CPR>(r16));
        fb_slot[ks] = A_CH + (wn0 + r16) * CPR + (ch ^ swz<CPR>(r16));
    }

    f32x4 acc[MI][NI];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int ktiles = (int)(((int64_t)p.K * In::kBytes) / 128);
    u32x4 fa[2][MI], fb[2][NI];

    typedef __attribute__((address_space(1))) const void* gptr_t;
    typedef __attribute__((address_space(3))) void* lptr_t;
#define MOYE_DMA(BASE, KOFF)                                                                          \
    _Pragma("unroll") for (int i = 0; i < LD; ++i) {                                                  \
        __builtin_amdgcn_global_load_lds((gptr_t)(gA + (int64_t)(8 * i) * pitch_a + (KOFF)),          \
                                         (lptr_t)((BASE) + dma_slot + 8 * CPR * i), 16, 0, 0);        \
        __builtin_amdgcn_global_load_lds((gptr_t)(gB + (int64_t)(8 * i) * pitch_b + (KOFF)),          \
                                         (lptr_t)((BASE) + A_CH + dma_slot + 8 * CPR * i), 16, 0, 0); \
    }
#define MOYE_WAIT_DMA() __builtin_amdgcn_s_waitcnt(0x0F70) /* vmcnt(0), leave expcnt and lgkmcnt alone */
#define MOYE_FRAGS(BASE, KS, BUF)                                                                     \
    _Pragma("unroll") for (int i = 0; i < MI; ++i) fa[BUF][i] = (BASE)[fa_slot[KS] + 16 * CPR * i];   \
    _Pragma("unroll") for (int j = 0; j < NI; ++j) fb[BUF][j] = (BASE)[fb_slot[KS] + 16 * CPR * j];
#define MOYE_MMA(BUF, I0, I1)                                                                         \
    _Pragma("unroll") for (int i = I0; i < I1; ++i)                                                   \
        _Pragma("unroll") for (int j = 0; j < NI; ++j) In::mma(fb[BUF][j], fa[BUF][i], acc[i][j]);

    // prologue
    MOYE_DMA(smem, 0)
    MOYE_WAIT_DMA();
    __syncthreads();
    MOYE_FRAGS(smem, 0, 0)

    for (int kt = 0; kt < ktiles; ++kt) {
        u32x4* const cur = smem + (kt & 1) * STAGE;
        u32x4* const nxt = smem + ((kt + 1) & 1) * STAGE;
        const bool more = kt + 1 < ktiles;
        MOYE_FRAGS(cur, 1, 1)
        if (more) {
            const int64_t koff = (int64_t)(kt + 1) * 128;
            MOYE_DMA(nxt, koff)
        }
        MOYE_MMA(0, 0, MI)
        MOYE_MMA(1, 0, MI / 2)
        __builtin_amdgcn_sched_barrier(0);  // keep the MFMAs above on this side of the wait
        MOYE_WAIT_DMA();
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
        if (more) {
            MOYE_FRAGS(nxt, 0, 0)
        }
        MOYE_MMA(1, MI / 2, MI)
    }
#undef MOYE_DMA
#undef MOYE_WAIT_DMA
#undef MOYE_FRAGS
#undef MOYE_MMA
    __syncthreads();  // every wave is done with the operand stages before they become C patches

    // ---- epilogue: alpha*acc + C -> OutT -> this wave's LDS patch -> 128-bit row stores ----
    // lane holds C[m = 16 i + r16][n = 16 j + 4 kq + e], e = 0..3
    const int64_t m_base = (int64_t)tm * BM + wm0, n_base = (int64_t)tn * BN + wn0;
    constexpr int EPC = 16 / (int)sizeof(OutT);  // elements per 16-byte chunk
    constexpr int CR = WN / EPC;                 // chunks per patch row
    constexpr int PASS_MI = 2, PASS_ROWS = PASS_MI * 16;
    static_assert(NWAVES * PASS_ROWS * WN * 4 <= 2 * STAGE * 16, "C patches fit in the operand stages");
    OutT* patch = reinterpret_cast<OutT*>(smem) + wave * (PASS_ROWS * WN);
    u32x4* patch16 = reinterpret_cast<u32x4*>(patch);

#pragma unroll
    for (int i0 = 0; i0 < MI; i0 += PASS_MI) {
#pragma unroll
        for (int ii = 0; ii < PASS_MI; ++ii) {
            const int i = i0 + ii;
#pragma unroll
            for (int j = 0; j < NI; ++j) {
                float v[4] = {acc[i][j].x * p.alpha, acc[i][j].y * p.alpha, acc[i][j].z * p.alpha,
                              acc[i][j].w * p.alpha};
                if (p.C) {
                    const int64_t m = m_base + 16 * i + r16, n = n_base + 16 * j + 4 * kq;
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] += Out::load(p.C, m * p.ldc_m + (n + e) * p.ldc_n);
                }
                const int row = 16 * ii + r16, col = 16 * j + 4 * kq;
                const int chunk = col / EPC, within = col % EPC;
                OutT* dst = patch + (row * CR + (chunk ^ (row & 7))) * EPC + within;
#pragma unroll
                for (int e = 0; e < 4; ++e) dst[e] = Out::cvt(v[e]);
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int t = 0; t < PASS_ROWS * CR / 64; ++t) {
            const int c = lane + 64 * t, row = c / CR, ch = c % CR;
            const u32x4 w = patch16[row * CR + (ch ^ (row & 7))];
            char* d = static_cast<char*>(p.D) +
                      ((m_base + 16 * i0 + row) * p.ldd + n_base) * (int64_t)sizeof(OutT) + ch * 16;
            *reinterpret_cast<u32x4*>(d) = w;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
}

template <typename In, typename Out, int WGM, int WGN>
static int32_t launch256(const GemmArgs& a, hipStream_t st) {
    constexpr int kLds = 2 * (256 + 256) * 128;  // two operand stages, 128 KiB
    auto kern = gemm_mfma_tn_256<In, Out, WGM, WGN>;
    static bool once = false;
    if (!once) {
        MOYE_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, kLds));
        once = true;
    }
    kern<<<dim3((unsigned)(a.tiles_m * a.tiles_n)), dim3(64 * WGM * WGN), kLds, st>>>(a);
    MOYE_HIP_CHECK(hipGetLastError());
    return MOYE_OK;
}

template <typename In>
static int32_t launch256_out(int32_t out_dt, const GemmArgs& a, int waves, hipStream_t st) {
    if (waves == 4) {
        switch (out_dt) {
            case MOYE_F32: return launch256<In, OutF32, 2, 2>(a, st);
            case MOYE_F16: return launch256<In, OutF16, 2, 2>(a, st);
            case MOYE_BF16: return launch256<In, OutBF16, 2, 2>(a, st);
            default: break;
        }
    }
    switch (out_dt) {
        case MOYE_F32: return launch256<In, OutF32, 2, 4>(a, st);
        case MOYE_F16: return launch256<In, OutF16, 2, 4>(a, st);
        case MOYE_BF16: return launch256<In, OutBF16, 2, 4>(a, st);
        default: return fail(MOYE_ERR_UNSUPPORTED, "gemm!: MFMA kernels write f32, f16 or bf16, not %s", dtype_name(out_dt));
    }
}

// 256 x 256 x (128 bytes of K) tile; the caller has checked divisibility and alignment.
int32_t gemm_mfma_tn_256_dispatch(int32_t in_dt, int32_t out_dt, GemmArgs a, int waves, hipStream_t st) {
    a.tiles_m = a.M / 256;
    a.tiles_n = a.N / 256;
    switch (in_dt) {
        case MOYE_F16: return launch256_out<InF16>(out_dt, a, waves, st);
        case MOYE_BF16: return launch256_out<InBF16>(out_dt, a, waves, st);
        case MOYE_F8E4M3: return launch256_out<InFP8>(out_dt, a, waves, st);
        default: return fail(MOYE_ERR_UNSUPPORTED, "gemm!: no MFMA atom for %s inputs", dtype_name(in_dt));
    }
}

}  // namespace moye

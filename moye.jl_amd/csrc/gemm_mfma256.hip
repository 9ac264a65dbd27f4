// gemm! on the matrix cores, large-tile schedule: one 256 x 256 x (128 bytes of K) CTA tile per
// compute unit; 2 x 4 waves with 128 x 64 wave tiles (the default: 128 accumulator registers per
// lane, two waves per SIMD) or 2 x 2 waves with 128 x 128 wave tiles (256 accumulators).
//
// Why this shape on gfx950: with 64 x 64 wave tiles the fragment reads need about as many LDS
// clocks as the MFMAs need SIMD clocks; larger wave tiles cut the LDS bytes per flop, and the
// 256 x 256 CTA tile halves the L2 bytes per flop of a 128 x 128 one.  4096 / 256 = 16, so a
// 4096^2 problem is exactly 256 workgroups: one per CU, no tail.
//
// Schedule per k-tile (two k-steps of 32 halves / 64 fp8), operand tiles double-buffered in LDS,
// fragments double-buffered in registers:
//   step 0: ds_read the fragments of step 1 (buffer 1) | MFMAs of step 0 (buffer 0)
//   s_waitcnt vmcnt(0) lgkmcnt(0), s_barrier: tile t+1 has landed, nobody reads tile t any more
//   global_load_lds_dwordx4 of tile t+2 -> the stage tile t just vacated: the loads have a whole
//     iteration to complete and go straight to LDS (no registers, no ds_write)
//   step 1: ds_read the fragments of step 0 of tile t+1 (buffer 0) | MFMAs of step 1 (buffer 1)
// so the MFMAs that follow a barrier always find their operands already in registers.
// A load-to-LDS instruction writes lane l's 16 bytes at base + 16 l, so the XOR swizzle is
// applied on the global side: lane l of a 64-chunk block fetches chunk (l%8)^(l/8) of row l/8.
//
// Same operand conventions as gemm_mfma.hip: K-major A and B, N-contiguous D, the MFMA issued
// with B rows as its first operand so a lane holds four consecutive n of one m.
#include <type_traits>

#include "mfma_epilogue.hpp"

namespace moye {

// kOps: the epilogue may apply an element-wise operation (GemmArgs::ep_op).  A separate instance, so that the code and
// the registers of that path never touch the kernel the plain gemm! runs.
//
// AMAJ / BMAJ = 1: that operand is stored with its unit stride along M (N) instead of K, the 'N' forms of
// src/arch/mma/make_mma_ops.jl:253-265 (GemmArgs::lda / ldb is then the pitch between consecutive k).  Its LDS tile is
// 64 k-rows of 256 operand rows (512 bytes), brought in by the same load-to-LDS instructions, and the fragments come
// out of it with ds_read_b64_tr_b16, the transposing LDS read of gfx950, where the reference has ldmatrix.trans
// (src/arch/copy/ldmatrix.jl:18-48): sixteen lanes that each point at four consecutive 16-bit values of a row get back
// the four values lane j's position holds in rows 0..3 of their group (measured on the hardware: result e of lane j of a
// group is value j % 4 of the lane 4 e + j / 4).  With lane l = 16 g + s pointing at k-row 8 g + s / 4 (+ 4 for the second
// read), m = m0 + 4 (s % 4), two reads give lane l the eight k of row m0 + l % 16 that the K-major ds_read_b128 would.
// The 32-byte piece index of a k-row is XORed with (row % 4) | 4 ((row / 8) % 2): the eight row pieces the 32 lanes of
// one pass read then lie in eight different bank groups.
//
// kRagged: M and N need not be multiples of 256 and K not of the k-tile (the intent of copyto_if!,
// src/algorithm/copy.jl:4-16, for whole tiles).  A row beyond the operand is read from the operand's last row instead and
// what is computed from it is never stored; in the last k-tile a lane whose 16-byte piece lies beyond K reads the
// row's first piece instead and every fragment piece beyond K is zeroed in registers before it reaches an MFMA; the
// epilogue is the general one with its row and column guards.
template <typename In, typename Out, int WGM, int WGN, bool kOps = false, int AMAJ = 0, int BMAJ = 0, bool kRagged = false>
__global__ __launch_bounds__(64 * WGM * WGN) void gemm_mfma_tn_256(GemmArgs p) {
    static_assert(!kRagged || (kOps && !AMAJ && !BMAJ), "ragged tiles: K-major operands, the general epilogue");
    constexpr int BM = 256, BN = 256, CPR = 8;  // 8 chunks of 16 bytes per tile row
    constexpr int A_CH = BM * CPR, B_CH = BN * CPR, STAGE = A_CH + B_CH;
    constexpr int NWAVES = WGM * WGN;
    constexpr int WROWS = BM / NWAVES;  // operand rows each wave brings in per tile
    constexpr int LD = WROWS / 8;       // load-to-LDS instructions per wave per operand (8 rows each)
    constexpr int WM = BM / WGM, WN = BN / WGN, MI = WM / 16, NI = WN / 16;

    extern __shared__ u32x4 smem[];

    int tm, tn;
    split_of_block(p);
    tile_of_block(p, &tm, &tn);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm0 = (wave / WGN) * WM, wn0 = (wave % WGN) * WN;
    const int r16 = lane & 15, kq = lane >> 4;

    const int64_t pitch_a = (int64_t)p.lda * In::kBytes, pitch_b = (int64_t)p.ldb * In::kBytes;
    // load-to-LDS: wave w fills rows WROWS w + 8 i + l/8 (i < LD) of each operand tile; lane l brings
    // the chunk that belongs in physical slot l % 8 of its row
    const int lrow = wave * WROWS + (lane >> 3), lch = (lane & 7) ^ (lane >> 3);
    const int row_a0 = tm * BM + lrow, row_b0 = tn * BN + lrow;
    const char* gA = static_cast<const char*>(p.A) + (int64_t)(kRagged ? min(row_a0, p.M - 1) : row_a0) * pitch_a + lch * 16;
    const char* gB = static_cast<const char*>(p.B) + (int64_t)(kRagged ? min(row_b0, p.N - 1) : row_b0) * pitch_b + lch * 16;
    // ragged tiles: how many rows below its first one this lane may go, and what to add to its address in the last k-tile
    [[maybe_unused]] const int more_a = max(p.M - 1 - row_a0, 0), more_b = max(p.N - 1 - row_b0, 0);
    [[maybe_unused]] const int k_rem = (int)((((int64_t)p.K * In::kBytes) % 128) / 16), k_valid = k_rem ? k_rem : 8;
    [[maybe_unused]] const int tail_delta = lch < k_valid ? 0 : -lch * 16;
    const int dma_slot = __builtin_amdgcn_readfirstlane(wave * WROWS * CPR);  // + 8 rows * CPR per i
    // An M-major (N-major) operand: wave w fills k-rows KROWS w + 2 i + l / 32 of the tile, two rows (1 KiB) per
    // instruction; lane l brings the 16-byte chunk that belongs in physical slot l % 32 of its row.
    constexpr int KROWS = 64 / NWAVES;
    static_assert(!(AMAJ || BMAJ) || (In::kBytes == 2 && KROWS == 2 * LD), "transposing fragment reads: 16-bit operands");
    auto tr_swz = [](int krow) { return (krow & 3) | (((krow >> 3) & 1) << 2); };
    [[maybe_unused]] int64_t tA[AMAJ ? LD : 1], tB[BMAJ ? LD : 1];  // byte offsets of this lane's chunk, per instruction, from the k-tile's first row
    if constexpr (AMAJ) {
#pragma unroll
        for (int i = 0; i < LD; ++i) {
            const int krow = wave * KROWS + 2 * i + (lane >> 5), p16 = lane & 31, l32 = (p16 >> 1) ^ tr_swz(krow);
            tA[i] = krow * pitch_a + ((int64_t)tm * BM) * In::kBytes + (l32 * 2 + (p16 & 1)) * 16;
        }
    }
    if constexpr (BMAJ) {
#pragma unroll
        for (int i = 0; i < LD; ++i) {
            const int krow = wave * KROWS + 2 * i + (lane >> 5), p16 = lane & 31, l32 = (p16 >> 1) ^ tr_swz(krow);
            tB[i] = krow * pitch_b + ((int64_t)tn * BN) * In::kBytes + (l32 * 2 + (p16 & 1)) * 16;
        }
    }
    const int dma_slot_t = __builtin_amdgcn_readfirstlane(wave * KROWS * 32);  // + 2 rows * 32 chunks per i

    // fragment slots: row = w?0 + 16 i + r16, chunk = 4 ks + kq
    int fa_slot[2], fb_slot[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
        const int ch = 4 * ks + kq;
        fa_slot[ks] = (wm0 + r16) * CPR + (ch ^ swz<CPR>(r16));
        fb_slot[ks] = A_CH + (wn0 + r16) * CPR + (ch ^ swz<CPR>(r16));
    }

    // transposed operands: byte offset of this lane's first read of 16-row block 0 of k-step 0 inside the operand tile;
    // block idx adds (idx << 5) by XOR (the piece index is swizzled), k-step ks adds 32 rows, the second read 4 rows
    const int fx = ((r16 >> 2) & 3) | ((kq & 1) << 2);
    const int ta_lane = (8 * kq + (r16 >> 2)) * 512 + (wm0 / 128) * 256 + ((((wm0 / 16) & 7) ^ fx) << 5) + 8 * (r16 & 3);
    const int tb_lane = (8 * kq + (r16 >> 2)) * 512 + (wn0 / 128) * 256 + ((((wn0 / 16) & 7) ^ fx) << 5) + 8 * (r16 & 3);

    f32x4 acc[MI][NI];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int ktiles = (int)(((int64_t)p.K * In::kBytes + (kRagged ? 127 : 0)) / 128);
    u32x4 fa[2][MI], fb[2][NI];
    typedef short v4s __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) v4s* tr_ptr_t;
    // the eight k of one row of a transposed operand tile: two transposing reads, 4 k-rows apart
    auto tr_frag = [&](const u32x4* tile16, int lane_off, int idx, int ks) __attribute__((always_inline)) -> u32x4 {
        const char* base = reinterpret_cast<const char*>(tile16) + ((lane_off ^ (idx << 5)) + ks * 32 * 512);
        const v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr_ptr_t)(base));
        const v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr_ptr_t)(base + 4 * 512));
        u32x2 l2, h2;
        __builtin_memcpy(&l2, &lo, 8);
        __builtin_memcpy(&h2, &hi, 8);
        return u32x4{l2.x, l2.y, h2.x, h2.y};
    };

    typedef __attribute__((address_space(1))) const void* gptr_t;
    typedef __attribute__((address_space(3))) void* lptr_t;
    // KT: index of the k-tile (128 bytes of K: 64 k of a 16-bit type)
#define MOYE_DMA(BASE, KT)                                                                            \
    _Pragma("unroll") for (int i = 0; i < LD; ++i) {                                                  \
        if constexpr (AMAJ)                                                                           \
            __builtin_amdgcn_global_load_lds((gptr_t)(static_cast<const char*>(p.A) + tA[i] + (int64_t)(KT) * 64 * pitch_a), \
                                             (lptr_t)((BASE) + dma_slot_t + 64 * i), 16, 0, 0);       \
        else if constexpr (kRagged)                                                                   \
            __builtin_amdgcn_global_load_lds((gptr_t)(gA + (int64_t)min(8 * i, more_a) * pitch_a + (int64_t)(KT) * 128 + ((KT) == ktiles - 1 ? tail_delta : 0)), \
                                             (lptr_t)((BASE) + dma_slot + 8 * CPR * i), 16, 0, 0);    \
        else                                                                                          \
            __builtin_amdgcn_global_load_lds((gptr_t)(gA + (int64_t)(8 * i) * pitch_a + (int64_t)(KT) * 128), \
                                             (lptr_t)((BASE) + dma_slot + 8 * CPR * i), 16, 0, 0);    \
        if constexpr (BMAJ)                                                                           \
            __builtin_amdgcn_global_load_lds((gptr_t)(static_cast<const char*>(p.B) + tB[i] + (int64_t)(KT) * 64 * pitch_b), \
                                             (lptr_t)((BASE) + A_CH + dma_slot_t + 64 * i), 16, 0, 0); \
        else if constexpr (kRagged)                                                                   \
            __builtin_amdgcn_global_load_lds((gptr_t)(gB + (int64_t)min(8 * i, more_b) * pitch_b + (int64_t)(KT) * 128 + ((KT) == ktiles - 1 ? tail_delta : 0)), \
                                             (lptr_t)((BASE) + A_CH + dma_slot + 8 * CPR * i), 16, 0, 0); \
        else                                                                                          \
            __builtin_amdgcn_global_load_lds((gptr_t)(gB + (int64_t)(8 * i) * pitch_b + (int64_t)(KT) * 128), \
                                             (lptr_t)((BASE) + A_CH + dma_slot + 8 * CPR * i), 16, 0, 0); \
    }
    // ragged K: the fragments of k-step KS of the last k-tile, in buffer BUF, keep only the pieces inside K
#define MOYE_MASK_TAIL(KS, BUF)                                                                       \
    if (kRagged && 4 * (KS) + kq >= k_valid) {                                                        \
        _Pragma("unroll") for (int i = 0; i < MI; ++i) fa[BUF][i] = u32x4{0u, 0u, 0u, 0u};            \
        _Pragma("unroll") for (int j = 0; j < NI; ++j) fb[BUF][j] = u32x4{0u, 0u, 0u, 0u};            \
    }
    // Wait until at most N of this wave's load-to-LDS instructions are in flight and its own LDS reads
    // have returned, then meet the other waves.  A bare s_barrier on purpose: __syncthreads() adds a
    // release fence that waits for ALL outstanding loads, which would drain the prefetch.  The waits
    // are the s_waitcnt builtin (not asm text) so that the compiler's own wait-count bookkeeping
    // sees them and does not add a second, stricter wait in front of the MFMAs.
#define MOYE_WAIT_BARRIER(N)                                                                           \
    {                                                                                                  \
        __builtin_amdgcn_s_waitcnt(((N) & 0xF) | (((N) >> 4) << 14) | 0x0070); /* vmcnt(N) lgkmcnt(0) */ \
        asm volatile("" ::: "memory");                                                                 \
        __builtin_amdgcn_s_barrier();                                                                  \
        asm volatile("" ::: "memory");                                                                 \
    }
#define MOYE_WAIT_LDS() __builtin_amdgcn_s_waitcnt(0xC07F) /* lgkmcnt(0) only */
#define MOYE_FRAGS(BASE, KS, BUF)                                                                     \
    _Pragma("unroll") for (int i = 0; i < MI; ++i) {                                                  \
        if constexpr (AMAJ) fa[BUF][i] = tr_frag((BASE), ta_lane, i, KS);                             \
        else fa[BUF][i] = (BASE)[fa_slot[KS] + 16 * CPR * i];                                         \
    }                                                                                                 \
    _Pragma("unroll") for (int j = 0; j < NI; ++j) {                                                  \
        if constexpr (BMAJ) fb[BUF][j] = tr_frag((BASE) + A_CH, tb_lane, j, KS);                      \
        else fb[BUF][j] = (BASE)[fb_slot[KS] + 16 * CPR * j];                                         \
    }
// Rows of the wave tile are walked back and forth, so that exactly one operand register set changes between
// consecutive MFMAs: with dense operands the part is power-limited, and an MFMA-only loop over an 8 x 4 register
// tile sustains 1.5-2 % more in this order than row by row (1980 against 1947 TFLOP/s).
#define MOYE_MMA(BUF, I0, I1)                                                                         \
    _Pragma("unroll") for (int i = I0; i < I1; ++i)                                                   \
        _Pragma("unroll") for (int jj = 0; jj < NI; ++jj) {                                           \
            const int j = (i & 1) ? NI - 1 - jj : jj;                                                 \
            In::mma(fb[BUF][j], fa[BUF][i], acc[i][j]);                                               \
        }

    // Issue order inside a k-step: the two waves of a SIMD leave the barrier together, so if each one
    // issued all its fragment reads first the MFMA pipe would idle for both.  Spread them instead:
    // NV load-to-LDS instructions each followed by kLoadGap MFMAs, then every ds_read followed by MFMAs.
    // (Two MFMAs between loads, measured against one, three, and loads and reads alternating: fp16 4096^3 1338 TFLOP/s
    // against 1305, 1340, 1310; with zero operands 1871 against 1773, 1846, 1761.  All eight waves of a workgroup leave the
    // barrier together, and 64 loads in as many MFMA slots are more than the vector memory pipe takes without holding
    // up the waves that issue them.)
    constexpr int kLoadGap = 2;
#define MOYE_INTERLEAVE(NV)                                                                           \
    _Pragma("unroll") for (int q = 0; q < (NV); ++q) {                                                \
        __builtin_amdgcn_sched_group_barrier(0x010, 1, 0); /* VMEM   */                               \
        __builtin_amdgcn_sched_group_barrier(0x008, kLoadGap, 0); /* MFMA   */                        \
    }                                                                                                 \
    _Pragma("unroll") for (int q = 0; q < MI + NI; ++q) {                                             \
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0); /* DS read */                              \
        __builtin_amdgcn_sched_group_barrier(0x008, (MI * NI - kLoadGap * (NV)) / (MI + NI), 0);      \
    }                                                                                                 \
    __builtin_amdgcn_sched_group_barrier(0x008, (MI * NI - kLoadGap * (NV)) % (MI + NI), 0);

    // Where in K this workgroup starts: the workgroups of one XCD (consecutive workgroup ids go to consecutive XCDs) walk K
    // together, so that the panels they share are fetched into their L2 once, but the eight XCDs start an eighth of K
    // apart, so that at any moment the chip asks memory for eight different column blocks of A and B instead of one
    // (with K-major operands and a power-of-two pitch one column block lives in few channels).  k_of() hands out the
    // indices of successive k-tiles in that rotated order; the sum over k starts elsewhere but is the same sum.
    int k_next = (!kRagged && (p.xcd_swizzle & kGemmRotateK)) ? (int)((int64_t)(blockIdx.x % 8) * ktiles / 8) : 0;  // (ragged: the last k-tile in time is the last in K)
    auto k_of = [&]() {
        const int kt_now = k_next;
        k_next = k_next + 1 == ktiles ? 0 : k_next + 1;
        return kt_now;
    };
    // prologue: tiles 0 and 1 on their way, wait for tile 0 only (LD loads per operand are younger)
    { const int ko = k_of(); MOYE_DMA(smem, ko) }
    if (ktiles > 1) {
        { const int ko = k_of(); MOYE_DMA(smem + STAGE, ko) }
        MOYE_WAIT_BARRIER(2 * LD)
    } else {
        MOYE_WAIT_BARRIER(0)
    }
    MOYE_FRAGS(smem, 0, 0)
    if (ktiles == 1) { MOYE_MASK_TAIL(0, 0) }

    // One k-tile.  DMA: tile KT+2 exists and is fetched; NEXT: tile KT+1 exists and its first fragments
    // are read.  The steady-state body has no branches, so each k-step is one scheduling region.
#define MOYE_TILE(KT, DMA, NEXT, TAIL)                                                                \
    {                                                                                                 \
        u32x4* const cur = smem + ((KT) & 1) * STAGE;                                                 \
        u32x4* const nxt = smem + (((KT) + 1) & 1) * STAGE;                                           \
        /* step 0: MFMAs on buffer 0 while the fragments of step 1 arrive in buffer 1.  Buffer 0 was  \
           requested a whole step ago; retiring those reads BEFORE the new ones are issued keeps the  \
           MFMAs from waiting on the reads they are meant to overlap with. */                         \
        MOYE_WAIT_LDS();                                                                              \
        __builtin_amdgcn_sched_barrier(0);                                                            \
        MOYE_FRAGS(cur, 1, 1)                                                                         \
        if ((TAIL) == 2) { MOYE_MASK_TAIL(1, 1) }                                                     \
        MOYE_MMA(0, 0, MI)                                                                            \
        MOYE_INTERLEAVE(0)                                                                            \
        __builtin_amdgcn_sched_barrier(0);                                                            \
        /* tile KT+1 has landed (the only loads in flight); this wave needs nothing more of tile KT */ \
        MOYE_WAIT_BARRIER(0)                                                                          \
        __builtin_amdgcn_sched_barrier(0);                                                            \
        /* step 1: the stage tile KT lived in is free, so tile KT+2 gets a whole iteration to arrive; \
           MFMAs on buffer 1 (already in registers) while step 0 of tile KT+1 arrives in buffer 0 */  \
        if (DMA) { const int ko = k_of(); MOYE_DMA(cur, ko) }                                     \
        if (NEXT) MOYE_FRAGS(nxt, 0, 0)                                                               \
        if ((TAIL) == 1) { MOYE_MASK_TAIL(0, 0) }                                                     \
        MOYE_MMA(1, 0, MI)                                                                            \
        if (NEXT) { MOYE_INTERLEAVE((DMA) ? 2 * LD : 0) }                                             \
        __builtin_amdgcn_sched_barrier(0);                                                            \
    }
    int kt = 0;
    for (; kt + 2 < ktiles; ++kt) MOYE_TILE(kt, true, true, 0)
    if (kt + 1 < ktiles) {
        MOYE_TILE(kt, false, true, 1)
        ++kt;
    }
    MOYE_TILE(kt, false, false, 2)
#undef MOYE_TILE
#undef MOYE_MASK_TAIL
#undef MOYE_INTERLEAVE
#undef MOYE_DMA
#undef MOYE_WAIT_BARRIER
#undef MOYE_WAIT_LDS
#undef MOYE_FRAGS
#undef MOYE_MMA
    __syncthreads();  // every wave is done with the operand stages before they become C patches

    // --- epilogue (mfma_epilogue.hpp): alpha*acc + C -> OutT -> this wave's LDS patch -> 128-bit row stores
    static_assert(NWAVES * 32 * WN * 4 <= 2 * STAGE * 16, "C patches (32 rows per wave and pass) fit in the operand stages");
    if constexpr (kRagged) store_c_tile_general<Out, MI, NI, true>(p, acc, smem, wave, lane, (int64_t)tm * BM + wm0, (int64_t)tn * BN + wn0);
    else store_c_tile<Out, MI, NI, kOps>(p, acc, smem, wave, lane, (int64_t)tm * BM + wm0, (int64_t)tn * BN + wn0);
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
    store_c_tile<Out, MI, NI, false>(p, acc, smem, wave, lane, (int64_t)tm * BM + wm0, (int64_t)tn * BN + wn0);
}

template <typename In, typename Out, int STAGES>
static int32_t launch256_ring(const GemmArgs& a, hipStream_t st) {
    constexpr int kLds = STAGES * (256 + 256) * 64;
    auto kern = gemm_mfma_tn_256_ring<In, Out, 2, 4, STAGES>;
    static LdsCap cap;
    if (int32_t e = raise_lds_cap(cap, reinterpret_cast<const void*>(kern), kLds)) return e;
    kern<<<dim3((unsigned)(a.tiles_m * a.tiles_n), (unsigned)(a.split > 1 ? a.split : 1)), dim3(512), kLds, st>>>(a);
    MOYE_HIP_CHECK(hipGetLastError());
    return MOYE_OK;
}

template <typename In, typename Out, int WGM, int WGN, bool kOps, int AMAJ, int BMAJ, bool kRagged = false>
static int32_t launch256_instance(const GemmArgs& a, hipStream_t st) {
    constexpr int kLds = 2 * (256 + 256) * 128;  // two operand stages, 128 KiB
    auto kern = gemm_mfma_tn_256<In, Out, WGM, WGN, kOps, AMAJ, BMAJ, kRagged>;
    static LdsCap cap;
    if (int32_t e = raise_lds_cap(cap, reinterpret_cast<const void*>(kern), kLds)) return e;
    kern<<<dim3((unsigned)(a.tiles_m * a.tiles_n), (unsigned)(a.split > 1 ? a.split : 1)), dim3(64 * WGM * WGN), kLds, st>>>(a);
    MOYE_HIP_CHECK(hipGetLastError());
    return MOYE_OK;
}

template <typename In, typename Out, int WGM, int WGN>
static int32_t launch256(const GemmArgs& a, hipStream_t st) {
    const bool am = a.xcd_swizzle & kGemmAMajorM, bm = a.xcd_swizzle & kGemmBMajorN;
    if (a.xcd_swizzle & kGemmRagged) {
        if constexpr (WGM * WGN == 8 && !std::is_same<In, InFP8>::value) {
            if (am || bm) return fail(MOYE_ERR_UNSUPPORTED, "gemm!: ragged 256 x 256 tiles take K-major operands");
            return launch256_instance<In, Out, WGM, WGN, true, 0, 0, true>(a, st);
        } else {
            return fail(MOYE_ERR_UNSUPPORTED, "gemm!: ragged 256 x 256 tiles run on eight waves with f16, bf16 or f32 operands");
        }
    }
    if (am || bm) {
        // operands that are not K-major: eight waves, 16-bit types (the host checked)
        if constexpr (WGM * WGN == 8 && In::kBytes == 2) {
            const bool ops = a.ep_op != MOYE_MAP_IDENTITY;
            if (am && bm) return ops ? launch256_instance<In, Out, WGM, WGN, true, 1, 1>(a, st) : launch256_instance<In, Out, WGM, WGN, false, 1, 1>(a, st);
            if (am) return ops ? launch256_instance<In, Out, WGM, WGN, true, 1, 0>(a, st) : launch256_instance<In, Out, WGM, WGN, false, 1, 0>(a, st);
            return ops ? launch256_instance<In, Out, WGM, WGN, true, 0, 1>(a, st) : launch256_instance<In, Out, WGM, WGN, false, 0, 1>(a, st);
        } else {
            return fail(MOYE_ERR_UNSUPPORTED, "gemm!: operands that are not K-major run natively with 16-bit types on eight waves only");
        }
    }
    if constexpr (WGM * WGN == 8) if (a.ep_op != MOYE_MAP_IDENTITY) return launch256_instance<In, Out, WGM, WGN, true, 0, 0>(a, st);
    return launch256_instance<In, Out, WGM, WGN, false, 0, 0>(a, st);
}

template <typename In>
static int32_t launch256_out(int32_t out_dt, const GemmArgs& a, int waves, int stages, hipStream_t st) {
    if (stages >= 3 && a.ep_op != MOYE_MAP_IDENTITY)
        return fail(MOYE_ERR_UNSUPPORTED, "gemm!: the ring schedules (stages >= 3) take no element-wise epilogue operation; leave stages at 0");
    if (stages >= 3) {
        const bool five = stages >= 5;
        switch (out_dt) {
            case MOYE_F32: return five ? launch256_ring<In, OutF32, 5>(a, st) : launch256_ring<In, OutF32, 4>(a, st);
            case MOYE_F16: return five ? launch256_ring<In, OutF16, 5>(a, st) : launch256_ring<In, OutF16, 4>(a, st);
            case MOYE_BF16: return five ? launch256_ring<In, OutBF16, 5>(a, st) : launch256_ring<In, OutBF16, 4>(a, st);
            default: break;
        }
    }
    if (waves == 4 && a.ep_op == MOYE_MAP_IDENTITY) {  // (with an element-wise operation the eight-wave form runs: 256 accumulators leave it no registers)
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
int32_t gemm_mfma_tn_256_dispatch(int32_t in_dt, int32_t out_dt, GemmArgs a, int waves, int stages, hipStream_t st) {
    a.tiles_m = (a.M + 255) / 256;  // (whole tiles unless kGemmRagged)
    a.tiles_n = (a.N + 255) / 256;
    switch (in_dt) {
        case MOYE_F16: return launch256_out<InF16>(out_dt, a, waves, stages, st);
        case MOYE_BF16: return launch256_out<InBF16>(out_dt, a, waves, stages, st);
        case MOYE_F8E4M3: return launch256_out<InFP8>(out_dt, a, waves, stages, st);
        case MOYE_F32: return launch256_out<InF32>(out_dt, a, waves, stages, st);
        default: return fail(MOYE_ERR_UNSUPPORTED, "gemm!: no MFMA atom for %s inputs", dtype_name(in_dt));
    }
}

}  // namespace moye

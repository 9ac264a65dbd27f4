// The k-loop and epilogue shared by the MFMA GEMM kernels that bring their operand tiles into LDS with load-to-LDS
// instructions: gemm_mfma_tn_256 (gemm_mfma256.hip: 256 x 256 CTA tile, eight or four waves, one workgroup per CU) and
// gemm_mfma_tn_128 (gemm_mfma128.hip: 128 x 128 CTA tile, four waves, two workgroups per CU).
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
#pragma once

#include <type_traits>

#include "mfma_epilogue.hpp"

namespace moye {


// kOps: the epilogue may apply an element-wise operation (GemmArgs::ep_op).  A separate instance, so that the code and
// the registers of that path never touch the kernel the plain gemm! runs.
//
// AMAJ / BMAJ = 1: that operand is stored with its unit stride along M (N) instead of K, the 'N' forms of
// src/arch/mma/make_mma_ops.jl:253-265 (GemmArgs::lda / ldb is then the pitch between consecutive k).  Its LDS tile is
// 64 k-rows of BM operand rows (512 or 256 bytes), brought in by the same load-to-LDS instructions, and the fragments come
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
// epilogues run with their row and column guards.
//
// kBias: the call's element-wise operation has a scalar, one-per-column or one-per-row operand or none and is no division
// (kGemmEpiLaneOp: a bias, a ReLU, a scale): an instance of its own that is the plain kernel with that operation in the
// lanes' own epilogue, nothing of the general one.
//
// AT = 32: the 32 x 32 MFMA forms (v_mfma_f32_32x32x16_{f16,bf16,fp8_fp8}, v_mfma_f32_32x32x2_f32), which the reference's
// make_tiled_mma takes like any other atom (src/atom/mma.jl:80-107).  A 32 x 32 MFMA reads 32 rows of each operand and
// half the K extent of the 16 x 16 form: lane l holds row l % 32 and the 16-byte chunk l / 32 of a 32-byte piece of that
// row, so a fragment of a k-step is two chunks (two MFMAs in a row per accumulator tile) and the LDS tile, the loads and
// the number of fragment reads are those of the 16 x 16 forms.  Whole tiles, K-major operands.
template <typename In, typename Out, int BM, int BN, int WGM, int WGN, bool kOps, int AMAJ, int BMAJ, bool kRagged, bool kBias = false, int AT = 16>
__device__ __forceinline__ void gemm_mfma_tn_lds_tile(GemmArgs p) {
    static_assert(AT == 16 || (AT == 32 && !AMAJ && !BMAJ && !kRagged), "32 x 32 MFMA tiles: whole tiles, K-major operands");
    static_assert(!kRagged || (!AMAJ && !BMAJ), "ragged tiles: K-major operands");
    static_assert(!kBias || (!kOps && !kRagged && !AMAJ && !BMAJ), "the bias instance: whole tiles, K-major operands");
    static_assert((BM == 256 && BN == 256) || (BM == 128 && BN == 128 && WGM == 2 && WGN == 2), "tile shapes");
    constexpr int CPR = 8;  // 8 chunks of 16 bytes per tile row
    constexpr int A_CH = BM * CPR, B_CH = BN * CPR, STAGE = A_CH + B_CH;
    constexpr int NWAVES = WGM * WGN;
    constexpr int WROWS = BM / NWAVES;  // operand rows each wave brings in per tile
    constexpr int LD = WROWS / 8;       // load-to-LDS instructions per wave per operand (8 rows each)
    constexpr int WM = BM / WGM, WN = BN / WGN, MI = WM / AT, NI = WN / AT;
    constexpr int FT = AT / 16;  // 16-byte chunks (MFMAs in a row) per fragment and k-step
    typedef float accv __attribute__((ext_vector_type(AT * AT / 64)));

    extern __shared__ u32x4 smem[];

    int tm, tn;
    split_of_block(p);
    tile_of_block(p, &tm, &tn);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm0 = (wave / WGN) * WM, wn0 = (wave % WGN) * WN;
    const int r16 = lane % AT, kq = lane / AT;  // row inside an MFMA tile, chunk inside the piece of a row one MFMA reads

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
    // (the 128 x 128 tile has registers to spare and half the MFMAs per load: its clamped row offsets are kept)
    constexpr bool kKeepRowOffsets = kRagged && BM == 128;
    [[maybe_unused]] int64_t ro_a[kKeepRowOffsets ? LD : 1], ro_b[kKeepRowOffsets ? LD : 1];
    if constexpr (kKeepRowOffsets) {
#pragma unroll
        for (int i = 0; i < LD; ++i) {
            ro_a[i] = (int64_t)min(8 * i, more_a) * pitch_a;
            ro_b[i] = (int64_t)min(8 * i, more_b) * pitch_b;
        }
    }
    const int dma_slot = __builtin_amdgcn_readfirstlane(wave * WROWS * CPR);  // + 8 rows * CPR per i
    // The 32 x 32 forms read rows r and r + 16 of a fragment in the same pass of a 128-bit LDS read (lanes l and l + 16), so
    // the chunk permutation of a row also looks at bit 4 of the row: rows 16-31 of every 32 trade neighbouring chunks.
    // On the load side that is the other 16-byte piece of a 32-byte pair for the instructions that bring such rows.
    static_assert(AT == 16 || WROWS % 32 == 0, "bit 4 of a tile row is bit 1 of the instruction index");
    [[maybe_unused]] const int pair_delta = (lch & 1) ? -16 : 16;
#define MOYE_PAIR(I) (AT == 32 && (((I) >> 1) & 1) ? pair_delta : 0)
    // An M-major (N-major) operand: a k-row of the tile is TROW bytes (BM 16-bit values); wave w fills k-rows
    // KROWS w + TRPI i + l / TLPR of the tile, TRPI rows (1 KiB) per instruction; lane l brings the 16-byte chunk that
    // belongs in physical slot l % TLPR of its row.
    constexpr int KROWS = 64 / NWAVES;
    constexpr int TROW = BM * 2, TLPR = TROW / 16, TRPI = 64 / TLPR;
    static_assert(!(AMAJ || BMAJ) || (In::kBytes == 2 && BM == BN && KROWS == TRPI * LD), "transposing fragment reads: 16-bit operands");
    auto tr_swz = [](int krow) { return (krow & 3) | (((krow >> 3) & 1) << 2); };
    [[maybe_unused]] int64_t tA[AMAJ ? LD : 1], tB[BMAJ ? LD : 1];  // byte offsets of this lane's chunk, per instruction, from the k-tile's first row
    if constexpr (AMAJ) {
#pragma unroll
        for (int i = 0; i < LD; ++i) {
            const int krow = wave * KROWS + TRPI * i + lane / TLPR, p16 = lane % TLPR, l32 = (p16 >> 1) ^ tr_swz(krow);
            tA[i] = krow * pitch_a + ((int64_t)tm * BM) * In::kBytes + (l32 * 2 + (p16 & 1)) * 16;
        }
    }
    if constexpr (BMAJ) {
#pragma unroll
        for (int i = 0; i < LD; ++i) {
            const int krow = wave * KROWS + TRPI * i + lane / TLPR, p16 = lane % TLPR, l32 = (p16 >> 1) ^ tr_swz(krow);
            tB[i] = krow * pitch_b + ((int64_t)tn * BN) * In::kBytes + (l32 * 2 + (p16 & 1)) * 16;
        }
    }
    const int dma_slot_t = __builtin_amdgcn_readfirstlane(wave * KROWS * TLPR);  // + 64 chunks (TRPI rows) per i

    // fragment slots: row = w?0 + AT i + r16, chunk = 4 ks + (4 / FT) t + kq
    int fa_slot[2][FT], fb_slot[2][FT];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks)
#pragma unroll
        for (int t = 0; t < FT; ++t) {
            const int ch = 4 * ks + (4 / FT) * t + kq, perm = swz<CPR>(r16) ^ (AT == 32 ? (r16 >> 4) & 1 : 0);
            fa_slot[ks][t] = (wm0 + r16) * CPR + (ch ^ perm);
            fb_slot[ks][t] = A_CH + (wn0 + r16) * CPR + (ch ^ perm);
        }

    // transposed operands: byte offset of this lane's first read of 16-row block 0 of k-step 0 inside the operand tile;
    // block idx adds (idx << 5) by XOR (the piece index is swizzled), k-step ks adds 32 rows, the second read 4 rows
    const int fx = ((r16 >> 2) & 3) | ((kq & 1) << 2);
    // (the blocks of a wave tile start at a piece index whose low bits are clear, so adding the block is an XOR too)
    const int ta_lane = (8 * kq + (r16 >> 2)) * TROW + (wm0 / 128) * 256 + ((((wm0 / 16) & 7) ^ fx) << 5) + 8 * (r16 & 3);
    const int tb_lane = (8 * kq + (r16 >> 2)) * TROW + (wn0 / 128) * 256 + ((((wn0 / 16) & 7) ^ fx) << 5) + 8 * (r16 & 3);

    accv acc[MI][NI];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j)
#pragma unroll
            for (int e = 0; e < AT * AT / 64; ++e) acc[i][j][e] = 0.f;

    const int ktiles = (int)(((int64_t)p.K * In::kBytes + (kRagged ? 127 : 0)) / 128);
    u32x4 fa[2][MI * FT], fb[2][NI * FT];  // (fragment i, chunk t at [FT i + t])
    typedef short v4s __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) v4s* tr_ptr_t;
    // the eight k of one row of a transposed operand tile: two transposing reads, 4 k-rows apart
    auto tr_frag = [&](const u32x4* tile16, int lane_off, int idx, int ks) __attribute__((always_inline)) -> u32x4 {
        const char* base = reinterpret_cast<const char*>(tile16) + ((lane_off ^ (idx << 5)) + ks * 32 * TROW);
        const v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr_ptr_t)(base));
        const v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr_ptr_t)(base + 4 * TROW));
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
            __builtin_amdgcn_global_load_lds((gptr_t)(gA + (kKeepRowOffsets ? ro_a[kKeepRowOffsets ? i : 0] : (int64_t)min(8 * i, more_a) * pitch_a) + (int64_t)(KT) * 128 + ((KT) == ktiles - 1 ? tail_delta : 0)), \
                                             (lptr_t)((BASE) + dma_slot + 8 * CPR * i), 16, 0, 0);    \
        else                                                                                          \
            __builtin_amdgcn_global_load_lds((gptr_t)(gA + (int64_t)(8 * i) * pitch_a + (int64_t)(KT) * 128 + MOYE_PAIR(i)), \
                                             (lptr_t)((BASE) + dma_slot + 8 * CPR * i), 16, 0, 0);    \
        if constexpr (BMAJ)                                                                           \
            __builtin_amdgcn_global_load_lds((gptr_t)(static_cast<const char*>(p.B) + tB[i] + (int64_t)(KT) * 64 * pitch_b), \
                                             (lptr_t)((BASE) + A_CH + dma_slot_t + 64 * i), 16, 0, 0); \
        else if constexpr (kRagged)                                                                   \
            __builtin_amdgcn_global_load_lds((gptr_t)(gB + (kKeepRowOffsets ? ro_b[kKeepRowOffsets ? i : 0] : (int64_t)min(8 * i, more_b) * pitch_b) + (int64_t)(KT) * 128 + ((KT) == ktiles - 1 ? tail_delta : 0)), \
                                             (lptr_t)((BASE) + A_CH + dma_slot + 8 * CPR * i), 16, 0, 0); \
        else                                                                                          \
            __builtin_amdgcn_global_load_lds((gptr_t)(gB + (int64_t)(8 * i) * pitch_b + (int64_t)(KT) * 128 + MOYE_PAIR(i)), \
                                             (lptr_t)((BASE) + A_CH + dma_slot + 8 * CPR * i), 16, 0, 0); \
    }
    // ragged K: the fragments of k-step KS of the last k-tile, in buffer BUF, keep only the pieces inside K
#define MOYE_MASK_TAIL(KS, BUF)                                                                       \
    if (kRagged && 4 * (KS) + kq >= k_valid) {                                                        \
        _Pragma("unroll") for (int i = 0; i < MI * FT; ++i) fa[BUF][i] = u32x4{0u, 0u, 0u, 0u};       \
        _Pragma("unroll") for (int j = 0; j < NI * FT; ++j) fb[BUF][j] = u32x4{0u, 0u, 0u, 0u};       \
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
    _Pragma("unroll") for (int i = 0; i < MI * FT; ++i) {                                             \
        if constexpr (AMAJ) fa[BUF][i] = tr_frag((BASE), ta_lane, i, KS);                             \
        else fa[BUF][i] = (BASE)[fa_slot[KS][i % FT] + AT * CPR * (i / FT)];                          \
    }                                                                                                 \
    _Pragma("unroll") for (int j = 0; j < NI * FT; ++j) {                                             \
        if constexpr (BMAJ) fb[BUF][j] = tr_frag((BASE) + A_CH, tb_lane, j, KS);                      \
        else fb[BUF][j] = (BASE)[fb_slot[KS][j % FT] + AT * CPR * (j / FT)];                          \
    }
// Rows of the wave tile are walked back and forth, so that exactly one operand register set changes between
// consecutive MFMAs: with dense operands the part is power-limited, and an MFMA-only loop over an 8 x 4 register
// tile sustains 1.5-2 % more in this order than row by row (1980 against 1947 TFLOP/s).
#define MOYE_MMA(BUF, I0, I1)                                                                         \
    _Pragma("unroll") for (int i = I0; i < I1; ++i)                                                   \
        _Pragma("unroll") for (int jj = 0; jj < NI; ++jj) {                                           \
            const int j = (i & 1) ? NI - 1 - jj : jj;                                                 \
            if constexpr (AT == 16) {                                                                 \
                In::mma(fb[BUF][j], fa[BUF][i], acc[i][j]);                                           \
            } else {                                                                                  \
                In::mma32(fb[BUF][2 * j], fa[BUF][2 * i], acc[i][j]);                                 \
                In::mma32(fb[BUF][2 * j + 1], fa[BUF][2 * i + 1], acc[i][j]);                         \
            }                                                                                         \
        }

    // Issue order inside a k-step: the two waves of a SIMD leave the barrier together, so if each one
    // issued all its fragment reads first the MFMA pipe would idle for both.  Spread them instead:
    // NV load-to-LDS instructions each followed by kLoadGap MFMAs, then every ds_read followed by MFMAs.
    // (Two MFMAs between loads, measured against one, three, and loads and reads alternating: fp16 4096^3 1338 TFLOP/s
    // against 1305, 1340, 1310; with zero operands 1871 against 1773, 1846, 1761.  All eight waves of a workgroup leave the
    // barrier together, and 64 loads in as many MFMA slots are more than the vector memory pipe takes without holding
    // up the waves that issue them.)
    // (the 32 x 32 forms: half as many MFMAs of twice the length per k-step, the same loads and fragment reads)
    constexpr int kLoadGap = AT == 16 ? 2 : 1;
    constexpr int NMMA = MI * NI * FT, NREAD = (MI + NI) * FT;  // per k-step (16-bit operands; more MFMAs per call otherwise)
#define MOYE_INTERLEAVE(NV)                                                                           \
    {                                                                                                 \
        _Pragma("unroll") for (int q = 0; q < (NV); ++q) {                                            \
            __builtin_amdgcn_sched_group_barrier(0x010, 1, 0); /* VMEM   */                           \
            __builtin_amdgcn_sched_group_barrier(0x008, kLoadGap, 0); /* MFMA   */                    \
        }                                                                                             \
        constexpr int kLeft = NMMA - kLoadGap * (NV); /* MFMAs after the loads */                     \
        if constexpr (kLeft >= NREAD || kLeft <= 0) {                                                 \
            _Pragma("unroll") for (int q = 0; q < NREAD; ++q) {                                       \
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0); /* DS read */                      \
                __builtin_amdgcn_sched_group_barrier(0x008, kLeft / NREAD, 0);                        \
            }                                                                                         \
            __builtin_amdgcn_sched_group_barrier(0x008, kLeft % NREAD, 0);                            \
        } else { /* fewer MFMAs than reads: several reads per MFMA */                                 \
            _Pragma("unroll") for (int q = 0; q < kLeft; ++q) {                                       \
                __builtin_amdgcn_sched_group_barrier(0x100, (NREAD + kLeft - 1) / kLeft, 0);          \
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                    \
            }                                                                                         \
        }                                                                                             \
    }

    // Where in K this workgroup starts: the workgroups of one XCD (consecutive workgroup ids go to consecutive XCDs) walk K
    // together, so that the panels they share are fetched into their L2 once, but the eight XCDs start an eighth of K
    // apart, so that at any moment the chip asks memory for eight different column blocks of A and B instead of one
    // (with K-major operands and a power-of-two pitch one column block lives in few channels).  k_of() hands out the
    // indices of successive k-tiles in that rotated order; the sum over k starts elsewhere but is the same sum.
    // (a K tail: the k-tile that holds it is masked as the last in time, so it has to be the last in K as well)
    int k_next = ((p.flags & kGemmRotateK) && !(kRagged && k_rem)) ? (int)((int64_t)(blockIdx.x % p.xcds) * ktiles / p.xcds) : 0;
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
#undef MOYE_PAIR
#undef MOYE_WAIT_BARRIER
#undef MOYE_WAIT_LDS
#undef MOYE_FRAGS
#undef MOYE_MMA
    __syncthreads();  // every wave is done with the operand stages before they become C patches

    // --- epilogue (mfma_epilogue.hpp): alpha*acc + C -> OutT -> this wave's LDS patch -> 128-bit row stores
    static_assert(NWAVES * 32 * WN * 4 <= 2 * STAGE * 16, "C patches (32 rows per wave and pass) fit in the operand stages");
    // (a kOps instance is only launched for calls with an operation or with ragged tiles: it carries the general
    // epilogue alone, which keeps the other one's registers out of its allocation)
    if constexpr (kBias) store_c_tile<Out, MI, NI, false, true, false, AT>(p, acc, smem, wave, lane, (int64_t)tm * BM + wm0, (int64_t)tn * BN + wn0);
    else if constexpr (kOps) store_c_tile_general<Out, MI, NI, kRagged, AT>(p, acc, smem, wave, lane, (int64_t)tm * BM + wm0, (int64_t)tn * BN + wn0);
    else store_c_tile<Out, MI, NI, kRagged, false, false, AT>(p, acc, smem, wave, lane, (int64_t)tm * BM + wm0, (int64_t)tn * BN + wn0);
}

}  // namespace moye

// gemm! on the matrix cores: D = alpha * A * B' + C for K-major ("TN") A:(M,K), B:(N,K) in
// f16 / bf16 / fp8-e4m3 with fp32 accumulation, written for gfx950 (64-lane waves, MFMA).
//
// Stands where the reference has its tensor-core user kernel and the loops under it
// (docs/src/manual/tensor_core.md:265-355 driving src/algorithm/blas.jl:74-131 and
// src/algorithm/copy.jl:106-130).  The reference's pieces map as follows:
//   cp.async gmem->smem   (src/arch/copy/copy_async.jl:8-24)  -> 128-bit global loads, staged in
//                          registers, written to LDS with an XOR swizzle on the 16-byte chunk
//   ldmatrix smem->reg    (src/arch/copy/ldmatrix.jl:18-48)   -> ds_read_b128 fragment loads that
//                          land directly in MFMA operand order
//   mma.sync              (src/arch/mma/make_mma_ops.jl:387-407) -> v_mfma_f32_16x16x32_{f16,bf16},
//                          v_mfma_f32_16x16x32_fp8_fp8
//   epilogue copyto!(tCgC, tCrC) (test/device/matmul.jl:51) -> registers -> LDS -> 128-bit stores
//
// Wave layout: 2 x 2 waves per workgroup, each wave owns a (BM/2) x (BN/2) block of C made of
// 16x16 MFMA tiles.  The MFMA is issued with the B-matrix rows as its first operand and the
// A-matrix rows as its second, so a lane ends up holding four CONSECUTIVE n of one m, which is
// what a row-major D wants.
#include "gemm_plan.hpp"
#include "mfma_common.hpp"

namespace moye {

// kEdge: M, N need not be multiples of the tile and K need not be a multiple of the k-tile (only of 16
// bytes): a row beyond M / N is read from the operand's last row instead (what is computed from it is never
// stored), k beyond K is read as zeros (the predication the reference's copyto_if! is meant for,
// src/algorithm/copy.jl:4-16; only loads of the last k-tile can take that branch) and the epilogue stores
// element by element inside the bounds.
//
// AT = 16 issues the 16x16 MFMA forms, AT = 32 the 32x32 ones (v_mfma_f32_32x32x16_{f16,bf16,fp8_fp8},
// v_mfma_f32_32x32x2_f32).  A 32x32 MFMA reads 32 rows of each operand and half the K extent of the
// 16x16 form: lane l holds row l % 32 and the 16-byte chunk l / 32 of a 32-byte piece of that row, and its 16
// accumulators are four groups of four consecutive n (n = 8 g + 4 (l / 32) + 0..3) of row m = l % 32.
template <typename In, typename Out, int BM, int BN, int BKB /* bytes of K per tile row */, bool kEdge = false, int AT = 16>
__global__ __launch_bounds__(256) void gemm_mfma_tn(GemmArgs p) {
    constexpr int CPR = BKB / 16;                 // 16-byte chunks per tile row
    constexpr int CS = 64 / AT;                   // chunks of a row that the lanes of one MFMA step cover
    constexpr int KSTEPS = CPR / CS;              // one step = one (fp8: two, fp32: four) MFMA k-slice
    constexpr int A_CH = BM * CPR, B_CH = BN * CPR;
    constexpr int A_LD = A_CH / 256, B_LD = B_CH / 256;
    constexpr int WM = BM / 2, WN = BN / 2, MI = WM / AT, NI = WN / AT;
    constexpr int G = AT * AT / 256;              // groups of four accumulators per lane and MFMA tile
    static_assert(A_CH % 256 == 0 && B_CH % 256 == 0 && CPR % 4 == 0 && (AT == 16 || AT == 32), "tile shape");
    typedef typename Out::type OutT;
    typedef float accv __attribute__((ext_vector_type(4 * G)));

    extern __shared__ u32x4 smem[];
    u32x4* const sA0 = smem;
    u32x4* const sB0 = smem + A_CH;
    constexpr int STAGE = A_CH + B_CH;

    int tm, tn;
    split_of_block(p);
    tile_of_block(p, &tm, &tn);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm0 = (wave >> 1) * WM, wn0 = (wave & 1) * WN;
    const int r16 = lane % AT, kq = lane / AT;   // row inside an MFMA tile, chunk inside a step

    // the chunk permutation of a tile row.  A 128-bit LDS read serves lanes l and l + 16 in one pass: with the 32x32 forms
    // those are rows r and r + 16 of a fragment, so bit 4 of the row takes part as well (rows 16-31 of every 32 trade
    // neighbouring chunks)
    auto perm = [](int row) { return swz<CPR>(row) ^ (AT == 32 ? (row >> 4) & 1 : 0); };
    const int64_t kbytes_a = (int64_t)p.lda * In::kBytes, kbytes_b = (int64_t)p.ldb * In::kBytes;
    const char* gA = static_cast<const char*>(p.A) + (int64_t)tm * BM * kbytes_a;
    const char* gB = static_cast<const char*>(p.B) + (int64_t)tn * BN * kbytes_b;

    // per-thread global chunk addresses and LDS slots (fixed for the whole k loop)
    const char* a_src[A_LD];
    const char* b_src[B_LD];
    int a_dst[A_LD], b_dst[B_LD];
    int a_lim[A_LD], b_lim[B_LD];  // kEdge: bytes of K this chunk may still read (0 for a row out of bounds)
    const int64_t kbytes = (int64_t)p.K * In::kBytes;
#pragma unroll
    for (int i = 0; i < A_LD; ++i) {
        const int c = tid + 256 * i, row = c / CPR, ch = c % CPR;
        a_src[i] = gA + (kEdge ? min(row, p.M - 1 - tm * BM) : row) * kbytes_a + ch * 16;
        a_dst[i] = row * CPR + (ch ^ perm(row));
        a_lim[i] = (int)(kbytes - ch * 16);
    }
#pragma unroll
    for (int i = 0; i < B_LD; ++i) {
        const int c = tid + 256 * i, row = c / CPR, ch = c % CPR;
        b_src[i] = gB + (kEdge ? min(row, p.N - 1 - tn * BN) : row) * kbytes_b + ch * 16;
        b_dst[i] = row * CPR + (ch ^ perm(row));
        b_lim[i] = (int)(kbytes - ch * 16);
    }
    // a chunk at byte offset koff of its row is inside the operand iff koff < lim
    auto load_a = [&](int i, int64_t koff) -> u32x4 {
        if (kEdge && koff >= a_lim[i]) return u32x4{0u, 0u, 0u, 0u};
        return *reinterpret_cast<const u32x4*>(a_src[i] + koff);
    };
    auto load_b = [&](int i, int64_t koff) -> u32x4 {
        if (kEdge && koff >= b_lim[i]) return u32x4{0u, 0u, 0u, 0u};
        return *reinterpret_cast<const u32x4*>(b_src[i] + koff);
    };

    accv acc[MI][NI];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j)
#pragma unroll
            for (int e = 0; e < 4 * G; ++e) acc[i][j][e] = 0.f;

    const int ktiles = (int)((kbytes + BKB - 1) / BKB);
    u32x4 ra[A_LD], rb[B_LD];

    // prologue: tile 0 -> LDS stage 0
#pragma unroll
    for (int i = 0; i < A_LD; ++i) ra[i] = load_a(i, 0);
#pragma unroll
    for (int i = 0; i < B_LD; ++i) rb[i] = load_b(i, 0);
#pragma unroll
    for (int i = 0; i < A_LD; ++i) sA0[a_dst[i]] = ra[i];
#pragma unroll
    for (int i = 0; i < B_LD; ++i) sB0[b_dst[i]] = rb[i];
    __syncthreads();

    for (int kt = 0; kt < ktiles; ++kt) {
        const u32x4* sA = sA0 + (kt & 1) * STAGE;
        const u32x4* sB = sB0 + (kt & 1) * STAGE;
        const bool more = kt + 1 < ktiles;
        if (more) {  // next tile: global -> registers, in flight during the MFMAs below
            const int64_t koff = (int64_t)(kt + 1) * BKB;
#pragma unroll
            for (int i = 0; i < A_LD; ++i) ra[i] = load_a(i, koff);
#pragma unroll
            for (int i = 0; i < B_LD; ++i) rb[i] = load_b(i, koff);
        }
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
            u32x4 fa[MI], fb[NI];
            const int ch = ks * CS + kq;
#pragma unroll
            for (int i = 0; i < MI; ++i) {
                const int row = wm0 + AT * i + r16;
                fa[i] = sA[row * CPR + (ch ^ perm(row))];
            }
#pragma unroll
            for (int j = 0; j < NI; ++j) {
                const int row = wn0 + AT * j + r16;
                fb[j] = sB[row * CPR + (ch ^ perm(row))];
            }
            // rows walked back and forth: one operand register set changes between consecutive MFMAs, which
            // costs less power than two (the part is power-limited with dense operands)
#pragma unroll
            for (int i = 0; i < MI; ++i)
#pragma unroll
                for (int jj = 0; jj < NI; ++jj) {
                    const int j = (i & 1) ? NI - 1 - jj : jj;
                    if constexpr (AT == 16) In::mma(fb[j], fa[i], acc[i][j]);
                    else In::mma32(fb[j], fa[i], acc[i][j]);
                }
        }
        if (more) {  // registers -> the other LDS stage
            u32x4* dA = sA0 + ((kt + 1) & 1) * STAGE;
            u32x4* dB = sB0 + ((kt + 1) & 1) * STAGE;
#pragma unroll
            for (int i = 0; i < A_LD; ++i) dA[a_dst[i]] = ra[i];
#pragma unroll
            for (int i = 0; i < B_LD; ++i) dB[b_dst[i]] = rb[i];
        }
        __syncthreads();
    }

    // ---- epilogue: alpha*acc + C -> OutT -> this wave's LDS patch -> 128-bit row stores ----
    // lane holds C[m = AT i + r16][n = AT j + 8 g + 4 kq + e], e = 0..3 (g = 0 only for the 16x16 forms)
    const int64_t m_base = (int64_t)tm * BM + wm0, n_base = (int64_t)tn * BN + wn0;
    // residue tiles, and any tile with an element-wise operation in the epilogue: every lane stores its own elements
    if (kEdge || p.ep_op != MOYE_MAP_IDENTITY) {
#pragma unroll
        for (int i = 0; i < MI; ++i) {
            const int64_t m = m_base + AT * i + r16;
            if (m >= p.M) continue;
#pragma unroll
            for (int j = 0; j < NI; ++j) {
#pragma unroll
                for (int g = 0; g < G; ++g) {
                    const int64_t n = n_base + AT * j + 8 * g + 4 * kq;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        if (n + e >= p.N) continue;
                        const float c = p.C ? Out::load(p.C, m * p.ldc_m + (n + e) * p.ldc_n) : 0.f;
                        static_cast<OutT*>(p.D)[m * p.ldd + n + e] = Out::cvt(epi_value(p, acc[i][j][4 * g + e], p.C != nullptr, c, m, n + e));
                    }
                }
            }
        }
        return;
    }
    constexpr int EPC = 16 / (int)sizeof(OutT);          // elements per 16-byte chunk
    constexpr int CR = WN / EPC;                         // chunks per patch row
    constexpr int PASS_MI = (sizeof(OutT) == 4 && MI > 1) ? MI / 2 : MI;  // keep the patch <= 8 KiB
    constexpr int PASS_ROWS = PASS_MI * AT;
    OutT* patch = reinterpret_cast<OutT*>(smem) + wave * (PASS_ROWS * WN);
    u32x4* patch16 = reinterpret_cast<u32x4*>(patch);
    // C with unit stride along n and 16-byte aligned rows (kGemmRowC) is read the way D is written, in 128-bit pieces
    // of whole rows, all requested up front, and handed to the lanes through the patch (see mfma_epilogue.hpp)
    constexpr int NCH = PASS_ROWS * CR / 64, PASSES = MI / PASS_MI;
    const bool row_c = p.C && (p.flags & kGemmRowC);
    u32x4 cw[PASSES][NCH];
    if (row_c) {
#pragma unroll
        for (int ps = 0; ps < PASSES; ++ps)
#pragma unroll
            for (int t = 0; t < NCH; ++t) {
                const int c = lane + 64 * t, row = c / CR, ch = c % CR;
                cw[ps][t] = *reinterpret_cast<const u32x4*>(static_cast<const char*>(p.C) +
                                                            ((m_base + PASS_ROWS * ps + row) * p.ldc_m + n_base) * (int64_t)sizeof(OutT) + ch * 16);
            }
    }

#pragma unroll
    for (int i0 = 0; i0 < MI; i0 += PASS_MI) {
        if (row_c) {
#pragma unroll
            for (int t = 0; t < NCH; ++t) {
                const int c = lane + 64 * t, row = c / CR, ch = c % CR;
                patch16[row * CR + (ch ^ (row & (CR - 1)))] = cw[i0 / PASS_MI][t];
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }
#pragma unroll
        for (int ii = 0; ii < PASS_MI; ++ii) {
            const int i = i0 + ii;
#pragma unroll
            for (int j = 0; j < NI; ++j) {
#pragma unroll
                for (int g = 0; g < G; ++g) {
                    const int row = AT * ii + r16, col = AT * j + 8 * g + 4 * kq;
                    const int chunk = col / EPC, within = col % EPC;
                    OutT* dst = patch + (row * CR + (chunk ^ (row & (CR - 1)))) * EPC + within;
                    const int64_t m = m_base + AT * i + r16, n = n_base + AT * j + 8 * g + 4 * kq;
                    float v[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        v[e] = __fmul_rn(acc[i][j][4 * g + e], p.alpha);
                        if (row_c) v[e] = __fadd_rn(v[e], __fmul_rn(p.beta, Out::load(dst, e)));
                        else if (p.C) v[e] = __fadd_rn(v[e], __fmul_rn(p.beta, Out::load(p.C, m * p.ldc_m + (n + e) * p.ldc_n)));
                    }
#pragma unroll
                    for (int e = 0; e < 4; ++e) dst[e] = Out::cvt(v[e]);
                }
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int t = 0; t < PASS_ROWS * CR / 64; ++t) {
            const int c = lane + 64 * t, row = c / CR, ch = c % CR;
            const u32x4 w = patch16[row * CR + (ch ^ (row & (CR - 1)))];
            char* d = static_cast<char*>(p.D) +
                      ((m_base + AT * i0 + row) * p.ldd + n_base) * (int64_t)sizeof(OutT) + ch * 16;
            store_d_chunk(p, d, w);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
}

template <typename In, typename Out, int BM, int BN, int BKB, bool kEdge = false, int AT = 16>
static int32_t launch(const GemmArgs& a, GemmPlan& plan) {
    typedef typename Out::type OutT;
    constexpr int kMain = 2 * (BM + BN) * BKB;
    constexpr int kEpi = (sizeof(OutT) == 4 && BM / 32 > 1 ? BM / 2 : BM) * BN * (int)sizeof(OutT);
    constexpr int kLds = kMain > kEpi ? kMain : kEpi;
    static LdsCap cap;
    plan.add_kernel(gemm_mfma_tn<In, Out, BM, BN, BKB, kEdge, AT>, a, (unsigned)(a.tiles_m * a.tiles_n), (unsigned)(a.split > 1 ? a.split : 1), 256, kLds,
                    kLds > 64 * 1024 ? &cap : nullptr, BM, BN, BKB, In::kDt, Out::kDt, "gemm_mfma_tn<%s,%s,%d,%d,%d,edge=%d,atom=%d>", In::kName,
                    Out::kName, BM, BN, BKB, (int)kEdge, AT);
    return MOYE_OK;
}

template <typename In, int BM, int BN, int BKB, bool kEdge = false, int AT = 16>
static int32_t launch_out(int32_t out_dt, const GemmArgs& a, GemmPlan& plan) {
    switch (out_dt) {
        case MOYE_F32: return launch<In, OutF32, BM, BN, BKB, kEdge, AT>(a, plan);
        case MOYE_F16: return launch<In, OutF16, BM, BN, BKB, kEdge, AT>(a, plan);
        case MOYE_BF16: return launch<In, OutBF16, BM, BN, BKB, kEdge, AT>(a, plan);
        default: return fail(MOYE_ERR_UNSUPPORTED, "gemm!: MFMA kernels write f32, f16 or bf16, not %s", dtype_name(out_dt));
    }
}

template <bool kEdge>
static int32_t launch_atom32(int32_t in_dt, int32_t out_dt, const GemmArgs& a, GemmPlan& plan) {
    switch (in_dt) {
        case MOYE_F16: return launch_out<InF16, 128, 128, 64, kEdge, 32>(out_dt, a, plan);
        case MOYE_BF16: return launch_out<InBF16, 128, 128, 64, kEdge, 32>(out_dt, a, plan);
        case MOYE_F8E4M3: return launch_out<InFP8, 128, 128, 64, kEdge, 32>(out_dt, a, plan);
        case MOYE_F32: return launch_out<InF32, 128, 128, 64, kEdge, 32>(out_dt, a, plan);
        default: return fail(MOYE_ERR_UNSUPPORTED, "gemm!: no MFMA atom for %s inputs", dtype_name(in_dt));
    }
}

// The 32x32 atoms: CTA tile 256x256 with 128 bytes of K per row on eight waves of 4 x 2 MFMA tiles each (whole tiles;
// gemm_mfma256_atom32.hip), or 128x128 with 64 bytes of K per row, four waves of 2 x 2 MFMA tiles each, residue tiles
// under the same rule as for the 16x16 atoms.  Left to the library: 256x256 tiles when they divide the problem and
// fill at least half of the chip.
static int32_t dispatch_atom32(int32_t in_dt, int32_t out_dt, int bm, int bn, int bk_elems, int waves, int stages, GemmArgs a, GemmPlan& plan) {
    const int eb = dtype_bytes(in_dt), ob = dtype_bytes(out_dt);
    const bool chosen_here = bm == 0 && bn == 0;
    const bool named256 = bm == 256 && bn == 256 && (bk_elems == 0 || bk_elems * eb == 128);
    if (!named256 && ((bm && bm != 128) || (bn && bn != 128) || (bk_elems && bk_elems * eb != 64)))
        return fail(MOYE_ERR_UNSUPPORTED, "gemm!: the 32x32 MFMA atoms run with CTA tile 256x256x%d or 128x128x%d, not %dx%dx%d", 128 / eb, 64 / eb, bm, bn,
                    bk_elems);
    if ((a.lda * eb) % 16 || (a.ldb * eb) % 16 || (reinterpret_cast<uintptr_t>(a.A) | reinterpret_cast<uintptr_t>(a.B)) % 16)
        return fail(MOYE_ERR_ALIGN, "gemm!: operands of the MFMA kernels need 16-byte aligned pointers and row pitches");
    const bool whole256 = a.M % 256 == 0 && a.N % 256 == 0 && a.K % (128 / eb) == 0;
    const bool aligned_d = !((a.ldd * ob) % 16 || reinterpret_cast<uintptr_t>(a.D) % 16);
    if (named256) {
        if (!whole256) return fail(MOYE_ERR_SHAPE, "gemm!: the 32x32 MFMA atoms take whole 256x256x%d tiles, the problem is %dx%dx%d", 128 / eb, a.M, a.N, a.K);
        if (!aligned_d) return fail(MOYE_ERR_ALIGN, "gemm!: operands of the MFMA kernels need 16-byte aligned pointers and row pitches");
        if ((waves > 1 && waves != 8) || stages >= 3 || (a.flags & (MOYE_GEMM_WAVE4 | MOYE_GEMM_PINGPONG)))
            return fail(MOYE_ERR_UNSUPPORTED, "gemm!: the 32x32 MFMA atoms on 256x256 tiles run on 2 x 4 waves with two LDS stages");
        return gemm_mfma_tn_256_atom32_dispatch(in_dt, out_dt, a, plan);
    }
    if (chosen_here && whole256 && aligned_d && (int64_t)(a.M / 256) * (a.N / 256) >= plan.shape.cus / 2 && stages < 3 &&
        !(a.flags & (MOYE_GEMM_WAVE4 | MOYE_GEMM_PINGPONG)))
        return gemm_mfma_tn_256_atom32_dispatch(in_dt, out_dt, a, plan);
    a.tiles_m = (a.M + 127) / 128;
    a.tiles_n = (a.N + 127) / 128;
    if (a.M % 128 || a.N % 128 || a.K % (64 / eb)) {
        if (!chosen_here && !(a.flags & MOYE_GEMM_PREDICATE))
            return fail(MOYE_ERR_SHAPE, "gemm!: CTA tile 128x128x%d does not divide the problem %dx%dx%d", 64 / eb, a.M, a.N, a.K);
        if (((int64_t)a.K * eb) % 16)
            return fail(MOYE_ERR_SHAPE, "gemm!: the predicated MFMA kernel needs K to be a multiple of %d elements (16 bytes), got %d",
                        16 / eb, a.K);
        return launch_atom32<true>(in_dt, out_dt, a, plan);
    }
    if ((a.ldd * ob) % 16 || reinterpret_cast<uintptr_t>(a.D) % 16)
        return fail(MOYE_ERR_ALIGN, "gemm!: operands of the MFMA kernels need 16-byte aligned pointers and row pitches");
    return launch_atom32<false>(in_dt, out_dt, a, plan);
}

// K-major A and B, N-contiguous D.  bk_elems = 0 picks the default K extent per tile.
// `lib`: the tile (and K ranges) the host chose together with the split when everything was left to the library
// (gemm_choose, gemm_plan.hpp); null where only the tile is open (a part of a larger problem, a split the caller named).
int32_t gemm_mfma_tn_dispatch(int32_t in_dt, int32_t out_dt, int bm, int bn, int bk_elems, int waves, int stages,
                              GemmArgs a, GemmPlan& plan, const TileChoice* lib) {
    const int eb = dtype_bytes(in_dt);
    const int cus = plan.shape.cus;
    if (a.flags & kGemmAtom32) return dispatch_atom32(in_dt, out_dt, bm, bn, bk_elems, waves, stages, a, plan);
    // a short A (at most 64 rows) is a bandwidth problem: stream B once, no CTA tiling
    if ((bm == 0 && bn == 0 && gemm_short_m(a.M, a.N, (int64_t)a.K * eb * (a.split > 1 ? a.split : 1), eb == 4, cus)) || (bm == a.M && bm <= 64 && bn == 16))
        return gemm_mfma_skinny_dispatch(in_dt, out_dt, a, plan);
    const bool chosen_here = bm == 0 && bn == 0;
    if (bm == 0 && bn == 0) {
        // the library chooses: 256 x 256 tiles, one per CU, where the cost model of gemm_plan.hpp prices them below
        // 128 x 128 and 64 x 64 tiles (they need not fill the chip: fp16 4096 x 2304 x 4096, 144 tiles, 73 us against 93;
        // 4096 x 2048 x 4096, 128 tiles, 72 us against 62 on 128 x 128 tiles)
        const int64_t rtiles = (int64_t)((a.M + 255) / 256) * ((a.N + 255) / 256);
        const int ranges = a.split > 1 ? a.split : 1;
        const int64_t k_bytes_all = (int64_t)a.K * eb * ranges;
        const bool whole256 = a.M % 256 == 0 && a.N % 256 == 0 && a.K % (128 / eb) == 0;
        const TileChoice choice = lib && lib->tile != 256 ? *lib
                                  : gemm_plan(a.M, a.N, k_bytes_all, eb == 4, a.M % 64 == 0 && a.N % 64 == 0 && ((int64_t)a.K * eb) % 128 == 0, 16, cus, ranges);
        // (operands that were left M- or N-major: the host made sure of whole 128 x 128 tiles, an aligned D and no K ranges;
        // such a call takes whole 256 x 256 or 128 x 128 tiles, never 64 x 64 ones, ragged ones or fringes)
        const bool majors = a.flags & (kGemmAMajorM | kGemmBMajorN);
        const bool prefer256 = lib ? lib->tile == 256
                               : ranges > 1 ? rtiles >= cus / 2
                                            : rtiles >= cus / 4 && gemm_plan_cost_256(a.M, a.N, k_bytes_all, eb == 4, !whole256, cus) <= choice.us;
        const bool big = whole256 && prefer256;
        // A large problem whose M or N is not a multiple of 256: the interior runs on 256x256 tiles, the fringe to the
        // right (all interior rows, the last N % 256 columns) and the fringe below (the last M % 256 rows, all columns)
        // on the kernels that take residue tiles.  Three launches on the same stream, disjoint parts of D.
        const int M0 = a.M / 256 * 256, N0 = a.N / 256 * 256, ob0 = dtype_bytes(out_dt);
        const bool aligned_ab = !((a.lda * eb) % 16 || (a.ldb * eb) % 16 ||
                                  (reinterpret_cast<uintptr_t>(a.A) | reinterpret_cast<uintptr_t>(a.B)) % 16);
        const bool aligned = aligned_ab && !((a.ldd * ob0) % 16 || reinterpret_cast<uintptr_t>(a.D) % 16);
        // Ragged tiles on the 256 x 256 kernel itself (its guarded instance: rows clamped, the K tail masked, stores
        // guarded) when that fills the chip, unless the fringes are thin enough for the short-M kernel, which then costs
        // less than a further round of tiles (fp16 4000 x 4096 x 4096: 170 us as interior + fringe on 128 x 128 tiles,
        // vendor library 96).  Not fp8: its fast kernel is the hand-ordered one, which has no guarded form.
        const int fr_m = a.M - M0, fr_n = a.N - N0;
        // (a D that is not 16-byte aligned: the interior then runs on the guarded instance, which stores such rows in
        // smaller pieces, and the short-M kernel writes D element by element anyway.)  Priced on its own: whole tiles for
        // the interior plus a short-M launch per fringe (4.5 us and its operands at 6 TB/s), against the plan for the
        // whole problem (fp16 4100 x 4100 x 4096: 17 x 17 ragged tiles are a second round for 33 tiles and cost more than
        // 128 x 128 tiles, 167-173 us either way; interior and two fringes 116)
        // (whole interior tiles with a D that is not aligned need the guarded instance: its conditions, as below)
        const bool guarded_takes_interior = in_dt != MOYE_F8E4M3 && stages < 3 && (waves <= 1 || waves == 8) &&
                                            !(a.flags & (MOYE_GEMM_WAVE4 | MOYE_GEMM_PINGPONG | kGemmAMajorM | kGemmBMajorN | kGemmAtom32));
        const bool thin_shape = (fr_m > 0 || fr_n > 0) && fr_m <= 64 && fr_n <= 64 && a.K % (128 / eb) == 0 && aligned_ab && ranges == 1 &&
                                (aligned || guarded_takes_interior);
        const double fringe_us = (fr_n > 0 ? 4.5 + (double)(M0 + fr_n) * (double)k_bytes_all / 6.0e6 : 0.0) +
                                 (fr_m > 0 ? 4.5 + (double)(a.N + fr_m) * (double)k_bytes_all / 6.0e6 : 0.0);
        const bool thin = thin_shape && (int64_t)(M0 / 256) * (N0 / 256) >= cus / 4 &&
                          gemm_plan_cost_256(M0, N0, k_bytes_all, eb == 4, false, cus) + fringe_us <= choice.us;
        // (the hand-ordered kernel's guarded forms: K of whole 16-byte pieces)
        const bool hand_ordered_ragged = (eb == 2 || eb == 4 || in_dt == MOYE_F8E4M3) && ((int64_t)a.K * eb) % 16 == 0 &&
                                         stages < 2 && row_offsets_fit(a, 256, eb);
        if ((!big || !aligned) && !thin && a.split <= 1 && bk_elems == 0 && aligned_ab && (in_dt != MOYE_F8E4M3 || hand_ordered_ragged) && ((int64_t)a.K * eb) % 16 == 0 &&
            prefer256 && stages < 3 && (waves <= 1 || waves == 8) &&
            !(a.flags & (MOYE_GEMM_WAVE4 | MOYE_GEMM_PINGPONG | kGemmAMajorM | kGemmBMajorN | kGemmAtom32))) {
            a.flags |= kGemmRagged;
            // the hand-ordered kernel's guarded forms (rows clamped, a K tail masked in registers; with a C or an
            // element-wise operation the instance whose epilogue is the general one)
            if (hand_ordered_ragged) return gemm_mfma_tn_256_w4_dispatch(in_dt, out_dt, a, 8, 128, false, plan);
            return gemm_mfma_tn_256_dispatch(in_dt, out_dt, a, 8, stages, plan);
        }
        if (!big && !majors && a.split <= 1 && bk_elems == 0 && (thin || (aligned && prefer256)) && a.K % (128 / eb) == 0 && (int64_t)(M0 / 256) * (N0 / 256) >= cus / 4) {
            GemmArgs part = a;
            part.M = M0; part.N = N0;
            if (int32_t e = gemm_mfma_tn_dispatch(in_dt, out_dt, 0, 0, 0, waves, stages, part, plan)) return e;
            if (a.N > N0 && a.N - N0 <= 64 && ((int64_t)a.K * eb) % 64 == 0) {
                // a narrow fringe is a short-M problem once transposed: D(:, N0:)' = B(N0:, :) * A'
                part = a;
                part.M = a.N - N0; part.N = M0;
                part.A = static_cast<const char*>(a.B) + (int64_t)N0 * a.ldb * eb; part.lda = a.ldb;
                part.B = a.A; part.ldb = a.lda;
                part.D = static_cast<char*>(a.D) + (int64_t)N0 * ob0; part.ldd = 1; part.ldd_n = a.ldd;
                if (a.C) part.C = static_cast<const char*>(a.C) + (int64_t)N0 * a.ldc_n * ob0;
                part.ldc_m = a.ldc_n; part.ldc_n = a.ldc_m;
                if (a.ep_x) part.ep_x = static_cast<const char*>(a.ep_x) + (int64_t)N0 * a.ep_xn * dtype_bytes(a.ep_xdt);
                part.ep_xm = a.ep_xn; part.ep_xn = a.ep_xm;
                if (int32_t e = gemm_mfma_skinny_dispatch(in_dt, out_dt, part, plan)) return e;
            } else if (a.N > N0) {
                part = a;
                part.M = M0; part.N = a.N - N0;
                part.B = static_cast<const char*>(a.B) + (int64_t)N0 * a.ldb * eb;
                part.D = static_cast<char*>(a.D) + (int64_t)N0 * ob0;
                if (a.C) part.C = static_cast<const char*>(a.C) + (int64_t)N0 * a.ldc_n * ob0;
                if (a.ep_x) part.ep_x = static_cast<const char*>(a.ep_x) + (int64_t)N0 * a.ep_xn * dtype_bytes(a.ep_xdt);
                if (int32_t e = gemm_mfma_tn_dispatch(in_dt, out_dt, 0, 0, 0, 0, 0, part, plan)) return e;
            }
            if (a.M > M0) {
                part = a;
                part.M = a.M - M0;
                part.A = static_cast<const char*>(a.A) + (int64_t)M0 * a.lda * eb;
                part.D = static_cast<char*>(a.D) + (int64_t)M0 * a.ldd * ob0;
                if (a.C) part.C = static_cast<const char*>(a.C) + (int64_t)M0 * a.ldc_m * ob0;
                if (a.ep_x) part.ep_x = static_cast<const char*>(a.ep_x) + (int64_t)M0 * a.ep_xm * dtype_bytes(a.ep_xdt);
                if (int32_t e = gemm_mfma_tn_dispatch(in_dt, out_dt, 0, 0, 0, 0, 0, part, plan)) return e;
            }
            return MOYE_OK;
        }
        // More whole 256 x 256 tiles than CUs, and a last round that fills a small part of the chip: two launches on the
        // same stream, the first on 256 x 256 tiles over as many tile rows (or columns) as the cost model likes, the
        // second over the rest on the tiles the library would choose for that problem alone (fp16 6144^3, 576 tiles:
        // 388 us in one launch, 344 as 20 + 4 tile rows, vendor library 366; 4608^3 185 -> 161-163, vendor 171;
        // 4608 x 4608 x 8192 318 -> 270-282; 5120^3, 400 tiles, gains nothing and the model says so).  Every
        // operand type, with everything left to the library; taken when the model sees 3 % or more (fp32: 12 %).
        if (big && a.split <= 1 && ranges == 1 && !majors && bk_elems == 0 && waves <= 1 && stages == 0 &&
            rtiles > cus && rtiles % cus && !(a.flags & (MOYE_GEMM_WAVE4 | MOYE_GEMM_PINGPONG | kGemmAtom32))) {
            const int tm = a.M / 256, tn = a.N / 256;
            const bool by_rows = tm >= tn;
            const int nt = by_rows ? tm : tn;
            auto alone = [&](int64_t m, int64_t n) {  // what the library would run the part as, priced
                const double on128 = gemm_plan(m, n, k_bytes_all, eb == 4, true, 16, cus, 1).us;
                const double on256 = gemm_plan_cost_256(m, n, k_bytes_all, eb == 4, false, cus);
                return (m / 256) * (n / 256) >= cus / 4 && on256 <= on128 ? on256 : on128;
            };
            const double whole_us = gemm_plan_cost_256(a.M, a.N, k_bytes_all, eb == 4, false, cus);
            // (fp32: the model prices a part-filled round like a full one, 7 % more than it takes, so it has to see 12 %;
            // every split it then takes was priced at 20 % or more and gains: 6144^3 4065 -> 3074 us, 4352 x 4352 x 2048
            // 912 -> 580, 7168 x 7168 x 2048 1833 -> 1494, 4608^3 2023 -> 1754)
            double best_us = (eb == 4 ? 0.88 : 0.97) * whole_us;
            int first = 0;
            for (int r = 1; r < nt; ++r) {
                const int64_t m1 = by_rows ? (int64_t)r * 256 : a.M, n1 = by_rows ? a.N : (int64_t)r * 256;
                const int64_t m2 = by_rows ? a.M - m1 : a.M, n2 = by_rows ? a.N : a.N - n1;
                const double us = gemm_plan_cost_256(m1, n1, k_bytes_all, eb == 4, false, cus) + 2.0 + alone(m2, n2);
                if (us < best_us) { best_us = us; first = r; }
            }
            if (first > 0) {
                GemmArgs part = a;
                (by_rows ? part.M : part.N) = first * 256;
                if (int32_t e = gemm_mfma_tn_dispatch(in_dt, out_dt, 256, 256, 128 / eb, 8, 0, part, plan)) return e;
                part = a;
                if (by_rows) {
                    const int64_t m1 = (int64_t)first * 256;
                    part.M = a.M - (int)m1;
                    part.A = static_cast<const char*>(a.A) + m1 * a.lda * eb;
                    part.D = static_cast<char*>(a.D) + m1 * a.ldd * ob0;
                    if (a.C) part.C = static_cast<const char*>(a.C) + m1 * a.ldc_m * ob0;
                    if (a.ep_x) part.ep_x = static_cast<const char*>(a.ep_x) + m1 * a.ep_xm * dtype_bytes(a.ep_xdt);
                } else {
                    const int64_t n1 = (int64_t)first * 256;
                    part.N = a.N - (int)n1;
                    part.B = static_cast<const char*>(a.B) + n1 * a.ldb * eb;
                    part.D = static_cast<char*>(a.D) + n1 * ob0;
                    if (a.C) part.C = static_cast<const char*>(a.C) + n1 * a.ldc_n * ob0;
                    if (a.ep_x) part.ep_x = static_cast<const char*>(a.ep_x) + n1 * a.ep_xn * dtype_bytes(a.ep_xdt);
                }
                return gemm_mfma_tn_dispatch(in_dt, out_dt, 0, 0, 0, 0, 0, part, plan);
            }
        }
        bm = bn = big ? 256 : 128;
        if (bk_elems == 0) bk_elems = big || a.K % (128 / eb) == 0 ? 128 / eb : 64 / eb;
        // smaller problems: 64 x 64 tiles (four times the workgroups, no ragged form) where the cost model prices them
        // below 128 x 128 tiles for the K ranges this call runs with (gemm_plan.hpp; fp16 1024^3: 8.3 us against 10.0)
        if (!big && !majors && aligned && a.M % 64 == 0 && a.N % 64 == 0 && a.K % bk_elems == 0 && !(a.flags & kGemmAtom32) && choice.tile == 64)
            bm = bn = 64;
        if (big && waves <= 1) waves = 8;
    }
    if (bm == 0) bm = 128;
    if (bn == 0) bn = 128;
    if (bk_elems == 0) bk_elems = 64 / eb;  // 64 bytes of K per row: 32 halves / 64 fp8
    const int bkb = bk_elems * eb;
    const int ob = dtype_bytes(out_dt);
    const bool misaligned_ab = (a.lda * eb) % 16 || (a.ldb * eb) % 16 ||
                               (reinterpret_cast<uintptr_t>(a.A) | reinterpret_cast<uintptr_t>(a.B)) % 16;
    const bool misaligned_d = (a.ldd * ob) % 16 || reinterpret_cast<uintptr_t>(a.D) % 16;
    const bool misaligned = misaligned_ab || misaligned_d;
    if (bm == 256 && bn == 256) {
        if (bkb != 128 && bkb != 64)
            return fail(MOYE_ERR_UNSUPPORTED, "gemm!: the 256x256 MFMA kernels take %d or %d elements of K per tile", 64 / eb, 128 / eb);
        // the ping-pong kernel has no element-wise operations in its epilogue (the hand-ordered one has them in its
        // eight-wave whole-line form and says so itself where a caller asks for another of its schedules)
        if ((a.flags & MOYE_GEMM_PINGPONG) && a.ep_op != MOYE_MAP_IDENTITY)
            return fail(MOYE_ERR_UNSUPPORTED, "gemm!: MOYE_GEMM_PINGPONG takes no element-wise epilogue operation; leave the schedule to the library");
        const bool majors256 = a.flags & (kGemmAMajorM | kGemmBMajorN);
        // an element-wise operation: the hand-ordered kernel's eight-wave whole-line form on K-major operands
        const bool ops_fit = a.ep_op == MOYE_MAP_IDENTITY || (waves != 4 && stages < 2 && !majors256);
        // fp8 runs at twice the 16-bit rate only on the 16x16x128 MFMA, which the hand-ordered kernel issues
        if (in_dt == MOYE_F8E4M3 && bkb == 128 && stages < 3 && !(a.flags & MOYE_GEMM_PINGPONG) && ops_fit)
            a.flags |= MOYE_GEMM_WAVE4;
        // ... and for the 16-bit types its form with whole 128-byte rows in two stages is the fastest k-loop of this build
        // (fp16 4096^3 97.6-98.6 us against 101.3-102.0 for the compiler-scheduled kernel on the same box, bf16 8192^3 726
        // against 754); a K tail stays with that kernel, and so does a call that asks for it: stages = 2 in the descriptor.
        // (operands that keep their M- / N-major form: its transposing fragment reads, eight waves, plain calls; fp16 4096^3 NN
        // against the compiler-scheduled kernel's: see the kernel's header)
        if (eb == 2 && bkb == 128 && stages < 2 && ops_fit &&
            (!majors256 || (waves != 4 && !(a.flags & kGemmEpiLaneOp))) &&
            !(a.flags & (MOYE_GEMM_PINGPONG | kGemmRagged | kGemmAtom32)) && row_offsets_fit(a, 256, eb))
            a.flags |= MOYE_GEMM_WAVE4;
        // fp32 operands: the hand-ordered kernel too (fp32 8192^3 152.8 TFLOP/s on whole-line stages, 147.8 on its ring of
        // 64-byte-row stages, 142.5 for the compiler-scheduled kernel)
        if (in_dt == MOYE_F32 && stages < 2 && ops_fit && (a.ep_op == MOYE_MAP_IDENTITY || bkb == 128) && a.K % 16 == 0 &&
            (!majors256 || (waves != 4 && bkb == 128)) &&
            !(a.flags & (MOYE_GEMM_PINGPONG | kGemmRagged | kGemmAtom32)) && row_offsets_fit(a, 256, eb))
            a.flags |= MOYE_GEMM_WAVE4;
        // hand-ordered kernel: k-steps of 64 bytes, or of 128 (fp8 always; the 16-bit types when the tile says so)
        const int w4_step = in_dt == MOYE_F8E4M3 || (bkb == 128 && (eb == 2 || eb == 4)) ? 128 : 64;
        const int kmult = (a.flags & MOYE_GEMM_WAVE4) ? w4_step / eb
                          : (a.flags & MOYE_GEMM_PINGPONG) ? 64 / eb : 128 / eb;
        if (a.M % 256 || a.N % 256 || a.K % kmult)
            return fail(MOYE_ERR_SHAPE, "gemm!: CTA tile 256x256x%d does not divide the problem %dx%dx%d", kmult,
                        a.M, a.N, a.K);
        if (misaligned)
            return fail(MOYE_ERR_ALIGN, "gemm!: operands of the MFMA kernels need 16-byte aligned pointers and row pitches");
        if (a.flags & MOYE_GEMM_WAVE4) return gemm_mfma_tn_256_w4_dispatch(in_dt, out_dt, a, waves, w4_step, stages >= 3, plan);
        if (a.flags & MOYE_GEMM_PINGPONG) return gemm_mfma_tn_256_pp_dispatch(in_dt, out_dt, a, plan);
        return gemm_mfma_tn_256_dispatch(in_dt, out_dt, a, waves, stages, plan);
    }
    if (bm == 64 && bn == 64 && (bkb == 64 || bkb == 128)) {
        // small problems: four times as many workgroups as with 128 x 128 tiles (no predicated form)
        if (a.M % 64 || a.N % 64 || a.K % bk_elems)
            return fail(MOYE_ERR_SHAPE, "gemm!: CTA tile 64x64x%d does not divide the problem %dx%dx%d", bk_elems, a.M, a.N, a.K);
        if (misaligned)
            return fail(MOYE_ERR_ALIGN, "gemm!: operands of the MFMA kernels need 16-byte aligned pointers and row pitches");
        a.tiles_m = a.M / 64;
        a.tiles_n = a.N / 64;
        const bool wide64 = bkb == 128;
        switch (in_dt) {
            case MOYE_F16: return wide64 ? launch_out<InF16, 64, 64, 128>(out_dt, a, plan) : launch_out<InF16, 64, 64, 64>(out_dt, a, plan);
            case MOYE_BF16: return wide64 ? launch_out<InBF16, 64, 64, 128>(out_dt, a, plan) : launch_out<InBF16, 64, 64, 64>(out_dt, a, plan);
            case MOYE_F8E4M3: return wide64 ? launch_out<InFP8, 64, 64, 128>(out_dt, a, plan) : launch_out<InFP8, 64, 64, 64>(out_dt, a, plan);
            case MOYE_F32: return wide64 ? launch_out<InF32, 64, 64, 128>(out_dt, a, plan) : launch_out<InF32, 64, 64, 64>(out_dt, a, plan);
            default: return fail(MOYE_ERR_UNSUPPORTED, "gemm!: no MFMA atom for %s inputs", dtype_name(in_dt));
        }
    }
    // 128 x 128 tiles with 128 bytes of K per tile run on the load-to-LDS kernel (gemm_mfma128.hip) when pointers and
    // pitches are 16-byte aligned: whole tiles, or -- where residue tiles are asked for (MOYE_GEMM_PREDICATE, or the
    // tile left to the library) -- tiles that reach beyond M, N and K, which also take a D that is not 16-byte aligned.
    // The kernel below keeps 64-byte k-tiles, the 32 x 32 atoms and operands that are not aligned.
    if (bm == 128 && bn == 128 && (bkb == 128 || chosen_here) && !misaligned_ab && ((int64_t)a.K * eb) % 16 == 0) {
        const bool whole = a.M % 128 == 0 && a.N % 128 == 0 && ((int64_t)a.K * eb) % 128 == 0 && !misaligned_d;
        // (plain f16 / bf16 calls with more tiles than CUs, so that some CUs hold two workgroups: the hand-ordered kernel's
        // 128 x 128 instance, gemm_mfma256w4.hip: fp16 4096^3 on these tiles 123-124 us against 128.5-129.7, 2560^3 37.5-38.0
        // against 39.6; with one workgroup per CU, whose load stalls then nobody covers, 2048^3 23.9 against 23.5)
        // (fp8 always: only this kernel issues the 16x16x128 MFMA on 128 x 128 tiles, twice the rate of the 16x16x32 one:
        // fp8 2560^3 29.9 -> 22.1 us, 2048^3 16.9 -> 13.7, 1536^3 14.0 -> 10.8; fp32 always as well: 4096^3 on these tiles
        // 1136 -> 914 us, 2048^3 128.8 -> 122.5)
        // (operands that keep their M- / N-major form: its transposing fragment reads, every operand type)
        const bool majors128 = a.flags & (kGemmAMajorM | kGemmBMajorN);
        if (whole && (majors128 || (int64_t)(a.M / 128) * (a.N / 128) > (eb == 2 ? cus : 0)) &&
            (eb == 2 || eb == 4 || in_dt == MOYE_F8E4M3) && a.ep_op == MOYE_MAP_IDENTITY && stages < 2 &&
            !(a.flags & kGemmEpiLaneOp) && row_offsets_fit(a, 128, eb))
            return gemm_mfma_tn_128_w4_dispatch(in_dt, out_dt, a, plan);
        if (whole) return gemm_mfma_tn_128_dispatch(in_dt, out_dt, a, plan);
        if (chosen_here || (a.flags & MOYE_GEMM_PREDICATE)) {
            a.flags |= kGemmRagged;
            // (no C, no operation, more tiles than CUs: the guarded form of the hand-ordered instance, which masks a K tail in registers)
            if ((int64_t)((a.M + 127) / 128) * ((a.N + 127) / 128) > (eb == 2 ? cus : 0) &&
                (eb == 2 || eb == 4 || in_dt == MOYE_F8E4M3) && ((int64_t)a.K * eb) % 16 == 0 &&
                a.ep_op == MOYE_MAP_IDENTITY && !a.C && stages < 2 && !(a.flags & (kGemmAMajorM | kGemmBMajorN | kGemmEpiLaneOp)) &&
                row_offsets_fit(a, 128, eb))
                return gemm_mfma_tn_128_w4_dispatch(in_dt, out_dt, a, plan);
            return gemm_mfma_tn_128_dispatch(in_dt, out_dt, a, plan);
        }
    }
    // The named tile 128 x 128 with 64 bytes of K per stage (128 x 128 x 32 for the 16-bit types: the tile the baseline's fp16
    // configuration names): plain f16 / bf16 calls on whole tiles, K a whole number of two-stage k-steps, run the
    // hand-ordered kernel's ring of four such stages (fp16 4096^3 125-127 us against 161-171); the rest the register-staged kernel.
    if (bm == 128 && bn == 128 && bkb == 64 && eb == 2 && !misaligned && a.M % 128 == 0 && a.N % 128 == 0 && ((int64_t)a.K * eb) % 128 == 0 &&
        a.ep_op == MOYE_MAP_IDENTITY && stages < 2 && !(a.flags & (kGemmAMajorM | kGemmBMajorN | kGemmEpiLaneOp | kGemmAtom32 | kGemmRagged | MOYE_GEMM_PINGPONG)) &&
        row_offsets_fit(a, 128, eb))
        return gemm_mfma_tn_128_w4_dispatch(in_dt, out_dt, a, plan, true);
    if (bm != 128 || bn != 128 || (bkb != 64 && bkb != 128))
        return fail(MOYE_ERR_UNSUPPORTED,
                    "gemm!: no MFMA kernel for CTA tile %dx%dx%d (%s); built: 64x64x{%d,%d}, 128x128x{%d,%d} and 256x256x%d", bm, bn,
                    bk_elems, dtype_name(in_dt), 64 / eb, 128 / eb, 64 / eb, 128 / eb, 128 / eb);
    if (a.M % bm || a.N % bn || a.K % bk_elems) {
        // the reference's kernels assert divisibility; residue tiles are computed when the caller asks for
        // predication or leaves the tile choice to the library
        if (!chosen_here && !(a.flags & MOYE_GEMM_PREDICATE))
            return fail(MOYE_ERR_SHAPE, "gemm!: CTA tile %dx%dx%d does not divide the problem %dx%dx%d", bm, bn,
                        bk_elems, a.M, a.N, a.K);
        if (((int64_t)a.K * eb) % 16)
            return fail(MOYE_ERR_SHAPE, "gemm!: the predicated MFMA kernel needs K to be a multiple of %d elements (16 bytes), got %d",
                        16 / eb, a.K);
        if ((a.lda * eb) % 16 || (a.ldb * eb) % 16 ||
            (reinterpret_cast<uintptr_t>(a.A) | reinterpret_cast<uintptr_t>(a.B)) % 16)
            return fail(MOYE_ERR_ALIGN, "gemm!: operands of the MFMA kernels need 16-byte aligned pointers and row pitches");
        a.tiles_m = (a.M + 127) / 128;
        a.tiles_n = (a.N + 127) / 128;
        // k-tiles of 128 bytes when the library chose the tile and K is long enough to matter (half the barriers)
        const bool wide_edge = chosen_here && (int64_t)a.K * eb >= 512;
        switch (in_dt) {
            case MOYE_F16: return wide_edge ? launch_out<InF16, 128, 128, 128, true>(out_dt, a, plan) : launch_out<InF16, 128, 128, 64, true>(out_dt, a, plan);
            case MOYE_BF16: return wide_edge ? launch_out<InBF16, 128, 128, 128, true>(out_dt, a, plan) : launch_out<InBF16, 128, 128, 64, true>(out_dt, a, plan);
            case MOYE_F8E4M3: return wide_edge ? launch_out<InFP8, 128, 128, 128, true>(out_dt, a, plan) : launch_out<InFP8, 128, 128, 64, true>(out_dt, a, plan);
            case MOYE_F32: return wide_edge ? launch_out<InF32, 128, 128, 128, true>(out_dt, a, plan) : launch_out<InF32, 128, 128, 64, true>(out_dt, a, plan);
            default: return fail(MOYE_ERR_UNSUPPORTED, "gemm!: no MFMA atom for %s inputs", dtype_name(in_dt));
        }
    }
    if (misaligned)
        return fail(MOYE_ERR_ALIGN, "gemm!: operands of the MFMA kernels need 16-byte aligned pointers and row pitches");
    a.tiles_m = a.M / bm;
    a.tiles_n = a.N / bn;
    const bool wide = bkb == 128;
    switch (in_dt) {
        case MOYE_F16:
            return wide ? launch_out<InF16, 128, 128, 128>(out_dt, a, plan) : launch_out<InF16, 128, 128, 64>(out_dt, a, plan);
        case MOYE_BF16:
            return wide ? launch_out<InBF16, 128, 128, 128>(out_dt, a, plan) : launch_out<InBF16, 128, 128, 64>(out_dt, a, plan);
        case MOYE_F8E4M3:
            return wide ? launch_out<InFP8, 128, 128, 128>(out_dt, a, plan) : launch_out<InFP8, 128, 128, 64>(out_dt, a, plan);
        case MOYE_F32:
            return wide ? launch_out<InF32, 128, 128, 128>(out_dt, a, plan) : launch_out<InF32, 128, 128, 64>(out_dt, a, plan);
        default:
            return fail(MOYE_ERR_UNSUPPORTED, "gemm!: no MFMA atom for %s inputs", dtype_name(in_dt));
    }
}

}  // namespace moye

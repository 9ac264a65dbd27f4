// MFMA GEMM for a short A: at most 64 rows against a long B (N x K), K-major operands.
// The work is streaming B from HBM once, so the kernel is laid out for bandwidth, not for the matrix pipe: one workgroup
// owns 16 or 32 rows of B (that many output columns) and all of A; its four waves split K into contiguous ranges of
// whole 128-byte lines, both operands go through LDS by load-to-LDS instructions that read whole lines, and the per-wave
// partial accumulators are summed through LDS in wave order, which makes the result independent of timing.  A (at most
// 64 x K) is re-read by every workgroup and lives in L2.  bf16 16 x 8192 x 8192: 21.0 us (0.80 of the HBM peak); a
// kernel whose lanes loaded their 16-byte pieces of B straight into MFMA operand registers took 32.4 us and is gone.
// K need only be a whole number of 16-byte pieces: what is left after the last whole line is a masked trip of its own.
//
// Stands where the reference's user kernel would run gemm! (src/algorithm/blas.jl:11-131) on a
// 16-row problem with its usual 128 x 128 tiles and waste 7/8 of each tile.
#include "mfma_common.hpp"
#include "gemm_plan.hpp"

namespace moye {

// Both operands are staged through LDS by load-to-LDS instructions.
// A lane that loads straight into MFMA operand registers must address row lane % 16: neighbouring lanes then ask for
// 16 bytes each of sixteen different cache lines, and the address path of the CU handles such an instruction several
// times slower than one whose lanes read consecutive addresses (measured on such a kernel with the lanes renumbered,
// results wrong on purpose, same bytes: 32.4 us as it was, 30.2 with four lanes per 64 bytes, 29.0 with eight lanes per
// 128-byte line).  Here every instruction reads eight whole 128-byte lines (eight rows of one operand, lane l the piece
// (l % 8) ^ (l / 8) of row l / 8), the pieces land in LDS in lane order, which is the XOR-swizzled row layout that
// ds_read_b128 reads back without bank conflicts, and no operand in flight holds a register.  Each wave streams its own
// K range through its own ring of kStages buffers of 128 bytes of K, so the k-loop has no barrier.
template <typename In, typename Out, int MT, int NTW, int WAVES, int kStages, int kAuxB = 2 /* nt: B is read once */>
__global__ __launch_bounds__(WAVES * 64) void gemm_mfma_skinny_lds(GemmArgs p) {
    typedef typename Out::type OutT;
    typedef __attribute__((address_space(1))) const void* gptr_t;
    typedef __attribute__((address_space(3))) void* lptr_t;
    constexpr int ROWS = 16 * NTW + 16 * MT;  // rows of B, then the rows of A
    constexpr int LD = ROWS / 8;              // load-to-LDS instructions per stage
    constexpr int STAGE = ROWS * 8;           // in 16-byte pieces
    static_assert(LD * kStages <= 63, "vmcnt counts to 63");
    static_assert(MT * NTW * 64 <= kStages * STAGE, "the partial sums fit where the rings were");
    extern __shared__ u32x4 smem[];
    split_of_block(p);
    const int wave = threadIdx.x / 64, lane = threadIdx.x % 64, r16 = lane % 16, kq = lane / 16;
    const int n0 = blockIdx.x * 16 * NTW;
    u32x4* const ring = smem + __builtin_amdgcn_readfirstlane(wave * kStages * STAGE);

    // the waves' K ranges: whole 128-byte lines, as even as they come (a wave may get none of a very short K); what is
    // left of K after the last whole line (1 to 7 pieces of 16 bytes) is one more trip of the last wave
    const int lines = (int)(((int64_t)p.K * In::kBytes) / 128);
    const int tail_pieces = (int)((((int64_t)p.K * In::kBytes) % 128) / 16);
    const int s0 = (int)((int64_t)lines * wave / WAVES), len = (int)((int64_t)lines * (wave + 1) / WAVES) - s0;
    // M and N need not be multiples of 16: a row beyond the operand is read from the last row instead, and what is
    // computed from it is not stored
    const int lrow = lane >> 3, lch = (lane & 7) ^ (lane >> 3);
    const char* src[LD];
#pragma unroll
    for (int j = 0; j < LD; ++j) {
        const int r = 8 * j + lrow;
        src[j] = j < 2 * NTW ? static_cast<const char*>(p.B) + (int64_t)min(n0 + r, p.N - 1) * p.ldb * In::kBytes + lch * 16
                             : static_cast<const char*>(p.A) + (int64_t)min(r - 16 * NTW, p.M - 1) * p.lda * In::kBytes + lch * 16;
    }
    // fragment of k-step ks (64 bytes of K): piece 4 ks + kq of row r16 of each 16-row block
    int slot[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) slot[ks] = r16 * 8 + ((4 * ks + kq) ^ (r16 & 7));

    f32x4 acc[MT][NTW];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int t = 0; t < NTW; ++t) acc[i][t] = f32x4{0.f, 0.f, 0.f, 0.f};

    // Workgroups that walk K in the same order ask their L2 for the same lines of A at the same moment, before any of
    // them has them: a workgroup starts its walk at a line that depends on its position within its L2's share of the
    // grid.  The order of a column's k-sum follows the workgroup, not the time, so results stay reproducible.
    const int first = len > 0 ? (int)((blockIdx.x / (unsigned)p.xcds) % (unsigned)len) : 0;
    auto line_of = [&](int t) { const int r = t + first; return s0 + (r >= len ? r - len : r); };
#define MOYE_STAGE_LOAD(T)                                                                                      \
    {                                                                                                           \
        const int64_t off_ = (int64_t)line_of(T) * 128;                                                         \
        u32x4* const dst_ = ring + ((T) % kStages) * STAGE;                                                     \
        _Pragma("unroll") for (int j = 0; j < 2 * NTW; ++j)                                                     \
            __builtin_amdgcn_global_load_lds((gptr_t)(src[j] + off_), (lptr_t)(dst_ + 64 * j), 16, 0, kAuxB);   \
        _Pragma("unroll") for (int j = 2 * NTW; j < LD; ++j)                                                    \
            __builtin_amdgcn_global_load_lds((gptr_t)(src[j] + off_), (lptr_t)(dst_ + 64 * j), 16, 0, 0);       \
    }
#pragma unroll
    for (int t = 0; t < kStages - 1; ++t)
        if (t < len) MOYE_STAGE_LOAD(t)
    for (int t = 0; t < len; ++t) {
        if (t + kStages - 1 < len) {
            __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the fragment reads of trip t - 1 are out of the buffer refilled now
            MOYE_STAGE_LOAD(t + kStages - 1)
            __builtin_amdgcn_s_waitcnt((((kStages - 1) * LD) & 0xF) | ((((kStages - 1) * LD) >> 4) << 14) | 0x0F70);
        } else {
            // the tail: fewer stages are behind this one; waiting for all of them costs little over so few trips
            __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
        }
        asm volatile("" ::: "memory");
        const u32x4* const cur = ring + (t % kStages) * STAGE;
        u32x4 b[2][NTW], a[2][MT];
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
            for (int j = 0; j < NTW; ++j) b[ks][j] = cur[16 * 8 * j + slot[ks]];
#pragma unroll
            for (int i = 0; i < MT; ++i) a[ks][i] = cur[16 * 8 * (NTW + i) + slot[ks]];
        }
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)
#pragma unroll
            for (int i = 0; i < MT; ++i)
#pragma unroll
                for (int j = 0; j < NTW; ++j) In::mma(b[ks][j], a[ks][i], acc[i][j]);
        asm volatile("" ::: "memory");
    }
    // The K tail (the intent of copyto_if!, src/algorithm/copy.jl:4-16, for the last line): a lane whose 16-byte piece lies
    // beyond K reads its row's first piece instead (nothing is read past a row's end), and every fragment piece beyond K
    // is zeroed in registers, of both operands (the bytes there may be NaN or Inf), before it reaches an MFMA.
    if (tail_pieces > 0 && wave == WAVES - 1) {
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the last trip's fragment reads are out of the buffer
        const int64_t off_ = (int64_t)lines * 128 + (lch < tail_pieces ? 0 : -lch * 16);
#pragma unroll
        for (int j = 0; j < 2 * NTW; ++j) __builtin_amdgcn_global_load_lds((gptr_t)(src[j] + off_), (lptr_t)(ring + 64 * j), 16, 0, kAuxB);
#pragma unroll
        for (int j = 2 * NTW; j < LD; ++j) __builtin_amdgcn_global_load_lds((gptr_t)(src[j] + off_), (lptr_t)(ring + 64 * j), 16, 0, 0);
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
        asm volatile("" ::: "memory");
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            const bool beyond = 4 * ks + kq >= tail_pieces;
            u32x4 b[NTW], a[MT];
#pragma unroll
            for (int j = 0; j < NTW; ++j) b[j] = beyond ? u32x4{0u, 0u, 0u, 0u} : ring[16 * 8 * j + slot[ks]];
#pragma unroll
            for (int i = 0; i < MT; ++i) a[i] = beyond ? u32x4{0u, 0u, 0u, 0u} : ring[16 * 8 * (NTW + i) + slot[ks]];
#pragma unroll
            for (int i = 0; i < MT; ++i)
#pragma unroll
                for (int j = 0; j < NTW; ++j) In::mma(b[j], a[i], acc[i][j]);
        }
        asm volatile("" ::: "memory");
    }
#undef MOYE_STAGE_LOAD

    __syncthreads();  // every wave is done with its ring before the partial sums go there
    f32x4* const part = reinterpret_cast<f32x4*>(smem);  // [WAVES][MT * NTW][64]
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int t = 0; t < NTW; ++t) part[(wave * MT * NTW + i * NTW + t) * 64 + lane] = acc[i][t];
    __syncthreads();
    // lane l of tile (i, t) holds C[m = 16 i + l % 16][n = n0 + 16 t + 4 (l / 16) + 0..3]
    for (int unit = threadIdx.x; unit < MT * NTW * 64; unit += WAVES * 64) {
        const int it = unit / 64, l = unit % 64;
        f32x4 v = part[unit];
#pragma unroll
        for (int w = 1; w < WAVES; ++w) v += part[w * MT * NTW * 64 + unit];
        const int m = 16 * (it / NTW) + l % 16, n = n0 + 16 * (it % NTW) + 4 * (l / 16);
        if (m >= p.M) continue;
        const int64_t sn = p.ldd_n ? p.ldd_n : 1;  // D may have its unit stride along m
        OutT* d = static_cast<OutT*>(p.D) + (int64_t)m * p.ldd + (int64_t)n * sn;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            if (n + e >= p.N) continue;
            const float c = p.C ? Out::load(p.C, (int64_t)m * p.ldc_m + (int64_t)(n + e) * p.ldc_n) : 0.f;
            d[e * sn] = Out::cvt(epi_value(p, v[e], p.C != nullptr, c, m, n + e));
        }
    }
}

constexpr int kSkinnyLdsWaves = 4;
static_assert(kSkinnyLineBytes == 128, "the host decides about K ranges by this");
template <typename In, typename Out, int MT, int W, int NTW, int S, int AUX>
static int32_t launch_skinny_lds_v(const GemmArgs& a, GemmPlan& plan) {
    constexpr int kLds = W * S * (16 * NTW + 16 * MT) * 128;
    static LdsCap cap;
    plan.add_kernel(gemm_mfma_skinny_lds<In, Out, MT, NTW, W, S, AUX>, a, (unsigned)((a.N + 16 * NTW - 1) / (16 * NTW)), (unsigned)(a.split > 1 ? a.split : 1),
                    W * 64, kLds, &cap, 0, 16 * NTW, 128, In::kDt, Out::kDt, "gemm_mfma_skinny_lds<%s,%s,mt=%d,ntw=%d,waves=%d,stages=%d>", In::kName, Out::kName,
                    MT, NTW, W, S);
    return MOYE_OK;
}
template <typename In, typename Out>
static int32_t launch_skinny_lds(const GemmArgs& a, GemmPlan& plan) {
    constexpr int W = kSkinnyLdsWaves;
    // Waves x buffers, bf16 16 x 8192 x 8192, 32 rows of B per workgroup: 8 x 3 27.2 us, 8 x 2 25.2, 4 x 2 21.2, 4 x 3 21.0,
    // 4 x 4 21.2, 2 x 4 21.0, 2 x 3 22.6, 1 x 8 30.0; 64 rows per workgroup (half as many workgroups as CUs) 28.0-30.1;
    // B without the non-temporal hint 23.6.  As with the transposes, less in flight is faster on this part, down to what
    // covers the latency.  32 rows per workgroup once that gives every CU one (bf16, K = 8192: N = 16384 40.1 us against
    // 45.3 with 16 rows; N = 4096 17.9 against 13.5).
    // (which of them: gemm_short_m_ntw, gemm_plan.hpp -- the rounds the workgroups of a launch need on the CUs decide)
    const int ranges = a.split > 1 ? a.split : 1;
    const int ntw = gemm_short_m_ntw(a.M, a.N, (int64_t)a.K * In::kBytes * ranges, plan.shape.cus, ranges);
    // (64 rows: two buffers instead of three, for the LDS; from 33 rows of A on, where every workgroup's reads of all of A
    // out of the L2s weigh most: bf16 64 x 28672 x 8192 118.8 us with 32 rows, 95.3 with 64)
    if (ntw == 4)
        return (a.M + 15) / 16 == 3 ? launch_skinny_lds_v<In, Out, 3, W, 4, 2, 2>(a, plan) : launch_skinny_lds_v<In, Out, 4, W, 4, 2, 2>(a, plan);
    if (ntw == 2) {
        switch ((a.M + 15) / 16) {
            case 1: return launch_skinny_lds_v<In, Out, 1, W, 2, 3, 2>(a, plan);
            case 2: return launch_skinny_lds_v<In, Out, 2, W, 2, 3, 2>(a, plan);
            case 3: return launch_skinny_lds_v<In, Out, 3, W, 2, 3, 2>(a, plan);
            default: return launch_skinny_lds_v<In, Out, 4, W, 2, 3, 2>(a, plan);
        }
    }
    switch ((a.M + 15) / 16) {
        case 1: return launch_skinny_lds_v<In, Out, 1, W, 1, 3, 2>(a, plan);
        case 2: return launch_skinny_lds_v<In, Out, 2, W, 1, 3, 2>(a, plan);
        case 3: return launch_skinny_lds_v<In, Out, 3, W, 1, 3, 2>(a, plan);
        default: return launch_skinny_lds_v<In, Out, 4, W, 1, 3, 2>(a, plan);
    }
}

template <typename In>
static int32_t launch_skinny_out(int32_t out_dt, const GemmArgs& a, GemmPlan& plan) {
    switch (out_dt) {
        case MOYE_F32: return launch_skinny_lds<In, OutF32>(a, plan);
        case MOYE_F16: return launch_skinny_lds<In, OutF16>(a, plan);
        case MOYE_BF16: return launch_skinny_lds<In, OutBF16>(a, plan);
        default: return fail(MOYE_ERR_UNSUPPORTED, "gemm!: MFMA kernels write f32, f16 or bf16, not %s", dtype_name(out_dt));
    }
}

// 1 <= M <= 64, any N, K a multiple of 16 bytes; pointers and pitches 16-byte aligned.
int32_t gemm_mfma_skinny_dispatch(int32_t in_dt, int32_t out_dt, const GemmArgs& a, GemmPlan& plan) {
    const int eb = dtype_bytes(in_dt);
    if (a.M < 1 || a.M > 64 || a.N < 1 || a.K < 1 || ((int64_t)a.K * eb) % 16)
        return fail(MOYE_ERR_SHAPE, "gemm!: the short-M MFMA kernel needs 1 <= M <= 64 and K %% %d == 0, got %dx%dx%d",
                    16 / eb, a.M, a.N, a.K);
    if ((a.lda * eb) % 16 || (a.ldb * eb) % 16 ||
        (reinterpret_cast<uintptr_t>(a.A) | reinterpret_cast<uintptr_t>(a.B)) % 16)
        return fail(MOYE_ERR_ALIGN, "gemm!: operands of the MFMA kernels need 16-byte aligned pointers and row pitches");
    switch (in_dt) {
        case MOYE_F16: return launch_skinny_out<InF16>(out_dt, a, plan);
        case MOYE_BF16: return launch_skinny_out<InBF16>(out_dt, a, plan);
        case MOYE_F8E4M3: return launch_skinny_out<InFP8>(out_dt, a, plan);
        case MOYE_F32: return launch_skinny_out<InF32>(out_dt, a, plan);
        default: return fail(MOYE_ERR_UNSUPPORTED, "gemm!: no MFMA atom for %s inputs", dtype_name(in_dt));
    }
}

}  // namespace moye

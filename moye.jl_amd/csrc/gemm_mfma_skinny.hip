// MFMA GEMM for a short A: at most 64 rows against a long B (N x K), K-major operands.
// The work is streaming B from HBM once, so the kernel is laid out for bandwidth, not for the
// matrix pipe: one workgroup owns 16 or 32 rows of B (that many output columns) and all of A; its waves split
// K into contiguous ranges, each lane streams 16-byte pieces of its B row straight into the MFMA
// operand registers (no LDS staging: nothing is reused inside a workgroup), and the per-wave
// partial accumulators are summed through LDS in wave order, which makes the result independent
// of timing.  A (at most 64 x K) is re-read by every workgroup and lives in L2; with 32 rows of B
// per workgroup each A fragment feeds two MFMAs, which halves that L2 traffic (measured 33 us
// against 38 us at 16 x 8192 x 8192 bf16; the bare B stream alone takes 22 us).  More requests in flight make it
// slower, not faster (same case, waves per workgroup x k-steps in flight per wave: 8 x 4 32.4 us, 4 x 8 34.3, 8 x 8 38.8,
// 16 x 2 39.9, 16 x 4 41.5, 8 x 16 55.1): the kernel is not short of memory-level parallelism.
//
// Stands where the reference's user kernel would run gemm! (src/algorithm/blas.jl:11-131) on a
// 16-row problem with its usual 128 x 128 tiles and waste 7/8 of each tile.
#include "mfma_common.hpp"

namespace moye {

template <typename In, typename Out, int MT, int NTW, int WAVES, int U = 4 /* 64-byte k-steps in flight per wave and row */>
__global__ __launch_bounds__(WAVES * 64) void gemm_mfma_skinny(GemmArgs p) {
    typedef typename Out::type OutT;
    split_of_block(p);
    __shared__ f32x4 part[WAVES][MT * NTW][64];
    const int wave = threadIdx.x / 64, lane = threadIdx.x % 64, r16 = lane % 16, kq = lane / 16;
    const int n0 = blockIdx.x * 16 * NTW;
    const int steps = (int)(((int64_t)p.K * In::kBytes) / 64);
    const int s0 = (int)((int64_t)steps * wave / WAVES), s1 = (int)((int64_t)steps * (wave + 1) / WAVES);
    // M and N need not be multiples of 16: a lane whose row lies beyond the operand reads the last row instead, and
    // what it computes is not stored
    const char* bp[NTW];
#pragma unroll
    for (int t = 0; t < NTW; ++t)
        bp[t] = static_cast<const char*>(p.B) + (int64_t)min(n0 + 16 * t + r16, p.N - 1) * p.ldb * In::kBytes + kq * 16;
    const char* ap[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i)
        ap[i] = static_cast<const char*>(p.A) + (int64_t)min(16 * i + r16, p.M - 1) * p.lda * In::kBytes + kq * 16;
    f32x4 acc[MT][NTW];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int t = 0; t < NTW; ++t) acc[i][t] = f32x4{0.f, 0.f, 0.f, 0.f};

    // Every workgroup needs all of A, and workgroups that walk K in the same order ask the L2 for the same lines of A
    // at the same moment, before any of them has them.  So a workgroup starts its walk at a step that depends on
    // its position within its L2's share of the grid (consecutive workgroups go to consecutive L2s), in units of U
    // steps so that a trip still covers whole 128-byte lines of B (measured at 16 x 8192 x 8192 bf16: 146 MiB
    // fetched instead of 161, 32.9 us instead of 34.0).  The order of a column's k-sum follows the workgroup, not
    // the time, so results stay reproducible.
    const int len = s1 - s0;
    const int first = len >= U && len % U == 0 ? U * (int)((blockIdx.x / 8) % (unsigned)(len / U)) : 0;
    auto step_of = [&](int t) { const int r = t + first; return s0 + (r >= len ? r - len : r); };
    int t0 = 0;
    for (; t0 + U <= len; t0 += U) {
        u32x4 b[NTW][U], a[MT][U];
        int64_t off[U];
#pragma unroll
        for (int u = 0; u < U; ++u) off[u] = (int64_t)step_of(t0 + u) * 64;
#pragma unroll
        for (int t = 0; t < NTW; ++t)
#pragma unroll
            for (int u = 0; u < U; ++u)
                b[t][u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(bp[t] + off[u]));
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int u = 0; u < U; ++u) a[i][u] = *reinterpret_cast<const u32x4*>(ap[i] + off[u]);
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int i = 0; i < MT; ++i)
#pragma unroll
                for (int t = 0; t < NTW; ++t) In::mma(b[t][u], a[i][u], acc[i][t]);
    }
    for (; t0 < len; ++t0) {
        const int64_t off = (int64_t)step_of(t0) * 64;
#pragma unroll
        for (int i = 0; i < MT; ++i) {
            const u32x4 a = *reinterpret_cast<const u32x4*>(ap[i] + off);
#pragma unroll
            for (int t = 0; t < NTW; ++t)
                In::mma(__builtin_nontemporal_load(reinterpret_cast<const u32x4*>(bp[t] + off)), a, acc[i][t]);
        }
    }

#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int t = 0; t < NTW; ++t) part[wave][i * NTW + t][lane] = acc[i][t];
    __syncthreads();
    // lane l of tile (i, t) holds C[m = 16 i + l % 16][n = n0 + 16 t + 4 (l / 16) + 0..3]
    for (int unit = threadIdx.x; unit < MT * NTW * 64; unit += WAVES * 64) {
        const int it = unit / 64, l = unit % 64;
        f32x4 v = part[0][it][l];
#pragma unroll
        for (int w = 1; w < WAVES; ++w) v += part[w][it][l];
        const int m = 16 * (it / NTW) + l % 16, n = n0 + 16 * (it % NTW) + 4 * (l / 16);
        if (m >= p.M) continue;
        const int64_t sn = p.ldd_n ? p.ldd_n : 1;  // D may have its unit stride along m (a column-major D, or the
                                                   // right-hand fringe of a large problem computed as its transpose)
        OutT* d = static_cast<OutT*>(p.D) + (int64_t)m * p.ldd + (int64_t)n * sn;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            if (n + e >= p.N) continue;
            const float c = p.C ? Out::load(p.C, (int64_t)m * p.ldc_m + (int64_t)(n + e) * p.ldc_n) : 0.f;
            d[e * sn] = Out::cvt(epi_value(p, v[e], p.C != nullptr, c, m, n + e));
        }
    }
}

template <typename In, typename Out>
static int32_t launch_skinny(const GemmArgs& a, hipStream_t st) {
    constexpr int W = 8;
    const dim3 block(W * 64);
    // With K split over two or more workgroups there are enough workgroups to give each one 64 rows of B: A, which every
    // workgroup reads whole (its K range of it), then crosses the L2-to-CU path half as often.  Pays from M = 33 on
    // (bf16 64 x 8192 x 8192: 44.8 us with two K ranges, the second pass included, against 52.5 unsplit; M = 48: 41.3
    // against 55.3); without the split the larger workgroup tile is slower (68.8 us).
    if (a.split > 1 && a.M > 32 && a.N % 64 == 0 && a.N / 64 >= 128) {
        const dim3 grid((unsigned)(a.N / 64), (unsigned)(a.split > 1 ? a.split : 1));
        if ((a.M + 15) / 16 == 3) gemm_mfma_skinny<In, Out, 3, 4, W><<<grid, block, 0, st>>>(a);
        else gemm_mfma_skinny<In, Out, 4, 4, W><<<grid, block, 0, st>>>(a);
        MOYE_HIP_CHECK(hipGetLastError());
        return MOYE_OK;
    }
    if (a.N % 32 == 0 && a.N / 32 >= 256) {  // two B tiles per wave once that still fills the chip
        const dim3 grid((unsigned)(a.N / 32), (unsigned)(a.split > 1 ? a.split : 1));
        switch ((a.M + 15) / 16) {
            case 1: gemm_mfma_skinny<In, Out, 1, 2, W><<<grid, block, 0, st>>>(a); break;
            case 2: gemm_mfma_skinny<In, Out, 2, 2, W><<<grid, block, 0, st>>>(a); break;
            case 3: gemm_mfma_skinny<In, Out, 3, 2, W><<<grid, block, 0, st>>>(a); break;
            default: gemm_mfma_skinny<In, Out, 4, 2, W><<<grid, block, 0, st>>>(a); break;
        }
    } else {
        const dim3 grid((unsigned)((a.N + 15) / 16), (unsigned)(a.split > 1 ? a.split : 1));
        switch ((a.M + 15) / 16) {
            case 1: gemm_mfma_skinny<In, Out, 1, 1, W><<<grid, block, 0, st>>>(a); break;
            case 2: gemm_mfma_skinny<In, Out, 2, 1, W><<<grid, block, 0, st>>>(a); break;
            case 3: gemm_mfma_skinny<In, Out, 3, 1, W><<<grid, block, 0, st>>>(a); break;
            default: gemm_mfma_skinny<In, Out, 4, 1, W><<<grid, block, 0, st>>>(a); break;
        }
    }
    MOYE_HIP_CHECK(hipGetLastError());
    return MOYE_OK;
}

template <typename In>
static int32_t launch_skinny_out(int32_t out_dt, const GemmArgs& a, hipStream_t st) {
    switch (out_dt) {
        case MOYE_F32: return launch_skinny<In, OutF32>(a, st);
        case MOYE_F16: return launch_skinny<In, OutF16>(a, st);
        case MOYE_BF16: return launch_skinny<In, OutBF16>(a, st);
        default: return fail(MOYE_ERR_UNSUPPORTED, "gemm!: MFMA kernels write f32, f16 or bf16, not %s", dtype_name(out_dt));
    }
}

// 1 <= M <= 64, any N, K a multiple of 64 bytes; pointers and pitches 16-byte aligned.
int32_t gemm_mfma_skinny_dispatch(int32_t in_dt, int32_t out_dt, const GemmArgs& a, hipStream_t st) {
    const int eb = dtype_bytes(in_dt);
    if (a.M < 1 || a.M > 64 || a.N < 1 || ((int64_t)a.K * eb) % 64)
        return fail(MOYE_ERR_SHAPE, "gemm!: the short-M MFMA kernel needs 1 <= M <= 64 and K %% %d == 0, got %dx%dx%d",
                    64 / eb, a.M, a.N, a.K);
    if ((a.lda * eb) % 16 || (a.ldb * eb) % 16 ||
        (reinterpret_cast<uintptr_t>(a.A) | reinterpret_cast<uintptr_t>(a.B)) % 16)
        return fail(MOYE_ERR_ALIGN, "gemm!: operands of the MFMA kernels need 16-byte aligned pointers and row pitches");
    switch (in_dt) {
        case MOYE_F16: return launch_skinny_out<InF16>(out_dt, a, st);
        case MOYE_BF16: return launch_skinny_out<InBF16>(out_dt, a, st);
        case MOYE_F8E4M3: return launch_skinny_out<InFP8>(out_dt, a, st);
        case MOYE_F32: return launch_skinny_out<InF32>(out_dt, a, st);
        default: return fail(MOYE_ERR_UNSUPPORTED, "gemm!: no MFMA atom for %s inputs", dtype_name(in_dt));
    }
}

}  // namespace moye

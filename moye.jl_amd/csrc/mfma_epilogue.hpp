// Epilogue shared by the MFMA GEMM kernels: alpha * acc + C -> OutT (round to nearest even,
// the conversion rule of src/arch/copy/copy.jl:38-43) -> the wave's own LDS patch -> 128-bit row
// stores.  The reference's kernels store accumulator fragments straight to global memory in
// fragment order (test/device/matmul.jl:51); going through LDS turns that into full-row writes.
#pragma once

#include "mfma_common.hpp"

namespace moye {

// acc[i][j] of a lane holds C[m = 16 i + lane % 16][n = 16 j + 4 (lane / 16) + e], e = 0..3,
// relative to (m_base, n_base).  `smem` must be free of operand data for all waves.
template <typename Out, int MI, int NI>
__device__ __forceinline__ void store_c_tile(const GemmArgs& p, const f32x4 (&acc)[MI][NI], u32x4* smem, int wave,
                                             int lane, int64_t m_base, int64_t n_base) {
    typedef typename Out::type OutT;
    constexpr int WN = NI * 16;
    constexpr int EPC = 16 / (int)sizeof(OutT);  // elements per 16-byte chunk
    constexpr int CR = WN / EPC;                 // chunks per patch row
    constexpr int PASS_MI = 2, PASS_ROWS = PASS_MI * 16;
    const int r16 = lane & 15, kq = lane >> 4;
    OutT* patch = reinterpret_cast<OutT*>(smem) + wave * (PASS_ROWS * WN);
    u32x4* patch16 = reinterpret_cast<u32x4*>(patch);
    // C with unit stride along n and 16-byte aligned rows (kGemmRowC, decided on the host) comes in the way D goes
    // out: 128-bit pieces of whole rows, through the patch, where each lane then finds its own four values.  The
    // pieces of the next AHEAD - 1 passes are already requested while a pass is worked on.  Any other C is read
    // element by element.
    constexpr int NCH = PASS_ROWS * CR / 64, PASSES = MI / PASS_MI;
    constexpr int AHEAD = sizeof(OutT) == 2 ? PASSES : (PASSES < 2 ? PASSES : 2);
    const bool row_c = p.C && (p.xcd_swizzle & kGemmRowC);
    u32x4 cw[AHEAD][NCH];
    auto fetch_c = [&](int pass, u32x4 (&into)[NCH]) __attribute__((always_inline)) {
#pragma unroll
        for (int t = 0; t < NCH; ++t) {
            const int c = lane + 64 * t, row = c / CR, ch = c % CR;
            into[t] = *reinterpret_cast<const u32x4*>(static_cast<const char*>(p.C) +
                                                      ((m_base + PASS_ROWS * pass + row) * p.ldc_m + n_base) * (int64_t)sizeof(OutT) + ch * 16);
        }
    };
    if (row_c) {
#pragma unroll
        for (int a = 0; a < AHEAD; ++a) fetch_c(a, cw[a]);
    }
#pragma unroll
    for (int i0 = 0; i0 < MI; i0 += PASS_MI) {
        if (row_c) {
            const int pass = i0 / PASS_MI;
#pragma unroll
            for (int t = 0; t < NCH; ++t) {
                const int c = lane + 64 * t, row = c / CR, ch = c % CR;
                patch16[row * CR + (ch ^ (row & 7))] = cw[pass % AHEAD][t];
            }
            if (pass + AHEAD < PASSES) fetch_c(pass + AHEAD, cw[pass % AHEAD]);
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }
#pragma unroll
        for (int ii = 0; ii < PASS_MI; ++ii) {
            const int i = i0 + ii;
#pragma unroll
            for (int j = 0; j < NI; ++j) {
                float v[4] = {acc[i][j].x * p.alpha, acc[i][j].y * p.alpha, acc[i][j].z * p.alpha,
                              acc[i][j].w * p.alpha};
                const int row = 16 * ii + r16, col = 16 * j + 4 * kq;
                const int chunk = col / EPC, within = col % EPC;
                OutT* dst = patch + (row * CR + (chunk ^ (row & 7))) * EPC + within;
                if (row_c) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] += Out::load(dst, e);
                } else if (p.C) {
                    const int64_t m = m_base + 16 * i + r16, n = n_base + 16 * j + 4 * kq;
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] += Out::load(p.C, m * p.ldc_m + (n + e) * p.ldc_n);
                }
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
            store_d_chunk(p, d, w);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
}

}  // namespace moye

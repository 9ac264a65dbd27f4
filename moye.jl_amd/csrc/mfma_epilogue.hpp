// Epilogue shared by the MFMA GEMM kernels: alpha * acc + C -> OutT (round to nearest even,
// the conversion rule of src/arch/copy/copy.jl:38-43) -> the wave's own LDS patch -> 128-bit row
// stores.  The reference's kernels store accumulator fragments straight to global memory in
// fragment order (test/device/matmul.jl:51); going through LDS turns that into full-row writes.
#pragma once

#include "mfma_common.hpp"

namespace moye {

// The same tile with an element-wise operation in the epilogue (GemmArgs::ep_op other than the identity).  The raw fp32
// accumulators go through the wave's LDS patch, 32 rows at a time; the lanes then read them back along rows, apply
// epi_value() (alpha, beta * C, the operation with its operand), convert and store 16-byte pieces.  The arithmetic
// exists once, in a loop over the passes that is not unrolled: unrolled over all accumulators it would be several
// thousand instructions per kernel.  `smem`: 32 x WN floats per wave.
// kGuard: the tile may reach beyond M or N, and D need not be 16-byte aligned; rows beyond M are skipped, a piece that
// crosses N is read and stored element by element up to N, and so is a piece of D that does not start on a 16-byte
// boundary (a pitch of D that is not a multiple of 16 bytes).
// AT: the MFMA tile (16 or 32; see store_c_tile).
template <typename Out, int MI, int NI, bool kGuard = false, int AT = 16>
__device__ __forceinline__ void store_c_tile_general(const GemmArgs& p, const float __attribute__((ext_vector_type(AT * AT / 64))) (&acc)[MI][NI],
                                                     u32x4* smem, int wave, int lane, int64_t m_base, int64_t n_base) {
    typedef typename Out::type OutT;
    constexpr int WN = NI * AT, PASS_MI = 32 / AT, PASS_ROWS = 32, PASSES = MI / PASS_MI, G = AT * AT / 256;
    constexpr int EPC = 16 / (int)sizeof(OutT);  // elements per 16-byte piece of D
    constexpr int CR = WN / 4;                   // 16-byte chunks of floats per patch row
    constexpr int OUT_CH = PASS_ROWS * (WN / EPC);  // 16-byte pieces of D per pass
    static_assert(CR >= 8 && OUT_CH % 64 == 0, "patch shape");
    const int r16 = lane % AT, kq = lane / AT;
    float* patch = reinterpret_cast<float*>(smem) + wave * (PASS_ROWS * WN);
    f32x4* patch16 = reinterpret_cast<f32x4*>(patch);
#pragma unroll 1
    for (int pass = 0; pass < PASSES; ++pass) {
        // accumulators of rows 32 pass .. 32 pass + 31 -> patch (the only part that names registers, hence the static index)
#pragma unroll
        for (int ps = 0; ps < PASSES; ++ps) {
            if (pass != ps) continue;
#pragma unroll
            for (int ii = 0; ii < PASS_MI; ++ii)
#pragma unroll
                for (int j = 0; j < NI; ++j)
#pragma unroll
                    for (int g = 0; g < G; ++g) {
                        const int row = AT * ii + r16, chunk = (AT / 4) * j + 2 * g + kq;
                        const auto& a = acc[ps * PASS_MI + ii][j];
                        patch16[row * CR + (chunk ^ (row & 7))] = f32x4{a[4 * g], a[4 * g + 1], a[4 * g + 2], a[4 * g + 3]};
                    }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll 1
        for (int t = 0; t < OUT_CH / 64; ++t) {
            const int c = lane + 64 * t, row = c / (WN / EPC), och = c % (WN / EPC);
            const int64_t m = m_base + PASS_ROWS * pass + row, n0 = n_base + och * EPC;
            if (kGuard && (m >= p.M || n0 >= p.N)) continue;
            const bool whole = !kGuard || n0 + EPC <= p.N;  // else only the first N - n0 elements exist
            char* const d16 = static_cast<char*>(p.D) + (m * p.ldd + n0) * (int64_t)sizeof(OutT);
            const bool store16 = whole && (!kGuard || (reinterpret_cast<uintptr_t>(d16) & 15) == 0);
            float v[EPC], x[EPC];
#pragma unroll
            for (int q = 0; q < EPC / 4; ++q) {
                const int chunk = och * (EPC / 4) + q;
                const f32x4 a = patch16[row * CR + (chunk ^ (row & 7))];
#pragma unroll
                for (int e = 0; e < 4; ++e) v[4 * q + e] = __fmul_rn(a[e], p.alpha);
            }
            // beta * C: a 16-byte piece of the row where C allows it (kGemmRowC), element by element otherwise
            if (p.C) {
                if ((p.flags & kGemmRowC) && whole) {
                    OutT cw[EPC];
                    const u32x4 w = *reinterpret_cast<const u32x4*>(static_cast<const char*>(p.C) + (m * p.ldc_m + n0) * (int64_t)sizeof(OutT));
                    __builtin_memcpy(cw, &w, 16);
#pragma unroll
                    for (int e = 0; e < EPC; ++e) v[e] = __fadd_rn(v[e], __fmul_rn(p.beta, Out::load(cw, e)));
                } else {
#pragma unroll
                    for (int e = 0; e < EPC; ++e)
                        if (whole || n0 + e < p.N) v[e] = __fadd_rn(v[e], __fmul_rn(p.beta, Out::load(p.C, m * p.ldc_m + (n0 + e) * p.ldc_n)));
                }
            }
            // the operand: a scalar, one value per row, a 16-byte piece (or two) of a row, or element by element
            if (!p.ep_x) {
#pragma unroll
                for (int e = 0; e < EPC; ++e) x[e] = p.ep_scalar;
            } else if (p.ep_xn == 0) {
                const float xr = epi_operand(p, m, 0);
#pragma unroll
                for (int e = 0; e < EPC; ++e) x[e] = xr;
            } else if ((p.flags & kGemmEpiRowX) && whole) {
                if (p.ep_xdt == MOYE_F32) {
                    const f32x4* xp = reinterpret_cast<const f32x4*>(static_cast<const float*>(p.ep_x) + m * p.ep_xm + n0);
#pragma unroll
                    for (int q = 0; q < EPC / 4; ++q) {
                        const f32x4 w = xp[q];
#pragma unroll
                        for (int e = 0; e < 4; ++e) x[4 * q + e] = w[e];
                    }
                } else {  // D's 16-bit type
                    OutT xw[EPC];
                    const u32x4 w = *reinterpret_cast<const u32x4*>(static_cast<const char*>(p.ep_x) + (m * p.ep_xm + n0) * (int64_t)sizeof(OutT));
                    __builtin_memcpy(xw, &w, 16);
#pragma unroll
                    for (int e = 0; e < EPC; ++e) x[e] = Out::load(xw, e);
                }
            } else {
#pragma unroll
                for (int e = 0; e < EPC; ++e) x[e] = whole || n0 + e < p.N ? epi_operand(p, m, n0 + e) : 0.f;
            }
            OutT out[EPC];
            switch (p.ep_op) {  // the operation is the same for every element: one branch per piece, not per element
#define MOYE_EPI_CASE(OP)                                                                              \
    case OP:                                                                                           \
        _Pragma("unroll") for (int e = 0; e < EPC; ++e) out[e] = Out::cvt(epi_op(OP, v[e], x[e]));     \
        break;
                MOYE_EPI_CASE(MOYE_MAP_ADD)
                MOYE_EPI_CASE(MOYE_MAP_SUB)
                MOYE_EPI_CASE(MOYE_MAP_MUL)
                MOYE_EPI_CASE(MOYE_MAP_DIV)
                MOYE_EPI_CASE(MOYE_MAP_MAX)
                MOYE_EPI_CASE(MOYE_MAP_MIN)
                MOYE_EPI_CASE(MOYE_MAP_NEG)
                MOYE_EPI_CASE(MOYE_MAP_ABS)
#undef MOYE_EPI_CASE
                default:
#pragma unroll
                    for (int e = 0; e < EPC; ++e) out[e] = Out::cvt(v[e]);
            }
            if (store16) {
                u32x4 w;
                __builtin_memcpy(&w, out, 16);
                store_d_chunk(p, d16, w);
            } else if (kGuard && whole && (reinterpret_cast<uintptr_t>(d16) & 7) == 0) {
                // a whole piece on an 8-byte boundary (a row pitch of 8 bytes modulo 16 puts every other row there)
                u32x2 h[2];
                __builtin_memcpy(h, out, 16);
                reinterpret_cast<u32x2*>(d16)[0] = h[0];
                reinterpret_cast<u32x2*>(d16)[1] = h[1];
            } else {
                OutT* d = static_cast<OutT*>(p.D) + m * p.ldd + n0;
#pragma unroll
                for (int e = 0; e < EPC; ++e)
                    if (whole || n0 + e < p.N) d[e] = out[e];
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
}

// acc[i][j] of a lane holds C[m = 16 i + lane % 16][n = 16 j + 4 (lane / 16) + e], e = 0..3,
// relative to (m_base, n_base); with the 32 x 32 MFMA tiles (AT = 32) its sixteen values are
// C[m = 32 i + lane % 32][n = 32 j + 8 g + 4 (lane / 32) + e], g = 0..3.  `smem` must be free of operand data for all waves.
// No element-wise operation here: a call with one runs an instance whose epilogue is store_c_tile_general alone (the host
// decides; the hand-ordered kernel has no such instance and is never sent one).
// kGuard: the tile may reach beyond M or N and D need not be 16-byte aligned: nothing is read or stored beyond them, a
// piece of D that crosses N or does not start on a 16-byte boundary goes out element by element.
// kLaneOp: the call's element-wise operation has a one-per-column, one-per-row or scalar operand or none, and is no
// division (kGemmEpiLaneOp: a bias, a ReLU, a scale): the lanes apply it to their own accumulators here, with the same
// roundings as the general epilogue, instead of sending the tile through it.
// kNoC: the caller has no C (GemmArgs::C is null, checked on the host): nothing of C's two read paths is compiled in,
// which frees their registers for instances that have few to spare.
// PR: rows of the wave tile per pass through the patch (32, or 16 where only half the room is there).
template <typename Out, int MI, int NI, bool kGuard = false, bool kLaneOp = false, bool kNoC = false, int AT = 16, int PR = 32>
__device__ __forceinline__ void store_c_tile(const GemmArgs& p, const float __attribute__((ext_vector_type(AT * AT / 64))) (&acc)[MI][NI], u32x4* smem,
                                             int wave, int lane, int64_t m_base, int64_t n_base) {
    typedef typename Out::type OutT;
    constexpr int WN = NI * AT, G = AT * AT / 256;  // G: groups of four consecutive n per lane and MFMA tile
    constexpr int EPC = 16 / (int)sizeof(OutT);  // elements per 16-byte chunk
    constexpr int CR = WN / EPC;                 // chunks per patch row
    static_assert(PR % AT == 0 && MI % (PR / AT) == 0, "whole MFMA tiles per pass");
    constexpr int PASS_MI = PR / AT, PASS_ROWS = PASS_MI * AT;
    const int r16 = lane % AT, kq = lane / AT;
    OutT* patch = reinterpret_cast<OutT*>(smem) + wave * (PASS_ROWS * WN);
    u32x4* patch16 = reinterpret_cast<u32x4*>(patch);
    // C with unit stride along n and 16-byte aligned rows (kGemmRowC, decided on the host) comes in the way D goes
    // out: 128-bit pieces of whole rows, through the patch, where each lane then finds its own four values.  The
    // pieces of the next AHEAD - 1 passes are already requested while a pass is worked on.  Any other C is read
    // element by element.
    constexpr int NCH = PASS_ROWS * CR / 64, PASSES = MI / PASS_MI;
    // (an instance that also applies an operation in the lanes has fewer registers to spare: one pass ahead)
    constexpr int AHEAD = kLaneOp ? 1 : sizeof(OutT) == 2 ? PASSES : (PASSES < 2 ? PASSES : 2);
    // (ragged tiles read C in whole pieces only when no piece crosses N)
    const bool row_c = !kNoC && p.C && (p.flags & kGemmRowC) && (!kGuard || p.N % EPC == 0);
    [[maybe_unused]] u32x4 cw[kNoC ? 1 : AHEAD][NCH];
    auto fetch_c = [&](int pass, u32x4 (&into)[NCH]) __attribute__((always_inline)) {
#pragma unroll
        for (int t = 0; t < NCH; ++t) {
            const int c = lane + 64 * t, row = c / CR, ch = c % CR;
            if (kGuard && (m_base + PASS_ROWS * pass + row >= p.M || n_base + ch * EPC >= p.N)) {
                into[t] = u32x4{0u, 0u, 0u, 0u};
                continue;
            }
            into[t] = *reinterpret_cast<const u32x4*>(static_cast<const char*>(p.C) +
                                                      ((m_base + PASS_ROWS * pass + row) * p.ldc_m + n_base) * (int64_t)sizeof(OutT) + ch * 16);
        }
    };
    if constexpr (!kNoC) {
        if (row_c) {
#pragma unroll
            for (int a = 0; a < AHEAD; ++a) fetch_c(a, cw[a]);
        }
    }
    // a lane's columns are n_base + AT j + 8 g + 4 kq + 0..3: the operand values of a one-per-column vector, once for all rows
    [[maybe_unused]] f32x4 xcol[kLaneOp ? NI * G : 1];
    [[maybe_unused]] const bool per_row = kLaneOp && p.ep_x && p.ep_xn == 0;
    if constexpr (kLaneOp) {
#pragma unroll
        for (int j = 0; j < NI * G; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e) xcol[j][e] = per_row ? 0.f : epi_operand(p, 0, n_base + AT * (j / G) + 8 * (j % G) + 4 * kq + e);
    }
#pragma unroll
    for (int i0 = 0; i0 < MI; i0 += PASS_MI) {
        if constexpr (!kNoC) {
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
        }
#pragma unroll
        for (int ii = 0; ii < PASS_MI; ++ii) {
            const int i = i0 + ii;
#pragma unroll
            for (int jg = 0; jg < NI * G; ++jg) {
                const int j = jg / G, g = jg % G;
                const int row = AT * ii + r16, col = AT * j + 8 * g + 4 * kq;
                const int chunk = col / EPC, within = col % EPC;
                OutT* dst = patch + (row * CR + (chunk ^ (row & 7))) * EPC + within;
                const int64_t m = m_base + AT * i + r16, n = n_base + col;
                [[maybe_unused]] float c[4] = {0.f, 0.f, 0.f, 0.f};
                if constexpr (!kNoC) {
                    if (row_c) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) c[e] = Out::load(dst, e);
                    } else if (p.C) {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            if (!kGuard || (m < p.M && n + e < p.N)) c[e] = Out::load(p.C, m * p.ldc_m + (n + e) * p.ldc_n);
                    }
                }
                float v[4] = {__fmul_rn(acc[i][j][4 * g], p.alpha), __fmul_rn(acc[i][j][4 * g + 1], p.alpha), __fmul_rn(acc[i][j][4 * g + 2], p.alpha),
                              __fmul_rn(acc[i][j][4 * g + 3], p.alpha)};
                if constexpr (!kNoC) {
                    if (p.C) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) v[e] = __fadd_rn(v[e], __fmul_rn(p.beta, c[e]));
                    }
                }
                if constexpr (kLaneOp) {
                    const float xrow = per_row ? epi_operand(p, m, 0) : 0.f;
                    // the same for every element: one uniform branch per four values; the addition (a bias) and the
                    // maximum (a ReLU) are asked first, so that they pay one or two compares and not a chain of them
#define MOYE_LANE_APPLY(OP) _Pragma("unroll") for (int e = 0; e < 4; ++e) v[e] = epi_op(OP, v[e], per_row ? xrow : xcol[jg][e]);
#define MOYE_LANE_CASE(OP) \
    case OP:               \
        MOYE_LANE_APPLY(OP) \
        break;
                    if (p.ep_op == MOYE_MAP_ADD) {
                        MOYE_LANE_APPLY(MOYE_MAP_ADD)
                    } else if (p.ep_op == MOYE_MAP_MAX) {
                        MOYE_LANE_APPLY(MOYE_MAP_MAX)
                    } else {
                        switch (p.ep_op) {
                            MOYE_LANE_CASE(MOYE_MAP_SUB)
                            MOYE_LANE_CASE(MOYE_MAP_MUL)
                            MOYE_LANE_CASE(MOYE_MAP_MIN)
                            MOYE_LANE_CASE(MOYE_MAP_NEG)
                            MOYE_LANE_CASE(MOYE_MAP_ABS)
                            default: break;
                        }
                    }
#undef MOYE_LANE_CASE
#undef MOYE_LANE_APPLY
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
                      ((m_base + AT * i0 + row) * p.ldd + n_base) * (int64_t)sizeof(OutT) + ch * 16;
            if constexpr (kGuard) {
                const int64_t m = m_base + AT * i0 + row, n0 = n_base + ch * EPC;
                if (m >= p.M || n0 >= p.N) continue;
                if (n0 + EPC <= p.N && (reinterpret_cast<uintptr_t>(d) & 15) == 8) {
                    // a whole piece on an 8-byte boundary (a row pitch of 8 bytes modulo 16 puts every other row there)
                    reinterpret_cast<u32x2*>(d)[0] = u32x2{w.x, w.y};
                    reinterpret_cast<u32x2*>(d)[1] = u32x2{w.z, w.w};
                    continue;
                }
                if (n0 + EPC > p.N || (reinterpret_cast<uintptr_t>(d) & 15)) {
                    OutT o[EPC];
                    __builtin_memcpy(o, &w, 16);
#pragma unroll
                    for (int e = 0; e < EPC; ++e)
                        if (n0 + e < p.N) reinterpret_cast<OutT*>(d)[e] = o[e];
                    continue;
                }
            }
            store_d_chunk(p, d, w);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
}

}  // namespace moye

// gemm! with the UniversalFMA atom on the device, arithmetic identical to the reference's:
//   d = (a * b) + c          (src/arch/mma/mma.jl:64, via src/traits/mma.jl:49-68)
// with `a * b` rounded in promote_type(TA, TB), the sum rounded in the accumulator type, never
// contracted into an fma, and k running ascending so every C element is the strict
// left-to-right sum the reference's loop nest produces (src/algorithm/blas.jl:63-67,83-85 inside
// the k-tile loop of test/device/matmul.jl:40-49).  The m/n visiting order and the CTA tile
// cannot change any element, so results are bit-identical to the CPU restatement for every
// tiling.  Any strides, any sizes (edges are predicated).
//
// This file is compiled with -ffp-contract=off.
#include "kernels.hpp"

namespace moye {

// (a NaN stays as it is; everything else through v_cvt_pk_bf16_f32, round to nearest even)
__device__ __forceinline__ float u_bf16_round(float f) {
    if (f != f) return f;
    return __uint_as_float((uint32_t)__builtin_bit_cast(uint16_t, (__bf16)f) << 16);
}

__device__ __forceinline__ float u_load(const void* p, int64_t i, int dt) {
    switch (dt) {
        case MOYE_F32: return static_cast<const float*>(p)[i];
        case MOYE_F16: return (float)static_cast<const _Float16*>(p)[i];
        default: return __uint_as_float((uint32_t)static_cast<const uint16_t*>(p)[i] << 16);  // bf16
    }
}

__device__ __forceinline__ void u_store(void* p, int64_t i, int dt, float v) {
    switch (dt) {
        case MOYE_F32: static_cast<float*>(p)[i] = v; break;
        case MOYE_F16: static_cast<_Float16*>(p)[i] = (_Float16)v; break;
        default: static_cast<uint16_t*>(p)[i] = (uint16_t)(__float_as_uint(u_bf16_round(v)) >> 16); break;
    }
}

// kProd / kAcc: 0 = fp32, 1 = fp16, 2 = bf16 — the type the product / the running sum is rounded in
template <int kT>
__device__ __forceinline__ float round_in(float x) {
    if constexpr (kT == 1) return (float)(_Float16)x;
    else if constexpr (kT == 2) return u_bf16_round(x);
    else return x;
}

template <int BM, int BN, int BK, int TM, int TN, int kProd, int kAcc>
__global__ __launch_bounds__(256) void gemm_universal_fma(UArgs p) {
    static_assert((BM / TM) * (BN / TN) == 256, "256 threads per workgroup");
    __shared__ float sA[BK][BM + 1];
    __shared__ float sB[BK][BN + 1];
    const int tid = threadIdx.x;
    const int m0 = blockIdx.x * BM, n0 = blockIdx.y * BN;
    constexpr int TX = BM / TM, TY = BN / TN;
    const int tx = tid % TX, ty = tid / TX;

    float acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int m = m0 + tx + TX * i, n = n0 + ty + TY * j;
            acc[i][j] = (p.C && p.alpha == 1.0f && m < p.M && n < p.N)
                            ? u_load(p.C, m * p.sc_m + n * p.sc_n, p.c_dt) : 0.0f;
        }

    const bool a_kfast = p.sa_k == 1, b_kfast = p.sb_k == 1;
    // Operand stages go global -> registers -> LDS, and the registers of stage t+1 are filled while stage t is
    // multiplied: a small problem (few workgroups per CU) would otherwise wait out one global round trip per stage.
    constexpr int LA = (BM * BK + 255) / 256, LB = (BN * BK + 255) / 256;
    float ra[LA], rb[LB];
    auto fetch = [&](int k0) {
        const int kmax = min(BK, p.K - k0);
#pragma unroll
        for (int q = 0; q < LA; ++q) {
            const int idx = tid + 256 * q;
            const int m = a_kfast ? idx / BK : idx % BM, k = a_kfast ? idx % BK : idx / BM;
            ra[q] = 0.0f;
            if (idx < BM * BK && m0 + m < p.M && k < kmax) ra[q] = u_load(p.A, (int64_t)(m0 + m) * p.sa_m + (int64_t)(k0 + k) * p.sa_k, p.a_dt);
        }
#pragma unroll
        for (int q = 0; q < LB; ++q) {
            const int idx = tid + 256 * q;
            const int n = b_kfast ? idx / BK : idx % BN, k = b_kfast ? idx % BK : idx / BN;
            rb[q] = 0.0f;
            if (idx < BN * BK && n0 + n < p.N && k < kmax) rb[q] = u_load(p.B, (int64_t)(n0 + n) * p.sb_n + (int64_t)(k0 + k) * p.sb_k, p.b_dt);
        }
    };
    auto stash = [&]() {
#pragma unroll
        for (int q = 0; q < LA; ++q) {
            const int idx = tid + 256 * q;
            const int m = a_kfast ? idx / BK : idx % BM, k = a_kfast ? idx % BK : idx / BM;
            if (idx < BM * BK) sA[k][m] = ra[q];
        }
#pragma unroll
        for (int q = 0; q < LB; ++q) {
            const int idx = tid + 256 * q;
            const int n = b_kfast ? idx / BK : idx % BN, k = b_kfast ? idx % BK : idx / BN;
            if (idx < BN * BK) sB[k][n] = rb[q];
        }
    };
    auto k_step = [&](int k) {
        float a[TM], b[TN];
#pragma unroll
        for (int i = 0; i < TM; ++i) a[i] = sA[k][tx + TX * i];
#pragma unroll
        for (int j = 0; j < TN; ++j) b[j] = sB[k][ty + TY * j];
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const float prod = round_in<kProd>(__fmul_rn(a[i], b[j]));
                acc[i][j] = round_in<kAcc>(__fadd_rn(prod, acc[i][j]));
            }
    };
    if (p.K > 0) {
        fetch(0);
        stash();
    }
    __syncthreads();
    for (int k0 = 0; k0 < p.K; k0 += BK) {
        const int kmax = min(BK, p.K - k0);
        const bool more = k0 + BK < p.K;
        if (more) fetch(k0 + BK);  // in flight during the arithmetic below
        if (kmax == BK && TM * TN <= 4) {
            // a whole stage of a small thread tile: the fragments of eight k are read from LDS before the first product, so
            // that one LDS latency is paid per eight k, not per k (there may be a single wave per SIMD to hide it)
#pragma unroll
            for (int kb = 0; kb < BK; kb += 8) {
                float a[8][TM], b[8][TN];
#pragma unroll
                for (int k = 0; k < 8; ++k) {
#pragma unroll
                    for (int i = 0; i < TM; ++i) a[k][i] = sA[kb + k][tx + TX * i];
#pragma unroll
                    for (int j = 0; j < TN; ++j) b[k][j] = sB[kb + k][ty + TY * j];
                }
#pragma unroll
                for (int k = 0; k < 8; ++k)
#pragma unroll
                    for (int i = 0; i < TM; ++i)
#pragma unroll
                        for (int j = 0; j < TN; ++j) {
                            const float prod = round_in<kProd>(__fmul_rn(a[k][i], b[k][j]));
                            acc[i][j] = round_in<kAcc>(__fadd_rn(prod, acc[i][j]));
                        }
            }
        } else if (kmax == BK) {   // a whole stage: unrolled, so that the LDS reads of later k are in flight under the arithmetic
#pragma unroll
            for (int k = 0; k < BK; ++k) k_step(k);
        } else {
            for (int k = 0; k < kmax; ++k) k_step(k);
        }
        __syncthreads();           // everybody is done reading this stage
        if (more) {
            stash();
            __syncthreads();
        }
    }

#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int m = m0 + tx + TX * i, n = n0 + ty + TY * j;
            if (m < p.M && n < p.N) {
                float v = acc[i][j];
                if (p.alpha != 1.0f) {
                    v = __fmul_rn(p.alpha, v);
                    if (p.C) v = __fadd_rn(v, u_load(p.C, m * p.sc_m + n * p.sc_n, p.c_dt));
                }
                u_store(p.D, m * p.sd_m + n * p.sd_n, p.d_dt, v);
            }
        }
}

template <int BM, int BN, int BK, int TM, int TN>
static int32_t launch_u(const UArgs& a, int prod, int accT, hipStream_t st) {
    const dim3 grid((a.M + BM - 1) / BM, (a.N + BN - 1) / BN);
#define MOYE_U(P, Q) gemm_universal_fma<BM, BN, BK, TM, TN, P, Q><<<grid, 256, 0, st>>>(a)
    if (prod == 0 && accT == 0) MOYE_U(0, 0);
    else if (prod == 1 && accT == 0) MOYE_U(1, 0);
    else if (prod == 2 && accT == 0) MOYE_U(2, 0);
    else if (prod == 1 && accT == 1) MOYE_U(1, 1);
    else if (prod == 2 && accT == 2) MOYE_U(2, 2);
    else return fail(MOYE_ERR_UNSUPPORTED, "gemm!: UniversalFMA has no kernel for this type combination");
#undef MOYE_U
    MOYE_HIP_CHECK(hipGetLastError());
    return MOYE_OK;
}

static int type_class(int dt) { return dt == MOYE_F16 ? 1 : dt == MOYE_BF16 ? 2 : 0; }

int32_t gemm_universal_dispatch(int bm, int bn, int bk, UArgs a, hipStream_t st) {
    for (int dt : {a.a_dt, a.b_dt, a.d_dt, a.C ? a.c_dt : MOYE_F32})
        if (dt != MOYE_F32 && dt != MOYE_F16 && dt != MOYE_BF16)
            return fail(MOYE_ERR_UNSUPPORTED, "gemm!: UniversalFMA kernels take f32, f16 or bf16, not %s", dtype_name(dt));
    // promote_type(TA, TB): the narrow type only when both operands have it
    const int prod = type_class(a.a_dt) == type_class(a.b_dt) ? type_class(a.a_dt) : 0;
    // the running sum lives in the accumulator type TC == TD
    const int accT = type_class(a.d_dt);
    if (accT != 0 && accT != prod)
        return fail(MOYE_ERR_UNSUPPORTED, "gemm!: a %s accumulator needs %s operands", dtype_name(a.d_dt), dtype_name(a.d_dt));
    if (a.C && a.c_dt != a.d_dt)
        return fail(MOYE_ERR_UNSUPPORTED, "gemm!: C and D must have the same element type");
    if (bm == 0 && bn == 0) {
        // measured, fp32: 1024^3 runs at 21.0 / 11.8 / 5.0 TFLOP/s on 32 / 64 / 128 tiles, 2048^3 at 28.0 / 36.5 / 20.3,
        // 4096^3 at 29.9 / 39.3 / 40.1 (every tile gives the same bits: k ascends strictly whatever the tile)
        const bool small = (int64_t)a.M * a.N <= 1024 * 1024;
        bm = bn = small ? 32 : 64;
    }
    if (bk == 0) bk = 8;
    // bK of the caller's tile is how many k the reference's kernel stages per trip; the sum over k is strictly ascending
    // whatever that number is, so the 32 x 32 tile, which small problems use with few waves per CU, stages 32 per trip (one
    // global round trip and one barrier pair per 32 k: fp32 256^3 17 us instead of 20, 1024^3 102 instead of 112)
    if (bm == 32 && bn == 32 && bk == 8) return launch_u<32, 32, 32, 2, 2>(a, prod, accT, st);
    if (bm == 32 && bn == 32 && bk == 8) return launch_u<32, 32, 8, 2, 2>(a, prod, accT, st);
    if (bm == 64 && bn == 64 && bk == 8) return launch_u<64, 64, 8, 4, 4>(a, prod, accT, st);
    if (bm == 128 && bn == 128 && bk == 8) return launch_u<128, 128, 8, 8, 8>(a, prod, accT, st);
    return fail(MOYE_ERR_UNSUPPORTED, "gemm!: UniversalFMA CTA tile %dx%dx%d not built (32x32x8, 64x64x8, 128x128x8)", bm, bn, bk);
}

}  // namespace moye

// Argument blocks and dispatch entry points shared by the kernel translation units and capi.hip.
#pragma once

#include "moye_common.hpp"

namespace moye {

// MFMA GEMM, K-major operands, N-contiguous output (gemm_mfma.hip)
struct GemmArgs {
    const void* A;  // (M,K), K contiguous, row pitch lda elements
    const void* B;  // (N,K), K contiguous, row pitch ldb
    const void* C;  // (M,N) or null, element strides ldc_m / ldc_n, dtype of D
    void* D;        // (M,N), N contiguous, row pitch ldd
    int M, N, K;
    int64_t lda, ldb, ldc_m, ldc_n, ldd;
    int64_t ldd_n;  // stride of D along n; 0 = contiguous.  Only the short-M kernel takes another value.
    float alpha;
    // the rest of the epilogue (moye_gemm_epilogue): D = op(alpha * acc + beta * C, x), see epi_value() in mfma_common.hpp
    float beta;        // applied to C; the host passes C = nullptr when beta == 0
    int ep_op;         // MOYE_MAP_*; MOYE_MAP_IDENTITY = none
    int ep_xdt;        // element type of ep_x: MOYE_F32, MOYE_F16 or MOYE_BF16
    float ep_scalar;   // second argument of op when ep_x is null
    const void* ep_x;  // (M,N) operand of op, element strides ep_xm / ep_xn (0 = repeated along that mode)
    int64_t ep_xm, ep_xn;
    int tiles_m, tiles_n;
    // split-K: gridDim.y ranges of K in one launch; range y reads A and B split_ab bytes further along their rows
    // and writes its product split_d bytes further (compact fp32 partial products, one after the other)
    int split;
    int64_t split_ab, split_d;
    int xcd_swizzle;  // bit 0: XCD-aware tile order; bits 8-15: MOYE_GEMM_* schedule flags; kGemmAtom32
};
constexpr int kGemmAtom32 = 0x10000;   // in GemmArgs::xcd_swizzle: issue the 32x32 MFMA forms
constexpr int kGemmRowC = 0x80000;    // in GemmArgs::xcd_swizzle: C has unit stride along n, 16-byte aligned rows: read in 128-bit pieces
constexpr int kGemmStreamD = 0x40000;  // in GemmArgs::xcd_swizzle: D is written with non-temporal stores
constexpr int kGemmAMajorM = 0x100000;  // in GemmArgs::xcd_swizzle: A has its unit stride along M, lda is the pitch between consecutive k
constexpr int kGemmBMajorN = 0x200000;  // the same for B and N (the 256 x 256 kernel's transposing fragment reads; 16-bit types)
constexpr int kGemmEpiRowX = 0x400000;  // in GemmArgs::xcd_swizzle: the epilogue operand has unit stride along n and 16-byte aligned rows (or one row)
constexpr int kGemmRagged = 0x800000;   // in GemmArgs::xcd_swizzle: the 256 x 256 kernel runs with tiles that reach beyond M, N or K (its guarded instance)
constexpr int kGemmEpiAddVec = 0x1000000;  // in GemmArgs::xcd_swizzle: the epilogue operation adds a one-per-column or one-per-row vector or a scalar
constexpr int kGemmRotateK = 0x20000;  // in GemmArgs::xcd_swizzle: each XCD starts its walk over K at its own eighth

// UniversalFMA GEMM, any strides (gemm_universal.hip)
struct UArgs {
    const void* A; const void* B; const void* C; void* D;
    int M, N, K;
    int64_t sa_m, sa_k, sb_n, sb_k, sc_m, sc_n, sd_m, sd_n;
    float alpha;
    int a_dt, b_dt, c_dt, d_dt;
};

int32_t copy_dispatch(const moye_tiled_copy* tc, const moye_tensor* dst, const moye_tensor* src, hipStream_t st);
int32_t copy_if_dispatch(const moye_tiled_copy* tc, const moye_tensor* dst, const moye_tensor* src, const moye_tensor* mask,
                         hipStream_t st);
int32_t gemm_mfma_tn_dispatch(int32_t in_dt, int32_t out_dt, int bm, int bn, int bk_elems, int waves, int stages,
                              GemmArgs a, hipStream_t st);
int32_t gemm_mfma_tn_256_dispatch(int32_t in_dt, int32_t out_dt, GemmArgs a, int waves, int stages, hipStream_t st);
int32_t gemm_mfma_tn_256_pp_dispatch(int32_t in_dt, int32_t out_dt, GemmArgs a, hipStream_t st);
int32_t gemm_mfma_tn_128_w4_dispatch(int32_t in_dt, int32_t out_dt, GemmArgs a, hipStream_t st);
int32_t gemm_mfma_tn_256_w4_dispatch(int32_t in_dt, int32_t out_dt, GemmArgs a, int waves, int kstep_bytes, bool ring, hipStream_t st);
int32_t gemm_mfma_tn_128_dispatch(int32_t in_dt, int32_t out_dt, GemmArgs a, hipStream_t st);
int32_t gemm_mfma_skinny_dispatch(int32_t in_dt, int32_t out_dt, const GemmArgs& a, hipStream_t st);
// The short-M kernel stages whole 128-byte lines of K through LDS, four waves with a K range each, when K is this many
// bytes or a multiple of it (else every lane loads its own 16-byte pieces).
constexpr int kSkinnyLineBytes = 128;
int32_t axpby_dispatch(double a, const moye_tensor* X, double b, const moye_tensor* Y, hipStream_t st);
int32_t fill_dispatch(const moye_tensor* X, double value, hipStream_t st);
int32_t map_dispatch(int32_t op, const moye_tensor* D, const moye_tensor* A, const moye_tensor* B, double scalar, hipStream_t st);
// sums the `split` partial products in P in ascending order and applies the epilogue of `e` (alpha, beta, op and operand;
// C with strides ldc_m / ldc_n; D with strides ldd / ldd_n), M x N elements
int32_t splitk_reduce_dispatch(const float* P, int split, int64_t M, int64_t N, const GemmArgs& e, int32_t out_dt, hipStream_t st);
int32_t mfma_ceiling(int32_t in_dt, int32_t random_operands, float seconds, float* tflops, float* clock_ghz, hipStream_t st);
int32_t gemm_universal_dispatch(int bm, int bn, int bk, UArgs a, hipStream_t st);

}  // namespace moye

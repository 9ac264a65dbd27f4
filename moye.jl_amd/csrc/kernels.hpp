// Argument blocks and dispatch entry points shared by the kernel translation units and capi.hip.
#pragma once

#include <vector>

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
    int flags;  // bit 0: XCD-aware tile order; bits 8-15: the MOYE_GEMM_* schedule flags of the descriptor; the kGemm* bits below
    int xcds;   // how many XCDs the hardware deals consecutive workgroup ids to (DeviceShape::xcds): the tile order and the K rotation count with it
};
// bits of GemmArgs::flags that the host sets for the kernels (the descriptor's own flags occupy bits 0-15)
constexpr int kGemmAtom32 = 0x10000;   // issue the 32x32 MFMA forms
constexpr int kGemmRotateK = 0x20000;  // each XCD starts its walk over K at its own share of K
constexpr int kGemmStreamD = 0x40000;  // D is written with non-temporal stores
constexpr int kGemmRowC = 0x80000;     // C has unit stride along n, 16-byte aligned rows: read in 128-bit pieces
constexpr int kGemmAMajorM = 0x100000;  // A has its unit stride along M, lda is the pitch between consecutive k
constexpr int kGemmBMajorN = 0x200000;  // the same for B and N (the kernels' transposing fragment reads)
constexpr int kGemmEpiRowX = 0x400000;  // the epilogue operand has unit stride along n and 16-byte aligned rows (or one row)
constexpr int kGemmRagged = 0x800000;   // tiles reach beyond M, N or K (the guarded instances)
constexpr int kGemmEpiLaneOp = 0x1000000;  // the epilogue operation (not a division) has a scalar, a one-per-column or a one-per-row operand, or none: a bias, a ReLU, a scale

// UniversalFMA GEMM, any strides (gemm_universal.hip)
struct UArgs {
    const void* A; const void* B; const void* C; void* D;
    int M, N, K;
    int64_t sa_m, sa_k, sb_n, sb_k, sc_m, sc_n, sd_m, sd_n;
    float alpha;
    int a_dt, b_dt, c_dt, d_dt;
};

// What the host needs to know of the chip to choose tiles: compute units, and the XCDs that consecutive workgroup ids are
// dealt to (32 CUs each on gfx950; a partitioned part shows fewer of both).  Read once per device; 256 / 8 when there is
// no device to ask (planning on a host without a GPU).
struct DeviceShape {
    int cus, xcds;
};
DeviceShape device_shape();
// `cus` > 0 overrides what the device says, for planning (moye_gemm_explain) and its tests
DeviceShape device_shape_for(int cus);

// The load-to-LDS kernels address operand rows as a uniform base plus a 32-bit lane offset: `rows` rows of either
// operand must span less than 4 GiB.
inline bool row_offsets_fit(const GemmArgs& a, int rows, int elem_bytes) {
    return (int64_t)rows * a.lda * elem_bytes < ((int64_t)1 << 32) && (int64_t)rows * a.ldb * elem_bytes < ((int64_t)1 << 32);
}

// ---- a gemm! call as a list of launches ---------------------------------------------------------------------------
// The host code that chooses kernels (capi.hip: gemm_plan_build; gemm_mfma.hip and the kernel files' dispatch functions)
// launches nothing: it appends steps to a GemmPlan.  gemm_plan_run (capi.hip) then enqueues them on a stream, and
// moye_gemm_explain prints them.  Building a plan touches no device, so it runs, and is tested, on hosts without one.
struct GemmStep {
    enum Kind { kKernel, kKMajorCopy, kSplitKReduce, kUniversal } kind = kKernel;
    // kKernel: one launch of an MFMA kernel instance
    char name[160] = {0};              // kernel function and template arguments, e.g. gemm_mfma_tn_256_w4<W4F16L,OutF16,waves=8>
    void (*kernel)(GemmArgs) = nullptr;
    GemmArgs args{};
    unsigned grid_x = 0, grid_y = 1, block = 0;
    int lds_bytes = 0;
    struct LdsCap* cap = nullptr;      // set when the kernel needs its dynamic-LDS cap raised (once per device)
    int tile_m = 0, tile_n = 0, tile_k_bytes = 0;  // CTA tile of the instance (0: the short-M kernels, which have none)
    int in_dt = 0, out_dt = 0;
    // kKMajorCopy: src (rows x cols with the unit stride along rows) -> dst (cols contiguous), through moye_copy's kernels
    moye_tensor copy_dst{}, copy_src{};
    // kSplitKReduce: sums `split` fp32 partial products of M x N in args.D's place (P) and applies the epilogue of `args`
    const float* partials = nullptr;
    int split = 0;
    // kUniversal: the UniversalFMA kernel on CTA tile (ubm, ubn, ubk)
    UArgs uargs{};
    int ubm = 0, ubn = 0, ubk = 0;
};
struct GemmPlan {
    std::vector<GemmStep> steps;
    DeviceShape shape{256, 8};
    size_t workspace_bytes = 0;  // what the steps use of the workspace (K-major operand copies, then split-K partial products)
    char* workspace = nullptr;   // where it is
    // appends a kernel launch; `name` is printf-style
    GemmStep& add_kernel(void (*kernel)(GemmArgs), const GemmArgs& a, unsigned grid_x, unsigned grid_y, unsigned block, int lds_bytes,
                         struct LdsCap* cap, int tile_m, int tile_n, int tile_k_bytes, int in_dt, int out_dt, const char* fmt, ...)
        __attribute__((format(printf, 14, 15)));
};
int32_t copy_dispatch(const moye_tiled_copy* tc, const moye_tensor* dst, const moye_tensor* src, hipStream_t st);
int32_t copy_if_dispatch(const moye_tiled_copy* tc, const moye_tensor* dst, const moye_tensor* src, const moye_tensor* mask,
                         hipStream_t st);
// The functions below choose kernel instances and append them to `plan`; none of them launches.
struct TileChoice;  // gemm_plan.hpp
int32_t gemm_mfma_tn_dispatch(int32_t in_dt, int32_t out_dt, int bm, int bn, int bk_elems, int waves, int stages,
                              GemmArgs a, GemmPlan& plan, const TileChoice* lib = nullptr);
int32_t gemm_mfma_tn_256_dispatch(int32_t in_dt, int32_t out_dt, GemmArgs a, int waves, int stages, GemmPlan& plan);
int32_t gemm_mfma_tn_256_pp_dispatch(int32_t in_dt, int32_t out_dt, GemmArgs a, GemmPlan& plan);
int32_t gemm_mfma_tn_256_atom32_dispatch(int32_t in_dt, int32_t out_dt, GemmArgs a, GemmPlan& plan);
int32_t gemm_mfma_tn_128_w4_dispatch(int32_t in_dt, int32_t out_dt, GemmArgs a, GemmPlan& plan, bool stage64 = false);
int32_t gemm_mfma_tn_256_w4_dispatch(int32_t in_dt, int32_t out_dt, GemmArgs a, int waves, int kstep_bytes, bool ring, GemmPlan& plan);
int32_t gemm_mfma_tn_128_dispatch(int32_t in_dt, int32_t out_dt, GemmArgs a, GemmPlan& plan);
int32_t gemm_mfma_skinny_dispatch(int32_t in_dt, int32_t out_dt, const GemmArgs& a, GemmPlan& plan);
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

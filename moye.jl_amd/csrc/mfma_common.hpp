// Element traits, LDS swizzle and tile mapping shared by the MFMA GEMM kernels.
#pragma once

#include "kernels.hpp"

namespace moye {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));

// ---- input element traits: how one pair of 16-byte chunks feeds the MFMA pipe ----------------
struct InF16 {
    static constexpr int kBytes = 2, kDt = MOYE_F16;
    static constexpr const char* kName = "InF16";
    static __device__ __forceinline__ void mma(const u32x4& a, const u32x4& b, f32x4& c) {
        c = __builtin_amdgcn_mfma_f32_16x16x32_f16((f16x8)a, (f16x8)b, c, 0, 0, 0);
    }
    // the 32x32x16 form: 32 rows per operand, a lane's chunk is half of a 32-byte piece of its row
    static __device__ __forceinline__ void mma32(const u32x4& a, const u32x4& b, f32x16& c) {
        c = __builtin_amdgcn_mfma_f32_32x32x16_f16((f16x8)a, (f16x8)b, c, 0, 0, 0);
    }
    // accumulator pinned in the AccVGPR file: its reads and write-backs then stay off the
    // ArchVGPR ports that the LDS fragment loads are writing through
    static __device__ __forceinline__ void mma_acc(const u32x4& a, const u32x4& b, f32x4& c) {
        asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
    }
};
struct InBF16 {
    static constexpr int kBytes = 2, kDt = MOYE_BF16;
    static constexpr const char* kName = "InBF16";
    static __device__ __forceinline__ void mma(const u32x4& a, const u32x4& b, f32x4& c) {
        c = __builtin_amdgcn_mfma_f32_16x16x32_bf16((bf16x8)a, (bf16x8)b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ void mma32(const u32x4& a, const u32x4& b, f32x16& c) {
        c = __builtin_amdgcn_mfma_f32_32x32x16_bf16((bf16x8)a, (bf16x8)b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ void mma_acc(const u32x4& a, const u32x4& b, f32x4& c) {
        asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
    }
};
// A 16-byte chunk holds 16 fp8 values = the k-slices of two MFMAs.  Both operands split the
// chunk the same way, so the pairing of products is unchanged.
struct InFP8 {
    static constexpr int kBytes = 1, kDt = MOYE_F8E4M3;
    static constexpr const char* kName = "InFP8";
    static __device__ __forceinline__ void mma(const u32x4& a, const u32x4& b, f32x4& c) {
        const long a0 = (long)(((uint64_t)a.y << 32) | a.x), a1 = (long)(((uint64_t)a.w << 32) | a.z);
        const long b0 = (long)(((uint64_t)b.y << 32) | b.x), b1 = (long)(((uint64_t)b.w << 32) | b.z);
        c = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(a0, b0, c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(a1, b1, c, 0, 0, 0);
    }
    static __device__ __forceinline__ void mma32(const u32x4& a, const u32x4& b, f32x16& c) {
        const long a0 = (long)(((uint64_t)a.y << 32) | a.x), a1 = (long)(((uint64_t)a.w << 32) | a.z);
        const long b0 = (long)(((uint64_t)b.y << 32) | b.x), b1 = (long)(((uint64_t)b.w << 32) | b.z);
        c = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(a0, b0, c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(a1, b1, c, 0, 0, 0);
    }
    static __device__ __forceinline__ void mma_acc(const u32x4& a, const u32x4& b, f32x4& c) {
        const u32x2 a0 = {a.x, a.y}, a1 = {a.z, a.w}, b0 = {b.x, b.y}, b1 = {b.z, b.w};
        asm volatile("v_mfma_f32_16x16x32_fp8_fp8 %0, %1, %2, %0" : "+a"(c) : "v"(a0), "v"(b0));
        asm volatile("v_mfma_f32_16x16x32_fp8_fp8 %0, %1, %2, %0" : "+a"(c) : "v"(a1), "v"(b1));
    }
};

// A 16-byte chunk holds 4 fp32 values of one row: element j of every lane's chunk goes to MFMA j, so
// MFMA j multiplies the k-slices {j, 4+j, 8+j, 12+j} of a 64-byte row piece; A and B are cut the
// same way, so every product a[m][k] * b[n][k] is formed exactly once.
struct InF32 {
    static constexpr int kBytes = 4, kDt = MOYE_F32;
    static constexpr const char* kName = "InF32";
    static __device__ __forceinline__ void mma(const u32x4& a, const u32x4& b, f32x4& c) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
            c = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(a[j]), __uint_as_float(b[j]), c, 0, 0, 0);
    }
    static __device__ __forceinline__ void mma32(const u32x4& a, const u32x4& b, f32x16& c) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
            c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a[j]), __uint_as_float(b[j]), c, 0, 0, 0);
    }
    static __device__ __forceinline__ void mma_acc(const u32x4& a, const u32x4& b, f32x4& c) { mma(a, b, c); }
};

// ---- output element traits: fp32 -> OutT, round to nearest even (src/arch/copy/copy.jl:38-43) ---
struct OutF32 {
    typedef float type;
    static constexpr int kDt = MOYE_F32;
    static constexpr const char* kName = "OutF32";
    static __device__ __forceinline__ float cvt(float x) { return x; }
    static __device__ __forceinline__ float load(const void* p, int64_t i) { return static_cast<const float*>(p)[i]; }
};
struct OutF16 {
    typedef _Float16 type;
    static constexpr int kDt = MOYE_F16;
    static constexpr const char* kName = "OutF16";
    static __device__ __forceinline__ _Float16 cvt(float x) { return (_Float16)x; }
    static __device__ __forceinline__ float load(const void* p, int64_t i) { return (float)static_cast<const _Float16*>(p)[i]; }
};
struct OutBF16 {
    typedef uint16_t type;
    static constexpr int kDt = MOYE_BF16;
    static constexpr const char* kName = "OutBF16";
    // v_cvt_pk_bf16_f32: round to nearest even, a NaN keeps its sign and upper payload bits and becomes quiet.  Checked on
    // the hardware over all 2^32 inputs against the integer form (add 0x7fff + the lowest kept bit, shift; NaN: shift, set
    // bit 6), which costs six instructions an element where this costs half of one.
    static __device__ __forceinline__ uint16_t cvt(float x) { return __builtin_bit_cast(uint16_t, (__bf16)x); }
    static __device__ __forceinline__ float load(const void* p, int64_t i) {
        return __uint_as_float((uint32_t)static_cast<const uint16_t*>(p)[i] << 16);
    }
};

// ---- the epilogue's arithmetic on one element (include/moye_hip.h, moye_gemm_epilogue) -------------------------------
// What the reference's user kernels do to the accumulator fragment after the k-loop: axpby! (src/algorithm/blas.jl:1-9)
// and one broadcast operation (src/broadcast.jl:5-41), in fp32, every operation rounded on its own (the intrinsics keep
// the compiler from contracting a product and a sum into one fused operation, which Julia does not do either).
__device__ __forceinline__ float epi_operand(const GemmArgs& p, int64_t m, int64_t n) {
    if (!p.ep_x) return p.ep_scalar;
    const int64_t i = m * p.ep_xm + n * p.ep_xn;
    switch (p.ep_xdt) {
        case MOYE_F16: return (float)static_cast<const _Float16*>(p.ep_x)[i];
        case MOYE_BF16: return __uint_as_float((uint32_t)static_cast<const uint16_t*>(p.ep_x)[i] << 16);
        default: return static_cast<const float*>(p.ep_x)[i];
    }
}
// max / min follow Julia: NaN if either argument is NaN, -0.0 < +0.0 (as moye_map)
__device__ __forceinline__ float epi_op(int op, float x, float y) {
    switch (op) {
        case MOYE_MAP_ADD: return __fadd_rn(x, y);
        case MOYE_MAP_SUB: return __fsub_rn(x, y);
        case MOYE_MAP_MUL: return __fmul_rn(x, y);
        case MOYE_MAP_DIV: return __fdiv_rn(x, y);
        // v_max_f32 / v_min_f32 order the zeros as Julia does (-0.0 < +0.0) and differ from it only when an operand is a NaN:
        // no lane of the wave has one (a wave-uniform test), and the instruction's result is the answer
        case MOYE_MAP_MAX:
            if (__builtin_amdgcn_ballot_w64((x != x) | (y != y)) == 0) return __builtin_fmaxf(x, y);
            return ((y > x) | (signbit(y) < signbit(x))) ? (x != x ? x : y) : (y != y ? y : x);
        case MOYE_MAP_MIN:
            if (__builtin_amdgcn_ballot_w64((x != x) | (y != y)) == 0) return __builtin_fminf(x, y);
            return ((y < x) | (signbit(y) > signbit(x))) ? (x != x ? x : y) : (y != y ? y : x);
        case MOYE_MAP_NEG: return -x;
        case MOYE_MAP_ABS: return signbit(x) ? -x : x;
        default: return x;
    }
}
// acc: the fp32 sum over k; c: the element of C (ignored unless has_c); (m, n): the element's position in the problem
__device__ __forceinline__ float epi_value(const GemmArgs& p, float acc, bool has_c, float c, int64_t m, int64_t n) {
    float t = __fmul_rn(acc, p.alpha);
    if (has_c) t = __fadd_rn(t, __fmul_rn(p.beta, c));
    if (p.ep_op != MOYE_MAP_IDENTITY) t = epi_op(p.ep_op, t, epi_operand(p, m, n));
    return t;
}

// XOR swizzle of the 16-byte chunk index inside an LDS tile row of CPR chunks.  The LDS has 32
// banks of 4 bytes, so 128 bytes (8 chunks) make one sweep of the banks and a 128-bit access is
// served 8 lanes per clock.  Rows that lie in different 128-byte sweeps get different chunk
// permutations, so 8 lanes reading the same logical chunk of 8 consecutive rows hit 8 different
// bank groups, and so do 8 lanes writing 8 consecutive chunks.
template <int CPR>
__device__ __forceinline__ int swz(int row) {
    if constexpr (CPR >= 8) return row & 7;
    else return (row / (8 / CPR)) & (CPR - 1);
}

// blockIdx.y -> the K range of a split-K launch (one range and no offsets for an ordinary launch)
__device__ __forceinline__ void split_of_block(GemmArgs& p) {
    if (gridDim.y > 1) {
        p.A = static_cast<const char*>(p.A) + (int64_t)blockIdx.y * p.split_ab;
        p.B = static_cast<const char*>(p.B) + (int64_t)blockIdx.y * p.split_ab;
        p.D = static_cast<char*>(p.D) + (int64_t)blockIdx.y * p.split_d;
    }
}

// One 16-byte piece of D.  With kGemmStreamD in GemmArgs::flags the store is non-temporal: when a launch has
// more tiles than the chip has CUs, results written the ordinary way sit in the L2s and push out the operand panels
// the next tiles are about to share.
__device__ __forceinline__ void store_d_chunk(const GemmArgs& p, char* d, const u32x4& w) {
    // (as text: the compiler merges an ordinary and a non-temporal store in the two arms of a branch into one ordinary
    // store; the nop covers the wait states a wide store needs before its data registers are written again)
    if (p.flags & kGemmStreamD) asm volatile("global_store_dwordx4 %0, %1, off nt\n\ts_nop 1" ::"v"(d), "v"(w) : "memory");
    else *reinterpret_cast<u32x4*>(d) = w;
}

// blockIdx -> (tile_m, tile_n).  Hardware deals consecutive workgroup ids round-robin to the 8
// XCDs; remapping id -> (id % 8) * (n / 8) + id / 8 hands each XCD one contiguous run of tiles,
// and inside a run tiles are walked in bands of 8 tile-rows so that the A and B panels an
// XCD's L2 holds are reused by the workgroups that follow.
// (`bid` of `n` tiles: a persistent kernel walks bid = blockIdx.x, blockIdx.x + gridDim.x, ... with gridDim.x a multiple of
// the number of XCDs, so every tile of a workgroup comes from its own XCD's run)
__device__ __forceinline__ void tile_of_index(int tiles_m, int tiles_n, int xcds, int flags, int bid, int n, int* tm, int* tn) {
    const int x = xcds;
    if ((flags & 1) && x > 1 && (n % x) == 0) bid = (bid % x) * (n / x) + bid / x;
    constexpr int kGroup = 8;
    const int per_group = kGroup * tiles_n;
    const int g = bid / per_group;
    const int first_m = g * kGroup;
    const int gsize = min(tiles_m - first_m, kGroup);
    const int r = bid - g * per_group;
    *tm = first_m + r % gsize;
    *tn = r / gsize;
}
__device__ __forceinline__ void tile_of_index(const GemmArgs& p, int bid, int n, int* tm, int* tn) {
    tile_of_index(p.tiles_m, p.tiles_n, p.xcds, p.flags, bid, n, tm, tn);
}
__device__ __forceinline__ void tile_of_block(const GemmArgs& p, int* tm, int* tn) { tile_of_index(p, blockIdx.x, gridDim.x, tm, tn); }

}  // namespace moye

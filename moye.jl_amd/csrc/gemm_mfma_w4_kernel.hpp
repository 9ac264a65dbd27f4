// gemm! on the matrix cores, every instruction of the k-loop placed by hand: one 256 x 256 CTA tile per compute unit,
// eight waves as 2 x 4 (wave tile 128 x 64, two waves per SIMD) or four as 2 x 2 (wave tile 128 x 128: 8 x 8 MFMA
// tiles, 256 accumulator registers per lane, pinned in the AccVGPR file).  Two forms of the operand stages in LDS:
//   whole lines  rows of 128 bytes of K, a stage is a k-step (64 KiB), two stages; a load-to-LDS instruction reads
//                eight whole 128-byte lines.  What a plain f16 / bf16 call on 256 x 256 tiles and every fp8 call run
//                (W4F16L, W4BF16L, W4FP8L; fp16 4096^3 97.4-98.7 us against 101.3-102.9 for the compiler-scheduled kernel
//                of gemm_mfma256.hip, fp8 8192^3 3050 TFLOP/s against 2745 on the ring), with an instance that adds a
//                bias and one for tiles that reach beyond M and N
//   ring         rows of 64 bytes in a ring of five 32 KiB stages, a k-step one stage or two (MOYE_GEMM_WAVE4 with
//                cta_tile_mnk[2] = 64 bytes of K, or with stages >= 3); how this kernel began, described below
//
// Why this shape: a 128 x 128 wave tile needs 16 fragments for 64 MFMAs (0.25 per MFMA; a
// 128 x 64 wave tile needs 0.375), and with one wave per SIMD the only workgroup-wide rendezvous
// is one s_barrier per k-step of 64 MFMAs.  Nothing else may hold the matrix pipe up, so the
// order of every instruction in the k-loop is fixed in the source:
//  * the MFMAs are inline assembly (their order is kept, and their "+a" constraints keep all 256
//    accumulators in AccVGPRs: with the builtins the register allocator moved accumulators
//    between the two register files, more copies than MFMAs);
//  * fragments are single-buffered and refilled in place: a fragment register is reloaded (for
//    the next k-step) right after the last MFMA of this k-step that reads it, and the MFMAs are
//    ordered so that every refill has at least 14 MFMAs (224 clocks) before its first use:
//      first half   rows 0-3, column by column      A0-3 are free after the last column
//      second half  row 4, row 5, then rows 6 and 7 column by column: B_j is free after its pair
//    the next k-step starts column by column again, so B_j is needed 4j MFMAs in;
//  * the fragment reads are inline assembly as well, with hand-placed s_waitcnt: the compiler's
//    wait-count pass drains every LDS read at the top of the loop once sixteen are in flight
//    across the back edge, and puts vmcnt(0) in front of LDS reads that follow load-to-LDS
//    instructions; neither is acceptable here.  The waits: the barrier's (all reads back, eight
//    MFMAs after the last one was issued), and partial ones in front of the first two columns;
//  * the loads of the stage(s) five ahead are spread evenly over the MFMAs that follow the barrier.
// A k-step is one stage (64 bytes of K) for f16/bf16/f32 and two stages for fp8, whose MFMA
// (16x16x128, 32 bytes per lane and operand) is the only fp8 form that runs at twice the
// 16-bit rate on gfx950.
//
// Ring: step s reads the fragments of step s+1 out of LDS, so when every wave has passed the
// barrier of step s (which sits after the MFMAs that consumed the last refills of step s-1) the
// stages of step s are free and receive the data five stages ahead.  Before the barrier a wave
// waits until its own share of step s+1 has landed: all but the youngest 5 - 2 SPS stages' loads.
//
// Operand conventions as in gemm_mfma256.hip: K-major A and B, N-contiguous D, the MFMA issued
// with B rows as its first operand so a lane holds four consecutive n of one m; the 16-byte chunk
// index of an LDS row is XORed with (row / 2) % 4, applied on the global side of the load-to-LDS.
#pragma once

#include <cstdlib>
#include <type_traits>
#include <utility>

#include "mfma_epilogue.hpp"

namespace moye {

typedef uint32_t u32x8 __attribute__((ext_vector_type(8)));

template <class F, int... Ps>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, Ps...>) {
    (f(std::integral_constant<int, Ps>{}), ...);
}
// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>), in order
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
    static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// The ND load-to-LDS instructions a wave issues per k-step go out evenly over the MFMA positions that
// follow the barrier (positions 8 .. NPOS - 1).  Returns the index of the load issued after MFMA P, or -1.
// With a ring of two stages the loads of a k-step must have landed by the next barrier: every other position from 8 on.
// (measured at fp16 4096^3, eight / four waves: every position 100.4 / 101.0 us, every other 97.7-98.7 / 97.4-98.6, every third
// 99.3 / 98.3; the barrier after MFMA 3, 5 or 11 instead of 7: 98.2, 99.9, 98.0 / 98.5, 99.4, 97.6)
constexpr int dma_index_early(int P, int ND) { return P >= 8 && P < 8 + 2 * ND && (P - 8) % 2 == 0 ? (P - 8) / 2 : -1; }
// The 128 x 128 tile: sixteen groups per k-step, the barrier after the fourth, eight loads over the twelve that follow.
constexpr int dma_index_128(int P, int ND) {
    for (int k = 0; k < ND; ++k)
        if (4 + (3 * k) / 2 == P) return k;
    return -1;
}
constexpr int dma_index(int P, int ND, int NPOS) {
    for (int k = 0; k < ND; ++k)
        if (8 + k * (NPOS - 8) / ND == P) return k;
    return -1;
}

// The same pointer, provably wave-uniform (an "s" operand of inline assembly is not legalised:
// a uniform value the compiler happened to compute in vector registers would be passed as is).
__device__ __forceinline__ const char* uniform_ptr(const char* p) {
    const uint64_t v = reinterpret_cast<uint64_t>(p);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return reinterpret_cast<const char*>(((uint64_t)hi << 32) | lo);
}

// 16 bytes from LDS byte address `addr` + OFF.  The compiler does not know that the result is in
// flight: the caller waits (s_waitcnt lgkmcnt) before the first use.
template <int OFF>
__device__ __forceinline__ u32x4 lds_read16(uint32_t addr) {
    u32x4 v;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
    return v;
}

// 8 bytes through the transposing LDS read of gfx950: sixteen lanes that each point at four consecutive 16-bit values
// get back, in lane j, value j % 4 of the lanes 4 e + j / 4 (e = 0..3).  In flight like lds_read16's result.
template <int OFF>
__device__ __forceinline__ u32x2 lds_read_tr8(uint32_t addr) {
    u32x2 v;
    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
    return v;
}
// The same for bytes (fp8): sixteen lanes that each point at eight consecutive bytes get back, in lane j, byte j % 8 of
// the lanes 2 e + j / 8 (e = 0..7) (measured on the hardware with a one-off probe, like the 16-bit form).
template <int OFF>
__device__ __forceinline__ u32x2 lds_read_tr8_b8(uint32_t addr) {
    u32x2 v;
    asm volatile("ds_read_b64_tr_b8 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
    return v;
}
template <int OFF>
__device__ __forceinline__ uint32_t lds_read4(uint32_t addr) {
    uint32_t v;
    asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
    return v;
}
// A fragment read out of an operand stage that is stored with its unit stride along M (N): four 8-byte halves, q0 q1
// the lane's k of the first 16 bytes of a K-major fragment, q2 q3 those of the second (see the kernel's AMAJ / BMAJ);
// for fp32 eight single values.
struct W4TrFrag { u32x2 q0, q1, q2, q3; };
struct W4TrFrag32 { uint32_t e[8]; };

// fragment = what one lane feeds to one MFMA group per operand; SPS = ring stages per k-step; kRow = bytes of K per row
// of a stage, kRing = stages in the ring
struct W4Ring64 { static constexpr int kRow = 64, kRing = 5; };
// (kDt / kName: the operand type of the instance, and its name in a plan)
struct W4F16 : W4Ring64 {
    static constexpr int kBytes = 2, SPS = 1, kDt = MOYE_F16;
    static constexpr const char* kName = "W4F16";
    typedef u32x4 frag;
    static __device__ __forceinline__ void mma(const frag& a, const frag& b, f32x4& c) {
        asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
    }
};
struct W4BF16 : W4Ring64 {
    static constexpr int kBytes = 2, SPS = 1, kDt = MOYE_BF16;
    static constexpr const char* kName = "W4BF16";
    typedef u32x4 frag;
    static __device__ __forceinline__ void mma(const frag& a, const frag& b, f32x4& c) {
        asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
    }
};
// The 16-bit types with k-steps of two stages (128 bytes of K): two MFMAs in a row on the same accumulator (which
// costs nothing: 16.4 clocks per MFMA either way) and half as many barriers per K.
struct W4F16x2 : W4Ring64 {
    static constexpr int kBytes = 2, SPS = 2, kDt = MOYE_F16;
    static constexpr const char* kName = "W4F16x2";
    struct frag { u32x4 lo, hi; };
    static __device__ __forceinline__ void mma(const frag& a, const frag& b, f32x4& c) {
        asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %3, %0\n\tv_mfma_f32_16x16x32_f16 %0, %2, %4, %0"
                     : "+a"(c) : "v"(a.lo), "v"(a.hi), "v"(b.lo), "v"(b.hi));
    }
};
struct W4BF16x2 : W4Ring64 {
    static constexpr int kBytes = 2, SPS = 2, kDt = MOYE_BF16;
    static constexpr const char* kName = "W4BF16x2";
    struct frag { u32x4 lo, hi; };
    static __device__ __forceinline__ void mma(const frag& a, const frag& b, f32x4& c) {
        asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %3, %0\n\tv_mfma_f32_16x16x32_bf16 %0, %2, %4, %0"
                     : "+a"(c) : "v"(a.lo), "v"(a.hi), "v"(b.lo), "v"(b.hi));
    }
};
// ... in a ring of four stages, i.e. two k-steps: what the 128 x 128 tile named with 64 bytes of K per stage runs on (64 KiB,
// two workgroups to a CU; fp16 4096^3: 125-127 us with the two halves of every 128-byte line requested back to back, 140-143
// a stage after the other, on the same box as 155-159 in a ring of five and 151-153 of six, one workgroup to a CU, and
// 161-171 for the register-staged kernel)
struct W4F16x2R4 : W4F16x2 {
    static constexpr int kRing = 4;
    static constexpr const char* kName = "W4F16x2R4";
};
struct W4BF16x2R4 : W4BF16x2 {
    static constexpr int kRing = 4;
    static constexpr const char* kName = "W4BF16x2R4";
};
// 32 bytes per lane: the chunk of stage 0 and the chunk of stage 1 of the k-step.  Which 32 of the
// 128 k-values a lane carries does not matter as long as A and B agree, and they do.
struct W4FP8 : W4Ring64 {
    static constexpr int kBytes = 1, SPS = 2, kDt = MOYE_F8E4M3;
    static constexpr const char* kName = "W4FP8";
    struct frag { u32x4 lo, hi; };
    static __device__ __forceinline__ void mma(const frag& a, const frag& b, f32x4& c) {
        const u32x8 a8 = __builtin_shufflevector(a.lo, a.hi, 0, 1, 2, 3, 4, 5, 6, 7);
        const u32x8 b8 = __builtin_shufflevector(b.lo, b.hi, 0, 1, 2, 3, 4, 5, 6, 7);
        asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0" : "+a"(c) : "v"(a8), "v"(b8));
    }
};
// The same MFMA fed from whole 128-byte rows: a stage is a k-step (64 KiB), two stages make the ring (the fragments of
// step s+1 are read out of one while the loads of step s+2 fill the other), a lane's 32 bytes are chunks kq and kq + 4
// of its row.  A load-to-LDS instruction then reads eight whole 128-byte lines instead of sixteen half lines.
struct W4FP8L {
    static constexpr int kBytes = 1, SPS = 1, kRow = 128, kRing = 2, kDt = MOYE_F8E4M3;
    static constexpr const char* kName = "W4FP8L";
    struct frag { u32x4 lo, hi; };
    static __device__ __forceinline__ void mma4(const u32x4& alo, const u32x4& ahi, const u32x4& blo, const u32x4& bhi, f32x4& c) {
        const u32x8 a8 = __builtin_shufflevector(alo, ahi, 0, 1, 2, 3, 4, 5, 6, 7);
        const u32x8 b8 = __builtin_shufflevector(blo, bhi, 0, 1, 2, 3, 4, 5, 6, 7);
        asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0" : "+a"(c) : "v"(a8), "v"(b8));
    }
    static __device__ __forceinline__ void mma(const frag& a, const frag& b, f32x4& c) { mma4(a.lo, a.hi, b.lo, b.hi, c); }
};
// The 16-bit types on whole-line stages: chunk kq feeds the first MFMA of an accumulator, chunk kq + 4 the second.
struct W4F16L {
    static constexpr int kBytes = 2, SPS = 1, kRow = 128, kRing = 2, kDt = MOYE_F16;
    static constexpr const char* kName = "W4F16L";
    struct frag { u32x4 lo, hi; };
    // the two MFMAs of an accumulator from the four 16-byte halves (what the transposing fragment reads assemble)
    static __device__ __forceinline__ void mma4(const u32x4& alo, const u32x4& ahi, const u32x4& blo, const u32x4& bhi, f32x4& c) {
        asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %3, %0\n\tv_mfma_f32_16x16x32_f16 %0, %2, %4, %0"
                     : "+a"(c) : "v"(alo), "v"(ahi), "v"(blo), "v"(bhi));
    }
    static __device__ __forceinline__ void mma(const frag& a, const frag& b, f32x4& c) { mma4(a.lo, a.hi, b.lo, b.hi, c); }
};
struct W4BF16L {
    static constexpr int kBytes = 2, SPS = 1, kRow = 128, kRing = 2, kDt = MOYE_BF16;
    static constexpr const char* kName = "W4BF16L";
    struct frag { u32x4 lo, hi; };
    static __device__ __forceinline__ void mma4(const u32x4& alo, const u32x4& ahi, const u32x4& blo, const u32x4& bhi, f32x4& c) {
        asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %3, %0\n\tv_mfma_f32_16x16x32_bf16 %0, %2, %4, %0"
                     : "+a"(c) : "v"(alo), "v"(ahi), "v"(blo), "v"(bhi));
    }
    static __device__ __forceinline__ void mma(const frag& a, const frag& b, f32x4& c) { mma4(a.lo, a.hi, b.lo, b.hi, c); }
};
// element j of the chunk goes to MFMA j (see InF32)
struct W4F32 : W4Ring64 {
    static constexpr int kBytes = 4, SPS = 1, kDt = MOYE_F32;
    static constexpr const char* kName = "W4F32";
    typedef u32x4 frag;
    static __device__ __forceinline__ void mma(const frag& a, const frag& b, f32x4& c) {
        asm volatile(
            "v_mfma_f32_16x16x4_f32 %0, %1, %5, %0\n\tv_mfma_f32_16x16x4_f32 %0, %2, %6, %0\n\t"
            "v_mfma_f32_16x16x4_f32 %0, %3, %7, %0\n\tv_mfma_f32_16x16x4_f32 %0, %4, %8, %0"
            : "+a"(c)
            : "v"(a.x), "v"(a.y), "v"(a.z), "v"(a.w), "v"(b.x), "v"(b.y), "v"(b.z), "v"(b.w));
    }
};

// WGN = 2: four waves (2 x 2), wave tile 128 x 128.  WGN = 4: eight waves (2 x 4), wave tile 128 x 64,
// two waves per SIMD, so that what stalls one wave's instruction stream (an M0 write, a taken branch,
// the barrier) leaves the matrix pipe to the other.
// kBias: the call's element-wise operation has a scalar, one-per-column or one-per-row operand (a bias, a ReLU, a scale:
// kGemmEpiLaneOp): the same kernel with that operation in the lanes' own epilogue (store_c_tile's kLaneOp, which asks
// for C one pass ahead only: with the plain form's four passes ahead the epilogue spilled 96 registers, so it spills 2-3).
// kNoC: the call has no C (checked on the host): C's read paths are not compiled in (fp16 4096^3 with a bias row: +1.8 %
// over the plain call, +4.2 % with the paths compiled in and not taken).
// kRagged: M and N need not be multiples of 256 and K only of 16 bytes (its tail: see tail_pieces): a lane whose row lies beyond
// the operand reads the operand's last row instead (its constant lane offset is computed from the clamped row), what is
// computed from it is never stored, and the epilogue runs with its row and column guards (a D that is not 16-byte
// aligned goes out element by element where it must).  For calls without C (its epilogue is compiled without C's read
// paths: with them and the guards it spilled 64-110 registers); a ragged call with C runs the kOps instance.
// kOps: the epilogue is store_c_tile_general (any element-wise operation, any C, whole or ragged tiles): the raw
// accumulators go through LDS 32 rows at a time and the arithmetic exists once, in a loop, which costs the 16-bit
// outputs 9-20 spilled registers after the last MFMA and none before.  Whole-line stages, eight waves, K-major operands.
//
// TILE = 128: the same kernel on a 128 x 128 CTA tile, four waves as 2 x 2 (wave tile 64 x 64, 4 x 4 MFMA tiles), two
// whole-line stages of 32 KiB, two workgroups per CU (what gemm_mfma128.hip's kernel is to gemm_mfma256.hip's): rows 0-1
// column by column, then rows 2-3 column by column; the barrier after the fourth MFMA group, the eight loads of a
// wave over the twelve groups that follow.
// fp32 on whole-line stages: a 128-byte row holds 32 k; chunk kq and chunk kq + 4 are four k each, element j of a chunk
// going to MFMA j (see W4F32): eight MFMAs in a row per accumulator and k-step.
struct W4F32L {
    static constexpr int kBytes = 4, SPS = 1, kRow = 128, kRing = 2, kDt = MOYE_F32;
    static constexpr const char* kName = "W4F32L";
    struct frag { u32x4 lo, hi; };
    // four MFMAs from four values of each operand
    static __device__ __forceinline__ void mma_quad(uint32_t a0, uint32_t a1, uint32_t a2, uint32_t a3, uint32_t b0, uint32_t b1, uint32_t b2, uint32_t b3, f32x4& c) {
        asm volatile(
            "v_mfma_f32_16x16x4_f32 %0, %1, %5, %0\n\tv_mfma_f32_16x16x4_f32 %0, %2, %6, %0\n\t"
            "v_mfma_f32_16x16x4_f32 %0, %3, %7, %0\n\tv_mfma_f32_16x16x4_f32 %0, %4, %8, %0"
            : "+a"(c)
            : "v"(a0), "v"(a1), "v"(a2), "v"(a3), "v"(b0), "v"(b1), "v"(b2), "v"(b3));
    }
    static __device__ __forceinline__ void mma(const frag& a, const frag& b, f32x4& c) {
        mma_quad(a.lo.x, a.lo.y, a.lo.z, a.lo.w, b.lo.x, b.lo.y, b.lo.z, b.lo.w, c);
        mma_quad(a.hi.x, a.hi.y, a.hi.z, a.hi.w, b.hi.x, b.hi.y, b.hi.z, b.hi.w, c);
    }
};

// AMAJ / BMAJ = 1: that operand is stored with its unit stride along M (N) instead of K, the 'N' forms of
// src/arch/mma/make_mma_ops.jl:253-265 (GemmArgs::lda / ldb is then the pitch between consecutive k).  Its half of a stage
// is 64 k-rows of 256 operand rows (512 bytes), filled by the same load-to-LDS instructions (two k-rows each), and the
// fragments come out of it with ds_read_b64_tr_b16, where the reference has ldmatrix.trans
// (src/arch/copy/ldmatrix.jl:18-48): lane 16 g + s points at k-row 8 g + s / 4 (+ 4, + 32, + 36 for the other three
// reads) and m = m0 + 4 (s % 4), and the four reads hand it the k of row m0 + s that chunks g and g + 4 of a K-major
// row would.  The 32-byte piece index of a k-row is XORed with (row % 4) | 4 ((row / 8) % 2), so that the eight row
// pieces the 32 lanes of one pass read lie in eight bank groups (the layout of gemm_mfma_lds_tile.hpp).  fp8 the same
// way through ds_read_b64_tr_b8 (k-rows of 256 bytes, 128 per stage; lane 16 g + s points at k-row 16 g + s / 2 (+ 8,
// + 64, + 72) and m = m0 + 8 (s % 2); the 16-byte piece index XORed with row % 8 and, in bit 3, with (row / 16) % 2: see
// tr_swz).  fp32 needs no transposing read: an
// MFMA takes one value per lane and operand, so a lane reads its eight values of row m0 + s with ds_read_b32 from
// k-rows 4 g + e and 16 + 4 g + e (k-rows of 1 KiB, 32 per stage; the 64-byte piece index XORed with (row / 4) % 2, so
// that the two k-rows the 32 lanes of a pass read lie in different halves of the banks).  Whole-line stages, plain calls
// on whole tiles: the 256 x 256 tile with eight waves, the 128 x 128 tile with four (k-rows of 128 operand rows).
template <typename In, typename Out, int WGN, bool kBias = false, bool kRagged = false, int TILE = 256, int AMAJ = 0, int BMAJ = 0, bool kOps = false, bool kNoC = false, bool kPersist = false>
__global__ __launch_bounds__(128 * WGN, TILE == 128 ? 2 : 1) void gemm_mfma_tn_256_w4(GemmArgs p) {
    static_assert(!(AMAJ || BMAJ) || (In::kRow == 128 && ((TILE == 256 && WGN == 4) || (TILE == 128 && WGN == 2)) && !kBias && !kRagged),
                  "operands that are not K-major: whole-line stages, eight waves, plain whole tiles");
    static_assert(!kRagged || (!kBias && In::kRow == 128 && !AMAJ && !BMAJ), "ragged tiles: the plain whole-line form, K-major operands");
    static_assert(!kOps || (In::kRow == 128 && TILE == 256 && WGN == 4 && !kBias && !AMAJ && !BMAJ), "epilogue operations: whole-line stages, eight waves, K-major operands");
    static_assert(!kPersist || (In::kRow == 128 && TILE == 256 && WGN == 4 && !kRagged && !kOps && !AMAJ && !BMAJ),
                  "the persistent form: whole-line stages, eight waves, whole tiles, K-major operands (its C patches lie beside the stages)");
    static_assert(TILE == 256 || (TILE == 128 && WGN == 2 && !kBias && (In::kRow == 128 || (In::SPS == 2 && !kRagged))),
                  "128 x 128 tiles: 2 x 2 waves; the whole-line form, plain or ragged, or the ring of 64-byte-row stages with k-steps of two stages");
    constexpr int BM = TILE, BN = TILE, kRow = In::kRow, CPR = kRow / 16, STAGES = In::kRing, SPS = In::SPS;
    constexpr bool kLine = kRow == 128;                        // a fragment is two chunks of one row of one stage
    constexpr int RPF = kLine ? 2 : SPS;                       // LDS reads per fragment
    constexpr int RPI = 64 / CPR;                              // rows one load-to-LDS instruction covers
    static_assert(!kLine || (SPS == 1 && STAGES == 2), "whole-line stages: one per k-step, two in the ring");
    constexpr int STAGE = (BM + BN) * CPR;  // in 16-byte chunks
    constexpr int NW = 2 * WGN, WN = BN / WGN;
    constexpr int MI = BM / 32, NI = WN / 16, NPOS = MI * NI, H = MI / 2;  // H: the rows of the first phase
    constexpr int BAR = TILE == 128 ? 3 : 7;  // the MFMA group after which the waves meet
    constexpr int RW = BM / NW, LD = RW / RPI;  // per wave and stage: RW rows, LD load-to-LDS instructions per operand
    typedef typename In::frag frag;
    typedef std::conditional_t<In::kBytes == 4, W4TrFrag32, W4TrFrag> frag_t;
    typedef std::conditional_t<AMAJ != 0, frag_t, frag> frag_a;
    typedef std::conditional_t<BMAJ != 0, frag_t, frag> frag_b;
    constexpr int RPT = In::kBytes == 4 ? 8 : 4;                    // LDS reads per fragment of a transposed operand
    constexpr int RPA = AMAJ ? RPT : RPF, RPB = BMAJ ? RPT : RPF;  // LDS reads per fragment of A and of B
    // transposed operand halves of a stage: k-rows of TROW bytes, a swizzle granule of 16 operand rows (GB bytes)
    constexpr int TROW = TILE * In::kBytes, TKROWS = 128 / In::kBytes, TLPR = TROW / 16, TRPI = 64 / TLPR, GB = 16 * In::kBytes;
    // (bytes: the 32 lanes of a pass read k-rows 0-7 and 16-23.  On the 256 x 256 tile a k-row has sixteen 16-byte granules
    // and bit 4 of the row picks the half of them; on the 128 x 128 tile it has eight, a k-row is half a sweep of the
    // banks, and the k-rows whose bit 4 is set are stored with their neighbour's place instead (tr_place), so that rows
    // j and 16 + j lie in different halves.  Without either, every such read took two more cycles.)
    auto tr_swz = [](int krow) {
        return In::kBytes == 2   ? ((krow & 3) | (((krow >> 3) & 1) << 2))
               : In::kBytes == 1 ? ((krow & 7) | (TROW >= 256 ? ((krow >> 4) & 1) << 3 : 0))
                                 : ((krow >> 2) & 1);
    };
    auto tr_place = [](int krow) { return In::kBytes == 1 && TROW < 256 ? krow ^ ((krow >> 4) & 1) : krow; };  // its own inverse

    extern __shared__ __attribute__((aligned(256))) u32x4 smem[];

    // kPersist: a workgroup per CU that takes tile blockIdx.x, blockIdx.x + gridDim.x, ... of the launch (problems with
    // more tiles than CUs).  The first two stages of the next tile are requested before the epilogue of the tile just
    // computed, whose C patches lie beside the operand stages, so the stores of one tile and the first loads of the next
    // are in flight together and a tile's k-loop starts on data that is already there.
    int tm, tn;
    split_of_block(p);
    [[maybe_unused]] int tile = blockIdx.x;
    [[maybe_unused]] const int ntiles = p.tiles_m * p.tiles_n;
    // (the persistent form: the tile's place comes out of integer divisions, which run on the vector unit; their inputs go
    // through an empty statement so that no reciprocal is kept in a vector register across the k-loop, and the results
    // are made scalars again)
    auto locate = [&](int bid) __attribute__((always_inline)) {
        int tiles_m = p.tiles_m, tiles_n = p.tiles_n, xcds = p.xcds, n = ntiles;
        asm volatile("" : "+s"(tiles_m), "+s"(tiles_n), "+s"(xcds), "+s"(n), "+s"(bid));
        tile_of_index(tiles_m, tiles_n, xcds, p.flags, bid, n, &tm, &tn);
        tm = __builtin_amdgcn_readfirstlane(tm);
        tn = __builtin_amdgcn_readfirstlane(tn);
    };
    if constexpr (kPersist) locate(tile);
    else tile_of_block(p, &tm, &tn);
    [[maybe_unused]] bool first_tile = true;
    // (a persistent workgroup comes back here for every tile.  Everything a lane computes from its number is computed
    // again: the lane number goes through an empty statement, so that none of it is kept in registers across the epilogue
    // of the tile before, which needs them itself; a spilled value would come back through a scratch load, and a wait for
    // that load is a wait for every store and load issued before it)
    for (;;) {
    int lane_now = threadIdx.x & 63;
    if constexpr (kPersist) asm volatile("" : "+v"(lane_now));
    const int tid = threadIdx.x, lane = lane_now, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm0 = (wave / WGN) * (BM / 2), wn0 = (wave % WGN) * WN;
    const int r16 = lane & 15, kq = lane >> 4;

    const int64_t pitch_a = (int64_t)p.lda * In::kBytes, pitch_b = (int64_t)p.ldb * In::kBytes;
    // LDS stage (32 KiB) = A tile (256 rows of 64 bytes) then B tile.  Lane l of a load-to-LDS
    // instruction lands in physical chunk l % 4 of row l / 4 of a 16-row group; wave w brings rows
    // RW w .. RW w + RW - 1 of each operand.
    const int lrow = wave * RW + lane / CPR, lch = (lane % CPR) ^ swz<CPR>(lane / CPR);
    // (an M-major operand: its tile starts BM elements further along the row of every k)
    const char* a_tile = static_cast<const char*>(p.A) + (AMAJ ? (int64_t)tm * BM * In::kBytes : (int64_t)tm * BM * pitch_a);  // uniform
    const char* b_tile = static_cast<const char*>(p.B) + (BMAJ ? (int64_t)tn * BN * In::kBytes : (int64_t)tn * BN * pitch_b);
    constexpr uint32_t kStageBytes = STAGE * 16, kATileBytes = BM * CPR * 16;

    f32x4 acc[MI][NI];

    // Ragged instances also take a K that ends inside a 128-byte row (a whole number of 16-byte pieces): the last stage
    // then holds tail_pieces valid pieces per row.  The lanes whose piece lies beyond K read the row's first piece of that
    // stage instead (inside the operand), and every fragment half that lies beyond K is zeroed in registers before the
    // last k-step's MFMAs (what was loaded there may be NaN or Inf, and must not reach an accumulator).
    [[maybe_unused]] const int tail_pieces = kRagged ? (int)((((int64_t)p.K * In::kBytes) % kRow) / 16) : 0;  // 0: whole rows
    const int nstages = (int)(((int64_t)p.K * In::kBytes + (kRagged ? kRow - 1 : 0)) / kRow);
    const int nsteps = nstages / SPS;
    frag_a fa[MI];
    frag_b fb[NI];

    typedef __attribute__((address_space(3))) void* lptr_t;
    const uint32_t lds0 = (uint32_t)(uintptr_t)(lptr_t)smem;  // LDS byte address of the ring
    // Load-to-LDS instruction Q (0 .. LD-1: A, LD .. 2 LD - 1: B) of this wave's share of a stage, in the scalar-base
    // form: a uniform 64-bit pointer to the stage's first row plus a per-lane 32-bit offset that never
    // changes, so no vector ALU work is left in the loop.  M0 carries the LDS destination of the
    // instruction's first lane.
    uint32_t voff[2 * LD];
    [[maybe_unused]] const int last_a = p.M - 1 - tm * BM, last_b = p.N - 1 - tn * BN;  // ragged: the last row of the operand, counted from the tile's first
    // an M-major (N-major) operand: instruction q % LD of wave w brings k-rows 8 w + 2 (q % LD) + lane / 32 of the stage,
    // lane l the 16-byte piece that belongs in physical slot l % 32 of its k-row
    static_assert(!(AMAJ || BMAJ) || TKROWS / NW == TRPI * LD, "a wave's k-rows of a transposed operand: LD instructions");
#pragma unroll
    for (int q = 0; q < 2 * LD; ++q) {
        if ((q < LD && AMAJ) || (q >= LD && BMAJ)) {
            // (the k-row whose place in the stage this lane fills)
            const int krow = tr_place(wave * (TKROWS / NW) + TRPI * (q % LD) + lane / TLPR), p16 = lane % TLPR;
            const int piece = (((p16 * 16 / GB) ^ tr_swz(krow)) * GB + (p16 * 16) % GB) / 16;  // the swizzle moves granules
            voff[q] = (uint32_t)(krow * (q < LD ? pitch_a : pitch_b) + piece * 16);
            continue;
        }
        int row = lrow + RPI * (q % LD);
        if constexpr (kRagged) row = min(row, q < LD ? last_a : last_b);
        voff[q] = (uint32_t)(row * (q < LD ? pitch_a : pitch_b) + lch * 16);
    }
    // stage g of this workgroup's walk over K is stage g + g0 (mod nstages) of the operands: the eight XCDs start an
    // eighth of K apart when the caller asks for it (see gemm_mfma256.hip); not with a K tail, whose stage has to be
    // the last in time as well
    const int g0 = ((p.flags & kGemmRotateK) && !tail_pieces) ? (int)((int64_t)(blockIdx.x % p.xcds) * nsteps / p.xcds) * SPS : 0;
    // what a lane whose piece lies beyond K in the last stage subtracts from its offset to land on the row's first piece
    [[maybe_unused]] const uint32_t tail_cut = (kRagged && tail_pieces && lch >= tail_pieces) ? (uint32_t)lch * 16 : 0;
    auto dma1 = [&](int g, int ring_slot, auto qc) __attribute__((always_inline)) {
        constexpr int Q = decltype(qc)::value;
        const int gr = g + g0 >= nstages ? g + g0 - nstages : g + g0;
        // (stage gr of a K-major operand starts kRow bytes further along every row, of an M-major one 64 k-rows further down)
        const char* const base = uniform_ptr(Q < LD ? a_tile + (AMAJ ? (int64_t)gr * TKROWS * pitch_a : (int64_t)gr * kRow)
                                                    : b_tile + (BMAJ ? (int64_t)gr * TKROWS * pitch_b : (int64_t)gr * kRow));
        const uint32_t dst = __builtin_amdgcn_readfirstlane(lds0 + ring_slot * kStageBytes + (Q < LD ? 0 : kATileBytes) +
                                                            (uint32_t)(wave * RW + RPI * (Q % LD)) * kRow);
        uint32_t lane_off = voff[Q];  // (a captured array element cannot be an asm operand of a generic lambda)
        if constexpr (kRagged) lane_off -= gr == nstages - 1 ? tail_cut : 0u;  // (a uniform choice; tail_cut is zero without a tail)
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(lane_off), "s"(base), "s"(dst)
                     : "memory");
    };
#define MOYE_VMCNT(N) (((N) & 0xF) | (((N) >> 4) << 14))
    // bare s_barrier: __syncthreads() would add a fence that drains the prefetch
#define MOYE_BARRIER()                      \
    {                                       \
        asm volatile("" ::: "memory");      \
        __builtin_amdgcn_s_barrier();       \
        asm volatile("" ::: "memory");      \
    }
    // LDS byte addresses of this lane's fragment chunk in ring slot 0; 16-row block BLK adds 1024 BLK
    const uint32_t frag_lane = (uint32_t)(r16 * kRow + ((kq ^ swz<CPR>(r16)) * 16));
    const uint32_t fa_byte = lds0 + wm0 * kRow + frag_lane;
    const uint32_t fb_byte = lds0 + kATileBytes + wn0 * kRow + frag_lane;
    // whole-line stages: the lane's second chunk, kq + 4, of the same row
    [[maybe_unused]] const uint32_t hi_delta = (uint32_t)((((kq + 4) ^ swz<CPR>(r16)) - (kq ^ swz<CPR>(r16))) * 16);
    // transposed operand halves: the byte address of this lane's first read of 16-row block 0 in ring slot 0; block BLK
    // XORs BLK << 5 into it (the piece index is swizzled, and a wave tile starts at a piece index whose low bits are clear)
    // (the lane's first k-row and its bytes inside the granule: 16-bit 8 kq + r16 / 4 and 8 (r16 % 4); bytes 16 kq + r16 / 2
    // and 8 (r16 % 2); fp32 4 kq and 4 r16)
    [[maybe_unused]] const int tr_row0 = In::kBytes == 2 ? 8 * kq + (r16 >> 2) : In::kBytes == 1 ? 16 * kq + (r16 >> 1) : 4 * kq;
    [[maybe_unused]] const int tr_in = In::kBytes == 2 ? 8 * (r16 & 3) : In::kBytes == 1 ? 8 * (r16 & 1) : 4 * r16;
    [[maybe_unused]] const int tr_fx = tr_swz(tr_row0);
    // (the other reads of a fragment add 8, 64 and 72 k-rows (bytes) to the first: neither bit 0, which tr_place may flip,
    // nor the bits the swizzle looks at change)
    [[maybe_unused]] const uint32_t ta_byte = lds0 + (uint32_t)(tr_place(tr_row0) * TROW + ((wm0 / 16) ^ tr_fx) * GB + tr_in);
    [[maybe_unused]] const uint32_t tb_byte = lds0 + kATileBytes + (uint32_t)(tr_place(tr_row0) * TROW + ((wn0 / 16) ^ tr_fx) * GB + tr_in);
    // the fragment of 16-row block BLK for the k-step whose stages start at byte offsets o0 (, o1)
    auto load_frag = [&](auto& f, uint32_t base, auto blk_c, uint32_t o0, uint32_t o1) __attribute__((always_inline)) {
        constexpr int OFF = 16 * kRow * decltype(blk_c)::value;
        if constexpr (std::is_same_v<std::remove_reference_t<decltype(f)>, W4TrFrag>) {
            const uint32_t at = (base ^ (uint32_t)(decltype(blk_c)::value * GB)) + o0;  // (stage offsets are multiples of 64 KiB)
            if constexpr (In::kBytes == 2) {
                f.q0 = lds_read_tr8<0>(at);
                f.q1 = lds_read_tr8<4 * TROW>(at);
                f.q2 = lds_read_tr8<32 * TROW>(at);
                f.q3 = lds_read_tr8<36 * TROW>(at);
            } else {
                f.q0 = lds_read_tr8_b8<0>(at);
                f.q1 = lds_read_tr8_b8<8 * TROW>(at);
                f.q2 = lds_read_tr8_b8<64 * TROW>(at);
                f.q3 = lds_read_tr8_b8<72 * TROW>(at);
            }
        } else if constexpr (std::is_same_v<std::remove_reference_t<decltype(f)>, W4TrFrag32>) {
            const uint32_t at = (base ^ (uint32_t)(decltype(blk_c)::value * GB)) + o0;
            f.e[0] = lds_read4<0>(at);
            f.e[1] = lds_read4<TROW>(at);
            f.e[2] = lds_read4<2 * TROW>(at);
            f.e[3] = lds_read4<3 * TROW>(at);
            f.e[4] = lds_read4<16 * TROW>(at);
            f.e[5] = lds_read4<17 * TROW>(at);
            f.e[6] = lds_read4<18 * TROW>(at);
            f.e[7] = lds_read4<19 * TROW>(at);
        } else if constexpr (kLine) {
            f.lo = lds_read16<OFF>(base + o0);
            f.hi = lds_read16<OFF>(base + hi_delta + o0);
        } else if constexpr (SPS == 1) {
            f = lds_read16<OFF>(base + o0);
        } else {
            f.lo = lds_read16<OFF>(base + o0);
            f.hi = lds_read16<OFF>(base + o1);
        }
    };
#define MOYE_BLK(N) std::integral_constant<int, (N)> {}

    // prologue: all stages of the ring requested, wait for the first k-step's
    auto request_ring = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int g = 0; g < STAGES; ++g)
            if (g < nstages) {
                static_for<2 * LD>([&](auto qc) __attribute__((always_inline)) { dma1(g, g, qc); });
            }
    };
    if (first_tile) request_ring();  // (a later tile of a persistent workgroup: requested before the epilogue of the tile before)
    // (the persistent form: a zero made here, so that the compiler does not keep one in vector registers across the tiles,
    // where it would be spilled and come back through a scratch load)
    float zero = 0.f;
    if constexpr (kPersist) asm volatile("v_mov_b32 %0, 0" : "=v"(zero));
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j) acc[i][j] = f32x4{zero, zero, zero, zero};
    // A later tile of a persistent workgroup: after this tile's two stages the wave issued the previous tile's epilogue,
    // at least sixteen 16-byte stores (128 x 64 values of 16 bits), and vector memory operations complete in the order
    // they were issued: with at most the second stage's loads and eight more operations in flight the first stage is there.
    constexpr int kEpilogueOps = 8;
    if (kPersist && !first_tile && nstages >= STAGES) __builtin_amdgcn_s_waitcnt(MOYE_VMCNT(2 * LD * (STAGES - SPS) + kEpilogueOps) | 0x0F70);
    else if (nstages >= STAGES) __builtin_amdgcn_s_waitcnt(MOYE_VMCNT(2 * LD * (STAGES - SPS)) | 0x0F70);
    else __builtin_amdgcn_s_waitcnt(0x0F70);
    MOYE_BARRIER()
    static_for<MI>([&](auto ic) __attribute__((always_inline)) {
        load_frag(fa[decltype(ic)::value], AMAJ ? ta_byte : fa_byte, ic, 0, kStageBytes);
        if ((decltype(ic)::value + 1) % (12 / RPA < 4 ? 12 / RPA : 4) == 0) __builtin_amdgcn_s_waitcnt(0xC07F);  // at most 15 reads in flight
    });
    static_for<NI>([&](auto jc) __attribute__((always_inline)) {
        load_frag(fb[decltype(jc)::value], BMAJ ? tb_byte : fb_byte, jc, 0, kStageBytes);
        if ((decltype(jc)::value + 1) % (12 / RPB < 4 ? 12 / RPB : 4) == 0) __builtin_amdgcn_s_waitcnt(0xC07F);
    });
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)

    // position P of the NPOS MFMA groups of a k-step -> (i, j): rows 0-3 column by column, row 4, row 5,
    // rows 6 and 7 column by column.
    // Inside each phase the walk goes back and forth, so that one operand register set changes between consecutive
    // MFMAs, not two (odd columns of rows 0-3 and of rows 6-7 run upwards, row 4 runs from the last column back): with
    // dense operands the part is power-limited and an MFMA-only loop sustains 1.5-2 % more in such an order.
    // (H = 4 rows first, rows 4 and 5 whole, rows 6 and 7 in pairs for the 256 x 256 tile; H = 2, no whole rows, rows 2
    // and 3 in pairs for the 128 x 128 one)
#define MOYE_I(P)                                                                                     \
    ((P) < H * NI ? ((((P) / H) & 1) ? H - 1 - (P) % H : (P) % H)                                      \
     : (P) < (MI - 2) * NI ? H + ((P) - H * NI) / NI                                                   \
                    : MI - 2 + ((((((P) - (MI - 2) * NI) / 2) & 1) ? 1 - (((P) - (MI - 2) * NI) & 1) : (((P) - (MI - 2) * NI) & 1))))
#define MOYE_J(P)                                                                                     \
    ((P) < H * NI ? (P) / H                                                                            \
     : (P) < (MI - 2) * NI ? (((((P) - H * NI) / NI) & 1) ? ((P) - H * NI) % NI : NI - 1 - ((P) - H * NI) % NI) \
                           : ((P) - (MI - 2) * NI) / 2)
    int slot;  // ring slot of the first stage of step s
    // One k-step.  MORE: step s+1 exists (its fragments are read); AHEAD: the stages five ahead exist
    // (they are requested, and the stages allowed to stay in flight at the barrier are the full 5 - 2 SPS).
    // Fragment reads in program order (128 x 128 wave tile): A3 A2 A1 A0 (after MFMA 28..31, each after its last
    // use in the upward last column) A4 (39) A5 (47) B0 (49) B1 (51) B2 B3 B4 B5 B6 (61) A7 (62) A6 B7 (63); the next
    // k-step needs B_j at MFMA 4 j and A0-3 at 0..3.  In general: rows 0-3 after 4 (NI - 1) .. 4 NI - 1, A4 after
    // 5 NI - 1, A5 after 6 NI - 1, B_j after 6 NI + 2 j + 1, rows 6 and 7 after 8 NI - 2 and 8 NI - 1.
    auto step = [&](auto more_c, auto ahead_c, int s) __attribute__((always_inline)) {
        constexpr bool MORE = decltype(more_c)::value, AHEAD = decltype(ahead_c)::value;
        if constexpr (kRagged && !MORE) {
            // the last k-step of a K that ends inside a row: the fragment halves beyond K become zeros (a lane's halves
            // are pieces kq and kq + 4 of its row).  In a block of its own, after every fragment read has returned.
            if (tail_pieces) {
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                const bool cut_lo = kq >= tail_pieces, cut_hi = kq + 4 >= tail_pieces;
                auto cut = [&](auto& f) __attribute__((always_inline)) {
                    // (only the two-piece fragments of the whole-line forms exist in ragged instances; the test keeps
                    // the other instantiations of this lambda well-formed)
                    if constexpr (std::is_class_v<std::remove_reference_t<decltype(f)>>) {
                        const u32x4 zero = {0u, 0u, 0u, 0u};
                        f.lo = cut_lo ? zero : f.lo;
                        f.hi = cut_hi ? zero : f.hi;
                    }
                };
#pragma unroll
                for (int i = 0; i < MI; ++i) cut(fa[i]);
#pragma unroll
                for (int j = 0; j < NI; ++j) cut(fb[j]);
            }
        }
        int slot_n = slot + SPS;  // first stage of step s+1
        if (slot_n >= STAGES) slot_n -= STAGES;
        const uint32_t o0 = (uint32_t)slot_n * kStageBytes;
        const uint32_t o1 = (uint32_t)(slot_n + 1 == STAGES ? 0 : slot_n + 1) * kStageBytes;
        const int g_new = s * SPS + STAGES;  // first global stage requested in this step
        static_for<NPOS>([&](auto pc) __attribute__((always_inline)) {
            constexpr int P = decltype(pc)::value;
            constexpr int i = MOYE_I(P), j = MOYE_J(P);
            // B0 is followed by NI + 1 fragment reads, B1 by NI; a stricter count costs nothing where the
            // older reads are hundreds of clocks old (fp8: two reads per fragment, 32-clock MFMAs)
            // (in reads: B1 .. B(NI-1) and the last two A fragments follow B0)
            constexpr int after_b0 = (NI - 1) * RPB + 2 * RPA, after_b1 = (NI - 2) * RPB + 2 * RPA;
            if (P == 0) __builtin_amdgcn_s_waitcnt(0xC07F | ((after_b0 < 12 ? after_b0 : 12) << 8));
            if (P == H) __builtin_amdgcn_s_waitcnt(0xC07F | ((after_b1 < 12 ? after_b1 : 12) << 8));
            if constexpr ((AMAJ || BMAJ) && In::kBytes == 4) {
                auto el = [](const auto& f, auto tc) __attribute__((always_inline)) {
                    constexpr int t = decltype(tc)::value;
                    if constexpr (std::is_same_v<std::remove_cv_t<std::remove_reference_t<decltype(f)>>, W4TrFrag32>) return f.e[t];
                    else if constexpr (t < 4) return f.lo[t];
                    else return f.hi[t - 4];
                };
#define MOYE_EL(F, T) el(F, std::integral_constant<int, T>{})
                In::mma_quad(MOYE_EL(fb[j], 0), MOYE_EL(fb[j], 1), MOYE_EL(fb[j], 2), MOYE_EL(fb[j], 3), MOYE_EL(fa[i], 0), MOYE_EL(fa[i], 1), MOYE_EL(fa[i], 2), MOYE_EL(fa[i], 3), acc[i][j]);
                In::mma_quad(MOYE_EL(fb[j], 4), MOYE_EL(fb[j], 5), MOYE_EL(fb[j], 6), MOYE_EL(fb[j], 7), MOYE_EL(fa[i], 4), MOYE_EL(fa[i], 5), MOYE_EL(fa[i], 6), MOYE_EL(fa[i], 7), acc[i][j]);
#undef MOYE_EL
            } else if constexpr (AMAJ || BMAJ) {
                // (the halves of a transposed fragment are joined where the MFMA names them: the register allocator puts
                // the two reads' results side by side; the build checks that nothing else touches them)
                auto lo = [](const auto& f) __attribute__((always_inline)) {
                    if constexpr (std::is_same_v<std::remove_cv_t<std::remove_reference_t<decltype(f)>>, W4TrFrag>) return __builtin_shufflevector(f.q0, f.q1, 0, 1, 2, 3);
                    else return f.lo;
                };
                auto hi = [](const auto& f) __attribute__((always_inline)) {
                    if constexpr (std::is_same_v<std::remove_cv_t<std::remove_reference_t<decltype(f)>>, W4TrFrag>) return __builtin_shufflevector(f.q2, f.q3, 0, 1, 2, 3);
                    else return f.hi;
                };
                In::mma4(lo(fb[j]), hi(fb[j]), lo(fa[i]), hi(fa[i]), acc[i][j]);
            } else {
                In::mma(fb[j], fa[i], acc[i][j]);
            }
            if (P == BAR) {
                // my share of step s+1 has landed and all my fragment reads have returned (the last were
                // issued eight MFMAs ago); after the barrier that holds for everybody
                if (AHEAD) {
                    __builtin_amdgcn_s_waitcnt(MOYE_VMCNT(2 * LD * (STAGES - 2 * SPS)) | 0x0070);
                } else {
                    // stages requested so far: min(nstages, g_new); needed: all below (s+2) SPS
                    const int allow = min(nstages, g_new) - (s + 2) * SPS;
                    if (allow >= 2) __builtin_amdgcn_s_waitcnt(MOYE_VMCNT(2 * LD * 2) | 0x0070);
                    else if (allow == 1) __builtin_amdgcn_s_waitcnt(MOYE_VMCNT(2 * LD) | 0x0070);
                    else __builtin_amdgcn_s_waitcnt(0x0070);
                }
                MOYE_BARRIER()
            }
            constexpr int dma_q = TILE == 128 ? dma_index_128(P, 2 * LD * SPS) : kLine ? dma_index_early(P, 2 * LD) : dma_index(P, 2 * LD * SPS, NPOS);
            if constexpr (dma_q >= 0) {
                constexpr int q = dma_q;  // 0 .. 2 LD SPS - 1
                // The 128 x 128 tile's k-steps of two 64-byte-row stages ask for the two halves of a 128-byte line one
                // right after the other, so that the second finds the line in the L1 the first brought it into (a stage
                // after the other, eight waves of two workgroups put 32 KiB between them: the L1's size); all loads of a
                // k-step are waited for together there (the ring holds two k-steps), so their order is free.
                constexpr bool kPairHalves = TILE == 128 && SPS == 2 && STAGES == 2 * SPS;
                constexpr int q_stage = kPairHalves ? q % 2 : q / (2 * LD), q_instr = kPairHalves ? q / 2 : q % (2 * LD);
                // in the drain a k-step of two stages may still have its first stage to request
                if (AHEAD || g_new + q_stage < nstages) {
                    int sl = slot + q_stage;
                    if (sl >= STAGES) sl -= STAGES;
                    dma1(g_new + q_stage, sl, std::integral_constant<int, q_instr>{});
                }
            }
            if (MORE) {
                constexpr int A0 = H * (NI - 1), B0 = (MI - 2) * NI;
                const uint32_t fa_at = AMAJ ? ta_byte : fa_byte, fb_at = BMAJ ? tb_byte : fb_byte;
                if constexpr (P >= A0 && P < A0 + H) load_frag(fa[i], fa_at, MOYE_BLK(i), o0, o1);  // the rows of the first phase: last use
                if constexpr (P >= H * NI && P < B0 && (P + 1) % NI == 0) load_frag(fa[i], fa_at, MOYE_BLK(i), o0, o1);  // a whole row: its end
                if constexpr (P >= NPOS - 2) load_frag(fa[i], fa_at, MOYE_BLK(i), o0, o1);          // the last two rows: last use
                if constexpr (P >= B0 && ((P - B0) & 1)) load_frag(fb[(P - B0) / 2], fb_at, MOYE_BLK((P - B0) / 2), o0, o1);
            }
        });
        slot = slot_n;
    };
    typedef std::integral_constant<bool, true> yes;
    typedef std::integral_constant<bool, false> no;
    int s = 0;
    slot = 0;
    for (; s * SPS + STAGES + SPS <= nstages; ++s) step(yes{}, yes{}, s);
    for (; s + 1 < nsteps; ++s) step(yes{}, no{}, s);
    step(no{}, no{}, s);
    // The accumulators were written by instructions whose latency the compiler does not know: let the last
    // ones retire before anything reads them.  The empty statements make every later read of an accumulator
    // depend on something that comes after the nops (volatile statements keep their order), so the epilogue's
    // v_accvgpr_read cannot be scheduled up to the MFMA that produced the value (seen in a variant of this
    // kernel: the read landed right behind the MFMA and returned the old value).  The build checks the
    // generated code for the other way this could go wrong: an accumulator register named, between MFMAs,
    // by anything that is not an MFMA (build.py, check_accumulator_hazards).
    asm volatile("s_nop 15\n\ts_nop 15\n\t; MOYE_ACC_SETTLED" ::: "memory");
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j) asm volatile("" : "+a"(acc[i][j]));
    __syncthreads();  // every wave is done with the operand ring before it becomes C patches (or the next tile's stages)

    if constexpr (kPersist) {
        const int64_t m_done = (int64_t)tm * BM + wm0, n_done = (int64_t)tn * BN + wn0;
        const int next = tile + (int)gridDim.x;
        if (next < ntiles) {
            locate(next);
            a_tile = static_cast<const char*>(p.A) + (int64_t)tm * BM * pitch_a;
            b_tile = static_cast<const char*>(p.B) + (int64_t)tn * BN * pitch_b;
            request_ring();
        }
        // the C patches: 32 rows of 64 16-bit values per wave (16 rows of 32-bit ones), 32 KiB beside the two stages.  (The lane number goes through
        // an empty statement so that nothing of the epilogue's per-lane address arithmetic is moved out of the loop over
        // the tiles: it would stay in registers through the k-loop, which has none to spare, and be spilled; a reload in
        // the epilogue waits for every store before it.)
        int lane_here = threadIdx.x & 63;
        asm volatile("" : "+v"(lane_here));
        store_c_tile<Out, MI, NI, false, kBias, kNoC, 16, sizeof(typename Out::type) == 2 ? 32 : 16>(p, acc, smem + STAGES * STAGE, wave, lane_here, m_done, n_done);
        if (next >= ntiles) break;
        tile = next;
        first_tile = false;
    } else {
        if constexpr (kOps)
            store_c_tile_general<Out, MI, NI, kRagged>(p, acc, smem, wave, lane, (int64_t)tm * BM + wm0, (int64_t)tn * BN + wn0);
        else
            store_c_tile<Out, MI, NI, kRagged, kBias, kRagged || kNoC>(p, acc, smem, wave, lane, (int64_t)tm * BM + wm0, (int64_t)tn * BN + wn0);
        break;
    }
    }  // for (;;)
#undef MOYE_BLK
#undef MOYE_I
#undef MOYE_J
#undef MOYE_VMCNT
#undef MOYE_BARRIER
}

template <typename In, typename Out, int WGN, bool kBias = false, bool kRagged = false, int TILE = 256, int AMAJ = 0, int BMAJ = 0, bool kOps = false, bool kNoC = false,
          bool kPersist = false>
static int32_t launch256_w4(const GemmArgs& a, GemmPlan& plan) {
    // all 160 KiB, or 128 KiB for two whole-line stages (64 KiB on 128 x 128 tiles); the persistent form: 32 KiB of C patches more
    constexpr int kLds = In::kRing * (TILE + TILE) * In::kRow + (kPersist ? 8 * 32 * 64 * 2 : 0);
    static LdsCap cap;
    unsigned grid = (unsigned)(a.tiles_m * a.tiles_n);
    if constexpr (kPersist) {
        // one workgroup per CU, a whole number of them per XCD
        const unsigned per_round = (unsigned)(plan.shape.cus / plan.shape.xcds * plan.shape.xcds);
        if (per_round && grid > per_round) grid = per_round;
    }
    plan.add_kernel(gemm_mfma_tn_256_w4<In, Out, WGN, kBias, kRagged, TILE, AMAJ, BMAJ, kOps, kNoC, kPersist>, a, grid,
                    (unsigned)(a.split > 1 ? a.split : 1), 128 * WGN, kLds, &cap, TILE, TILE, In::kRow * In::SPS, In::kDt, Out::kDt,
                    "gemm_mfma_tn_256_w4<%s,%s,waves=%d,bias=%d,ragged=%d,tile=%d,amaj=%d,bmaj=%d,ops=%d%s>", In::kName, Out::kName, 2 * WGN, (int)kBias, (int)kRagged,
                    TILE, AMAJ, BMAJ, (int)kOps, kPersist ? ",persist=1" : "");
    return MOYE_OK;
}

// The instances live in six translation units (so that they compile side by side): gemm_mfma256w4.hip (the 256 x 256
// tile with K-major operands), gemm_mfma256w4_majors.hip (operands that keep their M- / N-major form),
// gemm_mfma256w4_ops.hip (an element-wise operation in the epilogue), gemm_mfma256w4_persist.hip (one workgroup per CU
// that walks over the tiles), gemm_mfma128w4.hip (the 128 x 128 tile), gemm_mfma128w4_majors.hip (the 128 x 128 tile with
// M- / N-major operands).
int32_t launch256_w4_majors_dispatch(int32_t in_dt, int32_t out_dt, const GemmArgs& a, GemmPlan& plan);
int32_t launch256_w4_ops_dispatch(int32_t in_dt, int32_t out_dt, const GemmArgs& a, GemmPlan& plan);
int32_t launch128_w4_majors_dispatch(int32_t in_dt, int32_t out_dt, const GemmArgs& a, GemmPlan& plan);
int32_t launch256_w4_persist_dispatch(int32_t in_dt, int32_t out_dt, const GemmArgs& a, GemmPlan& plan);

}  // namespace moye

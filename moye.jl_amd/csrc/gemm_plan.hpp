// Host-side choice of CTA tile and K ranges for a gemm! whose tile is left to the library and that does not fill the chip
// with 256 x 256 tiles: a small cost model instead of thresholds.  Its per-k-tile times are fitted to bf16 timings on one
// MI355X with a different B on every call (operands that stay in the 256 MiB memory-side cache between calls run the
// kernels with one workgroup per CU up to 1.4 times faster, which real callers with several weight matrices do not see);
// the number of compute units that share the work is an argument (DeviceShape::cus).
//
//   time = 3 us + k-tiles per workgroup x t(tile, workgroups resident on a CU) [x rounds] + second pass of a K split
//
// with k-tiles of 128 bytes of K and, per k-tile and workgroup,
//   128 x 128 tiles (gemm_mfma128.hip, two workgroups fit a CU):   0.85 us alone on its CU, 1.08 us with a neighbour
//   64 x 64 tiles (gemm_mfma.hip, four fit):                       0.48 / 0.73 / 0.86 / 1.00 us for 1 / 2 / 3 / 4 on a CU
// (512 x 8192 x 8192 on 256 workgroups of 128 x 128: 111.8 us, in two K ranges on 512: 89.4; 1024 x 4096 x 14336 on 256:
// 198.5; 2048 x 4096 x 4096 on 512: 72.3; 2048^3 on 1024 workgroups of 64 x 64: 33.0; 512 x 4096 x 4096 on 512: 49.8), and a
// second pass that moves the fp32 partial products at about 6 TB/s (they are still in the caches) after 3 us of launch.
// Ragged tiles cost the 128 x 128 kernel 15 % more; the 64 x 64 kernel has no ragged form.  fp32 operands have their own
// per-k-tile times.
#pragma once

#include <cstdint>
#include <initializer_list>

namespace moye {

struct TileChoice {
    int tile;   // 64 or 128
    int split;  // K ranges
    double us;
};

inline double gemm_plan_cost(int tile, int split, int64_t M, int64_t N, int64_t k_bytes, bool f32_in, int cus) {
    const int64_t tiles = ((M + tile - 1) / tile) * ((N + tile - 1) / tile), ctas = tiles * split;
    const int slots = tile == 128 ? 2 : 4;
    // per k-tile and workgroup with 1 .. slots workgroups resident on a CU.  fp32 operands run on v_mfma_f32_16x16x4_f32,
    // an eighth of the 16-bit rate per byte of K, and are bound by it (2048^3 on 256 workgroups of 128 x 128: 124.5 us;
    // 4096 x 2048 x 4096 on 512: 465 us; 2560^3 on 400: 291 us; 3072^3 on 576: 522 us; 1024^3 on 256 workgroups of
    // 64 x 64: 25.7 us; 2048^3 on 1024: 156 us; 3072^3 on 2304: 509 us)
    static const double t128_16[3] = {0, 0.85, 1.08}, t64_16[5] = {0, 0.48, 0.73, 0.86, 1.00};
    static const double t128_32[3] = {0, 1.92, 3.62}, t64_32[5] = {0, 0.71, 1.25, 1.80, 2.40};
    const double* t = tile == 128 ? (f32_in ? t128_32 : t128_16) : (f32_in ? t64_32 : t64_16);
    const double ktiles = (double)((k_bytes / split + 127) / 128);
    // whole rounds of cus x slots workgroups, then the rest with fewer neighbours
    const int64_t full = ctas / ((int64_t)cus * slots), rest = ctas % ((int64_t)cus * slots);
    double us = 3.0 + ktiles * ((double)full * t[slots] + (rest ? t[(rest + cus - 1) / cus] : 0.0));
    if (tile == 128 && (M % 128 || N % 128 || k_bytes % 128)) us *= 1.15;
    if (split > 1) us += 3.0 + (2.0 * split * 4.0 + 4.0) * (double)M * (double)N / 6.0e6;
    return us;
}

// `max_split` = 1 forbids K ranges (no workspace); `fixed_split` > 0 asks for the best tile for that many ranges (the
// dispatch after the split has been made: k_bytes is then the whole K again, so both calls price the same candidates).
inline TileChoice gemm_plan(int64_t M, int64_t N, int64_t k_bytes, bool f32_in, bool tile64_ok, int max_split, int cus,
                            int fixed_split = 0) {
    TileChoice best{128, fixed_split > 0 ? fixed_split : 1, 1e30};
    for (int tile : {128, 64}) {
        if (tile == 64 && !tile64_ok) continue;
        // (one row of tiles: the 64 x 64 kernel has nothing to share B with, and the model does not know
        // -- bf16 64 x 65536 x 2048: 51.9 us against 43.3 on 128 x 128 tiles; 64 x 32768 x 2048: 26.7 against 27.4)
        if (tile == 64 && M <= 64) continue;
        for (int s = 1; s <= 16; s *= 2) {
            if (fixed_split > 0 && s != fixed_split) continue;
            if (fixed_split <= 0 && s > 1) {
                // equal ranges of whole k-tiles, at least four of them
                if (s > max_split || k_bytes % s || (k_bytes / s) % 128 || k_bytes / s < 512) continue;
            }
            const double us = gemm_plan_cost(tile, s, M, N, k_bytes, f32_in, cus);
            if (us < best.us) best = TileChoice{tile, s, us};
        }
    }
    return best;
}

// The same problem on 256 x 256 tiles, one workgroup per CU: 9 us + per k-tile 1.44 us in a round that fills the chip,
// 1.30 us in one that fills half of it or less, linear in between (bf16, B not cached: 512 x 8192 x 8192 on 64 tiles 176 us,
// in two K ranges 109.1, in four 79.4; with B cached 0.98 us per k-tile up to half the chip: fp16 K = 4096, 144 tiles 73 us,
// 128 72); a quarter more for the guarded instance (130 x 32768 x 4096 on 128 ragged tiles: 99 us).  `split` K ranges:
// that many times the workgroups with a share of K each, and the second pass.
inline double gemm_plan_cost_256(int64_t M, int64_t N, int64_t k_bytes, bool f32_in, bool ragged, int cus, int split = 1) {
    const int64_t tiles = ((M + 255) / 256) * ((N + 255) / 256) * split, full = tiles / cus, rest = tiles % cus;
    const int half = cus / 2 > 0 ? cus / 2 : 1;
    const double ktiles = (double)((k_bytes / split + 127) / 128);
    // (fp32: 7.05 us per k-tile however many CUs are busy: the matrix pipe alone sets the pace; 4096^3 909 us,
    // 3072^3 on 144 tiles 687 us, 4096 x 2048 x 4096 on 128 tiles 913 us)
    const double t_full = f32_in ? 7.05 : 1.44;
    const double t_rest = rest == 0 ? 0.0 : f32_in ? 7.05 : rest <= half ? 1.30 : 1.30 + (double)(rest - half) / (double)half * 0.14;
    double us = 9.0 + 6.0 * (double)(full + (rest ? 1 : 0) - 1) + ktiles * ((double)full * t_full + t_rest);
    if (ragged) us *= 1.25;
    if (split > 1) us += 3.0 + (2.0 * split * 4.0 + 4.0) * (double)M * (double)N / 6.0e6;  // the second pass, as in gemm_plan_cost
    return us;
}

// Everything left to the library (tile, waves, K ranges): the cheapest of 64 x 64 / 128 x 128 tiles with 1 .. max_split K
// ranges and of unsplit 256 x 256 tiles, which are considered from a quarter of the CUs' worth of tiles on.  The one
// place where tile and K ranges are chosen together: the workspace sizing and the dispatcher both take their answer
// from here.
inline TileChoice gemm_choose(int64_t M, int64_t N, int64_t k_bytes, bool f32_in, int max_split, int cus) {
    TileChoice best = gemm_plan(M, N, k_bytes, f32_in, M % 64 == 0 && N % 64 == 0 && k_bytes % 128 == 0, max_split, cus);
    const bool ragged = M % 256 || N % 256 || k_bytes % 128;
    if (((M + 255) / 256) * ((N + 255) / 256) >= cus / 4) {
        const double us = gemm_plan_cost_256(M, N, k_bytes, f32_in, ragged, cus);
        if (us <= best.us) best = TileChoice{256, 1, us};
    }
    // few whole 256 x 256 tiles and a long K: K ranges that bring the workgroups up to one per CU at most (bf16, a B that is
    // not cached: 512 x 8192 x 8192 on 128 x 128 tiles 111.8 us, in two ranges 89.4, on 256 x 256 tiles in four ranges
    // 79.4; 1024 x 4096 x 14336 198.5 / 145.2 / 113.5)
    if (!ragged && !f32_in) {
        const int64_t tiles = (M / 256) * (N / 256);
        for (int s = 2; s <= max_split && tiles * s <= cus; s *= 2) {
            if (k_bytes % s || (k_bytes / s) % 128 || k_bytes / s < 512) continue;
            const double us = gemm_plan_cost_256(M, N, k_bytes, f32_in, false, cus, s);
            if (us < best.us) best = TileChoice{256, s, us};
        }
    }
    return best;
}

// A short A (at most 64 rows, K in 16-byte pieces) goes to the kernel that streams B once and reads all of A per workgroup
// (gemm_mfma_skinny.hip) -- except more than 16 rows with many columns: that kernel then brings A out of the L2s as
// often as B out of memory and has one stage in flight per wave, which holds it near 5 TB/s of B, and 128 x 128 tiles,
// part empty as they are, take less once there are more of them than CUs (the hand-ordered instance with two workgroups
// on a CU) or, with a very short K, from three quarters of the CUs on.  bf16, us with a different B on every call (so
// that the memory-side cache does not serve it), that kernel / tiles: 64 x 65536 x 2048 63.8 / 47.1; 32 x 65536 x 2048
// 59.8 / 46.3; 64 x 36864 x 2048 44.9 / 40.0; 64 x 65536 x 4096 107.9 / 92.8; 64 x 65536 x 8192 201.3 / 181.5;
// 24 x 65536 x 1024 37.4 / 25.7; 64 x 262144 x 2048 265.0 / 209.7; 64 x 32768 x 1024 22.7 / 21.5; 64 x 24576 x 512
// 16.3 / 12.6.  But 64 x 32768 x 2048 32.7 / 36.7; 64 x 28672 x 8192 95.7 / 134.8; 48 x 49152 x 8192 132.8 / 149.3;
// 16 x 65536 x 2048 42.4 / 46 and 64 x 16384 x 2048 17.6 / 34.3.
// (fp32 operands stay on that kernel: their MFMA is slow enough for the empty part of a tile to cost more than it saves,
// 32 x 65536 x 1024 73.2 us against 138.5 on tiles, 64 x 65536 x 2048 165.2 against 252.3.)
inline bool gemm_short_m(int64_t M, int64_t N, int64_t k_bytes, bool f32_in, int cus) {
    if (M > 64 || k_bytes % 16) return false;
    if (M <= 16 || f32_in) return true;
    const int64_t tiles = (N + 127) / 128;
    if (tiles > cus) return !(k_bytes <= 8192 || (M > 48 && tiles >= 2 * (int64_t)cus));
    return !(4 * tiles >= 3 * (int64_t)cus && k_bytes <= 2048);
}

// The short-M kernel's workgroups take 16, 32 or (from 33 rows of A on) 64 rows of B and all of A, one workgroup on a CU
// at a time (its rings fill the LDS), and a workgroup streams its rows at about 64 GB/s whatever the others do (52 with
// 64 rows of B: two buffers instead of three).  A launch therefore takes as many rounds as its workgroups -- times the K
// ranges of a split -- need on the CUs: bf16 64 x 12288 x 8192 57.7 us on 384 workgroups of 32 rows, 46.3 on 192 of 64;
// 64 x 14336 x 4096 33.6 / 27.2; 48 x 10240 x 8192 51.1 / 40.1; but 64 x 8192 x 8192 31.1 on 256 of 32 rows, 43.8 on 128
// of 64; 64 x 4096 x 14336 42.0 unsplit on 256 workgroups of 16 rows, 47.0 in two K ranges on 512.  In microseconds:
// 4.5 (two launches of a split: 7.5, and never under 10.7) + the longer of all bytes at 6 TB/s and rounds x a workgroup's
// bytes at its rate.
inline double gemm_short_m_us(int64_t M, int64_t N, int64_t k_bytes, int cus, int ntw, int split) {
    const int mt = (int)((M + 15) / 16);
    const int64_t wgs = (N + 16 * ntw - 1) / (16 * ntw) * split, rounds = (wgs + cus - 1) / cus;
    const double wg_us = (double)(16 * ntw + 16 * mt) * ((double)k_bytes / split) / (ntw == 4 ? 52.0e3 : 64.0e3);
    const double floor_us = (double)(N + M) * (double)k_bytes / 6.0e6;
    const double t = floor_us > (double)rounds * wg_us ? floor_us : (double)rounds * wg_us;
    if (split > 1) return 7.5 + t > 10.7 ? 7.5 + t : 10.7;
    return 4.5 + t;
}
// 16-row blocks of B per workgroup for a launch in `split` K ranges: the cheapest, more rows on a tie (fewer rounds)
inline int gemm_short_m_ntw(int64_t M, int64_t N, int64_t k_bytes, int cus, int split, double* us = nullptr) {
    int best = 1;
    double best_us = 1e30;
    for (int ntw : {1, 2, 4}) {
        if (ntw == 4 && M <= 32) continue;
        const double t = gemm_short_m_us(M, N, k_bytes, cus, ntw, split);
        if (t <= best_us) { best_us = t; best = ntw; }
    }
    if (us) *us = best_us;
    return best;
}

}  // namespace moye

// copyto! on the device: layout-driven copy kernels for gfx950.
//
// Takes over the element loop of the reference's `copyto!`
// (src/algorithm/copy.jl:4-12,42-64 and :106-130): logical element i of src goes to logical
// element i of dst through both layouts.  Three kernels:
//   transpose_lds   rank-2, the unit-stride mode differs between src and dst: 128-bit global
//                   loads, 4x4 register transpose, XOR-swizzled LDS tile, 128-bit stores
//   copy_flat       both sides contiguous in the same order: 128-bit streaming copy
//   copy_generic    anything else: per-element gather/scatter with optional conversion
#include <algorithm>

#include "kernels.hpp"

namespace moye {

// ------------------------------------------------------------------------------------------
// transpose through a 64x64 LDS tile
// ------------------------------------------------------------------------------------------
// src(i, j) at i + j*lds   (i is the contiguous index),  dst(i, j) at i*ldd + j.
// One workgroup of 256 threads moves one 64x64 tile of 4-byte elements.
//
// LDS tile T[64 rows = i][16 chunks of 4 = j]; the chunk index is XORed with (row>>2)&15 so
// that the 16 lanes which write one float4 each to 16 different rows, and the 16 lanes which
// read 16 different chunks of one row, both touch all 64 banks exactly once.

constexpr int kTile = 64;
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));  // one 128-bit access

template <bool kSwizzle>
__device__ __forceinline__ int lds_chunk(int row, int chunk) {
    return kSwizzle ? (chunk ^ ((row >> 2) & 15)) : chunk;
}

// tile index -> (ti, tj): tiles are visited in square super-blocks of `sb` x `sb` tiles so
// that the workgroups in flight read and write runs of sb*256 contiguous bytes per row on
// BOTH sides (a plain row-major order makes one side hop a full leading dimension per tile).
__device__ __forceinline__ void tile_coords(int64_t t, int tiles_i, int tiles_j, int sb,
                                            int* ti, int* tj) {
    const int64_t per_band = (int64_t)sb * tiles_i;       // a band = sb tile-columns (j), all i
    const int band = (int)(t / per_band);
    const int64_t r = t - (int64_t)band * per_band;
    const int band_w = min(sb, tiles_j - band * sb);      // last band may be narrower
    const int blk = (int)(r / ((int64_t)sb * band_w));    // block of sb tiles along i
    const int64_t q = r - (int64_t)blk * sb * band_w;
    const int blk_h = min(sb, tiles_i - blk * sb);
    // inside a block: i fastest
    *ti = blk * sb + (int)(q % blk_h);
    *tj = band * sb + (int)(q / blk_h);
}

// One workgroup moves GI tiles that are neighbours along the source's contiguous index: every
// source row it touches is then a run of GI*256 bytes, which is what keeps DRAM pages open on the
// read side; all 4*GI loads of a thread are in flight before the first LDS write.
template <bool kSwizzle, int GI>
__global__ __launch_bounds__(256) void transpose_lds_b32(const uint32_t* __restrict__ src,
                                                         uint32_t* __restrict__ dst, int64_t lds_,
                                                         int64_t ldd, int groups_i, int tiles_j,
                                                         int sb, int64_t bs_src, int64_t bs_dst, int64_t bz_src, int64_t bz_dst) {
    extern __shared__ u32x4 tile[];  // GI tiles of 64 x 16 chunks
    src += (int64_t)blockIdx.y * bs_src + (int64_t)blockIdx.z * bz_src;  // blockIdx.y counts the matrices of a batch
    dst += (int64_t)blockIdx.y * bs_dst + (int64_t)blockIdx.z * bz_dst;
    int gi, tj;
    tile_coords(blockIdx.x, groups_i, tiles_j, sb, &gi, &tj);

    const int lane16 = threadIdx.x & 15;  // chunk of 4 along the contiguous index
    const int grp = threadIdx.x >> 4;     // 0..15

    // ---- load: rows j = 4*grp+q, columns i = 4*lane16 .. +3 of each tile ----
    const uint32_t* s = src + ((int64_t)tj * kTile + 4 * grp) * lds_ + (int64_t)gi * GI * kTile + 4 * lane16;
    u32x4 v[GI][4];
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int a = 0; a < GI; ++a)
            v[a][q] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(s + q * lds_ + a * kTile));

    // ---- 4x4 register transpose, store float4 over j into row i of the LDS tile ----
#pragma unroll
    for (int a = 0; a < GI; ++a)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int row = 4 * lane16 + e;  // i within the tile
            tile[a * 1024 + row * 16 + lds_chunk<kSwizzle>(row, grp)] = u32x4{v[a][0][e], v[a][1][e], v[a][2][e], v[a][3][e]};
        }
    __syncthreads();

    // ---- store: rows i = grp + 16*p, columns j = 4*lane16 .. +3 ----
    uint32_t* d = dst + ((int64_t)gi * GI * kTile + grp) * ldd + (int64_t)tj * kTile + 4 * lane16;
#pragma unroll
    for (int a = 0; a < GI; ++a)
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const int row = grp + 16 * p;
            const u32x4 w = tile[a * 1024 + row * 16 + lds_chunk<kSwizzle>(row, lane16)];
            __builtin_nontemporal_store(w, reinterpret_cast<u32x4*>(d + (int64_t)(a * kTile + 16 * p) * ldd));
        }
}

template <bool kSwizzle, int GI>
static int32_t launch_transpose(const uint32_t* s, uint32_t* d, int64_t lds_, int64_t ldd, int ti, int tj, hipStream_t st, int64_t bs_src = 0,
                              int64_t bs_dst = 0, int batch = 1, int64_t bz_src = 0, int64_t bz_dst = 0, int batch2 = 1) {
    auto kern = transpose_lds_b32<kSwizzle, GI>;
    constexpr int kLds = GI * kTile * kTile * 4;
    if (kLds > 48 * 1024) {
        static LdsCap cap;
        if (int32_t e = raise_lds_cap(cap, reinterpret_cast<const void*>(kern), kLds)) return e;
    }
    const int64_t groups = (int64_t)(ti / GI) * tj;
    if (groups >= (1 << 24)) return fail(MOYE_ERR_SHAPE, "copyto!: too many tiles for one launch (2^24 workgroups of 256)");
    // groups are walked with the source-contiguous index fastest in bands of 64 tile columns: the
    // workgroups in flight read whole source rows and write runs of several KiB per destination row
    kern<<<dim3((unsigned)groups, (unsigned)batch, (unsigned)batch2), 256, kLds, st>>>(s, d, lds_, ldd, ti / GI, tj, 64, bs_src, bs_dst, bz_src, bz_dst);
    MOYE_HIP_CHECK(hipGetLastError());
    return MOYE_OK;
}

// The form for large matrices: a workgroup moves GJ tiles that are neighbours along the DESTINATION's contiguous index
// (64 destination rows of GJ * 256 bytes each) and workgroups are numbered along that index first, so consecutive
// workgroups complete whole destination rows: 64 x ldd elements of contiguous memory per tj / GJ workgroups.  On this
// part writes are the side that needs the locality (measured on 16384^2, one side at a time with the other left out:
// reads of 256-byte pieces a pitch apart run at 6.9 TB/s whatever the order; writes run at 6.6-6.9 TB/s in this order
// against 5.1 with the source-contiguous index first), and fewer workgroups in flight do better than more: one per CU
// (6.25 TB/s) against two (6.15) or five (5.85), hence the LDS request above what the tiles need.
// 512 lanes, eight 16-byte loads each (same box, alternating runs, 16384^2: 256 lanes with sixteen loads each 6226-6252 GB/s,
// 512 with eight 6263-6300, 1024 with four 6236; two such workgroups per CU 6254; workgroups of 32 x 512, 128 x 256 or
// 64 x 512 elements 5.9-6.2; ordinary stores, or half of each row stored the ordinary way, 5.89; ordinary loads 5.90).
template <int GJ>
__global__ __launch_bounds__(512) void transpose_lds_b32_rows(const uint32_t* __restrict__ src, uint32_t* __restrict__ dst,
                                                              int64_t lds_, int64_t ldd, int groups_j, int64_t bs_src,
                                                              int64_t bs_dst, int64_t bz_src, int64_t bz_dst) {
    constexpr int TJ = GJ * kTile, JC = TJ / 4;  // the group's extent along j, in elements and in 16-byte chunks
    constexpr int NG = 512 / 16, NB = JC / NG;   // lanes come as 16 chunks along i x NG row quads along j
    static_assert(JC % NG == 0 && 512 % JC == 0, "group shape");
    extern __shared__ u32x4 tile[];  // 64 rows (i) of JC chunks (j), the chunk index XORed with (row / 4) % 8
    src += (int64_t)blockIdx.y * bs_src + (int64_t)blockIdx.z * bz_src;
    dst += (int64_t)blockIdx.y * bs_dst + (int64_t)blockIdx.z * bz_dst;
    const int gj = blockIdx.x % groups_j, ti = blockIdx.x / groups_j;
    const int ic = threadIdx.x & 15;  // chunk of 4 along i
    const int jr = threadIdx.x >> 4;  // 0..31: source rows 4 (jr + NG b) + q

    const uint32_t* s = src + ((int64_t)gj * TJ) * lds_ + (int64_t)ti * kTile + 4 * ic;
    u32x4 v[NB][4];
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int q = 0; q < 4; ++q)
            v[b][q] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(s + (int64_t)(4 * (jr + NG * b) + q) * lds_));
    // 4 x 4 register transpose: eight consecutive lanes write eight different rows-of-four, hence eight different bank groups
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int row = 4 * ic + e, c = jr + NG * b;
            tile[row * JC + (c ^ ((row >> 2) & 7))] = u32x4{v[b][0][e], v[b][1][e], v[b][2][e], v[b][3][e]};
        }
    __syncthreads();
    // ---- store: JC consecutive lanes write one destination row of the group (GJ * 256 bytes), 512 / JC rows per pass ----
    constexpr int RPP = 512 / JC;
    const int jc = threadIdx.x % JC, r0 = threadIdx.x / JC;
    uint32_t* d = dst + ((int64_t)ti * kTile + r0) * ldd + (int64_t)gj * TJ + 4 * jc;
#pragma unroll
    for (int p = 0; p < kTile / RPP; ++p) {
        const int row = r0 + RPP * p;
        const u32x4 w = tile[row * JC + (jc ^ ((row >> 2) & 7))];
        __builtin_nontemporal_store(w, reinterpret_cast<u32x4*>(d + (int64_t)(RPP * p) * ldd));
    }
}

template <int GJ>
static int32_t launch_transpose_rows(const uint32_t* s, uint32_t* d, int64_t lds_, int64_t ldd, int ti, int tj, hipStream_t st,
                                     int64_t bs_src = 0, int64_t bs_dst = 0, int batch = 1, int64_t bz_src = 0, int64_t bz_dst = 0, int batch2 = 1) {
    auto kern = transpose_lds_b32_rows<GJ>;
    constexpr int kLds = 96 * 1024;  // the tiles need GJ * 16 KiB; more than half of a CU's 160 KiB keeps it to one workgroup per CU
    static_assert(GJ * kTile * kTile * 4 <= kLds, "tiles fit");
    static LdsCap cap;
    if (int32_t e = raise_lds_cap(cap, reinterpret_cast<const void*>(kern), kLds)) return e;
    const int64_t groups = (int64_t)ti * (tj / GJ);
    if (groups >= (1 << 24)) return fail(MOYE_ERR_SHAPE, "copyto!: too many tiles for one launch (2^24 workgroups of 512)");
    kern<<<dim3((unsigned)groups, (unsigned)batch, (unsigned)batch2), 512, kLds, st>>>(s, d, lds_, ldd, tj / GJ, bs_src, bs_dst, bz_src, bz_dst);
    MOYE_HIP_CHECK(hipGetLastError());
    return MOYE_OK;
}

// ------------------------------------------------------------------------------------------
// the same for 8-byte elements (Float64 / Int64 matrices), destination rows first
// ------------------------------------------------------------------------------------------
// A workgroup moves 64 (i) x 128 (j) elements, 64 KiB like the 4-byte form: a source row's piece is 512 bytes (32 lanes of
// two elements), a destination row's 1 KiB (64 lanes of two elements).  A lane loads two elements along i from each of two
// neighbouring source rows, turns the 2 x 2 block in registers and writes two elements along j into each of two LDS rows;
// the chunk index of an LDS row is XORed with (row / 2) % 8.
constexpr int kTileJ64 = 128;
__global__ __launch_bounds__(512) void transpose_lds_b64_rows(const uint64_t* __restrict__ src, uint64_t* __restrict__ dst, int64_t lds_,
                                                              int64_t ldd, int groups_j, int64_t bs_src, int64_t bs_dst, int64_t bz_src, int64_t bz_dst) {
    constexpr int JC = kTileJ64 / 2;            // 16-byte chunks (two elements) per LDS row
    constexpr int NG = 512 / 32, NB = JC / NG;  // lanes come as 32 chunks along i x NG row pairs along j
    extern __shared__ u32x4 tile[];             // 64 rows (i) of JC chunks (j)
    src += (int64_t)blockIdx.y * bs_src + (int64_t)blockIdx.z * bz_src;
    dst += (int64_t)blockIdx.y * bs_dst + (int64_t)blockIdx.z * bz_dst;
    const int gj = blockIdx.x % groups_j, ti = blockIdx.x / groups_j;
    const int ic = threadIdx.x & 31;  // chunk of 2 along i
    const int jr = threadIdx.x >> 5;  // 0..15: source rows 2 (jr + NG b) + q
    const uint64_t* s = src + ((int64_t)gj * kTileJ64) * lds_ + (int64_t)ti * kTile + 2 * ic;
    u32x4 v[NB][2];
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int q = 0; q < 2; ++q)
            v[b][q] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(s + (int64_t)(2 * (jr + NG * b) + q) * lds_));
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const int row = 2 * ic + e, c = jr + NG * b;
            tile[row * JC + (c ^ ((row >> 1) & 7))] = u32x4{v[b][0][2 * e], v[b][0][2 * e + 1], v[b][1][2 * e], v[b][1][2 * e + 1]};
        }
    __syncthreads();
    // ---- store: JC consecutive lanes write one destination row of the group (1 KiB), 512 / JC rows per pass ----
    constexpr int RPP = 512 / JC;
    const int jc = threadIdx.x % JC, r0 = threadIdx.x / JC;
    uint64_t* d = dst + ((int64_t)ti * kTile + r0) * ldd + (int64_t)gj * kTileJ64 + 2 * jc;
#pragma unroll
    for (int p = 0; p < kTile / RPP; ++p) {
        const int row = r0 + RPP * p;
        const u32x4 w = tile[row * JC + (jc ^ ((row >> 1) & 7))];
        __builtin_nontemporal_store(w, reinterpret_cast<u32x4*>(d + (int64_t)(RPP * p) * ldd));
    }
}

static int32_t launch_transpose64_rows(const uint64_t* s, uint64_t* d, int64_t lds_, int64_t ldd, int ti, int tj, hipStream_t st,
                                       int64_t bs_src = 0, int64_t bs_dst = 0, int batch = 1, int64_t bz_src = 0, int64_t bz_dst = 0, int batch2 = 1) {
    auto kern = transpose_lds_b64_rows;
    constexpr int kLds = 96 * 1024;  // the tile needs 64 KiB; the request keeps it to one workgroup per CU
    static LdsCap cap;
    if (int32_t e = raise_lds_cap(cap, reinterpret_cast<const void*>(kern), kLds)) return e;
    const int64_t groups = (int64_t)ti * tj;
    if (groups >= (1 << 24)) return fail(MOYE_ERR_SHAPE, "copyto!: too many tiles for one launch (2^24 workgroups of 512)");
    kern<<<dim3((unsigned)groups, (unsigned)batch, (unsigned)batch2), 512, kLds, st>>>(s, d, lds_, ldd, tj, bs_src, bs_dst, bz_src, bz_dst);
    MOYE_HIP_CHECK(hipGetLastError());
    return MOYE_OK;
}

// ------------------------------------------------------------------------------------------
// the same for 2-byte elements (fp16 / bf16 matrices)
// ------------------------------------------------------------------------------------------
// A 64 x 64 tile is 64 source rows (j) of 128 bytes.  Rows go to LDS as they come, 16 bytes per lane,
// with the 16-byte chunk index XORed with j / 8; a lane then gathers the 8 values S[8c .. 8c+7][i]
// with 2-byte LDS reads (for a wave: 8 values of i, 8 values of c -> 32 different banks) and stores them
// as one 16-byte piece of destination row i, 8 lanes per 128-byte run.
template <int GI>
__global__ __launch_bounds__(256) void transpose_lds_b16(const uint16_t* __restrict__ src, uint16_t* __restrict__ dst,
                                                         int64_t lds_, int64_t ldd, int groups_i, int tiles_j, int sb,
                                                         int64_t bs_src, int64_t bs_dst, int64_t bz_src, int64_t bz_dst) {
    extern __shared__ u32x4 tile[];  // GI tiles of 64 rows x 8 chunks
    src += (int64_t)blockIdx.y * bs_src + (int64_t)blockIdx.z * bz_src;
    dst += (int64_t)blockIdx.y * bs_dst + (int64_t)blockIdx.z * bz_dst;
    int gi, tj;
    tile_coords(blockIdx.x, groups_i, tiles_j, sb, &gi, &tj);
    const int v = threadIdx.x & 7;   // 16-byte chunk inside a 128-byte run
    const int r = threadIdx.x >> 3;  // 0..31

    // ---- load: rows j = r and r + 32, elements i = 8v .. 8v+7 of each tile ----
    const uint16_t* s = src + ((int64_t)tj * kTile + r) * lds_ + (int64_t)gi * GI * kTile + 8 * v;
    u32x4 x[GI][2];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int a = 0; a < GI; ++a)
            x[a][h] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(s + (int64_t)(32 * h) * lds_ + a * kTile));
#pragma unroll
    for (int a = 0; a < GI; ++a)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int j = r + 32 * h;
            tile[a * 512 + j * 8 + (v ^ (j >> 3))] = x[a][h];
        }
    __syncthreads();

    // ---- store: destination rows i = r and r + 32, elements j = 8v .. 8v+7 ----
    const uint16_t* lds16 = reinterpret_cast<const uint16_t*>(tile);
    uint16_t* d = dst + ((int64_t)gi * GI * kTile + r) * ldd + (int64_t)tj * kTile + 8 * v;
#pragma unroll
    for (int a = 0; a < GI; ++a)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int i = r + 32 * h;
            uint16_t w[8];
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                const int j = 8 * v + q;  // j / 8 == v
                w[q] = lds16[a * 4096 + j * 64 + ((((i >> 3) ^ v) << 3) | (i & 7))];
            }
            u32x4 o;
            o.x = w[0] | ((uint32_t)w[1] << 16);
            o.y = w[2] | ((uint32_t)w[3] << 16);
            o.z = w[4] | ((uint32_t)w[5] << 16);
            o.w = w[6] | ((uint32_t)w[7] << 16);
            __builtin_nontemporal_store(o, reinterpret_cast<u32x4*>(d + (int64_t)(a * kTile + 32 * h) * ldd));
        }
}

template <int GI>
static int32_t launch_transpose16(const uint16_t* s, uint16_t* d, int64_t lds_, int64_t ldd, int ti, int tj, hipStream_t st, int64_t bs_src = 0,
                              int64_t bs_dst = 0, int batch = 1, int64_t bz_src = 0, int64_t bz_dst = 0, int batch2 = 1) {
    auto kern = transpose_lds_b16<GI>;
    constexpr int kLds = GI * kTile * kTile * 2;
    if (kLds > 48 * 1024) {
        static LdsCap cap;
        if (int32_t e = raise_lds_cap(cap, reinterpret_cast<const void*>(kern), kLds)) return e;
    }
    const int64_t groups = (int64_t)(ti / GI) * tj;
    if (groups >= (1 << 24)) return fail(MOYE_ERR_SHAPE, "copyto!: too many tiles for one launch (2^24 workgroups of 256)");
    kern<<<dim3((unsigned)groups, (unsigned)batch, (unsigned)batch2), 256, kLds, st>>>(s, d, lds_, ldd, ti / GI, tj, 64, bs_src, bs_dst, bz_src, bz_dst);
    MOYE_HIP_CHECK(hipGetLastError());
    return MOYE_OK;
}

// The same with destination rows first (see transpose_lds_b32_rows): a workgroup moves GJ tiles that are neighbours
// along the destination's contiguous index, 64 destination rows of GJ * 128 bytes, and workgroups are numbered along that
// index first; one workgroup per CU.
template <int GJ>
__global__ __launch_bounds__(256) void transpose_lds_b16_rows(const uint16_t* __restrict__ src, uint16_t* __restrict__ dst,
                                                              int64_t lds_, int64_t ldd, int groups_j, int64_t bs_src,
                                                              int64_t bs_dst, int64_t bz_src, int64_t bz_dst) {
    extern __shared__ u32x4 tile[];  // GJ tiles of 64 rows x 8 chunks
    src += (int64_t)blockIdx.y * bs_src + (int64_t)blockIdx.z * bz_src;
    dst += (int64_t)blockIdx.y * bs_dst + (int64_t)blockIdx.z * bz_dst;
    const int gj = blockIdx.x % groups_j, ti = blockIdx.x / groups_j;
    const int v = threadIdx.x & 7;   // 16-byte chunk inside a 128-byte run
    const int r = threadIdx.x >> 3;  // 0..31
    const uint16_t* s = src + ((int64_t)gj * GJ * kTile + r) * lds_ + (int64_t)ti * kTile + 8 * v;
    u32x4 x[GJ][2];
#pragma unroll
    for (int b = 0; b < GJ; ++b)
#pragma unroll
        for (int h = 0; h < 2; ++h)
            x[b][h] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(s + (int64_t)(b * kTile + 32 * h) * lds_));
#pragma unroll
    for (int b = 0; b < GJ; ++b)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int j = r + 32 * h;
            tile[b * 512 + j * 8 + (v ^ (j >> 3))] = x[b][h];
        }
    __syncthreads();
    const uint16_t* lds16 = reinterpret_cast<const uint16_t*>(tile);
    uint16_t* d = dst + ((int64_t)ti * kTile + r) * ldd + (int64_t)gj * GJ * kTile + 8 * v;
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int b = 0; b < GJ; ++b) {
            const int i = r + 32 * h;
            uint16_t w[8];
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                const int j = 8 * v + q;  // j / 8 == v
                w[q] = lds16[b * 4096 + j * 64 + ((((i >> 3) ^ v) << 3) | (i & 7))];
            }
            u32x4 o;
            o.x = w[0] | ((uint32_t)w[1] << 16);
            o.y = w[2] | ((uint32_t)w[3] << 16);
            o.z = w[4] | ((uint32_t)w[5] << 16);
            o.w = w[6] | ((uint32_t)w[7] << 16);
            __builtin_nontemporal_store(o, reinterpret_cast<u32x4*>(d + (int64_t)(32 * h) * ldd + b * kTile));
        }
}

template <int GJ>
static int32_t launch_transpose16_rows(const uint16_t* s, uint16_t* d, int64_t lds_, int64_t ldd, int ti, int tj, hipStream_t st,
                                       int64_t bs_src = 0, int64_t bs_dst = 0, int batch = 1, int64_t bz_src = 0, int64_t bz_dst = 0, int batch2 = 1) {
    auto kern = transpose_lds_b16_rows<GJ>;
    constexpr int kLds = 96 * 1024;  // the tiles need GJ * 8 KiB; the request keeps it to one workgroup per CU
    static_assert(GJ * kTile * kTile * 2 <= kLds, "tiles fit");
    static LdsCap cap;
    if (int32_t e = raise_lds_cap(cap, reinterpret_cast<const void*>(kern), kLds)) return e;
    const int64_t groups = (int64_t)ti * (tj / GJ);
    if (groups >= (1 << 24)) return fail(MOYE_ERR_SHAPE, "copyto!: too many tiles for one launch (2^24 workgroups of 256)");
    kern<<<dim3((unsigned)groups, (unsigned)batch, (unsigned)batch2), 256, kLds, st>>>(s, d, lds_, ldd, tj / GJ, bs_src, bs_dst, bz_src, bz_dst);
    MOYE_HIP_CHECK(hipGetLastError());
    return MOYE_OK;
}

// ------------------------------------------------------------------------------------------
// the same for 1-byte elements (fp8 matrices, bytes)
// ------------------------------------------------------------------------------------------
// A sub-tile is 256 source rows (j) of 64 bytes (i); a workgroup moves GI of them that are neighbours along i.  Rows go
// to LDS as they come, 16 bytes per lane.  A lane then owns a block of 4 (i) x 16 (j) bytes: it reads the 16 rows'
// dwords, transposes the bytes in registers and stores four 16-byte pieces, one to each of four consecutive
// destination rows.  A 64-byte LDS row spans 16 of the 64 banks, so rows that are a multiple of four apart share
// banks; the lanes of a wave read rows 16 apart, hence rows are stored with their two low index bits XORed with
// bits 4-5: the four rows a wave reads at once then lie in four different bank groups.
constexpr int kTileJ8 = 256;
__device__ __forceinline__ int lds_row_b8(int j) { return (j & ~3) | ((j & 3) ^ ((j >> 4) & 3)); }

template <int GI>
__global__ __launch_bounds__(256) void transpose_lds_b8(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst, int64_t lds_,
                                                        int64_t ldd, int groups_i, int tiles_j, int sb, int64_t bs_src,
                                                        int64_t bs_dst, int64_t bz_src, int64_t bz_dst) {
    extern __shared__ u32x4 tile[];  // GI sub-tiles of 256 rows x 4 chunks
    src += (int64_t)blockIdx.y * bs_src + (int64_t)blockIdx.z * bz_src;
    dst += (int64_t)blockIdx.y * bs_dst + (int64_t)blockIdx.z * bz_dst;
    int gi, tj;
    tile_coords(blockIdx.x, groups_i, tiles_j, sb, &gi, &tj);
    const int v = threadIdx.x & 3;   // 16-byte chunk of a 64-byte row
    const int r = threadIdx.x >> 2;  // 0..63

    // ---- load: rows j = r + 64 h, bytes i = 16 v .. 16 v + 15 of each sub-tile ----
    const uint8_t* s = src + ((int64_t)tj * kTileJ8 + r) * lds_ + (int64_t)gi * GI * kTile + 16 * v;
    u32x4 x[GI][4];
#pragma unroll
    for (int h = 0; h < 4; ++h)
#pragma unroll
        for (int a = 0; a < GI; ++a)
            x[a][h] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(s + (int64_t)(64 * h) * lds_ + a * kTile));
#pragma unroll
    for (int a = 0; a < GI; ++a)
#pragma unroll
        for (int h = 0; h < 4; ++h) tile[a * 1024 + lds_row_b8(r + 64 * h) * 4 + v] = x[a][h];
    __syncthreads();

    // ---- store: destination rows i = 4 ib .. 4 ib + 3, bytes j = 16 c .. 16 c + 15 ----
    const uint32_t* lds32 = reinterpret_cast<const uint32_t*>(tile);
    const int ib = threadIdx.x & 15, c = threadIdx.x >> 4;
    uint8_t* d = dst + ((int64_t)gi * GI * kTile + 4 * ib) * ldd + (int64_t)tj * kTileJ8 + 16 * c;
#pragma unroll
    for (int a = 0; a < GI; ++a) {
        uint32_t w[16];
#pragma unroll
        for (int q = 0; q < 16; ++q) w[q] = lds32[a * 4096 + lds_row_b8(16 * c + q) * 16 + ib];  // S[16 c + q][4 ib .. 4 ib + 3]
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            u32x4 o;
#pragma unroll
            for (int g = 0; g < 4; ++g)
                o[g] = ((w[4 * g] >> (8 * e)) & 0xffu) | (((w[4 * g + 1] >> (8 * e)) & 0xffu) << 8) |
                       (((w[4 * g + 2] >> (8 * e)) & 0xffu) << 16) | (((w[4 * g + 3] >> (8 * e)) & 0xffu) << 24);
            __builtin_nontemporal_store(o, reinterpret_cast<u32x4*>(d + (int64_t)(a * kTile + e) * ldd));
        }
    }
}

// The same for matrices whose source rows come in whole runs of 256 bytes: a workgroup moves a tile of 256 x 256 bytes,
// four of the sub-tiles above side by side along i, and both sides move whole 256-byte runs per instruction: a load
// instruction reads four source rows of 256 bytes (sixteen lanes each), a store instruction writes four destination rows
// of 256 bytes.  (The kernel above reads and writes 64-byte pieces of sixteen rows per instruction: half lines, which the
// address path takes several times slower, and four waves complete a destination row's run between them.)  A lane of the
// store phase owns 4 (i) x 16 (j) bytes of each sub-tile as above; the sixteen lanes of a run read LDS rows 16 apart and
// the four runs of a wave four neighbouring dwords, so besides the row swizzle above the dword position of a row is
// XORed with 4 ((j / 64) % 4): the 64 dwords a wave reads at once then lie in 64 banks.  The 4 x 4 byte blocks are
// transposed with v_perm_b32, eight per block.
// Workgroups are numbered along the destination's contiguous index first (see transpose_lds_b32_rows), one per CU.
__device__ __forceinline__ void transpose_bytes_4x4(uint32_t r0, uint32_t r1, uint32_t r2, uint32_t r3, uint32_t (&o)[4]) {
    const uint32_t t0 = __builtin_amdgcn_perm(r1, r0, 0x05010400u), t1 = __builtin_amdgcn_perm(r1, r0, 0x07030602u);
    const uint32_t t2 = __builtin_amdgcn_perm(r3, r2, 0x05010400u), t3 = __builtin_amdgcn_perm(r3, r2, 0x07030602u);
    o[0] = __builtin_amdgcn_perm(t2, t0, 0x05040100u);
    o[1] = __builtin_amdgcn_perm(t2, t0, 0x07060302u);
    o[2] = __builtin_amdgcn_perm(t3, t1, 0x05040100u);
    o[3] = __builtin_amdgcn_perm(t3, t1, 0x07060302u);
}

__global__ __launch_bounds__(256) void transpose_lds_b8_wide(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst, int64_t lds_,
                                                             int64_t ldd, int tiles_j, int64_t bs_src, int64_t bs_dst, int64_t bz_src, int64_t bz_dst) {
    extern __shared__ u32x4 tile[];  // four sub-tiles of 256 rows x 4 chunks
    src += (int64_t)blockIdx.y * bs_src + (int64_t)blockIdx.z * bz_src;
    dst += (int64_t)blockIdx.y * bs_dst + (int64_t)blockIdx.z * bz_dst;
    const int tj = blockIdx.x % tiles_j, gi = blockIdx.x / tiles_j;
    // ---- load: rows j = r + 16 h, bytes i = 64 a + 16 v .. + 15: a row's sixteen lanes read 256 contiguous bytes ----
    const int v = threadIdx.x & 3, a = (threadIdx.x >> 2) & 3, r = threadIdx.x >> 4;
    const uint8_t* s = src + ((int64_t)tj * kTileJ8 + r) * lds_ + (int64_t)gi * 4 * kTile + 64 * a + 16 * v;
    u32x4 x[16];
#pragma unroll
    for (int h = 0; h < 16; ++h) x[h] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(s + (int64_t)(16 * h) * lds_));
#pragma unroll
    for (int h = 0; h < 16; ++h) {
        const int j = r + 16 * h;
        tile[a * 1024 + lds_row_b8(j) * 4 + (v ^ ((j >> 6) & 3))] = x[h];
    }
    __syncthreads();

    // ---- store: destination rows i = 64 a + 4 ib .. + 3, bytes j = 16 c .. 16 c + 15: sixteen lanes write 256 contiguous bytes ----
    const uint32_t* lds32 = reinterpret_cast<const uint32_t*>(tile);
    const int c = threadIdx.x & 15, ib = threadIdx.x >> 4;
    uint8_t* d = dst + ((int64_t)gi * 4 * kTile + 4 * ib) * ldd + (int64_t)tj * kTileJ8 + 16 * c;
    const int pos = ib ^ ((c >> 2) << 2);  // (16 c + q) / 64 == c / 4
#pragma unroll
    for (int a2 = 0; a2 < 4; ++a2) {
        uint32_t w[16];
#pragma unroll
        for (int q = 0; q < 16; ++q) w[q] = lds32[a2 * 4096 + lds_row_b8(16 * c + q) * 16 + pos];  // S[16 c + q][64 a2 + 4 ib .. + 3]
        uint32_t o[4][4];  // [g][e]
#pragma unroll
        for (int g = 0; g < 4; ++g) transpose_bytes_4x4(w[4 * g], w[4 * g + 1], w[4 * g + 2], w[4 * g + 3], o[g]);
#pragma unroll
        for (int e = 0; e < 4; ++e)
            __builtin_nontemporal_store(u32x4{o[0][e], o[1][e], o[2][e], o[3][e]}, reinterpret_cast<u32x4*>(d + (int64_t)(a2 * kTile + e) * ldd));
    }
}

static int32_t launch_transpose8_wide(const uint8_t* s, uint8_t* d, int64_t lds_, int64_t ldd, int ti, int tj, hipStream_t st, int64_t bs_src = 0,
                                      int64_t bs_dst = 0, int batch = 1, int64_t bz_src = 0, int64_t bz_dst = 0, int batch2 = 1) {
    auto kern = transpose_lds_b8_wide;
    constexpr int kLds = 96 * 1024;  // the tile needs 64 KiB; the request keeps it to one workgroup per CU (+2-3 % on large matrices)
    static_assert(4 * kTileJ8 * kTile <= kLds, "the tile fits");
    static LdsCap cap;
    if (int32_t e = raise_lds_cap(cap, reinterpret_cast<const void*>(kern), kLds)) return e;
    const int64_t groups = (int64_t)(ti / 4) * tj;
    if (groups >= (1 << 24)) return fail(MOYE_ERR_SHAPE, "copyto!: too many tiles for one launch (2^24 workgroups of 256)");
    kern<<<dim3((unsigned)groups, (unsigned)batch, (unsigned)batch2), 256, kLds, st>>>(s, d, lds_, ldd, tj, bs_src, bs_dst, bz_src, bz_dst);
    MOYE_HIP_CHECK(hipGetLastError());
    return MOYE_OK;
}

template <int GI>
static int32_t launch_transpose8(const uint8_t* s, uint8_t* d, int64_t lds_, int64_t ldd, int ti, int tj, hipStream_t st, int64_t bs_src = 0,
                              int64_t bs_dst = 0, int batch = 1, int64_t bz_src = 0, int64_t bz_dst = 0, int batch2 = 1) {
    auto kern = transpose_lds_b8<GI>;
    constexpr int kLds = GI * kTileJ8 * kTile;
    if (kLds > 48 * 1024) {
        static LdsCap cap;
        if (int32_t e = raise_lds_cap(cap, reinterpret_cast<const void*>(kern), kLds)) return e;
    }
    const int64_t groups = (int64_t)(ti / GI) * tj;
    if (groups >= (1 << 24)) return fail(MOYE_ERR_SHAPE, "copyto!: too many tiles for one launch (2^24 workgroups of 256)");
    kern<<<dim3((unsigned)groups, (unsigned)batch, (unsigned)batch2), 256, kLds, st>>>(s, d, lds_, ldd, ti / GI, tj, 64, bs_src, bs_dst, bz_src, bz_dst);
    MOYE_HIP_CHECK(hipGetLastError());
    return MOYE_OK;
}

// ------------------------------------------------------------------------------------------
// contiguous streaming copy, 16 bytes per lane per step
// ------------------------------------------------------------------------------------------
// One 16-byte piece per lane, one workgroup per 4 KiB, non-temporal on both sides, no loop: measured on 1 GiB
// 6.56 TB/s against 6.09 for workgroups that walk 16 KiB chunks with four pieces of a lane in flight (6.04-6.25 with two
// or four pieces per lane and no loop, 4.3 with eight; 6.2 without the non-temporal hints).
__global__ __launch_bounds__(256) void copy_flat_b128(const u32x4* __restrict__ src,
                                                      u32x4* __restrict__ dst, int64_t n16) {
    const int64_t i = flat_piece();
    if (i < n16) __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
}

__global__ __launch_bounds__(256) void copy_flat_bytes(const uint8_t* __restrict__ src,
                                                       uint8_t* __restrict__ dst, int64_t n) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) dst[i] = src[i];
}

// ------------------------------------------------------------------------------------------
// generic gather/scatter with conversion
// ------------------------------------------------------------------------------------------
struct FlatLayout {
    int32_t rank;
    int64_t shape[MOYE_MAX_RANK];
    int64_t stride[MOYE_MAX_RANK];
};

// colexicographic decomposition of a 0-based linear index (src/stride.jl:20-31)
__device__ __forceinline__ int64_t layout_offset(const FlatLayout& l, int64_t i) {
    int64_t off = 0;
#pragma unroll 1
    for (int m = 0; m < l.rank; ++m) {
        const int64_t s = l.shape[m];
        const int64_t q = i / s;
        off += (i - q * s) * l.stride[m];
        i = q;
    }
    return off;
}

__device__ __forceinline__ float bf16_to_f32(uint16_t h) { return __uint_as_float((uint32_t)h << 16); }

// round to nearest even, a NaN made quiet: v_cvt_pk_bf16_f32 (the same bits as the integer form for all 2^32 inputs)
__device__ __forceinline__ uint16_t f32_to_bf16(float f) { return __builtin_bit_cast(uint16_t, (__bf16)f); }

// OCP e4m3fn <-> fp32 through v_cvt_f32_fp8 / v_cvt_pk_fp8_f32.  Narrowing rounds to nearest even and turns NaN, infinities
// and everything beyond the last tie (|x| > 464) into NaN, as the integer form these replaced did: a one-off kernel compared
// the two over all 2^32 inputs (and all 256 the other way) on the hardware.  They differ in one thing only, the sign of a NaN:
// the instructions make every NaN negative, here a NaN keeps the sign it came with.
__device__ __forceinline__ float f8e4m3_to_f32(uint8_t b) {
    return b == 0x7f ? __uint_as_float(0x7fc00000u) : __builtin_amdgcn_cvt_f32_fp8((int)b, 0);
}
__device__ __forceinline__ uint8_t f32_to_f8e4m3(float f) {
    const uint8_t h = (uint8_t)(__builtin_amdgcn_cvt_pk_fp8_f32(f, f, 0, false) & 0xff);
    return f != f ? (uint8_t)(((__float_as_uint(f) >> 24) & 0x80) | 0x7f) : h;
}

template <int kDt>
__device__ __forceinline__ double load_as_f64(const char* p) {
    if constexpr (kDt == MOYE_F32) return (double)*reinterpret_cast<const float*>(p);
    else if constexpr (kDt == MOYE_F16) return (double)(float)*reinterpret_cast<const _Float16*>(p);
    else if constexpr (kDt == MOYE_BF16) return (double)bf16_to_f32(*reinterpret_cast<const uint16_t*>(p));
    else if constexpr (kDt == MOYE_F8E4M3) return (double)f8e4m3_to_f32(*reinterpret_cast<const uint8_t*>(p));
    else return *reinterpret_cast<const double*>(p);
}

// Every narrower float format here embeds exactly in fp32 and fp32 in fp64, so one rounding
// step per conversion happens below (f64 -> f16/bf16/f8 goes through f32 only when the source
// was at most f32, which is then exact).
template <int kDt>
__device__ __forceinline__ void store_from(char* p, double v, bool src_is_f64) {
    if constexpr (kDt == MOYE_F64) *reinterpret_cast<double*>(p) = v;
    else if constexpr (kDt == MOYE_F32) *reinterpret_cast<float*>(p) = (float)v;
    else if constexpr (kDt == MOYE_F16)
        *reinterpret_cast<_Float16*>(p) = src_is_f64 ? (_Float16)v : (_Float16)(float)v;
    else if constexpr (kDt == MOYE_BF16) *reinterpret_cast<uint16_t*>(p) = f32_to_bf16((float)v);
    else *reinterpret_cast<uint8_t*>(p) = f32_to_f8e4m3((float)v);
}

// copyto_if! (src/algorithm/copy.jl:4-16): element i moves only where the mask's logical element i is nonzero
struct Mask {
    const uint8_t* ptr;  // null = every element moves
    FlatLayout l;
};
__device__ __forceinline__ bool masked_out(const Mask& m, int64_t i) { return m.ptr && !m.ptr[layout_offset(m.l, i)]; }

// layouts of one shape mode by mode, few enough pieces for 32-bit indices
static bool same_modes_32(const FlatLayout& a, const FlatLayout& b, int64_t n) {
    if (a.rank != b.rank || n >= ((int64_t)1 << 31)) return false;
    for (int m = 0; m < a.rank; ++m)
        if (a.shape[m] != b.shape[m] || a.shape[m] <= 0) return false;
    return true;
}

template <int kBytes>
__global__ __launch_bounds__(256) void copy_generic_bits(const char* __restrict__ src,
                                                         char* __restrict__ dst, FlatLayout ls,
                                                         FlatLayout ld, int64_t n, Mask mask) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        if (masked_out(mask, i)) continue;
        const char* s = src + layout_offset(ls, i) * kBytes;
        char* d = dst + layout_offset(ld, i) * kBytes;
        if constexpr (kBytes == 1) *reinterpret_cast<uint8_t*>(d) = *reinterpret_cast<const uint8_t*>(s);
        else if constexpr (kBytes == 2) *reinterpret_cast<uint16_t*>(d) = *reinterpret_cast<const uint16_t*>(s);
        else if constexpr (kBytes == 4) *reinterpret_cast<uint32_t*>(d) = *reinterpret_cast<const uint32_t*>(s);
        else if constexpr (kBytes == 8) *reinterpret_cast<uint64_t*>(d) = *reinterpret_cast<const uint64_t*>(s);
        else *reinterpret_cast<u32x4*>(d) = *reinterpret_cast<const u32x4*>(s);
    }
}

// The same for two layouts of one shape, mode by mode, and fewer than 2^31 pieces: the index is taken apart once, with
// 32-bit divisions, and the coordinates are weighed with both sides' strides (the general form divides 64-bit numbers
// twice per mode, which is most of its time: [16, 2048, 32, 128] -> [16, 32, 2048, 128] fp32 240 us against 172 this way).
// kStream: non-temporal accesses, for arrays far beyond the caches.
template <int kBytes, bool kStream>
__global__ __launch_bounds__(256) void copy_generic_bits_same(const char* __restrict__ src, char* __restrict__ dst, FlatLayout ls, FlatLayout ld,
                                                              uint32_t n) {
    typedef std::conditional_t<kBytes == 16, u32x4, std::conditional_t<kBytes == 8, uint64_t, std::conditional_t<kBytes == 4, uint32_t,
            std::conditional_t<kBytes == 2, uint16_t, uint8_t>>>> piece;
    const uint32_t stride = gridDim.x * blockDim.x;
    for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        int64_t so = 0, dof = 0;
        uint32_t rest = i;
#pragma unroll 1
        for (int m = 0; m < ls.rank; ++m) {
            const uint32_t extent = (uint32_t)ls.shape[m], q = rest / extent, c = rest - q * extent;
            so += (int64_t)c * ls.stride[m];
            dof += (int64_t)c * ld.stride[m];
            rest = q;
        }
        const piece* s = reinterpret_cast<const piece*>(src + so * kBytes);
        piece* d = reinterpret_cast<piece*>(dst + dof * kBytes);
        if constexpr (kStream) __builtin_nontemporal_store(__builtin_nontemporal_load(s), d);
        else *d = *s;
    }
}

template <int kBytes>
static void launch_generic_bits_same(const char* s, char* d, const FlatLayout& ls, const FlatLayout& ld, int64_t n, hipStream_t st) {
    const dim3 g((unsigned)std::min<int64_t>((n + 255) / 256, (int64_t)1 << 22));
    if (n * kBytes >= ((int64_t)64 << 20)) copy_generic_bits_same<kBytes, true><<<g, 256, 0, st>>>(s, d, ls, ld, (uint32_t)n);
    else copy_generic_bits_same<kBytes, false><<<g, 256, 0, st>>>(s, d, ls, ld, (uint32_t)n);
}
template <int kSrc, int kDst>
__global__ __launch_bounds__(256) void copy_generic_cvt(const char* __restrict__ src,
                                                        char* __restrict__ dst, FlatLayout ls,
                                                        FlatLayout ld, int64_t n, int sb, int db, Mask mask) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        if (masked_out(mask, i)) continue;
        const double v = load_as_f64<kSrc>(src + layout_offset(ls, i) * sb);
        store_from<kDst>(dst + layout_offset(ld, i) * db, v, kSrc == MOYE_F64);
    }
}

// The same element loops, V elements per lane: for arrays whose first mode (once the modes are ordered by stride) is a
// run of unit stride on every side -- pitched matrices, slices of larger arrays -- with V dividing its extent and every
// other stride, and aligned pointers.  The vectorisation the reference computes with max_common_vector
// (src/layout.jl:752-761) and leaves unused (src/algorithm/copy.jl:53-58), here also for converting copies (the wider
// side moves 16 bytes per lane) and for copyto_if! (the mask is read V bytes at a time; a group whose mask is all true
// goes out in one access, a mixed one element by element, so that elements whose mask is false are never written).
// The layouts count groups of V elements (extent of mode 0 and the other strides divided by V).  Same conversion per
// element as copy_generic_cvt; kSrc == kDst moves bits.
template <int N> struct BytesOf;
template <> struct BytesOf<1> { typedef uint8_t type; };
template <> struct BytesOf<2> { typedef uint16_t type; };
template <> struct BytesOf<4> { typedef uint32_t type; };
template <> struct BytesOf<8> { typedef uint64_t type; };
template <> struct BytesOf<16> { typedef u32x4 type; };
// kSame: the layouts (the mask's too) have one shape mode by mode and there are fewer than 2^31 groups: the index is taken
// apart once, with 32-bit divisions, for all of them (see copy_generic_bits_same).
template <int kSrc, int kDst, int SB, int DB, int V, bool kSame = false>
__global__ __launch_bounds__(256) void copy_groups(const char* __restrict__ src, char* __restrict__ dst, FlatLayout ls, FlatLayout ld,
                                                   int64_t ngroups, Mask mask) {
    typedef typename BytesOf<V * SB>::type SrcWord;
    typedef typename BytesOf<V * DB>::type DstWord;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; g < ngroups; g += stride) {
        int64_t so = 0, dof = 0, mo = 0;
        if constexpr (kSame) {
            uint32_t rest = (uint32_t)g;
#pragma unroll 1
            for (int m = 0; m < ls.rank; ++m) {
                const uint32_t extent = (uint32_t)ls.shape[m], q = rest / extent, c = rest - q * extent;
                so += (int64_t)c * ls.stride[m];
                dof += (int64_t)c * ld.stride[m];
                if (mask.ptr) mo += (int64_t)c * mask.l.stride[m];
                rest = q;
            }
        } else {
            so = layout_offset(ls, g);
            dof = layout_offset(ld, g);
            if (mask.ptr) mo = layout_offset(mask.l, g);
        }
        uint8_t keep[V];
        bool all = true, any = true;
        if (mask.ptr) {
            typedef typename BytesOf<V>::type MaskWord;
            const MaskWord mw = *reinterpret_cast<const MaskWord*>(mask.ptr + mo * V);
            __builtin_memcpy(keep, &mw, V);
            any = false;
#pragma unroll
            for (int e = 0; e < V; ++e) {
                all = all && keep[e];
                any = any || keep[e];
            }
            if (!any) continue;
        }
        const SrcWord in = *reinterpret_cast<const SrcWord*>(src + so * (V * SB));
        char* const d = dst + dof * (V * DB);
        DstWord out;
        if constexpr (kSrc == kDst) {
            static_assert(SB == DB, "bits");
            __builtin_memcpy(&out, &in, V * SB);
        } else {
#pragma unroll
            for (int e = 0; e < V; ++e) {
                char e_in[SB], e_out[DB];
                __builtin_memcpy(e_in, reinterpret_cast<const char*>(&in) + e * SB, SB);
                store_from<kDst>(e_out, load_as_f64<kSrc>(e_in), kSrc == MOYE_F64);
                __builtin_memcpy(reinterpret_cast<char*>(&out) + e * DB, e_out, DB);
            }
        }
        if (all) {
            *reinterpret_cast<DstWord*>(d) = out;
        } else if constexpr (V >= 8) {
            // some of a group of eight or sixteen: the destination's own values fill the gaps and the group goes out in one
            // piece (the elements the mask leaves out are written back as they were read; nothing else writes them during a
            // copyto_if!).  Element by element, a random mask cost eight partial stores per lane: fp16 8192^2 3.07 TB/s
            // against 4.64.  Groups of four gain nothing from it (f32 -> f16 4.46 against 4.10 this way).
            DstWord old = *reinterpret_cast<const DstWord*>(d);
#pragma unroll
            for (int e = 0; e < V; ++e)
                if (keep[e]) __builtin_memcpy(reinterpret_cast<char*>(&old) + e * DB, reinterpret_cast<const char*>(&out) + e * DB, DB);
            *reinterpret_cast<DstWord*>(d) = old;
        } else {
#pragma unroll
            for (int e = 0; e < V; ++e)
                if (keep[e]) __builtin_memcpy(d + e * DB, reinterpret_cast<const char*>(&out) + e * DB, DB);
        }
    }
}

// Converting copy between two dense, 16-byte aligned runs of elements of one width (fp16 <-> bf16): a lane converts the
// elements of one 16-byte piece; one workgroup per 256 pieces, no loop.  Element by element the same conversion as
// copy_generic_cvt.
template <int kSrc, int kDst, int SB, int DB>
__global__ __launch_bounds__(256) void copy_cvt_dense(const char* __restrict__ src, char* __restrict__ dst, int64_t nvec) {
    static_assert(SB == DB, "the widening and narrowing directions have kernels of their own");
    constexpr int E = 16 / SB;
    const u32x4* sv = reinterpret_cast<const u32x4*>(src);
    u32x4* dv = reinterpret_cast<u32x4*>(dst);
    const int64_t i = flat_piece();
    if (i >= nvec) return;
    const u32x4 in = __builtin_nontemporal_load(sv + i);
    u32x4 out;
#pragma unroll
    for (int k = 0; k < E; ++k) {
        char e_in[SB], e_out[DB];
        __builtin_memcpy(e_in, reinterpret_cast<const char*>(&in) + k * SB, SB);
        store_from<kDst>(e_out, load_as_f64<kSrc>(e_in), kSrc == MOYE_F64);
        __builtin_memcpy(reinterpret_cast<char*>(&out) + k * DB, e_out, DB);
    }
    __builtin_nontemporal_store(out, dv + i);
}

static FlatLayout flat_of(const moye_tensor& t) {
    FlatLayout f;
    f.rank = t.rank;
    for (int i = 0; i < MOYE_MAX_RANK; ++i) {
        f.shape[i] = i < t.rank ? t.shape[i] : 1;
        f.stride[i] = i < t.rank ? t.stride[i] : 0;
    }
    return f;
}

// Is the layout a dense run 0..size-1 visited in order (compact column-major after dropping
// size-1 modes)?
static bool is_contiguous(const moye_tensor& t) {
    int64_t expect = 1;
    for (int i = 0; i < t.rank; ++i) {
        if (t.shape[i] == 1) continue;
        if (t.stride[i] != expect) return false;
        expect *= t.shape[i];
    }
    return true;
}

// Are both one dense run in the same order: as written, or once the modes of both are ordered by stride (two row-major
// arrays of one shape: a copy may visit the elements in any order)?
static bool one_run_each(const moye_tensor& src, const moye_tensor& dst) {
    if (is_contiguous(src) && is_contiguous(dst)) return true;
    moye_tensor ts = src, td = dst;
    moye_tensor* both[2] = {&td, &ts};
    return order_modes_by_stride(both, 2) && is_contiguous(ts) && is_contiguous(td);
}

// The widening direction: a lane's 16-byte store holds EW = 16 / sizeof(dst) elements, which it reads as one access of
// EW * sizeof(src) bytes (8, 4 or 2), so that loads and stores of a wave are both contiguous; four of them in flight.
template <int NB> struct NarrowWord;
template <> struct NarrowWord<8> { typedef uint64_t type; };
template <> struct NarrowWord<4> { typedef uint32_t type; };
template <> struct NarrowWord<2> { typedef uint16_t type; };
template <int kSrc, int kDst, int SB, int DB>
__global__ __launch_bounds__(256) void copy_cvt_dense_widen(const char* __restrict__ src, char* __restrict__ dst, int64_t nvec) {
    constexpr int EW = 16 / DB, NB = EW * SB;
    typedef typename NarrowWord<NB>::type word;
    const word* sv = reinterpret_cast<const word*>(src);
    u32x4* dv = reinterpret_cast<u32x4*>(dst);
    auto convert = [](word in) {
        u32x4 out;
#pragma unroll
        for (int k = 0; k < EW; ++k) {
            char e_in[SB], e_out[DB];
            __builtin_memcpy(e_in, reinterpret_cast<const char*>(&in) + k * SB, SB);
            store_from<kDst>(e_out, load_as_f64<kSrc>(e_in), kSrc == MOYE_F64);
            __builtin_memcpy(reinterpret_cast<char*>(&out) + k * DB, e_out, DB);
        }
        return out;
    };
    // one piece per lane, one workgroup per 256 pieces, no loop (the form that is fastest for the plain copy)
    const int64_t i = flat_piece();
    if (i < nvec) __builtin_nontemporal_store(convert(__builtin_nontemporal_load(sv + i)), dv + i);
}

// The narrowing direction: a lane reads 16 bytes and stores the EN = 16 / sizeof(src) converted elements as one access of
// 2, 4 or 8 bytes; loads and stores of a wave are contiguous.
template <int kSrc, int kDst, int SB, int DB>
__global__ __launch_bounds__(256) void copy_cvt_dense_narrow(const char* __restrict__ src, char* __restrict__ dst, int64_t nvec) {
    constexpr int EN = 16 / SB, NB = EN * DB;
    typedef typename NarrowWord<NB>::type word;
    const u32x4* sv = reinterpret_cast<const u32x4*>(src);
    word* dv = reinterpret_cast<word*>(dst);
    auto convert = [](const u32x4& in) {
        word out;
#pragma unroll
        for (int k = 0; k < EN; ++k) {
            char e_in[SB], e_out[DB];
            __builtin_memcpy(e_in, reinterpret_cast<const char*>(&in) + k * SB, SB);
            store_from<kDst>(e_out, load_as_f64<kSrc>(e_in), kSrc == MOYE_F64);
            __builtin_memcpy(reinterpret_cast<char*>(&out) + k * DB, e_out, DB);
        }
        return out;
    };
    const int64_t i = flat_piece();
    if (i < nvec) __builtin_nontemporal_store(convert(__builtin_nontemporal_load(sv + i)), dv + i);
}

constexpr int float_bytes(int dt) { return dt == MOYE_F64 ? 8 : dt == MOYE_F32 ? 4 : dt == MOYE_F8E4M3 ? 1 : 2; }

// dense converting copy of the first n - n % E elements; returns how many elements it covered (0: not launched)
template <int kSrc, int kDst>
static int64_t launch_cvt_dense_pair(const char* s, char* d, int64_t n, hipStream_t st) {
    constexpr int SB = float_bytes(kSrc), DB = float_bytes(kDst), E = 16 / (SB < DB ? SB : DB);
    if constexpr (DB > SB) {
        constexpr int EW = 16 / DB;
        const int64_t nvec = n / EW;
        if (nvec == 0) return 0;
        copy_cvt_dense_widen<kSrc, kDst, SB, DB><<<flat_grid(nvec), 256, 0, st>>>(s, d, nvec);
        return nvec * EW;
    }
    if constexpr (SB > DB) {
        static_assert((16 / SB) * DB >= 2, "a lane's store is 2, 4 or 8 bytes");
        constexpr int EN = 16 / SB;
        const int64_t nvec = n / EN;
        if (nvec == 0) return 0;
        copy_cvt_dense_narrow<kSrc, kDst, SB, DB><<<flat_grid(nvec), 256, 0, st>>>(s, d, nvec);
        return nvec * EN;
    }
    if constexpr (SB == DB) {
        const int64_t nvec = n / E;
        if (nvec == 0) return 0;
        copy_cvt_dense<kSrc, kDst, SB, DB><<<flat_grid(nvec), 256, 0, st>>>(s, d, nvec);
        return nvec * E;
    }
    return 0;
}
template <int kSrc>
static int64_t launch_cvt_dense_dst(int32_t dd, const char* s, char* d, int64_t n, hipStream_t st) {
    switch (dd) {
        case MOYE_F32: if constexpr (kSrc != MOYE_F32) return launch_cvt_dense_pair<kSrc, MOYE_F32>(s, d, n, st); break;
        case MOYE_F16: if constexpr (kSrc != MOYE_F16) return launch_cvt_dense_pair<kSrc, MOYE_F16>(s, d, n, st); break;
        case MOYE_BF16: if constexpr (kSrc != MOYE_BF16) return launch_cvt_dense_pair<kSrc, MOYE_BF16>(s, d, n, st); break;
        case MOYE_F8E4M3: if constexpr (kSrc != MOYE_F8E4M3) return launch_cvt_dense_pair<kSrc, MOYE_F8E4M3>(s, d, n, st); break;
        case MOYE_F64: if constexpr (kSrc != MOYE_F64) return launch_cvt_dense_pair<kSrc, MOYE_F64>(s, d, n, st); break;
        default: break;
    }
    return 0;
}
static int64_t launch_cvt_dense(int32_t sd, int32_t dd, const char* s, char* d, int64_t n, hipStream_t st) {
    switch (sd) {
        case MOYE_F32: return launch_cvt_dense_dst<MOYE_F32>(dd, s, d, n, st);
        case MOYE_F16: return launch_cvt_dense_dst<MOYE_F16>(dd, s, d, n, st);
        case MOYE_BF16: return launch_cvt_dense_dst<MOYE_BF16>(dd, s, d, n, st);
        case MOYE_F8E4M3: return launch_cvt_dense_dst<MOYE_F8E4M3>(dd, s, d, n, st);
        case MOYE_F64: return launch_cvt_dense_dst<MOYE_F64>(dd, s, d, n, st);
        default: return 0;
    }
}

// ------------------------------------------------------------------------------------------
// a transpose that converts on the way (copyto! between arrays of different element types whose unit strides lie on
// different modes: src/algorithm/copy.jl:38-43 with the layouts of a transpose)
// ------------------------------------------------------------------------------------------
// A tile is TI elements along the source's contiguous index i (at least 128 bytes of a source row) by TJ along the
// destination's (at least 256 bytes of a destination row).  A lane loads 16-byte pieces of source rows, converts their
// elements and writes them one by one into an LDS tile of destination elements, [i][j]; a lane then reads 16 bytes of an
// LDS row and stores them as 16 bytes of a destination row.  Workgroups are numbered along j first, as in the other
// destination-order kernels.  An LDS row is 16 bytes longer than its data, which spreads the rows over the banks.
template <int kSrc, int kDst, int SB, int DB>
__global__ __launch_bounds__(256) void transpose_cvt_lds(const char* __restrict__ src, char* __restrict__ dst, int64_t lds_, int64_t ldd, int tiles_j,
                                                         int64_t bs_src, int64_t bs_dst, int64_t bz_src, int64_t bz_dst) {
    constexpr int TI = SB == 1 ? 128 : 64, TJ = DB == 1 ? 256 : 128;
    constexpr int ES = 16 / SB, ED = 16 / DB;  // elements per 16-byte piece
    constexpr int PI = TI / ES, RJ = 256 / PI, NL = TJ / RJ;  // pieces per source row of the tile, source rows per pass, passes
    constexpr int PITCH = TJ * DB + 16;
    extern __shared__ char cvt_tile[];  // TI rows of PITCH bytes
    src += ((int64_t)blockIdx.y * bs_src + (int64_t)blockIdx.z * bz_src) * SB;  // (a batch of matrices: their indices in the grid)
    dst += ((int64_t)blockIdx.y * bs_dst + (int64_t)blockIdx.z * bz_dst) * DB;
    const int tj = blockIdx.x % tiles_j, ti = blockIdx.x / tiles_j;
    const int pi = threadIdx.x % PI, jr = threadIdx.x / PI;
    const char* s = src + (((int64_t)tj * TJ + jr) * lds_ + (int64_t)ti * TI + ES * pi) * SB;
    constexpr int CH = NL < 8 ? NL : 8;  // loads in flight per lane
#pragma unroll 1
    for (int h0 = 0; h0 < NL; h0 += CH) {
        u32x4 x[CH];
#pragma unroll
        for (int h = 0; h < CH; ++h) x[h] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(s + (int64_t)(RJ * (h0 + h)) * lds_ * SB));
#pragma unroll
        for (int h = 0; h < CH; ++h) {
            const int j = jr + RJ * (h0 + h);
#pragma unroll
            for (int e = 0; e < ES; ++e) {
                char e_in[SB];
                __builtin_memcpy(e_in, reinterpret_cast<const char*>(&x[h]) + e * SB, SB);
                store_from<kDst>(cvt_tile + (ES * pi + e) * PITCH + j * DB, load_as_f64<kSrc>(e_in), kSrc == MOYE_F64);
            }
        }
    }
    __syncthreads();
    constexpr int PJ = TJ / ED, RP = 256 / PJ;  // pieces per destination row of the tile, destination rows per pass
    const int pj = threadIdx.x % PJ, r0 = threadIdx.x / PJ;
    char* d = dst + (((int64_t)ti * TI + r0) * ldd + (int64_t)tj * TJ + ED * pj) * DB;
#pragma unroll
    for (int p = 0; p < TI / RP; ++p) {
        const u32x4 w = *reinterpret_cast<const u32x4*>(cvt_tile + (r0 + RP * p) * PITCH + pj * 16);
        __builtin_nontemporal_store(w, reinterpret_cast<u32x4*>(d + (int64_t)(RP * p) * ldd * DB));
    }
}

// tile extents of transpose_cvt_lds for elements of sb and db bytes
static int cvt_tile_i(int sb) { return sb == 1 ? 128 : 64; }
static int cvt_tile_j(int db) { return db == 1 ? 256 : 128; }

template <int kSrc, int kDst, int SB, int DB>
static int32_t launch_transpose_cvt_pair(const char* s, char* d, int64_t lds_, int64_t ldd, int64_t ni, int64_t nj, hipStream_t st, const int64_t (&bt)[6]) {
    auto kern = transpose_cvt_lds<kSrc, kDst, SB, DB>;
    constexpr int TI = SB == 1 ? 128 : 64, TJ = DB == 1 ? 256 : 128, kLds = TI * (TJ * DB + 16);
    if (kLds > 48 * 1024) {
        static LdsCap cap;
        if (int32_t e = raise_lds_cap(cap, reinterpret_cast<const void*>(kern), kLds)) return e;
    }
    const int64_t groups = (ni / TI) * (nj / TJ);
    if (groups >= (1 << 24)) return fail(MOYE_ERR_SHAPE, "copyto!: too many tiles for one launch (2^24 workgroups of 256)");
    kern<<<dim3((unsigned)groups, (unsigned)bt[4], (unsigned)bt[5]), 256, kLds, st>>>(s, d, lds_, ldd, (int)(nj / TJ), bt[0], bt[1], bt[2], bt[3]);
    MOYE_HIP_CHECK(hipGetLastError());
    return MOYE_OK;
}
template <int kSrc, int SB>
static int32_t launch_transpose_cvt_dst(int32_t dd, const char* s, char* d, int64_t lds_, int64_t ldd, int64_t ni, int64_t nj, hipStream_t st, const int64_t (&bt)[6]) {
    switch (dd) {
        case MOYE_F32: if constexpr (kSrc != MOYE_F32) return launch_transpose_cvt_pair<kSrc, MOYE_F32, SB, 4>(s, d, lds_, ldd, ni, nj, st, bt); break;
        case MOYE_F16: if constexpr (kSrc != MOYE_F16) return launch_transpose_cvt_pair<kSrc, MOYE_F16, SB, 2>(s, d, lds_, ldd, ni, nj, st, bt); break;
        case MOYE_BF16: if constexpr (kSrc != MOYE_BF16) return launch_transpose_cvt_pair<kSrc, MOYE_BF16, SB, 2>(s, d, lds_, ldd, ni, nj, st, bt); break;
        case MOYE_F8E4M3: if constexpr (kSrc != MOYE_F8E4M3) return launch_transpose_cvt_pair<kSrc, MOYE_F8E4M3, SB, 1>(s, d, lds_, ldd, ni, nj, st, bt); break;
        case MOYE_F64: if constexpr (kSrc != MOYE_F64) return launch_transpose_cvt_pair<kSrc, MOYE_F64, SB, 8>(s, d, lds_, ldd, ni, nj, st, bt); break;
        default: break;
    }
    return fail(MOYE_ERR_UNSUPPORTED, "copyto!: no conversion between these element types");
}
// bt: the strides (in elements) of one or two modes that count matrices, source and destination, and their extents
// {bs_src, bs_dst, bz_src, bz_dst, batch, batch2}; {0, 0, 0, 0, 1, 1} for one matrix
static int32_t launch_transpose_cvt(int32_t sd, int32_t dd, const char* s, char* d, int64_t lds_, int64_t ldd, int64_t ni, int64_t nj, hipStream_t st,
                                    const int64_t (&bt)[6]) {
    switch (sd) {
        case MOYE_F32: return launch_transpose_cvt_dst<MOYE_F32, 4>(dd, s, d, lds_, ldd, ni, nj, st, bt);
        case MOYE_F16: return launch_transpose_cvt_dst<MOYE_F16, 2>(dd, s, d, lds_, ldd, ni, nj, st, bt);
        case MOYE_BF16: return launch_transpose_cvt_dst<MOYE_BF16, 2>(dd, s, d, lds_, ldd, ni, nj, st, bt);
        case MOYE_F8E4M3: return launch_transpose_cvt_dst<MOYE_F8E4M3, 1>(dd, s, d, lds_, ldd, ni, nj, st, bt);
        case MOYE_F64: return launch_transpose_cvt_dst<MOYE_F64, 8>(dd, s, d, lds_, ldd, ni, nj, st, bt);
        default: return fail(MOYE_ERR_UNSUPPORTED, "copyto!: no conversion between these element types");
    }
}

template <int kSrc>
static bool launch_cvt_dst(int32_t dd, dim3 g, hipStream_t st, const char* s, char* d, FlatLayout ls,
                           FlatLayout ld, int64_t n, int sb, int db, const Mask& mk) {
    switch (dd) {
        case MOYE_F32: copy_generic_cvt<kSrc, MOYE_F32><<<g, 256, 0, st>>>(s, d, ls, ld, n, sb, db, mk); return true;
        case MOYE_F16: copy_generic_cvt<kSrc, MOYE_F16><<<g, 256, 0, st>>>(s, d, ls, ld, n, sb, db, mk); return true;
        case MOYE_BF16: copy_generic_cvt<kSrc, MOYE_BF16><<<g, 256, 0, st>>>(s, d, ls, ld, n, sb, db, mk); return true;
        case MOYE_F8E4M3: copy_generic_cvt<kSrc, MOYE_F8E4M3><<<g, 256, 0, st>>>(s, d, ls, ld, n, sb, db, mk); return true;
        case MOYE_F64: copy_generic_cvt<kSrc, MOYE_F64><<<g, 256, 0, st>>>(s, d, ls, ld, n, sb, db, mk); return true;
        default: return false;
    }
}

// (the instance that takes the index apart once where the layouts, the mask's too, have one shape and the groups are few
// enough for 32-bit indices: 8192^2 inside a pitch of 16384, f32 -> f16 5.0 -> 5.4 TB/s, f16 -> f32 4.2 -> 5.4, f16 -> bf16 4.7 -> 6.7)
template <int kSrc, int kDst, int SB, int DB, int V>
static void run_groups(const char* s, char* d, const FlatLayout& ls, const FlatLayout& ld, int64_t ngroups, const Mask& mk, hipStream_t st) {
    if (same_modes_32(ls, ld, ngroups) && (!mk.ptr || same_modes_32(ls, mk.l, ngroups)))
        copy_groups<kSrc, kDst, SB, DB, V, true><<<strided_grid(ngroups), 256, 0, st>>>(s, d, ls, ld, ngroups, mk);
    else
        copy_groups<kSrc, kDst, SB, DB, V, false><<<strided_grid(ngroups), 256, 0, st>>>(s, d, ls, ld, ngroups, mk);
}
template <int kSrc, int kDst, int SB, int DB>
static void launch_groups_pair(const char* s, char* d, const FlatLayout& ls, const FlatLayout& ld, int64_t ngroups, const Mask& mk, hipStream_t st) {
    constexpr int V = 16 / (SB > DB ? SB : DB);
    static_assert(V >= 2, "groups of at least two elements");
    run_groups<kSrc, kDst, SB, DB, V>(s, d, ls, ld, ngroups, mk, st);
}
template <int kSrc, int SB>
static bool launch_groups_dst(int32_t dd, const char* s, char* d, const FlatLayout& ls, const FlatLayout& ld, int64_t ng, const Mask& mk, hipStream_t st) {
    switch (dd) {
        case MOYE_F32: launch_groups_pair<kSrc, MOYE_F32, SB, 4>(s, d, ls, ld, ng, mk, st); return true;
        case MOYE_F16: launch_groups_pair<kSrc, MOYE_F16, SB, 2>(s, d, ls, ld, ng, mk, st); return true;
        case MOYE_BF16: launch_groups_pair<kSrc, MOYE_BF16, SB, 2>(s, d, ls, ld, ng, mk, st); return true;
        case MOYE_F8E4M3: launch_groups_pair<kSrc, MOYE_F8E4M3, SB, 1>(s, d, ls, ld, ng, mk, st); return true;
        case MOYE_F64: launch_groups_pair<kSrc, MOYE_F64, SB, 8>(s, d, ls, ld, ng, mk, st); return true;
        default: return false;
    }
}
// Groups of V = 16 / (the wider element) elements along the first mode, when every layout of the call (the modes already
// ordered by stride) has it as a run of unit stride that V divides, V divides every other stride that is used, and the
// pointers are aligned to what a lane then accesses.  `same_bits`: a copy of bits (with a mask: copyto_if!).  Returns
// false, having launched nothing, when the call does not qualify.
static bool launch_groups(int32_t src_dt, int32_t dst_dt, const char* s, char* d, FlatLayout ls, FlatLayout ld, Mask mk, bool same_bits, int64_t n,
                          hipStream_t st) {
    const int sb = dtype_bytes(src_dt), db = dtype_bytes(dst_dt);
    const int V = 16 / std::max(sb, db);
    if (V < 2 || ls.rank < 1 || ld.rank != ls.rank) return false;
    auto fits = [&](const FlatLayout& l, const void* p, int elem_bytes) {
        if (l.stride[0] != 1 || l.shape[0] % V || reinterpret_cast<uintptr_t>(p) % (V * elem_bytes)) return false;
        for (int m = 1; m < MOYE_MAX_RANK; ++m)
            if (l.shape[m] > 1 && l.stride[m] % V) return false;
        return true;
    };
    if (ls.shape[0] != ld.shape[0] || !fits(ls, s, sb) || !fits(ld, d, db)) return false;
    if (mk.ptr && (mk.l.rank != ls.rank || mk.l.shape[0] != ls.shape[0] || !fits(mk.l, mk.ptr, 1))) return false;
    for (FlatLayout* l : {&ls, &ld, &mk.l}) {
        if (l == &mk.l && !mk.ptr) continue;
        l->shape[0] /= V;
        for (int m = 1; m < MOYE_MAX_RANK; ++m) l->stride[m] /= V;
    }
    const int64_t ng = n / V;
    if (same_bits) {
        switch (sb) {
            case 1: run_groups<MOYE_U8, MOYE_U8, 1, 1, 16>(s, d, ls, ld, ng, mk, st); return true;
            case 2: run_groups<MOYE_U16, MOYE_U16, 2, 2, 8>(s, d, ls, ld, ng, mk, st); return true;
            case 4: run_groups<MOYE_U32, MOYE_U32, 4, 4, 4>(s, d, ls, ld, ng, mk, st); return true;
            case 8: run_groups<MOYE_U64, MOYE_U64, 8, 8, 2>(s, d, ls, ld, ng, mk, st); return true;
            default: return false;
        }
    }
    switch (src_dt) {
        case MOYE_F32: return launch_groups_dst<MOYE_F32, 4>(dst_dt, s, d, ls, ld, ng, mk, st);
        case MOYE_F16: return launch_groups_dst<MOYE_F16, 2>(dst_dt, s, d, ls, ld, ng, mk, st);
        case MOYE_BF16: return launch_groups_dst<MOYE_BF16, 2>(dst_dt, s, d, ls, ld, ng, mk, st);
        case MOYE_F8E4M3: return launch_groups_dst<MOYE_F8E4M3, 1>(dst_dt, s, d, ls, ld, ng, mk, st);
        case MOYE_F64: return launch_groups_dst<MOYE_F64, 8>(dst_dt, s, d, ls, ld, ng, mk, st);
        default: return false;
    }
}

int32_t copy_dispatch(const moye_tiled_copy* tc, const moye_tensor* dst, const moye_tensor* src,
                      hipStream_t st) {
    return copy_if_dispatch(tc, dst, src, nullptr, st);
}

// `mask` null: copyto!; else copyto_if! with a mask array of one byte per logical element (nonzero = move)
int32_t copy_if_dispatch(const moye_tiled_copy* tc, const moye_tensor* dst, const moye_tensor* src,
                         const moye_tensor* mask, hipStream_t st) {
    if (int32_t e = check_tensor(dst, "dst")) return e;
    if (int32_t e = check_tensor(src, "src")) return e;
    int64_t n = tensor_size(*src);
    Mask mk{};
    if (mask) {
        if (int32_t e = check_tensor(mask, "mask")) return e;
        if (dtype_bytes(mask->dtype) != 1 || is_float_dtype(mask->dtype))
            return fail(MOYE_ERR_UNSUPPORTED, "copyto_if!: the mask holds one byte per element (Bool), not %s", dtype_name(mask->dtype));
        if (tensor_size(*mask) != n)
            return fail(MOYE_ERR_SHAPE, "copyto_if!: mask holds %lld elements, src %lld", (long long)tensor_size(*mask), (long long)n);
        mk.ptr = static_cast<const uint8_t*>(mask->ptr);
        mk.l = flat_of(*mask);
    }
    if (tensor_size(*dst) != n)
        return fail(MOYE_ERR_SHAPE, "copyto!: dst holds %lld elements, src %lld",
                    (long long)tensor_size(*dst), (long long)n);
    const int sb = dtype_bytes(src->dtype), db = dtype_bytes(dst->dtype);
    if (n == 0) return MOYE_OK;
    const bool same_bits = (src->dtype == dst->dtype) || (sb == db && !is_float_dtype(src->dtype) && !is_float_dtype(dst->dtype));
    if (!same_bits && !(is_float_dtype(src->dtype) && is_float_dtype(dst->dtype)))
        return fail(MOYE_ERR_UNSUPPORTED, "copyto!: no conversion %s -> %s", dtype_name(src->dtype),
                    dtype_name(dst->dtype));
    if (tc) {
        if (tc->op != MOYE_COPY_UNIVERSAL && tc->op != MOYE_COPY_LDS_TILED)
            return fail(MOYE_ERR_UNSUPPORTED, "copyto!: unknown copy op %d", tc->op);
        if (tc->vec_bits && (tc->vec_bits % 8 || tc->vec_bits > 128 || (tc->vec_bits & (tc->vec_bits - 1))))
            return fail(MOYE_ERR_ARG, "copyto!: vec_bits %d is not one of 8..128", tc->vec_bits);
        if (tc->vec_bits && tc->vec_bits % (8 * sb))
            return fail(MOYE_ERR_SHAPE, "copyto!: a %d-bit access does not hold whole %s values", tc->vec_bits,
                        dtype_name(src->dtype));
    }
    const char* s = static_cast<const char*>(src->ptr);
    char* d = static_cast<char*>(dst->ptr);

    // Arrays of one shape of rank three and more: modes of extent 1 go, and modes that are neighbours in memory on both
    // sides become one (NCHW -> NHWC: H and W), so that what follows sees a matrix or a batch of matrices where there is
    // one (the tiler of the descriptor speaks of the caller's modes: it is checked here, then dropped)
    if (!mask && src->rank == dst->rank && src->rank > 2) {
        bool same = true;
        for (int m = 0; m < src->rank; ++m) same = same && src->shape[m] == dst->shape[m];
        moye_tensor cs = *src, cd = *dst;
        int r = 0;
        for (int m = 0; same && m < src->rank; ++m) {
            if (src->shape[m] == 1) continue;
            if (r > 0 && src->stride[m] == cs.stride[r - 1] * cs.shape[r - 1] && dst->stride[m] == cd.stride[r - 1] * cd.shape[r - 1]) {
                cs.shape[r - 1] *= src->shape[m];
                cd.shape[r - 1] = cs.shape[r - 1];
            } else {
                cs.shape[r] = cd.shape[r] = src->shape[m];
                cs.stride[r] = src->stride[m];
                cd.stride[r] = dst->stride[m];
                ++r;
            }
        }
        if (same && r >= 1 && r < src->rank) {
            moye_tiled_copy plain{};
            if (tc) {
                if (tc->op == MOYE_COPY_LDS_TILED)
                    for (int m = 0; m < 2; ++m)
                        if (tc->tiler_mn[m] < 0 || (tc->tiler_mn[m] > 0 && src->shape[m] % tc->tiler_mn[m]))
                            return fail(MOYE_ERR_SHAPE, "copyto!: tiler extent %d does not divide mode %d of size %lld", tc->tiler_mn[m], m + 1,
                                        (long long)src->shape[m]);
                plain = *tc;
                plain.tiler_mn[0] = plain.tiler_mn[1] = 0;
            }
            cs.rank = cd.rank = r;
            return copy_if_dispatch(tc ? &plain : nullptr, &cd, &cs, nullptr, st);
        }
    }
    if (same_bits && !mask) {
        // (1) both sides one dense run in the same order
        if (one_run_each(*src, *dst)) {
            const int64_t bytes = n * sb;
            if (bytes % 16 == 0 && (reinterpret_cast<uintptr_t>(s) | reinterpret_cast<uintptr_t>(d)) % 16 == 0) {
                const int64_t n16 = bytes / 16;
                copy_flat_b128<<<flat_grid(n16), 256, 0, st>>>(reinterpret_cast<const u32x4*>(s), reinterpret_cast<u32x4*>(d), n16);
            } else {
                const int blocks = (int)std::min<int64_t>((bytes + 255) / 256, 256 * 32);
                copy_flat_bytes<<<blocks, 256, 0, st>>>(reinterpret_cast<const uint8_t*>(s), reinterpret_cast<uint8_t*>(d), bytes);
            }
            MOYE_HIP_CHECK(hipGetLastError());
            return MOYE_OK;
        }
        // whole tiles of an aligned matrix (or of `batch` such matrices bs / bd elements apart) through the LDS kernels
        auto tiled_launch = [&](const char* s_, char* d_, int64_t ni, int64_t nj, int64_t lds_, int64_t ldd, int64_t bs, int64_t bd,
                                int batch, int64_t bs2 = 0, int64_t bd2 = 0, int batch2 = 1) -> int32_t {
            const int tile_j = sb == 1 ? kTileJ8 : sb == 8 ? kTileJ64 : kTile;
            const int ti = (int)(ni / kTile), tj = (int)(nj / tile_j);
            if (sb == 8)
                return launch_transpose64_rows(reinterpret_cast<const uint64_t*>(s_), reinterpret_cast<uint64_t*>(d_), lds_, ldd, ti, tj, st, bs, bd, batch, bs2, bd2, batch2);
            if (sb == 1) {
                const uint8_t* s8 = reinterpret_cast<const uint8_t*>(s_);
                uint8_t* d8 = reinterpret_cast<uint8_t*>(d_);
                // whole 256-byte runs on both sides, destination rows first (measured, TB/s, the 64-byte-piece kernel in
                // super-block order / this one: 16384^2 2.91 / 4.82, 32768^2 3.20 / 5.89, 8192^2 3.29 / 4.94, 32768 x 4096
                // 3.32 / 5.70, 4096 x 32768 3.46 / 4.99, 65536 x 16384 3.09 / 6.12; this one in super-block order 4.35-5.05)
                if (ti % 4 == 0) return launch_transpose8_wide(s8, d8, lds_, ldd, ti, tj, st, bs, bd, batch, bs2, bd2, batch2);
                if (ti % 2 == 0) return launch_transpose8<2>(s8, d8, lds_, ldd, ti, tj, st, bs, bd, batch, bs2, bd2, batch2);
                return launch_transpose8<1>(s8, d8, lds_, ldd, ti, tj, st, bs, bd, batch, bs2, bd2, batch2);
            }
            if (sb == 2) {
                const uint16_t* s16 = reinterpret_cast<const uint16_t*>(s_);
                uint16_t* d16 = reinterpret_cast<uint16_t*>(d_);
                // measured, TB/s, source-first / destination-first: 16384^2 5.32 / 5.75, 4096^2 x 16 6.25 / 6.47, 32768 x 4096
                // 4.07 / 6.10; 2048^2 x 64 5.83 / 5.18, 4096 x 32768 5.65 / 4.46
                if (tj % 8 == 0 && ni >= nj && ni >= 3072)
                    return launch_transpose16_rows<8>(s16, d16, lds_, ldd, ti, tj, st, bs, bd, batch, bs2, bd2, batch2);
                if (ti % 8 == 0) return launch_transpose16<8>(s16, d16, lds_, ldd, ti, tj, st, bs, bd, batch, bs2, bd2, batch2);
                if (ti % 4 == 0) return launch_transpose16<4>(s16, d16, lds_, ldd, ti, tj, st, bs, bd, batch, bs2, bd2, batch2);
                if (ti % 2 == 0) return launch_transpose16<2>(s16, d16, lds_, ldd, ti, tj, st, bs, bd, batch, bs2, bd2, batch2);
                return launch_transpose16<1>(s16, d16, lds_, ldd, ti, tj, st, bs, bd, batch, bs2, bd2, batch2);
            }
            const uint32_t* s32 = reinterpret_cast<const uint32_t*>(s_);
            uint32_t* d32 = reinterpret_cast<uint32_t*>(d_);
            if (tc && (tc->flags & MOYE_GEMM_NO_LDS_SWIZZLE)) return launch_transpose<false, 1>(s32, d32, lds_, ldd, ti, tj, st, bs, bd, batch, bs2, bd2, batch2);
            // Destination rows first (transpose_lds_b32_rows) when the source's contiguous extent is at least the destination's
            // and 2048 or more; measured, TB/s, source-first / destination-first order: 16384^2 5.68 / 6.25, 12288^2 5.20 / 5.94,
            // 4096^2 x 16 5.81 / 6.02, 2048^2 x 64 6.30 / 6.48, 32768 x 4096 4.33 / 6.39; the other way round 4096 x 32768
            // 5.58 / 5.08, 2048 x 65536 5.77 / 4.52, 1024^2 x 128 6.03 / 5.86.
            if (tj % 4 == 0 && ni >= nj && ni >= 2048)
                return launch_transpose_rows<4>(s32, d32, lds_, ldd, ti, tj, st, bs, bd, batch, bs2, bd2, batch2);
            if (ti % 4 == 0) return launch_transpose<true, 4>(s32, d32, lds_, ldd, ti, tj, st, bs, bd, batch, bs2, bd2, batch2);
            if (ti % 2 == 0) return launch_transpose<true, 2>(s32, d32, lds_, ldd, ti, tj, st, bs, bd, batch, bs2, bd2, batch2);
            return launch_transpose<true, 1>(s32, d32, lds_, ldd, ti, tj, st, bs, bd, batch, bs2, bd2, batch2);
        };
        // (2) rank-2 transpose of 1-, 2- and 4-byte elements through LDS patches
        bool lds_pair = false;  // a rank-2 pair with the unit strides on different modes: what the LDS-tiled op is for
        // The tiler of the descriptor (tiler_MN of make_tiled_copy, src/atom/copy.jl:249-258; 32 x 32 in the reference's own
        // transpose kernel, test/host/copy_async.jl:51-76) must divide the array, as zipped_divide asserts; how the kernels
        // group elements into LDS patches (64 x 64, several per workgroup) is their own business and changes no result.
        if (tc && tc->op == MOYE_COPY_LDS_TILED && src->rank >= 2) {
            for (int m = 0; m < 2; ++m)
                if (tc->tiler_mn[m] < 0 || (tc->tiler_mn[m] > 0 && src->shape[m] % tc->tiler_mn[m]))
                    return fail(MOYE_ERR_SHAPE, "copyto!: tiler extent %d does not divide mode %d of size %lld", tc->tiler_mn[m], m + 1,
                                (long long)src->shape[m]);
        }
        if ((sb == 8 || sb == 4 || sb == 2 || sb == 1) && src->rank == 2 && dst->rank == 2 && src->shape[0] == dst->shape[0] &&
            src->shape[1] == dst->shape[1]) {
            const moye_tensor *a = src, *b = dst;
            bool ok = false, swap = false;
            if (a->stride[0] == 1 && b->stride[1] == 1) ok = true;
            else if (a->stride[1] == 1 && b->stride[0] == 1) ok = swap = true;
            lds_pair = ok;
            if (ok) {
                // normalise to: i = contiguous index of src, j = contiguous index of dst
                const int mi = swap ? 1 : 0, mj = swap ? 0 : 1;
                const int64_t ni = a->shape[mi], nj = a->shape[mj];
                const int64_t lds_ = a->stride[mj], ldd = b->stride[mi];
                const int per16 = 16 / sb;  // elements per 16-byte access
                const int tile_j = sb == 1 ? kTileJ8 : sb == 8 ? kTileJ64 : kTile;  // extent of a tile along the destination's contiguous index
                const bool aligned = ni % kTile == 0 && nj % tile_j == 0 && lds_ % per16 == 0 && ldd % per16 == 0 &&
                                     lds_ >= ni && ldd >= nj &&
                                     (reinterpret_cast<uintptr_t>(s) | reinterpret_cast<uintptr_t>(d)) % 16 == 0;
                if (aligned) return tiled_launch(s, d, ni, nj, lds_, ldd, 0, 0, 1);
                // Sizes that are not multiples of the tile (everything else in order): the interior goes through the
                // LDS tiles, the two strips that are left through the general kernel.  Three launches, disjoint parts.  (A strip
                // touches one page per row of the other side, so it costs far more per byte than the interior: 16400 x 16392
                // fp32 runs at 3.3 TB/s against 5.6 for 16384 x 16384; whole tiles pushed against the edge cost the same.)
                const int64_t ni0 = ni / kTile * kTile, nj0 = nj / tile_j * tile_j;
                if (ni0 > 0 && nj0 > 0 && lds_ % per16 == 0 && ldd % per16 == 0 &&
                    lds_ >= ni && ldd >= nj && (reinterpret_cast<uintptr_t>(s) | reinterpret_cast<uintptr_t>(d)) % 16 == 0) {
                    // sub-array [i0, i0 + ci) x [j0, j0 + cj) of both sides
                    auto part = [&](int64_t i0, int64_t ci, int64_t j0, int64_t cj) -> int32_t {
                        if (ci == 0 || cj == 0) return MOYE_OK;
                        moye_tensor ps = *src, pd = *dst;
                        for (moye_tensor* t : {&ps, &pd}) {
                            t->ptr = static_cast<char*>(t->ptr) + (i0 * t->stride[mi] + j0 * t->stride[mj]) * sb;
                            t->shape[mi] = ci;
                            t->shape[mj] = cj;
                        }
                        // the strips are not whole patches: they go through the general kernel whatever the descriptor says
                        const bool interior = i0 == 0 && j0 == 0 && ci == ni0 && cj == nj0;
                        return copy_if_dispatch(interior ? tc : nullptr, &pd, &ps, nullptr, st);
                    };
                    if (int32_t e = part(0, ni0, 0, nj0)) return e;
                    if (int32_t e = part(ni0, ni - ni0, 0, nj)) return e;
                    return part(0, ni0, nj0, nj - nj0);
                }
            }
        }
        // (2b) a batch of such transposes: arrays of one shape, rank above two, the unit strides of the two sides on
        // different modes of 64 and more; every other mode counts matrices.  One launch with the matrix index in the
        // grid when there are one or two such modes and the matrices are whole aligned tiles; else one rank-2 call per matrix while
        // the matrices are large enough to fill the chip on their own and few enough for the launches not to matter
        // (64 fp32 matrices of 2048 x 2048: 1.5 TB/s through the general kernel, which reads one side in single
        // elements a pitch apart).
        if ((sb == 8 || sb == 4 || sb == 2 || sb == 1) && src->rank == dst->rank && src->rank > 2) {
            const int r = src->rank;
            bool same = true;
            int mi = -1, mj = -1;
            for (int m = 0; m < r; ++m) {
                same = same && src->shape[m] == dst->shape[m];
                if (src->shape[m] > 1 && src->stride[m] == 1 && mi < 0) mi = m;
                if (dst->shape[m] > 1 && dst->stride[m] == 1 && mj < 0) mj = m;
            }
            if (same && mi >= 0 && mj >= 0 && mi != mj && src->shape[mi] >= kTile && src->shape[mj] >= kTile) {
                const int64_t per = src->shape[mi] * src->shape[mj], batch = n / per;
                // one or two batch modes, whole aligned tiles: one launch, the matrix indices in the grid
                // (fp16 [16, 2048, 32, 128] -> [16, 32, 128, 2048], 512 matrices in two modes: 1645 us as 512 launches)
                int bm[2] = {-1, -1}, nbatch_modes = 0;
                for (int m = 0; m < r; ++m)
                    if (m != mi && m != mj && src->shape[m] > 1) {
                        if (nbatch_modes < 2) bm[nbatch_modes] = m;
                        ++nbatch_modes;
                    }
                if (nbatch_modes == 1 || nbatch_modes == 2) {
                    const int64_t ni = src->shape[mi], nj = src->shape[mj], lds_ = src->stride[mj], ldd = dst->stride[mi];
                    const int per16 = 16 / sb, tile_j = sb == 1 ? kTileJ8 : sb == 8 ? kTileJ64 : kTile;
                    bool fits = ni % kTile == 0 && nj % tile_j == 0 && lds_ % per16 == 0 && ldd % per16 == 0 && lds_ >= ni && ldd >= nj &&
                                (reinterpret_cast<uintptr_t>(s) | reinterpret_cast<uintptr_t>(d)) % 16 == 0;
                    for (int b = 0; b < nbatch_modes; ++b)
                        fits = fits && src->shape[bm[b]] <= 65535 && src->stride[bm[b]] % per16 == 0 && dst->stride[bm[b]] % per16 == 0;
                    if (fits) {
                        const bool two = nbatch_modes == 2;
                        return tiled_launch(s, d, ni, nj, lds_, ldd, src->stride[bm[0]], dst->stride[bm[0]], (int)src->shape[bm[0]],
                                            two ? src->stride[bm[1]] : 0, two ? dst->stride[bm[1]] : 0, two ? (int)src->shape[bm[1]] : 1);
                    }
                }
                if (batch <= 4096 && per * sb >= (128 << 10)) {
                    moye_tensor ps = *src, pd = *dst;
                    ps.rank = pd.rank = 2;
                    ps.shape[0] = pd.shape[0] = src->shape[mi];
                    ps.shape[1] = pd.shape[1] = src->shape[mj];
                    ps.stride[0] = src->stride[mi]; ps.stride[1] = src->stride[mj];
                    pd.stride[0] = dst->stride[mi]; pd.stride[1] = dst->stride[mj];
                    int64_t idx[MOYE_MAX_RANK] = {0};
                    for (int64_t b = 0; b < batch; ++b) {
                        int64_t so = 0, dof = 0;
                        for (int m = 0; m < r; ++m)
                            if (m != mi && m != mj) { so += idx[m] * src->stride[m]; dof += idx[m] * dst->stride[m]; }
                        ps.ptr = const_cast<char*>(s) + so * sb;
                        pd.ptr = d + dof * sb;
                        if (int32_t e = copy_if_dispatch(tc, &pd, &ps, nullptr, st)) return e;
                        for (int m = 0; m < r; ++m) {  // next matrix, first mode fastest
                            if (m == mi || m == mj) continue;
                            if (++idx[m] < src->shape[m]) break;
                            idx[m] = 0;
                        }
                    }
                    return MOYE_OK;
                }
            }
        }
        // a pair the LDS-tiled op is meant for, but smaller than a patch or not 16-byte aligned: the general kernel moves it
        if (tc && tc->op == MOYE_COPY_LDS_TILED && !lds_pair)
            return fail(MOYE_ERR_UNSUPPORTED,
                        "copyto!: the LDS-tiled copy takes rank-2 operands (or a batch of them) of 1-, 2- or 4-byte elements "
                        "with the unit stride on different modes");
    }

    // (2c) a transpose that converts: a rank-2 pair of one shape, floating-point types that differ, the unit strides on
    // different modes.  Whole aligned tiles through transpose_cvt_lds; other sizes as an interior of whole tiles plus two
    // strips for the general kernel (8192^2 f32 -> f16: 294 us through the general kernel, which reads one side in single
    // elements a pitch apart).
    if (!same_bits && !mask && src->rank == 2 && dst->rank == 2 && src->shape[0] == dst->shape[0] && src->shape[1] == dst->shape[1] &&
        is_float_dtype(src->dtype) && is_float_dtype(dst->dtype) && !(tc && tc->op == MOYE_COPY_LDS_TILED && (tc->tiler_mn[0] || tc->tiler_mn[1]))) {
        int mi = -1;
        if (src->stride[0] == 1 && dst->stride[1] == 1) mi = 0;
        else if (src->stride[1] == 1 && dst->stride[0] == 1) mi = 1;
        if (mi >= 0) {
            const int mj = 1 - mi;
            const int64_t ni = src->shape[mi], nj = src->shape[mj], lds_ = src->stride[mj], ldd = dst->stride[mi];
            const int ti = cvt_tile_i(sb), tj = cvt_tile_j(db);
            const bool lines = (lds_ * sb) % 16 == 0 && (ldd * db) % 16 == 0 && lds_ >= ni && ldd >= nj &&
                               (reinterpret_cast<uintptr_t>(s) | reinterpret_cast<uintptr_t>(d)) % 16 == 0;
            if (lines && ni % ti == 0 && nj % tj == 0) return launch_transpose_cvt(src->dtype, dst->dtype, s, d, lds_, ldd, ni, nj, st, {0, 0, 0, 0, 1, 1});
            const int64_t ni0 = ni / ti * ti, nj0 = nj / tj * tj;
            if (lines && ni0 > 0 && nj0 > 0) {
                auto part = [&](int64_t i0, int64_t ci, int64_t j0, int64_t cj) -> int32_t {
                    if (ci == 0 || cj == 0) return MOYE_OK;
                    moye_tensor ps = *src, pd = *dst;
                    ps.ptr = static_cast<char*>(ps.ptr) + (i0 * ps.stride[mi] + j0 * ps.stride[mj]) * sb;
                    pd.ptr = static_cast<char*>(pd.ptr) + (i0 * pd.stride[mi] + j0 * pd.stride[mj]) * db;
                    ps.shape[mi] = pd.shape[mi] = ci;
                    ps.shape[mj] = pd.shape[mj] = cj;
                    return copy_if_dispatch(nullptr, &pd, &ps, nullptr, st);
                };
                if (int32_t e = part(0, ni0, 0, nj0)) return e;
                if (int32_t e = part(ni0, ni - ni0, 0, nj)) return e;
                return part(0, ni0, nj0, nj - nj0);
            }
        }
    }

    // (2d) a batch of such converting transposes, counted by one or two modes (NCHW f32 -> NHWC f16 after H and W have
    // become one mode): whole aligned tiles, one launch
    if (!same_bits && !mask && src->rank == dst->rank && src->rank > 2 && is_float_dtype(src->dtype) && is_float_dtype(dst->dtype) &&
        !(tc && tc->op == MOYE_COPY_LDS_TILED && (tc->tiler_mn[0] || tc->tiler_mn[1]))) {
        const int r = src->rank;
        bool same = true;
        int mi = -1, mj = -1;
        for (int m = 0; m < r; ++m) {
            same = same && src->shape[m] == dst->shape[m];
            if (src->shape[m] > 1 && src->stride[m] == 1 && mi < 0) mi = m;
            if (dst->shape[m] > 1 && dst->stride[m] == 1 && mj < 0) mj = m;
        }
        if (same && mi >= 0 && mj >= 0 && mi != mj) {
            int bm[2] = {-1, -1}, nb = 0;
            for (int m = 0; m < r; ++m)
                if (m != mi && m != mj && src->shape[m] > 1) {
                    if (nb < 2) bm[nb] = m;
                    ++nb;
                }
            const int64_t ni = src->shape[mi], nj = src->shape[mj], lds_ = src->stride[mj], ldd = dst->stride[mi];
            bool fits = (nb == 1 || nb == 2) && ni % cvt_tile_i(sb) == 0 && nj % cvt_tile_j(db) == 0 && (lds_ * sb) % 16 == 0 && (ldd * db) % 16 == 0 &&
                        lds_ >= ni && ldd >= nj && (reinterpret_cast<uintptr_t>(s) | reinterpret_cast<uintptr_t>(d)) % 16 == 0;
            for (int b = 0; fits && b < nb; ++b)
                fits = src->shape[bm[b]] <= 65535 && (src->stride[bm[b]] * sb) % 16 == 0 && (dst->stride[bm[b]] * db) % 16 == 0;
            if (fits) {
                const bool two = nb == 2;
                return launch_transpose_cvt(src->dtype, dst->dtype, s, d, lds_, ldd, ni, nj, st,
                                            {src->stride[bm[0]], dst->stride[bm[0]], two ? src->stride[bm[1]] : 0, two ? dst->stride[bm[1]] : 0,
                                             src->shape[bm[0]], two ? src->shape[bm[1]] : 1});
            }
        }
    }

    // (3) generic
    FlatLayout ls = flat_of(*src), ld = flat_of(*dst);
    // same shape mode by mode: visit the coordinates along the destination's smallest strides first (then the source's)
    {
        FlatLayout* all[3] = {&ld, &ls, mask ? &mk.l : nullptr};
        order_modes_by_stride(all, mask ? 3 : 2);
    }
    if (same_bits && !mask) {
        // Vectorise when the layouts allow it, which the reference computes (max_common_vector,
        // src/layout.jl:752-761) and then leaves unused (src/algorithm/copy.jl:53-58): if logical
        // neighbours are memory neighbours on both sides in runs of v elements, and every other stride
        // and both pointers are multiples of v, both layouts are recast to elements of v * sizeof(T)
        // bytes (the upcast of src/layout.jl:945-975 on flattened modes) and moved 4..16 bytes at a time.
        const auto run = [](const FlatLayout& l) { return l.rank >= 1 && l.stride[0] == 1 ? l.shape[0] : 1; };
        int64_t v = std::min(run(ls), run(ld));
        // logical index i -> mode-0 coordinate i % shape[0] on each side: the runs must line up
        if (ls.shape[0] != ld.shape[0]) v = std::__gcd(std::__gcd(ls.shape[0], ld.shape[0]), v);
        int64_t width = 16 / sb;  // widest access in elements
        while (width > 1) {
            bool fits = v % width == 0 && reinterpret_cast<uintptr_t>(s) % (width * sb) == 0 &&
                        reinterpret_cast<uintptr_t>(d) % (width * sb) == 0;
            for (int m = 1; m < MOYE_MAX_RANK && fits; ++m)
                fits = (ls.shape[m] == 1 || ls.stride[m] % width == 0) && (ld.shape[m] == 1 || ld.stride[m] % width == 0);
            if (fits) break;
            width /= 2;
        }
        if (width > 1 && sb * width <= 16) {
            for (FlatLayout* l : {&ls, &ld}) {
                l->shape[0] /= width;
                for (int m = 1; m < MOYE_MAX_RANK; ++m) l->stride[m] /= width;
            }
            const int64_t nv = n / width;
            if (same_modes_32(ls, ld, nv)) {
                switch (sb * width) {
                    case 2: launch_generic_bits_same<2>(s, d, ls, ld, nv, st); break;
                    case 4: launch_generic_bits_same<4>(s, d, ls, ld, nv, st); break;
                    case 8: launch_generic_bits_same<8>(s, d, ls, ld, nv, st); break;
                    default: launch_generic_bits_same<16>(s, d, ls, ld, nv, st); break;
                }
                MOYE_HIP_CHECK(hipGetLastError());
                return MOYE_OK;
            }
            const dim3 gv = strided_grid(nv);  // one piece per lane up to 16 GiB of 16-byte pieces
            switch (sb * width) {
                case 2: copy_generic_bits<2><<<gv, 256, 0, st>>>(s, d, ls, ld, nv, Mask{}); break;
                case 4: copy_generic_bits<4><<<gv, 256, 0, st>>>(s, d, ls, ld, nv, Mask{}); break;
                case 8: copy_generic_bits<8><<<gv, 256, 0, st>>>(s, d, ls, ld, nv, Mask{}); break;
                default: copy_generic_bits<16><<<gv, 256, 0, st>>>(s, d, ls, ld, nv, Mask{}); break;
            }
            MOYE_HIP_CHECK(hipGetLastError());
            return MOYE_OK;
        }
    }
    if (!same_bits && !mask && one_run_each(*src, *dst) &&
        (reinterpret_cast<uintptr_t>(s) | reinterpret_cast<uintptr_t>(d)) % 16 == 0) {
        // both sides one aligned run: 16-byte accesses for all whole groups, the general kernel for what is left
        const int64_t done = launch_cvt_dense(src->dtype, dst->dtype, s, d, n, st);
        if (done > 0) {
            MOYE_HIP_CHECK(hipGetLastError());
            if (done == n) return MOYE_OK;
            s += done * sb;
            d += done * db;
            n -= done;
            for (FlatLayout* l : {&ls, &ld}) {
                l->rank = 1;
                for (int m = 0; m < MOYE_MAX_RANK; ++m) { l->shape[m] = 1; l->stride[m] = 0; }
                l->shape[0] = n;
                l->stride[0] = 1;
            }
        }
    }
    // converting copies between pitched arrays, and copyto_if!: groups of elements along the first mode where the layouts
    // allow (a plain copy of bits has taken its vectorised path above)
    if ((!same_bits || mask) && launch_groups(src->dtype, dst->dtype, s, d, ls, ld, mk, same_bits, n, st)) {
        MOYE_HIP_CHECK(hipGetLastError());
        return MOYE_OK;
    }
    const dim3 g((unsigned)std::min<int64_t>((n + 255) / 256, 256 * 64));
    bool ok = true;
    if (same_bits) {
        switch (sb) {
            case 1: copy_generic_bits<1><<<g, 256, 0, st>>>(s, d, ls, ld, n, mk); break;
            case 2: copy_generic_bits<2><<<g, 256, 0, st>>>(s, d, ls, ld, n, mk); break;
            case 4: copy_generic_bits<4><<<g, 256, 0, st>>>(s, d, ls, ld, n, mk); break;
            case 8: copy_generic_bits<8><<<g, 256, 0, st>>>(s, d, ls, ld, n, mk); break;
            case 16: copy_generic_bits<16><<<g, 256, 0, st>>>(s, d, ls, ld, n, mk); break;
            default: ok = false;
        }
    } else {
        switch (src->dtype) {
            case MOYE_F32: ok = launch_cvt_dst<MOYE_F32>(dst->dtype, g, st, s, d, ls, ld, n, sb, db, mk); break;
            case MOYE_F16: ok = launch_cvt_dst<MOYE_F16>(dst->dtype, g, st, s, d, ls, ld, n, sb, db, mk); break;
            case MOYE_BF16: ok = launch_cvt_dst<MOYE_BF16>(dst->dtype, g, st, s, d, ls, ld, n, sb, db, mk); break;
            case MOYE_F8E4M3: ok = launch_cvt_dst<MOYE_F8E4M3>(dst->dtype, g, st, s, d, ls, ld, n, sb, db, mk); break;
            case MOYE_F64: ok = launch_cvt_dst<MOYE_F64>(dst->dtype, g, st, s, d, ls, ld, n, sb, db, mk); break;
            default: ok = false;
        }
    }
    if (!ok) return fail(MOYE_ERR_UNSUPPORTED, "copyto!: no kernel for %s -> %s", dtype_name(src->dtype), dtype_name(dst->dtype));
    MOYE_HIP_CHECK(hipGetLastError());
    return MOYE_OK;
}

}  // namespace moye

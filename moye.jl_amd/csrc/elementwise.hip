// axpby!, fill!/zeros! and broadcast-style element-wise maps on device arrays with arbitrary layouts.
//
//   axpby!(a, X, b, Y)  (src/algorithm/blas.jl:1-9):  y[i] = iszero(b) ? a*x[i] : a*x[i] + b*y[i]
//   fill!(x, val), zeros!(x)  (src/algorithm/array_algorithms.jl:158-182)
//   dst .= a .+ b, a .* s, max.(a, b), ...  (src/broadcast.jl:5-41; map! src/algorithm/array_algorithms.jl:192-210)
// over the logical elements i of both layouts.  X and Y have the same element type T; a and b are
// converted to T first and every operation is rounded in T (Julia's Float16 arithmetic computes in
// Float32 and rounds after each operation; so does this), products and the sum never contracted
// into an fma: the file is compiled with -ffp-contract=off.
#include <algorithm>
#include <cstring>
#include <type_traits>

#include "mfma_common.hpp"

namespace moye {

// Second pass of a split-K gemm!: D[m][n] = cvt(epilogue(P_0 + P_1 + ... )[m][n]).  The partial products P_s are
// fp32, compact, with n contiguous and one after the other; they are summed in ascending s, so the result does not
// depend on timing.  The epilogue (alpha, beta * C, op) is the one the GEMM kernels apply, epi_value().
template <typename Out>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ P, int split, int64_t M, int64_t N,
                                                            GemmArgs e) {
    const int64_t total = M * N;
    const int64_t d_cs = e.ldd_n ? e.ldd_n : 1;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        float sum = P[i];
        for (int s = 1; s < split; ++s) sum += P[(int64_t)s * total + i];
        const int64_t m = i / N, n = i % N;
        const float c = e.C ? Out::load(e.C, m * e.ldc_m + n * e.ldc_n) : 0.f;
        static_cast<typename Out::type*>(e.D)[m * e.ldd + n * d_cs] = Out::cvt(epi_value(e, sum, e.C != nullptr, c, m, n));
    }
}

// The same, four neighbouring columns per lane in 16-byte pieces of the partial products, one piece per lane and no loop
// (N a multiple of four, D row-major with rows that start on whole pieces of four results).  The additions and the
// epilogue are the scalar kernel's, element by element, in the same order: the same bits.  (bf16 512 x 8192 in four ranges,
// partial products still in the caches: 16.6 us with the scalar kernel, 12.7 with this one.)
template <typename Out>
__global__ __launch_bounds__(256) void splitk_reduce_vec4_kernel(const float* __restrict__ P, int split, int64_t M, int64_t N, GemmArgs e) {
    typedef typename Out::type OutT;
    const int64_t total = M * N, i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= total) return;
    f32x4 sum = *reinterpret_cast<const f32x4*>(P + i);
#pragma unroll 4
    for (int s = 1; s < split; ++s) {
        const f32x4 v = *reinterpret_cast<const f32x4*>(P + (int64_t)s * total + i);
        sum.x += v.x; sum.y += v.y; sum.z += v.z; sum.w += v.w;
    }
    const int64_t m = i / N, n = i - m * N;
    OutT out[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const float c = e.C ? Out::load(e.C, m * e.ldc_m + (n + k) * e.ldc_n) : 0.f;
        out[k] = Out::cvt(epi_value(e, sum[k], e.C != nullptr, c, m, n + k));
    }
    typedef typename std::conditional<sizeof(OutT) == 4, u32x4, u32x2>::type piece;
    piece w;
    __builtin_memcpy(&w, out, sizeof w);
    *reinterpret_cast<piece*>(static_cast<OutT*>(e.D) + m * e.ldd + n) = w;
}

int32_t splitk_reduce_dispatch(const float* P, int split, int64_t M, int64_t N, const GemmArgs& e, int32_t out_dt, hipStream_t st) {
    const int64_t ob = dtype_bytes(out_dt);
    if (N % 4 == 0 && (e.ldd_n == 0 || e.ldd_n == 1) && e.ldd % 4 == 0 && reinterpret_cast<uintptr_t>(e.D) % (4 * ob) == 0 &&
        reinterpret_cast<uintptr_t>(P) % 16 == 0 && (M * N / 4 + 255) / 256 < ((int64_t)1 << 31)) {
        const dim3 grid4((unsigned)((M * N / 4 + 255) / 256));
        switch (out_dt) {
            case MOYE_F32: splitk_reduce_vec4_kernel<OutF32><<<grid4, 256, 0, st>>>(P, split, M, N, e); break;
            case MOYE_F16: splitk_reduce_vec4_kernel<OutF16><<<grid4, 256, 0, st>>>(P, split, M, N, e); break;
            case MOYE_BF16: splitk_reduce_vec4_kernel<OutBF16><<<grid4, 256, 0, st>>>(P, split, M, N, e); break;
            default: return fail(MOYE_ERR_UNSUPPORTED, "gemm!: MFMA kernels write f32, f16 or bf16, not %s", dtype_name(out_dt));
        }
        MOYE_HIP_CHECK(hipGetLastError());
        return MOYE_OK;
    }
    const dim3 grid((unsigned)std::min<int64_t>((M * N + 255) / 256, 256 * 32));
    switch (out_dt) {
        case MOYE_F32: splitk_reduce_kernel<OutF32><<<grid, 256, 0, st>>>(P, split, M, N, e); break;
        case MOYE_F16: splitk_reduce_kernel<OutF16><<<grid, 256, 0, st>>>(P, split, M, N, e); break;
        case MOYE_BF16: splitk_reduce_kernel<OutBF16><<<grid, 256, 0, st>>>(P, split, M, N, e); break;
        default: return fail(MOYE_ERR_UNSUPPORTED, "gemm!: MFMA kernels write f32, f16 or bf16, not %s", dtype_name(out_dt));
    }
    MOYE_HIP_CHECK(hipGetLastError());
    return MOYE_OK;
}

namespace {
struct ELayout {
    int32_t rank;
    int64_t shape[MOYE_MAX_RANK];
    int64_t stride[MOYE_MAX_RANK];
};

// colexicographic decomposition of a 0-based linear index (src/stride.jl:20-31)
__device__ __forceinline__ int64_t e_offset(const ELayout& l, int64_t i) {
    int64_t off = 0;
#pragma unroll 1
    for (int m = 0; m < l.rank; ++m) {
        const int64_t s = l.shape[m], q = i / s;
        off += (i - q * s) * l.stride[m];
        i = q;
    }
    return off;
}

// The same for up to three layouts of one shape, mode by mode, and an index below 2^31: the index is taken apart once,
// with 32-bit divisions, and the coordinates are weighed with each layout's strides (the 64-bit divisions of e_offset,
// once per layout and mode, set the pace of these kernels otherwise).
__device__ __forceinline__ void e_offsets(const ELayout& a, const ELayout& b, const ELayout& c, uint32_t i, int64_t* oa, int64_t* ob, int64_t* oc) {
    int64_t xa = 0, xb = 0, xc = 0;
#pragma unroll 1
    for (int m = 0; m < a.rank; ++m) {
        const uint32_t extent = (uint32_t)a.shape[m], q = i / extent, r = i - q * extent;
        xa += (int64_t)r * a.stride[m];
        xb += (int64_t)r * b.stride[m];
        xc += (int64_t)r * c.stride[m];
        i = q;
    }
    *oa = xa;
    *ob = xb;
    *oc = xc;
}
// layouts of one shape mode by mode, few enough elements for 32-bit indices (host side)
bool same_modes_32(const ELayout& a, const ELayout& b, int64_t n) {
    if (a.rank != b.rank || n >= ((int64_t)1 << 31)) return false;
    for (int m = 0; m < a.rank; ++m)
        if (a.shape[m] != b.shape[m] || a.shape[m] <= 0) return false;
    return true;
}

ELayout elayout_of(const moye_tensor& t) {
    ELayout f;
    f.rank = t.rank;
    for (int i = 0; i < MOYE_MAX_RANK; ++i) {
        f.shape[i] = i < t.rank ? t.shape[i] : 1;
        f.stride[i] = i < t.rank ? t.stride[i] : 0;
    }
    return f;
}

// (a NaN stays as it is; everything else through v_cvt_pk_bf16_f32, round to nearest even)
__device__ __forceinline__ float e_bf16_round(float f) {
    if (f != f) return f;
    return __uint_as_float((uint32_t)__builtin_bit_cast(uint16_t, (__bf16)f) << 16);
}

// element traits: load to / store from the compute type, round a compute-type value to T
struct ElF32 {
    typedef float compute;
    typedef float storage;
    static __device__ __forceinline__ float load(const float* p) { return *p; }
    static __device__ __forceinline__ void store(float* p, float v) { *p = v; }
    static __device__ __forceinline__ float round(float v) { return v; }
};
struct ElF64 {
    typedef double compute;
    typedef double storage;
    static __device__ __forceinline__ double load(const double* p) { return *p; }
    static __device__ __forceinline__ void store(double* p, double v) { *p = v; }
    static __device__ __forceinline__ double round(double v) { return v; }
};
struct ElF16 {
    typedef float compute;
    typedef _Float16 storage;
    static __device__ __forceinline__ float load(const _Float16* p) { return (float)*p; }
    static __device__ __forceinline__ void store(_Float16* p, float v) { *p = (_Float16)v; }
    static __device__ __forceinline__ float round(float v) { return (float)(_Float16)v; }
};
struct ElBF16 {
    typedef float compute;
    typedef uint16_t storage;
    static __device__ __forceinline__ float load(const uint16_t* p) { return __uint_as_float((uint32_t)*p << 16); }
    static __device__ __forceinline__ void store(uint16_t* p, float v) { *p = (uint16_t)(__float_as_uint(e_bf16_round(v)) >> 16); }
    static __device__ __forceinline__ float round(float v) { return e_bf16_round(v); }
};

template <typename El>
__global__ __launch_bounds__(256) void axpby_kernel(typename El::compute a, const typename El::storage* x, ELayout lx,
                                                    typename El::compute b, typename El::storage* y, ELayout ly,
                                                    int64_t n, bool b_is_zero, bool same = false) {
    typedef typename El::compute T;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        int64_t ox, oy, unused;
        if (same) e_offsets(lx, ly, ly, (uint32_t)i, &ox, &oy, &unused);
        else ox = e_offset(lx, i), oy = e_offset(ly, i);
        const T ax = El::round(a * El::load(x + ox));
        typename El::storage* yp = y + oy;
        if (b_is_zero) {
            El::store(yp, ax);
        } else {
            const T by = El::round(b * El::load(yp));
            El::store(yp, El::round(ax + by));
        }
    }
}


template <typename T>
__device__ __forceinline__ T map_op(int32_t op, T x, T y) {
    switch (op) {
        case MOYE_MAP_ADD: return x + y;
        case MOYE_MAP_SUB: return x - y;
        case MOYE_MAP_MUL: return x * y;
        case MOYE_MAP_DIV: return x / y;
        // Julia's max/min for floats (base/math.jl): a NaN operand is returned; max(-0.0, 0.0) == 0.0
        case MOYE_MAP_MAX: return ((y > x) | (signbit(y) < signbit(x))) ? (x != x ? x : y) : (y != y ? y : x);
        case MOYE_MAP_MIN: return ((y < x) | (signbit(y) > signbit(x))) ? (x != x ? x : y) : (y != y ? y : x);
        case MOYE_MAP_NEG: return -x;
        case MOYE_MAP_ABS: return signbit(x) ? -x : x;
        default: return x;  // MOYE_MAP_IDENTITY
    }
}

// dst[i] = f(a[i], b[i % nb]) or f(a[i], s): b may be a whole array (nb == n) or span the leading modes of dst
// and repeat over the trailing ones (Julia's broadcasting of a lower-rank array), or absent (scalar operand)
template <typename El>
__global__ __launch_bounds__(256) void map_kernel(int32_t op, typename El::storage* d, ELayout ld,
                                                  const typename El::storage* a, ELayout la,
                                                  const typename El::storage* b, ELayout lb, int64_t nb,
                                                  typename El::compute s, int64_t n, bool same = false) {
    typedef typename El::compute T;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        int64_t oa, ob = 0, od;
        if (same) {
            e_offsets(la, lb, ld, (uint32_t)i, &oa, &ob, &od);  // (lb unused without b: its strides weigh nothing that is read)
        } else {
            oa = e_offset(la, i);
            if (b) ob = e_offset(lb, i % nb);
            od = e_offset(ld, i);
        }
        const T x = El::load(a + oa);
        const T y = b ? El::load(b + ob) : s;
        El::store(d + od, El::round(map_op(op, x, y)));
    }
}

template <int kBytes>
__global__ __launch_bounds__(256) void fill_kernel(char* x, ELayout lx, int64_t n, uint64_t bits) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        char* p = x + e_offset(lx, i) * kBytes;
        if constexpr (kBytes == 1) *reinterpret_cast<uint8_t*>(p) = (uint8_t)bits;
        else if constexpr (kBytes == 2) *reinterpret_cast<uint16_t*>(p) = (uint16_t)bits;
        else if constexpr (kBytes == 4) *reinterpret_cast<uint32_t*>(p) = (uint32_t)bits;
        else *reinterpret_cast<uint64_t*>(p) = bits;
    }
}

// ---- dense fast path ------------------------------------------------------------------------------------------
// When every array of a call is one run in logical order (compact column-major after dropping size-1 modes) and
// 16-byte aligned, logical index = memory index on all sides: 16 bytes per lane, one access per operand and lane, one
// workgroup per 4 KiB, no loop and no index arithmetic.  (Measured on 1 GiB arrays, a + b -> d: this form 6.4 TB/s with
// non-temporal accesses, 6.0 without; workgroups that loop over chunks with four accesses of a lane in flight 5.5-6.1
// whatever the grid; a fill 6.9 TB/s in this form with ordinary stores, 4.8-5.9 looping.)  The per-element arithmetic
// is the same code as in the general kernels.
template <typename El>
struct DenseVec {
    typedef typename El::storage S;
    static constexpr int N = 16 / (int)sizeof(S);
    typedef S type __attribute__((ext_vector_type(N)));
};

template <typename El>
__global__ __launch_bounds__(256) void axpby_dense_kernel(typename El::compute a, const typename El::storage* x,
                                                          typename El::compute b, typename El::storage* y, int64_t nvec,
                                                          bool b_is_zero) {
    typedef typename El::compute T;
    typedef typename El::storage S;
    typedef typename DenseVec<El>::type vec;
    constexpr int N = DenseVec<El>::N;
    const vec* xv = reinterpret_cast<const vec*>(x);
    vec* yv = reinterpret_cast<vec*>(y);
    auto one = [&](const vec& vx, const vec& vy) {
        vec r;
#pragma unroll
        for (int k = 0; k < N; ++k) {
            S ex = vx[k], ey = vy[k], er;
            const T ax = El::round(a * El::load(&ex));
            if (b_is_zero) El::store(&er, ax);
            else El::store(&er, El::round(ax + El::round(b * El::load(&ey))));
            r[k] = er;
        }
        return r;
    };
    const int64_t i = flat_piece();
    if (i >= nvec) return;
    const vec vx = __builtin_nontemporal_load(xv + i);
    __builtin_nontemporal_store(one(vx, b_is_zero ? vx : __builtin_nontemporal_load(yv + i)), yv + i);
}

template <typename El>
__global__ __launch_bounds__(256) void map_dense_kernel(int32_t op, typename El::storage* d, const typename El::storage* a,
                                                        const typename El::storage* b, typename El::compute s, int64_t nvec) {
    typedef typename El::compute T;
    typedef typename El::storage S;
    typedef typename DenseVec<El>::type vec;
    constexpr int N = DenseVec<El>::N;
    const vec* av = reinterpret_cast<const vec*>(a);
    const vec* bv = reinterpret_cast<const vec*>(b);
    vec* dv = reinterpret_cast<vec*>(d);
    auto one = [&](const vec& va, const vec& vb) {
        vec r;
#pragma unroll
        for (int k = 0; k < N; ++k) {
            S ea = va[k], eb = vb[k], er;
            const T x = El::load(&ea);
            const T y = b ? El::load(&eb) : s;
            El::store(&er, El::round(map_op(op, x, y)));
            r[k] = er;
        }
        return r;
    };
    const int64_t i = flat_piece();
    if (i >= nvec) return;
    // (d may be a or b: every lane reads its own piece before it writes it)
    const vec va = __builtin_nontemporal_load(av + i);
    __builtin_nontemporal_store(one(va, b ? __builtin_nontemporal_load(bv + i) : va), dv + i);
}

__global__ __launch_bounds__(256) void fill_dense_kernel(u32x4* x, int64_t nvec, u32x4 pattern) {
    const int64_t i = flat_piece();
    if (i < nvec) x[i] = pattern;
}

// ---- rows of 16-byte pieces -----------------------------------------------------------------------------------
// Arrays that are not one run but whose first mode (after the modes were ordered by stride) has unit stride on every
// side, in whole aligned 16-byte pieces: the layouts are recast to 16-byte elements (first extent and every other
// stride divided by the piece's element count) and each lane takes one piece per operand, with the arithmetic of the
// general kernels.
template <typename El>
__global__ __launch_bounds__(256) void axpby_rows_kernel(typename El::compute a, const typename El::storage* x, ELayout lx,
                                                         typename El::compute b, typename El::storage* y, ELayout ly, int64_t nvec,
                                                         bool b_is_zero, bool same) {
    typedef typename El::compute T;
    typedef typename El::storage S;
    typedef typename DenseVec<El>::type vec;
    constexpr int N = DenseVec<El>::N;
    const vec* xv = reinterpret_cast<const vec*>(x);
    vec* yv = reinterpret_cast<vec*>(y);
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < nvec; i += (int64_t)gridDim.x * 256) {
        int64_t ox, oy, unused;
        if (same) e_offsets(lx, ly, ly, (uint32_t)i, &ox, &oy, &unused);
        else ox = e_offset(lx, i), oy = e_offset(ly, i);
        const vec vx = xv[ox];
        vec* py = yv + oy;
        const vec vy = b_is_zero ? vx : *py;
        vec r;
#pragma unroll
        for (int k = 0; k < N; ++k) {
            S ex = vx[k], ey = vy[k], er;
            const T ax = El::round(a * El::load(&ex));
            if (b_is_zero) El::store(&er, ax);
            else El::store(&er, El::round(ax + El::round(b * El::load(&ey))));
            r[k] = er;
        }
        *py = r;
    }
}

template <typename El>
__global__ __launch_bounds__(256) void map_rows_kernel(int32_t op, typename El::storage* d, ELayout ld, const typename El::storage* a,
                                                       ELayout la, const typename El::storage* b, ELayout lb, typename El::compute s,
                                                       int64_t nvec, bool same) {
    typedef typename El::compute T;
    typedef typename El::storage S;
    typedef typename DenseVec<El>::type vec;
    constexpr int N = DenseVec<El>::N;
    const vec* av = reinterpret_cast<const vec*>(a);
    const vec* bv = reinterpret_cast<const vec*>(b);
    vec* dv = reinterpret_cast<vec*>(d);
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < nvec; i += (int64_t)gridDim.x * 256) {
        int64_t oa, ob = 0, od;
        if (same) {
            e_offsets(la, lb, ld, (uint32_t)i, &oa, &ob, &od);  // (lb unused without b: its strides weigh nothing that is read)
        } else {
            oa = e_offset(la, i);
            if (b) ob = e_offset(lb, i);
            od = e_offset(ld, i);
        }
        const vec va = av[oa];
        const vec vb = b ? bv[ob] : va;
        vec r;
#pragma unroll
        for (int k = 0; k < N; ++k) {
            S ea = va[k], eb = vb[k], er;
            const T x = El::load(&ea);
            const T y = b ? El::load(&eb) : s;
            El::store(&er, El::round(map_op(op, x, y)));
            r[k] = er;
        }
        dv[od] = r;
    }
}

__global__ __launch_bounds__(256) void fill_rows_kernel(u32x4* x, ELayout lx, int64_t nvec, u32x4 pattern) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < nvec; i += (int64_t)gridDim.x * 256) x[e_offset(lx, i)] = pattern;
}

// ---- an operand whose unit stride lies on another mode than the destination's -----------------------------------------
// (d = a + b' with b' a transposed view, axpby! between a column-major and a row-major array.)  The general kernels
// read such an operand in single elements a pitch apart.  Here a workgroup takes a TILE x TILE block of the two modes
// concerned -- mode 0, the destination's unit stride, and mode j, that operand's --, brings the operand's block into LDS
// along mode j (rows padded by one element: both directions free of bank conflicts for 4-byte elements) and computes
// along mode 0, reading the destination and every operand that is laid out like it directly.  The modes beside these
// two are taken apart once per workgroup.  The arithmetic is the general kernels'.
struct EwTiled {
    ELayout ld, l0, l1;      // destination, first and second operand (same modes, ordered by the destination's strides)
    int32_t j;               // the mode whose stride is 1 in the operands that go through LDS
    int32_t tiles_p, tiles_q;
    bool lds0, lds1, has1;
};

// V > 1: a lane takes that many neighbouring elements wherever it runs along a unit stride (eight 2-byte or two 4-byte
// elements); extents, pitches and pointers then have to be multiples of V (groups_ok below).
template <typename El, int TILE, int V, bool kMap>
__global__ __launch_bounds__(256) void ew_tiled_kernel(int32_t op, typename El::compute ca, typename El::compute cb, bool b_is_zero,
                                                       typename El::storage* d, const typename El::storage* u0,
                                                       const typename El::storage* u1, EwTiled g) {
    typedef typename El::compute T;
    typedef typename El::storage S;
    typedef S SV __attribute__((ext_vector_type(V)));
    extern __shared__ __align__(16) char tile_bytes[];  // one padded block per operand that goes through LDS
    S* const tile0 = reinterpret_cast<S*>(tile_bytes);
    S* const tile1 = tile0 + (g.lds0 ? TILE * (TILE + 1) : 0);
    const uint32_t bid = blockIdx.x;
    const uint32_t tp = bid % (uint32_t)g.tiles_p, rest0 = bid / (uint32_t)g.tiles_p;
    const uint32_t tq = rest0 % (uint32_t)g.tiles_q;
    uint32_t rest = rest0 / (uint32_t)g.tiles_q;
    int64_t bd = 0, b0 = 0, b1 = 0;  // where this workgroup's block starts in each array, the two tiled modes aside
#pragma unroll 1
    for (int m = 1; m < g.ld.rank; ++m) {
        if (m == g.j) continue;
        const uint32_t extent = (uint32_t)g.ld.shape[m], q = rest / extent, r = rest - q * extent;
        bd += (int64_t)r * g.ld.stride[m];
        b0 += (int64_t)r * g.l0.stride[m];
        b1 += (int64_t)r * g.l1.stride[m];
        rest = q;
    }
    const int64_t p0 = (int64_t)tp * TILE, q0 = (int64_t)tq * TILE;
    const int np = (int)min((int64_t)TILE, g.ld.shape[0] - p0), nq = (int)min((int64_t)TILE, g.ld.shape[g.j] - q0);
    constexpr int LR = TILE / V;  // lanes along a row of the block
    const int lo = V * (threadIdx.x % LR), hi0 = threadIdx.x / LR;
    constexpr int STEP = 256 / LR, IT = TILE / STEP;
    // (every loop below has IT trips with the bounds as predicates, so that a lane's IT loads are in flight together)
    // the operands that run along mode j: lanes along j, the block's rows of mode 0 one after the other
    if (g.lds0 || g.lds1) {
        SV r0[IT], r1[IT];
#pragma unroll
        for (int k = 0; k < IT; ++k) {
            const int lp = hi0 + k * STEP;
            r0[k] = r1[k] = SV(S(0));
            if (lo < nq && lp < np) {
                if (g.lds0) r0[k] = *reinterpret_cast<const SV*>(u0 + b0 + (p0 + lp) * g.l0.stride[0] + (q0 + lo));
                if (g.lds1) r1[k] = *reinterpret_cast<const SV*>(u1 + b1 + (p0 + lp) * g.l1.stride[0] + (q0 + lo));
            }
        }
#pragma unroll
        for (int k = 0; k < IT; ++k) {
            const int lp = hi0 + k * STEP;
#pragma unroll
            for (int e = 0; e < V; ++e) {
                if (g.lds0) tile0[lp * (TILE + 1) + lo + e] = r0[k][e];
                if (g.lds1) tile1[lp * (TILE + 1) + lo + e] = r1[k][e];
            }
        }
        __syncthreads();
    }
    SV e0[IT], e1[IT], old[IT];
#pragma unroll
    for (int k = 0; k < IT; ++k) {
        const int lq = hi0 + k * STEP;
        const bool in = lo < np && lq < nq;
        e0[k] = e1[k] = old[k] = SV(S(0));
        if (g.lds0) {
#pragma unroll
            for (int e = 0; e < V; ++e) e0[k][e] = tile0[(lo + e) * (TILE + 1) + lq];
        } else if (in) {
            // (V = 2: the host has made sure of a unit stride along mode 0 for every operand read here)
            e0[k] = *reinterpret_cast<const SV*>(u0 + b0 + (p0 + lo) * g.l0.stride[0] + (q0 + lq) * g.l0.stride[g.j]);
        }
        if (kMap && g.has1) {
            if (g.lds1) {
#pragma unroll
                for (int e = 0; e < V; ++e) e1[k][e] = tile1[(lo + e) * (TILE + 1) + lq];
            } else if (in) {
                e1[k] = *reinterpret_cast<const SV*>(u1 + b1 + (p0 + lo) * g.l1.stride[0] + (q0 + lq) * g.l1.stride[g.j]);
            }
        }
        if (!kMap && !b_is_zero && in) old[k] = *reinterpret_cast<const SV*>(d + bd + (p0 + lo) + (q0 + lq) * g.ld.stride[g.j]);
    }
#pragma unroll
    for (int k = 0; k < IT; ++k) {
        const int lq = hi0 + k * STEP;
        if (lo >= np || lq >= nq) continue;
        SV out;
#pragma unroll
        for (int e = 0; e < V; ++e) {
            const S xe = e0[k][e], ye = e1[k][e], oe = old[k][e];
            S re;
            const T x = El::load(&xe);
            if constexpr (kMap) {
                const T y = g.has1 ? El::load(&ye) : cb;  // (cb: the scalar operand)
                El::store(&re, El::round(map_op(op, x, y)));
            } else {
                const T ax = El::round(ca * x);
                if (b_is_zero) El::store(&re, ax);
                else El::store(&re, El::round(ax + El::round(cb * El::load(&oe))));
            }
            out[e] = re;
        }
        *reinterpret_cast<SV*>(d + bd + (p0 + lo) + (q0 + lq) * g.ld.stride[g.j]) = out;
    }
}

// May the lanes take groups of v?  Extents along the two tiled modes that are multiples of v, every array with a unit
// stride along the mode its lanes run on, strides elsewhere that are multiples of v and a pointer on a whole group.
bool groups_ok(const EwTiled& g, const void* d, const void* u0, const void* u1, size_t elem, int v) {
    if (g.ld.shape[0] % v || g.ld.shape[g.j] % v) return false;
    auto whole_but = [&](const ELayout& l, int unit) {
        if (l.stride[unit] != 1) return false;
        for (int m = 0; m < l.rank; ++m)
            if (m != unit && l.shape[m] != 1 && l.stride[m] % v) return false;
        return true;
    };
    auto on_group = [&](const void* p) { return reinterpret_cast<uintptr_t>(p) % (v * elem) == 0; };
    if (!whole_but(g.ld, 0) || !on_group(d)) return false;
    if (!whole_but(g.l0, g.lds0 ? g.j : 0) || !on_group(u0)) return false;
    if (g.has1 && (!whole_but(g.l1, g.lds1 ? g.j : 0) || !on_group(u1))) return false;
    return true;
}

// Does the tiled kernel apply?  Layouts of one shape, ordered by the destination's strides (order_modes_by_stride), the
// destination's unit stride on mode 0, and an operand whose unit stride lies on another mode j with at least 16
// elements along both; every other operand runs along mode 0 or along j as well, or is read as it comes.
bool plan_tiled(const ELayout& ld, const ELayout* const* ops, int nops, int tile, EwTiled* g) {
    if (ld.rank < 2 || ld.stride[0] != 1 || ld.shape[0] < 16) return false;
    int j = -1;
    for (int q = 0; q < nops && j < 0; ++q) {
        if (ops[q]->stride[0] == 1) continue;
        for (int m = 1; m < ld.rank; ++m)
            if (ops[q]->stride[m] == 1 && ld.shape[m] >= 16) { j = m; break; }
    }
    if (j < 0) return false;
    g->ld = ld;
    g->l0 = *ops[0];
    g->l1 = nops > 1 ? *ops[1] : *ops[0];
    g->has1 = nops > 1;
    g->j = j;
    g->lds0 = ops[0]->stride[0] != 1 && ops[0]->stride[j] == 1;
    g->lds1 = nops > 1 && ops[1]->stride[0] != 1 && ops[1]->stride[j] == 1;
    const int64_t tp = (ld.shape[0] + tile - 1) / tile, tq = (ld.shape[j] + tile - 1) / tile;
    int64_t rest = 1;
    for (int m = 1; m < ld.rank; ++m)
        if (m != j) rest *= ld.shape[m];
    if (tp * tq * rest >= ((int64_t)1 << 31) || rest >= ((int64_t)1 << 31)) return false;
    g->tiles_p = (int32_t)tp;
    g->tiles_q = (int32_t)tq;
    return true;
}
template <typename El>
constexpr int tiled_edge() { return sizeof(typename El::storage) == 8 ? 32 : 64; }
template <typename El>
constexpr int tiled_edge_pairs() { return sizeof(typename El::storage) == 2 ? 128 : 64; }
template <typename El>
size_t tiled_lds(const EwTiled& g, int edge) {
    return (size_t)((g.lds0 ? 1 : 0) + (g.lds1 ? 1 : 0)) * edge * (edge + 1) * sizeof(typename El::storage);
}
// (the block edge of the form with groups differs for 2-byte elements: the plan is made again for it)
template <typename El, bool kMap>
bool launch_tiled(int32_t op, typename El::compute ca, typename El::compute cb, bool b_is_zero, typename El::storage* d, const ELayout& ld,
                  const typename El::storage* u0, const typename El::storage* u1, const ELayout* const* ops, int nops, int64_t n, hipStream_t st) {
    EwTiled g;
    if (!plan_tiled(ld, ops, nops, tiled_edge<El>(), &g)) return false;
    const int64_t rest = n / (ld.shape[0] * ld.shape[g.j]);
    if constexpr (sizeof(typename El::storage) <= 4) {
        EwTiled g2;
        // (8192^2, axpby! with X transposed / map! add with b transposed, TB/s: f32 two per lane 3.95 / 4.01, four 3.64 / 3.97;
        // f16 two per lane 3.04 / 2.50, four 5.14 / 3.23, eight 5.90 / 3.61)
        constexpr int E2 = tiled_edge_pairs<El>(), V2 = sizeof(typename El::storage) == 2 ? 8 : 2;
        // (two 2-byte operands through LDS would take 66 KB: above what a launch gets without asking)
        if (groups_ok(g, d, u0, u1, sizeof(typename El::storage), V2) && plan_tiled(ld, ops, nops, E2, &g2) && tiled_lds<El>(g2, E2) <= 65536) {
            ew_tiled_kernel<El, E2, V2, kMap><<<(unsigned)((int64_t)g2.tiles_p * g2.tiles_q * rest), 256, tiled_lds<El>(g2, E2), st>>>(op, ca, cb, b_is_zero, d, u0, u1, g2);
            return true;
        }
    }
    constexpr int E1 = tiled_edge<El>();
    ew_tiled_kernel<El, E1, 1, kMap><<<(unsigned)((int64_t)g.tiles_p * g.tiles_q * rest), 256, tiled_lds<El>(g, E1), st>>>(op, ca, cb, b_is_zero, d, u0, u1, g);
    return true;
}

// Can every one of these (same-shape, stride-ordered) layouts be recast to pieces of `per` elements?  If so, does it.
bool recast_rows(ELayout* const* ls, const void* const* ptrs, int count, int per) {
    if (per <= 1) return false;
    for (int q = 0; q < count; ++q) {
        const ELayout& l = *ls[q];
        if (l.rank < 1 || l.stride[0] != 1 || l.shape[0] % per || reinterpret_cast<uintptr_t>(ptrs[q]) % 16) return false;
        for (int m = 1; m < l.rank; ++m)
            if (l.shape[m] != 1 && l.stride[m] % per) return false;
    }
    for (int q = 0; q < count; ++q) {
        ELayout& l = *ls[q];
        l.shape[0] /= per;
        for (int m = 1; m < l.rank; ++m) l.stride[m] /= per;
    }
    return true;
}

// one run in logical order?
bool dense(const moye_tensor& t) {
    int64_t expect = 1;
    for (int i = 0; i < t.rank; ++i) {
        if (t.shape[i] == 1) continue;
        if (t.stride[i] != expect) return false;
        expect *= t.shape[i];
    }
    return true;
}
// the same for a layout whose modes have been ordered by stride: an element-wise operation may visit the elements in
// any order, so a dense row-major array (or any permutation of a compact layout) is one run as well
bool dense_l(const ELayout& l) {
    int64_t expect = 1;
    for (int i = 0; i < l.rank; ++i) {
        if (l.shape[i] == 1) continue;
        if (l.stride[i] != expect) return false;
        expect *= l.shape[i];
    }
    return true;
}
bool aligned16(const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; }

ELayout run_layout(int64_t n) {  // a rank-1 run of n elements: what is left of a dense array behind its last whole 16 bytes
    ELayout l{};
    l.rank = 1;
    for (int i = 0; i < MOYE_MAX_RANK; ++i) { l.shape[i] = 1; l.stride[i] = 0; }
    l.shape[0] = n;
    l.stride[0] = 1;
    return l;
}

int64_t count(const moye_tensor& t) {
    int64_t n = 1;
    for (int i = 0; i < t.rank; ++i) n *= t.shape[i];
    return n;
}

// host-side rounding of the scalars to T, the same way the kernels round
float host_round_f16(float v) { return (float)(_Float16)v; }
float host_round_bf16(float f) {
    uint32_t u;
    std::memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return f;
    u += 0x7fffu + ((u >> 16) & 1u);
    u &= 0xffff0000u;
    std::memcpy(&f, &u, 4);
    return f;
}
}  // namespace

template <typename El>
static void launch_axpby(typename El::compute a, const void* x, const ELayout& lx, typename El::compute b, void* y, const ELayout& ly,
                         int64_t n, bool is_dense, bool rows, bool ordered, hipStream_t st) {
    typedef typename El::storage S;
    const S* xs = static_cast<const S*>(x);
    S* ys = static_cast<S*>(y);
    const bool b0 = b == (typename El::compute)0;
    if (!is_dense && rows) {  // lx, ly are in 16-byte pieces
        const int64_t nvec = n / DenseVec<El>::N;
        axpby_rows_kernel<El><<<strided_grid(nvec), 256, 0, st>>>(a, xs, lx, b, ys, ly, nvec, b0, same_modes_32(lx, ly, nvec));
        return;
    }
    if (!is_dense) {
        const ELayout* ops[1] = {&lx};
        if (ordered && launch_tiled<El, false>(0, a, b, b0, ys, ly, xs, xs, ops, 1, n, st)) return;
        const dim3 grid((unsigned)std::min<int64_t>((n + 255) / 256, 256 * 16));
        axpby_kernel<El><<<grid, 256, 0, st>>>(a, xs, lx, b, ys, ly, n, b0, same_modes_32(lx, ly, n));
        return;
    }
    constexpr int N = DenseVec<El>::N;
    const int64_t nvec = n / N, tail = n - nvec * N;
    if (nvec) axpby_dense_kernel<El><<<flat_grid(nvec), 256, 0, st>>>(a, xs, b, ys, nvec, b0);
    if (tail) axpby_kernel<El><<<1, 64, 0, st>>>(a, xs + nvec * N, run_layout(tail), b, ys + nvec * N, run_layout(tail), tail, b0);
}

template <typename El>
static void launch_map(int32_t op, void* d, const ELayout& ld, const void* a, const ELayout& la, const void* b, const ELayout& lb,
                       int64_t nb, typename El::compute s, int64_t n, bool is_dense, bool rows, bool ordered, hipStream_t st) {
    typedef typename El::storage S;
    S* ds = static_cast<S*>(d);
    const S* as = static_cast<const S*>(a);
    const S* bs = static_cast<const S*>(b);
    if (!is_dense && rows) {  // ld, la, lb are in 16-byte pieces
        const int64_t nvec = n / DenseVec<El>::N;
        map_rows_kernel<El><<<strided_grid(nvec), 256, 0, st>>>(op, ds, ld, as, la, bs, lb, s, nvec,
                                                                same_modes_32(ld, la, nvec) && (!bs || same_modes_32(ld, lb, nvec)));
        return;
    }
    if (!is_dense) {
        const ELayout* ops[2] = {&la, &lb};
        if (ordered && launch_tiled<El, true>(op, s, s, false, ds, ld, as, bs ? bs : as, ops, bs ? 2 : 1, n, st)) return;
        const dim3 grid((unsigned)std::min<int64_t>((n + 255) / 256, 256 * 16));
        map_kernel<El><<<grid, 256, 0, st>>>(op, ds, ld, as, la, bs, lb, nb, s, n,
                                             same_modes_32(ld, la, n) && (!bs || (nb == n && same_modes_32(ld, lb, n))));
        return;
    }
    constexpr int N = DenseVec<El>::N;
    const int64_t nvec = n / N, tail = n - nvec * N;
    if (nvec) map_dense_kernel<El><<<flat_grid(nvec), 256, 0, st>>>(op, ds, as, bs, s, nvec);
    if (tail)
        map_kernel<El><<<1, 64, 0, st>>>(op, ds + nvec * N, run_layout(tail), as + nvec * N, run_layout(tail), bs ? bs + nvec * N : nullptr,
                                         run_layout(tail), tail, s, tail);
}

int32_t axpby_dispatch(double a, const moye_tensor* X, double b, const moye_tensor* Y, hipStream_t st) {
    if (int32_t e = check_tensor(X, "X")) return e;
    if (int32_t e = check_tensor(Y, "Y")) return e;
    if (X->dtype != Y->dtype) return fail(MOYE_ERR_UNSUPPORTED, "axpby!: X and Y must have the same element type");
    const int64_t n = count(*X);
    if (count(*Y) != n) return fail(MOYE_ERR_SHAPE, "axpby!: X holds %lld elements, Y %lld", (long long)n, (long long)count(*Y));
    if (n == 0) return MOYE_OK;
    ELayout lx = elayout_of(*X), ly = elayout_of(*Y);
    bool fast = dense(*X) && dense(*Y) && aligned16(X->ptr) && aligned16(Y->ptr);
    bool rows = false, ordered = false;  // ordered: the layouts have one shape mode by mode and are sorted by Y's strides
    if (!fast) {
        ELayout* all[2] = {&ly, &lx};
        const void* ptrs[2] = {Y->ptr, X->ptr};
        if (order_modes_by_stride(all, 2)) {
            ordered = true;
            if (dense_l(lx) && dense_l(ly) && aligned16(X->ptr) && aligned16(Y->ptr)) fast = true;  // one run each, in the same order
            else rows = recast_rows(all, ptrs, 2, 16 / dtype_bytes(X->dtype));
        }
    }
    switch (X->dtype) {
        case MOYE_F32: launch_axpby<ElF32>((float)a, X->ptr, lx, (float)b, Y->ptr, ly, n, fast, rows, ordered, st); break;
        case MOYE_F64: launch_axpby<ElF64>(a, X->ptr, lx, b, Y->ptr, ly, n, fast, rows, ordered, st); break;
        case MOYE_F16: launch_axpby<ElF16>(host_round_f16((float)a), X->ptr, lx, host_round_f16((float)b), Y->ptr, ly, n, fast, rows, ordered, st); break;
        case MOYE_BF16: launch_axpby<ElBF16>(host_round_bf16((float)a), X->ptr, lx, host_round_bf16((float)b), Y->ptr, ly, n, fast, rows, ordered, st); break;
        default:
            return fail(MOYE_ERR_UNSUPPORTED, "axpby!: element type %s is not a floating-point type this build handles", dtype_name(X->dtype));
    }
    MOYE_HIP_CHECK(hipGetLastError());
    return MOYE_OK;
}


// dst .= op.(A, B) / op.(A, scalar) / op.(A): every array has the same floating-point element type T, the scalar
// is converted to T first and the result of the one operation is rounded in T
int32_t map_dispatch(int32_t op, const moye_tensor* D, const moye_tensor* A, const moye_tensor* B, double scalar,
                     hipStream_t st) {
    if (op < MOYE_MAP_IDENTITY || op > MOYE_MAP_ABS) return fail(MOYE_ERR_UNSUPPORTED, "map!: unknown operation %d", op);
    if (int32_t e = check_tensor(D, "dst")) return e;
    if (int32_t e = check_tensor(A, "a")) return e;
    if (B) if (int32_t e = check_tensor(B, "b")) return e;
    if (A->dtype != D->dtype || (B && B->dtype != D->dtype))
        return fail(MOYE_ERR_UNSUPPORTED, "map!: all arrays must have the element type of the destination (%s)", dtype_name(D->dtype));
    const int64_t n = count(*D);
    if (count(*A) != n) return fail(MOYE_ERR_SHAPE, "map!: dst holds %lld elements, a %lld", (long long)n, (long long)count(*A));
    int64_t nb = 1;
    if (B) {
        nb = count(*B);
        // b must be dst-sized or span a leading group of dst's modes
        bool ok = nb == n;
        int64_t lead = 1;
        for (int i = 0; i < D->rank && !ok; ++i) {
            lead *= D->shape[i];
            ok = lead == nb;
        }
        if (!ok && nb != 1)
            return fail(MOYE_ERR_SHAPE, "map!: cannot broadcast %lld elements of b over the %lld of dst", (long long)nb, (long long)n);
    }
    if (n == 0) return MOYE_OK;
    ELayout ld = elayout_of(*D), la = elayout_of(*A), lb = B ? elayout_of(*B) : ELayout{};
    const void* bp = B ? B->ptr : nullptr;
    bool fast = dense(*D) && dense(*A) && aligned16(D->ptr) && aligned16(A->ptr) &&
                (!B || (nb == n && dense(*B) && aligned16(B->ptr)));
    bool rows = false, ordered = false;
    if (!fast && (!B || nb == n)) {  // (a b that is broadcast is tied to the leading modes of dst as the caller wrote them)
        ELayout* all[3] = {&ld, &la, &lb};
        const void* ptrs[3] = {D->ptr, A->ptr, bp};
        if (order_modes_by_stride(all, B ? 3 : 2)) {
            ordered = true;
            if (dense_l(ld) && dense_l(la) && (!B || dense_l(lb)) && aligned16(D->ptr) && aligned16(A->ptr) && (!B || aligned16(B->ptr))) fast = true;
            else rows = recast_rows(all, ptrs, B ? 3 : 2, 16 / dtype_bytes(D->dtype));
        }
    }
    switch (D->dtype) {
        case MOYE_F32: launch_map<ElF32>(op, D->ptr, ld, A->ptr, la, bp, lb, nb, (float)scalar, n, fast, rows, ordered, st); break;
        case MOYE_F64: launch_map<ElF64>(op, D->ptr, ld, A->ptr, la, bp, lb, nb, scalar, n, fast, rows, ordered, st); break;
        case MOYE_F16: launch_map<ElF16>(op, D->ptr, ld, A->ptr, la, bp, lb, nb, host_round_f16((float)scalar), n, fast, rows, ordered, st); break;
        case MOYE_BF16: launch_map<ElBF16>(op, D->ptr, ld, A->ptr, la, bp, lb, nb, host_round_bf16((float)scalar), n, fast, rows, ordered, st); break;
        default:
            return fail(MOYE_ERR_UNSUPPORTED, "map!: element type %s is not a floating-point type this build handles", dtype_name(D->dtype));
    }
    MOYE_HIP_CHECK(hipGetLastError());
    return MOYE_OK;
}

// `value` is converted to the element type (floating-point types: round to nearest even; integer types: truncation)
int32_t fill_dispatch(const moye_tensor* X, double value, hipStream_t st) {
    if (int32_t e = check_tensor(X, "x")) return e;
    const int64_t n = count(*X);
    if (n == 0) return MOYE_OK;
    uint64_t bits = 0;
    switch (X->dtype) {
        case MOYE_F32: { const float f = (float)value; uint32_t u; std::memcpy(&u, &f, 4); bits = u; break; }
        case MOYE_F64: std::memcpy(&bits, &value, 8); break;
        case MOYE_F16: { const _Float16 h = (_Float16)(float)value; uint16_t u; std::memcpy(&u, &h, 2); bits = u; break; }
        case MOYE_BF16: { const float f = host_round_bf16((float)value); uint32_t u; std::memcpy(&u, &f, 4); bits = u >> 16; break; }
        case MOYE_U8: case MOYE_U16: case MOYE_U32: case MOYE_U64: bits = (uint64_t)(int64_t)value; break;
        default: return fail(MOYE_ERR_UNSUPPORTED, "fill!: no conversion to %s", dtype_name(X->dtype));
    }
    char* p = static_cast<char*>(X->ptr);
    const int eb = dtype_bytes(X->dtype);
    if (eb < 8) bits &= (1ull << (8 * eb)) - 1;  // integer values wrap to the element's width
    ELayout lx = elayout_of(*X);
    bool ordered = false;
    {
        ELayout* all[1] = {&lx};
        ordered = order_modes_by_stride(all, 1);
    }
    if ((dense(*X) || (ordered && dense_l(lx))) && aligned16(p)) {  // the value repeated over 16 bytes, then what is left behind the last whole 16 bytes
        uint64_t rep = bits;
        for (int w = eb; w < 8; w *= 2) rep |= rep << (8 * w);
        const u32x4 pattern = {(uint32_t)rep, (uint32_t)(rep >> 32), (uint32_t)rep, (uint32_t)(rep >> 32)};
        const int64_t nvec = n * eb / 16, tail = n - nvec * (16 / eb);
        if (nvec) fill_dense_kernel<<<flat_grid(nvec), 256, 0, st>>>(reinterpret_cast<u32x4*>(p), nvec, pattern);
        if (tail) {
            char* q = p + nvec * 16;
            switch (eb) {
                case 1: fill_kernel<1><<<1, 64, 0, st>>>(q, run_layout(tail), tail, bits); break;
                case 2: fill_kernel<2><<<1, 64, 0, st>>>(q, run_layout(tail), tail, bits); break;
                case 4: fill_kernel<4><<<1, 64, 0, st>>>(q, run_layout(tail), tail, bits); break;
                default: fill_kernel<8><<<1, 64, 0, st>>>(q, run_layout(tail), tail, bits); break;
            }
        }
        MOYE_HIP_CHECK(hipGetLastError());
        return MOYE_OK;
    }
    const dim3 grid((unsigned)std::min<int64_t>((n + 255) / 256, 256 * 16));
    {
        ELayout* all[1] = {&lx};
        const void* ptrs[1] = {p};
        if (ordered && recast_rows(all, ptrs, 1, 16 / eb)) {  // the value repeated over 16 bytes
            uint64_t rep = bits;
            for (int w = eb; w < 8; w *= 2) rep |= rep << (8 * w);
            const u32x4 pattern = {(uint32_t)rep, (uint32_t)(rep >> 32), (uint32_t)rep, (uint32_t)(rep >> 32)};
            const int64_t nvec = n / (16 / eb);
            fill_rows_kernel<<<strided_grid(nvec), 256, 0, st>>>(reinterpret_cast<u32x4*>(p), lx, nvec, pattern);
            MOYE_HIP_CHECK(hipGetLastError());
            return MOYE_OK;
        }
    }
    switch (eb) {
        case 1: fill_kernel<1><<<grid, 256, 0, st>>>(p, lx, n, bits); break;
        case 2: fill_kernel<2><<<grid, 256, 0, st>>>(p, lx, n, bits); break;
        case 4: fill_kernel<4><<<grid, 256, 0, st>>>(p, lx, n, bits); break;
        default: fill_kernel<8><<<grid, 256, 0, st>>>(p, lx, n, bits); break;
    }
    MOYE_HIP_CHECK(hipGetLastError());
    return MOYE_OK;
}

}  // namespace moye

// C entry points of libmoye_hip for the device loops and the small runtime helpers.
// Descriptor validation lives here: the shape/divisibility violations the reference raises as
// Julia assertions while tracing (src/algorithm/blas.jl:55-57,79-82, src/int_tuple.jl:88,
// src/atom/copy.jl:121-122) come back as status codes before any kernel is launched.
#include <cstring>
#include <map>
#include <mutex>
#include <utility>
#include <vector>

#include "kernels.hpp"
#include "gemm_plan.hpp"

namespace moye {

std::string& last_error() {
    thread_local std::string e;
    return e;
}

int32_t fail(moye_status st, const char* fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    last_error() = buf;
    return (int32_t)st;
}

int32_t check_tensor(const moye_tensor* t, const char* what) {
    if (!t) return fail(MOYE_ERR_ARG, "%s: null tensor descriptor", what);
    if (t->rank < 1 || t->rank > MOYE_MAX_RANK)
        return fail(MOYE_ERR_RANK, "%s: rank %d outside 1..%d", what, t->rank, MOYE_MAX_RANK);
    if (dtype_bytes(t->dtype) == 0) return fail(MOYE_ERR_UNSUPPORTED, "%s: unknown dtype %d", what, t->dtype);
    for (int i = 0; i < t->rank; ++i) {
        if (t->shape[i] < 0) return fail(MOYE_ERR_SHAPE, "%s: negative extent in mode %d", what, i + 1);
        if (t->stride[i] < 0) return fail(MOYE_ERR_UNSUPPORTED, "%s: negative strides are not supported", what);
    }
    if (tensor_size(*t) > 0 && !t->ptr) return fail(MOYE_ERR_ARG, "%s: null data pointer", what);
    if (t->memspace != MOYE_GMEM)
        return fail(MOYE_ERR_UNSUPPORTED, "%s: only global-memory arrays cross the C ABI (shared memory and registers "
                                          "live inside the kernels)", what);
    return MOYE_OK;
}

int32_t as_matrix(const moye_tensor* t, const char* what, Mat* m) {
    if (int32_t e = check_tensor(t, what)) return e;
    if (t->rank != 2) return fail(MOYE_ERR_RANK, "%s: gemm! operands are rank-2, got rank %d", what, t->rank);
    m->ptr = static_cast<char*>(t->ptr);
    m->rows = t->shape[0];
    m->cols = t->shape[1];
    m->rs = t->stride[0];
    m->cs = t->stride[1];
    m->dtype = t->dtype;
    return MOYE_OK;
}

static int32_t atom_input_dtype(int32_t atom) {
    switch (atom) {
        case MOYE_MFMA_F32_16x16x32_F16: case MOYE_MFMA_F32_32x32x16_F16: return MOYE_F16;
        case MOYE_MFMA_F32_16x16x32_BF16: case MOYE_MFMA_F32_32x32x16_BF16: return MOYE_BF16;
        case MOYE_MFMA_F32_16x16x32_FP8: case MOYE_MFMA_F32_32x32x16_FP8: return MOYE_F8E4M3;
        case MOYE_MFMA_F32_16x16x4_F32: case MOYE_MFMA_F32_32x32x2_F32: return MOYE_F32;
        default: return -1;
    }
}

// ---- workspace: K-major copies of operands that are not K-major, partial products of split-K -------
// moye_gemm_ex takes the workspace from its caller and allocates nothing.  moye_gemm keeps the
// library's own: one buffer per (device, stream), allocated on the first call that needs one (a
// synchronous hipMalloc inside that call) and replaced by a larger one when a larger call comes.  A
// replaced buffer is not freed in the call path, since work queued earlier on the stream may still
// use it: it is parked until moye_gemm_release_workspace().  g_ws_mutex is held from the lookup to
// the last enqueue of a call, so two host threads that share a stream cannot interleave the halves
// (transpose, GEMM, reduction) of their calls; calls on different streams have different buffers.
struct LibWorkspace {
    char* ptr = nullptr;
    size_t bytes = 0;
};
static std::mutex g_ws_mutex;
static std::map<std::pair<int, hipStream_t>, LibWorkspace> g_ws;
static std::vector<void*> g_ws_parked;

// caller holds g_ws_mutex
static int32_t library_workspace(size_t bytes, hipStream_t st, char** out) {
    int dev = 0;
    MOYE_HIP_CHECK(hipGetDevice(&dev));
    LibWorkspace& w = g_ws[{dev, st}];
    if (bytes > w.bytes) {
        // (at least twice the old size, so that calls that grow a little at a time park few buffers)
        const size_t grown = std::max(bytes, 2 * w.bytes);
        void* p = nullptr;
        if (hipMalloc(&p, grown) != hipSuccess) {
            (void)hipGetLastError();
            MOYE_HIP_CHECK(hipMalloc(&p, bytes));
            w.bytes = bytes;
        } else {
            w.bytes = grown;
        }
        if (w.ptr) g_ws_parked.push_back(w.ptr);
        w.ptr = static_cast<char*>(p);
    }
    *out = w.ptr;
    return MOYE_OK;
}

// ---- moye_gemm_noalloc: the workspace is a static device array ----------------------------------
// For callers that cannot allocate (under graph capture, in serving loops): the split-K partial
// products and the K-major operand copies go into this array instead of an allocated buffer.  Every
// GPU the library runs on holds its own copy at its own address until the process ends; the address
// is asked for once per device, with that device current, and only that address (never the array's
// name, which on the host is a stand-in) is handed to kernels.
constexpr size_t kScratchBytes = MOYE_NOALLOC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];
constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static char* g_scratch_ptr[kMaxDevices];

static int32_t scratch_of_current_device(char** out) {
    int dev = 0;
    MOYE_HIP_CHECK(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return fail(MOYE_ERR_ARG, "moye_gemm_noalloc: device index %d beyond %d", dev, kMaxDevices - 1);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        MOYE_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (!p) return fail(MOYE_ERR_HIP, "moye_gemm_noalloc: the static scratch array has no address on device %d", dev);
        g_scratch_ptr[dev] = static_cast<char*>(p);
    }
    *out = g_scratch_ptr[dev];
    return MOYE_OK;
}

// bytes of a K-major copy of an (rows x K) operand: row pitch rounded up to 16 bytes
static size_t kmajor_bytes(const Mat& m) {
    const int eb = dtype_bytes(m.dtype);
    const int64_t pitch = (m.cols * eb + 15) / 16 * 16;
    return (size_t)(m.rows * pitch + 255) / 256 * 256;
}

// K ranges for the short-M kernel that stages lines through LDS, when N is small and K long: N = 1024 puts 64 workgroups
// of 16 rows of B on 256 CUs, and a workgroup streams its rows at about 64 GB/s whatever the others do.  The model of
// gemm_short_m_us (gemm_plan.hpp), fitted to bf16 timings (M = 16: 1024 x 32768 37.8 unsplit, 18.3 in four ranges;
// 2048 x 16384 22.2, 17.1 in two; 1024 x 8192 12.1, 10.7 in four; 2048 x 8192 12.6, 11.7 in two: left alone; M = 32,
// 1024 x 8192 15.6, 10.7 in four; M = 64, 2048 x 8192 22.7, 17.9 in two, 20.4 in four).  Ranges are whole lines of 2 KiB
// and more; at most two above M = 32 (every workgroup reads its range of all of A, which then dominates); taken when
// the model gains a tenth, the fewest ranges within 5 % of the best.
static int skinny_lines_split(int64_t M, int64_t N, int64_t k_bytes, int cus) {
    if ((N + 31) / 32 >= cus) return 1;  // 32 rows of B per workgroup and every CU has one
    double t1;
    gemm_short_m_ntw(M, N, k_bytes, cus, 1, &t1);
    double t[9];
    double best = t1;
    const int max_split = M > 32 ? 2 : 8;
    for (int sp = 2; sp <= max_split; ++sp) {
        t[sp] = 1e30;
        if (k_bytes % ((int64_t)sp * kSkinnyLineBytes) || k_bytes / sp < 2048) continue;
        gemm_short_m_ntw(M, N, k_bytes, cus, sp, &t[sp]);
        best = std::min(best, t[sp]);
    }
    if (best > 0.9 * t1) return 1;
    for (int sp = 2; sp <= max_split; ++sp)
        if (t[sp] <= 1.05 * best) return sp;
    return 1;
}

// What the chip looks like to the planner (kernels.hpp).  Asked once per device; a host without a device plans for 256 / 8.
DeviceShape device_shape_for(int cus) {
    if (cus > 0) return DeviceShape{cus, cus >= 32 ? cus / 32 : 1};
    return device_shape();
}
DeviceShape device_shape() {
    static std::mutex m;
    static DeviceShape cached[kMaxDevices];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        (void)hipGetLastError();
        return DeviceShape{256, 8};
    }
    std::lock_guard<std::mutex> lock(m);
    if (cached[dev].cus == 0) {
        int cus = 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) {
            (void)hipGetLastError();
            return DeviceShape{256, 8};
        }
        cached[dev] = device_shape_for(cus);  // gfx950: 32 CUs to an XCD; a partitioned part shows fewer of both
    }
    return cached[dev];
}

GemmStep& GemmPlan::add_kernel(void (*kernel)(GemmArgs), const GemmArgs& a, unsigned grid_x, unsigned grid_y, unsigned block, int lds_bytes,
                               LdsCap* cap, int tile_m, int tile_n, int tile_k_bytes, int in_dt, int out_dt, const char* fmt, ...) {
    steps.emplace_back();
    GemmStep& st = steps.back();
    st.kind = GemmStep::kKernel;
    st.kernel = kernel;
    st.args = a;
    st.args.xcds = shape.xcds;
    st.grid_x = grid_x; st.grid_y = grid_y; st.block = block;
    st.lds_bytes = lds_bytes;
    st.cap = cap;
    st.tile_m = tile_m; st.tile_n = tile_n; st.tile_k_bytes = tile_k_bytes;
    st.in_dt = in_dt; st.out_dt = out_dt;
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(st.name, sizeof st.name, fmt, ap);
    va_end(ap);
    return st;
}

// What the library decides when tile, waves and K ranges are all left to it: one answer for the workspace sizing and the
// dispatcher (gemm_choose, gemm_plan.hpp).  `open`: the call leaves all of that open and runs on the MFMA kernels that
// take a choice (M above 64 or K not in whole 64-byte pieces; 16-byte pieces of K).
struct LibraryChoice {
    bool open = false;
    TileChoice tile{128, 1, 0.0};
};
static LibraryChoice library_choice(const moye_tiled_mma* mma, int64_t M, int64_t N, int64_t K, int eb, int cus) {
    LibraryChoice c;
    const bool short_m = gemm_short_m(M, N, K * eb, eb == 4, cus);
    if (mma->split_k >= 0 || mma->cta_tile_mnk[0] || mma->cta_tile_mnk[1] || mma->cta_tile_mnk[2] || short_m || (K * eb) % 16) return c;
    c.open = true;
    c.tile = gemm_choose(M, N, K * eb, eb == 4, (mma->flags & MOYE_GEMM_NO_WORKSPACE) ? 1 : 16, cus);
    return c;
}

// split_k of the descriptor -> number of K ranges.  Negative = the library chooses: with the tile left to the library too,
// what the cost model of gemm_plan.hpp finds cheapest together with the tile (none where 256 x 256 tiles come out
// cheapest); with a named tile, none when the problem's 128 x 128 tiles fill half the chip,
// else the largest count up to cus / tiles that cuts K into equal ranges of whole 128-byte pieces of at least 512 bytes.
static int split_count(const moye_tiled_mma* mma, int64_t M, int64_t N, int64_t K, int eb, int cus) {
    if (mma->split_k >= 0) return mma->split_k > 1 ? mma->split_k : 1;
    if (mma->flags & MOYE_GEMM_NO_WORKSPACE) return 1;  // nowhere to put the partial products
    if (mma->cta_tile_mnk[0] == 0 && mma->cta_tile_mnk[1] == 0 && gemm_short_m(M, N, K * eb, eb == 4, cus)) {
        // the short-M kernel (gemm_mfma_skinny.hip): fastest unsplit when its workgroups fill the chip (bf16 64 x 8192 x 8192:
        // 30.4 us against 41.3 with two ranges and the second pass); K ranges are whole lines
        return skinny_lines_split(M, N, K * eb, cus);
    }
    if (const LibraryChoice c = library_choice(mma, M, N, K, eb, cus); c.open) return c.tile.split;
    const int64_t tiles = ((M + 127) / 128) * ((N + 127) / 128);
    if (tiles <= 0 || tiles >= cus / 2) return 1;
    for (int64_t s = std::min<int64_t>(cus / tiles, K); s >= 2; --s)
        if (K % s == 0 && ((K / s) * eb) % 128 == 0 && (K / s) * eb >= 512) return (int)s;
    return 1;
}

// An operand with its unit stride along M (N) instead of K needs no K-major copy when the call runs on kernels whose
// fragment reads transpose: f16 / bf16 through the 16x16x32 atoms on whole 256 x 256 x 64 tiles on eight waves (the
// hand-ordered kernel, gemm_mfma256w4.hip, for plain calls; the load-to-LDS kernel otherwise) or whole 128 x 128 x 64 tiles
// (named, or the library's own choice for a problem of whole 128 x 128 tiles with more than 64 rows), the two-stage
// schedule, no K ranges; fp8 and fp32 on the hand-ordered kernel's whole 256 x 256 or 128 x 128 tiles with 128 bytes of K
// per k-step (named so, or left to the library: 256 x 256 tiles when the problem has at least 128 of them), plain calls; the operand dense
// along its rows with a pitch of whole 16-byte pieces, and D 16-byte aligned (the guarded instances, which take any D,
// read K-major operands only).
static bool majors_run_natively(const moye_tiled_mma* mma, const Mat& A, const Mat& B, const Mat& D, const moye_gemm_epilogue& ep,
                                bool has_c, int cus) {
    const bool b16 = mma->atom == MOYE_MFMA_F32_16x16x32_F16 || mma->atom == MOYE_MFMA_F32_16x16x32_BF16;
    const bool wide = mma->atom == MOYE_MFMA_F32_16x16x32_FP8 || mma->atom == MOYE_MFMA_F32_16x16x4_F32;  // hand-ordered kernel only
    if (!b16 && !wide) return false;
    if ((mma->flags & (MOYE_GEMM_PINGPONG | MOYE_GEMM_WAVE4)) || mma->stages >= 3) return false;
    if (mma->split_k != 0 && mma->split_k != 1) return false;  // the K ranges of a split need not be whole k-tiles
    const int64_t M = A.rows, N = B.rows, K = A.cols;
    const int eb = dtype_bytes(A.dtype);
    const int bm = mma->cta_tile_mnk[0], bn = mma->cta_tile_mnk[1], bk = mma->cta_tile_mnk[2];
    if ((K * eb) % 128) return false;
    const bool four_waves = mma->atom_layout_mnk[0] * mma->atom_layout_mnk[1] == 4;
    const bool named256 = bm == 256 && bn == 256 && (b16 ? (bk == 0 || bk == 64) : bk * eb == 128) && !four_waves && M % 256 == 0 && N % 256 == 0;
    const bool named128 = bm == 128 && bn == 128 && bk * eb == 128 && M % 128 == 0 && N % 128 == 0;
    const bool chosen = bm == 0 && bn == 0 && bk == 0 && M > 64 && M % 128 == 0 && N % 128 == 0;
    if (wide) {
        // (the hand-ordered kernel reads such operands in plain calls only, and fp32 and fp8 have no other kernel that does)
        if (ep.op != MOYE_MAP_IDENTITY || mma->stages >= 2) return false;
        // (left to the library: whole 256 x 256 or 128 x 128 tiles, whichever the cost model prefers)
        if (!named256 && !named128 && !chosen) return false;
        // (fp32, left to the library, fewer 128 x 128 tiles than CUs: K-major copies and 64 x 64 tiles cost less than a
        // part-filled chip on the slow fp32 MFMA: 1024^3 38.5 us against 68.9)
        if (chosen && eb == 4 && (M / 128) * (N / 128) < cus) return false;
    } else if (!named256 && !named128 && !chosen) {
        return false;
    }
    (void)has_c;
    const int64_t d_pitch = D.cs == 1 ? D.rs : D.cs;
    if ((D.cs != 1 && D.rs != 1) || (d_pitch * dtype_bytes(D.dtype)) % 16 || reinterpret_cast<uintptr_t>(D.ptr) % 16) return false;
    for (const Mat* x : {&A, &B}) {
        if (x->cs == 1 || x->cols == 1) continue;  // K-major already
        if (x->rs != 1 || (x->cs * eb) % 16 || reinterpret_cast<uintptr_t>(x->ptr) % 16 || x->cs < x->rows) return false;
        if (wide && 256 * x->cs * eb >= ((int64_t)1 << 32)) return false;  // (the kernel's 32-bit lane offsets)
    }
    return true;
}

// K-major copies of A and B where needed, then the fp32 partial products of a split-K call
static size_t gemm_workspace_bytes_impl(const moye_tiled_mma* mma, const Mat& A, const Mat& B, bool native, int cus) {
    if (mma->atom == MOYE_MMA_UNIVERSAL_FMA) return 0;
    size_t n = 0;
    if (!native && A.cs != 1 && A.cols > 1) n += kmajor_bytes(A);
    if (!native && B.cs != 1 && B.cols > 1) n += kmajor_bytes(B);
    const int split = split_count(mma, A.rows, B.rows, A.cols, dtype_bytes(A.dtype), cus);
    if (split > 1) n += (size_t)split * (size_t)A.rows * (size_t)B.rows * sizeof(float);
    return n;
}

static size_t gemm_workspace_bytes(const moye_tiled_mma* mma, const Mat& A, const Mat& B, const Mat& D, const moye_gemm_epilogue& ep, int cus) {
    return gemm_workspace_bytes_impl(mma, A, B, majors_run_natively(mma, A, B, D, ep, false, cus), cus);
}

// A step that transposes `m` (unit stride along its rows index) into ws as rows x K with K contiguous; rewrites `m`
static void plan_kmajor_copy(Mat* m, char* ws, GemmPlan& plan) {
    const int eb = dtype_bytes(m->dtype);
    const int64_t pitch_e = ((m->cols * eb + 15) / 16 * 16) / eb;
    plan.steps.emplace_back();
    GemmStep& st = plan.steps.back();
    st.kind = GemmStep::kKMajorCopy;
    moye_tensor& src = st.copy_src;
    src.ptr = m->ptr; src.dtype = m->dtype; src.rank = 2; src.memspace = MOYE_GMEM;
    src.shape[0] = m->rows; src.shape[1] = m->cols; src.stride[0] = m->rs; src.stride[1] = m->cs;
    st.copy_dst = src;
    st.copy_dst.ptr = ws; st.copy_dst.stride[0] = pitch_e; st.copy_dst.stride[1] = 1;
    snprintf(st.name, sizeof st.name, "kmajor_copy");
    m->ptr = ws; m->rs = pitch_e; m->cs = 1;
}

// C as the 256 x 256 kernels' epilogue likes it: unit stride along the kernel's n, rows that start on 16-byte boundaries
static bool rows_in_16_byte_pieces(const void* c, int64_t ld_m, int64_t ld_n, int32_t dt) {
    return c && ld_n == 1 && reinterpret_cast<uintptr_t>(c) % 16 == 0 && (ld_m * dtype_bytes(dt)) % 16 == 0;
}

// gemm!(mma, D, A, B, C) as moye_gemm has always computed it: D = alpha * A * B' + C
static moye_gemm_epilogue plain_epilogue(float alpha) {
    moye_gemm_epilogue e{};
    e.alpha = alpha;
    e.beta = 1.f;
    e.op = MOYE_MAP_IDENTITY;
    return e;
}


// the epilogue operand as the 256 x 256 kernels like it: unit stride along the kernel's n, 16-byte aligned rows (or one row)
static bool operand_rows_in_16_byte_pieces(const GemmArgs& g) {
    if (!g.ep_x || g.ep_xn != 1) return false;
    const int eb = dtype_bytes(g.ep_xdt);
    return reinterpret_cast<uintptr_t>(g.ep_x) % 16 == 0 && (g.ep_xm * eb) % 16 == 0;
}

// an epilogue operation the lanes can apply to their own accumulators: its operand is a scalar, one value per column or one
// per row, or it has none (a bias, a ReLU, a scale); a division stays with the general epilogue (its code is long, and the
// lanes' form is unrolled over all accumulators)
static bool lane_op(const GemmArgs& g) {
    return g.ep_op != MOYE_MAP_IDENTITY && g.ep_op != MOYE_MAP_DIV && (!g.ep_x || g.ep_xm == 0 || g.ep_xn == 0);
}

// gemm!(mma, D, A, B, C) with the epilogue `ep` as a list of launches.  Pure host arithmetic on the descriptors: nothing
// is launched, allocated or asked of a device (plan.shape says what the chip looks like).  `workspace(bytes, &ptr)` is
// asked once, and only when the call needs a workspace, for `bytes` bytes: the caller's buffer, the library's own, the
// static scratch array, or -- for moye_gemm_explain -- an address that is never dereferenced.
template <typename WorkspaceSource>
static int32_t gemm_plan_build(const moye_tiled_mma* mma, const moye_tensor* tD, const moye_tensor* tA, const moye_tensor* tB,
                               const moye_tensor* tC, const moye_gemm_epilogue& ep, WorkspaceSource&& workspace, GemmPlan& plan) {
    if (!mma) return fail(MOYE_ERR_ARG, "gemm!: null TiledMMA descriptor");
    const int cus = plan.shape.cus;
    const float alpha = ep.alpha;
    if (ep.beta == 0.f) tC = nullptr;  // axpby!'s iszero(b): C is not read
    if (ep.op < MOYE_MAP_IDENTITY || ep.op > MOYE_MAP_ABS) return fail(MOYE_ERR_UNSUPPORTED, "gemm!: unknown epilogue operation %d", ep.op);
    Mat A, B, C{}, D;
    if (int32_t e = as_matrix(tA, "A", &A)) return e;
    if (int32_t e = as_matrix(tB, "B", &B)) return e;
    if (int32_t e = as_matrix(tD, "D", &D)) return e;
    if (tC) {
        if (int32_t e = as_matrix(tC, "C", &C)) return e;
    }
    // the stride of a mode of extent 1 is never used: a one-row operand with unit stride along its columns gets the
    // pitch a dense row-major array of its shape would have, so that it is not taken for M-major or misaligned
    for (Mat* x : {&A, &B, &C, &D})
        if (x->rows == 1 && x->cs == 1) x->rs = x->cols;
    // blas.jl:55-57,79-82: size(A,1)==size(C,1), size(B,1)==size(C,2), size(A,2)==size(B,2)
    if (A.rows != D.rows) return fail(MOYE_ERR_SHAPE, "gemm!: M of A (%lld) and D (%lld) differ", (long long)A.rows, (long long)D.rows);
    if (B.rows != D.cols) return fail(MOYE_ERR_SHAPE, "gemm!: N of B (%lld) and D (%lld) differ", (long long)B.rows, (long long)D.cols);
    if (A.cols != B.cols) return fail(MOYE_ERR_SHAPE, "gemm!: K of A (%lld) and B (%lld) differ", (long long)A.cols, (long long)B.cols);
    if (tC && (C.rows != D.rows || C.cols != D.cols)) return fail(MOYE_ERR_SHAPE, "gemm!: C and D differ in shape");
    if (A.rows > 0x7fffffff || B.rows > 0x7fffffff || A.cols > 0x7fffffff)
        return fail(MOYE_ERR_SHAPE, "gemm!: extents above 2^31-1 are not supported");
    if (A.rows == 0 || B.rows == 0) return MOYE_OK;
    const int M = (int)A.rows, N = (int)B.rows, K = (int)A.cols;
    int bm = mma->cta_tile_mnk[0], bn = mma->cta_tile_mnk[1], bk = mma->cta_tile_mnk[2];

    if (mma->atom == MOYE_MMA_UNIVERSAL_FMA) {
        if (mma->split_k > 1)
            return fail(MOYE_ERR_UNSUPPORTED, "gemm!: UniversalFMA sums k in ascending order (src/algorithm/blas.jl:63-67); split_k would change that");
        if (ep.op != MOYE_MAP_IDENTITY || (tC && ep.beta != 1.f))
            return fail(MOYE_ERR_UNSUPPORTED, "gemm!: UniversalFMA accumulates onto C as the reference does (src/algorithm/blas.jl:39-88): "
                                              "beta other than 0 or 1 and element-wise epilogue operations belong to the MFMA atoms");
        plan.steps.emplace_back();
        GemmStep& st = plan.steps.back();
        st.kind = GemmStep::kUniversal;
        st.uargs = UArgs{A.ptr, B.ptr, tC ? C.ptr : nullptr, D.ptr, M, N, K, A.rs, A.cs, B.rs, B.cs,
                         C.rs, C.cs, D.rs, D.cs, alpha, A.dtype, B.dtype, tC ? C.dtype : D.dtype, D.dtype};
        st.ubm = bm; st.ubn = bn; st.ubk = bk;
        snprintf(st.name, sizeof st.name, "gemm_universal<%d,%d,%d>", bm, bn, bk);
        return MOYE_OK;
    }
    const int32_t in_dt = atom_input_dtype(mma->atom);
    if (in_dt < 0) return fail(MOYE_ERR_UNSUPPORTED, "gemm!: unknown MMA atom %d", mma->atom);
    if (A.dtype != in_dt || B.dtype != in_dt)
        return fail(MOYE_ERR_UNSUPPORTED, "gemm!: atom takes %s operands, got A %s and B %s", dtype_name(in_dt),
                    dtype_name(A.dtype), dtype_name(B.dtype));
    if (tC && C.dtype != D.dtype) return fail(MOYE_ERR_UNSUPPORTED, "gemm!: C and D must have the same element type");
    const bool atom32 = mma->atom == MOYE_MFMA_F32_32x32x2_F32 || mma->atom == MOYE_MFMA_F32_32x32x16_F16 ||
                        mma->atom == MOYE_MFMA_F32_32x32x16_BF16 || mma->atom == MOYE_MFMA_F32_32x32x16_FP8;
    if (K == 0) return fail(MOYE_ERR_SHAPE, "gemm!: K == 0");
    // NN / NT / TT (the naming of src/arch/mma/make_mma_ops.jl:253-265): operands whose unit stride is not
    // along K are brought to the K-major form the kernels read (one tiled transpose each)
    char* ws = nullptr;
    const bool native_majors = majors_run_natively(mma, A, B, D, ep, tC != nullptr, plan.shape.cus);
    int major_flags = 0;  // which of the kernel's operands keep their M- (N-) major form
    if (native_majors) {
        if (A.cs != 1 && A.cols > 1) { major_flags |= kGemmAMajorM; A.rs = A.cs; A.cs = 1; }  // Mat::rs now holds the pitch between consecutive k
        if (B.cs != 1 && B.cols > 1) { major_flags |= kGemmBMajorN; B.rs = B.cs; B.cs = 1; }
    }
    plan.workspace_bytes = gemm_workspace_bytes_impl(mma, A, B, native_majors, cus);
    if (plan.workspace_bytes) {
        if (mma->flags & MOYE_GEMM_NO_WORKSPACE)
            return fail(MOYE_ERR_UNSUPPORTED, "gemm!: the MFMA kernels need K-major A and B (stride 1 along K, the 'TN' form), split_k needs room "
                                              "for its partial products, and MOYE_GEMM_NO_WORKSPACE forbids the use of a workspace");
        if (int32_t e = workspace(plan.workspace_bytes, &ws)) return e;
        plan.workspace = ws;
        if (!native_majors && A.cs != 1 && A.cols > 1) {
            const size_t nb = kmajor_bytes(A);
            plan_kmajor_copy(&A, ws, plan);
            ws += nb;
        }
        if (!native_majors && B.cs != 1 && B.cols > 1) {
            const size_t nb = kmajor_bytes(B);
            plan_kmajor_copy(&B, ws, plan);
            ws += nb;
        }
    }
    GemmArgs g{};
    g.beta = ep.beta;
    g.ep_op = ep.op;
    g.ep_scalar = (float)ep.scalar;
    const bool binary_op = ep.op != MOYE_MAP_IDENTITY && ep.op != MOYE_MAP_NEG && ep.op != MOYE_MAP_ABS;
    Mat X{};
    if (binary_op && ep.operand) {
        if (int32_t e = as_matrix(ep.operand, "epilogue operand", &X)) return e;
        if (X.rows != D.rows || X.cols != D.cols)
            return fail(MOYE_ERR_SHAPE, "gemm!: the epilogue operand is (%lld,%lld), D is (%lld,%lld); repeat a vector with a stride of 0",
                        (long long)X.rows, (long long)X.cols, (long long)D.rows, (long long)D.cols);
        if (X.dtype != MOYE_F32 && X.dtype != D.dtype)
            return fail(MOYE_ERR_UNSUPPORTED, "gemm!: the epilogue operand holds f32 or D's element type, not %s", dtype_name(X.dtype));
        g.ep_x = X.ptr; g.ep_xdt = X.dtype; g.ep_xm = X.rs; g.ep_xn = X.cs;
    }
    // TiledMMA.atom_layout_mnk = how many waves tile the CTA along M and N (src/atom/mma.jl:84)
    int waves = mma->atom_layout_mnk[0] * mma->atom_layout_mnk[1];
    g.alpha = alpha;
    g.K = K;
    g.xcds = plan.shape.xcds;
    // The XCDs start their walk over K a share of K apart when the problem is large enough for the column blocks they
    // ask memory for at one time to matter: more 256 x 256 tiles than CUs, or rows of 32 KiB and more (measured, 256 x 256
    // tile, same box, alternating runs: bf16 8192^3 1408 TFLOP/s against 1372, fp16 4096 x 4096 x 16384 +4 %; fp16 4096^3
    // 1333 against 1338, so not there)
    // A problem with a short side leans on memory, and its workgroups all walk K in step: with a power-of-two pitch they
    // then ask few memory channels for everything at one time.  bf16, a B that is not in the memory-side cache, us without ->
    // with the XCDs an eighth of K apart: 64 x 65536 x 2048 on 128 x 128 tiles 68.2 -> 46.8; 64 x 65536 x 4096 124.2 -> 92.2;
    // 128 x 65536 x 4096 126.3 -> 98.1; 256 x 65536 x 2048 75.3 -> 68.3; 512 x 16384 x 4096 80.9 -> 77.3; 1024 x 16384 x 2048
    // 58.3 -> 57.1; 2048 x 8192 x 2048 57.5 -> 56.9; 4096 x 4096 x 2048 52.4 -> 52.2.  So: a side of at most 1024.
    const bool rotate_k = (int64_t)(M / 256) * (N / 256) > cus || (int64_t)K * dtype_bytes(in_dt) >= 32768 || std::min(M, N) <= 1024;
    // D written with non-temporal stores (measured, same box, alternating runs, ordinary -> non-temporal, TFLOP/s): fp16
    // 4096^3 fp16 out 1339 -> 1345, fp32 out 1285 -> 1253; fp16 8192^3 fp16 out 1382 -> 1401; bf16 8192^3 fp32 out 1412 ->
    // 1452; fp8 4096^3 bf16 out 2373 -> 2450, 8192^3 2760 -> 2745; fp16 2048^3 and 3072^3 +1.6 %.  So: 16-bit results
    // always, except for the fp8 kernel on more tiles than CUs; 32-bit results when the launch has more 256 x 256 tiles
    // than the chip has CUs (then the results of one round would sit in the L2s in place of the next round's operands;
    // in a single round they are better left there for the end of the kernel to write back)
    const bool many_tiles = (int64_t)(M / 256) * (N / 256) > cus;
    const bool stream_d = dtype_bytes(D.dtype) == 2 ? !(in_dt == MOYE_F8E4M3 && many_tiles) : many_tiles;
    g.flags = !(mma->flags & MOYE_GEMM_NO_XCD_SWIZZLE) | (mma->flags & 0xff00) | (atom32 ? kGemmAtom32 : 0) | (rotate_k ? kGemmRotateK : 0) |
              (stream_d ? kGemmStreamD : 0) | major_flags;
    // tile and K ranges, where both are left to the library, are one decision (gemm_choose)
    const LibraryChoice lib = library_choice(mma, M, N, K, dtype_bytes(in_dt), cus);
    const TileChoice* lib_tile = lib.open ? &lib.tile : nullptr;
    if (const int split = split_count(mma, M, N, K, dtype_bytes(in_dt), cus); split > 1) {
        // K is cut into `split` equal ranges, all in one launch (gridDim.y); each range writes its fp32 product, compact and
        // row-major, into the workspace; a second pass sums the ranges in ascending order, applies alpha and C and converts
        const int eb = dtype_bytes(in_dt);
        if (split > 65535) return fail(MOYE_ERR_ARG, "gemm!: split_k = %d is beyond the 65535 ranges one launch holds", split);
        if (K % split || ((int64_t)(K / split) * eb) % 16)
            return fail(MOYE_ERR_SHAPE, "gemm!: split_k = %d needs K = %d to split into equal ranges of whole 16-byte pieces", split, K);
        const int Ks = K / split;
        float* P = reinterpret_cast<float*>(ws);
        GemmArgs r = g;  // the epilogue belongs to the second pass
        r.C = tC ? C.ptr : nullptr; r.ldc_m = C.rs; r.ldc_n = C.cs; r.D = D.ptr; r.ldd = D.rs; r.ldd_n = D.cs;
        r.M = M; r.N = N;
        g.alpha = 1.f; g.beta = 0.f; g.ep_op = MOYE_MAP_IDENTITY; g.ep_x = nullptr;
        g.K = Ks; g.M = M; g.N = N; g.lda = A.rs; g.ldb = B.rs; g.ldd = N; g.C = nullptr;
        g.A = A.ptr; g.B = B.ptr; g.D = P;
        g.split = split; g.split_ab = (int64_t)Ks * eb; g.split_d = (int64_t)M * N * (int64_t)sizeof(float);
        g.flags &= ~kGemmStreamD;  // the partial products are read back at once
        if (int32_t e = gemm_mfma_tn_dispatch(in_dt, MOYE_F32, bm, bn, bk, waves, mma->stages, g, plan, lib_tile)) return e;
        plan.steps.emplace_back();
        GemmStep& st = plan.steps.back();
        st.kind = GemmStep::kSplitKReduce;
        st.partials = P; st.split = split; st.args = r; st.out_dt = D.dtype; st.in_dt = MOYE_F32;
        snprintf(st.name, sizeof st.name, "splitk_reduce");
        return MOYE_OK;
    }
    if (D.cs == 1) {  // row-major D
        g.A = A.ptr; g.B = B.ptr; g.M = M; g.N = N; g.lda = A.rs; g.ldb = B.rs; g.ldd = D.rs;
        g.C = tC ? C.ptr : nullptr; g.ldc_m = C.rs; g.ldc_n = C.cs; g.D = D.ptr;
        if (rows_in_16_byte_pieces(g.C, g.ldc_m, g.ldc_n, D.dtype)) g.flags |= kGemmRowC;
        if (operand_rows_in_16_byte_pieces(g)) g.flags |= kGemmEpiRowX;
        if (lane_op(g)) g.flags |= kGemmEpiLaneOp;
        return gemm_mfma_tn_dispatch(in_dt, D.dtype, bm, bn, bk, waves, mma->stages, g, plan, lib_tile);
    }
    if (D.rs == 1 && bm == 0 && bn == 0 && gemm_short_m(M, N, (int64_t)K * dtype_bytes(in_dt), dtype_bytes(in_dt) == 4, plan.shape.cus)) {
        // column-major D with a short A: the short-M kernel writes D through both of its strides
        g.A = A.ptr; g.B = B.ptr; g.M = M; g.N = N; g.lda = A.rs; g.ldb = B.rs; g.ldd = 1; g.ldd_n = D.cs;
        g.C = tC ? C.ptr : nullptr; g.ldc_m = C.rs; g.ldc_n = C.cs; g.D = D.ptr;
        return gemm_mfma_skinny_dispatch(in_dt, D.dtype, g, plan);
    }
    if (D.rs == 1) {  // column-major D: D' = B * A' is row-major
        g.A = B.ptr; g.B = A.ptr; g.M = N; g.N = M; g.lda = B.rs; g.ldb = A.rs; g.ldd = D.cs;
        g.C = tC ? C.ptr : nullptr; g.ldc_m = C.cs; g.ldc_n = C.rs; g.D = D.ptr;
        std::swap(g.ep_xm, g.ep_xn);  // the kernel's m is the caller's n
        g.flags = (g.flags & ~(kGemmAMajorM | kGemmBMajorN)) | ((major_flags & kGemmAMajorM) ? kGemmBMajorN : 0) |
                  ((major_flags & kGemmBMajorN) ? kGemmAMajorM : 0);
        if (rows_in_16_byte_pieces(g.C, g.ldc_m, g.ldc_n, D.dtype)) g.flags |= kGemmRowC;
        if (operand_rows_in_16_byte_pieces(g)) g.flags |= kGemmEpiRowX;
        if (lane_op(g)) g.flags |= kGemmEpiLaneOp;
        // (the library's choice was priced for (M, N); the cost model is symmetric in them)
        return gemm_mfma_tn_dispatch(in_dt, D.dtype, bn, bm, bk, waves, mma->stages, g, plan, lib_tile);
    }
    return fail(MOYE_ERR_UNSUPPORTED, "gemm!: D needs a unit stride along M or N");
}

// Enqueues the steps of a plan on `st`, in order.  The only part of gemm! that talks to the device.
static int32_t gemm_plan_run(const GemmPlan& plan, hipStream_t st) {
    for (const GemmStep& s : plan.steps) {
        switch (s.kind) {
            case GemmStep::kKernel:
                if (s.cap)
                    if (int32_t e = raise_lds_cap(*s.cap, reinterpret_cast<const void*>(s.kernel), s.lds_bytes)) return e;
                hipLaunchKernelGGL(s.kernel, dim3(s.grid_x, s.grid_y), dim3(s.block), s.lds_bytes, st, s.args);
                MOYE_HIP_CHECK(hipGetLastError());
                break;
            case GemmStep::kKMajorCopy:
                if (int32_t e = copy_dispatch(nullptr, &s.copy_dst, &s.copy_src, st)) return e;
                break;
            case GemmStep::kSplitKReduce:
                if (int32_t e = splitk_reduce_dispatch(s.partials, s.split, s.args.M, s.args.N, s.args, s.out_dt, st)) return e;
                break;
            case GemmStep::kUniversal:
                if (int32_t e = gemm_universal_dispatch(s.ubm, s.ubn, s.ubk, s.uargs, st)) return e;
                break;
        }
    }
    return MOYE_OK;
}

// `caller_ws` / `caller_ws_bytes`: the workspace when the caller brings one (it must hold what moye_gemm_workspace_size
// reports); with caller_brings_ws == false the library's own per-stream buffer is used.
static int32_t gemm_impl(const moye_tiled_mma* mma, const moye_tensor* tD, const moye_tensor* tA,
                         const moye_tensor* tB, const moye_tensor* tC, const moye_gemm_epilogue& ep, bool caller_brings_ws, char* caller_ws,
                         size_t caller_ws_bytes, hipStream_t st) {
    std::unique_lock<std::mutex> ws_lock(g_ws_mutex, std::defer_lock);
    GemmPlan plan;
    plan.shape = device_shape();
    auto workspace = [&](size_t bytes, char** out) -> int32_t {
        if (caller_brings_ws) {
            if (bytes > caller_ws_bytes)
                return fail(MOYE_ERR_ARG, "gemm!: this call needs a workspace of %zu bytes, the one passed holds %zu", bytes, caller_ws_bytes);
            if (reinterpret_cast<uintptr_t>(caller_ws) % 256)
                return fail(MOYE_ERR_ALIGN, "gemm!: the workspace must start on a 256-byte boundary");
            *out = caller_ws;
            return MOYE_OK;
        }
        ws_lock.lock();  // until every kernel of this call is enqueued
        return library_workspace(bytes, st, out);
    };
    if (int32_t e = gemm_plan_build(mma, tD, tA, tB, tC, ep, workspace, plan)) return e;
    return gemm_plan_run(plan, st);
}

// "A+123" / "ws+456": where a pointer of a step lies, relative to the caller's arrays or the workspace
static void where(char* out, size_t cap, const void* p, const GemmPlan& plan, const moye_tensor* tA, const moye_tensor* tB, const moye_tensor* tD,
                  const moye_tensor* tC) {
    const char* q = static_cast<const char*>(p);
    if (!p) { snprintf(out, cap, "null"); return; }
    if (plan.workspace && q >= plan.workspace && q < plan.workspace + plan.workspace_bytes) { snprintf(out, cap, "ws+%lld", (long long)(q - plan.workspace)); return; }
    struct { const char* name; const moye_tensor* t; } arrays[] = {{"A", tA}, {"B", tB}, {"D", tD}, {"C", tC}};
    for (auto& a : arrays) {
        if (!a.t || !a.t->ptr) continue;
        const char* base = static_cast<const char*>(a.t->ptr);
        const int64_t bytes = tensor_cosize(*a.t) * dtype_bytes(a.t->dtype);
        if (q >= base && q < base + bytes) { snprintf(out, cap, "%s+%lld", a.name, (long long)(q - base)); return; }
    }
    snprintf(out, cap, "?");
}

static std::string flag_names(int f) {
    std::string s;
    auto add = [&](bool on, const char* n) { if (on) { if (!s.empty()) s += '|'; s += n; } };
    add(f & 1, "xcd_order"); add(f & MOYE_GEMM_PINGPONG, "pingpong"); add(f & MOYE_GEMM_PREDICATE, "predicate"); add(f & MOYE_GEMM_WAVE4, "hand_ordered");
    add(f & kGemmAtom32, "atom32"); add(f & kGemmRotateK, "rotate_k"); add(f & kGemmStreamD, "stream_d"); add(f & kGemmRowC, "row_c");
    add(f & kGemmAMajorM, "a_m_major"); add(f & kGemmBMajorN, "b_n_major"); add(f & kGemmEpiRowX, "row_x"); add(f & kGemmRagged, "ragged");
    add(f & kGemmEpiLaneOp, "lane_op");
    return s.empty() ? "0" : s;
}

static std::string explain_plan(const GemmPlan& plan, const moye_tensor* tA, const moye_tensor* tB, const moye_tensor* tD, const moye_tensor* tC) {
    std::string out;
    char line[1024], wa[48], wb[48], wd[48], wc[48];
    snprintf(line, sizeof line, "plan: %zu step(s), workspace %zu bytes, %d CUs in %d XCDs\n", plan.steps.size(), plan.workspace_bytes, plan.shape.cus, plan.shape.xcds);
    out += line;
    for (size_t i = 0; i < plan.steps.size(); ++i) {
        const GemmStep& s = plan.steps[i];
        switch (s.kind) {
            case GemmStep::kKernel: {
                const GemmArgs& a = s.args;
                where(wa, sizeof wa, a.A, plan, tA, tB, tD, tC); where(wb, sizeof wb, a.B, plan, tA, tB, tD, tC);
                where(wd, sizeof wd, a.D, plan, tA, tB, tD, tC); where(wc, sizeof wc, a.C, plan, tA, tB, tD, tC);
                snprintf(line, sizeof line,
                         "step %zu: kernel %s grid=%ux%u block=%u lds=%d tile=%dx%dx%dB in=%s out=%s M=%d N=%d K=%d lda=%lld ldb=%lld ldd=%lld ldd_n=%lld "
                         "A=%s B=%s D=%s C=%s a16=%d b16=%d d16=%d split=%d alpha=%g beta=%g op=%d flags=%s\n",
                         i, s.name, s.grid_x, s.grid_y, s.block, s.lds_bytes, s.tile_m, s.tile_n, s.tile_k_bytes, dtype_name(s.in_dt), dtype_name(s.out_dt), a.M, a.N,
                         a.K, (long long)a.lda, (long long)a.ldb, (long long)a.ldd, (long long)a.ldd_n, wa, wb, wd, wc,
                         (int)(reinterpret_cast<uintptr_t>(a.A) % 16 == 0), (int)(reinterpret_cast<uintptr_t>(a.B) % 16 == 0),
                         (int)(reinterpret_cast<uintptr_t>(a.D) % 16 == 0), a.split > 1 ? a.split : 1, (double)a.alpha, (double)a.beta, a.ep_op,
                         flag_names(a.flags).c_str());
                break;
            }
            case GemmStep::kKMajorCopy:
                where(wa, sizeof wa, s.copy_src.ptr, plan, tA, tB, tD, tC); where(wd, sizeof wd, s.copy_dst.ptr, plan, tA, tB, tD, tC);
                snprintf(line, sizeof line, "step %zu: kmajor_copy %s (%lld x %lld %s, strides %lld,%lld) -> %s (pitch %lld)\n", i, wa, (long long)s.copy_src.shape[0],
                         (long long)s.copy_src.shape[1], dtype_name(s.copy_src.dtype), (long long)s.copy_src.stride[0], (long long)s.copy_src.stride[1], wd,
                         (long long)s.copy_dst.stride[0]);
                break;
            case GemmStep::kSplitKReduce:
                where(wa, sizeof wa, s.partials, plan, tA, tB, tD, tC); where(wd, sizeof wd, s.args.D, plan, tA, tB, tD, tC);
                snprintf(line, sizeof line, "step %zu: splitk_reduce split=%d M=%d N=%d partials=%s D=%s out=%s alpha=%g beta=%g op=%d\n", i, s.split, s.args.M, s.args.N, wa,
                         wd, dtype_name(s.out_dt), (double)s.args.alpha, (double)s.args.beta, s.args.ep_op);
                break;
            case GemmStep::kUniversal:
                snprintf(line, sizeof line, "step %zu: kernel %s M=%d N=%d K=%d\n", i, s.name, s.uargs.M, s.uargs.N, s.uargs.K);
                break;
        }
        out += line;
    }
    return out;
}

// Average launch time of `iters` back-to-back launches, HIP events on the launch stream.
template <typename F>
static int32_t time_launches(F&& launch, hipStream_t st, int warmup, int iters, float* ms) {
    if (!ms || iters <= 0 || warmup < 0) return fail(MOYE_ERR_ARG, "timing: bad arguments");
    for (int i = 0; i < warmup; ++i)
        if (int32_t e = launch()) return e;
    hipEvent_t t0 = nullptr, t1 = nullptr;
    MOYE_HIP_CHECK(hipEventCreate(&t0));
    struct Events {  // destroyed on every way out
        hipEvent_t &a, &b;
        ~Events() {
            if (a) (void)hipEventDestroy(a);
            if (b) (void)hipEventDestroy(b);
        }
    } events{t0, t1};
    MOYE_HIP_CHECK(hipEventCreate(&t1));
    MOYE_HIP_CHECK(hipEventRecord(t0, st));
    int32_t err = MOYE_OK;
    for (int i = 0; i < iters && !err; ++i) err = launch();
    MOYE_HIP_CHECK(hipEventRecord(t1, st));
    MOYE_HIP_CHECK(hipEventSynchronize(t1));
    float total = 0.f;
    MOYE_HIP_CHECK(hipEventElapsedTime(&total, t0, t1));
    if (err) return err;
    *ms = total / (float)iters;
    return MOYE_OK;
}

}  // namespace moye

using namespace moye;

extern "C" {

int32_t moye_copy(const moye_tiled_copy* tc, const moye_tensor* dst, const moye_tensor* src, void* stream) {
    return copy_dispatch(tc, dst, src, static_cast<hipStream_t>(stream));
}

int32_t moye_gemm(const moye_tiled_mma* mma, const moye_tensor* D, const moye_tensor* A, const moye_tensor* B,
                  const moye_tensor* C, float alpha, void* stream) {
    return gemm_impl(mma, D, A, B, C, plain_epilogue(alpha), false, nullptr, 0, static_cast<hipStream_t>(stream));
}

int32_t moye_gemm_ex(const moye_tiled_mma* mma, const moye_tensor* D, const moye_tensor* A, const moye_tensor* B,
                     const moye_tensor* C, const moye_gemm_epilogue* ep, void* workspace, size_t workspace_bytes,
                     void* stream) {
    if (!ep) return fail(MOYE_ERR_ARG, "moye_gemm_ex: null epilogue descriptor");
    if (!workspace && workspace_bytes) return fail(MOYE_ERR_ARG, "moye_gemm_ex: null workspace of %zu bytes", workspace_bytes);
    // a call that needs no workspace may pass none; one that needs it and passes none fails: this entry never allocates
    return gemm_impl(mma, D, A, B, C, *ep, true, static_cast<char*>(workspace), workspace_bytes, static_cast<hipStream_t>(stream));
}

int32_t moye_gemm_noalloc(const moye_tiled_mma* mma, const moye_tensor* D, const moye_tensor* A, const moye_tensor* B,
                          const moye_tensor* C, float alpha, void* stream) {
    if (!mma || !D || !A || !B) return fail(MOYE_ERR_ARG, "moye_gemm_noalloc: null argument");
    size_t need = 0;
    if (int32_t e = moye_gemm_workspace_size(mma, D, A, B, &need)) return e;
    if (need > kScratchBytes)
        return fail(MOYE_ERR_ARG, "moye_gemm_noalloc: this call needs %zu bytes of workspace, the static scratch array holds %zu; "
                                  "use moye_gemm_ex with a workspace of the caller's", need, kScratchBytes);
    char* ws = nullptr;
    if (int32_t e = scratch_of_current_device(&ws)) return e;
    // every byte of the scratch a call reads it has written before (whole K-major copies, whole partial products), so
    // nothing needs clearing between calls
    return gemm_impl(mma, D, A, B, C, plain_epilogue(alpha), true, ws, kScratchBytes, static_cast<hipStream_t>(stream));
}

int32_t moye_gemm_explain(const moye_tiled_mma* mma, const moye_tensor* D, const moye_tensor* A, const moye_tensor* B,
                          const moye_tensor* C, const moye_gemm_epilogue* ep, int32_t compute_units, char* out, size_t cap) {
    if (!mma || !D || !A || !B || !out || cap == 0) return fail(MOYE_ERR_ARG, "moye_gemm_explain: null argument");
    out[0] = 0;
    GemmPlan plan;
    plan.shape = device_shape_for(compute_units);
    // the workspace of a plan that is only printed: an address nothing is read from or written to
    auto workspace = [](size_t, char** p) -> int32_t {
        *p = reinterpret_cast<char*>(uintptr_t(1) << 40);
        return MOYE_OK;
    };
    const moye_gemm_epilogue plain = plain_epilogue(1.f);
    if (int32_t e = gemm_plan_build(mma, D, A, B, C, ep ? *ep : plain, workspace, plan)) return e;
    const std::string text = explain_plan(plan, A, B, D, C);
    if (text.size() + 1 > cap) return fail(MOYE_ERR_BUFFER, "moye_gemm_explain: the plan takes %zu bytes of text, the buffer holds %zu", text.size() + 1, cap);
    memcpy(out, text.c_str(), text.size() + 1);
    return MOYE_OK;
}

int32_t moye_gemm_release_workspace(void) {
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    int current = 0;
    MOYE_HIP_CHECK(hipGetDevice(&current));
    struct Restore {  // the caller's device is current again on every way out
        int dev;
        ~Restore() { (void)hipSetDevice(dev); }
    } restore{current};
    int last = -1;
    for (auto& kv : g_ws) {  // ordered by device: wait once for each device that holds a buffer
        if (kv.first.first != last) {
            last = kv.first.first;
            MOYE_HIP_CHECK(hipSetDevice(last));
            MOYE_HIP_CHECK(hipDeviceSynchronize());
        }
        if (kv.second.ptr) g_ws_parked.push_back(kv.second.ptr);
    }
    g_ws.clear();
    for (void* p : g_ws_parked) (void)hipFree(p);
    g_ws_parked.clear();
    return MOYE_OK;
}

int32_t moye_axpby(double a, const moye_tensor* X, double b, const moye_tensor* Y, void* stream) {
    return axpby_dispatch(a, X, b, Y, static_cast<hipStream_t>(stream));
}

int32_t moye_fill(const moye_tensor* X, double value, void* stream) {
    return fill_dispatch(X, value, static_cast<hipStream_t>(stream));
}

int32_t moye_map(int32_t op, const moye_tensor* dst, const moye_tensor* a, const moye_tensor* b, double scalar,
                 void* stream) {
    return map_dispatch(op, dst, a, b, scalar, static_cast<hipStream_t>(stream));
}

int32_t moye_copy_if(const moye_tensor* dst, const moye_tensor* src, const moye_tensor* mask, void* stream) {
    if (!dst || !src || !mask) return fail(MOYE_ERR_ARG, "copyto_if!: null argument");
    return copy_if_dispatch(nullptr, dst, src, mask, static_cast<hipStream_t>(stream));
}

int32_t moye_gemm_workspace_size(const moye_tiled_mma* mma, const moye_tensor* D, const moye_tensor* A,
                                 const moye_tensor* B, size_t* bytes) {
    const moye_gemm_epilogue plain = plain_epilogue(1.f);
    return moye_gemm_ex_workspace_size(mma, D, A, B, &plain, bytes);
}

int32_t moye_gemm_ex_workspace_size(const moye_tiled_mma* mma, const moye_tensor* D, const moye_tensor* A,
                                    const moye_tensor* B, const moye_gemm_epilogue* ep, size_t* bytes) {
    if (!mma || !D || !A || !B || !ep || !bytes) return fail(MOYE_ERR_ARG, "moye_gemm_workspace_size: null argument");
    *bytes = 0;
    Mat a, b, d;
    if (int32_t e = as_matrix(A, "A", &a)) return e;
    if (int32_t e = as_matrix(B, "B", &b)) return e;
    if (int32_t e = as_matrix(D, "D", &d)) return e;
    for (Mat* x : {&a, &b, &d})
        if (x->rows == 1 && x->cs == 1) x->rs = x->cols;
    if (!(mma->flags & MOYE_GEMM_NO_WORKSPACE)) *bytes = gemm_workspace_bytes(mma, a, b, d, *ep, device_shape().cus);
    return MOYE_OK;
}

int32_t moye_device_malloc(void** ptr, size_t bytes) {
    if (!ptr) return fail(MOYE_ERR_ARG, "moye_device_malloc: null out pointer");
    MOYE_HIP_CHECK(hipMalloc(ptr, bytes));
    return MOYE_OK;
}
int32_t moye_device_free(void* ptr) {
    MOYE_HIP_CHECK(hipFree(ptr));
    return MOYE_OK;
}
int32_t moye_memcpy_h2d(void* dst, const void* src, size_t bytes) {
    MOYE_HIP_CHECK(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice));
    return MOYE_OK;
}
int32_t moye_memcpy_d2h(void* dst, const void* src, size_t bytes) {
    MOYE_HIP_CHECK(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost));
    return MOYE_OK;
}
int32_t moye_memset(void* dst, int value, size_t bytes) {
    MOYE_HIP_CHECK(hipMemset(dst, value, bytes));
    return MOYE_OK;
}
int32_t moye_device_sync(void) {
    MOYE_HIP_CHECK(hipDeviceSynchronize());
    return MOYE_OK;
}
int32_t moye_device_info(char* name, size_t cap, int32_t* compute_units, int32_t* clock_khz, size_t* total_mem) {
    int dev = 0;
    MOYE_HIP_CHECK(hipGetDevice(&dev));
    hipDeviceProp_t prop;
    MOYE_HIP_CHECK(hipGetDeviceProperties(&prop, dev));
    if (name && cap) {
        snprintf(name, cap, "%s (%s)", prop.name, prop.gcnArchName);
    }
    if (compute_units) *compute_units = prop.multiProcessorCount;
    if (clock_khz) *clock_khz = prop.clockRate;
    if (total_mem) *total_mem = prop.totalGlobalMem;
    return MOYE_OK;
}

int32_t moye_time_gemm(const moye_tiled_mma* mma, const moye_tensor* D, const moye_tensor* A, const moye_tensor* B,
                       const moye_tensor* C, float alpha, void* stream, int32_t warmup, int32_t iters,
                       float* ms_per_launch) {
    hipStream_t st = static_cast<hipStream_t>(stream);
    return time_launches([&] { return gemm_impl(mma, D, A, B, C, plain_epilogue(alpha), false, nullptr, 0, st); }, st, warmup, iters, ms_per_launch);
}

int32_t moye_time_copy(const moye_tiled_copy* tc, const moye_tensor* dst, const moye_tensor* src, void* stream,
                       int32_t warmup, int32_t iters, float* ms_per_launch) {
    hipStream_t st = static_cast<hipStream_t>(stream);
    return time_launches([&] { return copy_dispatch(tc, dst, src, st); }, st, warmup, iters, ms_per_launch);
}

int32_t moye_mfma_ceiling(int32_t in_dtype, int32_t random_operands, float seconds, float* tflops, float* clock_ghz,
                          void* stream) {
    return mfma_ceiling(in_dtype, random_operands, seconds, tflops, clock_ghz, static_cast<hipStream_t>(stream));
}

const char* moye_last_error(void) { return last_error().c_str(); }
const char* moye_version(void) { return "moye_hip 0.1.0 (gfx950)"; }

}  // extern "C"

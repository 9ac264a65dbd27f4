/*
 * moye_hip.h — C ABI of libmoye_hip.so: gfx950 (MI355X) kernels behind MoYe.jl's
 * `copyto!` / `gemm!` and the host-side layout algebra that computes their descriptors.
 *
 * The reference (YichengDWu/MoYe.jl v4.0.1) has no FFI boundary of its own: its atoms call
 * NVPTX intrinsics from Julia device code.  Each entry point below names the Julia generic
 * function (reference file:line) whose device work it takes over.  A Julia caller binds
 * these with `ccall`, the Python mirror with `ctypes`; both pass the same plain structs.
 *
 * Conventions
 *   - every function returns a moye_status (0 = ok); moye_last_error() gives the
 *     thread-local message of the last failure on the calling thread;
 *   - pointers inside moye_tensor are BORROWED device pointers, 0-based offsets already
 *     folded in; descriptors are copied at call time;
 *   - shapes/strides are the FLATTENED layout of a MoYeArray (src/array.jl:53-59), strides
 *     in elements, non-negative;
 *   - kernels are enqueued on the caller's stream (NULL = default stream) and the call
 *     returns without waiting.
 */
#ifndef MOYE_HIP_H
#define MOYE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MOYE_MAX_RANK 8

typedef enum {
    MOYE_OK = 0,
    MOYE_ERR_RANK = 1,        /* DimensionMismatch: wrong number of modes                       */
    MOYE_ERR_SHAPE = 2,       /* size mismatch / tile does not divide (shape_div assert)        */
    MOYE_ERR_UNSUPPORTED = 3, /* dtype / atom / operand major this build has no kernel for      */
    MOYE_ERR_ALIGN = 4,       /* pointer or leading dimension not aligned for the vector width  */
    MOYE_ERR_HIP = 5,         /* a HIP runtime call failed                                       */
    MOYE_ERR_ARG = 6,         /* NULL or out-of-range argument                                   */
    MOYE_ERR_PARSE = 7,       /* malformed layout / tuple text                                   */
    MOYE_ERR_BUFFER = 8       /* output text buffer too small                                    */
} moye_status;

typedef enum {
    MOYE_F32 = 0, MOYE_F16 = 1, MOYE_BF16 = 2, MOYE_F8E4M3 = 3, MOYE_F64 = 4,
    MOYE_U8 = 5, MOYE_U16 = 6, MOYE_U32 = 7, MOYE_U64 = 8, MOYE_U128 = 9
} moye_dtype;

/* address-space tag of src/pointer.jl:1-7 (isgmem / issmem / isrmem) */
typedef enum { MOYE_GMEM = 0, MOYE_SMEM = 1, MOYE_RMEM = 2 } moye_memspace;

/* a MoYeArray over a ViewEngine (src/array.jl:53-59, src/engine.jl:6-50), flattened */
typedef struct {
    void*   ptr;
    int32_t dtype;      /* moye_dtype    */
    int32_t memspace;   /* moye_memspace */
    int32_t rank;       /* 1..MOYE_MAX_RANK */
    int32_t _pad;
    int64_t shape[MOYE_MAX_RANK];
    int64_t stride[MOYE_MAX_RANK];
} moye_tensor;

/* MMA atoms: UniversalFMA (src/arch/mma/mma.jl:53-64) plus the gfx950 MFMA instructions that
 * take the place of the reference's MMAOP_* table (src/arch/mma/make_mma_ops.jl:426-438).
 * The 16x16 forms run with every CTA tile moye_gemm offers (64x64, 128x128, 256x256 and the
 * short-M form), the 32x32 forms with the 256x256 tile (whole tiles, 2 x 4 waves) and the 128x128 tile (plain and
 * predicated); with the tile left to the library they take 256x256 tiles where those divide the problem and fill half
 * the chip. */
typedef enum {
    MOYE_MMA_UNIVERSAL_FMA = 0,
    MOYE_MFMA_F32_16x16x32_F16 = 1,
    MOYE_MFMA_F32_32x32x16_F16 = 2,
    MOYE_MFMA_F32_16x16x32_BF16 = 3,
    MOYE_MFMA_F32_32x32x16_BF16 = 4,
    MOYE_MFMA_F32_16x16x32_FP8 = 5,
    MOYE_MFMA_F32_32x32x16_FP8 = 6,
    MOYE_MFMA_F32_16x16x4_F32 = 7,
    MOYE_MFMA_F32_32x32x2_F32 = 8
} moye_mma_atom;

/* a TiledMMA (src/atom/mma.jl:80-92) plus the CTA tile the caller's shared-memory layouts
 * imply (bM,bN,bK of test/device/matmul.jl:11-13) and schedule options */
typedef struct {
    int32_t atom;                  /* moye_mma_atom                                           */
    int32_t atom_layout_mnk[3];    /* shape of TiledMMA.atom_layout_mnk (atom/mma.jl:84)       */
    int32_t tile_mnk[3];           /* tile_size(mma, 1..3) (atom/mma.jl:178-191); for the record: the
                                      kernels are chosen by cta_tile_mnk and atom_layout_mnk     */
    int32_t cta_tile_mnk[3];       /* bM, bN, bK; 0 = let the library choose                    */
    int32_t stages;                /* LDS pipeline depth, 0 = the library's choice (two); 2 = two
                                      stages on the compiler-scheduled kernel; 4, 5 = the rings   */
    int32_t split_k;               /* 0/1 = none; >1 = K cut into that many equal ranges (each a
                                      whole number of 16-byte pieces), all computed by one launch
                                      into fp32 partial products in the library's workspace and
                                      summed in ascending order by a second kernel (results do not
                                      depend on timing); MFMA atoms only.  < 0 = the library
                                      chooses: no split unless the problem's tiles (for M <= 64:
                                      its workgroups of 16 columns) fill less than half the chip
                                      and K is long                                              */
    int32_t flags;                 /* MOYE_GEMM_* bits                                          */
} moye_tiled_mma;

#define MOYE_GEMM_NO_XCD_SWIZZLE 1   /* keep blockIdx -> tile mapping linear (for A/B studies)  */
#define MOYE_GEMM_NO_LDS_SWIZZLE 2   /* in moye_tiled_copy.flags: the LDS-tiled 32-bit transpose keeps
                                        its tile linear (bank-conflict study); the GEMM kernels
                                        ignore it                                               */
#define MOYE_GEMM_NO_WORKSPACE 4      /* fail instead of transposing a non-K-major operand into the workspace */
#define MOYE_GEMM_PREDICATE 0x200     /* compute residue tiles (M, N, K not multiples of the 128x128 CTA tile)
                                        instead of failing as the reference's kernels assert; implied
                                        when cta_tile_mnk is left to the library                        */
#define MOYE_GEMM_PINGPONG 0x100      /* 256x256 tile only: the two waves of a SIMD alternate
                                        between MFMA and memory slots, k-tiles of 64 bytes in a
                                        five-stage LDS ring (cta_tile_mnk[2] = 64 bytes of K)    */
#define MOYE_GEMM_WAVE4 0x400         /* 256x256 tile only: the hand-ordered kernel by name, four
                                        waves (atom layout 2x2: 128x128 wave tiles, one per SIMD) or
                                        eight.  cta_tile_mnk[2] = 128 bytes of K (fp8 always): two
                                        LDS stages of whole 128-byte rows, or with stages >= 3 the
                                        ring of five stages of 64-byte rows; 64 bytes of K: that
                                        ring.  fp8 on the 16x16x128 MFMA.  Plain f16 / bf16 calls on
                                        256x256x(128 bytes) tiles and fp8 calls run this kernel
                                        without the flag; stages = 2 keeps a 16-bit call on the
                                        compiler-scheduled two-stage kernel                       */
#define MOYE_GEMM_NO_PERSIST 0x800    /* one workgroup per CTA tile also where the library would run
                                        one workgroup per CU that walks over the tiles (a problem
                                        with more 256x256 tiles than CUs; for A/B studies)        */

/* copy ops: UniversalCopy (src/arch/copy/copy.jl:26-51); the LDS-staged forms stand where the
 * reference has cp.async (copy_async.jl:8-24) and ldmatrix (ldmatrix.jl:18-48) */
typedef enum {
    MOYE_COPY_UNIVERSAL = 0,       /* element-wise through both layouts                        */
    MOYE_COPY_LDS_TILED = 1        /* 128-bit global loads -> XOR-swizzled LDS tile -> 128-bit  */
} moye_copy_op;

/* a TiledCopy (src/atom/copy.jl:86-90) reduced to what the kernels consume */
typedef struct {
    int32_t op;                    /* moye_copy_op                                             */
    int32_t vec_bits;              /* bits per access of the atom: 8..128 (UniversalCopy{UIntN}) */
    int32_t thr_shape[2];          /* thr_layout of make_tiled_copy (atom/copy.jl:249-258); for the
                                      record: the kernels' lane layouts are their own and no
                                      result depends on thr_shape / val_shape                    */
    int32_t val_shape[2];          /* val_layout                                                */
    int32_t tiler_mn[2];           /* tiler_MN, e.g. 64x64 or the reference's 32x32; 0 = none.  Must
                                      divide modes 1 and 2 of the array (zipped_divide's assertion) */
    int32_t flags;                 /* 0 or MOYE_GEMM_NO_LDS_SWIZZLE                              */
} moye_tiled_copy;

/* ---- device loops ------------------------------------------------------------------------ */

/* Base.copyto!(dest::MoYeArray, src::MoYeArray) (src/algorithm/copy.jl:42-64) and
 * Base.copyto!(tiled_copy, dst, src) (src/algorithm/copy.jl:106-130): logical element i of
 * src goes to logical element i of dst through both layouts; bit-exact when the dtypes
 * agree, round-to-nearest-even conversion otherwise (src/arch/copy/copy.jl:38-43).
 * `tc` may be NULL (plain copyto!). */
int32_t moye_copy(const moye_tiled_copy* tc, const moye_tensor* dst, const moye_tensor* src,
                  void* stream);
/* copyto_if!(dest, src, mask) (src/algorithm/copy.jl:4-16): as copyto!, but logical element i moves
 * only where mask(i) is true.  The reference takes any callable; across this boundary the mask is an
 * array of one byte per logical element (Bool: nonzero = move) with a layout of its own.  Elements
 * of dst whose mask is false keep their value. */
int32_t moye_copy_if(const moye_tensor* dst, const moye_tensor* src, const moye_tensor* mask,
                     void* stream);

/* gemm!(mma, D, A, B, C) (src/algorithm/blas.jl:11-17 and the dispatch tower :20-131) driven
 * over a whole problem the way the reference's user kernels drive it
 * (test/device/matmul.jl:3-53, docs/src/manual/tensor_core.md:265-355):
 * A:(M,K), B:(N,K), C,D:(M,N);  D = alpha * (A * B') + C.   C may be NULL (zero-init
 * accumulator, `zeros!(tCrC)`); D may alias C.  With MOYE_MMA_UNIVERSAL_FMA the arithmetic is
 * the reference's exactly (product rounded in the input type, unfused add, k ascending).
 * The library reads no environment variable: which kernel a call runs on follows from the descriptors alone
 * (moye_gemm_explain prints it).  The MFMA kernels sum k in an order that is fixed per kernel instance and position
 * in the grid, never by timing: a call repeated on the same device gives the same bits; the bits of an element may
 * differ between problem shapes, descriptors or devices that put it on another kernel instance or tile. */
int32_t moye_gemm(const moye_tiled_mma* mma, const moye_tensor* D, const moye_tensor* A,
                  const moye_tensor* B, const moye_tensor* C, float alpha, void* stream);

/* axpby!(a, X, b, Y) (src/algorithm/blas.jl:1-9): y[i] = iszero(b) ? a*x[i] : a*x[i] + b*y[i] over the
 * logical elements of both layouts; X and Y have the same floating-point element type T, a and b are
 * converted to T first, every operation is rounded in T and nothing is fused. */
int32_t moye_axpby(double a, const moye_tensor* X, double b, const moye_tensor* Y, void* stream);

/* fill!(x, value) / zeros!(x) (src/algorithm/array_algorithms.jl:158-182): value converted to x's
 * element type */
int32_t moye_fill(const moye_tensor* X, double value, void* stream);

/* Broadcast-style element-wise maps, dst .= op.(a, b) (src/broadcast.jl:5-41; map!,
 * src/algorithm/array_algorithms.jl:192-210), over the logical elements of the layouts.  All arrays have the
 * same floating-point element type T.  `b` may be NULL (the second operand is `scalar`, converted to T), hold
 * as many elements as dst, or as many as a leading group of dst's modes (it then repeats over the trailing
 * modes, as a lower-rank array does under Julia's broadcasting).  One operation, rounded in T. */
#define MOYE_MAP_IDENTITY 0   /* dst .= a                      */
#define MOYE_MAP_ADD 1        /* a .+ b                        */
#define MOYE_MAP_SUB 2        /* a .- b                        */
#define MOYE_MAP_MUL 3        /* a .* b                        */
#define MOYE_MAP_DIV 4        /* a ./ b                        */
#define MOYE_MAP_MAX 5        /* max.(a, b): NaN if either is  */
#define MOYE_MAP_MIN 6        /* min.(a, b)                    */
#define MOYE_MAP_NEG 7        /* .-a (b and scalar ignored)    */
#define MOYE_MAP_ABS 8        /* abs.(a)                       */
int32_t moye_map(int32_t op, const moye_tensor* dst, const moye_tensor* a, const moye_tensor* b, double scalar,
                 void* stream);

/* bytes of device workspace this gemm! call needs: the K-major copies of MFMA operands whose unit stride
 * is not along K (NN / NT / TT problems, src/arch/mma/make_mma_ops.jl:253-265) and split_k * M * N fp32
 * partial products of a split-K call; 0 for plain TN, for UniversalFMA, for f16 / bf16 operands of any major
 * that run on whole 256x256x64 or 128x128x64 tiles without K ranges, and for fp8 / fp32 operands of any major on whole
 * 256x256 tiles with 128 bytes of K per k-step (named so, or left to the library on problems of at least 128 such
 * tiles) -- all read where they lie.  Assumes the plain epilogue of moye_gemm (see moye_gemm_ex_workspace_size).
 *   moye_gemm     keeps a workspace of its own per (device, stream): allocated by the first call on that stream
 *                 that needs one (a synchronous hipMalloc inside that call, so not under stream capture),
 *                 replaced by a larger one when a larger call comes, never freed inside a call.  Calls on
 *                 different streams do not share a buffer; calls on one stream are ordered by the stream.
 *   moye_gemm_ex  takes the workspace from the caller (256-byte aligned, at least the size reported here;
 *                 NULL when the call needs none) and never allocates, frees or synchronises.            */
int32_t moye_gemm_workspace_size(const moye_tiled_mma* mma, const moye_tensor* D,
                                 const moye_tensor* A, const moye_tensor* B, size_t* bytes);
/* waits for the devices that hold workspaces of moye_gemm and frees them all (no counterpart in the
 * reference, whose kernels own no memory) */
int32_t moye_gemm_release_workspace(void);

/* What the reference's user kernels do to the accumulator fragment between the k-loop and the store
 * (axpby!, src/algorithm/blas.jl:1-9; a broadcast over the fragment, src/broadcast.jl:5-41), as part of the
 * GEMM's epilogue:   D = op(alpha * (A * B') + beta * C, operand)   in fp32, then one round-to-nearest-even
 * conversion to D's type (src/arch/copy/copy.jl:38-43).  Nothing is fused: alpha * acc, beta * c, their sum
 * and op are four separately rounded fp32 operations; with beta == 0 C is not read (axpby!'s iszero(b)). */
typedef struct {
    float   alpha;
    float   beta;
    int32_t op;                 /* MOYE_MAP_*; MOYE_MAP_IDENTITY = none                                */
    int32_t _pad;
    const moye_tensor* operand; /* second argument of op: an (M,N) array of f32 or of D's type with any
                                   strides, 0 = repeated along that mode (a bias vector is (M,N):(1,0) or
                                   (M,N):(0,1)); NULL = `scalar`                                        */
    double  scalar;
} moye_gemm_epilogue;

/* gemm! with the epilogue above and a caller-provided workspace */
int32_t moye_gemm_ex(const moye_tiled_mma* mma, const moye_tensor* D, const moye_tensor* A,
                     const moye_tensor* B, const moye_tensor* C, const moye_gemm_epilogue* ep,
                     void* workspace, size_t workspace_bytes, void* stream);
/* Which launches a gemm! call would make, as text; host arithmetic only: nothing is launched, allocated or asked of
 * a device, the data pointers of the descriptors are compared but never dereferenced (any distinct, suitably aligned
 * addresses will do).  No counterpart in the reference, whose kernels are written by its users; here it is how a
 * caller -- and this library's tests -- see what the dispatcher decided.  `ep` may be NULL (the plain epilogue of
 * moye_gemm).  `compute_units`: plan for a chip of that many CUs (32 to an XCD); 0 = the current device, or 256 CUs in 8
 * XCDs when there is none.  One line per step:
 *   plan: <n> step(s), workspace <bytes> bytes, <cus> CUs in <xcds> XCDs
 *   step <i>: kernel <function<template arguments>> grid=<x>x<y> block=<lanes> lds=<bytes> tile=<m>x<n>x<k bytes>B
 *             in=<dtype> out=<dtype> M= N= K= lda= ldb= ldd= ldd_n= A=<where> B= D= C= a16= b16= d16= split= alpha=
 *             beta= op= flags=<names joined by |>
 *   step <i>: kmajor_copy <where> (<rows> x <cols> <dtype>, strides ..) -> ws+<offset> (pitch <elements>)
 *   step <i>: splitk_reduce split= M= N= partials=ws+<offset> D=<where> out=<dtype> alpha= beta= op=
 * <where> is A+<bytes>, B+.., D+.., C+.. (inside the caller's arrays), ws+<bytes> (inside the workspace) or null;
 * M, N, K, the pitches and the operand roles are the kernel's (a column-major D runs the transposed problem).
 * MOYE_ERR_BUFFER when `cap` bytes do not hold the text. */
int32_t moye_gemm_explain(const moye_tiled_mma* mma, const moye_tensor* D, const moye_tensor* A,
                          const moye_tensor* B, const moye_tensor* C, const moye_gemm_epilogue* ep,
                          int32_t compute_units, char* out, size_t cap);

/* moye_gemm_workspace_size for a call of moye_gemm_ex with this epilogue.  The two differ in one case: fp8 and fp32
 * operands that are not K-major are read where they lie by plain calls only; with an element-wise operation in the
 * epilogue they need their K-major copies.  (No counterpart in the reference: its kernels own no memory.) */
int32_t moye_gemm_ex_workspace_size(const moye_tiled_mma* mma, const moye_tensor* D, const moye_tensor* A,
                                    const moye_tensor* B, const moye_gemm_epilogue* ep, size_t* bytes);

/* gemm! for callers that cannot allocate device memory (code under HIP graph capture, serving loops, harnesses
 * that forbid hipMalloc).  No counterpart in the reference.  Same arguments and results as moye_gemm, bit for bit;
 * the workspace (split-K partial products, K-major copies of operands that are not K-major) is a static device
 * array of MOYE_NOALLOC_SCRATCH_BYTES inside the library, one copy per GPU, held until the process ends.  A call
 * that needs more (moye_gemm_workspace_size) fails with MOYE_ERR_ARG before anything is launched.  Never calls
 * hipMalloc / hipFree or synchronises.  All calls on one GPU share that GPU's array: calls that overlap on one GPU
 * (different streams, or host threads that do not order their launches) race; calls on one stream are safe. */
#define MOYE_NOALLOC_SCRATCH_BYTES (32u << 20)
int32_t moye_gemm_noalloc(const moye_tiled_mma* mma, const moye_tensor* D, const moye_tensor* A,
                          const moye_tensor* B, const moye_tensor* C, float alpha, void* stream);

/* ---- host-side layout algebra (no GPU needed) ------------------------------------------- */
/* Text form of a layout: `shape:stride`, `_n` = static int, `n` = dynamic int, e.g.
 * "(_2, (_1, _6)):(_1, (_6, _2))"; a bare shape means the compact column-major layout
 * (make_layout(shape), src/layout.jl:141-144).  Tiles: a layout, an int, `:` or `<t1, t2, ..>`.
 * Results are written to `out` (capacity `cap` bytes, NUL-terminated). */
int32_t moye_layout_normalize(const char* layout, char* out, size_t cap);                    /* parse + print  */
int32_t moye_layout_eval(const char* layout, const char* coord, int64_t* index);             /* layout.jl:90-102 (1-based) */
/* the same with the result as text, which carries its integer type the way the reference's result does (Int32 stays
 * Int32: test/layout.jl:4-12, src/utilities.jl:1-11): "_7" static, "7" an Int, "7i32" an Int32.  In all text that
 * crosses this boundary a dynamic Int32 is written with the suffix `i32`; a result is static when every integer that
 * went into it is, an Int32 when its dynamic inputs all are, an Int otherwise; Int32 arithmetic wraps modulo 2^32. */
int32_t moye_layout_eval_typed(const char* layout, const char* coord, char* out, size_t cap);
int32_t moye_layout_size(const char* layout, int64_t* size);                                 /* layout.jl:302-304 */
int32_t moye_layout_cosize(const char* layout, int64_t* cosize);                             /* layout.jl:350-352 */
int32_t moye_layout_rank_depth(const char* layout, int32_t* rank, int32_t* depth);           /* layout.jl:321-343 */
int32_t moye_layout_flatten(const char* layout, char* out, size_t cap);                      /* layout.jl:292-294 */
int32_t moye_layout_coalesce(const char* layout, char* out, size_t cap);                     /* layout.jl:497-502 */
int32_t moye_layout_filter(const char* layout, char* out, size_t cap);                       /* layout.jl:515-517 */
int32_t moye_layout_composition(const char* lhs, const char* rhs_tile, char* out, size_t cap); /* layout.jl:593-612 */
int32_t moye_layout_complement(const char* layout, const char* cotarget, char* out, size_t cap); /* layout.jl:660-668; cotarget "" = cosize */
int32_t moye_layout_right_inverse(const char* layout, char* out, size_t cap);                /* layout.jl:717-730 */
int32_t moye_layout_left_inverse(const char* layout, char* out, size_t cap);                 /* layout.jl:738 */
int32_t moye_layout_max_common_vector(const char* a, const char* b, int64_t* n);             /* layout.jl:752-761 */
int32_t moye_layout_logical_product(const char* layout, const char* tile, char* out, size_t cap); /* layout.jl:826-838 */
int32_t moye_layout_zipped_product(const char* layout, const char* tile, char* out, size_t cap);  /* layout.jl:840-842 */
int32_t moye_layout_tiled_product(const char* layout, const char* tile, char* out, size_t cap);   /* layout.jl:844-847 */
int32_t moye_layout_blocked_product(const char* block, const char* layout, int32_t coalesce_result, char* out, size_t cap); /* layout.jl:880-889 */
int32_t moye_layout_raked_product(const char* block, const char* layout, int32_t coalesce_result, char* out, size_t cap);   /* layout.jl:919-928 */
int32_t moye_layout_logical_divide(const char* layout, const char* tile, char* out, size_t cap);  /* layout.jl:1058-1070 */
int32_t moye_layout_zipped_divide(const char* layout, const char* tile, char* out, size_t cap);   /* layout.jl:1114-1116 */
int32_t moye_layout_tiled_divide(const char* layout, const char* tile, char* out, size_t cap);    /* layout.jl:1123-1127 */
int32_t moye_layout_recast(const char* layout, int32_t new_bytes, int32_t old_bytes, char* out, size_t cap); /* layout.jl:999-1010 */
int32_t moye_layout_append(const char* layout, int32_t rank, char* out, size_t cap);         /* layout.jl:377-389 */
int32_t moye_layout_prepend(const char* layout, int32_t rank, char* out, size_t cap);        /* layout.jl:391-397 */
int32_t moye_layout_make_ordered(const char* shape, const char* order, char* out, size_t cap); /* layout.jl:216-218 */
int32_t moye_layout_make_fragment_like(const char* layout, char* out, size_t cap);           /* layout.jl:1143-1149 */
int32_t moye_layout_slice(const char* layout, const char* coord, char* out, size_t cap, int64_t* offset); /* slice_and_offset, layout.jl:368-371 */
int32_t moye_layout_make(const char* shape, int32_t row_major, char* out, size_t cap);
int32_t moye_layout_tile_to_shape(const char* layout, const char* trg_shape, const char* order, char* out, size_t cap); /* layout.jl:930-935; order "" = GenColMajor */
int32_t moye_layout_print(const char* layout, char* out, size_t cap);                       /* print_layout, print.jl:7-44: the index table of a rank-2 layout as text */
int32_t moye_layout_make_like(const char* layout, char* out, size_t cap);                   /* make_layout_like, layout.jl:223-225 */        /* make_layout(shape, GenColMajor|GenRowMajor), layout.jl:154-159 */

/* IntTuple helpers (src/int_tuple.jl, src/stride.jl, src/algorithm/tuple_algorithms.jl) on tuple text such as
 * "(3,(2,2))".  op = flatten | unflatten | product | capacity | product_each | rank | depth | shape_div |
 * elem_scale | filter_zeros | slice | dice | group(a, begin, end) | append(a, val[, n]) | prepend(a, val[, n]) |
 * zip2_by | compact_col_major | compact_row_major | compact_order | coord_to_index | index_to_coord |
 * coord_to_coord | iscompatible | colex_less | elem_less | increment */
int32_t moye_tuple_op(const char* op, const char* a, const char* b, const char* c, char* out, size_t cap);

/* @tile / local_tile (src/algorithm/array_algorithms.jl:113-120) and @parallelize /
 * local_partition (:36-47) on a layout: the sliced layout and the 0-based element offset.
 * `proj` may be "" (none). */
int32_t moye_local_tile(const char* layout, const char* tile, const char* coord, const char* proj,
                        char* out, size_t cap, int64_t* offset);
int32_t moye_local_partition(const char* layout, const char* thr_tile, const char* coord_or_index,
                             const char* proj, char* out, size_t cap, int64_t* offset);

/* TiledMMA (src/atom/mma.jl): `atom` is a moye_mma_atom or the name of one of the reference's
 * NVIDIA atoms kept as data for its tests ("MMAOP_16x8x8_F16F16F16F16_TN", ...).
 * what = "thr_layout_vmnk" | "tile_shape" | "layout_a" | "layout_b" | "layout_c" |
 *        "layoutA_TV" | "layoutB_TV" | "layoutC_TV" | "size" |
 *        "layoutA_MK" | "layoutB_NK" | "layoutC_MN" with "thrID_A" | "thrID_B" | "thrID_C"
 *        (get_layoutA_MK / B_NK / C_MN, atom/mma.jl:235-262: both values of each pair) |
 *        "print": the three tables print_typst(tiled_mma) draws (print.jl:46-93,317-323) as text,
 *        B as (K, N), then A (M, K), then C (M, N); a cell reads T<thread index>V<value index>,
 *        1-based as the reference prints them.  A table of a 256 x 256 tile needs about 1 MB.   */
int32_t moye_tiled_mma_query(const char* atom, const char* atom_layout, const char* permutation,
                             const char* what, char* out, size_t cap);
/* partition_A/B/C of get_slice(mma, thr_idx) (atom/mma.jl:171-175,292-308); operand = 'A'|'B'|'C' */
int32_t moye_tiled_mma_partition(const char* atom, const char* atom_layout, const char* permutation,
                                 int32_t thr_idx, char operand, const char* layout,
                                 char* out, size_t cap, int64_t* offset);
/* make_tiled_copy (atom/copy.jl:249-258): src/dst bits of UniversalCopy{S,D}, value bits of T.
 * what = "layout_tv" | "tiler" | "num_val_src" | "num_val_dst" | "size"                        */
int32_t moye_tiled_copy_query(int32_t src_bits, int32_t dst_bits, int32_t val_bits,
                              const char* thr_layout, const char* val_layout, const char* what,
                              char* out, size_t cap);
/* partition_S / partition_D of get_slice(tiled_copy, thr_idx) (atom/copy.jl:206-214); which = 'S'|'D' */
int32_t moye_tiled_copy_partition(int32_t src_bits, int32_t dst_bits, int32_t val_bits,
                                  const char* thr_layout, const char* val_layout, int32_t thr_idx,
                                  char which, const char* layout, char* out, size_t cap, int64_t* offset);
/* TiledCopy(atom, layout_tv, tiler) (atom/copy.jl:113-125): the form make_tiled_copy_A/B/C build from a
 * TiledMMA (atom/copy.jl:227-240: layout_tv = get_layoutA/B/C_TV(mma), tiler = its tile sizes).
 * what = "layoutS_TV" | "layoutD_TV" (atom/copy.jl:168-187) | "layoutS_MN" | "layoutD_MN"
 * (atom/copy.jl:175-179,188-192; their thread-id layout is size:1) | "num_val_src" | "num_val_dst" |
 * "size" | "print": the source and destination tables print_typst(tiled_copy) draws
 * (print.jl:200-233,337-345) as text, cells T<thread>V<value>.  The TV, MN and print names are
 * accepted by moye_tiled_copy_query too. */
int32_t moye_tiled_copy_tv_query(int32_t src_bits, int32_t dst_bits, int32_t val_bits, const char* layout_tv,
                                 const char* tiler, const char* what, char* out, size_t cap);
int32_t moye_tiled_copy_tv_partition(int32_t src_bits, int32_t dst_bits, int32_t val_bits, const char* layout_tv,
                                     const char* tiler, int32_t thr_idx, char which, const char* layout,
                                     char* out, size_t cap, int64_t* offset);
/* retile_S / retile_D (atom/copy.jl:151-166, 216-225) */
int32_t moye_tiled_copy_tv_retile(int32_t src_bits, int32_t dst_bits, int32_t val_bits, const char* layout_tv,
                                  const char* tiler, const char* layout, char* out, size_t cap);
/* fill a moye_tiled_mma from MoYe-level arguments (checks that the atom layout and the
 * permutation sizes describe a tile this build has a kernel for) */
int32_t moye_make_tiled_mma(int32_t atom, const char* atom_layout, const char* permutation,
                            moye_tiled_mma* out);

/* One execution of a hardware MMA atom by one wave, operands gathered and results scattered through
 * the atom's (thr,val) layouts (the tables behind layout_a/b/c of src/traits/mma.jl:26-31, which
 * partition_A/B/C apply): A is the (M,K) atom tile, B the (N,K) tile, D the (M,N) tile, all dense
 * column-major on the device; D = A * B'.  Allocates a small table buffer and synchronises `stream`:
 * a self-test for the atom tables, not a compute path. */
int32_t moye_mma_atom_probe(int32_t atom, const void* A, const void* B, float* D, void* stream);

/* ---- runtime helpers (thin wrappers so a non-HIP host language needs nothing else) ------- */
int32_t moye_device_malloc(void** ptr, size_t bytes);
int32_t moye_device_free(void* ptr);
int32_t moye_memcpy_h2d(void* dst, const void* src, size_t bytes);
int32_t moye_memcpy_d2h(void* dst, const void* src, size_t bytes);
int32_t moye_memset(void* dst, int value, size_t bytes);
int32_t moye_device_sync(void);
int32_t moye_device_info(char* name, size_t cap, int32_t* compute_units, int32_t* clock_khz,
                         size_t* total_mem);
/* time `iters` back-to-back launches of the same moye_gemm / moye_copy call with HIP events on
 * `stream`; returns the average milliseconds per launch */
int32_t moye_time_gemm(const moye_tiled_mma* mma, const moye_tensor* D, const moye_tensor* A,
                       const moye_tensor* B, const moye_tensor* C, float alpha, void* stream,
                       int32_t warmup, int32_t iters, float* ms_per_launch);
int32_t moye_time_copy(const moye_tiled_copy* tc, const moye_tensor* dst, const moye_tensor* src,
                       void* stream, int32_t warmup, int32_t iters, float* ms_per_launch);

/* The matrix pipe alone: every wave of every CU issues independent MFMAs of the given input type
 * (MOYE_F16 | MOYE_BF16 | MOYE_F8E4M3 | MOYE_F32) on register operands for about `seconds`, no memory
 * traffic.  Reports the rate and the clock the loop ran at (cycle counter over wall time); with
 * random_operands != 0 the operands are dense pseudo-random values, else zeros.  A yardstick for the
 * GEMM kernels' roofline fractions (the part does not hold its nominal clock under dense operands);
 * allocates a few KiB and synchronises. */
int32_t moye_mfma_ceiling(int32_t in_dtype, int32_t random_operands, float seconds, float* tflops,
                          float* clock_ghz, void* stream);

const char* moye_last_error(void);
const char* moye_version(void);

#ifdef __cplusplus
}
#endif
#endif /* MOYE_HIP_H */

# MoYeHIP.jl — `ccall` glue that routes MoYe's device verbs to libmoye_hip.so on AMD gfx950.
#
# This file is the reference-side binding of include/moye_hip.h.  It is written against MoYe.jl
# v4.0.1's own types and adds methods to its generic functions, so user code keeps calling
# `copyto!`, `gemm!`, `make_tiled_mma`, `@tile`, ... unchanged.  It has not been executed in this
# repository's build environment (no Julia runtime there); the ABI it binds is exercised by the
# ctypes mirror under moye_hip/, which declares the same signatures.
#
# Usage:
#   ENV["MOYE_HIP_LIB"] = "/path/to/libmoye_hip.so"
#   using MoYe; include("MoYeHIP.jl"); using .MoYeHIP
#   A = MoYeHIP.device_array(Float16, @Layout((4096,4096), GenRowMajor))  # (M,K), K contiguous
#   mma = MoYeHIP.make_tiled_mma(MoYeHIP.MFMA_F32_16x16x32_F16, @Layout((2,4,1)), (_256,_256,_64))
#   MoYeHIP.gemm!(mma, D, A, B)            # D = A * B'   on the GPU
module MoYeHIP

using MoYe
using MoYe: MoYeArray, Layout, StaticInt, static, shape, stride, flatten, rank

const LIB = get(ENV, "MOYE_HIP_LIB", "libmoye_hip.so")
const CAP = 1 << 16            # text buffer for layouts coming back

# ---- status -----------------------------------------------------------------------------------
struct MoYeHIPError <: Exception
    status::Int32
    msg::String
end
Base.showerror(io::IO, e::MoYeHIPError) = print(io, "MoYeHIP status ", e.status, ": ", e.msg)

last_error() = unsafe_string(ccall((:moye_last_error, LIB), Cstring, ()))
version() = unsafe_string(ccall((:moye_version, LIB), Cstring, ()))

# The library's status codes stand for the reference's exception classes.
function check(st::Int32)
    st == 0 && return nothing
    msg = last_error()
    st == 1 && throw(DimensionMismatch(msg))        # MOYE_ERR_RANK
    st == 2 && throw(DimensionMismatch(msg))        # MOYE_ERR_SHAPE (failed shape_div assert)
    st == 3 && throw(ArgumentError(msg))            # MOYE_ERR_UNSUPPORTED (no method)
    st == 6 && throw(ArgumentError(msg))            # MOYE_ERR_ARG
    throw(MoYeHIPError(st, msg))
end

# ---- descriptors (mirror the C structs field for field) ---------------------------------------
struct Tensor                     # moye_tensor
    ptr::Ptr{Cvoid}
    dtype::Int32
    memspace::Int32
    rank::Int32
    _pad::Int32
    shape::NTuple{8,Int64}
    stride::NTuple{8,Int64}
end

struct TiledMMADesc               # moye_tiled_mma
    atom::Int32
    atom_layout_mnk::NTuple{3,Int32}
    tile_mnk::NTuple{3,Int32}
    cta_tile_mnk::NTuple{3,Int32}
    stages::Int32
    split_k::Int32
    flags::Int32
end

struct TiledCopyDesc              # moye_tiled_copy
    op::Int32
    vec_bits::Int32
    thr_shape::NTuple{2,Int32}
    val_shape::NTuple{2,Int32}
    tiler_mn::NTuple{2,Int32}
    flags::Int32
end

struct GemmEpilogue               # moye_gemm_epilogue
    alpha::Cfloat
    beta::Cfloat
    op::Int32
    _pad::Int32
    operand::Ptr{Tensor}
    scalar::Cdouble
end

# moye_map / epilogue operations
const MAP_IDENTITY = Int32(0)
const MAP_ADD = Int32(1)
const MAP_SUB = Int32(2)
const MAP_MUL = Int32(3)
const MAP_DIV = Int32(4)
const MAP_MAX = Int32(5)
const MAP_MIN = Int32(6)
const MAP_NEG = Int32(7)
const MAP_ABS = Int32(8)

const UNIVERSAL_FMA = Int32(0)
const MFMA_F32_16x16x32_F16 = Int32(1)
const MFMA_F32_32x32x16_F16 = Int32(2)
const MFMA_F32_16x16x32_BF16 = Int32(3)
const MFMA_F32_32x32x16_BF16 = Int32(4)
const MFMA_F32_16x16x32_FP8 = Int32(5)
const MFMA_F32_32x32x16_FP8 = Int32(6)
const MFMA_F32_16x16x4_F32 = Int32(7)
const MFMA_F32_32x32x2_F32 = Int32(8)
# moye_tiled_mma.flags
const GEMM_NO_XCD_SWIZZLE = Int32(1)
const GEMM_NO_LDS_SWIZZLE = Int32(2)
const GEMM_NO_WORKSPACE = Int32(4)      # fail instead of transposing NN/NT/TT operands into the workspace
const GEMM_PINGPONG = Int32(0x100)      # 256x256 tile: ping-pong schedule over a five-stage LDS ring
const GEMM_WAVE4 = Int32(0x400)         # 256x256 tile: four waves with 128x128 wave tiles, fp8 on the 16x16x128 MFMA
const GEMM_PREDICATE = Int32(0x200)     # compute residue tiles instead of asserting divisibility
const GEMM_NO_PERSIST = Int32(0x800)    # one workgroup per CTA tile, never one per CU that walks over the tiles
const COPY_UNIVERSAL = Int32(0)
const COPY_LDS_TILED = Int32(1)

dtype_code(::Type{Float32}) = Int32(0)
dtype_code(::Type{Float16}) = Int32(1)
dtype_code(::Type{Float64}) = Int32(4)
dtype_code(::Type{UInt8}) = Int32(5)
dtype_code(::Type{UInt16}) = Int32(6)
dtype_code(::Type{UInt32}) = Int32(7)
dtype_code(::Type{Int32}) = Int32(7)
dtype_code(::Type{UInt64}) = Int32(8)
dtype_code(::Type{UInt128}) = Int32(9)
dtype_code(::Type{T}) where {T} =
    nameof(T) === :BFloat16 ? Int32(2) : throw(ArgumentError("MoYeHIP: no dtype code for $T"))

pad8(t, fill) = ntuple(i -> i <= length(t) ? Int64(t[i]) : Int64(fill), 8)

"Flatten a device MoYeArray into the descriptor the library consumes (borrowed pointer)."
function Tensor(x::MoYeArray{T}) where {T}
    l = flatten(MoYe.layout(x))
    r = rank(l)
    r <= 8 || throw(DimensionMismatch("MoYeHIP: more than 8 flattened modes"))
    Tensor(Ptr{Cvoid}(UInt(pointer(x))), dtype_code(T), Int32(0), Int32(r), Int32(0),
           pad8(shape(l), 1), pad8(stride(l), 0))
end

# ---- host-side layout algebra through the library -------------------------------------------
# Layouts cross the boundary in MoYe's own printed form (`string(layout)`), with `i32` added to run-time Int32 integers.
# The results are parsed back with MoYe's constructors by `parse_layout` below.

# Text form of an IntTuple for the library: MoYe prints an Int32 like an Int, so the width is added here ("5i32");
# results carry it back, and an index computed from Int32 and static integers only comes back as an Int32
# (test/layout.jl:4-12 of MoYe).
int_text(x::Int32) = string(x, "i32")
int_text(x::Colon) = ":"
int_text(x::Tuple) = length(x) == 1 ? string("(", int_text(x[1]), ",)") : string("(", join((int_text(e) for e in x), ", "), ")")
int_text(x) = string(x)
layout_text(l::Layout) = string(int_text(shape(l)), ":", int_text(stride(l)))

function parse_int_tuple(s::AbstractString)
    s = strip(s)
    if startswith(s, "(")
        depth = 0; parts = String[]; start = 2
        for (i, c) in pairs(s)
            c == '(' && (depth += 1)
            c == ')' && (depth -= 1)
            if (c == ',' && depth == 1) || (c == ')' && depth == 0)
                piece = strip(s[start:prevind(s, i)])
                isempty(piece) || push!(parts, piece)
                start = nextind(s, i)
            end
        end
        return Tuple(parse_int_tuple(p) for p in parts)
    elseif startswith(s, "_")
        return static(parse(Int, s[2:end]))
    elseif endswith(s, "i32")
        return parse(Int32, s[1:end-3])
    else
        return parse(Int, s)
    end
end

function parse_layout(s::AbstractString)
    depth = 0
    for (i, c) in pairs(s)
        c == '(' && (depth += 1)
        c == ')' && (depth -= 1)
        if c == ':' && depth == 0
            return MoYe.make_layout(parse_int_tuple(s[1:prevind(s, i)]), parse_int_tuple(s[nextind(s, i):end]))
        end
    end
    MoYe.make_layout(parse_int_tuple(s))
end

# any argument of the host algebra as text: layouts and IntTuples with their integer widths, text as it is
txt(x::Layout) = layout_text(x)
txt(x::AbstractString) = x
txt(x) = int_text(x)
tile_text(t::Tuple) = "<" * join((txt(x) for x in t), ", ") * ">"
tile_text(x) = txt(x)

macro layout_call(sym, args...)
    quote
        buf = Vector{UInt8}(undef, CAP)
        check(ccall(($(QuoteNode(sym)), LIB), Int32, ($(map(_ -> :Cstring, args)...), Ptr{UInt8}, Csize_t),
                    $(map(esc, args)...), buf, CAP))
        parse_layout(unsafe_string(pointer(buf)))
    end
end

coalesce(l::Layout) = @layout_call moye_layout_coalesce txt(l)
filter(l::Layout) = @layout_call moye_layout_filter txt(l)
flatten_layout(l::Layout) = @layout_call moye_layout_flatten txt(l)
composition(a::Layout, b) = @layout_call moye_layout_composition txt(a) tile_text(b)
complement(l::Layout, cotarget = "") = @layout_call moye_layout_complement txt(l) txt(cotarget)
right_inverse(l::Layout) = @layout_call moye_layout_right_inverse txt(l)
left_inverse(l::Layout) = @layout_call moye_layout_left_inverse txt(l)
logical_product(l::Layout, t) = @layout_call moye_layout_logical_product txt(l) tile_text(t)
zipped_product(l::Layout, t) = @layout_call moye_layout_zipped_product txt(l) tile_text(t)
tiled_product(l::Layout, t) = @layout_call moye_layout_tiled_product txt(l) tile_text(t)
logical_divide(l::Layout, t) = @layout_call moye_layout_logical_divide txt(l) tile_text(t)
zipped_divide(l::Layout, t) = @layout_call moye_layout_zipped_divide txt(l) tile_text(t)
tiled_divide(l::Layout, t) = @layout_call moye_layout_tiled_divide txt(l) tile_text(t)
make_fragment_like(l::Layout) = @layout_call moye_layout_make_fragment_like txt(l)
normalize(l::Layout) = @layout_call moye_layout_normalize txt(l)

function blocked_product(block::Layout, l::Layout, coalesce_result::Bool = false)
    buf = Vector{UInt8}(undef, CAP)
    check(ccall((:moye_layout_blocked_product, LIB), Int32, (Cstring, Cstring, Int32, Ptr{UInt8}, Csize_t),
                txt(block), txt(l), Int32(coalesce_result), buf, CAP))
    parse_layout(unsafe_string(pointer(buf)))
end

function raked_product(block::Layout, l::Layout, coalesce_result::Bool = false)
    buf = Vector{UInt8}(undef, CAP)
    check(ccall((:moye_layout_raked_product, LIB), Int32, (Cstring, Cstring, Int32, Ptr{UInt8}, Csize_t),
                txt(block), txt(l), Int32(coalesce_result), buf, CAP))
    parse_layout(unsafe_string(pointer(buf)))
end

function recast(l::Layout, ::Type{New}, ::Type{Old}) where {New,Old}
    buf = Vector{UInt8}(undef, CAP)
    check(ccall((:moye_layout_recast, LIB), Int32, (Cstring, Int32, Int32, Ptr{UInt8}, Csize_t),
                txt(l), Int32(sizeof(New)), Int32(sizeof(Old)), buf, CAP))
    parse_layout(unsafe_string(pointer(buf)))
end

# `layout(coord)`.  The result has the type MoYe's own arithmetic would give it: a StaticInt when layout and coordinate
# are static, an Int32 when their run-time integers all are (`@Layout((2,(2,2)),(2,(1,4)))(Int32(2)) isa Int32`,
# test/layout.jl:4-12), an Int otherwise.
function layout_index(l::Layout, coord)
    buf = Vector{UInt8}(undef, 64)
    check(ccall((:moye_layout_eval_typed, LIB), Int32, (Cstring, Cstring, Ptr{UInt8}, Csize_t),
                layout_text(l), int_text(coord), buf, 64))
    parse_int_tuple(unsafe_string(pointer(buf)))
end

function layout_size(l::Layout)
    n = Ref{Int64}(0)
    check(ccall((:moye_layout_size, LIB), Int32, (Cstring, Ptr{Int64}), txt(l), n)); n[]
end

function layout_cosize(l::Layout)
    n = Ref{Int64}(0)
    check(ccall((:moye_layout_cosize, LIB), Int32, (Cstring, Ptr{Int64}), txt(l), n)); n[]
end

function max_common_vector(a::Layout, b::Layout)
    n = Ref{Int64}(0)
    check(ccall((:moye_layout_max_common_vector, LIB), Int32, (Cstring, Cstring, Ptr{Int64}), txt(a), txt(b), n))
    n[]
end

function tuple_op(op::AbstractString, a, b = "", c = "")
    buf = Vector{UInt8}(undef, CAP)
    check(ccall((:moye_tuple_op, LIB), Int32, (Cstring, Cstring, Cstring, Cstring, Ptr{UInt8}, Csize_t),
                op, txt(a), txt(b), txt(c), buf, CAP))
    unsafe_string(pointer(buf))
end

"`@tile x tile coord` on a device array: the sub-array's layout and pointer, computed by the library."
function local_tile(x::MoYeArray{T}, tile::Tuple, coord::Tuple, proj = "") where {T}
    buf = Vector{UInt8}(undef, CAP); off = Ref{Int64}(0)
    check(ccall((:moye_local_tile, LIB), Int32, (Cstring, Cstring, Cstring, Cstring, Ptr{UInt8}, Csize_t, Ptr{Int64}),
                txt(MoYe.layout(x)), tile_text(tile), tile_text(coord), txt(proj), buf, CAP, off))
    MoYeArray(pointer(x) + off[] * sizeof(T), parse_layout(unsafe_string(pointer(buf))))
end

"`@parallelize x thr_layout thr_idx` on a device array."
function local_partition(x::MoYeArray{T}, thr::Layout, idx::Integer, proj = "") where {T}
    buf = Vector{UInt8}(undef, CAP); off = Ref{Int64}(0)
    check(ccall((:moye_local_partition, LIB), Int32,
                (Cstring, Cstring, Cstring, Cstring, Ptr{UInt8}, Csize_t, Ptr{Int64}),
                txt(MoYe.layout(x)), txt(thr), txt(idx), txt(proj), buf, CAP, off))
    MoYeArray(pointer(x) + off[] * sizeof(T), parse_layout(unsafe_string(pointer(buf))))
end

# ---- TiledMMA / TiledCopy ---------------------------------------------------------------------
"make_tiled_mma(op, atom_layout, permutation) for the gfx950 atoms; returns the POD descriptor."
function make_tiled_mma(atom::Int32, atom_layout::Layout, permutation::Tuple = ())
    d = Ref{TiledMMADesc}()
    check(ccall((:moye_make_tiled_mma, LIB), Int32, (Int32, Cstring, Cstring, Ptr{TiledMMADesc}),
                atom, txt(atom_layout), isempty(permutation) ? "" : tile_text(permutation), d))
    d[]
end

function tiled_mma_query(atom::AbstractString, atom_layout::Layout, permutation, what::AbstractString; cap = CAP)
    buf = Vector{UInt8}(undef, cap)
    check(ccall((:moye_tiled_mma_query, LIB), Int32, (Cstring, Cstring, Cstring, Cstring, Ptr{UInt8}, Csize_t),
                atom, txt(atom_layout), permutation === nothing ? "" : tile_text(permutation), what, buf, cap))
    unsafe_string(pointer(buf))
end

"The tables print_typst(tiled_mma) draws (src/print.jl:46-93,317-323) as text: B as (K, N), then A, then C."
print_tv(atom::AbstractString, atom_layout::Layout, permutation = nothing) =
    println(tiled_mma_query(atom, atom_layout, permutation, "print"; cap = 1 << 23))

"partition_A/B/C(get_slice(mma, thr_idx), x) computed by the library (operand = 'A', 'B' or 'C')."
function tiled_mma_partition(atom::AbstractString, atom_layout::Layout, permutation, thr_idx::Integer,
                             operand::Char, x::MoYeArray{T}) where {T}
    buf = Vector{UInt8}(undef, CAP); off = Ref{Int64}(0)
    check(ccall((:moye_tiled_mma_partition, LIB), Int32,
                (Cstring, Cstring, Cstring, Int32, Cchar, Cstring, Ptr{UInt8}, Csize_t, Ptr{Int64}),
                atom, txt(atom_layout), permutation === nothing ? "" : tile_text(permutation), Int32(thr_idx),
                Cchar(operand), txt(MoYe.layout(x)), buf, CAP, off))
    MoYeArray(pointer(x) + off[] * sizeof(T), parse_layout(unsafe_string(pointer(buf))))
end

function tiled_copy_query(src_bits, dst_bits, val_bits, thr::Layout, val::Layout, what::AbstractString; cap = CAP)
    buf = Vector{UInt8}(undef, cap)
    check(ccall((:moye_tiled_copy_query, LIB), Int32,
                (Int32, Int32, Int32, Cstring, Cstring, Cstring, Ptr{UInt8}, Csize_t),
                Int32(src_bits), Int32(dst_bits), Int32(val_bits), txt(thr), txt(val), what, buf, cap))
    unsafe_string(pointer(buf))
end

"The source and destination tables print_typst(tiled_copy) draws (src/print.jl:200-233,337-345) as text."
print_tv(src_bits::Integer, dst_bits::Integer, val_bits::Integer, thr::Layout, val::Layout) =
    println(tiled_copy_query(src_bits, dst_bits, val_bits, thr, val, "print"; cap = 1 << 23))

function tiled_copy_partition(src_bits, dst_bits, val_bits, thr::Layout, val::Layout, thr_idx::Integer,
                              which::Char, x::MoYeArray{T}) where {T}
    buf = Vector{UInt8}(undef, CAP); off = Ref{Int64}(0)
    check(ccall((:moye_tiled_copy_partition, LIB), Int32,
                (Int32, Int32, Int32, Cstring, Cstring, Int32, Cchar, Cstring, Ptr{UInt8}, Csize_t, Ptr{Int64}),
                Int32(src_bits), Int32(dst_bits), Int32(val_bits), txt(thr), txt(val), Int32(thr_idx),
                Cchar(which), txt(MoYe.layout(x)), buf, CAP, off))
    MoYeArray(pointer(x) + off[] * sizeof(T), parse_layout(unsafe_string(pointer(buf))))
end

# TiledCopy(atom, layout_tv, tiler): what make_tiled_copy_A/B/C build from a TiledMMA (src/atom/copy.jl:227-240)
function tiled_copy_tv_query(src_bits, dst_bits, val_bits, layout_tv::Layout, tiler::Tuple, what::AbstractString)
    buf = Vector{UInt8}(undef, CAP)
    check(ccall((:moye_tiled_copy_tv_query, LIB), Int32,
                (Int32, Int32, Int32, Cstring, Cstring, Cstring, Ptr{UInt8}, Csize_t),
                Int32(src_bits), Int32(dst_bits), Int32(val_bits), txt(layout_tv), txt(tiler), what, buf, CAP))
    unsafe_string(pointer(buf))
end

function tiled_copy_tv_partition(src_bits, dst_bits, val_bits, layout_tv::Layout, tiler::Tuple, thr_idx::Integer,
                                 which::Char, x::MoYeArray{T}) where {T}
    buf = Vector{UInt8}(undef, CAP); off = Ref{Int64}(0)
    check(ccall((:moye_tiled_copy_tv_partition, LIB), Int32,
                (Int32, Int32, Int32, Cstring, Cstring, Int32, Cchar, Cstring, Ptr{UInt8}, Csize_t, Ptr{Int64}),
                Int32(src_bits), Int32(dst_bits), Int32(val_bits), txt(layout_tv), txt(tiler), Int32(thr_idx),
                Cchar(which), txt(MoYe.layout(x)), buf, CAP, off))
    MoYeArray(pointer(x) + off[] * sizeof(T), parse_layout(unsafe_string(pointer(buf))))
end

"retile_S / retile_D (src/atom/copy.jl:151-166) of a fragment layout"
function tiled_copy_tv_retile(src_bits, dst_bits, val_bits, layout_tv::Layout, tiler::Tuple, l::Layout)
    buf = Vector{UInt8}(undef, CAP)
    check(ccall((:moye_tiled_copy_tv_retile, LIB), Int32,
                (Int32, Int32, Int32, Cstring, Cstring, Cstring, Ptr{UInt8}, Csize_t),
                Int32(src_bits), Int32(dst_bits), Int32(val_bits), txt(layout_tv), txt(tiler), txt(l), buf, CAP))
    parse_layout(unsafe_string(pointer(buf)))
end

function tile_to_shape(l::Layout, trg_shape::Tuple, order = "")
    buf = Vector{UInt8}(undef, CAP)
    check(ccall((:moye_layout_tile_to_shape, LIB), Int32, (Cstring, Cstring, Cstring, Ptr{UInt8}, Csize_t),
                txt(l), txt(trg_shape), txt(order), buf, CAP))
    parse_layout(unsafe_string(pointer(buf)))
end

make_layout_like(l::Layout) = @layout_call moye_layout_make_like txt(l)

"One wave executes the atom once through its (thr,val) tables: D(M,N) = A(M,K) * B(N,K)' on dense column-major device tiles."
mma_atom_probe(atom::Int32, A::Ptr{Cvoid}, B::Ptr{Cvoid}, D::Ptr{Cvoid}; stream = C_NULL) =
    check(ccall((:moye_mma_atom_probe, LIB), Int32, (Int32, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}), atom, A, B, D, stream))

"A TiledCopy for the device copy: atom of `vec_bits` bits, thread and value layouts, LDS tile."
function tiled_copy_desc(; op = COPY_UNIVERSAL, vec_bits = 128, thr = (16, 16), val = (4, 4), tiler = (64, 64))
    TiledCopyDesc(op, Int32(vec_bits), Int32.(thr), Int32.(val), Int32.(tiler), Int32(0))
end

# ---- the device verbs -------------------------------------------------------------------------
"""
    copyto!(dst, src; tiled_copy=nothing, stream=C_NULL)

`Base.copyto!(dest::MoYeArray, src::MoYeArray)` (src/algorithm/copy.jl:42-64) and
`copyto!(tiled_copy, dst, src)` (:106-130) for device arrays.  Asynchronous on `stream`.
"""
function copyto!(dst::MoYeArray, src::MoYeArray; tiled_copy::Union{Nothing,TiledCopyDesc} = nothing,
                 stream::Ptr{Cvoid} = C_NULL)
    d, s = Ref(Tensor(dst)), Ref(Tensor(src))
    GC.@preserve dst src begin
        if tiled_copy === nothing
            check(ccall((:moye_copy, LIB), Int32, (Ptr{Cvoid}, Ptr{Tensor}, Ptr{Tensor}, Ptr{Cvoid}), C_NULL, d, s, stream))
        else
            tc = Ref(tiled_copy)
            check(ccall((:moye_copy, LIB), Int32, (Ptr{TiledCopyDesc}, Ptr{Tensor}, Ptr{Tensor}, Ptr{Cvoid}), tc, d, s, stream))
        end
    end
    dst
end

"copyto_if!(dst, src, mask) (src/algorithm/copy.jl:4-16); `mask` is a MoYeArray{Bool} (one byte per logical element)."
function copyto_if!(dst::MoYeArray, src::MoYeArray, mask::MoYeArray{Bool}; stream::Ptr{Cvoid} = C_NULL)
    m = Tensor(recast(UInt8, mask))
    GC.@preserve dst src mask check(ccall((:moye_copy_if, LIB), Int32, (Ptr{Tensor}, Ptr{Tensor}, Ptr{Tensor}, Ptr{Cvoid}),
                                          Ref(Tensor(dst)), Ref(Tensor(src)), Ref(m), stream))
    dst
end

"""
    gemm!(mma, D, A, B[, C]; alpha=1f0, stream=C_NULL)

`gemm!(mma, D, A, B, C)` (src/algorithm/blas.jl:11-17) over whole device operands:
A:(M,K), B:(N,K), C,D:(M,N); D = alpha * A * B' + C.  Returns `nothing` like the reference.
"""
function gemm!(mma::TiledMMADesc, D::MoYeArray, A::MoYeArray, B::MoYeArray, C::Union{Nothing,MoYeArray} = nothing;
               alpha::Real = 1.0f0, stream::Ptr{Cvoid} = C_NULL)
    m, d, a, b = Ref(mma), Ref(Tensor(D)), Ref(Tensor(A)), Ref(Tensor(B))
    GC.@preserve D A B C begin
        if C === nothing
            check(ccall((:moye_gemm, LIB), Int32,
                        (Ptr{TiledMMADesc}, Ptr{Tensor}, Ptr{Tensor}, Ptr{Tensor}, Ptr{Cvoid}, Cfloat, Ptr{Cvoid}),
                        m, d, a, b, C_NULL, Float32(alpha), stream))
        else
            c = Ref(Tensor(C))
            check(ccall((:moye_gemm, LIB), Int32,
                        (Ptr{TiledMMADesc}, Ptr{Tensor}, Ptr{Tensor}, Ptr{Tensor}, Ptr{Tensor}, Cfloat, Ptr{Cvoid}),
                        m, d, a, b, c, Float32(alpha), stream))
        end
    end
    nothing
end

"""
    gemm_ex!(mma, D, A, B[, C]; alpha, beta, op, operand, scalar, workspace, workspace_bytes, stream)

gemm! with the epilogue a MoYe kernel applies to its accumulator fragment fused in: `axpby!` (src/algorithm/blas.jl:1-9)
and one broadcast operation (src/broadcast.jl:5-41), D = op.(alpha * A * B' + beta * C, operand).  `operand` is an
(M,N) MoYeArray (a stride of 0 repeats a bias vector along that mode) or `nothing` (then `scalar`).  The workspace, when
the call needs one (`gemm_workspace_size`), comes from the caller; this entry point never allocates.
"""
function gemm_ex!(mma::TiledMMADesc, D::MoYeArray, A::MoYeArray, B::MoYeArray, C::Union{Nothing,MoYeArray} = nothing;
                  alpha::Real = 1.0f0, beta::Real = C === nothing ? 0.0f0 : 1.0f0, op::Int32 = MAP_IDENTITY,
                  operand::Union{Nothing,MoYeArray} = nothing, scalar::Real = 0.0,
                  workspace::Ptr{Cvoid} = C_NULL, workspace_bytes::Integer = 0, stream::Ptr{Cvoid} = C_NULL)
    m, d, a, b = Ref(mma), Ref(Tensor(D)), Ref(Tensor(A)), Ref(Tensor(B))
    x = operand === nothing ? nothing : Ref(Tensor(operand))
    c = C === nothing ? nothing : Ref(Tensor(C))
    GC.@preserve D A B C operand x c begin
        xp = x === nothing ? Ptr{Tensor}(C_NULL) : Base.unsafe_convert(Ptr{Tensor}, x)
        cp = c === nothing ? Ptr{Tensor}(C_NULL) : Base.unsafe_convert(Ptr{Tensor}, c)
        ep = Ref(GemmEpilogue(Float32(alpha), Float32(beta), op, Int32(0), xp, Float64(scalar)))
        check(ccall((:moye_gemm_ex, LIB), Int32,
                    (Ptr{TiledMMADesc}, Ptr{Tensor}, Ptr{Tensor}, Ptr{Tensor}, Ptr{Tensor}, Ptr{GemmEpilogue}, Ptr{Cvoid}, Csize_t, Ptr{Cvoid}),
                    m, d, a, b, cp, ep, workspace, workspace_bytes, stream))
    end
    nothing
end

"""
    gemm_noalloc!(mma, D, A, B[, C]; alpha=1f0, stream=C_NULL)

gemm! for callers that cannot allocate device memory (under graph capture): the workspace is a static 32 MiB array
inside the library; a call that needs more throws an ArgumentError.
"""
function gemm_noalloc!(mma::TiledMMADesc, D::MoYeArray, A::MoYeArray, B::MoYeArray, C::Union{Nothing,MoYeArray} = nothing;
                       alpha::Real = 1.0f0, stream::Ptr{Cvoid} = C_NULL)
    m, d, a, b = Ref(mma), Ref(Tensor(D)), Ref(Tensor(A)), Ref(Tensor(B))
    c = C === nothing ? nothing : Ref(Tensor(C))
    GC.@preserve D A B C c begin
        cp = c === nothing ? Ptr{Tensor}(C_NULL) : Base.unsafe_convert(Ptr{Tensor}, c)
        check(ccall((:moye_gemm_noalloc, LIB), Int32,
                    (Ptr{TiledMMADesc}, Ptr{Tensor}, Ptr{Tensor}, Ptr{Tensor}, Ptr{Tensor}, Cfloat, Ptr{Cvoid}),
                    m, d, a, b, cp, Float32(alpha), stream))
    end
    nothing
end

"Frees the per-stream workspaces `gemm!` keeps for NN / NT / TT operands and split-K (waits for the device first)."
gemm_release_workspace() = check(ccall((:moye_gemm_release_workspace, LIB), Int32, ()))

"""
    axpby!(a, X, b, Y; stream=C_NULL)

`axpby!(a, X, b, Y)` (src/algorithm/blas.jl:1-9) for device arrays of one floating-point element type.
"""
function axpby!(a::Real, X::MoYeArray, b::Real, Y::MoYeArray; stream::Ptr{Cvoid} = C_NULL)
    GC.@preserve X Y check(ccall((:moye_axpby, LIB), Int32, (Cdouble, Ptr{Tensor}, Cdouble, Ptr{Tensor}, Ptr{Cvoid}),
                                 Float64(a), Ref(Tensor(X)), Float64(b), Ref(Tensor(Y)), stream))
    nothing
end

"`fill!(x, val)` / `zeros!(x)` (src/algorithm/array_algorithms.jl:158-182) for device arrays."
function fill!(x::MoYeArray, val::Real; stream::Ptr{Cvoid} = C_NULL)
    GC.@preserve x check(ccall((:moye_fill, LIB), Int32, (Ptr{Tensor}, Cdouble, Ptr{Cvoid}), Ref(Tensor(x)), Float64(val), stream))
    x
end
zeros!(x::MoYeArray; stream::Ptr{Cvoid} = C_NULL) = fill!(x, 0.0; stream = stream)

const MAP_OPS = Dict{Any,Int32}(identity => 0, (+) => 1, (-) => 2, (*) => 3, (/) => 4, max => 5, min => 6, abs => 8)

"""
    map!(f, dst, a, b; stream=C_NULL)     # dst .= f.(a, b), b an array or a number
    map!(f, dst, a; stream=C_NULL)        # dst .= f.(a) for identity, -, abs

The device form of the reference's broadcast (src/broadcast.jl:5-41) and `map!`
(src/algorithm/array_algorithms.jl:192-210) for `f` in `+ - * / max min abs identity`: one operation per
element, rounded in the arrays' element type.  A lower-rank `b` repeats over the trailing modes of `dst`.
"""
function map!(f, dst::MoYeArray, a::MoYeArray, b::MoYeArray; stream::Ptr{Cvoid} = C_NULL)
    GC.@preserve dst a b check(ccall((:moye_map, LIB), Int32, (Int32, Ptr{Tensor}, Ptr{Tensor}, Ptr{Tensor}, Cdouble, Ptr{Cvoid}),
                                     MAP_OPS[f], Ref(Tensor(dst)), Ref(Tensor(a)), Ref(Tensor(b)), 0.0, stream))
    dst
end
function map!(f, dst::MoYeArray, a::MoYeArray, b::Real; stream::Ptr{Cvoid} = C_NULL)
    GC.@preserve dst a check(ccall((:moye_map, LIB), Int32, (Int32, Ptr{Tensor}, Ptr{Tensor}, Ptr{Tensor}, Cdouble, Ptr{Cvoid}),
                                   MAP_OPS[f], Ref(Tensor(dst)), Ref(Tensor(a)), C_NULL, Float64(b), stream))
    dst
end
function map!(f, dst::MoYeArray, a::MoYeArray; stream::Ptr{Cvoid} = C_NULL)
    op = f === (-) ? Int32(7) : MAP_OPS[f]
    GC.@preserve dst a check(ccall((:moye_map, LIB), Int32, (Int32, Ptr{Tensor}, Ptr{Tensor}, Ptr{Tensor}, Cdouble, Ptr{Cvoid}),
                                   op, Ref(Tensor(dst)), Ref(Tensor(a)), C_NULL, 0.0, stream))
    dst
end

function gemm_workspace_size(mma::TiledMMADesc, D::MoYeArray, A::MoYeArray, B::MoYeArray)
    n = Ref{Csize_t}(0)
    check(ccall((:moye_gemm_workspace_size, LIB), Int32,
                (Ptr{TiledMMADesc}, Ptr{Tensor}, Ptr{Tensor}, Ptr{Tensor}, Ptr{Csize_t}),
                Ref(mma), Ref(Tensor(D)), Ref(Tensor(A)), Ref(Tensor(B)), n))
    Int(n[])
end

# the same for a gemm_ex! call whose epilogue applies `op` (fp8 / fp32 operands that are not K-major are read where they
# lie by plain calls only)
function gemm_ex_workspace_size(mma::TiledMMADesc, D::MoYeArray, A::MoYeArray, B::MoYeArray; op::Int32 = MAP_IDENTITY)
    n = Ref{Csize_t}(0)
    ep = Ref(GemmEpilogue(1.0f0, 0.0f0, op, Int32(0), Ptr{Tensor}(C_NULL), 0.0))
    check(ccall((:moye_gemm_ex_workspace_size, LIB), Int32,
                (Ptr{TiledMMADesc}, Ptr{Tensor}, Ptr{Tensor}, Ptr{Tensor}, Ptr{GemmEpilogue}, Ptr{Csize_t}),
                Ref(mma), Ref(Tensor(D)), Ref(Tensor(A)), Ref(Tensor(B)), ep, n))
    Int(n[])
end

"""
    gemm_explain(mma, D, A, B[, C]; op, compute_units) -> String

The launches `gemm!` / `gemm_ex!` would make for these descriptors (kernel instance, grid, tile, sub-problem, K ranges,
flags; one line per launch).  Host arithmetic only: nothing is launched and the arrays' memory is not touched.
"""
function gemm_explain(mma::TiledMMADesc, D::MoYeArray, A::MoYeArray, B::MoYeArray, C::Union{Nothing,MoYeArray} = nothing;
                      op::Int32 = MAP_IDENTITY, compute_units::Integer = 0)
    buf = Vector{UInt8}(undef, 1 << 16)
    c = C === nothing ? nothing : Ref(Tensor(C))
    GC.@preserve D A B C c buf begin
        cp = c === nothing ? Ptr{Tensor}(C_NULL) : Base.unsafe_convert(Ptr{Tensor}, c)
        ep = Ref(GemmEpilogue(1.0f0, C === nothing ? 0.0f0 : 1.0f0, op, Int32(0), Ptr{Tensor}(C_NULL), 0.0))
        check(ccall((:moye_gemm_explain, LIB), Int32,
                    (Ptr{TiledMMADesc}, Ptr{Tensor}, Ptr{Tensor}, Ptr{Tensor}, Ptr{Tensor}, Ptr{GemmEpilogue}, Int32, Ptr{UInt8}, Csize_t),
                    Ref(mma), Ref(Tensor(D)), Ref(Tensor(A)), Ref(Tensor(B)), cp, ep, Int32(compute_units), buf, length(buf)))
    end
    unsafe_string(pointer(buf))
end

# ---- device memory without a Julia GPU package ------------------------------------------------
function device_malloc(bytes::Integer)
    p = Ref{Ptr{Cvoid}}(C_NULL)
    check(ccall((:moye_device_malloc, LIB), Int32, (Ptr{Ptr{Cvoid}}, Csize_t), p, bytes)); p[]
end
device_free(p::Ptr{Cvoid}) = check(ccall((:moye_device_free, LIB), Int32, (Ptr{Cvoid},), p))
device_sync() = check(ccall((:moye_device_sync, LIB), Int32, ()))
memset(p::Ptr{Cvoid}, v::Integer, bytes::Integer) =
    check(ccall((:moye_memset, LIB), Int32, (Ptr{Cvoid}, Cint, Csize_t), p, v, bytes))

"A device MoYeArray of element type T with the given layout (caller frees with `device_free(pointer(x))`)."
function device_array(::Type{T}, l::Layout) where {T}
    p = device_malloc(layout_cosize(l) * sizeof(T))
    MoYeArray(Ptr{T}(p), l)
end

function upload!(dst::MoYeArray{T}, host::Array{T}) where {T}
    GC.@preserve host check(ccall((:moye_memcpy_h2d, LIB), Int32, (Ptr{Cvoid}, Ptr{Cvoid}, Csize_t),
                                  Ptr{Cvoid}(UInt(pointer(dst))), pointer(host), sizeof(host)))
    dst
end

function download!(host::Array{T}, src::MoYeArray{T}) where {T}
    GC.@preserve host check(ccall((:moye_memcpy_d2h, LIB), Int32, (Ptr{Cvoid}, Ptr{Cvoid}, Csize_t),
                                  pointer(host), Ptr{Cvoid}(UInt(pointer(src))), sizeof(host)))
    host
end

function device_info()
    name = Vector{UInt8}(undef, 256); cu = Ref{Int32}(0); khz = Ref{Int32}(0); mem = Ref{Csize_t}(0)
    check(ccall((:moye_device_info, LIB), Int32, (Ptr{UInt8}, Csize_t, Ptr{Int32}, Ptr{Int32}, Ptr{Csize_t}),
                name, 256, cu, khz, mem))
    (name = unsafe_string(pointer(name)), compute_units = cu[], clock_khz = khz[], total_mem = Int(mem[]))
end

"(TFLOP/s, GHz) of an MFMA-only loop on every CU: what the matrix pipe sustains on this part for this input type."
function mfma_ceiling(in_dtype::Int32; random_operands::Bool = true, seconds::Real = 0.3, stream = C_NULL)
    tf = Ref{Cfloat}(0); ghz = Ref{Cfloat}(0)
    check(ccall((:moye_mfma_ceiling, LIB), Int32, (Int32, Int32, Cfloat, Ptr{Cfloat}, Ptr{Cfloat}, Ptr{Cvoid}),
                in_dtype, Int32(random_operands), Float32(seconds), tf, ghz, stream))
    (tflops = tf[], clock_ghz = ghz[])
end

function print_layout(l::Layout)
    buf = Vector{UInt8}(undef, 1 << 20)
    check(ccall((:moye_layout_print, LIB), Int32, (Cstring, Ptr{UInt8}, Csize_t), txt(l), buf, 1 << 20))
    println(unsafe_string(pointer(buf)))
end

"Average milliseconds per launch of the same gemm! call, HIP events on `stream`."
function time_gemm(mma::TiledMMADesc, D, A, B; alpha = 1.0f0, stream = C_NULL, warmup = 3, iters = 20)
    ms = Ref{Cfloat}(0)
    check(ccall((:moye_time_gemm, LIB), Int32,
                (Ptr{TiledMMADesc}, Ptr{Tensor}, Ptr{Tensor}, Ptr{Tensor}, Ptr{Cvoid}, Cfloat, Ptr{Cvoid}, Int32, Int32, Ptr{Cfloat}),
                Ref(mma), Ref(Tensor(D)), Ref(Tensor(A)), Ref(Tensor(B)), C_NULL, Float32(alpha), stream,
                Int32(warmup), Int32(iters), ms))
    ms[]
end

function time_copy(dst, src; tiled_copy = tiled_copy_desc(), stream = C_NULL, warmup = 3, iters = 20)
    ms = Ref{Cfloat}(0)
    check(ccall((:moye_time_copy, LIB), Int32,
                (Ptr{TiledCopyDesc}, Ptr{Tensor}, Ptr{Tensor}, Ptr{Cvoid}, Int32, Int32, Ptr{Cfloat}),
                Ref(tiled_copy), Ref(Tensor(dst)), Ref(Tensor(src)), stream, Int32(warmup), Int32(iters), ms))
    ms[]
end

end # module

"""ctypes binding of libmoye_hip.so (the C ABI declared in include/moye_hip.h).

The library is built in-tree by `moye.jl_amd/build.py`; nothing here falls back to another
implementation: a missing library raises at import of the first symbol.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmoye_hip.so")

MAX_RANK = 8

# moye_status
OK, ERR_RANK, ERR_SHAPE, ERR_UNSUPPORTED, ERR_ALIGN, ERR_HIP, ERR_ARG, ERR_PARSE, ERR_BUFFER = range(9)
STATUS_NAMES = ["OK", "ERR_RANK", "ERR_SHAPE", "ERR_UNSUPPORTED", "ERR_ALIGN", "ERR_HIP", "ERR_ARG",
                "ERR_PARSE", "ERR_BUFFER"]
# moye_dtype
F32, F16, BF16, F8E4M3, F64, U8, U16, U32, U64, U128 = range(10)
DTYPE_BYTES = {F32: 4, F16: 2, BF16: 2, F8E4M3: 1, F64: 8, U8: 1, U16: 2, U32: 4, U64: 8, U128: 16}
GMEM, SMEM, RMEM = range(3)
# moye_mma_atom
(MMA_UNIVERSAL_FMA, MFMA_F32_16x16x32_F16, MFMA_F32_32x32x16_F16, MFMA_F32_16x16x32_BF16,
 MFMA_F32_32x32x16_BF16, MFMA_F32_16x16x32_FP8, MFMA_F32_32x32x16_FP8, MFMA_F32_16x16x4_F32,
 MFMA_F32_32x32x2_F32) = range(9)
COPY_UNIVERSAL, COPY_LDS_TILED = 0, 1
GEMM_NO_XCD_SWIZZLE, GEMM_NO_LDS_SWIZZLE, GEMM_NO_WORKSPACE, GEMM_PINGPONG, GEMM_PREDICATE = 1, 2, 4, 0x100, 0x200
GEMM_WAVE4 = 0x400
GEMM_NO_PERSIST = 0x800
# moye_map operations (include/moye_hip.h)
MAP_IDENTITY, MAP_ADD, MAP_SUB, MAP_MUL, MAP_DIV, MAP_MAX, MAP_MIN, MAP_NEG, MAP_ABS = range(9)
MAP_OPS = {"identity": 0, "add": 1, "sub": 2, "mul": 3, "div": 4, "max": 5, "min": 6, "neg": 7, "abs": 8}


class MoyeError(RuntimeError):
    """A non-zero moye_status; `.status` holds the code (the reference raises Julia
    DimensionMismatch / AssertionError / ArgumentError in the same situations)."""

    def __init__(self, status, message):
        super().__init__("%s: %s" % (STATUS_NAMES[status] if 0 <= status < len(STATUS_NAMES) else status, message))
        self.status = status


class Tensor(C.Structure):
    _fields_ = [("ptr", C.c_void_p), ("dtype", C.c_int32), ("memspace", C.c_int32), ("rank", C.c_int32),
                ("_pad", C.c_int32), ("shape", C.c_int64 * MAX_RANK), ("stride", C.c_int64 * MAX_RANK)]


class TiledMMA(C.Structure):
    _fields_ = [("atom", C.c_int32), ("atom_layout_mnk", C.c_int32 * 3), ("tile_mnk", C.c_int32 * 3),
                ("cta_tile_mnk", C.c_int32 * 3), ("stages", C.c_int32), ("split_k", C.c_int32),
                ("flags", C.c_int32)]


class TiledCopy(C.Structure):
    _fields_ = [("op", C.c_int32), ("vec_bits", C.c_int32), ("thr_shape", C.c_int32 * 2),
                ("val_shape", C.c_int32 * 2), ("tiler_mn", C.c_int32 * 2), ("flags", C.c_int32)]


class GemmEpilogue(C.Structure):
    _fields_ = [("alpha", C.c_float), ("beta", C.c_float), ("op", C.c_int32), ("_pad", C.c_int32),
                ("operand", C.POINTER(Tensor)), ("scalar", C.c_double)]


_lib = None


def lib():
    """The loaded library (loads on first use; raises if it has not been built)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError("libmoye_hip.so is not built: run `python moye.jl_amd/build.py` "
                              "(or __graft_entry__.build())")
        _lib = C.CDLL(LIB_PATH)
        _declare(_lib)
    return _lib


def _declare(l):
    P, S, I32, I64p = C.POINTER, C.c_size_t, C.c_int32, C.POINTER(C.c_int64)
    cs, vp = C.c_char_p, C.c_void_p
    l.moye_last_error.restype = cs
    l.moye_version.restype = cs
    sig = {
        "moye_copy": [P(TiledCopy), P(Tensor), P(Tensor), vp],
        "moye_copy_if": [P(Tensor), P(Tensor), P(Tensor), vp],
        "moye_gemm": [P(TiledMMA), P(Tensor), P(Tensor), P(Tensor), P(Tensor), C.c_float, vp],
        "moye_gemm_ex": [P(TiledMMA), P(Tensor), P(Tensor), P(Tensor), P(Tensor), P(GemmEpilogue), vp, S, vp],
        "moye_gemm_release_workspace": [],
        "moye_gemm_noalloc": [P(TiledMMA), P(Tensor), P(Tensor), P(Tensor), P(Tensor), C.c_float, vp],
        "moye_gemm_workspace_size": [P(TiledMMA), P(Tensor), P(Tensor), P(Tensor), P(S)],
        "moye_gemm_ex_workspace_size": [P(TiledMMA), P(Tensor), P(Tensor), P(Tensor), P(GemmEpilogue), P(S)],
        "moye_gemm_explain": [P(TiledMMA), P(Tensor), P(Tensor), P(Tensor), P(Tensor), P(GemmEpilogue), I32, cs, S],
        "moye_device_malloc": [P(vp), S], "moye_device_free": [vp],
        "moye_memcpy_h2d": [vp, vp, S], "moye_memcpy_d2h": [vp, vp, S], "moye_memset": [vp, C.c_int, S],
        "moye_device_sync": [],
        "moye_device_info": [cs, S, P(I32), P(I32), P(S)],
        "moye_time_gemm": [P(TiledMMA), P(Tensor), P(Tensor), P(Tensor), P(Tensor), C.c_float, vp, I32, I32,
                           P(C.c_float)],
        "moye_time_copy": [P(TiledCopy), P(Tensor), P(Tensor), vp, I32, I32, P(C.c_float)],
    }
    for name, args in sig.items():
        f = getattr(l, name)
        f.argtypes = args
        f.restype = I32
    del I64p


def check(status):
    if status != OK:
        raise MoyeError(status, lib().moye_last_error().decode())


def make_tensor(ptr, dtype, shape, stride, memspace=GMEM):
    """A moye_tensor over a flattened layout (shape/stride: sequences of ints, strides in elements)."""
    shape, stride = list(shape), list(stride)
    if len(shape) != len(stride):
        raise MoyeError(ERR_RANK, "shape and stride must be congruent")
    if not 1 <= len(shape) <= MAX_RANK:
        raise MoyeError(ERR_RANK, "rank %d outside 1..%d" % (len(shape), MAX_RANK))
    t = Tensor()
    t.ptr, t.dtype, t.memspace, t.rank = ptr, dtype, memspace, len(shape)
    for i, (s, d) in enumerate(zip(shape, stride)):
        t.shape[i], t.stride[i] = int(s), int(d)
    return t

"""ctypes wrapper of the C oracle (gemm_oracle.c).  Test infrastructure only."""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_PATH = os.path.join(_HERE, "_build", "libmoye_oracle.so")
_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_PATH):
            import build as _b  # oracle/build.py
            _b.build()
        _lib = C.CDLL(_PATH)
        fp = C.POINTER(C.c_float)
        _lib.moye_ref_gemm.argtypes = [C.c_int] * 3 + [fp, C.c_long, C.c_long, fp, C.c_long, C.c_long, fp, C.c_long,
                                                       C.c_long] + [C.c_int] * 5
        _lib.moye_ref_gemm.restype = None
        _lib.moye_ref_round_f16.argtypes = [C.c_float]
        _lib.moye_ref_round_f16.restype = C.c_float
        _lib.moye_ref_round_bf16.argtypes = [C.c_float]
        _lib.moye_ref_round_bf16.restype = C.c_float
        lp = C.POINTER(C.c_long)
        _lib.moye_ref_copy.argtypes = [C.c_int, lp, lp, C.c_int, lp, lp, C.c_void_p, C.c_void_p, C.c_long, C.c_int]
        _lib.moye_ref_copy.restype = None
    return _lib


PROD = {"f32": 0, "f16": 1, "bf16": 2}


def gemm(A, B, C0=None, prod="f32", tile=(32, 32, 8), threads=1):
    """C = A*B' + C0 for fp32 ndarrays A:(M,K), B:(N,K) of any strides; returns a new (M,N) array."""
    A = np.asarray(A, dtype=np.float32)
    B = np.asarray(B, dtype=np.float32)
    M, K = A.shape
    N = B.shape[0]
    Cm = np.zeros((M, N), np.float32) if C0 is None else np.array(C0, dtype=np.float32, order="C")
    fp = C.POINTER(C.c_float)
    lib().moye_ref_gemm(M, N, K, A.ctypes.data_as(fp), A.strides[0] // 4, A.strides[1] // 4,
                        B.ctypes.data_as(fp), B.strides[0] // 4, B.strides[1] // 4,
                        Cm.ctypes.data_as(fp), Cm.strides[0] // 4, Cm.strides[1] // 4,
                        PROD[prod], tile[0], tile[1], tile[2], threads)
    return Cm


def copy(dst, dshape, dstride, src, sshape, sstride):
    """copyto! over flattened layouts on numpy buffers of equal itemsize."""
    n = int(np.prod(sshape))
    assert n == int(np.prod(dshape)) and dst.itemsize == src.itemsize
    arr = lambda v: (C.c_long * len(v))(*[int(x) for x in v])
    lib().moye_ref_copy(len(dshape), arr(dshape), arr(dstride), len(sshape), arr(sshape), arr(sstride),
                        dst.ctypes.data, src.ctypes.data, n, dst.itemsize)
    return dst

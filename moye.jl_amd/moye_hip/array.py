"""MoYeArray, the tiling verbs, TiledMMA / TiledCopy and the two algorithms, mirroring
src/array.jl, src/algorithm/array_algorithms.jl, src/atom/{mma,copy}.jl and
src/algorithm/{copy,blas}.jl of the reference for arrays in device (global) memory."""
import ctypes as C

from . import _lib, device
from . import layout as L
from ._lib import MoyeError, check
from .layout import COLON, Layout, _b, _l, _text_out, _tile_text, tuple_text

_CAP = 8192


class MoYeArray:
    """A non-owning view: device pointer + element type + layout (src/array.jl:53-59 over a
    ViewEngine, src/engine.jl:6-50).  `ptr` is an integer address; the caller keeps the buffer alive."""

    __slots__ = ("ptr", "dtype", "layout", "memspace", "_keep")

    def __init__(self, ptr, dtype, layout, memspace=_lib.GMEM, keep=None):
        self.ptr, self.dtype, self.memspace, self._keep = int(ptr), dtype, memspace, keep
        self.layout = layout if isinstance(layout, Layout) else L.make_layout(layout)

    @classmethod
    def from_torch(cls, t, layout=None, transposed=False):
        """MoYeArray(x::AbstractArray[, layout]) (src/array.jl:95-110).  torch tensors are row-major,
        Julia arrays column-major: without a layout the tensor's own sizes and strides are used."""
        from .torch_interop import dtype_of
        if layout is None:
            shape, stride = tuple(t.shape), tuple(t.stride())
            if transposed:
                shape, stride = shape[::-1], stride[::-1]
            layout = Layout(shape, stride)
        return cls(t.data_ptr(), dtype_of(t), layout, keep=t)

    @property
    def elsize(self):
        return _lib.DTYPE_BYTES[self.dtype]

    def __len__(self):
        return L.size(self.layout)

    def __repr__(self):
        return "MoYeArray(0x%x, dtype=%d, %s)" % (self.ptr, self.dtype, self.layout)

    def tensor(self):
        """The flattened moye_tensor descriptor handed to the HIP library."""
        shape, stride = L.flat(self.layout)
        return _lib.make_tensor(self.ptr, self.dtype, shape, stride, self.memspace)

    def _with(self, layout, offset=0):
        return MoYeArray(self.ptr + offset * self.elsize, self.dtype, layout, self.memspace, self._keep)


def view(x, *coord):
    """view(x, coord...) (src/array.jl:221-237): sliced layout, pointer advanced by the offset."""
    c = coord[0] if len(coord) == 1 else tuple(coord)
    if c is COLON:
        return x._with(x.layout)
    sub, off = L.slice_and_offset(x.layout, c)
    return x._with(sub, off)


def transpose(x):
    """src/array.jl:247-249."""
    if L.rank(x.layout) != 2:
        raise MoyeError(_lib.ERR_RANK, "transpose needs a rank-2 array")
    return x._with(L.make_layout(x.layout[2], x.layout[1]))


def recast(x, new_dtype):
    """recast(NewType, x) (src/array.jl:294-314)."""
    nb, ob = _lib.DTYPE_BYTES[new_dtype], x.elsize
    return MoYeArray(x.ptr, new_dtype, L.recast(x.layout, nb, ob), x.memspace, x._keep)


def _sliced(fn, x, *args):
    off = C.c_int64()
    buf = C.create_string_buffer(_CAP)
    check(fn(_b(x.layout.text), *args, buf, _CAP, C.byref(off)))
    return x._with(Layout(buf.value.decode()), off.value)


def local_tile(x, tile, coord, proj=None):
    """`@tile x tile coord [proj]` (src/algorithm/array_algorithms.jl:113-120,146-156)."""
    return _sliced(_l().moye_local_tile, x, _b(_tile_text(tile)), _b(tuple_text(coord)),
                   _b("" if proj is None else tuple_text(proj)))


def local_partition(x, tile, coord_or_index, proj=None):
    """`@parallelize x thr_layout idx [proj]` (src/algorithm/array_algorithms.jl:36-47,101-111)."""
    return _sliced(_l().moye_local_partition, x, _b(_tile_text(tile)), _b(tuple_text(coord_or_index)),
                   _b("" if proj is None else tuple_text(proj)))


# ---- MMA -----------------------------------------------------------------------------------------
ATOM_NAMES = ["UniversalFMA", "MFMA_F32_16x16x32_F16", "MFMA_F32_32x32x16_F16", "MFMA_F32_16x16x32_BF16",
              "MFMA_F32_32x32x16_BF16", "MFMA_F32_16x16x32_FP8", "MFMA_F32_32x32x16_FP8", "MFMA_F32_16x16x4_F32",
              "MFMA_F32_32x32x2_F32"]


def _emit(text, file):
    if file is not False:
        print(text, file=file)
    return text


class TiledMMA:
    """make_tiled_mma(op, atom_layout, permutations) (src/atom/mma.jl:193-233).  `op` is a
    moye_mma_atom number or an atom name (the reference's NVIDIA atoms exist by name, as data)."""

    def __init__(self, op, atom_layout=None, permutations=None, cta_tile=None, stages=0, flags=0):
        self.op = op
        self.name = ATOM_NAMES[op] if isinstance(op, int) else op
        self.atom_layout = atom_layout if atom_layout is not None else L.static_layout((1, 1, 1))
        self.permutations = permutations
        self.cta_tile, self.stages, self.flags = cta_tile, stages, flags

    def _q(self, what):
        perm = "" if self.permutations is None else _tile_text(tuple(self.permutations))
        return _text_out(_l().moye_tiled_mma_query, _b(self.name), _b(self.atom_layout.text), _b(perm), _b(what))

    def thr_layout_vmnk(self):
        return Layout(self._q("thr_layout_vmnk"))

    def tile_shape(self):
        return L.parse_tuple(self._q("tile_shape"))

    def tile_size(self, i):
        return self.tile_shape()[i - 1]

    def size(self):
        return int(L.parse_tuple(self._q("size")))

    def layout_a(self):
        return Layout(self._q("layout_a"))

    def layout_b(self):
        return Layout(self._q("layout_b"))

    def layout_c(self):
        return Layout(self._q("layout_c"))

    def layout_tv(self, operand):
        return Layout(self._q("layout%s_TV" % operand))

    def layout_mn(self, operand):
        """get_layoutA_MK / get_layoutB_NK / get_layoutC_MN (src/atom/mma.jl:235-262): (layout, thread-id layout)."""
        return Layout(self._q({"A": "layoutA_MK", "B": "layoutB_NK", "C": "layoutC_MN"}[operand])), Layout(self._q("thrID_" + operand))

    def print_tv(self, file=None):
        """The three tables print_typst(tiled_mma) draws (src/print.jl:46-93,317-323), as text: B as (K, N), then A,
        then C; a cell reads T<thread index>V<value index>.  Returns the text; file=False only returns it."""
        return _emit(self._q("print"), file)

    def get_slice(self, thr_idx):
        return ThrMMA(self, thr_idx)

    def descriptor(self):
        """moye_tiled_mma for the device call."""
        if not isinstance(self.op, int):
            raise MoyeError(_lib.ERR_UNSUPPORTED, "atom %s has no gfx950 kernel" % self.name)
        d = _lib.TiledMMA()
        perm = "" if self.permutations is None else _tile_text(tuple(self.permutations))
        check(_l().moye_make_tiled_mma(self.op, _b(self.atom_layout.text), _b(perm), C.byref(d)))
        if self.cta_tile is not None:
            for i in range(3):
                d.cta_tile_mnk[i] = self.cta_tile[i]
        elif self.permutations is None:
            for i in range(3):
                d.cta_tile_mnk[i] = 0  # let the library choose
        d.stages, d.flags = self.stages, self.flags
        return d


def make_tiled_mma(op, atom_layout=None, permutations=None, **kw):
    return TiledMMA(op, atom_layout, permutations, **kw)


class ThrMMA:
    """get_slice(tiled_mma, thr_idx) (src/atom/mma.jl:171-175)."""

    def __init__(self, tiled_mma, thr_idx):
        self.tiled_mma, self.thr_idx = tiled_mma, thr_idx

    def _part(self, operand, x):
        m = self.tiled_mma
        perm = "" if m.permutations is None else _tile_text(tuple(m.permutations))
        off = C.c_int64()
        buf = C.create_string_buffer(_CAP)
        check(_l().moye_tiled_mma_partition(_b(m.name), _b(m.atom_layout.text), _b(perm), self.thr_idx,
                                            operand.encode(), _b(x.layout.text), buf, _CAP, C.byref(off)))
        return x._with(Layout(buf.value.decode()), off.value)

    def partition_A(self, a):
        return self._part("A", a)

    def partition_B(self, b):
        return self._part("B", b)

    def partition_C(self, c):
        return self._part("C", c)

    # partition_fragment_X / make_fragment_X (src/atom/mma.jl:26-47,310-337): the register-resident
    # counterpart of a partition.  Registers have no host address, so the mirror returns the
    # fragment's LAYOUT (what a device kernel would allocate), not an array.
    def partition_fragment_A(self, a):
        return L.make_fragment_like(self.partition_A(a).layout)

    def partition_fragment_B(self, b):
        return L.make_fragment_like(self.partition_B(b).layout)

    def partition_fragment_C(self, c):
        return L.make_fragment_like(self.partition_C(c).layout)

    make_fragment_A, make_fragment_B, make_fragment_C = partition_fragment_A, partition_fragment_B, partition_fragment_C


# ---- copy ------------------------------------------------------------------------------------------
class CopyAtom:
    """CopyAtom{UniversalCopy{S,D}, T}() (src/atom/copy.jl:31-59): S/D are the access widths in bits,
    T the value width in bits."""

    def __init__(self, src_bits, val_bits, dst_bits=None):
        self.src_bits, self.dst_bits, self.val_bits = src_bits, dst_bits or src_bits, val_bits


class TiledCopy:
    """make_tiled_copy(atom, thr_layout, val_layout) (src/atom/copy.jl:249-258)."""

    def __init__(self, atom, thr_layout, val_layout=None, op=_lib.COPY_UNIVERSAL, flags=0):
        self.atom, self.thr_layout = atom, thr_layout
        self.val_layout = val_layout if val_layout is not None else L.static_layout(1)
        self.op, self.flags = op, flags

    def _q(self, what):
        a = self.atom
        return _text_out(_l().moye_tiled_copy_query, a.src_bits, a.dst_bits, a.val_bits, _b(self.thr_layout.text),
                         _b(self.val_layout.text), _b(what))

    @property
    def tiled_layout_TV(self):
        return Layout(self._q("layout_tv"))

    @property
    def tiler_MN(self):
        return L.parse_tuple(self._q("tiler"))

    def size(self):
        return int(L.parse_tuple(self._q("size")))

    @property
    def num_val_src(self):
        return int(L.parse_tuple(self._q("num_val_src")))

    def get_slice(self, thr_idx):
        return ThrCopy(self, thr_idx)

    def get_layoutS_TV(self):
        return Layout(self._q("layoutS_TV"))

    def get_layoutD_TV(self):
        return Layout(self._q("layoutD_TV"))

    def get_layoutS_MN(self):
        """src/atom/copy.jl:175-179: (layout, thread-id layout)."""
        return Layout(self._q("layoutS_MN")), L.static_layout(self.size())

    def get_layoutD_MN(self):
        """src/atom/copy.jl:188-192."""
        return Layout(self._q("layoutD_MN")), L.static_layout(self.size())

    def print_tv(self, file=None):
        """The source and destination tables print_typst(tiled_copy) draws (src/print.jl:200-233,337-345), as text."""
        return _emit(self._q("print"), file)

    def descriptor(self):
        d = _lib.TiledCopy()
        d.op, d.vec_bits, d.flags = self.op, self.atom.src_bits, self.flags
        ts, vs = self.thr_layout.shape, self.val_layout.shape
        ts = ts if isinstance(ts, tuple) else (ts, 1)
        vs = vs if isinstance(vs, tuple) else (vs, 1)
        tiler = self.tiler_MN
        for i in range(2):
            d.thr_shape[i] = int(L.tuple_op("product", ts[i])) if i < len(ts) else 1
            d.val_shape[i] = int(L.tuple_op("product", vs[i])) if i < len(vs) else 1
            d.tiler_mn[i] = int(tiler[i]) if i < len(tiler) else 1
        return d


def make_tiled_copy(atom, thr_layout, val_layout=None, **kw):
    return TiledCopy(atom, thr_layout, val_layout, **kw)


class TiledCopyTV:
    """TiledCopy(atom, layout_tv, tiler) (src/atom/copy.jl:113-125), the form make_tiled_copy_A/B/C
    produce from a TiledMMA (src/atom/copy.jl:227-240)."""

    def __init__(self, atom, layout_tv, tiler):
        self.atom, self.tiled_layout_TV, self.tiler_MN = atom, layout_tv, tuple(tiler)

    def _args(self):
        a = self.atom
        return (a.src_bits, a.dst_bits, a.val_bits, _b(self.tiled_layout_TV.text), _b(L.tuple_text(self.tiler_MN)))

    def _q(self, what):
        return _text_out(_l().moye_tiled_copy_tv_query, *self._args(), _b(what))

    def size(self):
        return int(L.parse_tuple(self._q("size")))

    def get_layoutS_TV(self):
        return Layout(self._q("layoutS_TV"))

    def get_layoutD_TV(self):
        return Layout(self._q("layoutD_TV"))

    def get_layoutS_MN(self):
        return Layout(self._q("layoutS_MN")), L.static_layout(self.size())

    def get_layoutD_MN(self):
        return Layout(self._q("layoutD_MN")), L.static_layout(self.size())

    def print_tv(self, file=None):
        return _emit(self._q("print"), file)

    def retile(self, x):
        """retile_S / retile_D (src/atom/copy.jl:151-166) on a MoYeArray or a Layout."""
        lay = x if isinstance(x, Layout) else x.layout
        out = Layout(_text_out(_l().moye_tiled_copy_tv_retile, *self._args(), _b(lay.text)))
        return out if isinstance(x, Layout) else x._with(out, 0)

    def get_slice(self, thr_idx):
        return ThrCopyTV(self, thr_idx)


class ThrCopyTV:
    def __init__(self, tiled_copy, thr_idx):
        self.tiled_copy, self.thr_idx = tiled_copy, thr_idx

    def _part(self, which, x):
        off = C.c_int64()
        buf = C.create_string_buffer(_CAP)
        check(_l().moye_tiled_copy_tv_partition(*self.tiled_copy._args(), self.thr_idx, which.encode(),
                                                _b(x.layout.text), buf, _CAP, C.byref(off)))
        return x._with(Layout(buf.value.decode()), off.value)

    def partition_S(self, s):
        return self._part("S", s)

    def partition_D(self, d):
        return self._part("D", d)

    def retile_S(self, s):
        return self.tiled_copy.retile(s)

    retile_D = retile_S


def make_tiled_copy_A(atom, tiled_mma):
    """src/atom/copy.jl:227-230."""
    return TiledCopyTV(atom, tiled_mma.layout_tv("A"), (tiled_mma.tile_size(1), tiled_mma.tile_size(3)))


def make_tiled_copy_B(atom, tiled_mma):
    """src/atom/copy.jl:231-235."""
    return TiledCopyTV(atom, tiled_mma.layout_tv("B"), (tiled_mma.tile_size(2), tiled_mma.tile_size(3)))


def make_tiled_copy_C(atom, tiled_mma):
    """src/atom/copy.jl:236-240."""
    return TiledCopyTV(atom, tiled_mma.layout_tv("C"), (tiled_mma.tile_size(1), tiled_mma.tile_size(2)))


class ThrCopy:
    """get_slice(tiled_copy, thr_idx) (src/atom/copy.jl:198-214)."""

    def __init__(self, tiled_copy, thr_idx):
        self.tiled_copy, self.thr_idx = tiled_copy, thr_idx

    def _part(self, which, x):
        t, a = self.tiled_copy, self.tiled_copy.atom
        off = C.c_int64()
        buf = C.create_string_buffer(_CAP)
        check(_l().moye_tiled_copy_partition(a.src_bits, a.dst_bits, a.val_bits, _b(t.thr_layout.text),
                                             _b(t.val_layout.text), self.thr_idx, which.encode(),
                                             _b(x.layout.text), buf, _CAP, C.byref(off)))
        return x._with(Layout(buf.value.decode()), off.value)

    def partition_S(self, s):
        return self._part("S", s)

    def partition_D(self, d):
        return self._part("D", d)


# ---- the algorithms --------------------------------------------------------------------------------
def copyto_(dst, src, tiled_copy=None, stream=None):
    """copyto!(dst, src) / copyto!(tiled_copy, dst, src) (src/algorithm/copy.jl:42-46,106-110); returns dst."""
    tc = tiled_copy.descriptor() if isinstance(tiled_copy, TiledCopy) else tiled_copy
    d = dst if isinstance(dst, _lib.Tensor) else dst.tensor()   # raw descriptors pass straight through
    s = src if isinstance(src, _lib.Tensor) else src.tensor()
    device.copyto_(d, s, tc, stream)
    return dst


def copyto_if_(dst, src, mask, stream=None):
    """copyto_if!(dst, src, mask) (src/algorithm/copy.jl:4-16): element i moves where the mask's element i is true;
    the mask is a MoYeArray of bytes (Bool) with its own layout.  Returns dst."""
    t = [x if isinstance(x, _lib.Tensor) else x.tensor() for x in (dst, src, mask)]
    device.copyto_if_(t[0], t[1], t[2], stream)
    return dst


def gemm_(mma, D, A, B, C_=None, alpha=1.0, stream=None):
    """gemm!(mma, D, A, B, C) (src/algorithm/blas.jl:11-17): D = alpha * A * B' + C with A:(M,K), B:(N,K),
    C,D:(M,N).  gemm_(mma, A, B, C) with three arrays accumulates in place like the reference's 3-argument form."""
    if not isinstance(mma, (TiledMMA, _lib.TiledMMA)):  # gemm!(A, B, C): UniversalFMA
        A, B, C_, D = mma, D, A, A
        mma = TiledMMA(_lib.MMA_UNIVERSAL_FMA)
    d = mma.descriptor() if isinstance(mma, TiledMMA) else mma

    def t(x):
        return x if x is None or isinstance(x, _lib.Tensor) else x.tensor()

    device.gemm_(d, t(D), t(A), t(B), t(C_), alpha, stream)


def axpby_(a, X, b, Y, stream=None):
    """axpby!(a, X, b, Y) (src/algorithm/blas.jl:1-9): Y = a*X + b*Y element by element; returns Y."""
    x = X if isinstance(X, _lib.Tensor) else X.tensor()
    y = Y if isinstance(Y, _lib.Tensor) else Y.tensor()
    device.axpby_(a, x, b, y, stream)
    return Y


def fill_(X, value, stream=None):
    """fill!(x, value) (src/algorithm/array_algorithms.jl:158-164); returns X."""
    device.fill_(X if isinstance(X, _lib.Tensor) else X.tensor(), value, stream)
    return X


def map_(op, dst, A, B=None, scalar=0.0, stream=None):
    """dst .= op.(A, B) or op.(A, scalar) (src/broadcast.jl:5-41; map!, src/algorithm/array_algorithms.jl:192-210);
    op is one of "identity", "add", "sub", "mul", "div", "max", "min", "neg", "abs".  Returns dst."""
    t = lambda x: x if isinstance(x, _lib.Tensor) else x.tensor()
    device.map_(_lib.MAP_OPS[op] if isinstance(op, str) else op, t(dst), t(A), None if B is None else t(B), scalar, stream)
    return dst


def broadcast(op, A, B=None, scalar=0.0, stream=None):
    """op.(A, B): a new array with `make_layout_like(layout(A))`, as `similar` gives the reference's broadcast
    (src/broadcast.jl:27-31).  The memory is a torch tensor the result keeps alive."""
    import torch
    from .torch_interop import TORCH_DTYPES
    lay = L.make_layout_like(A.layout)
    buf = torch.empty(int(L.cosize(lay)), dtype=TORCH_DTYPES[A.dtype], device="cuda")
    out = MoYeArray(buf.data_ptr(), A.dtype, lay, keep=buf)
    return map_(op, out, A, B, scalar, stream)


def zeros_(X, stream=None):
    """zeros!(x) (src/algorithm/array_algorithms.jl:176-182)."""
    return fill_(X, 0.0, stream)

"""CPU oracle for MoYe's arrays, tiling verbs, atoms, copyto! and gemm!.

TEST INFRASTRUCTURE ONLY — see layout_oracle.py for the rules.  Restates
src/array.jl, src/algorithm/array_algorithms.jl, src/atom/{mma,copy}.jl,
src/traits/*.jl, src/algorithm/{copy,blas}.jl and src/arch/mma/mma.jl of the
reference over numpy buffers.  Pure-Python loops: for small cases only.

The tensor-core tables of the reference (`mma_sm70/75/80.jl`, `ldmatrix.jl`)
are reproduced as data because the reference's own tests and SVG fixtures are
expressed through them (pinned by tests/test_svg_fixtures.py against the figures
of the reference's manual); the gfx950 MFMA tables are new and are pinned on
hardware by the one-wave atom probe test (tests/test_gpu_gemm.py).

Parity unpinned in this file (the reference holds no vector for them): `copyto_if`
(src/algorithm/copy.jl:4-16 is never called with a mask in the reference's tests;
checked only against the element loop written out) and the printed form of
`get_layout{A,B,C}_{MK,NK,MN}` / `get_layout{S,D}_MN` (their function values are pinned
by the manual's figures and by inversion through the TV layouts,
tests/test_svg_fixtures.py).
"""
from __future__ import annotations

import numpy as np

from layout_oracle import (COLON, S, Layout, SL, _0, _1, append, lflatten, capacity, coalesce, composition,
                           complement, cosize, dice, dice_layout, get_congr_coord, is_static,
                           is_tuple, lappend, lgroup, logical_divide, logical_product, lprepend,
                           lrank, ltranspose, lzip, make_fragment_like, make_layout,
                           make_layout_like, product_each, raked_product, rank, recast_layout,
                           repeat, right_inverse, shape_div, size, slice_and_offset, smax, static,
                           tiled_product, upcast, withshape, zipped_divide, prepend)

# --------------------------------------------------------------------------
# MoYeArray (src/array.jl)
# --------------------------------------------------------------------------


class Array:
    """array.jl:53-59 — a buffer (1-D numpy array), an element offset and a layout."""

    def __init__(self, buf, layout, offset=0, memspace="gmem"):
        self.buf = buf
        self.layout = layout
        self.offset = int(offset)
        self.memspace = memspace

    @classmethod
    def undef(cls, dtype, layout, memspace="rmem"):
        """array.jl:61-66 — owning arrays need a static layout."""
        if not isinstance(layout, Layout):
            layout = make_layout(layout)
        if not (is_static(layout.shape) and is_static(layout.stride)):
            raise ValueError("Owning `MoYeArray` cannot be created from a dynamic layout")
        return cls(np.zeros(int(cosize(layout)), dtype=dtype), layout, 0, memspace)

    @classmethod
    def from_matrix(cls, a, transposed=False):
        """array.jl:95-103 — column-major over an array, row-major over a Transpose."""
        a = np.asarray(a)
        if transposed:  # `a` is the parent; the wrapper has the reversed size
            return cls(a.reshape(-1, order="F"), make_layout(tuple(reversed(a.shape)), "GenRowMajor"))
        return cls(a.reshape(-1, order="F"), make_layout(tuple(a.shape), "GenColMajor"))

    @property
    def dtype(self):
        return self.buf.dtype

    def index0(self, coord):
        return self.offset + int(self.layout(coord)) - 1

    def __getitem__(self, coord):
        return self.buf[self.index0(coord)]

    def __setitem__(self, coord, v):
        self.buf[self.index0(coord)] = v

    def __len__(self):
        return int(size(self.layout))

    def offsets(self):
        """0-based buffer offsets of the logical elements 1..size, in order.  Large arrays take the same
        colexicographic decomposition (stride.jl:20-31) over the flattened modes in numpy, all elements at once;
        tests/test_oracle_tiled.py checks the two forms against each other."""
        n = len(self)
        if n > 4096:
            return self.offsets_vectorised()
        return np.array([self.index0(i) for i in range(1, n + 1)], dtype=np.int64)

    def offsets_vectorised(self):
        flat = lflatten(self.layout)
        shp = flat.shape if isinstance(flat.shape, tuple) else (flat.shape,)
        strd = flat.stride if isinstance(flat.stride, tuple) else (flat.stride,)
        idx = np.arange(len(self), dtype=np.int64)
        off = np.full(len(self), self.offset, dtype=np.int64)
        for s_, d_ in zip(shp, strd):
            off += (idx % int(s_)) * int(d_)
            idx //= int(s_)
        return off

    def values(self):
        return self.buf[self.offsets()]


def view(x, *coord):
    """array.jl:221-237."""
    if len(coord) == 1 and coord[0] is COLON:
        return Array(x.buf, x.layout, x.offset, x.memspace)
    c = tuple(coord) if len(coord) > 1 else coord[0]
    sliced, off = slice_and_offset(x.layout, c)
    return Array(x.buf, sliced, x.offset + int(off), x.memspace)


def similar(x, dtype=None):
    """array.jl:239-245."""
    return Array.undef(dtype or x.dtype, make_layout_like(x.layout))


def transpose(x):
    """array.jl:247-249."""
    return Array(x.buf, ltranspose(x.layout), x.offset, x.memspace)


def append_dim(x, n):
    """array.jl:256-258."""
    return Array(x.buf, lappend(x.layout, n), x.offset, x.memspace)


def prepend_dim(x, n):
    """array.jl:265-267."""
    return Array(x.buf, lprepend(x.layout, n), x.offset, x.memspace)


def recast(dtype, x):
    """array.jl:294-314 (non-negative strides only)."""
    dtype = np.dtype(dtype)
    old = x.buf.dtype.itemsize
    new_layout = recast_layout(x.layout, dtype.itemsize, old)
    byte_off = x.offset * old
    assert byte_off % dtype.itemsize == 0
    return Array(x.buf.view(dtype), new_layout, byte_off // dtype.itemsize, x.memspace)


def local_tile(x, tile, coord, proj=None):
    """array_algorithms.jl:113-120 (`@tile`)."""
    if proj is not None:
        return local_tile(x, dice(tile, proj), dice(coord, proj))
    r1, r2 = len(tile), lrank(x.layout)
    z = Array(x.buf, zipped_divide(x.layout, tile), x.offset, x.memspace)
    return view(z, repeat(COLON, r1), append(coord, COLON, r2))


def local_partition(x, tile, index, proj=None):
    """array_algorithms.jl:36-47 (`@parallelize`)."""
    if isinstance(tile, Layout):
        if proj is not None:
            shp = dice(tuple(capacity(s) for s in tile.shape), proj)
            coord = get_congr_coord(dice_layout(tile, proj), index)
        else:
            shp = tuple(capacity(s) for s in tile.shape) if is_tuple(tile.shape) else (tile.shape,)
            coord = get_congr_coord(tile, index)
            if not is_tuple(coord):
                coord = (coord,)
        return local_partition(x, shp, coord)
    if proj is not None:
        return local_partition(x, dice(tile, proj), dice(index, proj))
    n = lrank(x.layout)
    z = Array(x.buf, zipped_divide(x.layout, tile), x.offset, x.memspace)
    return view(z, tuple(index), repeat(COLON, n))


# --------------------------------------------------------------------------
# MMA ops and traits
# --------------------------------------------------------------------------


class MMAOp:
    """arch/mma/mma.jl:5-64 + traits/mma.jl:33-42: value types, shape, thread and TV layouts."""

    def __init__(self, name, shape_mnk, thr_id, layout_a, layout_b, layout_c, types):
        self.name = name
        self.shape_mnk = static(shape_mnk)
        self.thr_id = thr_id
        self.layout_a, self.layout_b, self.layout_c = layout_a, layout_b, layout_c
        self.types = types  # (D, A, B, C) numpy dtypes or names


def UniversalFMA(d="f32", a="f32", b="f32", c="f32"):
    """traits/mma.jl:38-42."""
    return MMAOp("UniversalFMA", (1, 1, 1), SL(1), SL((1, 1)), SL((1, 1)), SL((1, 1)), (d, a, b, c))


# traits/mma_sm70.jl, mma_sm75.jl, mma_sm80.jl — only the rows the reference's tests and
# docstrings exercise.
REFERENCE_MMA_OPS = {
    "MMAOP_8x8x4_F32F16F16F32_NT": MMAOp(
        "MMAOP_8x8x4_F32F16F16F32_NT", (8, 8, 4), SL((4, 2), (1, 16)),
        SL(((4, 2), 4), ((8, 4), 1)), SL(((4, 2), 4), ((8, 4), 1)),
        SL(((2, 2, 2), (2, 2, 2)), ((1, 16, 4), (8, 2, 32))), ("f32", "f16", "f16", "f32")),
    "MMAOP_16x8x8_F16F16F16F16_TN": MMAOp(
        "MMAOP_16x8x8_F16F16F16F16_TN", (16, 8, 8), SL(32),
        SL(((4, 8), (2, 2)), ((32, 1), (16, 8))), SL(((4, 8), 2), ((16, 1), 8)),
        SL(((4, 8), (2, 2)), ((32, 1), (16, 8))), ("f16", "f16", "f16", "f16")),
    "MMAOP_16x8x16_F16F16F16F16_TN": MMAOp(
        "MMAOP_16x8x16_F16F16F16F16_TN", (16, 8, 16), SL(32),
        SL(((4, 8), (2, 2, 2)), ((32, 1), (16, 8, 128))), SL(((4, 8), (2, 2)), ((16, 1), (8, 64))),
        SL(((4, 8), (2, 2)), ((32, 1), (16, 8))), ("f16", "f16", "f16", "f16")),
    "MMAOP_16x8x8_F32TF32TF32F32_TN": MMAOp(
        "MMAOP_16x8x8_F32TF32TF32F32_TN", (16, 8, 8), SL(32),
        SL(((4, 8), (2, 2)), ((16, 1), (8, 64))), SL(((4, 8), 2), ((8, 1), 32)),
        SL(((4, 8), (2, 2)), ((32, 1), (16, 8))), ("f32", "tf32", "tf32", "f32")),
}

# gfx950 MFMA atoms (one 64-lane wave).  (thr, val) -> 1-based col-major index into the
# (M,K) / (N,K) / (M,N) atom tile.  Lane l of a 16x16xK atom holds A[l%16][8(l/16)..+7],
# B[l%16][same k] and D[4(l/16)+r][l%16]; a 32x32xK atom holds A[l%32][8(l/32)..+7] and
# D[8(r/4)+4(l/32)+r%4][l%32].
MFMA_OPS = {
    "MFMA_F32_16x16x32_F16": MMAOp(
        "MFMA_F32_16x16x32_F16", (16, 16, 32), SL(64),
        SL(((16, 4), 8), ((1, 128), 16)), SL(((16, 4), 8), ((1, 128), 16)),
        SL(((16, 4), 4), ((16, 4), 1)), ("f32", "f16", "f16", "f32")),
    "MFMA_F32_32x32x16_F16": MMAOp(
        "MFMA_F32_32x32x16_F16", (32, 32, 16), SL(64),
        SL(((32, 2), 8), ((1, 256), 32)), SL(((32, 2), 8), ((1, 256), 32)),
        SL(((32, 2), (4, 4)), ((32, 4), (1, 8))), ("f32", "f16", "f16", "f32")),
    "MFMA_F32_16x16x4_F32": MMAOp(
        "MFMA_F32_16x16x4_F32", (16, 16, 4), SL(64),
        SL(((16, 4), 1), ((1, 16), 0)), SL(((16, 4), 1), ((1, 16), 0)),
        SL(((16, 4), 4), ((16, 4), 1)), ("f32", "f32", "f32", "f32")),
    "MFMA_F32_32x32x2_F32": MMAOp(
        "MFMA_F32_32x32x2_F32", (32, 32, 2), SL(64),
        SL(((32, 2), 1), ((1, 32), 0)), SL(((32, 2), 1), ((1, 32), 0)),
        SL(((32, 2), (4, 4)), ((32, 4), (1, 8))), ("f32", "f32", "f32", "f32")),
}
for _n, _t in (("BF16", "bf16"), ("FP8", "f8e4m3")):
    for _g in ("16x16x32", "32x32x16"):
        _src = MFMA_OPS["MFMA_F32_%s_F16" % _g]
        MFMA_OPS["MFMA_F32_%s_%s" % (_g, _n)] = MMAOp(
            "MFMA_F32_%s_%s" % (_g, _n), tuple(int(v) for v in _src.shape_mnk), _src.thr_id,
            _src.layout_a, _src.layout_b, _src.layout_c, ("f32", _t, _t, "f32"))


class TiledMMA:
    """atom/mma.jl:80-199."""

    def __init__(self, atom, atom_layout=None, permutations=None):
        self.atom = atom
        al = atom_layout if atom_layout is not None else SL((1, 1, 1))
        self.atom_layout_mnk = lappend(al, 3)                       # atom/mma.jl:196
        perm = permutations if permutations is not None else (COLON, COLON, COLON)
        self.permutation_mnk = append(perm, COLON, 3)               # atom/mma.jl:197

    def thr_layout_vmnk(self):
        """atom/mma.jl:115-118."""
        return tiled_product(self.atom.thr_id, self.atom_layout_mnk)

    def size(self):
        return size(self.thr_layout_vmnk())

    def tile_size(self, i):
        """atom/mma.jl:178-189 (i is 1-based)."""
        core = self.atom.shape_mnk[i - 1] * size(self.thr_layout_vmnk(), i + 1)
        s = self.permutation_mnk[i - 1]
        if s is COLON:
            return core
        p = size(s) if isinstance(s, Layout) else s
        return smax(core, p)

    def tile_shape(self):
        return tuple(self.tile_size(i) for i in (1, 2, 3))

    def _thrfrg(self, l, i0, i1, tv, j0, j1):
        t = self.thr_layout_vmnk()
        mnk = self.atom.shape_mnk
        perm = self.permutation_mnk
        t_array = logical_divide(l, (perm[i0], perm[i1]))
        a_array = zipped_divide(t_array, (make_layout(mnk[i0]), make_layout(mnk[i1])))
        tv_array = composition(a_array, (tv, COLON))
        thr_tile = (COLON, (make_layout(size(t, j0)), make_layout(size(t, j1))))
        return zipped_divide(tv_array, thr_tile)

    def thrfrg_C(self, l):
        """atom/mma.jl:120-135."""
        return self._thrfrg(l, 0, 1, self.atom.layout_c, 2, 3)

    def thrfrg_A(self, l):
        """atom/mma.jl:137-152."""
        return self._thrfrg(l, 0, 2, self.atom.layout_a, 2, 4)

    def thrfrg_B(self, l):
        """atom/mma.jl:154-169."""
        return self._thrfrg(l, 1, 2, self.atom.layout_b, 3, 4)

    def get_slice(self, thr_idx):
        """atom/mma.jl:171-175."""
        return ThrMMA(self, get_congr_coord(self.thr_layout_vmnk(), thr_idx))

    # atom/mma.jl:264-289
    def get_layoutC_TV(self):
        ref = make_layout((self.tile_size(1), self.tile_size(2)))
        tv = self.thrfrg_C(ref)
        return composition(tv, (right_inverse(self.thr_layout_vmnk()), COLON))

    def get_layoutA_TV(self):
        ref = make_layout((self.tile_size(1), self.tile_size(3)))
        tv = self.thrfrg_A(ref)
        t = self.thr_layout_vmnk()
        atile = (COLON, (make_layout((size(t, 2), size(t, 3)), (_1, _0)), COLON))
        return composition(composition(tv, (atile, COLON)), (right_inverse(t), COLON))

    def get_layoutB_TV(self):
        ref = make_layout((self.tile_size(2), self.tile_size(3)))
        tv = self.thrfrg_B(ref)
        t = self.thr_layout_vmnk()
        btile = (COLON, (make_layout((size(t, 2), size(t, 3)), (_0, _1)), COLON))
        return composition(composition(tv, (btile, COLON)), (right_inverse(t), COLON))


    # atom/mma.jl:235-262: cell of the tile -> index into the un-permuted (thr, val) fragment layout, together with
    # the layout that turns the thread part of that index into a thread index (the other operand's atoms dropped)
    def get_layoutC_MN(self):
        ref = make_layout((self.tile_size(1), self.tile_size(2)))
        return withshape(right_inverse(self.thrfrg_C(ref)), ref.shape), self.thr_layout_vmnk()((COLON, COLON, COLON, _1))

    def get_layoutA_MK(self):
        ref = make_layout((self.tile_size(1), self.tile_size(3)))
        return withshape(right_inverse(self.thrfrg_A(ref)), ref.shape), self.thr_layout_vmnk()((COLON, COLON, _1, COLON))

    def get_layoutB_NK(self):
        ref = make_layout((self.tile_size(2), self.tile_size(3)))
        return withshape(right_inverse(self.thrfrg_B(ref)), ref.shape), self.thr_layout_vmnk()((COLON, _1, COLON, COLON))


def tv_table(layout_mn, thr_id):
    """The cells print_typst writes (src/print.jl:64-71,220-228): for cell (m, n) of the tile,
    `val_idx, thr = fldmod1(layout_mn(m, n), size(thr_id))` and `thr_idx = thr_id(thr)`; returns
    table[m][n] = (thr_idx, val_idx), both 1-based as the reference prints them."""
    nthr = int(size(thr_id))
    rows, cols = int(size(layout_mn, 1)), int(size(layout_mn, 2))
    out = []
    for m in range(1, rows + 1):
        row = []
        for n in range(1, cols + 1):
            idx = int(layout_mn((m, n))) - 1
            row.append((int(thr_id(idx % nthr + 1)), idx // nthr + 1))
        out.append(row)
    return out


def make_tiled_mma(op, atom_layout=None, permutations=None):
    """atom/mma.jl:193-199,229-233."""
    return TiledMMA(op, atom_layout, permutations)


class ThrMMA:
    """atom/mma.jl:86-92,292-308."""

    def __init__(self, tiled_mma, thr_vmnk):
        self.tiled_mma = tiled_mma
        self.thr_vmnk = thr_vmnk

    def _part(self, x, frg, i, j):
        arr = Array(x.buf, frg(x.layout), x.offset, x.memspace)
        v = self.thr_vmnk
        coord = (v[0], (v[i], v[j]))
        nrest = rank(arr.layout[2].shape[1])
        return view(arr, coord, (COLON, repeat(COLON, nrest)))

    def partition_C(self, c):
        return self._part(c, self.tiled_mma.thrfrg_C, 1, 2)

    def partition_A(self, a):
        return self._part(a, self.tiled_mma.thrfrg_A, 1, 3)

    def partition_B(self, b):
        return self._part(b, self.tiled_mma.thrfrg_B, 2, 3)

    def partition_fragment_C(self, c):
        """atom/mma.jl:26-31,310-313."""
        p = self.partition_C(c)
        return Array.undef(np.float32, make_layout(p.layout.shape))

    def partition_fragment_A(self, a):
        """atom/mma.jl:34-39,314-317."""
        return Array.undef(a.dtype, make_fragment_like(self.partition_A(a).layout))

    def partition_fragment_B(self, b):
        """atom/mma.jl:40-45,318-321."""
        return Array.undef(b.dtype, make_fragment_like(self.partition_B(b).layout))


# --------------------------------------------------------------------------
# copy ops, traits, atoms, tiled copies
# --------------------------------------------------------------------------


class CopyTraits:
    """traits/copy.jl:3-21 — thread id layout and *bit* layouts (thr, bit) for src/dst/ref."""

    def __init__(self, name, threadid, src, dst, ref=None):
        self.name, self.threadid, self.srclayout, self.dstlayout = name, threadid, src, dst
        self.reflayout = ref if ref is not None else src


def UniversalCopy(src_bits, dst_bits=None):
    """traits/copy.jl:16-21."""
    dst_bits = src_bits if dst_bits is None else dst_bits
    return CopyTraits("UniversalCopy", make_layout(_1), make_layout((_1, S(src_bits))),
                      make_layout((_1, S(dst_bits))))


def _ldsm(name, src, dst):
    return CopyTraits(name, SL(32), src, dst, dst)


# traits/ldmatrix.jl:1-41
LDSM = {
    "LDSM_U32x1_N": _ldsm("LDSM_U32x1_N", SL(((8, 4), 128), ((128, 0), 1)), SL((32, 32), (32, 1))),
    "LDSM_U32x2_N": _ldsm("LDSM_U32x2_N", SL(((16, 2), 128), ((128, 0), 1)),
                          SL((32, (32, 2)), (32, (1, 1024)))),
    "LDSM_U32x4_N": _ldsm("LDSM_U32x4_N", SL((32, 128), (128, 1)),
                          SL((32, (32, 4)), (32, (1, 1024)))),
    "LDSM_U16x2_T": _ldsm("LDSM_U16x2_T", SL(((8, 4), 128), ((128, 0), 1)),
                          SL(((4, 8), (16, 2)), ((256, 16), (1, 128)))),
    "LDSM_U16x4_T": _ldsm("LDSM_U16x4_T", SL(((16, 2), 128), ((128, 0), 1)),
                          SL(((4, 8), (16, 2, 2)), ((256, 16), (1, 128, 1024)))),
    "LDSM_U16x8_T": _ldsm("LDSM_U16x8_T", SL((32, 128), (128, 1)),
                          SL(((4, 8), (16, 2, 4)), ((256, 16), (1, 128, 1024)))),
}


class CopyAtom:
    """atom/copy.jl:3-59."""

    def __init__(self, traits, val_bits):
        self.traits = traits
        b = S(val_bits)
        self.val_layout_src = upcast(traits.srclayout, b)
        self.val_layout_dst = upcast(traits.dstlayout, b)
        self.val_layout_ref = upcast(traits.reflayout, b)
        n = size(traits.threadid)
        assert size(self.val_layout_src, 1) == n
        assert size(self.val_layout_dst, 1) == n
        assert size(self.val_layout_ref, 1) == n
        self.num_val_src = size(self.val_layout_src, 2)
        self.num_val_dst = size(self.val_layout_dst, 2)


class TiledCopy:
    """atom/copy.jl:86-125."""

    def __init__(self, atom, layout_tv, tiler_mn):
        assert int(size(layout_tv, 1)) % int(size(atom.val_layout_ref, 1)) == 0
        assert int(size(layout_tv, 2)) % int(size(atom.val_layout_ref, 2)) == 0
        self.copy_atom, self.tiled_layout_TV, self.tiler_MN = atom, layout_tv, tiler_mn

    def size(self):
        return size(self.tiled_layout_TV, 1)

    def tile2thrfrg(self, x, ref2trg):
        """atom/copy.jl:127-135."""
        ref = self.copy_atom.val_layout_ref
        atom_tv = zipped_divide(self.tiled_layout_TV, (size(ref, 1), size(ref, 2)))
        trg_tv = composition(atom_tv, (ref2trg, COLON))
        thrval2mn = coalesce(lzip(trg_tv), (_1, (_1, _1)))
        tv_array = composition(x, (thrval2mn, COLON))
        return tv_array(((COLON, COLON), COLON))

    def tidfrg_S(self, src):
        """atom/copy.jl:137-142."""
        a = self.copy_atom
        return self.tile2thrfrg(zipped_divide(src, self.tiler_MN),
                                composition(right_inverse(a.val_layout_ref), a.val_layout_src))

    def tidfrg_D(self, dst):
        """atom/copy.jl:144-149."""
        a = self.copy_atom
        return self.tile2thrfrg(zipped_divide(dst, self.tiler_MN),
                                composition(right_inverse(a.val_layout_ref), a.val_layout_dst))

    def get_layoutS_TV(self):
        """atom/copy.jl:168-173."""
        a = self.copy_atom
        ref = make_layout((self.tiler_MN, _1))
        return self.tile2thrfrg(ref, composition(right_inverse(a.val_layout_ref),
                                                 a.val_layout_src))((COLON, COLON, _1))

    def get_layoutD_TV(self):
        """atom/copy.jl:181-186."""
        a = self.copy_atom
        ref = make_layout((self.tiler_MN, _1))
        return self.tile2thrfrg(ref, composition(right_inverse(a.val_layout_ref),
                                                 a.val_layout_dst))((COLON, COLON, _1))

    def get_layoutS_MN(self):
        """atom/copy.jl:175-179."""
        return (composition(right_inverse(self.get_layoutS_TV()), make_layout(self.tiler_MN)),
                make_layout(size(self.tiled_layout_TV, 1)))

    def get_layoutD_MN(self):
        """atom/copy.jl:188-192."""
        return (composition(right_inverse(self.get_layoutD_TV()), make_layout(self.tiler_MN)),
                make_layout(size(self.tiled_layout_TV, 1)))

    def get_slice(self, thr_idx):
        return ThrCopy(self, thr_idx)

    def retile(self, x):
        """atom/copy.jl:151-166."""
        v = size(x, 1)
        tv = self.tiled_layout_TV
        shape_mn = self.tiler_MN
        atom_num_val = size(self.copy_atom.val_layout_ref, 2)
        num_thr = size(tv, 1)
        frg_mn = upcast(composition(right_inverse(tv), make_layout(shape_mn)), num_thr * v)
        frg_v = zipped_divide(logical_product(make_layout(v), right_inverse(frg_mn)),
                              make_layout(atom_num_val))
        t_array = zipped_divide(x, prepend(product_each(frg_mn.shape), v))
        v_array = composition(t_array, (frg_v, COLON))
        return v_array((COLON, append(_1, COLON, lrank(x))))


class ThrCopy:
    """atom/copy.jl:198-214."""

    def __init__(self, tiled_copy, thr_idx):
        self.tiled_copy, self.thr_idx = tiled_copy, thr_idx

    def partition_S(self, s):
        t = Array(s.buf, self.tiled_copy.tidfrg_S(s.layout), s.offset, s.memspace)
        return view(t, self.thr_idx, COLON, repeat(COLON, lrank(s.layout)))

    def partition_D(self, d):
        t = Array(d.buf, self.tiled_copy.tidfrg_D(d.layout), d.offset, d.memspace)
        return view(t, self.thr_idx, COLON, repeat(COLON, lrank(d.layout)))

    def retile_S(self, s):
        return Array(s.buf, self.tiled_copy.retile(s.layout), s.offset, s.memspace)

    retile_D = retile_S


def make_tiled_copy(atom, thr_layout, val_layout=None):
    """atom/copy.jl:249-258."""
    val_layout = val_layout if val_layout is not None else SL(1)
    layout_mn = raked_product(thr_layout, val_layout, True)
    layout_tv = composition(right_inverse(layout_mn),
                            make_layout((size(thr_layout), size(val_layout))))
    tiler = product_each(layout_mn.shape)
    return TiledCopy(atom, layout_tv, tiler)


def make_tiled_copy_A(atom, tiled_mma):
    """atom/copy.jl:227-230."""
    return TiledCopy(atom, tiled_mma.get_layoutA_TV(), (tiled_mma.tile_size(1), tiled_mma.tile_size(3)))


def make_tiled_copy_B(atom, tiled_mma):
    """atom/copy.jl:231-235."""
    return TiledCopy(atom, tiled_mma.get_layoutB_TV(), (tiled_mma.tile_size(2), tiled_mma.tile_size(3)))


def make_tiled_copy_C(atom, tiled_mma):
    """atom/copy.jl:236-240."""
    return TiledCopy(atom, tiled_mma.get_layoutC_TV(), (tiled_mma.tile_size(1), tiled_mma.tile_size(2)))


# --------------------------------------------------------------------------
# the loops: copyto! and gemm!
# --------------------------------------------------------------------------


def _convert(v, dtype):
    """arch/copy/copy.jl:38-43 — Julia `convert`: round to nearest even."""
    return np.asarray(v).astype(dtype)


def copyto(dst, src, tiled_copy=None):
    """algorithm/copy.jl:42-64 (plain) and :106-130 (with a copy atom).

    Logical element i of src goes to logical element i of dst through both layouts;
    bit-exact when the types agree, `convert` otherwise.  With a copy atom the value
    mode must hold a whole number of atom values (traits/copy.jl:33-36).
    """
    n = len(src)
    if len(dst) != n:
        raise ValueError("copyto!: size mismatch %d vs %d" % (len(dst), n))
    if tiled_copy is not None:
        atom = tiled_copy.copy_atom if hasattr(tiled_copy, "copy_atom") else tiled_copy
        assert int(size(src.layout, 1)) % int(atom.num_val_src) == 0
        assert int(size(dst.layout, 1)) % int(atom.num_val_dst) == 0
    so, do = src.offsets(), dst.offsets()
    vals = src.buf[so]
    if dst.dtype != src.dtype:
        vals = _convert(vals, dst.dtype)
    dst.buf[do] = vals
    return dst


def copyto_if(dst, src, mask):
    """algorithm/copy.jl:4-16: as copyto!, but logical element i moves only where mask(i) is true.  `mask` is an
    Array of bytes with its own layout (the reference takes any callable of the 1-based linear index)."""
    n = len(src)
    if len(dst) != n or len(mask) != n:
        raise ValueError("copyto_if!: size mismatch")
    so, do, mo = src.offsets(), dst.offsets(), mask.offsets()
    keep = mask.buf[mo] != 0
    vals = src.buf[so][keep]
    if dst.dtype != src.dtype:
        vals = _convert(vals, dst.dtype)
    dst.buf[do[keep]] = vals
    return dst


def round_bf16(x32):
    """fp32 -> bf16 (kept in fp32 storage), round to nearest even; NaN stays NaN."""
    x32 = np.asarray(x32, dtype=np.float32)
    u = x32.view(np.uint32).astype(np.uint64)
    lsb = (u >> 16) & 1
    r = ((u + 0x7FFF + lsb) >> 16) << 16
    out = r.astype(np.uint32).view(np.float32)
    return np.where(np.isnan(x32), x32, out)


def _product_rounder(ta, tb):
    """arch/mma/mma.jl:64 — `a .* b` is rounded in promote_type(TA, TB) before the add."""
    if ta == "f16" and tb == "f16":
        return lambda p: p.astype(np.float16).astype(np.float32)
    if ta == "bf16" and tb == "bf16":
        return round_bf16
    return lambda p: p


def gemm_universal_fma(A, B, C, ta="f32", tb="f32"):
    """algorithm/blas.jl:11-88 with UniversalFMA (arch/mma/mma.jl:64).

    A:(M,K), B:(N,K), C:(M,N) are fp32 ndarrays holding values representable in
    ta/tb.  k runs outermost and ascending, every C element is the strict
    left-to-right sum  c = fl32(round_T(a*b) + c), never fused.  The m/n visiting
    order (serpentine in blas.jl:63-67) does not affect any single element.
    """
    A = np.asarray(A, dtype=np.float32)
    B = np.asarray(B, dtype=np.float32)
    C = np.array(C, dtype=np.float32, copy=True)
    rnd = _product_rounder(ta, tb)
    for k in range(A.shape[1]):
        p = np.multiply.outer(A[:, k], B[:, k]).astype(np.float32)
        C = (rnd(p) + C).astype(np.float32)
    return C


def gemm_arrays(D, A, B, C):
    """blas.jl:39-88 over oracle Arrays of rank 2: D = A*B' + C, element by element."""
    m, n = int(size(C.layout, 1)), int(size(C.layout, 2))
    k = int(size(A.layout, 2))
    assert int(size(A.layout, 1)) == m and int(size(B.layout, 1)) == n
    assert int(size(B.layout, 2)) == k
    for kk in range(1, k + 1):
        for nn in range(1, n + 1):
            for mi in range(1, m + 1):
                ms = mi if nn & 1 else m + 1 - mi
                a = np.float32(A[(ms, kk)])
                b = np.float32(B[(nn, kk)])
                c = np.float32(C[(ms, nn)])
                D[(ms, nn)] = np.float32(np.float32(a * b) + c)
    return D


def axpby(a, X, b, Y):
    """blas.jl:1-9 — y[i] = iszero(b) ? a*x[i] : a*x[i] + b*y[i] over the logical elements of both
    arrays, every operation rounded in the arrays' element type (numpy's float16 arithmetic computes in
    float32 and rounds after each operation, as Julia's does; bf16 arrays are float32 buffers holding
    bf16 values and are rounded with round_bf16)."""
    assert len(X) == len(Y)
    ox, oy = X.offsets(), Y.offsets()
    bf16 = getattr(Y, "bf16", False)
    if bf16:
        rnd = lambda v: round_bf16(np.asarray(v, dtype=np.float32))
        af, bf_ = rnd(np.float32(a)), rnd(np.float32(b))
        x, y = X.buf[ox].astype(np.float32), Y.buf[oy].astype(np.float32)
        ax = rnd(af * x)
        Y.buf[oy] = ax if bf_ == 0 else rnd(ax + rnd(bf_ * y))
        return Y
    T = Y.buf.dtype.type
    at, bt = T(a), T(b)
    x, y = X.buf[ox], Y.buf[oy]
    ax = (at * x).astype(T)
    Y.buf[oy] = ax if bt == 0 else (ax + (bt * y).astype(T)).astype(T)
    return Y


def _julia_max(x, y):
    """base/math.jl max(x::T, y::T): ifelse((y > x) | (signbit(y) < signbit(x)), ifelse(isnan(x), x, y), ifelse(isnan(y), y, x))."""
    with np.errstate(invalid="ignore"):
        cond = (y > x) | (np.signbit(y) < np.signbit(x))
    return np.where(cond, np.where(np.isnan(x), x, y), np.where(np.isnan(y), y, x))


def _julia_min(x, y):
    with np.errstate(invalid="ignore"):
        cond = (y < x) | (np.signbit(y) > np.signbit(x))
    return np.where(cond, np.where(np.isnan(x), x, y), np.where(np.isnan(y), y, x))


BROADCAST_OPS = {
    "identity": lambda x, y: x, "add": lambda x, y: x + y, "sub": lambda x, y: x - y, "mul": lambda x, y: x * y,
    "div": lambda x, y: x / y, "max": _julia_max, "min": _julia_min, "neg": lambda x, y: -x, "abs": lambda x, y: np.abs(x),
}


def broadcast(op, A, B=None, scalar=0.0, out=None):
    """src/broadcast.jl:5-41 — `op.(A, B)` for arrays with static layouts.  The result is an owning array with
    `make_layout_like(layout(A))` (broadcast.jl:27-31, `similar`) unless `out` is given (`out .= op.(A, B)`).  B
    may be an array with as many elements as A, an array spanning a leading group of A's modes (a lower-rank
    array: Julia repeats it over the trailing modes), or None (the second operand is `scalar`).  One operation
    per element, rounded in the element type (Float16 computes in Float32 and rounds, as numpy does; bf16
    arrays are float32 buffers holding bf16 values)."""
    f = BROADCAST_OPS[op]
    n = len(A)
    oa = A.offsets()
    bf16 = getattr(A, "bf16", False)
    T = np.float32 if bf16 else A.buf.dtype.type
    x = A.buf[oa].astype(T)
    if B is None:
        y = round_bf16(np.float32(scalar)) if bf16 else T(scalar)
    else:
        nb = len(B)
        shp = lflatten(A.layout).shape
        shp = [int(v) for v in shp] if isinstance(shp, tuple) else [int(shp)]
        assert nb in (n, 1) or nb in list(np.cumprod(shp)), "cannot broadcast %d elements over %s" % (nb, shp)
        y = B.buf[B.offsets()].astype(T)[np.arange(n) % nb]
    with np.errstate(all="ignore"):
        r = np.asarray(f(x, y)).astype(T)
    if bf16:
        r = round_bf16(r)
    if out is None:
        out = Array.undef(A.buf.dtype.type, make_layout_like(A.layout))
        if bf16:
            out.bf16 = True
    out.buf[out.offsets()] = r
    return out


def gemm_epilogue(acc, alpha, beta, C, op, operand, scalar, out):
    """What a user kernel of the reference does to its fp32 accumulator fragment after the k-loop, composed of the
    reference's own pieces: axpby!(alpha, acc, beta, c) (blas.jl:1-9; iszero(beta) leaves C out), one broadcast
    `op.(t, operand)` (broadcast.jl:5-41), and the conversion of copyto! into the result type (arch/copy/copy.jl:38-43,
    round to nearest even).  acc: (M,N) float32; C: (M,N) in the result type or None; operand: anything numpy
    broadcasts to (M,N) (float32, float16 or bf16-valued float32) or None for `scalar`; out: "f32" | "f16" | "bf16".
    Every intermediate is float32 and every operation is rounded on its own."""
    M, N = acc.shape
    lay = make_layout((M, N))
    X = Array(np.ascontiguousarray(acc, dtype=np.float32).reshape(-1, order="F").copy(), lay)
    c32 = np.zeros((M, N), np.float32) if C is None else np.asarray(C).astype(np.float32)
    Y = Array(c32.reshape(-1, order="F").copy(), lay)
    axpby(np.float32(alpha), X, np.float32(beta if C is not None else 0.0), Y)
    if op not in (None, "identity"):
        if operand is None:
            Y = broadcast(op, Y, None, scalar, out=Y)
        else:
            full = np.broadcast_to(np.asarray(operand).astype(np.float32), (M, N))
            Y = broadcast(op, Y, Array(full.reshape(-1, order="F").copy(), lay), out=Y)
    r = Y.buf.reshape(M, N, order="F")
    if out == "f16":
        with np.errstate(over="ignore"):
            return r.astype(np.float16)
    if out == "bf16":
        return round_bf16(r)
    return r


def fill(X, value):
    """array_algorithms.jl:158-164 — every logical element of X becomes `value` (converted to eltype)."""
    X.buf[X.offsets()] = X.buf.dtype.type(value)
    return X


def gemm_fp64(A, B):
    """The tolerance oracle: exact-input fp64 product A*B' of (M,K) and (N,K)."""
    return np.asarray(A, dtype=np.float64) @ np.asarray(B, dtype=np.float64).T


def relerr(c, c64):
    """Norm-wise relative error  max|C - C64| / max|C64|."""
    c64 = np.asarray(c64, dtype=np.float64)
    return float(np.max(np.abs(np.asarray(c, dtype=np.float64) - c64)) / np.max(np.abs(c64)))

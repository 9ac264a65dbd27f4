"""moye_hip — host-side mirror of MoYe.jl's API over libmoye_hip.so (gfx950 / MI355X).

`copyto_` and `gemm_` (on MoYeArray views; `device.copyto_` / `device.gemm_` on raw descriptors) are `Base.copyto!` (src/algorithm/copy.jl:42-46,106-110 of the
reference) and `gemm!` (src/algorithm/blas.jl:11-17) for device arrays; they flatten the
arrays' layouts into plain descriptors and hand them to the HIP library.  There is no other
code path: without the built library every call raises.
"""
from . import _lib
from ._lib import (BF16, COPY_LDS_TILED, COPY_UNIVERSAL, F8E4M3, F16, F32, F64, GEMM_NO_LDS_SWIZZLE,
                   GEMM_NO_XCD_SWIZZLE, MFMA_F32_16x16x4_F32, MFMA_F32_16x16x32_BF16, MFMA_F32_16x16x32_F16,
                   MFMA_F32_16x16x32_FP8, MFMA_F32_32x32x2_F32, MFMA_F32_32x32x16_BF16,
                   MFMA_F32_32x32x16_F16, MFMA_F32_32x32x16_FP8, MMA_UNIVERSAL_FMA, U8, U16, U32, U64, U128,
                   MoyeError, Tensor, TiledCopy, TiledMMA, check, lib, make_tensor)
from . import device
from .device import device_info, gemm_epilogue, gemm_ex_, gemm_noalloc_, gemm_release_workspace, mfma_ceiling, mma_atom_probe, tiled_copy_desc, tiled_mma_desc, time_copy, time_gemm, gemm_workspace_size, gemm_explain, parse_plan, version
from .layout import (COLON, GenColMajor, GenRowMajor, Int32, Layout, StaticInt, append, blocked_product, coalesce,
                     compact_col_major, compact_row_major, complement, composition, coord_to_index, cosize, depth,
                     flatten, index_to_coord, left_inverse, logical_divide, logical_product, make_fragment_like,
                     make_layout, make_ordered_layout, max_common_vector, prepend, raked_product, rank, recast,
                     right_inverse, shape_div, size, slice_and_offset, static, static_layout, tiled_divide,
                     tiled_product, zipped_divide, zipped_product, unflatten, group, tuple_append, tuple_prepend,
                     zip2_by, product_each, capacity, elem_scale, filter_zeros, colex_less, elem_less, increment,
                     coord_to_coord, iscompatible, tile_to_shape, make_layout_like, print_layout)
from .array import (axpby_, fill_, zeros_, map_, broadcast, CopyAtom, MoYeArray, ThrCopy, ThrMMA, TiledCopy as TiledCopyOp, TiledMMA as TiledMMAOp, copyto_, copyto_if_,
                    gemm_, local_partition, local_tile, make_tiled_copy, make_tiled_copy_A, make_tiled_copy_B,
                    make_tiled_copy_C, make_tiled_mma, transpose, view)

__all__ = [n for n in dir() if not n.startswith("_")]

// Host-side layout algebra of MoYe (src/int_tuple.jl, src/stride.jl, src/layout.jl,
// src/algorithm/tuple_algorithms.jl of the reference), in C++.  No GPU involved: these functions
// compute the tile and partition shapes that are flattened into the descriptors of moye_hip.h.
//
// Integers keep the reference's static/dynamic distinction (Static.StaticInt{N} vs Int): two
// static operands give a static result, anything mixed is dynamic, a static zero absorbs a
// product.  Static-ness drives coalescing (only static modes merge, layout.jl:454-458), compact
// strides (a static size-1 mode gets stride _0, stride.jl:173-174) and the divisibility assert
// of shape_div (int_tuple.jl:87-90).
#pragma once

#include <cstdint>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/moye_hip.h"

namespace moye {
namespace host {

struct Error : std::runtime_error {
    moye_status status;
    Error(moye_status st, const std::string& msg) : std::runtime_error(msg), status(st) {}
};

// A dynamic integer is an Int (64 bits) or an Int32 (`w32`; src/utilities.jl:1-11: IntType = Union{Int, StaticInt,
// Int32}).  Julia's promotion decides the type of a result: static with static stays static, a static operand takes the
// other's type (promote_rule(StaticInt, Int32) = Int32), Int32 with Int32 is Int32, anything with an Int is an Int.
// Int32 results wrap modulo 2^32 as Julia's do.  In text a dynamic Int32 carries the suffix `i32` ("5i32").
struct Int {
    int64_t v = 0;
    bool s = false;    // static
    bool w32 = false;  // dynamic Int32 (never set on a static integer)
    Int() = default;
    Int(int64_t v_, bool s_, bool w32_ = false) : v(w32_ && !s_ ? (int64_t)(int32_t)v_ : v_), s(s_), w32(w32_ && !s_) {}
};
inline Int S(int64_t v) { return Int(v, true); }
inline Int D(int64_t v) { return Int(v, false); }
inline Int D32(int64_t v) { return Int(v, false, true); }
// the result of an operation on a and b / on a alone, with value v
inline Int promoted(int64_t v, Int a, Int b) { return Int(v, a.s && b.s, (a.s || a.w32) && (b.s || b.w32)); }
inline Int same_type(Int a, int64_t v) { return Int(v, a.s, a.w32); }

// An IntTuple: a leaf integer, a colon (only inside coordinates and tiles) or a tuple of IntTuples.
struct IT {
    enum Kind { LEAF, TUPLE, COLON } kind = LEAF;
    Int leaf;
    std::vector<IT> items;
    IT() = default;
    IT(Int i) : kind(LEAF), leaf(i) {}
    static IT tuple(std::vector<IT> v) {
        IT t;
        t.kind = TUPLE;
        t.items = std::move(v);
        return t;
    }
    static IT colon() {
        IT t;
        t.kind = COLON;
        return t;
    }
    bool is_tuple() const { return kind == TUPLE; }
    bool is_leaf() const { return kind == LEAF; }
    bool is_colon() const { return kind == COLON; }
    size_t size() const { return items.size(); }
    const IT& operator[](size_t i) const { return items[i]; }
};

struct Layout {
    IT shape, stride;
};

// A tile argument (src/layout.jl:64-67): a layout, an int, a colon, or a tuple of tiles.
struct Tile {
    enum Kind { LAYOUT, INT, COLON, TUPLE } kind = COLON;
    Layout layout;
    Int value;
    std::vector<Tile> items;
};

// ---- text ------------------------------------------------------------------------------------
IT parse_int_tuple(const std::string& text);
Layout parse_layout(const std::string& text);   // a bare shape gives the compact col-major layout
Tile parse_tile(const std::string& text);
std::string to_string(const IT& t);
std::string to_string(const Layout& l);

// ---- IntTuple (src/int_tuple.jl, src/algorithm/tuple_algorithms.jl) ---------------------------
int rank(const IT& t);
int depth(const IT& t);
Int product(const IT& t);
IT flatten(const IT& t);                 // an int stays an int
std::vector<Int> flat_leaves(const IT& t);
IT shape_div(const IT& a, const IT& b);
IT slice(const IT& a, const IT& index);
IT dice(const IT& a, const IT& index);
bool is_static(const IT& t);
bool iscompatible(const IT& a, const IT& b);
bool equal_values(const IT& a, const IT& b);

// ---- coordinates (src/stride.jl) ----------------------------------------------------------------
Int coord_to_index(const IT& coord, const IT& shape, const IT& stride);  // 1-based
Int coord_to_index_default(const IT& coord, const IT& shape);
IT index_to_coord(Int index, const IT& shape, const IT& stride);
IT compact_col_major(const IT& shape, Int current = S(1));
IT compact_row_major(const IT& shape, Int current = S(1));
IT compact_order(const IT& shape, const IT& order);

// ---- Layout (src/layout.jl) ----------------------------------------------------------------------
Layout make_layout(const IT& shape);
Layout make_layout(const IT& shape, const IT& stride);
Layout concat(const std::vector<Layout>& ls);
Layout mode(const Layout& l, int i);      // 1-based sub-layout
int rank(const Layout& l);
Int size(const Layout& l);
Int size(const Layout& l, int i);
Int cosize(const Layout& l);
Int eval(const Layout& l, const IT& coord);
Layout flatten(const Layout& l);
Layout coalesce(const Layout& l);
Layout coalesce(const Layout& l, const IT& profile);
Layout filter(const Layout& l);
Layout composition(const Layout& lhs, const Tile& rhs);
Layout composition(const Layout& lhs, const Layout& rhs);
Layout complement(const Layout& l, Int cotarget);
Layout complement(const Layout& l);
Layout right_inverse(const Layout& l);
Layout left_inverse(const Layout& l);
Int max_common_vector(const Layout& a, const Layout& b);
Layout logical_product(const Layout& l, const Tile& tile);
Layout zipped_product(const Layout& l, const Tile& tile);
Layout tiled_product(const Layout& l, const Tile& tile);
Layout blocked_product(const Layout& block, const Layout& l, bool coalesce_result);
Layout raked_product(const Layout& block, const Layout& l, bool coalesce_result);
Layout logical_divide(const Layout& l, const Tile& tile);
Layout zipped_divide(const Layout& l, const Tile& tile);
Layout tiled_divide(const Layout& l, const Tile& tile);
Layout upcast(const Layout& l, int64_t n);
Layout downcast(const Layout& l, int64_t n);
Layout recast(const Layout& l, int new_bytes, int old_bytes);
Layout append(const Layout& l, int n);    // pad with 1:0 modes to rank n
Layout prepend(const Layout& l, int n);
Layout make_ordered_layout(const IT& shape, const IT& order);
Layout make_fragment_like(const Layout& l);
Layout slice_layout(const Layout& l, const IT& coord);
Layout slice_and_offset(const Layout& l, const IT& coord, int64_t* offset);
Layout dice_layout(const Layout& l, const IT& coord);
IT get_congr_coord(const Layout& l, Int index);
Layout zip(const Layout& a, const Layout& b);
Layout zip(const Layout& a);
Layout transpose(const Layout& l);
Tile tile_of(const Layout& l);
Tile tile_of(Int v);
Tile tile_colon();
Tile tile_tuple(std::vector<Tile> v);
Tile tile_from_shape(const IT& t);        // ints -> by-mode tiler of ints

// ---- tiling verbs on layouts (src/algorithm/array_algorithms.jl) ----------------------------------
Layout local_tile(const Layout& l, const Tile& tile, const IT& coord, const IT* proj, int64_t* offset);

// more IntTuple helpers (src/algorithm/tuple_algorithms.jl, src/int_tuple.jl, src/stride.jl)
IT unflatten(const IT& flat, const IT& target);
IT group(const IT& t, int b, int e);
IT append_value(const IT& t, const IT& val, int n);    // n < 0: append once
IT prepend_value(const IT& t, const IT& val, int n);
IT zip2_by(const IT& t, const IT& guide);
IT product_each(const IT& t);
IT elem_scale(const IT& x, const IT& y);
IT filter_zeros(const IT& a, const IT& x);
bool colex_less(const IT& a, const IT& b);
bool elem_less(const IT& a, const IT& b);
IT increment(const IT& coord, const IT& shape);
IT coord_to_coord(const IT& coord, const IT& src_shape, const IT& dst_shape);
Layout tile_to_shape(const Layout& l, const IT& trg_shape, const IT* order);  // order null = GenColMajor
Layout make_layout_like(const Layout& l);
Layout local_partition(const Layout& l, const Tile& tile, const IT& coord_or_index, const IT* proj,
                       int64_t* offset);

}  // namespace host
}  // namespace moye

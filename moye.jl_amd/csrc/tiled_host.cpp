// Host-side TiledMMA / TiledCopy descriptors (src/atom/mma.jl, src/atom/copy.jl, src/traits/*.jl of
// the reference) on top of the layout algebra, and their C entry points.
#include <cstring>
#include <map>

#include "layout_host.hpp"
#include "moye_common.hpp"

namespace moye {
namespace host {

namespace {
[[noreturn]] void raise(moye_status st, const std::string& m) { throw Error(st, m); }
IT SI(int64_t v) { return IT(S(v)); }
IT tup(std::vector<IT> v) { return IT::tuple(std::move(v)); }
Layout L(const char* text) { return parse_layout(text); }
IT colons(int n) { return IT::tuple(std::vector<IT>((size_t)n, IT::colon())); }
}  // namespace

// An MMA atom: shape, thread-id layout and the (thr, val) -> tile-index layouts of A, B, C
// (src/traits/mma.jl:26-42).
struct MMAAtomDesc {
    std::string name;
    int64_t m, n, k;
    Layout thr_id, layout_a, layout_b, layout_c;
};

static const std::map<std::string, MMAAtomDesc>& atoms() {
    static const std::map<std::string, MMAAtomDesc> table = [] {
        std::map<std::string, MMAAtomDesc> t;
        auto add = [&](const char* name, int64_t m, int64_t n, int64_t k, const char* thr, const char* a,
                       const char* b, const char* c) {
            t[name] = MMAAtomDesc{name, m, n, k, L(thr), L(a), L(b), L(c)};
        };
        // src/traits/mma.jl:38-42
        add("UniversalFMA", 1, 1, 1, "_1:_0", "(_1,_1):(_0,_0)", "(_1,_1):(_0,_0)", "(_1,_1):(_0,_0)");
        // gfx950 MFMA, one 64-lane wave.  A 16x16xK atom: lane l holds A[l%16][8(l/16)..+7],
        // B[l%16][same k], D[4(l/16)+r][l%16]; a 32x32xK atom: A[l%32][8(l/32)..+7],
        // D[8(r/4)+4(l/32)+r%4][l%32].  Indices are 1-based column-major into (M,K)/(N,K)/(M,N).
        const char* a16 = "((_16,_4),_8):((_1,_128),_16)";
        const char* c16 = "((_16,_4),_4):((_16,_4),_1)";
        const char* a32 = "((_32,_2),_8):((_1,_256),_32)";
        const char* c32 = "((_32,_2),(_4,_4)):((_32,_4),(_1,_8))";
        for (const char* ty : {"F16", "BF16", "FP8"}) {
            add((std::string("MFMA_F32_16x16x32_") + ty).c_str(), 16, 16, 32, "_64:_1", a16, a16, c16);
            add((std::string("MFMA_F32_32x32x16_") + ty).c_str(), 32, 32, 16, "_64:_1", a32, a32, c32);
        }
        add("MFMA_F32_16x16x4_F32", 16, 16, 4, "_64:_1", "((_16,_4),_1):((_1,_16),_0)", "((_16,_4),_1):((_1,_16),_0)", c16);
        add("MFMA_F32_32x32x2_F32", 32, 32, 2, "_64:_1", "((_32,_2),_1):((_1,_32),_0)", "((_32,_2),_1):((_1,_32),_0)", c32);
        // the reference's NVIDIA atoms its tests and docstrings are written against, kept as data
        // (src/traits/mma_sm70.jl:1-25, mma_sm80.jl:1-115)
        add("MMAOP_8x8x4_F32F16F16F32_NT", 8, 8, 4, "(_4,_2):(_1,_16)", "((_4,_2),_4):((_8,_4),_1)",
            "((_4,_2),_4):((_8,_4),_1)", "((_2,_2,_2),(_2,_2,_2)):((_1,_16,_4),(_8,_2,_32))");
        add("MMAOP_16x8x8_F16F16F16F16_TN", 16, 8, 8, "_32:_1", "((_4,_8),(_2,_2)):((_32,_1),(_16,_8))",
            "((_4,_8),_2):((_16,_1),_8)", "((_4,_8),(_2,_2)):((_32,_1),(_16,_8))");
        add("MMAOP_16x8x16_F16F16F16F16_TN", 16, 8, 16, "_32:_1", "((_4,_8),(_2,_2,_2)):((_32,_1),(_16,_8,_128))",
            "((_4,_8),(_2,_2)):((_16,_1),(_8,_64))", "((_4,_8),(_2,_2)):((_32,_1),(_16,_8))");
        add("MMAOP_16x8x8_F32TF32TF32F32_TN", 16, 8, 8, "_32:_1", "((_4,_8),(_2,_2)):((_16,_1),(_8,_64))",
            "((_4,_8),_2):((_8,_1),_32)", "((_4,_8),(_2,_2)):((_32,_1),(_16,_8))");
        return t;
    }();
    return table;
}

static const char* kAtomNames[] = {"UniversalFMA", "MFMA_F32_16x16x32_F16", "MFMA_F32_32x32x16_F16",
                                   "MFMA_F32_16x16x32_BF16", "MFMA_F32_32x32x16_BF16", "MFMA_F32_16x16x32_FP8",
                                   "MFMA_F32_32x32x16_FP8", "MFMA_F32_16x16x4_F32", "MFMA_F32_32x32x2_F32"};

static const MMAAtomDesc& find_atom(const std::string& name_in) {
    std::string name = name_in;
    // a moye_mma_atom number is accepted too
    if (!name.empty() && std::isdigit((unsigned char)name[0])) {
        const int id = std::atoi(name.c_str());
        if (id < 0 || id > MOYE_MFMA_F32_32x32x2_F32) raise(MOYE_ERR_UNSUPPORTED, "unknown MMA atom " + name);
        name = kAtomNames[id];
    }
    auto it = atoms().find(name);
    if (it == atoms().end()) raise(MOYE_ERR_UNSUPPORTED, "unknown MMA atom \"" + name + "\"");
    return it->second;
}

// TiledMMA (src/atom/mma.jl:80-199)
struct TiledMMAHost {
    const MMAAtomDesc* atom;
    Layout atom_layout_mnk;        // padded to rank 3 (atom/mma.jl:196)
    std::vector<Tile> permutation;  // padded to 3 with ':' (atom/mma.jl:197)

    TiledMMAHost(const MMAAtomDesc& a, const std::string& atom_layout, const std::string& perm) : atom(&a) {
        const Layout al = atom_layout.empty() ? L("(_1,_1,_1)") : parse_layout(atom_layout);
        atom_layout_mnk = append(al, 3);
        if (!perm.empty()) {
            const Tile p = parse_tile(perm);
            if (p.kind != Tile::TUPLE) raise(MOYE_ERR_ARG, "permutations must be a tile tuple <m, n, k>");
            permutation = p.items;
        }
        if (permutation.size() > 3) raise(MOYE_ERR_RANK, "permutations has more than 3 modes");
        while (permutation.size() < 3) permutation.push_back(tile_colon());
    }
    Layout thr_layout_vmnk() const {  // atom/mma.jl:115-118
        return tiled_product(atom->thr_id, tile_of(atom_layout_mnk));
    }
    Int tile_size(int i) const {  // atom/mma.jl:178-189, i = 1..3
        const int64_t mnk[3] = {atom->m, atom->n, atom->k};
        const Int core = Int(mnk[i - 1] * size(thr_layout_vmnk(), i + 1).v, true);
        const Tile& s = permutation[i - 1];
        if (s.kind == Tile::COLON) return core;
        const Int p = s.kind == Tile::LAYOUT ? size(s.layout) : s.value;
        return Int(std::max(core.v, p.v), core.s && p.s);
    }
    Layout thrfrg(const Layout& l, int i0, int i1, const Layout& tv, int j0, int j1) const {  // atom/mma.jl:120-169
        const Layout t = thr_layout_vmnk();
        const int64_t mnk[3] = {atom->m, atom->n, atom->k};
        const Layout t_array = logical_divide(l, tile_tuple({permutation[i0], permutation[i1]}));
        const Layout a_array = zipped_divide(
            t_array, tile_tuple({tile_of(make_layout(SI(mnk[i0]))), tile_of(make_layout(SI(mnk[i1])))}));
        const Layout tv_array = composition(a_array, tile_tuple({tile_of(tv), tile_colon()}));
        const Tile thr_tile = tile_tuple({tile_colon(), tile_tuple({tile_of(make_layout(IT(size(t, j0)))),
                                                                     tile_of(make_layout(IT(size(t, j1))))})});
        return zipped_divide(tv_array, thr_tile);
    }
    Layout thrfrg_C(const Layout& l) const { return thrfrg(l, 0, 1, atom->layout_c, 2, 3); }
    Layout thrfrg_A(const Layout& l) const { return thrfrg(l, 0, 2, atom->layout_a, 2, 4); }
    Layout thrfrg_B(const Layout& l) const { return thrfrg(l, 1, 2, atom->layout_b, 3, 4); }

    // partition_X of get_slice(thr_idx) (atom/mma.jl:171-175,292-308)
    Layout partition(char operand, const Layout& l, int64_t thr_idx, int64_t* offset) const {
        const IT v = get_congr_coord(thr_layout_vmnk(), D(thr_idx));
        Layout frg;
        IT coord;
        switch (operand) {
            case 'C': frg = thrfrg_C(l); coord = tup({v[0], tup({v[1], v[2]})}); break;
            case 'A': frg = thrfrg_A(l); coord = tup({v[0], tup({v[1], v[3]})}); break;
            case 'B': frg = thrfrg_B(l); coord = tup({v[0], tup({v[2], v[3]})}); break;
            default: raise(MOYE_ERR_ARG, "operand must be 'A', 'B' or 'C'");
        }
        const int nrest = rank(mode(mode(frg, 2), 2).shape);
        return slice_and_offset(frg, tup({coord, tup({IT::colon(), colons(nrest)})}), offset);
    }
    // get_layoutX_TV (atom/mma.jl:264-289)
    Layout layout_tv(char operand) const {
        const Layout t = thr_layout_vmnk();
        const Tile inv = tile_of(right_inverse(t));
        if (operand == 'C') {
            const Layout ref = make_layout(tup({IT(tile_size(1)), IT(tile_size(2))}));
            return composition(thrfrg_C(ref), tile_tuple({inv, tile_colon()}));
        }
        const IT mn = tup({IT(size(t, 2)), IT(size(t, 3))});
        if (operand == 'A') {
            const Layout ref = make_layout(tup({IT(tile_size(1)), IT(tile_size(3))}));
            const Tile atile = tile_tuple({tile_colon(), tile_tuple({tile_of(make_layout(mn, tup({SI(1), SI(0)}))), tile_colon()})});
            return composition(composition(thrfrg_A(ref), tile_tuple({atile, tile_colon()})), tile_tuple({inv, tile_colon()}));
        }
        const Layout ref = make_layout(tup({IT(tile_size(2)), IT(tile_size(3))}));
        const Tile btile = tile_tuple({tile_colon(), tile_tuple({tile_of(make_layout(mn, tup({SI(0), SI(1)}))), tile_colon()})});
        return composition(composition(thrfrg_B(ref), tile_tuple({btile, tile_colon()})), tile_tuple({inv, tile_colon()}));
    }
    // get_layoutC_MN / get_layoutA_MK / get_layoutB_NK (atom/mma.jl:235-262): cell of the tile -> index into the
    // (thr, val) fragment layout, and the layout from the thread part of that index to the thread index
    std::pair<Layout, Layout> layout_mn(char operand) const {
        const Layout t = thr_layout_vmnk();
        const IT c = IT::colon(), one = SI(1);
        switch (operand) {
            case 'C': {
                const Layout ref = make_layout(tup({IT(tile_size(1)), IT(tile_size(2))}));
                return {composition(right_inverse(thrfrg_C(ref)), ref), slice_layout(t, tup({c, c, c, one}))};
            }
            case 'A': {
                const Layout ref = make_layout(tup({IT(tile_size(1)), IT(tile_size(3))}));
                return {composition(right_inverse(thrfrg_A(ref)), ref), slice_layout(t, tup({c, c, one, c}))};
            }
            case 'B': {
                const Layout ref = make_layout(tup({IT(tile_size(2)), IT(tile_size(3))}));
                return {composition(right_inverse(thrfrg_B(ref)), ref), slice_layout(t, tup({c, one, c, c}))};
            }
            default: raise(MOYE_ERR_ARG, "operand must be 'A', 'B' or 'C'");
        }
    }
};

// The table print_typst draws for one operand (src/print.jl:64-71,220-228) as text: cell (m, n) holds
// "T<thr_idx>V<val_idx>" with val_idx, thr = fldmod1(layout_mn(m, n), size(thr_id)) and thr_idx = thr_id(thr), all
// 1-based.  `transposed` draws cell (n, m) at row m, as the reference does for B above C.
static std::string tv_table_text(const std::string& title, const Layout& layout_mn, const Layout& thr_id, bool transposed) {
    const int64_t nthr = size(thr_id).v;
    const int64_t d1 = size(layout_mn, 1).v, d2 = size(layout_mn, 2).v;
    const int64_t rows = transposed ? d2 : d1, cols = transposed ? d1 : d2;
    const int64_t nval = (size(layout_mn).v + nthr - 1) / nthr;
    const int w = (int)("T" + std::to_string(cosize(thr_id).v) + "V" + std::to_string(nval)).size() + 2;
    auto lpad = [](const std::string& t, int n) { return (int)t.size() >= n ? t : std::string((size_t)n - t.size(), ' ') + t; };
    std::string sep = "     ";
    for (int64_t n = 0; n < cols; ++n) sep += "+" + std::string((size_t)w, '-');
    sep += "+";
    std::string r = title + "\n     ";
    for (int64_t n = 1; n <= cols; ++n) r += "  " + lpad(std::to_string(n), w - 2) + " ";
    for (int64_t m = 1; m <= rows; ++m) {
        r += "\n" + sep + "\n" + lpad(std::to_string(m), 3) + "  ";
        for (int64_t n = 1; n <= cols; ++n) {
            const int64_t idx = eval(layout_mn, transposed ? tup({IT(D(n)), IT(D(m))}) : tup({IT(D(m)), IT(D(n))})).v - 1;
            const int64_t thr = eval(thr_id, IT(D(idx % nthr + 1))).v;
            r += "| " + lpad("T" + std::to_string(thr) + "V" + std::to_string(idx / nthr + 1), w - 2) + " ";
        }
        r += "|";
    }
    return r + "\n" + sep + "\n";
}

// CopyAtom + TiledCopy (src/atom/copy.jl:3-59,86-258) for UniversalCopy{S,D} over values of val_bits
struct TiledCopyHost {
    Layout val_src, val_dst, val_ref;  // (thr, val) value layouts of the atom
    Layout layout_tv;
    IT tiler;

    TiledCopyHost(int src_bits, int dst_bits, int val_bits, const Layout& thr, const Layout& val) {
        if (src_bits <= 0 || dst_bits <= 0 || val_bits <= 0) raise(MOYE_ERR_ARG, "bit widths must be positive");
        // traits/copy.jl:16-21: one thread, src/dst bit layouts (1, bits)
        const Layout bs = make_layout(tup({SI(1), SI(src_bits)})), bd = make_layout(tup({SI(1), SI(dst_bits)}));
        val_src = upcast(bs, val_bits);  // atom/copy.jl:35-37
        val_dst = upcast(bd, val_bits);
        val_ref = val_src;
        // make_tiled_copy (atom/copy.jl:249-258)
        const Layout layout_mn = raked_product(thr, val, true);
        layout_tv = composition(right_inverse(layout_mn), make_layout(tup({IT(size(thr)), IT(size(val))})));
        std::vector<IT> t;
        for (const IT& s : (layout_mn.shape.is_tuple() ? layout_mn.shape.items : std::vector<IT>{layout_mn.shape}))
            t.push_back(IT(product(s)));
        tiler = IT::tuple(t);
        // TiledCopy constructor asserts (atom/copy.jl:121-122)
        if (size(layout_tv, 1).v % size(val_ref, 1).v) raise(MOYE_ERR_SHAPE, "thread count is not a multiple of the atom's");
        if (size(layout_tv, 2).v % size(val_ref, 2).v)
            raise(MOYE_ERR_SHAPE, "values per thread (" + std::to_string(size(layout_tv, 2).v) +
                                      ") are not a multiple of the atom's " + std::to_string(size(val_ref, 2).v));
    }
    // TiledCopy(atom, layout_tv, tiler) (atom/copy.jl:113-125): what make_tiled_copy_A/B/C build from a
    // TiledMMA's layouts (atom/copy.jl:227-240)
    TiledCopyHost(int src_bits, int dst_bits, int val_bits, const Layout& tv, const IT& tiler_mn) {
        if (src_bits <= 0 || dst_bits <= 0 || val_bits <= 0) raise(MOYE_ERR_ARG, "bit widths must be positive");
        const Layout bs = make_layout(tup({SI(1), SI(src_bits)})), bd = make_layout(tup({SI(1), SI(dst_bits)}));
        val_src = upcast(bs, val_bits);
        val_dst = upcast(bd, val_bits);
        val_ref = val_src;
        layout_tv = tv;
        tiler = tiler_mn;
        if (rank(layout_tv) != 2) raise(MOYE_ERR_RANK, "layout_tv must have a thread and a value mode");
        if (size(layout_tv, 1).v % size(val_ref, 1).v) raise(MOYE_ERR_SHAPE, "thread count is not a multiple of the atom's");
        if (size(layout_tv, 2).v % size(val_ref, 2).v)
            raise(MOYE_ERR_SHAPE, "values per thread (" + std::to_string(size(layout_tv, 2).v) +
                                      ") are not a multiple of the atom's " + std::to_string(size(val_ref, 2).v));
    }
    Int num_val_src() const { return size(val_src, 2); }
    Int num_val_dst() const { return size(val_dst, 2); }

    Layout tile2thrfrg(const Layout& x, const Layout& ref2trg) const {  // atom/copy.jl:127-135
        const Layout atom_tv =
            zipped_divide(layout_tv, tile_tuple({tile_of(size(val_ref, 1)), tile_of(size(val_ref, 2))}));
        const Layout trg_tv = composition(atom_tv, tile_tuple({tile_of(ref2trg), tile_colon()}));
        const Layout thrval2mn = coalesce(zip(trg_tv), tup({SI(1), tup({SI(1), SI(1)})}));
        const Layout tv_array = composition(x, tile_tuple({tile_of(thrval2mn), tile_colon()}));
        return slice_layout(tv_array, tup({tup({IT::colon(), IT::colon()}), IT::colon()}));
    }
    Layout tidfrg(char which, const Layout& l) const {  // atom/copy.jl:137-149
        if (rank(l) < rank(tiler)) raise(MOYE_ERR_RANK, "The dimension is too small to be tiled.");
        const Layout& trg = which == 'S' ? val_src : val_dst;
        return tile2thrfrg(zipped_divide(l, tile_from_shape(tiler)), composition(right_inverse(val_ref), trg));
    }
    Layout layout_TV(char which) const {  // get_layoutS_TV / get_layoutD_TV, atom/copy.jl:168-187
        if (which != 'S' && which != 'D') raise(MOYE_ERR_ARG, "which must be 'S' or 'D'");
        const Layout& trg = which == 'S' ? val_src : val_dst;
        const Layout ref = make_layout(tup({tiler, SI(1)}));
        const Layout t = tile2thrfrg(ref, composition(right_inverse(val_ref), trg));
        return slice_layout(t, tup({IT::colon(), IT::colon(), SI(1)}));
    }
    // get_layoutS_MN / get_layoutD_MN (atom/copy.jl:175-179,188-192)
    std::pair<Layout, Layout> layout_MN(char which) const {
        return {composition(right_inverse(layout_TV(which)), make_layout(tiler)), make_layout(IT(size(layout_tv, 1)))};
    }
    std::string print() const {  // print_typst(tiled_copy), src/print.jl:337-345
        const auto s = layout_MN('S'), d = layout_MN('D');
        return tv_table_text("S " + to_string(tiler), s.first, s.second, false) + "\n" +
               tv_table_text("D " + to_string(tiler), d.first, d.second, false);
    }
    Layout retile(const Layout& x) const {  // atom/copy.jl:151-166
        const Int v = size(x, 1);
        const Int atom_num_val = size(val_ref, 2);
        const Int num_thr = size(layout_tv, 1);
        const Layout frg_mn = upcast(composition(right_inverse(layout_tv), make_layout(tiler)), num_thr.v * v.v);
        const Layout frg_v = zipped_divide(logical_product(make_layout(IT(v)), tile_of(right_inverse(frg_mn))),
                                           tile_of(make_layout(IT(atom_num_val))));
        std::vector<Tile> by_mode{tile_of(v)};
        for (const IT& e : product_each(frg_mn.shape).items) by_mode.push_back(tile_of(e.leaf));
        const Layout t_array = zipped_divide(x, tile_tuple(by_mode));
        const Layout v_array = composition(t_array, tile_tuple({tile_of(frg_v), tile_colon()}));
        std::vector<IT> rest{SI(1)};
        for (int i = 1; i < rank(x); ++i) rest.push_back(IT::colon());
        return slice_layout(v_array, tup({IT::colon(), IT::tuple(rest)}));
    }
    Layout partition(char which, const Layout& l, int64_t thr_idx, int64_t* offset) const {  // atom/copy.jl:206-214
        if (which != 'S' && which != 'D') raise(MOYE_ERR_ARG, "which must be 'S' or 'D'");
        const Layout t = tidfrg(which, l);
        return slice_and_offset(t, tup({IT(D(thr_idx)), IT::colon(), colons(rank(l))}), offset);
    }
};

}  // namespace host
}  // namespace moye

// ------------------------------------------------------------------------------------------------
// C entry points
// ------------------------------------------------------------------------------------------------
using namespace moye;
using namespace moye::host;

namespace {
int32_t put(const std::string& s, char* out, size_t cap) {
    if (!out || cap == 0) return fail(MOYE_ERR_ARG, "null output buffer");
    if (s.size() + 1 > cap) return fail(MOYE_ERR_BUFFER, "output needs %zu bytes, buffer has %zu", s.size() + 1, cap);
    std::memcpy(out, s.c_str(), s.size() + 1);
    return MOYE_OK;
}
const char* nz(const char* s) { return s ? s : ""; }
int64_t leaf_of_text(const std::string& t) {
    const IT v = parse_int_tuple(t);
    if (!v.is_leaf()) throw Error(MOYE_ERR_ARG, "expected an integer, got " + t);
    return v.leaf.v;
}

template <typename F>
int32_t guarded(F&& f) {
    try {
        return f();
    } catch (const Error& e) {
        return fail(e.status, "%s", e.what());
    } catch (const std::exception& e) {
        return fail(MOYE_ERR_ARG, "%s", e.what());
    }
}
#define MOYE_REQUIRE(p) \
    if (!(p)) return fail(MOYE_ERR_ARG, "null argument: %s", #p)
}  // namespace


// ---------------------------------------------------------------------------------------------
// One-wave probe of an MFMA atom: every lane gathers its A and B fragment values through the
// atom's (thr, val) -> tile-index tables above, the wave executes the instruction once on a zero
// accumulator, and every lane scatters its D values through the C table.  If the tables describe
// the hardware, D = A * B' for any input; they are what partition_A/B/C hand to callers
// (src/atom/mma.jl:292-308), so this is their known-answer test on the machine itself.
// ---------------------------------------------------------------------------------------------
namespace {
typedef float probe_f32x4 __attribute__((ext_vector_type(4)));
typedef float probe_f32x16 __attribute__((ext_vector_type(16)));
typedef _Float16 probe_f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 probe_bf16x8 __attribute__((ext_vector_type(8)));

template <int ATOM>
__global__ __launch_bounds__(64) void mma_atom_probe_kernel(const void* A, const void* B, float* D, const int* ai,
                                                            const int* bi, const int* ci) {
    const int lane = threadIdx.x;
    constexpr bool k32 = ATOM == MOYE_MFMA_F32_32x32x16_F16 || ATOM == MOYE_MFMA_F32_32x32x16_BF16 ||
                         ATOM == MOYE_MFMA_F32_32x32x16_FP8 || ATOM == MOYE_MFMA_F32_32x32x2_F32;
    constexpr int VC = k32 ? 16 : 4;
    float out[VC];
    if constexpr (ATOM == MOYE_MFMA_F32_16x16x4_F32 || ATOM == MOYE_MFMA_F32_32x32x2_F32) {
        const float a = static_cast<const float*>(A)[ai[lane]], b = static_cast<const float*>(B)[bi[lane]];
        if constexpr (k32) {
            probe_f32x16 c = {};
            c = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
            for (int v = 0; v < VC; ++v) out[v] = c[v];
        } else {
            probe_f32x4 c = {};
            c = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
            for (int v = 0; v < VC; ++v) out[v] = c[v];
        }
    } else if constexpr (ATOM == MOYE_MFMA_F32_16x16x32_FP8 || ATOM == MOYE_MFMA_F32_32x32x16_FP8) {
        uint64_t a = 0, b = 0;
        for (int v = 0; v < 8; ++v) {
            a |= (uint64_t)static_cast<const uint8_t*>(A)[ai[lane * 8 + v]] << (8 * v);
            b |= (uint64_t)static_cast<const uint8_t*>(B)[bi[lane * 8 + v]] << (8 * v);
        }
        if constexpr (k32) {
            probe_f32x16 c = {};
            c = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8((long)a, (long)b, c, 0, 0, 0);
            for (int v = 0; v < VC; ++v) out[v] = c[v];
        } else {
            probe_f32x4 c = {};
            c = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8((long)a, (long)b, c, 0, 0, 0);
            for (int v = 0; v < VC; ++v) out[v] = c[v];
        }
    } else {
        uint16_t a[8], b[8];
        for (int v = 0; v < 8; ++v) {
            a[v] = static_cast<const uint16_t*>(A)[ai[lane * 8 + v]];
            b[v] = static_cast<const uint16_t*>(B)[bi[lane * 8 + v]];
        }
        if constexpr (ATOM == MOYE_MFMA_F32_16x16x32_F16 || ATOM == MOYE_MFMA_F32_32x32x16_F16) {
            probe_f16x8 fa, fb;
            __builtin_memcpy(&fa, a, 16);
            __builtin_memcpy(&fb, b, 16);
            if constexpr (k32) {
                probe_f32x16 c = {};
                c = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa, fb, c, 0, 0, 0);
                for (int v = 0; v < VC; ++v) out[v] = c[v];
            } else {
                probe_f32x4 c = {};
                c = __builtin_amdgcn_mfma_f32_16x16x32_f16(fa, fb, c, 0, 0, 0);
                for (int v = 0; v < VC; ++v) out[v] = c[v];
            }
        } else {
            probe_bf16x8 fa, fb;
            __builtin_memcpy(&fa, a, 16);
            __builtin_memcpy(&fb, b, 16);
            if constexpr (k32) {
                probe_f32x16 c = {};
                c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa, fb, c, 0, 0, 0);
                for (int v = 0; v < VC; ++v) out[v] = c[v];
            } else {
                probe_f32x4 c = {};
                c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa, fb, c, 0, 0, 0);
                for (int v = 0; v < VC; ++v) out[v] = c[v];
            }
        }
    }
    for (int v = 0; v < VC; ++v) D[ci[lane * VC + v]] = out[v];
}

// 0-based tile indices of every (lane, value) pair of a TV layout
std::vector<int> tv_table(const Layout& tv) {
    const int64_t nt = size(tv, 1).v, nv = size(tv, 2).v;
    std::vector<int> t((size_t)(nt * nv));
    for (int64_t l = 0; l < nt; ++l)
        for (int64_t v = 0; v < nv; ++v)
            t[(size_t)(l * nv + v)] = (int)(eval(tv, tup({IT(D(l + 1)), IT(D(v + 1))})).v - 1);
    return t;
}

int32_t mma_atom_probe_impl(int32_t atom, const void* A, const void* B, float* D, hipStream_t st) {
    if (atom < MOYE_MFMA_F32_16x16x32_F16 || atom > MOYE_MFMA_F32_32x32x2_F32)
        throw Error(MOYE_ERR_UNSUPPORTED, "moye_mma_atom_probe: not a hardware atom");
    const MMAAtomDesc& a = find_atom(std::to_string(atom));
    if (size(a.thr_id).v != 64) throw Error(MOYE_ERR_UNSUPPORTED, "moye_mma_atom_probe: atom is not one wave wide");
    const std::vector<int> ta = tv_table(a.layout_a), tb = tv_table(a.layout_b), tc = tv_table(a.layout_c);
    const size_t na = ta.size(), nb = tb.size(), nc = tc.size();
    int* dev = nullptr;
    MOYE_HIP_CHECK(hipMalloc(&dev, (na + nb + nc) * sizeof(int)));
    int32_t rc = MOYE_OK;
    auto copy = [&](int* d, const std::vector<int>& h) { return hipMemcpy(d, h.data(), h.size() * sizeof(int), hipMemcpyHostToDevice); };
    if (copy(dev, ta) != hipSuccess || copy(dev + na, tb) != hipSuccess || copy(dev + na + nb, tc) != hipSuccess) {
        rc = fail(MOYE_ERR_HIP, "moye_mma_atom_probe: table upload failed");
    } else {
        const int *ai = dev, *bi = dev + na, *ci = dev + na + nb;
        switch (atom) {
#define MOYE_PROBE_CASE(X) case X: mma_atom_probe_kernel<X><<<1, 64, 0, st>>>(A, B, D, ai, bi, ci); break;
            MOYE_PROBE_CASE(MOYE_MFMA_F32_16x16x32_F16)
            MOYE_PROBE_CASE(MOYE_MFMA_F32_32x32x16_F16)
            MOYE_PROBE_CASE(MOYE_MFMA_F32_16x16x32_BF16)
            MOYE_PROBE_CASE(MOYE_MFMA_F32_32x32x16_BF16)
            MOYE_PROBE_CASE(MOYE_MFMA_F32_16x16x32_FP8)
            MOYE_PROBE_CASE(MOYE_MFMA_F32_32x32x16_FP8)
            MOYE_PROBE_CASE(MOYE_MFMA_F32_16x16x4_F32)
            MOYE_PROBE_CASE(MOYE_MFMA_F32_32x32x2_F32)
#undef MOYE_PROBE_CASE
        }
        if (hipGetLastError() != hipSuccess || hipStreamSynchronize(st) != hipSuccess)
            rc = fail(MOYE_ERR_HIP, "moye_mma_atom_probe: launch failed");
    }
    (void)hipFree(dev);
    return rc;
}
}  // namespace

extern "C" {

int32_t moye_layout_normalize(const char* layout, char* out, size_t cap) {
    MOYE_REQUIRE(layout);
    return guarded([&] { return put(to_string(parse_layout(layout)), out, cap); });
}
int32_t moye_layout_eval(const char* layout, const char* coord, int64_t* index) {
    MOYE_REQUIRE(layout && coord && index);
    return guarded([&] {
        *index = eval(parse_layout(layout), parse_int_tuple(coord)).v;
        return (int32_t)MOYE_OK;
    });
}
int32_t moye_layout_eval_typed(const char* layout, const char* coord, char* out, size_t cap) {
    MOYE_REQUIRE(layout && coord && out);
    return guarded([&] { return put(to_string(IT(eval(parse_layout(layout), parse_int_tuple(coord)))), out, cap); });
}
int32_t moye_layout_size(const char* layout, int64_t* n) {
    MOYE_REQUIRE(layout && n);
    return guarded([&] {
        *n = size(parse_layout(layout)).v;
        return (int32_t)MOYE_OK;
    });
}
int32_t moye_layout_cosize(const char* layout, int64_t* n) {
    MOYE_REQUIRE(layout && n);
    return guarded([&] {
        *n = cosize(parse_layout(layout)).v;
        return (int32_t)MOYE_OK;
    });
}
int32_t moye_layout_rank_depth(const char* layout, int32_t* r, int32_t* d) {
    MOYE_REQUIRE(layout && r && d);
    return guarded([&] {
        const Layout l = parse_layout(layout);
        *r = rank(l);
        *d = depth(l.shape);
        return (int32_t)MOYE_OK;
    });
}
#define MOYE_UNARY(NAME, EXPR)                                                  \
    int32_t NAME(const char* layout, char* out, size_t cap) {                   \
        MOYE_REQUIRE(layout);                                                   \
        return guarded([&] {                                                    \
            const Layout l = parse_layout(layout);                              \
            return put(to_string(EXPR), out, cap);                              \
        });                                                                     \
    }
MOYE_UNARY(moye_layout_flatten, flatten(l))
MOYE_UNARY(moye_layout_coalesce, coalesce(l))
MOYE_UNARY(moye_layout_filter, filter(l))
MOYE_UNARY(moye_layout_right_inverse, right_inverse(l))
MOYE_UNARY(moye_layout_left_inverse, left_inverse(l))
MOYE_UNARY(moye_layout_make_fragment_like, make_fragment_like(l))
#undef MOYE_UNARY

#define MOYE_WITH_TILE(NAME, FN)                                                         \
    int32_t NAME(const char* layout, const char* tile, char* out, size_t cap) {          \
        MOYE_REQUIRE(layout && tile);                                                    \
        return guarded([&] {                                                             \
            return put(to_string(FN(parse_layout(layout), parse_tile(tile))), out, cap); \
        });                                                                              \
    }
MOYE_WITH_TILE(moye_layout_composition, composition)
MOYE_WITH_TILE(moye_layout_logical_product, logical_product)
MOYE_WITH_TILE(moye_layout_zipped_product, zipped_product)
MOYE_WITH_TILE(moye_layout_tiled_product, tiled_product)
MOYE_WITH_TILE(moye_layout_logical_divide, logical_divide)
MOYE_WITH_TILE(moye_layout_zipped_divide, zipped_divide)
MOYE_WITH_TILE(moye_layout_tiled_divide, tiled_divide)
#undef MOYE_WITH_TILE

int32_t moye_layout_complement(const char* layout, const char* cotarget, char* out, size_t cap) {
    MOYE_REQUIRE(layout);
    return guarded([&] {
        const Layout l = parse_layout(layout);
        const std::string c = nz(cotarget);
        if (c.empty()) return put(to_string(complement(l)), out, cap);
        const IT t = parse_int_tuple(c);
        if (!t.is_leaf()) throw Error(MOYE_ERR_ARG, "cotarget must be an integer");
        return put(to_string(complement(l, t.leaf)), out, cap);
    });
}
int32_t moye_layout_max_common_vector(const char* a, const char* b, int64_t* n) {
    MOYE_REQUIRE(a && b && n);
    return guarded([&] {
        *n = max_common_vector(parse_layout(a), parse_layout(b)).v;
        return (int32_t)MOYE_OK;
    });
}
int32_t moye_layout_blocked_product(const char* block, const char* layout, int32_t c, char* out, size_t cap) {
    MOYE_REQUIRE(block && layout);
    return guarded([&] { return put(to_string(blocked_product(parse_layout(block), parse_layout(layout), c != 0)), out, cap); });
}
int32_t moye_layout_raked_product(const char* block, const char* layout, int32_t c, char* out, size_t cap) {
    MOYE_REQUIRE(block && layout);
    return guarded([&] { return put(to_string(raked_product(parse_layout(block), parse_layout(layout), c != 0)), out, cap); });
}
int32_t moye_layout_recast(const char* layout, int32_t nb, int32_t ob, char* out, size_t cap) {
    MOYE_REQUIRE(layout);
    return guarded([&] { return put(to_string(recast(parse_layout(layout), nb, ob)), out, cap); });
}
int32_t moye_layout_append(const char* layout, int32_t r, char* out, size_t cap) {
    MOYE_REQUIRE(layout);
    return guarded([&] { return put(to_string(append(parse_layout(layout), r)), out, cap); });
}
int32_t moye_layout_prepend(const char* layout, int32_t r, char* out, size_t cap) {
    MOYE_REQUIRE(layout);
    return guarded([&] { return put(to_string(prepend(parse_layout(layout), r)), out, cap); });
}
int32_t moye_layout_make_ordered(const char* shape, const char* order, char* out, size_t cap) {
    MOYE_REQUIRE(shape && order);
    return guarded([&] { return put(to_string(make_ordered_layout(parse_int_tuple(shape), parse_int_tuple(order))), out, cap); });
}
int32_t moye_layout_make(const char* shape, int32_t row_major, char* out, size_t cap) {
    MOYE_REQUIRE(shape);
    return guarded([&] {
        const IT s = parse_int_tuple(shape);
        return put(to_string(Layout{s, row_major ? compact_row_major(s) : compact_col_major(s)}), out, cap);
    });
}
int32_t moye_layout_slice(const char* layout, const char* coord, char* out, size_t cap, int64_t* offset) {
    MOYE_REQUIRE(layout && coord);
    return guarded([&] { return put(to_string(slice_and_offset(parse_layout(layout), parse_int_tuple(coord), offset)), out, cap); });
}

// IntTuple / coordinate helpers by name
int32_t moye_tuple_op(const char* op_, const char* a_, const char* b_, const char* c_, char* out, size_t cap) {
    MOYE_REQUIRE(op_ && a_);
    return guarded([&] {
        const std::string op = op_, b = nz(b_), c = nz(c_);
        const IT a = parse_int_tuple(a_);
        auto B = [&] { return parse_int_tuple(b); };
        auto C = [&] { return parse_int_tuple(c); };
        if (op == "flatten") return put(to_string(flatten(a)), out, cap);
        if (op == "product" || op == "capacity") return put(to_string(IT(product(a))), out, cap);
        if (op == "rank") return put(std::to_string(rank(a)), out, cap);
        if (op == "depth") return put(std::to_string(depth(a)), out, cap);
        if (op == "shape_div") return put(to_string(shape_div(a, B())), out, cap);
        if (op == "slice") return put(to_string(slice(a, B())), out, cap);
        if (op == "dice") return put(to_string(dice(a, B())), out, cap);
        if (op == "compact_col_major") return put(to_string(compact_col_major(a)), out, cap);
        if (op == "compact_row_major") return put(to_string(compact_row_major(a)), out, cap);
        if (op == "compact_order") return put(to_string(compact_order(a, B())), out, cap);
        if (op == "coord_to_index")
            return put(to_string(IT(c.empty() ? coord_to_index_default(a, B()) : coord_to_index(a, B(), C()))), out, cap);
        if (op == "index_to_coord") {
            if (!a.is_leaf()) throw Error(MOYE_ERR_ARG, "index_to_coord takes an integer index");
            const IT shp = B();
            if (!c.empty()) {
                const IT st = C();
                if (shp.is_tuple() && st.is_tuple() && shp.size() != st.size())
                    throw Error(MOYE_ERR_RANK, "shape, and stride must have the same rank");
                return put(to_string(index_to_coord(a.leaf, shp, st)), out, cap);
            }
            return put(to_string(index_to_coord(a.leaf, shp, compact_col_major(shp))), out, cap);
        }
        if (op == "iscompatible") return put(iscompatible(a, B()) ? "true" : "false", out, cap);
        if (op == "unflatten") return put(to_string(unflatten(a, B())), out, cap);
        if (op == "group") return put(to_string(group(a, (int)leaf_of_text(b), (int)leaf_of_text(c))), out, cap);
        if (op == "append") return put(to_string(append_value(a, B(), c.empty() ? -1 : (int)leaf_of_text(c))), out, cap);
        if (op == "prepend") return put(to_string(prepend_value(a, B(), c.empty() ? -1 : (int)leaf_of_text(c))), out, cap);
        if (op == "zip2_by") return put(to_string(zip2_by(a, B())), out, cap);
        if (op == "product_each") return put(to_string(product_each(a)), out, cap);
        if (op == "elem_scale") return put(to_string(elem_scale(a, B())), out, cap);
        if (op == "filter_zeros") return put(to_string(filter_zeros(a, b.empty() ? a : B())), out, cap);
        if (op == "colex_less") return put(colex_less(a, B()) ? "true" : "false", out, cap);
        if (op == "elem_less") return put(elem_less(a, B()) ? "true" : "false", out, cap);
        if (op == "increment") return put(to_string(increment(a, B())), out, cap);
        if (op == "coord_to_coord") return put(to_string(coord_to_coord(a, B(), C())), out, cap);
        throw Error(MOYE_ERR_UNSUPPORTED, "unknown tuple op \"" + op + "\"");
    });
}

int32_t moye_local_tile(const char* layout, const char* tile, const char* coord, const char* proj, char* out, size_t cap,
                        int64_t* offset) {
    MOYE_REQUIRE(layout && tile && coord);
    return guarded([&] {
        const std::string pj = nz(proj);
        IT p;
        if (!pj.empty()) p = parse_int_tuple(pj);
        return put(to_string(local_tile(parse_layout(layout), parse_tile(tile), parse_int_tuple(coord),
                                        pj.empty() ? nullptr : &p, offset)),
                   out, cap);
    });
}
int32_t moye_local_partition(const char* layout, const char* thr_tile, const char* coord_or_index, const char* proj,
                             char* out, size_t cap, int64_t* offset) {
    MOYE_REQUIRE(layout && thr_tile && coord_or_index);
    return guarded([&] {
        const std::string pj = nz(proj);
        IT p;
        if (!pj.empty()) p = parse_int_tuple(pj);
        return put(to_string(local_partition(parse_layout(layout), parse_tile(thr_tile), parse_int_tuple(coord_or_index),
                                             pj.empty() ? nullptr : &p, offset)),
                   out, cap);
    });
}

int32_t moye_tiled_mma_query(const char* atom, const char* atom_layout, const char* permutation, const char* what_,
                             char* out, size_t cap) {
    MOYE_REQUIRE(atom && what_);
    return guarded([&] {
        const MMAAtomDesc& a = find_atom(atom);
        const TiledMMAHost m(a, nz(atom_layout), nz(permutation));
        const std::string what = what_;
        if (what == "thr_layout_vmnk") return put(to_string(m.thr_layout_vmnk()), out, cap);
        if (what == "tile_shape")
            return put(to_string(IT::tuple({IT(m.tile_size(1)), IT(m.tile_size(2)), IT(m.tile_size(3))})), out, cap);
        if (what == "size") return put(to_string(IT(size(m.thr_layout_vmnk()))), out, cap);
        if (what == "shape_mnk") return put(to_string(IT::tuple({IT(S(a.m)), IT(S(a.n)), IT(S(a.k))})), out, cap);
        if (what == "thr_id") return put(to_string(a.thr_id), out, cap);
        if (what == "layout_a") return put(to_string(a.layout_a), out, cap);
        if (what == "layout_b") return put(to_string(a.layout_b), out, cap);
        if (what == "layout_c") return put(to_string(a.layout_c), out, cap);
        if (what == "layoutA_TV") return put(to_string(m.layout_tv('A')), out, cap);
        if (what == "layoutB_TV") return put(to_string(m.layout_tv('B')), out, cap);
        if (what == "layoutC_TV") return put(to_string(m.layout_tv('C')), out, cap);
        if (what == "layoutA_MK") return put(to_string(m.layout_mn('A').first), out, cap);
        if (what == "layoutB_NK") return put(to_string(m.layout_mn('B').first), out, cap);
        if (what == "layoutC_MN") return put(to_string(m.layout_mn('C').first), out, cap);
        if (what == "thrID_A") return put(to_string(m.layout_mn('A').second), out, cap);
        if (what == "thrID_B") return put(to_string(m.layout_mn('B').second), out, cap);
        if (what == "thrID_C") return put(to_string(m.layout_mn('C').second), out, cap);
        if (what == "print") {  // print_typst(tiled_mma), src/print.jl:317-323: B drawn as (K, N), then A, then C
            const auto A = m.layout_mn('A'), B = m.layout_mn('B'), C = m.layout_mn('C');
            return put(tv_table_text("B (K, N)", B.first, B.second, true) + "\n" + tv_table_text("A (M, K)", A.first, A.second, false) +
                           "\n" + tv_table_text("C (M, N)", C.first, C.second, false), out, cap);
        }
        throw Error(MOYE_ERR_UNSUPPORTED, "unknown TiledMMA query \"" + what + "\"");
    });
}

int32_t moye_tiled_mma_partition(const char* atom, const char* atom_layout, const char* permutation, int32_t thr_idx,
                                 char operand, const char* layout, char* out, size_t cap, int64_t* offset) {
    MOYE_REQUIRE(atom && layout);
    return guarded([&] {
        const TiledMMAHost m(find_atom(atom), nz(atom_layout), nz(permutation));
        return put(to_string(m.partition(operand, parse_layout(layout), thr_idx, offset)), out, cap);
    });
}

int32_t moye_tiled_copy_query(int32_t src_bits, int32_t dst_bits, int32_t val_bits, const char* thr_layout,
                              const char* val_layout, const char* what_, char* out, size_t cap) {
    MOYE_REQUIRE(thr_layout && what_);
    return guarded([&] {
        const std::string vl = nz(val_layout);
        const TiledCopyHost tc(src_bits, dst_bits, val_bits, parse_layout(thr_layout), vl.empty() ? parse_layout("_1") : parse_layout(vl));
        const std::string what = what_;
        if (what == "layout_tv") return put(to_string(tc.layout_tv), out, cap);
        if (what == "layoutS_TV") return put(to_string(tc.layout_TV('S')), out, cap);
        if (what == "layoutD_TV") return put(to_string(tc.layout_TV('D')), out, cap);
        if (what == "layoutS_MN") return put(to_string(tc.layout_MN('S').first), out, cap);
        if (what == "layoutD_MN") return put(to_string(tc.layout_MN('D').first), out, cap);
        if (what == "print") return put(tc.print(), out, cap);
        if (what == "tiler") return put(to_string(tc.tiler), out, cap);
        if (what == "num_val_src") return put(to_string(IT(tc.num_val_src())), out, cap);
        if (what == "num_val_dst") return put(to_string(IT(tc.num_val_dst())), out, cap);
        if (what == "size") return put(to_string(IT(size(tc.layout_tv, 1))), out, cap);
        throw Error(MOYE_ERR_UNSUPPORTED, "unknown TiledCopy query \"" + what + "\"");
    });
}

int32_t moye_tiled_copy_partition(int32_t src_bits, int32_t dst_bits, int32_t val_bits, const char* thr_layout,
                                  const char* val_layout, int32_t thr_idx, char which, const char* layout, char* out,
                                  size_t cap, int64_t* offset) {
    MOYE_REQUIRE(thr_layout && layout);
    return guarded([&] {
        const std::string vl = nz(val_layout);
        const TiledCopyHost tc(src_bits, dst_bits, val_bits, parse_layout(thr_layout), vl.empty() ? parse_layout("_1") : parse_layout(vl));
        return put(to_string(tc.partition(which, parse_layout(layout), thr_idx, offset)), out, cap);
    });
}

int32_t moye_tiled_copy_tv_query(int32_t src_bits, int32_t dst_bits, int32_t val_bits, const char* layout_tv,
                                 const char* tiler, const char* what_, char* out, size_t cap) {
    MOYE_REQUIRE(layout_tv && tiler && what_);
    return guarded([&] {
        const TiledCopyHost tc(src_bits, dst_bits, val_bits, parse_layout(layout_tv), parse_int_tuple(tiler));
        const std::string what = what_;
        if (what == "layoutS_TV") return put(to_string(tc.layout_TV('S')), out, cap);
        if (what == "layoutD_TV") return put(to_string(tc.layout_TV('D')), out, cap);
        if (what == "layoutS_MN") return put(to_string(tc.layout_MN('S').first), out, cap);
        if (what == "layoutD_MN") return put(to_string(tc.layout_MN('D').first), out, cap);
        if (what == "print") return put(tc.print(), out, cap);
        if (what == "num_val_src") return put(to_string(IT(tc.num_val_src())), out, cap);
        if (what == "num_val_dst") return put(to_string(IT(tc.num_val_dst())), out, cap);
        if (what == "size") return put(to_string(IT(size(tc.layout_tv, 1))), out, cap);
        throw Error(MOYE_ERR_UNSUPPORTED, "unknown TiledCopy query \"" + what + "\"");
    });
}

int32_t moye_tiled_copy_tv_partition(int32_t src_bits, int32_t dst_bits, int32_t val_bits, const char* layout_tv,
                                     const char* tiler, int32_t thr_idx, char which, const char* layout, char* out,
                                     size_t cap, int64_t* offset) {
    MOYE_REQUIRE(layout_tv && tiler && layout);
    return guarded([&] {
        const TiledCopyHost tc(src_bits, dst_bits, val_bits, parse_layout(layout_tv), parse_int_tuple(tiler));
        return put(to_string(tc.partition(which, parse_layout(layout), thr_idx, offset)), out, cap);
    });
}

int32_t moye_tiled_copy_tv_retile(int32_t src_bits, int32_t dst_bits, int32_t val_bits, const char* layout_tv,
                                  const char* tiler, const char* layout, char* out, size_t cap) {
    MOYE_REQUIRE(layout_tv && tiler && layout);
    return guarded([&] {
        const TiledCopyHost tc(src_bits, dst_bits, val_bits, parse_layout(layout_tv), parse_int_tuple(tiler));
        return put(to_string(tc.retile(parse_layout(layout))), out, cap);
    });
}

int32_t moye_layout_tile_to_shape(const char* layout, const char* trg_shape, const char* order, char* out, size_t cap) {
    MOYE_REQUIRE(layout && trg_shape);
    return guarded([&] {
        const std::string od = nz(order);
        IT o;
        if (!od.empty()) o = parse_int_tuple(od);
        return put(to_string(tile_to_shape(parse_layout(layout), parse_int_tuple(trg_shape), od.empty() ? nullptr : &o)), out, cap);
    });
}

int32_t moye_layout_print(const char* layout, char* out, size_t cap) {  // print_layout, print.jl:7-44
    MOYE_REQUIRE(layout);
    return guarded([&] {
        const Layout l = parse_layout(layout);
        if (rank(l) != 2) throw Error(MOYE_ERR_RANK, "print_layout takes a rank-2 layout");
        const int64_t rows = size(l, 1).v, cols = size(l, 2).v;
        const int w = (int)std::to_string(cosize(l).v).size() + 2;
        auto lpad = [](const std::string& t, int n) { return (int)t.size() >= n ? t : std::string((size_t)n - t.size(), ' ') + t; };
        std::string sep = "    ";
        for (int64_t n = 0; n < cols; ++n) sep += "+" + std::string((size_t)w, '-');
        sep += "+";
        std::string r = to_string(l) + "\n    ";
        for (int64_t n = 1; n <= cols; ++n) r += "  " + lpad(std::to_string(n), w - 2) + " ";
        for (int64_t m = 1; m <= rows; ++m) {
            r += "\n" + sep + "\n" + lpad(std::to_string(m), 2) + "  ";
            for (int64_t n = 1; n <= cols; ++n)
                r += "| " + lpad(std::to_string(eval(l, tup({IT(D(m)), IT(D(n))})).v), w - 2) + " ";
            r += "|";
        }
        r += "\n" + sep;
        return put(r, out, cap);
    });
}

int32_t moye_layout_make_like(const char* layout, char* out, size_t cap) {
    MOYE_REQUIRE(layout);
    return guarded([&] { return put(to_string(make_layout_like(parse_layout(layout))), out, cap); });
}

int32_t moye_make_tiled_mma(int32_t atom, const char* atom_layout, const char* permutation, moye_tiled_mma* out) {
    MOYE_REQUIRE(out);
    return guarded([&] {
        const TiledMMAHost m(find_atom(std::to_string(atom)), nz(atom_layout), nz(permutation));
        std::memset(out, 0, sizeof *out);
        out->atom = atom;
        const Layout& al = m.atom_layout_mnk;
        for (int i = 0; i < 3; ++i) {
            out->atom_layout_mnk[i] = (int32_t)size(al, i + 1).v;
            out->tile_mnk[i] = (int32_t)m.tile_size(i + 1).v;
        }
        if (out->atom_layout_mnk[2] != 1)
            throw Error(MOYE_ERR_UNSUPPORTED, "atoms tiled along K inside a workgroup are not supported by the kernels");
        // the CTA tile follows the permutation sizes: that is what the caller's shared-memory layouts hold
        for (int i = 0; i < 3; ++i) out->cta_tile_mnk[i] = out->tile_mnk[i];
        return (int32_t)MOYE_OK;
    });
}

int32_t moye_mma_atom_probe(int32_t atom, const void* A, const void* B, float* D, void* stream) {
    MOYE_REQUIRE(A && B && D);
    return guarded([&] { return mma_atom_probe_impl(atom, A, B, D, static_cast<hipStream_t>(stream)); });
}

}  // extern "C"

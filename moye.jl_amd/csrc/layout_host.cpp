// Host-side layout algebra (see layout_host.hpp).  Each function cites the reference file:line
// whose semantics it keeps.
#include "layout_host.hpp"

#include <algorithm>
#include <cctype>
#include <cstdlib>

namespace moye {
namespace host {

namespace {

[[noreturn]] void raise(moye_status st, const std::string& m) { throw Error(st, m); }

// Julia `div` / `rem`: truncation toward zero, remainder with the sign of the dividend.
int64_t tdiv(int64_t a, int64_t b) {
    if (b == 0) raise(MOYE_ERR_SHAPE, "division by zero in layout arithmetic");
    return a / b;  // C++ truncates toward zero
}
int64_t trem(int64_t a, int64_t b) {
    if (b == 0) raise(MOYE_ERR_SHAPE, "division by zero in layout arithmetic");
    return a % b;
}

// Static.jl arithmetic: static op static -> static, mixed -> dynamic; a static zero absorbs `*`.
Int add(Int a, Int b) { return promoted(a.v + b.v, a, b); }
Int sub(Int a, Int b) { return promoted(a.v - b.v, a, b); }
Int mul(Int a, Int b) {
    if ((a.s && a.v == 0) || (b.s && b.v == 0)) return S(0);
    return promoted(a.v * b.v, a, b);
}
Int div(Int a, Int b) { return promoted(tdiv(a.v, b.v), a, b); }
Int rem(Int a, Int b) { return promoted(trem(a.v, b.v), a, b); }
Int imin(Int a, Int b) { return promoted(std::min(a.v, b.v), a, b); }
Int imax(Int a, Int b) { return promoted(std::max(a.v, b.v), a, b); }
Int iabs(Int a) { return same_type(a, std::llabs(a.v)); }
Int isign(Int a) { return same_type(a, (a.v > 0) - (a.v < 0)); }
Int cld(Int a, Int b) {
    if (b.v == 0) raise(MOYE_ERR_SHAPE, "division by zero in layout arithmetic");
    int64_t q = a.v / b.v;
    if ((a.v % b.v != 0) && ((a.v < 0) == (b.v < 0))) ++q;
    return promoted(q, a, b);
}
bool is_static_one(const IT& t) { return t.is_leaf() && t.leaf.s && t.leaf.v == 1; }
bool is_static_zero(const IT& t) { return t.is_leaf() && t.leaf.s && t.leaf.v == 0; }

std::vector<IT> as_items(const IT& t) { return t.is_tuple() ? t.items : std::vector<IT>{t}; }

const Int& leaf_of(const IT& t) {
    if (!t.is_leaf()) raise(MOYE_ERR_ARG, "expected an integer, got " + to_string(t));
    return t.leaf;
}

IT front(const IT& t) { return t.is_tuple() ? front(t.items.front()) : t; }

IT replace_front(const IT& t, const IT& v) {
    if (!t.is_tuple()) return v;
    IT r = t;
    r.items[0] = v;
    return r;
}

IT prepend_item(const IT& t, const IT& v) {
    std::vector<IT> out{v};
    for (const IT& e : as_items(t)) out.push_back(e);
    return IT::tuple(out);
}

IT unwrap(const IT& t) { return (t.is_tuple() && t.size() == 1) ? unwrap(t.items[0]) : t; }

}  // namespace

// ------------------------------------------------------------------------------------------------
// text
// ------------------------------------------------------------------------------------------------
namespace {
struct Parser {
    const std::string& s;
    size_t p = 0;
    explicit Parser(const std::string& str) : s(str) {}
    void ws() {
        while (p < s.size() && std::isspace((unsigned char)s[p])) ++p;
    }
    bool peek(char c) {
        ws();
        return p < s.size() && s[p] == c;
    }
    bool eat(char c) {
        if (peek(c)) {
            ++p;
            return true;
        }
        return false;
    }
    bool done() {
        ws();
        return p >= s.size();
    }
    [[noreturn]] void bad(const std::string& what) {
        raise(MOYE_ERR_PARSE, "cannot parse \"" + s + "\" at offset " + std::to_string(p) + ": " + what);
    }
    Int integer() {
        ws();
        bool st = false;
        if (p < s.size() && s[p] == '_') {
            st = true;
            ++p;
        }
        size_t q = p;
        if (q < s.size() && (s[q] == '-' || s[q] == '+')) ++q;
        size_t d0 = q;
        while (q < s.size() && std::isdigit((unsigned char)s[q])) ++q;
        if (q == d0) bad("expected an integer");
        int64_t v = std::strtoll(s.substr(p, q - p).c_str(), nullptr, 10);
        p = q;
        if (s.compare(p, 3, "i32") == 0) {  // a dynamic Int32
            if (st) bad("a static integer has no width");
            if (v < INT32_MIN || v > INT32_MAX) bad("value does not fit an Int32");
            p += 3;
            return D32(v);
        }
        return Int(v, st);
    }
    // int tuple item; colons allowed when `colons`
    IT item(bool colons) {
        ws();
        if (eat('(')) {
            std::vector<IT> v;
            while (!peek(')')) {
                v.push_back(item(colons));
                if (!eat(',') && !peek(')')) bad("expected ',' or ')'");
                if (p >= s.size()) bad("unterminated tuple");
            }
            eat(')');
            return IT::tuple(v);
        }
        if (colons && peek(':')) {
            ++p;
            return IT::colon();
        }
        return IT(integer());
    }
    // position of the top-level ':' that splits shape:stride, or npos
    static size_t split(const std::string& t) {
        int depth = 0;
        for (size_t i = 0; i < t.size(); ++i) {
            if (t[i] == '(' || t[i] == '<') ++depth;
            else if (t[i] == ')' || t[i] == '>') --depth;
            else if (t[i] == ':' && depth == 0) return i;
        }
        return std::string::npos;
    }
};

std::string trim(const std::string& t) {
    size_t a = 0, b = t.size();
    while (a < b && std::isspace((unsigned char)t[a])) ++a;
    while (b > a && std::isspace((unsigned char)t[b - 1])) --b;
    return t.substr(a, b - a);
}

void check_congruent(const IT& a, const IT& b, const std::string& text) {
    if (a.is_tuple() != b.is_tuple() || (a.is_tuple() && a.size() != b.size()))
        raise(MOYE_ERR_PARSE, "shape and stride of \"" + text + "\" are not congruent");
    if (a.is_tuple())
        for (size_t i = 0; i < a.size(); ++i) check_congruent(a[i], b[i], text);
}
}  // namespace

IT parse_int_tuple(const std::string& text) {
    Parser ps(text);
    IT r = ps.item(true);
    if (!ps.done()) ps.bad("trailing text");
    return r;
}

Layout parse_layout(const std::string& text_in) {
    const std::string text = trim(text_in);
    const size_t k = Parser::split(text);
    if (k == std::string::npos) {
        Parser ps(text);
        IT shape = ps.item(false);
        if (!ps.done()) ps.bad("trailing text");
        return make_layout(shape);
    }
    const std::string a = text.substr(0, k), b = text.substr(k + 1);
    Parser pa(a), pb(b);
    IT shape = pa.item(false);
    if (!pa.done()) pa.bad("trailing text");
    IT stride = pb.item(false);
    if (!pb.done()) pb.bad("trailing text");
    check_congruent(shape, stride, text);
    return Layout{shape, stride};
}

Tile parse_tile(const std::string& text_in) {
    const std::string text = trim(text_in);
    if (text.empty()) raise(MOYE_ERR_PARSE, "empty tile");
    Tile t;
    if (text == ":") {
        t.kind = Tile::COLON;
        return t;
    }
    if (text.front() == '<') {
        if (text.back() != '>') raise(MOYE_ERR_PARSE, "unterminated tile tuple \"" + text + "\"");
        t.kind = Tile::TUPLE;
        const std::string inner = text.substr(1, text.size() - 2);
        int depth = 0;
        size_t start = 0;
        for (size_t i = 0; i <= inner.size(); ++i) {
            if (i == inner.size() || (inner[i] == ',' && depth == 0)) {
                const std::string part = trim(inner.substr(start, i - start));
                if (!part.empty()) t.items.push_back(parse_tile(part));
                start = i + 1;
            } else if (inner[i] == '(' || inner[i] == '<') ++depth;
            else if (inner[i] == ')' || inner[i] == '>') --depth;
        }
        return t;
    }
    if (text.front() == '(' || Parser::split(text) != std::string::npos) {
        t.kind = Tile::LAYOUT;
        t.layout = parse_layout(text);
        return t;
    }
    Parser ps(text);
    t.kind = Tile::INT;
    t.value = ps.integer();
    if (!ps.done()) ps.bad("trailing text");
    return t;
}

std::string to_string(const IT& t) {
    if (t.is_colon()) return ":";
    if (t.is_leaf()) return (t.leaf.s ? "_" : "") + std::to_string(t.leaf.v) + (t.leaf.w32 ? "i32" : "");
    std::string r = "(";
    for (size_t i = 0; i < t.size(); ++i) {
        if (i) r += ", ";
        r += to_string(t[i]);
    }
    if (t.size() == 1) r += ",";
    return r + ")";
}

std::string to_string(const Layout& l) { return to_string(l.shape) + ":" + to_string(l.stride); }

// ------------------------------------------------------------------------------------------------
// IntTuple
// ------------------------------------------------------------------------------------------------
int rank(const IT& t) { return t.is_tuple() ? (int)t.size() : 1; }  // int_tuple.jl:30-32

int depth(const IT& t) {  // int_tuple.jl:41-44
    if (!t.is_tuple()) return 0;
    int d = 0;
    for (const IT& e : t.items) d = std::max(d, depth(e));
    return d + 1;
}

std::vector<Int> flat_leaves(const IT& t) {
    std::vector<Int> out;
    if (t.is_leaf()) out.push_back(t.leaf);
    else if (t.is_tuple())
        for (const IT& e : t.items) {
            auto v = flat_leaves(e);
            out.insert(out.end(), v.begin(), v.end());
        }
    return out;
}

IT flatten(const IT& t) {  // tuple_algorithms.jl:18-20
    if (!t.is_tuple()) return t;
    std::vector<IT> out;
    for (const IT& e : t.items) {
        if (e.is_tuple()) {
            IT f = flatten(e);
            out.insert(out.end(), f.items.begin(), f.items.end());
        } else {
            out.push_back(e);
        }
    }
    return IT::tuple(out);
}

Int product(const IT& t) {  // int_tuple.jl:48-50
    if (t.is_leaf()) return t.leaf;
    Int p = S(1);
    for (const Int& v : flat_leaves(t)) p = mul(p, v);
    return p;
}

bool is_static(const IT& t) {
    for (const Int& v : flat_leaves(t))
        if (!v.s) return false;
    return !t.is_colon();
}

bool equal_values(const IT& a, const IT& b) {
    if (a.kind != b.kind) return false;
    if (a.is_leaf()) return a.leaf.v == b.leaf.v;
    if (a.is_colon()) return true;
    if (a.size() != b.size()) return false;
    for (size_t i = 0; i < a.size(); ++i)
        if (!equal_values(a[i], b[i])) return false;
    return true;
}

namespace {
Int shape_div_int(Int a, Int b) {  // int_tuple.jl:84-90
    if (a.s && b.s && b.v != 0 && a.v != 0 && a.v % b.v != 0 && b.v % a.v != 0)
        raise(MOYE_ERR_SHAPE, "Cannot divide " + std::to_string(a.v) + " by " + std::to_string(b.v) + " or vice versa");
    if (b.v == 0) raise(MOYE_ERR_SHAPE, "shape_div by zero");
    const int64_t q = tdiv(a.v, b.v);
    const int64_t r = q != 0 ? q : isign(a).v * isign(b).v;
    return promoted(r, a, b);
}
}  // namespace

IT shape_div(const IT& a, const IT& b) {  // int_tuple.jl:84-101
    if (a.is_tuple()) {
        if (b.is_tuple()) {
            if (a.size() != b.size()) raise(MOYE_ERR_RANK, "shape_div: tuples of different length");
            std::vector<IT> out;
            for (size_t i = 0; i < a.size(); ++i) out.push_back(shape_div(a[i], b[i]));
            return IT::tuple(out);
        }
        std::vector<IT> out;
        IT rest = b;
        for (const IT& ai : a.items) {
            out.push_back(shape_div(ai, rest));
            rest = shape_div(rest, ai);
        }
        return IT::tuple(out);
    }
    if (b.is_tuple()) return shape_div(a, IT(product(b)));
    return IT(shape_div_int(leaf_of(a), leaf_of(b)));
}

IT elem_scale(const IT& x, const IT& y) {  // int_tuple.jl:103-109
    if (x.is_tuple()) {
        if (!y.is_tuple() || x.size() != y.size()) raise(MOYE_ERR_RANK, "elem_scale: incongruent tuples");
        std::vector<IT> out;
        for (size_t i = 0; i < x.size(); ++i) out.push_back(elem_scale(x[i], y[i]));
        return IT::tuple(out);
    }
    return IT(mul(leaf_of(x), product(y)));
}

IT filter_zeros(const IT& a, const IT& x) {  // int_tuple.jl:123-128
    if (a.is_tuple()) {
        std::vector<IT> out;
        for (size_t i = 0; i < a.size(); ++i) out.push_back(filter_zeros(a[i], x[i]));
        return IT::tuple(out);
    }
    return is_static_zero(a) ? IT(S(1)) : x;
}

namespace {
IT product_like(const IT& x, const IT& g) {  // int_tuple.jl:59-60
    if (g.is_tuple()) {
        if (!x.is_tuple() || x.size() != g.size()) raise(MOYE_ERR_RANK, "product_like: incongruent tuples");
        std::vector<IT> out;
        for (size_t i = 0; i < g.size(); ++i) out.push_back(product_like(x[i], g[i]));
        return IT::tuple(out);
    }
    return IT(product(x));
}

bool has_colon(const IT& t) {
    if (t.is_colon()) return true;
    if (t.is_tuple())
        for (const IT& e : t.items)
            if (has_colon(e)) return true;
    return false;
}
}  // namespace

bool iscompatible(const IT& a, const IT& b) {  // int_tuple.jl:116-120
    if (a.is_tuple()) {
        if (!b.is_tuple() || a.size() != b.size()) return false;
        for (size_t i = 0; i < a.size(); ++i)
            if (!iscompatible(a[i], b[i])) return false;
        return true;
    }
    return leaf_of(a).v == product(b).v;
}

IT slice(const IT& a, const IT& index) {  // int_tuple.jl:130-142
    if (index.is_colon()) return IT::tuple({a});
    if (index.is_tuple()) {
        const std::vector<IT> av = as_items(a);
        if (av.size() != index.size()) raise(MOYE_ERR_RANK, "Array and index must have the same rank");
        std::vector<IT> out;
        for (size_t i = 0; i < av.size(); ++i) {
            IT s = slice(av[i], index[i]);
            out.insert(out.end(), s.items.begin(), s.items.end());
        }
        return IT::tuple(out);
    }
    return IT::tuple({});
}

IT dice(const IT& a, const IT& index) {  // int_tuple.jl:143-156
    if (index.is_colon()) return IT::tuple({});
    if (index.is_tuple()) {
        const std::vector<IT> av = as_items(a);
        if (av.size() != index.size()) raise(MOYE_ERR_RANK, "Array and index must have the same rank");
        std::vector<IT> out;
        for (size_t i = 0; i < av.size(); ++i) {
            IT s = dice(av[i], index[i]);
            out.insert(out.end(), s.items.begin(), s.items.end());
        }
        return IT::tuple(out);
    }
    return IT::tuple({a});
}

// ------------------------------------------------------------------------------------------------
// coordinates (src/stride.jl)
// ------------------------------------------------------------------------------------------------
namespace {
Int c2i0_int(Int coord, const IT& shape, const IT& stride) {  // stride.jl:1-33
    const size_t n = shape.size();
    if (n == 1) {
        if (shape[0].is_tuple()) return c2i0_int(coord, shape[0], stride[0]);
        return mul(coord, leaf_of(stride[0]));
    }
    Int result = S(0);
    for (size_t i = 0; i < n; ++i) {
        const Int p = product(shape[i]);
        if (shape[i].is_tuple()) result = add(result, c2i0_int(rem(coord, p), shape[i], stride[i]));
        else result = add(result, mul(rem(coord, leaf_of(shape[i])), leaf_of(stride[i])));
        coord = div(coord, p);
    }
    return result;
}

Int c2i0(const IT& coord, const IT& shape, const IT& stride) {  // stride.jl:35-54, 0-based
    if (coord.is_leaf()) {
        if (shape.is_leaf()) return mul(coord.leaf, leaf_of(stride));
        return c2i0_int(coord.leaf, shape, stride);
    }
    if (!coord.is_tuple() || !shape.is_tuple() || coord.size() != shape.size())
        raise(MOYE_ERR_RANK, "coordinate " + to_string(coord) + " does not fit shape " + to_string(shape));
    Int acc = S(0);
    bool first = true;
    for (size_t i = 0; i < coord.size(); ++i) {
        const Int t = c2i0(coord[i], shape[i], stride[i]);
        acc = first ? t : add(acc, t);
        first = false;
    }
    return acc;
}

IT offset0(const IT& x) {  // stride.jl:72-80: 1-based -> 0-based, colon -> 0
    if (x.is_colon()) return IT(S(0));
    if (x.is_tuple()) {
        std::vector<IT> out;
        for (const IT& e : x.items) out.push_back(offset0(e));
        return IT::tuple(out);
    }
    return IT(same_type(x.leaf, x.leaf.v - 1));
}
}  // namespace

Int coord_to_index(const IT& coord, const IT& shape, const IT& stride) {  // stride.jl:82-89
    const Int idx = c2i0(offset0(coord), shape, stride);
    return same_type(idx, idx.v + 1);
}

Int coord_to_index_default(const IT& coord, const IT& shape) {  // stride.jl:56-70
    const IT c0 = offset0(coord);
    if (c0.is_leaf()) return same_type(c0.leaf, c0.leaf.v + 1);
    const std::vector<Int> fc = flat_leaves(c0);
    const std::vector<Int> fs = flat_leaves(product_like(shape, coord));
    Int acc = fc.back();
    for (size_t i = fc.size() - 1; i-- > 0;) acc = add(fc[i], mul(fs[i], acc));
    return same_type(acc, acc.v + 1);
}

namespace {
IT compact_impl(const IT& shape, Int& current, bool left) {  // stride.jl:168-236
    if (shape.is_tuple()) {
        std::vector<IT> res(shape.size());
        if (left)
            for (size_t i = 0; i < shape.size(); ++i) res[i] = compact_impl(shape[i], current, left);
        else
            for (size_t i = shape.size(); i-- > 0;) res[i] = compact_impl(shape[i], current, left);
        return IT::tuple(res);
    }
    if (is_static_one(shape)) return IT(S(0));
    const Int stride = current;
    current = mul(current, leaf_of(shape));
    return IT(stride);
}

IT compact_major(const IT& shape, const IT& current, bool left) {  // stride.jl:238-245
    if (current.is_tuple()) {
        if (!shape.is_tuple() || shape.size() != current.size())
            raise(MOYE_ERR_RANK, "shape and current must have the same rank");
        std::vector<IT> out;
        for (size_t i = 0; i < shape.size(); ++i) out.push_back(compact_major(shape[i], current[i], left));
        return IT::tuple(out);
    }
    Int cur = leaf_of(current);
    return compact_impl(shape, cur, left);
}
}  // namespace

IT compact_col_major(const IT& shape, Int current) { return compact_major(shape, IT(current), true); }
IT compact_row_major(const IT& shape, Int current) { return compact_major(shape, IT(current), false); }

IT index_to_coord(Int index, const IT& shape, const IT& stride_in) {  // stride.jl:91-128
    if (shape.is_tuple()) {
        IT stride = stride_in;
        if (!stride.is_tuple()) stride = compact_col_major(shape, leaf_of(stride));
        if (stride.size() != shape.size()) raise(MOYE_ERR_RANK, "shape, and stride must have the same rank");
        std::vector<IT> out;
        for (size_t i = 0; i < shape.size(); ++i) out.push_back(index_to_coord(index, shape[i], stride[i]));
        return IT::tuple(out);
    }
    if (is_static_one(shape)) return IT(S(0));
    const Int st = leaf_of(stride_in);
    const Int crd = rem(div(same_type(index, index.v - 1), st), leaf_of(shape));
    return IT(same_type(crd, crd.v + 1));
}

namespace {
IT unflatten_impl(const std::vector<IT>& flat, size_t& pos, const IT& target) {  // tuple_algorithms.jl:25-37
    if (target.is_tuple()) {
        std::vector<IT> out;
        for (const IT& t : target.items) out.push_back(unflatten_impl(flat, pos, t));
        return IT::tuple(out);
    }
    return flat.at(pos++);
}
}  // namespace

IT compact_order(const IT& shape, const IT& order) {  // stride.jl:253-276
    const IT pl = product_like(shape, order);
    const std::vector<Int> old_shape = flat_leaves(pl);
    const std::vector<Int> flat_order = flat_leaves(order);
    Int max_order = S(0);
    for (const Int& o : flat_order)
        if (o.s && max_order.v <= o.v) max_order = o;
    std::vector<IT> old_order;
    for (size_t i = 0; i < flat_order.size(); ++i)
        old_order.push_back(IT(flat_order[i].s ? flat_order[i] : S((int64_t)i + 1 + max_order.v)));
    size_t pos = 0;
    const IT new_order = unflatten_impl(old_order, pos, order);
    struct Rec {
        const std::vector<Int>& os;
        const std::vector<IT>& oo;
        IT operator()(const IT& sh, const IT& od) const {
            if (od.is_tuple()) {
                std::vector<IT> out;
                for (size_t i = 0; i < od.size(); ++i) out.push_back((*this)(sh[i], od[i]));
                return IT::tuple(out);
            }
            Int d = S(1);
            for (size_t i = 0; i < os.size(); ++i) d = mul(d, oo[i].leaf.v < od.leaf.v ? os[i] : S(1));
            return compact_col_major(sh, d);
        }
    } rec{old_shape, old_order};
    return rec(shape, new_order);
}

// ------------------------------------------------------------------------------------------------
// Layout
// ------------------------------------------------------------------------------------------------
Layout make_layout(const IT& shape) { return Layout{shape, compact_col_major(shape)}; }  // layout.jl:141-144

Layout make_layout(const IT& shape, const IT& stride) {  // layout.jl:133-140
    check_congruent(shape, stride, to_string(shape) + ":" + to_string(stride));
    return Layout{shape, stride};
}

Layout concat(const std::vector<Layout>& ls) {  // layout.jl:151-153
    std::vector<IT> sh, st;
    for (const Layout& l : ls) {
        sh.push_back(l.shape);
        st.push_back(l.stride);
    }
    return Layout{IT::tuple(sh), IT::tuple(st)};
}

int rank(const Layout& l) { return rank(l.shape); }

Layout mode(const Layout& l, int i) {  // layout.jl:233-236
    if (!l.shape.is_tuple()) {
        if (i != 1) raise(MOYE_ERR_RANK, "mode " + std::to_string(i) + " of a rank-1 layout");
        return l;
    }
    if (i < 1 || i > (int)l.shape.size()) raise(MOYE_ERR_RANK, "mode index out of range");
    return Layout{l.shape[i - 1], l.stride[i - 1]};
}

Int size(const Layout& l) { return product(l.shape); }  // layout.jl:302-304
Int size(const Layout& l, int i) { return product(mode(l, i).shape); }
Int eval(const Layout& l, const IT& coord) { return coord_to_index(coord, l.shape, l.stride); }  // layout.jl:90-95
Int cosize(const Layout& l) { return eval(l, IT(size(l))); }  // layout.jl:350-352

Layout flatten(const Layout& l) { return Layout{flatten(l.shape), flatten(l.stride)}; }  // layout.jl:292-294

namespace {
// layout.jl:441-479
Layout bw_coalesce(int n, const std::vector<IT>& old_shape, const std::vector<IT>& old_stride, IT new_shape,
                   IT new_stride) {
    for (int i = n - 1; i >= 0; --i) {
        const IT& s = old_shape[i];
        const IT& d = old_stride[i];
        if (is_static_one(s)) continue;
        if (is_static_one(new_shape)) {
            new_shape = s;
            new_stride = d;
        } else {
            const IT fs = front(new_shape), fd = front(new_stride);
            if (fs.leaf.s && s.leaf.s && d.leaf.s && fd.leaf.s && s.leaf.v * d.leaf.v == fd.leaf.v) {
                new_shape = replace_front(new_shape, IT(mul(s.leaf, fs.leaf)));
                new_stride = replace_front(new_stride, d);
            } else {
                new_shape = prepend_item(new_shape, s);
                new_stride = prepend_item(new_stride, d);
            }
        }
    }
    if (is_static_one(new_shape)) return Layout{IT(S(1)), IT(S(0))};
    return Layout{new_shape, new_stride};
}

// apply f by mode (layout.jl:408-439); without n the longer tail is kept
template <typename F>
Layout transform(F&& f, const Layout& a, const std::vector<Tile>& t, int n) {
    const int r1 = rank(a), r2 = (int)t.size();
    std::vector<Layout> out;
    if (n >= 0) {
        for (int i = 1; i <= n; ++i) out.push_back(f(mode(a, i), t[i - 1]));
        return concat(out);
    }
    for (int i = 1; i <= std::min(r1, r2); ++i) out.push_back(f(mode(a, i), t[i - 1]));
    if (r1 < r2) {
        for (int i = r1 + 1; i <= r2; ++i) {
            if (t[i - 1].kind != Tile::LAYOUT) raise(MOYE_ERR_RANK, "tile has more modes than the layout");
            out.push_back(t[i - 1].layout);
        }
    } else {
        for (int i = r2 + 1; i <= r1; ++i) out.push_back(mode(a, i));
    }
    return concat(out);
}
}  // namespace

Layout coalesce(const Layout& l) {  // layout.jl:497-502
    std::vector<IT> fs = as_items(flatten(l.shape)), fd = as_items(flatten(l.stride));
    return bw_coalesce((int)fs.size() - 1, fs, fd, fs.back(), fd.back());
}

Layout coalesce(const Layout& l, const IT& profile) {  // layout.jl:503-509
    if (!profile.is_tuple()) return coalesce(l);
    if ((int)profile.size() > rank(l)) raise(MOYE_ERR_RANK, "coalesce: profile longer than the layout");
    std::vector<Layout> out;
    for (int i = 1; i <= rank(l); ++i)
        out.push_back(i <= (int)profile.size() ? coalesce(mode(l, i), profile[i - 1]) : mode(l, i));
    return concat(out);
}

Layout filter(const Layout& l) {  // layout.jl:511-517
    return coalesce(Layout{filter_zeros(l.stride, l.shape), l.stride});
}

namespace {
void fold_shape(const std::vector<IT>& front_shape, IT rest, std::vector<IT>* out, IT* rest_out) {
    for (const IT& si : front_shape) {
        const Int a = iabs(leaf_of(si));
        out->push_back(IT(imin(a, leaf_of(rest))));
        rest = shape_div(rest, IT(a));
    }
    *rest_out = rest;
}

// layout.jl:520-575: A (flat shape ls, stride ld) after one B mode rs:rd
Layout compose1(const IT& ls, const IT& ld, const IT& rs, const IT& rd) {
    if (rs.is_tuple()) {
        std::vector<Layout> out;
        for (size_t i = 0; i < rs.size(); ++i) out.push_back(compose1(ls, ld, rs[i], rd[i]));
        return concat(out);
    }
    if (is_static_zero(rd)) return Layout{rs, rd};
    if (!ls.is_tuple()) return Layout{rs, IT(mul(leaf_of(ld), leaf_of(rd)))};
    const int n = (int)ls.size();
    const std::vector<IT> f_shape(ls.items.begin(), ls.items.end() - 1);
    const std::vector<IT> f_stride(ld.items.begin(), ld.items.end() - 1);
    if (is_static_one(rd)) {
        std::vector<IT> shape1;
        IT rest;
        fold_shape(f_shape, rs, &shape1, &rest);
        return bw_coalesce(n - 1, shape1, ld.items, rest, ld.items.back());
    }
    std::vector<IT> shape1;
    IT rest_stride = rd;
    for (const IT& di : f_shape) {
        shape1.push_back(shape_div(di, rest_stride));
        rest_stride = shape_div(rest_stride, di);
    }
    std::vector<IT> stride1;
    for (size_t i = 0; i < f_shape.size(); ++i)
        stride1.push_back(elem_scale(f_stride[i], shape_div(f_shape[i], shape1[i])));
    std::vector<IT> shape2;
    IT rest_shape;
    fold_shape(shape1, rs, &shape2, &rest_shape);
    return bw_coalesce(n - 1, shape2, stride1, rest_shape, IT(mul(leaf_of(rest_stride), leaf_of(ld.items.back()))));
}
}  // namespace

Layout composition(const Layout& lhs, const Layout& rhs) {  // layout.jl:593-597
    return compose1(flatten(lhs.shape), flatten(lhs.stride), rhs.shape, rhs.stride);
}

Layout composition(const Layout& lhs, const Tile& rhs) {  // layout.jl:598-608
    switch (rhs.kind) {
        case Tile::COLON: return lhs;
        case Tile::LAYOUT: return composition(lhs, rhs.layout);
        case Tile::INT: return composition(lhs, make_layout(IT(rhs.value)));
        default:
            if ((int)rhs.items.size() > rank(lhs)) raise(MOYE_ERR_RANK, "composition: tile has more modes than the layout");
            return transform([](const Layout& a, const Tile& t) { return composition(a, t); }, lhs, rhs.items,
                             (int)rhs.items.size());
    }
}

namespace {
Layout complement_impl(const IT& shp_in, const IT& strd_in, Int cotarget) {  // layout.jl:621-653
    if (!shp_in.is_tuple() && is_static_zero(strd_in)) return make_layout(IT(cotarget));
    std::vector<IT> shp = as_items(shp_in), strd = as_items(strd_in);
    for (const IT& d : strd)
        if (!d.is_leaf() || !d.leaf.s) raise(MOYE_ERR_UNSUPPORTED, "complement requires static strides");
    std::vector<IT> res_shape, res_stride{IT(S(1))};
    const size_t r = shp.size();
    for (size_t i = 0; i + 1 < r; ++i) {
        size_t k = 0;
        for (size_t j = 1; j < strd.size(); ++j)
            if (strd[j].leaf.v < strd[k].leaf.v) k = j;
        const Int m = strd[k].leaf;
        const Int new_shape = div(m, res_stride[i].leaf);
        const Int new_stride = mul(m, leaf_of(shp[k]));
        if (new_shape.v == 0) raise(MOYE_ERR_SHAPE, "complement: the layout is not injective");
        shp.erase(shp.begin() + k);
        strd.erase(strd.begin() + k);
        res_shape.push_back(IT(new_shape));
        res_stride.push_back(IT(new_stride));
    }
    const Int new_shape = div(strd[0].leaf, res_stride.back().leaf);
    if (new_shape.v == 0) raise(MOYE_ERR_SHAPE, "complement: the layout is not injective");
    res_shape.push_back(IT(new_shape));
    const Int new_stride = mul(leaf_of(shp[0]), strd[0].leaf);
    const IT rest_shape = IT(cld(cotarget, new_stride));
    const IT rest_stride = compact_col_major(rest_shape, new_stride);
    return coalesce(Layout{IT::tuple({IT::tuple(res_shape), rest_shape}), IT::tuple({IT::tuple(res_stride), rest_stride})});
}
}  // namespace

Layout complement(const Layout& l, Int cotarget) {  // layout.jl:660-663
    const Layout f = filter(l);
    return complement_impl(f.shape, f.stride, cotarget);
}

Layout complement(const Layout& l) {  // layout.jl:665-668
    const Layout f = filter(l);
    return complement_impl(f.shape, f.stride, cosize(f));
}

Layout right_inverse(const Layout& l) {  // layout.jl:670-730
    const Layout flat = coalesce(l);
    const std::vector<IT> shp = as_items(flat.shape), strd = as_items(flat.stride);
    int start = -1;
    for (size_t i = 0; i < strd.size(); ++i)
        if (strd[i].leaf.s && std::llabs(strd[i].leaf.v) == 1) {
            start = (int)i;
            break;
        }
    if (start < 0) return Layout{IT(S(1)), IT(S(0))};
    std::vector<int> seq{start};
    int cur = start;
    while (true) {
        const Int nxt = mul(iabs(strd[cur].leaf), shp[cur].leaf);
        if (!nxt.s) break;
        int found = -1;
        for (size_t j = 0; j < strd.size(); ++j)
            if (strd[j].leaf.s && std::llabs(strd[j].leaf.v) == nxt.v) {
                found = (int)j;
                break;
            }
        if (found < 0 || std::find(seq.begin(), seq.end(), found) != seq.end()) break;
        seq.push_back(found);
        cur = found;
    }
    const std::vector<IT> rstride = as_items(compact_col_major(flat.shape));
    std::vector<IT> rs, rd;
    for (int i : seq) {
        rs.push_back(shp[i]);
        rd.push_back(IT(mul(isign(strd[i].leaf), rstride[i].leaf)));
    }
    return Layout{unwrap(IT::tuple(rs)), unwrap(IT::tuple(rd))};
}

Layout left_inverse(const Layout& l) {  // layout.jl:738
    return right_inverse(concat({l, complement(l)}));
}

Int max_common_vector(const Layout& a, const Layout& b) {  // layout.jl:752-761
    const Layout common = coalesce(composition(a, right_inverse(b)));
    const IT s1 = common.shape.is_tuple() ? common.shape[0] : common.shape;
    const IT d1 = common.stride.is_tuple() ? common.stride[0] : common.stride;
    if (s1.is_leaf() && s1.leaf.s && d1.is_leaf() && d1.leaf.s && d1.leaf.v == 1) return s1.leaf;
    return S(1);
}

Layout zip(const Layout& a, const Layout& b) {  // layout.jl:767-770
    auto z = [](const IT& x, const IT& y) {
        if (x.is_tuple() && y.is_tuple()) {
            std::vector<IT> out;
            for (size_t i = 0; i < std::min(x.size(), y.size()); ++i) out.push_back(IT::tuple({x[i], y[i]}));
            return IT::tuple(out);
        }
        return IT::tuple({IT::tuple({x, y})});
    };
    return Layout{z(a.shape, b.shape), z(a.stride, b.stride)};
}

Layout zip(const Layout& a) {  // layout.jl:763-765
    auto z = [](const IT& t) {
        if (!t.is_tuple()) return t;
        bool all = !t.items.empty();
        size_t n = SIZE_MAX;
        for (const IT& e : t.items) {
            all = all && e.is_tuple();
            if (e.is_tuple()) n = std::min(n, e.size());
        }
        if (!all) return IT::tuple({t});
        std::vector<IT> out;
        for (size_t i = 0; i < n; ++i) {
            std::vector<IT> row;
            for (const IT& e : t.items) row.push_back(e[i]);
            out.push_back(IT::tuple(row));
        }
        return IT::tuple(out);
    };
    return Layout{z(a.shape), z(a.stride)};
}

Layout transpose(const Layout& l) {  // layout.jl:772-774
    if (rank(l) != 2) raise(MOYE_ERR_RANK, "transpose needs a rank-2 layout");
    return concat({mode(l, 2), mode(l, 1)});
}

Tile tile_of(const Layout& l) {
    Tile t;
    t.kind = Tile::LAYOUT;
    t.layout = l;
    return t;
}
Tile tile_of(Int v) {
    Tile t;
    t.kind = Tile::INT;
    t.value = v;
    return t;
}
Tile tile_colon() { return Tile{}; }
Tile tile_tuple(std::vector<Tile> v) {
    Tile t;
    t.kind = Tile::TUPLE;
    t.items = std::move(v);
    return t;
}
Tile tile_from_shape(const IT& t) {
    if (t.is_colon()) return tile_colon();
    if (t.is_leaf()) return tile_of(t.leaf);
    std::vector<Tile> v;
    for (const IT& e : t.items) v.push_back(tile_from_shape(e));
    return tile_tuple(v);
}

namespace {
// zip2_by (tuple_algorithms.jl:213-224) with the tile as guide: a Layout / int / colon is a leaf
void zip2_by(const IT& t, const Tile& guide, IT* first, IT* second) {
    if (guide.kind != Tile::TUPLE) {
        if (!t.is_tuple() || t.size() != 2) raise(MOYE_ERR_RANK, "zip2_by: expected a pair, got " + to_string(t));
        *first = t[0];
        *second = t[1];
        return;
    }
    const size_t gr = guide.items.size();
    if (!t.is_tuple() || gr > t.size()) raise(MOYE_ERR_RANK, "zip2_by: guide tuple is longer than input tuple");
    std::vector<IT> firsts, seconds;
    for (size_t i = 0; i < gr; ++i) {
        IT a, b;
        zip2_by(t[i], guide.items[i], &a, &b);
        firsts.push_back(a);
        seconds.push_back(b);
    }
    for (size_t i = gr; i < t.size(); ++i) seconds.push_back(t[i]);
    *first = IT::tuple(firsts);
    *second = IT::tuple(seconds);
}

Layout tile_unzip(const Layout& l, const Tile& tile) {  // layout.jl:776-778
    if (tile.kind != Tile::TUPLE) {
        if (!l.shape.is_tuple() || l.shape.size() != 2) raise(MOYE_ERR_RANK, "tile_unzip: expected a rank-2 layout");
        return l;
    }
    IT s1, s2, d1, d2;
    zip2_by(l.shape, tile, &s1, &s2);
    zip2_by(l.stride, tile, &d1, &d2);
    return Layout{IT::tuple({s1, s2}), IT::tuple({d1, d2})};
}

int tile_rank(const Tile& t) {
    if (t.kind == Tile::TUPLE) return (int)t.items.size();
    if (t.kind == Tile::LAYOUT) return rank(t.layout);
    return 1;
}

IT colons(int n) {
    std::vector<IT> v((size_t)n, IT::colon());
    return IT::tuple(v);
}
}  // namespace

Layout logical_product(const Layout& l, const Tile& tile) {  // layout.jl:826-838
    switch (tile.kind) {
        case Tile::COLON: return l;
        case Tile::INT: return logical_product(l, tile_of(make_layout(IT(tile.value))));
        case Tile::LAYOUT: {
            const Layout comp = complement(l, mul(size(l), cosize(tile.layout)));
            return concat({l, composition(comp, tile.layout)});
        }
        default:
            return transform([](const Layout& a, const Tile& t) { return logical_product(a, t); }, l, tile.items, -1);
    }
}

Layout zipped_product(const Layout& l, const Tile& tile) { return tile_unzip(logical_product(l, tile), tile); }

Layout tiled_product(const Layout& l, const Tile& tile) {  // layout.jl:844-847
    const Layout d = zipped_product(l, tile);
    return slice_layout(d, IT::tuple({IT::colon(), colons(tile_rank(tile))}));
}

Layout append(const Layout& l, int n) {  // layout.jl:377-389
    if (rank(l) == n) return l;
    if (rank(l) > n) raise(MOYE_ERR_RANK, "append: layout already has more modes");
    std::vector<IT> sh = as_items(l.shape), st = as_items(l.stride);
    while ((int)sh.size() < n) {
        sh.push_back(IT(S(1)));
        st.push_back(IT(S(0)));
    }
    return Layout{IT::tuple(sh), IT::tuple(st)};
}

Layout prepend(const Layout& l, int n) {  // layout.jl:391-397
    if (rank(l) > n) raise(MOYE_ERR_RANK, "prepend: layout already has more modes");
    std::vector<IT> sh = as_items(l.shape), st = as_items(l.stride);
    while ((int)sh.size() < n) {
        sh.insert(sh.begin(), IT(S(1)));
        st.insert(st.begin(), IT(S(0)));
    }
    return Layout{IT::tuple(sh), IT::tuple(st)};
}

namespace {
Layout product_zip(const Layout& block, const Layout& l, bool coalesce_result, bool raked) {  // layout.jl:880-928
    const int r = std::max(rank(block), rank(l));
    const Layout res = logical_product(append(block, r), tile_of(append(l, r)));
    const Layout z = raked ? zip(mode(res, 2), mode(res, 1)) : zip(mode(res, 1), mode(res, 2));
    if (!coalesce_result) return z;
    std::vector<IT> ones((size_t)r, IT(S(1)));
    return coalesce(z, IT::tuple(ones));
}
}  // namespace

Layout blocked_product(const Layout& block, const Layout& l, bool c) { return product_zip(block, l, c, false); }
Layout raked_product(const Layout& block, const Layout& l, bool c) { return product_zip(block, l, c, true); }

Layout logical_divide(const Layout& l, const Tile& tile) {  // layout.jl:1058-1070
    switch (tile.kind) {
        case Tile::COLON: return l;
        case Tile::INT: return logical_divide(l, tile_of(make_layout(IT(tile.value))));
        case Tile::LAYOUT:
            return composition(l, concat({tile.layout, complement(tile.layout, size(l))}));
        default:
            if ((int)tile.items.size() > rank(l)) raise(MOYE_ERR_RANK, "too many modes in tile");
            return transform([](const Layout& a, const Tile& t) { return logical_divide(a, t); }, l, tile.items, -1);
    }
}

Layout zipped_divide(const Layout& l, const Tile& tile) { return tile_unzip(logical_divide(l, tile), tile); }

Layout tiled_divide(const Layout& l, const Tile& tile) {  // layout.jl:1123-1127
    const Layout d = zipped_divide(l, tile);
    return slice_layout(d, IT::tuple({IT::colon(), colons(rank(mode(d, 2)))}));
}

Layout upcast(const Layout& l, int64_t n) {  // layout.jl:945-965
    struct F {
        int64_t n;
        Layout operator()(const IT& shp, const IT& strd) const {
            if (shp.is_tuple()) {
                std::vector<Layout> out;
                for (size_t i = 0; i < shp.size(); ++i) out.push_back((*this)(shp[i], strd[i]));
                return concat(out);
            }
            const Int d = leaf_of(strd);
            if (d.s) {
                if (d.v == 0) return Layout{shp, strd};
                const IT m = IT(S(n));
                return Layout{shape_div(shp, shape_div(m, IT(iabs(d)))), shape_div(strd, m)};
            }
            return Layout{shp, IT(same_type(d, tdiv(d.v, n)))};
        }
    };
    return F{n}(l.shape, l.stride);
}

Layout downcast(const Layout& l, int64_t n) {  // layout.jl:967-997
    struct F {
        int64_t n;
        Layout operator()(const IT& shp, const IT& strd) const {
            if (shp.is_tuple()) {
                std::vector<Layout> out;
                for (size_t i = 0; i < shp.size(); ++i) out.push_back((*this)(shp[i], strd[i]));
                return concat(out);
            }
            const Int d = leaf_of(strd);
            const bool unit = (d.v == 1) || (d.s && d.v == -1);
            if (unit) return Layout{IT(mul(leaf_of(shp), S(n))), strd};
            return Layout{shp, IT(mul(d, S(n)))};
        }
    };
    return F{n}(l.shape, l.stride);
}

Layout recast(const Layout& l, int new_bytes, int old_bytes) {  // layout.jl:999-1010
    if (new_bytes <= 0 || old_bytes <= 0) raise(MOYE_ERR_ARG, "recast: element sizes must be positive");
    if (new_bytes == old_bytes) return l;
    if (new_bytes > old_bytes) {
        if (new_bytes % old_bytes) raise(MOYE_ERR_SHAPE, "Cannot recast: sizes do not divide");
        return upcast(l, new_bytes / old_bytes);
    }
    if (old_bytes % new_bytes) raise(MOYE_ERR_SHAPE, "Cannot recast: sizes do not divide");
    return downcast(l, old_bytes / new_bytes);
}

Layout make_ordered_layout(const IT& shape, const IT& order) {  // layout.jl:216-218
    return Layout{shape, compact_order(shape, order)};
}

Layout make_fragment_like(const Layout& l) {  // layout.jl:1143-1149
    if (!(is_static(l.shape) && is_static(l.stride)) || rank(l) == 1) return make_layout(l.shape);
    std::vector<Layout> rest;
    for (int i = 2; i <= rank(l); ++i) rest.push_back(mode(l, i));
    const Layout r = concat(rest);
    return tiled_product(make_layout(l.shape[0]), tile_of(make_ordered_layout(r.shape, r.stride)));
}

Layout slice_layout(const Layout& l, const IT& coord) {  // layout.jl:364-366
    return Layout{slice(l.shape, coord), slice(l.stride, coord)};
}

Layout slice_and_offset(const Layout& l, const IT& coord, int64_t* offset) {  // layout.jl:368-371
    const Int idx = coord_to_index(coord, l.shape, l.stride);
    if (offset) *offset = idx.v - 1;
    return slice_layout(l, coord);
}

Layout dice_layout(const Layout& l, const IT& coord) {  // layout.jl:373-375
    return Layout{dice(l.shape, coord), dice(l.stride, coord)};
}

IT get_congr_coord(const Layout& l, Int index) {  // layout.jl:115-119
    const IT h = index_to_coord(index, l.shape, l.stride);
    if (!l.shape.is_tuple()) return IT::tuple({IT(coord_to_index_default(h, l.shape))});
    std::vector<IT> out;
    for (size_t i = 0; i < l.shape.size(); ++i) {
        // a static size-1 mode yields the coordinate _0 (stride.jl:91-93), kept as is
        if (h[i].is_leaf() && h[i].leaf.s && h[i].leaf.v == 0) out.push_back(IT(Int(0, true)));
        else out.push_back(IT(coord_to_index_default(h[i], l.shape[i])));
    }
    return IT::tuple(out);
}

// ------------------------------------------------------------------------------------------------
// tiling verbs (src/algorithm/array_algorithms.jl)
// ------------------------------------------------------------------------------------------------
namespace {
Tile dice_tile(const Tile& tile, const IT& proj) {
    if (tile.kind != Tile::TUPLE || !proj.is_tuple() || tile.items.size() != proj.size())
        raise(MOYE_ERR_RANK, "projection and tile must have the same rank");
    std::vector<Tile> out;
    for (size_t i = 0; i < proj.size(); ++i)
        if (!proj[i].is_colon()) out.push_back(tile.items[i]);
    return tile_tuple(out);
}
IT append_colons(const IT& coord, int n) {
    std::vector<IT> v = as_items(coord);
    if ((int)v.size() > n) raise(MOYE_ERR_RANK, "coordinate has more modes than the array");
    while ((int)v.size() < n) v.push_back(IT::colon());
    return IT::tuple(v);
}
}  // namespace

Layout local_tile(const Layout& l, const Tile& tile, const IT& coord, const IT* proj, int64_t* offset) {
    // array_algorithms.jl:113-120
    if (proj) return local_tile(l, dice_tile(tile, *proj), dice(coord, *proj), nullptr, offset);
    if (tile.kind != Tile::TUPLE) raise(MOYE_ERR_ARG, "@tile takes a tuple tile");
    const int r1 = (int)tile.items.size(), r2 = rank(l);
    const Layout z = zipped_divide(l, tile);
    return slice_and_offset(z, IT::tuple({colons(r1), append_colons(coord, r2)}), offset);
}

Layout local_partition(const Layout& l, const Tile& tile, const IT& coord_or_index, const IT* proj,
                       int64_t* offset) {
    // array_algorithms.jl:36-47
    if (tile.kind == Tile::LAYOUT) {
        const Layout& t = tile.layout;
        std::vector<IT> caps;
        for (const IT& s : as_items(t.shape)) caps.push_back(IT(product(s)));
        IT shp = IT::tuple(caps);
        IT coord;
        if (proj) {
            shp = dice(shp, *proj);
            coord = get_congr_coord(dice_layout(t, *proj), leaf_of(coord_or_index));
        } else {
            coord = get_congr_coord(t, leaf_of(coord_or_index));
        }
        return local_partition(l, tile_from_shape(shp), coord, nullptr, offset);
    }
    if (proj) return local_partition(l, dice_tile(tile, *proj), dice(coord_or_index, *proj), nullptr, offset);
    if (tile.kind != Tile::TUPLE) raise(MOYE_ERR_ARG, "@parallelize takes a thread layout or a tuple tile");
    const Layout z = zipped_divide(l, tile);
    return slice_and_offset(z, IT::tuple({coord_or_index, colons(rank(l))}), offset);
}

// ------------------------------------------------------------------------------------------------
// IntTuple helpers used by callers rather than by the algebra itself
// ------------------------------------------------------------------------------------------------
IT unflatten(const IT& flat, const IT& target) {  // tuple_algorithms.jl:25-37
    const std::vector<IT> items = as_items(flat);
    size_t need = flat_leaves(target).size();
    if (items.size() < need) raise(MOYE_ERR_RANK, "unflatten: not enough elements for the target profile");
    size_t pos = 0;
    return unflatten_impl(items, pos, target);
}

IT group(const IT& t, int b, int e) {  // tuple_algorithms.jl:101-112, modes b..e (1-based, inclusive)
    const std::vector<IT> items = as_items(t);
    if (b < 1 || e < b || (size_t)e > items.size()) raise(MOYE_ERR_ARG, "group: bad range");
    std::vector<IT> out(items.begin(), items.begin() + (b - 1));
    out.push_back(IT::tuple(std::vector<IT>(items.begin() + (b - 1), items.begin() + e)));
    out.insert(out.end(), items.begin() + e, items.end());
    return IT::tuple(out);
}

IT append_value(const IT& t, const IT& val, int n) {  // tuple_algorithms.jl:114-145
    std::vector<IT> items = as_items(t);
    if (n < 0) {
        items.push_back(val);
        return IT::tuple(items);
    }
    if (items.size() > (size_t)n)
        raise(MOYE_ERR_RANK, "input tuple of length " + std::to_string(items.size()) + ", requested " + std::to_string(n));
    while (items.size() < (size_t)n) items.push_back(val);
    return IT::tuple(items);
}

IT prepend_value(const IT& t, const IT& val, int n) {  // tuple_algorithms.jl:147-176
    std::vector<IT> items = as_items(t);
    if (n < 0) {
        items.insert(items.begin(), val);
        return IT::tuple(items);
    }
    if (items.size() > (size_t)n)
        raise(MOYE_ERR_RANK, "input tuple of length " + std::to_string(items.size()) + ", requested " + std::to_string(n));
    items.insert(items.begin(), (size_t)n - items.size(), val);
    return IT::tuple(items);
}

IT zip2_by(const IT& t, const IT& guide) {  // tuple_algorithms.jl:213-224
    if (!guide.is_tuple()) {
        if (!t.is_tuple() || t.size() != 2) raise(MOYE_ERR_RANK, "zip2_by: expected a pair");
        return t;
    }
    if (!t.is_tuple() || guide.size() > t.size()) raise(MOYE_ERR_RANK, "zip2_by: guide tuple is longer than input tuple");
    std::vector<IT> firsts, seconds;
    for (size_t i = 0; i < guide.size(); ++i) {
        const IT z = zip2_by(t[i], guide[i]);
        firsts.push_back(z[0]);
        seconds.push_back(z[1]);
    }
    for (size_t i = guide.size(); i < t.size(); ++i) seconds.push_back(t[i]);
    return IT::tuple({IT::tuple(firsts), IT::tuple(seconds)});
}

IT product_each(const IT& t) {
    std::vector<IT> out;
    for (const IT& e : as_items(t)) out.push_back(IT(product(e)));
    return IT::tuple(out);
}

namespace {
bool int_less(const IT& a, const IT& b) { return leaf_of(a).v < leaf_of(b).v; }
IT drop_last(const IT& t) { return IT::tuple(std::vector<IT>(t.items.begin(), t.items.end() - 1)); }
IT drop_first(const IT& t) { return IT::tuple(std::vector<IT>(t.items.begin() + 1, t.items.end())); }
IT repeat_like(const IT& t, Int x) {  // tuple_algorithms.jl:80-98
    if (!t.is_tuple()) return IT(x);
    std::vector<IT> out;
    for (const IT& e : t.items) out.push_back(repeat_like(e, x));
    return IT::tuple(out);
}
}  // namespace

bool colex_less(const IT& a, const IT& b) {  // int_tuple.jl:184-195
    if (!a.is_tuple() && !b.is_tuple()) return int_less(a, b);
    if (!a.is_tuple() || !b.is_tuple()) raise(MOYE_ERR_RANK, "colex_less: an integer against a tuple");
    if (a.size() == 0) return b.size() != 0;
    if (b.size() == 0) return false;
    const IT &x = a.items.back(), &y = b.items.back();
    if (!equal_values(x, y)) return colex_less(x, y);
    return colex_less(drop_last(a), drop_last(b));
}

bool elem_less(const IT& a, const IT& b) {  // int_tuple.jl:197-211
    if (!a.is_tuple() && !b.is_tuple()) return int_less(a, b);
    if (!a.is_tuple() || !b.is_tuple()) raise(MOYE_ERR_RANK, "elem_less: an integer against a tuple");
    if (a.size() == 0) return true;
    if (b.size() == 0) return false;
    const IT &x = a[0], &y = b[0];
    if (a.size() == 1 && b.size() == 1) return x.is_tuple() ? elem_less(x, y) : int_less(x, y);
    if (!(equal_values(x, y) || elem_less(x, y))) return false;
    return elem_less(drop_first(a), drop_first(b));
}

IT increment(const IT& coord, const IT& shape) {  // int_tuple.jl:218-232: next 1-based coordinate, wrapping
    if (!coord.is_tuple()) {
        const Int c = leaf_of(coord), s = leaf_of(shape);
        return c.v < s.v ? IT(same_type(c, c.v + 1)) : IT(same_type(c, 1));
    }
    if (!shape.is_tuple() || shape.size() != coord.size()) raise(MOYE_ERR_RANK, "increment: coordinate and shape differ in rank");
    const IT &c = coord[0], &s = shape[0];
    if (coord.size() == 1) return IT::tuple({increment(c, s)});
    if (!equal_values(c, s)) {
        IT r = coord;
        r.items[0] = increment(c, s);
        return r;
    }
    const bool st = is_static(c);
    std::vector<IT> out{repeat_like(s, Int(1, st))};
    for (const IT& e : increment(drop_first(coord), drop_first(shape)).items) out.push_back(e);
    return IT::tuple(out);
}

IT coord_to_coord(const IT& coord, const IT& src_shape, const IT& dst_shape) {  // stride.jl:133-141
    if (coord.is_tuple() && src_shape.is_tuple() && dst_shape.is_tuple()) {
        if (coord.size() != src_shape.size() || coord.size() != dst_shape.size())
            raise(MOYE_ERR_RANK, "coord, shape1, and shape2 must have the same rank");
        std::vector<IT> out;
        for (size_t i = 0; i < coord.size(); ++i) out.push_back(coord_to_coord(coord[i], src_shape[i], dst_shape[i]));
        return IT::tuple(out);
    }
    const Int idx = coord_to_index_default(coord, src_shape);
    if (!dst_shape.is_tuple()) return IT(idx);  // index_to_coord(index, shape::Int) is the index itself (stride.jl:118-121)
    return index_to_coord(idx, dst_shape, compact_col_major(dst_shape));
}

Layout tile_to_shape(const Layout& l, const IT& trg_shape, const IT* order) {  // layout.jl:930-935
    const int r = rank(trg_shape);
    if (rank(l) > r) raise(MOYE_ERR_RANK, "Cannot tile to a smaller shape");
    const Layout padded = append(l, r);
    const IT pshape = shape_div(product_each(trg_shape), product_each(padded.shape));
    const Layout ord = order ? make_ordered_layout(pshape, *order) : make_layout(pshape);
    return coalesce(blocked_product(padded, ord, false), pshape);
}

Layout make_layout_like(const Layout& l) {  // layout.jl:223-225
    return Layout{l.shape, compact_order(filter_zeros(l.stride, l.shape), l.stride)};
}

}  // namespace host
}  // namespace moye

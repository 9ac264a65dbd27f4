"""Host-side mirror of MoYe's layout API (src/layout.jl exports, src/MoYe.jl:59-101).

Every function here is a thin call into libmoye_hip.so's `moye_layout_*` / `moye_tuple_op`
entry points; the algebra itself lives in the library (csrc/layout_host.cpp).  Layouts travel as
text, `shape:stride`, with `_n` for a static integer (`Static.StaticInt`) and `n` for a dynamic one.
"""
import ctypes as C

from . import _lib
from ._lib import check, lib

_CAP = 8192
_BIG_CAP = 1 << 23


class StaticInt(int):
    """A compile-time integer, printed `_n` (the reference's `_1`, `_2`, ... constants)."""

    __slots__ = ()

    def __repr__(self):
        return "_%d" % int(self)


class Int32(int):
    """A run-time 32-bit integer (Julia `Int32`), written `5i32` in text: results computed from Int32 and static
    integers only stay Int32 (test/layout.jl:4-12 of the reference)."""

    __slots__ = ()

    def __repr__(self):
        return "%di32" % int(self)


class _Colon:
    def __repr__(self):
        return ":"


COLON = _Colon()
GenColMajor = "GenColMajor"
GenRowMajor = "GenRowMajor"


def static(x):
    """`static(x)`: make every integer of a (nested) tuple static."""
    if isinstance(x, tuple):
        return tuple(static(e) for e in x)
    if x is COLON:
        return x
    return StaticInt(x)


def tuple_text(t):
    if isinstance(t, tuple):
        inner = ", ".join(tuple_text(e) for e in t)
        return "(%s,)" % inner if len(t) == 1 else "(%s)" % inner
    if t is COLON or t is Ellipsis or t == ":":
        return ":"
    return repr(t) if isinstance(t, (StaticInt, Int32)) else str(int(t))


def parse_tuple(text):
    """Inverse of tuple_text."""
    text = text.strip()
    pos = [0]

    def item():
        while text[pos[0]] == " ":
            pos[0] += 1
        ch = text[pos[0]]
        if ch == "(":
            pos[0] += 1
            out = []
            while True:
                while text[pos[0]] in " ,":
                    pos[0] += 1
                if text[pos[0]] == ")":
                    pos[0] += 1
                    return tuple(out)
                out.append(item())
        if ch == ":":
            pos[0] += 1
            return COLON
        j = pos[0]
        while j < len(text) and (text[j].isdigit() or text[j] in "_-"):
            j += 1
        tok = text[pos[0]:j]
        if text.startswith("i32", j):
            pos[0] = j + 3
            return Int32(int(tok))
        pos[0] = j
        return StaticInt(int(tok[1:])) if tok.startswith("_") else int(tok)

    return item()


def _tile_text(t):
    """Tile argument: Layout | int | COLON | tuple of tiles -> text (`<a, b>` for tuples)."""
    if isinstance(t, Layout):
        return t.text
    if isinstance(t, tuple):
        return "<" + ", ".join(_tile_text(e) for e in t) + ">"
    if isinstance(t, str):
        return t
    return tuple_text(t)


def _text_out(fn, *args):
    buf = C.create_string_buffer(_CAP)
    status = fn(*args, buf, _CAP)
    if status == _lib.ERR_BUFFER:  # printed tables outgrow the usual buffer
        buf = C.create_string_buffer(_BIG_CAP)
        status = fn(*args, buf, _BIG_CAP)
    check(status)
    return buf.value.decode()


def _b(s):
    return s.encode() if isinstance(s, str) else s


_declared = False


def _l():
    global _declared
    l = lib()
    if not _declared:
        cs, S, I32 = C.c_char_p, C.c_size_t, C.c_int32
        I64p, I32p = C.POINTER(C.c_int64), C.POINTER(C.c_int32)
        un = ["flatten", "coalesce", "filter", "right_inverse", "left_inverse", "make_fragment_like", "normalize"]
        for n in un:
            getattr(l, "moye_layout_" + n).argtypes = [cs, cs, S]
        for n in ["composition", "logical_product", "zipped_product", "tiled_product", "logical_divide",
                  "zipped_divide", "tiled_divide", "complement", "make_ordered"]:
            getattr(l, "moye_layout_" + n).argtypes = [cs, cs, cs, S]
        for n in ["blocked_product", "raked_product"]:
            getattr(l, "moye_layout_" + n).argtypes = [cs, cs, I32, cs, S]
        l.moye_layout_recast.argtypes = [cs, I32, I32, cs, S]
        l.moye_layout_append.argtypes = [cs, I32, cs, S]
        l.moye_layout_prepend.argtypes = [cs, I32, cs, S]
        l.moye_layout_make.argtypes = [cs, I32, cs, S]
        l.moye_layout_slice.argtypes = [cs, cs, cs, S, I64p]
        l.moye_layout_eval.argtypes = [cs, cs, I64p]
        l.moye_layout_size.argtypes = [cs, I64p]
        l.moye_layout_cosize.argtypes = [cs, I64p]
        l.moye_layout_rank_depth.argtypes = [cs, I32p, I32p]
        l.moye_layout_max_common_vector.argtypes = [cs, cs, I64p]
        l.moye_tuple_op.argtypes = [cs, cs, cs, cs, cs, S]
        l.moye_local_tile.argtypes = [cs, cs, cs, cs, cs, S, I64p]
        l.moye_local_partition.argtypes = [cs, cs, cs, cs, cs, S, I64p]
        l.moye_tiled_mma_query.argtypes = [cs, cs, cs, cs, cs, S]
        l.moye_tiled_mma_partition.argtypes = [cs, cs, cs, I32, C.c_char, cs, cs, S, I64p]
        l.moye_tiled_copy_query.argtypes = [I32, I32, I32, cs, cs, cs, cs, S]
        l.moye_tiled_copy_partition.argtypes = [I32, I32, I32, cs, cs, I32, C.c_char, cs, cs, S, I64p]
        l.moye_make_tiled_mma.argtypes = [I32, cs, cs, C.POINTER(_lib.TiledMMA)]
        l.moye_tiled_copy_tv_query.argtypes = [I32, I32, I32, cs, cs, cs, cs, S]
        l.moye_tiled_copy_tv_partition.argtypes = [I32, I32, I32, cs, cs, I32, C.c_char, cs, cs, S, I64p]
        l.moye_tiled_copy_tv_retile.argtypes = [I32, I32, I32, cs, cs, cs, cs, S]
        l.moye_layout_tile_to_shape.argtypes = [cs, cs, cs, cs, S]
        l.moye_layout_make_like.argtypes = [cs, cs, S]
        l.moye_layout_print.argtypes = [cs, cs, S]
        _declared = True
    return l


class Layout:
    """`Layout(shape, stride)` (src/layout.jl:48-59).  Immutable; `.text` is the canonical form."""

    __slots__ = ("text",)

    def __init__(self, shape, stride=None):
        if stride is None and isinstance(shape, str):
            self.text = _text_out(_l().moye_layout_normalize, _b(shape))
        elif stride is None:
            self.text = _text_out(_l().moye_layout_make, _b(tuple_text(shape)), 0)
        else:
            self.text = _text_out(_l().moye_layout_normalize, _b(tuple_text(shape) + ":" + tuple_text(stride)))

    # ---- structure ----
    def _split(self):
        depth = 0
        for i, ch in enumerate(self.text):
            depth += ch == "("
            depth -= ch == ")"
            if ch == ":" and depth == 0:
                return self.text[:i], self.text[i + 1:]
        raise ValueError(self.text)

    @property
    def shape(self):
        return parse_tuple(self._split()[0])

    @property
    def stride(self):
        return parse_tuple(self._split()[1])

    def __repr__(self):
        return self.text

    def __eq__(self, other):  # numeric equality, like Julia's `==`
        return isinstance(other, Layout) and self.shape == other.shape and self.stride == other.stride

    def __hash__(self):
        return hash((self.shape, self.stride))

    def identical(self, other):
        """Same values and same static-ness (Julia `===`)."""
        return self.text == other.text

    def __call__(self, *coord):
        """layout(coord): 1-based index of a coordinate, or the sliced layout if it holds a colon."""
        c = coord[0] if len(coord) == 1 else tuple(coord)
        if _has_colon(c):
            return slice_and_offset(self, c)[0]
        # the typed form: a StaticInt, an Int32 or an int, as the reference's result type would be
        f = _l().moye_layout_eval_typed
        f.argtypes = [C.c_char_p, C.c_char_p, C.c_char_p, C.c_size_t]
        return parse_tuple(_text_out(f, _b(self.text), _b(tuple_text(c))))

    def __getitem__(self, i):
        s, d = self.shape, self.stride
        if not isinstance(s, tuple):
            if i != 1:
                raise IndexError(i)
            return self
        return Layout(s[i - 1], d[i - 1])

    def __len__(self):
        return rank(self)


def _has_colon(c):
    return c is COLON or (isinstance(c, tuple) and any(_has_colon(e) for e in c))


# ---- constructors (src/layout.jl:133-225) ----
def make_layout(*args):
    if args and all(isinstance(a, Layout) for a in args):
        return Layout(tuple(a.shape for a in args), tuple(a.stride for a in args))
    if len(args) == 1:
        return Layout(args[0])
    shape, second = args
    if second == GenColMajor:
        return Layout(shape)
    if second == GenRowMajor:
        return Layout(_text_out(_l().moye_layout_make, _b(tuple_text(shape)), 1))
    return Layout(shape, second)


def static_layout(shape, stride=None):
    """The `@Layout` macro (src/layout.jl:188-198)."""
    if stride is None or isinstance(stride, str):
        return make_layout(static(shape), *([stride] if stride else []))
    return make_layout(static(shape), static(stride))


def make_ordered_layout(shape, order):
    return Layout(_text_out(_l().moye_layout_make_ordered, _b(tuple_text(shape)), _b(tuple_text(order))))


# ---- queries ----
def size(l, i=None):
    out = C.c_int64()
    check(_l().moye_layout_size(_b((l if i is None else l[i]).text), C.byref(out)))
    return out.value


def cosize(l):
    out = C.c_int64()
    check(_l().moye_layout_cosize(_b(l.text), C.byref(out)))
    return out.value


def rank(l):
    r, d = C.c_int32(), C.c_int32()
    check(_l().moye_layout_rank_depth(_b(l.text), C.byref(r), C.byref(d)))
    return r.value


def depth(l):
    r, d = C.c_int32(), C.c_int32()
    check(_l().moye_layout_rank_depth(_b(l.text), C.byref(r), C.byref(d)))
    return d.value


def max_common_vector(a, b):
    out = C.c_int64()
    check(_l().moye_layout_max_common_vector(_b(a.text), _b(b.text), C.byref(out)))
    return out.value


# ---- algebra ----
def _unary(name):
    def f(l):
        return Layout(_text_out(getattr(_l(), "moye_layout_" + name), _b(l.text)))
    f.__name__ = name
    return f


flatten = _unary("flatten")
coalesce = _unary("coalesce")
filter = _unary("filter")  # noqa: A001 - the reference's name
right_inverse = _unary("right_inverse")
left_inverse = _unary("left_inverse")
make_fragment_like = _unary("make_fragment_like")


def _with_tile(name):
    def f(l, tile):
        return Layout(_text_out(getattr(_l(), "moye_layout_" + name), _b(l.text), _b(_tile_text(tile))))
    f.__name__ = name
    return f


composition = _with_tile("composition")
logical_product = _with_tile("logical_product")
zipped_product = _with_tile("zipped_product")
tiled_product = _with_tile("tiled_product")
logical_divide = _with_tile("logical_divide")
zipped_divide = _with_tile("zipped_divide")
tiled_divide = _with_tile("tiled_divide")


def complement(l, cotarget=None):
    ct = "" if cotarget is None else tuple_text(cotarget)
    return Layout(_text_out(_l().moye_layout_complement, _b(l.text), _b(ct)))


def blocked_product(block, l, coalesce_result=False):
    return Layout(_text_out(_l().moye_layout_blocked_product, _b(block.text), _b(l.text), int(coalesce_result)))


def raked_product(block, l, coalesce_result=False):
    return Layout(_text_out(_l().moye_layout_raked_product, _b(block.text), _b(l.text), int(coalesce_result)))


def recast(l, new_bytes, old_bytes):
    return Layout(_text_out(_l().moye_layout_recast, _b(l.text), new_bytes, old_bytes))


def append(l, n):
    return Layout(_text_out(_l().moye_layout_append, _b(l.text), n))


def prepend(l, n):
    return Layout(_text_out(_l().moye_layout_prepend, _b(l.text), n))


def slice_and_offset(l, coord):
    """(sliced layout, 0-based element offset) — src/layout.jl:368-371."""
    off = C.c_int64()
    buf = C.create_string_buffer(_CAP)
    check(_l().moye_layout_slice(_b(l.text), _b(tuple_text(coord)), buf, _CAP, C.byref(off)))
    return Layout(buf.value.decode()), off.value


def tuple_op(op, a, b=None, c=None):
    """IntTuple helpers of src/int_tuple.jl / src/stride.jl by name; returns a (nested) tuple or int."""
    tb = "" if b is None else tuple_text(b)
    tc = "" if c is None else tuple_text(c)
    out = _text_out(_l().moye_tuple_op, _b(op), _b(tuple_text(a)), _b(tb), _b(tc))
    if out in ("true", "false"):
        return out == "true"
    return parse_tuple(out)


def coord_to_index(coord, shape, stride=None):
    return tuple_op("coord_to_index", coord, shape, stride)


def index_to_coord(index, shape, stride=None):
    return tuple_op("index_to_coord", index, shape, stride)


def compact_col_major(shape):
    return tuple_op("compact_col_major", shape)


def compact_row_major(shape):
    return tuple_op("compact_row_major", shape)


def shape_div(a, b):
    return tuple_op("shape_div", a, b)


def flat(l):
    """Flattened (shape, stride) lists of ints: what a moye_tensor descriptor carries."""
    f = flatten(l)
    s, d = f.shape, f.stride
    if not isinstance(s, tuple):
        s, d = (s,), (d,)
    return [int(x) for x in s], [int(x) for x in d]


# ---- more IntTuple helpers (src/algorithm/tuple_algorithms.jl, src/int_tuple.jl, src/stride.jl) ----
def unflatten(flat_tuple, target):
    return tuple_op("unflatten", flat_tuple, target)


def group(t, b, e):
    """group modes b..e (1-based, inclusive) — tuple_algorithms.jl:101-112."""
    return tuple_op("group", t, b, e)


def tuple_append(t, val, n=None):
    return tuple_op("append", t, val, n)


def tuple_prepend(t, val, n=None):
    return tuple_op("prepend", t, val, n)


def zip2_by(t, guide):
    return tuple_op("zip2_by", t, guide)


def product_each(t):
    return tuple_op("product_each", t)


def capacity(t):
    return tuple_op("capacity", t)


def elem_scale(x, y):
    return tuple_op("elem_scale", x, y)


def filter_zeros(a, x=None):
    return tuple_op("filter_zeros", a, x)


def colex_less(a, b):
    return tuple_op("colex_less", a, b)


def elem_less(a, b):
    return tuple_op("elem_less", a, b)


def increment(coord, shape):
    return tuple_op("increment", coord, shape)


def coord_to_coord(coord, src_shape, dst_shape):
    return tuple_op("coord_to_coord", coord, src_shape, dst_shape)


def iscompatible(a, b):
    return tuple_op("iscompatible", a, b)


def tile_to_shape(l, trg_shape, order=None):
    """src/layout.jl:930-935; order None = GenColMajor."""
    return Layout(_text_out(_l().moye_layout_tile_to_shape, _b(l.text), _b(tuple_text(trg_shape)),
                            _b("" if order is None else tuple_text(order))))


def make_layout_like(l):
    """src/layout.jl:223-225."""
    return Layout(_text_out(_l().moye_layout_make_like, _b(l.text)))


def print_layout(l, file=None):
    """print_layout(layout) (src/print.jl:7-44): the index table of a rank-2 layout; returns the text."""
    buf = C.create_string_buffer(1 << 20)
    check(_l().moye_layout_print(_b(l.text), buf, 1 << 20))
    text = buf.value.decode()
    if file is not False:
        print(text, file=file)
    return text

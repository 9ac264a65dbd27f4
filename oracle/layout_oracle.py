"""CPU oracle for MoYe's host-side layout algebra.  TEST INFRASTRUCTURE ONLY.

Pure-Python restatement of the integer algorithms of the reference
(YichengDWu/MoYe.jl v4.0.1).  Nothing in the shipped package imports this
file: only tests, the smoke check and the CPU-baseline leg of the benchmark
may use it, and only as the checker.

Every function cites the reference file:line it follows.  Integers carry the
reference's static/dynamic distinction: `S(n)` is a `Static.StaticInt{n}`
(printed `_n`), a plain `int` is a run-time `Int`.  Arithmetic between two
static ints is static, anything mixed is dynamic, and a static zero absorbs a
product (Static.jl, compat "0.8, 1", is not vendored by the reference; these
three rules are its published behaviour).

Pinned by tests/test_oracle_layout.py against the reference's own known
answers (test/stride.jl, test/int_tuple.jl, test/tuple_alg.jl,
test/layout.jl, test/array.jl, test/tiling.jl, test/tiled_mma.jl,
test/copy.jl, the printed tables in the docstrings of src/layout.jl and
src/algorithm/array_algorithms.jl, docs/src/manual/tiled_matmul.md) and by
function-level invariants evaluated by brute force.

Parity unpinned (no reference vector exists and none can be generated without
a Julia runtime): the printed form (nesting, static-ness) of the results of
`retile`, `get_layout{A,B,C}_TV`, `make_tiled_copy_{A,B,C}`, `tile_to_shape`,
`left_inverse`, and of `compact_order` with mixed static/dynamic orders.  The
function values of the TV layouts and of make_tiled_copy_A/B are pinned by the
thread-ownership tables of the manual's figures (tests/test_svg_fixtures.py);
`retile`, `tile_to_shape` and `left_inverse` by invariants only.
"""
from __future__ import annotations

import re
from functools import reduce

# --------------------------------------------------------------------------
# static integers (Static.jl StaticInt; src/utilities.jl:1-62)
# --------------------------------------------------------------------------


class S(int):
    """A compile-time integer (`StaticInt{N}`), printed as `_N`."""

    __slots__ = ()

    def __repr__(self):
        return "_%d" % int(self)

    __str__ = __repr__

    def _w(self, other, r):
        if isinstance(other, S):
            return S(r)
        return I32(r) if isinstance(other, I32) else int(r)

    def __add__(self, o):
        return self._w(o, int(self) + int(o))

    __radd__ = __add__

    def __sub__(self, o):
        return self._w(o, int(self) - int(o))

    def __rsub__(self, o):
        return self._w(o, int(o) - int(self))

    def __mul__(self, o):
        if int(self) == 0:
            return S(0)
        return self._w(o, int(self) * int(o))

    __rmul__ = __mul__

    def __floordiv__(self, o):
        return self._w(o, tdiv(int(self), int(o)))

    def __rfloordiv__(self, o):
        return self._w(o, tdiv(int(o), int(self)))

    def __mod__(self, o):
        return self._w(o, trem(int(self), int(o)))

    def __rmod__(self, o):
        return self._w(o, trem(int(o), int(self)))

    def __neg__(self):
        return S(-int(self))

    def __abs__(self):
        return S(abs(int(self)))


def _wrap32(r):
    return (int(r) + 2 ** 31) % 2 ** 32 - 2 ** 31


class I32(int):
    """A run-time `Int32` (src/utilities.jl:1-11: IntType = Union{Int, StaticInt, Int32}), printed `5i32`.  Julia's
    promotion: with a static integer or another Int32 the result is an Int32 (promote_rule(StaticInt, Int32) = Int32),
    with an Int it is an Int; Int32 arithmetic wraps modulo 2^32."""

    __slots__ = ()

    def __new__(cls, v):
        return super().__new__(cls, _wrap32(v))

    def __repr__(self):
        return "%di32" % int(self)

    __str__ = __repr__

    def _w(self, other, r):
        return I32(r) if isinstance(other, (I32, S)) else int(r)

    def __add__(self, o):
        return self._w(o, int(self) + int(o))

    __radd__ = __add__

    def __sub__(self, o):
        return self._w(o, int(self) - int(o))

    def __rsub__(self, o):
        return self._w(o, int(o) - int(self))

    def __mul__(self, o):
        if isinstance(o, S) and int(o) == 0:
            return S(0)
        return self._w(o, int(self) * int(o))

    __rmul__ = __mul__

    def __floordiv__(self, o):
        return self._w(o, tdiv(int(self), int(o)))

    def __rfloordiv__(self, o):
        return self._w(o, tdiv(int(o), int(self)))

    def __mod__(self, o):
        return self._w(o, trem(int(self), int(o)))

    def __rmod__(self, o):
        return self._w(o, trem(int(o), int(self)))

    def __neg__(self):
        return I32(-int(self))

    def __abs__(self):
        return I32(abs(int(self)))


def one(x):
    """Julia `one(x)`: 1 in the type of x."""
    return _1 if isinstance(x, S) else I32(1) if isinstance(x, I32) else 1


def _promote(r, *xs):
    """r in the type Julia's promotion gives a result computed from xs."""
    if all(isinstance(x, S) for x in xs):
        return S(r)
    return I32(r) if all(isinstance(x, (S, I32)) for x in xs) else int(r)


def tdiv(a, b):
    """Julia `div`/`÷`: truncation toward zero."""
    q = abs(a) // abs(b)
    return q if (a >= 0) == (b >= 0) else -q


def trem(a, b):
    """Julia `rem`/`%`: sign of the dividend."""
    return a - b * tdiv(a, b)


class _Colon:
    def __repr__(self):
        return ":"


COLON = _Colon()
_0, _1 = S(0), S(1)


def is_int(x):
    return isinstance(x, int) and not isinstance(x, bool)


def is_tuple(x):
    return isinstance(x, tuple)


def is_static(x):
    if is_tuple(x):
        return all(is_static(e) for e in x)
    return isinstance(x, S)


def static(x):
    if is_tuple(x):
        return tuple(static(e) for e in x)
    if x is COLON:
        return x
    return S(x)


def dynamic(x):
    if is_tuple(x):
        return tuple(dynamic(e) for e in x)
    return int(x)


def smin(a, b):
    return _promote(min(int(a), int(b)), a, b)


def smax(a, b):
    return _promote(max(int(a), int(b)), a, b)


def sabs(a):
    return abs(a)


def ssign(a):
    return _promote((int(a) > 0) - (int(a) < 0), a)


def cld(a, b):
    return _promote(-((-int(a)) // int(b)), a, b)


# --------------------------------------------------------------------------
# tuple algorithms (src/algorithm/tuple_algorithms.jl)
# --------------------------------------------------------------------------


def flatten(x):
    """tuple_algorithms.jl:18-20 — remove all nesting; an int stays an int."""
    if not is_tuple(x):
        return x
    out = []
    for e in x:
        if is_tuple(e):
            out.extend(flatten(e))
        else:
            out.append(e)
    return tuple(out)


def flatten_to_tuple(x):
    """tuple_algorithms.jl:14-16."""
    f = flatten(x)
    return f if is_tuple(f) else (f,)


def unflatten(flat, target):
    """tuple_algorithms.jl:25-37 — re-nest `flat` after the profile `target`."""

    def impl(rem, t):
        if is_tuple(t):
            res = []
            for sub in t:
                r, rem = impl(rem, sub)
                res.append(r)
            return tuple(res), rem
        return rem[0], rem[1:]

    return impl(tuple(flat), target)[0]


def front(t):
    """tuple_algorithms.jl:1-3 — first leaf."""
    return front(t[0]) if is_tuple(t) else t


def back(t):
    """tuple_algorithms.jl:5-7 — last leaf."""
    return back(t[-1]) if is_tuple(t) else t


def unwrap(t):
    """tuple_algorithms.jl:9-10."""
    return unwrap(t[0]) if is_tuple(t) and len(t) == 1 else t


def tuple_cat(*ts):
    return tuple(e for t in ts for e in t)


def insert(t, x, n):
    """tuple_algorithms.jl:39-41 (1-based position n)."""
    return t[: n - 1] + (x,) + t[n - 1:]


def remove(t, n):
    """tuple_algorithms.jl:43-53 (1-based)."""
    if len(t) < n:
        return t
    return t[: n - 1] + t[n:]


def replace(t, x, n):
    """tuple_algorithms.jl:55-58 (1-based)."""
    return t[: n - 1] + (x,) + t[n:]


def replace_front(t, v):
    return (v,) + t[1:] if is_tuple(t) else v


def repeat(x, n):
    return tuple(x for _ in range(int(n)))


def repeat_like(t, x):
    """tuple_algorithms.jl:80-98."""
    return tuple(repeat_like(e, x) for e in t) if is_tuple(t) else x


def group(t, b, e):
    """tuple_algorithms.jl:101-112 — group modes b..e (1-based, inclusive)."""
    return t[: b - 1] + (t[b - 1: e],) + t[e:]


def _as_tuple(t):
    return t if is_tuple(t) else (t,)


def append(t, val, n=None):
    """tuple_algorithms.jl:114-145 — append `val` once, or pad to length n."""
    t = _as_tuple(t)
    if n is None:
        return t + (val,)
    if len(t) > n:
        raise ValueError("input tuple of length %d, requested %d" % (len(t), n))
    return t + (val,) * (int(n) - len(t))


def prepend(t, val, n=None):
    """tuple_algorithms.jl:147-176."""
    t = _as_tuple(t)
    if n is None:
        return (val,) + t
    if len(t) > n:
        raise ValueError("input tuple of length %d, requested %d" % (len(t), n))
    return (val,) * (int(n) - len(t)) + t


def escan(f, x, init):
    """tuple_algorithms.jl:192-207 — exclusive scan."""
    out = [init]
    for e in x[:-1]:
        out.append(f(out[-1], e))
    return tuple(out)


def zip_(t):
    """tuple_algorithms.jl:209-212 (`_zip`)."""
    if is_tuple(t) and len(t) > 0 and all(is_tuple(e) for e in t):
        return tuple(zip(*t))
    if is_tuple(t):
        return (t,)
    return t


def zip2_by(t, guide):
    """tuple_algorithms.jl:213-224."""
    if not is_tuple(guide):
        assert len(t) == 2
        return t
    tr, gr = len(t), len(guide)
    if gr > tr:
        raise ValueError("zip2_by: guide tuple is longer than input tuple")
    split = [zip2_by(t[i], guide[i]) for i in range(gr)]
    firsts = tuple(s[0] for s in split)
    seconds = tuple(s[1] for s in split)
    return (firsts, seconds + tuple(t[gr:]))


def hascolon(t):
    """tuple_algorithms.jl:226-227 — top level only."""
    return is_tuple(t) and any(e is COLON for e in t)


# --------------------------------------------------------------------------
# IntTuple (src/int_tuple.jl)
# --------------------------------------------------------------------------


def rank(x):
    """int_tuple.jl:30-32."""
    return len(x) if is_tuple(x) else 1


def depth(x):
    """int_tuple.jl:41-44."""
    if not is_tuple(x):
        return 0
    return max([depth(e) for e in x], default=0) + 1


def product(x):
    """int_tuple.jl:48-50."""
    if not is_tuple(x):
        return x
    return reduce(lambda a, b: a * b, flatten(x), _1) if len(x) else _1


capacity = product


def product_each(x):
    return tuple(product(e) for e in x)


def product_like(x, g):
    """int_tuple.jl:59-60 — one product of `x` per leaf of the guide `g`."""
    if is_tuple(g):
        return tuple(product_like(x[i], g[i]) for i in range(len(g)))
    return product(x)


def shape_div(a, b):
    """int_tuple.jl:84-101."""
    if is_tuple(a):
        if is_tuple(b):
            assert len(a) == len(b)
            return tuple(shape_div(x, y) for x, y in zip(a, b))
        res, rest = [], b
        for ai in a:
            res.append(shape_div(ai, rest))
            rest = shape_div(rest, ai)
        return tuple(res)
    if is_tuple(b):
        return shape_div(a, product(b))
    if isinstance(a, S) and isinstance(b, S):
        if int(a) % int(b) != 0 and int(b) % int(a) != 0:
            raise AssertionError("Cannot divide %d by %d or vice versa" % (a, b))
    q = tdiv(int(a), int(b))
    r = q if q != 0 else int(ssign(a)) * int(ssign(b))
    return _promote(r, a, b)


def elem_scale(x, y):
    """int_tuple.jl:103-109."""
    if is_tuple(x):
        assert len(x) == len(y)
        return tuple(elem_scale(a, b) for a, b in zip(x, y))
    return x * capacity(y)


def iscongruent(x, y):
    return repeat_like(x, 0) == repeat_like(y, 0)


def iscompatible(a, b):
    """int_tuple.jl:116-120 — every coordinate into a is a coordinate into b."""
    if is_tuple(a):
        if not is_tuple(b):
            return False
        return len(a) == len(b) and all(iscompatible(x, y) for x, y in zip(a, b))
    return int(a) == int(capacity(b))


def filter_zeros(a, x=None):
    """int_tuple.jl:123-128 — modes of x paired with a static 0 in a become _1."""
    if x is None:
        x = a
    if is_tuple(a):
        return tuple(filter_zeros(p, q) for p, q in zip(a, x))
    return _1 if (isinstance(a, S) and a == 0) else x


def slice_(a, index):
    """int_tuple.jl:130-142 — keep what a `:` selects."""
    if index is COLON:
        return (a,)
    if is_tuple(index):
        if not is_tuple(a):
            a = (a,)
        if len(a) != len(index):
            raise ValueError("Array and index must have the same rank")
        return tuple_cat(*[slice_(x, i) for x, i in zip(a, index)])
    return ()


def dice(a, index):
    """int_tuple.jl:143-156 — keep what an integer selects."""
    if index is COLON:
        return ()
    if is_tuple(index):
        if len(a) != len(index):
            raise ValueError("Array and index must have the same rank")
        return tuple_cat(*[dice(x, i) for x, i in zip(a, index)])
    return (a,)


def colex_less(t1, t2):
    """int_tuple.jl:184-195."""
    if not is_tuple(t1) and not is_tuple(t2):
        return t1 < t2
    if len(t1) == 0:
        return len(t2) != 0
    if len(t2) == 0:
        return False
    a, b = t1[-1], t2[-1]
    if a != b:
        return colex_less(a, b)
    return colex_less(t1[:-1], t2[:-1])


def elem_less(t1, t2):
    """int_tuple.jl:197-211."""
    if not is_tuple(t1) and not is_tuple(t2):
        return t1 < t2
    if len(t1) == 0:
        return True
    if len(t2) == 0:
        return False
    a, b = t1[0], t2[0]
    if len(t1) == len(t2) == 1:
        return elem_less(a, b) if is_tuple(a) else a < b
    if not (a == b or elem_less(a, b)):
        return False
    return elem_less(t1[1:], t2[1:])


def increment(coord, shape):
    """int_tuple.jl:218-232 — next 1-based coordinate, wrapping to all ones."""
    if not is_tuple(coord):
        return coord + 1 if coord < shape else 1
    c, s = coord[0], shape[0]
    if len(coord) == len(shape) == 1:
        return (increment(c, s),)
    if c != s:
        return (increment(c, s),) + tuple(coord[1:])
    return (repeat_like(s, 1),) + increment(coord[1:], shape[1:])


# --------------------------------------------------------------------------
# coordinate <-> index (src/stride.jl)
# --------------------------------------------------------------------------


def _c2i0_int(coord, shape, stride):
    """stride.jl:1-33 — integer coordinate into a tuple shape (colexicographic)."""
    n = len(shape)
    if n == 1:
        if is_tuple(shape[0]):
            return _c2i0_int(coord, shape[0], stride[0])
        return coord * stride[0]
    result = _0
    for i in range(n):
        p = product(shape[i])
        if is_tuple(shape[i]):
            result = result + _c2i0_int(coord % p, shape[i], stride[i])
        else:
            result = result + (coord % shape[i]) * stride[i]
        coord = coord // p
    return result


def coord_to_index0(coord, shape, stride=None):
    """stride.jl:35-70 — 0-based coordinate to 0-based offset."""
    if stride is None:
        if not is_tuple(coord):
            return coord
        fc = flatten(coord)
        fs = flatten(product_like(shape, coord))
        fs = fs if is_tuple(fs) else (fs,)
        acc = fc[-1]
        for c, s in zip(reversed(fc[:-1]), reversed(fs[:-1])):
            acc = c + s * acc
        return acc
    if not is_tuple(coord):
        if not is_tuple(shape):
            return coord * stride
        return _c2i0_int(coord, shape, stride)
    if not is_tuple(shape) or len(coord) != len(shape):
        raise ValueError("coordinate %r does not fit shape %r" % (coord, shape))
    acc = None
    for c, s, d in zip(coord, shape, stride):
        t = coord_to_index0(c, s, d)
        acc = t if acc is None else acc + t
    return acc if acc is not None else _0


def _offset(x):
    """stride.jl:72-80 — 1-based to 0-based; a colon counts as zero."""
    if x is COLON:
        return _0
    if is_tuple(x):
        return tuple(_offset(e) for e in x)
    return x - one(x)


def coord_to_index(coord, shape, stride=None):
    """stride.jl:82-89 — 1-based coordinate to 1-based index; `one(idx)` keeps the integer type."""
    idx = coord_to_index0(_offset(coord), shape, stride)
    return idx + one(idx)


def index_to_coord(index, shape, stride=None):
    """stride.jl:91-128 — 1-based index to a 1-based hierarchical coordinate."""
    if is_tuple(index):
        if stride is None:
            if len(index) != len(shape):
                raise ValueError("index and shape must have the same rank")
            return tuple(index_to_coord(i, s) for i, s in zip(index, shape))
        if not (len(index) == len(shape) == len(stride)):
            raise ValueError("index, shape, and stride must have the same rank")
        return tuple(index_to_coord(i, s, d) for i, s, d in zip(index, shape, stride))
    if stride is None:
        if not is_tuple(shape):
            return index
        stride = compact_col_major(shape, _1)
    if is_tuple(shape):
        if not is_tuple(stride):
            stride = compact_col_major(shape, stride)
        if len(shape) != len(stride):
            raise ValueError("shape, and stride must have the same rank")
        return tuple(index_to_coord(index, s, d) for s, d in zip(shape, stride))
    if isinstance(shape, S) and shape == 1:
        return _0
    crd = ((index - one(index)) // stride) % shape
    return crd + one(crd)


def coord_to_coord(coord, src_shape, dst_shape):
    """stride.jl:133-141."""
    if is_tuple(coord) and is_tuple(src_shape) and is_tuple(dst_shape):
        if not (len(coord) == len(src_shape) == len(dst_shape)):
            raise ValueError("coord, shape1, and shape2 must have the same rank")
        return tuple(coord_to_coord(c, s, d) for c, s, d in zip(coord, src_shape, dst_shape))
    return index_to_coord(coord_to_index(coord, src_shape), dst_shape)


def _compact(shape, current, left):
    """stride.jl:168-236 — (strides, next) ; a static size-1 mode gets stride _0."""
    if is_tuple(shape):
        res = []
        it = shape if left else tuple(reversed(shape))
        for si in it:
            r, current = _compact(si, current, left)
            if left:
                res.append(r)
            else:
                res.insert(0, r)
        return tuple(res), current
    if isinstance(shape, S) and shape == 1:
        return _0, current
    return current, current * shape


def _compact_major(shape, current, left):
    """stride.jl:238-245."""
    if is_tuple(current):
        if len(shape) != len(current):
            raise ValueError("shape and current must have the same rank")
        return tuple(_compact_major(s, c, left) for s, c in zip(shape, current))
    return _compact(shape, current, left)[0]


def compact_col_major(shape, current=_1):
    """stride.jl:249."""
    return _compact_major(shape, current, True)


def compact_row_major(shape, current=_1):
    """stride.jl:250."""
    return _compact_major(shape, current, False)


GenColMajor = "GenColMajor"
GenRowMajor = "GenRowMajor"


def compact_order(shape, order):
    """stride.jl:253-282 — compact strides following `order`.

    Dynamic order entries are replaced by their position placed after the
    largest static order (stride.jl:266-273).
    """
    if order == GenColMajor:
        return compact_col_major(shape)
    if order == GenRowMajor:
        return compact_row_major(shape)
    old_shape = flatten_to_tuple(product_like(shape, order))
    flat_order = flatten_to_tuple(order)
    max_order = _0
    for o in flat_order:
        if isinstance(o, S) and max_order <= o:
            max_order = o
    old_order = tuple(o if isinstance(o, S) else S(i + 1 + int(max_order))
                      for i, o in enumerate(flat_order))
    new_order = unflatten(old_order, order)

    def rec(sh, od):
        if is_tuple(od):
            return tuple(rec(s, o) for s, o in zip(sh, od))
        d = _1
        for s, o in zip(old_shape, old_order):
            d = d * (product(s) if o < od else _1)
        return compact_col_major(sh, d)

    return rec(shape, new_order)


# --------------------------------------------------------------------------
# Layout (src/layout.jl)
# --------------------------------------------------------------------------


def _fmt(x):
    if is_tuple(x):
        if len(x) == 1:
            return "(%s,)" % _fmt(x[0])
        return "(" + ", ".join(_fmt(e) for e in x) + ")"
    return repr(x)


class Layout:
    """layout.jl:48-59 — a shape and a congruent stride."""

    __slots__ = ("shape", "stride")

    def __init__(self, shape, stride):
        if is_tuple(shape) != is_tuple(stride):
            raise TypeError("shape and stride must be congruent")
        if is_tuple(shape) and len(shape) != len(stride):
            raise TypeError("shape and stride must be congruent")
        self.shape = shape
        self.stride = stride

    def __repr__(self):
        return "%s:%s" % (_fmt(self.shape), _fmt(self.stride))

    def __eq__(self, other):
        # numeric equality, like Julia's `==` on tuples of StaticInt / Int
        return isinstance(other, Layout) and self.shape == other.shape and \
            self.stride == other.stride

    def __hash__(self):
        return hash((self.shape, self.stride))

    def identical(self, other):
        """Structural equality including static-ness (Julia `===`)."""
        return self == other and _same_static(self.shape, other.shape) and \
            _same_static(self.stride, other.stride)

    # layout.jl:90-102 — call operator
    def __call__(self, *coord):
        if len(coord) > 1:
            coord = (tuple(coord),)
        c = coord[0]
        if c is COLON or hascolon(c) or _deep_colon(c):
            return slice_layout(self, c)
        return coord_to_index(c, self.shape, self.stride)

    # layout.jl:233-244
    def __getitem__(self, i):
        if isinstance(i, slice):
            r = range(*i.indices(rank(self) + 1))
            return tuple(self[k] for k in r)
        if not is_tuple(self.shape):
            if i != 1:
                raise IndexError(i)
            return self
        return Layout(self.shape[i - 1], self.stride[i - 1])

    def __len__(self):
        return rank(self.shape)

    def __iter__(self):
        return iter(self[k] for k in range(1, rank(self.shape) + 1))


def _same_static(a, b):
    if is_tuple(a):
        return is_tuple(b) and len(a) == len(b) and all(_same_static(x, y) for x, y in zip(a, b))
    return isinstance(a, S) == isinstance(b, S)


def _deep_colon(c):
    return is_tuple(c) and any(e is COLON or _deep_colon(e) for e in c)


def make_layout(*args):
    """layout.jl:133-168."""
    if len(args) >= 1 and all(isinstance(a, Layout) for a in args):
        return Layout(tuple(a.shape for a in args), tuple(a.stride for a in args))
    if len(args) == 1:
        return Layout(args[0], compact_col_major(args[0]))
    shape, second = args
    if second == GenColMajor:
        return Layout(shape, compact_col_major(shape))
    if second == GenRowMajor:
        return Layout(shape, compact_row_major(shape))
    return Layout(shape, second)


def static_layout(shape, stride=None):
    """The `@Layout` macro (layout.jl:188-198)."""
    if stride is None:
        return make_layout(static(shape))
    if isinstance(stride, str):
        return make_layout(static(shape), stride)
    return make_layout(static(shape), static(stride))


SL = static_layout


def make_ordered_layout(shape, order=None):
    """layout.jl:216-221."""
    if isinstance(shape, Layout):
        shape, order = shape.shape, shape.stride
    return make_layout(shape, compact_order(shape, order))


def make_layout_like(layout):
    """layout.jl:223-225."""
    return make_layout(layout.shape,
                       compact_order(filter_zeros(layout.stride, layout.shape), layout.stride))


def shape(l):
    return l.shape if isinstance(l, Layout) else l


def stride(l):
    return l.stride


def size(l, i=None):
    """layout.jl:302-307."""
    if i is None:
        return capacity(shape(l))
    s = shape(l)
    return capacity(s[i - 1] if is_tuple(s) else s)


def cosize(l):
    """layout.jl:350-352."""
    return l(size(l))


def lrank(l, i=None):
    s = shape(l)
    return rank(s if i is None else s[i - 1])


def ldepth(l):
    return depth(shape(l))


def lflatten(l):
    """layout.jl:292-294."""
    return Layout(flatten(l.shape), flatten(l.stride))


def slice_layout(l, coord):
    """layout.jl:364-366."""
    return Layout(slice_(l.shape, coord), slice_(l.stride, coord))


def slice_and_offset(l, coord):
    """layout.jl:368-371 — sliced layout and 0-based element offset."""
    idx = coord_to_index(coord, l.shape, l.stride)
    return slice_layout(l, coord), idx - 1


def dice_layout(l, coord):
    """layout.jl:373-375."""
    return Layout(dice(l.shape, coord), dice(l.stride, coord))


def lappend(l, n, x=None):
    """layout.jl:377-389 — pad with `1:0` modes up to rank n."""
    if x is None:
        x = Layout(_1, _0)
    if lrank(l) == n:
        return l
    return Layout(append(l.shape, x.shape, n), append(l.stride, x.stride, n))


def lprepend(l, n, x=None):
    """layout.jl:391-397."""
    if x is None:
        x = Layout(_1, _0)
    return Layout(prepend(l.shape, x.shape, n), prepend(l.stride, x.stride, n))


def lgroup(l, b, e):
    """layout.jl:404-406."""
    return Layout(group(l.shape, b, e), group(l.stride, b, e))


def get_hier_coord(l, index):
    """layout.jl:105-108."""
    return index_to_coord(index, l.shape, l.stride)


def get_congr_coord(l, index):
    """layout.jl:115-119 — flat 1-based coordinate per mode (0 for static size-1 modes)."""
    h = get_hier_coord(l, index)
    if not is_tuple(l.shape):
        return coord_to_coord(h, l.shape, _1)
    return coord_to_coord(h, l.shape, tuple(_1 for _ in l.shape))


def _transform(f, t1, t2, n=None):
    """layout.jl:408-439 — apply f by mode; without n the longer tail is kept."""
    r1, r2 = lrank(t1), rank(t2)
    if n is not None:
        return make_layout(*[f(t1[i], t2[i - 1]) for i in range(1, n + 1)])
    out = [f(t1[i], t2[i - 1]) for i in range(1, min(r1, r2) + 1)]
    if r1 < r2:
        out += [t2[i - 1] for i in range(r1 + 1, r2 + 1)]
    elif r1 > r2:
        out += [t1[i] for i in range(r2 + 1, r1 + 1)]
    return make_layout(*out)


def _bw_coalesce(n, old_shape, old_stride, new_shape, new_stride):
    """layout.jl:441-479 — fold modes n..1 into the running front."""
    for i in range(n - 1, -1, -1):
        s, d = old_shape[i], old_stride[i]
        if isinstance(s, S) and s == 1:
            continue
        if not is_tuple(new_shape) and isinstance(new_shape, S) and new_shape == 1:
            new_shape, new_stride = s, d
        elif (isinstance(front(new_shape), S) and isinstance(s, S) and isinstance(d, S)
              and isinstance(front(new_stride), S) and s * d == front(new_stride)):
            new_shape = replace_front(new_shape, s * front(new_shape))
            new_stride = replace_front(new_stride, d)
        else:
            new_shape = prepend(new_shape, s)
            new_stride = prepend(new_stride, d)
    if not is_tuple(new_shape) and isinstance(new_shape, S) and new_shape == 1:
        return Layout(_1, _0)
    return Layout(new_shape, new_stride)


def coalesce(l, trg_profile=None):
    """layout.jl:497-509."""
    if trg_profile is not None and is_tuple(trg_profile):
        assert rank(trg_profile) <= lrank(l)
        return _transform(coalesce, l, trg_profile)
    fs, fd = flatten(l.shape), flatten(l.stride)
    if not is_tuple(fs):
        fs, fd = (fs,), (fd,)
    return _bw_coalesce(len(fs) - 1, fs, fd, fs[-1], fd[-1])


def lfilter_zeros(l):
    """layout.jl:511-513."""
    return Layout(filter_zeros(l.stride, l.shape), l.stride)


def lfilter(l):
    """layout.jl:515-517."""
    return coalesce(lfilter_zeros(l))


def _fold_shape(front_shape, rest):
    res = []
    for si in front_shape:
        res.append(smin(sabs(si), rest))
        rest = shape_div(rest, sabs(si))
    return tuple(res), rest


def _compose(ls, ld, rs, rd):
    """layout.jl:520-575 — A (flat shape ls, stride ld) after one B mode rs:rd."""
    if is_tuple(rs):
        return make_layout(*[_compose(ls, ld, rs[i], rd[i]) for i in range(len(rs))])
    if isinstance(rd, S) and rd == 0:
        return Layout(rs, rd)
    if not is_tuple(ls):
        return Layout(rs, ld * rd)
    n = len(ls)
    f_shape, f_stride = ls[:-1], ld[:-1]
    if isinstance(rd, S) and rd == 1:
        shape1, rest_shape = _fold_shape(f_shape, rs)
        return _bw_coalesce(n - 1, shape1, ld, rest_shape, ld[-1])
    shape1, rest_stride = [], rd
    for di in f_shape:
        shape1.append(shape_div(di, rest_stride))
        rest_stride = shape_div(rest_stride, di)
    shape1 = tuple(shape1)
    stride1 = elem_scale(f_stride, shape_div(f_shape, shape1))
    shape2, rest_shape = _fold_shape(shape1, rs)
    return _bw_coalesce(n - 1, shape2, stride1, rest_shape, rest_stride * ld[-1])


def composition(lhs, rhs):
    """layout.jl:593-612 — the layout i -> lhs(rhs(i))."""
    if rhs is COLON:
        return lhs
    if isinstance(rhs, Layout):
        return _compose(flatten(lhs.shape), flatten(lhs.stride), rhs.shape, rhs.stride)
    if is_tuple(rhs):
        assert rank(rhs) <= lrank(lhs)
        return _transform(composition, lhs, rhs, rank(rhs))
    return composition(lhs, make_layout(rhs))


def withshape(l, *shp):
    """layout.jl:614-619."""
    return composition(l, make_layout(shp[0] if len(shp) == 1 else tuple(shp)))


def _complement(shp, strd, cotarget):
    """layout.jl:621-653."""
    if not is_tuple(shp):
        if isinstance(strd, S) and strd == 0:
            return make_layout(cotarget)
        shp, strd = (shp,), (strd,)
    if not is_static(strd):
        raise TypeError("complement requires static strides (layout.jl:640)")
    shp, strd = list(shp), list(strd)
    res_shape, res_stride = [], [_1]
    r = len(shp)
    for i in range(r - 1):
        m = min(strd, key=int)
        k = [int(x) for x in strd].index(int(m))
        new_shape = m // res_stride[i]
        new_stride = m * shp[k]
        assert int(new_shape) != 0
        del shp[k], strd[k]
        res_shape.append(new_shape)
        res_stride.append(new_stride)
    new_shape = strd[0] // res_stride[-1]
    assert int(new_shape) != 0
    res_shape.append(new_shape)
    new_stride = shp[0] * strd[0]
    rest_shape = cld(cotarget, new_stride)
    rest_stride = compact_col_major(rest_shape, new_stride)
    return coalesce(Layout((tuple(res_shape), rest_shape), (tuple(res_stride), rest_stride)))


def complement(l, cotarget=None):
    """layout.jl:660-668."""
    f = lfilter(l)
    if cotarget is None:
        cotarget = cosize(f)
    return _complement(f.shape, f.stride, cotarget)


def right_inverse(l):
    """layout.jl:670-730 — l(right_inverse(l)(i)) == i."""
    if l is COLON:
        return l
    flat = coalesce(l)
    shp = flat.shape if is_tuple(flat.shape) else (flat.shape,)
    strd = flat.stride if is_tuple(flat.stride) else (flat.stride,)
    astride = tuple(sabs(d) for d in strd)
    start = None
    for i, d in enumerate(astride):
        if isinstance(d, S) and d == 1:
            start = i
            break
    if start is None:
        return Layout(_1, _0)
    seq, cur, n = [start], start, len(shp)
    while True:
        nxt = astride[cur] * shp[cur]
        if not isinstance(nxt, S):
            break
        found = None
        for j, d in enumerate(astride):
            if isinstance(d, S) and d == nxt:
                found = j
                break
        if found is None or found in seq:
            break
        seq.append(found)
        cur = found
    rstride = compact_col_major(flat.shape)
    rstride = rstride if is_tuple(rstride) else (rstride,)
    return Layout(unwrap(tuple(shp[i] for i in seq)),
                  unwrap(tuple(ssign(strd[i]) * rstride[i] for i in seq)))


def left_inverse(l):
    """layout.jl:738."""
    if l is COLON:
        return l
    return right_inverse(make_layout(l, complement(l)))


def max_common_vector(a, b):
    """layout.jl:752-761."""
    common = coalesce(composition(a, right_inverse(b)))
    s1 = common.shape[0] if is_tuple(common.shape) else common.shape
    d1 = common.stride[0] if is_tuple(common.stride) else common.stride
    if isinstance(s1, S) and isinstance(d1, S) and d1 == 1:
        return s1
    return _1


def max_common_layout(a, b):
    """layout.jl:741-750."""
    inv_b = right_inverse(b)
    common = coalesce(composition(a, inv_b))
    s1 = common.shape[0] if is_tuple(common.shape) else common.shape
    d1 = common.stride[0] if is_tuple(common.stride) else common.stride
    if isinstance(s1, S) and isinstance(d1, S) and d1 == 1:
        return composition(inv_b, common[1])
    return Layout(_1, _0)


def lzip(a, b=None):
    """layout.jl:763-770."""
    if b is None:
        return Layout(zip_(a.shape), zip_(a.stride))
    return Layout(zip_((a.shape, b.shape)), zip_((a.stride, b.stride)))


def ltranspose(l):
    """layout.jl:772-774."""
    assert lrank(l) == 2
    return make_layout(l[2], l[1])


def _guide(tile):
    """A tile tuple viewed as a zip2_by guide: a Layout counts as a leaf."""
    if is_tuple(tile):
        return tuple(_guide(t) for t in tile)
    return 0


def tile_unzip(l, tile):
    """layout.jl:776-778."""
    g = _guide(tile)
    return Layout(zip2_by(l.shape, g), zip2_by(l.stride, g))


def logical_product(l, tile):
    """layout.jl:826-838."""
    if tile is COLON:
        return l
    if isinstance(tile, Layout):
        return make_layout(l, composition(complement(l, size(l) * cosize(tile)), tile))
    if is_tuple(tile):
        return _transform(logical_product, l, tile)
    return logical_product(l, make_layout(tile))


def _tile_rank(tile):
    return lrank(tile) if isinstance(tile, Layout) else rank(tile)


def zipped_product(l, tile):
    """layout.jl:840-842."""
    return tile_unzip(logical_product(l, tile), tile)


def tiled_product(l, tile):
    """layout.jl:844-847."""
    d = zipped_product(l, tile)
    return d((COLON, repeat(COLON, _tile_rank(tile))))


def blocked_product(block, l, coalesce_result=False):
    """layout.jl:880-889."""
    r = max(lrank(block), lrank(l))
    res = logical_product(lappend(block, r), lappend(l, r))
    res = lzip(res[1], res[2])
    return coalesce(res, repeat(_1, r)) if coalesce_result else res


def raked_product(block, l, coalesce_result=False):
    """layout.jl:919-928."""
    r = max(lrank(block), lrank(l))
    res = logical_product(lappend(block, r), lappend(l, r))
    res = lzip(res[2], res[1])
    return coalesce(res, repeat(_1, r)) if coalesce_result else res


def tile_to_shape(l, trg_shape, ord_shape=GenColMajor):
    """layout.jl:930-935."""
    r = rank(trg_shape)
    assert lrank(l) <= r, "Cannot tile to a smaller shape"
    padded = lappend(l, r)
    pshape = shape_div(product_each(trg_shape), product_each(_as_tuple(padded.shape)))
    return coalesce(blocked_product(padded, make_ordered_layout(pshape, ord_shape)), pshape)


def upcast(l, m):
    """layout.jl:945-965."""

    def f(shp, strd):
        if is_tuple(shp):
            return make_layout(*[f(s, d) for s, d in zip(shp, strd)])
        if isinstance(strd, S):
            if strd == 0:
                return Layout(shp, strd)
            return Layout(shape_div(shp, shape_div(m, sabs(strd))), shape_div(strd, m))
        return Layout(shp, _promote(tdiv(int(strd), int(m)), strd, m))  # safe_div(stride, m()), layout.jl:943,955-958: div keeps the stride's integer type

    return f(l.shape, l.stride)


def downcast(l, n):
    """layout.jl:967-997."""

    def f(shp, strd):
        if is_tuple(shp):
            return make_layout(*[f(s, d) for s, d in zip(shp, strd)])
        if int(strd) in (1, -1) and (isinstance(strd, S) or int(strd) == 1):
            return Layout(shp * n, strd)
        return Layout(shp, strd * n)

    return f(l.shape, l.stride)


def recast_layout(l, new_bytes, old_bytes):
    """layout.jl:999-1010."""
    if new_bytes == old_bytes:
        return l
    if new_bytes > old_bytes:
        assert new_bytes % old_bytes == 0
        return upcast(l, S(new_bytes // old_bytes))
    assert old_bytes % new_bytes == 0
    return downcast(l, S(old_bytes // new_bytes))


def logical_divide(l, tile):
    """layout.jl:1058-1070."""
    if tile is COLON:
        return l
    if isinstance(tile, Layout):
        return composition(l, make_layout(tile, complement(tile, size(l))))
    if is_tuple(tile):
        if len(tile) > lrank(l):
            raise ValueError("too many modes in tile")
        return _transform(logical_divide, l, tile)
    return logical_divide(l, make_layout(tile))


def zipped_divide(l, tile):
    """layout.jl:1114-1116."""
    return tile_unzip(logical_divide(l, tile), tile)


def tiled_divide(l, tile):
    """layout.jl:1123-1127."""
    d = zipped_divide(l, tile)
    return d((COLON, repeat(COLON, lrank(d, 2))))


def make_fragment_like(l):
    """layout.jl:1143-1149."""
    if not isinstance(l, Layout):
        return make_layout(l)
    if not (is_static(l.shape) and is_static(l.stride)) or lrank(l) == 1:
        return make_layout(l.shape)
    rest = make_layout(*[l[i] for i in range(2, lrank(l) + 1)])
    return tiled_product(make_layout(l.shape[0]), make_ordered_layout(rest))


# --------------------------------------------------------------------------
# text form:  "(_2, (_1, _6)):(_1, (_6, _2))"
# --------------------------------------------------------------------------

_TOK = re.compile(r"\s*(_?-?\d+(?:i32)?|[(),:])")


def print_layout(layout):
    """print.jl:7-44 — the rank-2 index table, as a string (lines joined by newlines, no trailing newline).
    Cells hold the 1-based index; the column width follows the number of digits of cosize."""
    assert lrank(layout) == 2
    idx_width = len(str(int(cosize(layout)))) + 2
    sep = "    " + ("+" + "-" * idx_width) * int(size(layout, 2)) + "+"
    lines = [str(layout), "    " + "".join("  " + str(n).rjust(idx_width - 2) + " " for n in range(1, int(size(layout, 2)) + 1))]
    for m in range(1, int(size(layout, 1)) + 1):
        lines.append(sep)
        lines.append(str(m).rjust(2) + "  " + "".join("| " + str(int(layout((m, n)))).rjust(idx_width - 2) + " "
                                                         for n in range(1, int(size(layout, 2)) + 1)) + "|")
    lines.append(sep)
    return "\n".join(lines)


def parse_int_tuple(text):
    toks = _TOK.findall(text)
    if "".join(toks) != re.sub(r"\s+", "", text):
        raise ValueError("cannot parse %r" % text)
    pos = [0]

    def item():
        t = toks[pos[0]]
        pos[0] += 1
        if t == "(":
            out = []
            while toks[pos[0]] != ")":
                out.append(item())
                if toks[pos[0]] == ",":
                    pos[0] += 1
            pos[0] += 1
            return tuple(out)
        if t == ":":
            return COLON
        if t.endswith("i32"):
            return I32(int(t[:-3]))
        return S(int(t[1:])) if t.startswith("_") else int(t)

    v = item()
    if pos[0] != len(toks):
        raise ValueError("trailing text in %r" % text)
    return v


def parse_layout(text):
    """Inverse of `repr(Layout)`; a bare shape gives the compact col-major layout."""
    depth_, split = 0, None
    for i, ch in enumerate(text):
        if ch == "(":
            depth_ += 1
        elif ch == ")":
            depth_ -= 1
        elif ch == ":" and depth_ == 0:
            split = i
            break
    if split is None:
        return make_layout(parse_int_tuple(text))
    return Layout(parse_int_tuple(text[:split]), parse_int_tuple(text[split + 1:]))


def all_indices(l):
    """[l(1), ..., l(size)] as plain ints — brute-force evaluation for invariants."""
    return [int(l(i)) for i in range(1, int(size(l)) + 1)]

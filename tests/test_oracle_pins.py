"""Independent pins for the parts of the oracle that no vector held by the reference covers.

tests/test_oracle_golden.py pins the oracle on the reference's own doctest / issue vectors and on
what the five benchmark configurations touch.  The GPU suite also leans on the oracle for every
scalar primitive, for stencils of every rank and width, stencil2, transform, fold1Seg and SIMD
vectors; here each of those is checked against arithmetic stated a second time in another
vocabulary -- Python's unbounded integers, numpy's fixed-width arrays, `struct`, brute force over
small grids -- chosen so that a slip in the oracle (a wrong shift direction, a floor where a
truncation belongs, a transposed stencil tuple, an offset used as a length) fails a case.
The Haskell facts restated (not taken from the oracle): fixed-width integers wrap; `quot`/`rem`
truncate and `div`/`mod` floor; `shiftR` is arithmetic on signed and logical on unsigned types and
shifts by the width or more give 0 or -1; `rotate` takes its count modulo the width; `countLeadingZeros`
/ `countTrailingZeros` of 0 are the width; `signum`; `max x y = if x <= y then y else x`;
`truncate`/`floor`/`ceiling`/`round` (half to even); `coerce` reinterprets bits.
"""
import math
import struct

import numpy as np
import pytest

from accelerate_amd import ir as A
from oracle import interp as O

from . import progs as Q
from .cases import NPT, same
from .scalar_cases import FLTS, INTS, scalar_cases

SCALAR = scalar_cases()


def _bits(ty):
    return np.iinfo(NPT[ty]).bits


def _signed(ty):
    return np.iinfo(NPT[ty]).min < 0


def _wrap(ty, v):
    """Python integer -> the value a `ty` holds (two's complement)."""
    b = _bits(ty)
    v &= (1 << b) - 1
    return v - (1 << b) if _signed(ty) and v >> (b - 1) else v


def _unsigned(ty, v):
    return int(v) & ((1 << _bits(ty)) - 1)


def _each(ty, f, *cols):
    return np.array([_wrap(ty, f(*[int(c) for c in row])) for row in zip(*cols)], NPT[ty])


def _trunc_div(a, b):
    q = abs(a) // abs(b)
    return q if (a < 0) == (b < 0) else -q


def _rot(ty, x, n):      # rotate left by n, count taken modulo the width (negative: to the right)
    b = _bits(ty)
    n %= b
    u = _unsigned(ty, x)
    return ((u << n) | (u >> (b - n))) if n else u


def _shr(ty, x, n):
    if n >= _bits(ty):
        return -1 if _signed(ty) and x < 0 else 0
    return x >> n if _signed(ty) else _unsigned(ty, x) >> n      # Python's >> on negatives is arithmetic


INT_BINARY = {
    "add": lambda ty, a, b: a + b, "sub": lambda ty, a, b: a - b, "mul": lambda ty, a, b: a * b,
    "band": lambda ty, a, b: a & b, "bor": lambda ty, a, b: a | b, "bxor": lambda ty, a, b: a ^ b,
    "min": lambda ty, a, b: a if a <= b else b, "max": lambda ty, a, b: b if a <= b else a,
    "quot": lambda ty, a, b: _trunc_div(a, b), "rem": lambda ty, a, b: a - _trunc_div(a, b) * b,
    "idiv": lambda ty, a, b: a // b, "mod": lambda ty, a, b: a % b,
    "shl": lambda ty, a, n: 0 if n >= _bits(ty) else a << n, "shr": _shr,
    "rotl": lambda ty, a, n: _rot(ty, a, n), "rotr": lambda ty, a, n: _rot(ty, a, -n),
}
INT_UNARY = {
    "neg": lambda ty, a: -a, "abs": lambda ty, a: abs(a), "sig": lambda ty, a: (a > 0) - (a < 0),
    "bnot": lambda ty, a: ~a,
}
INT_COUNT = {
    "popcount": lambda ty, a: bin(_unsigned(ty, a)).count("1"),
    "clz": lambda ty, a: _bits(ty) - _unsigned(ty, a).bit_length(),
    "ctz": lambda ty, a: _bits(ty) if _unsigned(ty, a) == 0 else (_unsigned(ty, a) & -_unsigned(ty, a)).bit_length() - 1,
}
COMPARE = {"lt": np.less, "gt": np.greater, "lte": np.less_equal, "gte": np.greater_equal, "eq": np.equal,
           "neq": np.not_equal}
FLT_BINARY = {"add": np.add, "sub": np.subtract, "mul": np.multiply, "fdiv": np.divide}
FLT_UNARY = {"neg": np.negative, "abs": np.abs, "sig": np.sign, "sqrt": np.sqrt, "sin": np.sin, "cos": np.cos,
             "tan": np.tan, "asin": np.arcsin, "acos": np.arccos, "atan": np.arctan, "sinh": np.sinh, "cosh": np.cosh,
             "tanh": np.tanh, "asinh": np.arcsinh, "acosh": np.arccosh, "atanh": np.arctanh, "exp": np.exp,
             "log": np.log}
TO_INT = {"truncate": math.trunc, "floor": math.floor, "ceiling": math.ceil,
          "round": lambda v: int(np.rint(v))}     # rint rounds half to even, as Haskell's round does


def independent(name, args):
    """What the named scalar case must yield, from Python / numpy arithmetic; (expected, ulps)."""
    head, _, rest = name.partition("_")
    if rest in INTS:
        ty = rest
        if head in INT_BINARY:
            return _each(ty, lambda a, b: INT_BINARY[head](ty, a, b), *args), None
        if head in ("quotrem", "divmod"):
            q, r = ("quot", "rem") if head == "quotrem" else ("idiv", "mod")
            return [_each(ty, lambda a, b: INT_BINARY[q](ty, a, b), *args),
                    _each(ty, lambda a, b: INT_BINARY[r](ty, a, b), *args)], None
        if head in INT_UNARY:
            return _each(ty, lambda a: INT_UNARY[head](ty, a), *args), None
        if head in INT_COUNT:
            return np.array([INT_COUNT[head](ty, int(a)) for a in args[0]], np.int64), None
        if head in COMPARE:
            return COMPARE[head](*args).astype(np.uint8), None
    if rest in FLTS:
        ty = rest
        t = NPT[ty]
        with np.errstate(all="ignore"):
            if head in FLT_BINARY:
                return FLT_BINARY[head](*args).astype(t), None
            if head in ("min", "max"):      # Ord's defaults: NaN in the first operand wins, in the second loses
                a, b = args
                le = a <= b
                return np.where(le, a, b).astype(t) if head == "min" else np.where(le, b, a).astype(t), None
            if head == "recip":
                return (t(1) / args[0]).astype(t), None
            if head in FLT_UNARY:
                exact = head in ("neg", "abs", "sig", "sqrt")
                return FLT_UNARY[head](args[0]).astype(t), None if exact else 4
            if head == "fpow":
                return np.power(*args).astype(t), 8
            if head == "logbase":           # logBase b x = log x / log b with (base, x) as operands
                return (np.log(args[1].astype(np.float64)) / np.log(args[0].astype(np.float64))).astype(t), 8
            if head == "atan2":
                return np.arctan2(*args).astype(t), 4
            if head in COMPARE:
                return COMPARE[head](*args).astype(np.uint8), None
            if head == "isnan":
                return np.isnan(args[0]).astype(np.uint8), None
            if head == "isinf":
                return np.isinf(args[0]).astype(np.uint8), None
            if head == "pi":
                return (t(math.pi) * args[0]).astype(t), None
            if head == "issue409":
                y = (t(1) / args[0]).astype(t)
                return (y + np.tanh(((-y) * y).astype(t)).astype(t)).astype(t), 4
    parts = name.split("_")
    if parts[0] == "fromintegral":
        return args[0].astype(NPT[parts[2]]), None        # numpy narrows by wrapping, widens by value
    if parts[0] == "tofloating":
        return args[0].astype(NPT[parts[2]]), None
    if parts[0] in TO_INT and len(parts) == 3:
        return np.array([_wrap(parts[2], TO_INT[parts[0]](float(v))) for v in args[0]], NPT[parts[2]]), None
    if name == "max_nan_f32" or name == "max_nan_f64":
        a, b = args
        with np.errstate(invalid="ignore"):
            return np.where(a <= b, b, a), None
    if name in ("add_f16", "mul_f16"):
        f = np.add if name == "add_f16" else np.multiply
        return f(args[0].astype(np.float32), args[1].astype(np.float32)).astype(np.float16), None
    if name == "land":
        return ((args[0] != 0) & (args[1] != 0)).astype(np.uint8), None
    if name == "lor":
        return ((args[0] != 0) | (args[1] != 0)).astype(np.uint8), None
    if name == "lnot":
        return (args[0] == 0).astype(np.uint8), None
    if name == "coerce_f32_u32":
        return np.array([struct.unpack("<I", struct.pack("<f", float(v)))[0] for v in args[0]], np.uint32), None
    if name == "minmaxbound":
        row = [np.iinfo(np.int8).min, np.iinfo(np.uint16).max, np.iinfo(np.int32).min, np.iinfo(np.int64).max,
               np.iinfo(np.uint64).max]
        dts = [np.int8, np.uint16, np.int32, np.int64, np.uint64]
        return [np.full(3, v, d) for v, d in zip(row, dts)], None
    if name == "while_collatz":
        def steps(n):
            k = 0
            while n > 1:
                n, k = (n // 2 if n % 2 == 0 else 3 * n + 1), k + 1
            return k
        return np.array([steps(int(n)) for n in args[0]], np.int64), None
    if name == "case_tag":
        def f(v):
            tag = v & 3
            return 10 if tag == 0 else _wrap("i64", v + 1) if tag == 1 else _wrap("i64", -v)
        return np.array([f(int(v)) for v in args[0]], np.int64), None
    if name == "cond_guards_index":
        xs = args[0]
        return np.array([xs[i] if i < len(xs) else -1 for i in range(40)], np.int64), None
    if name == "index_roundtrip":
        xs = args[0]
        lin = np.arange(xs.size, dtype=np.int64)
        ix = np.unravel_index(lin, xs.shape)                 # row-major, innermost fastest
        return [np.ravel_multi_index(ix, xs.shape).astype(np.int64), xs[ix]], None
    raise KeyError(name)


def _ulp_close(a, b, ulps):
    if isinstance(a, (list, tuple)):
        return len(a) == len(b) and all(_ulp_close(x, y, ulps) for x, y in zip(a, b))
    a, b = np.asarray(a), np.asarray(b)
    if a.shape != b.shape or a.dtype != b.dtype:
        return False
    with np.errstate(invalid="ignore"):
        both_nan = np.isnan(a) & np.isnan(b)
        spacing = np.spacing(np.maximum(np.abs(a), np.abs(b)).astype(a.dtype)).astype(np.float64)
        ok = (np.abs(a.astype(np.float64) - b.astype(np.float64)) <= ulps * spacing) | (a == b)
    return bool(np.all(ok | both_nan))


@pytest.mark.parametrize("case", SCALAR, ids=[c[0] for c in SCALAR])
def test_every_scalar_case_against_python_and_numpy(case):
    name, prog, args, _ = case
    want, ulps = independent(name, args)       # a case without an independent statement fails here
    got = O.run_n(prog.text(), *args)
    if ulps is None:
        assert same(got, want), (name, got, want)
    else:
        assert _ulp_close(got, want, ulps), (name, got, want)


def test_edge_counts_of_shifts_rotates_and_bit_counts():
    # the places where a plausible slip shows: count 0, width - 1, width, all ones, the sign bit
    for ty in INTS:
        b, t = _bits(ty), NPT[ty]
        lo, hi = np.iinfo(t).min, np.iinfo(t).max
        xs = np.array([0, 1, hi, lo, _wrap(ty, -1), _wrap(ty, 1 << (b - 1)), _wrap(ty, 0x5A5A5A5A5A5A5A5A)], t)
        for cnt in (0, 1, b - 1, b, b + 1, 2 * b):
            n = np.full(xs.size, cnt, np.int64)
            for op in ("shl", "shr", "rotl", "rotr"):
                prog = A.alam([A.tarray(1, ty), A.tarray(1, A.Int)], lambda a, c, op=op: A.zipwith(
                    ty, A.lam([ty, A.Int], lambda x, k: A.prim(op, ty, A.pair(x, k))), a, c))
                want = _each(ty, lambda x, k, op=op: INT_BINARY[op](ty, x, k), xs, n)
                assert same(O.run_n(prog.text(), xs, n), want), (ty, op, cnt)
        for op in INT_COUNT:
            prog = A.alam([A.tarray(1, ty)], lambda a, op=op: A.map_(A.Int, A.lam([ty], lambda x: A.prim(op, ty, x)), a))
            assert same(O.run_n(prog.text(), xs), np.array([INT_COUNT[op](ty, int(x)) for x in xs], np.int64)), (ty, op)
    # spot values nobody computes: the widths themselves
    one = lambda op, ty, v: int(O.run_n(A.alam([A.tarray(1, ty)], lambda a: A.map_(
        A.Int, A.lam([ty], lambda x: A.prim(op, ty, x)), a)).text(), np.array([v], NPT[ty]))[0])
    assert one("clz", "i16", 0) == 16 and one("ctz", "u32", 0) == 32 and one("popcount", "i8", -1) == 8
    assert one("clz", "i64", 1) == 63 and one("ctz", "i64", -(1 << 63)) == 63 and one("clz", "i32", -1) == 0


def test_rounding_of_halves_and_negatives():
    for ty in FLTS:
        xs = np.array([0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 2.0, -2.0, 0.49, -0.49, 7.99, -7.99, 1e9 + 0.5], NPT[ty])
        want = {"truncate": [0, 1, 2, 0, -1, -2, 2, -2, 0, 0, 7, -7], "floor": [0, 1, 2, -1, -2, -3, 2, -2, 0, -1, 7, -8],
                "ceiling": [1, 2, 3, 0, -1, -2, 2, -2, 1, 0, 8, -7], "round": [0, 2, 2, 0, -2, -2, 2, -2, 0, 0, 8, -8]}
        for op, exp in want.items():
            prog = A.alam([A.tarray(1, ty)], lambda a, op=op: A.map_(A.i64, A.lam([ty], lambda x: A.prim(op, [ty, A.i64], x)), a))
            got = O.run_n(prog.text(), xs)
            assert list(got[:12]) == exp, (ty, op, list(got))


# ---- SIMD vectors: pack / unpack against numpy slicing ---------------------------------------

@pytest.mark.parametrize("n", [2, 3, 4, 8, 16])
def test_vec_unpack_is_component_selection_and_pack_inverts_it(n):
    rng = np.random.default_rng(n)
    xs = rng.integers(-100, 100, (37, n)).astype(np.int32)
    for k in (0, n // 2, n - 1):
        assert same(O.run_n(Q.vec_extract(n, A.i32, k).text(), xs), xs[:, k])
    cols = [xs[:30 - j, j].copy() for j in range(min(n, 4))]
    if n <= 4:
        got = O.run_n(Q.vec_inject(n, A.i32).text(), *cols)
        m = min(len(c) for c in cols)
        assert same(got, np.stack([c[:m] for c in cols], axis=1))
    # component-wise sums: a scan of vectors is a scan per component
    assert same(O.run_n(Q.vec_scan(n, A.i32, "l").text(), xs), np.cumsum(xs, axis=0, dtype=np.int32))
    assert same(O.run_n(Q.vec_scan(n, A.i32, "r").text(), xs), np.cumsum(xs[::-1], axis=0, dtype=np.int32)[::-1])


# ---- stencils: brute force for every rank, width and boundary --------------------------------

def _remap(i, n, kind):
    """one index component under Clamp / Mirror / Wrap (Interpreter.hs:824-839 restated in words:
    clamp to the edge; reflect about the edge element without repeating it; continue on the
    far side)."""
    if 0 <= i < n:
        return i
    if kind == "clamp":
        return min(max(i, 0), n - 1)
    if kind == "mirror":
        return -i if i < 0 else 2 * (n - 1) - i
    return i % n


def _boundary_fn(ix):
    acc = 100
    for c in ix:
        acc = acc * 3 + c
    return acc


def _weighted_ref(g, widths, kind):
    """stencil_weighted by brute force: taps in row-major order over the offsets -k..+k of every
    dimension, outermost dimension slowest, tap number w (from 1) weighs w."""
    out = np.zeros_like(g)
    offs = [list(range(-(w // 2), w // 2 + 1)) for w in widths]
    for ix in np.ndindex(*g.shape):
        acc, w = 0, 0
        for d in np.ndindex(*[len(o) for o in offs]):
            w += 1
            p = tuple(i + offs[k][d[k]] for k, i in enumerate(ix))
            inside = all(0 <= c < n for c, n in zip(p, g.shape))
            if inside:
                v = int(g[p])
            elif kind == "constant":
                v = -3
            elif kind == "function":
                v = _boundary_fn(p)
            else:
                v = int(g[tuple(_remap(c, n, kind) for c, n in zip(p, g.shape))])
            acc += w * v
        out[ix] = acc
    return out


STENCILS = [([3], (9,)), ([5], (11,)), ([7], (9,)), ([9], (13,)), ([3, 3], (4, 6)), ([5, 5], (6, 7)), ([3, 5], (4, 9)),
            ([7, 7], (8, 9)), ([9, 9], (10, 11)), ([3, 3, 3], (3, 4, 5)), ([3, 3, 3], (2, 5, 3))]


@pytest.mark.parametrize("kind", ["clamp", "mirror", "wrap", "constant", "function"])
@pytest.mark.parametrize("widths,shape", STENCILS, ids=["x".join(map(str, w)) + "_" + "x".join(map(str, s)) for w, s in STENCILS])
def test_stencils_of_every_rank_and_width_by_brute_force(widths, shape, kind):
    if kind == "mirror" and any(s < w // 2 + 1 for w, s in zip(widths, shape)):
        pytest.skip("the remapped index is still outside: an error, tested below")
    rng = np.random.default_rng(sum(widths) + len(shape))
    g = rng.integers(-9, 9, shape).astype(np.int64)
    b = {"constant": A.constant(A.i64, -3), "function": Q.boundary_function(A.i64, len(shape))}.get(kind, kind)
    got = O.run_n(Q.stencil_weighted(A.i64, widths, b).text(), g)
    assert same(got, _weighted_ref(g, widths, kind))


@pytest.mark.parametrize("kind,shape", [("mirror", (1, 5)), ("mirror", (5, 1)), ("wrap", (3,)), ("mirror", (4,))])
def test_extents_too_short_for_mirror_or_wrap_are_index_errors(kind, shape):
    # Mirror on an extent <= halo, Wrap on an extent < halo: one remapping leaves the index outside
    # and the reference's indexCheck fires (Shape.hs:98-106)
    widths = [3, 3] if len(shape) == 2 else [9]
    g = np.ones(shape, np.int64)
    with pytest.raises(O.OracleError, match="index out of bounds"):
        O.run_n(Q.stencil_weighted(A.i64, widths, kind).text(), g)


@pytest.mark.parametrize("b1,b2", [("clamp", "wrap"), ("mirror", "clamp"), ("wrap", "mirror"),
                                   ("constant", "clamp"), ("function", "constant")])
def test_stencil2_by_brute_force(b1, b2):
    # two sources of different extents: the result has the intersection, each source is bounded
    # by its own extents (Interpreter.hs:652-668)
    rng = np.random.default_rng(5)
    x = rng.integers(-9, 9, (5, 8)).astype(np.int64)
    y = rng.integers(-9, 9, (7, 6)).astype(np.int64)
    mk = lambda k: {"constant": A.constant(A.i64, 4), "function": Q.boundary_function(A.i64, 2)}.get(k, k)
    got = O.run_n(Q.stencil2_sum(A.i64, mk(b1), mk(b2)).text(), x, y)

    def tap(g, p, kind):
        if all(0 <= c < n for c, n in zip(p, g.shape)):
            return int(g[p])
        if kind == "constant":
            return 4
        if kind == "function":
            return _boundary_fn(p)
        return int(g[tuple(_remap(c, n, kind) for c, n in zip(p, g.shape))])

    ref = np.zeros((5, 6), np.int64)
    for r in range(5):
        for c in range(6):
            # left + right of the first source's middle row, twice the second's centre, its top minus its bottom
            ref[r, c] = (tap(x, (r, c - 1), b1) + tap(x, (r, c + 1), b1) + 2 * tap(y, (r, c), b2)
                         + tap(y, (r - 1, c), b2) - tap(y, (r + 1, c), b2))
    assert same(got, ref)


# ---- fold1Seg, transform ---------------------------------------------------------------------

def _split_places(lens, xs):
    out, at = [], 0
    for n in lens:
        out.append(xs[at:at + n])
        at += n
    return out


@pytest.mark.parametrize("shape", [(40,), (3, 40), (2, 3, 40)])
def test_fold1seg_is_foldl1_over_split_places(shape):
    # the reference's own test reference: foldl1 over splitPlaces (Test/NoFib/Prelude/Fold.hs:254-269),
    # with an operator that is neither commutative nor blind to the split: the interval monoid
    rng = np.random.default_rng(len(shape))
    lens = np.array([3, 1, 10, 7, 2, 9], np.int64)           # 32 of the 40 elements, no empty segment
    a, b = rng.integers(-50, 50, shape).astype(np.int64), rng.integers(-50, 50, shape).astype(np.int64)
    got = O.run_n(Q.fold1seg_interval(len(shape)).text(), [a, b], lens)
    ra, rb = np.zeros(shape[:-1] + (len(lens),), np.int64), np.zeros(shape[:-1] + (len(lens),), np.int64)
    for outer in np.ndindex(*shape[:-1]):
        for s, (sa, sb) in enumerate(zip(_split_places(lens, a[outer]), _split_places(lens, b[outer]))):
            ra[outer + (s,)], rb[outer + (s,)] = sa[0], sb[-1]     # (first of the leftmost, second of the rightmost)
    assert same(got, [ra, rb])
    # and a sum, against numpy
    got = O.run_n(Q.fold1seg_sum(A.i64, len(shape)).text(), a, lens)
    used = a[..., :int(lens.sum())]                             # what lies behind the last segment is ignored
    ref = np.add.reduceat(used, np.concatenate([[0], np.cumsum(lens)[:-1]]), axis=-1)
    assert same(got, ref)


def test_fold1seg_of_an_empty_segment_is_an_error():
    with pytest.raises(O.OracleError, match="empty segment"):
        O.run_n(Q.fold1seg_sum(A.i64, 1).text(), np.arange(10, dtype=np.int64), np.array([3, 0, 4], np.int64))


def test_transform_is_map_after_backpermute():
    # Transform sh p f a: out[ix] = f (a ! p ix)   (Interpreter.hs:344-351)
    rng = np.random.default_rng(3)
    m = rng.integers(-100, 100, (5, 7)).astype(np.int64)
    got = O.run_n(Q.transform_transpose_affine().text(), m)
    assert same(got, 3 * m.T + 1)

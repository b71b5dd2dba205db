"""Programs that exercise every scalar primitive (PrimFun, AST.hs:661-753) and the scalar
control constructs through `map` / `zipWith`, with inputs that hit the places where Haskell
and C disagree (negative operands of div/mod, shifts by the width, rounding ties, NaN)."""
from __future__ import annotations

import numpy as np

from accelerate_amd import ir as A

from .cases import NPT

INTS = ["i8", "i16", "i32", "i64", "u8", "u16", "u32", "u64"]
FLTS = ["f32", "f64"]


def _map1(tin, tout, f):
    return A.alam([A.tarray(1, tin)], lambda xs: A.map_(tout, A.lam([tin], f), xs))


def _zip2(t1, t2, tout, f):
    return A.alam([A.tarray(1, t1), A.tarray(1, t2)], lambda xs, ys: A.zipwith(tout, A.lam([t1, t2], f), xs, ys))


def _ints(ty, rng, n=96):
    info = np.iinfo(NPT[ty])
    edge = [0, 1, 2, 3, 7, info.max, info.max - 1, info.min, info.min + 1]
    if info.min < 0:
        edge += [-1, -2, -3, -7]
    body = rng.integers(info.min, info.max, n - len(edge), dtype=np.int64 if ty != "u64" else np.uint64, endpoint=True)
    return np.concatenate([np.array(edge, dtype=NPT[ty]), body.astype(NPT[ty])])


def _flts(ty, rng, n=96):
    edge = [0.0, -0.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 1.0, -1.0, 3.75, -3.25, 1e-3, 100.25]
    return np.concatenate([np.array(edge, NPT[ty]), rng.uniform(-8, 8, n - len(edge)).astype(NPT[ty])])


def scalar_cases():
    """(id, program, args, ulps): ulps None = bit-exact, otherwise allowed distance in units
    of the last place of the result type (transcendental functions come from different
    math libraries on the two sides)."""
    rng = np.random.default_rng(77)
    out = []
    add = lambda *c: out.append(c)
    for ty in INTS:
        x, y = _ints(ty, rng), _ints(ty, rng)
        ynz = np.where(y == 0, NPT[ty](3), y)
        if np.iinfo(NPT[ty]).min < 0:       # minBound `quot` (-1) overflows in the reference
            ynz = np.where(ynz == NPT[ty](-1), NPT[ty](5), ynz)
        for name in ("add", "sub", "mul", "band", "bor", "bxor", "min", "max"):
            add("%s_%s" % (name, ty), _zip2(ty, ty, ty, lambda a, b, n=name: A.prim(n, ty, A.pair(a, b))), [x, y], None)
        for name in ("quot", "rem", "idiv", "mod"):
            add("%s_%s" % (name, ty), _zip2(ty, ty, ty, lambda a, b, n=name: A.prim(n, ty, A.pair(a, b))), [x, ynz], None)
        for name in ("quotrem", "divmod"):
            add("%s_%s" % (name, ty), _zip2(ty, ty, A.tpair(ty, ty), lambda a, b, n=name: A.prim(n, ty, A.pair(a, b))),
                [x, ynz], None)
        for name in ("neg", "abs", "sig", "bnot"):
            add("%s_%s" % (name, ty), _map1(ty, ty, lambda a, n=name: A.prim(n, ty, a)), [x], None)
        for name in ("popcount", "clz", "ctz"):
            add("%s_%s" % (name, ty), _map1(ty, A.Int, lambda a, n=name: A.prim(n, ty, a)), [x], None)
        bits = np.iinfo(NPT[ty]).bits
        sh = rng.integers(0, bits + 3, x.size).astype(np.int64)
        for name in ("shl", "shr"):
            add("%s_%s" % (name, ty), _zip2(ty, A.Int, ty, lambda a, b, n=name: A.prim(n, ty, A.pair(a, b))), [x, sh], None)
        rot = rng.integers(-2 * bits, 2 * bits, x.size).astype(np.int64)
        for name in ("rotl", "rotr"):
            add("%s_%s" % (name, ty), _zip2(ty, A.Int, ty, lambda a, b, n=name: A.prim(n, ty, A.pair(a, b))), [x, rot], None)
        for name in ("lt", "gt", "lte", "gte", "eq", "neq"):
            add("%s_%s" % (name, ty), _zip2(ty, ty, A.u8, lambda a, b, n=name: A.prim(n, ty, A.pair(a, b))), [x, x[::-1].copy()], None)
        for to in ("i8", "u16", "i32", "u64", "i64"):
            add("fromintegral_%s_%s" % (ty, to), _map1(ty, to, lambda a, t=to: A.fromintegral(ty, t, a)), [x], None)
        for to in FLTS:
            add("fromintegral_%s_%s" % (ty, to), _map1(ty, to, lambda a, t=to: A.fromintegral(ty, t, a)), [x], None)
    add("minmaxbound", A.generate(A.tarray(1, A.ttup(A.i8, A.u16, A.i32, A.i64, A.u64)), A.sh(3), A.lam(
        [A.tshape(1)], lambda ix: A.tup(A.minbound(A.i8), A.maxbound(A.u16), A.minbound(A.i32), A.maxbound(A.i64),
                                        A.maxbound(A.u64)))), [], None)
    for ty in FLTS:
        x, y = _flts(ty, rng), _flts(ty, rng)
        for name in ("add", "sub", "mul", "fdiv", "min", "max"):
            add("%s_%s" % (name, ty), _zip2(ty, ty, ty, lambda a, b, n=name: A.prim(n, ty, A.pair(a, b))), [x, y], None)
        for name in ("neg", "abs", "sig", "recip", "sqrt"):
            arg = np.abs(x) if name == "sqrt" else x
            add("%s_%s" % (name, ty), _map1(ty, ty, lambda a, n=name: A.prim(n, ty, a)), [arg], None)
        for name in ("sin", "cos", "tan", "atan", "sinh", "cosh", "tanh", "asinh", "exp"):
            add("%s_%s" % (name, ty), _map1(ty, ty, lambda a, n=name: A.prim(n, ty, a)), [x], 4)
        unit = (x / 9).astype(NPT[ty])
        for name in ("asin", "acos", "atanh"):
            add("%s_%s" % (name, ty), _map1(ty, ty, lambda a, n=name: A.prim(n, ty, a)), [unit], 4)
        pos = (np.abs(x) + NPT[ty](1.25)).astype(NPT[ty])
        for name in ("log", "acosh"):
            add("%s_%s" % (name, ty), _map1(ty, ty, lambda a, n=name: A.prim(n, ty, a)), [pos], 4)
        for name in ("fpow", "logbase"):
            add("%s_%s" % (name, ty), _zip2(ty, ty, ty, lambda a, b, n=name: A.prim(n, ty, A.pair(a, b))),
                [pos, (np.abs(y) + NPT[ty](1.5)).astype(NPT[ty])], 8)
        add("atan2_%s" % ty, _zip2(ty, ty, ty, lambda a, b: A.atan2(ty, a, b)), [x, y], 4)
        for name in ("truncate", "round", "floor", "ceiling"):
            for to in ("i32", "i64"):
                add("%s_%s_%s" % (name, ty, to), _map1(ty, to, lambda a, n=name, t=to: A.prim(n, [ty, t], a)), [x], None)
        # Issue409: y + tanh ((-y) * y) with y = recip x, at x = 1 (1 + tanh (-1))
        add("issue409_%s" % ty, _map1(ty, ty, lambda a: A.let(ty, A.recip(ty, a), lambda y: A.let(
            ty, A.mul(ty, A.neg(ty, y), y), lambda b: A.add(ty, y, A.tanh(ty, b))))), [np.array([1.0, 2.0, -0.5], NPT[ty])], 4)
        special = np.array([np.nan, np.inf, -np.inf, 0.0, 1.0], NPT[ty])
        add("isnan_%s" % ty, _map1(ty, A.u8, lambda a: A.isnan(ty, a)), [special], None)
        add("isinf_%s" % ty, _map1(ty, A.u8, lambda a: A.isinf(ty, a)), [special], None)
        add("max_nan_%s" % ty, _zip2(ty, ty, ty, lambda a, b: A.max_(ty, a, b)), [special, special[::-1].copy()], None)
        for name in ("lt", "gte", "eq"):
            add("%s_%s" % (name, ty), _zip2(ty, ty, A.u8, lambda a, b, n=name: A.prim(n, ty, A.pair(a, b))), [x, y], None)
        other = "f64" if ty == "f32" else "f32"
        add("tofloating_%s_%s" % (ty, other), _map1(ty, other, lambda a: A.tofloating(ty, other, a)), [x], None)
        add("pi_%s" % ty, _map1(ty, ty, lambda a: A.mul(ty, A.pi(ty), a)), [x], None)
    # Float16 arithmetic goes through Float32 on both sides
    h = _flts("f16", rng)
    add("add_f16", _zip2(A.f16, A.f16, A.f16, lambda a, b: A.add(A.f16, a, b)), [h, h[::-1].copy()], None)
    add("mul_f16", _zip2(A.f16, A.f16, A.f16, lambda a, b: A.mul(A.f16, a, b)), [h, h[::-1].copy()], None)
    # booleans, coercion, scalar control flow
    b1 = rng.integers(0, 2, 64).astype(np.uint8)
    b2 = rng.integers(0, 2, 64).astype(np.uint8)
    add("land", _zip2(A.u8, A.u8, A.u8, A.land), [b1, b2], None)
    add("lor", _zip2(A.u8, A.u8, A.u8, A.lor), [b1, b2], None)
    add("lnot", _map1(A.u8, A.u8, A.lnot), [b1], None)
    xf = _flts("f32", rng)
    add("coerce_f32_u32", _map1(A.f32, A.u32, lambda a: A.coerce(A.f32, A.u32, a)), [xf], None)
    xi = _ints("i64", rng)
    small = (np.abs(xi) % 50).astype(np.int64)
    # while: count the steps of the Collatz iteration (While, AST.hs:597-601)
    st2 = A.ttup(A.Int, A.Int)
    collatz = _map1(A.Int, A.Int, lambda n0: A.let(st2, A.while_(
        st2,
        lambda st: A.gt(A.Int, A.untup(st)[0], A.constI(1)),
        lambda st: A.tup(A.cond(A.eq(A.Int, A.band(A.Int, A.untup(st)[0], A.constI(1)), A.constI(0)),
                                A.quot(A.Int, A.untup(st)[0], A.constI(2)),
                                A.add(A.Int, A.mul(A.Int, A.constI(3), A.untup(st)[0]), A.constI(1))),
                         A.add(A.Int, A.untup(st)[1], A.constI(1))),
        A.tup(n0, A.constI(0))), lambda fin: A.untup(fin)[1]))
    add("while_collatz", collatz, [small + 1], None)
    # case on a tag with a default (Case, AST.hs:585-589)
    add("case_tag", _map1(A.Int, A.Int, lambda v: A.case(
        A.fromintegral(A.Int, A.u8, A.band(A.Int, v, A.constI(3))),
        [(0, A.constI(10)), (1, A.add(A.Int, v, A.constI(1)))], A.neg(A.Int, v))), [xi], None)
    # cond guarding an out-of-bounds index must stay a branch (Issue187)
    guard = A.alam([A.tarray(1, A.Int)], lambda xs: A.generate(
        A.tarray(1, A.Int), A.sh(40), A.lam([A.tshape(1)], lambda ix: A.cond(
            A.lt(A.Int, A.untup(ix)[0], A.untup_shape(xs)[0]),
            A.index(xs, A.vexp(ix)), A.constI(-1)))))
    add("cond_guards_index", guard, [np.arange(10, dtype=np.int64)], None)
    # index arithmetic: toIndex / fromIndex / shapeSize round trip on a rank-3 shape
    rt = A.alam([A.tarray(3, A.Int)], lambda xs: A.generate(
        A.tarray(1, A.ttup(A.Int, A.Int)), A.sh(A.shapesize(3, A.shape(xs))), A.lam([A.tshape(1)], lambda ix: A.let(
            A.tshape(3), A.fromindex(3, A.shape(xs), A.untup(ix)[0]),
            lambda i3: A.tup(A.toindex(3, A.shape(xs), A.vexp(i3)), A.index(xs, A.vexp(i3)))))))
    add("index_roundtrip", rt, [np.arange(2 * 3 * 5, dtype=np.int64).reshape(2, 3, 5) * 7], None)
    return out
